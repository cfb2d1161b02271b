// Standalone RMSNorm over the last dimension of a [rows, k] matrix:
//   y = gamma * x * rsqrt(mean(x^2) + eps)      (fp32 math, one rounding at the store)
// Counterpart of csrc/norm/rmsnorm_fp16_kernels.cu:35-126 in the reference (which every
// block re-reduces a whole row for 512 outputs); here one workgroup owns one row, reads it
// once with 128-bit loads into registers, reduces through DPP + LDS and writes it back.
#include "common.cuh"

namespace mui {

constexpr int kNormThreads = 256;

// VEC path: k % 8 == 0 and 16-byte aligned rows; up to CH*2048 elements stay in registers.
template <typename T, int CH>
__global__ void __launch_bounds__(kNormThreads) rmsnorm_vec_kernel(
    const uint16_t* gamma, const uint16_t* x, uint16_t* y,
    int k, float eps) {
  __shared__ float red[kNormThreads / kWave];
  const int t = threadIdx.x;
  const int kc = k >> 3;
  const uint16_t* xr = x + (long)blockIdx.x * k;
  uint16_t* yr = y + (long)blockIdx.x * k;

  float xf[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = t + kNormThreads * j;
    if (c < kc) {
      unpack8<T>(ld16(xr + (c << 3)), xf[j]);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss = fmaf(xf[j][i], xf[j][i], ss);
    }
  }
  ss = wave_sum(ss);
  if ((t & (kWave - 1)) == 0) red[t >> 6] = ss;
  __syncthreads();
  const float rs = rsqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)k + eps);
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = t + kNormThreads * j;
    if (c < kc) {
      float gf[8], o[8];
      unpack8<T>(ld16(gamma + (c << 3)), gf);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = gf[i] * (xf[j][i] * rs);
      *(u32x4*)(yr + (c << 3)) = pack8<T>(o);
    }
  }
}

// Generic path: any k, any alignment; two passes over the row (second one hits cache).
template <typename T>
__global__ void __launch_bounds__(kNormThreads) rmsnorm_any_kernel(
    const uint16_t* gamma, const uint16_t* x, uint16_t* y,
    int k, float eps) {
  __shared__ float red[kNormThreads / kWave];
  const int t = threadIdx.x;
  const uint16_t* xr = x + (long)blockIdx.x * k;
  uint16_t* yr = y + (long)blockIdx.x * k;
  float ss = 0.f;
  for (int i = t; i < k; i += kNormThreads) {
    const float v = T::one(xr[i]);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  if ((t & (kWave - 1)) == 0) red[t >> 6] = ss;
  __syncthreads();
  const float rs = rsqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)k + eps);
  for (int i = t; i < k; i += kNormThreads)
    yr[i] = T::pack(T::one(gamma[i]) * (T::one(xr[i]) * rs));
}

template <typename T>
static int launch_rmsnorm(hipStream_t s, const uint16_t* gamma, const uint16_t* x, uint16_t* y,
                          int rows, int k, float eps) {
  const bool vec = (k % 8 == 0) && aligned16(x) && aligned16(y) && aligned16(gamma) &&
                   k <= 8 * 8 * kNormThreads;
  dim3 grid(rows), block(kNormThreads);
  if (vec) {
    const int ch = ceil_div(k >> 3, kNormThreads);
    if (ch <= 1) hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 1>), grid, block, 0, s, gamma, x, y, k, eps);
    else if (ch <= 2) hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 2>), grid, block, 0, s, gamma, x, y, k, eps);
    else if (ch <= 4) hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 4>), grid, block, 0, s, gamma, x, y, k, eps);
    else hipLaunchKernelGGL((rmsnorm_vec_kernel<T, 8>), grid, block, 0, s, gamma, x, y, k, eps);
  } else {
    hipLaunchKernelGGL((rmsnorm_any_kernel<T>), grid, block, 0, s, gamma, x, y, k, eps);
  }
  return launch_status();
}

}  // namespace mui

using namespace mui;

extern "C" int mui_rmsnorm(mui_stream_t stream, int dtype, const void* weights, const void* x,
                           float epsilon, void* y, int rows, int k) {
  MUI_CHECK_ARG(weights && x && y);
  MUI_CHECK_ARG(rows > 0 && k > 0);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    return launch_rmsnorm<F16>(s, (const uint16_t*)weights, (const uint16_t*)x, (uint16_t*)y, rows, k, epsilon);
  if (dtype == MUI_DTYPE_BF16)
    return launch_rmsnorm<BF16>(s, (const uint16_t*)weights, (const uint16_t*)x, (uint16_t*)y, rows, k, epsilon);
  return MUI_ERR_INVALID_ARG;
}

// ---------------------------------------------------------------------------------------
// SiLU(gate) * up on an interleaved [rows, n, 2] buffer (the output of ONE matmul with the
// row-interleaved gate/up weights, used for prompts too long for the fused GEMV family):
// out[r, i] = silu(gu[r, 2i]) * gu[r, 2i + 1], fp32 math, one rounding.
// The reference runs two matmuls, an activation kernel and a multiply
// (muillm/modules/gateupdownmlp.py:343-359).
// ---------------------------------------------------------------------------------------
namespace mui {
template <typename T>
__global__ void __launch_bounds__(256) silu_mul_interleaved_kernel(const uint16_t* gu, uint16_t* out, long total8) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long c = (long)blockIdx.x * blockDim.x + threadIdx.x; c < total8; c += stride) {
    const u32x4 a = ld16(gu + c * 16), b = ld16(gu + c * 16 + 8);
    float fa[8], fb[8], o[8];
    unpack8<T>(a, fa);
    unpack8<T>(b, fb);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = silu_f32(fa[2 * i]) * fa[2 * i + 1];
      o[4 + i] = silu_f32(fb[2 * i]) * fb[2 * i + 1];
    }
    *(u32x4*)(out + c * 8) = pack8<T>(o);
  }
}
}  // namespace mui

extern "C" int mui_silu_mul_interleaved(mui_stream_t stream, int dtype, const void* gate_up, void* out,
                                        long rows, int n) {
  MUI_CHECK_ARG(gate_up && out && rows > 0 && n > 0);
  MUI_CHECK_ARG(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16);
  if (n % 8) return MUI_ERR_UNSUPPORTED;
  if ((((uintptr_t)gate_up | (uintptr_t)out) & 15u) != 0) return MUI_ERR_ALIGNMENT;
  const long total8 = rows * (n / 8);
  long blocks = (total8 + 255) / 256;
  const long cap = (long)mui::device_cus() * 16;
  if (blocks > cap) blocks = cap;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((mui::silu_mul_interleaved_kernel<mui::F16>), dim3((unsigned)blocks), dim3(256), 0, s,
                       (const uint16_t*)gate_up, (uint16_t*)out, total8);
  else
    hipLaunchKernelGGL((mui::silu_mul_interleaved_kernel<mui::BF16>), dim3((unsigned)blocks), dim3(256), 0, s,
                       (const uint16_t*)gate_up, (uint16_t*)out, total8);
  return mui::launch_status();
}
