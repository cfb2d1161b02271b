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
