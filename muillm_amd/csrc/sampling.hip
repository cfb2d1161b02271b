// Greedy token selection: argmax over each row of a [rows, vocab] 16-bit logits matrix,
// lowest index on ties. One workgroup of 1024 threads per row, 128-bit loads, wave reduce on
// (value, index) pairs, LDS across the 16 waves. It keeps the decode loop free of
// library reductions (which may record memset nodes when captured into a HIP graph).
// Reference counterpart: the greedy branch of the sampling loop, torch.argmax at
// muillm/sampling/generation.py:330-335.
#include "common.cuh"

namespace mui {

constexpr int kArgmaxThreads = 1024;

__device__ __forceinline__ void take_better(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

template <typename T>
__global__ void __launch_bounds__(kArgmaxThreads) argmax_rows_kernel(const uint16_t* logits, long row_stride,
                                                                    int64_t* out, int vocab) {
  __shared__ float sv[kArgmaxThreads / kWave];
  __shared__ int si[kArgmaxThreads / kWave];
  const uint16_t* row = logits + (long)blockIdx.x * row_stride;
  const int t = threadIdx.x;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  const bool vec = ((row_stride & 7) == 0) && ((((uintptr_t)logits) & 15u) == 0);
  const int nvec = vec ? (vocab >> 3) : 0;
  for (int c = t; c < nvec; c += kArgmaxThreads) {
    float f[8];
    unpack8<T>(ld16(row + (c << 3)), f);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // NaN never wins; strict > keeps the lowest index inside a thread's ascending scan
      if (f[i] > best) { best = f[i]; best_i = (c << 3) + i; }
    }
  }
  for (int i = (nvec << 3) + t; i < vocab; i += kArgmaxThreads) {
    const float f = T::one(row[i]);
    if (f > best) { best = f; best_i = i; }
  }
  // wave reduce with shuffles over (value, index)
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off);
    const int oi = __shfl_xor(best_i, off);
    take_better(best, best_i, ov, oi);
  }
  if ((t & (kWave - 1)) == 0) { sv[t >> 6] = best; si[t >> 6] = best_i; }
  __syncthreads();
  if (t == 0) {
    for (int w = 1; w < kArgmaxThreads / kWave; ++w) take_better(best, best_i, sv[w], si[w]);
    out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
  }
}

}  // namespace mui

using namespace mui;

extern "C" int mui_argmax(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                          int64_t* out_index, int rows, int vocab) {
  MUI_CHECK_ARG(logits && out_index && rows > 0 && vocab > 0 && row_stride >= vocab);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((argmax_rows_kernel<F16>), dim3(rows), dim3(kArgmaxThreads), 0, s,
                       (const uint16_t*)logits, row_stride, out_index, vocab);
  else if (dtype == MUI_DTYPE_BF16)
    hipLaunchKernelGGL((argmax_rows_kernel<BF16>), dim3(rows), dim3(kArgmaxThreads), 0, s,
                       (const uint16_t*)logits, row_stride, out_index, vocab);
  else
    return MUI_ERR_INVALID_ARG;
  return launch_status();
}
