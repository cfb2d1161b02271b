/*
 * muillm_amd.h -- C ABI of libmuillm_amd.so: muiLLM's decode-time hot path as
 * hand-written HIP kernels for AMD MI355X (gfx950).
 *
 * Every entry point
 *   - takes plain device pointers, sizes and a HIP stream (as void*), no framework types;
 *   - enqueues asynchronously on that stream and never synchronises or allocates;
 *   - owns nothing: outputs and scratch are caller-allocated;
 *   - returns MUI_OK (0) or a negative MUI_ERR_* code (mui_status_string() names it);
 *   - validates shapes/alignment on the host before launching anything.
 *
 * The comment above each declaration names the entry of the reference's pybind11
 * module `muillm_ext` (Epliz/muiLLM, csrc/module.cpp) that it stands in for.
 *
 * Tensors are dense row-major unless a stride argument says otherwise. "16-bit type"
 * means fp16 or bf16 selected by the `dtype` argument; all arithmetic is fp32 with a
 * single rounding at the store.
 */
#ifndef MUILLM_AMD_H
#define MUILLM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUI_ABI_VERSION 1

/* status codes (reference: TORCH_CHECK exceptions, csrc/linear/linear.cu:72-74;
 * muillm_error_t, csrc/base.h:4-7) */
#define MUI_OK 0
#define MUI_ERR_INVALID_ARG (-1) /* null pointer, non-positive size, bad enum */
#define MUI_ERR_UNSUPPORTED (-2) /* shape outside what the kernels cover */
#define MUI_ERR_LAUNCH (-3)      /* hipGetLastError() after the launch was not hipSuccess */
#define MUI_ERR_ALIGNMENT (-4)   /* a pointer or row pitch is not 16-byte aligned */
#define MUI_ERR_DEVICE (-5)      /* device query failed / not a gfx950 device */

#define MUI_DTYPE_F16 0
#define MUI_DTYPE_BF16 1

/* largest token batch the decode kernels accept in one call */
#define MUI_MAX_TOKENS 8

typedef void* mui_stream_t; /* a hipStream_t; NULL is the default stream */

/* What muillm_engine_init() (csrc/engine.cpp:3-26, csrc/gpu_info.cpp:7-69) records per
 * GPU, for the current device only. */
typedef struct mui_device_info {
  int device;              /* HIP ordinal */
  int compute_units;       /* 256 on MI355X */
  int wave_size;           /* 64 */
  int simd_lanes;          /* compute_units * 4 SIMDs * 16 lanes */
  int lds_bytes_per_block; /* max LDS per workgroup */
  int l2_bytes;
  int clock_khz;
  int is_gfx950;           /* 1 when gcnArchName starts with "gfx950" */
  uint64_t hbm_bytes;
  char arch[64];           /* gcnArchName */
} mui_device_info_t;

int mui_abi_version(void);
const char* mui_status_string(int status);

/* muillm_engine_init (csrc/module.cpp:283). Fills `out` for HIP device `device`. */
int mui_device_info(int device, mui_device_info_t* out);

/* ------------------------------------------------------------------------------------
 * Linear family
 * ---------------------------------------------------------------------------------- */

/* muillm_linear_forward / muillm_linear_module_forward (csrc/module.cpp:178,312;
 * csrc/linear/linear.cu:76-208; kernels csrc/linear/linear_fp16_kernels.cu:163-626).
 *
 *   y[t, n] = (sum_k W[n, k] * xn[t, k]) * mul_bias[n] + add_bias[n] + residual[t, n]
 *   xn[t, :] = norm_weights ? norm_weights * x[t, :] * rsqrt(mean(x[t, :]^2) + epsilon) : x[t, :]
 *
 * W is [n_out, k_in] with row pitch `w_pitch` elements (w_pitch == k_in when dense);
 * x is [tokens, k_in]; y, residual are [tokens, n_out]; norm_weights is [k_in];
 * mul_bias, add_bias are [n_out]. norm_weights, mul_bias, add_bias, residual may be NULL.
 * tokens in 1..MUI_MAX_TOKENS. epsilon is added to the mean (HuggingFace convention).
 * Requirements: k_in % 8 == 0, W and x 16-byte aligned, w_pitch % 8 == 0.
 * y may alias residual. */
int mui_linear(mui_stream_t stream, int dtype, const void* weights, long w_pitch,
               const void* x, const void* norm_weights, float epsilon,
               const void* mul_bias, const void* add_bias, const void* residual,
               void* y, int n_out, int k_in, int tokens);

/* muillm_rmsnorm_forward (csrc/module.cpp:251; csrc/norm/rmsnorm.cu:31-85; kernel
 * csrc/norm/rmsnorm_fp16_kernels.cu:35-126).
 *   y[r, :] = weights * x[r, :] * rsqrt(mean(x[r, :]^2) + epsilon), rows r < rows.
 * Any k >= 1; 16-byte aligned rows take the vector path. y may alias x. */
int mui_rmsnorm(mui_stream_t stream, int dtype, const void* weights, const void* x,
                float epsilon, void* y, int rows, int k);

/* First half of muillm_gateupsilu_forward (csrc/module.cpp:182; csrc/ffn/gateup.cu:88-219;
 * kernels csrc/ffn/gateup_fp16_kernels.cu:160-604):
 *   h[t, n] = silu(sum_k G[n, k] xn[t, k]) * (sum_k U[n, k] xn[t, k])
 * G and U are [n_inter, k_in] with a common row pitch `gu_pitch` elements. They may be two
 * separate dense matrices (gu_pitch == k_in) or the two interleaved halves of one packed
 * [n_inter, 2, k_in] buffer (up == gate + k_in, gu_pitch == 2 * k_in), which is the layout
 * the Python layer repacks to. xn as in mui_linear. h is [tokens, n_inter].
 * The second half (down projection + residual) is mui_linear with residual. */
int mui_gateup_silu(mui_stream_t stream, int dtype, const void* gate, const void* up,
                    long gu_pitch, const void* x, const void* norm_weights, float epsilon,
                    void* h, int n_inter, int k_in, int tokens);

#ifdef __cplusplus
}
#endif

#endif /* MUILLM_AMD_H */
