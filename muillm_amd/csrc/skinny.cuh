// Interface between the single-token GEMV entry points and the small-batch MFMA kernel.
#pragma once

#include "common.cuh"

namespace mui {

enum { WF_16BIT = 0, WF_I8_CHANNEL = 1, WF_U8_GROUP = 2 };
enum { SK_LINEAR = 0, SK_GATEUP = 1 };

struct SkinnyParams {
  const void* w0;       // linear: matrix; gate/up: gate rows
  const void* w1;       // gate/up: up rows
  long pitch;           // row pitch in weight elements
  const uint16_t* s0;   // I8_CHANNEL: scale of row n at s0[n*s_pitch]; U8_GROUP: pairs at s0 + n*s_pitch + 2g
  const uint16_t* s1;
  long s_pitch;
  int group_shift;
  const uint16_t* x;    // [tokens, k], token rows x_pitch elements apart (0: k)
  long x_pitch;         // honoured by the 1..4-token kernels (their K-segment calls); others need 0
  const uint16_t* gamma;
  const uint16_t* mul_bias;
  const uint16_t* add_bias;
  const uint16_t* residual;  // [tokens, n]
  uint16_t* y;               // [tokens, n]
  int n;       // outputs (weight rows, or gate/up pairs)
  int k;
  int tokens;  // 1..16
  float eps;
  void* workspace;         // optional scratch of the prompt GEMM (mui_linear_ws), zeroed once by the caller
  size_t workspace_bytes;
};

// Operands of the prompt GEMM (gemm_prefill.hip)
struct PrefillGemmParams {
  const uint8_t* w0;      // linear: matrix; gate/up: gate rows
  const uint8_t* w1;      // gate/up: up rows
  long pitch;             // weight row pitch in bytes
  const uint16_t* s0;     // per-channel int8: scale of row n at s0[n * s_pitch]; group format: (scale, min) pairs of row n at s0 + n * s_pitch + 2 g
  const uint16_t* s1;
  long s_pitch;
  int group_shift;        // group format: log2 of the codes per (scale, min) pair
  const uint16_t* x;      // [tokens, k] dense
  const uint16_t* gamma;
  const uint16_t* mul_bias;
  const uint16_t* add_bias;
  const uint16_t* residual;  // [tokens, n] dense
  uint16_t* y;               // [tokens, n]: row pitch y_pitch elements (n unless the launch covers a band of the outputs)
  long y_pitch;              // (the residual has the same pitch)
  int n;        // outputs (weight rows; gate/up pairs)
  int k;
  int tokens;
  float eps;
  int n_tiles;  // row tiles
  int t_tiles;  // token tiles
  // K split over workgroups (prefill_gemm_kernel<..., XS = true>): partial tiles and arrival counters
  int k_splits;
  int row_split;          // the XCDs divide the tile grid row_split ways by rows, 8 / row_split ways by tokens
  int row_group;          // row tiles per panel of an XCD's tile walk
  int total_blocks;       // software-pipelined tiles: tiles of the launch (row tiles rounded up to 8, times token tiles)
  float* part;            // [tiles * k_splits] partial tiles in fp32
  unsigned* part_count;   // [tiles], zero between launches
};

// B operand of one k-chunk: gamma * x rounded to the 16-bit type, sum of squares on the side.
// fp16: packed multiply (one rounding, same result as the fp32 product rounded once) and a
// packed dot for the squares.
template <typename T, bool NORM>
__device__ __forceinline__ u32x4 make_b(const u32x4 xv, const u32x4 gv, float& ss) {
  if constexpr (!NORM) {
    return xv;
  } else if constexpr (T::kDtype == MUI_DTYPE_F16) {
    const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f16x2 xx = __builtin_bit_cast(f16x2, xw[i]);
      ss = __builtin_amdgcn_fdot2(xx, xx, ss, false);
      o[i] = __builtin_bit_cast(uint32_t, xx * __builtin_bit_cast(f16x2, gw[i]));
    }
    u32x4 b = {o[0], o[1], o[2], o[3]};
    return b;
  } else {
    float xf[8], gf[8], o[8];
    unpack8<T>(xv, xf);
    unpack8<T>(gv, gf);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ss = fmaf(xf[i], xf[i], ss);
      o[i] = xf[i] * gf[i];
    }
    return pack8<T>(o);
  }
}

// v_mfma_f32_16x16x32: A = 16 rows x 32 k, B = 32 k x 16 columns; lane l supplies 8 k-values
// (k-chunk l / 16 of the step) of row / column l % 16
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T>
__device__ __forceinline__ f32x4 mfma16x16x32(u32x4 a, u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16x16x32<F16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16x16x32<BF16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// 8 int8/uint8 weights (two dwords) -> the 16-bit MFMA operand.
//   per-channel: exact integers (the row scale is applied in the epilogue). For fp16 the bytes
//   are dropped into the mantissa of 1024.0 (0x6400 | b = 1024 + b) with two byte permutes and
//   the offset is removed with a packed subtract: 5 VALU ops per dword instead of a convert
//   and a pack per weight.
//   group format: u8 * scale + min, rounded once to the 16-bit type.
template <typename T, int WF>
__device__ __forceinline__ u32x4 convert_a(uint32_t w0, uint32_t w1, const uint16_t* srow, int elem, int group_shift) {
  const uint32_t v[2] = {w0, w1};
  if constexpr (WF == WF_I8_CHANNEL && T::kDtype == MUI_DTYPE_F16) {
    u32x4 out;
    const f16x2 off = {(_Float16)1152.f, (_Float16)1152.f};  // 1024 + 128 (sign bit flipped below)
    uint32_t o[4];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const uint32_t u = v[m] ^ 0x80808080u;
      const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
      const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
      o[2 * m + 0] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, lo) - off);
      o[2 * m + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, hi) - off);
    }
    out.x = o[0]; out.y = o[1]; out.z = o[2]; out.w = o[3];
    return out;
  } else {
    float f[8];
    if constexpr (WF == WF_I8_CHANNEL) {
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int b = 0; b < 4; ++b) f[4 * m + b] = (float)(int)(int8_t)((v[m] >> (8 * b)) & 0xffu);
    } else {
      const uint32_t pr = ld4(srow + 2 * (elem >> group_shift));
      const float sc = T::lo(pr), mn = T::hi(pr);
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int b = 0; b < 4; ++b) f[4 * m + b] = fmaf((float)((v[m] >> (8 * b)) & 0xffu), sc, mn);
    }
    return pack8<T>(f);
  }
}

// group format with the (scale, min) pair already in a register: u8 * scale + min, rounded once
template <typename T>
__device__ __forceinline__ u32x4 convert_a_pair(uint32_t w0, uint32_t w1, uint32_t pair) {
  const uint32_t v[2] = {w0, w1};
  const float sc = T::lo(pair), mn = T::hi(pair);
  float f[8];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int b = 0; b < 4; ++b) f[4 * m + b] = fmaf((float)((v[m] >> (8 * b)) & 0xffu), sc, mn);
  return pack8<T>(f);
}

// tiled matrix-core GEMM for prompts (gemm_prefill.hip): any token count, 16-bit weights or int8 codes of either format
int launch_prefill_gemm(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
size_t prefill_workspace_bytes();  // what SkinnyParams::workspace must hold for the prompt GEMM to use it
// 17..128 tokens: 16 weight rows per workgroup, K split over its waves, token columns in up to 8 MFMA tiles (gemm_wide.hip)
int launch_gemm_wide(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
// launches gemm_skinny_kernel<dtype, weight format, epilogue>; returns a MUI_* status
int launch_skinny(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
// experiments: 0 disables the B-stationary persistent variant
void skinny_set_bstat(int on);
void skinny_set_lt(int on);  // 0: operands loaded straight from HBM in MFMA order (older kernels)

// 1..8 tokens, 16-bit weights: the single-token GEMV structure with the token operands packed
// in registers (gemv_multi.hip); returns MUI_ERR_UNSUPPORTED for shapes it does not cover
int launch_gemv_multi(hipStream_t s, int dtype, int epilogue, const SkinnyParams& p);
void gemv_multi_set_two(int min_passes);  // fewest row groups per workgroup for its two-set variant (0: never)
// MFMA skinny GEMM whose weight rows are read as contiguous runs and turned into operands
// through wave-private LDS (gemm_skinny_lt.hip); MUI_ERR_UNSUPPORTED for shapes it does not cover
int launch_skinny_lt(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
int int8_tuned_wgs_per_cu();  // mui_tune_int8's workgroups-per-CU override (0 = built-in)
int int8_tuned_rows();        // mui_tune_int8's rows-per-group override (0 = built-in)
int gemv_tuned_wgs_per_cu();  // mui_tune_gemv's workgroups-per-CU override (0 = built-in)
// 2..4 tokens, int8 weights, fp16 activations (int8_multi.hip); same contract
int launch_int8_multi(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
void skinny_set_int8_multi(int on);
// 1..4 tokens, int8 weights, fp16 activations on the 4 x 4 x 4 matrix instruction (int8_quad.hip); same contract
int launch_int8_quad(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
void int8_set_packed_dot(bool on);  // int8.hip: single fp16 token through int8_multi.hip

}  // namespace mui
