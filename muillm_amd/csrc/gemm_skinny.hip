// Small-batch (2..8 tokens) variants of the fused linears as skinny GEMMs on the matrix cores.
//
// The reference has no kernel for this case: anything but a single token falls back to an
// RMSNorm kernel + torch matmul + residual add (csrc/modules/linear_module.cpp:57-79,
// muillm/modules/gateupdownmlp.py:343-359). Here the weights are still streamed exactly
// once; the token batch rides along as the N dimension of v_mfma_f32_16x16x32 (padded to 16
// columns: the kernel stays HBM-bound, the MFMA pipe is <10 % busy at 8 tokens).
//
//   workgroup = 8 wave64s, one tile of 16 weight rows; the K range is split over the waves.
//   A operand  = weights: lane l loads 16 bytes of row (l % 16) at k-chunk (l / 16) of the
//                step, straight from HBM (non-temporal). int8 weights are converted to the
//                16-bit type in registers (per-channel: exact integers, scale applied in the
//                epilogue; group format: u8*scale+min rounded once to the 16-bit type).
//   B operand  = gamma * x of token (l % 16), same k-chunk, built on the fly from L2-resident
//                x and gamma (rounded to the 16-bit type like HF's normalised activations);
//                lanes of tokens >= batch feed zeros. sum(x^2) per token is accumulated by the
//                same lanes; rsqrt(mean + eps) is applied to the finished dot products.
//   C          = 16 rows x 16 tokens fp32 per wave; the 8 partial tiles are summed through LDS
//                and the epilogue (mul/add bias, residual, or SiLU(gate)*up on row pairs) writes
//                the 16-bit outputs.
// Because A and B label k identically (chunk index = lane / 16), the result does not depend
// on how the hardware orders k inside the instruction.
#include "skinny.cuh"

namespace mui {

constexpr int kSkWaves = 8;
constexpr int kSkThreads = kSkWaves * kWave;
constexpr int kSkUnroll = 8;  // 16-byte weight loads in flight per lane

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

// 8 weights of a chunk -> the 16-bit MFMA operand
template <typename T, int WF>
__device__ __forceinline__ u32x4 make_a(const void* rp, int chunk, const uint16_t* srow, int group_shift) {
  if constexpr (WF == WF_16BIT) {
    return ld16_stream((const uint16_t*)rp + (chunk << 3));
  } else {
    const u32x2 raw = ld8_stream((const uint8_t*)rp + (chunk << 3));
    float f[8];
    const uint32_t v[2] = {raw.x, raw.y};
    if constexpr (WF == WF_I8_CHANNEL) {
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int b = 0; b < 4; ++b) f[4 * m + b] = (float)(int)(int8_t)((v[m] >> (8 * b)) & 0xffu);
    } else {
      const uint32_t pr = *(const uint32_t*)(srow + 2 * ((chunk << 3) >> group_shift));
      const float sc = T::lo(pr), mn = T::hi(pr);
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int b = 0; b < 4; ++b) f[4 * m + b] = fmaf((float)((v[m] >> (8 * b)) & 0xffu), sc, mn);
    }
    return pack8<T>(f);
  }
}

template <typename T, int WF, bool NORM, int EPI>
__global__ void __launch_bounds__(kSkThreads) gemm_skinny_kernel(const SkinnyParams p) {
  __shared__ float tile[kSkWaves][16][17];
  __shared__ float ss_part[kSkWaves][kWave];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int r16 = lane & 15;  // A: row of the tile; B: token
  const int g = lane >> 4;    // k-chunk within a step
  const int tile_idx = blockIdx.x;

  // physical weight row behind tile row r16
  int out_row;
  const void* wbase;
  const uint16_t* sbase;
  if constexpr (EPI == SK_GATEUP) {
    out_row = tile_idx * 8 + (r16 >> 1);
    wbase = (r16 & 1) ? p.w1 : p.w0;
    sbase = (r16 & 1) ? p.s1 : p.s0;
  } else {
    out_row = tile_idx * 16 + r16;
    wbase = p.w0;
    sbase = p.s0;
  }
  const int row_c = out_row < p.n ? out_row : p.n - 1;
  constexpr int kWBytes = (WF == WF_16BIT) ? 2 : 1;
  const void* rp = (const char*)wbase + (long)row_c * p.pitch * kWBytes;
  const uint16_t* srow = (WF == WF_U8_GROUP) ? sbase + (long)row_c * p.s_pitch : nullptr;

  const int kc = p.k >> 3;                       // 8-element chunks per row
  const int steps = (kc + 3) >> 2;               // MFMA steps over the whole K
  const int per_wave = (steps + kSkWaves - 1) / kSkWaves;
  const int s_begin = wave * per_wave;
  const int s_end = (s_begin + per_wave) < steps ? (s_begin + per_wave) : steps;

  const bool tok_ok = r16 < p.tokens;
  const uint16_t* xrow = p.x + (long)(tok_ok ? r16 : 0) * p.k;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float ss = 0.f;

  for (int s0 = s_begin; s0 < s_end; s0 += kSkUnroll) {
    u32x4 a[kSkUnroll];
    u32x4 xv[kSkUnroll];
    u32x4 gv[kSkUnroll];
    bool ok[kSkUnroll];
#pragma unroll
    for (int u = 0; u < kSkUnroll; ++u) {
      const int chunk = ((s0 + u) << 2) + g;
      ok[u] = (s0 + u) < s_end && chunk < kc;
      const int cc = ok[u] ? chunk : 0;
      a[u] = make_a<T, WF>(rp, cc, srow, p.group_shift);
      xv[u] = ld16(xrow + (cc << 3));
      if constexpr (NORM) gv[u] = ld16(p.gamma + (cc << 3));
    }
#pragma unroll
    for (int u = 0; u < kSkUnroll; ++u) {
      u32x4 b = {0u, 0u, 0u, 0u};
      if (ok[u] && tok_ok) {
        if constexpr (NORM) {
          float xf[8], gf[8], o[8];
          unpack8<T>(xv[u], xf);
          unpack8<T>(gv[u], gf);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            ss = fmaf(xf[i], xf[i], ss);
            o[i] = xf[i] * gf[i];
          }
          b = pack8<T>(o);
        } else {
          b = xv[u];
        }
      }
      if (!ok[u]) a[u] = b;  // a clamped chunk must not contribute: b is zero there
      acc = mfma16x16x32<T>(a[u], b, acc);
    }
  }

  // C layout of the 16x16 tile: lane holds column (lane % 16) = token, rows 4*(lane/16)+r
#pragma unroll
  for (int r = 0; r < 4; ++r) tile[wave][4 * g + r][r16] = acc[r];
  if constexpr (NORM) ss_part[wave][lane] = ss;
  __syncthreads();

  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  if (t < OUT * 16) {
    const int i = t >> 4;   // output index inside the tile
    const int j = t & 15;   // token
    const int n = tile_idx * OUT + i;
    if (j < p.tokens && n < p.n) {
      float rs = 1.f;
      if constexpr (NORM) {
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < kSkWaves; ++w)
          tot += (ss_part[w][j] + ss_part[w][j + 16]) + (ss_part[w][j + 32] + ss_part[w][j + 48]);
        rs = rsqrtf(tot / (float)p.k + p.eps);
      }
      auto total = [&](int row) {
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kSkWaves; ++w) v += tile[w][row][j];
        return v;
      };
      float v;
      if constexpr (EPI == SK_GATEUP) {
        float gt = total(2 * i) * rs, up = total(2 * i + 1) * rs;
        if constexpr (WF == WF_I8_CHANNEL) {
          gt *= T::one(p.s0[(long)n * p.s_pitch]);
          up *= T::one(p.s1[(long)n * p.s_pitch]);
        }
        v = silu_f32(gt) * up;
      } else {
        v = total(i) * rs;
        if constexpr (WF == WF_I8_CHANNEL) v *= T::one(p.s0[(long)n * p.s_pitch]);
        if (p.mul_bias) v *= T::one(p.mul_bias[n]);
        if (p.add_bias) v += T::one(p.add_bias[n]);
        if (p.residual) v += T::one(p.residual[(long)j * p.n + n]);
      }
      p.y[(long)j * p.n + n] = T::pack(v);
    }
  }
}

template <typename T, int WF, int EPI>
static int launch_skinny_t(hipStream_t s, const SkinnyParams& p) {
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  const int grid = ceil_div(p.n, OUT);
  if (p.gamma)
    hipLaunchKernelGGL((gemm_skinny_kernel<T, WF, true, EPI>), dim3(grid), dim3(kSkThreads), 0, s, p);
  else
    hipLaunchKernelGGL((gemm_skinny_kernel<T, WF, false, EPI>), dim3(grid), dim3(kSkThreads), 0, s, p);
  return launch_status();
}

// entry used by gemv.hip / int8.hip for tokens >= 2
int launch_skinny(hipStream_t s, int dtype, int wf, int epi, const SkinnyParams& p) {
#define MUI_SK_CASE(TT, WFV, EPIV) \
  if (wf == WFV && epi == EPIV) return launch_skinny_t<TT, WFV, EPIV>(s, p);
  if (dtype == MUI_DTYPE_F16) {
    MUI_SK_CASE(F16, WF_16BIT, SK_LINEAR)
    MUI_SK_CASE(F16, WF_16BIT, SK_GATEUP)
    MUI_SK_CASE(F16, WF_I8_CHANNEL, SK_LINEAR)
    MUI_SK_CASE(F16, WF_I8_CHANNEL, SK_GATEUP)
    MUI_SK_CASE(F16, WF_U8_GROUP, SK_LINEAR)
    MUI_SK_CASE(F16, WF_U8_GROUP, SK_GATEUP)
  } else if (dtype == MUI_DTYPE_BF16) {
    MUI_SK_CASE(BF16, WF_16BIT, SK_LINEAR)
    MUI_SK_CASE(BF16, WF_16BIT, SK_GATEUP)
    MUI_SK_CASE(BF16, WF_I8_CHANNEL, SK_LINEAR)
    MUI_SK_CASE(BF16, WF_I8_CHANNEL, SK_GATEUP)
    MUI_SK_CASE(BF16, WF_U8_GROUP, SK_LINEAR)
    MUI_SK_CASE(BF16, WF_U8_GROUP, SK_GATEUP)
  }
#undef MUI_SK_CASE
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui
