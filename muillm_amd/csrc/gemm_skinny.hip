// Small-batch (2..16 tokens) variants of the fused linears as skinny GEMMs on the matrix cores,
// operands loaded in MFMA order straight from memory. Serves the 8-bit weight formats (whose
// conversion happens in operand layout); 16-bit weights take gemm_skinny_lt.hip first, which
// reads contiguous row runs and reorders them through LDS.
//
// The reference has no kernel for this case: anything but a single token falls back to an
// RMSNorm kernel + torch matmul + residual add (csrc/modules/linear_module.cpp:57-79,
// muillm/modules/gateupdownmlp.py:343-359). Here the weights are still streamed exactly
// once; the token batch rides along as the N dimension of v_mfma_f32_16x16x32 (padded to 16
// columns: the kernel stays HBM-bound, the MFMA pipe is <10 % busy at 8 tokens).
//
//   workgroup = 8 wave64s, one tile of 16 weight rows; the K range is split over the waves.
//   A operand  = weights: lane l loads 16 bytes of row (l % 16) at position (l / 16) of the
//                step, straight from HBM (non-temporal): one k-chunk of 8 16-bit weights, or
//                two k-chunks of 8-bit weights (two MFMAs), converted to the 16-bit type in
//                registers (per-channel: exact integers, scale applied in the epilogue;
//                group format: u8*scale+min rounded once to the 16-bit type).
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

  // A lane reads 16 bytes of its weight row per step: one 8-element k-chunk of 16-bit weights
  // or two of 8-bit weights (two MFMAs). A and B label k identically, so any k order works.
  constexpr int CPL = (WF == WF_16BIT) ? 1 : 2;  // k-chunks per lane and step
  constexpr int UNR = (WF == WF_16BIT) ? kSkUnroll : kSkUnroll / 2;
  const int kcl = p.k / (8 * CPL);               // lane-chunks per row
  const int steps = (kcl + 3) >> 2;
  const int per_wave = (steps + kSkWaves - 1) / kSkWaves;
  const int s_begin = wave * per_wave;
  const int s_end = (s_begin + per_wave) < steps ? (s_begin + per_wave) : steps;

  const bool tok_ok = r16 < p.tokens;
  const uint16_t* xrow = p.x + (long)(tok_ok ? r16 : 0) * p.k;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float ss = 0.f;

  // batches of UNR steps; without gamma two register sets: the next batch is in flight while
  // this one is used
  struct Batch {
    u32x4 a[UNR];
    u32x4 xv[UNR][CPL];
    u32x4 gv[UNR][CPL];
    bool ok[UNR];
    int cidx[UNR];
  };
  auto load_batch = [&](int s0, Batch& q) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int chunk = ((s0 + u) << 2) + g;
      q.ok[u] = (s0 + u) < s_end && chunk < kcl;
      const int cc = q.ok[u] ? chunk : 0;
      q.cidx[u] = cc;
      q.a[u] = ld16_stream((const char*)rp + ((long)cc << 4));
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        q.xv[u][c] = ld16(xrow + ((cc * CPL + c) << 3));
        if constexpr (NORM) q.gv[u][c] = ld16(p.gamma + ((cc * CPL + c) << 3));
      }
    }
  };
  auto use_batch = [&](const Batch& q) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        u32x4 b = {0u, 0u, 0u, 0u};
        if (q.ok[u] && tok_ok) b = make_b<T, NORM>(q.xv[u][c], q.gv[u][c], ss);
        u32x4 av;
        if constexpr (WF == WF_16BIT) {
          av = q.a[u];
        } else {
          av = convert_a<T, WF>(c == 0 ? q.a[u].x : q.a[u].z, c == 0 ? q.a[u].y : q.a[u].w, srow,
                                (q.cidx[u] * CPL + c) << 3, p.group_shift);
        }
        if (!q.ok[u]) av = b;  // a clamped chunk must not contribute: b is zero there
        acc = mfma16x16x32<T>(av, b, acc);
      }
    }
  };
  if constexpr (NORM) {
    // gamma doubles the registers of a batch: one set (measured faster than two here)
    Batch qa;
    for (int s0 = s_begin; s0 < s_end; s0 += UNR) {
      load_batch(s0, qa);
      use_batch(qa);
    }
  } else {
    Batch qa, qb;
    int s0 = s_begin;
    if (s0 < s_end) load_batch(s0, qa);
    while (s0 < s_end) {
      const int s1 = s0 + UNR;
      if (s1 < s_end) load_batch(s1, qb);
      use_batch(qa);
      if (s1 >= s_end) break;
      s0 = s1 + UNR;
      if (s0 < s_end) load_batch(s0, qa);
      use_batch(qb);
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

// ---------------------------------------------------------------------------------------
// B-stationary variant for K <= 4096: persistent workgroups, one per CU. Wave w always owns
// the same K range, so its B operands (gamma * x of the 16 token columns) are built ONCE and
// stay in registers while the workgroup walks over its weight tiles; the inner loop is weight
// loads + MFMAs only, and the next tile's weights are requested before the current tile is
// reduced (two register sets), so the HBM stream never drains between tiles. (Parking B in LDS
// to afford a third weight register set was measured slower: 54 vs 46 us on the gate/up shape.)
// ---------------------------------------------------------------------------------------
constexpr int kBsSteps = 16;  // MFMA steps (32 k-values each) per wave: K <= 8 * 16 * 32

template <typename T, int WF, bool NORM, int EPI, bool FULL>
__global__ void __launch_bounds__(kSkThreads) gemm_skinny_bstat_kernel(const SkinnyParams p, int n_tiles) {
  constexpr int CPL = (WF == WF_16BIT) ? 1 : 2;   // k-chunks (8 values) per 16-byte weight load
  constexpr int LCH = kBsSteps / CPL;             // 16-byte weight loads per lane and tile
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  constexpr int kWBytes = (WF == WF_16BIT) ? 2 : 1;
  __shared__ float tile[2][kSkWaves][16][17];
  __shared__ float ss_part[kSkWaves][kWave];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int r16 = lane & 15;
  const int g = lane >> 4;

  // K is a multiple of 32 lane-chunks (launcher): every wave owns jmax consecutive steps, and
  // 16-byte lane-chunk j of this lane is chunk lc0 + 4 * j of the row (a contiguous run per wave)
  // FULL: K is exactly 8 waves x 16 steps (4096), no step is ever skipped
  const int jmax = FULL ? LCH : ((p.k / (8 * CPL)) >> 5);
  const int lc0 = ((wave * jmax) << 2) + g;

  // ---- B operands, once ----
  const bool tok_ok = r16 < p.tokens;
  const uint16_t* xrow = p.x + (long)(tok_ok ? r16 : 0) * p.k;
  u32x4 bq[LCH][CPL];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < LCH; ++j) {
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      u32x4 b = {0u, 0u, 0u, 0u};
      if ((FULL || j < jmax) && tok_ok) {
        const int e = ((lc0 + 4 * j) * CPL + c) << 3;
        const u32x4 xv = ld16(xrow + e);
        u32x4 gv = xv;
        if constexpr (NORM) gv = ld16(p.gamma + e);
        b = make_b<T, NORM>(xv, gv, ss);
      }
      bq[j][c] = b;
    }
  }
  if constexpr (NORM) ss_part[wave][lane] = ss;

  auto row_ptr = [&](int tile_idx, const uint16_t*& srow) -> const char* {
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
    srow = (WF == WF_U8_GROUP) ? sbase + (long)row_c * p.s_pitch : nullptr;
    return (const char*)wbase + (long)row_c * p.pitch * kWBytes;
  };
  auto issue = [&](int tile_idx, u32x4 (&a)[LCH], const uint16_t*& srow) {
    const char* rp = row_ptr(tile_idx, srow) + (lc0 << 4);
#pragma unroll
    for (int j = 0; j < LCH; ++j)
      if (FULL || j < jmax) a[j] = ld16_stream(rp + (j << 6));
  };
  auto consume = [&](int tile_idx, const u32x4 (&a)[LCH], const uint16_t* srow, int buf) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < LCH; ++j) {
      if (FULL || j < jmax) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          u32x4 av;
          if constexpr (WF == WF_16BIT) {
            av = a[j];
          } else {
            av = convert_a<T, WF>(c == 0 ? a[j].x : a[j].z, c == 0 ? a[j].y : a[j].w, srow,
                                  ((lc0 + 4 * j) * CPL + c) << 3, p.group_shift);
          }
          acc = mfma16x16x32<T>(av, bq[j][c], acc);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) tile[buf][wave][4 * g + r][r16] = acc[r];
  };
  auto epilogue = [&](int tile_idx, int buf) {
    if (t < OUT * 16) {
      const int i = t >> 4;
      const int j = t & 15;
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
          for (int w = 0; w < kSkWaves; ++w) v += tile[buf][w][row][j];
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
  };

  // ---- tiles blockIdx.x, blockIdx.x + gridDim.x, ...; two register sets ----
  u32x4 a0[LCH], a1[LCH];
  const uint16_t* sr0 = nullptr;
  const uint16_t* sr1 = nullptr;
  int tl = blockIdx.x;
  if (tl < n_tiles) issue(tl, a0, sr0);
  while (tl < n_tiles) {
    const int t1 = tl + gridDim.x;
    if (t1 < n_tiles) issue(t1, a1, sr1);
    consume(tl, a0, sr0, 0);
    __syncthreads();
    epilogue(tl, 0);
    if (t1 >= n_tiles) break;
    const int t2 = t1 + gridDim.x;
    if (t2 < n_tiles) issue(t2, a0, sr0);
    consume(t1, a1, sr1, 1);
    __syncthreads();
    epilogue(t1, 1);
    tl = t2;
  }
}

static int g_skinny_bstat = 1;  // 0: always stream B (experiments)

template <typename T, int WF, int EPI>
static int launch_skinny_t(hipStream_t s, const SkinnyParams& p) {
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  const int n_tiles = ceil_div(p.n, OUT);
  constexpr int kGran = 256 * ((WF == WF_16BIT) ? 1 : 2);  // K covered by one lane-chunk index
  if (g_skinny_bstat && p.k <= kSkWaves * kBsSteps * 32 && p.k % kGran == 0) {
    const int grid = balanced_grid(n_tiles, 1);
    const bool full = p.k == kSkWaves * kBsSteps * 32;
#define MUI_BSTAT(NORMV, FULLV) \
  hipLaunchKernelGGL((gemm_skinny_bstat_kernel<T, WF, NORMV, EPI, FULLV>), dim3(grid), dim3(kSkThreads), 0, s, p, n_tiles)
    if (p.gamma) { if (full) MUI_BSTAT(true, true); else MUI_BSTAT(true, false); }
    else { if (full) MUI_BSTAT(false, true); else MUI_BSTAT(false, false); }
#undef MUI_BSTAT
    return launch_status();
  }
  if (p.gamma)
    hipLaunchKernelGGL((gemm_skinny_kernel<T, WF, true, EPI>), dim3(n_tiles), dim3(kSkThreads), 0, s, p);
  else
    hipLaunchKernelGGL((gemm_skinny_kernel<T, WF, false, EPI>), dim3(n_tiles), dim3(kSkThreads), 0, s, p);
  return launch_status();
}

static int g_skinny_lt = 1;     // LDS-transposed operand kernel (gemm_skinny_lt.hip) first
void skinny_set_bstat(int on) { g_skinny_bstat = on; }
void skinny_set_lt(int on) { g_skinny_lt = on; }

static int g_int8_multi = 1;  // 2..4 tokens of int8 weights: vector-ALU kernel (int8_multi.hip) first
void skinny_set_int8_multi(int on) { g_int8_multi = on; }

// entry used by gemv.hip / int8.hip for tokens >= 2
int launch_skinny(hipStream_t s, int dtype, int wf, int epi, const SkinnyParams& p) {
  // int8 at 2-4 tokens with fp16 activations: the 4 x 4 x 4 matrix-instruction kernel (int8_quad.hip:
  // QKV 6144 x 4096 at 4 tokens 7.6 us against 9.0 us on the vector ALUs, gate/up 2 x 14336 x 4096
  // 20.5 us against 22.9 us on the kernel below). What it declines (one token, bf16, the group format
  // up to two tokens, rows longer than 14336):
  // the vector-ALU kernel, except at 3-4 tokens long rows (down 4096 x
  // 14336 at 4 tokens: 13.6 vs 16.4 us) and tall gate/up matrices (2 x 14336 x 4096: a steady
  // 27 us against 27-34 us), where the matrix-core kernel measured faster -- with per-channel
  // scales and, for fp16 activations, with the reference's groups of 128 codes or more, which that
  // kernel scales once per group (gate/up at 4 tokens 24.3 vs 29.4 us, down 16.7 vs 18.9 us); smaller
  // groups and bf16 convert code by code there and stay on the vector-ALU kernel
  const bool lt_format = wf == WF_I8_CHANNEL || (wf == WF_U8_GROUP && p.group_shift >= 7 && dtype == MUI_DTYPE_F16);
  const bool lt_first = g_skinny_lt && lt_format && p.tokens >= 3 &&
                        (p.k > 8192 || (epi == SK_GATEUP && p.n >= 8192));
  if (wf != WF_16BIT && p.tokens <= 4) {
    const int st = launch_int8_quad(s, dtype, wf, epi, p);
    if (st != MUI_ERR_UNSUPPORTED) return st;
  }
  if (wf != WF_16BIT && g_int8_multi && p.tokens <= 4 && !lt_first) {
    const int st = launch_int8_multi(s, dtype, wf, epi, p);
    if (st != MUI_ERR_UNSUPPORTED) return st;
  }
  if (g_skinny_lt) {
    const int st = launch_skinny_lt(s, dtype, wf, epi, p);
    if (st != MUI_ERR_UNSUPPORTED) return st;
  }
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
