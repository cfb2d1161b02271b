// Fused linears for 1..2 tokens (3..4 and, on tall matrices, up to 8 on request) with 16-bit
// weights: the single-token GEMV structure (256 threads, thread t owns 16-byte chunks t, t+256, ...
// of every row, R rows in flight, next row group requested before the reduction, persistent
// balanced grid) with the token operands gamma * x packed 16-bit in registers and one packed dot
// (v_dot2_f32_f16) per two weights and token. The weights are streamed exactly once. From 3
// tokens on the matrix-core skinny GEMM (gemm_skinny_lt.hip) is the default: it measured 0.2-1 us
// per call faster there once it brought in only 8 token rows for up to 8 tokens.
//
// The reference has no kernel for this case (csrc/modules/linear_module.cpp:57-79 falls back to
// RMSNorm + torch matmul + add; muillm/modules/gateupdownmlp.py:343-359).
#include "skinny.cuh"

namespace mui {

constexpr int kMtThreads = 256;
constexpr int kMtWaves = kMtThreads / kWave;

template <typename T>
__device__ __forceinline__ float dot2_mt(uint32_t a, uint32_t b, float c);
template <>
__device__ __forceinline__ float dot2_mt<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}
typedef __bf16 bf16x2_mt __attribute__((ext_vector_type(2)));
template <>
__device__ __forceinline__ float dot2_mt<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_mt, a), __builtin_bit_cast(bf16x2_mt, b), c, false);
}

// TWO (one token, work lists of several row groups per workgroup -- the lm_head): two register
// sets; the weights of group i + 2 are requested as soon as group i has been multiplied, so a
// workgroup always has a whole group in flight while it reduces, synchronises and stores.
template <typename T, int R, int CH, bool NORM, int EPI, int TOK, bool TWO = false>
__global__ void __launch_bounds__(kMtThreads) gemv_multi_kernel(
    // scalars, hottest first (preloaded into SGPRs at wave launch)
    const uint16_t* w0, const uint16_t* w1, long pitch, const uint16_t* x, const uint16_t* gamma,
    uint16_t* y, int n, int k, int tokens, int x_pitch, float eps, const uint16_t* residual,
    const uint16_t* mul_bias, const uint16_t* add_bias) {
  constexpr int OUT = (EPI == SK_GATEUP) ? R / 2 : R;
  static_assert(EPI != SK_GATEUP || (R % 2 == 0), "gate/up needs row pairs");
  static_assert(16 * OUT * TOK <= kMtThreads, "sixteen epilogue lanes per output");
  constexpr int NV = R * TOK;  // partial sums per row group: value r * TOK + token
  __shared__ float red[2][kMtWaves * 4][NV];  // [buffer][wave * 4 + 16-lane row][value]
  __shared__ float red_ss[kMtWaves][TOK];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int kc = k >> 3;
  const int n_groups = (n + OUT - 1) / OUT;

  int coff[CH];
  bool cvalid[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = t + kMtThreads * j;
    cvalid[j] = c < kc;
    coff[j] = cvalid[j] ? (c << 3) : 0;
  }

  constexpr int NSET = TWO ? 2 : 1;
  struct Set {
    u32x4 w[R][CH];
    uint32_t res;  // residual (16-bit pattern) that belongs to the weights in w
  };
  Set sets[NSET];
#pragma unroll
  for (int u = 0; u < NSET; ++u) sets[u].res = 0;
  auto issue_w = [&](Set& st, int rg) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row;
      const uint16_t* base;
      if constexpr (EPI == SK_GATEUP) {
        row = rg * OUT + (r >> 1);
        base = (r & 1) ? w1 : w0;
      } else {
        row = rg * R + r;
        base = w0;
      }
      row = row < n ? row : n - 1;
      const uint16_t* rp = base + (long)row * pitch;
#pragma unroll
      for (int j = 0; j < CH; ++j) st.w[r][j] = ld16_stream(rp + coff[j]);
    }
  };
  // the residual value of a group's epilogue thread rides along with the weights: loaded inside
  // the epilogue it would add a memory round trip to the end of the kernel. With two sets every
  // thread requests it, from a clamped address: behind a branch the compiler could no longer count
  // the loads in flight and would wait for the other set's weights as well.
  auto issue_res = [&](Set& st, int rg) {
    if constexpr (EPI == SK_LINEAR) {
      // (the epilogue's finishing thread of output o, token tk is thread 16 * (o * TOK + tk))
      if constexpr (TWO) {
        int row = rg * OUT + ((t >> 4) / TOK < OUT ? (t >> 4) / TOK : OUT - 1);
        row = row < n ? row : n - 1;
        st.res = ld2(residual ? residual + row : x);
      } else {
        if (residual && (t & 15) == 0 && (t >> 4) < OUT * TOK) {
          const int row = rg * OUT + (t >> 4) / TOK, tk = (t >> 4) % TOK;
          if (row < n && tk < tokens) st.res = ld2(residual + (long)tk * n + row);
        }
      }
    }
  };
  // ---- token operands: gamma * x rounded once to the 16-bit type (zero past the row / batch).
  // They are requested before the first weights: loads return in order, so the operand
  // preparation (and a fused norm's reduction) then overlaps the flight of the first row group
  // instead of following it (measured on one device against weights-first, one token: C1 7.6 ->
  // 7.1 us, down 19.0 -> 18.7 us, o_proj 6.9 -> 6.8 us, QKV 9.3 -> 9.4 us). No load sits behind a
  // branch (clamped addresses, dead lanes zeroed by selects), and the first token's addresses
  // depend only on arguments that arrive preloaded in SGPRs.
  int rg = blockIdx.x;  // the grid never exceeds the number of row groups
  u32x4 xq[TOK][CH];
  u32x4 gq[CH];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    // (token 0 needs no arithmetic: its loads depend on nothing but preloaded arguments)
    const long xrow = tk == 0 ? 0 : (long)(tk < tokens ? tk : tokens - 1) * x_pitch;
#pragma unroll
    for (int j = 0; j < CH; ++j) xq[tk][j] = ld16(x + xrow + coff[j]);
  }
  if constexpr (NORM) {
#pragma unroll
    for (int j = 0; j < CH; ++j) gq[j] = ld16(gamma + coff[j]);
  }
  issue_w(sets[0], rg);
  issue_res(sets[0], rg);
  // group i of this workgroup is blockIdx.x + i * gridDim.x
  const int n_my = (n_groups - 1 - (int)blockIdx.x) / (int)gridDim.x + 1;
  auto group_of = [&](int i) -> int { return blockIdx.x + i * gridDim.x; };
  if constexpr (TWO) {
    // (a workgroup of a ragged grid that has a single group requests it twice)
    issue_w(sets[1], group_of(n_my > 1 ? 1 : 0));
    issue_res(sets[1], group_of(n_my > 1 ? 1 : 0));
  }

  float ss[TOK];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    ss[tk] = 0.f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const bool live = cvalid[j] && tk < tokens;
      float sq = 0.f;
      const u32x4 b = make_b<T, NORM>(xq[tk][j], NORM ? gq[j] : xq[tk][j], sq);
      const u32x4 zero = {0u, 0u, 0u, 0u};
      xq[tk][j] = live ? b : zero;
      ss[tk] += live ? sq : 0.f;
    }
  }
  float rs[TOK];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) rs[tk] = 1.f;
  if constexpr (NORM) {
#pragma unroll
    for (int tk = 0; tk < TOK; ++tk) {
      const float s = wave_sum(ss[tk]);
      if (lane == 0) red_ss[wave][tk] = s;
    }
    __syncthreads();
#pragma unroll
    for (int tk = 0; tk < TOK; ++tk) {
      const float tot = (red_ss[0][tk] + red_ss[1][tk]) + (red_ss[2][tk] + red_ss[3][tk]);
      rs[tk] = rsqrtf(tot / (float)k + eps);
    }
  }

  int buf = 0;
  if constexpr (!TWO) {
    // one register set: the next group is requested behind a (uniform) branch once the current one
    // has been multiplied. (Requested unconditionally, with the last pass peeled, the compiler gave
    // the refilled weights registers of their own and copied them back at the top of the loop: the
    // MLP at 2 tokens went from 56.6 to 70 us.)
    for (; rg < n_groups; rg += gridDim.x) {
      float acc[NV];
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int tk = 0; tk < TOK; ++tk) {
          float a = 0.f;
#pragma unroll
          for (int j = 0; j < CH; ++j) {
            a = dot2_mt<T>(sets[0].w[r][j].x, xq[tk][j].x, a);
            a = dot2_mt<T>(sets[0].w[r][j].y, xq[tk][j].y, a);
            a = dot2_mt<T>(sets[0].w[r][j].z, xq[tk][j].z, a);
            a = dot2_mt<T>(sets[0].w[r][j].w, xq[tk][j].w, a);
          }
          acc[r * TOK + tk] = a;
        }
      }
      const uint32_t res_cur = sets[0].res;
      const int nxt = rg + gridDim.x;
      if (nxt < n_groups) {  // keep the memory pipe full during the reduction
        issue_w(sets[0], nxt);
        issue_res(sets[0], nxt);
      }

      // all NV sums of a 16-lane row in one multi-value DPP reduction; the 16 row partials
      // (4 waves x 4 rows) are added by the epilogue threads
      row16_reduce_scatter<NV>(acc, lane);
      if ((lane & (16 / NV - 1)) == 0 || NV == 16) red[buf][t >> 4][(lane & 15) / (16 / NV)] = acc[0];
      __syncthreads();

      // sixteen lanes per output: each fetches one of the 16 row partials, a DPP butterfly adds them
      // (one thread adding all sixteen was a chain of sixteen dependent LDS reads at the end of the kernel)
      if (t < 16 * OUT * TOK) {
        const int part = t & 15, o = (t >> 4) / TOK, tk = (t >> 4) % TOK;
        const int row = rg * OUT + o;
        float v0 = row16_sum(red[buf][part][((EPI == SK_GATEUP) ? 2 * o : o) * TOK + tk]);
        float v1 = 0.f;
        if constexpr (EPI == SK_GATEUP) v1 = row16_sum(red[buf][part][(2 * o + 1) * TOK + tk]);
        if (part == 0 && row < n && tk < tokens) {
          float rsv = rs[0];
#pragma unroll
          for (int i = 1; i < TOK; ++i) rsv = (tk == i) ? rs[i] : rsv;
          float v;
          if constexpr (EPI == SK_GATEUP) {
            v = silu_f32(v0 * rsv) * (v1 * rsv);
          } else {
            v = v0 * rsv;
            if (mul_bias) v *= T::one(mul_bias[row]);
            if (add_bias) v += T::one(add_bias[row]);
            if (residual) v += T::one((uint16_t)res_cur);
          }
          y[(long)tk * n + row] = T::pack(v);
        }
      }
      buf ^= 1;
    }
  } else {
    // group `g` out of register set `st`; refill: the set is requested again for group `nxt` (its
    // weights once this group has been multiplied, the residual once the epilogue has used it)
    auto pass = [&](Set& st, int g, auto refill, int nxt) {
      float acc[NV];
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int tk = 0; tk < TOK; ++tk) {
          float a = 0.f;
#pragma unroll
          for (int j = 0; j < CH; ++j) {
            a = dot2_mt<T>(st.w[r][j].x, xq[tk][j].x, a);
            a = dot2_mt<T>(st.w[r][j].y, xq[tk][j].y, a);
            a = dot2_mt<T>(st.w[r][j].z, xq[tk][j].z, a);
            a = dot2_mt<T>(st.w[r][j].w, xq[tk][j].w, a);
          }
          acc[r * TOK + tk] = a;
        }
      }
      if constexpr (decltype(refill)::value) issue_w(st, nxt);  // keep the memory pipe full during the reduction

      // all NV sums of a 16-lane row in one multi-value DPP reduction; the 16 row partials
      // (4 waves x 4 rows) are added by the epilogue threads
      row16_reduce_scatter<NV>(acc, lane);
      if ((lane & (16 / NV - 1)) == 0 || NV == 16) red[buf][t >> 4][(lane & 15) / (16 / NV)] = acc[0];
      __syncthreads();

      if (t < 16 * OUT * TOK) {  // sixteen lanes per output, as above
        const int part = t & 15, o = (t >> 4) / TOK, tk = (t >> 4) % TOK;
        const int row = g * OUT + o;
        float v0 = row16_sum(red[buf][part][((EPI == SK_GATEUP) ? 2 * o : o) * TOK + tk]);
        float v1 = 0.f;
        if constexpr (EPI == SK_GATEUP) v1 = row16_sum(red[buf][part][(2 * o + 1) * TOK + tk]);
        if (part == 0 && row < n && tk < tokens) {
          float rsv = rs[0];
#pragma unroll
          for (int i = 1; i < TOK; ++i) rsv = (tk == i) ? rs[i] : rsv;
          float v;
          if constexpr (EPI == SK_GATEUP) {
            v = silu_f32(v0 * rsv) * (v1 * rsv);
          } else {
            v = v0 * rsv;
            if (mul_bias) v *= T::one(mul_bias[row]);
            if (add_bias) v += T::one(add_bias[row]);
            if (residual) v += T::one((uint16_t)st.res);
          }
          y[(long)tk * n + row] = T::pack(v);
        }
      }
      if constexpr (decltype(refill)::value) issue_res(st, nxt);
      buf ^= 1;
    };
    constexpr std::true_type kRefill{};
    constexpr std::false_type kLast{};
    // pairs of groups whose sets are both refilled, then the last one to three groups
    int i = 0;
    for (; i + 3 < n_my; i += 2) {
      pass(sets[0], group_of(i), kRefill, group_of(i + 2));
      pass(sets[1], group_of(i + 1), kRefill, group_of(i + 3));
    }
    const int rem = n_my - i;
    if (rem == 3) {
      pass(sets[0], group_of(i), kRefill, group_of(i + 2));
      pass(sets[1], group_of(i + 1), kLast, 0);
      pass(sets[0], group_of(i + 2), kLast, 0);
    } else if (rem == 2) {
      pass(sets[0], group_of(i), kLast, 0);
      pass(sets[1], group_of(i + 1), kLast, 0);
    } else {
      pass(sets[0], group_of(i), kLast, 0);
    }
  }
}

static int g_mt_two_min_passes = 4;  // fewest row groups per workgroup that take two register sets (0: never)
void gemv_multi_set_two(int min_passes) { g_mt_two_min_passes = min_passes; }

template <typename T, int R, int CH, int EPI, int TOK>
static int launch_mt_rc(hipStream_t s, const SkinnyParams& p, int grid) {
#define MUI_MT_LAUNCH(NORMV, TWOV)                                                                              \
  hipLaunchKernelGGL((gemv_multi_kernel<T, R, CH, NORMV, EPI, TOK, TWOV>), dim3(grid), dim3(kMtThreads), 0, s,  \
                     (const uint16_t*)p.w0, (const uint16_t*)p.w1, p.pitch, p.x, p.gamma, p.y, p.n, p.k,        \
                     p.tokens, (int)(p.x_pitch > 0 ? p.x_pitch : (long)p.k), p.eps, p.residual, p.mul_bias, p.add_bias)
  if constexpr (TOK == 1 && CH <= 2 && EPI == SK_LINEAR) {
    constexpr int OUT = R;
    if (g_mt_two_min_passes > 0 && ceil_div(p.n, OUT) >= (long)g_mt_two_min_passes * grid) {
      if (p.gamma) MUI_MT_LAUNCH(true, true); else MUI_MT_LAUNCH(false, true);
      return launch_status();
    }
  }
  if (p.gamma) MUI_MT_LAUNCH(true, false); else MUI_MT_LAUNCH(false, false);
#undef MUI_MT_LAUNCH
  return launch_status();
}

template <typename T, int EPI, int TOK>
static int launch_mt_t(hipStream_t s, const SkinnyParams& p) {
  const int ch = ceil_div(p.k >> 3, kMtThreads);
  if constexpr (TOK == 8) {
    // 8 tokens: 2 rows x 8 tokens = 16 partial sums per group; only rows of <= 2 chunks per thread
    // and only tall matrices. Opt-in (mui_tune_skinny): 43 us on the 2 x 14336 x 4096 gate/up
    // shape against 40 us for the matrix-core kernel of gemm_skinny_lt.hip
    if (ch > 2 || p.n < 8192) return MUI_ERR_UNSUPPORTED;
    constexpr int R = 2, OUT = (EPI == SK_GATEUP) ? 1 : 2;
    const int grid = balanced_grid(ceil_div(p.n, OUT), 4);
    if (ch <= 1) return launch_mt_rc<T, R, 1, EPI, TOK>(s, p, grid);
    return launch_mt_rc<T, R, 2, EPI, TOK>(s, p, grid);
  } else {
  if (ch <= 2) {
    constexpr int R = 4, OUT = (EPI == SK_GATEUP) ? 2 : 4;
    const int tuned = gemv_tuned_wgs_per_cu();
    const int grid = balanced_grid(ceil_div(p.n, OUT), tuned > 0 ? tuned : 3);
    if (ch <= 1) return launch_mt_rc<T, R, 1, EPI, TOK>(s, p, grid);
    return launch_mt_rc<T, R, 2, EPI, TOK>(s, p, grid);
  }
  constexpr int R = 2, OUT = (EPI == SK_GATEUP) ? 1 : 2;
  const int tuned = gemv_tuned_wgs_per_cu();
  // long rows: 2 workgroups per CU. One token, rows of 5+ chunks per thread and a row-group count
  // that fills 4 workgroups per CU evenly: 4 (18.35 against 18.65 us on 4096 x 14336). Elsewhere 4
  // measured slower (15360 x 5120: 26.6 against 24.9 us; 5120 x 13824, whose 2560 groups do not
  // split evenly: 23.1 against 22.0 us; with the operand registers of 4 tokens 22.3 against 21.3 us).
  const int n_groups = ceil_div(p.n, OUT);
  const bool four = TOK == 1 && ch > 4 && n_groups % (device_cus() * 4) == 0;
  const int grid = balanced_grid(n_groups, tuned > 0 ? tuned : (four ? 4 : 2));
  if (ch <= 4) return launch_mt_rc<T, R, 4, EPI, TOK>(s, p, grid);
  if (ch <= 7) return launch_mt_rc<T, R, 7, EPI, TOK>(s, p, grid);
  return MUI_ERR_UNSUPPORTED;
  }
}

// longest row one launch covers: 7 chunks of 8 values per thread
constexpr int kMtMaxK = 7 * 8 * kMtThreads;

int launch_gemv_multi(hipStream_t s, int dtype, int epilogue, const SkinnyParams& p) {
  if (p.tokens < 1 || p.tokens > 8) return MUI_ERR_UNSUPPORTED;
  if (p.k > kMtMaxK) {
    // Longer rows (down projections of 70B-class models): K segments, one launch each, every
    // launch after the first adding to y through the residual operand (the thread that loads
    // y[t, n] is the one that stores it). A fused norm needs the whole row and is not split.
    if (epilogue != SK_LINEAR || p.gamma) return MUI_ERR_UNSUPPORTED;
    SkinnyParams q = p;
    q.x_pitch = p.x_pitch > 0 ? p.x_pitch : (long)p.k;
    for (int done = 0; done < p.k; done += kMtMaxK) {
      q.k = p.k - done < kMtMaxK ? p.k - done : kMtMaxK;
      q.w0 = (const uint16_t*)p.w0 + done;
      q.x = p.x + done;
      q.residual = done == 0 ? p.residual : p.y;
      q.add_bias = done + q.k == p.k ? p.add_bias : nullptr;
      const int st = launch_gemv_multi(s, dtype, epilogue, q);
      if (st != MUI_OK) return st;
    }
    return MUI_OK;
  }
#define MUI_MT_CASE(TT, EPIV)                                            \
  if (epilogue == EPIV) {                                                \
    if (p.tokens <= 1) return launch_mt_t<TT, EPIV, 1>(s, p);            \
    if (p.tokens <= 2) return launch_mt_t<TT, EPIV, 2>(s, p);            \
    if (p.tokens <= 4) return launch_mt_t<TT, EPIV, 4>(s, p);            \
    return launch_mt_t<TT, EPIV, 8>(s, p);                               \
  }
  if (dtype == MUI_DTYPE_F16) {
    MUI_MT_CASE(F16, SK_LINEAR)
    MUI_MT_CASE(F16, SK_GATEUP)
  } else if (dtype == MUI_DTYPE_BF16) {
    MUI_MT_CASE(BF16, SK_LINEAR)
    MUI_MT_CASE(BF16, SK_GATEUP)
  }
#undef MUI_MT_CASE
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui
