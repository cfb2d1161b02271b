// Weight-only int8 linears for 1..4 tokens (fp16 activations) on the 4 x 4 x 4 matrix instruction.
//
// v_mfma_f32_4x4x4_16b_f16 multiplies sixteen independent 4 x 4 blocks per wave: lane 4 b + j
// supplies, for block b, four k-values of row j of the first operand and four k-values of column j
// of the second, and receives column j of the block's 4 x 4 result (row i in result register i).
// Sixteen independent blocks are what a GEMV-shaped read wants: with the (up to) four tokens as
// the rows of the first operand and four weight rows as the columns of the second, lane 4 b + j
// reads 16 consecutive codes of weight row j at 16 b -- a load instruction covers 256 contiguous
// bytes of each of four rows, the access shape of the vector-ALU kernels -- and no value has to
// change lanes on its way to the multiplier: no LDS tile, no transposing reads, and the token
// operands (gamma * x of token j at the lane's own k-values) are prepared once per lane instead
// of once per lane and token. Per 16 codes of a lane: 4 sign flips and 8 byte permutes (a byte
// dropped into the mantissa of 1024.0 is the fp16 number 1024 + byte; int8_multi.hip has the
// arithmetic) and 4 matrix instructions, where the packed-dot kernel issues 8 dots per token.
// The offset's correction term needs sum_k x_k of every token in the lanes of every weight row: the
// same instruction against a tile of ones delivers it in exactly that layout.
//
// A workgroup of WV waves works on groups of 4 U weight rows (U times two gate/up pairs); wave w
// takes Q consecutive 256-code segments of the rows, the sixteen blocks of a wave
// are added up in registers (DPP inside a row of 16 lanes, row swaps across rows) and the waves
// through LDS. One workgroup of eight waves per CU with eight rows per group measured best on the
// Llama-3-8B shapes: every workgroup prepares the token operands of its whole K range, so many
// small workgroups multiply that traffic (four waves x four rows x three workgroups per CU: QKV
// 6144 x 4096 at 4 tokens 9.1 us, against 7.6 us). Two register sets where that pays (launcher):
// the weights of group i + 2 are requested once group i has been multiplied, the values its
// epilogue needs from memory once group i's epilogue has used them (refilled any earlier, the
// compiler copies them between registers at the loop's edges and waits for the youngest loads).
//
// The reference has no kernel for more than one token (muillm/modules/quantized/int8linear.py:279-293
// dequantises the whole matrix and calls F.linear).
#include "skinny.cuh"

namespace mui {

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kDppRor4 = 0x124;  // row_ror:4: lane l of a row of 16 reads lane (l + 4) % 16
constexpr int kDppRor8 = 0x128;

struct Int8QuadArgs {
  const uint16_t* s0; const uint16_t* s1; long s_pitch; int group_shift;
  const uint16_t* add_bias; const uint16_t* residual;
};

__device__ __forceinline__ f32x4 mfma4(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, f32x4 c) {
  const u32x2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
}

// sum over the four 16-lane rows of a wave, the same value in all four (gfx950's row swaps:
// permlane16_swap exchanges rows 1, 3 of its first operand with rows 0, 2 of its second,
// permlane32_swap the upper half of the first with the lower half of the second)
__device__ __forceinline__ float quad_rows_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// GW (group format, groups of at least 128 codes): a wave's span of Q segments holds at most 16
// groups, so lane 4 b + j requests the span's pair number b of its row -- one load per lane and
// four rows -- and the pair of segment q is fetched from the lane that holds it with a
// ds_bpermute; one load per lane and segment otherwise. (The per-segment loads doubled the
// kernel's load instructions: gate/up 2 x 14336 x 4096 at 4 tokens 23.3 us with them, 21.3 us with
// the pairs taken out of the timing altogether, 20.5 us with per-channel scales.)
template <int WV, int Q, int U, bool NORM, int EPI, int WF, bool TWO, bool GW = false>
__global__ void __launch_bounds__(WV* kWave) int8_quad_kernel(
    // The first 14 dwords arrive in SGPRs at wave launch, the rest through scalar loads: everything
    // the addresses of the token rows and of the first weights are made of is among the former, and
    // nothing that needs the latter may move in front of those loads (sched_barrier below).
    const uint8_t* w0, const uint8_t* w1, const uint16_t* x, const uint16_t* gamma, int pitch, int n, int k,
    int tokens, int x_pitch, uint16_t* y, float eps, const Int8QuadArgs a) {
  using T = F16;
  constexpr int OUT4 = (EPI == SK_GATEUP) ? 2 : 4;  // outputs of four weight rows
  constexpr int OUT = OUT4 * U;                     // outputs per row group (U times four weight rows)
  constexpr int NP = WV;                            // partial results per output: one per wave
  constexpr int NSET = TWO ? 2 : 1;
  constexpr uint32_t kFlip = (WF == WF_I8_CHANNEL) ? 0x80808080u : 0u;
  constexpr float kOffset = (WF == WF_I8_CHANNEL) ? 1152.f : 1024.f;
  constexpr bool GROUP = WF == WF_U8_GROUP;
  __shared__ __attribute__((aligned(16))) float red[2][NP][4 * U][4];  // [buffer][partial][weight row][token]
  __shared__ float red_ss[NP][4];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int j = lane & 3;   // weight row inside the group; token of this lane's x operand
  const int b = lane >> 2;  // block: codes 16 b .. 16 b + 15 of each 256-code segment
  const int n_groups = (n + OUT - 1) / OUT;

  // segment q of this wave covers codes (wave * Q + q) * 256 .. + 255 of a row (a contiguous span per
  // wave: QKV 6144 x 4096 at 4 tokens 7.3 us, against 7.5 us with the waves interleaved segment by segment)
  int koff[Q];
  bool kval[Q];
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    const int kk = (wave * Q + q) * 256 + 16 * b;
    kval[q] = kk < k;
    koff[q] = kval[q] ? kk : 0;
  }

  // One register set: the weights of a row group, the (scale, min) pairs of the group format, and
  // what the epilogue thread of the group needs from memory (residual, per-channel scales; loaded
  // inside the epilogue they would add a memory round trip to the end of the kernel). Every thread
  // requests the epilogue values, from clamped addresses: behind a branch the compiler could no
  // longer count the loads in flight and would wait for the other set's weights as well.
  struct Set {
    u32x4 w[U][Q];
    uint32_t sp[U][GW ? 1 : Q];
    uint32_t res, s0, s1;
  };
  auto issue_w = [&](Set& st, int rg) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int row;
      const uint8_t* base;
      if constexpr (EPI == SK_GATEUP) {
        row = rg * OUT + u * OUT4 + (j >> 1);
        base = (j & 1) ? w1 : w0;
      } else {
        row = rg * OUT + u * OUT4 + j;
        base = w0;
      }
      row = row < n ? row : n - 1;
      const uint8_t* rp = base + (long)row * pitch;
#pragma unroll
      for (int q = 0; q < Q; ++q) st.w[u][q] = ld16_stream(rp + koff[q]);
    }
  };
  // the epilogue's mapping: thread o * 4 + tk finishes output o of the group for token tk
  const int ep_o = (t >> 2) < OUT ? (t >> 2) : OUT - 1;
  const int ep_tk = (t & 3) < tokens ? (t & 3) : tokens - 1;
  auto issue_extras = [&](Set& st, int rg) {
    int row = rg * OUT + ep_o;
    row = row < n ? row : n - 1;
    if constexpr (WF == WF_I8_CHANNEL) {
      st.s0 = ld2(a.s0 + (long)row * a.s_pitch);
      if constexpr (EPI == SK_GATEUP) st.s1 = ld2(a.s1 + (long)row * a.s_pitch);
    }
    if constexpr (EPI == SK_LINEAR) st.res = ld2(a.residual ? a.residual + ((long)ep_tk * n + row) : x);
  };

  // ---- token operand of this lane: gamma * x of token j at the lane's k-values, requested before
  // the first weights (loads return in order: the preparation then overlaps the flight of the first
  // row group instead of following it). No load sits behind a branch (clamped addresses, dead lanes
  // zeroed by selects).
  u32x4 xa[Q][2];
  {
    const long xrow = (long)(j < tokens ? j : tokens - 1) * x_pitch;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) xa[q][hf] = ld16(x + xrow + koff[q] + 8 * hf);
    }
  }
  u32x4 gq[NORM ? Q : 1][2];
  if constexpr (NORM) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) gq[q][hf] = ld16(gamma + koff[q] + 8 * hf);
    }
  }
  Set sets[NSET];
  issue_w(sets[0], blockIdx.x);
  __builtin_amdgcn_sched_barrier(0);  // nothing that waits for a scalar load moves in front of the loads above
  // The grid never exceeds the number of row groups; group i of this workgroup is blockIdx.x + i * gridDim.x.
  const int n_my = (n_groups - 1 - (int)blockIdx.x) / (int)gridDim.x + 1;
  auto group_of = [&](int i) -> int { return blockIdx.x + i * gridDim.x; };
  // GW: first group of this wave's span, the pair this lane requests (clamped to the row's last
  // group), and for every segment the byte address (lane * 4) of the lane holding its pair
  int gw_load = 0;
  int gw_src[GW ? Q : 1] = {};
  if constexpr (GW) {
    const int g0 = (wave * Q * 256) >> a.group_shift;
    const int g_last = ((k + (1 << a.group_shift) - 1) >> a.group_shift) - 1;
    gw_load = g0 + b < g_last ? g0 + b : g_last;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      int gi = ((((wave * Q + q) * 256) + 16 * b) >> a.group_shift) - g0;
      gi = gi < 15 ? gi : 15;
      gw_src[q] = (4 * gi + j) * 4;
    }
  }
  // the group format's (scale, min) pairs of a row group
  auto issue_pairs = [&](Set& st, int rg) {
    if constexpr (GROUP) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int row;
        const uint16_t* sbase;
        if constexpr (EPI == SK_GATEUP) {
          row = rg * OUT + u * OUT4 + (j >> 1);
          sbase = (j & 1) ? a.s1 : a.s0;
        } else {
          row = rg * OUT + u * OUT4 + j;
          sbase = a.s0;
        }
        row = row < n ? row : n - 1;
        if constexpr (GW) {
          st.sp[u][0] = ld4(sbase + (long)row * a.s_pitch + 2 * gw_load);
        } else {
#pragma unroll
          for (int q = 0; q < Q; ++q) st.sp[u][q] = ld4(sbase + (long)row * a.s_pitch + 2 * (koff[q] >> a.group_shift));
        }
      }
    }
  };
  auto issue = [&](Set& st, int rg) {
    issue_w(st, rg);
    issue_pairs(st, rg);
  };
  issue_pairs(sets[0], group_of(0));
  issue_extras(sets[0], group_of(0));
  if constexpr (TWO) {
    // (a workgroup of a ragged grid that has a single group requests it twice: one group of the launch)
    issue(sets[1], group_of(n_my > 1 ? 1 : 0));
    issue_extras(sets[1], group_of(n_my > 1 ? 1 : 0));
  }

  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    const bool live = kval[q] && j < tokens;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      float sq = 0.f;
      u32x4 v = make_b<T, NORM>(xa[q][hf], NORM ? gq[q][hf] : xa[q][hf], sq);
      const u32x4 zero = {0u, 0u, 0u, 0u};
      xa[q][hf] = live ? v : zero;
      ss += live ? sq : 0.f;
    }
  }
  // step s of segment q multiplies the lane's codes 4 s .. 4 s + 3 with these four token values
  auto xop = [&](int q, int s, uint32_t& lo, uint32_t& hi) {
    const u32x4 v = xa[q][s >> 1];
    lo = (s & 1) ? v.z : v.x;
    hi = (s & 1) ? v.w : v.y;
  };
  // sum of the token operands over the lane's block, for all four tokens (result register i = token
  // i): per segment for the group format, over all of them for per-channel scales
  constexpr uint32_t kOnes = 0x3C003C00u;
  f32x4 xs[GROUP ? Q : 1];
#pragma unroll
  for (int q = 0; q < (GROUP ? Q : 1); ++q) xs[q] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int q = 0; q < Q; ++q) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      uint32_t lo, hi;
      xop(q, s, lo, hi);
      xs[GROUP ? q : 0] = mfma4(lo, hi, kOnes, kOnes, xs[GROUP ? q : 0]);
    }
  }
  f32x4 acc_init = {0.f, 0.f, 0.f, 0.f};
  if constexpr (!GROUP) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc_init[i] = -kOffset * xs[0][i];
  }
  float rsv = 1.f;  // 1 / rms of the epilogue thread's token
  if constexpr (NORM) {
    ss += dpp_f32<kDppRor8>(ss);
    ss += dpp_f32<kDppRor4>(ss);
    ss = quad_rows_sum(ss);
    if (lane < 4) red_ss[wave][j] = ss;
    __syncthreads();
    if (t < OUT * 4) {
      float tot = 0.f;
#pragma unroll
      for (int p = 0; p < NP; ++p) tot += red_ss[p][t & 3];
      rsv = rsqrtf(tot / (float)k + eps);
    }
  }

  int buf = 0;
  // group `rg` out of register set `st`; refill: the set is requested again for group `nxt`
  auto pass = [&](Set& st, int rg, auto refill, int nxt) {
    f32x4 acc[U], acc1[U];  // two chains per four rows: matrix instructions back to back
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc[u] = acc_init;
      acc1[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int q = 0; q < Q; ++q) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const u32x4 wq = st.w[u][q];
        const uint32_t wv[4] = {wq.x ^ kFlip, wq.y ^ kFlip, wq.z ^ kFlip, wq.w ^ kFlip};
        f32x4 part = {0.f, 0.f, 0.f, 0.f}, part1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint32_t b0 = __builtin_amdgcn_perm(0x64646464u, wv[s], 0x04010400u);
          const uint32_t b1 = __builtin_amdgcn_perm(0x64646464u, wv[s], 0x04030402u);
          uint32_t lo, hi;
          xop(q, s, lo, hi);
          if constexpr (GROUP) {
            if (s & 1) part1 = mfma4(lo, hi, b0, b1, part1);
            else part = mfma4(lo, hi, b0, b1, part);
          } else {
            if (s & 1) acc1[u] = mfma4(lo, hi, b0, b1, acc1[u]);
            else acc[u] = mfma4(lo, hi, b0, b1, acc[u]);
          }
        }
        if constexpr (GROUP) {
          // w = u8 * scale + min over the segment's group: scale * (sum - 1024 xs) + min * xs
          uint32_t pair;
          if constexpr (GW) pair = (uint32_t)__builtin_amdgcn_ds_bpermute(gw_src[q], (int)st.sp[u][0]);
          else pair = st.sp[u][q];
          const float sc = T::lo(pair), cm = fmaf(-kOffset, sc, T::hi(pair));
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[u][i] = fmaf(sc, part[i] + part1[i], fmaf(cm, xs[q][i], acc[u][i]));
        }
      }
    }
    if constexpr (decltype(refill)::value) issue(st, nxt);
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = acc[u][i] + acc1[u][i];
        v += dpp_f32<kDppRor8>(v);
        v += dpp_f32<kDppRor4>(v);
        acc[u][i] = quad_rows_sum(v);
      }
      if (lane < 4) *(f32x4*)&red[buf][wave][u * 4 + j][0] = acc[u];
    }
    __syncthreads();

    if (t < OUT * 4) {
      const int o = t >> 2, tk = t & 3;
      const int row = rg * OUT + o;
      if (row < n && tk < tokens) {
        auto total = [&](int r) {
          float v = 0.f;
#pragma unroll
          for (int p = 0; p < NP; ++p) v += red[buf][p][r][tk];
          return v * rsv;
        };
        float v;
        if constexpr (EPI == SK_GATEUP) {
          float g = total(2 * o), up = total(2 * o + 1);
          if constexpr (WF == WF_I8_CHANNEL) {
            g *= T::one((uint16_t)st.s0);
            up *= T::one((uint16_t)st.s1);
          }
          v = silu_f32(g) * up;
        } else {
          v = total(o);
          if constexpr (WF == WF_I8_CHANNEL) v *= T::one((uint16_t)st.s0);
          if (a.add_bias) v += T::one(a.add_bias[row]);
          if (a.residual) v += T::one((uint16_t)st.res);
        }
        y[(long)tk * n + row] = T::pack(v);
      }
    }
    if constexpr (decltype(refill)::value) issue_extras(st, nxt);
    buf ^= 1;
  };
  constexpr std::true_type kRefill{};
  constexpr std::false_type kLast{};
  if constexpr (!TWO) {
    for (int i = 0; i + 1 < n_my; ++i) pass(sets[0], group_of(i), kRefill, group_of(i + 1));
    pass(sets[0], group_of(n_my - 1), kLast, 0);
  } else {
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

static int g_i8q_on = 1;       // mui_tune_int8_quad: 0 sends 2..4 tokens to the older kernels
static int g_i8q_min_tokens = 0;  // 0: two tokens with per-channel scales, three with the group format
static int g_i8q_per_cu = 0;   // workgroups per CU, 0 = built-in
static int g_i8q_sets = 0;     // 1: one register set everywhere
static int g_i8q_wide_pairs = 1;  // group format: one (scale, min) load per lane and four rows where groups allow

template <int WV, int Q, int U, int EPI, int WF, bool GW = false>
static int launch_i8q_wq(hipStream_t s, const SkinnyParams& p) {
  constexpr int OUT = ((EPI == SK_GATEUP) ? 2 : 4) * U;
  Int8QuadArgs a = {p.s0, p.s1, p.s_pitch, p.group_shift, p.add_bias, p.residual};
  const long x_pitch = p.x_pitch > 0 ? p.x_pitch : (long)p.k;
  if (p.pitch > 0x7fffffffL || x_pitch > 0x7fffffffL) return MUI_ERR_UNSUPPORTED;
  const int n_groups = ceil_div(p.n, OUT);
  // workgroups per CU: three of four waves, two of eight -- or what the registers of the instance
  // allow, asked once per instance (a grid larger than what is resident runs its tail as a second round)
  auto resident = [](auto kernel) {
    int nb = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel, WV * kWave, 0) != hipSuccess || nb < 1) nb = 1;
    return nb;
  };
  static const int res_two[2] = {resident(int8_quad_kernel<WV, Q, U, false, EPI, WF, true, GW>),
                                 resident(int8_quad_kernel<WV, Q, U, true, EPI, WF, true, GW>)};
  static const int res_one[2] = {resident(int8_quad_kernel<WV, Q, U, false, EPI, WF, false, GW>),
                                 resident(int8_quad_kernel<WV, Q, U, true, EPI, WF, false, GW>)};
  const int want = g_i8q_per_cu > 0 ? g_i8q_per_cu : (WV == 4 ? 3 : 1);
  const int nm = p.gamma ? 1 : 0;
  // Two register sets where workgroups have more than one group (a ragged grid's last ones may have
  // one) -- by default only behind a fused norm, whose reduction and barrier the second set's
  // flight covers, or with more than two groups per workgroup: o_proj 4096 x 4096 at 4 tokens, two
  // groups per workgroup and no norm, measured 5.7 us with one set against 6.2 us with two, QKV
  // 6144 x 4096 (norm, three groups) 8.6 against 7.6 us, down 4096 x 14336 (four groups) 15.0
  // against 13.6 us.
  int per_cu = want < res_two[nm] ? want : res_two[nm];
  int grid = balanced_grid(n_groups, per_cu);
  bool two = n_groups > grid;
  if (g_i8q_sets == 1) two = false;
  else if (g_i8q_sets == 0) two = two && (p.gamma || n_groups > 2 * grid);
  if (!two) {
    per_cu = want < res_one[nm] ? want : res_one[nm];
    grid = balanced_grid(n_groups, per_cu);
  }
#define MUI_I8Q_LAUNCH(NORMV, TWOV)                                                                             \
  hipLaunchKernelGGL((int8_quad_kernel<WV, Q, U, NORMV, EPI, WF, TWOV, GW>), dim3(grid), dim3(WV* kWave), 0, s,         \
                     (const uint8_t*)p.w0, (const uint8_t*)p.w1, p.x, p.gamma, (int)p.pitch, p.n, p.k, p.tokens, \
                     (int)x_pitch, p.y, p.eps, a)
  if (two) { if (p.gamma) MUI_I8Q_LAUNCH(true, true); else MUI_I8Q_LAUNCH(false, true); }
  else { if (p.gamma) MUI_I8Q_LAUNCH(true, false); else MUI_I8Q_LAUNCH(false, false); }
#undef MUI_I8Q_LAUNCH
  return launch_status();
}

template <int EPI, int WF>
static int launch_i8q_t(hipStream_t s, const SkinnyParams& p) {
  const int segs = ceil_div(p.k, 256);
  if constexpr (WF == WF_U8_GROUP) {
    if (p.group_shift >= 7 && g_i8q_wide_pairs) {
      if (segs <= 4) return launch_i8q_wq<4, 1, 2, EPI, WF, true>(s, p);
      if (segs <= 8) return launch_i8q_wq<8, 1, 2, EPI, WF, true>(s, p);
      if (segs <= 16) return launch_i8q_wq<8, 2, 2, EPI, WF, true>(s, p);
      if (segs <= 32) return launch_i8q_wq<8, 4, 1, EPI, WF, true>(s, p);
      if (segs <= 56) return launch_i8q_wq<8, 7, 1, EPI, WF, true>(s, p);
      return MUI_ERR_UNSUPPORTED;
    }
  }
  if (segs <= 4) return launch_i8q_wq<4, 1, 2, EPI, WF>(s, p);
  if (segs <= 8) return launch_i8q_wq<8, 1, 2, EPI, WF>(s, p);
  if (segs <= 16) return launch_i8q_wq<8, 2, 2, EPI, WF>(s, p);
  if (segs <= 32) return launch_i8q_wq<8, 4, 1, EPI, WF>(s, p);
  if (segs <= 56) return launch_i8q_wq<8, 7, 1, EPI, WF>(s, p);
  return MUI_ERR_UNSUPPORTED;
}

// 1..4 tokens, int8 weights, fp16 activations; MUI_ERR_UNSUPPORTED for what it does not cover
// (bf16, rows longer than 14336, groups smaller than 16 codes, a multiplicative bias)
int launch_int8_quad(hipStream_t s, int dtype, int wf, int epilogue, const SkinnyParams& p) {
  // One token stays on the packed-dot kernel (QKV 6144 x 4096: 6.5 against 7.3 us here); the group
  // format, whose (scale, min) pairs double this kernel's load instructions, up to two tokens.
  const int min_tokens = g_i8q_min_tokens > 0 ? g_i8q_min_tokens : (wf == WF_U8_GROUP ? 3 : 2);
  if (!g_i8q_on || dtype != MUI_DTYPE_F16 || p.tokens < min_tokens || p.tokens > 4) return MUI_ERR_UNSUPPORTED;
  if (p.mul_bias || (p.k & 15)) return MUI_ERR_UNSUPPORTED;
  if (wf == WF_U8_GROUP && p.group_shift < 4) return MUI_ERR_UNSUPPORTED;
#define MUI_I8Q_CASE(WFV, EPIV) \
  if (wf == WFV && epilogue == EPIV) return launch_i8q_t<EPIV, WFV>(s, p);
  MUI_I8Q_CASE(WF_I8_CHANNEL, SK_LINEAR)
  MUI_I8Q_CASE(WF_I8_CHANNEL, SK_GATEUP)
  MUI_I8Q_CASE(WF_U8_GROUP, SK_LINEAR)
  MUI_I8Q_CASE(WF_U8_GROUP, SK_GATEUP)
#undef MUI_I8Q_CASE
  return MUI_ERR_UNSUPPORTED;
}

}  // namespace mui

extern "C" int mui_tune_int8_quad(int on, int min_tokens, int workgroups_per_cu, int sets) {
  MUI_TUNE_GUARD();
  if (min_tokens < 0 || min_tokens > 5 || workgroups_per_cu < 0 || workgroups_per_cu > 16 || sets < 0 || sets > 2)
    return MUI_ERR_INVALID_ARG;
  mui::g_i8q_on = on ? 1 : 0;
  mui::g_i8q_min_tokens = min_tokens;
  mui::g_i8q_per_cu = workgroups_per_cu;
  mui::g_i8q_sets = sets;
  return MUI_OK;
}
