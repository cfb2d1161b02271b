// Weight-only int8 linears for 2..4 tokens (fp16 activations): the single-token int8 GEMV
// structure (int8.hip) with the token operands gamma * x packed fp16 in registers.
//
// Dequantisation without a convert per weight: a byte b dropped into the mantissa of 1024.0
// (0x6400 | b, two byte permutes per dword) IS the fp16 number 1024 + b, so
//     sum_k (1024 + b_k) x_k  -  1024 sum_k x_k  =  sum_k b_k x_k
// with one v_dot2_f32_f16 per two weights and token; the correction term is folded into the
// accumulator's start value (per-channel format, where the sign bit is flipped first: offset
// 1024 + 128) or applied per group together with (scale, min) (the reference's group format,
// muillm/quantization/rtnquantizer.py:49-88). The products are exact in fp32 and the offset is
// 16x the largest weight, so the cancellation costs about 4 bits of the fp32 accumulator.
//
// The reference has no kernel for more than one token (muillm/modules/quantized/int8linear.py:279-293
// dequantises the whole matrix and calls F.linear).
#include "skinny.cuh"

namespace mui {

constexpr int kI8mThreads = 256;
constexpr int kI8mWaves = kI8mThreads / kWave;

struct Int8MultiArgs {
  const uint16_t* s0; const uint16_t* s1; long s_pitch; int group_shift;
  const uint16_t* add_bias; const uint16_t* residual;
};

template <int R, int CH, bool NORM, int EPI, int WF, int TOK>
__global__ void __launch_bounds__(kI8mThreads) int8_multi_kernel(
    // The first 14 dwords arrive in SGPRs at wave launch, the rest through scalar loads: everything
    // the addresses of the token rows and of the first weights are made of is among the former, and
    // nothing that needs the latter is allowed in front of those loads (sched_barrier below) --
    // with `tokens`, the bias pointers or the grid size consumed early, the compiler put the wait
    // for the scalar loads in front of the first vector load (QKV 6144 x 4096 and o_proj at one token).
    const uint8_t* w0, const uint8_t* w1, const uint16_t* x, const uint16_t* gamma, int pitch, int n, int k,
    int tokens, int x_pitch, uint16_t* y, float eps, const Int8MultiArgs a) {
  using T = F16;
  constexpr int OUT = (EPI == SK_GATEUP) ? R / 2 : R;
  constexpr int NV = R * TOK;             // partial sums per row group
  constexpr int NH = NV > 16 ? 2 : 1;     // reduced 16 at a time
  constexpr int NVH = NV / NH;
  constexpr uint32_t kFlip = (WF == WF_I8_CHANNEL) ? 0x80808080u : 0u;
  constexpr float kOffset = (WF == WF_I8_CHANNEL) ? 1152.f : 1024.f;
  static_assert(NV <= 32 && (R % 2 == 0) && NVH <= 16, "shape");
  __shared__ float red[2][kI8mWaves * 4][NV];
  __shared__ float red_ss[kI8mWaves][TOK];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int kc = k >> 4;  // 16-byte chunks (16 weights) per row
  const int n_groups = (n + OUT - 1) / OUT;

  int coff[CH];
  bool cvalid[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = t + kI8mThreads * j;
    cvalid[j] = c < kc;
    coff[j] = cvalid[j] ? (c << 4) : 0;
  }

  // The weights of a row group, the (scale, min) pairs of the group format, and what the epilogue
  // thread of the group needs from memory (residual, per-channel scales): loaded inside the
  // epilogue that would add a memory round trip to the end of the kernel. Every thread requests
  // the epilogue values, from clamped addresses (no load behind a branch).
  struct Set {
    u32x4 w[R][CH];
    uint32_t sm[R][CH];
    uint32_t res, s0, s1;
  };
  // the epilogue gives every output sixteen lanes; lane 0 of them, thread 16 * (o * TOK + tk), finishes it
  static_assert(16 * OUT * TOK <= kI8mThreads, "sixteen epilogue lanes per output");
  const int ep_o = ((t >> 4) / TOK) < OUT ? (t >> 4) / TOK : OUT - 1;
  const int ep_tk = ((t >> 4) % TOK) < tokens ? (t >> 4) % TOK : tokens - 1;
  auto issue_w = [&](Set& st, int rg) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row;
      const uint8_t* base;
      if constexpr (EPI == SK_GATEUP) {
        row = rg * OUT + (r >> 1);
        base = (r & 1) ? w1 : w0;
      } else {
        row = rg * R + r;
        base = w0;
      }
      row = row < n ? row : n - 1;
      const uint8_t* rp = base + (long)row * pitch;
#pragma unroll
      for (int j = 0; j < CH; ++j) st.w[r][j] = ld16_stream(rp + coff[j]);
    }
  };
  // the group format's (scale, min) pairs and the epilogue's values: their addresses need scalars
  // that are not preloaded
  auto issue_rest = [&](Set& st, int rg) {
    if constexpr (WF == WF_U8_GROUP) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        int row;
        const uint16_t* sbase;
        if constexpr (EPI == SK_GATEUP) {
          row = rg * OUT + (r >> 1);
          sbase = (r & 1) ? a.s1 : a.s0;
        } else {
          row = rg * R + r;
          sbase = a.s0;
        }
        row = row < n ? row : n - 1;
#pragma unroll
        for (int j = 0; j < CH; ++j) st.sm[r][j] = ld4(sbase + (long)row * a.s_pitch + 2 * (coff[j] >> a.group_shift));
      }
    }
    int row = rg * OUT + ep_o;
    row = row < n ? row : n - 1;
    if constexpr (WF == WF_I8_CHANNEL) {
      st.s0 = ld2(a.s0 + (long)row * a.s_pitch);
      if constexpr (EPI == SK_GATEUP) st.s1 = ld2(a.s1 + (long)row * a.s_pitch);
    }
    if constexpr (EPI == SK_LINEAR) st.res = ld2(a.residual ? a.residual + ((long)ep_tk * n + row) : x);
  };
  // ---- token operands: gamma * x as packed fp16, the chunk's sum of them on the side. They are
  // requested before the first weights: loads return in order, so the operand preparation (and a
  // fused norm's reduction) then overlaps the flight of the first row group instead of following
  // it (QKV with fused norm 7.5 -> 6.4 us at one token). No load sits behind a branch (clamped
  // addresses, dead lanes zeroed by selects).
  u32x4 xq[TOK][CH][2];
  u32x4 gq[CH][2];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    const long xrow = tk == 0 ? 0 : (long)(tk < tokens ? tk : tokens - 1) * x_pitch;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) xq[tk][j][hf] = ld16(x + xrow + coff[j] + 8 * hf);
    }
  }
  if constexpr (NORM) {
#pragma unroll
    for (int j = 0; j < CH; ++j) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) gq[j][hf] = ld16(gamma + coff[j] + 8 * hf);
    }
  }
  Set set;
  issue_w(set, blockIdx.x);
  __builtin_amdgcn_sched_barrier(0);  // nothing that waits for a scalar load moves in front of the loads above
  // The grid never exceeds the number of row groups; group i of this workgroup is blockIdx.x + i * gridDim.x.
  const int n_my = (n_groups - 1 - (int)blockIdx.x) / (int)gridDim.x + 1;
  auto group_of = [&](int i) -> int { return blockIdx.x + i * gridDim.x; };
  issue_rest(set, blockIdx.x);

  float xsum[TOK][CH];
  float ss[TOK];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    ss[tk] = 0.f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      xsum[tk][j] = 0.f;
      const bool live = cvalid[j] && tk < tokens;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        float sq = 0.f;
        u32x4 b = make_b<T, NORM>(xq[tk][j][hf], NORM ? gq[j][hf] : xq[tk][j][hf], sq);
        const u32x4 zero = {0u, 0u, 0u, 0u};
        b = live ? b : zero;
        ss[tk] += live ? sq : 0.f;
        xq[tk][j][hf] = b;
        // sum of the eight operands: packed dots against (1, 1)
        const uint32_t bw[4] = {b.x, b.y, b.z, b.w};
        const f16x2 one2 = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
        for (int d = 0; d < 4; ++d)
          xsum[tk][j] = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, bw[d]), one2, xsum[tk][j], false);
      }
    }
  }
  float acc_init[TOK];  // per-channel: -(1024 + 128) * sum of this thread's operands
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < CH; ++j) s += xsum[tk][j];
    acc_init[tk] = -kOffset * s;
  }
  float rsv = 1.f;  // 1 / rms of the epilogue thread's token
  if constexpr (NORM) {
#pragma unroll
    for (int tk = 0; tk < TOK; ++tk) {
      const float s = wave_sum(ss[tk]);
      if (lane == 0) red_ss[wave][tk] = s;
    }
    __syncthreads();
    if (t < 16 * OUT * TOK) {
      const int tk = (t >> 4) % TOK;
      const float tot = (red_ss[0][tk] + red_ss[1][tk]) + (red_ss[2][tk] + red_ss[3][tk]);
      rsv = rsqrtf(tot / (float)k + eps);
    }
  }

  int buf = 0;
  // group `rg` out of register set `st`; REFILL: the set is requested again for group `nxt`
  auto pass = [&](Set& st, int rg, auto refill, int nxt) {
    float acc[NH][NVH];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float ar[TOK];
#pragma unroll
      for (int tk = 0; tk < TOK; ++tk) ar[tk] = (WF == WF_I8_CHANNEL) ? acc_init[tk] : 0.f;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        // 16 bytes -> 8 packed pairs (1024 + b): pairs 0..3 meet xq[..][0], pairs 4..7 meet xq[..][1]
        const uint32_t wv[4] = {st.w[r][j].x ^ kFlip, st.w[r][j].y ^ kFlip, st.w[r][j].z ^ kFlip, st.w[r][j].w ^ kFlip};
        uint32_t pr[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          pr[2 * d + 0] = __builtin_amdgcn_perm(0x64646464u, wv[d], 0x04010400u);
          pr[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, wv[d], 0x04030402u);
        }
#pragma unroll
        for (int tk = 0; tk < TOK; ++tk) {
          float s = (WF == WF_I8_CHANNEL) ? ar[tk] : 0.f;
          // components go through scalars: __builtin_bit_cast applied directly to a vector
          // component (q.y) was compiled as a read of component 0 by this toolchain
          const u32x4 q0 = xq[tk][j][0], q1 = xq[tk][j][1];
          const uint32_t qa[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
          for (int d = 0; d < 8; ++d)
            s = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pr[d]), __builtin_bit_cast(f16x2, qa[d]), s, false);
          if constexpr (WF == WF_I8_CHANNEL) {
            ar[tk] = s;
          } else {
            // w = u8 * scale + min over this chunk's group: scale * (s - 1024 xsum) + min * xsum
            const float sc = T::lo(st.sm[r][j]), mn = T::hi(st.sm[r][j]);
            ar[tk] = fmaf(sc, fmaf(-kOffset, xsum[tk][j], s), fmaf(mn, xsum[tk][j], ar[tk]));
          }
        }
      }
#pragma unroll
      for (int tk = 0; tk < TOK; ++tk) {
        const int v = r * TOK + tk;
        acc[v / NVH][v % NVH] = ar[tk];
      }
    }
    const uint32_t cur_res = st.res, cur_s0 = st.s0, cur_s1 = st.s1;
    if constexpr (decltype(refill)::value) {
      issue_w(st, nxt);
      issue_rest(st, nxt);
    }

#pragma unroll
    for (int h = 0; h < NH; ++h) {
      row16_reduce_scatter<NVH>(acc[h], lane);
      if ((lane & (16 / NVH - 1)) == 0 || NVH == 16) red[buf][t >> 4][h * NVH + (lane & 15) / (16 / NVH)] = acc[h][0];
    }
    __syncthreads();

    // sixteen lanes per output: each fetches one of the 16 row partials, a DPP butterfly adds them
    // (one thread adding all sixteen was a chain of sixteen dependent LDS reads at the end of the kernel)
    if (t < 16 * OUT * TOK) {
      const int part = t & 15, o = (t >> 4) / TOK, tk = (t >> 4) % TOK;
      const int row = rg * OUT + o;
      const float v0 = row16_sum(red[buf][part][((EPI == SK_GATEUP) ? 2 * o : o) * TOK + tk]) * rsv;
      float v1 = 0.f;
      if constexpr (EPI == SK_GATEUP) v1 = row16_sum(red[buf][part][(2 * o + 1) * TOK + tk]) * rsv;
      if (part == 0 && row < n && tk < tokens) {
        float v;
        if constexpr (EPI == SK_GATEUP) {
          float g = v0, u = v1;
          if constexpr (WF == WF_I8_CHANNEL) {
            g *= T::one((uint16_t)cur_s0);
            u *= T::one((uint16_t)cur_s1);
          }
          v = silu_f32(g) * u;
        } else {
          v = v0;
          if constexpr (WF == WF_I8_CHANNEL) v *= T::one((uint16_t)cur_s0);
          if (a.add_bias) v += T::one(a.add_bias[row]);
          if (a.residual) v += T::one((uint16_t)cur_res);
        }
        y[(long)tk * n + row] = T::pack(v);
      }
    }
    buf ^= 1;
  };
  constexpr std::true_type kRefill{};
  constexpr std::false_type kLast{};
  for (int i = 0; i + 1 < n_my; ++i) pass(set, group_of(i), kRefill, group_of(i + 1));
  pass(set, group_of(n_my - 1), kLast, 0);
}

template <int R, int CH, int EPI, int WF, int TOK>
static int launch_i8m_rc(hipStream_t s, const SkinnyParams& p, int grid) {
  Int8MultiArgs a = {p.s0, p.s1, p.s_pitch, p.group_shift, p.add_bias, p.residual};
  const long x_pitch = p.x_pitch > 0 ? p.x_pitch : (long)p.k;
  if (p.pitch > 0x7fffffffL || x_pitch > 0x7fffffffL) return MUI_ERR_UNSUPPORTED;
#define MUI_I8M_LAUNCH(NORMV)                                                                              \
  hipLaunchKernelGGL((int8_multi_kernel<R, CH, NORMV, EPI, WF, TOK>), dim3(grid), dim3(kI8mThreads), 0, s,  \
                     (const uint8_t*)p.w0, (const uint8_t*)p.w1, p.x, p.gamma, (int)p.pitch, p.n, p.k,      \
                     p.tokens, (int)x_pitch, p.y, p.eps, a)
  if (p.gamma) MUI_I8M_LAUNCH(true); else MUI_I8M_LAUNCH(false);
#undef MUI_I8M_LAUNCH
  return launch_status();
}

template <int EPI, int WF, int TOK>
static int launch_i8m_t(hipStream_t s, const SkinnyParams& p) {
  const int ch = ceil_div(p.k >> 4, kI8mThreads);
  const int per_cu = int8_tuned_wgs_per_cu();
  if (ch <= 1) {
    if constexpr (TOK == 1) {
      if (int8_tuned_rows() == 16) {
        constexpr int R = 16, OUT = (EPI == SK_GATEUP) ? R / 2 : R;
        return launch_i8m_rc<R, 1, EPI, WF, TOK>(s, p, balanced_grid(ceil_div(p.n, OUT), per_cu > 0 ? per_cu : 2));
      }
    }
    // short rows: 8 rows in flight at 2 tokens, 4 at 4 (at most 32 partial sums per group)
    constexpr int R = (TOK <= 2) ? 8 : 4;
    constexpr int OUT = (EPI == SK_GATEUP) ? R / 2 : R;
    return launch_i8m_rc<R, 1, EPI, WF, TOK>(s, p, balanced_grid(ceil_div(p.n, OUT), per_cu > 0 ? per_cu : 3));
  }
  constexpr int R = 2, OUT = (EPI == SK_GATEUP) ? 1 : 2;
  const int grid = balanced_grid(ceil_div(p.n, OUT), per_cu > 0 ? per_cu : 2);
  if (ch <= 2) return launch_i8m_rc<R, 2, EPI, WF, TOK>(s, p, grid);
  if (ch <= 4) return launch_i8m_rc<R, 4, EPI, WF, TOK>(s, p, grid);
  return MUI_ERR_UNSUPPORTED;
}

// longest row one launch covers: 4 chunks of 16 weights per thread
constexpr int kI8mMaxK = 4 * 16 * kI8mThreads;

int launch_int8_multi(hipStream_t s, int dtype, int wf, int epilogue, const SkinnyParams& p) {
  if (dtype != MUI_DTYPE_F16 || p.tokens < 1 || p.tokens > 4) return MUI_ERR_UNSUPPORTED;
  if (p.mul_bias) return MUI_ERR_UNSUPPORTED;
  if (p.k > kI8mMaxK) {
    // Longer rows: K segments, one launch each, every launch after the first adding to y through
    // the residual operand (row scale and (scale, min) pairs are linear in the segment sums; a
    // segment starts on a group boundary). A fused norm needs the whole row and is not split.
    if (epilogue != SK_LINEAR || p.gamma) return MUI_ERR_UNSUPPORTED;
    if (wf == WF_U8_GROUP && (p.group_shift > 14)) return MUI_ERR_UNSUPPORTED;
    SkinnyParams q = p;
    q.x_pitch = p.x_pitch > 0 ? p.x_pitch : (long)p.k;
    for (int done = 0; done < p.k; done += kI8mMaxK) {
      q.k = p.k - done < kI8mMaxK ? p.k - done : kI8mMaxK;
      q.w0 = (const uint8_t*)p.w0 + done;
      q.x = p.x + done;
      if (wf == WF_U8_GROUP) q.s0 = p.s0 + 2 * (done >> p.group_shift);
      q.residual = done == 0 ? p.residual : p.y;
      q.add_bias = done + q.k == p.k ? p.add_bias : nullptr;
      const int st = launch_int8_multi(s, dtype, wf, epilogue, q);
      if (st != MUI_OK) return st;
    }
    return MUI_OK;
  }
#define MUI_I8M_CASE(WFV, EPIV)                                          \
  if (wf == WFV && epilogue == EPIV) {                                   \
    if (p.tokens <= 1) return launch_i8m_t<EPIV, WFV, 1>(s, p);          \
    if (p.tokens <= 2) return launch_i8m_t<EPIV, WFV, 2>(s, p);          \
    return launch_i8m_t<EPIV, WFV, 4>(s, p);                             \
  }
  MUI_I8M_CASE(WF_I8_CHANNEL, SK_LINEAR)
  MUI_I8M_CASE(WF_I8_CHANNEL, SK_GATEUP)
  MUI_I8M_CASE(WF_U8_GROUP, SK_LINEAR)
  MUI_I8M_CASE(WF_U8_GROUP, SK_GATEUP)
#undef MUI_I8M_CASE
  return MUI_ERR_UNSUPPORTED;
}

}  // namespace mui
