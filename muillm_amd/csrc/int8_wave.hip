// Weight-only int8 linears for 1..4 tokens (fp16 activations) on rows of at most 4096 weights:
// one WAVE per output row.
//
// int8_multi.hip deals the 16-byte chunks of a row out to the 256 threads of a workgroup, so every
// group of rows ends in a reduction across four waves (LDS, a barrier, an epilogue thread that adds
// sixteen partials). A 4096-byte row is only four wave-wide loads long, and that tail is then a large
// share of the kernel (QKV 6144 x 4096 at one token: 6.5 us against 5.0 us for just reading the
// bytes; at four tokens 8.9 us). Here lane l of a wave owns chunks l, l + 64, l + 128, l + 192 of
// EVERY row its wave handles: a wave-wide load still covers 1 KiB of contiguous weights, the token
// operands gamma * x of all of K sit in the wave's registers, and a row's sum is finished inside the
// wave (one multi-value DPP reduction per 16-lane row, two row swaps across the four rows) -- no
// LDS, no barrier, no hand-off between waves; the four waves of a workgroup never meet. A wave works
// on RW output rows (or gate/up pairs) at a time and requests the next ones before it reduces.
//
// Arithmetic is that of int8_multi.hip (bytes dropped into the mantissa of 1024.0, v_dot2_f32_f16,
// offset folded into the accumulator's start value or applied per group with (scale, min)); only
// the order in which a row's partial sums are added differs.
//
// The reference's kernel for this case: csrc/int8_linear_kernels.cu:238-431 (one token),
// csrc/int8_gateup_kernels.cu:255-520; it has none for more than one token.
#include "skinny.cuh"

namespace mui {

constexpr int kI8wThreads = 256;
constexpr int kI8wWaves = kI8wThreads / kWave;

struct Int8WaveArgs {
  const uint16_t* s0; const uint16_t* s1; long s_pitch; int group_shift;
  const uint16_t* add_bias; const uint16_t* residual; long x_pitch;
};

// sum over the four 16-lane rows of a wave, the same value in all four (row swaps in the vector
// ALU: rows (0, 1) and (2, 3) first, then the two halves)
__device__ __forceinline__ float i8w_rows_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

template <int RW, int CH, bool NORM, int EPI, int WF, int TOK>
__global__ void __launch_bounds__(kI8wThreads) int8_wave_kernel(
    // scalars, hottest first (preloaded into SGPRs at wave launch)
    const uint8_t* w0, const uint8_t* w1, long pitch, const uint16_t* x, const uint16_t* gamma,
    uint16_t* y, int n, int k, int tokens, float eps, const Int8WaveArgs a) {
  using T = F16;
  constexpr int RR = (EPI == SK_GATEUP) ? 2 * RW : RW;  // weight rows a wave has in flight
  // values a wave reduces per step, in NH halves of NVH: linear -> value r * TOK + tk; gate/up ->
  // half 0 holds the gate sums, half 1 the up sums, both at index p * TOK + tk, so that the lane
  // that finishes output (p, tk) finds both in its own registers
  constexpr int NV = RR * TOK;
  constexpr int NH = (EPI == SK_GATEUP) ? 2 : (NV > 16 ? 2 : 1);
  constexpr int NVH = NV / NH;
  static_assert(NVH == 2 || NVH == 4 || NVH == 8 || NVH == 16, "2..16 values per reduction");
  constexpr uint32_t kFlip = (WF == WF_I8_CHANNEL) ? 0x80808080u : 0u;
  constexpr float kOffset = (WF == WF_I8_CHANNEL) ? 1152.f : 1024.f;

  const int lane = threadIdx.x & (kWave - 1);
  const int gw = blockIdx.x * kI8wWaves + (threadIdx.x >> 6);  // this wave among all waves
  const int n_waves = gridDim.x * kI8wWaves;
  const int kc = k >> 4;  // 16-byte chunks (16 weights) per row
  const int n_units = (n + RW - 1) / RW;

  int coff[CH];
  bool cvalid[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = lane + kWave * j;
    cvalid[j] = c < kc;
    coff[j] = cvalid[j] ? (c << 4) : 0;
  }

  // the lane that finishes value `eidx` of each half (lanes 0, 16 / NVH, ... of the first 16)
  constexpr int kStep = 16 / NVH;
  const bool elane = lane < 16 && (lane % kStep) == 0;
  const int eidx = lane / kStep;

  u32x4 w[RR][CH];
  uint32_t sm[RR][CH];  // group format: packed (scale, min) of the chunk's group
  uint32_t ep_res[NH], ep_s0[NH], ep_s1[NH];
#pragma unroll
  for (int h = 0; h < NH; ++h) ep_res[h] = ep_s0[h] = ep_s1[h] = 0;

  auto issue = [&](int u) {
#pragma unroll
    for (int r = 0; r < RR; ++r) {
      int row;
      const uint8_t* base;
      const uint16_t* sbase;
      if constexpr (EPI == SK_GATEUP) {
        row = u * RW + (r >> 1);
        base = (r & 1) ? w1 : w0;
        sbase = (r & 1) ? a.s1 : a.s0;
      } else {
        row = u * RW + r;
        base = w0;
        sbase = a.s0;
      }
      row = row < n ? row : n - 1;
      const uint8_t* rp = base + (long)row * pitch;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        w[r][j] = ld16_stream(rp + coff[j]);
        if constexpr (WF == WF_U8_GROUP)
          sm[r][j] = ld4(sbase + (long)row * a.s_pitch + 2 * (coff[j] >> a.group_shift));
      }
    }
    // what the finishing lanes need from memory rides along with the weights
    if (elane) {
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        if (EPI == SK_GATEUP && h > 0) continue;  // one output per lane: gate and up share the index
        const int v = (EPI == SK_GATEUP) ? eidx : h * NVH + eidx;
        const int row = u * RW + v / TOK, tk = v % TOK;
        if (row < n && tk < tokens) {
          if constexpr (WF == WF_I8_CHANNEL) {
            ep_s0[h] = ld2(a.s0 + (long)row * a.s_pitch);
            if constexpr (EPI == SK_GATEUP) ep_s1[h] = ld2(a.s1 + (long)row * a.s_pitch);
          }
          if constexpr (EPI == SK_LINEAR) {
            if (a.residual) ep_res[h] = ld2(a.residual + (long)tk * n + row);
          }
        }
      }
    }
  };

  // ---- token operands: gamma * x as packed fp16 (requested before the first weights: loads return
  // in order), the chunk's sum of them on the side. No load sits behind a branch.
  int u = gw;  // the launcher never starts more waves than there are units
  u32x4 xq[TOK][CH][2];
  u32x4 gq[CH][2];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    const long xrow = tk == 0 ? 0 : (long)(tk < tokens ? tk : tokens - 1) * a.x_pitch;
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
  issue(u < n_units ? u : n_units - 1);

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
        float bf[8];
        unpack8<T>(b, bf);
        xsum[tk][j] += ((bf[0] + bf[1]) + (bf[2] + bf[3])) + ((bf[4] + bf[5]) + (bf[6] + bf[7]));
      }
    }
  }
  float acc_init[TOK];  // per-channel: -(1024 + 128) * sum of this lane's operands
  float rs[TOK];
#pragma unroll
  for (int tk = 0; tk < TOK; ++tk) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < CH; ++j) s += xsum[tk][j];
    acc_init[tk] = -kOffset * s;
    rs[tk] = 1.f;
    if constexpr (NORM) rs[tk] = rsqrtf(wave_sum(ss[tk]) / (float)k + eps);  // the wave holds all of x
  }

  for (; u < n_units; u += n_waves) {
    float acc[NH][NVH];
#pragma unroll
    for (int r = 0; r < RR; ++r) {
      float ar[TOK];
#pragma unroll
      for (int tk = 0; tk < TOK; ++tk) ar[tk] = (WF == WF_I8_CHANNEL) ? acc_init[tk] : 0.f;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        // 16 bytes -> 8 packed pairs (1024 + b): pairs 0..3 meet xq[..][0], pairs 4..7 meet xq[..][1]
        const uint32_t wv[4] = {w[r][j].x ^ kFlip, w[r][j].y ^ kFlip, w[r][j].z ^ kFlip, w[r][j].w ^ kFlip};
        uint32_t pr[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          pr[2 * d + 0] = __builtin_amdgcn_perm(0x64646464u, wv[d], 0x04010400u);
          pr[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, wv[d], 0x04030402u);
        }
#pragma unroll
        for (int tk = 0; tk < TOK; ++tk) {
          float s = (WF == WF_I8_CHANNEL) ? ar[tk] : 0.f;
          // (components go through scalars: a bit cast applied directly to a vector component was
          // compiled as a read of component 0 by this toolchain)
          const u32x4 q0 = xq[tk][j][0], q1 = xq[tk][j][1];
          const uint32_t qa[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
          for (int d = 0; d < 8; ++d)
            s = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pr[d]), __builtin_bit_cast(f16x2, qa[d]), s, false);
          if constexpr (WF == WF_I8_CHANNEL) {
            ar[tk] = s;
          } else {
            // w = u8 * scale + min over this chunk's group: scale * (s - 1024 xsum) + min * xsum
            const float sc = T::lo(sm[r][j]), mn = T::hi(sm[r][j]);
            ar[tk] = fmaf(sc, fmaf(-kOffset, xsum[tk][j], s), fmaf(mn, xsum[tk][j], ar[tk]));
          }
        }
      }
#pragma unroll
      for (int tk = 0; tk < TOK; ++tk) {
        if constexpr (EPI == SK_GATEUP) {
          acc[r & 1][(r >> 1) * TOK + tk] = ar[tk];
        } else {
          const int v = r * TOK + tk;
          acc[v / NVH][v % NVH] = ar[tk];
        }
      }
    }
    uint32_t cur_res[NH], cur_s0[NH], cur_s1[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) { cur_res[h] = ep_res[h]; cur_s0[h] = ep_s0[h]; cur_s1[h] = ep_s1[h]; }
    const int cur = u;
    const int nxt = u + n_waves;
    if (nxt < n_units) issue(nxt);  // keep the memory pipe full during the reduction

    float tot[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      row16_reduce_scatter<NVH>(acc[h], lane);
      tot[h] = i8w_rows_sum(acc[h][0]);
    }
    if (elane) {
      if constexpr (EPI == SK_GATEUP) {
        const int row = cur * RW + eidx / TOK, tk = eidx % TOK;
        if (row < n && tk < tokens) {
          float rsv = rs[0];
#pragma unroll
          for (int i = 1; i < TOK; ++i) rsv = (tk == i) ? rs[i] : rsv;
          float g = tot[0] * rsv, up = tot[1] * rsv;
          if constexpr (WF == WF_I8_CHANNEL) {
            g *= T::one((uint16_t)cur_s0[0]);
            up *= T::one((uint16_t)cur_s1[0]);
          }
          y[(long)tk * n + row] = T::pack(silu_f32(g) * up);
        }
      } else {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
          const int v = h * NVH + eidx;
          const int row = cur * RW + v / TOK, tk = v % TOK;
          if (row < n && tk < tokens) {
            float rsv = rs[0];
#pragma unroll
            for (int i = 1; i < TOK; ++i) rsv = (tk == i) ? rs[i] : rsv;
            float val = tot[h] * rsv;
            if constexpr (WF == WF_I8_CHANNEL) val *= T::one((uint16_t)cur_s0[h]);
            if (a.add_bias) val += T::one(a.add_bias[row]);
            if (a.residual) val += T::one((uint16_t)cur_res[h]);
            y[(long)tk * n + row] = T::pack(val);
          }
        }
      }
    }
  }
}

static int g_int8_wave_per_cu = 0;  // 0: built-in choice of workgroups per CU

template <int RW, int CH, int EPI, int WF, int TOK>
static int launch_i8w_rc(hipStream_t s, const SkinnyParams& p) {
  const int n_units = ceil_div(p.n, RW);
  const int wg_units = ceil_div(n_units, kI8wWaves);  // a workgroup is four independent waves
  const int per_cu = g_int8_wave_per_cu > 0 ? g_int8_wave_per_cu : (TOK >= 4 ? 2 : 3);
  const int grid = balanced_grid(wg_units, per_cu);
  Int8WaveArgs a = {p.s0, p.s1, p.s_pitch, p.group_shift, p.add_bias, p.residual,
                    p.x_pitch > 0 ? p.x_pitch : (long)p.k};
#define MUI_I8W_LAUNCH(NORMV)                                                                             \
  hipLaunchKernelGGL((int8_wave_kernel<RW, CH, NORMV, EPI, WF, TOK>), dim3(grid), dim3(kI8wThreads), 0, s, \
                     (const uint8_t*)p.w0, (const uint8_t*)p.w1, p.pitch, p.x, p.gamma, p.y, p.n, p.k,     \
                     p.tokens, p.eps, a)
  if (p.gamma) MUI_I8W_LAUNCH(true); else MUI_I8W_LAUNCH(false);
#undef MUI_I8W_LAUNCH
  return launch_status();
}

template <int EPI, int WF, int TOK>
static int launch_i8w_t(hipStream_t s, const SkinnyParams& p) {
  // rows (pairs) per wave and step: eight 16-byte loads per lane in flight on 4096-byte rows, and at
  // least two values per reduction
  constexpr int RW = (EPI == SK_GATEUP) ? (TOK == 1 ? 2 : 1) : 2;
  const int ch = ceil_div(p.k >> 4, kWave);
  if (ch <= 2) return launch_i8w_rc<RW, 2, EPI, WF, TOK>(s, p);
  if (ch <= 4) return launch_i8w_rc<RW, 4, EPI, WF, TOK>(s, p);
  return MUI_ERR_UNSUPPORTED;
}

void int8_wave_set_per_cu(int per_cu) { g_int8_wave_per_cu = per_cu; }

// 1..4 fp16 tokens on rows of at most 4096 int8 weights; MUI_ERR_UNSUPPORTED for anything else
int launch_int8_wave(hipStream_t s, int dtype, int wf, int epilogue, const SkinnyParams& p) {
  if (dtype != MUI_DTYPE_F16 || p.tokens < 1 || p.tokens > 4 || p.mul_bias) return MUI_ERR_UNSUPPORTED;
  if (p.k > 4 * 16 * kWave || p.n < 1) return MUI_ERR_UNSUPPORTED;
#define MUI_I8W_CASE(WFV, EPIV)                                          \
  if (wf == WFV && epilogue == EPIV) {                                   \
    if (p.tokens <= 1) return launch_i8w_t<EPIV, WFV, 1>(s, p);          \
    if (p.tokens <= 2) return launch_i8w_t<EPIV, WFV, 2>(s, p);          \
    return launch_i8w_t<EPIV, WFV, 4>(s, p);                             \
  }
  MUI_I8W_CASE(WF_I8_CHANNEL, SK_LINEAR)
  MUI_I8W_CASE(WF_I8_CHANNEL, SK_GATEUP)
  MUI_I8W_CASE(WF_U8_GROUP, SK_LINEAR)
  MUI_I8W_CASE(WF_U8_GROUP, SK_GATEUP)
#undef MUI_I8W_CASE
  return MUI_ERR_UNSUPPORTED;
}

}  // namespace mui
