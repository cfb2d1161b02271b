// Weight-only int8 GEMVs for one token, dequantisation fused into the weight stream.
//
// Two on-device formats:
//   FMT_CHANNEL  int8 [N, K] + one 16-bit scale per output row (symmetric, s = max|row|/127).
//                y[n] = s[n] * sum_k q[n,k] xn[k].  The scale is applied once per row in the
//                epilogue; the inner loop is integer->fp32 convert + fma only.
//   FMT_GROUP    the reference's RTN format (muillm/quantization/rtnquantizer.py:49-88):
//                uint8 [N, K] + (scale, min) 16-bit pairs per group of 2^shift inputs,
//                w = u8 * scale + min, accumulated as scale * sum(u8 x) + min * sum(x) per
//                group like csrc/int8_linear_kernels.cu:213-236.
// Reference kernels: csrc/int8_linear_kernels.cu:238-697 (GEMV), csrc/int8_gateup_kernels.cu:255-865
// (gate/up + SiLU), csrc/int8_dequantization_kernel.cu:74-150 (dequantise).
//
// Same workgroup shape as the 16-bit GEMV (4 wave64s, thread t owns 16-byte chunks
// t, t+256, ... of every row, xn in fp32 registers) but a chunk now carries 16 weights, so
// twice as many rows are kept in flight to have the same bytes outstanding per thread.
// Signed bytes are converted with the unsigned byte->float instruction after flipping the
// sign bit (q + 128), and the 128 * sum(x) correction is folded into the accumulator's
// initial value, so dequantisation costs one VALU op per weight.
#include "common.cuh"
#include "skinny.cuh"

namespace mui {

enum { FMT_CHANNEL = 0, FMT_GROUP = 1 };
enum { EPI8_LINEAR = 0, EPI8_GATEUP = 1 };

struct Int8Params {
  const uint8_t* w0;   // linear: the matrix; gate/up: gate rows
  const uint8_t* w1;   // gate/up: up rows
  long pitch;          // row pitch in bytes
  const uint16_t* s0;  // CHANNEL: scale of row n at s0[n * s_pitch]; GROUP: pairs at s0 + n*s_pitch + 2g
  const uint16_t* s1;  // same for the up rows
  long s_pitch;        // in 16-bit elements
  int group_shift;     // GROUP only
  const uint16_t* x;
  const uint16_t* gamma;
  const uint16_t* add_bias;
  const uint16_t* residual;
  uint16_t* y;
  int n;
  int k;
  float eps;
};

constexpr int kThreads8 = 256;
constexpr int kWaves8 = kThreads8 / kWave;

// 16 weights of one chunk -> fp32; `bias` is 0x80808080 for signed storage (value + 128)
__device__ __forceinline__ void unpack16_u8(const u32x4 w, uint32_t flip, float (&f)[16]) {
  const uint32_t v[4] = {w.x ^ flip, w.y ^ flip, w.z ^ flip, w.w ^ flip};
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    f[4 * m + 0] = (float)(v[m] & 0xffu);
    f[4 * m + 1] = (float)((v[m] >> 8) & 0xffu);
    f[4 * m + 2] = (float)((v[m] >> 16) & 0xffu);
    f[4 * m + 3] = (float)(v[m] >> 24);
  }
}

template <typename T, int R, int CH, bool NORM, int EPI, int FMT>
__global__ void __launch_bounds__(kThreads8) int8_gemv_kernel(
    // scalars, hottest first: the first 16 argument dwords are preloaded into SGPRs at wave launch
    const uint8_t* a_w0, const uint8_t* a_w1, long a_pitch, const uint16_t* a_x, const uint16_t* a_gamma,
    uint16_t* a_y, int a_n, int a_k, const uint16_t* a_s0, const uint16_t* a_s1, long a_s_pitch,
    int a_group_shift, float a_eps, const uint16_t* a_add_bias, const uint16_t* a_residual) {
  const Int8Params p = {a_w0, a_w1, a_pitch, a_s0, a_s1, a_s_pitch, a_group_shift, a_x, a_gamma,
                        a_add_bias, a_residual, a_y, a_n, a_k, a_eps};
  constexpr int OUT = (EPI == EPI8_GATEUP) ? R / 2 : R;
  static_assert(EPI != EPI8_GATEUP || (R % 2 == 0), "gate/up needs row pairs");
  constexpr uint32_t kFlip = (FMT == FMT_CHANNEL) ? 0x80808080u : 0u;

  __shared__ float red[2][kWaves8][R];
  __shared__ float red_ss[kWaves8];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int kc = p.k >> 4;  // 16-byte chunks (16 weights) per row
  const int n_groups = (p.n + OUT - 1) / OUT;

  int coff[CH];
  bool cvalid[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = t + kThreads8 * j;
    cvalid[j] = c < kc;
    coff[j] = cvalid[j] ? (c << 4) : 0;
  }

  u32x4 w[R][CH];
  uint32_t sm[R][CH];  // GROUP: packed (scale, min) of the chunk's group
  auto issue = [&](int rg) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row;
      const uint8_t* base;
      const uint16_t* sbase;
      if constexpr (EPI == EPI8_GATEUP) {
        row = rg * OUT + (r >> 1);
        base = (r & 1) ? p.w1 : p.w0;
        sbase = (r & 1) ? p.s1 : p.s0;
      } else {
        row = rg * R + r;
        base = p.w0;
        sbase = p.s0;
      }
      row = row < p.n ? row : p.n - 1;
      const uint8_t* rp = base + (long)row * p.pitch;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        w[r][j] = ld16_stream(rp + coff[j]);
        if constexpr (FMT == FMT_GROUP) {
          const uint16_t* sp = sbase + (long)row * p.s_pitch + 2 * (coff[j] >> p.group_shift);
          sm[r][j] = *(const uint32_t*)sp;
        }
      }
    }
  };

  int rg = blockIdx.x;
  if (rg < n_groups) issue(rg);

  // ---- inputs ----
  float xs[CH][16];
  float xsum[CH];  // sum of the chunk's inputs (offset / min correction)
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    xsum[j] = 0.f;
    if (cvalid[j]) {
#pragma unroll
      for (int hlf = 0; hlf < 2; ++hlf) {
        float xf[8];
        unpack8<T>(ld16(p.x + coff[j] + 8 * hlf), xf);
        if constexpr (NORM) {
          float gf[8];
          unpack8<T>(ld16(p.gamma + coff[j] + 8 * hlf), gf);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            ss = fmaf(xf[i], xf[i], ss);
            xs[j][8 * hlf + i] = xf[i] * gf[i];
          }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) xs[j][8 * hlf + i] = xf[i];
        }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) xsum[j] += xs[j][i];
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) xs[j][i] = 0.f;
    }
  }
  float acc_init = 0.f;  // CHANNEL: -128 * sum of this thread's inputs
  if constexpr (FMT == FMT_CHANNEL) {
#pragma unroll
    for (int j = 0; j < CH; ++j) acc_init -= 128.f * xsum[j];
  }

  float rs = 1.f;
  if constexpr (NORM) {
    ss = wave_sum(ss);
    if (lane == 0) red_ss[wave] = ss;
    __syncthreads();
    const float tot = (red_ss[0] + red_ss[1]) + (red_ss[2] + red_ss[3]);
    rs = rsqrtf(tot / (float)p.k + p.eps);
  }

  int buf = 0;
  for (; rg < n_groups; rg += gridDim.x) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float a = acc_init;
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        float wf[16];
        unpack16_u8(w[r][j], kFlip, wf);
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          a0 = fmaf(wf[i], xs[j][i], a0);
          a1 = fmaf(wf[i + 1], xs[j][i + 1], a1);
        }
        if constexpr (FMT == FMT_GROUP) {
          const float sc = T::lo(sm[r][j]), mn = T::hi(sm[r][j]);
          a = fmaf(sc, a0 + a1, a);
          a = fmaf(mn, xsum[j], a);
        } else {
          a += a0 + a1;
        }
      }
      acc[r] = a;
    }

    const int nxt = rg + gridDim.x;
    if (nxt < n_groups) issue(nxt);

#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) red[buf][wave][r] = acc[r];
    }
    __syncthreads();

    if (t < OUT) {
      const int n = rg * OUT + t;
      if (n < p.n) {
        auto total = [&](int r) {
          return (red[buf][0][r] + red[buf][1][r]) + (red[buf][2][r] + red[buf][3][r]);
        };
        float v;
        if constexpr (EPI == EPI8_GATEUP) {
          float g = total(2 * t) * rs, u = total(2 * t + 1) * rs;
          if constexpr (FMT == FMT_CHANNEL) {
            g *= T::one(p.s0[(long)n * p.s_pitch]);
            u *= T::one(p.s1[(long)n * p.s_pitch]);
          }
          v = silu_f32(g) * u;
        } else {
          v = total(t) * rs;
          if constexpr (FMT == FMT_CHANNEL) v *= T::one(p.s0[(long)n * p.s_pitch]);
          if (p.add_bias) v += T::one(p.add_bias[n]);
          if (p.residual) v += T::one(p.residual[n]);
        }
        p.y[n] = T::pack(v);
      }
    }
    buf ^= 1;
  }
}

// ---------------------------------------------------------------------------------------
// dequantise to a dense 16-bit matrix (bit-exact definitions)
//   CHANNEL: out = T(float(q) * float(s[n]))          -- exact product, one rounding
//   GROUP:   out = T(fma(float(u8), scale, min))      -- csrc/int8_dequantization_kernel.cu:50-59
// one thread per 16-byte chunk of weights, grid-stride.
// ---------------------------------------------------------------------------------------
template <typename T, int FMT>
__global__ void __launch_bounds__(256) int8_dequant_kernel(
    const uint8_t* q, long q_pitch, const uint16_t* s, long s_pitch, int group_shift,
    uint16_t* out, long out_pitch, int n, int k) {
  const int kc = k >> 4;
  const long total = (long)n * kc;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int row = (int)(idx / kc);
    const int c = (int)(idx - (long)row * kc);
    const u32x4 wv = ld16_stream(q + (long)row * q_pitch + ((long)c << 4));
    const uint32_t v[4] = {wv.x, wv.y, wv.z, wv.w};
    float scale, mn = 0.f;
    if constexpr (FMT == FMT_CHANNEL) {
      scale = T::one(s[(long)row * s_pitch]);
    } else {
      const uint32_t pr = *(const uint32_t*)(s + (long)row * s_pitch + 2 * ((c << 4) >> group_shift));
      scale = T::lo(pr);
      mn = T::hi(pr);
    }
    float o[16];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte = (v[m] >> (8 * b)) & 0xffu;
        if constexpr (FMT == FMT_CHANNEL) {
          o[4 * m + b] = (float)(int)(int8_t)byte * scale;
        } else {
          o[4 * m + b] = __builtin_fmaf((float)byte, scale, mn);
        }
      }
    }
    float lo8[8], hi8[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { lo8[i] = o[i]; hi8[i] = o[8 + i]; }
    uint16_t* op = out + (long)row * out_pitch + ((long)c << 4);
    *(u32x4*)op = pack8<T>(lo8);
    *(u32x4*)(op + 8) = pack8<T>(hi8);
  }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
// fp16 activations: a single token also takes the packed-dot kernel of int8_multi.hip (measured
// 5-15 % faster than the convert + fma kernel below, which remains the bf16 path)
static int g_int8_dot2 = 1;
static int g_int8_wgs_per_cu = 0;
static int g_int8_rows = 0;

template <typename T, int R, int CH, int EPI, int FMT>
static int launch8_rc(hipStream_t s, const Int8Params& p, int grid) {
  if (p.gamma)
    hipLaunchKernelGGL((int8_gemv_kernel<T, R, CH, true, EPI, FMT>), dim3(grid), dim3(kThreads8), 0, s, p.w0, p.w1,
                       p.pitch, p.x, p.gamma, p.y, p.n, p.k, p.s0, p.s1, p.s_pitch, p.group_shift, p.eps, p.add_bias,
                       p.residual);
  else
    hipLaunchKernelGGL((int8_gemv_kernel<T, R, CH, false, EPI, FMT>), dim3(grid), dim3(kThreads8), 0, s, p.w0, p.w1,
                       p.pitch, p.x, p.gamma, p.y, p.n, p.k, p.s0, p.s1, p.s_pitch, p.group_shift, p.eps, p.add_bias,
                       p.residual);
  return launch_status();
}

template <typename T, int R, int EPI, int FMT>
static int launch8_r(hipStream_t s, const Int8Params& p, int ch) {
  constexpr int OUT = (EPI == EPI8_GATEUP) ? R / 2 : R;
  const int n_groups = ceil_div(p.n, OUT);
  const int per_cu = g_int8_wgs_per_cu > 0 ? g_int8_wgs_per_cu : 3;
  const int grid = balanced_grid(n_groups, per_cu);
  if (ch <= 1) return launch8_rc<T, R, 1, EPI, FMT>(s, p, grid);
  if constexpr (R <= 4) {
    if (ch <= 2) return launch8_rc<T, R, 2, EPI, FMT>(s, p, grid);
  }
  if constexpr (R <= 2) {
    if (ch <= 4) return launch8_rc<T, R, 4, EPI, FMT>(s, p, grid);
  }
  return MUI_ERR_UNSUPPORTED;
}

template <typename T, int EPI, int FMT>
static int launch8_t(hipStream_t s, const Int8Params& p) {
  const int ch = ceil_div(p.k >> 4, kThreads8);
  int rows = g_int8_rows;
  if (rows == 0 || rows == 16) rows = ch > 1 ? 4 : 8;
  if (rows == 8 && ch == 1) return launch8_r<T, 8, EPI, FMT>(s, p, ch);
  if (rows >= 4 && ch <= 2) return launch8_r<T, 4, EPI, FMT>(s, p, ch);
  return launch8_r<T, 2, EPI, FMT>(s, p, ch);
}

template <int EPI, int FMT>
static int launch8(hipStream_t s, int dtype, const Int8Params& p) {
  if (dtype == MUI_DTYPE_F16) return launch8_t<F16, EPI, FMT>(s, p);
  if (dtype == MUI_DTYPE_BF16) return launch8_t<BF16, EPI, FMT>(s, p);
  return MUI_ERR_INVALID_ARG;
}

static int check_int8_common(int dtype, const void* w, long pitch, const void* x,
                             const void* gamma, int n, int k, int tokens, bool any_token_count = false) {
  if (!(w && x)) return MUI_ERR_INVALID_ARG;
  if (!(n > 0 && k > 0 && tokens > 0)) return MUI_ERR_INVALID_ARG;
  if (!(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16)) return MUI_ERR_INVALID_ARG;
  if (tokens > MUI_MAX_TOKENS && !any_token_count) return MUI_ERR_UNSUPPORTED;
  if (pitch < k) return MUI_ERR_INVALID_ARG;
  if ((k & 15) || (pitch & 15)) return MUI_ERR_UNSUPPORTED;
  if (!aligned16(w) || !aligned16(x) || (gamma && !aligned16(gamma))) return MUI_ERR_ALIGNMENT;
  return MUI_OK;
}

}  // namespace mui

using namespace mui;

namespace mui {
void int8_set_packed_dot(bool on) { g_int8_dot2 = on ? 1 : 0; }
int int8_tuned_wgs_per_cu() { return g_int8_wgs_per_cu; }
int int8_tuned_rows() { return g_int8_rows; }
}  // namespace mui

extern "C" int mui_tune_int8(int rows, int wgs_per_cu) {
  MUI_TUNE_GUARD();
  if (!(rows == 0 || rows == 2 || rows == 4 || rows == 8 || rows == 16)) return MUI_ERR_INVALID_ARG;
  if (wgs_per_cu < 0 || wgs_per_cu > 32) return MUI_ERR_INVALID_ARG;
  g_int8_rows = rows;
  g_int8_wgs_per_cu = wgs_per_cu;
  return MUI_OK;
}

extern "C" int mui_int8_linear(mui_stream_t stream, int dtype, const void* weights_i8, long w_pitch,
                               const void* scales, const void* x, const void* norm_weights,
                               float epsilon, const void* add_bias, const void* residual, void* y,
                               int n_out, int k_in, int tokens) {
  int st = check_int8_common(dtype, weights_i8, w_pitch, x, norm_weights, n_out, k_in, tokens, true);
  if (st != MUI_OK) return st;
  MUI_CHECK_ARG(scales && y);
  hipStream_t s = (hipStream_t)stream;
  if (tokens > MUI_MAX_TOKENS) {  // a prompt: the tiled matrix-core GEMM, codes converted on the way to LDS
    SkinnyParams sp = {};
    sp.w0 = weights_i8; sp.pitch = w_pitch; sp.s0 = (const uint16_t*)scales; sp.s_pitch = 1;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.add_bias = (const uint16_t*)add_bias; sp.residual = (const uint16_t*)residual;
    sp.y = (uint16_t*)y; sp.n = n_out; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_prefill_gemm(s, dtype, WF_I8_CHANNEL, SK_LINEAR, sp);
  }
  if (tokens >= 2 || (g_int8_dot2 && dtype == MUI_DTYPE_F16)) {
    SkinnyParams sp = {};
    sp.w0 = weights_i8; sp.pitch = w_pitch; sp.s0 = (const uint16_t*)scales; sp.s_pitch = 1;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.add_bias = (const uint16_t*)add_bias; sp.residual = (const uint16_t*)residual;
    sp.y = (uint16_t*)y; sp.n = n_out; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_skinny(s, dtype, WF_I8_CHANNEL, SK_LINEAR, sp);
  }
  for (int tkn = 0; tkn < tokens; ++tkn) {
    Int8Params p = {};
    p.w0 = (const uint8_t*)weights_i8;
    p.pitch = w_pitch;
    p.s0 = (const uint16_t*)scales;
    p.s_pitch = 1;
    p.x = (const uint16_t*)x + (long)tkn * k_in;
    p.gamma = (const uint16_t*)norm_weights;
    p.add_bias = (const uint16_t*)add_bias;
    p.residual = residual ? (const uint16_t*)residual + (long)tkn * n_out : nullptr;
    p.y = (uint16_t*)y + (long)tkn * n_out;
    p.n = n_out;
    p.k = k_in;
    p.eps = epsilon;
    st = launch8<EPI8_LINEAR, FMT_CHANNEL>(s, dtype, p);
    if (st != MUI_OK) return st;
  }
  return MUI_OK;
}

extern "C" int mui_int8_gateup_silu(mui_stream_t stream, int dtype, const void* gate_i8,
                                    const void* up_i8, long gu_pitch, const void* gate_scales,
                                    const void* up_scales, long scale_stride, const void* x,
                                    const void* norm_weights, float epsilon, void* h, int n_inter,
                                    int k_in, int tokens) {
  int st = check_int8_common(dtype, gate_i8, gu_pitch, x, norm_weights, n_inter, k_in, tokens, true);
  if (st != MUI_OK) return st;
  MUI_CHECK_ARG(up_i8 && gate_scales && up_scales && h && scale_stride >= 1);
  if (!aligned16(up_i8)) return MUI_ERR_ALIGNMENT;
  hipStream_t s = (hipStream_t)stream;
  if (tokens > MUI_MAX_TOKENS) {
    SkinnyParams sp = {};
    sp.w0 = gate_i8; sp.w1 = up_i8; sp.pitch = gu_pitch;
    sp.s0 = (const uint16_t*)gate_scales; sp.s1 = (const uint16_t*)up_scales; sp.s_pitch = scale_stride;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.y = (uint16_t*)h; sp.n = n_inter; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_prefill_gemm(s, dtype, WF_I8_CHANNEL, SK_GATEUP, sp);
  }
  if (tokens >= 2 || (g_int8_dot2 && dtype == MUI_DTYPE_F16)) {
    SkinnyParams sp = {};
    sp.w0 = gate_i8; sp.w1 = up_i8; sp.pitch = gu_pitch;
    sp.s0 = (const uint16_t*)gate_scales; sp.s1 = (const uint16_t*)up_scales; sp.s_pitch = scale_stride;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.y = (uint16_t*)h; sp.n = n_inter; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_skinny(s, dtype, WF_I8_CHANNEL, SK_GATEUP, sp);
  }
  for (int tkn = 0; tkn < tokens; ++tkn) {
    Int8Params p = {};
    p.w0 = (const uint8_t*)gate_i8;
    p.w1 = (const uint8_t*)up_i8;
    p.pitch = gu_pitch;
    p.s0 = (const uint16_t*)gate_scales;
    p.s1 = (const uint16_t*)up_scales;
    p.s_pitch = scale_stride;
    p.x = (const uint16_t*)x + (long)tkn * k_in;
    p.gamma = (const uint16_t*)norm_weights;
    p.y = (uint16_t*)h + (long)tkn * n_inter;
    p.n = n_inter;
    p.k = k_in;
    p.eps = epsilon;
    st = launch8<EPI8_GATEUP, FMT_CHANNEL>(s, dtype, p);
    if (st != MUI_OK) return st;
  }
  return MUI_OK;
}

extern "C" int mui_int8_group_linear(mui_stream_t stream, int dtype, const void* weights_u8,
                                     long w_pitch, const void* scales_min_vals, int group_size_shift,
                                     const void* x, const void* norm_weights, float epsilon,
                                     const void* add_bias, const void* residual, void* y, int n_out,
                                     int k_in, int tokens) {
  int st = check_int8_common(dtype, weights_u8, w_pitch, x, norm_weights, n_out, k_in, tokens, true);
  if (st != MUI_OK) return st;
  MUI_CHECK_ARG(scales_min_vals && y);
  if (group_size_shift < 4 || group_size_shift > 30) return MUI_ERR_UNSUPPORTED;
  if (k_in & ((1 << group_size_shift) - 1)) return MUI_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  if (tokens > MUI_MAX_TOKENS) {  // a prompt: the tiled matrix-core GEMM, codes dequantised on the way to LDS
    SkinnyParams sp = {};
    sp.w0 = weights_u8; sp.pitch = w_pitch; sp.s0 = (const uint16_t*)scales_min_vals;
    sp.s_pitch = 2L * (k_in >> group_size_shift); sp.group_shift = group_size_shift;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.add_bias = (const uint16_t*)add_bias; sp.residual = (const uint16_t*)residual;
    sp.y = (uint16_t*)y; sp.n = n_out; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_prefill_gemm(s, dtype, WF_U8_GROUP, SK_LINEAR, sp);
  }
  if (tokens >= 2 || (g_int8_dot2 && dtype == MUI_DTYPE_F16)) {
    SkinnyParams sp = {};
    sp.w0 = weights_u8; sp.pitch = w_pitch; sp.s0 = (const uint16_t*)scales_min_vals;
    sp.s_pitch = 2L * (k_in >> group_size_shift); sp.group_shift = group_size_shift;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.add_bias = (const uint16_t*)add_bias; sp.residual = (const uint16_t*)residual;
    sp.y = (uint16_t*)y; sp.n = n_out; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_skinny(s, dtype, WF_U8_GROUP, SK_LINEAR, sp);
  }
  for (int tkn = 0; tkn < tokens; ++tkn) {
    Int8Params p = {};
    p.w0 = (const uint8_t*)weights_u8;
    p.pitch = w_pitch;
    p.s0 = (const uint16_t*)scales_min_vals;
    p.s_pitch = 2L * (k_in >> group_size_shift);
    p.group_shift = group_size_shift;
    p.x = (const uint16_t*)x + (long)tkn * k_in;
    p.gamma = (const uint16_t*)norm_weights;
    p.add_bias = (const uint16_t*)add_bias;
    p.residual = residual ? (const uint16_t*)residual + (long)tkn * n_out : nullptr;
    p.y = (uint16_t*)y + (long)tkn * n_out;
    p.n = n_out;
    p.k = k_in;
    p.eps = epsilon;
    st = launch8<EPI8_LINEAR, FMT_GROUP>(s, dtype, p);
    if (st != MUI_OK) return st;
  }
  return MUI_OK;
}

extern "C" int mui_int8_group_gateup_silu(mui_stream_t stream, int dtype, const void* gate_u8,
                                          const void* up_u8, long gu_pitch, const void* gate_smv,
                                          const void* up_smv, long smv_pitch, int group_size_shift,
                                          const void* x, const void* norm_weights, float epsilon,
                                          void* h, int n_inter, int k_in, int tokens) {
  int st = check_int8_common(dtype, gate_u8, gu_pitch, x, norm_weights, n_inter, k_in, tokens, true);
  if (st != MUI_OK) return st;
  MUI_CHECK_ARG(up_u8 && gate_smv && up_smv && h);
  if (!aligned16(up_u8)) return MUI_ERR_ALIGNMENT;
  if (group_size_shift < 4 || group_size_shift > 30) return MUI_ERR_UNSUPPORTED;
  if (k_in & ((1 << group_size_shift) - 1)) return MUI_ERR_UNSUPPORTED;
  if (smv_pitch < 2L * (k_in >> group_size_shift) || (smv_pitch & 1)) return MUI_ERR_INVALID_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (tokens > MUI_MAX_TOKENS) {
    SkinnyParams sp = {};
    sp.w0 = gate_u8; sp.w1 = up_u8; sp.pitch = gu_pitch;
    sp.s0 = (const uint16_t*)gate_smv; sp.s1 = (const uint16_t*)up_smv; sp.s_pitch = smv_pitch;
    sp.group_shift = group_size_shift;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.y = (uint16_t*)h; sp.n = n_inter; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_prefill_gemm(s, dtype, WF_U8_GROUP, SK_GATEUP, sp);
  }
  if (tokens >= 2 || (g_int8_dot2 && dtype == MUI_DTYPE_F16)) {
    SkinnyParams sp = {};
    sp.w0 = gate_u8; sp.w1 = up_u8; sp.pitch = gu_pitch;
    sp.s0 = (const uint16_t*)gate_smv; sp.s1 = (const uint16_t*)up_smv; sp.s_pitch = smv_pitch;
    sp.group_shift = group_size_shift;
    sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.y = (uint16_t*)h; sp.n = n_inter; sp.k = k_in; sp.tokens = tokens; sp.eps = epsilon;
    return launch_skinny(s, dtype, WF_U8_GROUP, SK_GATEUP, sp);
  }
  for (int tkn = 0; tkn < tokens; ++tkn) {
    Int8Params p = {};
    p.w0 = (const uint8_t*)gate_u8;
    p.w1 = (const uint8_t*)up_u8;
    p.pitch = gu_pitch;
    p.s0 = (const uint16_t*)gate_smv;
    p.s1 = (const uint16_t*)up_smv;
    p.s_pitch = smv_pitch;
    p.group_shift = group_size_shift;
    p.x = (const uint16_t*)x + (long)tkn * k_in;
    p.gamma = (const uint16_t*)norm_weights;
    p.y = (uint16_t*)h + (long)tkn * n_inter;
    p.n = n_inter;
    p.k = k_in;
    p.eps = epsilon;
    st = launch8<EPI8_GATEUP, FMT_GROUP>(s, dtype, p);
    if (st != MUI_OK) return st;
  }
  return MUI_OK;
}

extern "C" int mui_int8_dequantize(mui_stream_t stream, int dtype, const void* weights_i8,
                                   long w_pitch, const void* scales, long scale_stride, void* out,
                                   long out_pitch, int n, int k) {
  MUI_CHECK_ARG(weights_i8 && scales && out && n > 0 && k > 0 && scale_stride >= 1);
  if ((k & 15) || (w_pitch & 15) || (out_pitch & 7)) return MUI_ERR_UNSUPPORTED;
  if (w_pitch < k || out_pitch < k) return MUI_ERR_INVALID_ARG;
  if (!aligned16(weights_i8) || !aligned16(out)) return MUI_ERR_ALIGNMENT;
  const long chunks = (long)n * (k >> 4);
  const int grid = (int)((chunks + 255) / 256 < 65536 ? (chunks + 255) / 256 : 65536);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((int8_dequant_kernel<F16, FMT_CHANNEL>), dim3(grid), dim3(256), 0, s,
                       (const uint8_t*)weights_i8, w_pitch, (const uint16_t*)scales, scale_stride, 0,
                       (uint16_t*)out, out_pitch, n, k);
  else if (dtype == MUI_DTYPE_BF16)
    hipLaunchKernelGGL((int8_dequant_kernel<BF16, FMT_CHANNEL>), dim3(grid), dim3(256), 0, s,
                       (const uint8_t*)weights_i8, w_pitch, (const uint16_t*)scales, scale_stride, 0,
                       (uint16_t*)out, out_pitch, n, k);
  else
    return MUI_ERR_INVALID_ARG;
  return launch_status();
}

extern "C" int mui_int8_group_dequantize(mui_stream_t stream, int dtype, const void* weights_u8,
                                         long w_pitch, const void* scales_min_vals, long smv_pitch,
                                         int group_size_shift, void* out, long out_pitch, int n, int k) {
  MUI_CHECK_ARG(weights_u8 && scales_min_vals && out && n > 0 && k > 0);
  if ((k & 15) || (w_pitch & 15) || (out_pitch & 7)) return MUI_ERR_UNSUPPORTED;
  if (group_size_shift < 4 || group_size_shift > 30) return MUI_ERR_UNSUPPORTED;
  if (k & ((1 << group_size_shift) - 1)) return MUI_ERR_UNSUPPORTED;
  if (w_pitch < k || out_pitch < k) return MUI_ERR_INVALID_ARG;
  if (smv_pitch < 2L * (k >> group_size_shift) || (smv_pitch & 1)) return MUI_ERR_INVALID_ARG;
  if (!aligned16(weights_u8) || !aligned16(out)) return MUI_ERR_ALIGNMENT;
  const long chunks = (long)n * (k >> 4);
  const int grid = (int)((chunks + 255) / 256 < 65536 ? (chunks + 255) / 256 : 65536);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((int8_dequant_kernel<F16, FMT_GROUP>), dim3(grid), dim3(256), 0, s,
                       (const uint8_t*)weights_u8, w_pitch, (const uint16_t*)scales_min_vals, smv_pitch,
                       group_size_shift, (uint16_t*)out, out_pitch, n, k);
  else if (dtype == MUI_DTYPE_BF16)
    hipLaunchKernelGGL((int8_dequant_kernel<BF16, FMT_GROUP>), dim3(grid), dim3(256), 0, s,
                       (const uint8_t*)weights_u8, w_pitch, (const uint16_t*)scales_min_vals, smv_pitch,
                       group_size_shift, (uint16_t*)out, out_pitch, n, k);
  else
    return MUI_ERR_INVALID_ARG;
  return launch_status();
}

// ---------------------------------------------------------------------------------------
// One-time conversion of the reference's packed gate/up format into the row-interleaved one the
// kernels stream: weights [N, K, 2] (gate and up of one input feature adjacent,
// muillm/modules/quantized/int8gateupdownmlp.py:211-230) -> [N, 2, K]; (scale, min) pairs
// [N * G, 2, 2] (group, gate|up, scale|min) -> [N, 2, G, 2]. One thread moves 16 input bytes
// (8 gate + 8 up codes); the first N * G * 2 threads also move one (scale, min) pair each.
// ---------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) int8_repack_gateup_kernel(const uint8_t* in, const uint32_t* smv_in,
                                                                 uint8_t* out, uint32_t* smv_out, int n, int k,
                                                                 int groups) {
  const long total = (long)n * (k >> 3);  // 16-byte input chunks
  const long pairs = (long)n * groups * 2;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / (k >> 3);
    const int c = (int)(idx - row * (k >> 3));  // covers input features 8c .. 8c+7
    const u32x4 v = *(const u32x4*)(in + row * 2L * k + ((long)c << 4));
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t g[2], u[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      // dword = (g0, u0, g1, u1): even bytes are gate codes, odd bytes up codes
      g[h] = __builtin_amdgcn_perm(w[2 * h + 1], w[2 * h], 0x06040200u);
      u[h] = __builtin_amdgcn_perm(w[2 * h + 1], w[2 * h], 0x07050301u);
    }
    uint32_t* go = (uint32_t*)(out + row * 2L * k + ((long)c << 3));
    uint32_t* uo = (uint32_t*)(out + row * 2L * k + k + ((long)c << 3));
    go[0] = g[0]; go[1] = g[1];
    uo[0] = u[0]; uo[1] = u[1];
    if (smv_in && idx < pairs) {
      // idx enumerates the input pairs (row, group, which)
      const long r = idx / (2L * groups);
      const int rem = (int)(idx - r * 2L * groups);
      const int grp = rem >> 1, which = rem & 1;
      smv_out[(r * 2 + which) * groups + grp] = smv_in[idx];
    }
  }
}

extern "C" int mui_int8_repack_gateup(mui_stream_t stream, const void* gate_up_nk2, const void* smv_ng22,
                                      int group_size_shift, void* gate_up_n2k, void* smv_n2g2, int n_inter,
                                      int k_in) {
  MUI_CHECK_ARG(gate_up_nk2 && gate_up_n2k && n_inter > 0 && k_in > 0);
  MUI_CHECK_ARG((smv_ng22 == nullptr) == (smv_n2g2 == nullptr));
  MUI_CHECK_ARG(gate_up_nk2 != gate_up_n2k && (smv_ng22 == nullptr || smv_ng22 != smv_n2g2));
  if (k_in & 15) return MUI_ERR_UNSUPPORTED;
  int groups = 0;
  if (smv_ng22) {
    if (group_size_shift < 4 || group_size_shift > 30 || (k_in & ((1 << group_size_shift) - 1)))
      return MUI_ERR_UNSUPPORTED;
    groups = k_in >> group_size_shift;
    if (((uintptr_t)smv_ng22 & 3) || ((uintptr_t)smv_n2g2 & 3)) return MUI_ERR_ALIGNMENT;
  }
  if (!aligned16(gate_up_nk2) || !aligned16(gate_up_n2k)) return MUI_ERR_ALIGNMENT;
  // every (scale, min) pair needs a thread: 2 G pairs per row against K / 8 chunks per row
  if (2L * groups > (k_in >> 3)) return MUI_ERR_UNSUPPORTED;
  const long chunks = (long)n_inter * (k_in >> 3);
  const int grid = (int)((chunks + 255) / 256 < 65536 ? (chunks + 255) / 256 : 65536);
  hipLaunchKernelGGL(int8_repack_gateup_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)gate_up_nk2, (const uint32_t*)smv_ng22, (uint8_t*)gate_up_n2k,
                     (uint32_t*)smv_n2g2, n_inter, k_in, groups);
  return launch_status();
}
