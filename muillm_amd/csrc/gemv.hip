// Single-token fused GEMV family for gfx950:
//   linear      y = (W . xn) * mul_bias + add_bias + residual
//   gate/up     h = silu(G . xn) * (U . xn)
// with xn = x (plain) or gamma * x * rsqrt(mean(x^2) + eps) (RMSNorm fused in).
//
// Counterpart of the reference's single-token kernels (csrc/linear/linear_fp16_kernels.cu:163-626,
// csrc/ffn/gateup_fp16_kernels.cu:160-604) but laid out for CDNA4:
//   * a workgroup is 4 wave64s; thread t owns the 16-byte weight chunks t, t+256, ... of
//     every row, so each wave-level load instruction covers 1 KiB of contiguous weights and
//     the 4 waves cover 4 KiB -- whole DRAM pages, perfectly coalesced;
//   * gamma*x lives in fp32 registers for the lifetime of the workgroup (CH chunks of 8),
//     loaded once; sum(x^2) is reduced once per workgroup while the first weights are in flight;
//   * R rows are in flight together (R*CH 128-bit loads per thread) and the next row group
//     is requested before the current one is reduced, so a persistent workgroup never
//     drains its memory pipeline;
//   * the k-split is reduced with DPP inside a wave and through LDS across the 4 waves; one
//     barrier per row group (double-buffered LDS);
//   * the rsqrt factor is applied to the finished dot product, not to the 4096 inputs.
#include "common.cuh"
#include "skinny.cuh"

namespace mui {

enum { EPI_LINEAR = 0, EPI_GATEUP = 1 };

struct GemvParams {
  const uint16_t* w0;  // linear: the matrix; gate/up: gate rows
  const uint16_t* w1;  // gate/up: up rows
  long pitch;          // row pitch in elements
  const uint16_t* x;   // [K]
  const uint16_t* gamma;
  const uint16_t* mul_bias;
  const uint16_t* add_bias;
  const uint16_t* residual;
  uint16_t* y;
  int n;  // outputs (rows of W, or gate/up pairs)
  int k;
  float eps;
};

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

// The arguments are scalars, the ones every wave needs first in front: the first 16 dwords
// of the kernel-argument segment are preloaded into SGPRs at wave launch (build flag
// -amdgpu-kernarg-preload-count), so the first weight loads do not wait for a scalar load.
template <typename T, int R, int CH, bool NORM, int EPI>
__global__ void __launch_bounds__(kThreads) gemv_kernel(const uint16_t* a_w0, const uint16_t* a_w1, long a_pitch,
                                                        const uint16_t* a_x, const uint16_t* a_gamma,
                                                        uint16_t* a_y, int a_n, int a_k, float a_eps,
                                                        const uint16_t* a_residual, const uint16_t* a_mul_bias,
                                                        const uint16_t* a_add_bias) {
  const GemvParams p = {a_w0, a_w1, a_pitch, a_x, a_gamma, a_mul_bias, a_add_bias, a_residual, a_y, a_n, a_k, a_eps};
  constexpr int OUT = (EPI == EPI_GATEUP) ? R / 2 : R;  // outputs per row group
  static_assert(EPI != EPI_GATEUP || (R % 2 == 0), "gate/up needs row pairs");

  __shared__ float red[2][kWaves][R];
  __shared__ float red_ss[kWaves];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int kc = p.k >> 3;  // 16-byte chunks per row
  const int n_groups = (p.n + OUT - 1) / OUT;

  // chunk offsets (in elements); chunks past the end of the row are redirected to chunk 0
  // and meet xs == 0 there, so the hot loop has no predication at all.
  int coff[CH];
  bool cvalid[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int c = t + kThreads * j;
    cvalid[j] = c < kc;
    coff[j] = cvalid[j] ? (c << 3) : 0;
  }

  u32x4 w[R][CH];
  auto issue = [&](int rg) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row;
      const uint16_t* base;
      if constexpr (EPI == EPI_GATEUP) {
        row = rg * OUT + (r >> 1);
        base = (r & 1) ? p.w1 : p.w0;
      } else {
        row = rg * R + r;
        base = p.w0;
      }
      row = row < p.n ? row : p.n - 1;  // clamp: result is dropped in the epilogue
      const uint16_t* rp = base + (long)row * p.pitch;
#pragma unroll
      for (int j = 0; j < CH; ++j) w[r][j] = ld16_stream(rp + coff[j]);
    }
  };

  // epilogue operands (biases, residual) of a row group are fetched together with its
  // weights, one group ahead, so no dependent global load sits behind the final barrier
  float e_mb = 1.f, e_ab = 0.f, e_res = 0.f;
  auto issue_epi = [&](int rg) {
    if constexpr (EPI == EPI_LINEAR) {
      if (t < OUT) {
        int n = rg * OUT + t;
        n = n < p.n ? n : p.n - 1;
        e_mb = p.mul_bias ? T::one(p.mul_bias[n]) : 1.f;
        e_ab = p.add_bias ? T::one(p.add_bias[n]) : 0.f;
        e_res = p.residual ? T::one(p.residual[n]) : 0.f;
      }
    }
  };

  int rg = blockIdx.x;
  if (rg < n_groups) {
    issue(rg);  // weights first: they are the long pole
    issue_epi(rg);
  }

  // ---- inputs: gamma * x in fp32 registers, sum of squares on the side ----
  float xs[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    if (cvalid[j]) {
      float xf[8];
      unpack8<T>(ld16(p.x + coff[j]), xf);
      if constexpr (NORM) {
        float gf[8];
        unpack8<T>(ld16(p.gamma + coff[j]), gf);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          ss = fmaf(xf[i], xf[i], ss);
          xs[j][i] = xf[i] * gf[i];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) xs[j][i] = xf[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) xs[j][i] = 0.f;
    }
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
      float a0 = 0.f, a1 = 0.f;  // two chains per row to shorten the dependency
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        float wf[8];
        unpack8<T>(w[r][j], wf);
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
          a0 = fmaf(wf[i], xs[j][i], a0);
          a1 = fmaf(wf[i + 1], xs[j][i + 1], a1);
        }
      }
      acc[r] = a0 + a1;
    }

    const float c_mb = e_mb, c_ab = e_ab, c_res = e_res;
    const int nxt = rg + gridDim.x;
    if (nxt < n_groups) {  // keep the memory pipe full during the reduction
      issue(nxt);
      issue_epi(nxt);
    }

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
        float v;
        if constexpr (EPI == EPI_GATEUP) {
          const int rg_ = 2 * t, ru_ = 2 * t + 1;
          const float g = ((red[buf][0][rg_] + red[buf][1][rg_]) + (red[buf][2][rg_] + red[buf][3][rg_])) * rs;
          const float u = ((red[buf][0][ru_] + red[buf][1][ru_]) + (red[buf][2][ru_] + red[buf][3][ru_])) * rs;
          v = silu_f32(g) * u;
        } else {
          v = ((red[buf][0][t] + red[buf][1][t]) + (red[buf][2][t] + red[buf][3][t])) * rs;
          v = fmaf(v, c_mb, c_ab) + c_res;
        }
        p.y[n] = T::pack(v);
      }
    }
    buf ^= 1;
  }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
struct Tuning {
  int rows_linear = 0;  // 0 = pick per shape; 2 or 4 force R for the linear kernel
  int wgs_per_cu = 0;   // 0 = pick per shape; else cap on workgroups per CU for persistent grids
};
static Tuning g_tune;
int gemv_tuned_wgs_per_cu() { return g_tune.wgs_per_cu; }  // shared with gemv_multi.hip

template <typename T, int R, int CH, int EPI>
static int launch_rc(hipStream_t s, const GemvParams& p, int grid) {
  if (p.gamma)
    hipLaunchKernelGGL((gemv_kernel<T, R, CH, true, EPI>), dim3(grid), dim3(kThreads), 0, s, p.w0, p.w1, p.pitch, p.x,
                       p.gamma, p.y, p.n, p.k, p.eps, p.residual, p.mul_bias, p.add_bias);
  else
    hipLaunchKernelGGL((gemv_kernel<T, R, CH, false, EPI>), dim3(grid), dim3(kThreads), 0, s, p.w0, p.w1, p.pitch, p.x,
                       p.gamma, p.y, p.n, p.k, p.eps, p.residual, p.mul_bias, p.add_bias);
  return launch_status();
}

template <typename T, int R, int EPI>
static int launch_r(hipStream_t s, const GemvParams& p, int ch) {
  constexpr int OUT = (EPI == EPI_GATEUP) ? R / 2 : R;
  const int n_groups = ceil_div(p.n, OUT);
  // measured on MI355X: 2-3 resident workgroups per CU with the next row group prefetched
  // saturate HBM; more only adds tail imbalance.
  int per_cu = g_tune.wgs_per_cu > 0 ? g_tune.wgs_per_cu : (ch > 2 ? 2 : 3);
  const int grid = balanced_grid(n_groups, per_cu);
  if (ch <= 1) return launch_rc<T, R, 1, EPI>(s, p, grid);
  if (ch <= 2) return launch_rc<T, R, 2, EPI>(s, p, grid);
  if (ch <= 4) return launch_rc<T, R, 4, EPI>(s, p, grid);
  if (ch <= 7) return launch_rc<T, R, 7, EPI>(s, p, grid);
  if (ch <= 8) return launch_rc<T, R, 8, EPI>(s, p, grid);
  return MUI_ERR_UNSUPPORTED;
}

template <typename T, int EPI>
static int launch_t(hipStream_t s, const GemvParams& p) {
  const int ch = ceil_div(p.k >> 3, kThreads);
  if (EPI == EPI_GATEUP) {
    // 4 rows = 2 gate/up pairs while a row fits 2 chunks per thread, else one pair
    return ch > 2 ? launch_r<T, 2, EPI>(s, p, ch) : launch_r<T, 4, EPI>(s, p, ch);
  }
  int rows = g_tune.rows_linear;
  if (rows == 0) rows = ch > 2 ? 2 : 4;  // long rows already give 14+ loads in flight at R=2
  return rows == 2 ? launch_r<T, 2, EPI>(s, p, ch) : launch_r<T, 4, EPI>(s, p, ch);
}

template <int EPI>
static int launch_gemv(hipStream_t s, int dtype, const GemvParams& p) {
  if (dtype == MUI_DTYPE_F16) return launch_t<F16, EPI>(s, p);
  if (dtype == MUI_DTYPE_BF16) return launch_t<BF16, EPI>(s, p);
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui

using namespace mui;

// token count from which the MFMA skinny-GEMM kernel takes over (below: one GEMV per token)
static int g_skinny_min_tokens = 2;
// A single fp16 token of a plain linear also takes the packed-dot kernel of gemv_multi.hip
// (gamma * x rounded once to fp16 like HuggingFace's normalised activations, half the multiply
// instructions, half the operand registers): o_proj 8.2 -> 7.0 us, down 20.9 -> 19.2 us, decode
// +3 % on MI355X. The gate/up kernel measured slower that way (36.2 vs 35.5 us) and stays on
// gemv_kernel. bf16 takes the same route with v_dot2_f32_bf16.
static int g_gemv_dot2 = 1;
// largest token count that takes the multi-token GEMV (gemv_multi.hip) instead of the MFMA kernel
// (3-4 tokens measured 1.8 us per decoder layer slower on it than on the MFMA kernel)
static int g_multi_max_tokens = 2;

extern "C" int mui_tune_skinny(int min_tokens, int stream_b, int multi_max_tokens) {
  MUI_TUNE_GUARD();
  if (min_tokens < 1 || min_tokens > MUI_MAX_TOKENS + 1) return MUI_ERR_INVALID_ARG;
  if (multi_max_tokens < 0 || multi_max_tokens > 8) return MUI_ERR_INVALID_ARG;
  g_skinny_min_tokens = min_tokens;
  skinny_set_bstat(stream_b != 1);
  skinny_set_lt(stream_b == 0);
  g_multi_max_tokens = multi_max_tokens == 0 ? 2 : multi_max_tokens;
  skinny_set_int8_multi(g_multi_max_tokens >= 2);
  return MUI_OK;
}

extern "C" int mui_tune_packed_dot(int linear_on, int int8_on) {
  MUI_TUNE_GUARD();
  g_gemv_dot2 = linear_on != 0;
  int8_set_packed_dot(int8_on != 0);
  return MUI_OK;
}

extern "C" int mui_tune_gemv(int rows_linear, int wgs_per_cu) {
  MUI_TUNE_GUARD();
  if (rows_linear >= 100) {  // experiments: 100 + n = fewest row groups per workgroup for two register sets (100: never)
    gemv_multi_set_two(rows_linear - 100);
    rows_linear = 0;
  }
  if (!(rows_linear == 0 || rows_linear == 2 || rows_linear == 4)) return MUI_ERR_INVALID_ARG;
  if (wgs_per_cu < 0 || wgs_per_cu > 32) return MUI_ERR_INVALID_ARG;
  g_tune.rows_linear = rows_linear;
  g_tune.wgs_per_cu = wgs_per_cu;
  return MUI_OK;
}

extern "C" size_t mui_linear_workspace_bytes(void) { return prefill_workspace_bytes(); }

// rows per row group of the single-token kernels (gemv_multi.hip launch_mt_t, int8_multi.hip
// launch_i8m_t at one token) times the row pitch
extern "C" int mui_linear_row_group_bytes(int weight_bits, int k, long pitch_bytes) {
  if (k <= 0 || pitch_bytes <= 0 || !(weight_bits == 16 || weight_bits == 8)) return 0;
  const int chunks = weight_bits == 16 ? ceil_div(k >> 3, 256) : ceil_div(k >> 4, 256);
  const int rows = weight_bits == 16 ? (chunks <= 2 ? 4 : 2) : (chunks <= 1 ? 8 : 2);
  const long bytes = rows * pitch_bytes;
  return bytes > (1 << 30) ? 0 : (int)bytes;
}

extern "C" int mui_linear(mui_stream_t stream, int dtype, const void* weights, long w_pitch,
                          const void* x, const void* norm_weights, float epsilon,
                          const void* mul_bias, const void* add_bias, const void* residual,
                          void* y, int n_out, int k_in, int tokens) {
  return mui_linear_ws(stream, dtype, weights, w_pitch, x, norm_weights, epsilon, mul_bias, add_bias, residual, y,
                       n_out, k_in, tokens, nullptr, 0);
}

extern "C" int mui_linear_ws(mui_stream_t stream, int dtype, const void* weights, long w_pitch,
                             const void* x, const void* norm_weights, float epsilon,
                             const void* mul_bias, const void* add_bias, const void* residual,
                             void* y, int n_out, int k_in, int tokens, void* workspace,
                             size_t workspace_bytes) {
  MUI_CHECK_ARG(weights && x && y);
  MUI_CHECK_ARG(workspace || workspace_bytes == 0);
  MUI_CHECK_ARG(n_out > 0 && k_in > 0 && tokens > 0);
  MUI_CHECK_ARG(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16);
  if (w_pitch < k_in) return MUI_ERR_INVALID_ARG;
  if ((k_in & 7) || (w_pitch & 7)) return MUI_ERR_UNSUPPORTED;
  if (!aligned16(weights) || !aligned16(x) || (norm_weights && !aligned16(norm_weights)))
    return MUI_ERR_ALIGNMENT;

  hipStream_t s = (hipStream_t)stream;
  if (tokens > MUI_MAX_TOKENS) {  // a prompt: the tiled matrix-core GEMM
    SkinnyParams sp = {};
    sp.w0 = weights; sp.pitch = w_pitch; sp.x = (const uint16_t*)x; sp.gamma = (const uint16_t*)norm_weights;
    sp.mul_bias = (const uint16_t*)mul_bias; sp.add_bias = (const uint16_t*)add_bias;
    sp.residual = (const uint16_t*)residual; sp.y = (uint16_t*)y; sp.n = n_out; sp.k = k_in; sp.tokens = tokens;
    sp.eps = epsilon;
    sp.workspace = workspace; sp.workspace_bytes = workspace_bytes;
    return launch_prefill_gemm(s, dtype, WF_16BIT, SK_LINEAR, sp);
  }
  if (tokens >= g_skinny_min_tokens || g_gemv_dot2) {
    SkinnyParams sp = {};
    sp.w0 = weights;
    sp.pitch = w_pitch;
    sp.x = (const uint16_t*)x;
    sp.gamma = (const uint16_t*)norm_weights;
    sp.mul_bias = (const uint16_t*)mul_bias;
    sp.add_bias = (const uint16_t*)add_bias;
    sp.residual = (const uint16_t*)residual;
    sp.y = (uint16_t*)y;
    sp.n = n_out;
    sp.k = k_in;
    sp.tokens = tokens;
    sp.eps = epsilon;
    if (tokens <= g_multi_max_tokens) {
      const int st = launch_gemv_multi(s, dtype, SK_LINEAR, sp);
      if (st != MUI_ERR_UNSUPPORTED) return st;
    }
    if (tokens >= g_skinny_min_tokens) return launch_skinny(s, dtype, WF_16BIT, SK_LINEAR, sp);
  }
  if (k_in > 8 * 8 * kThreads) return MUI_ERR_UNSUPPORTED;  // the per-token kernel below: 8 chunks per thread
  for (int tkn = 0; tkn < tokens; ++tkn) {
    GemvParams p;
    p.w0 = (const uint16_t*)weights;
    p.w1 = nullptr;
    p.pitch = w_pitch;
    p.x = (const uint16_t*)x + (long)tkn * k_in;
    p.gamma = (const uint16_t*)norm_weights;
    p.mul_bias = (const uint16_t*)mul_bias;
    p.add_bias = (const uint16_t*)add_bias;
    p.residual = residual ? (const uint16_t*)residual + (long)tkn * n_out : nullptr;
    p.y = (uint16_t*)y + (long)tkn * n_out;
    p.n = n_out;
    p.k = k_in;
    p.eps = epsilon;
    int st = launch_gemv<EPI_LINEAR>(s, dtype, p);
    if (st != MUI_OK) return st;
  }
  return MUI_OK;
}

extern "C" int mui_gateup_silu(mui_stream_t stream, int dtype, const void* gate, const void* up,
                               long gu_pitch, const void* x, const void* norm_weights,
                               float epsilon, void* h, int n_inter, int k_in, int tokens) {
  MUI_CHECK_ARG(gate && up && x && h);
  MUI_CHECK_ARG(n_inter > 0 && k_in > 0 && tokens > 0);
  MUI_CHECK_ARG(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16);
  if (gu_pitch < k_in) return MUI_ERR_INVALID_ARG;
  if ((k_in & 7) || (gu_pitch & 7)) return MUI_ERR_UNSUPPORTED;
  if (!aligned16(gate) || !aligned16(up) || !aligned16(x) ||
      (norm_weights && !aligned16(norm_weights)))
    return MUI_ERR_ALIGNMENT;

  hipStream_t s = (hipStream_t)stream;
  if (tokens > MUI_MAX_TOKENS) {  // a prompt: the tiled matrix-core GEMM
    SkinnyParams sp = {};
    sp.w0 = gate; sp.w1 = up; sp.pitch = gu_pitch; sp.x = (const uint16_t*)x;
    sp.gamma = (const uint16_t*)norm_weights; sp.y = (uint16_t*)h; sp.n = n_inter; sp.k = k_in;
    sp.tokens = tokens; sp.eps = epsilon;
    return launch_prefill_gemm(s, dtype, WF_16BIT, SK_GATEUP, sp);
  }
  // bf16 has no mixed-precision fma: a single bf16 token takes the packed-dot kernel here too
  if (tokens >= g_skinny_min_tokens || (g_gemv_dot2 && dtype == MUI_DTYPE_BF16)) {
    SkinnyParams sp = {};
    sp.w0 = gate;
    sp.w1 = up;
    sp.pitch = gu_pitch;
    sp.x = (const uint16_t*)x;
    sp.gamma = (const uint16_t*)norm_weights;
    sp.y = (uint16_t*)h;
    sp.n = n_inter;
    sp.k = k_in;
    sp.tokens = tokens;
    sp.eps = epsilon;
    if (tokens <= g_multi_max_tokens) {
      const int st = launch_gemv_multi(s, dtype, SK_GATEUP, sp);
      if (st != MUI_ERR_UNSUPPORTED) return st;
    }
    if (tokens >= g_skinny_min_tokens) return launch_skinny(s, dtype, WF_16BIT, SK_GATEUP, sp);
  }
  if (k_in > 8 * 8 * kThreads) return MUI_ERR_UNSUPPORTED;  // the per-token kernel below: 8 chunks per thread
  for (int tkn = 0; tkn < tokens; ++tkn) {
    GemvParams p;
    p.w0 = (const uint16_t*)gate;
    p.w1 = (const uint16_t*)up;
    p.pitch = gu_pitch;
    p.x = (const uint16_t*)x + (long)tkn * k_in;
    p.gamma = (const uint16_t*)norm_weights;
    p.mul_bias = p.add_bias = p.residual = nullptr;
    p.y = (uint16_t*)h + (long)tkn * n_inter;
    p.n = n_inter;
    p.k = k_in;
    p.eps = epsilon;
    int st = launch_gemv<EPI_GATEUP>(s, dtype, p);
    if (st != MUI_OK) return st;
  }
  return MUI_OK;
}
