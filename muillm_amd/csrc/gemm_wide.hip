// Linear layers for 17..128 tokens (short prompts, prompt chunks): still bound by the weight
// stream, so the structure is the decode kernels' -- few weight rows per workgroup, many
// workgroups, the K range split over the waves of a workgroup -- with the token columns widened
// to up to eight MFMA tiles.
//
// The reference hands these calls to the framework's GEMM after a standalone RMSNorm kernel
// (csrc/modules/linear_module.cpp:57-79; muillm/modules/gateupdownmlp.py:343-359;
// muillm/modules/quantized/int8linear.py:279-293 dequantises the whole matrix first).
//
// Work layout (wave64, v_mfma_f32_16x16x32):
//   a workgroup of 8 waves owns 16 weight rows (8 gate + 8 up rows under the gate/up epilogue)
//   and ALL tokens (NT tiles of 16). Wave w takes the k-steps w, w + 8, ... of 32 (int8: 64)
//   k-values: one 16-byte load per lane brings the A operand of a step straight from HBM (the 8
//   waves together cover 512 contiguous bytes of every row), NT loads bring the B operands from
//   the token rows (L2-resident: every workgroup reads all of x), gamma is applied to them in
//   registers (rounded once to the 16-bit type) and the sum of squares is gathered on the side.
//   No LDS and no barrier in the K loop; the next step's loads are in flight while the current
//   step is multiplied. At the end the 8 partial tiles per token tile are summed through LDS and
//   the epilogue (rsqrt factor, int8 row scale, biases, residual, or SiLU * mul) is applied.
//   Weights are read exactly once; x is re-read by every workgroup from L2.
#include "skinny.cuh"

namespace mui {

constexpr int kWideThreads = 512;
constexpr int kWideWaves = kWideThreads / kWave;

struct WideParams {
  const uint8_t* w0; const uint8_t* w1; long pitch;  // bytes
  const uint16_t* s0; const uint16_t* s1; long s_pitch;
  const uint16_t* x; const uint16_t* gamma; const uint16_t* mul_bias; const uint16_t* add_bias;
  const uint16_t* residual; uint16_t* y;
  int n, k, tokens; float eps;
};

template <typename T, int WF, bool NORM, int EPI, int NT>
__global__ void __launch_bounds__(kWideThreads) gemm_wide_kernel(const WideParams p) {
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;      // outputs per workgroup
  constexpr int KSTEP = (WF == WF_16BIT) ? 32 : 64;     // k-values per wave step
  constexpr int SUB = KSTEP / 32;                       // MFMA k-blocks per step
  constexpr int TOK = NT * 16;
  // partial tiles [wave pair][token tile][token][row]: the upper four waves hand theirs to the lower
  // four first, which keeps the buffer within the 64 KB of statically declared LDS
  __shared__ __align__(16) float red[kWideWaves / 2][NT][16][16];
  __shared__ float ss_red[NORM ? kWideWaves : 1][4][TOK];
  __shared__ float rs_lds[TOK];

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int lrow = lane & 15;   // A: weight row of the tile; B: token of the tile
  const int lchunk = lane >> 4; // which quarter of the step's k-values
  const int o0 = blockIdx.x * OUT;

  // A row of this lane
  const uint8_t* arow;
  {
    int o;
    const uint8_t* base = p.w0;
    if constexpr (EPI == SK_GATEUP) {
      o = o0 + (lrow & 7);
      base = (lrow & 8) ? p.w1 : p.w0;
    } else {
      o = o0 + lrow;
    }
    o = o < p.n ? o : p.n - 1;
    arow = base + (long)o * p.pitch;
  }
  // B rows (tokens) of this lane, one per token tile; tokens past the end read the last token
  const uint16_t* brow[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    int tk = j * 16 + lrow;
    tk = tk < p.tokens ? tk : p.tokens - 1;
    brow[j] = p.x + (long)tk * p.k;
  }

  const int total_steps = (p.k + KSTEP - 1) / KSTEP;
  const int my_steps = (total_steps - wave + kWideWaves - 1) / kWideWaves;  // steps wave, wave + 8, ...

  u32x4 a_nx, g_nx[SUB], b_nx[SUB][NT];
  bool live_nx[SUB];
  // k-values of lane chunk c in MFMA block u of step s: s*KSTEP + c*(8*SUB) + u*8 .. +8 (any
  // assignment works as long as A and B agree; this one makes a lane's bytes contiguous)
  auto load_step = [&](int i) {
    int s = wave + kWideWaves * i;
    s = s < total_steps ? s : 0;  // a wave past its last step re-reads step 0 (never multiplied in)
    const int kb = s * KSTEP + lchunk * (8 * SUB);
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
      const int kk = kb + u * 8;
      live_nx[u] = kk + 8 <= p.k;
      const int ko = live_nx[u] ? kk : 0;
#pragma unroll
      for (int j = 0; j < NT; ++j) b_nx[u][j] = ld16(brow[j] + ko);
      if constexpr (NORM) g_nx[u] = ld16(p.gamma + ko);
    }
    if constexpr (WF == WF_16BIT) {
      a_nx = ld16_stream(arow + 2L * (live_nx[0] ? kb : 0));
    } else {
      a_nx = ld16_stream(arow + (live_nx[0] ? kb : 0));
    }
  };

  f32x4 acc[NT];
  float ss[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) { acc[j] = f32x4{0.f, 0.f, 0.f, 0.f}; ss[j] = 0.f; }

  load_step(0);
  for (int i = 0; i < my_steps; ++i) {
    const u32x4 a_cu = a_nx;
    u32x4 g_cu[SUB], b_cu[SUB][NT];
    bool live_cu[SUB];
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
      live_cu[u] = live_nx[u];
      if constexpr (NORM) g_cu[u] = g_nx[u];
#pragma unroll
      for (int j = 0; j < NT; ++j) b_cu[u][j] = b_nx[u][j];
    }
    load_step(i + 1);  // in flight during this step's multiplications
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int u = 0; u < SUB; ++u) {
      u32x4 a;
      if constexpr (WF == WF_16BIT) a = a_cu;
      else a = (u == 0) ? convert_a<T, WF>(a_cu.x, a_cu.y, nullptr, 0, 0) : convert_a<T, WF>(a_cu.z, a_cu.w, nullptr, 0, 0);
      a = live_cu[u] ? a : zero;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        float sq = 0.f;
        const u32x4 b = make_b<T, NORM>(b_cu[u][j], NORM ? g_cu[u] : b_cu[u][j], sq);
        ss[j] += live_cu[u] ? sq : 0.f;
        acc[j] = mfma16x16x32<T>(a, b, acc[j]);
      }
    }
  }

  // ---- sum the waves' partial tiles; acc[j][e]: token 16 j + lane % 16, row 4 (lane / 16) + e
  constexpr int HW = kWideWaves / 2;
  if (wave >= HW) {
#pragma unroll
    for (int j = 0; j < NT; ++j) *(f32x4*)&red[wave - HW][j][lrow][lchunk * 4] = acc[j];
  }
  if constexpr (NORM) {
#pragma unroll
    for (int j = 0; j < NT; ++j) ss_red[wave][lchunk][j * 16 + lrow] = ss[j];
  }
  __syncthreads();
  if (wave < HW) {
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] += *(const f32x4*)&red[wave][j][lrow][lchunk * 4];
  }
  __syncthreads();
  if (wave < HW) {
#pragma unroll
    for (int j = 0; j < NT; ++j) *(f32x4*)&red[wave][j][lrow][lchunk * 4] = acc[j];
  }
  __syncthreads();
  if constexpr (NORM) {
    if (t < TOK) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < kWideWaves; ++w)
#pragma unroll
        for (int c = 0; c < 4; ++c) v += ss_red[w][c][t];
      rs_lds[t] = rsqrtf(v / (float)p.k + p.eps);
    }
    __syncthreads();
  }
  // outputs of the workgroup: OUT rows x tokens; thread -> (token, output), output fastest
  for (int idx = t; idx < OUT * TOK; idx += kWideThreads) {
    const int tk = idx / OUT, r = idx % OUT;
    const int o = o0 + r;
    if (tk >= p.tokens || o >= p.n) continue;
    const int j = tk >> 4, tl = tk & 15;
    const float rs = NORM ? rs_lds[tk] : 1.f;
    auto total = [&](int row) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < HW; ++w) v += red[w][j][tl][row];
      return v * rs;
    };
    float v;
    if constexpr (EPI == SK_GATEUP) {
      float g = total(r), u = total(r + 8);
      if constexpr (WF == WF_I8_CHANNEL) {
        g *= T::one(p.s0[(long)o * p.s_pitch]);
        u *= T::one(p.s1[(long)o * p.s_pitch]);
      }
      v = silu_f32(g) * u;
    } else {
      v = total(r);
      if constexpr (WF == WF_I8_CHANNEL) v *= T::one(p.s0[(long)o * p.s_pitch]);
      if (p.mul_bias) v *= T::one(p.mul_bias[o]);
      if (p.add_bias) v += T::one(p.add_bias[o]);
      if (p.residual) v += T::one(p.residual[(long)tk * p.n + o]);
    }
    p.y[(long)tk * p.n + o] = T::pack(v);
  }
}

template <typename T, int WF, int EPI, int NT>
static int launch_wide_nt(hipStream_t s, const WideParams& p) {
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  const int grid = ceil_div(p.n, OUT);
  if (p.gamma)
    hipLaunchKernelGGL((gemm_wide_kernel<T, WF, true, EPI, NT>), dim3(grid), dim3(kWideThreads), 0, s, p);
  else
    hipLaunchKernelGGL((gemm_wide_kernel<T, WF, false, EPI, NT>), dim3(grid), dim3(kWideThreads), 0, s, p);
  return launch_status();
}

template <typename T, int WF, int EPI>
static int launch_wide_t(hipStream_t s, const WideParams& p) {
  if (p.tokens <= 32) return launch_wide_nt<T, WF, EPI, 2>(s, p);
  if (p.tokens <= 64) return launch_wide_nt<T, WF, EPI, 4>(s, p);
  return launch_wide_nt<T, WF, EPI, 8>(s, p);
}

// 1..128 tokens (meant for 17..128), 16-bit weights or per-channel int8 codes, x / residual / y dense
int launch_gemm_wide(hipStream_t s, int dtype, int wf, int epilogue, const SkinnyParams& q) {
  if (q.tokens < 1 || q.tokens > 128 || q.n < 1 || q.k < 1) return MUI_ERR_UNSUPPORTED;
  if (!(wf == WF_16BIT || wf == WF_I8_CHANNEL)) return MUI_ERR_UNSUPPORTED;
  if (q.k % (wf == WF_16BIT ? 8 : 16)) return MUI_ERR_UNSUPPORTED;
  if (q.x_pitch != 0 && q.x_pitch != q.k) return MUI_ERR_UNSUPPORTED;
  WideParams p = {};
  const long esz = (wf == WF_16BIT) ? 2 : 1;
  p.w0 = (const uint8_t*)q.w0; p.w1 = (const uint8_t*)q.w1; p.pitch = q.pitch * esz;
  p.s0 = q.s0; p.s1 = q.s1; p.s_pitch = q.s_pitch;
  p.x = q.x; p.gamma = q.gamma; p.mul_bias = q.mul_bias; p.add_bias = q.add_bias; p.residual = q.residual;
  p.y = q.y; p.n = q.n; p.k = q.k; p.tokens = q.tokens; p.eps = q.eps;
#define MUI_WIDE_CASE(TT, WFV, EPIV) \
  if (dtype == TT::kDtype && wf == WFV && epilogue == EPIV) return launch_wide_t<TT, WFV, EPIV>(s, p);
  MUI_WIDE_CASE(F16, WF_16BIT, SK_LINEAR)
  MUI_WIDE_CASE(F16, WF_16BIT, SK_GATEUP)
  MUI_WIDE_CASE(F16, WF_I8_CHANNEL, SK_LINEAR)
  MUI_WIDE_CASE(F16, WF_I8_CHANNEL, SK_GATEUP)
  MUI_WIDE_CASE(BF16, WF_16BIT, SK_LINEAR)
  MUI_WIDE_CASE(BF16, WF_16BIT, SK_GATEUP)
  MUI_WIDE_CASE(BF16, WF_I8_CHANNEL, SK_LINEAR)
  MUI_WIDE_CASE(BF16, WF_I8_CHANNEL, SK_GATEUP)
#undef MUI_WIDE_CASE
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui
