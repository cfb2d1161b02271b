// Small-batch (5..16 tokens) fused linears with 16-bit weights on the matrix cores, with the
// weight rows read the way the single-token GEMV reads them.
//
// An MFMA A operand wants lane l to hold 16 bytes of row l % 16, so loading operands straight
// from HBM touches 16 rows x 64 bytes per instruction; measured on this part that pattern
// streams 17-40 % slower than instructions that each cover one contiguous kilobyte (13.0 vs
// 9.4 us for a 6144 x 4096 fp16 matrix). Here every load instruction covers 512-byte runs of two
// rows; the registers are written to a wave-private LDS tile (row pitch +16
// bytes: the 16 lanes of a b128 read phase hit 64 distinct banks) and read back in operand
// order. LDS traffic is one write and one read per weight byte, far below its bandwidth, and
// no workgroup barrier is involved: a wave only ever reads what it wrote itself.
//
// A pass of a wave is 16 rows x 256 k-values (8 load instructions of two 512-byte runs, then 8
// MFMAs): small enough that converting one pass overlaps the arrival of the next ones.
//   B-stationary mode (K <= 4096, K % 256 == 0): wave w owns the same K range of every tile
//     (two passes per tile); its B operands (gamma * x of the 16 token columns) are built once
//     and stay in registers; four register sets = two tiles in flight.
//   streaming mode (any K % 8 == 0, no fused norm): the wave walks its K range in passes and
//     brings the token rows through LDS the same way as the weight rows; two register sets.
// Both are persistent (one workgroup per CU, balanced tile counts).
//
// The reference has no kernel for this case (csrc/modules/linear_module.cpp:57-79 falls back to
// RMSNorm + torch matmul + add; muillm/modules/gateupdownmlp.py:343-359).
#include "skinny.cuh"

namespace mui {

constexpr int kLtWaves = 8;
constexpr int kLtThreads = kLtWaves * kWave;
constexpr int kLtSub = 256;                 // k-values per wave and pass
constexpr int kLtPitch = kLtSub * 2 + 16;   // LDS row pitch in bytes
constexpr int kLtLoads = 8;                 // load instructions per 16-row operand tile (2 rows each)
constexpr int kLtSteps = kLtSub / 32;       // MFMAs per pass

template <typename T, bool NORM, int EPI, bool BSTAT, bool FULL>
__global__ void __launch_bounds__(kLtThreads) gemm_skinny_lt_kernel(
    // scalars, hottest first (the leading ones are preloaded into SGPRs at wave launch)
    const void* w0, const void* w1, long pitch, const uint16_t* x, int n, int k, int tokens, int n_tiles, int spw,
    const uint16_t* gamma, uint16_t* y, float eps, const uint16_t* residual, const uint16_t* mul_bias,
    const uint16_t* add_bias) {
  SkinnyParams p = {};
  p.w0 = w0; p.w1 = w1; p.pitch = pitch; p.x = x; p.n = n; p.k = k; p.tokens = tokens;
  p.gamma = gamma; p.y = y; p.eps = eps; p.residual = residual; p.mul_bias = mul_bias; p.add_bias = add_bias;
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  constexpr int NOPS = BSTAT ? 1 : 2;   // operand tiles per wave in LDS: A, or A and B
  constexpr int NSET = BSTAT ? 4 : 2;   // register sets = passes in flight per wave
  constexpr int NB = BSTAT ? 1 : kLtLoads;
  static_assert(BSTAT || !NORM, "streaming mode has no fused norm");

  __shared__ __attribute__((aligned(16))) char op_lds[kLtWaves][NOPS][16 * kLtPitch];
  __shared__ float tile[2][kLtWaves][16][17];
  __shared__ float ss_part[kLtWaves][16];  // sum(x^2) of token j over wave w's K range

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int ld_row = lane >> 5;     // row inside a load instruction
  const int ld_chunk = lane & 31;   // 16-byte chunk inside the 512-byte row segment
  char* la = &op_lds[wave][0][0];
  char* lb = &op_lds[wave][NOPS - 1][0];

  // B-stationary: this wave's K range is jmax MFMA steps = jmax * 64 bytes of every row, walked
  // in two passes of 8 steps; streaming: spw passes of 256 k-values per tile
  const int jmax = BSTAT ? (FULL ? 2 * kLtSteps : (p.k >> 8)) : 0;
  const int passes = BSTAT ? 2 : spw;
  const int my_tiles = blockIdx.x < n_tiles ? (n_tiles - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
  const int n_items = my_tiles * passes;  // pass i: tile blockIdx.x + (i / passes) * gridDim.x, sub-block i % passes

  auto row_base = [&](int tl, int q) -> const char* {
    const int r = q * 2 + ld_row;  // row of the tile
    int out_row;
    const void* wbase;
    if constexpr (EPI == SK_GATEUP) {
      out_row = tl * 8 + q;
      wbase = ld_row ? p.w1 : p.w0;
    } else {
      out_row = tl * 16 + r;
      wbase = p.w0;
    }
    const int row_c = out_row < p.n ? out_row : p.n - 1;
    return (const char*)wbase + (long)row_c * p.pitch * 2;
  };

  // Lanes, token rows and passes with nothing to fetch issue no load at all (measured: feeding
  // them dummy addresses to keep the code branch-free costs more than the compiler's coarser
  // load-counter waits behind the branches).
  auto lane_k0 = [&](int i, bool& ok) -> int {  // first k-value of this lane's chunk in pass i
    const int sub = i % passes;
    if constexpr (BSTAT) {
      const int c = sub * 32 + ld_chunk;  // chunk inside the wave's range
      ok = FULL || c < 4 * jmax;
      return (wave * jmax * 4 + c) << 3;
    } else {
      const int k0 = ((wave * spw + sub) << 8) + (ld_chunk << 3);
      ok = k0 < p.k;
      return k0;
    }
  };
  // Epilogue thread t < 16 * OUT handles token t / OUT, output t % OUT of the tile (consecutive
  // threads write consecutive outputs of one token). Its residual value travels with the
  // register set of the tile's last pass and is requested right after that pass's weights.
  auto issue_residual = [&](int i, uint32_t& res) {  // 32-bit holder: never packed with another one
    if constexpr (EPI == SK_LINEAR) {
      const int tl = blockIdx.x + (i / passes) * gridDim.x;
      const int n = tl * OUT + (t % OUT), j = t / OUT;
      const bool want = p.residual && i < n_items && (i % passes) == passes - 1 && t < OUT * 16 && j < p.tokens && n < p.n;
      if (want) res = p.residual[(long)j * p.n + n];
    }
  };
  auto issue = [&](int i, u32x4 (&a)[kLtLoads], u32x4 (&b)[NB]) {
    if (i >= n_items) return;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const int tl = blockIdx.x + (i / passes) * gridDim.x;
    bool ok;
    const int k0 = lane_k0(i, ok);
#pragma unroll
    for (int q = 0; q < kLtLoads; ++q) a[q] = ok ? ld16_stream(row_base(tl, q) + ((long)k0 << 1)) : zero;
    if constexpr (!BSTAT) {
#pragma unroll
      for (int q = 0; q < kLtLoads; ++q) {
        const int tok = q * 2 + ld_row;
        b[q] = (ok && tok < p.tokens) ? ld16(p.x + (long)tok * p.k + k0) : zero;
      }
    }
  };

  auto epilogue = [&](int tl, int buf, float res) {
    if (t < OUT * 16) {
      const int i = t % OUT;
      const int j = t / OUT;
      const int n = tl * OUT + i;
      if (j < p.tokens && n < p.n) {
        float rs = 1.f;
        if constexpr (NORM) {
          float tot = 0.f;
#pragma unroll
          for (int w = 0; w < kLtWaves; ++w) tot += ss_part[w][j];
          rs = rsqrtf(tot / (float)p.k + p.eps);
        }
        auto total = [&](int row) {
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < kLtWaves; ++w) v += tile[buf][w][row][j];
          return v;
        };
        float v;
        if constexpr (EPI == SK_GATEUP) {
          v = silu_f32(total(2 * i) * rs) * (total(2 * i + 1) * rs);
        } else {
          v = total(i) * rs;
          if (p.mul_bias) v *= T::one(p.mul_bias[n]);
          if (p.add_bias) v += T::one(p.add_bias[n]);
          if (p.residual) v += res;
        }
        p.y[(long)j * p.n + n] = T::pack(v);
      }
    }
  };

  u32x4 bq[BSTAT ? 2 * kLtSteps : 1];
  f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};  // two chains: MFMAs back to back
  int buf = 0;
  auto stage = [&](const u32x4 (&a)[kLtLoads], const u32x4 (&b)[NB]) {  // registers -> LDS tile
#pragma unroll
    for (int q = 0; q < kLtLoads; ++q) *(u32x4*)(la + (q * 2 + ld_row) * kLtPitch + ld_chunk * 16) = a[q];
    if constexpr (!BSTAT) {
#pragma unroll
      for (int q = 0; q < kLtLoads; ++q) *(u32x4*)(lb + (q * 2 + ld_row) * kLtPitch + ld_chunk * 16) = b[q];
    }
    __builtin_amdgcn_wave_barrier();
  };
  // operand order back into the registers the pass came from (all reads in flight at once)
  auto gather = [&](u32x4 (&a)[kLtLoads], u32x4 (&b)[NB]) {
#pragma unroll
    for (int s = 0; s < kLtSteps; ++s) a[s] = *(const u32x4*)(la + r16 * kLtPitch + (4 * s + g) * 16);
    if constexpr (!BSTAT) {
#pragma unroll
      for (int s = 0; s < kLtSteps; ++s) b[s] = *(const u32x4*)(lb + r16 * kLtPitch + (4 * s + g) * 16);
    }
  };
  auto mma = [&](const u32x4 (&a)[kLtLoads], const u32x4 (&b)[NB], const int half) {
#pragma unroll
    for (int s = 0; s < kLtSteps; ++s) {
      if (BSTAT && !FULL && half * kLtSteps + s >= jmax) break;
      u32x4 bv;
      if constexpr (BSTAT) bv = bq[half * kLtSteps + s];
      else bv = b[s];
      if (s & 1) acc1 = mfma16x16x32<T>(a[s], bv, acc1);
      else acc = mfma16x16x32<T>(a[s], bv, acc);
    }
    __builtin_amdgcn_wave_barrier();
  };
  auto finish = [&](int i, const uint32_t res_bits) {
    if ((i % passes) == passes - 1 && i < n_items) {  // last pass of the tile: reduce over the waves
#pragma unroll
      for (int r = 0; r < 4; ++r) tile[buf][wave][4 * g + r][r16] = acc[r] + acc1[r];
      acc = f32x4{0.f, 0.f, 0.f, 0.f};
      acc1 = f32x4{0.f, 0.f, 0.f, 0.f};
      __syncthreads();
      epilogue(blockIdx.x + (i / passes) * gridDim.x, buf, T::one((uint16_t)res_bits));
      buf ^= 1;
    }
  };

  // The token operands are built while the first weight passes are already on their way: token
  // rows are read like weight rows (lane l = 16-byte chunk l of this wave's K range, one
  // contiguous kilobyte per token), multiplied by gamma, and turned into operand order through
  // the wave's LDS tile, one half of the range at a time; sum(x^2) per token is reduced over
  // the wave on the side. Their loads are issued before the weight loads: loads return in
  // order, so the build only waits for the L2-resident token rows, not for the weight passes
  // behind them.
  u32x4 gv = {0u, 0u, 0u, 0u};
  u32x4 xv[BSTAT ? 16 : 1];
  if constexpr (BSTAT) {
    const bool b_ok = FULL || lane < 4 * jmax;
    const int e = (wave * jmax * 4 + lane) << 3;  // element offset of this lane's chunk inside a row
    if constexpr (NORM) { if (b_ok) gv = ld16(p.gamma + e); }
#pragma unroll
    for (int tk = 0; tk < 16; ++tk) {
      xv[tk] = u32x4{0u, 0u, 0u, 0u};
      if (b_ok && tk < p.tokens) xv[tk] = ld16(p.x + (long)tk * p.k + e);
    }
  }

  // two passes go out before the build, the rest after it (the token rows, the build's
  // registers and four register sets do not fit the register file together)
  u32x4 as[NSET][kLtLoads], bs[NSET][NB];
  uint32_t rs_bits[NSET] = {};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    issue(u, as[u], bs[u]);
    issue_residual(u, rs_bits[u]);
  }

  if constexpr (BSTAT) {
#pragma unroll
    for (int tk = 0; tk < 16; ++tk) {
      float ss = 0.f;
      xv[tk] = make_b<T, NORM>(xv[tk], gv, ss);  // zero rows stay zero
      if constexpr (NORM) {
        ss = wave_sum(ss);
        if (lane == 0) ss_part[wave][tk] = ss;
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if ((lane >> 5) == h) {
#pragma unroll
        for (int tk = 0; tk < 16; ++tk) *(u32x4*)(la + tk * kLtPitch + ld_chunk * 16) = xv[tk];
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < kLtSteps; ++j) bq[h * kLtSteps + j] = *(const u32x4*)(la + r16 * kLtPitch + (4 * j + g) * 16);
      __builtin_amdgcn_wave_barrier();
    }
  }

#pragma unroll
  for (int u = 2; u < NSET; ++u) {
    issue(u, as[u], bs[u]);
    issue_residual(u, rs_bits[u]);
  }

  // passes in rounds of NSET
  for (int i = 0; i < n_items; i += NSET) {
#pragma unroll
    for (int u = 0; u < NSET; ++u) {
      const bool live = i + u < n_items;
      if (live) {
        stage(as[u], bs[u]);
        gather(as[u], bs[u]);
        mma(as[u], bs[u], u & 1);
      }
      issue(i + u + NSET, as[u], bs[u]);  // the set is free again
      if (live) finish(i + u, rs_bits[u]);
      issue_residual(i + u + NSET, rs_bits[u]);
    }
  }
}

template <typename T, int EPI>
static int launch_lt_t(hipStream_t s, const SkinnyParams& p) {
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  const int n_tiles = ceil_div(p.n, OUT);
  const int grid = balanced_grid(n_tiles, 1);  // ~150 KB of LDS: one workgroup per CU
#define MUI_LT(NORMV, BSTATV, FULLV, SPW)                                                               \
  hipLaunchKernelGGL((gemm_skinny_lt_kernel<T, NORMV, EPI, BSTATV, FULLV>), dim3(grid), dim3(kLtThreads), \
                     0, s, p.w0, p.w1, p.pitch, p.x, p.n, p.k, p.tokens, n_tiles, SPW, p.gamma, p.y, p.eps,        \
                     p.residual, p.mul_bias, p.add_bias)
  if (p.k <= kLtWaves * 2 * kLtSub && p.k % 256 == 0) {
    const bool full = p.k == kLtWaves * 2 * kLtSub;
    if (p.gamma) { if (full) MUI_LT(true, true, true, 1); else MUI_LT(true, true, false, 1); }
    else { if (full) MUI_LT(false, true, true, 1); else MUI_LT(false, true, false, 1); }
    return launch_status();
  }
  if (p.gamma || (p.k & 7)) return MUI_ERR_UNSUPPORTED;
  const int spw = ceil_div(ceil_div(p.k, 256), kLtWaves);
  MUI_LT(false, false, false, spw);
#undef MUI_LT
  return launch_status();
}

int launch_skinny_lt(hipStream_t s, int dtype, int epilogue, const SkinnyParams& p) {
  if (p.tokens < 1 || p.tokens > 16) return MUI_ERR_UNSUPPORTED;
  if (dtype == MUI_DTYPE_F16) {
    if (epilogue == SK_LINEAR) return launch_lt_t<F16, SK_LINEAR>(s, p);
    if (epilogue == SK_GATEUP) return launch_lt_t<F16, SK_GATEUP>(s, p);
  } else if (dtype == MUI_DTYPE_BF16) {
    if (epilogue == SK_LINEAR) return launch_lt_t<BF16, SK_LINEAR>(s, p);
    if (epilogue == SK_GATEUP) return launch_lt_t<BF16, SK_GATEUP>(s, p);
  }
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui
