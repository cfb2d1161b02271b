// Small-batch (up to 16 tokens) fused linears on the matrix cores, with the weight rows read
// the way the single-token GEMV reads them.
//
// An MFMA A operand wants lane l to hold the k-chunk l / 16 of row l % 16, so loading operands
// straight from HBM touches 16 rows x 64 bytes per instruction; measured on this part that
// pattern streams 17-40 % slower than instructions that cover contiguous runs of 512 bytes or
// more (13.0 vs 9.4 us for a 6144 x 4096 fp16 matrix). Here every load instruction covers
// contiguous runs (512 bytes of two rows with 16-bit weights, 256 bytes of four rows with 8-bit
// weights); the registers are written to a wave-private LDS tile (row pitch +16 bytes: the
// lanes of a read phase hit distinct banks) and read back in operand order. LDS traffic is one
// write and one read per weight byte, far below its bandwidth, and no workgroup barrier is
// involved: a wave only ever reads what it wrote itself. 8-bit weights cross LDS as bytes and
// are converted to the 16-bit type in operand layout (per-channel: exact integers, the row scale
// applied in the epilogue; group format: u8 * scale + min rounded once).
//
// A pass of a wave is 16 rows x 256 k-values (then 8 MFMAs): small enough that converting one
// pass overlaps the arrival of the next ones.
//   B-stationary mode (K <= 4096, K % 256 == 0): wave w owns the same K range of every tile
//     (two passes per tile); its B operands (gamma * x of the 16 token columns) are built once
//     and stay in registers.
//   streaming mode (longer rows): the wave walks its K range in passes and brings the token rows
//     through LDS the same way as the weight rows (a fused norm multiplies them by gamma on the
//     way and gathers sum(x^2) during the first tile). At up to 8 tokens only 8 token rows are
//     brought in per pass (down 4096 x 14336 at 8 tokens: 23.1 -> 21.8 us).
// Two register sets: the next pass is in flight while the current one is multiplied.
// Both are persistent (one workgroup per CU, balanced tile counts). The number of passes of a
// workgroup is a multiple of half the register sets (launcher).
//
// The reference has no kernel for this case (csrc/modules/linear_module.cpp:57-79 falls back to
// RMSNorm + torch matmul + add; muillm/modules/gateupdownmlp.py:343-359).
#include "skinny.cuh"

namespace mui {

constexpr int kLtWaves = 8;
constexpr int kLtThreads = kLtWaves * kWave;
constexpr int kLtSub = 256;                  // k-values per wave and pass
constexpr int kLtSteps = kLtSub / 32;        // MFMAs per pass
constexpr int kLtXPitch = kLtSub * 2 + 16;   // LDS row pitch of a 16-bit operand tile, bytes
constexpr int kLtXLoads = 8;                 // load instructions per 16-row tile of 16-bit values

// GP (group format): (scale, min) pairs per pass that travel with the pass's weights -- 2 for groups
// of 128 codes, 1 for groups of 256 or more; 0: the pair of every MFMA step is loaded where it is
// used (any group size >= 16). A load inside the multiply phase is the youngest one outstanding and
// waiting for it waits for the prefetched pass behind which it queued (loads return in order): down
// 4096 x 14336 at 4 tokens ran 20.7 us that way against 13.5 us with per-channel scales.
template <typename T, int WF, bool NORM, int EPI, bool BSTAT, bool FULL, bool HB, int GP = 0>
__global__ void __launch_bounds__(kLtThreads) gemm_skinny_lt_kernel(
    // scalars, hottest first (the leading ones are preloaded into SGPRs at wave launch)
    const void* w0, const void* w1, long pitch, const uint16_t* x, int n, int k, int tokens, int n_tiles, int spw,
    const uint16_t* gamma, uint16_t* y, float eps, const uint16_t* residual, const uint16_t* mul_bias,
    const uint16_t* add_bias, const uint16_t* s0, const uint16_t* s1, long s_pitch, int group_shift) {
  SkinnyParams p = {};
  p.w0 = w0; p.w1 = w1; p.pitch = pitch; p.x = x; p.n = n; p.k = k; p.tokens = tokens;
  p.gamma = gamma; p.y = y; p.eps = eps; p.residual = residual; p.mul_bias = mul_bias; p.add_bias = add_bias;
  p.s0 = s0; p.s1 = s1; p.s_pitch = s_pitch; p.group_shift = group_shift;
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  constexpr int WB = (WF == WF_16BIT) ? 2 : 1;   // bytes per weight
  // Group format with fp16 activations and groups of at least 128 codes: the codes reach the matrix
  // cores as the integers 1024 + u8 (a byte dropped into the mantissa of 1024.0: two byte permutes
  // per four codes instead of a convert, a multiply-add and a pack per code), the products of a
  // group's k-steps are accumulated on their own and folded into the running sums once per group:
  //   sum_k (u8_k * scale + min) x_k = scale * (sum_k (1024 + u8_k) x_k) + (min - 1024 scale) * sum_k x_k
  // with sum_k x_k from one more matrix instruction against a tile of ones. For (scale, min) to be
  // one pair per lane the product is taken transposed -- token rows as the first operand, weight
  // rows as the second --, so that lane (g, i) holds tokens 4 g .. 4 g + 3 of weight row i, the row
  // whose pairs it already loads for the conversion layout.
  constexpr bool GACC = WF == WF_U8_GROUP && GP > 0 && T::kDtype == MUI_DTYPE_F16;
  // Per-channel int8 with fp16 activations, same idea: the codes enter as 1024 + 128 + q (sign bit
  // flipped, byte dropped into the mantissa of 1024.0) and 1152 * sum_k x_k is taken off the finished
  // sums -- sum_k x_k over a wave's K range is a constant of the wave in B-stationary mode (sixteen
  // matrix instructions against a tile of ones, once), and one more matrix instruction per step in
  // streaming mode -- instead of a packed subtract per two codes on the way to the operand.
  constexpr bool CACC = WF == WF_I8_CHANNEL && T::kDtype == MUI_DTYPE_F16;
  const u32x4 ones16 = {0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u};
  f32x4 xs_wave = {0.f, 0.f, 0.f, 0.f};  // CACC, B-stationary: sum of this wave's token operands per token column
  f32x4 xs_run = {0.f, 0.f, 0.f, 0.f};   // CACC, streaming: the same over the passes of the current tile
  // k-values per wave and pass: 256 (512 bytes of a 16-bit row, 256 of an 8-bit one). (Passes of 512
  // codes for per-channel int8 -- 512 contiguous bytes per row again -- were ahead while the codes
  // were converted with a packed subtract per pair; with the offset taken off the finished sums
  // instead the finer passes win on every shape: gate/up 2 x 14336 x 4096 at 4 / 8 / 16 tokens 22.7 /
  // 23.4 / 25.4 us against 26.5 / 27.2 / 28.8 us.)
  constexpr int SUB = kLtSub;
  constexpr int STEPS = SUB / 32;                // MFMAs per pass
  constexpr int PB = 2 * kLtSub / SUB;           // B-stationary: passes per tile (2 or 1)
  constexpr int ROWB = SUB * WB;                 // bytes of a row segment of one pass
  constexpr int PITCH = ROWB + 16;               // LDS row pitch of the weight tile
  constexpr int RPI = 1024 / ROWB;               // rows covered by one load instruction (2 / 4)
  constexpr int NLD = 16 / RPI;                  // load instructions per weight tile (8 / 4)
  constexpr int LPR = kWave / RPI;               // lanes per row (32 / 16)
  constexpr int KPC = 16 / WB;                   // k-values per 16-byte chunk (8 / 16)
  constexpr int NOPS = BSTAT ? 1 : 2;            // operand tiles per wave in LDS: A, or A and B
  // register sets = passes in flight per wave (four measured no faster with 8-bit weights and
  // spill with 16-bit ones)
  constexpr int NSET = 2;
  constexpr int NB = BSTAT ? 1 : kLtXLoads;
  // streaming mode at up to 8 tokens: only the first 8 token rows are brought in (the other
  // rows of the LDS tile keep whatever they held: their output columns are never stored)
  constexpr int XL = HB ? kLtXLoads / 2 : kLtXLoads;

  __shared__ __attribute__((aligned(16))) char op_lds[kLtWaves][NOPS][16 * kLtXPitch];
  __shared__ float tile[2][kLtWaves][16][17];
  __shared__ float ss_part[kLtWaves][16];  // sum(x^2) of token j over wave w's K range

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int r16 = lane & 15;
  const int g = lane >> 4;
  const int ld_row = lane / LPR;     // weight tile: row inside a load instruction
  const int ld_chunk = lane % LPR;   //              16-byte chunk inside the row segment
  const int xl_row = lane >> 5;      // 16-bit token tile: the same for two rows x 512 bytes
  const int xl_chunk = lane & 31;
  char* la = &op_lds[wave][0][0];
  char* lb = &op_lds[wave][NOPS - 1][0];

  // B-stationary: this wave's K range is jmax MFMA steps = 32 * jmax k-values of every row,
  // walked in PB passes of STEPS steps; streaming: spw passes of 256 k-values per tile
  const int jmax = BSTAT ? (FULL ? 2 * kLtSteps : (p.k >> 8)) : 0;
  const int passes = BSTAT ? PB : spw;
  const int my_tiles = blockIdx.x < n_tiles ? (n_tiles - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
  const int n_items = my_tiles * passes;  // pass i: tile blockIdx.x + (i / passes) * gridDim.x, sub-block i % passes

  auto row_base = [&](int tl, int q) -> const char* {
    const int r = q * RPI + ld_row;  // row of the tile
    int out_row;
    const void* wbase;
    if constexpr (EPI == SK_GATEUP) {
      out_row = tl * 8 + (r >> 1);
      wbase = (r & 1) ? w1 : w0;
    } else {
      out_row = tl * 16 + r;
      wbase = p.w0;
    }
    const int row_c = out_row < p.n ? out_row : p.n - 1;
    return (const char*)wbase + (long)row_c * p.pitch * WB;
  };
  // group format: (scale, min) pairs of the weight row behind tile row r16 (operand layout)
  auto scale_row = [&](int tl) -> const uint16_t* {
    if constexpr (WF != WF_U8_GROUP) return nullptr;
    int out_row;
    const uint16_t* sbase;
    if constexpr (EPI == SK_GATEUP) {
      out_row = tl * 8 + (r16 >> 1);
      sbase = (r16 & 1) ? s1 : s0;
    } else {
      out_row = tl * 16 + r16;
      sbase = p.s0;
    }
    const int row_c = out_row < p.n ? out_row : p.n - 1;
    return sbase + (long)row_c * p.s_pitch;
  };

  // first k-value of pass i of this wave
  auto pass_k0 = [&](int i) -> int {
    const int sub = i % passes;
    if constexpr (BSTAT) return wave * jmax * 32 + sub * SUB;
    else return (wave * spw + sub) * SUB;
  };
  // k-values of pass i that exist (B-stationary: inside the wave's range; streaming: inside the row)
  auto pass_len = [&](int i) -> int {
    if constexpr (BSTAT) return FULL ? SUB : jmax * 32 - (i % passes) * SUB;
    else return p.k - pass_k0(i);
  };

  // No load of the steady state sits behind a branch: the compiler's load-counter waits are
  // exact only in straight-line code (behind a branch it waits for everything outstanding,
  // the newest prefetch included, which costs a full memory latency per pass). So nothing is
  // predicated: lanes past the end of the K range read the start of their row instead and are
  // zeroed on the way to LDS; token rows past the batch read the last token again (their
  // output columns are never stored); the tail without refills is peeled off the loop.
  // The epilogue lanes of output o = t / S_EX handle token o / OUT, output o % OUT of the tile.
  // Their residual value and per-channel scales
  // travel with the register set of each pass, requested right after that pass's weights: a
  // load inside the epilogue would be the youngest one outstanding, and waiting for it would
  // wait for every prefetched pass.
  struct Extras { uint32_t res, sc0, sc1; };  // 32-bit holders: never packed with one another
  constexpr int S_EX = kLtThreads / (OUT * 16);  // lanes per output in the epilogue
  const int tok_last = p.tokens - 1;
  auto issue_extras = [&](int i, Extras& e) {
    const int tl = blockIdx.x + (i / passes) * gridDim.x;
    int nn = tl * OUT + ((t / S_EX) % OUT), j = (t / S_EX) / OUT;  // the epilogue's mapping
    nn = nn < p.n ? nn : p.n - 1;
    j = j < p.tokens ? j : tok_last;
    if constexpr (EPI == SK_LINEAR) {
      const uint16_t* rp = p.residual ? p.residual + ((long)j * p.n + nn) : p.x;
      e.res = ld2(rp);
    }
    if constexpr (WF == WF_I8_CHANNEL) {
      e.sc0 = ld2(p.s0 + (long)nn * p.s_pitch);
      if constexpr (EPI == SK_GATEUP) e.sc1 = ld2(p.s1 + (long)nn * p.s_pitch);
    }
  };
  // k-value of this lane's weight chunk in pass i, or -1 past the end of the range
  auto weight_k = [&](int i) -> int {
    const int kk = ld_chunk * KPC;
    return (FULL || kk < pass_len(i)) ? pass_k0(i) + kk : -1;
  };
  auto issue = [&](int i, u32x4 (&a)[NLD], u32x4 (&b)[NB], u32x4& gm, uint32_t (&sp)[2]) {  // needs i < n_items
    const int tl = blockIdx.x + (i / passes) * gridDim.x;
    const int wk = weight_k(i);
    const long woff = (long)(wk < 0 ? 0 : wk) * WB;
#pragma unroll
    for (int q = 0; q < NLD; ++q) a[q] = ld16_stream(row_base(tl, q) + woff);
    if constexpr (WF == WF_U8_GROUP && GP > 0) {
      // the pass's (scale, min) pairs of the row this lane converts (operand layout: row r16)
      const uint16_t* srow = scale_row(tl);
#pragma unroll
      for (int q = 0; q < GP; ++q) {
        const int ke = pass_k0(i) + q * (SUB / GP);
        sp[q] = ld4(srow + 2 * ((ke < p.k ? ke : p.k - 1) >> p.group_shift));
      }
    }
    if constexpr (!BSTAT) {
      const int xk = pass_k0(i) + xl_chunk * 8;
      const int xoff = xk < p.k ? xk : 0;  // (the weights of those k-values are zeroed)
      if constexpr (NORM) gm = ld16(p.gamma + xoff);
#pragma unroll
      for (int q = 0; q < XL; ++q) {
        const int tok = q * 2 + xl_row;
        b[q] = ld16(p.x + (long)(tok < p.tokens ? tok : tok_last) * p.k + xoff);
      }
    }
  };

  // Epilogue of a tile: all 512 threads take part. Output o = t / S (S = 2 lanes per output for
  // the linear epilogue, 4 for gate/up) is output o % OUT of token o / OUT, so the lanes that
  // store write consecutive outputs of one token; each of the S lanes adds up the partial tiles
  // of 8 / S waves, the lanes are added with two DPP steps at most, and lane 0 of the group
  // finishes. (With one thread per output the two waves doing 16 dependent LDS reads each were
  // the tail of every tile: gate/up at 8 tokens 38.1 us with, 36.3 us without its epilogue.)
  constexpr int NOUT = OUT * 16;
  constexpr int S = kLtThreads / NOUT;
  constexpr int WPP = kLtWaves / S;
  auto epilogue = [&](int tl, int buf, const Extras& ex) {
    const int ep_o = t / S, ep_part = t % S;
    const int ep_i = ep_o % OUT, ep_j = ep_o / OUT;
    const int nn = tl * OUT + ep_i;
    float v0 = 0.f, v1 = 0.f;
#pragma unroll
    for (int w = 0; w < WPP; ++w) {
      const int wv = ep_part * WPP + w;
      if constexpr (EPI == SK_GATEUP) {
        v0 += tile[buf][wv][2 * ep_i][ep_j];
        v1 += tile[buf][wv][2 * ep_i + 1][ep_j];
      } else {
        v0 += tile[buf][wv][ep_i][ep_j];
      }
    }
    // quad permutes: lane ^ 1 (0xB1), lane ^ 2 (0x4E)
    v0 += dpp_f32<0xB1>(v0);
    if constexpr (S == 4) v0 += dpp_f32<0x4E>(v0);
    if constexpr (EPI == SK_GATEUP) {
      v1 += dpp_f32<0xB1>(v1);
      if constexpr (S == 4) v1 += dpp_f32<0x4E>(v1);
    }
    if (ep_part == 0 && ep_j < p.tokens && nn < p.n) {
      float ep_rs = 1.f;
      if constexpr (NORM) {
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < kLtWaves; ++w) tot += ss_part[w][ep_j];
        ep_rs = rsqrtf(tot / (float)p.k + p.eps);
      }
      float v;
      if constexpr (EPI == SK_GATEUP) {
        float gt = v0 * ep_rs, up = v1 * ep_rs;
        if constexpr (WF == WF_I8_CHANNEL) {
          gt *= T::one((uint16_t)ex.sc0);
          up *= T::one((uint16_t)ex.sc1);
        }
        v = silu_f32(gt) * up;
      } else {
        v = v0 * ep_rs;
        if constexpr (WF == WF_I8_CHANNEL) v *= T::one((uint16_t)ex.sc0);
        if (p.mul_bias) v *= T::one(p.mul_bias[nn]);
        if (p.add_bias) v += T::one(p.add_bias[nn]);
        if (p.residual) v += T::one((uint16_t)ex.res);
      }
      p.y[(long)ep_j * p.n + nn] = T::pack(v);
    }
  };

  u32x4 bq[BSTAT ? 2 * kLtSteps : 1];
  f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};  // two chains: MFMAs back to back
  int buf = 0;
  // streaming mode with a fused norm: sum(x^2) of tokens 2 q + xl_row over this lane's chunks,
  // gathered during the wave's passes over the first tile (later tiles read the same token rows)
  float ssx[(NORM && !BSTAT) ? kLtXLoads : 1] = {};
  auto stage = [&](int i, const u32x4 (&a)[NLD], const u32x4 (&b)[NB], const u32x4& gm) {  // registers -> LDS tiles
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const bool ok = FULL || weight_k(i) >= 0;
#pragma unroll
    for (int q = 0; q < NLD; ++q) *(u32x4*)(la + (q * RPI + ld_row) * PITCH + ld_chunk * 16) = ok ? a[q] : zero;
    if constexpr (!BSTAT) {
      const bool x_ok = pass_k0(i) + xl_chunk * 8 < p.k;
      const bool count = NORM && i < passes && x_ok;
#pragma unroll
      for (int q = 0; q < XL; ++q) {
        u32x4 v = b[q];
        // group format: a code zeroed past the row end still stands for `min` (or 1024 + 0), so the
        // token values of those k-values are zeroed as well
        if constexpr (WF != WF_16BIT) v = x_ok ? v : zero;
        if constexpr (NORM) {
          float sq = 0.f;
          v = make_b<T, true>(v, gm, sq);
          ssx[q] += count ? sq : 0.f;
        }
        *(u32x4*)(lb + (q * 2 + xl_row) * kLtXPitch + xl_chunk * 16) = v;
      }
    }
    __builtin_amdgcn_wave_barrier();
  };
  // one pass in operand order: STEPS MFMA steps of 32 k-values (half: which part of the wave's
  // range the pass covers in B-stationary mode; the register set fixes it)
  // (the operands are read back into the registers the pass came from: NLD = 8 = steps with
  // 16-bit weights, and the token tile of streaming mode has 8 loads as well)
  auto multiply = [&](int i, const int half, u32x4 (&a16)[NLD], u32x4 (&bx)[NB], const uint32_t (&sp)[2]) {
    u32x2 a8[WF == WF_16BIT ? 1 : STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {  // all reads in flight at once
      if constexpr (WF == WF_16BIT) a16[s] = *(const u32x4*)(la + r16 * PITCH + (4 * s + g) * 16);
      else a8[s] = *(const u32x2*)(la + r16 * PITCH + (4 * s + g) * 8);
      if constexpr (!BSTAT) bx[s] = *(const u32x4*)(lb + r16 * kLtXPitch + (4 * s + g) * 16);
    }
    const uint16_t* srow = scale_row(blockIdx.x + (i / passes) * gridDim.x);
    const int k0 = pass_k0(i);
    if constexpr (GACC) {
      constexpr int SEG = STEPS / GP;  // k-steps that share a (scale, min) pair
#pragma unroll
      for (int q = 0; q < GP; ++q) {
        f32x4 part = {0.f, 0.f, 0.f, 0.f}, part1 = {0.f, 0.f, 0.f, 0.f}, xs = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < SEG; ++s2) {
          const int s = q * SEG + s2;
          // (steps past the wave's range in a partial B-stationary pass multiply zeroed weights)
          u32x4 av, bv;
          av.x = __builtin_amdgcn_perm(0x64646464u, a8[s].x, 0x04010400u);
          av.y = __builtin_amdgcn_perm(0x64646464u, a8[s].x, 0x04030402u);
          av.z = __builtin_amdgcn_perm(0x64646464u, a8[s].y, 0x04010400u);
          av.w = __builtin_amdgcn_perm(0x64646464u, a8[s].y, 0x04030402u);
          if constexpr (BSTAT) bv = bq[half * STEPS + s];
          else bv = bx[s];
          if (s2 & 1) part1 = mfma16x16x32<T>(bv, av, part1);
          else part = mfma16x16x32<T>(bv, av, part);
          xs = mfma16x16x32<T>(bv, ones16, xs);
        }
        const float sc = T::lo(sp[q]), cm = fmaf(-1024.f, sc, T::hi(sp[q]));
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = fmaf(sc, part[r] + part1[r], fmaf(cm, xs[r], acc[r]));
      }
      __builtin_amdgcn_wave_barrier();
      return;
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (BSTAT && !FULL && half * STEPS + s >= jmax) break;
      u32x4 av, bv;
      if constexpr (WF == WF_16BIT) av = a16[s];
      else {
        if constexpr (CACC) {
          const uint32_t u0 = a8[s].x ^ 0x80808080u, u1 = a8[s].y ^ 0x80808080u;
          av.x = __builtin_amdgcn_perm(0x64646464u, u0, 0x04010400u);
          av.y = __builtin_amdgcn_perm(0x64646464u, u0, 0x04030402u);
          av.z = __builtin_amdgcn_perm(0x64646464u, u1, 0x04010400u);
          av.w = __builtin_amdgcn_perm(0x64646464u, u1, 0x04030402u);
        } else if constexpr (WF == WF_U8_GROUP && GP > 0) {
          av = convert_a_pair<T>(a8[s].x, a8[s].y, sp[s / (STEPS / GP)]);
        } else {
          const int ke = k0 + 32 * s + 8 * g;  // (clamped: the scale pair of a k past the row end is never used)
          av = convert_a<T, WF>(a8[s].x, a8[s].y, srow, ke < p.k ? ke : p.k - 1, p.group_shift);
        }
      }
      if constexpr (BSTAT) bv = bq[half * STEPS + s];
      else bv = bx[s];
      if (s & 1) acc1 = mfma16x16x32<T>(av, bv, acc1);
      else acc = mfma16x16x32<T>(av, bv, acc);
      if constexpr (CACC && !BSTAT) xs_run = mfma16x16x32<T>(ones16, bv, xs_run);
    }
    __builtin_amdgcn_wave_barrier();
  };
  auto finish = [&](int i, const Extras& ex) {
    if ((i % passes) == passes - 1) {  // last pass of the tile: reduce over the waves
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if constexpr (GACC) tile[buf][wave][r16][4 * g + r] = acc[r];  // transposed product: [weight row][token]
        else if constexpr (CACC) tile[buf][wave][4 * g + r][r16] = fmaf(-1152.f, BSTAT ? xs_wave[r] : xs_run[r], acc[r] + acc1[r]);
        else tile[buf][wave][4 * g + r][r16] = acc[r] + acc1[r];
      }
      xs_run = f32x4{0.f, 0.f, 0.f, 0.f};
      acc = f32x4{0.f, 0.f, 0.f, 0.f};
      acc1 = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (NORM && !BSTAT) {
        if (i < passes) {  // first tile done: this wave has seen its whole K range of every token
#pragma unroll
          for (int q = 0; q < XL; ++q) {
            const float even = wave_sum(lane < 32 ? ssx[q] : 0.f), odd = wave_sum(lane < 32 ? 0.f : ssx[q]);
            if (lane == 0) {
              ss_part[wave][2 * q] = even;
              ss_part[wave][2 * q + 1] = odd;
            }
          }
        }
      }
      __syncthreads();
      epilogue(blockIdx.x + (i / passes) * gridDim.x, buf, ex);
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
  constexpr int XT = HB ? 8 : 16;  // token rows brought in (B-stationary mode: built into operands)
  u32x4 xv[BSTAT ? XT : 1];
  const bool b_ok = FULL || lane < 4 * jmax;
  if constexpr (BSTAT) {
    const int e = b_ok ? (wave * jmax * 4 + lane) << 3 : 0;  // element offset of this lane's chunk inside a row
    if constexpr (NORM) gv = ld16(p.gamma + e);
#pragma unroll
    for (int tk = 0; tk < XT; ++tk) xv[tk] = ld16(p.x + (long)(tk < p.tokens ? tk : tok_last) * p.k + e);
  }
  auto build_b = [&]() {
    if constexpr (BSTAT) {
      const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int tk = 0; tk < XT; ++tk) {
        float ss = 0.f;
        xv[tk] = make_b<T, NORM>(b_ok ? xv[tk] : zero, gv, ss);
        if constexpr (NORM) {
          ss = wave_sum(ss);
          if (lane == 0) ss_part[wave][tk] = ss;
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if ((lane >> 5) == h) {
#pragma unroll
          for (int tk = 0; tk < XT; ++tk) *(u32x4*)(la + tk * kLtXPitch + xl_chunk * 16) = xv[tk];
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < kLtSteps; ++j) bq[h * kLtSteps + j] = *(const u32x4*)(la + r16 * kLtXPitch + (4 * j + g) * 16);
        __builtin_amdgcn_wave_barrier();
      }
      if constexpr (CACC) {
#pragma unroll
        for (int j = 0; j < 2 * kLtSteps; ++j) xs_wave = mfma16x16x32<T>(ones16, bq[j], xs_wave);
      }
    }
  };

  u32x4 as[NSET][NLD], bs[NSET][NB];
  u32x4 gs[NSET] = {};  // streaming mode with a fused norm: gamma chunk of the pass
  uint32_t sps[NSET][2] = {};  // group format: the pass's (scale, min) pairs
  Extras ex[NSET] = {};
  // pass i on register set U (U = i % NSET); REFILL: the set is requested again for pass i + NSET
#define MUI_LT_PASS(i_, U, REFILL)                    \
  {                                                   \
    stage((i_), as[U], bs[U], gs[U]);                 \
    multiply((i_), (U) % PB, as[U], bs[U], sps[U]);   \
    if (REFILL) issue((i_) + NSET, as[U], bs[U], gs[U], sps[U]); \
    finish((i_), ex[U]);                              \
    if (REFILL) issue_extras((i_) + NSET, ex[U]);     \
  }

  if (n_items >= NSET) {
    // two passes go out before the build, the rest after it (the token rows, the build's
    // registers and all register sets do not fit the register file together)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      issue(u, as[u], bs[u], gs[u], sps[u]);
      issue_extras(u, ex[u]);
    }
    build_b();
#pragma unroll
    for (int u = 2; u < NSET; ++u) {
      issue(u, as[u], bs[u], gs[u], sps[u]);
      issue_extras(u, ex[u]);
    }
    // passes with a refill in rounds of NSET, a half round if their number asks for it (it is
    // a multiple of NSET / 2), then the last NSET passes without refills
    const int n_main = n_items - NSET;
    int i = 0;
    for (; i + NSET <= n_main; i += NSET) {
#pragma unroll
      for (int u = 0; u < NSET; ++u) MUI_LT_PASS(i + u, u, true)
    }
    if (i < n_main) {
#pragma unroll
      for (int u = 0; u < NSET / 2; ++u) MUI_LT_PASS(i + u, u, true)
#pragma unroll
      for (int v = 0; v < NSET; ++v) MUI_LT_PASS(i + NSET / 2 + v, (NSET / 2 + v) % NSET, false)
    } else {
#pragma unroll
      for (int v = 0; v < NSET; ++v) MUI_LT_PASS(i + v, v, false)
    }
  } else {
    // fewer passes than register sets (one small tile per workgroup): everything is requested
    // up front and multiplied once it is there
#pragma unroll
    for (int u = 0; u < NSET; ++u) {
      if (u < n_items) {
        issue(u, as[u], bs[u], gs[u], sps[u]);
        issue_extras(u, ex[u]);
      }
    }
    build_b();
#pragma unroll
    for (int u = 0; u < NSET; ++u) {
      if (u < n_items) MUI_LT_PASS(u, u, false)
    }
  }
#undef MUI_LT_PASS
}

template <typename T, int WF, int EPI>
static int launch_lt_t(hipStream_t s, const SkinnyParams& p) {
  constexpr int OUT = (EPI == SK_GATEUP) ? 8 : 16;
  const int n_tiles = ceil_div(p.n, OUT);
  const int grid = balanced_grid(n_tiles, 1);  // ~150 KB of LDS: one workgroup per CU
#define MUI_LT_G(NORMV, BSTATV, FULLV, HBV, GPV, SPW)                                                                 \
  hipLaunchKernelGGL((gemm_skinny_lt_kernel<T, WF, NORMV, EPI, BSTATV, FULLV, HBV, GPV>), dim3(grid),                 \
                     dim3(kLtThreads), 0, s, p.w0, p.w1, p.pitch, p.x, p.n, p.k, p.tokens, n_tiles, SPW, p.gamma, p.y, \
                     p.eps, p.residual, p.mul_bias, p.add_bias, p.s0, p.s1, p.s_pitch, p.group_shift)
  // group format: groups of 128 codes carry two (scale, min) pairs with every 256-value pass, larger
  // groups one; smaller groups load the pair of each MFMA step where it is used
#define MUI_LT(NORMV, BSTATV, FULLV, HBV, SPW)                                \
  do {                                                                        \
    if constexpr (WF == WF_U8_GROUP) {                                        \
      if (p.group_shift == 7) MUI_LT_G(NORMV, BSTATV, FULLV, HBV, 2, SPW);    \
      else if (p.group_shift >= 8) MUI_LT_G(NORMV, BSTATV, FULLV, HBV, 1, SPW); \
      else MUI_LT_G(NORMV, BSTATV, FULLV, HBV, 0, SPW);                       \
    } else {                                                                  \
      MUI_LT_G(NORMV, BSTATV, FULLV, HBV, 0, SPW);                            \
    }                                                                         \
  } while (0)
  if (p.k <= kLtWaves * 2 * kLtSub && p.k % 256 == 0) {
    const bool full = p.k == kLtWaves * 2 * kLtSub;
    const bool hb = p.tokens <= 8;
#define MUI_LT_HB(NORMV, FULLV) \
  { if (hb) MUI_LT(NORMV, true, FULLV, true, 1); else MUI_LT(NORMV, true, FULLV, false, 1); }
    if (p.gamma) { if (full) MUI_LT_HB(true, true) else MUI_LT_HB(true, false) }
    else { if (full) MUI_LT_HB(false, true) else MUI_LT_HB(false, false) }
#undef MUI_LT_HB
    return launch_status();
  }
  // streaming: 16-byte chunks of weights and of token rows must not straddle the row end
  if (p.k % (WF == WF_16BIT ? 8 : 16)) return MUI_ERR_UNSUPPORTED;
  const int spw = ceil_div(ceil_div(p.k, kLtSub), kLtWaves);
  const bool hb = p.tokens <= 8;
  if (p.gamma) { if (hb) MUI_LT(true, false, false, true, spw); else MUI_LT(true, false, false, false, spw); }
  else { if (hb) MUI_LT(false, false, false, true, spw); else MUI_LT(false, false, false, false, spw); }
#undef MUI_LT
#undef MUI_LT_G
  return launch_status();
}

int launch_skinny_lt(hipStream_t s, int dtype, int wf, int epilogue, const SkinnyParams& p) {
  if (p.tokens < 1 || p.tokens > 16) return MUI_ERR_UNSUPPORTED;
#define MUI_LT_CASE(TT, WFV, EPIV) \
  if (wf == WFV && epilogue == EPIV) return launch_lt_t<TT, WFV, EPIV>(s, p);
  if (dtype == MUI_DTYPE_F16) {
    MUI_LT_CASE(F16, WF_16BIT, SK_LINEAR)
    MUI_LT_CASE(F16, WF_16BIT, SK_GATEUP)
    MUI_LT_CASE(F16, WF_I8_CHANNEL, SK_LINEAR)
    MUI_LT_CASE(F16, WF_I8_CHANNEL, SK_GATEUP)
    MUI_LT_CASE(F16, WF_U8_GROUP, SK_LINEAR)
    MUI_LT_CASE(F16, WF_U8_GROUP, SK_GATEUP)
  } else if (dtype == MUI_DTYPE_BF16) {
    MUI_LT_CASE(BF16, WF_16BIT, SK_LINEAR)
    MUI_LT_CASE(BF16, WF_16BIT, SK_GATEUP)
    MUI_LT_CASE(BF16, WF_I8_CHANNEL, SK_LINEAR)
    MUI_LT_CASE(BF16, WF_I8_CHANNEL, SK_GATEUP)
    MUI_LT_CASE(BF16, WF_U8_GROUP, SK_LINEAR)
    MUI_LT_CASE(BF16, WF_U8_GROUP, SK_GATEUP)
  }
#undef MUI_LT_CASE
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui
