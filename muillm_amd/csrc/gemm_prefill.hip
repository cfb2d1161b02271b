// Linear layers for more than MUI_MAX_TOKENS tokens (prompts): a tiled matrix-core GEMM with the
// same fused prologue / epilogues as the decode GEMVs.
//
// The reference hands every multi-token call to the framework's GEMM after a standalone RMSNorm
// kernel (csrc/modules/linear_module.cpp:57-79; muillm/modules/linear.py:324-333;
// muillm/modules/gateupdownmlp.py:343-359: norm, two matmuls, SiLU, multiply, matmul, add;
// int8: dequantise the whole matrix first, muillm/modules/quantized/int8linear.py:279-293).
// Here one kernel does y = (W . (gamma * x)) * rsqrt(mean(x^2) + eps) [* scale] [* mul_bias]
// [+ add_bias] [+ residual], or h = silu(G xn) * (U xn), for 16-bit or per-channel int8 weights
// (gamma optional: the host layer normalises prompts with one rmsnorm launch in front, which is
// cheaper than redoing the norm in every row tile).
//
// Work layout (wave64, v_mfma_f32_16x16x32):
//   a workgroup owns a tile of weight rows x tokens and walks K in steps: the weight tile (int8
//   rows converted on the way) and the token tile (gamma * x rounded once to the 16-bit type, sum
//   of squares gathered on the side) are staged through LDS in unpadded rows whose 16-byte
//   chunks are XOR-swizzled (conflict-free 128-bit reads and writes); the loads of step s + 2 are
//   in flight and step s + 1 is on its way into the other LDS stage while step s is multiplied.
//   Tile shapes, chosen per call by rounds of workgroups x cost per round (launch_prefill_t):
//   256 rows x 256 tokens x 64 k on eight waves (4 x 2; sixteen where a norm is fused or the loads
//   cannot go straight into LDS), 128 x 256 x 64 on sixteen (4 x 4), 192 x 256 x 64 on
//   twelve (3 x 4) while the grid covers most of the chip; 128 x 128 x 64 and 96 x 128 x 64 on four
//   waves (2 x 2), two workgroups per CU; 64 x 128 x 128 and 32 x 64 x 256 with a single LDS stage
//   for small matrices. For grids of a round or two of workgroups (short prompts, matrices of a few
//   thousand rows) shapes whose waves ALSO split K, each taking every fourth 32-value chunk of a
//   k-step: 128 x 128 x 128, 128 x 64 x 128 and 64 x 128 x 128 on sixteen waves, 64 x 64 x 256 and
//   32 x 64 x 256 on eight -- the LDS traffic per matrix instruction of a larger tile and four waves per SIMD
//   although there is one workgroup per CU; their partial tiles are exchanged through LDS in three
//   rounds at the end. (int8 weights keep eight / four waves where more would leave threads
//   without a chunk to stage.) With a caller-provided workspace a long K is shared between
//   workgroups as well (XS below).
//   Under the gate/up epilogue half of a wave's rows are gate rows and the other half the up
//   rows of the same outputs, so SiLU * mul happens in registers.
//   Token tiles of one row tile are placed on the same XCD (workgroup id modulo 8) so that the
//   re-reads of its weights hit that XCD's L2.
#include <type_traits>

#include "skinny.cuh"

namespace mui {

// NWR x NWT x NWK waves per workgroup, WR x WT MFMA tiles (16 x 16) per wave: the workgroup tile
// is 16 WR NWR weight rows x 16 WT NWT tokens; KS k-values per step, of which the NWK wave groups
// take every NWK-th 32-value chunk each (their partial tiles are added through LDS at the end).
// dynamically sized LDS: two stages of the 128 x 128 tile exceed the 64 KB a kernel may declare statically
extern __shared__ __align__(16) unsigned char pf_smem[];

template <int ROWS, int TOKS, int KS, int NBUF>
constexpr size_t prefill_lds_bytes() {
  return (size_t)NBUF * (ROWS + TOKS) * KS * 2 + TOKS * 4;
}
// The software-pipelined loop on three stages: three of the weight tile, and of the token tile three
// where 160 KB hold them, else two (the weights come from HBM, the token rows mostly from L2: the
// weights get the extra k-step of lead)
constexpr size_t kLdsPerWorkgroup = 160 * 1024;
template <int ROWS, int TOKS, int KS, int NBUF>
constexpr int pipe_x_stages() {
  return (NBUF == 3 && prefill_lds_bytes<ROWS, TOKS, KS, 3>() > kLdsPerWorkgroup) ? 2 : NBUF;
}
template <int ROWS, int TOKS, int KS, int NBUF>
constexpr size_t pipe_lds_bytes() {  // (no fused norm in this loop: no per-token sums behind the stages)
  return (size_t)(NBUF * ROWS + pipe_x_stages<ROWS, TOKS, KS, NBUF>() * TOKS) * KS * 2;
}

// partial tiles between workgroups: agent-scope relaxed atomics (write-through stores, loads that
// bypass the non-coherent caches; the XCDs do not share an L2)
__device__ __forceinline__ void xs_store(float* dst, f32x4 v) {
  __hip_atomic_store((uint64_t*)dst, ((uint64_t)__float_as_uint(v.y) << 32) | __float_as_uint(v.x), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store((uint64_t*)dst + 1, ((uint64_t)__float_as_uint(v.w) << 32) | __float_as_uint(v.z),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x4 xs_load(const float* src) {
  const uint64_t a = __hip_atomic_load((const uint64_t*)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t b = __hip_atomic_load((const uint64_t*)src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return f32x4{__uint_as_float((uint32_t)a), __uint_as_float((uint32_t)(a >> 32)), __uint_as_float((uint32_t)b),
               __uint_as_float((uint32_t)(b >> 32))};
}

// SiLU(g) * u of the gate/up epilogues, the product rounded to fp32 before it is rounded to the 16-bit
// type. Left alone the compiler merges the product and the conversion into one mixed-precision
// instruction (v_fma_mixlo_f16) for some outputs and not for others, depending on the code around
// them, and the instruction does not round like the pair it replaces: two kernels of the same tile
// then differ in the last place of a few outputs in a hundred thousand. The empty asm keeps the
// product a value of its own.
__device__ __forceinline__ float gateup_f32(float g, float u) {
  float r = silu_f32(g) * u;
  asm volatile("" : "+v"(r));
  return r;
}

// XS: K is also split over p.k_splits workgroups per tile (short prompts on matrices of few row
// tiles, where one workgroup per tile would leave most CUs idle and a long K to each): every
// workgroup delivers its partial tile in fp32 and counts itself in; whoever arrives last adds the
// partials up in index order (the same sum whichever workgroup that is) and runs the epilogue.
// Nobody waits for anybody.
// DMA: both operand tiles go from global memory straight into the LDS stages
// (global_load_lds_dwordx4: lane i of a wave instruction delivers its 16 bytes to LDS slot i of a
// 1 KB block, i.e. eight 128-byte rows of a tile), without staging registers. Staged through
// registers, the tile's sixteen waves have none to spare (128 each), the compiler lets the loaded
// values share registers with the matrix operands and therefore sinks the loads of step s + 2 to the
// end of step s's multiplications -- a barrier and a few instructions before step s + 1 waits for
// them: most of an L2 round trip per k-step with the matrix pipes idle. With the DMA the loads of
// step s + 1 are issued before step s is multiplied and are waited for after it. The swizzle is
// applied on the global side: slot (row r, chunk s) receives logical chunk s ^ swz(r). Needs 16-bit
// weights, K a multiple of the k-step, no fused norm (a prompt's norm is a launch of its own).
// PIPE (with DMA; the 256 x 256 tile on eight waves of 64 x 128): the software-pipelined loop. A wave
// holds the operands of both halves of a k-step in registers; the LDS reads of one half and the
// loads of the step after next are dealt out between the matrix instructions of the other half in
// a pinned order, and the one barrier per step has thirty-two matrix instructions of every wave
// behind it. Timed with the shader's own cycle counter the loop runs at 2283 cycles per k-step of
// 2048 matrix-pipe cycles per SIMD (2150 with the loads taken out) -- and at a shader clock of 1.36 GHz,
// which is what a microsecond figure on this part reflects: the board's power limit sets the clock
// under this load, and operand bytes read from LDS per matrix instruction are what the eight waves
// save over sixteen (192 instead of 256 KB per k-step).
template <typename T, int WF, bool NORM, int EPI, int WR, int WT, int NWR, int NWT, int NWK, int KS, int NBUF,
          bool XS = false, bool DMA = false, bool PIPE = false>
// one tile: the work of workgroup id `vb` of a grid of one workgroup per tile
__device__ __forceinline__ void prefill_gemm_tile(const PrefillGemmParams& p, const unsigned vb) {
  constexpr int kPfThreads = 64 * NWR * NWT * NWK;
  static_assert(!XS || (!NORM && EPI == SK_LINEAR && NBUF == 2), "workgroups that split K: plain linear, two stages");
  static_assert((KS / 32) % NWK == 0 && WT % NWK == 0, "k-split of the waves");
  constexpr int ROWS = 16 * WR * NWR, TOKS = 16 * WT * NWT;
  // The big tiles run in grids of several rounds in which the token tiles of a row tile share its
  // weights through L2: ordinary loads (gate/up at 4096 tokens 893 -> 865 us, down at 2048 350 ->
  // 312 us against non-temporal ones). The small tiles of short prompts stream the weights about
  // once: non-temporal (down at 512 tokens 116 vs 133 us).
  constexpr bool kStreamW = ROWS * TOKS < 128 * 128;
  // LDS rows are unpadded; 16-byte chunk c of row r lives at chunk c ^ swz(r), chosen so that the
  // 16 lanes of a 128-bit access (16 consecutive rows of one logical chunk when reading operands,
  // 16 consecutive chunks when staging) fall into 16 different groups of four banks
  constexpr int PITCH = KS;
  constexpr int CPR = KS / 8;            // 16-byte chunks of 8 elements per row and step
  constexpr int OUT_TILE = (EPI == SK_GATEUP) ? ROWS / 2 : ROWS;  // outputs per workgroup
  // chunks of a k-step per tile and per thread; where the threads do not divide them (twelve
  // waves), the last round of chunks is staged by the first waves only: the others load a valid
  // address all the same (rows and tokens are clamped) and skip the LDS write
  constexpr int XCHUNKS = TOKS * CPR;
  constexpr int WCHUNKS = ROWS * ((WF == WF_16BIT) ? CPR : KS / 16);
  constexpr int XCH = (XCHUNKS + kPfThreads - 1) / kPfThreads;     // token loads per thread and step
  constexpr int WCH = (WCHUNKS + kPfThreads - 1) / kPfThreads;
  constexpr bool XEXACT = XCHUNKS % kPfThreads == 0, WEXACT = WCHUNKS % kPfThreads == 0;
  static_assert(EPI != SK_GATEUP || WR % 2 == 0, "gate/up needs an even number of row tiles per wave");
  static_assert(XCH >= 1 && WCH >= 1 && kPfThreads % CPR == 0, "tile shape");
  static_assert(XCHUNKS >= kPfThreads && WCHUNKS >= kPfThreads, "every thread stages at least one chunk of each operand");
  static_assert((XEXACT || XCHUNKS % 64 == 0) && (WEXACT || WCHUNKS % 64 == 0), "whole waves stage the last round of chunks");
  // NBUF == 2: step s + 1 is written to the other LDS stage while step s is multiplied, one
  // barrier per step instead of two
  typedef uint16_t WStage[ROWS * PITCH];
  typedef uint16_t XStage[TOKS * PITCH];
  WStage* w_lds = (WStage*)pf_smem;
  constexpr int XB = PIPE ? pipe_x_stages<ROWS, TOKS, KS, NBUF>() : NBUF;  // stages of the token tile
  XStage* x_lds = (XStage*)(pf_smem + (size_t)NBUF * sizeof(WStage));
  float* rs_lds = (float*)(pf_smem + (size_t)NBUF * sizeof(WStage) + (size_t)XB * sizeof(XStage));  // (NORM only)

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int wk = wave / (NWR * NWT);         // which share of every k-step
  const int wr = (wave % (NWR * NWT)) / NWT;  // which band of the rows
  const int wt = wave % NWT;                  // which band of the tokens
  // bank group of (row r, chunk c) is (r * chunks-per-row + c) mod 16
  auto swz = [](int r) { return CPR == 8 ? ((r >> 1) & 7) : (r & 15); };

  // workgroup -> (row tile, token tile): consecutive workgroup ids are dealt round-robin to the
  // 8 XCDs, so ids that share id % 8 share an L2; give each XCD whole row tiles
  // (XS: the share of K is the fastest index -- with 8 shares it is the XCD, whose L2 then holds
  // one k-range of x for all row tiles)
  const int xs_share = XS ? (int)(vb % (unsigned)p.k_splits) : 0;
  const int xs_tile = XS ? (int)(vb / (unsigned)p.k_splits) : 0;
  const int xcd = vb & 7, slot = vb >> 3;
  // The eight XCDs (each with an L2 of its own) divide the tile grid p.row_split ways by rows and
  // 8 / p.row_split ways by tokens, interleaved: what every XCD fetches is its share of the weights
  // and its share of x, and the split that fetches least depends on which of the two is bigger (the
  // launcher chooses). Inside its share an XCD's slots walk panels of p.row_group row tiles x all its
  // token tiles, rows fastest: the 32 workgroups that it runs at a time then share few row tiles AND
  // few token tiles (4 x 8 instead of 1 x 32 at 8192 tokens), a third of the fetches again.
  int tile_n, tile_t;
  if constexpr (XS) {
    tile_n = xs_tile / p.t_tiles;
    tile_t = xs_tile % p.t_tiles;
  } else {
    const int rs = p.row_split, ts = 8 / rs;
    const int xr = xcd % rs, xt = xcd / rs;
    const int rows_x = (p.n_tiles + rs - 1) / rs, toks_x = (p.t_tiles + ts - 1) / ts;  // this XCD's share (its edge may lie outside)
    const int per_panel = p.row_group * toks_x;
    const int panel = slot / per_panel, w = slot - panel * per_panel;
    int rows_here = rows_x - panel * p.row_group;
    rows_here = rows_here < p.row_group ? rows_here : p.row_group;
    tile_n = (panel * p.row_group + w % rows_here) * rs + xr;
    tile_t = (w / rows_here) * ts + xt;
  }
  if (tile_n >= p.n_tiles || tile_t >= p.t_tiles) return;  // uniform for the workgroup, before any barrier
  const int o0 = tile_n * OUT_TILE;  // first output of the tile
  const int t0 = tile_t * TOKS;      // first token of the tile

  // local weight row r -> matrix row. linear: o0 + r. gate/up: of a wave's 16 WR rows the first
  // half are gate rows, the second half the up rows of the same outputs. Rows past the matrix read
  // its last row (their outputs are never stored). Kept as 32-bit indices: the addresses are
  // formed at the loads, 64-bit pointers per staged chunk would cost twice the registers.
  auto weight_row = [&](int r, bool& up) -> int {
    int o;
    if constexpr (EPI == SK_GATEUP) {
      constexpr int HALF = 8 * WR;  // outputs per wave
      const int h = r / (2 * HALF), within = r % (2 * HALF);
      o = o0 + h * HALF + within % HALF;
      up = within >= HALF;
    } else {
      o = o0 + r;
      up = false;
    }
    return o < p.n ? o : p.n - 1;
  };

  // ---- staging assignment: 16-byte chunk c = t + threads * i of a tile is row c / chunks-per-row,
  // column c % chunks-per-row (the column is the same for every i)
  const int xcol = t % CPR;
  int xtok[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int tk = t0 + (t + kPfThreads * i) / CPR;
    xtok[i] = tk < p.tokens ? tk : p.tokens - 1;
  }
  constexpr int WCPR = (WF == WF_16BIT) ? CPR : KS / 16;  // weight chunks per row (int8: 16 codes each)
  const int wcol = t % WCPR;
  int wrow[WCH];     // matrix row; bit 30 set: a row of the up matrix
#pragma unroll
  for (int i = 0; i < WCH; ++i) {
    bool up;
    const int o = weight_row((t + kPfThreads * i) / WCPR, up);
    wrow[i] = o | (up ? (1 << 30) : 0);
  }
  auto wptr = [&](int i) -> const uint8_t* {
    if constexpr (EPI == SK_GATEUP)
      return ((wrow[i] >> 30) ? p.w1 : p.w0) + (long)(wrow[i] & ((1 << 30) - 1)) * p.pitch;
    else
      return p.w0 + (long)wrow[i] * p.pitch;
  };

  const int n_steps = (p.k + KS - 1) / KS;
  // DMA: per wave instruction q the source of this lane's slot (fixed but for the k-step's offset)
  constexpr int kNWaves = kPfThreads / 64;
  constexpr int DRI = 64 / CPR;  // tile rows per load instruction (8 with k-steps of 64, 4 with 128, 2 with 256)
  constexpr int WQ = DMA ? ROWS / (DRI * kNWaves) : 1, XQ = DMA ? TOKS / (DRI * kNWaves) : 1;
  // per wave instruction q: a base address that is the same for the wave's lanes (the matrix, or the
  // up matrix for the instructions that cover up rows: eight consecutive tile rows never straddle
  // the two) and this lane's 32-bit byte offset from it; only the base moves with the k-step
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  unsigned dma_wo[WQ], dma_xo[XQ];
  if constexpr (DMA) {
    static_assert(!DMA || (WF == WF_16BIT && !NORM && NBUF >= 2 && !XS && CPR >= 8 && CPR <= 64), "what the DMA path covers");
    static_assert(!DMA || (WQ >= 1 && XQ >= 1 && WQ * DRI * kNWaves == ROWS && XQ * DRI * kNWaves == TOKS), "whole 1 KB blocks per wave");
    static_assert(!DMA || EPI != SK_GATEUP || (8 * WR) % DRI == 0, "gate and up rows change at multiples of a block's rows");
    const int sr = lane / CPR, sc = lane % CPR;
#pragma unroll
    for (int q = 0; q < WQ; ++q) {
      const int r = (q * kNWaves + wave) * DRI + sr;
      bool up;
      const int o = weight_row(r, up);
      dma_wo[q] = (unsigned)((long)o * p.pitch + ((sc ^ swz(r)) * 16));
    }
#pragma unroll
    for (int q = 0; q < XQ; ++q) {
      const int r = (q * kNWaves + wave) * DRI + sr;
      int tk = t0 + r;
      tk = tk < p.tokens ? tk : p.tokens - 1;
      dma_xo[q] = (unsigned)((long)tk * p.k * 2 + ((sc ^ swz(r)) * 16));
    }
  }
  // load instruction i of a k-step: the weight blocks first, then the token blocks
  auto dma_one = [&](int step, int buf, int i) {
    const long kb = (long)step * KS * 2;
    // (the lane offset is made opaque to the optimiser: widened to 64 bits outside the loop it would
    // cost a register pair and a 64-bit add per load instead of the scalar-base addressing mode)
    if (i < WQ) {
      const int q = i;
      bool up;
      weight_row((q * kNWaves + wave_u) * DRI, up);
      const uint8_t* base = ((EPI == SK_GATEUP && up) ? p.w1 : p.w0) + kb;
      unsigned off = dma_wo[q];
      asm volatile("" : "+v"(off));
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + off),
                                       (__attribute__((address_space(3))) void*)&w_lds[buf][(q * kNWaves + wave_u) * DRI * PITCH],
                                       16, 0, 0);
    } else {
      const int q = i - WQ;
      unsigned off = dma_xo[q];
      asm volatile("" : "+v"(off));
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)((const uint8_t*)p.x + kb + off),
                                       (__attribute__((address_space(3))) void*)&x_lds[buf][(q * kNWaves + wave_u) * DRI * PITCH],
                                       16, 0, 0);
    }
  };
  auto dma_step = [&](int step, int buf) {
#pragma unroll
    for (int i = 0; i < WQ + XQ; ++i) dma_one(step, buf, i);
  };
  // one k-step of the tile in registers, on its way from global memory to LDS
  struct Stage { u32x4 w[WCH], x[XCH], g; uint32_t pr[WF == WF_U8_GROUP ? WCH : 1]; };  // pr: the (scale, min) pair of a chunk of codes
  auto load_step = [&](int step, Stage& r) {
    // steps past the last one re-read step 0 (never stored): that keeps the loads out of branches;
    // chunks past the end of the row read the row's first chunk and are zeroed on the way to LDS
    const int k0 = step < n_steps ? step * KS : 0;
    const int xk = k0 + xcol * 8;
    const int xoff = xk + 8 <= p.k ? xk : 0;
#pragma unroll
    for (int i = 0; i < XCH; ++i) r.x[i] = ld16(p.x + (long)xtok[i] * p.k + xoff);
    if constexpr (NORM) r.g = ld16(p.gamma + xoff);
    if constexpr (WF == WF_16BIT) {
#pragma unroll
      for (int i = 0; i < WCH; ++i) r.w[i] = ld16_sel<kStreamW>(wptr(i) + 2L * xoff);
    } else {
      const int wk = k0 + wcol * 16;
      const int woff = wk + 16 <= p.k ? wk : 0;
#pragma unroll
      for (int i = 0; i < WCH; ++i) r.w[i] = ld16_sel<kStreamW>(wptr(i) + woff);
      if constexpr (WF == WF_U8_GROUP) {  // a chunk of 16 codes lies in one group (groups of 16 or more)
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
          const uint16_t* pairs = ((EPI == SK_GATEUP && (wrow[i] >> 30)) ? p.s1 : p.s0) + (long)(wrow[i] & ((1 << 30) - 1)) * p.s_pitch;
          r.pr[i] = ld4(pairs + 2 * (woff >> p.group_shift));
        }
      }
    }
  };

  float ss[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) ss[i] = 0.f;
  auto store_step = [&](int step, int buf, const Stage& r) {
    const int k0 = step * KS;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const bool xlive = k0 + xcol * 8 + 8 <= p.k;
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      if (!XEXACT && t + kPfThreads * i >= XCHUNKS) continue;  // uniform per wave
      float sq = 0.f;
      u32x4 b = make_b<T, NORM>(r.x[i], NORM ? r.g : r.x[i], sq);
      b = xlive ? b : zero;
      ss[i] += xlive ? sq : 0.f;
      const int row = (t + kPfThreads * i) / CPR;
      *(u32x4*)&x_lds[buf][row * PITCH + ((xcol ^ swz(row)) * 8)] = b;
    }
    if constexpr (WF == WF_16BIT) {
#pragma unroll
      for (int i = 0; i < WCH; ++i) {
        if (!WEXACT && t + kPfThreads * i >= WCHUNKS) continue;
        const int row = (t + kPfThreads * i) / CPR;
        *(u32x4*)&w_lds[buf][row * PITCH + ((xcol ^ swz(row)) * 8)] = xlive ? r.w[i] : zero;
      }
    } else {
      const bool wlive = k0 + wcol * 16 + 16 <= p.k;
#pragma unroll
      for (int i = 0; i < WCH; ++i) {
        if (!WEXACT && t + kPfThreads * i >= WCHUNKS) continue;
        u32x4 lo, hi;
        if constexpr (WF == WF_U8_GROUP) {  // u8 * scale + min rounded once: what the dequantisation kernel writes
          lo = convert_a_pair<T>(r.w[i].x, r.w[i].y, r.pr[i]);
          hi = convert_a_pair<T>(r.w[i].z, r.w[i].w, r.pr[i]);
        } else {
          lo = convert_a<T, WF>(r.w[i].x, r.w[i].y, nullptr, 0, 0);
          hi = convert_a<T, WF>(r.w[i].z, r.w[i].w, nullptr, 0, 0);
        }
        const int row = (t + kPfThreads * i) / WCPR;
        uint16_t* dst = &w_lds[buf][row * PITCH];
        *(u32x4*)(dst + (((2 * wcol) ^ swz(row)) * 8)) = wlive ? lo : zero;
        *(u32x4*)(dst + (((2 * wcol + 1) ^ swz(row)) * 8)) = wlive ? hi : zero;
      }
    }
  };

  f32x4 acc[WR][WT];
#pragma unroll
  for (int i = 0; i < WR; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if constexpr (NORM) {
    for (int i = t; i < TOKS; i += kPfThreads) rs_lds[i] = 0.f;
  }

  const int a_base = (wr * 16 * WR + (lane & 15)) * PITCH;  // rows 16 i + lane % 16: the swizzle depends on the lane only
  const int b_base = (wt * 16 * WT + (lane & 15)) * PITCH;
  const int lsw = swz(lane & 15), lg = lane >> 4;
  auto multiply = [&](int buf) {
#pragma unroll
    for (int kk = 0; kk < KS / 32 / NWK; ++kk) {
      const int ks = kk * NWK + wk;
      u32x4 a[WR], b[WT];
#pragma unroll
      for (int j = 0; j < WT; ++j) b[j] = *(const u32x4*)&x_lds[buf][b_base + j * 16 * PITCH + (((ks * 4 + lg) ^ lsw) * 8)];
#pragma unroll
      for (int i = 0; i < WR; ++i) a[i] = *(const u32x4*)&w_lds[buf][a_base + i * 16 * PITCH + (((ks * 4 + lg) ^ lsw) * 8)];
#pragma unroll
      for (int i = 0; i < WR; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = mfma16x16x32<T>(a[i], b[j], acc[i][j]);
    }
  };
  // k-steps of this workgroup: all of them, or its share
  const int sb = XS ? (int)((long)n_steps * xs_share / p.k_splits) : 0;
  const int se = XS ? (int)((long)n_steps * (xs_share + 1) / p.k_splits) : n_steps;
  Stage r0;
  if constexpr (DMA && PIPE) {
    // Two operand register sets per wave: the LDS reads of one half of a k-step are issued while the
    // other half is multiplied, one read per two matrix instructions, so a wave always has sixteen
    // or more matrix instructions to issue that wait for nothing; the barrier sits between the two
    // halves of a step, with the second half's multiplications behind it.
    static_assert(!PIPE || (KS == 64 && NWK == 1), "two halves per k-step");
    u32x4 a[2][WR], b[2][WT];
    // operand read i of a half step: the WT token operands first, then the WR weight operands
    // (bw / bx: the stage of the weight tile / of the token tile)
    auto read_one = [&](int bw, int bx, int kk, int set, int i) {
      if (i < WT) b[set][i] = *(const u32x4*)&x_lds[bx][b_base + i * 16 * PITCH + (((kk * 4 + lg) ^ lsw) * 8)];
      else a[set][i - WT] = *(const u32x4*)&w_lds[bw][a_base + (i - WT) * 16 * PITCH + (((kk * 4 + lg) ^ lsw) * 8)];
    };
    auto read_ops = [&](int bw, int bx, int kk, int set) {
#pragma unroll
      for (int i = 0; i < WT + WR; ++i) read_one(bw, bx, kk, set, i);
    };
    auto mm = [&](int set, int i0, int i1) {
#pragma unroll
      for (int i = i0; i < i1; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = mfma16x16x32<T>(a[set][i], b[set][j], acc[i][j]);
    };
    // pinned order of a region: `per` matrix instructions, then one instruction of the masked kind
    // (0x100 LDS read, 0x010 memory load), `n` times; then the remaining matrix instructions
    auto pin = [&](auto maskc, auto perc, auto nc, auto totalc) {
      constexpr int MASK = decltype(maskc)::value, PER = decltype(perc)::value, N = decltype(nc)::value,
                    TOTAL = decltype(totalc)::value;
#pragma unroll
      for (int r = 0; r < N; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
        __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
      }
      if constexpr (TOTAL > PER * N) __builtin_amdgcn_sched_group_barrier(0x008, TOTAL - PER * N, 0);
    };
    static_assert(!PIPE || WR * WT >= 2 * (WR + WT), "two matrix instructions per read");
    // NBUF stages: the loads of step s + NBUF are issued in the second half of step s, into the stage
    // that step s has just finished reading, and must have landed by the middle of step s + NBUF - 1:
    // one k-step of lead with two stages, two with three (the 128 x 256 tile, whose k-step is too short
    // to cover a trip to L2 under load). Where 160 KB do not hold three stages of both tiles the token
    // tile keeps two (XB): a step then issues the token loads of step s + 2 FIRST and the weight loads
    // of step s + 3 after them, so that "all but the newest WQ loads" is what the middle of the next
    // step waits for.
    static_assert(!PIPE || NBUF == 2 || NBUF == 3, "stages of the pipelined loop");
    static_assert(!PIPE || (NBUF - 1) * (WQ + XQ) <= 63, "the waits' load counts");
    // s_waitcnt immediate for "at most n loads outstanding" (six bits: [3:0] and [15:14])
    constexpr auto vm = [](int n) { return (n & 15) | ((n >> 4) << 14); };
    if constexpr (NBUF == 2) {
      dma_step(sb, 0);
      if (sb + 1 < se) dma_step(sb + 1, 1);
      if (sb + 1 < se) __builtin_amdgcn_s_waitcnt(0x0F70 | (WQ + XQ));  // all but the second step's loads
      else __builtin_amdgcn_s_waitcnt(0x0F70);
    } else if constexpr (XB == NBUF) {
#pragma unroll
      for (int a = 0; a < NBUF; ++a) dma_step(sb + a < se ? sb + a : se - 1, a);
      __builtin_amdgcn_s_waitcnt(0x0F70 | vm((NBUF - 1) * (WQ + XQ)));  // the first step's loads
    } else {
      static_assert(!PIPE || XB == NBUF || (NBUF == 3 && XB == 2), "stages of the token tile");
#pragma unroll
      for (int a = 0; a < NBUF; ++a) {  // W(0) X(0) W(1) X(1) W(2)
        const int st = sb + a < se ? sb + a : se - 1;
#pragma unroll
        for (int i = 0; i < WQ; ++i) dma_one(st, a, i);
        if (a < XB) {
#pragma unroll
          for (int i = 0; i < XQ; ++i) dma_one(st, a, WQ + i);
        }
      }
      __builtin_amdgcn_s_waitcnt(0x0F70 | vm(2 * WQ + XQ));  // the first step's loads
    }
    __syncthreads();
    read_ops(0, 0, 0, 0);
    int buf = 0, bx = 0;
    for (int s = sb; s < se; ++s) {
      const int nbuf = buf + 1 == NBUF ? 0 : buf + 1;
      const int nbx = bx + 1 == XB ? 0 : bx + 1;
      read_ops(buf, bx, 1, 1);
      mm(0, 0, WR);
      pin(std::integral_constant<int, 0x100>{}, std::integral_constant<int, 2>{}, std::integral_constant<int, WR + WT>{},
          std::integral_constant<int, WR * WT>{});
      __builtin_amdgcn_sched_barrier(0);
      // this wave's reads of the stage have returned, its share of the next stage has landed (loads
      // return in order: all but those of the NBUF - 2 steps after it)
      __builtin_amdgcn_s_waitcnt(0x0070 | vm(XB == NBUF ? (NBUF - 2) * (WQ + XQ) : WQ));
      __syncthreads();
      // (the last two steps load the last step once more, into a stage that nobody reads any more,
      // and read stale operands that nobody multiplies: no branch, one schedule)
      // second half: one row of matrix instructions per region, each with its share of the next
      // half's operand reads and of the loads of the step after next -- spread over the whole half,
      // so that the eight waves, which all leave the barrier together, do not queue their loads
      // faster than the CU's memory pipeline takes them (a wave that waits to issue a load does not
      // issue the matrix instructions behind it either)
      const int nxt = s + NBUF < se ? s + NBUF : se - 1;
      const int nxt_x = s + XB < se ? s + XB : se - 1;
      // (the reads in all but the last region where they fit there: the first matrix instruction of
      // the next half waits for the last of them)
      constexpr int NL = WQ + XQ, NR = WR + WT;
      constexpr int LD = (NL + WR - 1) / WR;                             // loads per region
      constexpr int RD_EARLY = (NR + WR - 2) / (WR - 1);                 // reads per region, last region free
      constexpr bool EARLY = RD_EARLY + LD <= WT;
      constexpr int RD = EARLY ? RD_EARLY : (NR + WR - 1) / WR;
      static_assert(!PIPE || RD + LD <= WT, "schedule of the second half: a matrix instruction per read and load");
      auto region = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        constexpr int nl = NL - i * LD < 0 ? 0 : (NL - i * LD < LD ? NL - i * LD : LD);
        constexpr int nr = (EARLY && i == WR - 1) || NR - i * RD < 0 ? 0 : (NR - i * RD < RD ? NR - i * RD : RD);
#pragma unroll
        for (int l = 0; l < nl; ++l) {
          constexpr int j = i * LD;
          if constexpr (XB == NBUF) {
            dma_one(nxt, buf, j + l);
          } else {  // token blocks first
            if (j + l < XQ) dma_one(nxt_x, bx, WQ + j + l);
            else dma_one(nxt, buf, j + l - XQ);
          }
        }
#pragma unroll
        for (int r = 0; r < nr; ++r) read_one(nbuf, nbx, 0, 0, i * RD + r);
        mm(1, i, i + 1);
        // a matrix instruction, a load, ..., a matrix instruction, a read, ... (loads first: they have the longer way)
#pragma unroll
        for (int g = 0; g < nl; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
#pragma unroll
        for (int g = 0; g < nr; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        if constexpr (WT - nl - nr > 0) __builtin_amdgcn_sched_group_barrier(0x008, WT - nl - nr, 0);
        __builtin_amdgcn_sched_barrier(0);
      };
      static_assert(!PIPE || (WR >= 2 && WR <= 4), "regions of the second half");
      region(std::integral_constant<int, 0>{});
      region(std::integral_constant<int, 1>{});
      if constexpr (WR > 2) region(std::integral_constant<int, 2>{});
      if constexpr (WR > 3) region(std::integral_constant<int, 3>{});
      buf = nbuf;
      bx = nbx;
    }
  } else if constexpr (DMA) {
    // NBUF stages, NBUF - 1 k-steps of loads in flight. Every pass issues a step's loads -- past the
    // last step the last one once more, into a stage nobody reads any more --, so that "all but the
    // newest (NBUF - 2) steps' loads" is a fixed count to wait for (loads return in order). (Used with
    // two stages; three stages on the short prompts' tiles whose waves split K lost to their
    // register-staged loops.)
    constexpr int LEAD = NBUF - 1;
    static_assert(!DMA || PIPE || (LEAD - 1) * (WQ + XQ) <= 15, "the wait's load count");
#pragma unroll
    for (int a = 0; a < LEAD; ++a) dma_step(sb + a < se ? sb + a : se - 1, a);
    int buf = 0, fill = LEAD;  // stage of step s; stage that step s + LEAD goes to (= the one step s - 1 used)
    for (int s = sb; s < se; ++s) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | ((LEAD - 1) * (WQ + XQ)));  // this wave's blocks of step s have landed
      __syncthreads();  // ... and everybody's; everybody is done reading step s - 1
      dma_step(s + LEAD < se ? s + LEAD : se - 1, fill);
      multiply(buf);
      buf = buf + 1 == NBUF ? 0 : buf + 1;
      fill = fill + 1 == NBUF ? 0 : fill + 1;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();  // the stages are free (and no load is still on its way into them)
  } else if constexpr (NBUF == 2) {
    load_step(sb, r0);
    // two LDS stages: step s + 1 moves from the registers to the other stage and step s + 2 is
    // requested from memory before step s is multiplied, so that the LDS writes and the loads
    // proceed under the matrix instructions; one barrier per step. (A second register stage
    // pushes the 128 x 128 tile past 256 registers per lane: one workgroup per CU instead of two,
    // 686 -> 846 us on 2048 x 28672 x 4096; on the tiles whose waves split K, which have the
    // registers to spare, it bought nothing either: 46 vs 41 us on 256 x 6144 x 4096 -- the
    // staging rate of a CU, about 35 GB/s from L2 in every shape, is the limit, not the latency.)
    store_step(sb, 0, r0);
    load_step(sb + 1, r0);
    __syncthreads();
    for (int s = sb; s < se; ++s) {
      if (s + 1 < se) store_step(s + 1, (s + 1 - sb) & 1, r0);  // uniform branch, no loads inside
      load_step(s + 2, r0);
      multiply((s - sb) & 1);
      if constexpr (NWR * NWT * NWK == 12) {
        // twelve waves have 168 registers each: the global loads stay in front of the multiply
        // (left alone the compiler sinks them to its end, a barrier before they are needed) and
        // the next operands are requested while the current ones are multiplied (QKV at 4096
        // tokens 208 -> 204 us)
        __builtin_amdgcn_sched_group_barrier(0x020, WCH + XCH + (NORM ? 1 : 0), 0);
        static_assert(NWR * NWT * NWK != 12 || (WR == 4 && WT == 4 && KS / 32 / NWK == 2), "pinned order of the twelve-wave tile");
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);  // b0-3, a0, a1
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // a2
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // a3
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // second half of the k-step: b0, b1
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);  // b2, b3, a0, a1
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      }
      __syncthreads();
    }
  } else {
    load_step(sb, r0);
    for (int s = 0; s < n_steps; ++s) {
      __syncthreads();  // the previous step's operands have been read
      store_step(s, 0, r0);
      __syncthreads();
      load_step(s + 1, r0);  // in flight during this step's multiplications
      multiply(0);
    }
  }

  // ---- waves that split K: wave group g keeps token tiles [g JW, (g + 1) JW) of its tile and
  // receives the other groups' partial sums for them through LDS (the stage buffers are free: the
  // loop ended with a barrier)
  constexpr int JW = WT / NWK;
  if constexpr (NWK > 1) {
    // NWK - 1 rounds: in round r group g hands the tiles of group (g + r) % NWK to it and takes its
    // own from group (g - r) % NWK; one area per wave
    constexpr int AREA = WR * JW * 64;  // f32x4 slots per wave and round
    static_assert((size_t)NWK * NWR * NWT * AREA * 16 <= (size_t)NBUF * (ROWS + TOKS) * KS * 2,
                  "the partial tiles of a round must fit the stage buffers");
    f32x4* red = (f32x4*)pf_smem;
    const int wrt = wave % (NWR * NWT);
#pragma unroll
    for (int r = 1; r < NWK; ++r) {
      const int to = (wk + r) % NWK, from = (wk + NWK - r) % NWK;
      f32x4* out = red + ((long)wrt * NWK + wk) * AREA;
#pragma unroll
      for (int d = 0; d < NWK; ++d) {
        if (d != to) continue;  // uniform per wave; d is a constant inside
#pragma unroll
        for (int i = 0; i < WR; ++i)
#pragma unroll
          for (int jj = 0; jj < JW; ++jj) out[(i * JW + jj) * 64 + lane] = acc[i][d * JW + jj];
      }
      __syncthreads();
      const f32x4* in = red + ((long)wrt * NWK + from) * AREA;
#pragma unroll
      for (int d = 0; d < NWK; ++d) {
        if (d != wk) continue;
#pragma unroll
        for (int i = 0; i < WR; ++i)
#pragma unroll
          for (int jj = 0; jj < JW; ++jj) {
            const f32x4 v = in[(i * JW + jj) * 64 + lane];
            f32x4& a = acc[i][d * JW + jj];
            a = f32x4{a.x + v.x, a.y + v.y, a.z + v.z, a.w + v.w};
          }
      }
      __syncthreads();
    }
  }

  // ---- workgroups that split K: deliver, count, and the last one adds up
  if constexpr (XS) {
    constexpr int SLOT = (kPfThreads / 64) * WR * JW * 64 * 4;  // floats per partial tile
    float* mine = p.part + ((long)xs_tile * p.k_splits + xs_share) * SLOT;
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      if (NWK > 1 && j / JW != wk) continue;  // tiles of another wave group (already handed over)
#pragma unroll
      for (int i = 0; i < WR; ++i) xs_store(mine + (((wave * WR + i) * JW + j % JW) * 64 + lane) * 4, acc[i][j]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's stores have arrived
    __syncthreads();                                    // ... and everybody's
    __shared__ unsigned xs_arrived;
    // release (everybody's partial tile, ordered before this thread by the barrier, is visible
    // device-wide before the count goes up) and acquire (the workgroup that sees the full count sees
    // every tile): the ordering the memory model gives, not one chip's write acknowledgements
    if (t == 0) xs_arrived = __hip_atomic_fetch_add(&p.part_count[xs_tile], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (xs_arrived + 1 != (unsigned)p.k_splits) return;  // uniform: somebody else finishes the tile
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      if (NWK > 1 && j / JW != wk) continue;
#pragma unroll
      for (int i = 0; i < WR; ++i) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int c = 0; c < p.k_splits; ++c) {
      const float* theirs = p.part + ((long)xs_tile * p.k_splits + c) * SLOT;
#pragma unroll
      for (int j = 0; j < WT; ++j) {
        if (NWK > 1 && j / JW != wk) continue;
#pragma unroll
        for (int i = 0; i < WR; ++i) {
          const f32x4 v = xs_load(theirs + (((wave * WR + i) * JW + j % JW) * 64 + lane) * 4);
          f32x4& a = acc[i][j];
          a = f32x4{a.x + v.x, a.y + v.y, a.z + v.z, a.w + v.w};
        }
      }
    }
    if (t == 0) __hip_atomic_store(&p.part_count[xs_tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- per-token rsqrt(mean(x^2) + eps): every thread adds the squares it staged to its tokens
  if constexpr (NORM) {
#pragma unroll
    for (int i = 0; i < XCH; ++i)
      if (XEXACT || t + kPfThreads * i < XCHUNKS) atomicAdd(&rs_lds[(t + kPfThreads * i) / CPR], ss[i]);
    __syncthreads();
    for (int i = t; i < TOKS; i += kPfThreads) rs_lds[i] = rsqrtf(rs_lds[i] / (float)p.k + p.eps);
    __syncthreads();
  }

  // ---- epilogue. acc[i][j][e]: token t0 + 16 WT wt + 16 j + lane % 16, local row 16 WR wr + 16 i +
  // 4 (lane / 16) + e
  const int tok_l = wt * 16 * WT + (lane & 15);
  const int sub = (lane >> 4) * 4;
  constexpr int OT = (EPI == SK_GATEUP) ? WR / 2 : WR;  // output row tiles per wave
  // Whole tiles of the software-pipelined kernels leave through LDS: a lane's accumulators are four
  // outputs of one token (8 bytes of a row of y, sixteen rows per store instruction), which reaches
  // memory as 32-byte pieces -- and the residual the same way. Instead the wave's block of y goes
  // through a wave-private LDS tile [token][output] (the operand stages are free by now) and is
  // loaded / stored 16 bytes per lane in whole rows of the wave tile (128 bytes per token with 64
  // outputs per wave): the residual rows come in that way, are picked up in accumulator layout,
  // replaced in place by the rounded results and leave that way. 64 tokens per pass. Chunk c of
  // row r sits in slot (c + r) % 8 of its 128-byte LDS row.
  if constexpr (PIPE) {
    constexpr int OW = 16 * OT;                  // outputs per wave
    constexpr int CE = OW / 8;                   // 16-byte chunks per row of the wave's block
    constexpr int LPR = CE > 4 ? 8 : 4;          // lanes per row in the row-wise phases
    constexpr int RPI = kWave / LPR;             // rows per row-wise instruction
    constexpr int JG = WT < 4 ? WT : 4;          // token tiles of 16 per pass
    constexpr int NI = 16 * JG / RPI;            // row-wise instructions per pass
    static_assert(!PIPE || (WT % JG == 0 && CE <= 8 && (size_t)kNWaves * 16 * JG * 128 <= (size_t)NBUF * sizeof(WStage) + (size_t)XB * sizeof(XStage)),
                  "the waves' epilogue tiles fit the operand stages");
    const bool whole = t0 + TOKS <= p.tokens && o0 + OUT_TILE <= p.n && (p.y_pitch & 7) == 0 &&
                       (((uintptr_t)p.y | (uintptr_t)p.residual) & 15) == 0;  // uniform
    if (whole) {
      __builtin_amdgcn_s_waitcnt(0x0070);  // this wave's last (unused) loads have landed, its reads returned
      __syncthreads();                     // ... and everybody's: the stages are free
      unsigned char* et = pf_smem + (size_t)wave_u * (16 * JG * 128);
      const int ow0 = o0 + wr * OW;                    // first output of the wave
      const int rrow = lane / LPR, rch = lane % LPR;   // row-wise phases: row inside an instruction, chunk
      const int arow = lane & 15, ag = lane >> 4;      // accumulator layout: token row, group of four outputs
#pragma unroll
      for (int j0 = 0; j0 < WT; j0 += JG) {
        const int tw0 = t0 + wt * 16 * WT + 16 * j0;   // first token of the pass
        if constexpr (EPI != SK_GATEUP) {
          if (p.residual) {
            u32x4 rr[NI];
#pragma unroll
            for (int it = 0; it < NI; ++it) {
              const int row = it * RPI + rrow;
              rr[it] = ld16(p.residual + (long)(tw0 + row) * p.y_pitch + ow0 + (rch < CE ? rch : 0) * 8);
            }
#pragma unroll
            for (int it = 0; it < NI; ++it) {
              const int row = it * RPI + rrow;
              if (rch < CE) *(u32x4*)(et + row * 128 + ((rch + row) & 7) * 16) = rr[it];
            }
          }
        }
#pragma unroll
        for (int jj = 0; jj < JG; ++jj) {
          const int j = j0 + jj;
          const int row = 16 * jj + arow;
#pragma unroll
          for (int i = 0; i < OT; ++i) {
            unsigned char* slot = et + row * 128 + (((2 * i + (ag >> 1)) + row) & 7) * 16 + (ag & 1) * 8;
            float v[4];
            float res4[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (EPI != SK_GATEUP) {
              if (p.residual) {
                const u32x2 rq = *(const u32x2*)slot;
                res4[0] = T::one((uint16_t)(rq.x & 0xffffu)); res4[1] = T::one((uint16_t)(rq.x >> 16));
                res4[2] = T::one((uint16_t)(rq.y & 0xffffu)); res4[3] = T::one((uint16_t)(rq.y >> 16));
              }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int oe = ow0 + 16 * i + 4 * ag + e;
              if constexpr (EPI == SK_GATEUP) {
                v[e] = gateup_f32(acc[i][j][e], acc[i + OT][j][e]);
              } else {
                float r = acc[i][j][e];
                if (p.mul_bias) r *= T::one(p.mul_bias[oe]);
                if (p.add_bias) r += T::one(p.add_bias[oe]);
                if (p.residual) r += res4[e];
                v[e] = r;
              }
            }
            u32x2 pk;
            pk.x = (uint32_t)T::pack(v[0]) | ((uint32_t)T::pack(v[1]) << 16);
            pk.y = (uint32_t)T::pack(v[2]) | ((uint32_t)T::pack(v[3]) << 16);
            *(u32x2*)slot = pk;
          }
        }
#pragma unroll
        for (int it = 0; it < NI; ++it) {
          const int row = it * RPI + rrow;
          if (rch < CE) {
            const u32x4 out = *(const u32x4*)(et + row * 128 + ((rch + row) & 7) * 16);
            *(u32x4*)(p.y + (long)(tw0 + row) * p.y_pitch + ow0 + rch * 8) = out;
          }
        }
      }
      return;
    }
  }
  // The four residual values of a lane and tile are adjacent: one 8-byte load where the row allows
  // it, and all of a wave's loads requested before the first store (y may be the residual itself:
  // every lane reads exactly what it writes later; behind a store the compiler has to keep a load
  // where it is). Four 2-byte loads per output, each waited for, cost the 256 x 256 tile 39 us of
  // epilogue against 10 us without a residual.
  const bool res_quads = EPI != SK_GATEUP && p.residual != nullptr && (p.y_pitch & 3) == 0;
  u32x2 resq[WT][OT];
  if constexpr (EPI != SK_GATEUP) {
    if (res_quads) {
#pragma unroll
      for (int j = 0; j < WT; ++j) {
        if (NWK > 1 && j / JW != wk) continue;
        int tok = t0 + tok_l + 16 * j;
        tok = tok < p.tokens ? tok : p.tokens - 1;
#pragma unroll
        for (int i = 0; i < OT; ++i) {
          int o = o0 + wr * 16 * OT + 16 * i + sub;
          o = o + 3 < p.n ? o : 0;  // (never used then)
          resq[j][i] = *(const u32x2*)(p.residual + (long)tok * p.y_pitch + o);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < WT; ++j) {
    if (NWK > 1 && j / JW != wk) continue;  // another wave group finishes this token tile
    const int tl = tok_l + 16 * j;
    const int tok = t0 + tl;
    if (tok >= p.tokens) continue;
    const float rs = NORM ? rs_lds[tl] : 1.f;
#pragma unroll
    for (int i = 0; i < OT; ++i) {
      const int o = o0 + wr * 16 * OT + 16 * i + sub;
      if (o >= p.n) continue;
      float v[4];
      const bool quad = o + 3 < p.n && (p.y_pitch & 3) == 0;
      float res4[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (EPI != SK_GATEUP) {
        if (res_quads && quad) {
          const u32x2 rq = resq[j][i];
          res4[0] = T::one((uint16_t)(rq.x & 0xffffu)); res4[1] = T::one((uint16_t)(rq.x >> 16));
          res4[2] = T::one((uint16_t)(rq.y & 0xffffu)); res4[3] = T::one((uint16_t)(rq.y >> 16));
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int oe = o + e < p.n ? o + e : p.n - 1;
        if constexpr (EPI == SK_GATEUP) {
          float g = acc[i][j][e] * rs, u = acc[i + OT][j][e] * rs;
          if constexpr (WF == WF_I8_CHANNEL) {
            g *= T::one(p.s0[(long)oe * p.s_pitch]);
            u *= T::one(p.s1[(long)oe * p.s_pitch]);
          }
          v[e] = gateup_f32(g, u);
        } else {
          float r = acc[i][j][e] * rs;
          if constexpr (WF == WF_I8_CHANNEL) r *= T::one(p.s0[(long)oe * p.s_pitch]);
          if (p.mul_bias) r *= T::one(p.mul_bias[oe]);
          if (p.add_bias) r += T::one(p.add_bias[oe]);
          if (p.residual) r += quad ? res4[e] : T::one(p.residual[(long)tok * p.y_pitch + oe]);
          v[e] = r;
        }
      }
      uint16_t* dst = p.y + (long)tok * p.y_pitch + o;
      if (quad) {
        u32x2 pk;
        pk.x = (uint32_t)T::pack(v[0]) | ((uint32_t)T::pack(v[1]) << 16);
        pk.y = (uint32_t)T::pack(v[2]) | ((uint32_t)T::pack(v[3]) << 16);
        *(u32x2*)dst = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (o + e < p.n) dst[e] = T::pack(v[e]);
      }
    }
  }
}

// The kernel: one tile per workgroup, or -- the software-pipelined tiles, whose grids are rounds of
// one workgroup per CU -- a grid of at most p.persist_blocks workgroups that each walk the tiles
// vb, vb + gridDim.x, ... (the grid is a multiple of 8, so a workgroup stays with its XCD's row
// tiles): no new workgroup has to be set up between two tiles of a CU, and a tile's stores drain
// while the next tile's first loads are on their way.
template <typename T, int WF, bool NORM, int EPI, int WR, int WT, int NWR, int NWT, int NWK, int KS, int NBUF,
          bool XS = false, bool DMA = false, bool PIPE = false>
// (twelve waves: three per SIMD, so let the compiler use the registers of three)
__global__ void __launch_bounds__(64 * NWR * NWT * NWK)
    __attribute__((amdgpu_waves_per_eu(1, (NWR * NWT * NWK == 12) ? 3 : 8)))
    prefill_gemm_kernel(const PrefillGemmParams p) {
  if constexpr (PIPE) {
    for (unsigned vb = blockIdx.x; vb < (unsigned)p.total_blocks; vb += gridDim.x) {
      if (vb != blockIdx.x) __syncthreads();  // every wave has left the tile before: its LDS is free
      prefill_gemm_tile<T, WF, NORM, EPI, WR, WT, NWR, NWT, NWK, KS, NBUF, XS, DMA, PIPE>(p, vb);
    }
  } else {
    prefill_gemm_tile<T, WF, NORM, EPI, WR, WT, NWR, NWT, NWK, KS, NBUF, XS, DMA, PIPE>(p, blockIdx.x);
  }
}

static int g_prefill_tile = 0;  // experiments: 0 = built-in choice, 1 = 128 x 128, 2 = 64 x 128, 3 = 32 x 64, 4 = 256 x 256,
                                // 5 = 64 x 128 on eight waves that split K four ways, 6 = 32 x 64 on four waves that split K,
                                // 7 = 128 x 256, 8 = 192 x 256, 9 = 128 x 128 on eight waves that split K four ways,
                                // 10 = 96 x 128 (linear only), 11 = 128 x 64 on sixteen waves that split K four ways,
                                // 12 = 64 x 64 on eight waves that split K four ways (linear only)

static int g_prefill_pipe_small = 1;  // experiments: the pipelined loop on the 128 x 256 and 192 x 256 tiles too
static int g_prefill_dma = 1;   // 0: operand tiles staged through registers everywhere
static int g_prefill_row_group = 4;   // row tiles per panel of an XCD's tile walk (experiments: 1 = one row tile after another)
static int g_prefill_row_split = 0;   // experiments: 8, 4 or 2 forces the XCDs' split of the grid (0: the launcher's choice)
static int g_prefill_bands = 1;       // experiments: 0 keeps gate/up in one launch whatever its last round holds
static int g_prefill_persistent = 1;  // experiments: 0 launches one workgroup per tile on the pipelined tiles too
static int g_prefill_stages3_big = 1;  // experiments: 0 keeps the pipelined 192 x 256 and 256 x 256 tiles on two stages of both tiles
static int g_prefill_stages3 = 1;     // experiments: 0 keeps the pipelined 128 x 256 tile on two LDS stages

// what the LDS-direct loads need: whole k-steps, 16-byte aligned rows, 32-bit byte offsets from
// the operands' bases
static bool lds_direct_loads_serve(const PrefillGemmParams& p, int k_step = 64) {
  return g_prefill_dma && p.k % k_step == 0 && p.pitch % 16 == 0 && (long)p.n * p.pitch < (1L << 32) &&
         (long)p.tokens * p.k * 2 < (1L << 32);
}
static bool pipelined_loop_serves(const PrefillGemmParams& p) { return lds_direct_loads_serve(p); }

template <typename T, int WF, int EPI, int WR, int WT, int NWR, int NWT, int NWK, int KS, int NBUF, bool PIPE = false>
static int launch_prefill_cfg(hipStream_t s, PrefillGemmParams p) {
  constexpr int ROWS = 16 * WR * NWR, TOKS = 16 * WT * NWT;
  p.n_tiles = ceil_div(p.n, EPI == SK_GATEUP ? ROWS / 2 : ROWS);
  p.t_tiles = ceil_div(p.tokens, TOKS);
  // The XCDs' split of the grid: rows alone (8 x 1), or 4 x 2 / 2 x 4 rows x tokens where that cuts
  // the bytes the eight L2s fetch between them -- weights x token splits + x x row splits -- by a
  // fifth or more (down 4096 x 14336 at 4096 tokens: 0.70 instead of 1.06 GB; gate/up keeps 8 x 1).
  p.row_split = 8;
  if (g_prefill_row_split) {
    p.row_split = g_prefill_row_split;
  } else {
    const double wb = (double)(EPI == SK_GATEUP ? 2 : 1) * p.n * p.k * (WF == WF_16BIT ? 2 : 1), xb = (double)p.tokens * p.k * 2;
    double best = wb + 8 * xb;
    for (int rs = 4; rs >= 2; rs /= 2) {
      const double c = wb * (8 / rs) + xb * rs;
      if (c < 0.8 * best && p.t_tiles >= 8 / rs * 4 && p.n_tiles >= rs * 4) { best = c; p.row_split = rs; }
    }
  }
  // every XCD gets the same number of slots: its share rounded up, the surplus exits
  const long grid = (long)ceil_div(p.n_tiles, p.row_split) * ceil_div(p.t_tiles, 8 / p.row_split) * 8;
  if (grid > 0x7fffffffL) return MUI_ERR_UNSUPPORTED;
  constexpr size_t lds = PIPE ? pipe_lds_bytes<ROWS, TOKS, KS, NBUF>() : prefill_lds_bytes<ROWS, TOKS, KS, NBUF>();
  static_assert(lds <= kLdsPerWorkgroup, "LDS of a workgroup");
  auto launch = [&](auto kernel) {
    if constexpr (lds > 65536) {
      // more dynamic LDS than the default limit: raised once per kernel (and device)
      static int raised_for = -1;
      int dev = 0;
      if (hipGetDevice(&dev) != hipSuccess) return MUI_ERR_DEVICE;
      if (raised_for != dev) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
          return MUI_ERR_LAUNCH;
        raised_for = dev;
      }
    }
    long blocks = grid;
    if constexpr (PIPE) {  // a round of workgroups that walk the tiles (a multiple of 8: a workgroup keeps its XCD)
      const long round = device_cus() / 8 * 8;
      if (g_prefill_persistent && round >= 8 && blocks > round) blocks = round;
    }
    hipLaunchKernelGGL(kernel, dim3((int)blocks), dim3(64 * NWR * NWT * NWK), lds, s, p);
    return launch_status();
  };
  p.total_blocks = (int)grid;
  p.row_group = g_prefill_row_group;
  if constexpr (!PIPE) {
    if (p.gamma) return launch(prefill_gemm_kernel<T, WF, true, EPI, WR, WT, NWR, NWT, NWK, KS, NBUF>);
  }
  constexpr int kWaves8 = 8 * NWR * NWT * NWK;
  if constexpr (WF == WF_16BIT && (NBUF == 2 || (PIPE && NBUF == 3)) && NWK == 1 && KS == 64 && ROWS % kWaves8 == 0 &&
                TOKS % kWaves8 == 0 && (PIPE || ROWS * TOKS >= 256 * 256)) {
    // LDS-direct operand loads: always with the software-pipelined loop; with the sixteen-wave loop
    // on the 256 x 256 tile only, where a k-step (2048 matrix-pipe cycles per SIMD) covers an L2
    // round trip (gate/up at 4096 tokens 834 -> 800 us, down 410 -> 390 us, o_proj 136 -> 123 us);
    // with that loop on 128 x 256, half of that, they lose (down at 2048 tokens 264 -> 293 us,
    // o_proj 77 -> 88 us, gate/up at 256 88 -> 99 us).
    if (lds_direct_loads_serve(p))
      return launch(prefill_gemm_kernel<T, WF, false, EPI, WR, WT, NWR, NWT, NWK, KS, NBUF, false, true, PIPE>);
  }
  if constexpr (PIPE) return MUI_ERR_UNSUPPORTED;  // the caller falls back to the sixteen-wave tile
  else return launch(prefill_gemm_kernel<T, WF, false, EPI, WR, WT, NWR, NWT, NWK, KS, NBUF>);
}

// Workspace of the K split over workgroups (mui_linear_ws): arrival counters, then partial tiles
constexpr int kXsMaxTiles = 1024;                              // counters
constexpr int kXsMaxWorkgroups = 512;                          // partial tiles
constexpr size_t kXsSlotBytes = 128 * 128 * sizeof(float);     // one 128 x 128 partial tile
constexpr size_t kXsCounterBytes = kXsMaxTiles * sizeof(unsigned);
size_t prefill_workspace_bytes() { return kXsCounterBytes + kXsMaxWorkgroups * kXsSlotBytes; }

// shares of K per 128 x 128 tile worth taking, or 0: the grid of whole tiles leaves at least three
// quarters of the CUs idle and every share keeps at least twelve k-steps of 128 -- the exchange
// (write-through of the partial tile, the counter, the last workgroup's reads) costs 10-15 us, so
// it pays on long rows only. Measured on MI355X: down 4096 x 14336 at 64 tokens 59 -> 44 us, at 256
// tokens 109 -> 57 us (8 and 4 shares); o_proj 4096 x 4096 at 64 tokens would go 20 -> 31 us.
static int xs_shares(const PrefillGemmParams& p) {
  const long tiles = (long)ceil_div(p.n, 128) * ceil_div(p.tokens, 128);
  const long cus = device_cus();
  if (tiles > kXsMaxTiles) return 0;
  long c = cus / tiles;
  const long steps = ceil_div(p.k, 128);
  if (c > steps / 12) c = steps / 12;
  if (c > 8) c = 8;
  if (tiles * c > kXsMaxWorkgroups) c = kXsMaxWorkgroups / tiles;
  return c >= 4 ? (int)c : 0;
}

template <typename T>
static int launch_prefill_xs(hipStream_t s, PrefillGemmParams p, int shares, void* workspace) {
  constexpr int WR = 4, WT = 4, NWR = 2, NWT = 2, NWK = 4, KS = 128;  // the K-splitting 128 x 128 tile
  constexpr int ROWS = 16 * WR * NWR, TOKS = 16 * WT * NWT;
  static_assert((size_t)ROWS * TOKS * sizeof(float) == kXsSlotBytes, "partial tile size");
  p.n_tiles = ceil_div(p.n, ROWS);
  p.t_tiles = ceil_div(p.tokens, TOKS);
  p.k_splits = shares;
  p.part_count = (unsigned*)workspace;
  p.part = (float*)((char*)workspace + kXsCounterBytes);
  const long grid = (long)p.n_tiles * p.t_tiles * shares;
  constexpr size_t lds = prefill_lds_bytes<ROWS, TOKS, KS, 2>();
  auto kernel = prefill_gemm_kernel<T, WF_16BIT, false, SK_LINEAR, WR, WT, NWR, NWT, NWK, KS, 2, true>;
  static int raised_for = -1;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return MUI_ERR_DEVICE;
  if (raised_for != dev) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return MUI_ERR_LAUNCH;
    raised_for = dev;
  }
  hipLaunchKernelGGL(kernel, dim3((int)grid), dim3(64 * NWR * NWT * NWK), lds, s, p);
  return launch_status();
}

// Gate/up whose 256 x 256 tiles (128 outputs each) end in a round that is at most half full: the
// number of row tiles that make whole rounds of workgroups, for a launch of their own -- or 0
static long gateup_bands(const PrefillGemmParams& p) {
  if (!g_prefill_bands) return 0;
  const long cus = device_cus();
  const long tt = ceil_div(p.tokens, 256), row_tiles = ceil_div(p.n, 128);
  if (cus % tt != 0 || cus / tt < 2) return 0;
  const long per_round = cus / tt, whole_rows = row_tiles / per_round * per_round, rest = row_tiles - whole_rows;
  return (whole_rows > 0 && rest > 0 && 2 * rest <= per_round) ? whole_rows : 0;
}

template <typename T, int WF, int EPI>
static int launch_prefill_t(hipStream_t s, const PrefillGemmParams& p) {
  // Big tiles re-read x and the weights least and keep the LDS traffic per matrix instruction
  // low, but a grid much smaller than the chip leaves the work to too few CUs, and a grid of one
  // and a bit rounds of workgroups costs two rounds. Each shape has a cost per round of
  // workgroups (microseconds at K = 4096 on MI355X; only the ratios matter); the number of
  // rounds the grid needs decides between them. Measured on the Llama-3-8B shapes: QKV at 1536
  // tokens is 144 tiles of 256 x 256 (116 us) but 192 of 192 x 256 (92 us), at 2048 tokens 192
  // (122 us) against 256 (99 us); o_proj and down at 2048 tokens are 128 tiles of 256 x 256 (112 / 363 us)
  // and 256 of 128 x 256 (78 / 270 us); QKV at 512 is 192 tiles of 128 x 128 (68 us), 256 of
  // 96 x 128 (62 us). Below three workgroups of 128 x 128 per four CUs: 64 x 128, then 32 x 64 (up
  // to 256 tokens on the 4096-row matrices).
  const long rows = (EPI == SK_GATEUP) ? 2L * p.n : p.n;
  const long cus = device_cus();
  const long want = 3L * cus / 4;
  auto tiles = [&](int r, int tk) { return (long)ceil_div((int)rows, r) * ceil_div(p.tokens, tk); };
  int which = g_prefill_tile;
  if (which == 0) {
    // few output tiles (short prompts on the 4096-row matrices): one workgroup per tile whose
    // waves split every k-step between them -- four waves that each hold the whole 32 x 64 tile,
    // or eight waves in two token halves of a 64 x 128 or 128 x 128 tile: the LDS traffic per
    // matrix instruction of a larger tile, and enough waves per CU although the grid is a single
    // round of workgroups (their 96-128 KB of LDS leave one per CU). 32 x 64 for up to 64 tokens
    // on 8192 rows (o_proj at 128 tokens 21.7 vs 28.3 us, down 60 vs 91 us).
    if (EPI == SK_LINEAR && tiles(32, 64) <= cus) which = 6;
    // ... and 64 x 64 while that is still a single round: QKV at 128 tokens 33 -> 24.5 us, o_proj at
    // 256 tokens 32 -> 23.5 us (k-steps of 128 instead of 256: 28.6 / 27.2 us)
    else if (EPI == SK_LINEAR && tiles(64, 64) <= cus) which = 12;
    else if (tiles(256, 256) >= 5 * cus / 8 || 2 * tiles(64, 128) > cus) {
      // one workgroup per CU (eight waves): rounds x cost, a little more per round once the
      // rounds follow each other (their weights compete for the L2)
      auto whole = [&](long n_tiles, float one, float many) {
        const long r = (n_tiles + cus - 1) / cus;
        return (float)r * (r > 1 ? many : one);
      };
      // two workgroups per CU (four waves): up to `cus` tiles run one per CU, the next `cus` join them
      auto pairs = [&](long n_tiles, float single, float twin) {
        const long full = n_tiles / (2 * cus), rest = n_tiles % (2 * cus);
        const float last = rest == 0 ? 0.f : rest <= cus ? single : single + (twin - single) * (float)(rest - cus) / (float)cus;
        return (float)full * twin + last;
      };
      // (the three big tiles cost less per round where the software-pipelined loop serves them)
      const bool pipe = WF == WF_16BIT && !p.gamma && pipelined_loop_serves(p);
      float best = whole(tiles(256, 256), pipe ? 96.f : 100.f, pipe ? 100.f : 111.f);
      which = 4;
      // (gate/up in two launches, see below: whole rounds of 256 x 256 and one round of 128 x 256)
      if constexpr (WF == WF_16BIT && EPI == SK_GATEUP) {
        if (pipe && gateup_bands(p) > 0) best = (float)((tiles(256, 256) + cus - 1) / cus - 1) * 100.f + 53.f;
      }
      auto offer = [&](int id, float cost) {
        if (cost < best * 0.97f) { best = cost; which = id; }  // bigger tiles win ties
      };
      if (pipe && EPI == SK_LINEAR) offer(8, whole(tiles(192, 256), 74.f, 80.f));
      else if (pipe) offer(8, whole(tiles(192, 256), 92.f, 98.f));  // gate/up: twelve waves beside pipelined 256 x 256 and 128 x 256
      else offer(8, whole(tiles(192, 256), 85.f, 92.f));
      if (pipe) offer(7, whole(tiles(128, 256), 53.f, 58.f));  // (three LDS stages; 63 / 66 with two)
      else offer(7, whole(tiles(128, 256), WF == WF_16BIT ? 67.f : 73.f, WF == WF_16BIT ? 70.f : 76.f));
      offer(1, pairs(tiles(128, 128), 68.f, 92.f));
      if (EPI == SK_LINEAR && WF == WF_16BIT) offer(10, pairs(tiles(96, 128), 60.f, 76.f));
      // 128 x 128 on waves that split K: the fastest single tile (QKV at 512 tokens 43 vs 62 us,
      // o_proj at 1024 44 vs 68 us, down at 1024 139 vs 219 us), one per CU
      offer(9, whole(tiles(128, 128), 42.f, 40.f));
      // the same with 64-token tiles: half the token bytes per workgroup for prompts of up to 64
      // tokens (gate/up at 64 tokens 57 -> 50 us)
      offer(11, whole(tiles(128, 64), 37.f, 36.5f));
      // 64 x 128 likewise (o_proj at 512 tokens 32 us, down 99 us, QKV at 256 33 us; four waves
      // that each held the whole tile took 40 / 118 / 41 us)
      offer(5, whole(tiles(64, 128), 32.5f, 31.f));
    } else {
      which = (tiles(64, 128) >= want || EPI == SK_GATEUP) ? 2 : 3;
    }
  }
  // Where the software-pipelined eight-wave loop does not apply (fused norm, int8 weights, K not a
  // multiple of 64): sixteen waves per workgroup (four per SIMD, at most 128 registers each) on all
  // but the smallest shapes, with the compiler's own schedule 3-16 % ahead of eight waves with twice
  // the wave tile, although a wave then reads 8
  // instead of 6 KB of operands per 16 matrix instructions -- more waves to fill the gaps between
  // a step's phases (256 x 256: o_proj at 2048 tokens 115 -> 104 us, down 375 -> 323 us, gate/up at
  // 4096 881 -> 854 us; 128 x 256: 75 -> 68 us per round; 128 x 128 splitting K: 46 -> 42 us).
  // int8 rows hold a quarter of the 16-byte chunks per k-step: where sixteen waves would leave
  // threads without a chunk to stage, the int8 kernels keep eight.
  if constexpr (WF == WF_16BIT && EPI == SK_GATEUP) {
    // Gate/up whose 256 x 256 tiles end in a round that is at most half full (2048 tokens: 896 tiles
    // = 3.5 rounds of 256 CUs): the outputs of the whole rounds in one launch, the rest as one round
    // of 128 x 256 tiles in a second one (a half-empty round of the big tile costs as much as a full
    // one, a round of the small tile two thirds of it).
    if (g_prefill_tile == 0 && which == 4 && !p.gamma && pipelined_loop_serves(p)) {
      {
        const long whole_rows = gateup_bands(p);
        if (whole_rows > 0) {
          PrefillGemmParams a = p, b = p;
          a.n = (int)(whole_rows * 128);
          b.n = p.n - a.n;
          b.w0 += (long)a.n * p.pitch;
          b.w1 += (long)a.n * p.pitch;
          b.y += a.n;
          int st = g_prefill_stages3_big ? launch_prefill_cfg<T, WF, EPI, 4, 8, 4, 2, 1, 64, 3, true>(s, a)
                                         : launch_prefill_cfg<T, WF, EPI, 4, 8, 4, 2, 1, 64, 2, true>(s, a);
          if (st == MUI_OK) st = g_prefill_stages3 ? launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 4, 1, 64, 3, true>(s, b)
                                                  : launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 4, 1, 64, 2, true>(s, b);
          if (st != MUI_ERR_UNSUPPORTED) return st;
        }
      }
    }
  }
  if constexpr (WF == WF_16BIT) {
    // 256 x 256 on 4 x 2 waves of 64 x 128 with two operand register sets (the software-pipelined
    // loop): where its loads can go straight into LDS it is 5-8 % ahead of the sixteen waves below
    // (gate/up at 4096 tokens 775 -> 736 us, down 386 -> 356 us, QKV 224 -> 209 us, down at 2048
    // tokens 345 -> 315 us; bit-equal results: the same products in the same order)
    if (which == 4 && !p.gamma) {
      const int st = g_prefill_stages3_big ? launch_prefill_cfg<T, WF, EPI, 4, 8, 4, 2, 1, 64, 3, true>(s, p)
                                           : launch_prefill_cfg<T, WF, EPI, 4, 8, 4, 2, 1, 64, 2, true>(s, p);
      if (st != MUI_ERR_UNSUPPORTED) return st;
    }
  }
  if (which == 13) which = 4;  // the sixteen-wave kernel on request
  if constexpr (WF == WF_16BIT) {
    if (g_prefill_pipe_small && !p.gamma) {
      int st = MUI_ERR_UNSUPPORTED;
      // 128 x 256, 2 x 4 waves of 64 x 64, three LDS stages
      if (which == 7) st = g_prefill_stages3 ? launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 4, 1, 64, 3, true>(s, p)
                                             : launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 4, 1, 64, 2, true>(s, p);
      if constexpr (EPI == SK_LINEAR) {
        // 192 x 256, 4 x 2 waves of 48 x 128
        if (which == 8) st = g_prefill_stages3_big ? launch_prefill_cfg<T, WF, EPI, 3, 8, 4, 2, 1, 64, 3, true>(s, p)
                                                   : launch_prefill_cfg<T, WF, EPI, 3, 8, 4, 2, 1, 64, 2, true>(s, p);
      }
      if (st != MUI_ERR_UNSUPPORTED) return st;
    }
  }
  if (which == 4) return launch_prefill_cfg<T, WF, EPI, 4, 4, 4, 4, 1, 64, 2>(s, p);      // 256 x 256, 4 x 4 waves of 64 x 64
  // 192 x 256 on twelve waves (3 x 4 of 64 x 64, the wave tile of the 256 x 256 kernel; the token
  // chunks of a k-step do not divide by 768 threads: the last round is staged by eight of the
  // waves): QKV at 2048 tokens 119 -> 108 us, at 4096 232 -> 208 us against eight waves of 96 x 64
  if (which == 8) return launch_prefill_cfg<T, WF, EPI, 4, 4, 3, 4, 1, 64, 2>(s, p);
  if constexpr (WF == WF_16BIT) {
    if (which == 7) return launch_prefill_cfg<T, WF, EPI, 2, 4, 4, 4, 1, 64, 2>(s, p);    // 128 x 256, 4 x 4 waves of 32 x 64
    if (which == 5) return launch_prefill_cfg<T, WF, EPI, 2, 4, 2, 2, 4, 128, 2>(s, p);   // 64 x 128, 2 x 2 waves x 4 shares of K
    if constexpr (EPI == SK_LINEAR) {
      if (which == 10) return launch_prefill_cfg<T, WF, EPI, 3, 4, 2, 2, 1, 64, 2>(s, p);  // 96 x 128, 2 x 2 waves of 48 x 64
    }
  }
  if (which == 10) which = 1;  // int8 weights, gate/up
  if (which == 7) return launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 4, 1, 64, 2>(s, p);      // 128 x 256, 2 x 4 waves of 64 x 64
  if (which == 9) return launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 2, 4, 128, 2>(s, p);     // 128 x 128, 2 x 2 waves x 4 shares of K
  if (which == 11) return launch_prefill_cfg<T, WF, EPI, 2, 4, 4, 1, 4, 128, 2>(s, p);    // 128 x 64, 4 x 1 waves x 4 shares of K
  if (which == 5) return launch_prefill_cfg<T, WF, EPI, 4, 4, 1, 2, 4, 128, 2>(s, p);     // 64 x 128, 2 token halves x 4 shares of K
  if constexpr (EPI == SK_LINEAR && WF == WF_16BIT) {
    // 32 x 64 on eight waves (2 row halves x 4 shares of K): QKV at 64 tokens 21.7 -> 20.7 us, o_proj 20.2 -> 19.1 us
    if (which == 6) return launch_prefill_cfg<T, WF, EPI, 1, 4, 2, 1, 4, 256, 2>(s, p);
    if (which == 12) return launch_prefill_cfg<T, WF, EPI, 2, 4, 2, 1, 4, 256, 2>(s, p);  // 64 x 64 likewise
  }
  if constexpr (EPI == SK_LINEAR) {
    if (which == 12) return launch_prefill_cfg<T, WF, EPI, 4, 4, 1, 1, 4, 256, 2>(s, p);  // int8: four waves that each hold the 64 x 64 tile
  }
  if (which == 12) which = 5;
  if (which == 6) return launch_prefill_cfg<T, WF, EPI, 2, 4, 1, 1, 4, 256, 2>(s, p);   // 32 x 64, four waves that each hold the tile split K
  if (which == 1) return launch_prefill_cfg<T, WF, EPI, 4, 4, 2, 2, 1, 64, 2>(s, p);
  if constexpr (EPI == SK_GATEUP) {
    return launch_prefill_cfg<T, WF, EPI, 2, 4, 2, 2, 1, 128, 1>(s, p);
  } else {
    if (which == 2) return launch_prefill_cfg<T, WF, EPI, 2, 4, 2, 2, 1, 128, 1>(s, p);
    return launch_prefill_cfg<T, WF, EPI, 1, 2, 2, 2, 1, 256, 1>(s, p);
  }
}

constexpr int kWideDefaultMaxTokens = 0;  // 0: the built-in rule below
static int g_wide_max_tokens = kWideDefaultMaxTokens;  // longest prompt taken by gemm_wide.hip

// Any number of tokens >= 1 (meant for more than MUI_MAX_TOKENS), 16-bit weights or per-channel
// int8 codes; SkinnyParams as for the decode kernels (x, residual and y dense).
int launch_prefill_gemm(hipStream_t s, int dtype, int wf, int epilogue, const SkinnyParams& q) {
  if (q.tokens < 1 || q.n < 1 || q.k < 1) return MUI_ERR_INVALID_ARG;
  // the shortest prompts are bound by the weight stream: 16 rows per workgroup, K split over the
  // waves, no LDS tiling (gemm_wide.hip). It wins while its grid is a single round of workgroups
  // and the token tiles are few: up to 40 tokens (o_proj at 33 tokens 16.0 vs 20.4 us for the
  // smallest LDS tile, 19.6 vs 20.6 at 48, 23.1 vs 21.2 at 64)
  PrefillGemmParams p = {};
  const long esz = (wf == WF_16BIT) ? 2 : 1;
  p.w0 = (const uint8_t*)q.w0; p.w1 = (const uint8_t*)q.w1; p.pitch = q.pitch * esz;
  p.s0 = q.s0; p.s1 = q.s1; p.s_pitch = q.s_pitch; p.group_shift = q.group_shift;
  p.x = q.x; p.gamma = q.gamma; p.mul_bias = q.mul_bias; p.add_bias = q.add_bias; p.residual = q.residual;
  p.y = q.y; p.y_pitch = q.n; p.n = q.n; p.k = q.k; p.tokens = q.tokens; p.eps = q.eps;
  // a caller-provided workspace lets a long K be shared between workgroups when the tiles are few
  // (in front of the 16-rows-per-workgroup kernel only for K beyond 8192: down at 33 tokens 31 vs 50 us)
  const bool wide_default = q.tokens <= 40 && epilogue == SK_LINEAR && ceil_div(q.n, 16) <= device_cus();
  const bool wide = g_wide_max_tokens == kWideDefaultMaxTokens ? wide_default : q.tokens <= g_wide_max_tokens;
  if (q.workspace && g_prefill_tile == 0 && g_wide_max_tokens == kWideDefaultMaxTokens && wf == WF_16BIT &&
      epilogue == SK_LINEAR && !q.gamma && q.k % 8 == 0 && (q.x_pitch == 0 || q.x_pitch == q.k) &&
      ((uintptr_t)q.workspace & 255u) == 0 && q.workspace_bytes >= prefill_workspace_bytes() &&
      (!wide || q.k > 8192)) {
    const int shares = xs_shares(p);
    if (shares) {
      if (dtype == MUI_DTYPE_F16) return launch_prefill_xs<F16>(s, p, shares, q.workspace);
      if (dtype == MUI_DTYPE_BF16) return launch_prefill_xs<BF16>(s, p, shares, q.workspace);
    }
  }
  if (wide && wf != WF_U8_GROUP) return launch_gemm_wide(s, dtype, wf, epilogue, q);  // (that kernel has no group format)
  if (!(wf == WF_16BIT || wf == WF_I8_CHANNEL || wf == WF_U8_GROUP)) return MUI_ERR_UNSUPPORTED;
  if (wf == WF_U8_GROUP && (q.group_shift < 4 || (q.k & ((1 << q.group_shift) - 1)))) return MUI_ERR_UNSUPPORTED;
  if (q.k % (wf == WF_16BIT ? 8 : 16)) return MUI_ERR_UNSUPPORTED;
  if (q.x_pitch != 0 && q.x_pitch != q.k) return MUI_ERR_UNSUPPORTED;
#define MUI_PF_CASE(TT, WFV, EPIV) \
  if (dtype == TT::kDtype && wf == WFV && epilogue == EPIV) return launch_prefill_t<TT, WFV, EPIV>(s, p);
  MUI_PF_CASE(F16, WF_16BIT, SK_LINEAR)
  MUI_PF_CASE(F16, WF_16BIT, SK_GATEUP)
  MUI_PF_CASE(F16, WF_I8_CHANNEL, SK_LINEAR)
  MUI_PF_CASE(F16, WF_I8_CHANNEL, SK_GATEUP)
  MUI_PF_CASE(F16, WF_U8_GROUP, SK_LINEAR)
  MUI_PF_CASE(F16, WF_U8_GROUP, SK_GATEUP)
  MUI_PF_CASE(BF16, WF_16BIT, SK_LINEAR)
  MUI_PF_CASE(BF16, WF_16BIT, SK_GATEUP)
  MUI_PF_CASE(BF16, WF_I8_CHANNEL, SK_LINEAR)
  MUI_PF_CASE(BF16, WF_I8_CHANNEL, SK_GATEUP)
  MUI_PF_CASE(BF16, WF_U8_GROUP, SK_LINEAR)
  MUI_PF_CASE(BF16, WF_U8_GROUP, SK_GATEUP)
#undef MUI_PF_CASE
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui

extern "C" int mui_tune_prefill(int tile, int wide_max_tokens) {
  MUI_TUNE_GUARD();
  // experiments: 200 + tile keeps the 128 x 256 and 192 x 256 tiles off the software-pipelined loop,
  // 100 + tile keeps every operand tile on the register-staged path
  // 6400 + tile / 12800 + tile / 19200 + tile: the XCDs split the tile grid 8 x 1 / 4 x 2 / 2 x 4 (rows x tokens)
  const int stages3_big = tile >= 51200 ? 0 : 1;  // 51200 + tile: the pipelined 192 x 256 and 256 x 256 tiles on two LDS stages
  if (tile >= 51200) tile -= 51200;
  const int stages3 = tile >= 25600 ? 0 : 1;  // 25600 + tile: the pipelined 128 x 256 tile on two LDS stages
  if (tile >= 25600) tile -= 25600;
  const int row_split = tile >= 19200 ? 2 : tile >= 12800 ? 4 : tile >= 6400 ? 8 : 0;
  if (tile >= 6400) tile -= tile >= 19200 ? 19200 : tile >= 12800 ? 12800 : 6400;
  // 3200 + tile: gate/up stays one launch whatever its last round of tiles holds
  const int bands = tile >= 3200 ? 0 : 1;
  if (tile >= 3200) tile -= 3200;
  // 800 + tile: an XCD walks one row tile after another; 1600 + tile / 2400 + tile: panels of 8 / 2 row tiles
  const int row_group = tile >= 2400 ? 2 : tile >= 1600 ? 8 : tile >= 800 ? 1 : 4;
  if (tile >= 800) tile -= tile >= 2400 ? 2400 : tile >= 1600 ? 1600 : 800;
  const int persistent = tile >= 400 ? 0 : 1;  // 400 + tile: one workgroup per tile on the pipelined tiles too
  if (tile >= 400) tile -= 400;
  const int pipe_small = tile >= 200 ? 0 : 1;
  if (tile >= 200) tile -= 200;
  const int dma = tile >= 100 ? 0 : 1;
  if (tile >= 100) tile -= 100;
  if (tile < 0 || tile > 13 || wide_max_tokens > 128) return MUI_ERR_INVALID_ARG;
  mui::g_prefill_stages3_big = stages3_big;
  mui::g_prefill_stages3 = stages3;
  mui::g_prefill_row_split = row_split;
  mui::g_prefill_bands = bands;
  mui::g_prefill_row_group = row_group;
  mui::g_prefill_persistent = persistent;
  mui::g_prefill_pipe_small = pipe_small;
  mui::g_prefill_dma = dma;
  mui::g_prefill_tile = tile;
  mui::g_wide_max_tokens = wide_max_tokens;  // 0: built-in rule; negative: never; n: prompts up to n tokens
  return MUI_OK;
}
