// Decode-time attention for gfx950: flash decoding over a static KV cache with the RoPE of
// the new token and its cache write-out fused in.
//
// Reference counterparts: RoPE + static-cache write (csrc/rope/rotary_fp16_kernels.cu:575-765),
// cache update (csrc/kvcaches/static_kvcache_xx16_kernels.cu:26-123), flash decoding partial
// pass and final reduce (csrc/attention/flash_decoding_fp16_kernels.cu:199-586, 642-785).
//
// Layout of the work (T = 1 new token per batch row, head_dim 128):
//   grid = (splits of the cached sequence, blocks of G query heads, batch).
//   Normally G = Hq/Hkv: a workgroup serves ALL query heads that share its KV head, so K and V
//   are read from HBM exactly once (the reference re-reads them once per query head); that
//   shape runs on the matrix cores (attn_decode_mfma_kernel below). What follows describes the
//   vector-ALU kernel, which serves the other shape:
//   Short sequences at small batch are latency-bound instead: there the launcher uses G = 1
//   and no sequence split (one workgroup per query head, the few hundred KB of K/V re-read
//   from cache by the heads of a group), which needs no second kernel to merge splits.
//   Inside a wave, the 16 lanes of a DPP row own the 16 x 16-byte chunks of ONE token's K/V
//   row; the 4 rows of a wave take 4 consecutive tokens, so one load instruction covers 1 KiB
//   of contiguous cache. q.k is a packed-fp16 dot (v_dot2_f32_f16) reduced over the 16 lanes
//   with DPP; softmax runs online in fp32 with one rescale per block of U tokens; p.v is
//   accumulated in fp32. Each DPP row therefore is an independent online-softmax worker over
//   its tokens; the 16 workers of a workgroup are merged through LDS (log-sum-exp combine),
//   and workgroups are merged by a small second kernel (fp32 partials, unlike the
//   reference's fp16 max/denominator).
//   The new token: every workgroup rotates the G query heads it needs on the fly (fp32 math,
//   rounded once to the 16-bit type); the workgroup whose split contains the new slot rotates
//   k, writes k/v into the cache and folds them in from LDS, so no workgroup ever reads the
//   slot that is being written.
//   The sequence length can come from device memory (cache_position[0] + 1), which keeps
//   the launch shape fixed under HIP-graph replay.
#include <mutex>
#include <type_traits>

#include "common.cuh"

namespace mui {

constexpr int kHeadDim = 128;
// A workgroup is NW wave64s (4 or 16). Each wave holds 4 DPP rows = 4 token workers, so a
// pass of the workgroup covers NW * 4 * U tokens. 16 waves (4 per SIMD) hide the dependent
// latency of the per-token math far better than 4; they need <= 128 VGPRs per lane, which
// rules them out for 8 query heads per KV head.
constexpr float kLog2e = 1.4426950408889634f;

struct AttnParams {
  const uint16_t* q;      // [B, Hq, D] (strides below), un-rotated when cos != null
  long q_bs, q_hs;
  const uint16_t* k_new;  // [B, Hkv, D] or null (no new token: attend over the cache as is)
  long k_bs, k_hs;
  const uint16_t* v_new;
  long v_bs, v_hs;
  const float* cos;       // [max_pos, rope_stride] fp32 tables, or null (no rotation)
  const float* sin;
  int rope_stride;
  int rope_rows;          // height of the tables: positions are clamped into [0, rope_rows)
  const int64_t* position_ids;  // rotary position of the new token per batch row, or null
  long pos_bs;
  const int64_t* cache_position;  // device scalar: cache slot of the new token
  int seq_len;            // valid cache length incl. the new token; < 0: cache_position[0] + 1
  uint16_t* k_cache;      // [B, Hkv, max_t, D]
  uint16_t* v_cache;
  long c_bs, c_hs, c_ts;
  const uint16_t* mask;   // [B, >= seq_len]: 0 keeps a key, anything else drops it; or null
  long mask_bs;
  uint16_t* q_out;        // optional dense [B, Hq, D] rotated queries
  float* part_acc;        // [B, Hq, n_splits, D]
  float* part_ml;         // [B, Hq, n_splits, 2]
  uint16_t* out;          // [B, Hq * D]
  int hq, hkv, n_splits, max_t;
  float scale_log2;       // log2(e) / sqrt(D)
  // optional: bytes the next kernel will stream (its weights), pulled on chip by extra workgroups
  // of the unsplit head-parallel launch, which leaves most CUs idle (see warm_cache)
  const char* warm;
  long warm_bytes;
  int warm_slab, warm_wgs, warm_delay;
};

template <typename T>
__device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float c);
template <>
__device__ __forceinline__ float dot2_acc<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}
typedef __bf16 bf16x2_at __attribute__((ext_vector_type(2)));
template <>
__device__ __forceinline__ float dot2_acc<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_at, a), __builtin_bit_cast(bf16x2_at, b), c, false);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Maximum / sum over the four 16-lane rows of a wave (lanes i, i + 16, i + 32, i + 48), the same
// value in all four: gfx950's row-swap instructions exchange rows between two registers in the
// vector ALU, without the LDS round trip of ds_bpermute that a shuffle by 16 or 32 lanes costs.
// (permlane16_swap: rows 1, 3 of the first operand <-> rows 0, 2 of the second; permlane32_swap:
// upper half of the first <-> lower half of the second.) The additions pair the rows as the two
// shuffles did -- (r0 + r1) + (r2 + r3) --, so the results are bit-identical.
__device__ __forceinline__ float rows_max(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
// The two registers of one swap: OFF = 16 -> a = rows (0, 0, 2, 2), b = rows (1, 1, 3, 3) of v;
// OFF = 32 -> a = rows (0, 1, 0, 1), b = rows (2, 3, 2, 3). Every row sees its own value in one of
// them and its partner's (lane ^ OFF) in the other, in the same order in all rows.
template <int OFF>
__device__ __forceinline__ void rows_pair(float v, float& a, float& b) {
  const unsigned u = __float_as_uint(v);
  if constexpr (OFF == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
  } else {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
  }
}

// rotate-half RoPE of element d of a 128-wide head held at `src` (16-bit), fp32 math:
//   r = x * cos[d mod 64] + (d < 64 ? -x[d+64] : x[d-64]) * sin[d mod 64]
template <typename T>
__device__ __forceinline__ float rope_elem(const uint16_t* src, int d, const float* cos_row,
                                           const float* sin_row) {
  const float x = T::one(src[d]);
  if (cos_row == nullptr) return x;
  constexpr int half = kHeadDim / 2;
  const float partner = d < half ? -T::one(src[d + half]) : T::one(src[d - half]);
  const int f = d & (half - 1);
  return fmaf(partner, sin_row[f], x * cos_row[f]);
}

// One block of UU tokens per DPP row: scores, online-softmax update, p.v accumulation.
template <typename T, int G, int UU>
__device__ __forceinline__ void attend_block(const u32x4 (&kreg)[UU], const u32x4 (&vreg)[UU],
                                             const bool (&valid)[UU], const float (&mask_add)[UU],
                                             const uint32_t (&qreg)[G][4], float scale_log2,
                                             float (&m)[G], float (&l)[G], float (&acc)[G][8]) {
  float s2[UU][G];
#pragma unroll
  for (int u = 0; u < UU; ++u) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float s = dot2_acc<T>(kreg[u].x, qreg[g][0], 0.f);
      s = dot2_acc<T>(kreg[u].y, qreg[g][1], s);
      s = dot2_acc<T>(kreg[u].z, qreg[g][2], s);
      s = dot2_acc<T>(kreg[u].w, qreg[g][3], s);
      s = row16_sum(s);
      s2[u][g] = valid[u] ? fmaf(s, scale_log2, mask_add[u]) : -INFINITY;
    }
  }
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float m_new = m[g];
#pragma unroll
    for (int u = 0; u < UU; ++u) m_new = fmaxf(m_new, s2[u][g]);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = fast_exp2(m[g] - m_use);
    float p[UU];
    float psum = 0.f;
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      p[u] = fast_exp2(s2[u][g] - m_use);
      psum += p[u];
    }
    l[g] = fmaf(l[g], corr, psum);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] *= corr;
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      float vf[8];
      unpack8<T>(vreg[u], vf);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(p[u], vf[i], acc[g][i]);
    }
    m[g] = m_new;
  }
}

// The arguments in front are copies of the struct's fields: leading scalar arguments arrive in
// SGPRs at wave launch (14 dwords), a struct only through scalar loads, and the kernel's first act
// is a dependent load through one of them (the cache slot), which then starts together with the
// loads of the struct instead of after them.
template <typename T, int G, int U, int NW, bool DIRECT>
__global__ void __launch_bounds__(NW * kWave) attn_decode_kernel(
    const int64_t* cache_position, const int64_t* position_ids, long pos_bs, const uint16_t* q, uint16_t* k_cache,
    uint16_t* v_cache, const float* cos_table, const AttnParams pr) {
  AttnParams p = pr;
  p.cache_position = cache_position; p.position_ids = position_ids; p.pos_bs = pos_bs; p.q = q; p.k_cache = k_cache;
  p.v_cache = v_cache; p.cos = cos_table;
  // the two device scalars everything else waits for, requested before anything waits for the
  // struct (their addresses are in SGPRs already)
  const long slot_dev = cache_position ? (long)cache_position[0] : -1;
  const long pos_dev = position_ids ? (long)position_ids[(long)blockIdx.z * pos_bs] : -1;
  __builtin_amdgcn_sched_barrier(0);
  constexpr int kAttnThreads = NW * kWave;
  constexpr int kWorkers = NW * 4;      // DPP rows per workgroup
  constexpr bool kPipe = (NW <= 8);     // <= 2 waves per SIMD: double-buffer K/V in registers
  __shared__ __attribute__((aligned(16))) uint16_t q_lds[G][kHeadDim];
  __shared__ __attribute__((aligned(16))) uint16_t kn_lds[kHeadDim];
  __shared__ __attribute__((aligned(16))) uint16_t vn_lds[kHeadDim];
  __shared__ float lds_m[NW][G];
  __shared__ float lds_l[NW][G];
  __shared__ __attribute__((aligned(16))) float tile[NW][G][kHeadDim];

  if constexpr (DIRECT && G == 1) {
    // workgroups past the query heads: cache warmers for the next kernel (batch row 0 only)
    if ((int)blockIdx.y >= p.hq) {
      if (blockIdx.z == 0)
        warm_cache(p.warm, p.warm_bytes, p.warm_slab, (int)blockIdx.y - p.hq, p.warm_wgs, threadIdx.x, kAttnThreads,
                   p.warm_delay);
      return;
    }
  }
  const int split = blockIdx.x, b = blockIdx.z;
  const int head0 = blockIdx.y * G;          // first query head of this workgroup
  const int group = p.hq / p.hkv;            // query heads per KV head (a multiple of G)
  const int kvh = head0 / group;
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int ts = lane >> 4;  // DPP row = token sub-index
  const int dc = lane & 15;  // 16-byte chunk of the head
  const int wk = wave * 4 + ts;

  const bool has_new = p.k_new != nullptr;
  const int slot = has_new ? (int)slot_dev : -1;
  int S = p.seq_len >= 0 ? p.seq_len : slot + 1;
  S = S < p.max_t ? S : p.max_t;
  long pos = p.position_ids ? pos_dev : (long)(slot >= 0 ? slot : S - 1);
  pos = pos < 0 ? 0 : (pos >= p.rope_rows ? p.rope_rows - 1 : pos);  // never index past the tables

  constexpr int kBlock = kWorkers * U;  // tokens per workgroup iteration
  int chunk = (S + p.n_splits - 1) / p.n_splits;
  chunk = ((chunk + kBlock - 1) / kBlock) * kBlock;
  const int t_begin = split * chunk;
  const int t_end = (t_begin + chunk) < S ? (t_begin + chunk) : S;
  const bool owner = has_new && slot >= t_begin && slot < t_begin + chunk && slot < S;
  const bool writer = owner && (head0 % group == 0);  // one workgroup per KV head stores the slot

  const float* cos_row = p.cos ? p.cos + pos * p.rope_stride : nullptr;
  const float* sin_row = p.sin ? p.sin + pos * p.rope_stride : nullptr;

  // ---- K/V streaming state; the first block is requested before anything else so that the
  //      query rotation below overlaps with its latency (the new slot is never read) ----
  const uint16_t* kc = p.k_cache + (long)b * p.c_bs + (long)kvh * p.c_hs + dc * 8;
  const uint16_t* vc = p.v_cache + (long)b * p.c_bs + (long)kvh * p.c_hs + dc * 8;
  const uint16_t* mrow = p.mask ? p.mask + (long)b * p.mask_bs : nullptr;
  // No K/V load sits behind a branch: the compiler's load-counter waits are exact only in
  // straight-line code (behind a branch it waits for everything outstanding, the block just
  // requested included, which would serialise the two register sets). Tokens past the end,
  // the new slot and whole blocks past the last one read row 0 of the head instead (always
  // there) and are marked invalid. MASKED adds the per-token mask read of padded batches.
  auto load_block = [&](int base, bool live, u32x4 (&kreg)[U], u32x4 (&vreg)[U], bool (&valid)[U],
                        auto masked) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int tok = base + u * kWorkers + wk;
      valid[u] = live && (tok < t_end) && (tok != slot);
      const int tk = valid[u] ? tok : 0;
      // split (long) sequences stream K/V once: non-temporal; the unsplit short case re-reads
      // rows that the previous steps left in cache
      kreg[u] = ld16_sel<!DIRECT>(kc + (long)tk * p.c_ts);
      vreg[u] = ld16_sel<!DIRECT>(vc + (long)tk * p.c_ts);
      if constexpr (decltype(masked)::value) {
        if (T::one(ld2(mrow + tk)) != 0.f) valid[u] = false;
      }
    }
  };
  u32x4 ka[U], va[U], kb[U], vb[U];
  bool valid_a[U], valid_b[U];
  // The workgroups of a launch start at addresses that are large powers of two apart and
  // advance at the same speed, so they would all hit the same memory channels at the same
  // time; softmax does not care about order, so each workgroup starts at its own block and
  // wraps around.
  const int n_blocks = t_end > t_begin ? (t_end - t_begin + kBlock - 1) / kBlock : 0;
  const int rot = n_blocks > 0 ? (int)((blockIdx.x * 7u + blockIdx.y * 13u + blockIdx.z * 29u) % (unsigned)n_blocks) : 0;
  auto block_base = [&](int bi) {  // any bi < 2 * n_blocks (blocks past the last one are not live)
    int blk = bi + rot;
    blk = blk >= n_blocks ? blk - n_blocks : blk;
    return t_begin + blk * kBlock;
  };
  auto fetch = [&](int bi, u32x4 (&kreg)[U], u32x4 (&vreg)[U], bool (&valid)[U], auto masked) {
    const bool live = bi < n_blocks;
    load_block(block_base(live ? bi : 0), live, kreg, vreg, valid, masked);
  };
  const bool use_mask = mrow != nullptr;
  if (use_mask) fetch(0, ka, va, valid_a, std::true_type{});
  else fetch(0, ka, va, valid_a, std::false_type{});

  // ---- rotate the G query heads of this KV head into LDS (16-bit, rounded once); the owner of
  //      the new slot also rotates k, writes k/v to the cache and keeps them in LDS. One index
  //      space over the threads (q elements, then k, then v): with 128 + 128 + 128 elements on
  //      512 threads every element has its own thread and the three groups' loads are in flight
  //      together, instead of the first two waves doing q and then k, one round trip after the other ----
  {
    constexpr int NQ = G * kHeadDim;
    const int total = NQ + (owner ? 2 * kHeadDim : 0);
    const long coff = (long)b * p.c_bs + (long)kvh * p.c_hs + (long)(slot >= 0 ? slot : 0) * p.c_ts;
    for (int e = t; e < total; e += kAttnThreads) {
      if (e < NQ) {
        const int g = e / kHeadDim, d = e % kHeadDim;
        const int head = head0 + g;
        const uint16_t* qp = p.q + (long)b * p.q_bs + (long)head * p.q_hs;
        const uint16_t r = T::pack(rope_elem<T>(qp, d, cos_row, sin_row));
        q_lds[g][d] = r;
        if (p.q_out && split == 0) p.q_out[((long)b * p.hq + head) * kHeadDim + d] = r;
      } else if (e < NQ + kHeadDim) {
        const int d = e - NQ;
        const uint16_t* kp = p.k_new + (long)b * p.k_bs + (long)kvh * p.k_hs;
        const uint16_t r = T::pack(rope_elem<T>(kp, d, cos_row, sin_row));
        kn_lds[d] = r;
        if (writer) p.k_cache[coff + d] = r;
      } else {
        const int d = e - NQ - kHeadDim;
        const uint16_t v = p.v_new[(long)b * p.v_bs + (long)kvh * p.v_hs + d];
        vn_lds[d] = v;
        if (writer) p.v_cache[coff + d] = v;
      }
    }
  }
  __syncthreads();

  uint32_t qreg[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const u32x4 qv = *(const u32x4*)&q_lds[g][dc * 8];
    qreg[g][0] = qv.x; qreg[g][1] = qv.y; qreg[g][2] = qv.z; qreg[g][3] = qv.w;
  }

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
  }

  {
    float madd[U];
#pragma unroll
    for (int u = 0; u < U; ++u) madd[u] = 0.f;
    auto sweep = [&](auto masked) {
      if constexpr (kPipe) {
        // two register sets: the next block is in flight while the current one is consumed;
        // the branch-free rounds run while both of their fetches are real, the last one or
        // two blocks are peeled (short sequences consist of that tail only)
        int bi = 0;
        for (; bi + 2 < n_blocks; bi += 2) {
          fetch(bi + 1, kb, vb, valid_b, masked);
          attend_block<T, G, U>(ka, va, valid_a, madd, qreg, p.scale_log2, m, l, acc);
          fetch(bi + 2, ka, va, valid_a, masked);
          attend_block<T, G, U>(kb, vb, valid_b, madd, qreg, p.scale_log2, m, l, acc);
        }
        if (bi + 1 < n_blocks) {
          fetch(bi + 1, kb, vb, valid_b, masked);
          attend_block<T, G, U>(ka, va, valid_a, madd, qreg, p.scale_log2, m, l, acc);
          attend_block<T, G, U>(kb, vb, valid_b, madd, qreg, p.scale_log2, m, l, acc);
        } else if (bi < n_blocks) {
          attend_block<T, G, U>(ka, va, valid_a, madd, qreg, p.scale_log2, m, l, acc);
        }
      } else {
        // 4 waves per SIMD overlap each other's loads; one register set keeps the kernel
        // under 128 VGPRs
        for (int bi = 0; bi < n_blocks; ++bi) {
          attend_block<T, G, U>(ka, va, valid_a, madd, qreg, p.scale_log2, m, l, acc);
          if (bi + 1 < n_blocks) fetch(bi + 1, ka, va, valid_a, masked);
        }
      }
    };
    if (use_mask) sweep(std::true_type{}); else sweep(std::false_type{});
  }

  if (owner && wave == 0) {  // the new token, straight from LDS, on DPP row 0 of wave 0
    u32x4 kreg[1], vreg[1];
    bool valid[1];
    float madd[1] = {0.f};
    kreg[0] = *(const u32x4*)&kn_lds[dc * 8];
    vreg[0] = *(const u32x4*)&vn_lds[dc * 8];
    valid[0] = (ts == 0);
    if (mrow != nullptr && T::one(mrow[slot]) != 0.f) valid[0] = false;
    attend_block<T, G, 1>(kreg, vreg, valid, madd, qreg, p.scale_log2, m, l, acc);
  }

  // ---- stage 1: merge the 4 workers (DPP rows) of each wave with row swaps in the vector ALU
  //      (no LDS round trips); every row ends up with the wave's combined (m, l, acc) ----
  auto merge_rows = [&](auto off_tag) {
    constexpr int OFF = decltype(off_tag)::value;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float ma, mb, la, lb;
      rows_pair<OFF>(m[g], ma, mb);
      rows_pair<OFF>(l[g], la, lb);
      const float mn = fmaxf(ma, mb);
      const float mu = (mn == -INFINITY) ? 0.f : mn;
      const float fa = fast_exp2(ma - mu), fb = fast_exp2(mb - mu);
      l[g] = la * fa + lb * fb;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float xa, xb;
        rows_pair<OFF>(acc[g][i], xa, xb);
        acc[g][i] = xa * fa + xb * fb;
      }
      m[g] = mn;
    }
  };
  merge_rows(std::integral_constant<int, 16>{});
  merge_rows(std::integral_constant<int, 32>{});
  // ---- stage 2: merge the NW waves through LDS: every wave leaves its (m, l, acc) as they are,
  //      one barrier, and the output threads scale by 2^(m_wave - max) as they add (the products
  //      and their order are the ones of scaling before the store, without that store's barrier) ----
  if (ts == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (dc == 0) {
        lds_m[wave][g] = m[g];
        lds_l[wave][g] = l[g];
      }
      f32x4 a0 = {acc[g][0], acc[g][1], acc[g][2], acc[g][3]};
      f32x4 a1 = {acc[g][4], acc[g][5], acc[g][6], acc[g][7]};
      *(f32x4*)&tile[wave][g][dc * 8] = a0;
      *(f32x4*)&tile[wave][g][dc * 8 + 4] = a1;
    }
  }
  __syncthreads();

  for (int e = t; e < G * kHeadDim; e += kAttnThreads) {
    const int g = e / kHeadDim, d = e % kHeadDim;
    const int head = head0 + g;
    float mx = lds_m[0][g];
#pragma unroll
    for (int w2 = 1; w2 < NW; ++w2) mx = fmaxf(mx, lds_m[w2][g]);
    const float m_use = (mx == -INFINITY) ? 0.f : mx;
    float a = 0.f, lsum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) {
      const float f = fast_exp2(lds_m[w2][g] - m_use);
      a += tile[w2][g][d] * f;
      lsum += lds_l[w2][g] * f;
    }
    if constexpr (DIRECT) {
      p.out[((long)b * p.hq + head) * kHeadDim + d] = T::pack(lsum > 0.f ? a / lsum : 0.f);
    } else {
      const long pi = ((long)b * p.hq + head) * p.n_splits + split;
      p.part_acc[pi * kHeadDim + d] = a;
      if (d == 0) {
        p.part_ml[pi * 2 + 0] = mx;
        p.part_ml[pi * 2 + 1] = lsum;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Matrix-core formulation: the kernel the launcher uses whenever a workgroup serves a whole KV
// group (G = Hq/Hkv; the vector kernel above keeps the unsplit G = 1 mode of short sequences).
// Same grid and merge as above, but a wave now owns blocks of 32 consecutive tokens. K and V
// are both loaded in their natural layout (lane = 16-byte chunk of a token row, four whole
// rows per instruction), parked in wave-private LDS tiles and read from there: loading K
// straight in MFMA operand layout touches 16 rows x 64 bytes per instruction and streams
// markedly slower. One register set; the tiles hold the block being multiplied while the
// registers receive the next one.
//   scores   S^T[token, head] = K[token, :] . q[head, :]   two v_mfma_f32_16x16x32 chains over
//            D = 128 (A = K rows from the LDS tile in operand layout: lane
//            (g = lane / 16, i = lane % 16) reads 16-byte chunk g + 4j of token i; B = rotated
//            q of head i from LDS, zero for i >= G). C puts head i's scores of tokens 4g + r
//            (r < 4) in lane (g, i): softmax needs one running max per lane column, shared by
//            the four lane groups with two shuffles.
//   output   O^T[d, head] += V^T[d, token] . P[token, head]   8 MFMAs (16 values of d each),
//            contraction over the block's 32 tokens. P comes straight from the score
//            registers (k-slots of lane group g = tokens 4g + r and 16 + 4g + r). V is read
//            back from its tile TRANSPOSED with ds_read_b64_tr_b16: within a 16-lane group, lane i receives
//            element i % 4 of the 8-byte rows addressed by lanes i/4, i/4 + 4, i/4 + 8,
//            i/4 + 12, i.e. four tokens of one d when those lanes point at token rows
//            4g .. 4g + 3 at column 16 * block + 4 * (lane % 4).
// About 100 instructions per 16 KiB of K/V per wave instead of about 600 on the vector ALUs.
// ---------------------------------------------------------------------------------------
typedef _Float16 af16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 abf16x8 __attribute__((ext_vector_type(8)));
typedef short ai16x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ f32x4 attn_mfma(u32x4 a, u32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 attn_mfma<F16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(af16x8, a), __builtin_bit_cast(af16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 attn_mfma<BF16>(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(abf16x8, a), __builtin_bit_cast(abf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* lds_ptr) {
  typedef ai16x4 __attribute__((address_space(3))) * lds_v4;
  const ai16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4)lds_ptr);
  return __builtin_bit_cast(u32x2, r);
}

constexpr int kMfTok = 32;        // tokens per wave block
constexpr int kMfKStride = 136;   // 16-bit elements per K tile row (256 + 16 bytes)
constexpr int kMfVStride = 144;   // 16-bit elements per V tile row: 288 bytes keep the transposed reads spread over the banks

template <typename T, int G, int NW, bool DIRECT>
__global__ void __launch_bounds__(NW * kWave) attn_decode_mfma_kernel(
    // leading copies of the struct's fields, as in attn_decode_kernel
    const int64_t* cache_position, const int64_t* position_ids, long pos_bs, const uint16_t* q, uint16_t* k_cache,
    uint16_t* v_cache, const float* cos_table, const AttnParams pr) {
  AttnParams p = pr;
  p.cache_position = cache_position; p.position_ids = position_ids; p.pos_bs = pos_bs; p.q = q; p.k_cache = k_cache;
  p.v_cache = v_cache; p.cos = cos_table;
  const long slot_dev = cache_position ? (long)cache_position[0] : -1;
  const long pos_dev = position_ids ? (long)position_ids[(long)blockIdx.z * pos_bs] : -1;
  __builtin_amdgcn_sched_barrier(0);
  constexpr int kAttnThreads = NW * kWave;
  constexpr int kBlock = NW * kMfTok;  // tokens per workgroup pass
  __shared__ __attribute__((aligned(16))) uint16_t q_lds[16][kHeadDim];
  __shared__ __attribute__((aligned(16))) uint16_t kn_lds[kHeadDim];
  __shared__ __attribute__((aligned(16))) uint16_t vn_lds[kHeadDim];
  __shared__ float lds_m[NW][G];
  __shared__ float lds_l[NW][G];
  // the V tiles during the sweep, the cross-wave merge buffer afterwards
  constexpr int kVBytes = NW * kMfTok * kMfVStride * 2;
  constexpr int kMergeBytes = NW * G * kHeadDim * 4;
  __shared__ __attribute__((aligned(16))) char big_lds[kVBytes > kMergeBytes ? kVBytes : kMergeBytes];
  uint16_t (*v_lds)[kMfVStride] = (uint16_t (*)[kMfVStride])(big_lds + (size_t)(threadIdx.x >> 6) * kMfTok * kMfVStride * 2);
  // K tile of the wave's block: rows of 256 + 16 bytes (the 16 lanes of an operand read phase
  // hit 64 distinct banks)
  __shared__ __attribute__((aligned(16))) uint16_t k_tiles[NW][kMfTok][kMfKStride];
  uint16_t (*k_lds)[kMfKStride] = k_tiles[threadIdx.x >> 6];
  float (*tile)[G][kHeadDim] = (float (*)[G][kHeadDim])big_lds;

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int head0 = kvh * G;
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int g = lane >> 4;
  const int i = lane & 15;

  const bool has_new = p.k_new != nullptr;
  const int slot = has_new ? (int)slot_dev : -1;
  int S = p.seq_len >= 0 ? p.seq_len : slot + 1;
  S = S < p.max_t ? S : p.max_t;
  long pos = p.position_ids ? pos_dev : (long)(slot >= 0 ? slot : S - 1);
  pos = pos < 0 ? 0 : (pos >= p.rope_rows ? p.rope_rows - 1 : pos);  // never index past the tables

  int chunk = (S + p.n_splits - 1) / p.n_splits;
  chunk = ((chunk + kBlock - 1) / kBlock) * kBlock;
  const int t_begin = split * chunk;
  const int t_end = (t_begin + chunk) < S ? (t_begin + chunk) : S;
  const bool owner = has_new && slot >= t_begin && slot < t_begin + chunk && slot < S;

  const float* cos_row = p.cos ? p.cos + pos * p.rope_stride : nullptr;
  const float* sin_row = p.sin ? p.sin + pos * p.rope_stride : nullptr;

  const uint16_t* kc = p.k_cache + (long)b * p.c_bs + (long)kvh * p.c_hs;
  const uint16_t* vc = p.v_cache + (long)b * p.c_bs + (long)kvh * p.c_hs;
  const uint16_t* mrow = p.mask ? p.mask + (long)b * p.mask_bs : nullptr;
  const int safe_row = t_begin < S ? t_begin : 0;  // a readable row for out-of-range lanes

  // K and V are both loaded in the natural layout (a load instruction covers four whole token
  // rows = 1 KB of a dense cache; loading K straight in operand layout would touch 16 rows x 64
  // bytes per instruction, which streams markedly slower) and reach the MFMAs through LDS.
  struct Block {
    u32x4 k[8];  // token base + 4 * u + g, chunk i
    u32x4 v[8];
  };
  auto load_block = [&](int base, Block& q) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int tok = base + 4 * u + g;
      const long off = (long)(tok < t_end ? tok : safe_row) * p.c_ts + i * 8;
      q.k[u] = ld16_sel<!DIRECT>(kc + off);
      q.v[u] = ld16_sel<!DIRECT>(vc + off);
    }
  };

  // (K/V loads are never behind a branch, see attn_decode_kernel: blocks past the end read the
  // safe row and are masked out by their token indices)
  // One register set: the LDS tiles hold the block being multiplied while the registers
  // already receive the next one.
  Block blk;
  const int base0 = t_begin + wave * kMfTok;
  const int n_blk = base0 < t_end ? (t_end - base0 + kBlock - 1) / kBlock : 0;  // blocks of this wave
  load_block(base0, blk);

  // ---- rotate the G query heads into LDS (rows >= G stay zero: the padded MFMA columns) ----
  for (int e = t; e < 16 * kHeadDim; e += kAttnThreads) {
    const int hh = e / kHeadDim, d = e % kHeadDim;
    uint16_t r = 0;
    if (hh < G) {
      const int head = head0 + hh;
      const uint16_t* qp = p.q + (long)b * p.q_bs + (long)head * p.q_hs;
      r = T::pack(rope_elem<T>(qp, d, cos_row, sin_row));
      if (p.q_out && split == 0) p.q_out[((long)b * p.hq + head) * kHeadDim + d] = r;
    }
    q_lds[hh][d] = r;
  }
  if (owner) {
    const long coff = (long)b * p.c_bs + (long)kvh * p.c_hs + (long)slot * p.c_ts;
    if (t < kHeadDim) {
      const uint16_t* kp = p.k_new + (long)b * p.k_bs + (long)kvh * p.k_hs;
      const uint16_t r = T::pack(rope_elem<T>(kp, t, cos_row, sin_row));
      kn_lds[t] = r;
      p.k_cache[coff + t] = r;
    } else if (t < 2 * kHeadDim) {
      const int d = t - kHeadDim;
      const uint16_t v = p.v_new[(long)b * p.v_bs + (long)kvh * p.v_hs + d];
      vn_lds[d] = v;
      p.v_cache[coff + d] = v;
    }
  }
  __syncthreads();

  u32x4 qreg[4];  // B operand of the score MFMAs: head i, chunk g + 4j
#pragma unroll
  for (int j = 0; j < 4; ++j) qreg[j] = *(const u32x4*)&q_lds[i][(g + 4 * j) * 8];

  float m = -INFINITY, l = 0.f;  // of head i (replicated over the lane groups; l is a partial sum)
  f32x4 acc[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto park = [&](int base, const Block& q) {
    // K and V (natural layout) into this wave's tiles
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      *(u32x4*)&k_lds[4 * u + g][i * 8] = q.k[u];
      *(u32x4*)&v_lds[4 * u + g][i * 8] = q.v[u];
    }
    // the new token's row comes from LDS, never from the cache slot written above: it
    // overwrites its row of the tiles (LDS operations of a wave execute in order)
    if (owner && slot >= base && slot < base + kMfTok && g == 0) {
      *(u32x4*)&k_lds[slot - base][i * 8] = *(const u32x4*)&kn_lds[i * 8];
      *(u32x4*)&v_lds[slot - base][i * 8] = *(const u32x4*)&vn_lds[i * 8];
    }
    __builtin_amdgcn_wave_barrier();
  };
  auto attend = [&](int base, auto masked) {
    f32x4 s1 = {0.f, 0.f, 0.f, 0.f}, s2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // A operands: token 16 * half + i, chunk g + 4 * step
      s1 = attn_mfma<T>(*(const u32x4*)&k_lds[i][(g + 4 * j) * 8], qreg[j], s1);
      s2 = attn_mfma<T>(*(const u32x4*)&k_lds[16 + i][(g + 4 * j) * 8], qreg[j], s2);
    }
    float sc[8];
    float m_loc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int tok = base + (r < 4 ? 4 * g + r : 16 + 4 * g + (r - 4));
      bool ok = tok < t_end;
      if constexpr (decltype(masked)::value) ok = ok && T::one(ld2(mrow + (ok ? tok : 0))) == 0.f;
      const float raw = r < 4 ? s1[r] : s2[r - 4];
      sc[r] = ok ? raw * p.scale_log2 : -INFINITY;
      m_loc = fmaxf(m_loc, sc[r]);
    }
    m_loc = rows_max(m_loc);
    const float m_new = fmaxf(m, m_loc);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = fast_exp2(m - m_use);
    float pr[8];
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      pr[r] = fast_exp2(sc[r] - m_use);
      psum += pr[r];
    }
    l = fmaf(l, corr, psum);
    m = m_new;
    u32x4 pb;  // B operand: k-slots 8g .. 8g+7 = tokens 4g+r, 16+4g+r
    pb.x = (uint32_t)T::pack(pr[0]) | ((uint32_t)T::pack(pr[1]) << 16);
    pb.y = (uint32_t)T::pack(pr[2]) | ((uint32_t)T::pack(pr[3]) << 16);
    pb.z = (uint32_t)T::pack(pr[4]) | ((uint32_t)T::pack(pr[5]) << 16);
    pb.w = (uint32_t)T::pack(pr[6]) | ((uint32_t)T::pack(pr[7]) << 16);
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const u32x2 lo = lds_read_tr16(&v_lds[4 * g + (i >> 2)][16 * db + 4 * (i & 3)]);
      const u32x2 hi = lds_read_tr16(&v_lds[16 + 4 * g + (i >> 2)][16 * db + 4 * (i & 3)]);
      const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
      f32x4 a = acc[db];
      a.x *= corr; a.y *= corr; a.z *= corr; a.w *= corr;
      acc[db] = attn_mfma<T>(va, pb, a);
    }
  };

  auto sweep = [&](auto masked) {
    for (int kb = 0; kb < n_blk; ++kb) {
      const int base = base0 + kb * kBlock;
      park(base, blk);
      load_block(base + kBlock, blk);
      attend(base, masked);
      __builtin_amdgcn_wave_barrier();  // the tiles are rewritten by the next park
    }
  };
  if (mrow != nullptr) sweep(std::true_type{}); else sweep(std::false_type{});

  // ---- the wave's totals: l summed over the four lane groups (m is already shared) ----
  l = rows_sum(l);

  // ---- merge the NW waves through LDS (the V tiles are dead: every wave has finished) ----
  __syncthreads();
  if (g == 0 && i < G) lds_m[wave][i] = m;
  __syncthreads();
  float mx = -INFINITY;
  if (i < G) {
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) mx = fmaxf(mx, lds_m[w2][i]);
  }
  const float f = fast_exp2(m - ((mx == -INFINITY) ? 0.f : mx));
  if (i < G) {
    if (g == 0) lds_l[wave][i] = l * f;
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      // C layout: lane (g, i) holds O^T[d = 16 db + 4 g + r][head i]
      f32x4 o = acc[db];
      o.x *= f; o.y *= f; o.z *= f; o.w *= f;
      *(f32x4*)&tile[wave][i][16 * db + 4 * g] = o;
    }
  }
  __syncthreads();

  for (int e = t; e < G * kHeadDim; e += kAttnThreads) {
    const int hh = e / kHeadDim, d = e % kHeadDim;
    const int head = head0 + hh;
    float a = 0.f, lsum = 0.f, mxx = lds_m[0][hh];
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) {
      a += tile[w2][hh][d];
      lsum += lds_l[w2][hh];
      mxx = fmaxf(mxx, lds_m[w2][hh]);
    }
    if constexpr (DIRECT) {
      p.out[((long)b * p.hq + head) * kHeadDim + d] = T::pack(lsum > 0.f ? a / lsum : 0.f);
    } else {
      const long pi = ((long)b * p.hq + head) * p.n_splits + split;
      p.part_acc[pi * kHeadDim + d] = a;
      if (d == 0) {
        p.part_ml[pi * 2 + 0] = mxx;
        p.part_ml[pi * 2 + 1] = lsum;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Causal attention for T > 1 new tokens (prefill) on the matrix cores: the same formulation as
// attn_decode_mfma_kernel with the 16 MFMA columns holding 16 consecutive QUERY POSITIONS of one
// head instead of the heads of a group. grid = (ceil(T / 16), Hq, B), 4 waves; every wave walks
// 32-token K/V blocks of the causal range [0, q_start + t0 + 16) and the waves are merged through
// LDS. q is already rotated ([B, Hq, T, D] dense, as rope_kv_write_kernel leaves it) and the new
// K/V rows are already in the cache. The reference hands this case to torch SDPA
// (muillm/modules/attention/sdpaattention.py:221-245).
// ---------------------------------------------------------------------------------------
struct PrefillParams {
  const uint16_t* q;        // [B, Hq, T, D]
  const uint16_t* k_cache;  // [B, Hkv, >= S, D] by strides
  const uint16_t* v_cache;
  long c_bs, c_hs, c_ts;
  uint16_t* out;            // [B, T, Hq * D]
  int hq, hkv, tokens, seq_len, q_start;  // query t sits at key position q_start + t; keys [0, seq_len)
  float scale_log2;
  const uint16_t* key_mask;  // optional [B, >= seq_len rounded up to 8]: non-zero = key hidden from every query
  long mask_bs;
};

// four consecutive 16-bit mask entries -> is entry r hidden (anything but +-0)
__device__ __forceinline__ bool key_hidden(const u32x2 m4, int r) {
  const uint32_t w = (r & 2) ? m4.y : m4.x;
  return (((r & 1) ? (w >> 16) : w) & 0x7fffu) != 0u;
}

template <typename T, int NW, bool MASKED>
__global__ void __launch_bounds__(NW * kWave) attn_prefill_mfma_kernel(const PrefillParams p) {
  constexpr int kAttnThreads = NW * kWave;
  constexpr int kBlock = NW * kMfTok;
  __shared__ __attribute__((aligned(16))) uint16_t q_lds[16][kHeadDim];
  __shared__ float lds_m[NW][16];
  __shared__ float lds_l[NW][16];
  constexpr int kVBytes = NW * kMfTok * kMfVStride * 2;
  constexpr int kMergeBytes = NW * 16 * kHeadDim * 4;
  __shared__ __attribute__((aligned(16))) char big_lds[kVBytes > kMergeBytes ? kVBytes : kMergeBytes];
  uint16_t (*v_lds)[kMfVStride] = (uint16_t (*)[kMfVStride])(big_lds + (size_t)(threadIdx.x >> 6) * kMfTok * kMfVStride * 2);
  float (*tile)[16][kHeadDim] = (float (*)[16][kHeadDim])big_lds;
  __shared__ __attribute__((aligned(16))) uint16_t k_tiles[NW][kMfTok][kMfKStride];
  uint16_t (*k_lds)[kMfKStride] = k_tiles[threadIdx.x >> 6];

  // grid = (Hq * B, position tiles): x is handed out first, so every head's long tiles start first
  const int t0 = (gridDim.y - 1 - blockIdx.y) * 16, head = blockIdx.x % p.hq, b = blockIdx.x / p.hq;
  const int kvh = head / (p.hq / p.hkv);
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int g = lane >> 4;
  const int i = lane & 15;

  // keys this tile can see: [0, kv_end); column i (query t0 + i) sees tokens < limit_i
  int kv_end = p.q_start + t0 + 16;
  kv_end = kv_end < p.seq_len ? kv_end : p.seq_len;
  const bool col_ok = (t0 + i) < p.tokens;
  int limit_i = p.q_start + t0 + i + 1;
  limit_i = limit_i < p.seq_len ? limit_i : p.seq_len;
  if (!col_ok) limit_i = 0;

  const uint16_t* kc = p.k_cache + (long)b * p.c_bs + (long)kvh * p.c_hs;
  const uint16_t* vc = p.v_cache + (long)b * p.c_bs + (long)kvh * p.c_hs;

  // K and V in their natural layout (four whole token rows per load instruction), through LDS
  // tiles into the MFMAs; one register set, the tiles being the second buffer; no load behind a
  // branch (see attn_decode_mfma_kernel)
  struct Block {
    u32x4 k[8];  // token base + 4 * u + g, chunk i
    u32x4 v[8];
    u32x2 hidden[2];  // MASKED: mask entries of tokens base + 4 g .. + 3 and base + 16 + 4 g .. + 3
  };
  const uint16_t* mrow = MASKED ? p.key_mask + (long)b * p.mask_bs : nullptr;
  auto load_block = [&](int base, Block& q) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int tok = base + 4 * u + g;
      const long off = (long)(tok < kv_end ? tok : 0) * p.c_ts + i * 8;
      q.k[u] = ld16(kc + off);
      q.v[u] = ld16(vc + off);
    }
    if constexpr (MASKED) {  // groups past the key range read the row's first entries (those tokens are out of range anyway)
      const int m0 = base + 4 * g, m1 = base + 16 + 4 * g;
      q.hidden[0] = ld8(mrow + (m0 < kv_end ? m0 : 0));
      q.hidden[1] = ld8(mrow + (m1 < kv_end ? m1 : 0));
    }
  };

  Block blk;
  const int base0 = wave * kMfTok;
  const int n_blk = base0 < kv_end ? (kv_end - base0 + kBlock - 1) / kBlock : 0;
  load_block(base0, blk);

  for (int e = t; e < 16 * kHeadDim; e += kAttnThreads) {
    const int qi = e / kHeadDim, d = e % kHeadDim;
    uint16_t r = 0;
    if (t0 + qi < p.tokens) r = p.q[(((long)b * p.hq + head) * p.tokens + t0 + qi) * kHeadDim + d];
    q_lds[qi][d] = r;
  }
  __syncthreads();
  u32x4 qreg[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) qreg[j] = *(const u32x4*)&q_lds[i][(g + 4 * j) * 8];

  float m = -INFINITY, l = 0.f;
  f32x4 acc[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x2 hidden_now[2] = {u32x2{0u, 0u}, u32x2{0u, 0u}};  // mask entries of the block in the LDS tiles
  auto park = [&](const Block& q) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      *(u32x4*)&k_lds[4 * u + g][i * 8] = q.k[u];
      *(u32x4*)&v_lds[4 * u + g][i * 8] = q.v[u];
    }
    if constexpr (MASKED) { hidden_now[0] = q.hidden[0]; hidden_now[1] = q.hidden[1]; }
    __builtin_amdgcn_wave_barrier();
  };
  auto attend = [&](int base) {
    f32x4 s1 = {0.f, 0.f, 0.f, 0.f}, s2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // A operands: token 16 * half + i, chunk g + 4 * step
      s1 = attn_mfma<T>(*(const u32x4*)&k_lds[i][(g + 4 * j) * 8], qreg[j], s1);
      s2 = attn_mfma<T>(*(const u32x4*)&k_lds[16 + i][(g + 4 * j) * 8], qreg[j], s2);
    }
    float sc[8];
    float m_loc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int tok = base + (r < 4 ? 4 * g + r : 16 + 4 * g + (r - 4));
      const float raw = r < 4 ? s1[r] : s2[r - 4];
      bool seen = tok < limit_i;
      if constexpr (MASKED) seen = seen && !key_hidden(hidden_now[r >> 2], r & 3);
      sc[r] = seen ? raw * p.scale_log2 : -INFINITY;
      m_loc = fmaxf(m_loc, sc[r]);
    }
    m_loc = rows_max(m_loc);
    const float m_new = fmaxf(m, m_loc);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = fast_exp2(m - m_use);
    float pr[8];
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      pr[r] = fast_exp2(sc[r] - m_use);
      psum += pr[r];
    }
    l = fmaf(l, corr, psum);
    m = m_new;
    u32x4 pb;
    pb.x = (uint32_t)T::pack(pr[0]) | ((uint32_t)T::pack(pr[1]) << 16);
    pb.y = (uint32_t)T::pack(pr[2]) | ((uint32_t)T::pack(pr[3]) << 16);
    pb.z = (uint32_t)T::pack(pr[4]) | ((uint32_t)T::pack(pr[5]) << 16);
    pb.w = (uint32_t)T::pack(pr[6]) | ((uint32_t)T::pack(pr[7]) << 16);
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const u32x2 lo = lds_read_tr16(&v_lds[4 * g + (i >> 2)][16 * db + 4 * (i & 3)]);
      const u32x2 hi = lds_read_tr16(&v_lds[16 + 4 * g + (i >> 2)][16 * db + 4 * (i & 3)]);
      const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
      f32x4 a = acc[db];
      a.x *= corr; a.y *= corr; a.z *= corr; a.w *= corr;
      acc[db] = attn_mfma<T>(va, pb, a);
    }
  };

  for (int kb = 0; kb < n_blk; ++kb) {
    const int base = base0 + kb * kBlock;
    park(blk);
    load_block(base + kBlock, blk);
    attend(base);
    __builtin_amdgcn_wave_barrier();  // the tiles are rewritten by the next park
  }

  l = rows_sum(l);

  __syncthreads();
  if (g == 0) lds_m[wave][i] = m;
  __syncthreads();
  float mx = -INFINITY;
#pragma unroll
  for (int w2 = 0; w2 < NW; ++w2) mx = fmaxf(mx, lds_m[w2][i]);
  const float f = fast_exp2(m - ((mx == -INFINITY) ? 0.f : mx));
  if (g == 0) lds_l[wave][i] = l * f;
#pragma unroll
  for (int db = 0; db < 8; ++db) {
    f32x4 o = acc[db];
    o.x *= f; o.y *= f; o.z *= f; o.w *= f;
    *(f32x4*)&tile[wave][i][16 * db + 4 * g] = o;
  }
  __syncthreads();

  for (int e = t; e < 16 * kHeadDim; e += kAttnThreads) {
    const int qi = e / kHeadDim, d = e % kHeadDim;
    if (t0 + qi >= p.tokens) continue;
    float a = 0.f, lsum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) {
      a += tile[w2][qi][d];
      lsum += lds_l[w2][qi];
    }
    p.out[((long)b * p.tokens + t0 + qi) * ((long)p.hq * kHeadDim) + (long)head * kHeadDim + d] =
        T::pack(lsum > 0.f ? a / lsum : 0.f);
  }
}

// ---------------------------------------------------------------------------------------
// Causal attention for long prompts: every K/V row that crosses LDS serves 32 query positions of
// ALL query heads of its KV head.
//
// grid = (Hkv * B, position tiles): workgroups are handed out x first, so the heaviest (last)
// position tile of EVERY KV head starts before any lighter tile -- with the tiles of one head
// after another the last heads' long tiles started when the chip was half done (64 % of the CU
// time busy at 4096 tokens) --, and with Hkv * B a multiple of the eight XCDs each XCD's L2 sees
// the K/V of its own heads only. A workgroup has one wave
// per (query head of the KV group, block of 32 query positions): NW = 4 waves for 1, 2 or 4 heads
// per KV head (4, 2, 1 position blocks), 8 waves for 8. The workgroup walks the causal key range
// in blocks of 64 tokens: all threads load the block's K and V rows in their natural layout (whole
// 256-byte rows, the next block in flight while the current one is multiplied) into ONE LDS tile
// pair that every wave reads -- K as MFMA A operands, V transposed with ds_read_b64_tr_b16, as
// in attn_decode_mfma_kernel. Per 32 tokens a wave issues 32 MFMAs (two query tiles of 16
// positions share each operand read), keeps its own online softmax (fp32, one rescale per 32
// tokens) and needs no merge with other waves. K/V are read from HBM/L2 once per 32 query
// positions of a KV head (attn_prefill_mfma_kernel: once per 16 positions of every query head).
// The reference hands this case to torch SDPA after repeat_kv
// (muillm/modules/attention/sdpaattention.py:221-245).
// ---------------------------------------------------------------------------------------
constexpr int kPgTok = 64;  // tokens per LDS block

// DMA: the K and V rows of a block go from global memory straight into one of TWO LDS tile pairs
// (global_load_lds_dwordx4: a wave instruction delivers four whole 256-byte rows), the block after
// the current one while the current one is multiplied: no staging registers, no copy into LDS
// between two barriers (a fifth of a block's time), one barrier per block. The rows are unpadded;
// 16-byte chunk c of row r sits in chunk slot c ^ (r % 16), applied on the global side of the load
// and in every LDS address (the sixteen rows of an operand read, and the rows of a transposing
// read, then fall into different banks). Needs 16-byte aligned cache rows.
extern __shared__ __align__(16) unsigned char pg_smem[];
template <typename T, int G, bool MASKED, bool DMA = false>
__global__ void __launch_bounds__((G == 8 ? 8 : 4) * kWave, (G == 8 ? 1 : 2)) attn_prefill_group_kernel(const PrefillParams p) {
  constexpr int NW = (G == 8) ? 8 : 4;
  constexpr int kThreads = NW * kWave;
  constexpr int PB = NW / G;           // blocks of 32 query positions per workgroup
  constexpr int POS = PB * 32;
  constexpr int LCH = kPgTok * 16 / kThreads;  // 16-byte chunks of K (and of V) per thread and block
  constexpr int KROW = DMA ? kHeadDim : kMfKStride, VROW = DMA ? kHeadDim : kMfVStride;  // elements per LDS row
  constexpr int NST = DMA ? 2 : 1;                                                      // LDS stages
  __shared__ __attribute__((aligned(16))) uint16_t k_static[DMA ? 8 : kPgTok * kMfKStride];
  __shared__ __attribute__((aligned(16))) uint16_t v_static[DMA ? 8 : kPgTok * kMfVStride];
  uint16_t* k_lds = DMA ? (uint16_t*)pg_smem : k_static;                                // [NST][kPgTok][KROW]
  uint16_t* v_lds = DMA ? (uint16_t*)pg_smem + NST * kPgTok * KROW : v_static;          // [NST][kPgTok][VROW]
  __shared__ __attribute__((aligned(16))) uint16_t hidden_lds[MASKED ? NST * kPgTok : 8];  // mask entries of the block
  int cur = 0;  // stage the current block is in
  // element offset of 16-bit element `col` of row `row` of the current K / V tile
  auto k_at = [&](int row, int col) -> const uint16_t* {
    if constexpr (DMA) return k_lds + (cur * kPgTok + row) * KROW + ((((col >> 3) ^ row) & 15) << 3) + (col & 7);
    else return k_lds + row * KROW + col;
  };
  auto v_at = [&](int row, int col) -> const uint16_t* {
    if constexpr (DMA) return v_lds + (cur * kPgTok + row) * VROW + ((((col >> 3) ^ row) & 15) << 3) + (col & 7);
    else return v_lds + row * VROW + col;
  };

  const int tile = gridDim.y - 1 - blockIdx.y;  // long key ranges first
  const int kvh = blockIdx.x % p.hkv, b = blockIdx.x / p.hkv;
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  const int g = lane >> 4;
  const int i = lane & 15;
  const int head = kvh * G + (wave % G);
  const int tpos = tile * POS + (wave / G) * 32;  // first query position of this wave

  // keys the workgroup can see: [0, kv_end); query column i of tile qt sees tokens < limit[qt]
  int kv_end = p.q_start + tile * POS + POS;
  kv_end = kv_end < p.seq_len ? kv_end : p.seq_len;
  int limit[2], wave_end = 0;
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const int pos = tpos + 16 * qt + i;
    int lim = p.q_start + pos + 1;
    lim = lim < p.seq_len ? lim : p.seq_len;
    limit[qt] = pos < p.tokens ? lim : 0;
  }
  {
    int last = tpos + 31 < p.tokens - 1 ? tpos + 31 : p.tokens - 1;  // last live position of the wave
    wave_end = last >= tpos ? p.q_start + last + 1 : 0;
    wave_end = wave_end < p.seq_len ? wave_end : p.seq_len;
  }
  // keys below this are seen by every query of the wave: no causal test needed for such blocks
  int wave_all_see = p.q_start + tpos + 1;
  wave_all_see = wave_all_see < p.seq_len ? wave_all_see : p.seq_len;

  const uint16_t* kc = p.k_cache + (long)b * p.c_bs + (long)kvh * p.c_hs;
  const uint16_t* vc = p.v_cache + (long)b * p.c_bs + (long)kvh * p.c_hs;

  u32x4 kreg[LCH], vreg[LCH];
  u32x2 hreg = {0u, 0u};
  const uint16_t* mrow = MASKED ? p.key_mask + (long)b * p.mask_bs : nullptr;
  auto load_block = [&](int base) {
#pragma unroll
    for (int u = 0; u < LCH; ++u) {
      const int c = t + kThreads * u;
      const int tok = base + (c >> 4);
      // rows past the key range read row 0 (their scores are masked): no load behind a branch
      const long off = (long)(tok < kv_end ? tok : 0) * p.c_ts + (c & 15) * 8;
      kreg[u] = ld16(kc + off);
      vreg[u] = ld16(vc + off);
    }
    if constexpr (MASKED) {  // every thread reads the four entries of group t % 16 (no load behind a branch); 16 threads keep them
      const int m0 = base + 4 * (t & 15);
      hreg = ld8(mrow + (m0 < kv_end ? m0 : 0));
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int u = 0; u < LCH; ++u) {
      const int c = t + kThreads * u;
      *(u32x4*)&k_lds[(c >> 4) * KROW + (c & 15) * 8] = kreg[u];
      *(u32x4*)&v_lds[(c >> 4) * VROW + (c & 15) * 8] = vreg[u];
    }
    if constexpr (MASKED) {
      if (t < 16) *(u32x2*)&hidden_lds[4 * t] = hreg;
    }
  };
  // DMA: the block's 16 + 16 groups of four rows are dealt to the waves; lane l of an instruction
  // fills chunk slot l % 16 of row l / 16 of its group
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto dma_block = [&](int base, int stage) {
    constexpr int NI = 16 / NW;  // instructions per wave and tile
#pragma unroll
    for (int q = 0; q < NI; ++q) {
      const int grp = q * NW + wave_u;
      const int row = 4 * grp + (lane >> 4);
      const int tok = base + row;
      // rows past the key range read row 0 (their scores are masked)
      const long off = (long)(tok < kv_end ? tok : 0) * p.c_ts + (((lane ^ row) & 15) << 3);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kc + off),
                                       (__attribute__((address_space(3))) void*)(k_lds + (stage * kPgTok + 4 * grp) * KROW),
                                       16, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vc + off),
                                       (__attribute__((address_space(3))) void*)(v_lds + (stage * kPgTok + 4 * grp) * VROW),
                                       16, 0, 0);
    }
  };
  auto load_hidden = [&](int base) {  // DMA path: the mask entries still travel through a register
    if constexpr (MASKED) {
      const int m0 = base + 4 * (t & 15);
      hreg = ld8(mrow + (m0 < kv_end ? m0 : 0));
    }
  };

  const int n_blk = (kv_end + kPgTok - 1) / kPgTok;
  if constexpr (DMA) {
    dma_block(0, 0);
    load_hidden(0);
  } else {
    load_block(0);
  }

  // B operands: rotated q of this wave's head, positions tpos + 16 qt + i, chunk g + 4 j
  u32x4 qreg[2][4];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    int pos = tpos + 16 * qt + i;
    pos = pos < p.tokens ? pos : p.tokens - 1;
    const uint16_t* qrow = p.q + (((long)b * p.hq + head) * p.tokens + pos) * kHeadDim;
#pragma unroll
    for (int j = 0; j < 4; ++j) qreg[qt][j] = ld16(qrow + (g + 4 * j) * 8);
  }

  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  f32x4 acc[2][8];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int db = 0; db < 8; ++db) acc[qt][db] = f32x4{0.f, 0.f, 0.f, 0.f};

  // one 32-token half of the LDS block (rows r0 .. r0 + 31), key positions base ..; below_diag: every
  // query of the wave sees every key of the half (no causal test, the common case)
  auto attend = [&](int r0, int base, auto below_diag) {
    f32x4 s1[2], s2[2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) { s1[qt] = f32x4{0.f, 0.f, 0.f, 0.f}; s2[qt] = f32x4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4 ka1 = *(const u32x4*)k_at(r0 + i, (g + 4 * j) * 8);
      const u32x4 ka2 = *(const u32x4*)k_at(r0 + 16 + i, (g + 4 * j) * 8);
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        s1[qt] = attn_mfma<T>(ka1, qreg[qt][j], s1[qt]);
        s2[qt] = attn_mfma<T>(ka2, qreg[qt][j], s2[qt]);
      }
    }
    u32x4 pb[2];
    float corr[2];
    u32x2 hid[2] = {u32x2{0u, 0u}, u32x2{0u, 0u}};
    if constexpr (MASKED) {
      hid[0] = *(const u32x2*)&hidden_lds[cur * kPgTok + r0 + 4 * g];
      hid[1] = *(const u32x2*)&hidden_lds[cur * kPgTok + r0 + 16 + 4 * g];
    }
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      // raw scores; the scale (positive) goes into the exponent's fma: p = 2^(raw * scale - m)
      float raw[8];
      float m_raw = -INFINITY;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const int tok = base + (r < 4 ? 4 * g + r : 16 + 4 * g + (r - 4));
        raw[r] = r < 4 ? s1[qt][r] : s2[qt][r - 4];
        if constexpr (!(decltype(below_diag)::value && !MASKED)) {
          bool seen = tok < limit[qt];
          if constexpr (MASKED) seen = seen && !key_hidden(hid[r >> 2], r & 3);
          raw[r] = seen ? raw[r] : -INFINITY;
        }
        m_raw = fmaxf(m_raw, raw[r]);
      }
      m_raw = rows_max(m_raw);
      const float m_new = fmaxf(m[qt], m_raw * p.scale_log2);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      corr[qt] = fast_exp2(m[qt] - m_use);
      float pr[8];
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        pr[r] = fast_exp2(fmaf(raw[r], p.scale_log2, -m_use));
        psum += pr[r];
      }
      l[qt] = fmaf(l[qt], corr[qt], psum);
      m[qt] = m_new;
      pb[qt].x = T::pack2(pr[0], pr[1]);
      pb[qt].y = T::pack2(pr[2], pr[3]);
      pb[qt].z = T::pack2(pr[4], pr[5]);
      pb[qt].w = T::pack2(pr[6], pr[7]);
    }
    // the running maxima settle after the first blocks: the 64 accumulator rescalings are skipped
    // whenever no lane of the wave raised its maximum (exp2(0) is exactly 1)
    if (__builtin_amdgcn_ballot_w64(corr[0] != 1.f || corr[1] != 1.f) != 0) {
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int db = 0; db < 8; ++db) {
          f32x4 a = acc[qt][db];
          a.x *= corr[qt]; a.y *= corr[qt]; a.z *= corr[qt]; a.w *= corr[qt];
          acc[qt][db] = a;
        }
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      const u32x2 lo = lds_read_tr16(v_at(r0 + 4 * g + (i >> 2), 16 * db + 4 * (i & 3)));
      const u32x2 hi = lds_read_tr16(v_at(r0 + 16 + 4 * g + (i >> 2), 16 * db + 4 * (i & 3)));
      const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) acc[qt][db] = attn_mfma<T>(va, pb[qt], acc[qt][db]);
    }
  };

  // a whole 64-token block that every query of the wave sees (the bulk of a long prompt): all 32
  // score MFMAs first, ONE online-softmax step over the 16 scores per lane and query tile, then all
  // 32 value MFMAs -- half the shuffles, rescale tests and exponentials of the running maxima of
  // two 32-token steps, and the softmax arithmetic of one query tile can run under the matrix
  // instructions of the other
  auto attend_block = [&]() {
    f32x4 sc4[2][4];  // [query tile][rows 0-15, 16-31, 32-47, 48-63 of the block]
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int h = 0; h < 4; ++h) sc4[qt][h] = f32x4{0.f, 0.f, 0.f, 0.f};
    // the wave that multiplies goes first: the other wave of the SIMD fits its softmax arithmetic
    // between the matrix instructions
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const u32x4 ka = *(const u32x4*)k_at(16 * h + i, (g + 4 * j) * 8);
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) sc4[qt][h] = attn_mfma<T>(ka, qreg[qt][j], sc4[qt][h]);
      }
    }
    // pinned order: the K operands of two k-slices requested up front, then eight matrix
    // instructions per four further reads (left alone the compiler reuses one operand register
    // set and waits for an LDS read right before half of the multiplies)
    {
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      __builtin_amdgcn_sched_barrier(0x6);  // only scalar and vector ALU work may move across
    }
    __builtin_amdgcn_s_setprio(0);
    u32x4 pb[2][2];
    float corr[2];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      float m_raw = -INFINITY;
#pragma unroll
      for (int h = 0; h < 4; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) m_raw = fmaxf(m_raw, sc4[qt][h][r]);
      m_raw = rows_max(m_raw);
      const float m_new = fmaxf(m[qt], m_raw * p.scale_log2);  // finite: the block is fully visible
      corr[qt] = fast_exp2(m[qt] - m_new);
      float pr[4][4];
      float psum = 0.f;
#pragma unroll
      for (int h = 0; h < 4; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          pr[h][r] = fast_exp2(fmaf(sc4[qt][h][r], p.scale_log2, -m_new));
          psum += pr[h][r];
        }
      l[qt] = fmaf(l[qt], corr[qt], psum);
      m[qt] = m_new;
#pragma unroll
      for (int half = 0; half < 2; ++half) {  // B operand of a 32-token half: tokens 4 g + r, then 16 + 4 g + r
        pb[qt][half].x = T::pack2(pr[2 * half][0], pr[2 * half][1]);
        pb[qt][half].y = T::pack2(pr[2 * half][2], pr[2 * half][3]);
        pb[qt][half].z = T::pack2(pr[2 * half + 1][0], pr[2 * half + 1][1]);
        pb[qt][half].w = T::pack2(pr[2 * half + 1][2], pr[2 * half + 1][3]);
      }
    }
    if (__builtin_amdgcn_ballot_w64(corr[0] != 1.f || corr[1] != 1.f) != 0) {
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int db = 0; db < 8; ++db) {
          f32x4 a = acc[qt][db];
          a.x *= corr[qt]; a.y *= corr[qt]; a.z *= corr[qt]; a.w *= corr[qt];
          acc[qt][db] = a;
        }
    }
    __builtin_amdgcn_sched_barrier(0x6);
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        const u32x2 lo = lds_read_tr16(v_at(32 * half + 4 * g + (i >> 2), 16 * db + 4 * (i & 3)));
        const u32x2 hi = lds_read_tr16(v_at(32 * half + 16 + 4 * g + (i >> 2), 16 * db + 4 * (i & 3)));
        const u32x4 va = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) acc[qt][db] = attn_mfma<T>(va, pb[qt][half], acc[qt][db]);
      }
    {  // four value tiles requested ahead, then two reads per two matrix instructions
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 1);
#pragma unroll
      for (int r = 0; r < 12; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 1);
    }
    __builtin_amdgcn_s_setprio(0);
  };

  for (int kb = 0; kb < n_blk; ++kb) {
    const int base = kb * kPgTok;
    if constexpr (DMA) {
      cur = kb & 1;
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's rows of the block have landed (and its mask entries)
      if constexpr (MASKED) {
        if (t < 16) *(u32x2*)&hidden_lds[cur * kPgTok + 4 * t] = hreg;
      }
      __syncthreads();  // ... and everybody's; every wave is done with the block before, whose stage is free
      dma_block(base + kPgTok, cur ^ 1);  // in flight while this block is multiplied (past the range: row 0, never read)
      load_hidden(base + kPgTok);
    } else {
      __syncthreads();  // every wave is done with the previous block
      park();
      __syncthreads();
      load_block(base + kPgTok);  // in flight while this block is multiplied
    }
    // a block without hidden keys (all but the padded edge of a prompt) is handled like an unmasked one
    bool block_clear = true;
    if constexpr (MASKED) {
      const u32x2 h4 = *(const u32x2*)&hidden_lds[cur * kPgTok + 4 * (lane & 15)];
      block_clear = __builtin_amdgcn_ballot_w64(((h4.x | h4.y) & 0x7fff7fffu) != 0u) == 0;
    }
    // a wave whose last query cannot see the half skips it (uniform per wave; LDS reads only)
    if (block_clear && base + 64 <= wave_all_see) {
      attend_block();
    } else {
      if (base + 32 <= wave_all_see) attend(0, base, std::true_type{});
      else if (base < wave_end) attend(0, base, std::false_type{});
      if (base + 64 <= wave_all_see) attend(32, base + 32, std::true_type{});
      else if (base + 32 < wave_end) attend(32, base + 32, std::false_type{});
    }
  }

  if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0x0F70);  // the last block's (unused) successor has landed
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    float lt = l[qt];
    lt = rows_sum(lt);
    const int pos = tpos + 16 * qt + i;
    if (pos >= p.tokens) continue;
    const float inv = lt > 0.f ? 1.f / lt : 0.f;
    uint16_t* orow = p.out + ((long)b * p.tokens + pos) * ((long)p.hq * kHeadDim) + (long)head * kHeadDim;
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      // acc[qt][db][e]: d = 16 db + 4 g + e of query column i
      const f32x4 o = acc[qt][db];
      u32x2 pk;
      pk.x = (uint32_t)T::pack(o.x * inv) | ((uint32_t)T::pack(o.y * inv) << 16);
      pk.y = (uint32_t)T::pack(o.z * inv) | ((uint32_t)T::pack(o.w * inv) << 16);
      *(u32x2*)(orow + 16 * db + 4 * g) = pk;
    }
  }
}

// log-sum-exp merge of the per-split partials: one workgroup of 128 threads per (head, batch).
// The split weights are computed once into LDS; the accumulation loop then has no dependent
// loads, so the partial rows of all splits are in flight together.
constexpr int kMaxSplits = 256;
template <typename T>
__global__ void __launch_bounds__(kHeadDim) attn_combine_kernel(const float* part_acc,
                                                                const float* part_ml,
                                                                uint16_t* out, int hq, int n_splits) {
  __shared__ float w_lds[kMaxSplits];
  __shared__ float red[2][2];
  const int head = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const long base = ((long)b * hq + head) * n_splits;
  float mx = -INFINITY;
  for (int s = d; s < n_splits; s += kHeadDim) mx = fmaxf(mx, part_ml[(base + s) * 2]);
  mx = wave_max(mx);
  if ((d & (kWave - 1)) == 0) red[0][d >> 6] = mx;
  __syncthreads();
  mx = fmaxf(red[0][0], red[0][1]);
  const float m_use = (mx == -INFINITY) ? 0.f : mx;
  float lpart = 0.f;
  for (int s = d; s < n_splits; s += kHeadDim) {
    const float w = fast_exp2(part_ml[(base + s) * 2] - m_use);
    w_lds[s] = w;
    lpart = fmaf(w, part_ml[(base + s) * 2 + 1], lpart);
  }
  lpart = wave_sum(lpart);
  if ((d & (kWave - 1)) == 0) red[1][d >> 6] = lpart;
  __syncthreads();
  const float lsum = red[1][0] + red[1][1];
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  const float* pa = part_acc + base * kHeadDim + d;
  int s = 0;
  for (; s + 4 <= n_splits; s += 4) {
    a0 = fmaf(w_lds[s + 0], pa[(long)(s + 0) * kHeadDim], a0);
    a1 = fmaf(w_lds[s + 1], pa[(long)(s + 1) * kHeadDim], a1);
    a2 = fmaf(w_lds[s + 2], pa[(long)(s + 2) * kHeadDim], a2);
    a3 = fmaf(w_lds[s + 3], pa[(long)(s + 3) * kHeadDim], a3);
  }
  for (; s < n_splits; ++s) a0 = fmaf(w_lds[s], pa[(long)s * kHeadDim], a0);
  const float a = (a0 + a1) + (a2 + a3);
  out[((long)b * hq + head) * kHeadDim + d] = T::pack(lsum > 0.f ? a / lsum : 0.f);
}

// RoPE of q (-> q_out) and k (-> cache slot or dense k_out), copy of v, for T tokens.
// grid = (Hq + 2*Hkv, T, B), 128 threads.
struct RopeParams {
  const uint16_t* q; long q_bs, q_ts, q_hs;   // [B, T, Hq, D] by strides; may be null
  const uint16_t* k; long k_bs, k_ts, k_hs;   // may be null
  const uint16_t* v; long v_bs, v_ts, v_hs;   // may be null
  const float* cos; const float* sin; int rope_stride;  // null: no rotation (plain cache update)
  int rope_rows;                              // height of the tables (positions are clamped to it)
  const int64_t* position_ids; long pos_bs;   // [B, T] (pos_bs = 0 broadcasts one row)
  const int64_t* cache_position;              // [T] slots; null: k_out/v_out are dense [B, Hkv, T, D]
  uint16_t* q_out;                            // dense [B, Hq, T, D]
  uint16_t* k_out; uint16_t* v_out; long c_bs, c_hs, c_ts;
  int hq, hkv, tokens, max_t;
};

template <typename T>
__global__ void __launch_bounds__(kHeadDim) rope_kv_write_kernel(const RopeParams p) {
  const int h = blockIdx.x, tkn = blockIdx.y, b = blockIdx.z, d = threadIdx.x;
  const float* cos_row = nullptr;
  const float* sin_row = nullptr;
  if (p.cos) {
    long pos = p.position_ids[(long)b * p.pos_bs + tkn];
    pos = pos < 0 ? 0 : (pos >= p.rope_rows ? p.rope_rows - 1 : pos);
    cos_row = p.cos + pos * p.rope_stride;
    sin_row = p.sin + pos * p.rope_stride;
  }
  if (h < p.hq) {
    if (p.q == nullptr) return;
    const uint16_t* src = p.q + (long)b * p.q_bs + (long)tkn * p.q_ts + (long)h * p.q_hs;
    p.q_out[(((long)b * p.hq + h) * p.tokens + tkn) * kHeadDim + d] = T::pack(rope_elem<T>(src, d, cos_row, sin_row));
    return;
  }
  long slot = tkn;
  if (p.cache_position) {
    slot = p.cache_position[tkn];
    if (slot < 0 || slot >= p.max_t) return;  // out-of-range slots are dropped, never written
  }
  if (h < p.hq + p.hkv) {
    if (p.k == nullptr) return;
    const int kh = h - p.hq;
    const uint16_t* src = p.k + (long)b * p.k_bs + (long)tkn * p.k_ts + (long)kh * p.k_hs;
    p.k_out[(long)b * p.c_bs + (long)kh * p.c_hs + slot * p.c_ts + d] = T::pack(rope_elem<T>(src, d, cos_row, sin_row));
  } else {
    if (p.v == nullptr) return;
    const int vh = h - p.hq - p.hkv;
    const uint16_t* src = p.v + (long)b * p.v_bs + (long)tkn * p.v_ts + (long)vh * p.v_hs;
    p.v_out[(long)b * p.c_bs + (long)vh * p.c_hs + slot * p.c_ts + d] = src[d];
  }
}

// The same with 128-bit accesses, for 16-byte aligned operands: eight threads per head row, each
// with 16-byte chunks c and c + 8 of it (the two halves that rotate into each other, so every
// input is read once); rows are numbered with the heads of a token next to each other, like the
// fused QKV projection leaves them. Same arithmetic per element as rope_elem.
// (512 tokens of 32 + 8 + 8 heads: 13 -> 4 us against one element per thread.)
template <typename T>
__global__ void __launch_bounds__(256) rope_kv_write_vec_kernel(const RopeParams p, long n_rows) {
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  const long row = gid >> 3;
  const int c = (int)(gid & 7);
  if (row >= n_rows) return;
  const int heads = p.hq + 2 * p.hkv;
  const int h = (int)(row % heads);
  const int tkn = (int)((row / heads) % p.tokens);
  const int b = (int)(row / ((long)heads * p.tokens));
  const uint16_t* src;
  uint16_t* dst;
  bool rotate = p.cos != nullptr;
  if (h < p.hq) {
    src = p.q + (long)b * p.q_bs + (long)tkn * p.q_ts + (long)h * p.q_hs;
    dst = p.q_out + (((long)b * p.hq + h) * p.tokens + tkn) * kHeadDim;
  } else {
    long slot = tkn;
    if (p.cache_position) {
      slot = p.cache_position[tkn];
      if (slot < 0 || slot >= p.max_t) return;  // out-of-range slots are dropped, never written
    }
    if (h < p.hq + p.hkv) {
      if (p.k == nullptr) return;
      const int kh = h - p.hq;
      src = p.k + (long)b * p.k_bs + (long)tkn * p.k_ts + (long)kh * p.k_hs;
      dst = p.k_out + (long)b * p.c_bs + (long)kh * p.c_hs + slot * p.c_ts;
    } else {
      if (p.v == nullptr) return;
      const int vh = h - p.hq - p.hkv;
      src = p.v + (long)b * p.v_bs + (long)tkn * p.v_ts + (long)vh * p.v_hs;
      dst = p.v_out + (long)b * p.c_bs + (long)vh * p.c_hs + slot * p.c_ts;
      rotate = false;
    }
  }
  const u32x4 lo = ld16(src + 8 * c), hi = ld16(src + 8 * c + kHeadDim / 2);
  if (!rotate) {
    *(u32x4*)(dst + 8 * c) = lo;
    *(u32x4*)(dst + 8 * c + kHeadDim / 2) = hi;
    return;
  }
  long pos = p.position_ids[(long)b * p.pos_bs + tkn];
  pos = pos < 0 ? 0 : (pos >= p.rope_rows ? p.rope_rows - 1 : pos);
  const float* cs = p.cos + pos * p.rope_stride + 8 * c;
  const float* sn = p.sin + pos * p.rope_stride + 8 * c;
  const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w}, hw[4] = {hi.x, hi.y, hi.z, hi.w};
  uint32_t ol[4], oh[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float l0 = T::lo(lw[j]), l1 = T::hi(lw[j]), h0 = T::lo(hw[j]), h1 = T::hi(hw[j]);
    const float c0 = cs[2 * j], c1 = cs[2 * j + 1], s0 = sn[2 * j], s1 = sn[2 * j + 1];
    // d < 64: x cos - x[d + 64] sin; d >= 64: x cos + x[d - 64] sin
    ol[j] = (uint32_t)T::pack(fmaf(-h0, s0, l0 * c0)) | ((uint32_t)T::pack(fmaf(-h1, s1, l1 * c1)) << 16);
    oh[j] = (uint32_t)T::pack(fmaf(l0, s0, h0 * c0)) | ((uint32_t)T::pack(fmaf(l1, s1, h1 * c1)) << 16);
  }
  *(u32x4*)(dst + 8 * c) = u32x4{ol[0], ol[1], ol[2], ol[3]};
  *(u32x4*)(dst + 8 * c + kHeadDim / 2) = u32x4{oh[0], oh[1], oh[2], oh[3]};
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
// tokens per worker and pass: 4 with 4 or 8 waves (<= 256 VGPRs available), 2 with 16 waves
// (128 VGPRs)
constexpr int unroll_for(int nw) { return nw == 16 ? 2 : 4; }

static int g_attn_waves = 0;  // 0: built-in choice; 4, 8 or 16 forces the workgroup size
static int g_attn_head_parallel = 1;  // unsplit decodes at small batch: workgroup per query head
static int g_attn_direct_tokens = 0;  // 0: built-in choice; longest sequence decoded unsplit
// Matrix-core kernel (attn_decode_mfma_kernel). 0 = built-in choice: whenever a workgroup
// handles a whole KV group, i.e. everywhere except the unsplit head-parallel mode of short
// sequences (32k context: 30 vs 35 us at batch 1, 163 vs 174 us at batch 8; on par at 1k).
// > 0: also instead of the head-parallel mode from that many tokens on; < 0: never.
static int g_attn_mfma_tokens = 0;

static inline bool attn_force_mfma(const AttnParams& p) {
  if (g_attn_mfma_tokens <= 0) return false;
  const int hint = p.seq_len > 0 ? p.seq_len : p.max_t;
  return hint >= g_attn_mfma_tokens;
}

// waves per workgroup for a given number of query heads per KV head
static inline int attn_waves_for(int g) {
  if (g > 4) return 4;  // 8 heads per group: ~240 VGPRs, one wave per SIMD
  return g_attn_waves ? g_attn_waves : 8;
}

template <typename T, int G, int NW>
static void launch_attn_nw(hipStream_t s, const AttnParams& p, dim3 grid) {
  if (p.n_splits == 1)
    hipLaunchKernelGGL((attn_decode_kernel<T, G, unroll_for(NW), NW, true>), grid, dim3(NW * kWave), 0, s,
                       p.cache_position, p.position_ids, p.pos_bs, p.q, p.k_cache, p.v_cache, p.cos, p);
  else
    hipLaunchKernelGGL((attn_decode_kernel<T, G, unroll_for(NW), NW, false>), grid, dim3(NW * kWave), 0, s,
                       p.cache_position, p.position_ids, p.pos_bs, p.q, p.k_cache, p.v_cache, p.cos, p);
}

template <typename T, int G, bool MFMA_ONLY = false>
static int launch_attn_g(hipStream_t s, const AttnParams& p, int batch) {
  dim3 grid(p.n_splits, p.hq / G, batch);
  const int nw = attn_waves_for(G);
  const bool mfma = MFMA_ONLY || (G == p.hq / p.hkv && g_attn_mfma_tokens >= 0);
  // cache warmers ride along with the unsplit one-workgroup-per-query-head launch of the vector
  // kernel only (the other shapes fill the chip themselves); they sit behind the head workgroups
  // in y, and hq % 8 == 0 keeps their XCD the one warm_cache() counts on
  if (G == 1 && !mfma && p.n_splits == 1 && p.warm && p.warm_wgs > 0 && p.hq % 8 == 0) grid.y += p.warm_wgs;
  if (mfma) {
    if (p.n_splits == 1)
      hipLaunchKernelGGL((attn_decode_mfma_kernel<T, G, 8, true>), grid, dim3(8 * kWave), 0, s, p.cache_position,
                         p.position_ids, p.pos_bs, p.q, p.k_cache, p.v_cache, p.cos, p);
    else
      hipLaunchKernelGGL((attn_decode_mfma_kernel<T, G, 8, false>), grid, dim3(8 * kWave), 0, s, p.cache_position,
                         p.position_ids, p.pos_bs, p.q, p.k_cache, p.v_cache, p.cos, p);
  } else if constexpr (MFMA_ONLY) {
    return MUI_ERR_UNSUPPORTED;
  } else if constexpr (G <= 4) {
    if (nw == 16) launch_attn_nw<T, G, 16>(s, p, grid);
    else if (nw == 8) launch_attn_nw<T, G, 8>(s, p, grid);
    else launch_attn_nw<T, G, 4>(s, p, grid);
  } else {
    launch_attn_nw<T, G, 4>(s, p, grid);
  }
  int st = launch_status();
  if (st != MUI_OK) return st;
  if (p.n_splits > 1) {
    hipLaunchKernelGGL((attn_combine_kernel<T>), dim3(p.hq, batch), dim3(kHeadDim), 0, s,
                       (const float*)p.part_acc, (const float*)p.part_ml, p.out, p.hq, p.n_splits);
    st = launch_status();
  }
  return st;
}

template <typename T>
static int launch_attn_t(hipStream_t s, const AttnParams& p, int batch) {
  // unsplit and too few KV heads to occupy the GPU: one workgroup per query head
  if (p.n_splits == 1 && g_attn_head_parallel && batch * p.hkv * 8 <= device_cus() && !attn_force_mfma(p))
    return launch_attn_g<T, 1>(s, p, batch);
  switch (p.hq / p.hkv) {
    case 1: return launch_attn_g<T, 1>(s, p, batch);
    case 2: return launch_attn_g<T, 2>(s, p, batch);
    case 4: return launch_attn_g<T, 4>(s, p, batch);
    case 8: return launch_attn_g<T, 8>(s, p, batch);
    // other group sizes: the matrix-core kernel pads the heads of a group to 16 columns anyway
    case 3: if (g_attn_mfma_tokens >= 0) return launch_attn_g<T, 3, true>(s, p, batch); break;
    case 5: if (g_attn_mfma_tokens >= 0) return launch_attn_g<T, 5, true>(s, p, batch); break;
    case 6: if (g_attn_mfma_tokens >= 0) return launch_attn_g<T, 6, true>(s, p, batch); break;
    case 7: if (g_attn_mfma_tokens >= 0) return launch_attn_g<T, 7, true>(s, p, batch); break;
    default: break;
  }
  // any other ratio: one workgroup per query head (K/V re-read by the heads of a group)
  return launch_attn_g<T, 1>(s, p, batch);
}

static int launch_attn(hipStream_t s, int dtype, const AttnParams& p, int batch) {
  if (dtype == MUI_DTYPE_F16) return launch_attn_t<F16>(s, p, batch);
  if (dtype == MUI_DTYPE_BF16) return launch_attn_t<BF16>(s, p, batch);
  return MUI_ERR_INVALID_ARG;
}

}  // namespace mui

using namespace mui;

static int g_attn_min_tokens = 0;  // 0: built-in choice; else fewest tokens worth a split
// prompt attention: 0 = built-in choice (the KV-group kernel from 512 query tokens), n > 0 = from n
// tokens, negative = never
static int g_prefill_group_tokens = 0;
static int g_prefill_attn_direct = 1;  // 0: K / V rows staged through registers

extern "C" int mui_tune_prefill_attention(int group_kernel_min_tokens) {
  MUI_TUNE_GUARD();
  // experiments: 1000000 + n keeps the K / V rows of the KV-group kernel on the register-staged path
  g_prefill_attn_direct = group_kernel_min_tokens >= 1000000 ? 0 : 1;
  if (group_kernel_min_tokens >= 1000000) group_kernel_min_tokens -= 1000000;
  g_prefill_group_tokens = group_kernel_min_tokens;
  return MUI_OK;
}

// launch of a KV-group kernel variant that needs the dynamic LDS limit raised (once per kernel and device)
template <typename K>
static int launch_pg_direct(K kernel, dim3 grid, int threads, int lds, hipStream_t s, const PrefillParams& p) {
  static int raised_for = -1;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return MUI_ERR_DEVICE;
  if (raised_for != dev) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return MUI_ERR_LAUNCH;
    raised_for = dev;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(threads), lds, s, p);
  return MUI_OK;
}

extern "C" int mui_tune_attention(int waves_per_workgroup, int min_tokens_per_split, int direct_tokens,
                                  int mfma_tokens) {
  MUI_TUNE_GUARD();
  if (!(waves_per_workgroup == 0 || waves_per_workgroup == 4 || waves_per_workgroup == 8 || waves_per_workgroup == 16))
    return MUI_ERR_INVALID_ARG;
  if (min_tokens_per_split < 0) return MUI_ERR_INVALID_ARG;
  g_attn_waves = waves_per_workgroup;
  g_attn_min_tokens = min_tokens_per_split;
  g_attn_head_parallel = direct_tokens >= 0;
  g_attn_direct_tokens = direct_tokens > 0 ? direct_tokens : 0;
  g_attn_mfma_tokens = mfma_tokens;
  return MUI_OK;
}

extern "C" int mui_flash_decode_splits(int batch, int n_q_heads, int n_kv_heads, int seq_len_hint) {
  if (batch <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || seq_len_hint <= 0) return 1;
  const int nw = attn_waves_for(n_q_heads / n_kv_heads);
  const int kBlock = nw * 4 * unroll_for(nw);  // tokens per workgroup pass
  // Splitting buys parallelism but every split beyond the first costs the combine launch
  // (~4 us) and partial traffic, so a split must carry a few passes of work. (Merging the
  // splits inside the kernel with a device-scope fence + counter was measured slower than
  // the combine launch on MI355X.) The total is one workgroup per CU: measured best at 32
  // splits for batch 1 and 4 splits for batch 8 with 8 KV heads.
  // Short sequences at small batch: one unsplit workgroup per query head beats split + merge.
  const int direct = g_attn_direct_tokens > 0 ? g_attn_direct_tokens : 1536;
  if (g_attn_head_parallel && seq_len_hint <= direct && batch * n_kv_heads * 8 <= device_cus()) return 1;
  const int min_tokens = g_attn_min_tokens > 0 ? g_attn_min_tokens : 2 * kBlock;
  const int max_useful = ceil_div(seq_len_hint, min_tokens);
  int want = device_cus() / (batch * n_kv_heads);  // one workgroup per CU, never a ragged second round
  if (want > 32) want = 32;
  int n = want < max_useful ? want : max_useful;
  if (n < 1) n = 1;
  return n;
}

extern "C" size_t mui_flash_decode_scratch_bytes(int batch, int n_q_heads, int head_dim, int n_splits) {
  if (batch <= 0 || n_q_heads <= 0 || head_dim <= 0 || n_splits <= 1) return 0;
  return (size_t)batch * n_q_heads * n_splits * (head_dim + 2) * sizeof(float);
}

static int check_attn_shape(int dtype, int batch, int hq, int hkv, int head_dim, int n_splits,
                            int max_t) {
  if (!(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16)) return MUI_ERR_INVALID_ARG;
  if (batch <= 0 || hq <= 0 || hkv <= 0 || n_splits <= 0 || max_t <= 0) return MUI_ERR_INVALID_ARG;
  if (n_splits > kMaxSplits) return MUI_ERR_UNSUPPORTED;
  if (head_dim != kHeadDim) return MUI_ERR_UNSUPPORTED;
  if (hq % hkv != 0) return MUI_ERR_INVALID_ARG;
  if (batch > 65535 || hq > 65535) return MUI_ERR_UNSUPPORTED;
  return MUI_OK;
}

extern "C" int mui_flash_decode(mui_stream_t stream, int dtype, const void* q, const void* k_cache,
                                const void* v_cache, long cache_batch_stride, long cache_head_stride,
                                long cache_token_stride, const void* mask, long mask_batch_stride,
                                int seq_len, void* scratch, int n_splits, void* out, int batch,
                                int n_q_heads, int n_kv_heads, int head_dim, int max_cache_len) {
  int st = check_attn_shape(dtype, batch, n_q_heads, n_kv_heads, head_dim, n_splits, max_cache_len);
  if (st != MUI_OK) return st;
  MUI_CHECK_ARG(q && k_cache && v_cache && out);
  MUI_CHECK_ARG(seq_len > 0 && seq_len <= max_cache_len);
  if (n_splits > 1 && !scratch) return MUI_ERR_INVALID_ARG;
  if ((cache_token_stride & 7) || (cache_head_stride & 7) || (cache_batch_stride & 7)) return MUI_ERR_ALIGNMENT;
  if (!aligned16(k_cache) || !aligned16(v_cache)) return MUI_ERR_ALIGNMENT;
  AttnParams p = {};
  p.q = (const uint16_t*)q;
  p.q_bs = (long)n_q_heads * head_dim;
  p.q_hs = head_dim;
  p.seq_len = seq_len;
  p.k_cache = (uint16_t*)k_cache;
  p.v_cache = (uint16_t*)v_cache;
  p.c_bs = cache_batch_stride;
  p.c_hs = cache_head_stride;
  p.c_ts = cache_token_stride;
  p.mask = (const uint16_t*)mask;
  p.mask_bs = mask_batch_stride;
  p.part_acc = (float*)scratch;
  p.part_ml = scratch ? (float*)scratch + (size_t)batch * n_q_heads * n_splits * head_dim : nullptr;
  p.out = (uint16_t*)out;
  p.hq = n_q_heads;
  p.hkv = n_kv_heads;
  p.n_splits = n_splits;
  p.max_t = max_cache_len;
  p.scale_log2 = kLog2e / sqrtf((float)head_dim);
  return launch_attn((hipStream_t)stream, dtype, p, batch);
}

// ---------------------------------------------------------------------------------------
// mui_flash_decode for callers that cannot allocate: the split partials live in a file-scope
// device array. Every GPU the library runs on holds its own copy of it, at its own address,
// until the process ends.
// ---------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = MUI_FLASH_DECODE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` per HIP ordinal. In host code the array's name is only a handle
// for hipGetSymbolAddress, never an address a kernel may use.
constexpr int kMaxDevices = 64;
static void* g_static_scratch_ptr[kMaxDevices] = {};
static std::mutex g_static_scratch_lock;

static int static_scratch_for_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MUI_ERR_DEVICE;
  std::lock_guard<std::mutex> guard(g_static_scratch_lock);
  if (!g_static_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return MUI_ERR_DEVICE;
    g_static_scratch_ptr[dev] = ptr;
  }
  *out = g_static_scratch_ptr[dev];
  return MUI_OK;
}

extern "C" size_t mui_flash_decode_static_scratch_limit(void) { return kStaticScratchBytes; }

extern "C" int mui_flash_decode_static(mui_stream_t stream, int dtype, const void* q, const void* k_cache,
                                       const void* v_cache, long cache_batch_stride, long cache_head_stride,
                                       long cache_token_stride, const void* mask, long mask_batch_stride,
                                       int seq_len, int n_splits, void* out, int batch, int n_q_heads,
                                       int n_kv_heads, int head_dim, int max_cache_len) {
  int st = check_attn_shape(dtype, batch, n_q_heads, n_kv_heads, head_dim, n_splits, max_cache_len);
  if (st != MUI_OK) return st;
  // partials of (batch, query head, split): beyond the array's size the call is refused, it
  // never falls back to an allocation
  if (mui_flash_decode_scratch_bytes(batch, n_q_heads, head_dim, n_splits) > kStaticScratchBytes)
    return MUI_ERR_SCRATCH_LIMIT;
  void* ptr = nullptr;
  if (n_splits > 1) {
    st = static_scratch_for_current_device(&ptr);
    if (st != MUI_OK) return st;
  }
  // Nothing in the array has to start at zero: every (row, head, split) slot the merge kernel
  // reads is written by the pass before it, empty splits included.
  return mui_flash_decode(stream, dtype, q, k_cache, v_cache, cache_batch_stride, cache_head_stride,
                          cache_token_stride, mask, mask_batch_stride, seq_len, ptr, n_splits, out, batch,
                          n_q_heads, n_kv_heads, head_dim, max_cache_len);
}

// Cache warming is OFF unless a caller opts in with mui_tune_warm(workgroups > 0, ...): measured on
// MI355X (Llama-3-8B shapes, 64 cached tokens) the warmed o_proj GEMV runs in 3.6 us instead of 6.8 us
// -- the L2s and the memory-side cache keep the matrix across the kernel boundary --, but the attention
// launch that carries the 33.5 MB fetch takes 8.7-9.4 us instead of 5.65 us (its two dependent round
// trips queue behind the fetch, a head start of 1-2.5 us for them does not help), so the pair costs
// 12.4-13.1 us against 12.3 us without and the decode rate is 373-380 against 380 tokens/s.
static int g_warm_wgs = 0;      // <= 0: cache warming off; > 0: warm workgroups added to the launch
static int g_warm_percent = 0;  // 0: built-in choice; share of the announced bytes that is warmed
static int g_warm_delay = -1;   // < 0: built-in choice; head start of the attention workgroups (s_sleep 8 units)

extern "C" int mui_tune_warm(int workgroups, int percent, int delay) {
  MUI_TUNE_GUARD();
  if (percent < 0 || percent > 100 || (workgroups > 0 && workgroups % 8 != 0) || delay > 64) return MUI_ERR_INVALID_ARG;
  g_warm_wgs = workgroups;
  g_warm_percent = percent;
  g_warm_delay = delay;
  return MUI_OK;
}

extern "C" int mui_attn_decode_fused_warm(mui_stream_t stream, int dtype, const void* q, long q_batch_stride,
                                          const void* k_new, long k_batch_stride, const void* v_new,
                                          long v_batch_stride, const float* cos_table, const float* sin_table,
                                          int rope_row_stride, int rope_rows, const int64_t* position_ids,
                                          long position_batch_stride, const int64_t* cache_position,
                                          int seq_len, void* k_cache, void* v_cache, long cache_batch_stride,
                                          long cache_head_stride, long cache_token_stride, const void* mask,
                                          long mask_batch_stride, void* q_out, void* scratch, int n_splits,
                                          void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                                          int max_cache_len, const void* next_weights, size_t next_weight_bytes,
                                          int next_slab_bytes) {
  int st = check_attn_shape(dtype, batch, n_q_heads, n_kv_heads, head_dim, n_splits, max_cache_len);
  if (st != MUI_OK) return st;
  MUI_CHECK_ARG(q && k_new && v_new && k_cache && v_cache && out && cache_position);
  MUI_CHECK_ARG((cos_table == nullptr) == (sin_table == nullptr));
  MUI_CHECK_ARG(seq_len <= max_cache_len);
  if (cos_table && (rope_row_stride < head_dim / 2 || rope_rows <= 0)) return MUI_ERR_INVALID_ARG;
  if (n_splits > 1 && !scratch) return MUI_ERR_INVALID_ARG;
  if ((cache_token_stride & 7) || (cache_head_stride & 7) || (cache_batch_stride & 7)) return MUI_ERR_ALIGNMENT;
  if (!aligned16(k_cache) || !aligned16(v_cache)) return MUI_ERR_ALIGNMENT;
  AttnParams p = {};
  p.q = (const uint16_t*)q;
  p.q_bs = q_batch_stride;
  p.q_hs = head_dim;
  p.k_new = (const uint16_t*)k_new;
  p.k_bs = k_batch_stride;
  p.k_hs = head_dim;
  p.v_new = (const uint16_t*)v_new;
  p.v_bs = v_batch_stride;
  p.v_hs = head_dim;
  p.cos = cos_table;
  p.sin = sin_table;
  p.rope_stride = rope_row_stride;
  p.rope_rows = rope_rows;
  p.position_ids = position_ids;
  p.pos_bs = position_batch_stride;
  p.cache_position = cache_position;
  p.seq_len = seq_len;
  p.k_cache = (uint16_t*)k_cache;
  p.v_cache = (uint16_t*)v_cache;
  p.c_bs = cache_batch_stride;
  p.c_hs = cache_head_stride;
  p.c_ts = cache_token_stride;
  p.mask = (const uint16_t*)mask;
  p.mask_bs = mask_batch_stride;
  p.q_out = (uint16_t*)q_out;
  p.part_acc = (float*)scratch;
  p.part_ml = scratch ? (float*)scratch + (size_t)batch * n_q_heads * n_splits * head_dim : nullptr;
  p.out = (uint16_t*)out;
  p.hq = n_q_heads;
  p.hkv = n_kv_heads;
  p.n_splits = n_splits;
  p.max_t = max_cache_len;
  p.scale_log2 = kLog2e / sqrtf((float)head_dim);
  if (next_weights && next_weight_bytes >= 16 && g_warm_wgs > 0) {
    MUI_CHECK_ARG(aligned16(next_weights) && next_slab_bytes >= 16 && next_slab_bytes % 16 == 0);
    // the eight L2s hold 32 MB together; the share beyond what fits would only push out its own head
    const int percent = g_warm_percent > 0 ? g_warm_percent : 100;
    size_t bytes = next_weight_bytes / 100 * percent;
    bytes -= bytes % (size_t)next_slab_bytes;
    if (bytes >= (size_t)next_slab_bytes) {
      p.warm = (const char*)next_weights;
      p.warm_bytes = (long)bytes;
      p.warm_slab = next_slab_bytes;
      p.warm_wgs = g_warm_wgs;
      p.warm_delay = g_warm_delay >= 0 ? g_warm_delay : 0;
    }
  }
  return launch_attn((hipStream_t)stream, dtype, p, batch);
}

extern "C" int mui_attn_decode_fused(mui_stream_t stream, int dtype, const void* q, long q_batch_stride,
                                     const void* k_new, long k_batch_stride, const void* v_new,
                                     long v_batch_stride, const float* cos_table, const float* sin_table,
                                     int rope_row_stride, int rope_rows, const int64_t* position_ids,
                                     long position_batch_stride, const int64_t* cache_position,
                                     int seq_len, void* k_cache, void* v_cache, long cache_batch_stride,
                                     long cache_head_stride, long cache_token_stride, const void* mask,
                                     long mask_batch_stride, void* q_out, void* scratch, int n_splits,
                                     void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                                     int max_cache_len) {
  return mui_attn_decode_fused_warm(stream, dtype, q, q_batch_stride, k_new, k_batch_stride, v_new, v_batch_stride,
                                    cos_table, sin_table, rope_row_stride, rope_rows, position_ids,
                                    position_batch_stride, cache_position, seq_len, k_cache, v_cache,
                                    cache_batch_stride, cache_head_stride, cache_token_stride, mask,
                                    mask_batch_stride, q_out, scratch, n_splits, out, batch, n_q_heads, n_kv_heads,
                                    head_dim, max_cache_len, nullptr, 0, 0);
}

extern "C" int mui_rope_kv_write(mui_stream_t stream, int dtype, const void* q, long q_batch_stride,
                                 long q_token_stride, long q_head_stride, const void* k,
                                 long k_batch_stride, long k_token_stride, long k_head_stride,
                                 const void* v, long v_batch_stride, long v_token_stride,
                                 long v_head_stride, const float* cos_table, const float* sin_table,
                                 int rope_row_stride, int rope_rows, const int64_t* position_ids,
                                 long position_batch_stride, const int64_t* cache_position, void* q_out,
                                 void* k_out, void* v_out, long out_batch_stride, long out_head_stride,
                                 long out_token_stride, int batch, int tokens, int n_q_heads,
                                 int n_kv_heads, int head_dim, int max_cache_len) {
  MUI_CHECK_ARG(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16);
  MUI_CHECK_ARG(batch > 0 && tokens > 0 && n_q_heads >= 0 && n_kv_heads >= 0 && max_cache_len > 0);
  MUI_CHECK_ARG((cos_table == nullptr) == (sin_table == nullptr));
  MUI_CHECK_ARG(!cos_table || position_ids);
  MUI_CHECK_ARG(!q || q_out);
  MUI_CHECK_ARG(!k || k_out);
  MUI_CHECK_ARG(!v || v_out);
  if (head_dim != kHeadDim) return MUI_ERR_UNSUPPORTED;
  if (cos_table && (rope_row_stride < head_dim / 2 || rope_rows <= 0)) return MUI_ERR_INVALID_ARG;
  if (tokens > 65535 || batch > 65535) return MUI_ERR_UNSUPPORTED;
  RopeParams p = {};
  p.q = (const uint16_t*)q; p.q_bs = q_batch_stride; p.q_ts = q_token_stride; p.q_hs = q_head_stride;
  p.k = (const uint16_t*)k; p.k_bs = k_batch_stride; p.k_ts = k_token_stride; p.k_hs = k_head_stride;
  p.v = (const uint16_t*)v; p.v_bs = v_batch_stride; p.v_ts = v_token_stride; p.v_hs = v_head_stride;
  p.cos = cos_table; p.sin = sin_table; p.rope_stride = rope_row_stride; p.rope_rows = rope_rows;
  p.position_ids = position_ids; p.pos_bs = position_batch_stride;
  p.cache_position = cache_position;
  p.q_out = (uint16_t*)q_out; p.k_out = (uint16_t*)k_out; p.v_out = (uint16_t*)v_out;
  p.c_bs = out_batch_stride; p.c_hs = out_head_stride; p.c_ts = out_token_stride;
  p.hq = q ? n_q_heads : 0; p.hkv = n_kv_heads; p.tokens = tokens; p.max_t = max_cache_len;
  const int heads = p.hq + 2 * n_kv_heads;
  if (heads == 0) return MUI_OK;
  hipStream_t s = (hipStream_t)stream;
  // 16-byte aligned rows everywhere (and every tensor that is read has its output): 128-bit accesses
  auto vec_ok = [](const void* ptr, std::initializer_list<long> strides) {
    if ((uintptr_t)ptr & 15u) return false;
    for (long st : strides)
      if (st & 7) return false;
    return true;
  };
  const bool vec = vec_ok(q, {q_batch_stride, q_token_stride, q_head_stride}) &&
                   vec_ok(k, {k_batch_stride, k_token_stride, k_head_stride}) &&
                   vec_ok(v, {v_batch_stride, v_token_stride, v_head_stride}) && vec_ok(q_out, {}) &&
                   vec_ok(k_out, {out_batch_stride, out_head_stride, out_token_stride}) && vec_ok(v_out, {}) &&
                   (!cos_table || (((uintptr_t)cos_table | (uintptr_t)sin_table) & 3u) == 0);
  if (vec) {
    const long n_rows = (long)batch * tokens * heads;
    const long blocks = (n_rows * 8 + 255) / 256;
    if (blocks > 0x7fffffffL) return MUI_ERR_UNSUPPORTED;
    if (dtype == MUI_DTYPE_F16) hipLaunchKernelGGL((rope_kv_write_vec_kernel<F16>), dim3((unsigned)blocks), dim3(256), 0, s, p, n_rows);
    else hipLaunchKernelGGL((rope_kv_write_vec_kernel<BF16>), dim3((unsigned)blocks), dim3(256), 0, s, p, n_rows);
    return launch_status();
  }
  dim3 grid(heads, tokens, batch), block(kHeadDim);
  if (dtype == MUI_DTYPE_F16) hipLaunchKernelGGL((rope_kv_write_kernel<F16>), grid, block, 0, s, p);
  else hipLaunchKernelGGL((rope_kv_write_kernel<BF16>), grid, block, 0, s, p);
  return launch_status();
}

static int prefill_attention_impl(mui_stream_t stream, int dtype, const void* q_rotated, const void* k_cache,
                                  const void* v_cache, long cache_batch_stride, long cache_head_stride,
                                  long cache_token_stride, int seq_len, int q_start, const void* key_mask,
                                  long mask_batch_stride, void* out, int batch, int n_q_heads, int n_kv_heads,
                                  int tokens, int head_dim) {
  MUI_CHECK_ARG(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16);
  MUI_CHECK_ARG(q_rotated && k_cache && v_cache && out);
  MUI_CHECK_ARG(batch > 0 && n_q_heads > 0 && n_kv_heads > 0 && tokens > 0 && seq_len > 0 && q_start >= 0);
  MUI_CHECK_ARG(q_start + tokens <= seq_len);
  if (head_dim != kHeadDim) return MUI_ERR_UNSUPPORTED;
  if (n_q_heads % n_kv_heads != 0) return MUI_ERR_INVALID_ARG;
  if (batch > 65535 || n_q_heads > 65535) return MUI_ERR_UNSUPPORTED;
  if ((cache_token_stride & 7) || (cache_head_stride & 7) || (cache_batch_stride & 7)) return MUI_ERR_ALIGNMENT;
  if (!aligned16(k_cache) || !aligned16(v_cache)) return MUI_ERR_ALIGNMENT;
  if (key_mask) {  // read four entries at a time
    if (((uintptr_t)key_mask & 7) || (mask_batch_stride & 3)) return MUI_ERR_ALIGNMENT;
    if (mask_batch_stride < (long)((seq_len + 3) / 4) * 4) return MUI_ERR_INVALID_ARG;
  }
  PrefillParams p = {};
  p.q = (const uint16_t*)q_rotated;
  p.k_cache = (const uint16_t*)k_cache;
  p.v_cache = (const uint16_t*)v_cache;
  p.c_bs = cache_batch_stride; p.c_hs = cache_head_stride; p.c_ts = cache_token_stride;
  p.out = (uint16_t*)out;
  p.hq = n_q_heads; p.hkv = n_kv_heads; p.tokens = tokens; p.seq_len = seq_len; p.q_start = q_start;
  p.scale_log2 = kLog2e / sqrtf((float)head_dim);
  p.key_mask = (const uint16_t*)key_mask; p.mask_bs = mask_batch_stride;
  const bool masked = key_mask != nullptr;
  hipStream_t s = (hipStream_t)stream;
  // Long prompts with 1, 2, 4 or 8 query heads per KV head: K/V rows cross LDS once per 32 query
  // positions of the whole KV group. Short prompts keep the kernel that splits the key range of
  // 16 query positions over four waves (more workgroups, shorter chains) up to 256 tokens, while
  // its grid (32 heads x 16 tiles) is a single round of workgroups: both take 7-12 us there; at 272
  // tokens it is 15.8 us against 11.6 us.
  const int group = n_q_heads / n_kv_heads;
  const bool grouped = (group == 1 || group == 2 || group == 4 || group == 8) &&
                       (g_prefill_group_tokens > 0 ? tokens >= g_prefill_group_tokens : g_prefill_group_tokens == 0 && tokens > 256);
  if (grouped) {
    if (ceil_div(tokens, 16) > 65535) return MUI_ERR_UNSUPPORTED;  // position tiles are the grid's y
    // K / V rows straight into LDS where every cache row is 16-byte aligned
    const bool direct = g_prefill_attn_direct && ((((uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0) &&
                        ((cache_batch_stride | cache_head_stride | cache_token_stride) & 7) == 0;
#define MUI_PG_LAUNCH(TT, GG)                                                                          \
    do {                                                                                                 \
      const dim3 pg_grid(n_kv_heads * batch, ceil_div(tokens, 128 / (GG == 8 ? 4 : GG)));                 \
      if (direct) {                                                                                      \
        constexpr int kDirectLds = 2 * kPgTok * 2 * kHeadDim * 2; /* two stages of a K and a V tile */   \
        int st;                                                                                          \
        if (masked) st = launch_pg_direct(attn_prefill_group_kernel<TT, GG, true, true>, pg_grid, (GG == 8 ? 8 : 4) * kWave, kDirectLds, s, p); \
        else st = launch_pg_direct(attn_prefill_group_kernel<TT, GG, false, true>, pg_grid, (GG == 8 ? 8 : 4) * kWave, kDirectLds, s, p);       \
        if (st != MUI_OK) return st;                                                                     \
      } else if (masked) hipLaunchKernelGGL((attn_prefill_group_kernel<TT, GG, true>), pg_grid, dim3((GG == 8 ? 8 : 4) * kWave), 0, s, p); \
      else hipLaunchKernelGGL((attn_prefill_group_kernel<TT, GG, false>), pg_grid, dim3((GG == 8 ? 8 : 4) * kWave), 0, s, p);       \
    } while (0)
    if (dtype == MUI_DTYPE_F16) {
      if (group == 1) MUI_PG_LAUNCH(F16, 1); else if (group == 2) MUI_PG_LAUNCH(F16, 2);
      else if (group == 4) MUI_PG_LAUNCH(F16, 4); else MUI_PG_LAUNCH(F16, 8);
    } else {
      if (group == 1) MUI_PG_LAUNCH(BF16, 1); else if (group == 2) MUI_PG_LAUNCH(BF16, 2);
      else if (group == 4) MUI_PG_LAUNCH(BF16, 4); else MUI_PG_LAUNCH(BF16, 8);
    }
#undef MUI_PG_LAUNCH
    return launch_status();
  }
  if (ceil_div(tokens, 16) > 65535) return MUI_ERR_UNSUPPORTED;
  dim3 grid(n_q_heads * batch, ceil_div(tokens, 16));
  if (dtype == MUI_DTYPE_F16) {
    if (masked) hipLaunchKernelGGL((attn_prefill_mfma_kernel<F16, 4, true>), grid, dim3(4 * kWave), 0, s, p);
    else hipLaunchKernelGGL((attn_prefill_mfma_kernel<F16, 4, false>), grid, dim3(4 * kWave), 0, s, p);
  } else {
    if (masked) hipLaunchKernelGGL((attn_prefill_mfma_kernel<BF16, 4, true>), grid, dim3(4 * kWave), 0, s, p);
    else hipLaunchKernelGGL((attn_prefill_mfma_kernel<BF16, 4, false>), grid, dim3(4 * kWave), 0, s, p);
  }
  return launch_status();
}

extern "C" int mui_prefill_attention(mui_stream_t stream, int dtype, const void* q_rotated, const void* k_cache,
                                     const void* v_cache, long cache_batch_stride, long cache_head_stride,
                                     long cache_token_stride, int seq_len, int q_start, void* out, int batch,
                                     int n_q_heads, int n_kv_heads, int tokens, int head_dim) {
  return prefill_attention_impl(stream, dtype, q_rotated, k_cache, v_cache, cache_batch_stride, cache_head_stride,
                                cache_token_stride, seq_len, q_start, nullptr, 0, out, batch, n_q_heads, n_kv_heads,
                                tokens, head_dim);
}

extern "C" int mui_prefill_attention_masked(mui_stream_t stream, int dtype, const void* q_rotated, const void* k_cache,
                                            const void* v_cache, long cache_batch_stride, long cache_head_stride,
                                            long cache_token_stride, int seq_len, int q_start, const void* key_mask,
                                            long mask_batch_stride, void* out, int batch, int n_q_heads,
                                            int n_kv_heads, int tokens, int head_dim) {
  MUI_CHECK_ARG(key_mask);
  return prefill_attention_impl(stream, dtype, q_rotated, k_cache, v_cache, cache_batch_stride, cache_head_stride,
                                cache_token_stride, seq_len, q_start, key_mask, mask_batch_stride, out, batch,
                                n_q_heads, n_kv_heads, tokens, head_dim);
}
