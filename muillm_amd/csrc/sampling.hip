// Greedy token selection: argmax over each row of a [rows, vocab] 16-bit logits matrix,
// lowest index on ties. One workgroup of 1024 threads per row, 128-bit loads, wave reduce on
// (value, index) pairs, LDS across the 16 waves. It keeps the decode loop free of
// library reductions (which may record memset nodes when captured into a HIP graph).
// Reference counterpart: the greedy branch of the sampling loop, torch.argmax at
// muillm/sampling/generation.py:330-335.
#include "common.cuh"

namespace mui {

constexpr int kArgmaxThreads = 1024;

__device__ __forceinline__ void take_better(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

// argmax over part `part` of `n_parts` of one row by the whole workgroup (the 16-byte chunks are
// dealt out in contiguous ranges; the elements behind the last whole chunk go to the last part).
// Valid on thread 0: the largest value and its lowest index, or index 0x7fffffff when no element
// of the part is greater than -inf (NaN never wins).
template <typename T>
__device__ __forceinline__ void slice_argmax(const uint16_t* row, bool vec, int vocab, int part, int n_parts,
                                             float& best_out, int& best_i_out) {
  __shared__ float sv[kArgmaxThreads / kWave];
  __shared__ int si[kArgmaxThreads / kWave];
  const int t = threadIdx.x;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  const int nvec = vec ? (vocab >> 3) : 0;
  const int per = (nvec + n_parts - 1) / n_parts;
  const int c_begin = part * per;
  const int c_end = c_begin + per < nvec ? c_begin + per : nvec;
  // four chunks per thread requested together: one load at a time made the scan of a 128k-entry
  // row a chain of 16 memory latencies (12.5 us; 4 in flight: about a third of that)
  constexpr int kInFlight = 4;
  for (int c0 = c_begin + t; c0 < c_end; c0 += kArgmaxThreads * kInFlight) {
    u32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int c = c0 + u * kArgmaxThreads;
      v[u] = ld16(row + ((c < c_end ? c : c0) << 3));  // clamped, not branched around
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int c = c0 + u * kArgmaxThreads;
      float f[8];
      unpack8<T>(v[u], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // NaN never wins; strict > keeps the lowest index inside a thread's ascending scan
        if (c < c_end && f[i] > best) { best = f[i]; best_i = (c << 3) + i; }
      }
    }
  }
  if (part == n_parts - 1) {
    for (int i = (nvec << 3) + t; i < vocab; i += kArgmaxThreads) {
      const float f = T::one(row[i]);
      if (f > best) { best = f; best_i = i; }
    }
  }
  // wave reduce with shuffles over (value, index)
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off);
    const int oi = __shfl_xor(best_i, off);
    take_better(best, best_i, ov, oi);
  }
  if ((t & (kWave - 1)) == 0) { sv[t >> 6] = best; si[t >> 6] = best_i; }
  __syncthreads();
  if (t == 0) {
    for (int w = 1; w < kArgmaxThreads / kWave; ++w) take_better(best, best_i, sv[w], si[w]);
  }
  best_out = best;
  best_i_out = best_i;
}

// argmax of one row by the whole workgroup; the result is valid on thread 0
template <typename T>
__device__ __forceinline__ int row_argmax(const uint16_t* row, bool vec, int vocab) {
  float best;
  int best_i;
  slice_argmax<T>(row, vec, vocab, 0, 1, best, best_i);
  return best_i == 0x7fffffff ? 0 : best_i;
}

template <typename T>
__global__ void __launch_bounds__(kArgmaxThreads) argmax_rows_kernel(const uint16_t* logits, long row_stride,
                                                                    int64_t* out, int vocab) {
  const bool vec = ((row_stride & 7) == 0) && ((((uintptr_t)logits) & 15u) == 0);
  const int best_i = row_argmax<T>(logits + (long)blockIdx.x * row_stride, vec, vocab);
  if (threadIdx.x == 0) out[blockIdx.x] = best_i;
}

// Greedy choice plus everything the decode loop does with it, for batch row blockIdx.x:
//   tok = argmax(logits[b]); finished rows emit pad_token instead (eos criterion)
//   tokens_out[b, step[b]] = tok; next_ids[b] = tok; position_ids[b] += 1; step[b] += 1
//   cache_position[0] += 1 (row 0 only); unfinished[b] &= tok is no eos and steps remain
// Every row owns its own counters, so the workgroups never read what another one writes.
struct GreedyParams {
  const uint16_t* logits; long row_stride; int vocab;
  int64_t* next_ids;        // [B]
  int64_t* position_ids;    // [B] or null
  int64_t* cache_position;  // [1] or null
  int64_t* step;            // [B]
  int64_t* tokens_out; long tokens_stride; int max_steps;  // [B, >= max_steps]
  int64_t* unfinished;      // [B] or null
  const int64_t* eos_ids; int n_eos; long pad_token;
  // optional: the chosen token's embedding row, for the next step's first layer
  const uint16_t* embed_table; long embed_stride; uint16_t* embed_out; int embed_dim;  // out [B, embed_dim] dense
};

// what thread 0 does with row b's choice
__device__ __forceinline__ int64_t greedy_finish(const GreedyParams& p, int b, int best_i) {
  int64_t tok = best_i;
  const bool was_unfinished = p.unfinished ? (p.unfinished[b] != 0) : true;
  if (p.unfinished && p.n_eos > 0 && !was_unfinished) tok = p.pad_token;
  const int64_t st = p.step[b];
  if (st >= 0 && st < p.max_steps) p.tokens_out[(long)b * p.tokens_stride + st] = tok;
  p.next_ids[b] = tok;
  if (p.position_ids) p.position_ids[b] += 1;
  p.step[b] = st + 1;
  if (b == 0 && p.cache_position) p.cache_position[0] += 1;
  if (p.unfinished) {
    bool unfinished = was_unfinished && (st + 1 < p.max_steps);
    for (int i = 0; i < p.n_eos; ++i) unfinished = unfinished && (tok != p.eos_ids[i]);
    p.unfinished[b] = unfinished ? 1 : 0;
  }
  return tok;
}

// The workgroup that finished row b hands the token to all its threads (thread 0 calls with the
// token, the others with anything) and copies that row of the embedding table to embed_out[b]:
// the embedding gather at the head of the next decode step, a launch of two dependent loads
// (token id, then the row), becomes the tail of this one. `mine` is uniform per workgroup.
__device__ __forceinline__ void gather_embedding(const GreedyParams& p, int b, int64_t tok, bool mine) {
  __shared__ long long tok_s;
  if (p.embed_table == nullptr) return;  // uniform
  if (threadIdx.x == 0) tok_s = mine ? tok : -1;
  __syncthreads();
  const long long tk = tok_s;
  if (tk < 0) return;
  const uint16_t* src = p.embed_table + tk * p.embed_stride;
  uint16_t* dst = p.embed_out + (long)b * p.embed_dim;
  const bool vec = ((p.embed_dim | p.embed_stride) & 7) == 0 && (((uintptr_t)p.embed_table | (uintptr_t)p.embed_out) & 15u) == 0;
  if (vec) {
    for (int c = threadIdx.x; c < (p.embed_dim >> 3); c += kArgmaxThreads) *(u32x4*)(dst + (c << 3)) = ld16(src + (c << 3));
  } else {
    for (int i = threadIdx.x; i < p.embed_dim; i += kArgmaxThreads) dst[i] = src[i];
  }
}

template <typename T>
__global__ void __launch_bounds__(kArgmaxThreads) greedy_advance_kernel(const GreedyParams p) {
  const int b = blockIdx.x;
  const bool vec = ((p.row_stride & 7) == 0) && ((((uintptr_t)p.logits) & 15u) == 0);
  const int best_i = row_argmax<T>(p.logits + (long)b * p.row_stride, vec, p.vocab);
  int64_t tok = 0;
  if (threadIdx.x == 0) tok = greedy_finish(p, b, best_i);
  gather_embedding(p, b, tok, true);
}

// The same with the scan of a row dealt out to gridDim.x workgroups (one workgroup pulls a 128k-entry
// row through a single CU's load path: 9.4 us). Every workgroup folds its candidate into the row's
// word of the workspace -- (order-preserving image of the value, ~index) under a 64-bit atomic max,
// so the largest value wins and among equal values the lowest index, as in the single-workgroup
// scan -- and counts itself in; whoever arrives last reads the word, returns word and counter to
// zero and finishes the step. Agent-scope atomics; nobody waits for anybody.
template <typename T>
__global__ void __launch_bounds__(kArgmaxThreads) greedy_advance_parts_kernel(const GreedyParams p,
                                                                             unsigned long long* best_word,
                                                                             unsigned* arrived) {
  const int part = blockIdx.x, n_parts = gridDim.x, b = blockIdx.y;
  float best;
  int best_i;
  slice_argmax<T>(p.logits + (long)b * p.row_stride, true, p.vocab, part, n_parts, best, best_i);
  int64_t tok = 0;
  bool last = false;
  if (threadIdx.x == 0) {
    if (best_i != 0x7fffffff) {
      const uint32_t u = __float_as_uint(best + 0.f);  // -0 counts as +0, as it does under ==
      const uint32_t image = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
      const unsigned long long key = ((unsigned long long)image << 32) | (0xffffffffu - (uint32_t)best_i);
      __hip_atomic_fetch_max(best_word + b, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // release: the candidate is visible device-wide before the count goes up; acquire: whoever sees
    // the full count sees every candidate (the memory model's own ordering, not a property of one
    // chip generation's write acknowledgements)
    const unsigned before = __hip_atomic_fetch_add(arrived + b, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    last = before + 1 == (unsigned)n_parts;
    if (last) {
      const unsigned long long w = __hip_atomic_load(best_word + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(best_word + b, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(arrived + b, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      tok = greedy_finish(p, b, w ? (int)(0xffffffffu - (uint32_t)(w & 0xffffffffu)) : 0);
    }
  }
  gather_embedding(p, b, tok, last);  // the last arriver's workgroup copies, the others leave
}

}  // namespace mui

using namespace mui;

extern "C" int mui_argmax(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                          int64_t* out_index, int rows, int vocab) {
  MUI_CHECK_ARG(logits && out_index && rows > 0 && vocab > 0 && row_stride >= vocab);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((argmax_rows_kernel<F16>), dim3(rows), dim3(kArgmaxThreads), 0, s,
                       (const uint16_t*)logits, row_stride, out_index, vocab);
  else if (dtype == MUI_DTYPE_BF16)
    hipLaunchKernelGGL((argmax_rows_kernel<BF16>), dim3(rows), dim3(kArgmaxThreads), 0, s,
                       (const uint16_t*)logits, row_stride, out_index, vocab);
  else
    return MUI_ERR_INVALID_ARG;
  return launch_status();
}

extern "C" size_t mui_greedy_workspace_bytes(int rows) { return rows > 0 ? (size_t)rows * 16 : 0; }

extern "C" int mui_greedy_advance_ws(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                                     int rows, int vocab, int64_t* next_ids, int64_t* position_ids,
                                     int64_t* cache_position, int64_t* step, int64_t* tokens_out,
                                     long tokens_stride, int max_steps, int64_t* unfinished,
                                     const int64_t* eos_ids, int n_eos, long pad_token, void* workspace,
                                     size_t workspace_bytes, const void* embed_table, long embed_row_stride,
                                     void* embed_out, int embed_dim) {
  MUI_CHECK_ARG(logits && next_ids && step && tokens_out && rows > 0 && vocab > 0 && row_stride >= vocab);
  MUI_CHECK_ARG((embed_table == nullptr) == (embed_out == nullptr));
  MUI_CHECK_ARG(!embed_table || (embed_dim > 0 && embed_row_stride >= embed_dim && pad_token >= 0 && pad_token < vocab));
  MUI_CHECK_ARG(max_steps >= 0 && tokens_stride >= max_steps && n_eos >= 0 && (n_eos == 0 || eos_ids));
  MUI_CHECK_ARG(workspace || workspace_bytes == 0);
  if (dtype != MUI_DTYPE_F16 && dtype != MUI_DTYPE_BF16) return MUI_ERR_INVALID_ARG;
  if (rows > 65535) return MUI_ERR_UNSUPPORTED;
  GreedyParams p = {};
  p.logits = (const uint16_t*)logits; p.row_stride = row_stride; p.vocab = vocab;
  p.next_ids = next_ids; p.position_ids = position_ids; p.cache_position = cache_position;
  p.step = step; p.tokens_out = tokens_out; p.tokens_stride = tokens_stride; p.max_steps = max_steps;
  p.unfinished = unfinished; p.eos_ids = eos_ids; p.n_eos = n_eos; p.pad_token = pad_token;
  p.embed_table = (const uint16_t*)embed_table; p.embed_stride = embed_row_stride;
  p.embed_out = (uint16_t*)embed_out; p.embed_dim = embed_dim;
  hipStream_t s = (hipStream_t)stream;
  // one workgroup per 1024 chunks of 16 bytes (one load per thread), 32 at most; rows that cannot be
  // read in 16-byte chunks, rows of a single part and calls without a workspace take one workgroup
  const bool vec = ((row_stride & 7) == 0) && ((((uintptr_t)logits) & 15u) == 0);
  int parts = vec ? ((vocab >> 3) + kArgmaxThreads - 1) / kArgmaxThreads : 1;
  parts = parts > 32 ? 32 : parts;
  if (parts > 1 && workspace && (((uintptr_t)workspace) & 7u) == 0 && workspace_bytes >= mui_greedy_workspace_bytes(rows)) {
    unsigned long long* best_word = (unsigned long long*)workspace;
    unsigned* arrived = (unsigned*)(best_word + rows);
    if (dtype == MUI_DTYPE_F16)
      hipLaunchKernelGGL((greedy_advance_parts_kernel<F16>), dim3(parts, rows), dim3(kArgmaxThreads), 0, s, p, best_word, arrived);
    else
      hipLaunchKernelGGL((greedy_advance_parts_kernel<BF16>), dim3(parts, rows), dim3(kArgmaxThreads), 0, s, p, best_word, arrived);
    return launch_status();
  }
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((greedy_advance_kernel<F16>), dim3(rows), dim3(kArgmaxThreads), 0, s, p);
  else
    hipLaunchKernelGGL((greedy_advance_kernel<BF16>), dim3(rows), dim3(kArgmaxThreads), 0, s, p);
  return launch_status();
}

extern "C" int mui_greedy_advance(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                                  int rows, int vocab, int64_t* next_ids, int64_t* position_ids,
                                  int64_t* cache_position, int64_t* step, int64_t* tokens_out,
                                  long tokens_stride, int max_steps, int64_t* unfinished,
                                  const int64_t* eos_ids, int n_eos, long pad_token) {
  return mui_greedy_advance_ws(stream, dtype, logits, row_stride, rows, vocab, next_ids, position_ids, cache_position,
                               step, tokens_out, tokens_stride, max_steps, unfinished, eos_ids, n_eos, pad_token,
                               nullptr, 0, nullptr, 0, nullptr, 0);
}
