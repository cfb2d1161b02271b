// Generation-loop helpers that keep a decode step on the device: embedding gather and
// sync-free sampling.
//
// Reference counterparts: the embedding kernels (csrc/embedding/embedding_xx16_kernels.cu:26-112,
// dispatched from csrc/embedding/embedding.cu:31-100) and the sampling branch of the generation
// loop, softmax -> muillm_multinomial_sample_one_no_sync = argmax(probs / q), q ~ Exp(1)
// (muillm/sampling/multinomial.py:4-6, muillm/sampling/generation.py:330-404), followed by
// muillm_add_tokens_check_finished (csrc/generation/generation.cu:29-113).
//
// Sampling here is one kernel per step: argmax_v(logit_v / temperature - log q_v) is the same
// draw as argmax(softmax(logits / temperature) / q) without materialising the probabilities.
// The exponential variates come from a counter-based generator (Philox4x32-10 keyed by the
// seed, counter = (vocab index / 4, row, step)), so a captured step replays with fresh noise
// as long as the device-side step counter advances, and a host can reproduce every draw.
#include "common.cuh"

namespace mui {

// ---------------------------------------------------------------------------------------
// embedding gather: out[t, :] = table[ids[t], :]; one workgroup per token, 16 bytes per thread
// ---------------------------------------------------------------------------------------
template <typename IDX>
__global__ void __launch_bounds__(256) embedding_kernel(const uint16_t* table, long row_pitch, const IDX* ids,
                                                        uint16_t* out, int dim, int vocab) {
  const long tok = blockIdx.x;
  long id = (long)ids[tok];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // clamp instead of reading out of bounds
  const uint16_t* src = table + id * row_pitch;
  uint16_t* dst = out + tok * dim;
  const bool vec = ((dim & 7) == 0) && ((row_pitch & 7) == 0) && (((uintptr_t)table | (uintptr_t)out) & 15u) == 0;
  if (vec) {
    for (int c = threadIdx.x; c < (dim >> 3); c += blockDim.x) *(u32x4*)(dst + (c << 3)) = ld16(src + (c << 3));
  } else {
    for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = src[i];
  }
}

// ---------------------------------------------------------------------------------------
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11)
// ---------------------------------------------------------------------------------------
struct Philox4 { uint32_t x, y, z, w; };

__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                 uint32_t k0, uint32_t k1) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(M0, c0), lo0 = M0 * c0;
    const uint32_t hi1 = __umulhi(M1, c2), lo1 = M1 * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += W0; k1 += W1;
  }
  return Philox4{c0, c1, c2, c3};
}

// 32 random bits -> uniform in (0, 1]: (bits >> 8 + 1) * 2^-24, then -log(-log u) is finite or +inf-free
__device__ __forceinline__ float gumbel_from_bits(uint32_t bits) {
  const float u = ((float)(bits >> 8) + 1.0f) * 5.9604644775390625e-08f;  // (0, 1]
  const float q = -__logf(u);                                             // Exp(1) variate in [0, 16.7]
  return -__logf(fmaxf(q, 1e-30f));                                       // -log q
}

constexpr int kSampleThreads = 1024;

struct SampleParams {
  const uint16_t* logits; long row_stride; int vocab;
  float inv_temperature;
  uint64_t seed;
  int64_t* next_ids; int64_t* position_ids; int64_t* cache_position; int64_t* step;
  int64_t* tokens_out; long tokens_stride; int max_steps;
  int64_t* unfinished; const int64_t* eos_ids; int n_eos; long pad_token;
};

__device__ __forceinline__ void take_better_s(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

template <typename T>
__global__ void __launch_bounds__(kSampleThreads) sample_advance_kernel(const SampleParams p) {
  __shared__ float sv[kSampleThreads / kWave];
  __shared__ int si[kSampleThreads / kWave];
  const int b = blockIdx.x, t = threadIdx.x;
  const uint16_t* row = p.logits + (long)b * p.row_stride;
  const uint32_t st_lo = (uint32_t)p.step[b];
  const uint32_t k0 = (uint32_t)p.seed, k1 = (uint32_t)(p.seed >> 32);
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  // groups of 4 consecutive vocabulary entries share one Philox block
  const int n4 = (p.vocab + 3) >> 2;
  for (int c = t; c < n4; c += kSampleThreads) {
    const Philox4 r = philox4x32_10((uint32_t)c, (uint32_t)b, st_lo, 0u, k0, k1);
    const uint32_t bits[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int v = (c << 2) + j;
      if (v < p.vocab) {
        const float lg = T::one(row[v]);
        // -inf logits (filtered by top-k / top-p processors) can never win; NaN neither
        const float s = fmaf(lg, p.inv_temperature, gumbel_from_bits(bits[j]));
        if (s > best) { best = s; best_i = v; }
      }
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(best, off);
    const int oi = __shfl_xor(best_i, off);
    take_better_s(best, best_i, ov, oi);
  }
  if ((t & (kWave - 1)) == 0) { sv[t >> 6] = best; si[t >> 6] = best_i; }
  __syncthreads();
  if (t != 0) return;
  for (int w = 1; w < kSampleThreads / kWave; ++w) take_better_s(best, best_i, sv[w], si[w]);
  int64_t tok = best_i == 0x7fffffff ? 0 : best_i;
  // bookkeeping identical to the greedy variant
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
}

}  // namespace mui

using namespace mui;

extern "C" int mui_embedding(mui_stream_t stream, int dtype, const void* table, long row_pitch,
                             const void* ids, int ids_are_int32, void* out, int n_tokens, int dim,
                             int vocab) {
  MUI_CHECK_ARG(table && ids && out && n_tokens > 0 && dim > 0 && vocab > 0 && row_pitch >= dim);
  MUI_CHECK_ARG(dtype == MUI_DTYPE_F16 || dtype == MUI_DTYPE_BF16);
  hipStream_t s = (hipStream_t)stream;
  if (ids_are_int32)
    hipLaunchKernelGGL((embedding_kernel<int32_t>), dim3(n_tokens), dim3(256), 0, s, (const uint16_t*)table,
                       row_pitch, (const int32_t*)ids, (uint16_t*)out, dim, vocab);
  else
    hipLaunchKernelGGL((embedding_kernel<int64_t>), dim3(n_tokens), dim3(256), 0, s, (const uint16_t*)table,
                       row_pitch, (const int64_t*)ids, (uint16_t*)out, dim, vocab);
  return launch_status();
}

extern "C" int mui_sample_advance(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                                  int rows, int vocab, float temperature, uint64_t seed,
                                  int64_t* next_ids, int64_t* position_ids, int64_t* cache_position,
                                  int64_t* step, int64_t* tokens_out, long tokens_stride, int max_steps,
                                  int64_t* unfinished, const int64_t* eos_ids, int n_eos, long pad_token) {
  MUI_CHECK_ARG(logits && next_ids && step && tokens_out && rows > 0 && vocab > 0 && row_stride >= vocab);
  MUI_CHECK_ARG(max_steps >= 0 && tokens_stride >= max_steps && n_eos >= 0 && (n_eos == 0 || eos_ids));
  MUI_CHECK_ARG(temperature > 0.f);
  SampleParams p = {};
  p.logits = (const uint16_t*)logits; p.row_stride = row_stride; p.vocab = vocab;
  p.inv_temperature = 1.0f / temperature; p.seed = seed;
  p.next_ids = next_ids; p.position_ids = position_ids; p.cache_position = cache_position;
  p.step = step; p.tokens_out = tokens_out; p.tokens_stride = tokens_stride; p.max_steps = max_steps;
  p.unfinished = unfinished; p.eos_ids = eos_ids; p.n_eos = n_eos; p.pad_token = pad_token;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MUI_DTYPE_F16)
    hipLaunchKernelGGL((sample_advance_kernel<F16>), dim3(rows), dim3(kSampleThreads), 0, s, p);
  else if (dtype == MUI_DTYPE_BF16)
    hipLaunchKernelGGL((sample_advance_kernel<BF16>), dim3(rows), dim3(kSampleThreads), 0, s, p);
  else
    return MUI_ERR_INVALID_ARG;
  return launch_status();
}
