/*
 * muillm_amd.h -- C ABI of libmuillm_amd.so: muiLLM's decode-time hot path as
 * hand-written HIP kernels for AMD MI355X (gfx950).
 *
 * Every entry point
 *   - takes plain device pointers, sizes and a HIP stream (as void*), no framework types;
 *   - enqueues asynchronously on that stream and never synchronises or allocates;
 *   - owns nothing: outputs and scratch are caller-allocated;
 *   - returns MUI_OK (0) or a negative MUI_ERR_* code (mui_status_string() names it);
 *   - validates shapes/alignment on the host before launching anything;
 *   - keeps no state between calls (the sweep aids that do are declared apart, in
 *     muillm_amd_tune.h).
 *
 * The comment above each declaration names the entry of the reference's pybind11
 * module `muillm_ext` (Epliz/muiLLM, csrc/module.cpp) that it stands in for.
 *
 * Tensors are dense row-major unless a stride argument says otherwise. "16-bit type"
 * means fp16 or bf16 selected by the `dtype` argument; all arithmetic is fp32 with a
 * single rounding at the store.
 */
#ifndef MUILLM_AMD_H
#define MUILLM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* bumped whenever a struct below changes layout or an entry point changes its arguments;
 * mui_abi_version() returns the value the library was built with */
#define MUI_ABI_VERSION 3

/* status codes (reference: TORCH_CHECK exceptions, csrc/linear/linear.cu:72-74;
 * muillm_error_t, csrc/base.h:4-7) */
#define MUI_OK 0
#define MUI_ERR_INVALID_ARG (-1) /* null pointer, non-positive size, bad enum */
#define MUI_ERR_UNSUPPORTED (-2) /* shape outside what the kernels cover */
#define MUI_ERR_LAUNCH (-3)      /* hipGetLastError() after the launch was not hipSuccess */
#define MUI_ERR_ALIGNMENT (-4)   /* a pointer or row pitch is not 16-byte aligned */
#define MUI_ERR_DEVICE (-5)      /* device query failed / not a gfx950 device */
#define MUI_ERR_SCRATCH_LIMIT (-6) /* needs more scratch than the library's built-in array holds */

#define MUI_DTYPE_F16 0
#define MUI_DTYPE_BF16 1

/* largest token batch of the weight-streaming decode kernels (and of mui_decoder_stack_step); the
 * linear entry points take more tokens than this through their tiled GEMM */
#define MUI_MAX_TOKENS 16

typedef void* mui_stream_t; /* a hipStream_t; NULL is the default stream */

/* What muillm_engine_init() (csrc/engine.cpp:3-26, csrc/gpu_info.cpp:7-69) records per
 * GPU, for the current device only. */
typedef struct mui_device_info {
  int device;              /* HIP ordinal */
  int compute_units;       /* 256 on MI355X */
  int wave_size;           /* 64 */
  int simd_lanes;          /* compute_units * 4 SIMDs * 16 lanes */
  int lds_bytes_per_block; /* max LDS per workgroup */
  int l2_bytes;
  int clock_khz;
  int is_gfx950;           /* 1 when gcnArchName starts with "gfx950" */
  uint64_t hbm_bytes;
  char arch[64];           /* gcnArchName */
} mui_device_info_t;

int mui_abi_version(void);
const char* mui_status_string(int status);

/* muillm_engine_init (csrc/module.cpp:283). Fills `out` for HIP device `device`. */
int mui_device_info(int device, mui_device_info_t* out);

/* ------------------------------------------------------------------------------------
 * Linear family
 * ---------------------------------------------------------------------------------- */

/* muillm_linear_forward / muillm_linear_module_forward (csrc/module.cpp:178,312;
 * csrc/linear/linear.cu:76-208; kernels csrc/linear/linear_fp16_kernels.cu:163-626).
 *
 *   y[t, n] = (sum_k W[n, k] * xn[t, k]) * mul_bias[n] + add_bias[n] + residual[t, n]
 *   xn[t, :] = norm_weights ? norm_weights * x[t, :] * rsqrt(mean(x[t, :]^2) + epsilon) : x[t, :]
 *
 * W is [n_out, k_in] with row pitch `w_pitch` elements (w_pitch == k_in when dense);
 * x is [tokens, k_in]; y, residual are [tokens, n_out]; norm_weights is [k_in];
 * mul_bias, add_bias are [n_out]. norm_weights, mul_bias, add_bias, residual may be NULL.
 * tokens >= 1: up to MUI_MAX_TOKENS the weight-streaming decode kernels (weights read once per
 * call), beyond that a tiled matrix-core GEMM (weights read once per 128 tokens) -- the reference
 * hands every multi-token call to the framework's GEMM after a separate RMSNorm kernel
 * (csrc/modules/linear_module.cpp:57-79). epsilon is added to the mean (HuggingFace convention).
 * Requirements: k_in % 8 == 0, W and x 16-byte aligned, w_pitch % 8 == 0.
 * y may alias residual. */
int mui_linear(mui_stream_t stream, int dtype, const void* weights, long w_pitch,
               const void* x, const void* norm_weights, float epsilon,
               const void* mul_bias, const void* add_bias, const void* residual,
               void* y, int n_out, int k_in, int tokens);

/* mui_linear with a scratch buffer for prompts. No counterpart in the reference (which allocates
 * inside its calls, csrc/linear/linear.cu:178-189). With more than MUI_MAX_TOKENS tokens on a matrix of
 * few rows and a long K (the down projection up to about 256 tokens) one workgroup per output tile
 * would leave most of the chip idle: given a workspace, K is shared between several workgroups per
 * tile, which exchange fp32 partial tiles through it (4096 x 14336 at 64 tokens: 44 instead of
 * 59 us, at 256 tokens 57 instead of 109 us). workspace: mui_linear_workspace_bytes() bytes of device memory, 256-byte aligned,
 * zero-filled ONCE by the caller before its first use (the kernels leave its counters at zero);
 * calls that may overlap on the device (different streams) need a workspace each. workspace may
 * be NULL (workspace_bytes 0): then, or when norm_weights is given, or for shapes that do not
 * profit, the call is mui_linear. Results do not depend on which workgroup arrives last (the
 * partials are added in a fixed order). */
size_t mui_linear_workspace_bytes(void);
int mui_linear_ws(mui_stream_t stream, int dtype, const void* weights, long w_pitch,
                  const void* x, const void* norm_weights, float epsilon,
                  const void* mul_bias, const void* add_bias, const void* residual,
                  void* y, int n_out, int k_in, int tokens, void* workspace, size_t workspace_bytes);

/* muillm_rmsnorm_forward (csrc/module.cpp:251; csrc/norm/rmsnorm.cu:31-85; kernel
 * csrc/norm/rmsnorm_fp16_kernels.cu:35-126).
 *   y[r, :] = weights * x[r, :] * rsqrt(mean(x[r, :]^2) + epsilon), rows r < rows.
 * Any k >= 1; 16-byte aligned rows take the vector path. y may alias x. */
int mui_rmsnorm(mui_stream_t stream, int dtype, const void* weights, const void* x,
                float epsilon, void* y, int rows, int k);

/* First half of muillm_gateupsilu_forward (csrc/module.cpp:182; csrc/ffn/gateup.cu:88-219;
 * kernels csrc/ffn/gateup_fp16_kernels.cu:160-604):
 *   h[t, n] = silu(sum_k G[n, k] xn[t, k]) * (sum_k U[n, k] xn[t, k])
 * G and U are [n_inter, k_in] with a common row pitch `gu_pitch` elements. They may be two
 * separate dense matrices (gu_pitch == k_in) or the two interleaved halves of one packed
 * [n_inter, 2, k_in] buffer (up == gate + k_in, gu_pitch == 2 * k_in), which is the layout
 * the Python layer repacks to. xn and the token range as in mui_linear. h is [tokens, n_inter].
 * The second half (down projection + residual) is mui_linear with residual. */
int mui_gateup_silu(mui_stream_t stream, int dtype, const void* gate, const void* up,
                    long gu_pitch, const void* x, const void* norm_weights, float epsilon,
                    void* h, int n_inter, int k_in, int tokens);

/* Activation step of the unfused MLP route for prompts longer than MUI_MAX_TOKENS tokens
 * (muillm/modules/gateupdownmlp.py:343-359: two matmuls, SiLU, multiply): with the gate and up
 * rows interleaved in one buffer, one matmul yields gate_up [rows, n, 2] and this call
 * computes out[r, i] = silu(gate_up[r, i, 0]) * gate_up[r, i, 1] (fp32 math, one rounding).
 * n % 8 == 0; 16-byte aligned buffers. */
int mui_silu_mul_interleaved(mui_stream_t stream, int dtype, const void* gate_up, void* out,
                             long rows, int n);

/* ------------------------------------------------------------------------------------
 * int8 weight-only family
 * ---------------------------------------------------------------------------------- */

/* muillm_int8_linear_forward (csrc/module.cpp:31-54,181; csrc/int8_linear_kernels.cu:703-785)
 * on the symmetric per-output-channel format of the decode benchmarks:
 *   weights_i8 int8 [n_out, k_in] (row pitch w_pitch bytes), scales 16-bit [n_out],
 *   w[n, k] = q[n, k] * scales[n];   y = W xn + add_bias + residual   (xn as in mui_linear).
 * The reference passes the residual through add_bias (int8linear.py:53-57); here both exist.
 * Any tokens >= 1 (as mui_linear: beyond MUI_MAX_TOKENS the tiled GEMM converts the codes on their
 * way to LDS; the reference dequantises the whole matrix and calls the framework's GEMM,
 * muillm/modules/quantized/int8linear.py:279-293).
 * Requirements: k_in % 16 == 0, k_in <= 16384, 16-byte aligned rows. */
int mui_int8_linear(mui_stream_t stream, int dtype, const void* weights_i8, long w_pitch,
                    const void* scales, const void* x, const void* norm_weights, float epsilon,
                    const void* add_bias, const void* residual, void* y, int n_out, int k_in,
                    int tokens);

/* muillm_int8_gateupsilu_forward (csrc/module.cpp:248; csrc/int8_gateup_kernels.cu:871-940),
 * per-channel format. gate/up are int8 [n_inter, k_in] sharing the row pitch gu_pitch (bytes):
 * two dense matrices, or the two halves of a row-interleaved [n_inter, 2, k_in] buffer
 * (up == gate + k_in, gu_pitch == 2 * k_in). Scale of row n: gate_scales[n * scale_stride],
 * up_scales[n * scale_stride] (scale_stride 2 for an interleaved [n_inter, 2] scale buffer).
 *   h[t, n] = silu(sg[n] * Gq[n,:] . xn[t]) * (su[n] * Uq[n,:] . xn[t]) */
int mui_int8_gateup_silu(mui_stream_t stream, int dtype, const void* gate_i8, const void* up_i8,
                         long gu_pitch, const void* gate_scales, const void* up_scales,
                         long scale_stride, const void* x, const void* norm_weights, float epsilon,
                         void* h, int n_inter, int k_in, int tokens);

/* muillm_int8_linear_forward on the reference's own RTN format
 * (muillm/quantization/rtnquantizer.py:49-88): weights_u8 uint8 [n_out, k_in],
 * scales_min_vals 16-bit [n_out * G, 2] = (scale, min) per group of 2^group_size_shift
 * inputs, w = u8 * scale + min. Requirements as above plus group size >= 16. Any tokens >= 1:
 * beyond MUI_MAX_TOKENS the tiled GEMM turns every chunk of codes into u8 * scale + min, rounded
 * once to the 16-bit type -- the values mui_int8_group_dequantize writes -- on its way to LDS. */
int mui_int8_group_linear(mui_stream_t stream, int dtype, const void* weights_u8, long w_pitch,
                          const void* scales_min_vals, int group_size_shift, const void* x,
                          const void* norm_weights, float epsilon, const void* add_bias,
                          const void* residual, void* y, int n_out, int k_in, int tokens);

/* muillm_int8_gateupsilu_forward on the reference's RTN format. gate/up rows share gu_pitch
 * (bytes); the (scale, min) pairs of row n start at gate_smv + n * smv_pitch and
 * up_smv + n * smv_pitch (16-bit elements; 2 * G when dense, 4 * G when row-interleaved).
 * Any tokens >= 1, as mui_int8_group_linear. */
int mui_int8_group_gateup_silu(mui_stream_t stream, int dtype, const void* gate_u8,
                               const void* up_u8, long gu_pitch, const void* gate_smv,
                               const void* up_smv, long smv_pitch, int group_size_shift,
                               const void* x, const void* norm_weights, float epsilon, void* h,
                               int n_inter, int k_in, int tokens);

/* The reference packs gate and up per element: gate_up_weights uint8 [n_inter, k_in, 2] and
 * gate_up_scales_min_vals 16-bit [n_inter * G, 2, 2] (group, gate|up, scale|min)
 * (muillm/modules/quantized/int8gateupdownmlp.py:211-230; read that way by
 * csrc/int8_gateup_kernels.cu:255-296). The kernels here stream row-interleaved buffers,
 * [n_inter, 2, k_in] and [n_inter, 2, G, 2]. This call converts the first form into the second,
 * once per weight (out of place; smv_* may both be NULL to convert only the codes), so that
 * tensors made by the reference's Python classes can be handed to mui_int8_group_gateup_silu /
 * mui_int8_group_dequantize. k_in % 16 == 0, group size >= 16. */
int mui_int8_repack_gateup(mui_stream_t stream, const void* gate_up_nk2, const void* smv_ng22,
                           int group_size_shift, void* gate_up_n2k, void* smv_n2g2, int n_inter,
                           int k_in);

/* Dense dequantisation of the per-channel format (the non-single-token branch of
 * muillm/modules/quantized/int8linear.py:279-293): out[n, k] = T(float(q[n,k]) * float(s[n])),
 * bit-identical to torch's q.to(T) * s[:, None]. scale of row n at scales[n * scale_stride]. */
int mui_int8_dequantize(mui_stream_t stream, int dtype, const void* weights_i8, long w_pitch,
                        const void* scales, long scale_stride, void* out, long out_pitch, int n,
                        int k);

/* muillm_int8_dequantize_forward (csrc/module.cpp:180; csrc/int8_dequantization_kernel.cu:50-59,156-193):
 * out[n, k] = T(fma(float(u8), float(scale_g), float(min_g))). */
int mui_int8_group_dequantize(mui_stream_t stream, int dtype, const void* weights_u8, long w_pitch,
                              const void* scales_min_vals, long smv_pitch, int group_size_shift,
                              void* out, long out_pitch, int n, int k);

/* ------------------------------------------------------------------------------------
 * RoPE, static KV cache, decode attention (head_dim 128; any whole number of query heads per KV
 * head: 1..8 read K/V once per KV head, other ratios once per query head)
 *
 * Common conventions: q/k/v inputs and the cache have unit inner stride; all other strides
 * are in elements. cos/sin tables are fp32 [rope_rows, rope_row_stride] with
 * rope_row_stride >= head_dim/2 and column f (f < head_dim/2) holding cos/sin(pos * inv_freq[f])
 * (the first half of the reference's cos_cached/sin_cached rows,
 * muillm/modules/attention/rotaryembedding.py:313-337); rotation is the HF rotate-half form
 * q' = q*cos + rotate_half(q)*sin in fp32, rounded once. position_ids / cache_position are
 * int64 device arrays like the reference's (csrc/rope/rotary.cu:209-211). Positions are read on
 * the device, so the table height rope_rows travels with the tables: a position outside
 * [0, rope_rows) uses the nearest table row instead of reading past the tables (the reference
 * reads out of bounds, csrc/rope/rotary_fp16_kernels.cu:674-685); callers that can know the
 * positions on the host should refuse such a request before it gets here. The cache is
 * [batch, n_kv_heads, max_cache_len, head_dim] (muillm/modules/kvcache/cache_utils.py:113-204).
 * ---------------------------------------------------------------------------------- */

/* muillm_rope_forward_static_cache / muillm_rope_forward_no_cache / muillm_static_kvcache_update
 * (csrc/module.cpp:266-268,272; csrc/rope/rotary.cu:603-756; csrc/kvcaches/static_kvcache.cpp:35-121)
 * for `tokens` new tokens per batch row:
 *   q_out[b, h, t, :]               = rope(q[b, t, h, :], position_ids[b, t])     (dense [B,Hq,T,D])
 *   k_out[b, h, slot(t), :]         = rope(k[b, t, h, :], position_ids[b, t])
 *   v_out[b, h, slot(t), :]         = v[b, t, h, :]
 * slot(t) = cache_position[t] when cache_position != NULL (k_out/v_out are the caches; slots
 * outside [0, max_cache_len) are skipped), else t (k_out/v_out are dense [B,Hkv,T,D] given by
 * the out strides). q, k or v may be NULL to skip that part; cos_table == NULL copies without
 * rotating (plain cache update). position_batch_stride 0 shares one row of positions. */
int mui_rope_kv_write(mui_stream_t stream, int dtype, const void* q, long q_batch_stride,
                      long q_token_stride, long q_head_stride, const void* k, long k_batch_stride,
                      long k_token_stride, long k_head_stride, const void* v, long v_batch_stride,
                      long v_token_stride, long v_head_stride, const float* cos_table,
                      const float* sin_table, int rope_row_stride, int rope_rows,
                      const int64_t* position_ids, long position_batch_stride,
                      const int64_t* cache_position, void* q_out,
                      void* k_out, void* v_out, long out_batch_stride, long out_head_stride,
                      long out_token_stride, int batch, int tokens, int n_q_heads, int n_kv_heads,
                      int head_dim, int max_cache_len);

/* Number of sequence splits to use for a decode over about seq_len_hint cached tokens
 * (enough workgroups to fill the GPU, at least two passes of work per split), and the
 * scratch size in bytes that mui_flash_decode / mui_attn_decode_fused need for it (0 when
 * n_splits == 1). The reference fixes 4 tokens per group (csrc/attention/flash_decoding.cu:15,153-158)
 * and allocates its partials inside the call. */
int mui_flash_decode_splits(int batch, int n_q_heads, int n_kv_heads, int seq_len_hint);
size_t mui_flash_decode_scratch_bytes(int batch, int n_q_heads, int head_dim, int n_splits);

/* muillm_causal_transformer_decoding_no_mask / _masked (csrc/module.cpp:276-277;
 * csrc/attention/flash_decoding.cu:99-325) for one query token per batch row:
 *   out[b, h*D:(h+1)*D] = softmax_s(q[b,h,:] . K[b, h/(Hq/Hkv), s, :] / sqrt(D)) V[b, h/(Hq/Hkv), s, :]
 * over s < seq_len. q is dense [batch, n_q_heads, head_dim] (already rotated); out is
 * [batch, n_q_heads * head_dim]. mask (optional, 16-bit, [batch, >= seq_len] rows
 * mask_batch_stride apart): 0 keeps key s, any other value drops it
 * (csrc/attention/flash_decoding_fp16_kernels.cu:386-393); a fully masked row yields 0.
 * scratch: mui_flash_decode_scratch_bytes() bytes, may be NULL when n_splits == 1.
 * n_splits <= 256. */
int mui_flash_decode(mui_stream_t stream, int dtype, const void* q, const void* k_cache,
                     const void* v_cache, long cache_batch_stride, long cache_head_stride,
                     long cache_token_stride, const void* mask, long mask_batch_stride, int seq_len,
                     void* scratch, int n_splits, void* out, int batch, int n_q_heads,
                     int n_kv_heads, int head_dim, int max_cache_len);

/* mui_flash_decode for callers that cannot allocate device memory (code under HIP-graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the
 * reference, whose flash decoding allocates its partials inside every call
 * (csrc/attention/flash_decoding.cu:156-158). Same arguments and results as mui_flash_decode
 * minus `scratch`: the split partials go to an array built into the library
 * (MUI_FLASH_DECODE_STATIC_SCRATCH_BYTES per GPU, held until the process ends), so the call
 * performs no allocation of any kind. A shape whose partials
 * (mui_flash_decode_scratch_bytes(batch, n_q_heads, head_dim, n_splits)) exceed that size is
 * refused with MUI_ERR_SCRATCH_LIMIT; at batch * n_q_heads * n_splits <= 8065 it fits. All calls
 * on one GPU share the array: calls that overlap in time on one GPU (different streams) race;
 * calls on one stream, or serialised by events, are safe. The device that is current at the
 * call must be the one the pointers belong to. */
#define MUI_FLASH_DECODE_STATIC_SCRATCH_BYTES (4u << 20)
size_t mui_flash_decode_static_scratch_limit(void);
int mui_flash_decode_static(mui_stream_t stream, int dtype, const void* q, const void* k_cache,
                            const void* v_cache, long cache_batch_stride, long cache_head_stride,
                            long cache_token_stride, const void* mask, long mask_batch_stride,
                            int seq_len, int n_splits, void* out, int batch, int n_q_heads,
                            int n_kv_heads, int head_dim, int max_cache_len);

/* One call for what the reference does in three (muillm_rotary_embedding_module_forward
 * csrc/module.cpp:381 -> RoPE + cache write kernel, then the two flash-decoding kernels,
 * muillm/modules/attention/sdpaattention.py:189-209): rotate q and the new k at
 * position_ids[b], write rotated k and v into cache slot cache_position[0], and attend over
 * cache rows [0, seq_len) including the new one. seq_len < 0 means cache_position[0] + 1,
 * read on the device, so the launch is replayable from a HIP graph as the sequence grows.
 * q, k_new, v_new: [batch, heads, head_dim] with head stride head_dim and the given batch
 * strides (views into a fused QKV output). q_out (optional): dense rotated queries. */
int mui_attn_decode_fused(mui_stream_t stream, int dtype, const void* q, long q_batch_stride,
                          const void* k_new, long k_batch_stride, const void* v_new,
                          long v_batch_stride, const float* cos_table, const float* sin_table,
                          int rope_row_stride, int rope_rows, const int64_t* position_ids,
                          long position_batch_stride, const int64_t* cache_position, int seq_len,
                          void* k_cache, void* v_cache, long cache_batch_stride,
                          long cache_head_stride, long cache_token_stride, const void* mask,
                          long mask_batch_stride, void* q_out, void* scratch, int n_splits,
                          void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                          int max_cache_len);

/* mui_attn_decode_fused that also announces what the NEXT kernel on the stream will stream:
 * next_weights / next_weight_bytes (16-byte aligned; NULL / 0: nothing) -- in a decoder layer the
 * o_proj matrix (csrc/modules/parallel_decoder_module.cpp:22-62 of the reference gives the order).
 * At short context and small batch the attention launch occupies one workgroup per query head
 * and is bound by latency: the rest of the chip and the whole memory system idle for its
 * duration. With this call, extra workgroups of the same launch pull those bytes on chip (L2 of
 * the XCD whose workgroups will read them, and the memory-side cache) and discard them; results
 * are those of mui_attn_decode_fused bit for bit. next_slab_bytes (a multiple of 16) is the
 * contiguous run one consumer workgroup reads at a time (for the GEMVs here: rows per group x
 * row pitch, see mui_linear_row_group_bytes); slab i is fetched by a workgroup on XCD i mod 8.
 * Launch shapes that fill the chip themselves (split sequences, larger batches) ignore the hint,
 * and so does every launch unless the process has opted in with mui_tune_warm (muillm_amd_tune.h):
 * on MI355X the faster o_proj (3.6 instead of 6.8 us) is paid for by a slower attention launch
 * (8.7-9.4 instead of 5.65 us). No counterpart in the reference. */
int mui_attn_decode_fused_warm(mui_stream_t stream, int dtype, const void* q, long q_batch_stride,
                               const void* k_new, long k_batch_stride, const void* v_new,
                               long v_batch_stride, const float* cos_table, const float* sin_table,
                               int rope_row_stride, int rope_rows, const int64_t* position_ids,
                               long position_batch_stride, const int64_t* cache_position, int seq_len,
                               void* k_cache, void* v_cache, long cache_batch_stride,
                               long cache_head_stride, long cache_token_stride, const void* mask,
                               long mask_batch_stride, void* q_out, void* scratch, int n_splits,
                               void* out, int batch, int n_q_heads, int n_kv_heads, int head_dim,
                               int max_cache_len, const void* next_weights, size_t next_weight_bytes,
                               int next_slab_bytes);

/* Bytes of weight matrix that one workgroup of the single-token linear kernels reads per step
 * (rows per row group x pitch_bytes), for mui_attn_decode_fused_warm; weight_bits 16 or 8. */
int mui_linear_row_group_bytes(int weight_bits, int k, long pitch_bytes);

/* Causal attention of `tokens` > 1 new query tokens per batch row (prefill, or a chunk of it)
 * over a static cache that already holds their rotated keys and values:
 *   out[b, t, h*D:(h+1)*D] = softmax_{s <= q_start + t}(q[b,h,t,:] . K[b, h/(Hq/Hkv), s, :] / sqrt(D)) V[...]
 * q_rotated is dense [batch, n_q_heads, tokens, head_dim] (what mui_rope_kv_write produces), query t
 * sits at key position q_start + t, keys are cache rows [0, seq_len), q_start + tokens <= seq_len.
 * The reference hands T > 1 to torch's scaled_dot_product_attention
 * (muillm/modules/attention/sdpaattention.py:221-245) after repeat_kv; here K/V are read per KV
 * head and no mask tensor is built. tokens may be at most 16 * 65535 (MUI_ERR_UNSUPPORTED beyond:
 * the position tiles are one dimension of the grid). */
int mui_prefill_attention(mui_stream_t stream, int dtype, const void* q_rotated, const void* k_cache,
                          const void* v_cache, long cache_batch_stride, long cache_head_stride,
                          long cache_token_stride, int seq_len, int q_start, void* out, int batch,
                          int n_q_heads, int n_kv_heads, int tokens, int head_dim);

/* The same with a key-padding mask (padded batches of prompts): key_mask is [batch, >= seq_len
 * rounded up to a multiple of 4] 16-bit entries, rows mask_batch_stride entries apart, 8-byte
 * aligned; a key whose entry is not zero is hidden from every query, on top of causality (what the
 * reference's additive 4-D mask amounts to when it is built from a 2-D attention mask,
 * muillm/modules/models/llama/model.py:437-613). A query whose every visible key is hidden gets
 * zeros. Reference route: torch SDPA with the 4-D mask (muillm/modules/attention/sdpaattention.py:221-245). */
int mui_prefill_attention_masked(mui_stream_t stream, int dtype, const void* q_rotated, const void* k_cache,
                                 const void* v_cache, long cache_batch_stride, long cache_head_stride,
                                 long cache_token_stride, int seq_len, int q_start, const void* key_mask,
                                 long mask_batch_stride, void* out, int batch, int n_q_heads,
                                 int n_kv_heads, int tokens, int head_dim);

/* Greedy token choice: out_index[r] = argmax_v logits[r, v] (lowest index on ties, NaN never
 * wins) for a 16-bit [rows, vocab] matrix with row pitch row_stride elements. Stands in for
 * the torch.argmax of the reference's greedy sampling branch
 * (muillm/sampling/generation.py:330-335) so that a captured decode step contains no
 * library reduction. */
int mui_argmax(mui_stream_t stream, int dtype, const void* logits, long row_stride,
               int64_t* out_index, int rows, int vocab);

/* One launch for the tail of a greedy decode step, per batch row b (all buffers on the device):
 *   tok = argmax_v logits[b, v]        (as mui_argmax)
 *   if unfinished != NULL and n_eos > 0 and unfinished[b] == 0: tok = pad_token
 *   tokens_out[b, step[b]] = tok  (when step[b] < max_steps);  next_ids[b] = tok
 *   position_ids[b] += 1;  step[b] += 1;  cache_position[0] += 1 (once)
 *   unfinished[b] &= (tok is none of eos_ids) && (step[b] < max_steps)
 * It folds the reference's torch.argmax + muillm_add_tokens_check_finished
 * (csrc/generation/generation.cu:29-113,115-195; muillm/sampling/generation.py:330-404) and
 * the position bookkeeping of its sampling loop into one kernel that a HIP graph can replay:
 * the token history is written in place at a device-side column counter instead of being
 * re-allocated as [B, T+1] every step. position_ids, cache_position and unfinished may be
 * NULL. */
int mui_greedy_advance(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                       int rows, int vocab, int64_t* next_ids, int64_t* position_ids,
                       int64_t* cache_position, int64_t* step, int64_t* tokens_out,
                       long tokens_stride, int max_steps, int64_t* unfinished,
                       const int64_t* eos_ids, int n_eos, long pad_token);

/* mui_greedy_advance with the scan of a long row dealt out to several workgroups (one workgroup per
 * 1024 chunks of 16 bytes, at most 32): a single workgroup pulls a 128k-entry row through one CU's
 * load path. No counterpart in the reference (its argmax is torch's). `workspace` is
 * mui_greedy_workspace_bytes(rows) bytes of 8-byte aligned device memory, zero-filled once by the
 * caller before the first call; every call leaves it zero-filled again, so one buffer serves all the
 * steps of a decode loop (and the replays of a captured one), but calls that share a buffer must not
 * overlap. The result is the one mui_greedy_advance gives, bit for bit. With workspace == NULL (and
 * workspace_bytes == 0), a buffer that is too small or misaligned, or rows that fit one workgroup,
 * this is mui_greedy_advance.
 * embed_table / embed_out (both or neither): the workgroup that finishes row b also copies row
 * `tok` of the 16-bit embedding table (rows embed_row_stride elements apart, embed_dim wide) to
 * embed_out[b, :] (dense [rows, embed_dim]), so that the next decode step starts from the embedding
 * without a gather launch of its own (whose two dependent loads -- token id, then the row -- cost
 * 4.8 us at the head of every step); pad_token must then be a row of the table (< vocab). */
size_t mui_greedy_workspace_bytes(int rows);
int mui_greedy_advance_ws(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                          int rows, int vocab, int64_t* next_ids, int64_t* position_ids,
                          int64_t* cache_position, int64_t* step, int64_t* tokens_out,
                          long tokens_stride, int max_steps, int64_t* unfinished,
                          const int64_t* eos_ids, int n_eos, long pad_token, void* workspace,
                          size_t workspace_bytes, const void* embed_table, long embed_row_stride,
                          void* embed_out, int embed_dim);

/* Sampling twin of mui_greedy_advance: tok = argmax_v(logits[b, v] / temperature - log q_v) with
 * q_v ~ Exp(1), which is the draw of the reference's sync-free multinomial
 * argmax(softmax(logits / temperature) / q) (muillm/sampling/multinomial.py:4-6) without
 * materialising the probabilities; -inf logits (top-k / top-p filters) never win. The variates
 * come from Philox4x32-10 keyed by `seed` with counter (v / 4, b, step[b] mod 2^32, 0), lane
 * v % 4 of the block: u = ((bits >> 8) + 1) * 2^-24, q = -log u. Token store, eos/pad rule and
 * counters exactly as mui_greedy_advance; replaying a captured launch draws fresh noise because
 * step[b] advances on the device. temperature > 0. */
int mui_sample_advance(mui_stream_t stream, int dtype, const void* logits, long row_stride,
                       int rows, int vocab, float temperature, uint64_t seed, int64_t* next_ids,
                       int64_t* position_ids, int64_t* cache_position, int64_t* step,
                       int64_t* tokens_out, long tokens_stride, int max_steps, int64_t* unfinished,
                       const int64_t* eos_ids, int n_eos, long pad_token);

/* ------------------------------------------------------------------------------------
 * decoder layers of one decode step in a single call
 * ---------------------------------------------------------------------------------- */

/* What MuiDecoderLayer.forward does for one token per batch row
 * (muillm/modules/decoder/decoder.py:130-165), for all layers, enqueued by one call; the
 * reference has a C++ layer loop only under tensor parallelism
 * (csrc/modules/parallel_decoder_stack.cpp, csrc/modules/parallel_decoder_module.cpp:22-62).
 * Per layer: qkv = Wqkv rmsnorm(h); attn = flash decoding with RoPE and cache write
 * (mui_attn_decode_fused); h' = Wo attn + h; mid = silu(Wg n) * (Wu n) with n = rmsnorm(h');
 * out = Wd mid + h'. Activations, norms, caches and 16-bit weights are device memory of the
 * 16-bit type `dtype`; any projection may instead hold int8 weights, with per-channel scales or
 * in the reference's group-wise (scale, min) format (muillm/modules/quantized/int8linear.py,
 * int8gateupdownmlp.py, muillm/quantization/rtnquantizer.py:49-88). The caller owns everything. */
typedef struct mui_decoder_layer {
  const void* input_norm;   /* [hidden] gamma of the RMSNorm fused into the QKV projection */
  const void* qkv_weight;   /* [(Hq + 2 Hkv) * D, hidden], rows q | k | v */
  long qkv_pitch;           /* row pitches in elements */
  const void* o_weight;     /* [hidden, Hq * D] */
  long o_pitch;
  const void* post_norm;    /* [hidden] gamma of the RMSNorm fused into gate/up */
  const void* gate_weight;  /* [intermediate, hidden] */
  const void* up_weight;    /* [intermediate, hidden], same pitch (interleaved storage allowed) */
  long gateup_pitch;
  const void* down_weight;  /* [hidden, intermediate] */
  long down_pitch;
  void* k_cache;            /* [batch, Hkv, max_cache_len, D] with the strides below */
  void* v_cache;
  /* Weight-only int8 projections (per-output-channel scales, the mui_int8_linear /
   * mui_int8_gateup_silu format): a non-NULL scales pointer says that projection's weights are
   * int8 codes (pitch in bytes) and are multiplied by these 16-bit scales; NULL = 16-bit
   * weights. gate and up are int8 together or not at all. */
  const void* qkv_scales;   /* [(Hq + 2 Hkv) * D] */
  const void* o_scales;     /* [hidden] */
  const void* gate_scales;  /* scale of row n at [n * gateup_scale_stride] */
  const void* up_scales;
  long gateup_scale_stride;
  const void* down_scales;  /* [hidden] */
  /* 0: the *_scales above are per-channel scales. s >= 4: the int8 projections of this layer are in
   * the reference's group format instead (muillm/quantization/rtnquantizer.py:49-88; the
   * mui_int8_group_linear / mui_int8_group_gateup_silu format): uint8 codes, groups of 2^s inputs,
   * and every non-NULL *_scales pointer addresses 16-bit (scale, min) pairs, [rows * G, 2] with
   * G = inputs >> s; for gate and up the pairs of row n start at gate_scales / up_scales +
   * n * gateup_scale_stride elements. */
  int int8_group_size_shift;
} mui_decoder_layer_t;

typedef struct mui_decoder_stack {
  int dtype, n_layers, hidden, n_q_heads, n_kv_heads, head_dim, intermediate;
  float norm_eps;
  const mui_decoder_layer_t* layers; /* host array of n_layers entries */
  const float* cos_table;            /* fp32 [rope_rows, rope_row_stride] rotary tables */
  const float* sin_table;
  long rope_row_stride;
  long rope_rows;
  long cache_batch_stride, cache_head_stride, cache_token_stride; /* elements */
  int max_cache_len;
} mui_decoder_stack_t;

/* Bytes of device workspace mui_decoder_stack_step needs (activations between the kernels
 * and the flash-decoding partials for n_splits); 0 on bad arguments. */
size_t mui_decoder_stack_workspace_bytes(const mui_decoder_stack_t* model, int batch, int n_splits);

/* hidden_in [batch, hidden] (token embeddings) -> hidden_out [batch, hidden] (output of the
 * last layer, before the final norm). position_ids, cache_position, seq_len, mask and
 * n_splits as in mui_attn_decode_fused (n_splits from mui_flash_decode_splits). workspace:
 * 256-byte aligned, mui_decoder_stack_workspace_bytes() bytes. batch <= MUI_MAX_TOKENS.
 * Asynchronous on `stream`, allocates nothing: capturable into a HIP graph. */
int mui_decoder_stack_step(mui_stream_t stream, const mui_decoder_stack_t* model, int batch,
                           const void* hidden_in, void* hidden_out, const int64_t* position_ids,
                           long position_batch_stride, const int64_t* cache_position, int seq_len,
                           const void* mask, long mask_batch_stride, int n_splits, void* workspace);

/* muillm_embedding_module_forward (csrc/module.cpp:320; csrc/embedding/embedding.cu:31-100; kernels
 * csrc/embedding/embedding_xx16_kernels.cu:26-112): out[t, :] = table[ids[t], :] for a 16-bit
 * [vocab, dim] table with row pitch row_pitch elements; ids int64, or int32 when ids_are_int32.
 * Ids outside [0, vocab) are clamped (the reference reads out of bounds). out is dense
 * [n_tokens, dim]. */
int mui_embedding(mui_stream_t stream, int dtype, const void* table, long row_pitch,
                  const void* ids, int ids_are_int32, void* out, int n_tokens, int dim, int vocab);

#ifdef __cplusplus
}
#endif

#endif /* MUILLM_AMD_H */
