/*
 * muillm_amd_tune.h -- measurement aids of libmuillm_amd.so, kept apart from the product ABI
 * (muillm_amd.h), whose entry points are stateless once mui_tune_lock() has been called (or in a
 * process that never calls anything declared here).
 *
 * The mui_tune_* calls set PROCESS-GLOBAL launch-shape overrides that the product entry points
 * read at launch time; they are for benchmark sweeps and for tests that pin one kernel variant,
 * are not thread-safe and must not be called while another thread launches work. A process that
 * never calls them gets the built-in choices. mui_probe_read is a bandwidth probe. None of them
 * has a counterpart in the reference, whose launch shapes are compile-time constants
 * (csrc/linear/linear_fp16_kernels.cu:646-654).
 */
#ifndef MUILLM_AMD_TUNE_H
#define MUILLM_AMD_TUNE_H

#include "muillm_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* One-way switch: after this call every mui_tune_* call returns MUI_ERR_UNSUPPORTED and changes
 * nothing, for the rest of the process. A deployment calls it once after start-up, so that the
 * product entry points behave as the stateless functions muillm_amd.h describes whatever else is
 * loaded into the process. */
int mui_tune_lock(void);

/* Launch-shape knobs (0 restores the built-in choice). */
/* rows_per_group: 0, 2 or 4; or 100 + n: the fewest row groups per workgroup from which the
 * one-token GEMV keeps two of them in flight (built-in: 4, i.e. the lm_head; 100: never) */
int mui_tune_gemv(int rows_per_group, int workgroups_per_cu);
/* single-token routing: linear_on -> mui_linear (and bf16 mui_gateup_silu) through the packed-dot
 * kernel of the multi-token GEMV (default on); int8_on -> a single fp16 token of the int8 entry
 * points through the packed-dot int8 kernel (default on) */
int mui_tune_packed_dot(int linear_on, int int8_on);
int mui_tune_int8(int rows_per_group, int workgroups_per_cu);
/* the 4 x 4 x 4 matrix-instruction int8 kernel (fp16 activations, up to 4 tokens): on = 0 sends its
 * shapes to the older kernels; min_tokens = fewest tokens it takes (0 = default: 2 with per-channel
 * scales, 3 with the group format); workgroups per
 * CU (0 = built-in); register sets = row groups in flight per workgroup: 0 = built-in choice (two
 * where a norm is fused or a workgroup has more than two groups), 1 = one, 2 = two wherever a
 * workgroup has more than one group */
int mui_tune_int8_quad(int on, int min_tokens, int workgroups_per_cu, int sets);
/* waves per attention workgroup (4, 8 = default for <= 4 query heads per KV head, 16), the
 * fewest cached tokens that justify one more sequence split (default: two passes), and the
 * longest sequence that mui_flash_decode_splits leaves unsplit at small batch (default 1536;
 * negative: never use the unsplit one-workgroup-per-query-head mode), and mfma_tokens for the
 * matrix-core decode kernel: 0 = default (whenever a workgroup handles a whole KV group, i.e.
 * everywhere but in the unsplit one-workgroup-per-query-head mode), n > 0 = also instead of
 * that mode for sequences (or cache capacities, when the length is read on the device) of at
 * least n tokens, negative = never (vector-ALU kernel only) */
int mui_tune_attention(int waves_per_workgroup, int min_tokens_per_split, int direct_tokens,
                       int mfma_tokens);
/* fewest tokens that leave the one-GEMV-per-token loop (default 2; MUI_MAX_TOKENS + 1 keeps the
 * loop); stream_b selects older MFMA variants for 16-bit weights instead of the default one
 * that turns contiguous row runs into operands through LDS: 2 = operands loaded in MFMA order
 * straight from memory, token operands kept in registers (K <= 4096), 1 = the same with the
 * token operands re-read per weight tile; multi_max_tokens: largest token count served by the
 * multi-token GEMV rather than the MFMA kernel (16-bit weights; 0 = default 2; 5..8 only
 * qualify on matrices of >= 8192 rows with K <= 4096; 1 = never) */
int mui_tune_skinny(int min_tokens, int stream_b, int multi_max_tokens);

/* Prompt GEMM (more than MUI_MAX_TOKENS tokens): tile = 0 built-in choice, 1 = 128 rows x 128
 * tokens, 2 = 64 x 128, 3 = 32 x 64 (linear only), 4 = 256 x 256, 5 = 64 x 128 whose waves split K
 * four ways (2 x 2 wave tiles; int8: two token halves), 6 = 32 x 64 on four waves that split K,
 * 7 = 128 x 256, 8 = 192 x 256, 9 = 128 x 128 and 11 = 128 x 64 with waves that split K like 5,
 * 10 = 96 x 128 (linear only), 12 = 64 x 64 with waves that split K like 6 (linear only),
 * 13 = 256 x 256 on sixteen waves (4, 7 and 8 themselves run on eight software-pipelined waves where
 * they can: 16-bit weights, no fused norm, K a multiple of 64; 8 for linear only); shapes that a weight
 * format or epilogue lacks fall back to the next one that it has. A forced tile also keeps
 * mui_linear_ws from sharing K between workgroups.
 * 100 + tile: the same, and no tile loads its operands straight into LDS (all are staged through
 * registers, on sixteen or twelve waves). 200 + tile: the same as tile, but 128 x 256 and 192 x 256
 * keep their sixteen / twelve waves. 400 + tile: the software-pipelined tiles are launched as one
 * workgroup per tile instead of a persistent round of workgroups. 800 + tile: an XCD's workgroups
 * walk one row tile after another instead of panels of four row tiles (1600 + tile: panels of
 * eight, 2400 + tile: of two). 3200 + tile: gate/up stays one launch whatever its last round of
 * tiles holds. 6400 / 12800 / 19200 + tile: the XCDs divide the tile grid 8 x 1 / 4 x 2 / 2 x 4 ways
 * (rows x tokens) instead of the launcher's choice. 25600 + tile: the software-pipelined 128 x 256 tile
 * keeps two LDS stages instead of three. 51200 + tile: the software-pipelined 192 x 256 and 256 x 256 tiles
 * keep two stages of the weight tile instead of three. The offsets add up (e.g. 1204 = 800 + 400 + 4).
 * wide_max_tokens = longest prompt served by the weight-streaming 16-rows-per-workgroup kernel
 * instead of the LDS-tiled one (0 restores the built-in choice; at most 128; negative: never) */
int mui_tune_prefill(int tile, int wide_max_tokens);

/* Prompt attention (mui_prefill_attention): fewest query tokens that take the kernel sharing each
 * K/V block between all query heads of a KV head (0 = built-in choice, negative = never);
 * 1000000 + n: the same as n, and that kernel stages its K/V rows through registers instead of
 * loading them straight into LDS */
int mui_tune_prefill_attention(int group_kernel_min_tokens);

/* Cache warming by the idle workgroups of the unsplit decode-attention launch
 * (mui_attn_decode_fused_warm) is off by default (it measured no gain: the o_proj GEMV that follows
 * gets 3 us faster, the attention launch 3-4 us slower). workgroups = warm workgroups added to the
 * launch (a multiple of 8; > 0 switches it on, <= 0 off), percent = share of the announced bytes
 * that is fetched (0 = all), delay = head start of the attention workgroups in units of s_sleep 8,
 * about a quarter microsecond each (negative = built-in choice, at most 64) */
int mui_tune_warm(int workgroups, int percent, int delay);

/* Measurement aid without a counterpart in the reference: reads `bytes` (a multiple of 16, from
 * a 16-byte aligned address) of device memory once with the access shape of the GEMV kernels and
 * discards them. One launch takes the least time any kernel that must read that many bytes can
 * take on this device, launch latency included. `sink` is any 256-byte device buffer (written
 * only if the data matches a fixed 16-byte pattern). */
int mui_probe_read(mui_stream_t stream, const void* src, uint64_t bytes, void* sink);

/* Measurement aid without a counterpart in the reference: a chain of n_launches dependent fp16
 * GEMVs x_{i+1} = W_i . x_i (square matrices n == k <= 4096, used round-robin from the host array
 * `weights`; launch i reads xa or xb and writes the other), to price a kernel boundary against a
 * hand-off through memory. mode 0: ordinary launches. mode 1 / 2: launches that may start before
 * their predecessor has finished; each requests its first weight rows, then waits -- at most
 * spin_limit polls, after which it sets *err and goes on -- for the arrival counters its
 * predecessor bumps after its last store, and reads x with agent-scope loads (1) or ordinary ones
 * (2). `flags`: mui_probe_chain_flag_bytes(n_launches) bytes, zeroed by the caller before every
 * call; `err`: one zeroed uint32; workgroups: grid size (a multiple of 8; 0 = built-in choice). */
size_t mui_probe_chain_flag_bytes(int n_launches);
int mui_probe_gemv_chain(mui_stream_t stream, int mode, const void* const* weights, int n_mats,
                         int n_launches, int n, int k, void* xa, void* xb, void* flags, void* err,
                         int workgroups, int spin_limit);
/* The same chain dealt alternately to two streams (ordinary launches; a kernel meets its predecessor,
 * which runs on the other stream, through the arrival counters): mode 0 independent GEMVs without
 * hand-off, 1 the hand-off of mode 1 above, 2 / 3 a variant whose fifth wave polls and fetches x
 * while the other four have one / two row groups of weights in flight. */
int mui_probe_gemv_chain2(mui_stream_t stream_a, mui_stream_t stream_b, int mode,
                          const void* const* weights, int n_mats, int n_launches, int n, int k, void* xa,
                          void* xb, void* flags, void* err, int workgroups, int spin_limit);

#ifdef __cplusplus
}
#endif

#endif /* MUILLM_AMD_TUNE_H */
