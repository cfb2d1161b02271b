// One call for the decoder layers of a decode step.
//
// The reference walks its layers from C++ only under tensor parallelism
// (csrc/modules/parallel_decoder_stack.cpp; per-layer order in
// csrc/modules/parallel_decoder_module.cpp:22-62: fused-norm QKV, attention with RoPE and
// cache write, o_proj + residual, fused-norm gate/up + SiLU, down + residual); on one GPU it
// goes through its Python modules (muillm/modules/decoder/decoder.py:130-165). Here the same
// order is enqueued by one C call, which removes the per-launch host work of an interpreter
// loop (about 160 launches per token) when the step is not replayed from a HIP graph. Each
// projection takes 16-bit weights or int8 codes, the latter with per-channel scales or in the
// reference's group-wise (scale, min) format (muillm/modules/quantized/int8linear.py:279-293,
// int8gateupdownmlp.py, muillm/quantization/rtnquantizer.py:49-88).
#include "common.cuh"

using namespace mui;

namespace {

inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct StackWorkspace {
  char* h_a;      // [batch, hidden]   o_proj output (residual stream after attention)
  char* h_b;      // [batch, hidden]   layer output
  char* qkv;      // [batch, (Hq + 2 Hkv) * D]
  char* attn;     // [batch, Hq * D]
  char* mid;      // [batch, intermediate]
  char* scratch;  // flash-decoding partials
  size_t total;
};

StackWorkspace carve(const mui_decoder_stack_t* m, int batch, int n_splits, char* base) {
  StackWorkspace w;
  const size_t e = 2;  // 16-bit activations
  const size_t hid = align256((size_t)batch * m->hidden * e);
  const size_t qkv = align256((size_t)batch * (m->n_q_heads + 2 * m->n_kv_heads) * m->head_dim * e);
  const size_t att = align256((size_t)batch * m->n_q_heads * m->head_dim * e);
  const size_t mid = align256((size_t)batch * m->intermediate * e);
  const size_t scr = align256(mui_flash_decode_scratch_bytes(batch, m->n_q_heads, m->head_dim, n_splits));
  size_t off = 0;
  w.h_a = base + off; off += hid;
  w.h_b = base + off; off += hid;
  w.qkv = base + off; off += qkv;
  w.attn = base + off; off += att;
  w.mid = base + off; off += mid;
  w.scratch = base + off; off += scr;
  w.total = off;
  return w;
}

}  // namespace

extern "C" size_t mui_decoder_stack_workspace_bytes(const mui_decoder_stack_t* m, int batch, int n_splits) {
  if (!m || batch < 1 || n_splits < 1) return 0;
  return carve(m, batch, n_splits, nullptr).total;
}

extern "C" int mui_decoder_stack_step(mui_stream_t stream, const mui_decoder_stack_t* m, int batch,
                                      const void* hidden_in, void* hidden_out,
                                      const int64_t* position_ids, long position_batch_stride,
                                      const int64_t* cache_position, int seq_len, const void* mask,
                                      long mask_batch_stride, int n_splits, void* workspace) {
  MUI_CHECK_ARG(m && m->layers && m->n_layers > 0 && hidden_in && hidden_out && workspace);
  MUI_CHECK_ARG(batch >= 1 && batch <= MUI_MAX_TOKENS && n_splits >= 1);
  MUI_CHECK_ARG(position_ids && cache_position);
  MUI_CHECK_ARG(((uintptr_t)workspace & 255u) == 0);
  const StackWorkspace w = carve(m, batch, n_splits, (char*)workspace);
  const int qd = m->n_q_heads * m->head_dim, kvd = m->n_kv_heads * m->head_dim;
  const int qkv_n = qd + 2 * kvd;
  const char* h = (const char*)hidden_in;  // residual stream entering the layer
  for (int l = 0; l < m->n_layers; ++l) {
    const mui_decoder_layer_t& L = m->layers[l];
    char* out = (l + 1 == m->n_layers) ? (char*)hidden_out : w.h_b;
    const int gs = L.int8_group_size_shift;  // 0: per-channel scales; else the reference's group format
    if (gs < 0) return MUI_ERR_INVALID_ARG;
    int st = !L.qkv_scales
                 ? mui_linear(stream, m->dtype, L.qkv_weight, L.qkv_pitch, h, L.input_norm, m->norm_eps, nullptr,
                              nullptr, nullptr, w.qkv, qkv_n, m->hidden, batch)
             : gs ? mui_int8_group_linear(stream, m->dtype, L.qkv_weight, L.qkv_pitch, L.qkv_scales, gs, h,
                                          L.input_norm, m->norm_eps, nullptr, nullptr, w.qkv, qkv_n, m->hidden,
                                          batch)
                  : mui_int8_linear(stream, m->dtype, L.qkv_weight, L.qkv_pitch, L.qkv_scales, h, L.input_norm,
                                    m->norm_eps, nullptr, nullptr, w.qkv, qkv_n, m->hidden, batch);
    if (st != MUI_OK) return st;
    const char* q = w.qkv;
    // the attention launch is told what follows it: at short context its idle workgroups fetch the
    // o_proj matrix on chip while the few busy ones wait on latency
    const int o_bits = L.o_scales ? 8 : 16;
    const long o_pitch_bytes = L.o_pitch * (o_bits / 8);
    const int o_slab = batch == 1 ? mui_linear_row_group_bytes(o_bits, qd, o_pitch_bytes) : 0;
    const size_t o_bytes = o_slab > 0 ? (size_t)m->hidden * (size_t)o_pitch_bytes : 0;
    st = mui_attn_decode_fused_warm(stream, m->dtype, q, qkv_n, q + (size_t)qd * 2, qkv_n,
                                    q + (size_t)(qd + kvd) * 2, qkv_n, m->cos_table, m->sin_table, (int)m->rope_row_stride, (int)m->rope_rows,
                                    position_ids, position_batch_stride, cache_position, seq_len, L.k_cache,
                                    L.v_cache, m->cache_batch_stride, m->cache_head_stride, m->cache_token_stride,
                                    mask, mask_batch_stride, nullptr, w.scratch, n_splits, w.attn, batch,
                                    m->n_q_heads, m->n_kv_heads, m->head_dim, m->max_cache_len,
                                    o_bytes ? L.o_weight : nullptr, o_bytes, o_slab);
    if (st != MUI_OK) return st;
    st = !L.o_scales ? mui_linear(stream, m->dtype, L.o_weight, L.o_pitch, w.attn, nullptr, 0.f, nullptr, nullptr, h,
                                  w.h_a, m->hidden, qd, batch)
         : gs ? mui_int8_group_linear(stream, m->dtype, L.o_weight, L.o_pitch, L.o_scales, gs, w.attn, nullptr, 0.f,
                                      nullptr, h, w.h_a, m->hidden, qd, batch)
              : mui_int8_linear(stream, m->dtype, L.o_weight, L.o_pitch, L.o_scales, w.attn, nullptr, 0.f, nullptr, h,
                                w.h_a, m->hidden, qd, batch);
    if (st != MUI_OK) return st;
    if ((L.gate_scales == nullptr) != (L.up_scales == nullptr)) return MUI_ERR_INVALID_ARG;
    st = !L.gate_scales
             ? mui_gateup_silu(stream, m->dtype, L.gate_weight, L.up_weight, L.gateup_pitch, w.h_a, L.post_norm,
                               m->norm_eps, w.mid, m->intermediate, m->hidden, batch)
         : gs ? mui_int8_group_gateup_silu(stream, m->dtype, L.gate_weight, L.up_weight, L.gateup_pitch,
                                           L.gate_scales, L.up_scales, L.gateup_scale_stride, gs, w.h_a,
                                           L.post_norm, m->norm_eps, w.mid, m->intermediate, m->hidden, batch)
              : mui_int8_gateup_silu(stream, m->dtype, L.gate_weight, L.up_weight, L.gateup_pitch, L.gate_scales,
                                     L.up_scales, L.gateup_scale_stride, w.h_a, L.post_norm, m->norm_eps, w.mid,
                                     m->intermediate, m->hidden, batch);
    if (st != MUI_OK) return st;
    st = !L.down_scales ? mui_linear(stream, m->dtype, L.down_weight, L.down_pitch, w.mid, nullptr, 0.f, nullptr,
                                     nullptr, w.h_a, out, m->hidden, m->intermediate, batch)
         : gs ? mui_int8_group_linear(stream, m->dtype, L.down_weight, L.down_pitch, L.down_scales, gs, w.mid,
                                      nullptr, 0.f, nullptr, w.h_a, out, m->hidden, m->intermediate, batch)
              : mui_int8_linear(stream, m->dtype, L.down_weight, L.down_pitch, L.down_scales, w.mid, nullptr, 0.f,
                                nullptr, w.h_a, out, m->hidden, m->intermediate, batch);
    if (st != MUI_OK) return st;
    h = out;
  }
  return MUI_OK;
}
