"""MuiSdpaAttention -- muillm/modules/attention/sdpaattention.py:27-256: as MuiBaseAttention;
multi-token inputs (prefill) run the library's causal kernels (with the key padding of a padded
batch when the model hands it over), torch's scaled_dot_product_attention only for masks of another
kind, fp32 or CPU tensors."""
from typing import Optional, Tuple

import torch

from ... import muillm_ext

from .baseattention import MuiBaseAttention
from .kvcache import repeat_kv


def _ignore_causal_mask_sdpa(attention_mask: Optional[torch.Tensor], inputs_shape, past_key_values_length: int,
                             sliding_window: Optional[int] = None, all_ones_mask: Optional[bool] = None,
                             is_training: bool = False) -> bool:
    """True when neither the user mask nor an explicit causal mask is needed and SDPA's
    is_causal flag suffices (no padding; one query token or no past). The all_ones_mask
    flag avoids the torch.all() device sync (sdpaattention.py:27-84 of the reference)."""
    query_length = inputs_shape[1]
    key_value_length = query_length + past_key_values_length
    if sliding_window is not None and key_value_length >= sliding_window:
        return False
    if attention_mask is None:
        return query_length == 1 or key_value_length == query_length
    if len(attention_mask.shape) == 4:
        return False
    no_padding = all_ones_mask if all_ones_mask is not None else bool(torch.all(attention_mask == 1))
    return bool(no_padding) and (query_length == 1 or key_value_length == query_length)


class MuiSdpaAttention(MuiBaseAttention):
    # Unpadded prompts of any length run the library's causal kernels (measured on MI355X, 32/8 heads
    # x 128, against repeat_kv + torch SDPA: 12 vs 36 us at 128 tokens, 20 vs 52 us at 512, 90 vs
    # 170 us at 2048, 0.77 vs 1.37 ms at 8192); None = no limit, a number restores the SDPA route
    # beyond that many tokens
    prefill_kernel_max_tokens = None

    def _prefill_kernel_ok(self, q, k, v, attention_mask, all_ones_mask, q_len, key_padding_mask=None) -> bool:
        """T > 1 whose mask is causal, or causal plus a key-padding mask handed over as such
        (key_padding_mask: what the model built its 4-D mask from), 16-bit CUDA tensors, head_dim
        128, K/V being equally strided views with unit inner stride (the static cache)."""
        if q_len <= 1 or not (all_ones_mask or attention_mask is None or key_padding_mask is not None):
            return False
        if not (q.is_cuda and q.dtype in (torch.float16, torch.bfloat16) and k.dtype == q.dtype and v.dtype == q.dtype):
            return False
        if self.head_dim != 128 or k.shape[2] < q_len or self.training:
            return False
        if self.prefill_kernel_max_tokens is not None and q_len > self.prefill_kernel_max_tokens:
            return False
        return (k.stride() == v.stride() and k.stride(3) == 1 and all(st % 8 == 0 for st in k.stride()[:3])
                and k.data_ptr() % 16 == 0 and v.data_ptr() % 16 == 0)

    def forward(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                attention_mask: Optional[torch.Tensor] = None, position_ids: Optional[torch.LongTensor] = None,
                past_key_value=None, output_attentions: bool = False, use_cache: bool = False,
                cache_position: Optional[torch.LongTensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                all_ones_mask: Optional[bool] = None, residual: Optional[torch.Tensor] = None, **kwargs):
        if output_attentions:
            return super().forward(
                query_states=query_states, key_states=key_states, value_states=value_states,
                attention_mask=attention_mask, position_ids=position_ids, past_key_value=past_key_value,
                output_attentions=output_attentions, use_cache=use_cache, cache_position=cache_position,
                position_embeddings=position_embeddings, all_ones_mask=all_ones_mask, residual=residual)
        if all_ones_mask is None:
            all_ones_mask = False
        bsz, q_len, _ = query_states.size()

        if self._fused_decode_ok(query_states, past_key_value, q_len):
            attn_output = self._fused_decode(query_states, key_states, value_states, attention_mask,
                                             position_ids, past_key_value, cache_position, all_ones_mask)
        else:
            q, k, v = self._split_heads(query_states, key_states, value_states)
            q, k, v = self.rotary_emb.apply_rotary_pos_emb_write_kv_cache(
                q, k, position_ids, position_embeddings, v, past_key_value, cache_position)
            attn_output = self._decode_or_none(q, k, v, attention_mask, all_ones_mask, q_len)
            key_padding_mask = None if all_ones_mask else kwargs.get("key_padding_mask")
            if attn_output is None and self._prefill_kernel_ok(q, k, v, attention_mask, all_ones_mask, q_len,
                                                               key_padding_mask):
                # causal attention of the new tokens over the cache views that already hold them
                attn_output = muillm_ext.mui_prefill_attention(q, k, v, key_mask=key_padding_mask)
            if attn_output is None:
                k = repeat_kv(k, self.num_key_value_groups)
                v = repeat_kv(v, self.num_key_value_groups)
                causal_mask = attention_mask
                if q.device.type == "cuda" and causal_mask is not None:
                    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
                is_causal = True if causal_mask is None and q_len > 1 else False
                attn_output = torch.nn.functional.scaled_dot_product_attention(
                    q, k, v, attn_mask=causal_mask,
                    dropout_p=self.attention_dropout if self.training else 0.0, is_causal=is_causal)
                attn_output = attn_output.transpose(1, 2).contiguous()
        attn_output = attn_output.reshape(bsz, q_len, self.hidden_size)
        attn_output = self.o_proj(attn_output, residual=residual)
        return attn_output, None, past_key_value
