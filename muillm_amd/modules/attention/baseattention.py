"""MuiBaseAttention -- muillm/modules/attention/baseattention.py:28-260: attention over
pre-projected q/k/v (the QKV projection lives in the decoder layer's MuiMultiLinear), RoPE +
KV-cache write, decode or eager attention, then o_proj with the residual fused in."""
import math
from typing import Optional, Tuple

import torch
import torch.nn as nn

from ... import muillm_ext
from ..._hf import head_dim_of
from ...engineconfig import MuiEngineConfig
from ...replacement.replacementcontext import MuiReplacementContext
from ..kvcache.cache_utils import MuiStaticCache
from ..linear import MuiLinear
from ..module import MuiModule
from .causaltransformerdecoding import mui_causally_decode, mui_causally_decode_masked
from .kvcache import repeat_kv
from .rotaryembedding import MuiRotaryEmbedding


class MuiBaseAttention(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, config, rotary_emb: MuiRotaryEmbedding, o_proj: MuiLinear,
                 layer_idx: Optional[int] = None, device=None, dtype=None):
        super().__init__(engine_config=engine_config)
        self.config = config
        self.layer_idx = layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = head_dim_of(config)
        kvh = getattr(config, "num_key_value_heads", None)
        self.num_key_value_heads = self.num_heads if kvh is None else kvh
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.max_position_embeddings = config.max_position_embeddings
        self.is_causal = True
        self.attention_dropout = getattr(config, "attention_dropout", 0.0)
        if (self.head_dim * self.num_heads) != self.hidden_size:
            raise ValueError(
                f"hidden_size must be divisible by num_heads (got `hidden_size`: {self.hidden_size}"
                f" and `num_heads`: {self.num_heads}).")
        self.o_proj = o_proj
        self.rotary_emb = rotary_emb

    @staticmethod
    def _create_rotary_embeddings(engine_config: MuiEngineConfig, config, layer_idx: int, device=None,
                                  dtype=None) -> MuiRotaryEmbedding:
        return MuiRotaryEmbedding(engine_config, config, layer_idx=layer_idx, device=device, dtype=dtype)

    @classmethod
    def replace(cls, replacement_context: MuiReplacementContext, prev_module) -> "MuiBaseAttention":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        dtype = prev_module.o_proj.weight.dtype
        layer_idx = prev_module.layer_idx
        config = prev_module.config
        rotary_emb = MuiBaseAttention._create_rotary_embeddings(engine_config, config, layer_idx, device, dtype)
        new_o_proj = MuiLinear.replace(replacement_context, prev_module.o_proj)
        return cls(engine_config=engine_config, config=config, rotary_emb=rotary_emb, o_proj=new_o_proj,
                   layer_idx=layer_idx, device=device, dtype=dtype)

    # ---- pieces shared with MuiSdpaAttention ----
    def _split_heads(self, query_states, key_states, value_states):
        bsz, q_len, _ = query_states.size()
        q = query_states.view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
        k = key_states.view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        v = value_states.view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        return q, k, v

    def _fused_decode_ok(self, query_states, past_key_value, q_len: int) -> bool:
        return (q_len == 1 and isinstance(past_key_value, MuiStaticCache) and query_states.is_cuda
                and query_states.dtype in (torch.float16, torch.bfloat16) and self.head_dim == 128
                and self.rotary_emb.dispatchable
                and past_key_value.key_cache[self.layer_idx].dtype == query_states.dtype)

    def _fused_decode(self, query_states, key_states, value_states, attention_mask, position_ids,
                      cache: MuiStaticCache, cache_position, all_ones_mask):
        """One token per batch row: RoPE, cache write and flash decoding in a single call."""
        if cache_position is None:
            raise ValueError("cache_position is needed")
        if self.layer_idx == 0:
            cache._seen_tokens += 1
            if cache.cpp_module is not None:
                cache.cpp_module.seen_tokens = cache._seen_tokens
        seq_len = None if cache.device_length_mode else cache._seen_tokens
        mask = None if (all_ones_mask or attention_mask is None) else attention_mask
        if position_ids is None:
            position_ids = cache_position.unsqueeze(0)
        return muillm_ext.mui_attention_decode_fused(
            query_states[:, 0, :], key_states[:, 0, :], value_states[:, 0, :],
            self.rotary_emb.cos32, self.rotary_emb.sin32, position_ids, cache_position,
            cache.key_cache[self.layer_idx], cache.value_cache[self.layer_idx],
            seq_len=seq_len, mask=mask, seq_len_hint=cache.max_cache_len, next_weights=self._next_weights())

    def _next_weights(self):
        """The matrix o_proj will stream right after the attention kernel (16-bit weights or int8 codes)."""
        o = self.o_proj
        w = getattr(o, "weights_int8", None)
        if w is None:
            w = getattr(o, "weights_uint8", None)
        if w is None:
            w = getattr(o, "weight", None)
        return w if isinstance(w, torch.Tensor) else None

    def _decode_or_none(self, q, k, v, attention_mask, all_ones_mask, q_len):
        """The two-step decode path (already rotated q, cache views) for T == 1."""
        if q_len == 1 and q.is_cuda and q.dtype in (torch.float16, torch.bfloat16) and self.head_dim == 128:
            if all_ones_mask or (attention_mask is None):
                return mui_causally_decode(q.contiguous(), k, v)
            return mui_causally_decode_masked(q.contiguous(), k, v, attention_mask)
        return None

    def _eager(self, q, k, v, attention_mask):
        bsz, _, q_len, _ = q.shape
        k = repeat_kv(k, self.num_key_value_groups)
        v = repeat_kv(v, self.num_key_value_groups)
        attn_weights = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(self.head_dim)
        if attention_mask is not None:
            attn_weights = attn_weights + attention_mask
        attn_weights = nn.functional.softmax(attn_weights, dim=-1, dtype=torch.float32).to(q.dtype)
        attn_weights = nn.functional.dropout(attn_weights, p=self.attention_dropout, training=self.training)
        attn_output = torch.matmul(attn_weights, v)
        attn_output = attn_output.transpose(1, 2).contiguous().reshape(bsz, q_len, self.hidden_size)
        return attn_output, attn_weights

    def forward(self, query_states: torch.Tensor, key_states: torch.Tensor, value_states: torch.Tensor,
                attention_mask: Optional[torch.Tensor] = None, position_ids: Optional[torch.LongTensor] = None,
                past_key_value=None, output_attentions: bool = False, use_cache: bool = False,
                cache_position: Optional[torch.LongTensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                all_ones_mask: Optional[bool] = None, residual: Optional[torch.Tensor] = None, **kwargs):
        if all_ones_mask is None:
            all_ones_mask = False
        bsz, q_len, _ = query_states.size()
        attn_weights = None
        if not output_attentions and self._fused_decode_ok(query_states, past_key_value, q_len):
            attn_output = self._fused_decode(query_states, key_states, value_states, attention_mask,
                                             position_ids, past_key_value, cache_position, all_ones_mask)
        else:
            q, k, v = self._split_heads(query_states, key_states, value_states)
            q, k, v = self.rotary_emb.apply_rotary_pos_emb_write_kv_cache(
                q, k, position_ids, position_embeddings, v, past_key_value, cache_position)
            attn_output = None if output_attentions else self._decode_or_none(
                q, k, v, attention_mask, all_ones_mask, q_len)
            if attn_output is None:
                attn_output, attn_weights = self._eager(q, k, v, attention_mask)
        attn_output = attn_output.reshape(bsz, q_len, self.hidden_size)
        attn_output = self.o_proj(attn_output, residual=residual)
        if not output_attentions:
            attn_weights = None
        return attn_output, attn_weights, past_key_value
