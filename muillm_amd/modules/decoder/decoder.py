"""MuiDecoderLayer: a Llama / Mistral decoder layer as three fused blocks (API of
muillm/modules/decoder/decoder.py:22-165 in the reference: replace / forward, `qkv_proj`,
`self_attn`, `mlp`):

    q, k, v = qkv_proj(h)                    input RMSNorm inside the fused QKV projection
    h = self_attn(q, k, v, residual=h)       RoPE + cache write + attention + o_proj + residual
    h = mlp(h, residual=h)                   post-attention RMSNorm inside gate/up, residual in down
"""
from typing import Optional, Tuple, Union

import torch

from ..._hf import LlamaDecoderLayer, MistralDecoderLayer
from ...engineconfig import MuiEngineConfig
from ...memorymanagement.gc import trigger_gc
from ...replacement.replacementcontext import MuiReplacementContext
from ..attention.baseattention import MuiBaseAttention
from ..attention.sdpaattention import MuiSdpaAttention
from ..gateupdownmlp import MuiGateUpDownMLP
from ..module import MuiModule
from ..multilinear import MuiMultiLinear

_PROJECTIONS = ("q_proj", "k_proj", "v_proj", "o_proj")
_ABSORBED_CHILDREN = ("self_attn", "mlp", "input_layernorm", "post_attention_layernorm")


class MuiDecoderLayer(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, qkv_proj: MuiMultiLinear, self_attn: MuiBaseAttention,
                 mlp: MuiGateUpDownMLP):
        super().__init__(engine_config=engine_config)
        self.qkv_proj = qkv_proj
        self.self_attn = self_attn
        self.mlp = mlp

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiDecoderLayer", LlamaDecoderLayer, MistralDecoderLayer]) -> "MuiDecoderLayer":
        """Build the fused layer out of a HuggingFace decoder layer and strip that layer of the
        children whose parameters moved (so their memory can be reclaimed while the model is
        converted layer by layer)."""
        if isinstance(prev_module, MuiDecoderLayer):
            return prev_module
        if replacement_context.device is None:
            raise ValueError("the replacement context names no target device")
        attention = prev_module.self_attn
        missing = [name for name in _PROJECTIONS if not hasattr(attention, name)]
        if missing:
            raise ValueError(f"{type(attention).__name__} has no {missing}: not a layer this build can convert")
        layer = MuiDecoderLayer(
            replacement_context.engine_config,
            qkv_proj=MuiMultiLinear.replace(replacement_context,
                                            prev_modules=[attention.q_proj, attention.k_proj, attention.v_proj],
                                            prev_layernorm_module=prev_module.input_layernorm),
            self_attn=MuiSdpaAttention.replace(replacement_context, attention),
            # an already converted MLP is rebuilt as well: it has to absorb the norm in front of it
            mlp=MuiGateUpDownMLP.replace(replacement_context, prev_module=prev_module.mlp,
                                         prev_layernorm_module=prev_module.post_attention_layernorm))
        for child in _ABSORBED_CHILDREN:
            delattr(prev_module, child)
        trigger_gc()
        return layer

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                position_ids: Optional[torch.LongTensor] = None, past_key_value=None,
                output_attentions: Optional[bool] = False, use_cache: Optional[bool] = False,
                cache_position: Optional[torch.LongTensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                all_ones_mask: Optional[bool] = None, **kwargs):
        """Returns (hidden_states[, attention weights][, cache]) like a HuggingFace decoder layer."""
        q, k, v = self.qkv_proj(hidden_states)
        after_attention, attention_weights, cache = self.self_attn(
            query_states=q, key_states=k, value_states=v, attention_mask=attention_mask,
            position_ids=position_ids, past_key_value=past_key_value, output_attentions=output_attentions,
            use_cache=use_cache, cache_position=cache_position, position_embeddings=position_embeddings,
            all_ones_mask=all_ones_mask, residual=hidden_states,
            key_padding_mask=kwargs.get("key_padding_mask"))
        result = [self.mlp(after_attention, residual=after_attention)]
        if output_attentions:
            result.append(attention_weights)
        if use_cache:
            result.append(cache)
        return tuple(result)
