"""MuiDecoderLayer -- muillm/modules/decoder/decoder.py:22-165:
   q, k, v = qkv_proj(h)                      (input RMSNorm fused into the GEMV)
   h = self_attn(q, k, v, ..., residual=h)    (RoPE + cache write + attention + o_proj + residual)
   h = mlp(h, residual=h)                     (post-attention RMSNorm fused into gate/up)"""
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
        engine_config = replacement_context.engine_config
        if replacement_context.device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiDecoderLayer):
            return prev_module
        prev_attn = prev_module.self_attn
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            if not hasattr(prev_attn, name):
                raise ValueError(f"Not supported {type(prev_attn)}")
        qkv_proj = MuiMultiLinear.replace(
            replacement_context, prev_modules=[prev_attn.q_proj, prev_attn.k_proj, prev_attn.v_proj],
            prev_layernorm_module=prev_module.input_layernorm)
        self_attn = MuiSdpaAttention.replace(replacement_context, prev_attn)
        # a MuiGateUpDownMLP is rebuilt too, to take the layernorm in
        mlp = MuiGateUpDownMLP.replace(replacement_context, prev_module=prev_module.mlp,
                                       prev_layernorm_module=prev_module.post_attention_layernorm)
        new_decoder = MuiDecoderLayer(engine_config=engine_config, qkv_proj=qkv_proj, self_attn=self_attn, mlp=mlp)
        del prev_module.self_attn
        del prev_module.mlp
        del prev_module.input_layernorm
        del prev_module.post_attention_layernorm
        trigger_gc()
        return new_decoder

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                position_ids: Optional[torch.LongTensor] = None, past_key_value=None,
                output_attentions: Optional[bool] = False, use_cache: Optional[bool] = False,
                cache_position: Optional[torch.LongTensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                all_ones_mask: Optional[bool] = None, **kwargs):
        residual = hidden_states
        query_states, key_states, value_states = self.qkv_proj(hidden_states)
        hidden_states, self_attn_weights, present_key_value = self.self_attn(
            query_states=query_states, key_states=key_states, value_states=value_states,
            attention_mask=attention_mask, position_ids=position_ids, past_key_value=past_key_value,
            output_attentions=output_attentions, use_cache=use_cache, cache_position=cache_position,
            position_embeddings=position_embeddings, all_ones_mask=all_ones_mask, residual=residual)
        residual = hidden_states
        hidden_states = self.mlp(hidden_states, residual=residual)
        outputs = (hidden_states,)
        if output_attentions:
            outputs += (self_attn_weights,)
        if use_cache:
            outputs += (present_key_value,)
        return outputs
