"""MuiLlamaModel / MuiLlamaForCausalLM -- the decoder harness around the fused layers
(muillm/modules/models/llama/model.py:75-873 of the reference; its Mistral file differs in
feeding config.sliding_window into the mask -- here the Mistral names alias the Llama classes,
whose forward() does the same whenever the config carries a sliding window).

Semantics kept from the reference: embed -> N x MuiDecoderLayer -> final MuiRMSNorm ->
lm_head (MuiLinear) -> fp32 logits; a MuiStaticCache with power-of-two capacity is created
on first use and grown when needed; the causal mask is dropped when there is no padding
(all_ones_mask), decode steps then need no mask at all.

The classes are plain torch modules (the reference derives them from HuggingFace's
PreTrainedModel / GenerationMixin, whose interfaces differ between transformers versions);
replace() accepts HuggingFace LlamaModel / LlamaForCausalLM (and Mistral) instances, and
from_config() builds a randomly initialised model straight from a config for benchmarks.
Greedy generation is provided by generate_greedy(), with the decode step optionally
captured once into a HIP graph and replayed (see graphdecoder.py)."""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple, Union

import torch
import torch.nn as nn

from .... import muillm_ext
from ...._hf import (LlamaForCausalLM, LlamaModel, MistralForCausalLM, MistralModel, head_dim_of)
from ....engineconfig import MuiEngineConfig
from ....memorymanagement.gc import trigger_gc
from ....replacement.replacementcontext import MuiReplacementContext
from ...attention.rotaryembedding import MuiRotaryEmbedding, is_hf_static_cache
from ...attention.sdpaattention import MuiSdpaAttention, _ignore_causal_mask_sdpa
from ...decoder.decoder import MuiDecoderLayer
from ...decoder.decoderstack import MuiDecoderStack
from ...embedding import MuiEmbedding
from ...gateupdownmlp import MuiGateUpDownMLP
from ...kvcache.cache_utils import (MuiCache, MuiStaticCache, create_static_cache,
                                    grow_static_cache_if_needed)
from ...linear import MuiLinear
from ...module import MuiModule
from ...multilinear import MuiMultiLinear
from ...norm.rmsnorm import MuiRMSNorm


@dataclass
class MuiDecoderConfig:
    """The fields of a Llama/Mistral config that the decoder reads (duck-typed stand-in for
    transformers' LlamaConfig / MistralConfig)."""
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    max_position_embeddings: int = 8192
    rope_theta: float = 500000.0
    head_dim: Optional[int] = None
    rope_scaling: Optional[Dict[str, Any]] = None
    attention_dropout: float = 0.0
    attention_bias: bool = False
    mlp_bias: bool = False
    pad_token_id: Optional[int] = None
    tie_word_embeddings: bool = False

    @staticmethod
    def llama3_8b(**overrides) -> "MuiDecoderConfig":
        return MuiDecoderConfig(**overrides)

    @staticmethod
    def mistral_7b(**overrides) -> "MuiDecoderConfig":
        base = dict(vocab_size=32000, rope_theta=10000.0, max_position_embeddings=32768, rms_norm_eps=1e-5)
        base.update(overrides)
        return MuiDecoderConfig(**base)


@dataclass
class MuiModelOutput:
    last_hidden_state: torch.Tensor
    past_key_values: Optional[MuiCache] = None
    hidden_states: Optional[Tuple[torch.Tensor, ...]] = None
    attentions: Optional[Tuple[torch.Tensor, ...]] = None


@dataclass
class MuiCausalLMOutput:
    logits: torch.Tensor
    past_key_values: Optional[MuiCache] = None
    hidden_states: Optional[Tuple[torch.Tensor, ...]] = None
    attentions: Optional[Tuple[torch.Tensor, ...]] = None
    loss: Optional[torch.Tensor] = None


class MuiLlamaModel(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, config, embed_tokens: nn.Embedding, layers,
                 norm: MuiRMSNorm, rotary_emb: MuiRotaryEmbedding):
        super().__init__(engine_config=engine_config)
        self.config = config
        self.cpp_engine = engine_config.cpp_engine
        self.mdevice = embed_tokens.weight.device
        self.mdtype = embed_tokens.weight.dtype
        self.padding_idx = getattr(config, "pad_token_id", None)
        self.vocab_size = config.vocab_size
        self.embed_tokens = embed_tokens
        self.layers = layers if isinstance(layers, nn.ModuleList) else nn.ModuleList(layers)
        self.norm = norm
        self.rotary_emb = rotary_emb
        self.use_decoder_stack = True  # False: always walk the layer modules from Python
        self._stack: Optional[MuiDecoderStack] = None
        self._stack_rejected = None

    def finalize_init(self):
        self.mdevice = self.embed_tokens.weight.device
        self.mdtype = self.embed_tokens.weight.dtype

    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_model) -> "MuiLlamaModel":
        if isinstance(prev_model, MuiLlamaModel):
            return prev_model
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        config = prev_model.config
        embed_tokens = MuiEmbedding.replace(replacement_context, prev_model.embed_tokens)
        dtype = embed_tokens.weight.dtype
        layers = []
        for i in range(len(prev_model.layers)):
            layers.append(MuiDecoderLayer.replace(replacement_context, prev_model.layers[i]))
            prev_model.layers[i] = None  # release the source layer as we go
        norm = MuiRMSNorm.replace(replacement_context, prev_model.norm)
        rotary_emb = MuiRotaryEmbedding(engine_config, config, layer_idx=0, device=device, dtype=dtype)
        new_model = MuiLlamaModel(engine_config, config, embed_tokens, layers, norm, rotary_emb)
        trigger_gc()
        return new_model

    def get_input_embeddings(self):
        return self.embed_tokens

    def set_input_embeddings(self, value):
        self.embed_tokens = value

    def _decode_stack(self, cache, batch_size: int, hidden_states) -> Optional[MuiDecoderStack]:
        """The single-call layer stack for this cache and batch size, or None when the model does
        not qualify (quantized layers, biases, foreign cache, ...); rebuilt when the cache moves."""
        if not self.use_decoder_stack or not hidden_states.is_cuda or not isinstance(cache, MuiStaticCache):
            return None
        st = self._stack
        if st is not None and st.matches(self.layers, cache, batch_size):
            return st
        self._stack = None
        # a model that did not qualify is not examined again until its modules or cache change
        key = tuple(id(m) for l in self.layers for m in (getattr(l, "qkv_proj", None), getattr(l, "mlp", None)))
        key += (id(cache), batch_size)
        if key == self._stack_rejected:
            return None
        if MuiDecoderStack.eligible(self.layers, self.rotary_emb, cache, batch_size):
            self._stack = MuiDecoderStack(self.layers, self.rotary_emb, cache, batch_size)
        else:
            self._stack_rejected = key
        return self._stack

    def _update_causal_mask(self, attention_mask, inputs_shape, cache_position, past_key_values,
                            output_attentions, all_ones_mask, past_seen_tokens: int,
                            sliding_window: Optional[int] = None):
        """Additive 4-D mask [B, 1, T, S_total] (0 keep / finfo.min drop), or None when SDPA's
        is_causal / the mask-free decode kernel suffice (llama/model.py:437-613 of the reference).
        sliding_window=W also drops the keys at or before position - W, so that every query sees
        its last W keys (mistral/model.py:590-602 of the reference)."""
        if (not output_attentions) and _ignore_causal_mask_sdpa(
                attention_mask, inputs_shape, past_seen_tokens, sliding_window=sliding_window,
                all_ones_mask=all_ones_mask, is_training=self.training):
            return None
        bsz, q_len = inputs_shape[0], inputs_shape[1]
        target_length = past_seen_tokens + q_len
        dtype, device = self.mdtype, self.mdevice
        min_dtype = torch.finfo(dtype).min
        if attention_mask is not None and attention_mask.dim() == 4:
            return attention_mask
        causal = torch.full((q_len, target_length), fill_value=min_dtype, dtype=dtype, device=device)
        keys = torch.arange(target_length, device=device)
        hidden = keys > cache_position.reshape(-1, 1)
        if sliding_window is not None:
            hidden = hidden | (keys <= cache_position.reshape(-1, 1) - int(sliding_window))
        causal = causal * hidden
        causal = causal[None, None, :, :].expand(bsz, 1, -1, -1)
        if attention_mask is not None:
            causal = causal.clone()
            mask_length = attention_mask.shape[-1]
            padding = causal[:, :, :, :mask_length] + attention_mask[:, None, None, :].to(dtype)
            causal[:, :, :, :mask_length] = causal[:, :, :, :mask_length].masked_fill(padding == 0, min_dtype)
        return causal

    def forward(self, input_ids: torch.LongTensor = None, attention_mask: Optional[torch.Tensor] = None,
                position_ids: Optional[torch.LongTensor] = None, past_key_values=None,
                inputs_embeds: Optional[torch.Tensor] = None, use_cache: Optional[bool] = None,
                output_attentions: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                return_dict: Optional[bool] = None, cache_position: Optional[torch.LongTensor] = None,
                all_ones_mask: Optional[bool] = None, skip_final_norm: bool = False):
        """skip_final_norm=True returns the un-normalised last hidden state: the causal-LM head
        then applies the final RMSNorm inside its GEMV kernel (single-token decode)."""
        output_attentions = bool(output_attentions)
        output_hidden_states = bool(output_hidden_states)
        use_cache = True if use_cache is None else use_cache
        if (input_ids is None) == (inputs_embeds is None):
            raise ValueError(
                "You cannot specify both input_ids and inputs_embeds at the same time, and must specify either one")
        inputs_shape = input_ids.shape if input_ids is not None else inputs_embeds.shape
        batch_size, q_len = inputs_shape[0], inputs_shape[1]
        if past_key_values is not None and not isinstance(past_key_values, MuiCache) \
                and not is_hf_static_cache(past_key_values):
            past_key_values = None  # other foreign cache types are dropped, a static cache is built instead
        # (a HuggingFace StaticCache is written in place by the rotary / cache-write kernel; its layers
        # take the per-layer route, the single-call decode step needs a MuiStaticCache)
        past_seen_tokens = int(past_key_values.get_seq_length()) if past_key_values is not None else 0
        tot_seq_len = past_seen_tokens + q_len
        # the rotary tables have max_position_embeddings rows and the kernels index them with
        # device-side positions: refuse here what would run past them
        if tot_seq_len > self.rotary_emb.max_seq_len_cached:
            raise ValueError(f"{tot_seq_len} tokens exceed the {self.rotary_emb.max_seq_len_cached} rotary positions "
                             "of this model (max_position_embeddings)")
        if isinstance(past_key_values, MuiStaticCache) and batch_size > past_key_values.max_batch_size:
            raise ValueError(f"batch {batch_size} exceeds the cache's max_batch_size {past_key_values.max_batch_size}")
        # Mistral's sliding-window attention, as the reference does it: config.sliding_window goes into
        # the mask (muillm/modules/models/mistral/model.py:484,593-602). Up to the window it is plain
        # causal attention; beyond it the mask hides the keys at or before position - window, single
        # tokens take the masked decode kernel and prompts the 4-D-mask route. (A 4-D mask from the
        # caller is used as it is: the device-resident decode loop maintains the window in its own.)
        window = getattr(self.config, "sliding_window", None)
        windowed = bool(window) and tot_seq_len > int(window)

        if use_cache:
            if past_key_values is None:
                past_key_values = create_static_cache(self.engine_config, self.config, batch_size, tot_seq_len,
                                                      self.mdevice, self.mdtype)
            elif isinstance(past_key_values, MuiStaticCache):
                grow_static_cache_if_needed(past_key_values, tot_seq_len, self.config.max_position_embeddings)

        if cache_position is None:
            cache_position = torch.arange(past_seen_tokens, tot_seq_len, device=self.mdevice)
        if position_ids is None:
            position_ids = cache_position.unsqueeze(0)

        if all_ones_mask is None:
            all_ones_mask = attention_mask is None
        causal_mask = None
        if not all_ones_mask or q_len > 1 or windowed:
            causal_mask = self._update_causal_mask(attention_mask, inputs_shape, cache_position, past_key_values,
                                                   output_attentions, all_ones_mask, past_seen_tokens,
                                                   sliding_window=int(window) if windowed else None)
        if all_ones_mask and q_len == 1 and not windowed:
            causal_mask = None
        elif causal_mask is not None:
            causal_mask = causal_mask[:, :, :, :tot_seq_len]
        if windowed:
            all_ones_mask = False  # the layers must apply the mask even without padding
        # a padded prompt whose 4-D mask was built right here from a 2-D one: the attention layers
        # get the key padding as such and keep the library's prompt kernel (a 4-D mask from the
        # caller may hold anything and stays with SDPA)
        key_padding_mask = None
        if (causal_mask is not None and q_len > 1 and attention_mask is not None and attention_mask.dim() == 2
                and not windowed and torch.device(self.mdevice).type == "cuda" and self.mdtype in (torch.float16, torch.bfloat16)):
            key_padding_mask = muillm_ext.key_padding_mask16(attention_mask, self.mdtype, tot_seq_len)
        position_ids = position_ids.contiguous()

        if inputs_embeds is None:
            inputs_embeds = self.embed_tokens(input_ids)
        hidden_states = inputs_embeds

        # shared position embeddings for the layers that take the unfused route
        position_embeddings = None
        if not (q_len == 1 and isinstance(past_key_values, MuiStaticCache) and hidden_states.is_cuda):
            position_embeddings = self.rotary_emb(hidden_states, position_ids)

        all_hidden_states = () if output_hidden_states else None
        all_self_attns = () if output_attentions else None
        stack = None
        if q_len == 1 and use_cache and not output_hidden_states and not output_attentions:
            stack = self._decode_stack(past_key_values, batch_size, hidden_states)
        if stack is not None:
            # every layer through one library call (what the loop below does, layer by layer)
            past_key_values._seen_tokens += 1
            if past_key_values.cpp_module is not None:
                past_key_values.cpp_module.seen_tokens = past_key_values._seen_tokens
            seq_len = None if past_key_values.device_length_mode else past_key_values._seen_tokens
            hidden_states = stack.step(hidden_states, position_ids, cache_position, seq_len,
                                       None if all_ones_mask else causal_mask)
        for decoder_layer in (self.layers if stack is None else ()):
            if output_hidden_states:
                all_hidden_states += (hidden_states,)
            layer_outputs = decoder_layer(
                hidden_states=hidden_states, attention_mask=causal_mask, position_ids=position_ids,
                past_key_value=past_key_values if use_cache else None, output_attentions=output_attentions,
                use_cache=use_cache, cache_position=cache_position, position_embeddings=position_embeddings,
                all_ones_mask=all_ones_mask, key_padding_mask=key_padding_mask)
            hidden_states = layer_outputs[0]
            if output_attentions:
                all_self_attns += (layer_outputs[1],)

        if not skip_final_norm:
            hidden_states = self.norm(hidden_states)
        if output_hidden_states:
            all_hidden_states += (hidden_states,)
        if use_cache and isinstance(past_key_values, MuiCache):
            past_key_values.sync_back()
        return MuiModelOutput(last_hidden_state=hidden_states,
                              past_key_values=past_key_values if use_cache else None,
                              hidden_states=all_hidden_states, attentions=all_self_attns)


class MuiLlamaForCausalLM(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, config, model: MuiLlamaModel, lm_head: MuiLinear):
        super().__init__(engine_config=engine_config)
        self.config = config
        self.model = model
        self.vocab_size = config.vocab_size
        self.lm_head = lm_head
        self._graph_decoder = None

    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_model) -> "MuiLlamaForCausalLM":
        if isinstance(prev_model, MuiLlamaForCausalLM):
            return prev_model
        engine_config = replacement_context.engine_config
        new_lm_head = MuiLinear.replace(replacement_context, prev_model.lm_head)
        new_model = MuiLlamaModel.replace(replacement_context, prev_model.model)
        return MuiLlamaForCausalLM(engine_config, prev_model.config, new_model, new_lm_head)

    @staticmethod
    def from_config(engine_config: MuiEngineConfig, config, dtype=torch.float16, device="cuda", seed: int = 0,
                    init_std: float = 0.02, finalize: bool = True) -> "MuiLlamaForCausalLM":
        """Randomly initialised model (weights ~ N(0, init_std), norm weights 1) built layer by
        layer on `device`; no checkpoint involved."""
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        hid, inter = config.hidden_size, config.intermediate_size
        d = head_dim_of(config)
        hq = config.num_attention_heads
        hkv = config.num_key_value_heads if getattr(config, "num_key_value_heads", None) else hq
        eps = config.rms_norm_eps

        def rnd_(p):
            p.data.normal_(0.0, init_std, generator=gen)

        embed = MuiEmbedding(engine_config, config.vocab_size, hid, device=device, dtype=dtype)
        rnd_(embed.weight)
        layers = []
        for i in range(config.num_hidden_layers):
            qkv = MuiMultiLinear(engine_config, hid, [hq * d, hkv * d, hkv * d], bias=False,
                                 variance_epsilon=eps, normalize=True, device=device, dtype=dtype)
            rnd_(qkv.linear.weight)
            o_proj = MuiLinear(engine_config, hq * d, hid, bias=False, device=device, dtype=dtype)
            rnd_(o_proj.weight)
            rope = MuiRotaryEmbedding(engine_config, config, layer_idx=i, device=device, dtype=dtype)
            attn = MuiSdpaAttention(engine_config, config, rope, o_proj, layer_idx=i, device=device, dtype=dtype)
            mlp = MuiGateUpDownMLP(engine_config, hid, inter, nn.SiLU(), variance_epsilon=eps, normalize=True,
                                   device=device, dtype=dtype)
            rnd_(mlp.gate_proj.weight)
            rnd_(mlp.up_proj.weight)
            rnd_(mlp.down_proj.weight)
            layers.append(MuiDecoderLayer(engine_config, qkv, attn, mlp))
        norm = MuiRMSNorm(engine_config, hid, eps=eps, device=device, dtype=dtype)
        rotary = MuiRotaryEmbedding(engine_config, config, layer_idx=0, device=device, dtype=dtype)
        model = MuiLlamaModel(engine_config, config, embed, layers, norm, rotary)
        lm_head = MuiLinear(engine_config, hid, config.vocab_size, bias=False, device=device, dtype=dtype)
        rnd_(lm_head.weight)
        lm = MuiLlamaForCausalLM(engine_config, config, model, lm_head)
        lm.eval()
        if finalize:
            from ....engine import _finalize_module
            _finalize_module(lm)
        setattr(lm, "muillm_config", engine_config)
        return lm

    def get_input_embeddings(self):
        return self.model.embed_tokens

    def get_output_embeddings(self):
        return self.lm_head

    def forward(self, input_ids: torch.LongTensor = None, attention_mask: Optional[torch.Tensor] = None,
                position_ids: Optional[torch.LongTensor] = None, past_key_values=None,
                inputs_embeds: Optional[torch.Tensor] = None, labels=None, use_cache: Optional[bool] = None,
                output_attentions: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                return_dict: Optional[bool] = None, cache_position: Optional[torch.LongTensor] = None,
                all_ones_mask: Optional[bool] = None, num_logits_to_keep: int = 0, float_logits: bool = True):
        if labels is not None:
            raise NotImplementedError("inference only: labels/loss are not supported")
        shape = input_ids.shape if input_ids is not None else inputs_embeds.shape
        head, norm = self.lm_head, self.model.norm
        # single-token decode: the final RMSNorm rides inside the lm_head GEMV
        fuse_norm = (shape[1] == 1 and not output_hidden_states and type(head) is MuiLinear and head.dispatchable
                     and not head.normalize and norm.dispatchable and head.weight.dtype == norm.weight.dtype)
        outputs = self.model(
            input_ids=input_ids, attention_mask=attention_mask, position_ids=position_ids,
            past_key_values=past_key_values, inputs_embeds=inputs_embeds, use_cache=use_cache,
            output_attentions=output_attentions, output_hidden_states=output_hidden_states,
            cache_position=cache_position, all_ones_mask=all_ones_mask, skip_final_norm=fuse_norm)
        hidden_states = outputs.last_hidden_state
        if num_logits_to_keep:
            hidden_states = hidden_states[:, -num_logits_to_keep:, :]
        if fuse_norm and hidden_states.is_cuda:
            logits = muillm_ext.muillm_linear_forward(self.engine_config.cpp_engine, hidden_states, head.weight, norm.weight, norm.variance_epsilon,
                                                      None, head.bias, None)
        else:
            if fuse_norm:
                hidden_states = norm(hidden_states)
            logits = self.lm_head(hidden_states)
        if float_logits:
            logits = logits.float()
        return MuiCausalLMOutput(logits=logits, past_key_values=outputs.past_key_values,
                                 hidden_states=outputs.hidden_states, attentions=outputs.attentions)

    @torch.no_grad()
    def generate_greedy(self, input_ids: torch.LongTensor, max_new_tokens: int, use_graph: Optional[bool] = None,
                        cache: Optional[MuiStaticCache] = None, return_logits: bool = False):
        """Prefill on the prompt, then max_new_tokens greedy decode steps at the prompt's batch
        size. Returns int64 [B, prompt + max_new_tokens] (and, optionally, the per-step fp16
        logits of the decode steps).

        use_graph=True captures the decode step (model forward, argmax, position bookkeeping,
        all on the device) into a HIP graph and replays it; False enqueues the same step on the
        stream every time; None (default) lets the decoder choose (MuiGraphDecoder: stream launches
        when the layer stack is one library call, graph replay otherwise)."""
        dec = self._decoder_for(use_graph=use_graph)
        cache = self._reusable_cache(dec, cache, input_ids)
        return dec.generate(input_ids, max_new_tokens, cache=cache, return_logits=return_logits)

    def _decoder_for(self, **options):
        """The MuiGraphDecoder for these options; the last one is kept, so that repeated generate()
        calls replay the graph captured by the first instead of warming up and capturing again."""
        from ..graphdecoder import MuiGraphDecoder

        key = tuple(sorted((k, tuple(v) if isinstance(v, (list, tuple)) else v) for k, v in options.items()))
        if self._graph_decoder is None or self._graph_decoder[0] != key:
            self._graph_decoder = (key, MuiGraphDecoder(self, **options))
        return self._graph_decoder[1]

    @staticmethod
    def _reusable_cache(dec, cache, input_ids):
        """Without a cache from the caller, a kept decoder starts again on its own (emptied) cache
        when the batch size fits: same buffers, so its captured graph stays valid. A cache that a
        caller handed to an earlier call is the caller's (multi-turn state) and is never touched."""
        if cache is None and dec.cache is not None and dec.owns_cache \
                and dec.cache.max_batch_size == input_ids.shape[0] \
                and dec.cache.key_cache[0].device == input_ids.device:
            dec.cache.reset()
            return dec.cache
        return cache

    @torch.no_grad()
    def generate(self, input_ids: torch.LongTensor = None, attention_mask: Optional[torch.Tensor] = None,
                 max_new_tokens: int = 20, do_sample: bool = False, temperature: float = 1.0,
                 top_k: Optional[int] = None, top_p: Optional[float] = None,
                 eos_token_id=None, pad_token_id: Optional[int] = None, seed: int = 0, use_graph: Optional[bool] = None,
                 cache: Optional[MuiStaticCache] = None, **unused):
        """HuggingFace-style entry point over the device-resident decode loop (the reference routes
        generate() through its MuiGenerationMixin._sample, muillm/sampling/generation.py:77-408).
        Greedy (do_sample=False) or temperature sampling; left-padded batches via attention_mask;
        rows stop at eos_token_id (int or list) and are filled with pad_token_id afterwards.
        Returns int64 [B, prompt_len + max_new_tokens]. top_k / top_p filter the logits with torch
        ops in front of the sampling kernel (the loop then runs eagerly instead of from the HIP
        graph); other logit processors (penalties, ...) are not part of this loop."""
        dropped = {k: v for k, v in unused.items() if v is not None and k in ("repetition_penalty", "num_beams")}
        if dropped:
            raise NotImplementedError(f"generate(): unsupported options {sorted(dropped)}")
        eos = None
        if eos_token_id is not None:
            eos = [int(eos_token_id)] if isinstance(eos_token_id, int) else [int(e) for e in eos_token_id]
        if pad_token_id is None:
            pad_token_id = eos[0] if eos else 0
        dec = self._decoder_for(use_graph=use_graph, eos_token_ids=eos, pad_token_id=pad_token_id,
                                do_sample=do_sample, temperature=temperature, seed=seed,
                                top_k=top_k if do_sample else None, top_p=top_p if do_sample else None)
        cache = self._reusable_cache(dec, cache, input_ids)
        # with an eos criterion the loop polls, without blocking, whether every row has finished
        return dec.generate(input_ids, max_new_tokens, cache=cache, attention_mask=attention_mask,
                            stop_check_every=8 if eos else 0)


# Mistral shares the Llama implementation; config.sliding_window, where set, goes into the attention
# mask once a sequence outgrows it (forward() above; the reference's mistral/model.py:484,593-602)
MuiMistralModel = MuiLlamaModel
MuiMistralForCausalLM = MuiLlamaForCausalLM
