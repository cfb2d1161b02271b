"""MuiRotaryEmbedding -- muillm/modules/attention/rotaryembedding.py:23-464 (Llama/Mistral
rotate-half RoPE; the Llama-4 complex variant is not part of this build).

Tables: inv_freq from the rope type ('default', 'linear', 'llama3'), freqs = outer(arange(max_pos),
inv_freq) in fp32, emb = cat(freqs, freqs), cos/sin scaled by attention_scaling. cos_cached /
sin_cached are kept in the requested dtype like the reference's; the kernels read fp32
tables built from the same fp32 angles (no 16-bit rounding of cos/sin). The fp32 tables are
shared between the per-layer modules of a model instead of being rebuilt 32 times."""
import math
from typing import Any, Dict, Optional, Tuple

import torch

from ... import muillm_ext
from ..._hf import LlamaRotaryEmbedding, MistralRotaryEmbedding, head_dim_of, rope_scaling_of, rope_theta_of
from ...engineconfig import MuiEngineConfig
from ...replacement.replacementcontext import MuiReplacementContext
from ..kvcache.cache_utils import MuiCache
from ..module import MuiModule


def rotate_half(x):
    """Rotates half the hidden dims of the input."""
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim: int = 1):
    """q' = q*cos + rotate_half(q)*sin with cos/sin [B, T, D] broadcast over heads."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def _default_inv_freq(theta: float, dim: int, device=None) -> torch.Tensor:
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64, device=device).to(torch.float32) / dim))


def compute_rope_inv_freq(rope_type: str, theta: float, dim: int, scaling: Optional[Dict[str, Any]] = None,
                          device=None) -> Tuple[torch.Tensor, float]:
    """(inv_freq [dim/2] fp32, attention_scaling) for the supported rope types, restating the
    published HuggingFace ROPE_INIT_FUNCTIONS formulas."""
    inv_freq = _default_inv_freq(theta, dim, device)
    if rope_type in (None, "default"):
        return inv_freq, 1.0
    if rope_type == "linear":
        return inv_freq / float(scaling["factor"]), 1.0
    if rope_type == "llama3":
        factor = float(scaling["factor"])
        low_freq_factor = float(scaling["low_freq_factor"])
        high_freq_factor = float(scaling["high_freq_factor"])
        old_context_len = float(scaling["original_max_position_embeddings"])
        low_freq_wavelen = old_context_len / low_freq_factor
        high_freq_wavelen = old_context_len / high_freq_factor
        wavelen = 2 * math.pi / inv_freq
        inv_freq_llama = torch.where(wavelen > low_freq_wavelen, inv_freq / factor, inv_freq)
        smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        smoothed = (1 - smooth) * inv_freq_llama / factor + smooth * inv_freq_llama
        is_medium = ~(wavelen < high_freq_wavelen) * ~(wavelen > low_freq_wavelen)
        return torch.where(is_medium, smoothed, inv_freq_llama), 1.0
    raise ValueError(f"unsupported rope type {rope_type!r}")


_SHARED_TABLES: Dict[tuple, Tuple[torch.Tensor, torch.Tensor]] = {}


def _shared_f32_tables(key, inv_freq: torch.Tensor, max_pos: int, attention_scaling: float, device):
    """fp32 [max_pos, dim/2] cos/sin on `device`, one copy per distinct rope configuration."""
    full_key = key + (str(device),)
    hit = _SHARED_TABLES.get(full_key)
    if hit is not None:
        return hit
    t = torch.arange(max_pos, device=inv_freq.device, dtype=torch.int64).type_as(inv_freq)
    freqs = torch.outer(t, inv_freq)
    cos = (freqs.cos() * attention_scaling).to(device=device, dtype=torch.float32).contiguous()
    sin = (freqs.sin() * attention_scaling).to(device=device, dtype=torch.float32).contiguous()
    _SHARED_TABLES[full_key] = (cos, sin)
    return cos, sin


class _MuiRotaryNoCache(torch.autograd.Function):
    @staticmethod
    def forward(ctx, positions_ids, cos_cached, sin_cached, q, k):
        return muillm_ext.muillm_rope_forward_no_cache(positions_ids, cos_cached, sin_cached, q, k)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("rotary backward not implemented")


def is_hf_static_cache(cache) -> bool:
    """A HuggingFace StaticCache of either generation (see _hf_static_cache_layer)."""
    if cache is None or isinstance(cache, MuiCache):
        return False
    layers = getattr(cache, "layers", None)
    if isinstance(layers, (list, tuple)) and len(layers) > 0:
        return all(type(layer).__name__ == "StaticLayer" for layer in layers)
    return isinstance(getattr(cache, "key_cache", None), list) and hasattr(cache, "max_cache_len")


def _hf_static_cache_layer(cache, layer_idx: int, k: torch.Tensor, v: torch.Tensor, cache_position=None):
    """(k_cache, v_cache, seen tokens after this update) of a HuggingFace StaticCache, or None for
    any other object. Two generations of that class are recognised by their attributes: per-layer
    objects (`cache.layers[i]` of type StaticLayer with `keys` / `values` / `max_cache_len`, allocated
    on first use, a device-side `cumulative_length`) and the older lists `key_cache` / `value_cache`
    with `max_cache_len`. The seen-token count is read from cache_position by the first layer (one
    device-to-host copy per forward; the reference keeps a counter on the cache object,
    rotaryembedding.py:394-396 there, which a reset of the cache would leave stale) and kept on the
    cache object for the other layers; the per-layer length counter of the newer class is advanced
    as its own update() would."""
    new_tokens = k.shape[-2]
    layers = getattr(cache, "layers", None)
    if isinstance(layers, (list, tuple)) and layer_idx < len(layers) and type(layers[layer_idx]).__name__ == "StaticLayer":
        layer = layers[layer_idx]
        if not getattr(layer, "is_initialized", True):
            layer.lazy_initialization(k, v)
        k_cache, v_cache = layer.keys, layer.values
        if isinstance(getattr(layer, "cumulative_length", None), torch.Tensor):
            layer.cumulative_length.add_(new_tokens)
    elif isinstance(getattr(cache, "key_cache", None), list) and hasattr(cache, "max_cache_len") \
            and layer_idx < len(cache.key_cache) and not isinstance(cache, MuiCache):
        k_cache, v_cache = cache.key_cache[layer_idx], cache.value_cache[layer_idx]
    else:
        return None
    if not (torch.is_tensor(k_cache) and k_cache.dim() == 4 and k_cache.shape == v_cache.shape
            and k_cache.dtype == k.dtype and k_cache.device == k.device and k_cache.stride(3) == 1):
        return None
    if cache_position is None:
        raise ValueError("cache_position is needed")
    if layer_idx == 0 or not hasattr(cache, "_mui_seen_tokens"):
        cache._mui_seen_tokens = int(cache_position.reshape(-1)[-1]) + 1
    return k_cache, v_cache, min(int(cache._mui_seen_tokens), k_cache.shape[2])


class _MuiRotaryCacheModule(torch.autograd.Function):
    @staticmethod
    def forward(ctx, module, cache, q, k, v, position_ids, cos_sin, cache_positions):
        return muillm_ext.muillm_rotary_embedding_module_forward(
            module, cache, q, k, v, position_ids, cos_sin, cache_positions)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("rotary backward not implemented")


class MuiRotaryEmbedding(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, config, rope_kwargs: Dict[str, Any] = None,
                 layer_idx: int = 0, output_complex: Optional[bool] = None, device=None, dtype=None):
        super().__init__(engine_config=engine_config)
        if output_complex:
            raise ValueError("complex (Llama-4) rotary embeddings are not part of this build")
        self.cpp_engine = engine_config.cpp_engine
        self.config = config
        self.rope_kwargs = {}
        self.output_complex = False
        self.layer_idx = layer_idx
        dtype = dtype if dtype is not None else torch.float32

        if config is not None:
            scaling = rope_scaling_of(config)
            self.rope_type = "default" if scaling is None else scaling.get("rope_type", scaling.get("type", "default"))
            theta = rope_theta_of(config)
            dim = head_dim_of(config)
            max_position_embeddings = config.max_position_embeddings
        else:
            if rope_kwargs is None:
                raise ValueError("Either config or rope_kwargs should be not None")
            self.rope_kwargs = rope_kwargs
            self.rope_type = rope_kwargs.get("rope_type", "default")
            scaling = rope_kwargs
            theta = float(rope_kwargs.get("base", rope_kwargs.get("rope_theta", 10000.0)))
            dim = int(rope_kwargs["dim"])
            max_position_embeddings = rope_kwargs["max_position_embeddings"]

        self.max_position_embeddings = max_position_embeddings
        self.rope_theta = theta
        self.head_dim = dim
        inv_freq, self.attention_scaling = compute_rope_inv_freq(self.rope_type, theta, dim, scaling, device)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        self._table_key = (self.rope_type, float(theta), int(dim), int(max_position_embeddings),
                           tuple(sorted((k, str(v)) for k, v in (scaling or {}).items())))
        self._set_cos_sin_cache(seq_len=max_position_embeddings, device=device, dtype=dtype)
        self.dtype = dtype
        self._check_dispatchable()
        self.cpp_module = None

    def _check_dispatchable(self):
        self.dispatchable = self.inv_freq.is_cuda and self.dtype in (torch.float16, torch.bfloat16) \
            and self.head_dim == 128

    def _set_cos_sin_cache(self, seq_len, device, dtype):
        self.max_seq_len_cached = seq_len
        cos32, sin32 = _shared_f32_tables(self._table_key, self.inv_freq, seq_len, self.attention_scaling,
                                          self.inv_freq.device)
        self.cos32, self.sin32 = cos32, sin32  # [max_pos, dim/2] fp32, shared between layers
        # the reference's [max_pos, dim] tables in the module dtype (views would not survive
        # the dtype change, so these are per-dtype copies, again shared through the buffers)
        self.register_buffer("cos_cached", torch.cat((cos32, cos32), dim=-1).to(dtype), persistent=False)
        self.register_buffer("sin_cached", torch.cat((sin32, sin32), dim=-1).to(dtype), persistent=False)

    def finalize_init(self):
        dev = self.inv_freq.device
        if self.cos32.device != dev:
            self.cos32, self.sin32 = _shared_f32_tables(self._table_key, self.inv_freq, self.max_seq_len_cached,
                                                        self.attention_scaling, dev)
        self._check_dispatchable()
        if self.cpp_module is not None:
            muillm_ext.muillm_rotary_embedding_module_deinit(self.cpp_module)
        self.cpp_module = muillm_ext.MuiRotaryModuleHandle.__new__(muillm_ext.MuiRotaryModuleHandle)
        self.cpp_module.engine = self.cpp_engine
        self.cpp_module.layer_idx = self.layer_idx
        self.cpp_module.cos_cached = self.cos_cached
        self.cpp_module.sin_cached = self.sin_cached
        self.cpp_module.cos32 = self.cos32
        self.cpp_module.sin32 = self.sin32

    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_module) -> "MuiRotaryEmbedding":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiRotaryEmbedding):
            return prev_module
        if not isinstance(prev_module, (LlamaRotaryEmbedding, MistralRotaryEmbedding)):
            raise ValueError(f"Unsupported type of module: {prev_module.__class__.__name__}")
        return MuiRotaryEmbedding(engine_config=engine_config, config=prev_module.config, device=device,
                                  dtype=prev_module.inv_freq.dtype)

    def forward(self, x, position_ids):
        """cos, sin gathered at position_ids: [B, T, D] in x's dtype."""
        dtype = x.dtype
        return self.cos_cached[position_ids].to(dtype=dtype), self.sin_cached[position_ids].to(dtype=dtype)

    def apply_rotary_pos_emb_write_kv_cache(self, q: torch.Tensor, k: torch.Tensor, position_ids: torch.Tensor,
                                            position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]],
                                            v: Optional[torch.Tensor] = None, cache=None,
                                            cache_position: Optional[torch.LongTensor] = None):
        """q/k/v [B, H, T, D] -> (q_rot, keys, values); with a cache the new k/v are written
        at cache_position and keys/values are the cache narrowed to the seen tokens."""
        kernel_ok = self.dispatchable and q.is_cuda and q.dtype in (torch.float16, torch.bfloat16) \
            and self.cpp_module is not None
        if kernel_ok:
            if cache is None:
                q_out, k_out = _MuiRotaryNoCache.apply(position_ids, self.cos32, self.sin32, q, k)
                return q_out, k_out, v
            if isinstance(cache, MuiCache):
                if cache_position is None:
                    raise ValueError("cache_position is needed")
                return _MuiRotaryCacheModule.apply(self.cpp_module, cache.cpp_module, q, k, v, position_ids,
                                                   position_embeddings, cache_position)
            hf_static = _hf_static_cache_layer(cache, self.layer_idx, k, v, cache_position)
            if hf_static is not None:
                # HuggingFace's StaticCache (muillm/modules/attention/rotaryembedding.py:392-418 of the
                # reference): its per-layer buffers are written in place by the same kernel
                k_cache, v_cache, seen = hf_static
                return muillm_ext.muillm_rope_forward_static_cache(
                    position_ids, self.cos32, self.sin32, q, k, v, k_cache, v_cache, cache_position, seen)
            raise ValueError(f"Unsupported cache type: {type(cache).__name__}")

        if position_embeddings is None:
            cos, sin = self.forward(k, position_ids)
        else:
            cos, sin = position_embeddings
        query_states, key_states = apply_rotary_pos_emb(q, k, cos, sin)
        value_states = v
        if cache is not None:
            cache_kwargs = {"sin": sin, "cos": cos, "cache_position": cache_position}
            key_states, value_states = cache.update(key_states, v, self.layer_idx, cache_kwargs)
        return query_states, key_states, value_states
