"""Static KV cache -- muillm/modules/kvcache/cache_utils.py:47-52,113-288,681-719.

Per layer key_cache[l], value_cache[l]: [max_batch, n_kv_heads, max_cache_len, head_dim],
zero-initialised, capacity a power of two; `_seen_tokens` is a host counter bumped once per
model step (on layer 0). The reference derives this class from HuggingFace's StaticCache;
this one depends on torch only (the HF constructor changed between versions) and keeps the
same fields and methods."""
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from ... import muillm_ext
from ..._hf import head_dim_of
from ...engineconfig import MuiEngineConfig


def _get_num_key_value_heads(config) -> int:
    kvh = getattr(config, "num_key_value_heads", None)
    return config.num_attention_heads if kvh is None else kvh


class MuiCache:
    def sync_back(self):
        pass


class MuiStaticCache(MuiCache):
    def __init__(self, engine_config: MuiEngineConfig, config, max_batch_size: int,
                 max_cache_len: Optional[int] = None, device: Union[torch.device, str, None] = None,
                 dtype: torch.dtype = torch.float32, tensor_parallelism: int = 1) -> None:
        if tensor_parallelism != 1:
            raise ValueError("tensor parallelism is not supported by this build")
        self.engine_config = engine_config
        self.cpp_engine = engine_config.cpp_engine
        self.max_batch_size = max_batch_size
        self.max_cache_len = config.max_position_embeddings if max_cache_len is None else max_cache_len
        self.head_dim = head_dim_of(config)
        self.num_key_value_heads = _get_num_key_value_heads(config)
        self.dtype = dtype
        self.device = device
        shape = (max_batch_size, self.num_key_value_heads, self.max_cache_len, self.head_dim)
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        for _ in range(config.num_hidden_layers):
            self.key_cache.append(torch.zeros(shape, dtype=dtype, device=device))
            self.value_cache.append(torch.zeros(shape, dtype=dtype, device=device))
        self._seen_tokens = 0
        # When True the decode kernels take the sequence length from the device-resident
        # cache_position instead of this host counter (set by the HIP-graph decode runner).
        self.device_length_mode = False
        self.cpp_module = None
        self.finalize_init()

    def finalize_init(self):
        if self.cpp_module is not None:
            muillm_ext.muillm_static_kvcache_module_deinit(self.cpp_module)
        self.cpp_module = muillm_ext.muillm_static_kvcache_module_init(
            self.cpp_engine, self.key_cache, self.value_cache, self._seen_tokens)

    def _sync_seen_tokens(self):
        if self.cpp_module is not None:
            self._seen_tokens = muillm_ext.muillm_kvcache_module_get_set_seen_tokens(
                self.cpp_module, self._seen_tokens)

    def sync_back(self):
        self.key_cache, self.value_cache = muillm_ext.muillm_static_kvcache_module_sync_back(self.cpp_module)
        self._sync_seen_tokens()

    def __len__(self):
        return len(self.key_cache)

    def _kernel_ok(self, t: torch.Tensor) -> bool:
        return t.is_cuda and t.dtype in (torch.float16, torch.bfloat16) and self.head_dim == 128

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Write the new rows at cache_kwargs['cache_position'] (dim 2) and return the caches
        narrowed to the tokens seen so far (cache_utils.py:185-204 of the reference)."""
        cache_position = None if cache_kwargs is None else cache_kwargs.get("cache_position")
        if cache_position is None:
            cache_position = torch.arange(self._seen_tokens, self._seen_tokens + key_states.shape[-2],
                                          device=key_states.device)
        k_out, v_out = self.key_cache[layer_idx], self.value_cache[layer_idx]
        if layer_idx == 0:
            self._seen_tokens += key_states.shape[-2]
            self._sync_seen_tokens()
        if self._kernel_ok(key_states) and key_states.dtype == k_out.dtype:
            return muillm_ext.muillm_static_kvcache_update(k_out, v_out, key_states, value_states,
                                                           cache_position, self._seen_tokens)
        k_out.index_copy_(2, cache_position, key_states.to(k_out.dtype))
        v_out.index_copy_(2, cache_position, value_states.to(v_out.dtype))
        return torch.narrow(k_out, 2, 0, self._seen_tokens), torch.narrow(v_out, 2, 0, self._seen_tokens)

    def grow_cache(self, capacity: int, max_capacity: int) -> None:
        """Grow to the next power of two >= capacity (capped), keeping the contents."""
        required_capacity = min(_next_pow2(capacity), max_capacity)
        if self.max_cache_len >= required_capacity:
            return
        diff = required_capacity - self.max_cache_len
        for layer_idx in range(len(self.key_cache)):
            prev_k, prev_v = self.key_cache[layer_idx], self.value_cache[layer_idx]
            b, h, _, d = prev_k.shape
            pad_k = torch.zeros((b, h, diff, d), dtype=prev_k.dtype, device=prev_k.device)
            pad_v = torch.zeros((b, h, diff, d), dtype=prev_v.dtype, device=prev_v.device)
            self.key_cache[layer_idx] = torch.cat([prev_k, pad_k], dim=-2)
            self.value_cache[layer_idx] = torch.cat([prev_v, pad_v], dim=-2)
            del prev_k, prev_v
        self.max_cache_len = required_capacity
        self.finalize_init()  # the kernel-side handle aliases the tensors: rebuild it

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        """Tokens seen so far; a host counter, so no CPU<->GPU sync."""
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        return self.max_cache_len

    def get_max_cache_shape(self) -> Optional[int]:
        return self.max_cache_len

    def reset(self):
        for k, v in zip(self.key_cache, self.value_cache):
            k.zero_()
            v.zero_()
        self._seen_tokens = 0
        if self.cpp_module is not None:
            self.cpp_module.seen_tokens = 0


def _next_pow2(x: int) -> int:
    if x < 0:
        raise ValueError("x should be positive")
    p = 1
    while p < x:
        p = p * 2
    return p


def create_static_cache(engine_config: MuiEngineConfig, config, max_batch_size, seq_len, device, dtype) -> MuiStaticCache:
    """Capacity follows a power-of-two schedule to avoid frequent re-allocation."""
    return MuiStaticCache(engine_config=engine_config, config=config, max_cache_len=_next_pow2(seq_len),
                          device=device, dtype=dtype, tensor_parallelism=engine_config.tensor_parallelism,
                          max_batch_size=max_batch_size)


def grow_static_cache_if_needed(cache: MuiStaticCache, capacity: int, max_capacity: int) -> MuiStaticCache:
    cache.grow_cache(capacity=capacity, max_capacity=max_capacity)
    return cache
