"""All decoder layers of a decode step through one library call.

The reference walks its layers from C++ only under tensor parallelism
(muillm/modules/models/llama/model.py:331-358 -> csrc/modules/parallel_decoder_stack.cpp); on
one GPU it calls its Python layer modules one by one (muillm/modules/decoder/decoder.py:130-165).
Here `mui_decoder_stack_step` enqueues the same per-layer sequence for every layer, so a step
that is not replayed from a HIP graph pays the host cost of one call instead of ~160.
"""
import ctypes
from typing import Optional

import torch
import torch.nn as nn

from ... import _lib, muillm_ext
from ..attention.baseattention import MuiBaseAttention
from ..gateupdownmlp import MuiGateUpDownMLP
from ..kvcache.cache_utils import MuiStaticCache
from ..linear import MuiLinear
from ..multilinear import MuiMultiLinear
from ..quantized.int8gateupdownmlp import MuiInt8GateUpDownMLP
from ..quantized.int8linear import MuiInt8Linear


def _group_shift(m) -> int:
    """0 for a 16-bit or per-channel int8 module, the group size's log2 for the group format."""
    if type(m) is MuiInt8Linear and not m.per_channel:
        return int(m.quantizer.group_size_shift)
    if type(m) is MuiInt8GateUpDownMLP and not m.per_channel:
        return int(m.group_size_shift)
    return 0


def _plain_linear(m, normalize: Optional[bool] = None) -> bool:
    """A bias-free MuiLinear, or a bias-free MuiInt8Linear (per-channel, or the group format with
    groups of at least 16 that divide the rows)."""
    if type(m) is MuiInt8Linear:
        if m.bias is not None or not m.dispatchable or (normalize is not None and bool(m.normalize) != normalize):
            return False
        if m.per_channel:
            return m.weights_int8.is_contiguous() and m.scales.is_contiguous()
        return (m.quantizer.group_size_shift >= 4 and m.in_features % 16 == 0 and m.weights_uint8.is_contiguous()
                and m.scales_min_vals.is_contiguous())
    return (type(m) is MuiLinear and m.bias is None and m.weight.is_cuda and m.weight.stride(1) == 1
            and (normalize is None or bool(m.normalize) == normalize))


def _linear_fields(m):
    """(weight tensor, row pitch, scales tensor or None, [(owner, attribute, object)]) of a projection;
    "scales" are per-channel scales or, in the group format, the (scale, min) pairs."""
    if type(m) is MuiInt8Linear:
        if m.per_channel:
            return m.weights_int8, m.weights_int8.stride(0), m.scales, [(m, "weights_int8", m.weights_int8),
                                                                         (m, "scales", m.scales)]
        return m.weights_uint8, m.weights_uint8.stride(0), m.scales_min_vals, [
            (m, "weights_uint8", m.weights_uint8), (m, "scales_min_vals", m.scales_min_vals)]
    return m.weight, m.weight.stride(0), None, [(m, "weight", m.weight)]


def _ptr(t) -> Optional[int]:
    return None if t is None else t.data_ptr()


class MuiDecoderStack:
    """Descriptor + workspace of `mui_decoder_stack_step` for one model, cache and batch size.

    Holds plain pointers: it has to be rebuilt when the cache is re-allocated (`matches`)."""

    def __init__(self, layers, rotary_emb, cache: MuiStaticCache, batch: int):
        self.lib = _lib.load()
        first = layers[0]
        attn0: MuiBaseAttention = first.self_attn
        self.dtype, self.device = first.qkv_proj.linear.norm_weights.dtype, first.qkv_proj.linear.norm_weights.device
        self.batch = batch
        self.hidden = first.qkv_proj.linear.in_features
        self.hq, self.hkv, self.d = attn0.num_heads, attn0.num_key_value_heads, attn0.head_dim
        self.cos32, self.sin32 = rotary_emb.cos32, rotary_emb.sin32
        kc0 = cache.key_cache[0]
        cb, chs, cts = kc0.stride(0), kc0.stride(1), kc0.stride(2)
        self.max_cache_len = kc0.shape[2]
        self._cache_ptrs = tuple(t.data_ptr() for t in cache.key_cache) + tuple(t.data_ptr() for t in cache.value_cache)
        self._keep = []  # tensors the descriptor points into
        self._layer_list = layers
        self._owners = []  # (module, attribute name, object) the descriptor was built from
        arr = (_lib.MuiDecoderLayerDesc * len(layers))()
        for i, layer in enumerate(layers):
            qkv, attn, mlp = layer.qkv_proj.linear, layer.self_attn, layer.mlp
            kc, vc = cache.key_cache[attn.layer_idx], cache.value_cache[attn.layer_idx]
            if (kc.stride(), vc.stride()) != (kc0.stride(), kc0.stride()):
                raise ValueError("cache layers must share one layout")
            qw, qp, qs, q_own = _linear_fields(qkv)
            ow, op, osc, o_own = _linear_fields(attn.o_proj)
            dw, dp, ds, d_own = _linear_fields(mlp.down_proj)
            shift = max(_group_shift(m) for m in (qkv, attn.o_proj, mlp, mlp.down_proj))
            if type(mlp) is MuiInt8GateUpDownMLP:
                gu = mlp.gate_up_weights  # [inter, 2, hidden] codes
                g_ptr, u_ptr, g_pitch = gu.data_ptr(), gu.data_ptr() + gu.stride(1), gu.stride(0)
                if mlp.per_channel:
                    gs, gs_name = mlp.gate_up_scales, "gate_up_scales"  # [inter, 2] scales
                else:
                    gs, gs_name = mlp.gate_up_scales_min_vals, "gate_up_scales_min_vals"  # [inter, 2, G, 2] pairs
                gs_ptr, us_ptr = gs.data_ptr(), gs.data_ptr() + gs.stride(1) * gs.element_size()
                gs_stride = gs.stride(0)
                gu_keep = [gu, gs]
                gu_own = [(mlp, "gate_up_weights", gu), (mlp, gs_name, gs)]
            else:
                g, u = mlp.gate_proj.weight, mlp.up_proj.weight
                g_ptr, u_ptr, g_pitch = g.data_ptr(), u.data_ptr(), g.stride(0)
                gs_ptr, us_ptr, gs_stride = None, None, 0
                gu_keep = [g, u]
                gu_own = [(mlp.gate_proj, "weight", g), (mlp.up_proj, "weight", u)]
            arr[i] = _lib.MuiDecoderLayerDesc(
                qkv.norm_weights.data_ptr(), qw.data_ptr(), qp, ow.data_ptr(), op,
                mlp.norm_weights.data_ptr(), g_ptr, u_ptr, g_pitch, dw.data_ptr(), dp, kc.data_ptr(), vc.data_ptr(),
                _ptr(qs), _ptr(osc), gs_ptr, us_ptr, gs_stride, _ptr(ds), shift)
            self._keep += [qkv.norm_weights, qw, qs, ow, osc, mlp.norm_weights, dw, ds, kc, vc] + gu_keep
            self._owners += [(layer, "qkv_proj", layer.qkv_proj), (layer, "self_attn", attn), (layer, "mlp", mlp),
                             (layer.qkv_proj, "linear", qkv), (qkv, "norm_weights", qkv.norm_weights),
                             (attn, "o_proj", attn.o_proj), (mlp, "norm_weights", mlp.norm_weights),
                             (mlp, "down_proj", mlp.down_proj)] + q_own + o_own + d_own + gu_own
        self._layers = arr
        self.desc = _lib.MuiDecoderStackDesc(
            muillm_ext._dtype_code(first.qkv_proj.linear.norm_weights), len(layers), self.hidden, self.hq, self.hkv,
            self.d, first.mlp.intermediate_size, float(first.qkv_proj.linear.variance_epsilon),
            ctypes.cast(arr, ctypes.POINTER(_lib.MuiDecoderLayerDesc)), self.cos32.data_ptr(), self.sin32.data_ptr(),
            self.cos32.stride(0), self.cos32.shape[0], cb, chs, cts, self.max_cache_len)
        self._ws = None
        self._ws_splits = 0

    @staticmethod
    def eligible(layers, rotary_emb, cache, batch: int) -> bool:
        """fp16 / bf16 Llama-shaped layers without biases on a static cache, head_dim 128; every
        projection 16-bit or int8 (per-channel, or the reference's group format)."""
        if not isinstance(cache, MuiStaticCache) or len(layers) == 0 or batch > _lib.MUI_MAX_TOKENS:
            return False
        if not getattr(rotary_emb, "dispatchable", False):
            return False
        eps, dtype = None, None
        for layer in layers:
            qkv, attn, mlp = getattr(layer, "qkv_proj", None), getattr(layer, "self_attn", None), getattr(layer, "mlp", None)
            if type(qkv) is not MuiMultiLinear or not _plain_linear(qkv.linear, True):
                return False
            if not isinstance(attn, MuiBaseAttention) or not _plain_linear(attn.o_proj, False):
                return False
            if attn.head_dim != 128:
                return False
            if type(mlp) is MuiGateUpDownMLP:
                if not all(_plain_linear(m, False) and type(m) is MuiLinear for m in (mlp.gate_proj, mlp.up_proj)):
                    return False
                if mlp.gate_proj.weight.stride(0) != mlp.up_proj.weight.stride(0):
                    return False
            elif type(mlp) is MuiInt8GateUpDownMLP:
                if not (mlp.dispatchable and mlp.gate_up_weights.is_contiguous()):
                    return False
                sc = mlp.gate_up_scales if mlp.per_channel else mlp.gate_up_scales_min_vals
                if not sc.is_contiguous() or (not mlp.per_channel and mlp.group_size_shift < 4):
                    return False
            else:
                return False
            if not mlp.normalize or not isinstance(mlp.activation_function, nn.SiLU):
                return False
            if not _plain_linear(mlp.down_proj, False):
                return False
            w = qkv.linear.norm_weights
            if w is None or mlp.norm_weights is None or w.dtype not in (torch.float16, torch.bfloat16):
                return False
            if cache.key_cache[attn.layer_idx].dtype != w.dtype or (dtype is not None and w.dtype != dtype):
                return False
            dtype = w.dtype
            for m in (qkv.linear, attn.o_proj, mlp.down_proj):
                if type(m) is MuiInt8Linear:
                    wd = m.scales.dtype if m.per_channel else m.scales_min_vals.dtype
                else:
                    wd = m.weight.dtype
                if wd != dtype:
                    return False
            # the int8 projections of a layer share one format: all per-channel, or all in the group
            # format with one group size (the layer descriptor carries a single shift)
            int8_mods = [m for m in (qkv.linear, attn.o_proj, mlp, mlp.down_proj)
                         if type(m) in (MuiInt8Linear, MuiInt8GateUpDownMLP)]
            if len({_group_shift(m) for m in int8_mods}) > 1:
                return False
            e = (float(qkv.linear.variance_epsilon), float(mlp.variance_epsilon))
            if e[0] != e[1] or (eps is not None and e != eps):
                return False
            eps = e
        return True

    def matches(self, layers, cache: MuiStaticCache, batch: int) -> bool:
        """Still valid for this step? The cache tensors are where they were, and every module and
        parameter the descriptor was built from is still the object in place (a later
        quantize_layers / .to() / weight swap replaces them)."""
        if batch != self.batch or layers is not self._layer_list:
            return False
        for owner, name, obj in self._owners:
            if getattr(owner, name, None) is not obj:
                return False
        ptrs = tuple(t.data_ptr() for t in cache.key_cache) + tuple(t.data_ptr() for t in cache.value_cache)
        return ptrs == self._cache_ptrs

    def step(self, hidden_in: torch.Tensor, position_ids: torch.Tensor, cache_position: torch.Tensor,
             seq_len: Optional[int], mask: Optional[torch.Tensor]) -> torch.Tensor:
        """hidden_in [B, 1, hidden] -> output of the last layer [B, 1, hidden]."""
        lib, b = self.lib, self.batch
        x = hidden_in.reshape(b, self.hidden)
        if not x.is_contiguous():
            x = x.contiguous()
        hint = seq_len if seq_len is not None else self.max_cache_len
        n_splits = lib.mui_flash_decode_splits(b, self.hq, self.hkv, int(hint))
        if self._ws is None or n_splits > self._ws_splits:
            nbytes = lib.mui_decoder_stack_workspace_bytes(ctypes.byref(self.desc), b, n_splits)
            self._ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=self.device)
            self._ws_splits = n_splits
        ws_ptr = (self._ws.data_ptr() + 255) & ~255
        pos = position_ids.reshape(-1)
        if pos.dtype != torch.int64 or cache_position.dtype != torch.int64:
            raise RuntimeError("position_ids and cache_position must be int64")
        mask_ptr, mask_bs = None, 0
        if mask is not None:
            mask = muillm_ext._mask_rows(mask, b, x.dtype)
            mask_ptr, mask_bs = mask.data_ptr(), mask.stride(0)
        out = torch.empty((b, 1, self.hidden), dtype=x.dtype, device=x.device)
        muillm_ext.check(
            lib.mui_decoder_stack_step(muillm_ext._stream(x), ctypes.byref(self.desc), b, x.data_ptr(), out.data_ptr(),
                                       pos.data_ptr(), 1 if pos.numel() > 1 else 0, cache_position.data_ptr(),
                                       -1 if seq_len is None else int(seq_len), mask_ptr, mask_bs, n_splits, ws_ptr),
            "mui_decoder_stack_step")
        return out
