"""Round-to-nearest weight quantisers (host side, run once per layer).

RTNQuantizer follows muillm/quantization/rtnquantizer.py:12-102 (asymmetric, group-wise,
unsigned 8 bit). ChannelRTNQuantizer is the symmetric per-output-channel int8 rule of the
int8 decode GEMVs: s = half(max|row| / 127), q = clamp(round_half_even(w / s), -127, 127)."""
import math
from typing import Tuple

import torch


def _ispow2(x: int) -> bool:
    return x != 0 and (x & (x - 1)) == 0


class RTNQuantizer:
    def __init__(self, n_bit: int = 8, groupsize: int = 128, min_bias=0, max_bias=0, f=1.0):
        if n_bit != 8:
            raise ValueError("only 8-bit RTN is supported")
        if not _ispow2(groupsize):
            raise ValueError(
                f"RTNQuantizer only supports power of two group sizes, but the provided groupsize {groupsize} is not")
        self.n_bit = n_bit
        self.group_size_shift = int(math.log2(groupsize))
        self.min_bias = min_bias
        self.max_bias = max_bias
        self.f = f

    @property
    def group_size(self) -> int:
        return 1 << self.group_size_shift

    def _check(self, w: torch.Tensor) -> None:
        if w.dim() != 2:
            raise ValueError(f"Only 2D tensors can be quantized, but w has {w.dim()} dimensions")
        if w.shape[-1] % self.group_size != 0:
            raise ValueError(
                f"groupsize must divide the weight dimension but {self.group_size} doesn't divide {w.shape[-1]}")

    def group_quantize_tensor(self, w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """-> (uint8 [N, K], cat(scale, min) [N*G, 2] in w's dtype)."""
        self._check(w)
        to_quant = w.reshape(-1, self.group_size).to(torch.float32)
        if torch.isnan(to_quant).any():
            raise ValueError("Cannot quantize tensors with NaN values")
        max_val = to_quant.amax(dim=1, keepdim=True) + self.max_bias
        min_val = to_quant.amin(dim=1, keepdim=True) + self.min_bias
        uint_range = 2 ** self.n_bit - 1
        val_range = (self.f * (max_val - min_val)).clamp(min=1e-6)
        val_center = (min_val + max_val) * 0.5
        min_val = val_center - val_range * 0.5
        scales = val_range / uint_range
        q = (to_quant.sub(min_val).div(scales).clamp(0, uint_range).round().to(torch.uint8).reshape_as(w))
        return q, torch.concat([scales, min_val], dim=-1).to(dtype=w.dtype)

    def group_dequantize_tensor(self, w_uint8: torch.Tensor, scales_min_vals: torch.Tensor,
                                dtype: torch.dtype) -> torch.Tensor:
        """The Python fallback: multiply then add in the scale dtype (two roundings)."""
        self._check(w_uint8)
        grouped = w_uint8.reshape(-1, self.group_size)
        scales = scales_min_vals[:, None, 0]
        mins = scales_min_vals[:, None, 1]
        return grouped.mul(scales).add(mins).reshape_as(w_uint8).to(dtype=dtype)


class ChannelRTNQuantizer:
    """Symmetric per-output-channel int8."""

    def quantize_tensor(self, w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """-> (int8 [N, K], scales [N] in w's dtype)."""
        if w.dim() != 2:
            raise ValueError(f"Only 2D tensors can be quantized, but w has {w.dim()} dimensions")
        wf = w.to(torch.float32)
        if torch.isnan(wf).any():
            raise ValueError("Cannot quantize tensors with NaN values")
        s = (wf.abs().amax(dim=1) / 127.0).to(w.dtype)
        tiny = torch.tensor(torch.finfo(w.dtype).tiny if w.dtype != torch.float16 else 2.0 ** -24,
                            dtype=w.dtype, device=w.device)
        s = torch.where(s > 0, s, tiny)
        q = torch.round(wf / s.to(torch.float32)[:, None]).clamp(-127, 127).to(torch.int8)
        return q, s

    def dequantize_tensor(self, q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
        return q.to(s.dtype) * s[:, None]
