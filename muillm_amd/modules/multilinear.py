"""MuiMultiLinear: several projections of the same input (q, k, v) as ONE MuiLinear over their
row-concatenated matrices, with the input RMSNorm absorbed; forward returns one last-dim view per
projection (API of muillm/modules/multilinear.py:28-237 in the reference: replace / copy_modules /
replace_back / forward, `linear`, `slice_starts`, `slice_ends`)."""
from itertools import accumulate
from typing import List, Tuple, Union

import torch
import torch.nn as nn
from torch import Tensor

from .._hf import LlamaRMSNorm, MistralRMSNorm
from ..engineconfig import MuiEngineConfig
from ..replacement.replacementcontext import MuiReplacementContext
from ._fusion import AbsorbedNorm, uniform_flag
from .linear import MuiLinear
from .module import MuiModule
from .norm.rmsnorm import MuiRMSNorm


class MuiMultiLinear(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, in_features: int, out_features: List[int],
                 bias: bool = True, variance_epsilon: float = 0.0, normalize: bool = False,
                 device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.in_features = in_features
        self.out_features = list(out_features)
        ends = list(accumulate(self.out_features))
        self.slice_ends = ends
        self.slice_starts = [0] + ends[:-1]
        self.linear = MuiLinear(engine_config, in_features=in_features, out_features=ends[-1], bias=bias,
                                variance_epsilon=variance_epsilon, normalize=normalize, device=device, dtype=dtype)

    def finalize_init(self):
        self.linear.finalize_init()

    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_modules: List[Union[MuiLinear, nn.Linear]],
                prev_layernorm_module: Union[MuiRMSNorm, LlamaRMSNorm, MistralRMSNorm] = None) -> "MuiMultiLinear":
        device = replacement_context.device
        if device is None:
            raise ValueError("the replacement context names no target device")
        if not prev_modules:
            raise ValueError("nothing to fuse: the list of projections is empty")
        sources = [replacement_context.to_local_module(m).to(device) for m in prev_modules]
        if len({m.in_features for m in sources}) != 1:
            raise ValueError("the projections to fuse must read the same input width")
        with_bias = uniform_flag([m.bias is not None for m in sources], "bias")
        absorbed = None
        if prev_layernorm_module is not None:
            absorbed = AbsorbedNorm.of(replacement_context.to_local_module(prev_layernorm_module).to(device))
        fused = MuiMultiLinear(replacement_context.engine_config, in_features=sources[0].in_features,
                               out_features=[m.out_features for m in sources], bias=with_bias,
                               variance_epsilon=0.0 if absorbed is None else absorbed.eps,
                               normalize=absorbed is not None, dtype=sources[0].weight.dtype, device=device)
        fused.copy_modules(sources, norm_weights=None if absorbed is None else absorbed.gain, device=device)
        return fused

    def copy_modules(self, prev_modules: List[Union[MuiLinear, nn.Linear]], norm_weights: torch.Tensor = None,
                     device=None):
        """Stack the projections' matrices (and biases) row-wise into the single layer."""
        if device is None:
            raise ValueError("copy_modules needs the target device")
        stacked_w = torch.cat([m.weight.detach() for m in prev_modules], dim=0)
        w_grad = uniform_flag([m.weight.requires_grad for m in prev_modules], "requires_grad of the weights")
        stacked_b, b_grad = None, None
        if self.linear.bias is not None:
            stacked_b = torch.cat([m.bias.detach() for m in prev_modules], dim=0)
            b_grad = uniform_flag([m.bias.requires_grad for m in prev_modules], "requires_grad of the biases")
        self.linear.load_tensors(stacked_w, stacked_b, norm_weights, weight_requires_grad=w_grad,
                                 bias_requires_grad=b_grad)
        self.to(device=device)

    def replace_back(self) -> Tuple[List[nn.Linear], torch.Tensor]:
        """Undo the fusion: one nn.Linear per projection (views of the stacked parameters) and the
        absorbed gain vector."""
        fused = self.linear
        parts = []
        for lo, hi in zip(self.slice_starts, self.slice_ends):
            part = nn.Linear(self.in_features, hi - lo, bias=fused.bias is not None, dtype=fused.weight.dtype,
                             device=fused.weight.device)
            part.weight = nn.Parameter(fused.weight[lo:hi].detach(), requires_grad=fused.weight.requires_grad)
            if fused.bias is not None:
                part.bias = nn.Parameter(fused.bias[lo:hi].detach(), requires_grad=fused.bias.requires_grad)
            parts.append(part)
        return parts, fused.norm_weights

    def forward(self, input: Tensor) -> Tuple[Tensor, ...]:
        y = self.linear(input)
        return tuple(y[..., lo:hi] for lo, hi in zip(self.slice_starts, self.slice_ends))
