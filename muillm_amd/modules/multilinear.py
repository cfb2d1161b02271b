"""MuiMultiLinear -- muillm/modules/multilinear.py:28-237: several linears over the same
input (q, k, v) fused into one MuiLinear over the row-concatenated weights, with the input
RMSNorm fused in; the outputs are last-dim views of the single result."""
from typing import Iterable, List, Tuple, Union

import torch
import torch.nn as nn
from torch import Tensor

from .._hf import LlamaRMSNorm, MistralRMSNorm
from ..engineconfig import MuiEngineConfig
from ..replacement.replacementcontext import MuiReplacementContext
from .linear import MuiLinear
from .module import MuiModule
from .norm.rmsnorm import MuiRMSNorm


def _all_or_none(it: Iterable[bool], exception_message) -> bool:
    vals = list(it)
    if any(vals) and not all(vals):
        raise ValueError(exception_message)
    return all(vals)


class MuiMultiLinear(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, in_features: int, out_features: List[int],
                 bias: bool = True, variance_epsilon: float = 0.0, normalize: bool = False,
                 device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.linear = MuiLinear(engine_config=engine_config, in_features=in_features,
                                out_features=sum(out_features), bias=bias,
                                variance_epsilon=variance_epsilon, normalize=normalize,
                                device=device, dtype=dtype)
        self.in_features = in_features
        self.out_features = list(out_features)
        self.slice_starts, self.slice_ends = [], []
        start = 0
        for out_feature in out_features:
            self.slice_starts.append(start)
            self.slice_ends.append(start + out_feature)
            start += out_feature

    def finalize_init(self):
        self.linear.finalize_init()

    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_modules: List[Union[MuiLinear, nn.Linear]],
                prev_layernorm_module: Union[MuiRMSNorm, LlamaRMSNorm, MistralRMSNorm] = None) -> "MuiMultiLinear":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if len(prev_modules) < 1:
            raise ValueError("MuiMultiLinear needs some linear layers passed in but none were provided")
        prev_modules = [replacement_context.to_local_module(m).to(device) for m in prev_modules]
        if prev_layernorm_module is not None:
            prev_layernorm_module = replacement_context.to_local_module(prev_layernorm_module).to(device)
        has_bias = _all_or_none(
            [m.bias is not None for m in prev_modules],
            "All linear modules or none must have a bias to merge into a MuiMultiLinear layer")
        normalize = prev_layernorm_module is not None
        variance_epsilon = MuiRMSNorm._extract_eps(prev_layernorm_module) if normalize else 0.0
        norm_weights = prev_layernorm_module.weight if normalize else None
        new_module = MuiMultiLinear(
            engine_config=engine_config, in_features=prev_modules[0].in_features,
            out_features=[m.out_features for m in prev_modules], bias=has_bias,
            variance_epsilon=variance_epsilon, normalize=normalize,
            dtype=prev_modules[0].weight.dtype, device=device)
        new_module.copy_modules(prev_modules=prev_modules, norm_weights=norm_weights, device=device)
        return new_module

    def _get_linear_back(self, slice_start: int, slice_end: int) -> nn.Linear:
        has_bias = self.linear.bias is not None
        weight = self.linear.weight[slice_start:slice_end, ...]
        linear = nn.Linear(in_features=self.in_features, out_features=slice_end - slice_start, bias=has_bias,
                           dtype=weight.dtype, device=weight.device)
        linear.weight = nn.Parameter(weight.detach(), requires_grad=self.linear.weight.requires_grad)
        if has_bias:
            linear.bias = nn.Parameter(self.linear.bias[slice_start:slice_end].detach(),
                                       requires_grad=self.linear.bias.requires_grad)
        return linear

    def replace_back(self) -> Tuple[List[nn.Linear], torch.Tensor]:
        """Split back into the individual linears (+ the norm weights)."""
        linears = [self._get_linear_back(s, e) for s, e in zip(self.slice_starts, self.slice_ends)]
        return linears, self.linear.norm_weights

    def copy_modules(self, prev_modules: List[Union[MuiLinear, nn.Linear]], norm_weights: torch.Tensor = None,
                     device=None):
        if device is None:
            raise ValueError("device was None")
        weights_rg = _all_or_none([m.weight.requires_grad for m in prev_modules],
                                  "all or none weights must required grads but got a mix")
        self.linear._set_weights(torch.cat([m.weight.detach() for m in prev_modules], dim=0), weights_rg)
        if self.linear.bias is not None:
            bias_rg = _all_or_none([m.bias.requires_grad for m in prev_modules],
                                   "all or none biases must required grads but got a mix")
            self.linear._set_bias(torch.cat([m.bias.detach() for m in prev_modules], dim=0), bias_rg)
        if norm_weights is not None:
            self.linear._set_norm_weights(norm_weights)
        self.to(device=device)

    def forward(self, input: Tensor) -> Tuple[Tensor, ...]:
        all_outputs = self.linear(input)
        return tuple(all_outputs[..., s:e] for s, e in zip(self.slice_starts, self.slice_ends))
