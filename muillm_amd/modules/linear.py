"""MuiLinear -- muillm/modules/linear.py:19-333: nn.Linear with an optional fused input
RMSNorm and a fused residual add."""
from typing import Optional, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from .. import muillm_ext
from .._hf import LlamaRMSNorm, MistralRMSNorm
from ..engineconfig import MuiEngineConfig
from ..replacement.replacementcontext import MuiReplacementContext
from .module import MuiModule
from .norm.rmsnorm import MuiRMSNorm, _MuiRMSNorm


class _MuiLinear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, module, x, residual):
        return muillm_ext.muillm_linear_module_forward(module, x, residual=residual)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("MuiLinear backward is not implemented")


class MuiLinear(MuiModule, nn.Linear):
    def __init__(self, engine_config: MuiEngineConfig, in_features: int, out_features: int, bias: bool = True,
                 variance_epsilon: float = 0.0, normalize: bool = False, device=None, dtype=None) -> None:
        MuiModule.__init__(self, engine_config=engine_config)
        nn.Linear.__init__(self, in_features=in_features, out_features=out_features, bias=bias,
                           device=device, dtype=dtype)
        self.cpp_engine = engine_config.cpp_engine
        self.device = self.weight.device
        self.dtype = self.weight.dtype
        self.normalize = normalize
        self.variance_epsilon = variance_epsilon
        self.norm_weights = nn.Parameter(torch.ones(in_features, dtype=dtype, device=device)) if normalize else None
        self._check_dispatchable()
        # the kernel-side handle is created at the end of all layer replacements
        self.cpp_module = None

    def _check_dispatchable(self):
        self.dispatchable = self.weight.is_cuda and self.weight.dtype in (torch.float16, torch.bfloat16)

    def finalize_init(self):
        if self.cpp_module is not None:
            muillm_ext.muillm_linear_module_deinit(self.cpp_module)
        self.cpp_module = muillm_ext.muillm_linear_module_init(
            self.cpp_engine, self.weight, self.norm_weights, self.variance_epsilon, None, self.bias)
        self._check_dispatchable()

    def finalize_deinit(self):
        cpp_module = self.__dict__.get("cpp_module", None)
        if cpp_module is not None:
            muillm_ext.muillm_linear_module_deinit(cpp_module)
            self.cpp_module = None

    @staticmethod
    def _set_requires_grads(param: nn.Parameter, requires_grads: bool) -> None:
        if param is not None:
            param.requires_grad = requires_grads

    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_module: Union["MuiLinear", nn.Linear],
                prev_layernorm_module: Union[MuiRMSNorm, LlamaRMSNorm, MistralRMSNorm] = None) -> "MuiLinear":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiLinear) and (prev_layernorm_module is None):
            return prev_module
        if not isinstance(prev_module, nn.Linear):
            raise ValueError(f"Unsupported replacement to MuiLinear: {prev_module.__class__.__name__}")
        prev_module = replacement_context.to_local_module(prev_module).to(device)
        if prev_layernorm_module is not None:
            prev_layernorm_module = replacement_context.to_local_module(prev_layernorm_module).to(device)

        if isinstance(prev_module, MuiLinear) and prev_module.normalize:
            if prev_layernorm_module is not None:
                raise ValueError("both norm weights in MuiLinear and layernorm module provided")
            normalize, variance_epsilon, norm_weights = True, prev_module.variance_epsilon, None
        elif prev_layernorm_module is not None:
            normalize = True
            variance_epsilon = MuiRMSNorm._extract_eps(prev_layernorm_module)
            norm_weights = prev_layernorm_module.weight
        else:
            normalize, variance_epsilon, norm_weights = False, 0.0, None

        new_module = MuiLinear(
            engine_config=engine_config, in_features=prev_module.in_features,
            out_features=prev_module.out_features, bias=prev_module.bias is not None,
            variance_epsilon=variance_epsilon, normalize=normalize,
            dtype=prev_module.weight.dtype, device=device)
        new_module.copy_module(prev_module=prev_module, norm_weights=norm_weights, device=device)
        return new_module

    def _set_weights(self, weights: torch.Tensor, requires_grads: Optional[bool] = None) -> None:
        rg = weights.requires_grad if requires_grads is None else requires_grads
        self.weight.data.copy_(weights.data)
        MuiLinear._set_requires_grads(self.weight, rg)

    def _set_bias(self, bias: torch.Tensor, requires_grads: Optional[bool] = None) -> None:
        if bias is not None:
            rg = bias.requires_grad if requires_grads is None else requires_grads
            self.bias.data.copy_(bias.data)
            MuiLinear._set_requires_grads(self.bias, rg)
        else:
            self.bias = None

    def _set_norm_weights(self, norm_weights: torch.Tensor, requires_grads: Optional[bool] = None) -> None:
        rg = norm_weights.requires_grad if requires_grads is None else requires_grads
        self.norm_weights.data.copy_(norm_weights.data)
        MuiLinear._set_requires_grads(self.norm_weights, rg)

    def copy_module(self, prev_module: Union["MuiLinear", nn.Linear], norm_weights: torch.Tensor = None,
                    device=None):
        """Copies weights/bias (and norm weights). Unlike the reference (linear.py:272-309) the
        epsilon given to the constructor is kept instead of being reset to 0."""
        if device is None:
            raise ValueError("device was None")
        self._set_weights(prev_module.weight)
        if prev_module.bias is not None:
            self._set_bias(prev_module.bias)
        if isinstance(prev_module, MuiLinear):
            if (prev_module.norm_weights is not None) and (norm_weights is not None):
                raise ValueError("both norm weights in MuiLinear and norm_weight provided")
            if prev_module.normalize:
                norm_weights = prev_module.norm_weights
        elif not isinstance(prev_module, nn.Linear):
            raise ValueError(f"Unsupported replacement: {prev_module.__class__.__name__}")
        if norm_weights is not None:
            # the norm weights stay separate from the matrix (folding them in is numerically unstable)
            self._set_norm_weights(norm_weights)
        self.to(device=device)
        self._check_dispatchable()

    def forward(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self.cpp_module is not None:
            return _MuiLinear.apply(self.cpp_module, input, residual)
        if self.normalize:
            if self.dispatchable and input.is_cuda:
                input = _MuiRMSNorm.apply(input, self.norm_weights, self.variance_epsilon)
            else:
                h = input.to(torch.float32)
                h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
                input = self.norm_weights * h.to(input.dtype)
        output = F.linear(input, self.weight, self.bias)
        if residual is not None:
            output = output + residual
        return output
