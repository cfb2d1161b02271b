"""MuiLinear: nn.Linear that can apply the RMSNorm in front of it and add a residual behind it,
all inside one kernel (API of muillm/modules/linear.py:19-333 in the reference: replace /
copy_module / finalize_init / finalize_deinit / forward(input, residual), `normalize`,
`variance_epsilon`, `norm_weights`).

The gain vector stays a separate parameter (multiplying it into the matrix would change the
rounding). One deliberate difference from the reference: the epsilon passed to the constructor
survives copy_module (there it falls back to 0 whenever norm weights are handed over,
linear.py:272-309)."""
from typing import Optional, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from .. import muillm_ext
from .._hf import LlamaRMSNorm, MistralRMSNorm
from ..engineconfig import MuiEngineConfig
from ..replacement.replacementcontext import MuiReplacementContext
from ._fusion import AbsorbedNorm, fill_parameter, is_kernel_dtype, rmsnorm_reference
from .module import MuiModule
from .norm.rmsnorm import MuiRMSNorm, _MuiRMSNorm


class _MuiLinear(torch.autograd.Function):
    """The library call as an autograd node without a backward (inference only)."""

    @staticmethod
    def forward(ctx, module, x, residual):
        return muillm_ext.muillm_linear_module_forward(module, x, residual=residual)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("inference only: MuiLinear has no backward")


class MuiLinear(MuiModule, nn.Linear):
    def __init__(self, engine_config: MuiEngineConfig, in_features: int, out_features: int, bias: bool = True,
                 variance_epsilon: float = 0.0, normalize: bool = False, device=None, dtype=None) -> None:
        MuiModule.__init__(self, engine_config=engine_config)
        nn.Linear.__init__(self, in_features=in_features, out_features=out_features, bias=bias,
                           device=device, dtype=dtype)
        self.cpp_engine = engine_config.cpp_engine
        self.device, self.dtype = self.weight.device, self.weight.dtype
        self.normalize = bool(normalize)
        self.variance_epsilon = variance_epsilon
        self.norm_weights = None
        if self.normalize:
            self.norm_weights = nn.Parameter(torch.ones(in_features, dtype=dtype, device=device))
        self.dispatchable = is_kernel_dtype(self.weight)
        self.cpp_module = None  # the library-side handle; made by finalize_init once every layer is in place

    # ---- life cycle --------------------------------------------------------------------------
    def finalize_init(self):
        self.finalize_deinit()
        self.dispatchable = is_kernel_dtype(self.weight)
        self.cpp_module = muillm_ext.muillm_linear_module_init(
            self.cpp_engine, self.weight, self.norm_weights, self.variance_epsilon, None, self.bias)

    def finalize_deinit(self):
        handle = self.__dict__.get("cpp_module")
        if handle is not None:
            muillm_ext.muillm_linear_module_deinit(handle)
            self.cpp_module = None

    # ---- construction from other layers ------------------------------------------------------
    @staticmethod
    def replace(replacement_context: MuiReplacementContext, prev_module: Union["MuiLinear", nn.Linear],
                prev_layernorm_module: Union[MuiRMSNorm, LlamaRMSNorm, MistralRMSNorm] = None) -> "MuiLinear":
        """A MuiLinear holding prev_module's parameters; with prev_layernorm_module, that norm is
        absorbed (the caller drops the norm layer). A MuiLinear passes through unchanged unless a
        norm is to be absorbed into it."""
        device = replacement_context.device
        if device is None:
            raise ValueError("the replacement context names no target device")
        already_ours = isinstance(prev_module, MuiLinear)
        if already_ours and prev_layernorm_module is None:
            return prev_module
        if not isinstance(prev_module, nn.Linear):
            raise ValueError(f"MuiLinear can stand in for nn.Linear layers, not for {type(prev_module).__name__}")
        if already_ours and prev_module.normalize and prev_layernorm_module is not None:
            raise ValueError("this MuiLinear already applies a norm; a second one cannot be absorbed")

        source = replacement_context.to_local_module(prev_module).to(device)
        absorbed = None
        if prev_layernorm_module is not None:
            absorbed = AbsorbedNorm.of(replacement_context.to_local_module(prev_layernorm_module).to(device))
        carries_norm = already_ours and source.normalize
        eps = absorbed.eps if absorbed is not None else (source.variance_epsilon if carries_norm else 0.0)

        layer = MuiLinear(replacement_context.engine_config, in_features=source.in_features,
                          out_features=source.out_features, bias=source.bias is not None, variance_epsilon=eps,
                          normalize=absorbed is not None or carries_norm, dtype=source.weight.dtype, device=device)
        layer.copy_module(source, norm_weights=None if absorbed is None else absorbed.gain, device=device)
        return layer

    def load_tensors(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     norm_weights: Optional[torch.Tensor] = None, weight_requires_grad: Optional[bool] = None,
                     bias_requires_grad: Optional[bool] = None) -> None:
        """Fill the parameters in place from plain tensors (shapes must match the constructor's)."""
        fill_parameter(self.weight, weight, weight_requires_grad)
        if self.bias is not None:
            if bias is None:
                raise ValueError("this layer was built with a bias but none was supplied")
            fill_parameter(self.bias, bias, bias_requires_grad)
        elif bias is not None:
            raise ValueError("this layer was built without a bias")
        if norm_weights is not None:
            if self.norm_weights is None:
                raise ValueError("this layer was built without a fused norm")
            fill_parameter(self.norm_weights, norm_weights)

    def copy_module(self, prev_module: Union["MuiLinear", nn.Linear], norm_weights: torch.Tensor = None,
                    device=None):
        """Take over prev_module's matrix and bias, plus a gain vector: either norm_weights or the
        one prev_module (a MuiLinear) already carries, never both."""
        if device is None:
            raise ValueError("copy_module needs the target device")
        if not isinstance(prev_module, nn.Linear):
            raise ValueError(f"cannot copy from {type(prev_module).__name__}")
        own_gain = prev_module.norm_weights if isinstance(prev_module, MuiLinear) and prev_module.normalize else None
        if own_gain is not None and norm_weights is not None:
            raise ValueError("two gain vectors: the source layer carries one and another was passed")
        self.load_tensors(prev_module.weight, prev_module.bias if self.bias is not None else None,
                          norm_weights if norm_weights is not None else own_gain)
        self.to(device=device)
        self.dispatchable = is_kernel_dtype(self.weight)

    # ---- forward -----------------------------------------------------------------------------
    def forward(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self.cpp_module is not None:
            return _MuiLinear.apply(self.cpp_module, input, residual)
        # before finalize_init: plain torch, with the library's norm kernel where it applies
        x = input
        if self.normalize:
            if self.dispatchable and x.is_cuda:
                x = _MuiRMSNorm.apply(x, self.norm_weights, self.variance_epsilon)
            else:
                x = rmsnorm_reference(x, self.norm_weights, self.variance_epsilon)
        y = F.linear(x, self.weight, self.bias)
        return y if residual is None else y + residual
