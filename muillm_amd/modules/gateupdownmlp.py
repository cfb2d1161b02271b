"""MuiGateUpDownMLP -- muillm/modules/gateupdownmlp.py:24-423:
   out = down(silu(gate(xn)) * up(xn)) + residual, xn = rmsnorm(x) when a norm is fused in.

At finalize_init the gate and up matrices are repacked into ONE row-interleaved buffer
[intermediate, 2, hidden] (row n of gate followed by row n of up); gate_proj.weight and
up_proj.weight become strided views of it, so no memory is duplicated and the unfused torch
path keeps working. The fused kernel streams both rows of a pair together and applies
SiLU * mul in registers before the single write of the intermediate."""
from enum import Enum
from typing import Optional, Union

import torch
import torch.nn as nn
from torch import Tensor

from .. import muillm_ext
from .._hf import LlamaMLP, LlamaRMSNorm, MistralMLP, MistralRMSNorm
from ..engineconfig import MuiEngineConfig
from ..memorymanagement.gc import trigger_gc
from ..replacement.replacementcontext import MuiReplacementContext
from .linear import MuiLinear
from .module import MuiModule
from ._fusion import AbsorbedNorm
from .norm.rmsnorm import MuiRMSNorm, _MuiRMSNorm


class _MuiGateUpSiLUMethod(Enum):
    # gate / up projections and the multiply done as separate ops
    GATEUPSILU_UNFUSED = 0
    # gate / up projections + SiLU * mul fused in one kernel
    GATEUPSILU_FUSED = 1
    # the reference's split-K variant; served by the same gfx950 kernel
    GATEUPSILU_SPLIT = 2


class _MuiGateUpSiLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, engine, inputs, norm_weights, variance_epsilon, gate_weights, up_weights,
                down_weights, residual):
        return muillm_ext.muillm_gateupsilu_forward(
            engine, norm_weights, variance_epsilon, gate_weights, up_weights, down_weights, residual, inputs)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("GateUpSiLU backward is not implemented")


class _MuiGateUpSiLUSplit(torch.autograd.Function):
    @staticmethod
    def forward(ctx, engine, inputs, norm_weights, variance_epsilon, gate_weights, up_weights,
                down_weights, residual):
        return muillm_ext.muillm_gateupsilu_split_forward(
            engine, norm_weights, variance_epsilon, gate_weights, up_weights, down_weights, residual, inputs)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("GateUpSiLU split K backward is not implemented")


class MuiGateUpDownMLP(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, hidden_size: int, intermediate_size: int,
                 activation_function: nn.Module, variance_epsilon: float = 0.0, normalize: bool = False,
                 device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.cpp_engine = engine_config.cpp_engine
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.normalize = normalize
        self.variance_epsilon = variance_epsilon
        self.norm_weights = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device)) if normalize else None
        self.gate_proj = MuiLinear(engine_config, hidden_size, intermediate_size, bias=False, device=device, dtype=dtype)
        self.up_proj = MuiLinear(engine_config, hidden_size, intermediate_size, bias=False, device=device, dtype=dtype)
        self.down_proj = MuiLinear(engine_config, intermediate_size, hidden_size, bias=False, device=device, dtype=dtype)
        self.activation_function = activation_function
        self._check_dispatchable()
        self.method = _MuiGateUpSiLUMethod.GATEUPSILU_FUSED
        self.gate_up_packed = None  # [intermediate, 2, hidden] once finalized on a GPU

    def _check_dispatchable(self):
        w = self.gate_proj.weight
        self.dispatchable = (isinstance(self.activation_function, nn.SiLU) and w.is_cuda
                             and w.dtype in (torch.float16, torch.bfloat16))

    def _pack_gate_up(self):
        """Row-interleave gate and up into one buffer and alias the two weights onto it."""
        g, u = self.gate_proj.weight, self.up_proj.weight
        if self.gate_up_packed is not None and g.data_ptr() == self.gate_up_packed.data_ptr():
            return
        packed = torch.empty((self.intermediate_size, 2, self.hidden_size), dtype=g.dtype, device=g.device)
        packed[:, 0, :].copy_(g.detach())
        packed[:, 1, :].copy_(u.detach())
        rg_g, rg_u = g.requires_grad, u.requires_grad
        self.gate_proj.weight = nn.Parameter(packed[:, 0, :], requires_grad=rg_g)
        self.up_proj.weight = nn.Parameter(packed[:, 1, :], requires_grad=rg_u)
        self.gate_up_packed = packed
        del g, u

    def finalize_init(self):
        self._check_dispatchable()
        if self.dispatchable:
            self._pack_gate_up()
        self.gate_proj.finalize_init()
        self.up_proj.finalize_init()
        self.down_proj.finalize_init()

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiGateUpDownMLP", LlamaMLP, MistralMLP],
                prev_layernorm_module: Union[MuiRMSNorm, LlamaRMSNorm, MistralRMSNorm] = None) -> "MuiGateUpDownMLP":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiGateUpDownMLP) and (prev_layernorm_module is None):
            return prev_module
        for name in ("gate_proj", "up_proj", "down_proj"):
            if not hasattr(prev_module, name):
                raise ValueError(f"Unsupported module type {type(prev_module)} for replacement")
        prev_module = replacement_context.to_local_module(prev_module).to(device)
        if prev_layernorm_module is not None:
            prev_layernorm_module = replacement_context.to_local_module(prev_layernorm_module).to(device)

        if isinstance(prev_module, MuiGateUpDownMLP):
            activation_function = prev_module.activation_function
        elif hasattr(prev_module, "act_fn"):
            activation_function = prev_module.act_fn
        elif hasattr(prev_module, "activation_fn"):
            activation_function = prev_module.activation_fn
        else:
            raise ValueError(f"Unsupported module type {type(prev_module)} for replacement")
        if type(activation_function).__name__ in ("SiLUActivation", "SiLU") and not isinstance(activation_function, nn.SiLU):
            activation_function = nn.SiLU()

        if isinstance(prev_module, MuiGateUpDownMLP) and prev_module.normalize:
            if prev_layernorm_module is not None:
                raise ValueError("both norm weights in MuiGateUpDownMLP and layernorm module provided")
            normalize, variance_epsilon, norm_weights = True, prev_module.variance_epsilon, None
        elif prev_layernorm_module is not None:
            normalize = True
            variance_epsilon = AbsorbedNorm.of(prev_layernorm_module).eps
            norm_weights = prev_layernorm_module.weight
        else:
            normalize, variance_epsilon, norm_weights = False, 0.0, None

        new_module = MuiGateUpDownMLP(
            engine_config=engine_config, hidden_size=prev_module.gate_proj.in_features,
            intermediate_size=prev_module.up_proj.out_features, activation_function=activation_function,
            variance_epsilon=variance_epsilon, normalize=normalize,
            dtype=prev_module.gate_proj.weight.dtype, device=device)
        new_module.copy_module(prev_module=prev_module, norm_weights=norm_weights, device=device)

        if not isinstance(prev_module, MuiGateUpDownMLP):
            # free the source weights
            del prev_module.gate_proj
            del prev_module.up_proj
            del prev_module.down_proj
            trigger_gc()
        return new_module

    def copy_module(self, prev_module, norm_weights: torch.Tensor = None, device=None):
        if device is None:
            raise ValueError("device was None")
        self.gate_proj.copy_module(prev_module.gate_proj, device=device)
        self.up_proj.copy_module(prev_module.up_proj, device=device)
        if isinstance(prev_module, MuiGateUpDownMLP):
            if (prev_module.norm_weights is not None) and (norm_weights is not None):
                raise ValueError("both norm weights in MuiGateUpDownMLP and norm_weight provided")
            if prev_module.norm_weights is not None:
                norm_weights = prev_module.norm_weights
        if norm_weights is not None:
            # own copy (the reference ends up aliasing the source parameter, gateupdownmlp.py:330-333)
            self.norm_weights = nn.Parameter(norm_weights.detach().clone(), requires_grad=norm_weights.requires_grad)
        self.down_proj.copy_module(prev_module.down_proj, device=device)
        self.to(device=device)
        self._check_dispatchable()

    def _forward_unfused(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self.normalize:
            if self.dispatchable and input.is_cuda:
                input = _MuiRMSNorm.apply(input, self.norm_weights, self.variance_epsilon)
            else:
                h = input.to(torch.float32)
                h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
                input = self.norm_weights * h.to(input.dtype)
        packed = self.gate_up_packed
        if (packed is not None and input.is_cuda and input.dtype == packed.dtype and self.intermediate_size % 8 == 0
                and self.gate_proj.bias is None and self.up_proj.bias is None
                and self.gate_proj.weight.data_ptr() == packed.data_ptr()):
            # long prompts: ONE matmul over the interleaved gate/up rows, one SiLU*mul kernel, and
            # the residual in the epilogue of the down projection
            gu = torch.nn.functional.linear(input, packed.view(2 * self.intermediate_size, self.hidden_size))
            return self.down_proj(muillm_ext.mui_silu_mul_interleaved(gu), residual=residual)
        g = self.gate_proj(input)
        u = self.up_proj(input)
        output = self.down_proj(self.activation_function(g) * u)
        if residual is not None:
            output = output + residual
        return output

    def _kernel_ok(self, input: Tensor) -> bool:
        return (self.dispatchable and muillm_ext.kernel_dispatchable(input)
                and isinstance(self.gate_proj, MuiLinear) and isinstance(self.up_proj, MuiLinear))

    def _forward_fused(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self._kernel_ok(input):
            return _MuiGateUpSiLU.apply(self.cpp_engine, input, self.norm_weights, self.variance_epsilon,
                                        self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, residual)
        return self._forward_unfused(input=input, residual=residual)

    def _forward_split(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self._kernel_ok(input):
            return _MuiGateUpSiLUSplit.apply(self.cpp_engine, input, self.norm_weights, self.variance_epsilon,
                                             self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, residual)
        return self._forward_unfused(input=input, residual=residual)

    def forward(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self.method == _MuiGateUpSiLUMethod.GATEUPSILU_FUSED:
            return self._forward_fused(input=input, residual=residual)
        elif self.method == _MuiGateUpSiLUMethod.GATEUPSILU_UNFUSED:
            return self._forward_unfused(input=input, residual=residual)
        elif self.method == _MuiGateUpSiLUMethod.GATEUPSILU_SPLIT:
            return self._forward_split(input=input, residual=residual)
        raise ValueError("Unsupported Gate/Up Silu method")
