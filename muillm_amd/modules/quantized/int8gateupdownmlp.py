"""MuiInt8GateUpDownMLP -- muillm/modules/quantized/int8gateupdownmlp.py:22-345: int8
gate/up + SiLU fused kernel followed by an int8 down projection with the residual.

gate and up are packed row-interleaved: gate_up_weights [N, 2, K] (row n of gate, then row n
of up) with gate_up_scales [N, 2] (per-channel format) or gate_up_scales_min_vals
[N, 2, G, 2] (group format). The reference packs per element ([N, K, 2],
int8gateupdownmlp.py:211-230); per-row packing keeps every row a contiguous stream of
128-bit loads while still serving both rows of a pair from one workgroup."""
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from ... import muillm_ext
from ...engineconfig import MuiEngineConfig
from ...quantization.quantizationmethod import Int8WeightOnlyQuantizationMethod
from ...replacement.replacementcontext import MuiReplacementContext
from ..gateupdownmlp import MuiGateUpDownMLP
from ..module import MuiModule
from ..norm.rmsnorm import _MuiRMSNorm
from .int8linear import MuiInt8Linear


class MuiInt8GateUpDownMLP(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, quantization_method: Int8WeightOnlyQuantizationMethod,
                 hidden_size: int, intermediate_size: int, activation_function: nn.Module,
                 variance_epsilon: float = 0.0, normalize: bool = False, device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.weight_dtype = dtype
        self.quantization_method = quantization_method
        self.per_channel = quantization_method.per_channel
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.normalize = normalize
        self.variance_epsilon = variance_epsilon
        self.norm_weights = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device)) if normalize else None
        qdtype = torch.int8 if self.per_channel else torch.uint8
        self.gate_up_weights = nn.Parameter(
            torch.zeros((intermediate_size, 2, hidden_size), dtype=qdtype, device=device), requires_grad=False)
        if self.per_channel:
            self.group_size_shift = 0
            self.gate_up_scales = nn.Parameter(
                torch.zeros((intermediate_size, 2), dtype=dtype, device=device), requires_grad=False)
        else:
            gs = quantization_method.group_size
            self.group_size_shift = gs.bit_length() - 1
            self.gate_up_scales_min_vals = nn.Parameter(
                torch.zeros((intermediate_size, 2, hidden_size // gs, 2), dtype=dtype, device=device),
                requires_grad=False)
        self.down_proj = MuiInt8Linear(engine_config, quantization_method, intermediate_size, hidden_size,
                                       bias=False, device=device, dtype=dtype)
        self.activation_function = activation_function
        self._check_dispatchable()

    def _check_dispatchable(self):
        self.dispatchable = (isinstance(self.activation_function, nn.SiLU) and self.gate_up_weights.is_cuda
                             and self.weight_dtype in (torch.float16, torch.bfloat16)
                             and (self.per_channel or self.group_size_shift >= 4))

    def finalize_init(self):
        self._check_dispatchable()
        self.down_proj.finalize_init()

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiInt8GateUpDownMLP", MuiGateUpDownMLP]) -> "MuiInt8GateUpDownMLP":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiInt8GateUpDownMLP):
            return prev_module
        if not isinstance(prev_module, MuiGateUpDownMLP):
            raise ValueError(f"Unsupported replacement to MuiInt8GateUpDownMLP: {prev_module.__class__.__name__}")
        prev_module = prev_module.to(device)
        new_module = MuiInt8GateUpDownMLP(
            engine_config=engine_config, quantization_method=engine_config.quantization_method,
            hidden_size=prev_module.hidden_size, intermediate_size=prev_module.intermediate_size,
            activation_function=prev_module.activation_function,
            variance_epsilon=prev_module.variance_epsilon, normalize=bool(prev_module.normalize),
            dtype=prev_module.gate_proj.weight.dtype, device=device)
        new_module.copy_module(prev_module=prev_module, device=device)
        return new_module

    def _quantize(self, linear) -> Tuple[torch.Tensor, torch.Tensor]:
        q = self.down_proj.quantizer
        w = linear.weight.detach()
        return q.quantize_tensor(w) if self.per_channel else q.group_quantize_tensor(w)

    def copy_module(self, prev_module: MuiGateUpDownMLP, device=None):
        if device is None:
            raise ValueError("device was None")
        if prev_module.norm_weights is not None:
            self.norm_weights = nn.Parameter(prev_module.norm_weights.detach().clone(), requires_grad=False)
        qg, sg = self._quantize(prev_module.gate_proj)
        qu, su = self._quantize(prev_module.up_proj)
        n = self.intermediate_size
        self.gate_up_weights = nn.Parameter(torch.stack([qg, qu], dim=1).contiguous(), requires_grad=False)
        if self.per_channel:
            self.gate_up_scales = nn.Parameter(torch.stack([sg, su], dim=1).contiguous(), requires_grad=False)
        else:
            self.gate_up_scales_min_vals = nn.Parameter(
                torch.stack([sg.reshape(n, -1, 2), su.reshape(n, -1, 2)], dim=1).contiguous(), requires_grad=False)
        self.down_proj.copy_module(prev_module.down_proj, device=device)
        self.to(device=device)
        self._check_dispatchable()

    def _dequantize_gateup_weights(self) -> Tuple[torch.Tensor, torch.Tensor]:
        gw, uw = self.gate_up_weights[:, 0, :], self.gate_up_weights[:, 1, :]
        if self.per_channel:
            sg, su = self.gate_up_scales[:, 0], self.gate_up_scales[:, 1]
            if self.dispatchable:
                return (muillm_ext.mui_int8_channel_dequantize_forward(gw, sg),
                        muillm_ext.mui_int8_channel_dequantize_forward(uw, su))
            return gw.to(sg.dtype) * sg[:, None], uw.to(su.dtype) * su[:, None]
        if self.dispatchable:
            return muillm_ext.muillm_int8_gateupsilu_dequantize_forward(
                self.gate_up_weights, self.gate_up_scales_min_vals, self.group_size_shift)
        q = self.down_proj.quantizer
        smv = self.gate_up_scales_min_vals
        return (q.group_dequantize_tensor(gw, smv[:, 0].reshape(-1, 2), dtype=self.weight_dtype),
                q.group_dequantize_tensor(uw, smv[:, 1].reshape(-1, 2), dtype=self.weight_dtype))

    def forward(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self.dispatchable and muillm_ext.int8_kernel_dispatchable(input):
            if self.per_channel:
                gateup = muillm_ext.mui_int8_channel_gateupsilu_forward(
                    self.norm_weights, self.variance_epsilon, self.gate_up_weights[:, 0, :],
                    self.gate_up_weights[:, 1, :], self.gate_up_scales[:, 0], self.gate_up_scales[:, 1], input)
            else:
                gateup = muillm_ext.muillm_int8_gateupsilu_forward(
                    self.norm_weights, self.variance_epsilon, self.gate_up_weights,
                    self.gate_up_scales_min_vals, self.group_size_shift, input)
            return self.down_proj(gateup, residual=residual)
        if self.normalize:
            if input.is_cuda and input.dtype in (torch.float16, torch.bfloat16):
                input = _MuiRMSNorm.apply(input, self.norm_weights, self.variance_epsilon)
            else:
                h = input.to(torch.float32)
                h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
                input = self.norm_weights * h.to(input.dtype)
        gate_weights, up_weights = self._dequantize_gateup_weights()
        g = F.linear(input, gate_weights)
        u = F.linear(input, up_weights)
        output = self.down_proj(self.activation_function(g) * u)
        if residual is not None:
            output = output + residual
        return output
