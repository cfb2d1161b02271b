"""MuiInt8Linear -- muillm/modules/quantized/int8linear.py:22-293: weight-only int8 linear
with optional fused input RMSNorm and residual.

Two storage formats, chosen by the Int8WeightOnlyQuantizationMethod:
  * group_size > 0  the reference's: weights_uint8 [N, K] + scales_min_vals [N*G, 2]
  * group_size == 0 per-output-channel symmetric: weights_int8 [N, K] + scales [N]
The decode kernels serve 1..8 tokens; more tokens dequantise the matrix and use torch's
matmul, like the reference's non-single-token branch (int8linear.py:279-293)."""
from typing import Optional, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor

from ... import muillm_ext
from ...engineconfig import MuiEngineConfig
from ...quantization.quantizationmethod import Int8WeightOnlyQuantizationMethod
from ...quantization.rtnquantizer import ChannelRTNQuantizer, RTNQuantizer
from ...replacement.replacementcontext import MuiReplacementContext
from ..linear import MuiLinear
from ..module import MuiModule
from ..norm.rmsnorm import _MuiRMSNorm


class _MuiInt8Dequantize(torch.autograd.Function):
    @staticmethod
    def forward(ctx, weights, scales_min_vals, group_size_shift):
        return muillm_ext.muillm_int8_dequantize_forward(weights, scales_min_vals, group_size_shift)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("Int8Dequantize backward is not implemented")


class _MuiInt8Linear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weights, scales_min_vals, group_size_shift, norm_weights, variance_epsilon, add_bias,
                residual):
        return muillm_ext.muillm_int8_linear_forward(
            x, weights, scales_min_vals, group_size_shift, norm_weights, variance_epsilon,
            mul_bias=None, add_bias=add_bias, residual=residual)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("Int8Linear backward is not implemented")


class MuiInt8Linear(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, quantization_method: Int8WeightOnlyQuantizationMethod,
                 in_features: int, out_features: int, bias: bool = True, variance_epsilon: float = 0.0,
                 normalize: bool = False, device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.quantization_method = quantization_method
        self.per_channel = quantization_method.per_channel
        self.in_features = in_features
        self.out_features = out_features
        self.weight_dtype = dtype
        self.normalize = normalize
        self.variance_epsilon = variance_epsilon
        self.norm_weights = nn.Parameter(torch.ones(in_features, dtype=dtype, device=device)) if normalize else None
        if self.per_channel:
            self.quantizer = ChannelRTNQuantizer()
            self.weights_int8 = nn.Parameter(
                torch.zeros((out_features, in_features), dtype=torch.int8, device=device), requires_grad=False)
            self.scales = nn.Parameter(torch.zeros((out_features,), dtype=dtype, device=device), requires_grad=False)
        else:
            self.quantizer = RTNQuantizer(n_bit=8, groupsize=quantization_method.group_size, f=quantization_method.f)
            num_groups = in_features // quantization_method.group_size
            # integer tensors cannot require grad
            self.weights_uint8 = nn.Parameter(
                torch.zeros((out_features, in_features), dtype=torch.uint8, device=device), requires_grad=False)
            self.scales_min_vals = nn.Parameter(
                torch.zeros((out_features * num_groups, 2), dtype=dtype, device=device), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros((out_features,), dtype=dtype, device=device)) if bias else None
        self._check_dispatchable()

    def _qweight(self) -> torch.Tensor:
        return self.weights_int8 if self.per_channel else self.weights_uint8

    def _check_dispatchable(self):
        self.dispatchable = self._qweight().is_cuda and self.weight_dtype in (torch.float16, torch.bfloat16)

    def finalize_init(self):
        self._check_dispatchable()

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiInt8Linear", nn.Linear, MuiLinear]) -> "MuiInt8Linear":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiInt8Linear):
            return prev_module
        if not isinstance(prev_module, nn.Linear):
            raise ValueError(f"Unsupported replacement to MuiInt8Linear: {prev_module.__class__.__name__}")
        prev_module = replacement_context.to_local_module(prev_module).to(device)
        normalize, variance_epsilon, norm_weights = False, 0.0, None
        if isinstance(prev_module, MuiLinear) and prev_module.normalize:
            normalize = True
            variance_epsilon = prev_module.variance_epsilon
            norm_weights = prev_module.norm_weights
        new_module = MuiInt8Linear(
            engine_config=engine_config, quantization_method=engine_config.quantization_method,
            in_features=prev_module.in_features, out_features=prev_module.out_features,
            bias=prev_module.bias is not None, variance_epsilon=variance_epsilon, normalize=normalize,
            dtype=prev_module.weight.dtype, device=device)
        new_module.copy_module(prev_module=prev_module, norm_weights=norm_weights, device=device)
        return new_module

    def copy_module(self, prev_module: nn.Linear, norm_weights: torch.Tensor = None, device=None):
        if device is None:
            raise ValueError("device was None")
        w = prev_module.weight.detach()
        if self.per_channel:
            q, s = self.quantizer.quantize_tensor(w)
            self.weights_int8 = nn.Parameter(q.contiguous(), requires_grad=False)
            self.scales = nn.Parameter(s.contiguous(), requires_grad=False)
        else:
            q, smv = self.quantizer.group_quantize_tensor(w)
            self.weights_uint8 = nn.Parameter(q.contiguous(), requires_grad=False)
            self.scales_min_vals = nn.Parameter(smv.contiguous(), requires_grad=False)
        if prev_module.bias is not None:
            self.bias = nn.Parameter(prev_module.bias.detach().clone(), requires_grad=False)
        if norm_weights is not None:
            self.norm_weights = nn.Parameter(norm_weights.detach().clone(), requires_grad=False)
        self.to(device=device)
        self._check_dispatchable()

    def _dequantize_weights(self) -> torch.Tensor:
        if self.per_channel:
            if self.dispatchable:
                return muillm_ext.mui_int8_channel_dequantize_forward(self.weights_int8, self.scales)
            return self.quantizer.dequantize_tensor(self.weights_int8, self.scales)
        if self.dispatchable and self.quantizer.group_size_shift >= 4 and self.in_features % 16 == 0:
            return _MuiInt8Dequantize.apply(self.weights_uint8, self.scales_min_vals, self.quantizer.group_size_shift)
        return self.quantizer.group_dequantize_tensor(self.weights_uint8, self.scales_min_vals, dtype=self.weight_dtype)

    def forward(self, input: Tensor, residual: Optional[Tensor] = None) -> Tensor:
        if self.dispatchable and muillm_ext.int8_kernel_dispatchable(input):
            if self.per_channel:
                return muillm_ext.mui_int8_channel_linear_forward(
                    input, self.weights_int8, self.scales, self.norm_weights, self.variance_epsilon,
                    self.bias, residual)
            if self.quantizer.group_size_shift >= 4:
                return _MuiInt8Linear.apply(input, self.weights_uint8, self.scales_min_vals,
                                            self.quantizer.group_size_shift, self.norm_weights,
                                            self.variance_epsilon, self.bias, residual)
        if self.normalize:
            if self.dispatchable and input.is_cuda:
                input = _MuiRMSNorm.apply(input, self.norm_weights, self.variance_epsilon)
            else:
                h = input.to(torch.float32)
                h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
                input = self.norm_weights * h.to(input.dtype)
        output = F.linear(input, self._dequantize_weights(), self.bias)
        if residual is not None:
            output = output + residual
        return output
