"""MuiRMSNorm: the standalone RMSNorm layer (API of muillm/modules/norm/rmsnorm.py:21-146 in the
reference: replace / copy_module / finalize_init / forward, `weight`, `variance_epsilon`).

On fp16 / bf16 CUDA tensors the library's kernel computes gain * x * rsqrt(mean(x^2) + eps) in
fp32 with one rounding; anything else takes the HuggingFace formula in torch."""
from typing import Union

import torch
import torch.nn as nn
from torch import Tensor

from ... import muillm_ext
from ..._hf import LlamaRMSNorm, MistralRMSNorm
from ...engineconfig import MuiEngineConfig
from ...replacement.replacementcontext import MuiReplacementContext
from .._fusion import AbsorbedNorm, is_kernel_dtype, rmsnorm_reference
from ..module import MuiModule


class _MuiRMSNorm(torch.autograd.Function):
    """The kernel call as an autograd node without a backward (inference only)."""

    @staticmethod
    def forward(ctx, inputs, weights, epsilon):
        return muillm_ext.muillm_rmsnorm_forward(weights, inputs, epsilon)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("inference only: RMSNorm has no backward here")


class MuiRMSNorm(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, hidden_size, eps=1e-6, device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.variance_epsilon = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype))
        self.dispatchable = is_kernel_dtype(self.weight)

    def finalize_init(self):
        self.dispatchable = is_kernel_dtype(self.weight)

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiRMSNorm", LlamaRMSNorm, MistralRMSNorm]) -> "MuiRMSNorm":
        if isinstance(prev_module, MuiRMSNorm):
            return prev_module
        device = replacement_context.device
        if device is None:
            raise ValueError("the replacement context names no target device")
        source = replacement_context.to_local_module(prev_module).to(device=device)
        norm = AbsorbedNorm.of(source)
        layer = MuiRMSNorm(replacement_context.engine_config, hidden_size=norm.gain.numel(), eps=norm.eps,
                           dtype=norm.gain.dtype, device=device)
        layer.copy_module(norm.gain, device=device)
        return layer

    def copy_module(self, prev_module: nn.Parameter, device=None):
        """Take over a gain vector (a clone of it) and move to `device`."""
        if device is None:
            raise ValueError("copy_module needs the target device")
        self.weight = nn.Parameter(prev_module.detach().clone(), requires_grad=prev_module.requires_grad)
        self.to(device=device)
        self.dispatchable = is_kernel_dtype(self.weight)

    def forward(self, input: Tensor) -> Tensor:
        if self.dispatchable and input.is_cuda and input.dtype == self.weight.dtype:
            return _MuiRMSNorm.apply(input, self.weight, self.variance_epsilon)
        return rmsnorm_reference(input, self.weight, self.variance_epsilon)
