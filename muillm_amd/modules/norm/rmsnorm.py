"""MuiRMSNorm -- muillm/modules/norm/rmsnorm.py:21-146."""
from typing import Union

import torch
import torch.nn as nn
from torch import Tensor

from ... import muillm_ext
from ..._hf import LlamaRMSNorm, MistralRMSNorm
from ...engineconfig import MuiEngineConfig
from ...replacement.replacementcontext import MuiReplacementContext
from ..module import MuiModule


class _MuiRMSNorm(torch.autograd.Function):
    """Named wrapper around the kernel call (inference only, like the reference)."""

    @staticmethod
    def forward(ctx, inputs, weights, epsilon):
        return muillm_ext.muillm_rmsnorm_forward(weights, inputs, epsilon)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("RMSNorm backward is not implemented")


class MuiRMSNorm(MuiModule):
    def __init__(self, engine_config: MuiEngineConfig, hidden_size, eps=1e-6, device=None, dtype=None) -> None:
        super().__init__(engine_config=engine_config)
        self.weight = nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype))
        self.variance_epsilon = eps
        self._check_dispatchable()

    def _check_dispatchable(self):
        wdtype = self.weight.dtype
        self.dispatchable = self.weight.is_cuda and wdtype in (torch.float16, torch.bfloat16)

    def finalize_init(self):
        self._check_dispatchable()

    @staticmethod
    def _extract_eps(prev_module) -> float:
        for attr in ("variance_epsilon", "eps"):
            if hasattr(prev_module, attr):
                return getattr(prev_module, attr)
        raise ValueError(f"cannot find the epsilon of {type(prev_module).__name__}")

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiRMSNorm", LlamaRMSNorm, MistralRMSNorm]) -> "MuiRMSNorm":
        engine_config = replacement_context.engine_config
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        if isinstance(prev_module, MuiRMSNorm):
            return prev_module
        prev_module = replacement_context.to_local_module(prev_module).to(device=device)
        new_module = MuiRMSNorm(
            engine_config=engine_config,
            hidden_size=prev_module.weight.shape[0],
            eps=MuiRMSNorm._extract_eps(prev_module),
            dtype=prev_module.weight.dtype,
            device=device,
        )
        new_module.copy_module(prev_module.weight, device=device)
        return new_module

    def copy_module(self, prev_module: nn.Parameter, device=None):
        if device is None:
            raise ValueError("device was None")
        requires_grad = prev_module.requires_grad
        self.weight = nn.Parameter(prev_module.detach().clone(), requires_grad=requires_grad)
        self.to(device=device)
        self._check_dispatchable()

    def forward(self, input: Tensor) -> Tensor:
        if self.dispatchable and input.is_cuda and input.dtype == self.weight.dtype:
            return _MuiRMSNorm.apply(input, self.weight, self.variance_epsilon)
        # non-fused form (rmsnorm.py:138-146 of the reference)
        input_dtype = input.dtype
        hidden_states = input.to(torch.float32)
        variance = hidden_states.pow(2).mean(-1, keepdim=True)
        hidden_states = hidden_states * torch.rsqrt(variance + self.variance_epsilon)
        return self.weight * hidden_states.to(input_dtype)
