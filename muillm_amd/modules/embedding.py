"""MuiEmbedding -- muillm/modules/embedding.py:13-140 of the reference: an nn.Embedding whose
forward is a gather kernel for 16-bit tables on the GPU (int32 or int64 ids), so that the
lookup of a decode step is a plain kernel launch that a HIP graph can replay."""
from typing import Optional, Union

import torch
import torch.nn as nn

from .. import muillm_ext
from ..engineconfig import MuiEngineConfig
from ..replacement.replacementcontext import MuiReplacementContext
from .module import MuiModule


class _MuiEmbedding(torch.autograd.Function):
    @staticmethod
    def forward(ctx, module, x):
        return muillm_ext.muillm_embedding_module_forward(module, x)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("embedding backward is not implemented")


class MuiEmbedding(MuiModule, nn.Module):
    def __init__(self, engine_config: MuiEngineConfig, num_embeddings: int, embedding_dim: int,
                 padding_idx: Optional[int] = None, device=None, dtype=None):
        MuiModule.__init__(self, engine_config)
        nn.Module.__init__(self)
        self.cpp_engine = engine_config.cpp_engine
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.padding_idx = padding_idx
        self.weight = nn.Parameter(torch.empty(num_embeddings, embedding_dim, device=device, dtype=dtype),
                                   requires_grad=False)
        nn.init.normal_(self.weight)
        self.cpp_module = None
        self._check_dispatchable()

    def _check_dispatchable(self):
        self.dispatchable = self.weight.is_cuda and self.weight.dtype in (torch.float16, torch.bfloat16)

    def finalize_init(self):
        if self.cpp_module is not None:
            muillm_ext.muillm_embedding_module_deinit(self.cpp_module)
        self.cpp_module = muillm_ext.muillm_embedding_module_init(self.cpp_engine, self.weight)
        self._check_dispatchable()

    def finalize_deinit(self):
        if self.cpp_module is not None:
            muillm_ext.muillm_embedding_module_deinit(self.cpp_module)
            self.cpp_module = None

    @staticmethod
    def replace(replacement_context: MuiReplacementContext,
                prev_module: Union["MuiEmbedding", nn.Embedding]) -> "MuiEmbedding":
        if isinstance(prev_module, MuiEmbedding):
            return prev_module
        device = replacement_context.device
        if device is None:
            raise ValueError("device was None")
        prev_module = replacement_context.to_local_module(prev_module).to(device)
        new_module = MuiEmbedding(replacement_context.engine_config, prev_module.num_embeddings,
                                  prev_module.embedding_dim, padding_idx=prev_module.padding_idx,
                                  device=device, dtype=prev_module.weight.dtype)
        new_module.copy_module(prev_module)
        return new_module

    def copy_module(self, prev_module: nn.Embedding):
        self.weight = nn.Parameter(prev_module.weight.detach(), requires_grad=False)
        self._check_dispatchable()

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if self.dispatchable and self.cpp_module is not None and input.is_cuda and input.dtype in (torch.int32, torch.int64):
            return _MuiEmbedding.apply(self.cpp_module, input)
        return nn.functional.embedding(input, self.weight, self.padding_idx)
