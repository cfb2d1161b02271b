"""MuiEngineConfig -- muillm/engineconfig.py:11-65 of the reference, single GPU only."""
from typing import Optional

import torch

from . import muillm_ext
from .quantization.quantizationmethod import QuantizationMethod


class MuiEngineConfig:
    """Holds the quantisation method and the engine handle (device facts of the GPU in use).

    Tensor parallelism is not part of this build: any value other than 1 is rejected.
    On a machine without a GPU the config can still be built (cpp_engine is None) so that
    host-side logic runs; CUDA tensors always go through the HIP library."""

    def __init__(self, quantization_method: Optional[QuantizationMethod] = None,
                 tensor_parallelism: Optional[int] = 1):
        self.quantization_method = quantization_method
        if tensor_parallelism not in (None, 1):
            raise ValueError(
                f"tensor_parallelism {tensor_parallelism} is not supported: this build drives one GPU")
        self.tensor_parallelism = 1
        self.comms = None
        # the library must be there even when no GPU is visible: there is no fallback for it
        from . import _lib
        _lib.load()
        self.cpp_engine = muillm_ext.muillm_engine_init() if torch.cuda.is_available() else None

    def rank(self) -> int:
        return 0

    def is_rank0(self) -> bool:
        return True
