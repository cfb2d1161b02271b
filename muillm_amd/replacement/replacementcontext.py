"""MuiReplacementContext -- muillm/replacement/replacementcontext.py:7-42."""
import torch.nn as nn

from ..engineconfig import MuiEngineConfig


class MuiReplacementContext:
    """What a replace() call needs: the engine config, the model being rewritten and the
    target device."""

    def __init__(self, engine_config: MuiEngineConfig, model: nn.Module, device: str = "cuda"):
        self.engine_config = engine_config
        self.model = model
        self.device = device

    def _get_module_name(self, module: nn.Module) -> str:
        for name, mod in self.model.named_modules():
            if mod is module:
                return name
        raise ValueError(f"Module {module} not found in the model.")

    def to_local_module(self, module: nn.Module) -> nn.Module:
        """The reference converts DTensor-sharded HF modules to local ones here; with one GPU
        every module already is local."""
        return module
