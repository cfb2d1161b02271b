"""MuiReplacementContext: what every replace() receives (API of
muillm/replacement/replacementcontext.py:7-42 in the reference: engine_config, model, device,
to_local_module)."""
import torch.nn as nn

from ..engineconfig import MuiEngineConfig


class MuiReplacementContext:
    def __init__(self, engine_config: MuiEngineConfig, model: nn.Module, device: str = "cuda"):
        self.engine_config = engine_config
        self.model = model      # the tree being rewritten (None when layers are converted on their own)
        self.device = device    # where converted layers end up

    def qualified_name(self, module: nn.Module) -> str:
        """Dotted name of `module` inside the model."""
        if self.model is not None:
            for name, candidate in self.model.named_modules():
                if candidate is module:
                    return name
        raise ValueError(f"{type(module).__name__} is not part of the model being converted")

    def to_local_module(self, module: nn.Module) -> nn.Module:
        """Hook for sharded checkpoints: the reference gathers DTensor-sharded HuggingFace modules
        here. One GPU: every module is local already."""
        return module
