"""init_engine -- muillm/engine.py:12-62: swap a model's layers for the fused ones, optionally
quantise, move to the device, then run finalize_init() post-order."""
from typing import Optional

import torch
import torch.nn as nn

from .engineconfig import MuiEngineConfig
from .quantization.quantizationmethod import QuantizationMethod


def _finalize_module(module: nn.Module):
    from .modules.module import MuiModule

    for sub_module in module.children():
        _finalize_module(sub_module)
    if isinstance(module, MuiModule):
        module.finalize_init()


def init_engine(model: nn.Module, device="cuda", quantization_method: QuantizationMethod = None,
                tensor_parallelism: Optional[int] = 1, engine_config: MuiEngineConfig = None) -> nn.Module:
    from .quantization.quantizedreplacements import quantize_layers
    from .replacement.replacementcontext import MuiReplacementContext
    from .replacement.replacements import replace_layers

    if engine_config is None:
        engine_config = MuiEngineConfig(quantization_method, tensor_parallelism=tensor_parallelism)
    quantization_method = engine_config.quantization_method

    # no_grad so that no autograd references keep the replaced modules alive
    with torch.no_grad():
        replacement_context = MuiReplacementContext(engine_config, model=model, device=device)
        model = replace_layers(module=model, replacement_context=replacement_context)
        if quantization_method is not None:
            replacement_context.model = model
            quantize_layers(model=model, engine_config=engine_config, device=device)
        if device is not None:
            model = model.to(device=device)
    setattr(model, "muillm_config", engine_config)
    _finalize_module(model)
    return model
