"""init_engine(model): the one call a user makes (API of muillm/engine.py:12-62 in the reference).

Order of work: layer replacement (HuggingFace layers -> fused layers, parents before children),
optional int8 quantisation of the replaced layers, move to the device, then finalize_init() on
every MuiModule children-first, so that a parent's finalize sees finished children."""
from typing import Optional

import torch
import torch.nn as nn

from .engineconfig import MuiEngineConfig
from .quantization.quantizationmethod import QuantizationMethod


def _finalize_module(module: nn.Module) -> None:
    """finalize_init() on every MuiModule of the tree, children before parents."""
    from .modules.module import MuiModule

    pending = [(module, False)]
    while pending:
        node, children_done = pending.pop()
        if children_done:
            if isinstance(node, MuiModule):
                node.finalize_init()
            continue
        pending.append((node, True))
        pending.extend((child, False) for child in reversed(list(node.children())))


def init_engine(model: nn.Module, device="cuda", quantization_method: QuantizationMethod = None,
                tensor_parallelism: Optional[int] = 1, engine_config: MuiEngineConfig = None) -> nn.Module:
    """Returns the converted model (the input object's layers are consumed). Either pass a ready
    engine_config or let one be made from quantization_method / tensor_parallelism (this build
    drives one GPU: any other tensor_parallelism is refused by MuiEngineConfig)."""
    from .quantization.quantizedreplacements import quantize_layers
    from .replacement.replacementcontext import MuiReplacementContext
    from .replacement.replacements import replace_layers

    config = engine_config or MuiEngineConfig(quantization_method, tensor_parallelism=tensor_parallelism)
    with torch.no_grad():  # keeps autograd from holding on to the layers that are being replaced
        context = MuiReplacementContext(config, model=model, device=device)
        converted = replace_layers(module=model, replacement_context=context)
        if config.quantization_method is not None:
            context.model = converted
            quantize_layers(model=converted, engine_config=config, device=device)
        if device is not None:
            converted = converted.to(device=device)
    converted.muillm_config = config
    _finalize_module(converted)
    return converted
