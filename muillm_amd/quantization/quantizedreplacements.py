"""quantize_layers -- muillm/quantization/quantizedreplacements.py:17-78: after the layer
replacement pass, swap MuiLinear / MuiGateUpDownMLP modules whose qualified name matches
one of the method's substrings for their int8 counterparts (all of them when no list is
given). The reference's glue calls replace() with a stale signature; this implements what
it intends: quantise in place, carrying a fused norm over."""
from typing import List

import torch.nn as nn

from ..engineconfig import MuiEngineConfig
from ..memorymanagement.gc import trigger_gc
from ..modules.gateupdownmlp import MuiGateUpDownMLP
from ..modules.linear import MuiLinear
from ..modules.quantized.int8gateupdownmlp import MuiInt8GateUpDownMLP
from ..modules.quantized.int8linear import MuiInt8Linear
from ..replacement.replacementcontext import MuiReplacementContext
from .quantizationmethod import Int8WeightOnlyQuantizationMethod

_INT8_LAYER_REPLACEMENTS = {
    nn.Linear: MuiInt8Linear,
    MuiLinear: MuiInt8Linear,
    MuiGateUpDownMLP: MuiInt8GateUpDownMLP,
}


def _recursive_setattr(model: nn.Module, module_name: str, new_module: nn.Module):
    """Put new_module where the dotted name points (the parent is found through get_submodule)."""
    parent_name, _, leaf = module_name.rpartition(".")
    setattr(model.get_submodule(parent_name) if parent_name else model, leaf, new_module)


def _module_name_matches(module_name: str, modules: List[str]) -> bool:
    return any(m in module_name for m in modules)


def quantize_layers(model: nn.Module, engine_config: MuiEngineConfig, device="cuda", verbose: bool = False):
    quantization_method = engine_config.quantization_method
    if not isinstance(quantization_method, Int8WeightOnlyQuantizationMethod):
        raise ValueError(f"The quantization method {quantization_method} is not supported")
    context = MuiReplacementContext(engine_config, model=model, device=device)
    # snapshot the names first: the tree is edited while walking it
    targets = [(name, module) for name, module in model.named_modules() if type(module) in _INT8_LAYER_REPLACEMENTS]
    replaced_prefixes: List[str] = []
    for module_name, module in targets:
        if any(module_name.startswith(p + ".") for p in replaced_prefixes):
            continue  # child of an MLP that was quantised as a whole
        if quantization_method.modules is not None and not _module_name_matches(module_name, quantization_method.modules):
            continue
        if verbose and engine_config.is_rank0():
            print(f"Quantizing {module_name}...")
        new_module = _INT8_LAYER_REPLACEMENTS[type(module)].replace(context, module)
        if module_name == "":
            model = new_module
        else:
            _recursive_setattr(model, module_name, new_module)
        if isinstance(new_module, MuiInt8GateUpDownMLP):
            replaced_prefixes.append(module_name)
        if new_module is not module:
            del module
        trigger_gc()
    return model
