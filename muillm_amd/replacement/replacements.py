"""replace_layers -- muillm/replacement/replacements.py:66-207: type-keyed table of layer
replacements applied top-down; after a module is replaced only the immediate children of the
NEW module are visited (the original children may no longer exist)."""
import torch.nn as nn

from .. import _hf
from ..memorymanagement.gc import trigger_gc
from ..modules.attention.rotaryembedding import MuiRotaryEmbedding
from ..modules.decoder.decoder import MuiDecoderLayer
from ..modules.gateupdownmlp import MuiGateUpDownMLP
from ..modules.linear import MuiLinear
from ..modules.models.llama.model import (MuiLlamaForCausalLM, MuiLlamaModel, MuiMistralForCausalLM,
                                          MuiMistralModel)
from ..modules.embedding import MuiEmbedding
from ..modules.norm.rmsnorm import MuiRMSNorm
from .replacementcontext import MuiReplacementContext

_LAYER_REPLACEMENTS = {
    # Linear
    nn.Linear: MuiLinear,
    # Embedding
    nn.Embedding: MuiEmbedding,
    # MLPs
    _hf.MistralMLP: MuiGateUpDownMLP,
    _hf.LlamaMLP: MuiGateUpDownMLP,
    # Norm layers
    _hf.MistralRMSNorm: MuiRMSNorm,
    _hf.LlamaRMSNorm: MuiRMSNorm,
    # Rotary embeddings
    _hf.MistralRotaryEmbedding: MuiRotaryEmbedding,
    _hf.LlamaRotaryEmbedding: MuiRotaryEmbedding,
    # Decoders: replaced as a whole so that the norms end up fused into the right GEMVs
    _hf.MistralDecoderLayer: MuiDecoderLayer,
    _hf.LlamaDecoderLayer: MuiDecoderLayer,
    # full models
    _hf.MistralModel: MuiMistralModel,
    _hf.LlamaModel: MuiLlamaModel,
    _hf.MistralForCausalLM: MuiMistralForCausalLM,
    _hf.LlamaForCausalLM: MuiLlamaForCausalLM,
}


def _recursive_setattr(model: nn.Module, module_name: str, new_module: nn.Module):
    """Put new_module where the dotted name points (the parent is found through get_submodule)."""
    parent_name, _, leaf = module_name.rpartition(".")
    setattr(model.get_submodule(parent_name) if parent_name else model, leaf, new_module)


def _no_further_replacement(module: nn.Module) -> bool:
    return bool(getattr(module, "_muillm_no_further_replacement", False))


def replace_layers(module: nn.Module, replacement_context: MuiReplacementContext, name_prefix="",
                   verbose: bool = False) -> nn.Module:
    engine_config = replacement_context.engine_config
    if engine_config.tensor_parallelism > 1:
        raise ValueError("tensor parallelism is not supported by this build")
    module_type = type(module)
    if (module_type in _LAYER_REPLACEMENTS) and not _no_further_replacement(module):
        new_module_type = _LAYER_REPLACEMENTS[module_type]
        if verbose and engine_config.is_rank0():
            print(f"Replacing {name_prefix} ({module_type} to {new_module_type}) ...")
        new_module = new_module_type.replace(replacement_context, module)
        if new_module is not module:
            del module
        trigger_gc()
        module = new_module
    for sub_module_name, sub_module in list(module.named_children()):
        full_module_name = name_prefix + "." + sub_module_name if name_prefix != "" else sub_module_name
        new_sub_module = replace_layers(sub_module, replacement_context=replacement_context,
                                        name_prefix=full_module_name, verbose=verbose)
        if new_sub_module is not sub_module:
            _recursive_setattr(module, sub_module_name, new_sub_module)
    return module
