"""Mistral models share the Llama implementation (muillm/modules/models/mistral/model.py of
the reference is a renamed copy of the Llama file)."""
from ..llama.model import MuiLlamaForCausalLM as MuiMistralForCausalLM  # noqa: F401
from ..llama.model import MuiLlamaModel as MuiMistralModel  # noqa: F401
