"""Mistral models are the Llama classes under their Mistral names. What the reference's
muillm/modules/models/mistral/model.py adds to its Llama file -- config.sliding_window in the mask
decision and in the 4-D mask (:480-488, :590-602 there) -- lives in MuiLlamaModel.forward /
_update_causal_mask, which apply it whenever the config has a sliding window, and in
MuiGraphDecoder, which keeps the window in the static mask of the device-resident decode loop."""
from ..llama.model import MuiLlamaForCausalLM as MuiMistralForCausalLM  # noqa: F401
from ..llama.model import MuiLlamaModel as MuiMistralModel  # noqa: F401
