"""Optional HuggingFace Transformers types used as replace() inputs and table keys.

The layer classes depend on torch only; when transformers is importable its Llama/Mistral
layer classes become valid inputs to the replace() constructors (as in the reference, which
pins transformers 4.52.4, setup.py:145). Placeholders keep isinstance() checks valid when
it is not."""


def _placeholder(name):
    return type(name, (), {"__doc__": f"placeholder for transformers' {name} (transformers not installed)"})


try:  # pragma: no cover - exercised wherever transformers is installed
    from transformers.models.llama.configuration_llama import LlamaConfig
    from transformers.models.llama.modeling_llama import (
        LlamaAttention,
        LlamaDecoderLayer,
        LlamaForCausalLM,
        LlamaMLP,
        LlamaModel,
        LlamaRMSNorm,
        LlamaRotaryEmbedding,
    )
    from transformers.models.mistral.configuration_mistral import MistralConfig
    from transformers.models.mistral.modeling_mistral import (
        MistralAttention,
        MistralDecoderLayer,
        MistralForCausalLM,
        MistralMLP,
        MistralModel,
        MistralRMSNorm,
        MistralRotaryEmbedding,
    )

    HAVE_TRANSFORMERS = True
except Exception:  # pragma: no cover
    HAVE_TRANSFORMERS = False
    for _n in (
        "LlamaConfig", "LlamaAttention", "LlamaDecoderLayer", "LlamaForCausalLM", "LlamaMLP", "LlamaModel",
        "LlamaRMSNorm", "LlamaRotaryEmbedding", "MistralConfig", "MistralAttention", "MistralDecoderLayer",
        "MistralForCausalLM", "MistralMLP", "MistralModel", "MistralRMSNorm", "MistralRotaryEmbedding",
    ):
        globals()[_n] = _placeholder(_n)


def rope_theta_of(config) -> float:
    """rope_theta across transformers versions (attribute in 4.x, rope_parameters dict in 5.x)."""
    rp = getattr(config, "rope_parameters", None)
    if isinstance(rp, dict) and "rope_theta" in rp:
        return float(rp["rope_theta"])
    theta = getattr(config, "rope_theta", None)
    return float(theta) if theta is not None else 10000.0


def rope_scaling_of(config):
    """The rope scaling dict (None for plain RoPE)."""
    rs = getattr(config, "rope_scaling", None)
    if rs is None:
        rp = getattr(config, "rope_parameters", None)
        if isinstance(rp, dict) and rp.get("rope_type", "default") not in (None, "default"):
            rs = rp
    return rs


def head_dim_of(config) -> int:
    hd = getattr(config, "head_dim", None)
    return int(hd) if hd else config.hidden_size // config.num_attention_heads
