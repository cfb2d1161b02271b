"""mui_causally_decode(_masked) -- muillm/modules/attention/causaltransformerdecoding.py:7-58."""
import torch

from ... import muillm_ext


class _MuiCausalDecoding(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v):
        return muillm_ext.muillm_causal_transformer_decoding_no_mask(q, k, v)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("causal decoding backward not implemented")


class _MuiMaskedCausalDecoding(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, m):
        return muillm_ext.muillm_causal_transformer_decoding_masked(q, k, v, m)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("causal decoding backward not implemented")


def mui_causally_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """q [B, Hq, 1, D], k/v [B, Hkv, S, D] -> [B, 1, Hq*D]."""
    return _MuiCausalDecoding.apply(q, k, v)


def mui_causally_decode_masked(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, m: torch.Tensor) -> torch.Tensor:
    """As above with m [B, 1, 1, S]: 0 keeps a key, torch.finfo(dtype).min (anything non-zero) drops it."""
    return _MuiMaskedCausalDecoding.apply(q, k, v, m)
