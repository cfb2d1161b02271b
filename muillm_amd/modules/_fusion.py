"""Host-side helpers shared by the layer classes: what a layer needs to know about an RMSNorm it
absorbs, the torch formula used where no kernel applies, and parameter loading."""
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn


@dataclass
class AbsorbedNorm:
    """An RMSNorm that a following projection applies itself: its gain vector and epsilon."""
    gain: torch.Tensor
    eps: float

    @staticmethod
    def of(norm_module: Optional[nn.Module]) -> Optional["AbsorbedNorm"]:
        """Read gain and epsilon off any RMSNorm-like module (HuggingFace spells the epsilon
        `variance_epsilon`, torch's own RMSNorm `eps`)."""
        if norm_module is None:
            return None
        eps = getattr(norm_module, "variance_epsilon", None)
        if eps is None:
            eps = getattr(norm_module, "eps", None)
        if eps is None:
            raise ValueError(f"{type(norm_module).__name__} carries no epsilon: not an RMSNorm this build can absorb")
        return AbsorbedNorm(gain=norm_module.weight, eps=float(eps))


def rmsnorm_reference(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """gain * (x / sqrt(mean(x^2) + eps)) with the statistics in fp32 and the normalised value
    rounded to x's dtype before the gain (muillm/modules/norm/rmsnorm.py:138-146: the HuggingFace form)."""
    x32 = x.float()
    inv = torch.rsqrt(x32.square().mean(dim=-1, keepdim=True) + eps)
    return gain * (x32 * inv).to(x.dtype)


def fill_parameter(param: nn.Parameter, values: torch.Tensor, requires_grad: Optional[bool] = None) -> None:
    """Overwrite a parameter in place (its storage, device and dtype stay); the gradient flag
    follows the source tensor unless given."""
    with torch.no_grad():
        param.copy_(values)
    param.requires_grad = values.requires_grad if requires_grad is None else bool(requires_grad)


def uniform_flag(flags, what: str) -> bool:
    """The common value of a list of booleans; a mixture is an error."""
    flags = [bool(f) for f in flags]
    if len(set(flags)) > 1:
        raise ValueError(f"{what}: the fused layers must agree, got {flags}")
    return flags[0] if flags else False


def is_kernel_dtype(t: torch.Tensor) -> bool:
    return t.is_cuda and t.dtype in (torch.float16, torch.bfloat16)
