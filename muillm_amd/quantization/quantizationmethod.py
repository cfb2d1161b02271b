"""Quantisation method descriptors -- muillm/quantization/quantizationmethod.py:1-24."""
from typing import List, Optional


class QuantizationMethod:
    """Base class of the supported quantisation methods. `modules` restricts quantisation to
    modules whose qualified name contains one of the given substrings."""

    def __init__(self, modules: Optional[List[str]] = None):
        self.modules = list(modules) if modules is not None else None


class Int8WeightOnlyQuantizationMethod(QuantizationMethod):
    """Weight-only 8-bit round-to-nearest.

    group_size > 0: the reference's asymmetric group-wise uint8 format (scale, min per group
    of `group_size` inputs; default 128 as in the reference).
    group_size == 0 (or None): symmetric per-output-channel int8 with one 16-bit scale per
    row, s = max|row| / 127 -- the format of the int8 decode benchmarks."""

    def __init__(self, group_size: Optional[int] = 128, f: float = 1.0, modules: Optional[List[str]] = None):
        super().__init__(modules)
        self.group_size = int(group_size) if group_size else 0
        self.f = f

    @property
    def per_channel(self) -> bool:
        return self.group_size == 0
