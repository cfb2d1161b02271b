"""muillm_amd: muiLLM's decode-time hot path for AMD MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (libmuillm_amd.so, include/muillm_amd.h) with a
Python layer that keeps the reference's module API (MuiLinear, MuiMultiLinear,
MuiGateUpDownMLP, MuiRMSNorm, attention + static KV cache, init_engine).
"""

__version__ = "0.1.0"
