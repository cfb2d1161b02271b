"""`muillm_ext`-shaped operator layer over the C ABI.

The reference binds its HIP kernels through a pybind11 module called `muillm_ext`
(csrc/module.cpp:177-432).  This module keeps those function names, argument orders and
error behaviour (RuntimeError/ValueError instead of TORCH_CHECK) so the layer classes in
muillm_amd.modules read like the reference's, but every function here only validates its
tensors, allocates the output with torch and hands raw device pointers plus the current HIP
stream to libmuillm_amd.so.

Dispatch rule (csrc/modules/linear_module.cpp:39-80): the fused kernels serve 16-bit CUDA
tensors holding 1..MUI_MAX_TOKENS tokens; anything else (prefill, fp32) takes the
reference's own unfused route -- RMSNorm kernel, torch matmul, residual add -- on the same
device.  There is no CPU fallback for CUDA inputs and no silent one for a missing library.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib
from ._lib import MUI_DTYPE_BF16, MUI_DTYPE_F16, MUI_MAX_TOKENS, check


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------
def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return MUI_DTYPE_F16
    if t.dtype == torch.bfloat16:
        return MUI_DTYPE_BF16
    raise ValueError(f"unsupported dtype {t.dtype}: the fused kernels take fp16 or bf16")


def _is_16bit(t: torch.Tensor) -> bool:
    return t.dtype in (torch.float16, torch.bfloat16)


def _check_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")


def _check_contiguous(t: torch.Tensor, name: str) -> None:
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _row_pitch(w: torch.Tensor, name: str) -> int:
    """Row pitch (elements) of a 2-D weight whose rows are dense."""
    if w.dim() != 2 or w.stride(1) != 1:
        raise RuntimeError(f"{name} must be 2-D with unit inner stride")
    return w.stride(0) if w.shape[0] > 1 else max(w.stride(0), w.shape[1])


def _num_tokens(x: torch.Tensor) -> int:
    return x.numel() // x.shape[-1]


def kernel_dispatchable(x: torch.Tensor) -> bool:
    """True when the fused decode kernels take this input."""
    return x.is_cuda and _is_16bit(x) and 1 <= _num_tokens(x) <= MUI_MAX_TOKENS and x.shape[-1] % 8 == 0


# --------------------------------------------------------------------------------------
# engine  (csrc/module.cpp:283, csrc/engine.cpp:3-26)
# --------------------------------------------------------------------------------------
class MuiEngine:
    """Stand-in for muillm_engine_ptr: device facts for the current GPU."""

    def __init__(self, device_index: int):
        self.device_index = device_index
        self.info = _lib.device_info(device_index)

    @property
    def simd_lanes(self) -> int:
        return int(self.info["simd_lanes"])


def muillm_engine_init() -> MuiEngine:
    _lib.load()
    if not torch.cuda.is_available():
        raise RuntimeError("muillm_engine_init: no HIP device is visible")
    return MuiEngine(torch.cuda.current_device())


# --------------------------------------------------------------------------------------
# RMSNorm  (csrc/module.cpp:251, csrc/norm/rmsnorm.cu:31-85)
# --------------------------------------------------------------------------------------
def muillm_rmsnorm_forward(weights: torch.Tensor, inputs: torch.Tensor, epsilon: float) -> torch.Tensor:
    _check_cuda(weights, "weights")
    _check_cuda(inputs, "inputs")
    _check_contiguous(weights, "weights")
    if inputs.dtype != weights.dtype:
        raise RuntimeError("rmsnorm: inputs and weights must have the same dtype")
    x = inputs.contiguous()
    k = x.shape[-1]
    if weights.numel() != k:
        raise RuntimeError("rmsnorm: weights must have as many elements as the last input dim")
    y = torch.empty_like(x)
    rows = x.numel() // k
    if rows == 0:
        return y
    check(
        _lib.load().mui_rmsnorm(_stream(x), _dtype_code(x), weights.data_ptr(), x.data_ptr(),
                                float(epsilon), y.data_ptr(), rows, k),
        "mui_rmsnorm",
    )
    return y


# --------------------------------------------------------------------------------------
# Linear  (csrc/module.cpp:178,310-312; csrc/linear/linear.cu:76-208;
#          csrc/modules/linear_module.cpp:39-80)
# --------------------------------------------------------------------------------------
def _linear_unfused(x, weights, norm_weights, epsilon, mul_bias, add_bias, residual):
    """The reference's non-single-token branch (csrc/modules/linear_module.cpp:57-79)."""
    if norm_weights is not None:
        x = muillm_rmsnorm_forward(norm_weights, x, epsilon) if (x.is_cuda and _is_16bit(x)) else _rmsnorm_torch(x, norm_weights, epsilon)
    out = F.linear(x, weights, None)
    if mul_bias is not None:
        out = out * mul_bias
    if add_bias is not None:
        out = out + add_bias
    if residual is not None:
        out = out + residual
    return out


def _rmsnorm_torch(x, w, eps):
    h = x.to(torch.float32)
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return w * h.to(x.dtype)


def muillm_linear_forward(
    engine: Optional[MuiEngine],
    x: torch.Tensor,
    weights: torch.Tensor,
    norm_weights: Optional[torch.Tensor] = None,
    epsilon: float = 0.0,
    mul_bias: Optional[torch.Tensor] = None,
    add_bias: Optional[torch.Tensor] = None,
    residual: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """y = (W . rmsnorm?(x)) * mul_bias + add_bias + residual, output shape x.shape[:-1] + [N]."""
    if weights.dim() != 2:
        raise RuntimeError("weights must be 2-D [out_features, in_features]")
    n, k = weights.shape
    if x.shape[-1] != k:
        raise RuntimeError(f"input has {x.shape[-1]} features but weights expect {k}")
    if x.device != weights.device:
        raise RuntimeError("x and weights must be on the same device")

    if not (kernel_dispatchable(x) and weights.dtype == x.dtype):
        return _linear_unfused(x, weights, norm_weights, epsilon, mul_bias, add_bias, residual)

    _check_cuda(weights, "weights")
    pitch = _row_pitch(weights, "weights")
    x = x.contiguous()
    for name, t, size in (("norm_weights", norm_weights, k), ("mul_bias", mul_bias, n), ("add_bias", add_bias, n)):
        if t is not None:
            _check_cuda(t, name)
            _check_contiguous(t, name)
            if t.dtype != x.dtype or t.numel() != size:
                raise RuntimeError(f"{name} must be a {x.dtype} vector of {size} elements")
    tokens = _num_tokens(x)
    out_shape = list(x.shape[:-1]) + [n]
    if residual is not None:
        _check_cuda(residual, "residual")
        if residual.dtype != x.dtype or residual.numel() != tokens * n:
            raise RuntimeError("residual must match the output's shape and dtype")
        residual = residual.contiguous()
    y = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    check(
        _lib.load().mui_linear(
            _stream(x), _dtype_code(x), weights.data_ptr(), pitch, x.data_ptr(),
            _ptr(norm_weights), float(epsilon), _ptr(mul_bias), _ptr(add_bias), _ptr(residual),
            y.data_ptr(), n, k, tokens,
        ),
        "mui_linear",
    )
    return y


class MuiLinearModuleHandle:
    """Stand-in for muillm_linear_module_ptr (csrc/modules/linear_module.h:43-45): aliases
    the Python-owned tensors, owns nothing."""

    def __init__(self, engine, weights, norm_weights, epsilon, mul_bias, add_bias):
        self.engine = engine
        self.weights = weights
        self.norm_weights = norm_weights
        self.epsilon = float(epsilon)
        self.mul_bias = mul_bias
        self.add_bias = add_bias


def muillm_linear_module_init(engine, weights, norm_weights=None, epsilon=0.0, mul_bias=None, add_bias=None):
    return MuiLinearModuleHandle(engine, weights, norm_weights, epsilon, mul_bias, add_bias)


def muillm_linear_module_deinit(module: MuiLinearModuleHandle) -> None:
    module.weights = module.norm_weights = module.mul_bias = module.add_bias = None


def muillm_linear_module_forward(module: MuiLinearModuleHandle, inputs: torch.Tensor, residual=None):
    return muillm_linear_forward(
        module.engine, inputs, module.weights, module.norm_weights, module.epsilon,
        module.mul_bias, module.add_bias, residual,
    )


# --------------------------------------------------------------------------------------
# Gate/Up/Down MLP  (csrc/module.cpp:182,215; csrc/ffn/gateup.cu:88-391)
# --------------------------------------------------------------------------------------
def mui_gateup_silu(norm_weights, epsilon, gate_weights, up_weights, x) -> torch.Tensor:
    """h = silu(G xn) * (U xn) for 1..MUI_MAX_TOKENS tokens; gate/up may be views into one
    interleaved [N, 2, K] buffer (common row pitch)."""
    n, k = gate_weights.shape
    if up_weights.shape != gate_weights.shape:
        raise RuntimeError("gate and up weights must have the same shape")
    pitch = _row_pitch(gate_weights, "gate_weights")
    if _row_pitch(up_weights, "up_weights") != pitch:
        raise RuntimeError("gate and up weights must share one row pitch")
    x = x.contiguous()
    tokens = _num_tokens(x)
    h = torch.empty(list(x.shape[:-1]) + [n], dtype=x.dtype, device=x.device)
    check(
        _lib.load().mui_gateup_silu(
            _stream(x), _dtype_code(x), gate_weights.data_ptr(), up_weights.data_ptr(), pitch,
            x.data_ptr(), _ptr(norm_weights), float(epsilon), h.data_ptr(), n, k, tokens,
        ),
        "mui_gateup_silu",
    )
    return h


def muillm_gateupsilu_forward(engine, norm_weights, epsilon, gate_weights, up_weights, down_weights,
                              residual, x) -> torch.Tensor:
    """out = Wd (silu(Wg xn) * (Wu xn)) + residual, argument order of csrc/module.cpp:182."""
    if not (kernel_dispatchable(x) and gate_weights.dtype == x.dtype):
        raise RuntimeError("muillm_gateupsilu_forward needs 1..8 tokens of a 16-bit CUDA tensor")
    h = mui_gateup_silu(norm_weights, epsilon, gate_weights, up_weights, x)
    return muillm_linear_forward(engine, h, down_weights, residual=residual)


def muillm_gateupsilu_split_forward(engine, norm_weights, epsilon, gate_weights, up_weights,
                                    down_weights, residual, x) -> torch.Tensor:
    """The reference's split-K variant (csrc/module.cpp:215) exists to create more blocks on
    MI300; the gfx950 kernel already sizes its grid to the CU count, so both names run the
    same path."""
    return muillm_gateupsilu_forward(engine, norm_weights, epsilon, gate_weights, up_weights,
                                     down_weights, residual, x)
