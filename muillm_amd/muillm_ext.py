"""`muillm_ext`-shaped operator layer over the C ABI.

The reference binds its HIP kernels through a pybind11 module called `muillm_ext`
(csrc/module.cpp:177-432).  This module keeps those function names, argument orders and
error behaviour (RuntimeError/ValueError instead of TORCH_CHECK) so the layer classes in
muillm_amd.modules read like the reference's, but every function here only validates its
tensors, allocates the output with torch and hands raw device pointers plus the current HIP
stream to libmuillm_amd.so.

Dispatch rule (csrc/modules/linear_module.cpp:39-80 hands everything but a single token to the
framework's GEMM): here the library's kernels serve 16-bit CUDA tensors of any token count --
1..MUI_MAX_TOKENS tokens the weight-streaming decode kernels, more tokens the tiled matrix-core GEMM
behind the same entry points (FUSED_CHUNK_MAX_TOKENS can send short prompts through the decode
kernels in chunks instead). Only fp32 and CPU
tensors take the reference's unfused route (RMSNorm, torch matmul, residual add).  There is no
CPU fallback for CUDA inputs and no silent one for a missing library.
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


_MAX_CALL_TOKENS = 1 << 20  # tokens one library call may carry (a sanity bound, not a kernel limit)


def _check_activations(x: torch.Tensor, k: int, what: str, max_tokens: int, *others) -> None:
    """What every fused entry point needs of its operands before raw pointers go to a kernel: a
    16-bit CUDA activation tensor with k features and a token count the kernels take, and every
    other operand on the same device. The kernels read k values per token: a shorter x would be
    read out of bounds."""
    _check_cuda(x, what + " input")
    if not _is_16bit(x):
        raise RuntimeError(f"{what}: activations must be fp16 or bf16, got {x.dtype}")
    if x.dim() < 1 or x.shape[-1] != k:
        raise RuntimeError(f"{what}: input has {x.shape[-1] if x.dim() else 0} features but the weights expect {k}")
    tokens = _num_tokens(x)
    if not 1 <= tokens <= max_tokens:
        raise RuntimeError(f"{what}: {tokens} tokens, the fused kernels take 1..{max_tokens}")
    for o in others:
        if o is not None and (not o.is_cuda or o.device != x.device):
            raise RuntimeError(f"{what}: every operand must live on the activations' device {x.device}")


# Up to this many tokens go through the decode kernels in chunks of MUI_MAX_TOKENS (each chunk
# streams the weights once more); more take the tiled matrix-core GEMM of the same entry points in
# one call. MUI_MAX_TOKENS = no chunking: an 8B-shaped prefill of 17-32 tokens takes 5.4-5.5 ms on the
# GEMM against 5.8-6.3 ms in two chunks.
FUSED_CHUNK_MAX_TOKENS = MUI_MAX_TOKENS


def kernel_dispatchable(x: torch.Tensor) -> bool:
    """True when the library's kernels take this input: any number of 16-bit CUDA tokens."""
    return x.is_cuda and _is_16bit(x) and _num_tokens(x) >= 1 and x.shape[-1] % 8 == 0


# False: prompts keep the RMSNorm fused into the tiled GEMM (the C entry points take either form)
PROMPT_NORM_FIRST = True


def _norm_first(x: torch.Tensor, norm_weights: Optional[torch.Tensor], epsilon: float, chunk_max: int):
    """Prompts (more tokens than the decode kernels take in chunks) are normalised by one rmsnorm
    launch before the tiled GEMM instead of inside it: every row tile of the GEMM would redo
    gamma * x and the sums of squares for its token tile, which costs 8-13 us per call from 33
    tokens on and 10 % at 2048-4096 tokens (gate/up at 2048 tokens 511 us fused, 458 + 5.5 us
    apart); the decode kernels read x once per call and keep the norm fused. Same arithmetic as
    the reference's multi-token route (rmsnorm kernel, then the GEMM; muillm/modules/linear.py:324-333)."""
    if PROMPT_NORM_FIRST and norm_weights is not None and _num_tokens(x) > chunk_max:
        return muillm_rmsnorm_forward(norm_weights, x.contiguous(), epsilon), None
    return x, norm_weights


# Scratch of the prompt GEMM (mui_linear_ws), one per device and stream: calls on one stream follow
# each other and can share it, calls on different streams may overlap. Zero-filled once.
_PROMPT_WORKSPACES: dict = {}


def _prompt_workspace(x: torch.Tensor) -> Optional[torch.Tensor]:
    key = (x.device.index, torch.cuda.current_stream(x.device).cuda_stream)
    ws = _PROMPT_WORKSPACES.get(key)
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            return None  # no allocation inside a capture: the call runs without the workspace
        ws = torch.zeros(_lib.load().mui_linear_workspace_bytes(), dtype=torch.uint8, device=x.device)
        _PROMPT_WORKSPACES[key] = ws
    return ws


def _token_calls(tokens: int, chunk_max: int):
    """(first token, count) of the library calls that cover `tokens` rows: chunks of MUI_MAX_TOKENS
    for the decode kernels up to chunk_max tokens, one call (the tiled GEMM) beyond."""
    if tokens > chunk_max:
        return [(0, tokens)]
    return [(off, min(MUI_MAX_TOKENS, tokens - off)) for off in range(0, tokens, MUI_MAX_TOKENS)]


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
    if residual is not None and mul_bias is None and x.is_cuda and _is_16bit(x) and residual.dtype == x.dtype:
        # the residual (and bias) ride in the GEMM epilogue: one kernel, one rounding
        out = torch.addmm(residual.reshape(-1, weights.shape[0]), x.reshape(-1, x.shape[-1]), weights.t())
        out = out.reshape(x.shape[:-1] + (weights.shape[0],))
        return out if add_bias is None else out + add_bias
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
    if k > 16384 and norm_weights is not None and _num_tokens(x) <= FUSED_CHUNK_MAX_TOKENS:
        # a fused norm needs the whole row in one pass of the 1..4-token kernels: norm kernel first
        x = muillm_rmsnorm_forward(norm_weights, x, epsilon)
        norm_weights = None

    _check_cuda(weights, "weights")
    pitch = _row_pitch(weights, "weights")
    x = x.contiguous()
    for name, t, size in (("norm_weights", norm_weights, k), ("mul_bias", mul_bias, n), ("add_bias", add_bias, n)):
        if t is not None:
            _check_cuda(t, name)
            _check_contiguous(t, name)
            if t.dtype != x.dtype or t.numel() != size:
                raise RuntimeError(f"{name} must be a {x.dtype} vector of {size} elements")
    x, norm_weights = _norm_first(x, norm_weights, epsilon, FUSED_CHUNK_MAX_TOKENS)
    tokens = _num_tokens(x)
    out_shape = list(x.shape[:-1]) + [n]
    if residual is not None:
        _check_cuda(residual, "residual")
        if residual.dtype != x.dtype or residual.numel() != tokens * n:
            raise RuntimeError("residual must match the output's shape and dtype")
        residual = residual.contiguous()
    y = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    lib, stream, code, esz = _lib.load(), _stream(x), _dtype_code(x), x.element_size()
    ws = _prompt_workspace(x) if tokens > FUSED_CHUNK_MAX_TOKENS else None
    for off, cnt in _token_calls(tokens, FUSED_CHUNK_MAX_TOKENS):
        check(
            lib.mui_linear_ws(
                stream, code, weights.data_ptr(), pitch, x.data_ptr() + off * k * esz,
                _ptr(norm_weights), float(epsilon), _ptr(mul_bias), _ptr(add_bias),
                None if residual is None else residual.data_ptr() + off * n * esz,
                y.data_ptr() + off * n * esz, n, k, cnt,
                None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(),
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
    _check_activations(x, k, "mui_gateup_silu", _MAX_CALL_TOKENS, gate_weights, up_weights, norm_weights)
    if gate_weights.dtype != x.dtype or up_weights.dtype != x.dtype or \
            (norm_weights is not None and (norm_weights.dtype != x.dtype or norm_weights.numel() != k)):
        raise RuntimeError("mui_gateup_silu: weights and norm weights must have the activations' dtype "
                           "(norm weights: one value per input feature)")
    x = x.contiguous()
    x, norm_weights = _norm_first(x, norm_weights, epsilon, FUSED_CHUNK_MAX_TOKENS)
    tokens = _num_tokens(x)
    h = torch.empty(list(x.shape[:-1]) + [n], dtype=x.dtype, device=x.device)
    lib, stream, code, esz = _lib.load(), _stream(x), _dtype_code(x), x.element_size()
    for off, cnt in _token_calls(tokens, FUSED_CHUNK_MAX_TOKENS):
        check(
            lib.mui_gateup_silu(
                stream, code, gate_weights.data_ptr(), up_weights.data_ptr(), pitch,
                x.data_ptr() + off * k * esz, _ptr(norm_weights), float(epsilon),
                h.data_ptr() + off * n * esz, n, k, cnt,
            ),
            "mui_gateup_silu",
        )
    return h


def mui_silu_mul_interleaved(gate_up: torch.Tensor) -> torch.Tensor:
    """[..., 2 * n] with (gate, up) pairs adjacent -> silu(gate) * up, [..., n]."""
    _check_cuda(gate_up, "gate_up")
    n = gate_up.shape[-1] // 2
    gu = gate_up if gate_up.is_contiguous() else gate_up.contiguous()
    out = torch.empty(gu.shape[:-1] + (n,), dtype=gu.dtype, device=gu.device)
    check(_lib.load().mui_silu_mul_interleaved(_stream(gu), _dtype_code(gu), gu.data_ptr(), out.data_ptr(),
                                               gu.numel() // (2 * n), n), "mui_silu_mul_interleaved")
    return out


def muillm_gateupsilu_forward(engine, norm_weights, epsilon, gate_weights, up_weights, down_weights,
                              residual, x) -> torch.Tensor:
    """out = Wd (silu(Wg xn) * (Wu xn)) + residual, argument order of csrc/module.cpp:182."""
    if not (kernel_dispatchable(x) and gate_weights.dtype == x.dtype):
        raise RuntimeError("muillm_gateupsilu_forward needs fp16 / bf16 CUDA tensors with k % 8 == 0")
    h = mui_gateup_silu(norm_weights, epsilon, gate_weights, up_weights, x)
    return muillm_linear_forward(engine, h, down_weights, residual=residual)


def muillm_gateupsilu_split_forward(engine, norm_weights, epsilon, gate_weights, up_weights,
                                    down_weights, residual, x) -> torch.Tensor:
    """The reference's split-K variant (csrc/module.cpp:215) exists to create more blocks on
    MI300; the gfx950 kernel already sizes its grid to the CU count, so both names run the
    same path."""
    return muillm_gateupsilu_forward(engine, norm_weights, epsilon, gate_weights, up_weights,
                                     down_weights, residual, x)


# --------------------------------------------------------------------------------------
# int8 weight-only  (csrc/module.cpp:180-181,247-248)
# --------------------------------------------------------------------------------------
def _byte_pitch(w: torch.Tensor, name: str) -> int:
    if w.dim() != 2 or w.stride(1) != 1 or w.element_size() != 1:
        raise RuntimeError(f"{name} must be a 2-D 8-bit tensor with unit inner stride")
    return w.stride(0) if w.shape[0] > 1 else max(w.stride(0), w.shape[1])


# int8 weights: the decode kernels take chunks of MUI_MAX_TOKENS up to this many tokens; beyond, the
# tiled matrix-core GEMM converts the codes on their way to LDS (per-channel format: no chunking,
# 64 tokens of an 8B-shaped prefill take 5.6 ms on the GEMM against 8.9 ms in four chunks; group
# format: 17..32 tokens 6.4 ms on the GEMM against 7.1 ms in two chunks); long prompts run on the
# matrix dequantised by the library's kernel (about 4 ms per 8B-shaped pass).
INT8_CHUNK_MAX_TOKENS = MUI_MAX_TOKENS
INT8_GROUP_CHUNK_MAX_TOKENS = MUI_MAX_TOKENS
# Per-channel format from this many tokens: the matrix is dequantised once per call (12–32 µs per
# Llama-3-8B matrix) and the GEMM runs its software-pipelined loop on 16-bit weights, which the
# converting loop cannot use (at 4096 tokens QKV 227 -> 182 µs, o_proj 128 -> 118, down 389 -> 381,
# gate/up 817 -> 762; an 8B-shaped prefill 27.5 -> 25.8 ms at 1536 tokens, while at 1024 tokens the
# conversion on the way to LDS is still ahead, 17.7 against 19.5 ms).
INT8_DEQUANT_MIN_TOKENS = 1280
# The group format likewise, from 1024 tokens; 33 .. 1023 tokens go to the GEMM that applies (scale, min)
# on the way to LDS (an 8B-shaped prefill of 64 tokens 9.4 -> 6.1 ms, 512 tokens 14.3 -> 12.1 ms, level at
# 1024, 35.0 against 29.9 ms at 2048).
INT8_GROUP_DEQUANT_MIN_TOKENS = 1024


def int8_kernel_dispatchable(x: torch.Tensor) -> bool:
    # rows longer than 16384: fp16 activations only (K segments / the streaming matrix-core kernel)
    return x.is_cuda and _is_16bit(x) and _num_tokens(x) >= 1 \
        and x.shape[-1] % 16 == 0 and (x.shape[-1] <= 16384 or x.dtype == torch.float16)


def _token_chunks(tokens: int, group_format: bool = False):
    """(first token, count) of the int8 calls that cover `tokens` rows."""
    return _token_calls(tokens, INT8_GROUP_CHUNK_MAX_TOKENS if group_format else INT8_CHUNK_MAX_TOKENS)


def mui_int8_channel_dequantize_forward(weights_i8: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """Per-channel format: out = T(float(q) * float(s[n])), bit-identical to q.to(T) * s[:, None]."""
    _check_cuda(weights_i8, "weights")
    n, k = weights_i8.shape
    if weights_i8.dtype != torch.int8:
        raise RuntimeError("per-channel weights must be int8")
    if k % 16 != 0:
        return weights_i8.to(scales.dtype) * scales.reshape(-1, 1)
    out = torch.empty((n, k), dtype=scales.dtype, device=weights_i8.device)
    sstride = scales.stride(0) if scales.dim() >= 1 and scales.numel() > 1 else 1
    check(
        _lib.load().mui_int8_dequantize(_stream(weights_i8), _dtype_code(scales), weights_i8.data_ptr(),
                                        _byte_pitch(weights_i8, "weights"), scales.data_ptr(), sstride,
                                        out.data_ptr(), k, n, k),
        "mui_int8_dequantize",
    )
    return out


def mui_int8_channel_linear_forward(x, weights_i8, scales, norm_weights=None, epsilon=0.0,
                                    add_bias=None, residual=None) -> torch.Tensor:
    """y = (q * s) xn + add_bias + residual on the symmetric per-channel format."""
    n, k = weights_i8.shape
    if x.shape[-1] != k:
        raise RuntimeError(f"input has {x.shape[-1]} features but weights expect {k}")
    if not int8_kernel_dispatchable(x):
        w = mui_int8_channel_dequantize_forward(weights_i8, scales)
        return _linear_unfused(x, w, norm_weights, epsilon, None, add_bias, residual)
    _check_cuda(weights_i8, "weights")
    _check_contiguous(scales, "scales")
    if scales.dtype != x.dtype or scales.numel() != n:
        raise RuntimeError("scales must be one value per output row in the activation dtype")
    x = x.contiguous()
    x, norm_weights = _norm_first(x, norm_weights, epsilon, INT8_CHUNK_MAX_TOKENS)
    tokens = _num_tokens(x)
    if tokens >= INT8_DEQUANT_MIN_TOKENS and k % 16 == 0:
        w = mui_int8_channel_dequantize_forward(weights_i8, scales)
        return muillm_linear_forward(None, x, w, norm_weights, epsilon, None, add_bias, residual)
    if residual is not None:
        residual = residual.contiguous()
    y = torch.empty(list(x.shape[:-1]) + [n], dtype=x.dtype, device=x.device)
    esz = x.element_size()
    for off, cnt in _token_chunks(tokens):
        check(
            _lib.load().mui_int8_linear(_stream(x), _dtype_code(x), weights_i8.data_ptr(),
                                        _byte_pitch(weights_i8, "weights"), scales.data_ptr(),
                                        x.data_ptr() + off * k * esz, _ptr(norm_weights), float(epsilon),
                                        _ptr(add_bias),
                                        None if residual is None else residual.data_ptr() + off * n * esz,
                                        y.data_ptr() + off * n * esz, n, k, cnt),
            "mui_int8_linear",
        )
    return y


def mui_int8_channel_gateupsilu_forward(norm_weights, epsilon, gate_i8, up_i8, gate_scales, up_scales, x):
    """h = silu(sg * Gq xn) * (su * Uq xn); gate/up (and their scales) may be views into
    row-interleaved [N, 2, K] / [N, 2] buffers."""
    n, k = gate_i8.shape
    pitch = _byte_pitch(gate_i8, "gate weights")
    if _byte_pitch(up_i8, "up weights") != pitch or up_i8.shape != gate_i8.shape:
        raise RuntimeError("gate and up weights must share shape and row pitch")
    sstride = gate_scales.stride(0) if gate_scales.numel() > 1 else 1
    if (up_scales.stride(0) if up_scales.numel() > 1 else 1) != sstride:
        raise RuntimeError("gate and up scales must share one stride")
    _check_activations(x, k, "mui_int8_channel_gateupsilu_forward", _MAX_CALL_TOKENS,
                       gate_i8, up_i8, gate_scales, up_scales, norm_weights)
    if not int8_kernel_dispatchable(x):
        raise RuntimeError("mui_int8_channel_gateupsilu_forward: the int8 kernels need k % 16 == 0 "
                           "(and fp16 activations beyond 16384 features)")
    if gate_i8.dtype != torch.int8 or up_i8.dtype != torch.int8:
        raise RuntimeError("per-channel gate/up weights must be int8")
    if gate_scales.dtype != x.dtype or up_scales.dtype != x.dtype or gate_scales.numel() != n or up_scales.numel() != n:
        raise RuntimeError("gate/up scales must be one value per row in the activation dtype")
    if norm_weights is not None and (norm_weights.dtype != x.dtype or norm_weights.numel() != k):
        raise RuntimeError("norm weights must be one value per input feature in the activation dtype")
    x = x.contiguous()
    x, norm_weights = _norm_first(x, norm_weights, epsilon, INT8_CHUNK_MAX_TOKENS)
    tokens = _num_tokens(x)
    if tokens >= INT8_DEQUANT_MIN_TOKENS:
        return mui_gateup_silu(norm_weights, epsilon, mui_int8_channel_dequantize_forward(gate_i8, gate_scales),
                               mui_int8_channel_dequantize_forward(up_i8, up_scales), x)
    h = torch.empty(list(x.shape[:-1]) + [n], dtype=x.dtype, device=x.device)
    esz = x.element_size()
    for off, cnt in _token_chunks(tokens):
        check(
            _lib.load().mui_int8_gateup_silu(_stream(x), _dtype_code(x), gate_i8.data_ptr(), up_i8.data_ptr(),
                                             pitch, gate_scales.data_ptr(), up_scales.data_ptr(), sstride,
                                             x.data_ptr() + off * k * esz, _ptr(norm_weights), float(epsilon),
                                             h.data_ptr() + off * n * esz, n, k, cnt),
            "mui_int8_gateup_silu",
        )
    return h


def muillm_int8_dequantize_forward(weights: torch.Tensor, scales_min_vals: torch.Tensor,
                                   group_size_shift: int) -> torch.Tensor:
    """Reference RTN group format -> dense 16-bit weights (csrc/module.cpp:180)."""
    _check_cuda(weights, "weights")
    n, k = weights.shape
    g = k >> group_size_shift
    out = torch.empty((n, k), dtype=scales_min_vals.dtype, device=weights.device)
    smv = scales_min_vals
    smv_pitch = 2 * g if smv.is_contiguous() and smv.numel() == n * g * 2 else smv.reshape(n, -1).stride(0)
    check(
        _lib.load().mui_int8_group_dequantize(_stream(weights), _dtype_code(smv), weights.data_ptr(),
                                              _byte_pitch(weights, "weights"), smv.data_ptr(), smv_pitch,
                                              int(group_size_shift), out.data_ptr(), k, n, k),
        "mui_int8_group_dequantize",
    )
    return out


def muillm_int8_linear_forward(x, weights, scales_min_vals, group_size_shift, norm_weights=None,
                               epsilon=0.0, mul_bias=None, add_bias=None, residual=None) -> torch.Tensor:
    """csrc/module.cpp:181 on the reference's uint8 group format. `residual` is an extension:
    the reference routes it through add_bias (muillm/modules/quantized/int8linear.py:53-57)."""
    if mul_bias is not None:
        raise RuntimeError("mul_bias is not supported by the int8 kernels")
    n, k = weights.shape
    if not (int8_kernel_dispatchable(x) and group_size_shift >= 4):
        w = muillm_int8_dequantize_forward(weights, scales_min_vals, group_size_shift)
        return _linear_unfused(x, w, norm_weights, epsilon, None, add_bias, residual)
    if weights.dtype != torch.uint8:
        raise RuntimeError("group-quantised weights must be uint8")
    _check_contiguous(scales_min_vals, "scales_min_vals")
    _check_activations(x, k, "muillm_int8_linear_forward", _MAX_CALL_TOKENS, weights,
                       scales_min_vals, norm_weights, add_bias, residual)
    if _num_tokens(x) >= INT8_GROUP_DEQUANT_MIN_TOKENS:
        # a long prompt: the reference's route (dequantise the matrix, then a GEMM,
        # muillm/modules/quantized/int8linear.py:279-293) on this library's kernels; shorter ones go
        # to the GEMM that dequantises the codes on their way to LDS (one call below)
        w = muillm_int8_dequantize_forward(weights, scales_min_vals, group_size_shift)
        return muillm_linear_forward(None, x, w, norm_weights, epsilon, None, add_bias, residual)
    if scales_min_vals.dtype != x.dtype or scales_min_vals.numel() != 2 * n * (k >> group_size_shift):
        raise RuntimeError("scales_min_vals must be [N * K / group, 2] (scale, min) pairs in the activation dtype")
    if norm_weights is not None and (norm_weights.dtype != x.dtype or norm_weights.numel() != k):
        raise RuntimeError("norm weights must be one value per input feature in the activation dtype")
    x = x.contiguous()
    x, norm_weights = _norm_first(x, norm_weights, epsilon, INT8_GROUP_CHUNK_MAX_TOKENS)
    tokens = _num_tokens(x)
    if add_bias is not None and add_bias.numel() == tokens * n and residual is None and tokens > 1:
        residual, add_bias = add_bias, None
    if residual is not None:
        residual = residual.contiguous()
    y = torch.empty(list(x.shape[:-1]) + [n], dtype=x.dtype, device=x.device)
    esz = x.element_size()
    for off, cnt in _token_chunks(tokens, group_format=True):
        check(
            _lib.load().mui_int8_group_linear(_stream(x), _dtype_code(x), weights.data_ptr(),
                                              _byte_pitch(weights, "weights"), scales_min_vals.data_ptr(),
                                              int(group_size_shift), x.data_ptr() + off * k * esz,
                                              _ptr(norm_weights), float(epsilon), _ptr(add_bias),
                                              None if residual is None else residual.data_ptr() + off * n * esz,
                                              y.data_ptr() + off * n * esz, n, k, cnt),
            "mui_int8_group_linear",
        )
    return y


# Row-interleaved twins of gate/up buffers that arrived in the reference's per-element packing,
# keyed by the address and version of the source tensors (bounded: one entry per quantised MLP).
# An entry also holds weak references to the two source tensors' storages: a hit counts only while
# both are alive (an address handed out again by the allocator after the first model is freed must
# not find the first model's twin), and an entry whose sources have died is dropped.
_REPACKED_GATEUP: "OrderedDict" = None
_REPACKED_GATEUP_MAX = 256


def _storage_ref(t: torch.Tensor):
    """A callable that gives the identity (`_cdata`) of t's storage while that storage is alive and
    None once it has been freed; holds no reference that would keep the tensor alive."""
    import weakref

    st = t.untyped_storage()
    cdata = st._cdata
    alive = weakref.ref(st)  # dies with the Python storage object, which t keeps alive through its base
    holder = weakref.ref(t)
    return lambda: cdata if (holder() is not None or alive() is not None) else None


def _is_reference_gateup_packing(gate_up_weights: torch.Tensor) -> bool:
    """[N, K, 2] (the reference's per-element interleave) as opposed to [N, 2, K]."""
    return gate_up_weights.dim() == 3 and gate_up_weights.shape[2] == 2 and gate_up_weights.shape[1] != 2


def _row_interleaved_gateup(gate_up_weights: torch.Tensor, gate_up_scales_min_vals: torch.Tensor,
                            group_size_shift: int):
    """(weights [N, 2, K], scales_min_vals [N, 2, G, 2]) of a gate/up pair in either packing.

    The reference's own tensors ([N, K, 2] + [N*G, 2, 2], int8gateupdownmlp.py:211-230) are
    converted on first use by mui_int8_repack_gateup and the result is kept for as long as the
    source tensors are unchanged (same storage, same version counter), so a reference module that
    calls this entry point every step pays the conversion once. The twin costs as much device
    memory as the original."""
    global _REPACKED_GATEUP
    if not _is_reference_gateup_packing(gate_up_weights):
        if gate_up_weights.dim() != 3 or gate_up_weights.shape[1] != 2:
            raise RuntimeError("gate_up_weights must be [N, 2, K] (row-interleaved) or [N, K, 2] (the reference's)")
        return gate_up_weights, gate_up_scales_min_vals
    from collections import OrderedDict

    if _REPACKED_GATEUP is None:
        _REPACKED_GATEUP = OrderedDict()
    w, smv = gate_up_weights, gate_up_scales_min_vals
    _check_cuda(w, "gate_up_weights")
    _check_cuda(smv, "gate_up_scales_min_vals")
    n, k, _ = w.shape
    g = k >> group_size_shift
    if w.dtype != torch.uint8 or not w.is_contiguous() or not smv.is_contiguous() or smv.numel() != n * g * 4:
        raise RuntimeError("reference packing: gate_up_weights uint8 [N, K, 2] and gate_up_scales_min_vals "
                           "[N * K / group, 2, 2], both contiguous")
    key = (w.data_ptr(), smv.data_ptr(), w._version, smv._version, n, k, int(group_size_shift), smv.dtype)
    hit = _REPACKED_GATEUP.get(key)
    if hit is not None:
        out_w, out_smv, w_ref, smv_ref = hit
        if w_ref() == w.untyped_storage()._cdata and smv_ref() == smv.untyped_storage()._cdata:
            _REPACKED_GATEUP.move_to_end(key)
            return out_w, out_smv
        del _REPACKED_GATEUP[key]  # same address, other (or dead) storage: a stale twin
    for stale in [kk for kk, v in _REPACKED_GATEUP.items() if v[2]() is None or v[3]() is None]:
        del _REPACKED_GATEUP[stale]
    out_w = torch.empty((n, 2, k), dtype=torch.uint8, device=w.device)
    out_smv = torch.empty((n, 2, g, 2), dtype=smv.dtype, device=smv.device)
    check(_lib.load().mui_int8_repack_gateup(_stream(w), w.data_ptr(), smv.data_ptr(), int(group_size_shift),
                                             out_w.data_ptr(), out_smv.data_ptr(), n, k), "mui_int8_repack_gateup")
    _REPACKED_GATEUP[key] = (out_w, out_smv, _storage_ref(w), _storage_ref(smv))
    while len(_REPACKED_GATEUP) > _REPACKED_GATEUP_MAX:
        _REPACKED_GATEUP.popitem(last=False)
    return out_w, out_smv


def muillm_int8_gateupsilu_forward(norm_weights, epsilon, gate_up_weights, gate_up_scales_min_vals,
                                   group_size_shift, x) -> torch.Tensor:
    """csrc/module.cpp:248. Takes the reference's packing -- gate_up_weights uint8 [N, K, 2],
    gate_up_scales_min_vals [N*G, 2, 2] (int8gateupdownmlp.py:211-230) -- or this build's
    row-interleaved one, [N, 2, K] (row n of gate, then row n of up) with [N, 2, G, 2], which
    keeps each row one contiguous 128-bit-loadable stream; the first is converted once (see
    _row_interleaved_gateup)."""
    gate_up_weights, gate_up_scales_min_vals = _row_interleaved_gateup(gate_up_weights, gate_up_scales_min_vals,
                                                                       group_size_shift)
    n, two, k = gate_up_weights.shape
    g = k >> group_size_shift
    _check_activations(x, k, "muillm_int8_gateupsilu_forward", _MAX_CALL_TOKENS,
                       gate_up_weights, gate_up_scales_min_vals, norm_weights)
    if not int8_kernel_dispatchable(x) or group_size_shift < 4:
        raise RuntimeError("muillm_int8_gateupsilu_forward: the int8 kernels need k % 16 == 0 and groups of >= 16")
    if gate_up_weights.dtype != torch.uint8 or not gate_up_weights.is_contiguous():
        raise RuntimeError("gate_up_weights must be a contiguous uint8 tensor")
    if gate_up_scales_min_vals.dtype != x.dtype or gate_up_scales_min_vals.numel() != n * 2 * g * 2 \
            or not gate_up_scales_min_vals.is_contiguous():
        raise RuntimeError("gate_up_scales_min_vals must hold N * 2 * K / group (scale, min) pairs in the activation dtype")
    if norm_weights is not None and (norm_weights.dtype != x.dtype or norm_weights.numel() != k):
        raise RuntimeError("norm weights must be one value per input feature in the activation dtype")
    if _num_tokens(x) >= INT8_GROUP_DEQUANT_MIN_TOKENS:
        # a long prompt: dequantise gate and up once, then the tiled GEMM with the SiLU * mul epilogue
        gd, ud = muillm_int8_gateupsilu_dequantize_forward(gate_up_weights, gate_up_scales_min_vals, group_size_shift)
        return mui_gateup_silu(norm_weights, epsilon, gd, ud, x)
    smv = gate_up_scales_min_vals.reshape(n, 2, g, 2)
    x = x.contiguous()
    x, norm_weights = _norm_first(x, norm_weights, epsilon, INT8_GROUP_CHUNK_MAX_TOKENS)
    tokens = _num_tokens(x)
    h = torch.empty(list(x.shape[:-1]) + [n], dtype=x.dtype, device=x.device)
    gw, uw = gate_up_weights[:, 0, :], gate_up_weights[:, 1, :]
    esz = x.element_size()
    for off, cnt in _token_chunks(tokens, group_format=True):
        check(
            _lib.load().mui_int8_group_gateup_silu(_stream(x), _dtype_code(x), gw.data_ptr(), uw.data_ptr(),
                                                   2 * k, smv[:, 0].data_ptr(), smv[:, 1].data_ptr(), 4 * g,
                                                   int(group_size_shift), x.data_ptr() + off * k * esz,
                                                   _ptr(norm_weights), float(epsilon),
                                                   h.data_ptr() + off * n * esz, n, k, cnt),
            "mui_int8_group_gateup_silu",
        )
    return h


def muillm_int8_gateupsilu_dequantize_forward(gate_up_weights, gate_up_scales_min_vals, group_size_shift):
    """csrc/module.cpp:247: packed uint8 gate/up ([N, K, 2] as in the reference, or [N, 2, K]) ->
    (gate, up) dense 16-bit matrices."""
    gate_up_weights, gate_up_scales_min_vals = _row_interleaved_gateup(gate_up_weights, gate_up_scales_min_vals,
                                                                       group_size_shift)
    n, _, k = gate_up_weights.shape
    g = k >> group_size_shift
    smv = gate_up_scales_min_vals.reshape(n, 2, g, 2)
    outs = []
    for s in range(2):
        w = gate_up_weights[:, s, :]
        out = torch.empty((n, k), dtype=smv.dtype, device=w.device)
        check(
            _lib.load().mui_int8_group_dequantize(_stream(w), _dtype_code(smv), w.data_ptr(), 2 * k,
                                                  smv[:, s].data_ptr(), 4 * g, int(group_size_shift),
                                                  out.data_ptr(), k, n, k),
            "mui_int8_group_dequantize",
        )
        outs.append(out)
    return outs[0], outs[1]


# --------------------------------------------------------------------------------------
# RoPE + static KV cache  (csrc/module.cpp:266-272,357-362,379-381)
# --------------------------------------------------------------------------------------
def _f32_table(t: torch.Tensor) -> torch.Tensor:
    if t.dtype != torch.float32:
        t = t.float()
    if t.dim() != 2 or t.stride(1) != 1:
        t = t.reshape(-1, t.shape[-1]).contiguous()
    return t


def _bhtd_strides(t: torch.Tensor, name: str):
    """Element strides (batch, token, head) of a [B, H, T, D] tensor with unit inner stride."""
    if t.dim() != 4 or t.stride(3) != 1:
        raise RuntimeError(f"{name} must be [B, H, T, D] with unit inner stride")
    return t.stride(0), t.stride(2), t.stride(1)


def _positions(position_ids: torch.Tensor, cos: torch.Tensor, b: int, t: int):
    """Returns (tables, position_ids[B or 1, T] int64, batch stride). cos/sin given already
    gathered as [B, T, E] are used as a table indexed by b*T + t
    (csrc/rope/rotary_position_layout.h:4-9)."""
    if cos.dim() == 3:
        rows = cos.shape[0] * cos.shape[1]
        pos = torch.arange(rows, device=cos.device, dtype=torch.int64).reshape(cos.shape[0], cos.shape[1])
        return pos, (t if cos.shape[0] > 1 else 0)
    pos = position_ids.to(torch.int64).reshape(-1, t).contiguous()
    return pos, (t if pos.shape[0] > 1 else 0)


def mui_rope_kv_write(q, k, v, cos, sin, position_ids, cache_position, k_out, v_out, max_cache_len):
    """q/k/v: [B, H, T, D] views; returns q_out [B, Hq, T, D]. k_out/v_out: caches
    [B, Hkv, MAX_T, D] (cache_position given) or dense outputs."""
    ref_t = q if q is not None else k
    b, _, t, d = ref_t.shape
    hq = q.shape[1] if q is not None else 0
    hkv = k.shape[1] if k is not None else (v.shape[1] if v is not None else 0)
    q_out = torch.empty((b, hq, t, d), dtype=q.dtype, device=q.device) if q is not None else None
    qs = _bhtd_strides(q, "q") if q is not None else (0, 0, 0)
    ks = _bhtd_strides(k, "k") if k is not None else (0, 0, 0)
    vs = _bhtd_strides(v, "v") if v is not None else (0, 0, 0)
    pos, pos_bs = (None, 0)
    cos32 = sin32 = None
    if cos is not None:
        pos, pos_bs = _positions(position_ids, cos, b, t)
        cos32, sin32 = _f32_table(cos), _f32_table(sin)
    out_ref = k_out if k_out is not None else v_out
    if out_ref is not None:
        if out_ref.dim() != 4 or out_ref.stride(3) != 1:
            raise RuntimeError("k/v outputs must be [B, H, T, D] with unit inner stride")
        ob, oh, ot = out_ref.stride(0), out_ref.stride(1), out_ref.stride(2)
        if b > out_ref.shape[0]:
            raise RuntimeError(f"batch {b} exceeds the batch capacity {out_ref.shape[0]} of the k/v outputs")
        if k_out is not None and v_out is not None and k_out.stride() != v_out.stride():
            raise RuntimeError("k and v outputs must share strides")
    else:
        ob = oh = ot = 0
    if cache_position is not None:
        cache_position = cache_position.to(torch.int64).contiguous()
    check(
        _lib.load().mui_rope_kv_write(
            _stream(ref_t), _dtype_code(ref_t),
            _ptr(q), qs[0], qs[1], qs[2], _ptr(k), ks[0], ks[1], ks[2], _ptr(v), vs[0], vs[1], vs[2],
            _ptr(cos32), _ptr(sin32), cos32.stride(0) if cos32 is not None else 0,
            cos32.shape[0] if cos32 is not None else 0,
            _ptr(pos), pos_bs, _ptr(cache_position), _ptr(q_out), _ptr(k_out), _ptr(v_out), ob, oh, ot,
            b, t, hq, hkv, d, int(max_cache_len)),
        "mui_rope_kv_write",
    )
    return q_out


def muillm_rope_forward_no_cache(position_ids, cos_cached, sin_cached, q, k) -> Tuple[torch.Tensor, torch.Tensor]:
    """csrc/module.cpp:266: rotated (q, k) as dense [B, H, T, D]."""
    b, hk, t, d = k.shape
    k_out = torch.empty((b, hk, t, d), dtype=k.dtype, device=k.device)
    q_out = mui_rope_kv_write(q, k, None, cos_cached, sin_cached, position_ids, None, k_out, None, t)
    return q_out, k_out


def muillm_static_kvcache_update(k_cache, v_cache, k, v, cache_position, seen_tokens: int):
    """csrc/module.cpp:272: scatter new k/v rows at cache_position (no rotation), return the
    caches narrowed to `seen_tokens`."""
    mui_rope_kv_write(None, k, v, None, None, None, cache_position, k_cache, v_cache, k_cache.shape[2])
    return k_cache.narrow(2, 0, seen_tokens), v_cache.narrow(2, 0, seen_tokens)


def muillm_rope_forward_static_cache(position_ids, cos_cached, sin_cached, q, k, v, k_cache, v_cache,
                                     cache_position, seen_tokens: int):
    """csrc/module.cpp:268: rotate q and k, write rotated k and v into the static cache at
    cache_position, return (q_rot, k_cache[:, :, :seen], v_cache[:, :, :seen])."""
    q_out = mui_rope_kv_write(q, k, v, cos_cached, sin_cached, position_ids, cache_position,
                              k_cache, v_cache, k_cache.shape[2])
    return q_out, k_cache.narrow(2, 0, seen_tokens), v_cache.narrow(2, 0, seen_tokens)


class MuiStaticKVCacheHandle:
    """Stand-in for the C++ MuillmStaticKVCache (csrc/modules/static_kvcache.cpp:3-49,
    csrc/modules/kvcache.h:13-48): aliases the per-layer cache tensors, mirrors seen_tokens."""

    def __init__(self, engine, key_cache: List[torch.Tensor], value_cache: List[torch.Tensor], seen_tokens: int):
        self.engine = engine
        self.key_cache = key_cache
        self.value_cache = value_cache
        self.seen_tokens = int(seen_tokens)


def muillm_static_kvcache_module_init(engine, key_cache, value_cache, seen_tokens):
    return MuiStaticKVCacheHandle(engine, key_cache, value_cache, seen_tokens)


def muillm_static_kvcache_module_deinit(module: MuiStaticKVCacheHandle) -> None:
    module.key_cache = module.value_cache = None


def muillm_static_kvcache_module_sync_back(module: MuiStaticKVCacheHandle):
    return module.key_cache, module.value_cache


def muillm_kvcache_module_get_set_seen_tokens(module: MuiStaticKVCacheHandle, seen_tokens: int) -> int:
    """Keeps the larger of the two counters (csrc/modules/kvcache.h:27-33)."""
    module.seen_tokens = max(module.seen_tokens, int(seen_tokens))
    return module.seen_tokens


class MuiRotaryModuleHandle:
    """Stand-in for MuillmRotaryEmbedding (csrc/modules/rotary_module.cpp:25-125)."""

    def __init__(self, engine, layer_idx, cos_cached, sin_cached):
        self.engine = engine
        self.layer_idx = layer_idx
        self.cos_cached = cos_cached
        self.sin_cached = sin_cached
        self.cos32 = _f32_table(cos_cached)
        self.sin32 = _f32_table(sin_cached)


def muillm_rotary_embedding_module_init(engine, layer_idx, cos_cached, sin_cached):
    return MuiRotaryModuleHandle(engine, layer_idx, cos_cached, sin_cached)


def muillm_rotary_embedding_module_deinit(module: MuiRotaryModuleHandle) -> None:
    module.cos_cached = module.sin_cached = module.cos32 = module.sin32 = None


def muillm_rotary_embedding_module_forward(module, cache, q, k, v, position_ids, cos_sin, cache_positions):
    """csrc/module.cpp:381 / rotary_module.cpp:25-94: bump seen_tokens on layer 0, rotate,
    write the cache, return (q_rot, k_view, v_view). The module's own fp32 tables indexed by
    position_ids are used (same values as cos_sin, without the 16-bit rounding)."""
    t = k.shape[2]
    if module.layer_idx == 0:
        cache.seen_tokens += t
    k_cache = cache.key_cache[module.layer_idx]
    v_cache = cache.value_cache[module.layer_idx]
    if position_ids is not None:
        cos, sin = module.cos32, module.sin32
    else:
        cos, sin = cos_sin
    q_out = mui_rope_kv_write(q, k, v, cos, sin, position_ids, cache_positions, k_cache, v_cache,
                              k_cache.shape[2])
    seen = cache.seen_tokens
    return q_out, k_cache.narrow(2, 0, seen), v_cache.narrow(2, 0, seen)


# --------------------------------------------------------------------------------------
# Decode attention  (csrc/module.cpp:276-277)
# --------------------------------------------------------------------------------------
def _cache_strides(k: torch.Tensor, v: torch.Tensor):
    if k.dim() != 4 or k.stride(3) != 1 or v.stride(3) != 1:
        raise RuntimeError("k innermost stride must be 1")
    if k.stride() != v.stride():
        raise RuntimeError("k and v strides must match")
    return k.stride(0), k.stride(1), k.stride(2)


def _scratch(lib, x: torch.Tensor, b: int, hq: int, d: int, n_splits: int) -> Optional[torch.Tensor]:
    nbytes = lib.mui_flash_decode_scratch_bytes(b, hq, d, n_splits)
    if nbytes == 0:
        return None
    return torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)


def _decode(q, k, v, m, n_splits=None) -> torch.Tensor:
    lib = _lib.load()
    _check_cuda(q, "q")
    _check_cuda(k, "k")
    _check_cuda(v, "v")
    _check_contiguous(q, "q")
    b, hq, t, d = q.shape
    if t != 1:
        raise RuntimeError("T > 1 not supported")
    hkv, s = k.shape[1], k.shape[2]
    cb, chs, cts = _cache_strides(k, v)
    mask_ptr, mask_bs = None, 0
    if m is not None:
        _check_cuda(m, "m")
        m = m.reshape(b, -1)
        if m.shape[1] < s or m.dtype != q.dtype:
            raise RuntimeError("mask must be [B, 1, 1, S] in the query dtype")
        m = m.contiguous()
        mask_ptr, mask_bs = m.data_ptr(), m.stride(0)
    if n_splits is None:
        n_splits = lib.mui_flash_decode_splits(b, hq, hkv, s)
    scratch = _scratch(lib, q, b, hq, d, n_splits)
    out = torch.empty((b, 1, hq * d), dtype=q.dtype, device=q.device)
    # max_cache_len: rows reachable through the view (the view is narrowed to s already)
    check(
        lib.mui_flash_decode(_stream(q), _dtype_code(q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                             cb, chs, cts, mask_ptr, mask_bs, s, _ptr(scratch), n_splits, out.data_ptr(),
                             b, hq, hkv, d, s),
        "mui_flash_decode",
    )
    return out


def _mask_rows(mask: torch.Tensor, b: int, dtype) -> torch.Tensor:
    """A [B, S] view with unit inner stride of a decode mask, without copying when possible."""
    _check_cuda(mask, "mask")
    if mask.dtype != dtype:
        raise RuntimeError("mask must have the query dtype")
    if mask.dim() == 4 and mask.shape[1] == 1 and mask.shape[2] == 1:
        rows = mask[:, 0, 0, :]
    elif mask.dim() == 2:
        rows = mask
    else:
        rows = mask.reshape(b, -1)
    if rows.shape[0] != b:
        raise RuntimeError("mask must have one row per batch entry")
    if rows.stride(1) != 1:
        rows = rows.contiguous()
    return rows


def muillm_causal_transformer_decoding_no_mask(q, k, v, n_splits=None) -> torch.Tensor:
    """q [B, Hq, 1, D] contiguous (rotated), k/v [B, Hkv, S, D] cache views -> [B, 1, Hq*D]."""
    return _decode(q, k, v, None, n_splits)


def muillm_causal_transformer_decoding_masked(q, k, v, m, n_splits=None) -> torch.Tensor:
    """As above with a [B, 1, 1, S] mask: 0 keeps a key, anything else drops it."""
    return _decode(q, k, v, m, n_splits)


def mui_attention_decode_fused(q, k, v, cos32, sin32, position_ids, cache_position, k_cache, v_cache,
                               seq_len: Optional[int] = None, mask=None, n_splits: Optional[int] = None,
                               seq_len_hint: Optional[int] = None, want_q_out: bool = False,
                               next_weights: Optional[torch.Tensor] = None):
    """RoPE(q, k) + cache write + flash decoding in one call.

    next_weights: the 2-D weight matrix (16-bit, or 8-bit codes) that the next single-token linear on
    this stream will read (a decoder layer's o_proj): when the launch leaves most of the chip idle
    -- one token at short context --, its spare workgroups fetch that matrix on chip meanwhile
    (mui_attn_decode_fused_warm); results do not change.

    q [B, Hq*D], k/v [B, Hkv*D]: un-rotated rows of the new token (views into the fused QKV
    output are fine: unit inner stride, any batch stride). cos32/sin32: fp32 tables.
    position_ids [B] or [B, 1] int64 (device), cache_position [1] int64 (device).
    seq_len=None reads the length from cache_position on the device (graph-replayable);
    the split count then comes from seq_len_hint (default: cache capacity)."""
    lib = _lib.load()
    b = q.shape[0]
    if b > k_cache.shape[0] or b > v_cache.shape[0]:
        raise RuntimeError(f"batch {b} exceeds the cache's batch capacity {k_cache.shape[0]}")
    q2, k2, v2 = q.reshape(b, -1), k.reshape(b, -1), v.reshape(b, -1)
    for name, tns in (("q", q2), ("k", k2), ("v", v2)):
        _check_cuda(tns, name)
        if tns.stride(1) != 1:
            raise RuntimeError(f"{name} must have unit inner stride")
    hkv, max_t, d = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    hq = q2.shape[1] // d
    cb, chs, cts = _cache_strides(k_cache, v_cache)
    pos = position_ids.reshape(-1)
    if pos.dtype != torch.int64 or cache_position.dtype != torch.int64:
        raise RuntimeError("position_ids and cache_position must be int64")
    pos_bs = 1 if pos.numel() > 1 else 0
    mask_ptr, mask_bs = None, 0
    if mask is not None:
        # [B, 1, 1, S] (or [B, S]); a view into a wider static buffer is used in place: under graph
        # replay the kernel reads up to the device-side sequence length, beyond the view's width
        mask = _mask_rows(mask, b, q.dtype)
        mask_ptr, mask_bs = mask.data_ptr(), mask.stride(0)
    if n_splits is None:
        hint = seq_len if seq_len is not None else (seq_len_hint if seq_len_hint is not None else max_t)
        n_splits = lib.mui_flash_decode_splits(b, hq, hkv, int(hint))
    scratch = _scratch(lib, q2, b, hq, d, n_splits)
    out = torch.empty((b, 1, hq * d), dtype=q.dtype, device=q.device)
    q_out = torch.empty((b, hq, 1, d), dtype=q.dtype, device=q.device) if want_q_out else None
    bs = lambda tns: tns.stride(0) if b > 1 else tns.shape[1]
    warm_ptr, warm_bytes, warm_slab = None, 0, 0
    if (next_weights is not None and b == 1 and next_weights.is_cuda and next_weights.dim() == 2
            and next_weights.stride(1) == 1 and next_weights.element_size() in (1, 2)
            and next_weights.data_ptr() % 16 == 0):
        pitch_bytes = next_weights.stride(0) * next_weights.element_size()
        warm_slab = lib.mui_linear_row_group_bytes(8 * next_weights.element_size(), next_weights.shape[1], pitch_bytes)
        if warm_slab > 0 and warm_slab % 16 == 0:
            warm_ptr, warm_bytes = next_weights.data_ptr(), next_weights.shape[0] * pitch_bytes
    check(
        lib.mui_attn_decode_fused_warm(
            _stream(q2), _dtype_code(q2), q2.data_ptr(), bs(q2), k2.data_ptr(), bs(k2), v2.data_ptr(), bs(v2),
            _ptr(cos32), _ptr(sin32), cos32.stride(0) if cos32 is not None else 0,
            cos32.shape[0] if cos32 is not None else 0,
            pos.data_ptr(), pos_bs, cache_position.data_ptr(), -1 if seq_len is None else int(seq_len),
            k_cache.data_ptr(), v_cache.data_ptr(), cb, chs, cts, mask_ptr, mask_bs, _ptr(q_out),
            _ptr(scratch), n_splits, out.data_ptr(), b, hq, hkv, d, max_t, warm_ptr, warm_bytes, warm_slab),
        "mui_attn_decode_fused_warm",
    )
    return (out, q_out) if want_q_out else out


# --------------------------------------------------------------------------------------
# greedy sampling helper
# --------------------------------------------------------------------------------------
def mui_argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """argmax over the last dim of 16-bit CUDA logits [..., V] -> int64 [...]; lowest index on ties."""
    _check_cuda(logits, "logits")
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    v = logits.shape[-1]
    l2 = logits.reshape(-1, v)
    rows = l2.shape[0]
    if out is None:
        out = torch.empty(logits.shape[:-1], dtype=torch.int64, device=logits.device)
    check(
        _lib.load().mui_argmax(_stream(l2), _dtype_code(l2), l2.data_ptr(), l2.stride(0) if rows > 1 else v,
                               out.data_ptr(), rows, v),
        "mui_argmax",
    )
    return out


def mui_greedy_advance(logits: torch.Tensor, next_ids: torch.Tensor, step: torch.Tensor, tokens_out: torch.Tensor,
                       position_ids: Optional[torch.Tensor] = None, cache_position: Optional[torch.Tensor] = None,
                       unfinished: Optional[torch.Tensor] = None, eos_token_ids: Optional[torch.Tensor] = None,
                       pad_token_id: int = 0, workspace: Optional[torch.Tensor] = None,
                       embed_table: Optional[torch.Tensor] = None, embed_out: Optional[torch.Tensor] = None) -> None:
    """Tail of a greedy decode step in one launch (everything in place, on the device):
    argmax of each logits row -> tokens_out[b, step[b]], next_ids[b]; position_ids[b], step[b]
    and cache_position[0] advance by one; unfinished[b] is cleared on an eos token or when
    tokens_out is full (finished rows emit pad_token_id, as the reference's
    muillm_add_tokens_check_finished does).

    logits [B, V] 16-bit; next_ids [B] or [B, 1]; step [B]; tokens_out [B, max_steps];
    position_ids [B] or [B, 1]; cache_position [1]; unfinished [B]; all integers int64.

    workspace (see greedy_workspace): lets the scan of a long row run on several workgroups; the
    same tokens either way. embed_table [V, H] / embed_out [B, H] or [B, 1, H] (16-bit, the logits'
    dtype): the chosen token's embedding row is copied to embed_out[b] in the same launch, for a
    next step that starts from inputs_embeds."""
    _check_cuda(logits, "logits")
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    v = logits.shape[-1]
    l2 = logits.reshape(-1, v)
    rows = l2.shape[0]
    for name, tns, n in (("next_ids", next_ids, rows), ("step", step, rows), ("position_ids", position_ids, rows),
                         ("cache_position", cache_position, 1), ("unfinished", unfinished, rows)):
        if tns is None:
            continue
        _check_cuda(tns, name)
        if tns.dtype != torch.int64 or tns.numel() != n or not tns.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous int64 tensor with {n} element(s)")
    _check_cuda(tokens_out, "tokens_out")
    if tokens_out.dtype != torch.int64 or tokens_out.dim() != 2 or tokens_out.shape[0] != rows or tokens_out.stride(1) != 1:
        raise RuntimeError("tokens_out must be int64 [B, max_steps] with unit inner stride")
    n_eos = 0
    if eos_token_ids is not None:
        _check_cuda(eos_token_ids, "eos_token_ids")
        if eos_token_ids.dtype != torch.int64 or not eos_token_ids.is_contiguous():
            raise RuntimeError("eos_token_ids must be a contiguous int64 tensor")
        n_eos = eos_token_ids.numel()
    ws_bytes = 0
    if workspace is not None:
        _check_cuda(workspace, "workspace")
        if workspace.dtype != torch.uint8 or not workspace.is_contiguous():
            raise RuntimeError("workspace must be a contiguous uint8 tensor (greedy_workspace makes one)")
        ws_bytes = workspace.numel()
    e_stride = e_dim = 0
    if (embed_table is None) != (embed_out is None):
        raise RuntimeError("embed_table and embed_out go together")
    if embed_table is not None:
        _check_cuda(embed_table, "embed_table")
        _check_cuda(embed_out, "embed_out")
        e_dim = embed_table.shape[-1]
        if (embed_table.dim() != 2 or embed_table.dtype != l2.dtype or embed_table.stride(1) != 1 or embed_table.shape[0] < v
                or embed_out.dtype != l2.dtype or not embed_out.is_contiguous() or embed_out.numel() != rows * e_dim):
            raise RuntimeError("embed_table must be [>= V, H] and embed_out a contiguous [B, H], both in the logits' dtype")
        e_stride = embed_table.stride(0)
    check(
        _lib.load().mui_greedy_advance_ws(
            _stream(l2), _dtype_code(l2), l2.data_ptr(), l2.stride(0) if rows > 1 else v, rows, v,
            next_ids.data_ptr(), _ptr(position_ids), _ptr(cache_position), step.data_ptr(), tokens_out.data_ptr(),
            tokens_out.stride(0), tokens_out.shape[1], _ptr(unfinished), _ptr(eos_token_ids), n_eos, int(pad_token_id),
            _ptr(workspace), ws_bytes, _ptr(embed_table), e_stride, _ptr(embed_out), e_dim),
        "mui_greedy_advance_ws",
    )


def greedy_workspace(rows: int, device) -> torch.Tensor:
    """Zero-filled workspace for mui_greedy_advance on `rows` logits rows: one per decode loop (calls
    that share it must not overlap); every call leaves it zero-filled again."""
    return torch.zeros(_lib.load().mui_greedy_workspace_bytes(int(rows)), dtype=torch.uint8, device=device)


def mui_sample_advance(logits: torch.Tensor, next_ids: torch.Tensor, step: torch.Tensor, tokens_out: torch.Tensor,
                       temperature: float = 1.0, seed: int = 0, position_ids: Optional[torch.Tensor] = None,
                       cache_position: Optional[torch.Tensor] = None, unfinished: Optional[torch.Tensor] = None,
                       eos_token_ids: Optional[torch.Tensor] = None, pad_token_id: int = 0) -> None:
    """Sampling twin of mui_greedy_advance: draws each row's token from softmax(logits / temperature)
    without a host sync or a probability tensor (argmax of logit / T - log q, q ~ Exp(1) from a
    counter-based generator keyed by `seed` and the device-side step counter), then does the same
    in-place bookkeeping. Logits filtered to -inf (top-k / top-p) are never drawn."""
    _check_cuda(logits, "logits")
    if logits.stride(-1) != 1:
        logits = logits.contiguous()
    v = logits.shape[-1]
    l2 = logits.reshape(-1, v)
    rows = l2.shape[0]
    if not temperature > 0:
        raise ValueError("temperature must be positive (use mui_greedy_advance for greedy decoding)")
    for name, tns, n in (("next_ids", next_ids, rows), ("step", step, rows), ("position_ids", position_ids, rows),
                         ("cache_position", cache_position, 1), ("unfinished", unfinished, rows)):
        if tns is None:
            continue
        _check_cuda(tns, name)
        if tns.dtype != torch.int64 or tns.numel() != n or not tns.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous int64 tensor with {n} element(s)")
    _check_cuda(tokens_out, "tokens_out")
    if tokens_out.dtype != torch.int64 or tokens_out.dim() != 2 or tokens_out.shape[0] != rows or tokens_out.stride(1) != 1:
        raise RuntimeError("tokens_out must be int64 [B, max_steps] with unit inner stride")
    n_eos = 0
    if eos_token_ids is not None:
        _check_cuda(eos_token_ids, "eos_token_ids")
        if eos_token_ids.dtype != torch.int64 or not eos_token_ids.is_contiguous():
            raise RuntimeError("eos_token_ids must be a contiguous int64 tensor")
        n_eos = eos_token_ids.numel()
    check(
        _lib.load().mui_sample_advance(
            _stream(l2), _dtype_code(l2), l2.data_ptr(), l2.stride(0) if rows > 1 else v, rows, v,
            float(temperature), int(seed) & 0xFFFFFFFFFFFFFFFF, next_ids.data_ptr(), _ptr(position_ids),
            _ptr(cache_position), step.data_ptr(), tokens_out.data_ptr(), tokens_out.stride(0), tokens_out.shape[1],
            _ptr(unfinished), _ptr(eos_token_ids), n_eos, int(pad_token_id)),
        "mui_sample_advance",
    )


# --------------------------------------------------------------------------------------
# embedding (csrc/module.cpp:314-320 of the reference)
# --------------------------------------------------------------------------------------
class MuiEmbeddingModule:
    """Handle returned by muillm_embedding_module_init: aliases the weight table."""

    def __init__(self, engine, weights: torch.Tensor):
        self.engine = engine
        self.weights = weights


def muillm_embedding_module_init(engine, weights: torch.Tensor) -> MuiEmbeddingModule:
    if weights.dim() != 2:
        raise RuntimeError("embedding weights must be 2-D [num_embeddings, embedding_dim]")
    return MuiEmbeddingModule(engine, weights)


def muillm_embedding_module_deinit(module: MuiEmbeddingModule) -> None:
    module.weights = None


def muillm_embedding_forward(engine, weights: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """out[..., :] = weights[x[...], :] for a 16-bit CUDA table and int32/int64 CUDA ids."""
    _check_cuda(weights, "weights")
    _check_cuda(x, "x")
    if weights.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("unsupported embedding type: only float16 and bfloat16 are supported")
    if x.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("unsupported index type: only int32 and int64 are supported")
    if weights.stride(1) != 1:
        raise RuntimeError("weights must have unit inner stride")
    xc = x.contiguous()
    dim = weights.shape[1]
    out = torch.empty(tuple(x.shape) + (dim,), dtype=weights.dtype, device=weights.device)
    if xc.numel() == 0:
        return out
    check(
        _lib.load().mui_embedding(_stream(weights), _dtype_code(weights), weights.data_ptr(), weights.stride(0),
                                  xc.data_ptr(), 1 if x.dtype == torch.int32 else 0, out.data_ptr(), xc.numel(), dim,
                                  weights.shape[0]),
        "mui_embedding",
    )
    return out


def muillm_embedding_module_forward(module: MuiEmbeddingModule, x: torch.Tensor) -> torch.Tensor:
    return muillm_embedding_forward(module.engine, module.weights, x)


def key_padding_mask16(attention_mask: torch.Tensor, dtype: torch.dtype, seq_len: Optional[int] = None) -> torch.Tensor:
    """The [B, S] 0 / 1 attention mask of a padded batch as mui_prefill_attention's key mask: 16-bit,
    1 where the key is padding, rows padded with zeros to a multiple of 8 entries (the kernel reads
    four entries at a time)."""
    b, s_mask = attention_mask.shape
    s = s_mask if seq_len is None else max(int(seq_len), s_mask)
    out = torch.zeros((b, (s + 7) // 8 * 8), dtype=dtype, device=attention_mask.device)
    out[:, :s_mask] = (attention_mask == 0).to(dtype)
    return out


def mui_prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_start: Optional[int] = None,
                          key_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of T > 1 new tokens over cache views that already contain them.

    q [B, Hq, T, D] rotated (made dense if it is not), k/v [B, Hkv, S, D] views of the static cache
    (unit inner stride, equal strides); query t sits at key position q_start + t (default S - T).
    key_mask (padded batches, see key_padding_mask16): [B, >= S rounded up to 4] in q's dtype, non-zero
    hides the key from every query. Returns [B, T, Hq * D]."""
    _check_cuda(q, "q")
    _check_cuda(k, "k")
    _check_cuda(v, "v")
    b, hq, t, d = q.shape
    hkv, s = k.shape[1], k.shape[2]
    if q_start is None:
        q_start = s - t
    if q_start < 0 or q_start + t > s:
        raise RuntimeError("the new tokens must lie inside the key sequence")
    qc = q.contiguous()
    cb, chs, cts = _cache_strides(k, v)
    out = torch.empty((b, t, hq * d), dtype=q.dtype, device=q.device)
    if key_mask is not None:
        _check_cuda(key_mask, "key_mask")
        if key_mask.dtype != q.dtype or key_mask.dim() != 2 or key_mask.shape[0] != b or key_mask.stride(1) != 1 \
                or key_mask.shape[1] < (s + 3) // 4 * 4 or key_mask.device != q.device:
            raise RuntimeError("key_mask must be [batch, >= keys rounded up to 4] in the activations' dtype, on their device")
        check(
            _lib.load().mui_prefill_attention_masked(_stream(qc), _dtype_code(qc), qc.data_ptr(), k.data_ptr(), v.data_ptr(),
                                                     cb, chs, cts, s, int(q_start), key_mask.data_ptr(), key_mask.stride(0),
                                                     out.data_ptr(), b, hq, hkv, t, d),
            "mui_prefill_attention_masked",
        )
        return out
    check(
        _lib.load().mui_prefill_attention(_stream(qc), _dtype_code(qc), qc.data_ptr(), k.data_ptr(), v.data_ptr(),
                                          cb, chs, cts, s, int(q_start), out.data_ptr(), b, hq, hkv, t, d),
        "mui_prefill_attention",
    )
    return out
