"""ctypes binding of libmuillm_amd.so (the C ABI declared in include/muillm_amd.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""

from __future__ import annotations

import ctypes
import os
import re
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
from typing import Dict, List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmuillm_amd.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "muillm_amd.h")
# measurement aids (process-global launch-shape overrides, bandwidth probe): not product ABI
TUNE_HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "muillm_amd_tune.h")

MUI_OK = 0
MUI_DTYPE_F16 = 0
MUI_DTYPE_BF16 = 1
MUI_MAX_TOKENS = 16


class MuiDeviceInfo(ctypes.Structure):
    _fields_ = [
        ("device", c_int),
        ("compute_units", c_int),
        ("wave_size", c_int),
        ("simd_lanes", c_int),
        ("lds_bytes_per_block", c_int),
        ("l2_bytes", c_int),
        ("clock_khz", c_int),
        ("is_gfx950", c_int),
        ("hbm_bytes", ctypes.c_uint64),
        ("arch", ctypes.c_char * 64),
    ]


class MuiLibraryError(RuntimeError):
    pass


_P = c_void_p
# name -> (restype, argtypes).  Must list every function include/muillm_amd.h declares.
_SIGNATURES = {
    "mui_abi_version": (c_int, []),
    "mui_status_string": (c_char_p, [c_int]),
    "mui_device_info": (c_int, [c_int, ctypes.POINTER(MuiDeviceInfo)]),
    "mui_linear": (c_int, [_P, c_int, _P, c_long, _P, _P, c_float, _P, _P, _P, _P, c_int, c_int, c_int]),
    "mui_linear_ws": (c_int, [_P, c_int, _P, c_long, _P, _P, c_float, _P, _P, _P, _P, c_int, c_int, c_int, _P,
                              ctypes.c_size_t]),
    "mui_linear_workspace_bytes": (ctypes.c_size_t, []),
    "mui_rmsnorm": (c_int, [_P, c_int, _P, _P, c_float, _P, c_int, c_int]),
    "mui_gateup_silu": (c_int, [_P, c_int, _P, _P, c_long, _P, _P, c_float, _P, c_int, c_int, c_int]),
    "mui_silu_mul_interleaved": (c_int, [_P, c_int, _P, _P, c_long, c_int]),
    "mui_int8_linear": (c_int, [_P, c_int, _P, c_long, _P, _P, _P, c_float, _P, _P, _P, c_int, c_int, c_int]),
    "mui_int8_gateup_silu": (c_int, [_P, c_int, _P, _P, c_long, _P, _P, c_long, _P, _P, c_float, _P, c_int, c_int, c_int]),
    "mui_int8_group_linear": (c_int, [_P, c_int, _P, c_long, _P, c_int, _P, _P, c_float, _P, _P, _P, c_int, c_int, c_int]),
    "mui_int8_group_gateup_silu": (c_int, [_P, c_int, _P, _P, c_long, _P, _P, c_long, c_int, _P, _P, c_float, _P, c_int, c_int, c_int]),
    "mui_int8_repack_gateup": (c_int, [_P, _P, _P, c_int, _P, _P, c_int, c_int]),
    "mui_int8_dequantize": (c_int, [_P, c_int, _P, c_long, _P, c_long, _P, c_long, c_int, c_int]),
    "mui_int8_group_dequantize": (c_int, [_P, c_int, _P, c_long, _P, c_long, c_int, _P, c_long, c_int, c_int]),
    "mui_rope_kv_write": (c_int, [_P, c_int, _P, c_long, c_long, c_long, _P, c_long, c_long, c_long,
                                  _P, c_long, c_long, c_long, _P, _P, c_int, c_int, _P, c_long, _P, _P, _P, _P,
                                  c_long, c_long, c_long, c_int, c_int, c_int, c_int, c_int, c_int]),
    "mui_flash_decode_splits": (c_int, [c_int, c_int, c_int, c_int]),
    "mui_tune_attention": (c_int, [c_int, c_int, c_int, c_int]),
    "mui_flash_decode_scratch_bytes": (ctypes.c_size_t, [c_int, c_int, c_int, c_int]),
    "mui_flash_decode": (c_int, [_P, c_int, _P, _P, _P, c_long, c_long, c_long, _P, c_long, c_int, _P,
                                 c_int, _P, c_int, c_int, c_int, c_int, c_int]),
    "mui_flash_decode_static_scratch_limit": (ctypes.c_size_t, []),
    "mui_flash_decode_static": (c_int, [_P, c_int, _P, _P, _P, c_long, c_long, c_long, _P, c_long, c_int,
                                        c_int, _P, c_int, c_int, c_int, c_int, c_int]),
    "mui_attn_decode_fused": (c_int, [_P, c_int, _P, c_long, _P, c_long, _P, c_long, _P, _P, c_int, c_int, _P,
                                      c_long, _P, c_int, _P, _P, c_long, c_long, c_long, _P, c_long, _P,
                                      _P, c_int, _P, c_int, c_int, c_int, c_int, c_int]),
    "mui_attn_decode_fused_warm": (c_int, [_P, c_int, _P, c_long, _P, c_long, _P, c_long, _P, _P, c_int, c_int, _P,
                                           c_long, _P, c_int, _P, _P, c_long, c_long, c_long, _P, c_long, _P,
                                           _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, _P, ctypes.c_size_t, c_int]),
    "mui_linear_row_group_bytes": (c_int, [c_int, c_int, c_long]),
    "mui_prefill_attention": (c_int, [_P, c_int, _P, _P, _P, c_long, c_long, c_long, c_int, c_int, _P, c_int, c_int,
                                      c_int, c_int, c_int]),
    "mui_prefill_attention_masked": (c_int, [_P, c_int, _P, _P, _P, c_long, c_long, c_long, c_int, c_int, _P, c_long, _P,
                                             c_int, c_int, c_int, c_int, c_int]),
    "mui_argmax": (c_int, [_P, c_int, _P, c_long, _P, c_int, c_int]),
    "mui_greedy_advance": (c_int, [_P, c_int, _P, c_long, c_int, c_int, _P, _P, _P, _P, _P, c_long, c_int, _P, _P,
                                   c_int, c_long]),
    "mui_greedy_workspace_bytes": (ctypes.c_size_t, [c_int]),
    "mui_greedy_advance_ws": (c_int, [_P, c_int, _P, c_long, c_int, c_int, _P, _P, _P, _P, _P, c_long, c_int, _P, _P,
                                      c_int, c_long, _P, ctypes.c_size_t, _P, c_long, _P, c_int]),
    "mui_sample_advance": (c_int, [_P, c_int, _P, c_long, c_int, c_int, c_float, ctypes.c_uint64, _P, _P, _P, _P, _P,
                                   c_long, c_int, _P, _P, c_int, c_long]),
    "mui_embedding": (c_int, [_P, c_int, _P, c_long, _P, c_int, _P, c_int, c_int, c_int]),
    "mui_decoder_stack_workspace_bytes": (ctypes.c_size_t, [_P, c_int, c_int]),
    "mui_decoder_stack_step": (c_int, [_P, _P, c_int, _P, _P, _P, c_long, _P, c_int, _P, c_long, c_int, _P]),
    "mui_probe_read": (c_int, [_P, _P, ctypes.c_uint64, _P]),
    "mui_tune_lock": (c_int, []),
    "mui_tune_gemv": (c_int, [c_int, c_int]),
    "mui_tune_packed_dot": (c_int, [c_int, c_int]),
    "mui_tune_int8": (c_int, [c_int, c_int]),
    "mui_tune_int8_quad": (c_int, [c_int, c_int, c_int, c_int]),
    "mui_tune_skinny": (c_int, [c_int, c_int, c_int]),
    "mui_tune_prefill": (c_int, [c_int, c_int]),
    "mui_tune_prefill_attention": (c_int, [c_int]),
    "mui_tune_warm": (c_int, [c_int, c_int, c_int]),
    "mui_probe_chain_flag_bytes": (ctypes.c_size_t, [c_int]),
    "mui_probe_gemv_chain": (c_int, [_P, c_int, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, c_int, c_int]),
    "mui_probe_gemv_chain2": (c_int, [_P, _P, c_int, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, c_int, c_int]),
}



class MuiDecoderLayerDesc(ctypes.Structure):
    """struct mui_decoder_layer of the public header."""
    _fields_ = [("input_norm", _P), ("qkv_weight", _P), ("qkv_pitch", c_long), ("o_weight", _P),
                ("o_pitch", c_long), ("post_norm", _P), ("gate_weight", _P), ("up_weight", _P),
                ("gateup_pitch", c_long), ("down_weight", _P), ("down_pitch", c_long), ("k_cache", _P),
                ("v_cache", _P), ("qkv_scales", _P), ("o_scales", _P), ("gate_scales", _P), ("up_scales", _P),
                ("gateup_scale_stride", c_long), ("down_scales", _P), ("int8_group_size_shift", c_int)]


class MuiDecoderStackDesc(ctypes.Structure):
    """struct mui_decoder_stack of the public header."""
    _fields_ = [("dtype", c_int), ("n_layers", c_int), ("hidden", c_int), ("n_q_heads", c_int),
                ("n_kv_heads", c_int), ("head_dim", c_int), ("intermediate", c_int), ("norm_eps", c_float),
                ("layers", ctypes.POINTER(MuiDecoderLayerDesc)), ("cos_table", _P), ("sin_table", _P),
                ("rope_row_stride", c_long), ("rope_rows", c_long), ("cache_batch_stride", c_long), ("cache_head_stride", c_long),
                ("cache_token_stride", c_long), ("max_cache_len", c_int)]


MUI_ABI_VERSION = 3  # MUI_ABI_VERSION of the public header: layout of the structs above

_lib: Optional[ctypes.CDLL] = None


def header_text(*paths: str) -> str:
    """Concatenated text of the given headers (default: both) with comments removed."""
    out = []
    for path in paths or (HEADER_PATH, TUNE_HEADER_PATH):
        with open(path, "r") as f:
            out.append(re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S))
    return "\n".join(out)


def declared_functions(*paths: str) -> List[str]:
    """Names of the functions the given headers (default: product + tuning header) declare."""
    return sorted(set(re.findall(r"\b(mui_[a-z0-9_]+)\s*\(", header_text(*paths))))


def load() -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MuiLibraryError(
            f"{LIB_PATH} is missing: build it with `make -C muillm_amd/csrc` "
            "(or __graft_entry__.build()). There is no CPU fallback."
        )
    # torch ships its own HIP runtime with the same SONAME; importing it first makes the
    # kernels and torch's allocator/streams share one runtime instance.
    import torch  # noqa: F401

    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.mui_abi_version() != MUI_ABI_VERSION:
        raise MuiLibraryError(
            f"{LIB_PATH} has ABI version {lib.mui_abi_version()}, this package expects {MUI_ABI_VERSION} "
            "(the descriptor structs differ): rebuild it with `make -C muillm_amd/csrc`.")
    _lib = lib
    return lib


def status_string(status: int) -> str:
    return load().mui_status_string(status).decode()


def check(status: int, what: str) -> None:
    if status != MUI_OK:
        raise MuiLibraryError(f"{what} failed: {status_string(status)} (status {status})")


def device_info(device: int = 0) -> Dict[str, object]:
    info = MuiDeviceInfo()
    check(load().mui_device_info(device, ctypes.byref(info)), "mui_device_info")
    out = {name: getattr(info, name) for name, _ in MuiDeviceInfo._fields_}
    out["arch"] = info.arch.decode()
    return out
