"""mui_flash_decode_static, the entry point that allocates nothing: its split partials live in
an array built into the library.  Called through the C ABI (ctypes) and checked, bit for bit,
against mui_flash_decode with caller-allocated scratch (same kernels, deterministic), and
against the oracle to the attention gate (2e-3 absolute); two calls in a row on the one GPU,
the second with a smaller input, so that what the first call left in the array must not leak
into the second."""

import pytest
import torch

import oracle
from muillm_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = 128
ATOL = 2e-3


def _case(seed, b, hq, hkv, s, cap, n_splits, dtype=torch.float16):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    q = torch.randn((b, hq, 1, D), generator=g).to(dtype)
    k = torch.randn((b, hkv, cap, D), generator=g).to(dtype)
    v = torch.randn((b, hkv, cap, D), generator=g).to(dtype)
    return q, k, v, s, n_splits


def _run(lib, q, k, v, s, n_splits, static):
    b, hq = q.shape[0], q.shape[1]
    hkv, cap = k.shape[1], k.shape[2]
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    out = torch.zeros((b, 1, hq * D), dtype=q.dtype, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    code = _lib.MUI_DTYPE_F16 if q.dtype == torch.float16 else _lib.MUI_DTYPE_BF16
    if static:
        st = lib.mui_flash_decode_static(stream, code, qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), kd.stride(0),
                                         kd.stride(1), kd.stride(2), None, 0, s, n_splits, out.data_ptr(), b, hq,
                                         hkv, D, cap)
    else:
        nbytes = lib.mui_flash_decode_scratch_bytes(b, hq, D, n_splits)
        scratch = torch.empty(max(nbytes, 4) // 4, dtype=torch.float32, device=DEV)
        st = lib.mui_flash_decode(stream, code, qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), kd.stride(0),
                                  kd.stride(1), kd.stride(2), None, 0, s, scratch.data_ptr(), n_splits,
                                  out.data_ptr(), b, hq, hkv, D, cap)
    torch.cuda.synchronize()
    return st, out


def test_static_scratch_matches_caller_scratch_on_two_calls_in_a_row():
    lib = _lib.load()
    # first call: 8 rows x 32 heads x 16 splits fills 2 MiB of the array; second: a smaller shape
    # whose partial slots overlap the first call's
    big = _case(0, 8, 32, 8, 3000, 4096, 16)
    small = _case(1, 1, 32, 8, 700, 1024, 5)
    for q, k, v, s, n_splits in (big, small):
        st, got = _run(lib, q, k, v, s, n_splits, static=True)
        assert st == 0, _lib.status_string(st)
        st, want = _run(lib, q, k, v, s, n_splits, static=False)
        assert st == 0, _lib.status_string(st)
        assert torch.equal(got, want), "static-scratch call differs from the caller-scratch call"
        ref = oracle.decode_attention(q, k[:, :, :s], v[:, :, :s])
        err = float((got.cpu().double().reshape(-1) - ref.double().reshape(-1)).abs().max())
        assert err <= ATOL, err


def test_static_scratch_unsplit_and_bf16():
    lib = _lib.load()
    for dtype, n_splits in ((torch.float16, 1), (torch.bfloat16, 7)):
        q, k, v, s, n_splits = _case(2, 2, 8, 2, 333, 512, n_splits, dtype)
        st, got = _run(lib, q, k, v, s, n_splits, static=True)
        assert st == 0, _lib.status_string(st)
        st, want = _run(lib, q, k, v, s, n_splits, static=False)
        assert st == 0 and torch.equal(got, want)


def test_static_scratch_limit_is_refused_without_launching():
    lib = _lib.load()
    limit = lib.mui_flash_decode_static_scratch_limit()
    assert limit == 4 << 20
    # 16 rows x 32 heads x 32 splits x 130 floats = 8.1 MiB > limit
    q, k, v, s, n_splits = _case(3, 16, 32, 8, 64, 64, 32)
    assert lib.mui_flash_decode_scratch_bytes(16, 32, D, 32) > limit
    st, out = _run(lib, q, k, v, s, n_splits, static=True)
    assert st == -6 and "scratch" in _lib.status_string(st)
    assert not out.any(), "a refused call must not write the output"
