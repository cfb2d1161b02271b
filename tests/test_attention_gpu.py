"""GPU parity of RoPE + static-cache write + flash decoding (config 4) through the C ABI.

Gates: attention outputs within 2e-3 absolute of the high-precision oracle; the cache slot
written by the fused kernel is bit-identical to the standalone rotation; every other cache
slot is untouched.  The reference has no test for these kernels; the recipes here are the
closed forms of softmax attention plus the prefill-then-decode sequence of the reference's
static-cache test (tests/test_static_kvcache.py:52-112 there)."""

import functools
import math
import os

import pytest
import torch

import oracle
from muillm_amd import _lib, muillm_ext
from tests.util import record_error

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = 128
ATOL = 2e-3


@pytest.fixture(params=["auto", "matrix-core", "vector"], autouse=True)
def attention_kernel_choice(request):
    """Every test runs three times: with the built-in kernel choice (matrix-core decode kernel
    except in the unsplit one-workgroup-per-query-head mode of short sequences), with the
    matrix-core kernel forced everywhere, and with the vector-ALU kernel only."""
    lib = _lib.load()
    if request.param == "matrix-core":
        _lib.check(lib.mui_tune_attention(0, 0, 0, 1), "mui_tune_attention")
    elif request.param == "vector":
        _lib.check(lib.mui_tune_attention(0, 0, 0, -1), "mui_tune_attention")
    yield request.param
    _lib.check(lib.mui_tune_attention(0, 0, 0, 0), "mui_tune_attention")


def _gen(seed=0):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _mk(shape, g, std=1.0, dtype=torch.float16):
    return (std * torch.randn(shape, generator=g)).to(dtype)


BF16_PROMPT_ATOL = 4e-3


def _attn_err(got, ref):
    """What the attention gate (<= 2e-3 absolute) is held against. fp16 outputs: max |got - ref|.
    bf16 outputs: the same after taking off half a unit in the last place of a bf16 number of the
    reference's size (at most 2^-8 |ref|) -- the rounding of the stored result, which alone exceeds
    2e-3 once |ref| reaches 0.5 and has nothing to do with how the attention was computed."""
    if got.dtype != torch.bfloat16:
        return _max_abs(got, ref)
    g, r = got.detach().cpu().double().reshape(-1), ref.double().reshape(-1)
    err = float(((g - r).abs() - r.abs() * 2.0 ** -8).clamp_min(0).max())
    test = os.environ.get("PYTEST_CURRENT_TEST", "").split("::")[-1].split(" ")[0]
    record_error("%s [bfloat16]" % test, err, ATOL, "max_abs_beyond_half_ulp_of_output")
    return err


def _max_abs(got, ref):
    err = float((got.detach().cpu().double().reshape(-1) - ref.double().reshape(-1)).abs().max())
    test = os.environ.get("PYTEST_CURRENT_TEST", "").split("::")[-1].split(" ")[0]
    record_error("%s [%s]" % (test, str(got.dtype).replace("torch.", "")), err, ATOL, "max_abs")
    return err


# ------------------------------------------------------------------------------------
# standalone RoPE / cache write
# ------------------------------------------------------------------------------------
@pytest.mark.parametrize("b,t,hq,hkv", [(1, 1, 32, 8), (2, 5, 8, 2), (1, 64, 32, 8), (8, 1, 32, 8)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rope_no_cache(b, t, hq, hkv, dtype):
    g = _gen(0)
    cos, sin = oracle.rope_tables(500000.0, D, 4096)
    qkv = _mk((b, t, (hq + 2 * hkv) * D), g, dtype=dtype).to(DEV)  # fused-QKV-like buffer
    q = qkv[..., : hq * D].view(b, t, hq, D).transpose(1, 2)       # strided views
    k = qkv[..., hq * D : (hq + hkv) * D].view(b, t, hkv, D).transpose(1, 2)
    pos = torch.randint(0, 4096, (b, t), generator=g)
    rq, rk = oracle.apply_rope(q.cpu(), k.cpu(), cos, sin, pos)
    q_out, k_out = muillm_ext.muillm_rope_forward_no_cache(pos.to(DEV), cos.to(DEV), sin.to(DEV), q, k)
    assert q_out.shape == (b, hq, t, D) and q_out.is_contiguous() and k_out.shape == (b, hkv, t, D)
    tol = 2.5e-3 if dtype == torch.float16 else 2e-2  # half an ulp at |x| <= 4
    assert _max_abs(q_out, rq) <= tol * max(1.0, float(rq.abs().max()) / 4)
    assert _max_abs(k_out, rk) <= tol * max(1.0, float(rk.abs().max()) / 4)
    # exact rounding: equals the fp64 result rounded once, up to 1 ulp flips
    ulp_off = (q_out.cpu().view(torch.int16).int() - rq.to(dtype).view(torch.int16).int()).abs().max()
    assert int(ulp_off) <= 1


def test_rope_invariants():
    g = _gen(1)
    cos, sin = oracle.rope_tables(500000.0, D, 1024)
    q = _mk((1, 4, 1, D), g).to(DEV)
    k = _mk((1, 4, 1, D), g).to(DEV)
    z = torch.zeros(1, 1, dtype=torch.int64, device=DEV)
    q0, k0 = muillm_ext.muillm_rope_forward_no_cache(z, cos.to(DEV), sin.to(DEV), q, k)
    assert torch.equal(q0, q) and torch.equal(k0, k)  # position 0 is the identity
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    def dots(m, n):
        pm = torch.full((1, 1), m, dtype=torch.int64, device=DEV)
        pn = torch.full((1, 1), n, dtype=torch.int64, device=DEV)
        qm, _ = muillm_ext.muillm_rope_forward_no_cache(pm, cos.to(DEV), sin.to(DEV), q, k)
        _, kn = muillm_ext.muillm_rope_forward_no_cache(pn, cos.to(DEV), sin.to(DEV), q, k)
        return (qm.float() * kn.float()).sum(-1)
    assert torch.allclose(dots(10, 3), dots(507, 500), atol=0.15)
    # norms of the (i, i + D/2) pairs are preserved
    p = torch.full((1, 1), 777, dtype=torch.int64, device=DEV)
    qr, _ = muillm_ext.muillm_rope_forward_no_cache(p, cos.to(DEV), sin.to(DEV), q, k)
    n0 = q.float()[..., :64] ** 2 + q.float()[..., 64:] ** 2
    n1 = qr.float()[..., :64] ** 2 + qr.float()[..., 64:] ** 2
    assert torch.allclose(n0, n1, rtol=5e-3, atol=5e-3)


def test_static_cache_prefill_then_decode():
    """Prefill 64 tokens, then 16 single-token updates: the narrowed views equal the
    concatenation of everything written (reference tests/test_static_kvcache.py:52-112),
    slots never written stay zero."""
    g = _gen(2)
    b, hkv, cap = 2, 8, 128
    k_cache = torch.zeros(b, hkv, cap, D, dtype=torch.float16, device=DEV)
    v_cache = torch.zeros_like(k_cache)
    ks, vs, seen = [], [], 0
    for step, t in enumerate([64] + [1] * 16):
        k = _mk((b, hkv, t, D), g).to(DEV)
        v = _mk((b, hkv, t, D), g).to(DEV)
        cp = torch.arange(seen, seen + t, device=DEV)
        seen += t
        kv, vv = muillm_ext.muillm_static_kvcache_update(k_cache, v_cache, k, v, cp, seen)
        ks.append(k)
        vs.append(v)
        assert kv.shape == (b, hkv, seen, D)
        assert torch.equal(kv, torch.cat(ks, dim=2)) and torch.equal(vv, torch.cat(vs, dim=2))
    assert not k_cache[:, :, seen:].any() and not v_cache[:, :, seen:].any()
    # out-of-range slots are ignored rather than written
    bad = torch.tensor([cap + 5], device=DEV)
    before = k_cache.clone()
    muillm_ext.muillm_static_kvcache_update(k_cache, v_cache, ks[-1], vs[-1], bad, seen)
    assert torch.equal(before, k_cache)


# ------------------------------------------------------------------------------------
# flash decoding over an existing cache
# ------------------------------------------------------------------------------------
@pytest.mark.parametrize("b,hq,hkv,s,cap", [
    (1, 32, 8, 1, 16), (1, 32, 8, 5, 8), (1, 32, 8, 63, 64), (2, 32, 8, 64, 128), (1, 32, 8, 65, 128),
    (1, 32, 8, 1024, 1024), (3, 32, 8, 1000, 1024), (8, 32, 8, 1024, 2048),
    (1, 8, 8, 300, 512), (1, 16, 8, 300, 512), (2, 64, 8, 300, 512),
    # other GQA ratios: 3, 5, 6, 7 (matrix-core kernel) and 12, 16 (one workgroup per query head)
    (1, 24, 8, 300, 512), (2, 20, 4, 700, 1024), (1, 12, 2, 300, 512), (1, 14, 2, 2000, 2048),
    (1, 12, 1, 300, 512), (1, 32, 2, 2000, 2048),
])
@pytest.mark.parametrize("splits", [None, 1, 7])
def test_flash_decode(b, hq, hkv, s, cap, splits):
    g = _gen(3)
    q = _mk((b, hq, 1, D), g)
    kc = _mk((b, hkv, cap, D), g)
    vc = _mk((b, hkv, cap, D), g)
    kc[:, :, s:] = float("nan")  # anything beyond the sequence must never be read
    vc[:, :, s:] = float("nan")
    ref = oracle.decode_attention(q, kc[:, :, :s], vc[:, :, :s])
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = muillm_ext.muillm_causal_transformer_decoding_no_mask(q.to(DEV), kd[:, :, :s], vd[:, :, :s], n_splits=splits)
    assert out.shape == (b, 1, hq * D)
    assert torch.isfinite(out).all()
    assert _max_abs(out, ref) <= ATOL


@pytest.mark.parametrize("b,s", [(1, 4096), (4, 16384), (1, 32768), (8, 4096)])
def test_flash_decode_config4_lengths(b, s):
    g = _gen(4)
    hq, hkv = 32, 8
    cap = oracle.next_pow2(s)
    q = _mk((b, hq, 1, D), g)
    kc = _mk((b, hkv, cap, D), g)
    vc = _mk((b, hkv, cap, D), g)
    ref = oracle.decode_attention(q, kc[:, :, :s], vc[:, :, :s])
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = muillm_ext.muillm_causal_transformer_decoding_no_mask(q.to(DEV), kd[:, :, :s], vd[:, :, :s])
    assert _max_abs(out, ref) <= ATOL
    # split-count invariance (size-independent property)
    out1 = muillm_ext.muillm_causal_transformer_decoding_no_mask(q.to(DEV), kd[:, :, :s], vd[:, :, :s], n_splits=3)
    assert _max_abs(out1, out.cpu()) <= 1e-3


def test_flash_decode_closed_forms():
    g = _gen(5)
    hq, hkv, s = 32, 8, 200
    q = _mk((1, hq, 1, D), g).to(DEV)
    v = _mk((1, hkv, s, D), g).to(DEV)
    # S = 1 -> out = v0 exactly
    out = muillm_ext.muillm_causal_transformer_decoding_no_mask(q, v[:, :, :1].contiguous(), v[:, :, :1].contiguous())
    assert torch.equal(out.view(hq, D), v[0, :, 0].repeat_interleave(4, dim=0))
    # identical keys -> uniform weights -> mean of V
    k_same = _mk((1, hkv, 1, D), g).to(DEV).expand(1, hkv, s, D).contiguous()
    out = muillm_ext.muillm_causal_transformer_decoding_no_mask(q, k_same, v)
    mean_v = v.float().mean(2)[0].repeat_interleave(4, dim=0)
    assert (out.view(hq, D).float() - mean_v).abs().max() <= ATOL
    # one dominant key -> its value; heads 4j..4j+3 share KV head j
    k = torch.zeros(1, hkv, s, D, dtype=torch.float16, device=DEV)
    qq = torch.zeros(1, hq, 1, D, dtype=torch.float16, device=DEV)
    qq[..., 0] = 30.0
    for j in range(hkv):
        k[0, j, 10 + j, 0] = 30.0
    out = muillm_ext.muillm_causal_transformer_decoding_no_mask(qq, k, v).view(hq, D)
    for h in range(hq):
        assert (out[h].float() - v[0, h // 4, 10 + h // 4].float()).abs().max() <= ATOL


def test_flash_decode_masked():
    g = _gen(6)
    b, hq, hkv, s = 2, 32, 8, 333
    q, k, v = _mk((b, hq, 1, D), g), _mk((b, hkv, s, D), g), _mk((b, hkv, s, D), g)
    drop = torch.rand(b, s, generator=g) < 0.3
    drop[0, :40] = True  # left padding
    drop[:, -1] = False
    minv = torch.finfo(torch.float16).min
    m = torch.zeros(b, 1, 1, s, dtype=torch.float16)
    m[drop[:, None, None, :]] = minv
    add = torch.zeros(b, 1, 1, s, dtype=torch.float64)
    add[drop[:, None, None, :]] = float("-inf")
    ref = oracle.decode_attention(q, k, v, add)
    out = muillm_ext.muillm_causal_transformer_decoding_masked(q.to(DEV), k.to(DEV), v.to(DEV), m.to(DEV))
    assert _max_abs(out, ref) <= ATOL
    out7 = muillm_ext.muillm_causal_transformer_decoding_masked(q.to(DEV), k.to(DEV), v.to(DEV), m.to(DEV), n_splits=5)
    assert _max_abs(out7, ref) <= ATOL


# ------------------------------------------------------------------------------------
# fused RoPE + cache write + decode
# ------------------------------------------------------------------------------------
@pytest.mark.parametrize("b,s,cap", [(1, 1, 16), (1, 33, 64), (2, 257, 512), (1, 1024, 1024), (4, 4096, 4096), (8, 1000, 1024)])
@pytest.mark.parametrize("device_len", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_decode(b, s, cap, device_len, dtype):
    """Config 4 recipe: cache pre-filled for s-1 positions, new token at position s-1."""
    _fused_decode_case(b, s, cap, device_len, dtype, 32, 8)


@pytest.mark.parametrize("b,s", [(1, 16384), (8, 16384), (1, 32768), (8, 32768)])
def test_fused_decode_long_context(b, s):
    """Config 4 at its long contexts, batch 1 and 8, through the entry point the decoder calls
    (RoPE + cache write + split flash decoding + merge); fp16, and bf16 at batch 1. Every batch
    row is checked against the oracle."""
    _fused_decode_case(b, s, s, True, torch.float16, 32, 8)
    if b == 1:
        _fused_decode_case(b, s, s, False, torch.bfloat16, 32, 8)


@pytest.mark.parametrize("rows,cols,esize", [(4096, 4096, 2), (1000, 1096, 2), (4096, 4096, 1), (8, 128, 2), (3, 64, 1)])
@pytest.mark.parametrize("s", [1, 33, 700, 3000])
def test_fused_decode_with_cache_warming(rows, cols, esize, s):
    """mui_attn_decode_fused_warm: announcing the next kernel's weight matrix (full size, ragged,
    tiny, 8-bit) changes neither the attention output nor the cache, bit for bit, whether the launch
    takes the hint (unsplit short sequences) or ignores it (split ones); the matrix is only read."""
    cap = 4096
    cos, sin, qkv, kc, vc, pos, cpos, v, rk, ref = _fused_decode_inputs(1, s, cap, torch.float16, 32, 8)
    lib = _lib.load()
    _lib.check(lib.mui_tune_warm(256 if rows % 2 == 0 else 64, 0, 2 if s == 33 else 0), "mui_tune_warm")  # opt in
    try:
        _warm_case(rows, cols, esize, s, cos, sin, qkv, kc, vc, pos, cpos, ref)
    finally:
        _lib.check(lib.mui_tune_warm(0, 0, -1), "mui_tune_warm")


def _warm_case(rows, cols, esize, s, cos, sin, qkv, kc, vc, pos, cpos, ref):
    w = torch.randint(-128, 127, (rows, cols * esize), dtype=torch.int8, device=DEV)
    w = w.view(torch.float16) if esize == 2 else w
    w_before = w.clone()
    outs = []
    for hint in (None, w):
        qkv_d, kd, vd = qkv.to(DEV), kc.to(DEV), vc.to(DEV)
        out = muillm_ext.mui_attention_decode_fused(
            qkv_d[:, 0, : 32 * D], qkv_d[:, 0, 32 * D : 40 * D], qkv_d[:, 0, 40 * D :], cos.to(DEV), sin.to(DEV),
            pos.to(DEV), cpos.to(DEV), kd, vd, seq_len=s, next_weights=hint)
        torch.cuda.synchronize()
        outs.append((out, kd, vd))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][2], outs[1][2])
    assert torch.equal(w.view(torch.int8), w_before.view(torch.int8))  # (random bit patterns: compared as integers)
    assert _max_abs(outs[1][0], ref) <= ATOL


@pytest.mark.parametrize("hq,hkv", [(24, 8), (20, 4), (12, 2), (14, 2), (32, 2), (12, 1)])
@pytest.mark.parametrize("b,s,cap", [(1, 257, 512), (2, 3000, 4096)])
def test_fused_decode_other_group_sizes(hq, hkv, b, s, cap):
    """Query heads per KV head other than 1, 2, 4, 8 (Llama-3.2-3B has 3): unsplit and split."""
    _fused_decode_case(b, s, cap, True, torch.float16, hq, hkv)


@functools.lru_cache(maxsize=8)
def _fused_decode_inputs(b, s, cap, dtype, hq, hkv):
    """Seeded inputs and the oracle's result of one fused-decode case (kept for the runs of the
    same case under the other kernel choices: the long contexts take seconds to generate)."""
    g = _gen(7)
    cos, sin = oracle.rope_tables(500000.0, D, cap)
    qkv = _mk((b, 1, (hq + 2 * hkv) * D), g, dtype=dtype)
    kc = torch.zeros(b, hkv, cap, D, dtype=dtype)
    vc = torch.zeros(b, hkv, cap, D, dtype=dtype)
    kc[:, :, : s - 1] = _mk((b, hkv, s - 1, D), g, dtype=dtype)
    vc[:, :, : s - 1] = _mk((b, hkv, s - 1, D), g, dtype=dtype)
    pos = torch.full((b, 1), s - 1, dtype=torch.int64)
    cpos = torch.tensor([s - 1], dtype=torch.int64)

    q = qkv[..., : hq * D].view(b, 1, hq, D).transpose(1, 2)
    k = qkv[..., hq * D : (hq + hkv) * D].view(b, 1, hkv, D).transpose(1, 2)
    v = qkv[..., (hq + hkv) * D :].view(b, 1, hkv, D).transpose(1, 2)
    rq, rk = oracle.apply_rope(q, k, cos, sin, pos)
    rq, rk = rq.to(dtype), rk.to(dtype)
    kref, vref = kc.clone(), vc.clone()
    kk, vv, _ = oracle.static_cache_update(kref, vref, rk, v, cpos, s - 1)
    ref = oracle.decode_attention(rq, kk, vv)
    return cos, sin, qkv, kc, vc, pos, cpos, v, rk, ref


def _fused_decode_case(b, s, cap, device_len, dtype, hq, hkv):
    cos, sin, qkv, kc, vc, pos, cpos, v, rk, ref = _fused_decode_inputs(b, s, cap, dtype, hq, hkv)

    qkv_d, kd, vd = qkv.to(DEV), kc.to(DEV), vc.to(DEV)
    qd = qkv_d[:, 0, : hq * D]
    kn = qkv_d[:, 0, hq * D : (hq + hkv) * D]
    vn = qkv_d[:, 0, (hq + hkv) * D :]
    out, q_out = muillm_ext.mui_attention_decode_fused(
        qd, kn, vn, cos.to(DEV), sin.to(DEV), pos.to(DEV), cpos.to(DEV), kd, vd,
        seq_len=None if device_len else s, seq_len_hint=s, want_q_out=True)
    assert out.shape == (b, 1, hq * D)
    assert _attn_err(out, ref) <= ATOL

    # the written slot is bit-identical to the standalone rotation; all other slots untouched
    q_sa, k_sa = muillm_ext.muillm_rope_forward_no_cache(
        pos.to(DEV), cos.to(DEV), sin.to(DEV),
        qkv_d[..., : hq * D].view(b, 1, hq, D).transpose(1, 2),
        qkv_d[..., hq * D : (hq + hkv) * D].view(b, 1, hkv, D).transpose(1, 2))
    assert torch.equal(kd[:, :, s - 1], k_sa[:, :, 0])
    assert torch.equal(q_out, q_sa)
    assert torch.equal(vd[:, :, s - 1].cpu(), v[:, :, 0])
    keep = torch.ones(cap, dtype=torch.bool)
    keep[s - 1] = False
    assert torch.equal(kd.cpu()[:, :, keep], kc[:, :, keep]) and torch.equal(vd.cpu()[:, :, keep], vc[:, :, keep])
    # 1-ulp agreement of the slot with the oracle's rotation rounded once
    off = (kd[:, :, s - 1].cpu().view(torch.int16).int() - rk[:, :, 0].view(torch.int16).int()).abs().max()
    assert int(off) <= 1


def test_fused_decode_sequence_matches_oracle_steps():
    """Eight consecutive decode steps with the length read from device memory: the cache
    grows in place and every step matches the oracle run on the same growing cache."""
    g = _gen(8)
    b, hq, hkv, cap, start = 2, 32, 8, 128, 37
    cos, sin = oracle.rope_tables(500000.0, D, cap)
    kc = torch.zeros(b, hkv, cap, D, dtype=torch.float16)
    vc = torch.zeros_like(kc)
    kc[:, :, :start] = _mk((b, hkv, start, D), g)
    vc[:, :, :start] = _mk((b, hkv, start, D), g)
    kd, vd = kc.to(DEV), vc.to(DEV)
    cpos_d = torch.tensor([start], dtype=torch.int64, device=DEV)
    pos_d = torch.full((b,), start, dtype=torch.int64, device=DEV)
    cosd, sind = cos.to(DEV), sin.to(DEV)
    seen = start
    for step in range(8):
        qkv = _mk((b, (hq + 2 * hkv) * D), g)
        qkv_d = qkv.to(DEV)
        out = muillm_ext.mui_attention_decode_fused(
            qkv_d[:, : hq * D], qkv_d[:, hq * D : (hq + hkv) * D], qkv_d[:, (hq + hkv) * D :],
            cosd, sind, pos_d, cpos_d, kd, vd, seq_len=None, n_splits=2)
        pos = torch.full((b, 1), seen, dtype=torch.int64)
        q = qkv[:, : hq * D].view(b, 1, hq, D).transpose(1, 2)
        k = qkv[:, hq * D : (hq + hkv) * D].view(b, 1, hkv, D).transpose(1, 2)
        v = qkv[:, (hq + hkv) * D :].view(b, 1, hkv, D).transpose(1, 2)
        rq, rk = oracle.apply_rope(q, k, cos, sin, pos)
        kk, vv, seen = oracle.static_cache_update(kc, vc, rk.half(), v, torch.tensor([seen]), seen)
        ref = oracle.decode_attention(rq.half(), kk, vv)
        assert _max_abs(out, ref) <= ATOL, f"step {step}"
        cpos_d += 1  # device-side counters, as a HIP-graph replay would advance them
        pos_d += 1
    assert (kd.cpu()[:, :, :seen].float() - kc[:, :, :seen].float()).abs().max() <= 8e-3


# ------------------------------------------------------------------------------------
# causal attention of T > 1 new tokens (prefill)
# ------------------------------------------------------------------------------------
def _causal_mask(t, s, q_start):
    m = torch.zeros(1, 1, t, s, dtype=torch.float64)
    key = torch.arange(s)[None, :]
    qry = q_start + torch.arange(t)[:, None]
    m[0, 0][key > qry] = float("-inf")
    return m


@pytest.mark.parametrize("b,hq,hkv,t,past", [
    (1, 32, 8, 32, 0), (2, 8, 2, 5, 0), (1, 32, 8, 16, 100), (1, 4, 4, 77, 3), (3, 16, 2, 33, 31), (1, 32, 8, 300, 0),
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefill_attention(b, hq, hkv, t, past, dtype):
    g = _gen(21)
    s = past + t
    cap = oracle.next_pow2(s)
    q = _mk((b, hq, t, D), g, dtype=dtype)
    kc = _mk((b, hkv, cap, D), g, dtype=dtype)
    vc = _mk((b, hkv, cap, D), g, dtype=dtype)
    kc[:, :, s:] = float("nan")  # rows beyond the sequence must never be read
    vc[:, :, s:] = float("nan")
    ref = oracle.decode_attention(q, kc[:, :, :s], vc[:, :, :s], _causal_mask(t, s, past))
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = muillm_ext.mui_prefill_attention(q.to(DEV), kd[:, :, :s], vd[:, :, :s])
    assert out.shape == (b, t, hq * D) and torch.isfinite(out).all()
    # bf16 prompts: the probabilities enter the matrix cores with bf16's 8 bits, which costs up to
    # 2^-9 max |V| per key beyond the rounding of the stored output (measured 2.6e-3): held at 4e-3
    assert _attn_err(out, ref) <= (ATOL if dtype == torch.float16 else BF16_PROMPT_ATOL)


@pytest.mark.parametrize("choice", ["auto", "kv-group", "kv-group-register-staged", "per-head"])
@pytest.mark.parametrize("b,hq,hkv,t,past", [
    (1, 32, 8, 2048, 0),     # the kernel shared by the four query heads of a KV head
    (1, 32, 8, 1000, 24),    # ragged: not a multiple of the 32-position blocks, continues a cache
    (2, 8, 8, 130, 5),       # one query head per KV head: four position blocks per workgroup
    (1, 16, 8, 260, 0),      # two
    (1, 64, 8, 140, 0),      # eight (8 waves)
    (1, 24, 8, 300, 0),      # three: no kv-group variant, the per-head kernel serves it
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefill_attention_long_prompts(b, hq, hkv, t, past, dtype, choice):
    """Prompt attention under each kernel choice (built-in; K/V shared by the query heads of a KV
    head; one workgroup per 16 positions of one head), a sample of query rows against the oracle."""
    if dtype == torch.bfloat16 and t > 1000:
        t = 520
    lib = _lib.load()
    _lib.check(lib.mui_tune_prefill_attention({"auto": 0, "kv-group": 1, "kv-group-register-staged": 1000001, "per-head": -1}[choice]), "tune")
    try:
        g = _gen(23)
        s = past + t
        cap = oracle.next_pow2(s)
        q = _mk((b, hq, t, D), g, dtype=dtype)
        kc = _mk((b, hkv, cap, D), g, dtype=dtype)
        vc = _mk((b, hkv, cap, D), g, dtype=dtype)
        kc[:, :, s:] = float("nan")  # rows beyond the sequence must never be read
        vc[:, :, s:] = float("nan")
        kd, vd = kc.to(DEV), vc.to(DEV)
        out = muillm_ext.mui_prefill_attention(q.to(DEV), kd[:, :, :s], vd[:, :, :s])
        assert out.shape == (b, t, hq * D) and torch.isfinite(out).all()
        rows = sorted(set(list(range(0, min(t, 40))) + list(range(t // 2 - 20, t // 2 + 20)) + list(range(t - 40, t))))
        rows = torch.tensor([r for r in rows if 0 <= r < t])
        mask = _causal_mask(t, s, past)[:, :, rows]
        ref = oracle.decode_attention(q[:, :, rows], kc[:, :, :s], vc[:, :, :s], mask)
        assert _attn_err(out[:, rows], ref) <= (ATOL if dtype == torch.float16 else BF16_PROMPT_ATOL)
    finally:
        _lib.check(lib.mui_tune_prefill_attention(0), "tune")


@pytest.mark.parametrize("choice", ["kv-group", "kv-group-register-staged", "per-head"])
@pytest.mark.parametrize("b,hq,hkv,t,past,padding", [
    (3, 32, 8, 200, 0, "left"),      # the reference's padded batches (tokenizer padding on the left)
    (2, 32, 8, 610, 0, "left"),
    (2, 8, 8, 97, 7, "right"),       # ragged, continues a cache, padding behind the prompt
    (2, 16, 8, 300, 0, "holes"),     # arbitrary hidden keys
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_prefill_attention_key_padding_mask(b, hq, hkv, t, past, padding, dtype, choice):
    """Prompt attention with a key-padding mask (mui_prefill_attention_masked) under both prompt
    kernels against the oracle with the additive 4-D mask the reference would build
    (muillm/modules/models/llama/model.py:437-613): every row that sees a key; rows that see none
    (padding queries of a left-padded row) come out as zeros."""
    lib = _lib.load()
    _lib.check(lib.mui_tune_prefill_attention({"kv-group": 1, "kv-group-register-staged": 1000001, "per-head": -1}[choice]), "tune")
    try:
        g = _gen(29)
        s = past + t
        q = _mk((b, hq, t, D), g, dtype=dtype)
        kc = _mk((b, hkv, s, D), g, dtype=dtype)
        vc = _mk((b, hkv, s, D), g, dtype=dtype)
        keep = torch.ones(b, s, dtype=torch.long)
        for row in range(b):
            n_pad = (37 * (row + 1)) % (t // 2)
            if padding == "left":
                keep[row, :n_pad] = 0
            elif padding == "right":
                keep[row, s - n_pad:] = 0
            else:
                keep[row, torch.randperm(s, generator=g)[:n_pad]] = 0
        key_mask = muillm_ext.key_padding_mask16(keep.to(DEV), dtype)
        assert key_mask.shape[1] % 8 == 0 and key_mask.shape[1] >= s
        out = muillm_ext.mui_prefill_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), key_mask=key_mask)
        assert out.shape == (b, t, hq * D) and torch.isfinite(out).all()
        mask4 = _causal_mask(t, s, past).expand(b, 1, t, s).clone()
        mask4 = mask4.masked_fill(keep[:, None, None, :] == 0, float("-inf"))
        sees_a_key = torch.isfinite(mask4).any(dim=-1)[:, 0]          # [b, t]
        safe = mask4.clone()
        safe[~sees_a_key[:, None].expand(b, 1, t)] = 0.0                # any finite row: those outputs are not compared
        ref = oracle.decode_attention(q, kc, vc, safe).reshape(b, t, hq * D)
        got = out.cpu().float()
        assert _attn_err(out.cpu()[sees_a_key], ref[sees_a_key]) <= (ATOL if dtype == torch.float16 else BF16_PROMPT_ATOL)
        if (~sees_a_key).any():
            assert float(got[~sees_a_key].abs().max()) == 0.0
    finally:
        _lib.check(lib.mui_tune_prefill_attention(0), "tune")


def test_prefill_attention_masked_abi_errors():
    lib = _lib.load()
    q = torch.zeros(1, 8, 32, D, dtype=torch.float16, device=DEV)
    kv = torch.zeros(1, 8, 32, D, dtype=torch.float16, device=DEV)
    out = torch.empty(1, 32, 8 * D, dtype=torch.float16, device=DEV)
    mask = torch.zeros(1, 32, dtype=torch.float16, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    args = (st, 0, q.data_ptr(), kv.data_ptr(), kv.data_ptr(), 8 * 32 * D, 32 * D, D, 32, 0)
    tail = (out.data_ptr(), 1, 8, 8, 32, D)
    assert lib.mui_prefill_attention_masked(*args, None, 32, *tail) == -1             # no mask
    assert lib.mui_prefill_attention_masked(*args, mask.data_ptr() + 2, 32, *tail) == -4  # misaligned
    assert lib.mui_prefill_attention_masked(*args, mask.data_ptr(), 30, *tail) == -4   # stride not a multiple of 4
    assert lib.mui_prefill_attention_masked(*args, mask.data_ptr(), 28, *tail) == -1   # rows shorter than the keys
    with pytest.raises(RuntimeError, match="key_mask"):
        muillm_ext.mui_prefill_attention(q, kv, kv, key_mask=mask.to(torch.bfloat16))


def test_prefill_attention_8k_rows_vs_oracle_and_kernels_agree():
    """An 8192-token prompt (32 / 8 heads): sampled rows against the oracle, and the two prompt
    kernels against each other on every row."""
    lib = _lib.load()
    g = _gen(24)
    t = 8192
    q, kc, vc = _mk((1, 32, t, D), g), _mk((1, 8, t, D), g), _mk((1, 8, t, D), g)
    qd, kd, vd = q.to(DEV), kc.to(DEV), vc.to(DEV)
    outs = {}
    for name, knob in (("kv-group", 1), ("kv-group-register-staged", 1000001), ("per-head", -1)):
        _lib.check(lib.mui_tune_prefill_attention(knob), "tune")
        try:
            outs[name] = muillm_ext.mui_prefill_attention(qd, kd, vd)
        finally:
            _lib.check(lib.mui_tune_prefill_attention(0), "tune")
    assert float((outs["kv-group"].float() - outs["per-head"].float()).abs().max()) <= 2 * ATOL
    # K / V rows loaded straight into LDS or staged through registers: the same arithmetic
    assert torch.equal(outs["kv-group"], outs["kv-group-register-staged"])
    rows = torch.tensor(list(range(0, 24)) + list(range(4085, 4110)) + list(range(t - 24, t)))
    ref = oracle.decode_attention(q[:, :, rows], kc, vc, _causal_mask(t, t, 0)[:, :, rows])
    assert _max_abs(outs["kv-group"][:, rows], ref) <= ATOL


def test_prefill_attention_closed_forms():
    g = _gen(22)
    hq, hkv, t = 8, 2, 40
    q = _mk((1, hq, t, D), g).to(DEV)
    k = _mk((1, hkv, t, D), g).to(DEV)
    v = _mk((1, hkv, t, D), g).to(DEV)
    out = muillm_ext.mui_prefill_attention(q, k, v).view(t, hq, D)
    # the first query sees only key 0 -> its value, exactly
    assert torch.equal(out[0], v[0, :, 0].repeat_interleave(hq // hkv, dim=0))
    # the last query row equals single-token decoding over the same keys
    dec = muillm_ext.muillm_causal_transformer_decoding_no_mask(q[:, :, -1:].contiguous(), k, v).view(hq, D)
    assert (out[-1].float() - dec.float()).abs().max() <= 1e-3
    # changing a FUTURE key/value must not change earlier rows (causality)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 30:] += 3.0
    v2[:, :, 30:] -= 2.0
    out2 = muillm_ext.mui_prefill_attention(q, k2, v2).view(t, hq, D)
    assert torch.equal(out2[:30], out[:30]) and not torch.equal(out2[30:], out[30:])


def test_attention_abi_errors():
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    q = torch.zeros(1, 32, 128, dtype=torch.float16, device=DEV)
    kc = torch.zeros(1, 8, 16, 128, dtype=torch.float16, device=DEV)
    out = torch.zeros(1, 32 * 128, dtype=torch.float16, device=DEV)
    args = (kc.stride(0), kc.stride(1), kc.stride(2), None, 0)
    assert lib.mui_flash_decode(s, 0, q.data_ptr(), kc.data_ptr(), kc.data_ptr(), *args, 4, None, 1, out.data_ptr(), 1, 32, 8, 64, 16) == -2
    assert lib.mui_flash_decode(s, 0, q.data_ptr(), kc.data_ptr(), kc.data_ptr(), *args, 4, None, 1, out.data_ptr(), 1, 32, 5, 128, 16) == -1
    assert lib.mui_flash_decode(s, 0, q.data_ptr(), kc.data_ptr(), kc.data_ptr(), *args, 40, None, 1, out.data_ptr(), 1, 32, 8, 128, 16) == -1
    assert lib.mui_flash_decode(s, 0, q.data_ptr(), kc.data_ptr(), kc.data_ptr(), *args, 4, None, 2, out.data_ptr(), 1, 32, 8, 128, 16) == -1
    assert lib.mui_flash_decode_scratch_bytes(2, 32, 128, 1) == 0
    assert lib.mui_flash_decode_scratch_bytes(2, 32, 128, 4) == 2 * 32 * 4 * 130 * 4
    with pytest.raises(RuntimeError):
        muillm_ext.muillm_causal_transformer_decoding_no_mask(torch.zeros(1, 32, 2, 128, dtype=torch.float16, device=DEV), kc, kc)


def test_rope_positions_outside_the_tables_and_batch_capacity():
    """Positions are read on the device, so the kernels get the table height: a position beyond
    the tables uses the last row instead of reading past it; a batch larger than the cache is
    refused by the wrappers; a table height of zero by the C ABI."""
    lib = _lib.load()
    g = _gen(12)
    rows = 64
    cos, sin = oracle.rope_tables(500000.0, D, rows)
    q, k = _mk((1, 4, 1, D), g).to(DEV), _mk((1, 1, 1, D), g).to(DEV)
    last = torch.full((1, 1), rows - 1, dtype=torch.int64, device=DEV)
    beyond = torch.full((1, 1), rows + 1000, dtype=torch.int64, device=DEV)
    negative = torch.full((1, 1), -5, dtype=torch.int64, device=DEV)
    zero = torch.zeros((1, 1), dtype=torch.int64, device=DEV)
    q_last, k_last = muillm_ext.muillm_rope_forward_no_cache(last, cos.to(DEV), sin.to(DEV), q, k)
    q_far, k_far = muillm_ext.muillm_rope_forward_no_cache(beyond, cos.to(DEV), sin.to(DEV), q, k)
    q_neg, _ = muillm_ext.muillm_rope_forward_no_cache(negative, cos.to(DEV), sin.to(DEV), q, k)
    q_zero, _ = muillm_ext.muillm_rope_forward_no_cache(zero, cos.to(DEV), sin.to(DEV), q, k)
    assert torch.equal(q_far, q_last) and torch.equal(k_far, k_last) and torch.equal(q_neg, q_zero)
    # fused decode entry: same clamp
    kc = torch.zeros(1, 1, 16, D, dtype=torch.float16, device=DEV)
    vc = torch.zeros_like(kc)
    cpos = torch.zeros(1, dtype=torch.int64, device=DEV)
    qkv = _mk((1, 6 * D), g).to(DEV)
    outs = []
    for pos in (last, beyond):
        kc.zero_(); vc.zero_()
        outs.append((muillm_ext.mui_attention_decode_fused(qkv[:, : 4 * D], qkv[:, 4 * D : 5 * D], qkv[:, 5 * D :],
                                                           cos.to(DEV), sin.to(DEV), pos, cpos, kc, vc, seq_len=1),
                     kc.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    # wrappers refuse a batch the cache cannot hold
    qkv2 = _mk((2, 6 * D), g).to(DEV)
    with pytest.raises(RuntimeError, match="batch"):
        muillm_ext.mui_attention_decode_fused(qkv2[:, : 4 * D], qkv2[:, 4 * D : 5 * D], qkv2[:, 5 * D :], cos.to(DEV),
                                              sin.to(DEV), torch.zeros(2, 1, dtype=torch.int64, device=DEV), cpos,
                                              kc, vc, seq_len=1)
    with pytest.raises(RuntimeError, match="batch"):
        muillm_ext.muillm_static_kvcache_update(kc, vc, _mk((2, 1, 1, D), g).to(DEV), _mk((2, 1, 1, D), g).to(DEV),
                                                cpos, 1)
    # C ABI: tables without a height are an invalid argument
    s = torch.cuda.current_stream().cuda_stream
    c32, s32 = cos.to(DEV), sin.to(DEV)
    out = torch.zeros(1, 4 * D, dtype=torch.float16, device=DEV)
    st = lib.mui_attn_decode_fused(s, 0, qkv.data_ptr(), 6 * D, qkv.data_ptr() + 8 * D, 6 * D, qkv.data_ptr() + 10 * D,
                                   6 * D, c32.data_ptr(), s32.data_ptr(), D // 2, 0, zero.data_ptr(), 1, cpos.data_ptr(),
                                   1, kc.data_ptr(), vc.data_ptr(), kc.stride(0), kc.stride(1), kc.stride(2), None, 0,
                                   None, None, 1, out.data_ptr(), 1, 4, 1, D, 16)
    assert st == -1
