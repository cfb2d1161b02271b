"""GPU parity of the linear entry points at prompt sizes (more than MUI_MAX_TOKENS tokens): the
tiled matrix-core GEMM with fused RMSNorm prologue and residual / bias / SiLU*mul epilogues, for
16-bit weights and int8 weights, against the CPU oracle.

The reference hands these calls to the framework's GEMM (csrc/modules/linear_module.cpp:57-79);
its own tests compare batch-4 layers with HuggingFace at allclose(rtol 1e-4, atol 1e-1)
(tests/test_linear.py, tests/test_gateupdownmlp.py there).  Gate here: the fp16/bf16 output
gate of the decode kernels (max error over max |ref| <= 1e-2 fp16 / 2e-2 bf16, elementwise form
included), plus that reference tolerance."""

import functools

import pytest
import torch

import oracle
from muillm_amd import _lib, muillm_ext
from tests.util import assert_parity, reference_allclose

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(params=["auto", "wide", "tile-256x256", "tile-128x128", "tile-64x128", "tile-32x64", "ksplit-64x128", "ksplit-32x64", "tile-128x256", "tile-192x256", "tile-96x128", "ksplit-128x128", "ksplit-128x64", "ksplit-64x64", "tile-256x256-16-waves", "tile-256x256-register-staged"], autouse=True)
def prompt_kernel_choice(request):
    """Every test runs with the built-in kernel choice and with each prompt kernel forced: the
    16-rows-per-workgroup kernel without LDS tiling (up to 128 tokens; longer prompts keep the
    built-in choice) and the shapes of the LDS-tiled kernel (the gate/up epilogue has no
    32 x 64, 64 x 64 and 96 x 128 shapes and takes 64 x 128 / 128 x 128 then; int8 weights have no
    96-row shape and take 128 x 128)."""
    lib = _lib.load()
    knobs = {"auto": (0, 0), "wide": (0, 128), "tile-256x256": (4, -1), "ksplit-64x128": (5, -1), "ksplit-32x64": (6, -1), "tile-128x128": (1, -1), "tile-64x128": (2, -1), "tile-32x64": (3, -1),
             "tile-128x256": (7, -1), "tile-192x256": (8, -1), "tile-96x128": (10, -1), "ksplit-128x128": (9, -1), "ksplit-128x64": (11, -1), "ksplit-64x64": (12, -1),
             "tile-256x256-16-waves": (13, -1), "tile-256x256-register-staged": (104, -1)}
    _lib.check(lib.mui_tune_prefill(*knobs[request.param]), "mui_tune_prefill")
    # the built-in choice runs as shipped (prompts normalised by one rmsnorm launch in front of
    # the GEMM); the forced kernels keep the norm fused into the GEMM, which the C entry points
    # still offer
    muillm_ext.PROMPT_NORM_FIRST = request.param == "auto"
    yield request.param
    muillm_ext.PROMPT_NORM_FIRST = True
    _lib.check(lib.mui_tune_prefill(0, 0), "mui_tune_prefill")


@functools.lru_cache(maxsize=64)
def _oracle_linear_case(tokens, n, k, norm, res, bias):
    """Seeded inputs and the oracle's result, shared by the runs of a case under each kernel choice."""
    g = _gen(0)
    w = _mk((n, k), g, 0.02)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0) if norm else None
    r = _mk((tokens, n), g) if res else None
    b = _mk((n,), g, 0.5) if bias else None
    return w, x, gamma, r, b, oracle.linear(x, w, gamma, 1e-5, b, r)


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _mk(shape, g, std=1.0, mean=0.0, dtype=torch.float16):
    return (mean + std * torch.randn(shape, generator=g)).to(dtype)


@pytest.mark.parametrize("tokens", [33, 64, 128, 512])
@pytest.mark.parametrize("n,k,norm,res,bias", [
    (4096, 4096, True, True, False),     # config 1 as a prompt
    (6144, 4096, True, False, False),    # fused QKV
    (4096, 14336, False, True, False),   # down projection
    (1000, 2056, True, True, True),      # rows not a multiple of the tile, K not a multiple of the step
    (130, 72, False, False, True),       # smaller than one tile / barely over one step
    (33, 8, True, True, False),          # a single k-chunk, odd row count (scalar stores)
])
def test_linear_prompt(tokens, n, k, norm, res, bias):
    if tokens == 512 and n * k > 4096 * 4096:
        tokens = 300  # keeps the float64 oracle quick; still three token tiles with a ragged last one
    w, x, gamma, r, b, ref = _oracle_linear_case(tokens, n, k, norm, res, bias)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), None if gamma is None else gamma.to(DEV), 1e-5,
                                         None, None if b is None else b.to(DEV), None if r is None else r.to(DEV))
    assert y.shape == (tokens, n)
    assert_parity(y, ref, 1e-2, f"prompt linear {tokens}x{n}x{k}", tight=5e-3)
    assert reference_allclose(y, ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tokens", [33, 128, 257])
def test_linear_prompt_mul_bias_and_bf16(tokens, dtype):
    g = _gen(1)
    n, k = 520, 1024
    w, x = _mk((n, k), g, 0.02, dtype=dtype), _mk((2, tokens, k), g, dtype=dtype)   # [B, T, K] input
    gamma, mb = _mk((k,), g, 0.1, 1.0, dtype=dtype), _mk((n,), g, 0.2, 1.0, dtype=dtype)
    ab, r = _mk((n,), g, 0.5, dtype=dtype), _mk((2, tokens, n), g, dtype=dtype)
    ref = (oracle.linear(x, w, gamma, 1e-5).double() * mb.double() + ab.double() + r.double())
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), gamma.to(DEV), 1e-5, mb.to(DEV), ab.to(DEV), r.to(DEV))
    assert y.shape == (2, tokens, n) and y.dtype == dtype
    assert_parity(y, ref, 1e-2, f"prompt linear mul_bias {dtype}")


@pytest.mark.parametrize("tokens", [33, 64, 128, 512])
@pytest.mark.parametrize("n,k", [(14336, 4096), (700, 520)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gateup_prompt(tokens, n, k, dtype):
    if n * k > 4096 * 4096 and (dtype == torch.bfloat16 or tokens == 512):
        tokens = min(tokens, 200)
    g = _gen(2)
    wg, wu = _mk((n, k), g, 0.02, dtype=dtype), _mk((n, k), g, 0.02, dtype=dtype)
    x, gamma = _mk((tokens, k), g, dtype=dtype), _mk((k,), g, 0.1, 1.0, dtype=dtype)
    ref = oracle.gateup_silu(x, wg, wu, gamma, 1e-5)
    packed = torch.stack([wg, wu], dim=1).contiguous().to(DEV)   # the module's interleaved [N, 2, K] buffer
    h = muillm_ext.mui_gateup_silu(gamma.to(DEV), 1e-5, packed[:, 0], packed[:, 1], x.to(DEV))
    # The stated gate -- max error over max |ref| <= 1e-2 -- holds in both types (bf16 measures 3.8e-3).
    # The additional elementwise form is held at 1e-2 for fp16. For bf16 it is 4e-2 here, and only
    # here and in the model-level tests: the matrix cores read gamma * x rounded to bf16's 8 bits, and
    # under SiLU * mul single elements then sit up to 3.3e-2 of |ref| + rms(ref) away from the oracle
    # with exact operands. That level belongs to the format, not to the kernel:
    # tests/test_oracle_cpu.py::test_bf16_gateup_elementwise_error_is_set_by_the_8_bit_operands finds
    # it with everything but the operand rounding exact, for this rounding and for the reference's
    # own (its RMSNorm fallback rounds twice, muillm/modules/norm/rmsnorm.py:140-146).
    assert_parity(h, ref, 1e-2, f"prompt gate/up {tokens}x{n}x{k} {dtype}",
                  elementwise=None if dtype == torch.float16 else 4e-2)
    h2 = muillm_ext.mui_gateup_silu(gamma.to(DEV), 1e-5, wg.to(DEV), wu.to(DEV), x.to(DEV))  # two dense matrices
    assert torch.equal(h, h2)


def test_mlp_prompt_matches_chunked_decode_kernels():
    """The whole MLP at 40 tokens: the tiled GEMM against the same call cut into 16-token chunks of
    the decode kernels (two independent kernel families) and against the oracle."""
    g = _gen(3)
    hid, inter, tokens = 1024, 2816, 40
    wg, wu, wd = _mk((inter, hid), g, 0.02), _mk((inter, hid), g, 0.02), _mk((hid, inter), g, 0.02)
    x, r, gamma = _mk((tokens, hid), g), _mk((tokens, hid), g), _mk((hid,), g, 0.1, 1.0)
    ref = oracle.gateupdown_mlp(x, wg, wu, wd, gamma, 1e-5, r)
    args = (gamma.to(DEV), 1e-5, wg.to(DEV), wu.to(DEV), wd.to(DEV), r.to(DEV), x.to(DEV))
    out = muillm_ext.muillm_gateupsilu_forward(None, *args)
    old = muillm_ext.FUSED_CHUNK_MAX_TOKENS
    try:
        muillm_ext.FUSED_CHUNK_MAX_TOKENS = 64
        chunked = muillm_ext.muillm_gateupsilu_forward(None, *args)
    finally:
        muillm_ext.FUSED_CHUNK_MAX_TOKENS = old
    assert_parity(out, ref, 1e-2, "prompt MLP (tiled GEMM)")
    assert_parity(chunked, ref, 1e-2, "prompt MLP (decode kernels in chunks)")
    assert float((out.float() - chunked.float()).abs().max()) <= 2e-2


@pytest.mark.parametrize("tokens", [65, 128, 300])
@pytest.mark.parametrize("n,k", [(6144, 4096), (4096, 14336), (200, 528)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_int8_channel_linear_prompt(tokens, n, k, dtype):
    g = _gen(4)
    w = _mk((n, k), g, 0.02)
    q, s = oracle.rtn_quantize_channel(w)
    s = s.to(dtype)
    x, gamma, r = _mk((tokens, k), g, dtype=dtype), _mk((k,), g, 0.1, 1.0, dtype=dtype), _mk((tokens, n), g, dtype=dtype)
    wexact = q.double() * s.double()[:, None]
    ref = oracle.linear(x, wexact, gamma, 1e-5, None, r)
    y = muillm_ext.mui_int8_channel_linear_forward(x.to(DEV), q.to(DEV), s.to(DEV), gamma.to(DEV), 1e-5, None, r.to(DEV))
    assert_parity(y, ref, 1e-2, f"int8 prompt linear {tokens}x{n}x{k} {dtype}")


@pytest.mark.parametrize("tokens", [65, 200])
@pytest.mark.parametrize("n,k", [(14336, 4096), (136, 272)])
def test_int8_channel_gateup_prompt(tokens, n, k):
    g = _gen(5)
    qg, sg = oracle.rtn_quantize_channel(_mk((n, k), g, 0.02))
    qu, su = oracle.rtn_quantize_channel(_mk((n, k), g, 0.02))
    x, gamma = _mk((tokens, k), g), _mk((k,), g, 0.1, 1.0)
    ref = oracle.gateup_silu(x, qg.double() * sg.double()[:, None], qu.double() * su.double()[:, None], gamma, 1e-5)
    pw = torch.stack([qg, qu], dim=1).contiguous().to(DEV)
    ps = torch.stack([sg, su], dim=1).contiguous().to(DEV)
    h = muillm_ext.mui_int8_channel_gateupsilu_forward(gamma.to(DEV), 1e-5, pw[:, 0], pw[:, 1], ps[:, 0], ps[:, 1], x.to(DEV))
    assert_parity(h, ref, 1e-2, f"int8 prompt gate/up {tokens}x{n}x{k}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_int8_channel_long_prompt_dequantises_once(dtype, monkeypatch):
    """From INT8_DEQUANT_MIN_TOKENS tokens the per-channel matrix is dequantised once per call
    (T(float(q) * float(s)), the rounding of the dequantisation kernel) and the GEMM runs on 16-bit
    weights. Gate 1e-2 against the oracle on the exact q * s, as for the converting GEMM, which must
    also agree with it to 1e-2 of the output's maximum on the same inputs."""
    g = _gen(14)
    tokens, n, k = muillm_ext.INT8_DEQUANT_MIN_TOKENS, 520, 1024
    q, s = oracle.rtn_quantize_channel(_mk((n, k), g, 0.02))
    s = s.to(dtype)
    x, gamma, r = _mk((tokens, k), g, dtype=dtype), _mk((k,), g, 0.1, 1.0, dtype=dtype), _mk((tokens, n), g, dtype=dtype)
    ref = oracle.linear(x, q.double() * s.double()[:, None], gamma, 1e-5, None, r)
    args = (x.to(DEV), q.to(DEV), s.to(DEV), gamma.to(DEV), 1e-5, None, r.to(DEV))
    y = muillm_ext.mui_int8_channel_linear_forward(*args)
    assert_parity(y, ref, 1e-2, f"int8 long prompt linear (dequantised once) {dtype}")
    qu, su = oracle.rtn_quantize_channel(_mk((n, k), g, 0.02))
    su = su.to(dtype)
    refh = oracle.gateup_silu(x, q.double() * s.double()[:, None], qu.double() * su.double()[:, None], gamma, 1e-5)
    pw = torch.stack([q, qu], dim=1).contiguous().to(DEV)
    ps = torch.stack([s, su], dim=1).contiguous().to(DEV)
    gargs = (gamma.to(DEV), 1e-5, pw[:, 0], pw[:, 1], ps[:, 0], ps[:, 1], x.to(DEV))
    h = muillm_ext.mui_int8_channel_gateupsilu_forward(*gargs)
    # bf16 gate/up: two 8-bit-mantissa operands of SiLU * mul set the elementwise floor (4e-2), as for 16-bit weights
    assert_parity(h, refh, 1e-2, f"int8 long prompt gate/up (dequantised once) {dtype}",
                  elementwise=None if dtype == torch.float16 else 4e-2)
    # the same calls on the GEMM that converts the codes on their way to LDS
    monkeypatch.setattr(muillm_ext, "INT8_DEQUANT_MIN_TOKENS", 1 << 30)
    y2 = muillm_ext.mui_int8_channel_linear_forward(*args)
    h2 = muillm_ext.mui_int8_channel_gateupsilu_forward(*gargs)
    for name, a_, b_ in (("linear", y, y2), ("gate/up", h, h2)):
        d = float((a_.float() - b_.float()).abs().max() / b_.float().abs().max())
        print(f"[parity] int8 long prompt {name} {dtype}: dequantise-once vs converting GEMM {d:.2e} of max (gate 1e-2)")
        assert d <= 1e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("route", ["scale-and-min-on-the-way-to-LDS", "dequantise-once"])
@pytest.mark.parametrize("tokens", [17, 40, 65, 150])
def test_int8_group_format_prompt(tokens, route, dtype, monkeypatch):
    """The reference's group format at prompt sizes, on both routes the host layer has: the tiled GEMM
    that turns a chunk of codes into u8 * scale + min, rounded once, on its way to LDS (prompts of
    17 .. INT8_GROUP_DEQUANT_MIN_TOKENS - 1 tokens), and the matrix dequantised by the library's
    kernel (the same values, bit-exact definition) followed by the 16-bit GEMM -- the reference's
    own route (int8linear.py:279-293), taken for longer prompts."""
    monkeypatch.setattr(muillm_ext, "INT8_GROUP_DEQUANT_MIN_TOKENS", 17 if route == "dequantise-once" else 1 << 30)
    g = _gen(6)
    n, k, gs = 1040, 1024, 128
    qw, smv = oracle.rtn_quantize_group(_mk((n, k), g, 0.02), gs)
    smv = smv.to(dtype)                                                # (scale, min) pairs in the activation dtype
    x, gamma, r = _mk((tokens, k), g, dtype=dtype), _mk((k,), g, 0.1, 1.0, dtype=dtype), _mk((tokens, n), g, dtype=dtype)
    wd = oracle.rtn_dequantize_group(qw, smv, gs, dtype=dtype)         # what the dequantisation kernel produces
    ref = oracle.linear(x, wd, gamma, 1e-5, None, r)
    y = muillm_ext.muillm_int8_linear_forward(x.to(DEV), qw.to(DEV), smv.to(DEV), 7, gamma.to(DEV), 1e-5,
                                              residual=r.to(DEV))
    assert_parity(y, ref, 1e-2, f"group-format prompt linear {dtype}")
    qu, smu = oracle.rtn_quantize_group(_mk((n, k), g, 0.02), gs)
    smu = smu.to(dtype)
    pw = torch.stack([qw, qu], dim=1).contiguous().to(DEV)
    ps = torch.stack([smv.reshape(n, -1, 2), smu.reshape(n, -1, 2)], dim=1).contiguous().to(DEV)
    h = muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, pw, ps, 7, x.to(DEV))
    refh = oracle.gateup_silu(x, wd, oracle.rtn_dequantize_group(qu, smu, gs, dtype=dtype), gamma, 1e-5)
    # bf16 gate/up: two 8-bit-mantissa operands of SiLU * mul set the elementwise floor (4e-2), as for 16-bit weights
    assert_parity(h, refh, 1e-2, f"group-format prompt gate/up {dtype}", elementwise=None if dtype == torch.float16 else 4e-2)


def test_prompt_abi_direct_and_errors():
    """Straight through the C ABI (ctypes): 48 tokens, and the argument checks of the tiled path."""
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    g = _gen(7)
    n, k, tokens = 256, 512, 48
    w, x, r = _mk((n, k), g, 0.02).to(DEV), _mk((tokens, k), g).to(DEV), _mk((tokens, n), g).to(DEV)
    y = torch.zeros(tokens, n, dtype=torch.float16, device=DEV)
    st = lib.mui_linear(s, 0, w.data_ptr(), k, x.data_ptr(), None, 0.0, None, None, r.data_ptr(), y.data_ptr(), n, k, tokens)
    assert st == 0
    assert_parity(y, oracle.linear(x.cpu(), w.cpu(), residual=r.cpu()), 1e-2, "ABI prompt linear")
    assert lib.mui_linear(s, 0, w.data_ptr(), k, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), n, 12, tokens) == -2
    assert lib.mui_linear(s, 0, w.data_ptr() + 2, k, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), n, k, tokens) == -4
    assert lib.mui_linear(s, 7, w.data_ptr(), k, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), n, k, tokens) == -1


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_group_format_prompt_abi_with_fused_norm(dtype):
    """mui_int8_group_linear / mui_int8_group_gateup_silu straight through the C ABI with 48 tokens
    AND norm weights: the tiled GEMM normalises the token rows while staging them (the host layer
    would normalise first) and applies (scale, min) to the codes on their way to LDS. Refused: groups
    smaller than 16 codes and a K that is not a whole number of groups."""
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    g = _gen(15)
    n, k, gs, tokens = 272, 1024, 128, 48
    code = 0 if dtype == torch.float16 else 1
    qw, smv = oracle.rtn_quantize_group(_mk((n, k), g, 0.02), gs)
    qu, smu = oracle.rtn_quantize_group(_mk((n, k), g, 0.02), gs)
    smv, smu = smv.to(dtype), smu.to(dtype)
    x, gamma, r = _mk((tokens, k), g, dtype=dtype), _mk((k,), g, 0.1, 1.0, dtype=dtype), _mk((tokens, n), g, dtype=dtype)
    wd, ud = oracle.rtn_dequantize_group(qw, smv, gs, dtype=dtype), oracle.rtn_dequantize_group(qu, smu, gs, dtype=dtype)
    qd, sd, xd, gd, rd = qw.to(DEV), smv.to(DEV), x.to(DEV), gamma.to(DEV), r.to(DEV)
    y = torch.zeros(tokens, n, dtype=dtype, device=DEV)
    st = lib.mui_int8_group_linear(s, code, qd.data_ptr(), k, sd.data_ptr(), 7, xd.data_ptr(), gd.data_ptr(), 1e-5, None,
                                   rd.data_ptr(), y.data_ptr(), n, k, tokens)
    assert st == 0
    tol = 1e-2
    assert_parity(y, oracle.linear(x, wd, gamma, 1e-5, None, r), tol, f"ABI group-format prompt linear, fused norm {dtype}")
    pw = torch.stack([qw, qu], dim=1).contiguous().to(DEV)
    ps = torch.stack([smv.reshape(n, -1, 2), smu.reshape(n, -1, 2)], dim=1).contiguous().to(DEV)
    h = torch.zeros(tokens, n, dtype=dtype, device=DEV)
    gcount = k // gs
    st = lib.mui_int8_group_gateup_silu(s, code, pw.data_ptr(), pw.data_ptr() + k, 2 * k, ps.data_ptr(),
                                        ps.data_ptr() + 2 * gcount * ps.element_size(), 4 * gcount, 7, xd.data_ptr(),
                                        gd.data_ptr(), 1e-5, h.data_ptr(), n, k, tokens)
    assert st == 0
    assert_parity(h, oracle.gateup_silu(x, wd, ud, gamma, 1e-5), tol, f"ABI group-format prompt gate/up, fused norm {dtype}",
                  elementwise=None if dtype == torch.float16 else 4e-2)
    assert lib.mui_int8_group_linear(s, code, qd.data_ptr(), k, sd.data_ptr(), 3, xd.data_ptr(), None, 0.0, None, None,
                                     y.data_ptr(), n, k, tokens) == -2
    assert lib.mui_int8_group_linear(s, code, qd.data_ptr(), k, sd.data_ptr(), 9, xd.data_ptr(), None, 0.0, None, None,
                                     y.data_ptr(), n, 1024 - 256, tokens) == -2
