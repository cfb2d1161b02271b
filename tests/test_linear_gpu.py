"""GPU parity: fused (RMSNorm ->) GEMV (+bias, +residual), standalone RMSNorm and the fused
gate/up + SiLU MLP, called through the C ABI, against the CPU oracle on identical seeded
inputs.  Gate: max relative error <= 1e-2 vs the high-precision oracle (fp16/bf16 outputs).

Shapes follow the benchmark configurations (4096->4096, 4096->6144 QKV, 4096->2x14336,
14336->4096) plus the ragged / tiny / strided cases the reference kernels special-case
(csrc/linear/linear_fp16_kernels.cu:227-320) and the batch-4 recipes of the reference's own
tests (tests/test_linear.py, tests/test_rmsnorm.py there)."""

import pytest
import torch

import oracle
from muillm_amd import _lib, muillm_ext
from tests.util import assert_parity, reference_allclose

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _gen(seed=0):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _mk(shape, g, std=1.0, mean=0.0, dtype=torch.float16):
    return (mean + std * torch.randn(shape, generator=g)).to(dtype)


@pytest.mark.parametrize(
    "n,k,norm,res,bias",
    [
        (4096, 4096, True, True, False),   # config 1
        (4096, 4096, False, False, False),
        (6144, 4096, True, False, False),  # fused QKV shape
        (4096, 14336, False, True, False),  # down projection
        (1024, 2048, True, True, True),
        (4097, 4096, True, True, True),    # N not a multiple of the row group
        (13, 4096, False, True, False),
        (1, 8, False, False, False),
        (5, 24, True, True, True),         # K smaller than one pass of the workgroup
        (64, 2056, True, False, False),    # K just above a 2048 boundary
        (32, 11008, True, True, False),
        (16, 16384, False, False, True),   # largest K of the register-resident path
        (128256 // 8, 4096, False, False, False),  # lm_head-like tall matrix (1/8 height)
    ],
)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_single_token(n, k, norm, res, bias, dtype):
    g = _gen(0)
    w = _mk((n, k), g, 0.02, dtype=dtype)
    x = _mk((1, k), g, dtype=dtype)
    gamma = _mk((k,), g, 0.1, 1.0, dtype=dtype) if norm else None
    r = _mk((1, n), g, dtype=dtype) if res else None
    b = _mk((n,), g, 0.5, dtype=dtype) if bias else None
    eps = 1e-5
    ref = oracle.linear(x, w, gamma, eps, b, r)
    y = muillm_ext.muillm_linear_forward(
        None, x.to(DEV), w.to(DEV), None if gamma is None else gamma.to(DEV), eps,
        None, None if b is None else b.to(DEV), None if r is None else r.to(DEV))
    assert y.shape == (1, n) and y.dtype == dtype
    # one gate for both 16-bit types (measured on MI355X: bf16 worst 3.9e-3 of max |ref|, 4.8e-3 on
    # the elementwise form); `tight` is a sanity bound in units of rms(ref), wider for bf16's 8 bits
    tight = 4e-3 if dtype == torch.float16 else 3e-2
    assert_parity(y, ref, 1e-2, f"linear {n}x{k}", tight=tight)


def test_linear_config1_reference_tolerance():
    """Config 1 exactly, also under the reference suite's own allclose(rtol 1e-4, atol 1e-1)."""
    torch.manual_seed(0)
    gamma = (1 + 0.1 * torch.randn(4096)).half()
    w = (0.02 * torch.randn(4096, 4096)).half()
    x = torch.randn(4096).half()
    res = torch.randn(4096).half()
    ref = oracle.linear(x, w, gamma, 1e-5, None, res)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), gamma.to(DEV), 1e-5, residual=res.to(DEV))
    assert y.shape == (4096,)
    assert_parity(y, ref, 1e-2, "config1", tight=3e-3)
    assert reference_allclose(y, ref)
    # the reference fallback executed literally in fp16 on CPU agrees as well
    ref16 = oracle.linear(x, w, gamma, 1e-5, None, res, reference_path=True)
    assert_parity(y, ref16, 1e-2, "config1 vs fp16 reference path")


def test_linear_closed_forms():
    k = 4096
    g = _gen(1)
    x = _mk((k,), g)
    eye = torch.eye(k, dtype=torch.float16)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), eye.to(DEV))
    assert torch.equal(y.cpu(), x)  # identity: exact
    ones = torch.ones(4, k, dtype=torch.float16)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), ones.to(DEV))
    s = x.double().sum()
    assert torch.allclose(y.cpu().double(), s.expand(4), rtol=2e-3, atol=2e-2)
    onehot = torch.zeros(8, k, dtype=torch.float16)
    idx = torch.tensor([0, 1, 7, 8, 255, 256, 2047, 4095])
    onehot[torch.arange(8), idx] = 1
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), onehot.to(DEV))
    assert torch.equal(y.cpu(), x[idx])  # gather: exact, catches any chunk mis-indexing
    # residual only: W = 0
    r = _mk((k,), g)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), torch.zeros(k, k, dtype=torch.float16, device=DEV), residual=r.to(DEV))
    assert torch.equal(y.cpu(), r)


def test_linear_norm_invariants():
    """Fused RMSNorm: scale invariance and the constant-row closed form."""
    k, n = 4096, 64
    g = _gen(2)
    w = _mk((n, k), g, 0.02)
    gamma = _mk((k,), g, 0.1, 1.0)
    x = _mk((k,), g)
    y1 = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), gamma.to(DEV), 0.0)
    y2 = muillm_ext.muillm_linear_forward(None, (x * 4).to(DEV), w.to(DEV), gamma.to(DEV), 0.0)
    assert torch.allclose(y1.float(), y2.float(), rtol=2e-3, atol=2e-3)
    # x = c * 1, gamma = 1, eps = 0  ->  xn = sign(c) * 1  ->  y = sign(c) * rowsum(W)
    xc = torch.full((k,), -3.0, dtype=torch.float16)
    y = muillm_ext.muillm_linear_forward(None, xc.to(DEV), w.to(DEV), torch.ones(k, dtype=torch.float16, device=DEV), 0.0)
    assert torch.allclose(y.cpu().double(), -w.double().sum(1), rtol=2e-3, atol=2e-3)


def test_linear_strided_weights():
    """Rows with a pitch larger than K (a view into a wider buffer)."""
    g = _gen(3)
    n, k = 96, 4096
    big = _mk((n, 2, k), g, 0.02)
    x = _mk((k,), g)
    bigd = big.to(DEV)
    for s in range(2):
        y = muillm_ext.muillm_linear_forward(None, x.to(DEV), bigd[:, s, :])
        assert_parity(y, oracle.linear(x, big[:, s, :]), 1e-2, f"strided {s}", tight=4e-3)


@pytest.mark.parametrize("tokens", [2, 3, 4, 5, 8, 13, 16])
@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 14336), (100, 512), (8208, 5120)])
def test_linear_small_batch(tokens, n, k):
    g = _gen(4)
    w = _mk((n, k), g, 0.02)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    r = _mk((tokens, n), g)
    ref = oracle.linear(x, w, gamma, 1e-5, None, r)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), gamma.to(DEV), 1e-5, residual=r.to(DEV))
    assert y.shape == (tokens, n)
    assert_parity(y, ref, 1e-2, f"batch {tokens} {n}x{k}", tight=4e-3)


@pytest.mark.parametrize("tokens", [5, 9, 16])
@pytest.mark.parametrize("n,k", [(24, 256), (33, 3840), (64, 4104), (40, 8192), (17, 14336), (130, 2056), (9, 24)])
@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_small_batch_edge_shapes(tokens, n, k, norm, dtype):
    """The matrix-core path at its seams: K below / at / above what a workgroup keeps stationary
    (4096), K that is not a multiple of the 256-value pass, rows that do not fill a 16-row tile,
    fused norm on long rows (the streaming mode applies gamma on the way to LDS and gathers
    sum(x^2) during its first tile), with residual and both biases."""
    g = _gen(40 + tokens)
    w = _mk((n, k), g, 0.02, dtype=dtype)
    x = _mk((tokens, k), g, dtype=dtype)
    gamma = _mk((k,), g, 0.1, 1.0, dtype=dtype) if norm else None
    r = _mk((tokens, n), g, dtype=dtype)
    mb = _mk((n,), g, 0.1, 1.0, dtype=dtype)
    ab = _mk((n,), g, 0.1, dtype=dtype)
    ref = oracle.linear(x, w, gamma, 1e-5, ab, r, mul_bias=mb)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), None if gamma is None else gamma.to(DEV),
                                         1e-5, mul_bias=mb.to(DEV), add_bias=ab.to(DEV), residual=r.to(DEV))
    assert y.shape == (tokens, n) and y.dtype == dtype
    assert_parity(y, ref, 1e-2, f"edge {tokens} {n}x{k} norm={norm} {dtype}")


@pytest.mark.parametrize("tokens", [5, 16])
@pytest.mark.parametrize("n,k", [(40, 256), (100, 3840), (24, 8192), (9, 2056), (4100, 5120)])
@pytest.mark.parametrize("norm", [True, False])
def test_gateup_small_batch_edge_shapes(tokens, n, k, norm):
    g = _gen(60 + tokens)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0) if norm else None
    ref = oracle.gateup_silu(x, wg, wu, gamma, 1e-5)
    packed = torch.stack((wg, wu), dim=1).to(DEV)
    h = muillm_ext.mui_gateup_silu(None if gamma is None else gamma.to(DEV), 1e-5, packed[:, 0], packed[:, 1], x.to(DEV))
    assert h.shape == (tokens, n)
    assert_parity(h, ref, 1e-2, f"gate/up edge {tokens} {n}x{k} norm={norm}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,n", [(17, 64), (300, 14336), (5, 8)])
def test_silu_mul_interleaved(rows, n, dtype):
    g = _gen(70)
    gu = _mk((rows, 2 * n), g, dtype=dtype)
    ref = torch.nn.functional.silu(gu[:, 0::2].double()) * gu[:, 1::2].double()
    out = muillm_ext.mui_silu_mul_interleaved(gu.to(DEV))
    assert out.shape == (rows, n) and out.dtype == dtype
    assert_parity(out, ref.float(), 1e-2, f"silu*mul {rows}x{n}")


@pytest.mark.parametrize("tokens", [1, 3, 8])
@pytest.mark.parametrize("k", [28672, 16392])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_rows_longer_than_one_pass(tokens, k, dtype):
    """Down projections of 70B-class models (K = 28672): up to 4 tokens go through K segments that
    accumulate through the residual operand, more tokens through the streaming matrix-core kernel."""
    g = _gen(80 + tokens)
    n = 72
    w = _mk((n, k), g, 0.02, dtype=dtype)
    x = _mk((tokens, k), g, dtype=dtype)
    r = _mk((tokens, n), g, dtype=dtype)
    mb = _mk((n,), g, 0.1, 1.0, dtype=dtype)
    ab = _mk((n,), g, 0.1, dtype=dtype)
    ref = oracle.linear(x, w, None, 0.0, ab, r, mul_bias=mb)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), mul_bias=mb.to(DEV), add_bias=ab.to(DEV),
                                         residual=r.to(DEV))
    assert y.shape == (tokens, n) and y.dtype == dtype
    assert_parity(y, ref, 1e-2, f"long rows {tokens} x {k} {dtype}")


def test_linear_reference_recipe_batch4():
    """tests/test_linear.py:13-43 of the reference: randn weights (seed 0), rand inputs of
    batch 4, compared with allclose(rtol 1e-4, atol 1e-1)."""
    torch.manual_seed(0)
    lin = torch.nn.Linear(2048, 1024, bias=True).half()
    lin.weight.data = torch.randn(1024, 2048).half() * 0.05
    x = torch.rand(4, 2048).half()
    ref = oracle.linear(x, lin.weight.data, bias=lin.bias.data)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), lin.weight.data.to(DEV), add_bias=lin.bias.data.to(DEV))
    assert reference_allclose(y, ref)
    assert_parity(y, ref, 1e-2, "recipe batch4")


def test_linear_abi_errors():
    lib = _lib.load()
    w = torch.zeros(8, 16, dtype=torch.float16, device=DEV)
    x = torch.zeros(16, dtype=torch.float16, device=DEV)
    y = torch.zeros(8, dtype=torch.float16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.mui_linear(s, 0, None, 16, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), 8, 16, 1) == -1
    assert lib.mui_linear(s, 7, w.data_ptr(), 16, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), 8, 16, 1) == -1
    assert lib.mui_linear(s, 0, w.data_ptr(), 12, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), 8, 12, 1) == -2
    assert lib.mui_linear(s, 0, w.data_ptr(), 16, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), 8, 16, 0) == -1
    assert lib.mui_linear(s, 0, w.data_ptr() + 2, 16, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(), 4, 8, 1) == -4
    assert b"aligned" in lib.mui_status_string(-4)
    with pytest.raises(RuntimeError):
        muillm_ext.muillm_linear_forward(None, x, torch.zeros(8, 24, dtype=torch.float16, device=DEV))
    # K % 8 != 0 and fp32 inputs take the unfused route and still compute the right thing
    w12 = torch.randn(8, 12, device=DEV).half()
    x12 = torch.randn(12, device=DEV).half()
    y12 = muillm_ext.muillm_linear_forward(None, x12, w12)
    assert_parity(y12, oracle.linear(x12.cpu(), w12.cpu()), 1e-2, "K=12 unfused")


# ------------------------------------------------------------------------------------
# RMSNorm
# ------------------------------------------------------------------------------------
@pytest.mark.parametrize("rows,k", [(4, 256), (1, 4096), (32, 4096), (8, 14336), (3, 100), (2, 7), (5, 2056), (1, 16384)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rmsnorm(rows, k, dtype):
    g = _gen(5)
    x = _mk((rows, k), g, dtype=dtype)
    w = _mk((k,), g, 0.1, 1.0, dtype=dtype)
    for eps in (1e-5, 1e-6):
        y = muillm_ext.muillm_rmsnorm_forward(w.to(DEV), x.to(DEV), eps)
        assert y.shape == x.shape and y.dtype == dtype
        assert_parity(y, oracle.rmsnorm(x, w, eps), 1e-2, f"rmsnorm {rows}x{k}",
                      tight=2e-3 if dtype == torch.float16 else 2e-2)


def test_rmsnorm_closed_forms():
    k = 4096
    ones = torch.ones(k, dtype=torch.float16)
    xc = torch.full((2, k), 5.0, dtype=torch.float16)
    xc[1] = -0.25
    y = muillm_ext.muillm_rmsnorm_forward(ones.to(DEV), xc.to(DEV), 0.0).cpu()
    assert torch.equal(y[0], ones) and torch.equal(y[1], -ones)  # x = c*1 -> sign(c)
    g = _gen(6)
    x = _mk((3, k), g)
    y = muillm_ext.muillm_rmsnorm_forward(ones.to(DEV), x.to(DEV), 0.0).cpu().double()
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(3, dtype=torch.float64), rtol=2e-3)
    y2 = muillm_ext.muillm_rmsnorm_forward(ones.to(DEV), (x * 8).to(DEV), 0.0).cpu().double()
    assert torch.allclose(y, y2, rtol=1e-3, atol=1e-3)  # scale invariance


# ------------------------------------------------------------------------------------
# gate/up + SiLU and the whole MLP
# ------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,k", [(14336, 4096), (11008, 4096), (257, 512), (3, 8), (64, 2056)])
@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("packed", [True, False])
def test_gateup_silu(n, k, norm, packed):
    g = _gen(7)
    wg = _mk((n, k), g, 0.02)
    wu = _mk((n, k), g, 0.02)
    x = _mk((1, k), g)
    gamma = _mk((k,), g, 0.1, 1.0) if norm else None
    ref = oracle.gateup_silu(x, wg, wu, gamma, 1e-5)
    if packed:
        gu = torch.stack([wg, wu], dim=1).to(DEV)  # [N, 2, K]: gate row n then up row n
        dg, du = gu[:, 0, :], gu[:, 1, :]
    else:
        dg, du = wg.to(DEV), wu.to(DEV)
    h = muillm_ext.mui_gateup_silu(None if gamma is None else gamma.to(DEV), 1e-5, dg, du, x.to(DEV))
    assert h.shape == (1, n)
    assert_parity(h, ref, 1e-2, f"gateup {n}x{k}", tight=6e-3)


@pytest.mark.parametrize("tokens", [1, 2, 4, 8, 16])
def test_mlp_config2(tokens):
    """Config 2: Mistral-7B-shaped MLP with fused norm and residual."""
    g = _gen(8)
    hid, inter = 4096, 14336
    wg = _mk((inter, hid), g, 0.02)
    wu = _mk((inter, hid), g, 0.02)
    wd = _mk((hid, inter), g, 0.02)
    gamma = _mk((hid,), g, 0.1, 1.0)
    x = _mk((tokens, hid), g)
    r = _mk((tokens, hid), g)
    ref = oracle.gateupdown_mlp(x, wg, wu, wd, gamma, 1e-5, r)
    out = muillm_ext.muillm_gateupsilu_forward(None, gamma.to(DEV), 1e-5, wg.to(DEV), wu.to(DEV), wd.to(DEV), r.to(DEV), x.to(DEV))
    assert out.shape == (tokens, hid)
    assert_parity(out, ref, 1e-2, f"mlp b={tokens}", tight=5e-3)
    ref_rounded = oracle.gateupdown_mlp(x, wg, wu, wd, gamma, 1e-5, r, round_intermediate=torch.float16)
    assert_parity(out, ref_rounded, 1e-2, f"mlp b={tokens} (rounded intermediate)", tight=3e-3)


def test_mlp_closed_forms():
    g = _gen(9)
    hid, inter = 512, 1024
    wd = _mk((hid, inter), g, 0.02).to(DEV)
    w = _mk((inter, hid), g, 0.02).to(DEV)
    z = torch.zeros(inter, hid, dtype=torch.float16, device=DEV)
    x = _mk((1, hid), g).to(DEV)
    r = _mk((1, hid), g).to(DEV)
    # Wg = 0 -> silu(0) = 0 -> out = residual ; Wu = 0 -> out = residual
    assert torch.equal(muillm_ext.muillm_gateupsilu_forward(None, None, 0.0, z, w, wd, r, x), r)
    assert torch.equal(muillm_ext.muillm_gateupsilu_forward(None, None, 0.0, w, z, wd, r, x), r)


def test_lm_head_full_size_gather_property():
    """At the full lm_head size (128256 x 4096, 1.05 GB) the oracle is too slow; a one-hot input
    turns the GEMV into a column gather, which must be bit-exact, and linearity ties a random
    input to two such runs (size-independent properties)."""
    from muillm_amd import muillm_ext
    g = torch.Generator(device="cuda").manual_seed(0)
    n, k = 128256, 4096
    w = torch.randn(n, k, device="cuda", dtype=torch.float16, generator=g) * 0.02
    for j in (0, 1, 2047, 4095):
        x = torch.zeros(1, k, device="cuda", dtype=torch.float16)
        x[0, j] = 1.0
        y = muillm_ext.muillm_linear_forward(None, x, w)
        assert torch.equal(y[0], w[:, j])
    # rows of ones -> sum of the inputs, for every one of the 128256 outputs
    w1 = torch.ones(n, 64, device="cuda", dtype=torch.float16)
    x = torch.randn(1, 64, device="cuda", dtype=torch.float16, generator=g)
    y = muillm_ext.muillm_linear_forward(None, x, w1)
    want = x.float().sum()
    assert float((y.float() - want).abs().max()) <= 2e-3 * max(1.0, abs(float(want)))
    # a random input against torch's fp32 matmul on a strided sample of rows
    x = torch.randn(1, k, device="cuda", dtype=torch.float16, generator=g)
    y = muillm_ext.muillm_linear_forward(None, x, w)
    rows = torch.arange(0, n, 257, device="cuda")
    ref = (w[rows].float() @ x[0].float())
    assert float((y[0, rows].float() - ref).abs().max()) <= 1e-2 * float(ref.abs().max())


def test_read_probe_reads_and_discards():
    """The read probe leaves source and sink untouched (the sink is written only when the XOR of
    everything a lane read equals a fixed pattern), covers sizes that are not a multiple of its
    chunk, and rejects misaligned requests."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    sink = torch.zeros(64, dtype=torch.int32, device=DEV)
    for nbytes in (16, 4096 * 8 + 48, 33554432):
        src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=DEV)
        keep = src.clone()
        assert lib.mui_probe_read(stream, src.data_ptr(), nbytes, sink.data_ptr()) == 0
        torch.cuda.synchronize()
        assert torch.equal(src, keep) and int(sink.abs().sum()) == 0
    assert lib.mui_probe_read(stream, src.data_ptr() + 8, 64, sink.data_ptr()) != 0
    assert lib.mui_probe_read(stream, src.data_ptr(), 24, sink.data_ptr()) != 0
    assert lib.mui_probe_read(stream, None, 64, sink.data_ptr()) != 0


@pytest.mark.parametrize("chunk_max", [16, 32])
@pytest.mark.parametrize("tokens", [17, 32])
def test_short_prompt_on_the_library_kernels(tokens, chunk_max, monkeypatch):
    """17..32 tokens: the tiled GEMM in one call (the default: FUSED_CHUNK_MAX_TOKENS = MUI_MAX_TOKENS),
    or two calls of the 16-token kernels when the chunk limit is raised -- never norm + library GEMM + add."""
    assert muillm_ext.FUSED_CHUNK_MAX_TOKENS == 16
    monkeypatch.setattr(muillm_ext, "FUSED_CHUNK_MAX_TOKENS", chunk_max)
    g = _gen(90 + tokens)
    n, k = 520, 1024
    w = _mk((n, k), g, 0.02)
    x = _mk((2, tokens // 2 if tokens % 2 == 0 else 1, k), g) if tokens % 2 == 0 else _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    r = _mk(tuple(x.shape[:-1]) + (n,), g)
    assert muillm_ext.kernel_dispatchable(x.to(DEV))
    ref = oracle.linear(x, w, gamma, 1e-5, None, r)
    y = muillm_ext.muillm_linear_forward(None, x.to(DEV), w.to(DEV), gamma.to(DEV), 1e-5, residual=r.to(DEV))
    assert y.shape == r.shape
    assert_parity(y, ref, 1e-2, f"chunked linear {tokens}", tight=4e-3)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    packed = torch.stack((wg, wu), dim=1).to(DEV)
    h = muillm_ext.mui_gateup_silu(gamma.to(DEV), 1e-5, packed[:, 0], packed[:, 1], x.to(DEV))
    assert_parity(h, oracle.gateup_silu(x, wg, wu, gamma, 1e-5), 1e-2, f"chunked gate/up {tokens}")
    # longer prompts stay on the library's kernels too (the tiled GEMM of the same entry points)
    assert muillm_ext.kernel_dispatchable(torch.zeros(33, k, dtype=torch.float16, device=DEV))
    assert muillm_ext._token_calls(32, 32) == [(0, 16), (16, 16)] and muillm_ext._token_calls(33, 32) == [(0, 33)]
    assert not muillm_ext.kernel_dispatchable(torch.zeros(33, k, dtype=torch.float32, device=DEV))
