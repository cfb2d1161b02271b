"""GPU parity of the int8 weight-only path (config 3): symmetric per-output-channel int8 with
fp16 scales on the Llama-3-8B decode GEMV shapes, plus the reference's own asymmetric
group-wise uint8 RTN format.  Dequantised weights must be bit-exact; GEMV outputs within
1e-2 relative of the high-precision oracle on the dequantised matrix."""

import pytest
import torch

import oracle
from muillm_amd import _lib, muillm_ext
from tests.util import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _gen(seed=0):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _mk(shape, g, std=1.0, mean=0.0, dtype=torch.float16):
    return (mean + std * torch.randn(shape, generator=g)).to(dtype)


SHAPES = [
    (6144, 4096),    # fused QKV
    (4096, 4096),    # o_proj
    (4096, 14336),   # down
    (1000, 2048),
    (7, 16),
    (33, 4112),      # K just above one pass of the workgroup
    (12, 8192),
]


@pytest.mark.parametrize("n,k", SHAPES)
def test_channel_dequant_bit_exact(n, k):
    g = _gen(0)
    w = _mk((n, k), g, 0.02)
    w[0] = 0  # all-zero row
    if n > 2:
        w[1] = w[1] * 1e-4  # tiny scale (fp16 subnormal products)
    q, s = oracle.rtn_quantize_channel(w)
    ref = oracle.rtn_dequantize_channel(q, s)
    assert torch.equal(ref, q.to(torch.float16) * s[:, None])  # the oracle's own closed form
    dq = muillm_ext.mui_int8_channel_dequantize_forward(q.to(DEV), s.to(DEV))
    assert dq.dtype == torch.float16
    assert torch.equal(dq.cpu().view(torch.int16), ref.view(torch.int16)), "dequantised weights are not bit-exact"


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("tokens", [1, 2, 4, 7, 16])
@pytest.mark.parametrize("norm", [True, False])
def test_channel_linear(n, k, tokens, norm):
    g = _gen(1)
    w = _mk((n, k), g, 0.02)
    q, s = oracle.rtn_quantize_channel(w)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0) if norm else None
    r = _mk((tokens, n), g)
    ref = oracle.int8_channel_linear(x, q, s, gamma, 1e-5, None, r)
    y = muillm_ext.mui_int8_channel_linear_forward(
        x.to(DEV), q.to(DEV), s.to(DEV), None if gamma is None else gamma.to(DEV), 1e-5, None, r.to(DEV))
    assert y.shape == (tokens, n)
    assert_parity(y, ref, 1e-2, f"int8 channel {n}x{k} b={tokens}", tight=4e-3)
    # and it tracks the unquantised fp16 layer to quantisation accuracy
    full = oracle.linear(x, w, gamma, 1e-5, None, r)
    assert oracle.rel_err(y.cpu(), full) < 3e-2


@pytest.mark.parametrize("tokens", [1, 3, 8])
@pytest.mark.parametrize("k", [28672, 16400])
def test_channel_linear_rows_longer_than_one_pass(tokens, k):
    """K = 28672 (down projection of a 70B-class model): K segments accumulating through the
    residual operand at up to 4 tokens, the streaming matrix-core kernel beyond."""
    g = _gen(11)
    n = 40
    w = _mk((n, k), g, 0.02)
    q, s = oracle.rtn_quantize_channel(w)
    x = _mk((tokens, k), g)
    r = _mk((tokens, n), g)
    ref = oracle.int8_channel_linear(x, q, s, None, 0.0, None, r)
    y = muillm_ext.mui_int8_channel_linear_forward(x.to(DEV), q.to(DEV), s.to(DEV), None, 0.0, None, r.to(DEV))
    assert_parity(y, ref, 1e-2, f"int8 long rows {tokens} x {k}", tight=4e-3)


@pytest.mark.parametrize("n,k", [(14336, 4096), (300, 1024), (5, 16)])
@pytest.mark.parametrize("tokens", [1, 2, 4, 7, 16])
@pytest.mark.parametrize("packed", [True, False])
def test_channel_gateup(n, k, tokens, packed):
    g = _gen(2)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    qg, sg = oracle.rtn_quantize_channel(wg)
    qu, su = oracle.rtn_quantize_channel(wu)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    ref = oracle.gateup_silu(x, oracle.rtn_dequantize_channel(qg, sg), oracle.rtn_dequantize_channel(qu, su), gamma, 1e-5)
    if packed:
        qq = torch.stack([qg, qu], dim=1).to(DEV)
        ss = torch.stack([sg, su], dim=1).to(DEV)
        a = (qq[:, 0], qq[:, 1], ss[:, 0], ss[:, 1])
    else:
        a = (qg.to(DEV), qu.to(DEV), sg.to(DEV), su.to(DEV))
    h = muillm_ext.mui_int8_channel_gateupsilu_forward(gamma.to(DEV), 1e-5, a[0], a[1], a[2], a[3], x.to(DEV))
    assert_parity(h, ref, 1e-2, f"int8 gateup {n}x{k}", tight=9e-3)  # activations enter the packed dot rounded to fp16


def test_channel_closed_forms():
    k = 4096
    g = _gen(3)
    x = _mk((k,), g)
    # q = 127 * I, s = 1/127 (exactly representable? no: use s = 2^-7 and q = 64 -> w = 0.5)
    q = torch.zeros(k, k, dtype=torch.int8)
    q[torch.arange(k), torch.arange(k)] = 64
    s = torch.full((k,), 2.0 ** -7, dtype=torch.float16)
    y = muillm_ext.mui_int8_channel_linear_forward(x.to(DEV), q.to(DEV), s.to(DEV))
    assert torch.allclose(y.cpu().float(), 0.5 * x.float(), rtol=1e-3, atol=1e-3)
    # extreme codes: all -127 / +127 rows
    q2 = torch.full((4, k), -127, dtype=torch.int8)
    q2[1] = 127
    q2[2, ::2] = 127
    s2 = torch.full((4,), 2.0 ** -10, dtype=torch.float16)
    ref = oracle.int8_channel_linear(x, q2, s2)
    y = muillm_ext.mui_int8_channel_linear_forward(x.to(DEV), q2.to(DEV), s2.to(DEV))
    assert torch.allclose(y.cpu().double(), ref, rtol=2e-3, atol=2e-2)


# ------------------------------------------------------------------------------------
# the reference's group-wise uint8 format
# ------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,k,gs", [(4096, 4096, 128), (4096, 14336, 2048), (6144, 4096, 32), (50, 256, 16), (9, 4096, 4096)])
def test_group_dequant_bit_exact(n, k, gs):
    g = _gen(4)
    w = _mk((n, k), g, 0.02)
    q, smv = oracle.rtn_quantize_group(w, gs)
    shift = gs.bit_length() - 1
    ref = oracle.rtn_dequantize_group(q, smv, gs, torch.float16, kernel_form=True)
    dq = muillm_ext.muillm_int8_dequantize_forward(q.to(DEV), smv.to(DEV), shift)
    assert torch.equal(dq.cpu().view(torch.int16), ref.view(torch.int16))
    # the reference's Python fallback rounds twice; it may differ from the kernel form by an ulp
    ref_py = oracle.rtn_dequantize_group(q, smv, gs, torch.float16, kernel_form=False)
    assert (dq.cpu().float() - ref_py.float()).abs().max() <= 2 * smv[:, 0].float().max()


@pytest.mark.parametrize("n,k,gs", [(4096, 4096, 128), (4096, 14336, 1024), (6144, 4096, 64), (50, 256, 16)])
@pytest.mark.parametrize("tokens", [1, 2, 4, 7, 16])
def test_group_linear(n, k, gs, tokens):
    g = _gen(5)
    w = _mk((n, k), g, 0.02)
    q, smv = oracle.rtn_quantize_group(w, gs)
    shift = gs.bit_length() - 1
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    r = _mk((tokens, n), g)
    ref = oracle.int8_group_linear(x, q, smv, gs, gamma, 1e-5, None, r)
    y = muillm_ext.muillm_int8_linear_forward(x.to(DEV), q.to(DEV), smv.to(DEV), shift, gamma.to(DEV), 1e-5,
                                              None, None, r.to(DEV))
    assert_parity(y, ref, 1e-2, f"int8 group {n}x{k} gs={gs}", tight=4e-3)
    assert oracle.rel_err(y.cpu(), oracle.linear(x, w, gamma, 1e-5, None, r)) < 3e-2


@pytest.mark.parametrize("matrix_cores", [False, True])
@pytest.mark.parametrize("n,k,gs", [(4096, 14336, 128), (64, 4224, 128), (40, 8448, 256), (33, 4096, 128), (4096, 4096, 4096)])
@pytest.mark.parametrize("tokens", [3, 4, 8, 16])
def test_group_linear_long_rows_and_group_accumulation(n, k, gs, tokens, matrix_cores):
    """Groups of 128 codes and more on the matrix-core kernel (its default from 5 tokens; forced here
    from 3): rows streamed in passes (K = 14336), a last pass that ends inside the row (K = 4224,
    8448), rows that do not fill a 16-row tile, one group per row -- the per-group accumulation
    must give what the oracle's dequantise-then-multiply gives."""
    lib = _lib.load()
    if matrix_cores:
        _lib.check(lib.mui_tune_skinny(2, 0, 1), "mui_tune_skinny")
    try:
        g = _gen(25)
        w = _mk((n, k), g, 0.02)
        q, smv = oracle.rtn_quantize_group(w, gs)
        shift = gs.bit_length() - 1
        x = _mk((tokens, k), g)
        gamma = _mk((k,), g, 0.1, 1.0) if k <= 4224 else None
        r = _mk((tokens, n), g)
        ref = oracle.int8_group_linear(x, q, smv, gs, gamma, 1e-5, None, r)
        y = muillm_ext.muillm_int8_linear_forward(x.to(DEV), q.to(DEV), smv.to(DEV), shift,
                                                  None if gamma is None else gamma.to(DEV), 1e-5, None, None, r.to(DEV))
        assert_parity(y, ref, 1e-2, f"int8 group {n}x{k} gs={gs} b={tokens} mfma={matrix_cores}", tight=4e-3)
    finally:
        _lib.check(lib.mui_tune_skinny(2, 0, 0), "mui_tune_skinny")


@pytest.mark.parametrize("n,k,gs", [(14336, 4096, 128), (300, 1024, 64), (5, 64, 16)])
@pytest.mark.parametrize("tokens", [2, 3, 4, 8])
def test_group_gateup_small_batches(n, k, gs, tokens):
    g = _gen(16)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    qg, smg = oracle.rtn_quantize_group(wg, gs)
    qu, smu = oracle.rtn_quantize_group(wu, gs)
    shift = gs.bit_length() - 1
    ng = k // gs
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    wgd = (qg.reshape(-1, gs).double() * smg[:, None, 0].double() + smg[:, None, 1].double()).reshape(n, k)
    wud = (qu.reshape(-1, gs).double() * smu[:, None, 0].double() + smu[:, None, 1].double()).reshape(n, k)
    ref = oracle.gateup_silu(x, wgd, wud, gamma, 1e-5)
    packed_w = torch.stack([qg, qu], dim=1).to(DEV)
    packed_s = torch.stack([smg.reshape(n, ng, 2), smu.reshape(n, ng, 2)], dim=1).to(DEV)
    h = muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, packed_w, packed_s, shift, x.to(DEV))
    assert h.shape == (tokens, n)
    assert_parity(h, ref, 1e-2, f"int8 group gateup {n}x{k} b={tokens}", tight=9e-3)


QUAD_SHAPES = [
    # (n, k): one case per (waves, segments-per-wave) instance of the 4 x 4 x 4 kernel and its tails
    (6144, 4096),   # 4 waves x 4 segments, two row groups per workgroup
    (4096, 14336),  # 8 x 7
    (1030, 1024),   # 4 x 1, n not a multiple of 4
    (515, 2032),    # 4 x 2, last segment ends inside the row
    (64, 4112),     # 8 x 4, one block past 4096
    (9, 8192),      # 8 x 4 full
    (3, 16),        # a single block
    (10000, 512),   # many groups per workgroup: the loop over pairs of register sets
]


@pytest.mark.parametrize("sets", [0, 1, 2])
@pytest.mark.parametrize("n,k", QUAD_SHAPES)
@pytest.mark.parametrize("tokens", [1, 2, 3, 4])
def test_quad_kernel_channel_linear(n, k, tokens, sets):
    """Per-channel int8 at 1..4 tokens on the 4 x 4 x 4 matrix-instruction kernel (forced from one
    token; its default starts at two), with the launcher's choice of register sets, with one and with two, with and without the
    fused norm, bias and residual -- against the oracle, and against the older kernels' output."""
    lib = _lib.load()
    g = _gen(31)
    w = _mk((n, k), g, 0.02)
    q, s = oracle.rtn_quantize_channel(w)
    x = _mk((tokens, k), g)
    r = _mk((tokens, n), g)
    bias = _mk((n,), g, 0.1)
    for norm, use_bias, use_res in [(True, False, True), (False, True, False), (True, True, True)]:
        gamma = _mk((k,), g, 0.1, 1.0) if norm else None
        ref = oracle.int8_channel_linear(x, q, s, gamma, 1e-5, bias if use_bias else None, r if use_res else None)
        args = (x.to(DEV), q.to(DEV), s.to(DEV), None if gamma is None else gamma.to(DEV), 1e-5,
                bias.to(DEV) if use_bias else None, r.to(DEV) if use_res else None)
        _lib.check(lib.mui_tune_int8_quad(1, 1, 0, sets), "mui_tune_int8_quad")
        try:
            y = muillm_ext.mui_int8_channel_linear_forward(*args)
            _lib.check(lib.mui_tune_int8_quad(0, 0, 0, 0), "mui_tune_int8_quad")
            y_old = muillm_ext.mui_int8_channel_linear_forward(*args)
        finally:
            _lib.check(lib.mui_tune_int8_quad(1, 0, 0, 0), "mui_tune_int8_quad")
        what = f"int8 channel quad {n}x{k} b={tokens} sets={sets} norm={norm} bias={use_bias} res={use_res}"
        assert_parity(y, ref, 1e-2, what, tight=4e-3)
        assert_parity(y, y_old.float().cpu(), 1e-2, what + " vs older kernels", tight=4e-3)


@pytest.mark.parametrize("n,k,gs", [(6144, 4096, 128), (4096, 14336, 128), (515, 2032, 16), (64, 4224, 64),
                                    (33, 4096, 4096), (10000, 512, 32)])
@pytest.mark.parametrize("tokens", [1, 2, 3, 4])
def test_quad_kernel_group_linear(n, k, gs, tokens):
    """The reference's group format on the same kernel: (scale, min) folded in once per lane and
    256-code segment on separately accumulated products."""
    lib = _lib.load()
    g = _gen(32)
    w = _mk((n, k), g, 0.02)
    q, smv = oracle.rtn_quantize_group(w, gs)
    shift = gs.bit_length() - 1
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    r = _mk((tokens, n), g)
    ref = oracle.int8_group_linear(x, q, smv, gs, gamma, 1e-5, None, r)
    _lib.check(lib.mui_tune_int8_quad(1, 1, 0, 0), "mui_tune_int8_quad")
    try:
        y = muillm_ext.muillm_int8_linear_forward(x.to(DEV), q.to(DEV), smv.to(DEV), shift, gamma.to(DEV), 1e-5,
                                                  None, None, r.to(DEV))
    finally:
        _lib.check(lib.mui_tune_int8_quad(1, 0, 0, 0), "mui_tune_int8_quad")
    assert_parity(y, ref, 1e-2, f"int8 group quad {n}x{k} gs={gs} b={tokens}", tight=4e-3)


@pytest.mark.parametrize("fmt", ["channel", "group"])
@pytest.mark.parametrize("n,k", [(14336, 4096), (301, 1024), (5, 272), (2000, 8192)])
@pytest.mark.parametrize("tokens", [1, 2, 3, 4])
def test_quad_kernel_gateup(n, k, tokens, fmt):
    lib = _lib.load()
    g = _gen(33)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    _lib.check(lib.mui_tune_int8_quad(1, 1, 0, 0), "mui_tune_int8_quad")
    try:
        if fmt == "channel":
            qg, sg = oracle.rtn_quantize_channel(wg)
            qu, su = oracle.rtn_quantize_channel(wu)
            ref = oracle.gateup_silu(x, oracle.rtn_dequantize_channel(qg, sg), oracle.rtn_dequantize_channel(qu, su), gamma, 1e-5)
            h = muillm_ext.mui_int8_channel_gateupsilu_forward(gamma.to(DEV), 1e-5, qg.to(DEV), qu.to(DEV), sg.to(DEV),
                                                               su.to(DEV), x.to(DEV))
        else:
            gs = 16 if k % 128 else 128
            qg, smg = oracle.rtn_quantize_group(wg, gs)
            qu, smu = oracle.rtn_quantize_group(wu, gs)
            ng = k // gs
            wgd = (qg.reshape(-1, gs).double() * smg[:, None, 0].double() + smg[:, None, 1].double()).reshape(n, k)
            wud = (qu.reshape(-1, gs).double() * smu[:, None, 0].double() + smu[:, None, 1].double()).reshape(n, k)
            ref = oracle.gateup_silu(x, wgd, wud, gamma, 1e-5)
            packed_w = torch.stack([qg, qu], dim=1).to(DEV)
            packed_s = torch.stack([smg.reshape(n, ng, 2), smu.reshape(n, ng, 2)], dim=1).to(DEV)
            h = muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, packed_w, packed_s, gs.bit_length() - 1,
                                                          x.to(DEV))
    finally:
        _lib.check(lib.mui_tune_int8_quad(1, 0, 0, 0), "mui_tune_int8_quad")
    assert h.shape == (tokens, n)
    assert_parity(h, ref, 1e-2, f"int8 {fmt} gateup quad {n}x{k} b={tokens}", tight=9e-3)


@pytest.mark.parametrize("n,k,gs", [(14336, 4096, 128), (100, 512, 32)])
def test_group_gateup(n, k, gs):
    g = _gen(6)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    qg, smg = oracle.rtn_quantize_group(wg, gs)
    qu, smu = oracle.rtn_quantize_group(wu, gs)
    shift = gs.bit_length() - 1
    ng = k // gs
    x = _mk((1, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    wgd = (qg.reshape(-1, gs).double() * smg[:, None, 0].double() + smg[:, None, 1].double()).reshape(n, k)
    wud = (qu.reshape(-1, gs).double() * smu[:, None, 0].double() + smu[:, None, 1].double()).reshape(n, k)
    ref = oracle.gateup_silu(x, wgd, wud, gamma, 1e-5)
    packed_w = torch.stack([qg, qu], dim=1).to(DEV)                                   # [N, 2, K]
    packed_s = torch.stack([smg.reshape(n, ng, 2), smu.reshape(n, ng, 2)], dim=1).to(DEV)  # [N, 2, G, 2]
    h = muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, packed_w, packed_s, shift, x.to(DEV))
    assert_parity(h, ref, 1e-2, f"int8 group gateup {n}x{k}", tight=9e-3)
    dg, du = muillm_ext.muillm_int8_gateupsilu_dequantize_forward(packed_w, packed_s, shift)
    assert torch.equal(dg.cpu(), oracle.rtn_dequantize_group(qg, smg, gs))
    assert torch.equal(du.cpu(), oracle.rtn_dequantize_group(qu, smu, gs))
    # the reference's own packing (muillm/modules/quantized/int8gateupdownmlp.py:211-230: codes
    # concatenated on a new last axis, (scale, min) rows on a new middle axis) gives the same bits
    ref_w = torch.cat([qg[:, :, None], qu[:, :, None]], dim=2).to(DEV)               # [N, K, 2]
    ref_s = torch.cat([smg[:, None, :], smu[:, None, :]], dim=1).to(DEV)             # [N*G, 2, 2]
    assert ref_w.shape == (n, k, 2) and ref_s.shape == (n * ng, 2, 2)
    h_ref = muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, ref_w, ref_s, shift, x.to(DEV))
    assert torch.equal(h_ref, h)
    rg, ru = muillm_ext.muillm_int8_gateupsilu_dequantize_forward(ref_w, ref_s, shift)
    assert torch.equal(rg, dg) and torch.equal(ru, du)
    # converted once: a second call finds the row-interleaved twin; an in-place edit of the source drops it
    twins = len(muillm_ext._REPACKED_GATEUP)
    muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, ref_w, ref_s, shift, x.to(DEV))
    assert len(muillm_ext._REPACKED_GATEUP) == twins
    ref_w[0, 0, 0] += 1
    h_edit = muillm_ext.muillm_int8_gateupsilu_forward(gamma.to(DEV), 1e-5, ref_w, ref_s, shift, x.to(DEV))
    assert len(muillm_ext._REPACKED_GATEUP) == twins + 1 and not torch.equal(h_edit[..., 0], h[..., 0])
    # the conversion itself, through the C ABI, against torch's permute
    lib = _lib.load()
    out_w = torch.empty((n, 2, k), dtype=torch.uint8, device=DEV)
    out_s = torch.empty((n, 2, ng, 2), dtype=torch.float16, device=DEV)
    st = lib.mui_int8_repack_gateup(torch.cuda.current_stream().cuda_stream, ref_w.data_ptr(), ref_s.data_ptr(), shift,
                                    out_w.data_ptr(), out_s.data_ptr(), n, k)
    assert st == 0
    assert torch.equal(out_w, ref_w.permute(0, 2, 1)) and torch.equal(out_s, ref_s.reshape(n, ng, 2, 2).permute(0, 2, 1, 3))
    assert lib.mui_int8_repack_gateup(None, ref_w.data_ptr(), ref_s.data_ptr(), 3, out_w.data_ptr(), out_s.data_ptr(), n, k) == -2
    assert lib.mui_int8_repack_gateup(None, ref_w.data_ptr(), None, shift, out_w.data_ptr(), out_s.data_ptr(), n, k) == -1


def test_int8_abi_errors():
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    w = torch.zeros(8, 32, dtype=torch.int8, device=DEV)
    sc = torch.ones(8, dtype=torch.float16, device=DEV)
    x = torch.zeros(32, dtype=torch.float16, device=DEV)
    y = torch.zeros(8, dtype=torch.float16, device=DEV)
    assert lib.mui_int8_linear(s, 0, w.data_ptr(), 32, None, x.data_ptr(), None, 0.0, None, None, y.data_ptr(), 8, 32, 1) == -1
    assert lib.mui_int8_linear(s, 0, w.data_ptr(), 24, sc.data_ptr(), x.data_ptr(), None, 0.0, None, None, y.data_ptr(), 8, 24, 1) == -2
    assert lib.mui_int8_group_linear(s, 0, w.data_ptr(), 32, sc.data_ptr(), 3, x.data_ptr(), None, 0.0, None, None, y.data_ptr(), 8, 32, 1) == -2
    # K % 16 != 0 goes through dequantise + matmul and is still right
    g = _gen(7)
    wf = _mk((8, 24), g, 0.02)
    q, s_ = oracle.rtn_quantize_channel(wf)
    xx = _mk((24,), g)
    yy = muillm_ext.mui_int8_channel_linear_forward(xx.to(DEV), q.to(DEV), s_.to(DEV))
    assert_parity(yy, oracle.int8_channel_linear(xx, q, s_), 1e-2, "K=24")


@pytest.mark.parametrize("chunk_max", [16, 64])
@pytest.mark.parametrize("tokens", [17, 40, 64])
def test_channel_linear_and_gateup_short_prompts(tokens, chunk_max, monkeypatch):
    """17..64 tokens: the tiled GEMM converting the codes on the way (the default), or the 16-token
    int8 kernels in chunks when the chunk limit is raised -- never a dequantised matrix for a
    library GEMM."""
    assert muillm_ext.INT8_CHUNK_MAX_TOKENS == 16 and muillm_ext.INT8_GROUP_CHUNK_MAX_TOKENS == 16
    monkeypatch.setattr(muillm_ext, "INT8_CHUNK_MAX_TOKENS", chunk_max)
    g = _gen(31)
    n, k = 264, 1024
    w = _mk((n, k), g, 0.02)
    q, s = oracle.rtn_quantize_channel(w)
    x = _mk((tokens, k), g)
    gamma = _mk((k,), g, 0.1, 1.0)
    r = _mk((tokens, n), g)
    assert muillm_ext.int8_kernel_dispatchable(x.to(DEV))
    ref = oracle.int8_channel_linear(x, q, s, gamma, 1e-5, None, r)
    y = muillm_ext.mui_int8_channel_linear_forward(x.to(DEV), q.to(DEV), s.to(DEV), gamma.to(DEV), 1e-5, None, r.to(DEV))
    assert y.shape == (tokens, n)
    assert_parity(y, ref, 1e-2, f"int8 chunks {tokens}", tight=4e-3)
    wg, wu = _mk((n, k), g, 0.02), _mk((n, k), g, 0.02)
    (qg, sg), (qu, su) = oracle.rtn_quantize_channel(wg), oracle.rtn_quantize_channel(wu)
    h = muillm_ext.mui_int8_channel_gateupsilu_forward(gamma.to(DEV), 1e-5, qg.to(DEV), qu.to(DEV), sg.to(DEV),
                                                       su.to(DEV), x.to(DEV))
    ref_h = oracle.gateup_silu(x, oracle.rtn_dequantize_channel(qg, sg), oracle.rtn_dequantize_channel(qu, su), gamma, 1e-5)
    assert_parity(h, ref_h, 1e-2, f"int8 gate/up chunks {tokens}")
    # longer prompts stay on the library's kernels too (the tiled GEMM of the same entry points)
    assert muillm_ext.int8_kernel_dispatchable(torch.zeros(65, k, dtype=torch.float16, device=DEV))
    assert muillm_ext._token_calls(64, 64) == [(0, 16), (16, 16), (32, 16), (48, 16)] and muillm_ext._token_calls(65, 64) == [(0, 65)]
    assert muillm_ext._token_chunks(16, group_format=True) == [(0, 16)] and muillm_ext._token_chunks(17, group_format=True) == [(0, 17)]


def test_wrappers_refuse_mismatched_operands():
    """The drop-in entry points hand raw pointers to the kernels: a short activation row, a CPU
    tensor, scales in another 16-bit type or too many tokens are refused with RuntimeError."""
    g = _gen(41)
    n, k = 64, 256
    q, s = oracle.rtn_quantize_channel(_mk((n, k), g, 0.02))
    qd, sd = q.to(DEV), s.to(DEV)
    x = _mk((1, k), g).to(DEV)
    with pytest.raises(RuntimeError, match="features"):
        muillm_ext.mui_int8_channel_gateupsilu_forward(None, 0.0, qd, qd, sd, sd, x[:, : k - 16])
    with pytest.raises(RuntimeError, match="CUDA"):
        muillm_ext.mui_int8_channel_gateupsilu_forward(None, 0.0, qd, qd, sd, sd, x.cpu())
    with pytest.raises(RuntimeError, match="dtype"):
        muillm_ext.mui_int8_channel_gateupsilu_forward(None, 0.0, qd, qd, sd.bfloat16(), sd.bfloat16(), x)
    with pytest.raises(RuntimeError, match="tokens"):
        muillm_ext.mui_int8_channel_gateupsilu_forward(None, 0.0, qd, qd, sd, sd, torch.zeros(0, k, dtype=torch.float16, device=DEV))
    qu, smv = oracle.rtn_quantize_group(_mk((n, k), g, 0.02), 128)
    qu, smv = qu.to(DEV), smv.to(DEV)
    with pytest.raises(RuntimeError, match="dtype"):
        muillm_ext.muillm_int8_linear_forward(x.bfloat16(), qu, smv, 7)        # bf16 activations, fp16 (scale, min)
    packed = torch.stack([qu, qu], dim=1).contiguous()
    psmv = torch.stack([smv.reshape(n, -1, 2)] * 2, dim=1).contiguous()
    with pytest.raises(RuntimeError, match="features"):
        muillm_ext.muillm_int8_gateupsilu_forward(None, 0.0, packed, psmv, 7, x[:, : k - 16])
    with pytest.raises(RuntimeError, match="tokens"):
        muillm_ext.muillm_int8_gateupsilu_forward(None, 0.0, packed, psmv, 7, torch.zeros(0, k, dtype=torch.float16, device=DEV))
    w = _mk((n, k), g, 0.02).to(DEV)
    with pytest.raises(RuntimeError, match="features"):
        muillm_ext.mui_gateup_silu(None, 0.0, w, w, x[:, : k - 8])
    with pytest.raises(RuntimeError, match="dtype"):
        muillm_ext.mui_gateup_silu(None, 0.0, w, w, x.bfloat16())
    with pytest.raises(RuntimeError, match="CUDA"):
        muillm_ext.muillm_gateupsilu_forward(None, None, 0.0, w, w, w[:k, :n] if False else w, None, x.cpu())
