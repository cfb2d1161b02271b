"""GPU parity of the software-pipelined prompt tiles (mui_linear / mui_gateup_silu beyond
MUI_MAX_TOKENS tokens, 16-bit weights, no fused norm, K a multiple of 64): 256 x 256, 128 x 256 and
192 x 256 (linear only) on eight waves with two operand register sets each, operands loaded
straight into LDS. Checked against the CPU oracle at the decode kernels' gate (max error over
max |ref| <= 1e-2) and bit for bit against the older kernels of the same tiles, which multiply the
same products in the same order.

The reference hands these calls to the framework's GEMM (csrc/modules/linear_module.cpp:57-79)."""

import pytest
import torch

import oracle
from muillm_amd import _lib
from tests.util import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _mk(shape, g, std=1.0, mean=0.0, dtype=torch.float16):
    return (mean + std * torch.randn(shape, generator=g)).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k,tokens,gateup", [
    (1000, 1024, 300, False),   # ragged rows and tokens: clamped rows and tokens in the last tiles
    (512, 64, 256, False),      # a single k-step
    (256, 128, 257, False),     # two k-steps, one token past a tile
    (4096, 14336, 520, False),  # down projection: 224 k-steps
    (700, 512, 400, True),      # gate/up, ragged
    (14336, 4096, 512, True),   # gate/up at the benchmark shape
])
def test_software_pipelined_tiles(dtype, n, k, tokens, gateup):
    """Tile choices 4 (256 x 256), 7 (128 x 256) and 8 (192 x 256; the gate/up epilogue has none and
    takes its twelve-wave kernel) run the software-pipelined loop here, 7 on three LDS stages and
    25607 the same tile on two, 4 and 8 on three stages of the weight tile and two of the token tile
    and 51204 / 51208 on two of both; 13, 207, 208 and 104 are the older kernels of the same tiles (sixteen /
    sixteen / twelve waves, LDS-direct or register-staged operands). The shapes with one and two
    k-steps run the three-stage loop with fewer steps than stages."""
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    g = _gen(11)
    code = 0 if dtype == torch.float16 else 1
    x = _mk((tokens, k), g, dtype=dtype)
    if gateup:
        wg, wu = _mk((n, k), g, 0.02, dtype=dtype), _mk((n, k), g, 0.02, dtype=dtype)
        ref = oracle.gateup_silu(x, wg, wu)
        wgd, wud, r, b = wg.to(DEV), wu.to(DEV), None, None
    else:
        w, r, b = _mk((n, k), g, 0.02, dtype=dtype), _mk((tokens, n), g, dtype=dtype), _mk((n,), g, 0.5, dtype=dtype)
        ref = oracle.linear(x, w, None, 1e-5, b, r)
        wd, r, b = w.to(DEV), r.to(DEV), b.to(DEV)
    xd = x.to(DEV)
    outs = {}
    for choice in (4, 51204, 13, 104, 7, 25607, 207, 8, 51208, 208):
        _lib.check(lib.mui_tune_prefill(choice, -1), "mui_tune_prefill")
        y = torch.zeros(tokens, n, dtype=dtype, device=DEV)
        if gateup:
            st = lib.mui_gateup_silu(s, code, wgd.data_ptr(), wud.data_ptr(), k, xd.data_ptr(), None, 0.0, y.data_ptr(), n, k, tokens)
        else:
            st = lib.mui_linear(s, code, wd.data_ptr(), k, xd.data_ptr(), None, 0.0, None, b.data_ptr(), r.data_ptr(), y.data_ptr(),
                                n, k, tokens)
        assert st == 0
        torch.cuda.synchronize()
        outs[choice] = y
    _lib.check(lib.mui_tune_prefill(0, 0), "mui_tune_prefill")
    for choice in (4, 7, 8):
        assert_parity(outs[choice], ref, 1e-2, f"pipelined tile choice {choice} {dtype} {tokens}x{n}x{k} gateup={gateup}")
    assert torch.equal(outs[4], outs[13]) and torch.equal(outs[4], outs[104])
    assert torch.equal(outs[7], outs[207]) and torch.equal(outs[8], outs[208]) and torch.equal(outs[4], outs[7])
    assert torch.equal(outs[7], outs[25607]) and torch.equal(outs[4], outs[51204]) and torch.equal(outs[8], outs[51208])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k,tokens", [
    (4608, 256, 2048),     # 36 row tiles of the 256 x 256 tile at 8 token tiles: one whole round of 32 and a tail of 4
    (4700, 128, 2000),     # the same with ragged outputs and tokens
    (14336, 4096, 2048),   # the benchmark shape: 3.5 rounds
])
def test_gateup_whole_rounds_and_tail_in_two_launches(dtype, n, k, tokens):
    """Gate/up whose 256 x 256 tiles end in a round that is at most half full is launched as the whole
    rounds on that tile and the remaining outputs on 128 x 256 tiles (the built-in choice; on a
    256-CU device these shapes take it): bit for bit what one launch on the 256 x 256 tile gives
    (tile choice 4, checked against the oracle above), and against the oracle on the small shapes."""
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    g = _gen(12)
    code = 0 if dtype == torch.float16 else 1
    x = _mk((tokens, k), g, dtype=dtype)
    wg, wu = _mk((n, k), g, 0.02, dtype=dtype), _mk((n, k), g, 0.02, dtype=dtype)
    xd, wgd, wud = x.to(DEV), wg.to(DEV), wu.to(DEV)
    outs = {}
    for choice in (0, 4, 3200):
        _lib.check(lib.mui_tune_prefill(choice, 0 if choice != 4 else -1), "mui_tune_prefill")
        y = torch.zeros(tokens, n, dtype=dtype, device=DEV)
        assert lib.mui_gateup_silu(s, code, wgd.data_ptr(), wud.data_ptr(), k, xd.data_ptr(), None, 0.0, y.data_ptr(), n, k, tokens) == 0
        torch.cuda.synchronize()
        outs[choice] = y
    _lib.check(lib.mui_tune_prefill(0, 0), "mui_tune_prefill")
    assert torch.equal(outs[0], outs[4]) and torch.equal(outs[0], outs[3200])
    if k <= 256:
        assert_parity(outs[0], oracle.gateup_silu(x, wg, wu), 1e-2, f"gate/up in two launches {dtype} {tokens}x{n}x{k}")


@pytest.mark.parametrize("n,k,tokens", [
    (4096, 14336, 4096),   # down: one round of 256 x 256 tiles, the XCDs split rows x tokens 4 x 2, 224 k-steps
    (6144, 4096, 4096),    # QKV: two rounds of 192 x 256 tiles walked by a persistent round of workgroups
    (4096, 4096, 8192),    # o_proj: two rounds of 256 x 256 tiles in panels of four row tiles
    (4096, 4096, 2048),    # o_proj: one round of 128 x 256 tiles on three LDS stages
])
def test_full_size_prompt_linears_against_the_older_kernels(n, k, tokens):
    """The Llama-3-8B projections at whole-prompt sizes, where the built-in choice walks several rounds
    of tiles, splits the grid over the XCDs by rows and tokens and keeps three LDS stages: bit for bit
    what the sixteen- / twelve-wave kernels of the same tiles give with every such choice switched
    off (100 + tile: register-staged operands; 800: one row tile after another; 6400: rows-only split;
    51200 / 25600: two LDS stages), and within 1e-2 of the maximum of an fp32 product of the same
    operands on the device (the CPU oracle takes minutes at these sizes; it gates the same kernels
    on smaller shapes above)."""
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    g = _gen(13)
    x = _mk((tokens, k), g).to(DEV)
    w = _mk((n, k), g, 0.02).to(DEV)
    r = _mk((tokens, n), g).to(DEV)
    ref = x.float() @ w.float().t() + r.float()
    which = 8 if n == 6144 else 7 if tokens == 2048 else 4
    outs = {}
    for choice in (0, 100 + which + 800 + 6400, 51200 + 25600 + which):
        _lib.check(lib.mui_tune_prefill(choice, 0 if choice == 0 else -1), "mui_tune_prefill")
        y = torch.zeros(tokens, n, dtype=torch.float16, device=DEV)
        assert lib.mui_linear(s, 0, w.data_ptr(), k, x.data_ptr(), None, 0.0, None, None, r.data_ptr(), y.data_ptr(), n, k, tokens) == 0
        torch.cuda.synchronize()
        outs[choice] = y
    _lib.check(lib.mui_tune_prefill(0, 0), "mui_tune_prefill")
    err = float((outs[0].float() - ref).abs().max() / ref.abs().max())
    print(f"[parity] full-size prompt linear {tokens}x{n}x{k}: max err over max |ref| {err:.2e} (gate 1e-2)")
    assert err <= 1e-2
    for choice, y in outs.items():
        assert torch.equal(outs[0], y), f"choice {choice} differs from the built-in one"
