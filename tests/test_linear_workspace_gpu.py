"""mui_linear_ws: the prompt linear with a caller-provided workspace (parity gate: north_star's 1e-2
relative against the fp32-accumulating oracle; bit-equal results call after call)."""
import pytest
import torch

from muillm_amd import _lib
import oracle
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
@pytest.mark.parametrize("tokens,n,k", [(64, 4096, 14336), (256, 4096, 14336), (33, 4096, 14336), (200, 1000, 6152)])
def test_linear_workspace_entry_shares_k_between_workgroups(tokens, n, k, dtype):
    """mui_linear_ws through the C ABI: few output tiles and a long K, so K is shared between
    workgroups that exchange partial tiles through the caller's workspace. Checked against the oracle
    and against the call without a workspace; three calls in a row on the same workspace (its
    counters must be back at zero after each) give the same bits, whichever workgroup arrived last."""
    lib = _lib.load()
    s = torch.cuda.current_stream().cuda_stream
    g = _gen(11)
    w, x = _mk((n, k), g, 0.02, dtype=dtype), _mk((tokens, k), g, dtype=dtype)
    r, b = _mk((tokens, n), g, dtype=dtype), _mk((n,), g, 0.5, dtype=dtype)
    ref = oracle.linear(x, w, None, 0.0, b, r)
    wd, xd, rd, bd = w.to(DEV), x.to(DEV), r.to(DEV), b.to(DEV)
    ws = torch.zeros(lib.mui_linear_workspace_bytes(), dtype=torch.uint8, device=DEV)
    code = 0 if dtype == torch.float16 else 1
    outs = []
    for _ in range(3):
        y = torch.zeros(tokens, n, dtype=dtype, device=DEV)
        st = lib.mui_linear_ws(s, code, wd.data_ptr(), k, xd.data_ptr(), None, 0.0, None, bd.data_ptr(), rd.data_ptr(),
                               y.data_ptr(), n, k, tokens, ws.data_ptr(), ws.numel())
        assert st == 0
        outs.append(y)
    torch.cuda.synchronize()
    assert_parity(outs[0], ref, 1e-2, f"prompt linear with workspace {tokens}x{n}x{k}")
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert int(ws[:4096].to(torch.int32).sum()) == 0  # every counter returned to zero
    plain = torch.zeros(tokens, n, dtype=dtype, device=DEV)
    assert lib.mui_linear(s, code, wd.data_ptr(), k, xd.data_ptr(), None, 0.0, None, bd.data_ptr(), rd.data_ptr(),
                          plain.data_ptr(), n, k, tokens) == 0
    assert_parity(outs[0], plain.double().cpu(), 1e-2, "workspace vs plain call",
                  elementwise=None)
    # a workspace that is too small or misaligned is not used (the call is then mui_linear); a size without a pointer is refused
    small = torch.zeros(tokens, n, dtype=dtype, device=DEV)
    assert lib.mui_linear_ws(s, code, wd.data_ptr(), k, xd.data_ptr(), None, 0.0, None, bd.data_ptr(), rd.data_ptr(),
                             small.data_ptr(), n, k, tokens, ws.data_ptr(), 1024) == 0
    assert torch.equal(small, plain)
    assert lib.mui_linear_ws(s, code, wd.data_ptr(), k, xd.data_ptr(), None, 0.0, None, bd.data_ptr(), rd.data_ptr(),
                             small.data_ptr(), n, k, tokens, None, 4096) == -1
