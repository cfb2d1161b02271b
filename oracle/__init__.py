"""CPU oracle for the decode hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A plain-PyTorch (CPU) restatement of the layer definitions that the reference
(Epliz/muiLLM) falls back to when its fused kernels do not apply, i.e. the semantics its
HIP kernels are meant to reproduce.  Each function cites the reference file:line it follows.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package, and only as the checker.  Nothing under muillm_amd/ imports it; the product path
raises if the HIP library is missing instead of falling back to anything here.

Two flavours per layer:
  * `*_exact`-style behaviour (default): inputs are upcast to float64, every reduction is
    done in float64 and nothing is rounded on the way.  This is the fp32-accumulated
    reference the tolerances are stated against (float64 so that the oracle's own
    rounding is negligible).
  * `reference_path=True` where offered: the reference's fallback executed literally in the
    tensors' own 16-bit dtype on CPU (F.linear on fp16, HF rounding points).  That is what
    bench.py times as the CPU baseline.

How each function is pinned (tests/test_oracle_*.py, all CPU):
  rmsnorm / linear / mlp      closed forms (identity weights, constant rows, scale
                              invariance), float64 numpy brute force, HuggingFace
                              LlamaRMSNorm / LlamaMLP fixtures in tests/golden/.
  rtn_quantize_group          closed form (range end points map to 0 and 255, |w-dq|<=scale/2),
                              brute-force numpy restatement on tiny groups.
  rtn_quantize_channel        closed form (row max -> +-127, |w-dq| <= s/2, zero rows).
  rope                        position 0 = identity, norm preservation, relative-position
                              property, float64 complex-rotation brute force, HuggingFace
                              apply_rotary_pos_emb fixture.
  static cache update         prefill-then-decode sequence equals concatenation.
  decode attention            S=1, identical keys -> mean of V, dominant key, split
                              invariance, numpy brute force, HuggingFace eager attention fixture.
"""

from .layers import *  # noqa: F401,F403
