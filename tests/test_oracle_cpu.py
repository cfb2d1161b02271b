"""Pins the CPU oracle itself (no GPU): every oracle function is checked against something
that does not retype its formula -- golden vectors written by the HuggingFace library
(tests/golden/hf_llama_small.npz, made by tests/golden/make_fixtures.py), closed forms,
invariants, and float64 numpy brute force on tiny inputs -- chosen so that a dropped term,
a wrong sign/index or a transposed operand fails at least one of them."""

import math
import os

import numpy as np
import pytest
import torch

import oracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hf_llama_small.npz")


@pytest.fixture(scope="module")
def gold():
    z = np.load(GOLD, allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files if k != "versions"}


# ------------------------------------------------------------------------------------
# golden vectors from the HuggingFace library
# ------------------------------------------------------------------------------------
def test_rmsnorm_vs_hf(gold):
    y = oracle.rmsnorm(gold["norm_x"], gold["norm_w"], 1e-5)
    assert torch.allclose(y, gold["norm_y"].double(), atol=1e-6)
    y16 = oracle.rmsnorm(gold["norm_x"], gold["norm_w"], 1e-5, reference_path=True)
    assert torch.allclose(y16, gold["norm_y"], atol=1e-6)


def test_mlp_vs_hf(gold):
    y = oracle.gateupdown_mlp(gold["mlp_x"], gold["mlp_wg"], gold["mlp_wu"], gold["mlp_wd"])
    assert torch.allclose(y, gold["mlp_y"].double(), atol=1e-5)
    # swapping gate and up must change the result (silu is applied to gate only)
    y_sw = oracle.gateupdown_mlp(gold["mlp_x"], gold["mlp_wu"], gold["mlp_wg"], gold["mlp_wd"])
    assert not torch.allclose(y_sw, gold["mlp_y"].double(), atol=1e-3)


def test_rope_vs_hf(gold):
    inv = oracle.rope_inv_freq(500000.0, 64)
    assert torch.equal(inv, gold["rope_inv_freq"])
    cos, sin = oracle.rope_tables(500000.0, 64, 96)
    pos = gold["rope_pos"]
    assert torch.allclose(cos[pos], gold["rope_cos"], atol=1e-6) and torch.allclose(sin[pos], gold["rope_sin"], atol=1e-6)
    qr, kr = oracle.apply_rope(gold["rope_q"], gold["rope_k"], cos, sin, pos)
    assert torch.allclose(qr, gold["rope_qr"].double(), atol=1e-5)
    assert torch.allclose(kr, gold["rope_kr"].double(), atol=1e-5)


def test_llama3_rope_scaling_vs_hf(gold):
    from muillm_amd.modules.attention.rotaryembedding import compute_rope_inv_freq

    inv, scale = compute_rope_inv_freq("llama3", 500000.0, 128, dict(
        factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192))
    assert scale == 1.0 and torch.allclose(inv, gold["llama3_inv_freq"], rtol=1e-6, atol=0)
    inv_d, _ = compute_rope_inv_freq("default", 500000.0, 64)
    assert torch.equal(inv_d, gold["rope_inv_freq"])


def test_attention_vs_hf(gold):
    out = oracle.decode_attention(gold["attn_q"], gold["attn_k"], gold["attn_v"], gold["attn_mask"])
    ref = gold["attn_out"].reshape(2, 1, 4 * 64).double()  # HF returns [B, T, H, D]
    assert torch.allclose(out, ref, atol=1e-5)
    out16 = oracle.decode_attention(gold["attn_q"], gold["attn_k"], gold["attn_v"], gold["attn_mask"], reference_path=True)
    assert torch.allclose(out16.double(), ref, atol=1e-5)


def test_whole_model_vs_hf(gold):
    """decoder_layer / decoder_model_step compose to HF's LlamaForCausalLM logits."""
    sd = {k[3:]: v.float() for k, v in gold.items() if k.startswith("sd.")}
    layers = []
    for i in range(2):
        p = f"model.layers.{i}."
        layers.append(dict(ln1=sd[p + "input_layernorm.weight"], wq=sd[p + "self_attn.q_proj.weight"],
                           wk=sd[p + "self_attn.k_proj.weight"], wv=sd[p + "self_attn.v_proj.weight"],
                           wo=sd[p + "self_attn.o_proj.weight"], ln2=sd[p + "post_attention_layernorm.weight"],
                           wg=sd[p + "mlp.gate_proj.weight"], wu=sd[p + "mlp.up_proj.weight"],
                           wd=sd[p + "mlp.down_proj.weight"], eps=1e-5))
    params = dict(embed=sd["model.embed_tokens.weight"], layers=layers, norm=sd["model.norm.weight"],
                  lm_head=sd["lm_head.weight"], eps=1e-5)
    cos, sin = oracle.rope_tables(500000.0, 64, 32)
    ids = gold["model_ids"]
    mk = lambda: [torch.zeros(2, 1, 16, 64, dtype=torch.float64) for _ in range(2)]
    kc, vc = mk(), mk()
    logits, seen = oracle.decoder_model_step(ids, params, kc, vc, cos, sin, 0, 2, 1, store_dtype=torch.float64)
    assert seen == 10
    assert torch.allclose(logits, gold["model_logits"].double(), atol=2e-5)
    # prefill 7 tokens then three single-token steps give the same logits (static cache path)
    kc, vc = mk(), mk()
    lg, seen = oracle.decoder_model_step(ids[:, :7], params, kc, vc, cos, sin, 0, 2, 1, store_dtype=torch.float64)
    for t in range(7, 10):
        lg, seen = oracle.decoder_model_step(ids[:, t : t + 1], params, kc, vc, cos, sin, seen, 2, 1, store_dtype=torch.float64)
        assert torch.allclose(lg[:, 0], gold["model_logits"][:, t].double(), atol=2e-5)


# ------------------------------------------------------------------------------------
# closed forms, invariants, brute force
# ------------------------------------------------------------------------------------
def test_linear_brute_force_and_closed_forms():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((5, 7))
    x = rng.standard_normal((2, 7))
    g = rng.standard_normal(7)
    b, r, mb = rng.standard_normal(5), rng.standard_normal((2, 5)), rng.standard_normal(5)
    eps = 1e-3
    ref = np.zeros((2, 5))
    for t in range(2):
        ms = sum(x[t, k] ** 2 for k in range(7)) / 7
        xn = [g[k] * x[t, k] / math.sqrt(ms + eps) for k in range(7)]
        for n in range(5):
            ref[t, n] = sum(w[n, k] * xn[k] for k in range(7)) * mb[n] + b[n] + r[t, n]
    T = torch.from_numpy
    got = oracle.linear(T(x), T(w), T(g), eps, T(b), T(r), T(mb))
    assert np.allclose(got.numpy(), ref, atol=1e-12)
    xx = torch.randn(3, 16)
    assert torch.allclose(oracle.linear(xx, torch.eye(16)), xx.double())
    assert torch.allclose(oracle.linear(xx, torch.ones(2, 16)), xx.double().sum(-1, keepdim=True).expand(3, 2))
    outs = oracle.multilinear(xx, [torch.eye(16)[:4], torch.eye(16)[4:6]])
    assert torch.allclose(outs[0], xx[:, :4].double()) and torch.allclose(outs[1], xx[:, 4:6].double())


def test_rmsnorm_invariants():
    x = torch.randn(4, 64)
    ones = torch.ones(64)
    y = oracle.rmsnorm(x, ones, 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(4, dtype=torch.float64))
    assert torch.allclose(oracle.rmsnorm(x * 7, ones, 0.0), y)
    c = torch.full((1, 64), -2.5)
    assert torch.allclose(oracle.rmsnorm(c, ones, 0.0), -torch.ones(1, 64, dtype=torch.float64))
    # eps is added to the mean, not divided by K
    assert torch.allclose(oracle.rmsnorm(torch.zeros(1, 64) + 1e-4, ones, 1.0), torch.full((1, 64), 1e-4, dtype=torch.float64), rtol=1e-6)


def test_mlp_closed_forms():
    x, r = torch.randn(2, 8), torch.randn(2, 8)
    w, wd, z = torch.randn(12, 8), torch.randn(8, 12), torch.zeros(12, 8)
    assert torch.allclose(oracle.gateupdown_mlp(x, z, w, wd, residual=r), r.double())
    assert torch.allclose(oracle.gateupdown_mlp(x, w, z, wd, residual=r), r.double())
    g = oracle.gateup_silu(x, w, w)
    a = x.double() @ w.double().T
    assert torch.allclose(g, a * a / (1 + torch.exp(-a)))


def test_group_rtn_brute_force():
    rng = np.random.default_rng(1)
    w = rng.standard_normal((3, 8)).astype(np.float32)
    q, smv = oracle.rtn_quantize_group(torch.from_numpy(w), group_size=4)
    for n in range(3):
        for gi in range(2):
            grp = w[n, 4 * gi : 4 * gi + 4]
            lo, hi = float(grp.min()), float(grp.max())
            scale = (hi - lo) / 255
            assert abs(float(smv[n * 2 + gi, 0]) - scale) < 1e-6 and abs(float(smv[n * 2 + gi, 1]) - lo) < 1e-6
            for j in range(4):
                assert int(q[n, 4 * gi + j]) == int(np.clip(np.round((grp[j] - lo) / scale), 0, 255))
    dq = oracle.rtn_dequantize_group(q, smv, 4, torch.float32)
    assert float((dq - torch.from_numpy(w)).abs().max()) <= float(smv[:, 0].max()) * 0.5 + 1e-6
    # constant group -> range clamp, no division by zero
    q0, smv0 = oracle.rtn_quantize_group(torch.full((1, 4), 0.25), 4)
    assert torch.isfinite(smv0).all() and torch.allclose(oracle.rtn_dequantize_group(q0, smv0, 4, torch.float32), torch.full((1, 4), 0.25), atol=1e-5)


def test_group_dequant_kernel_form_vs_python_form():
    w = (torch.randn(8, 64) * 0.02).half()
    q, smv = oracle.rtn_quantize_group(w, 16)
    a = oracle.rtn_dequantize_group(q, smv, 16, torch.float16, kernel_form=True)
    b = oracle.rtn_dequantize_group(q, smv, 16, torch.float16, kernel_form=False)
    exact = (q.reshape(-1, 16).double() * smv[:, None, 0].double() + smv[:, None, 1].double()).reshape(8, 64)
    assert float((a.double() - exact).abs().max()) <= float((b.double() - exact).abs().max()) + 1e-9
    assert torch.equal(a, exact.float().half())  # fp32 fma then one rounding == exact value rounded twice in order


def test_channel_rtn_closed_forms():
    w = torch.tensor([[0.5, -1.0, 0.25, 0.0], [0.0, 0.0, 0.0, 0.0], [2.0, 1.0, -0.5, 0.125]], dtype=torch.float16)
    q, s = oracle.rtn_quantize_channel(w)
    assert q.dtype == torch.int8 and s.dtype == torch.float16
    assert int(q[0, 1]) == -127 and int(q[2, 0]) == 127 and not q[1].any() and float(s[1]) > 0
    assert abs(float(s[0]) - 1.0 / 127) < 1e-5
    dq = oracle.rtn_dequantize_channel(q, s)
    assert torch.equal(dq, q.half() * s[:, None])
    assert bool(((dq.float() - w.float()).abs() <= s.float()[:, None] * 0.5 + w.float().abs() * 2.0 ** -9).all())
    # round-half-even: 2.5 steps -> 2, 3.5 -> 4 (scale exactly 1/64 -> max 127/64)
    w2 = torch.tensor([[127 / 64, 2.5 / 64, 3.5 / 64, -2.5 / 64]], dtype=torch.float16)
    q2, s2 = oracle.rtn_quantize_channel(w2)
    assert float(s2[0]) == 1 / 64 and q2.tolist() == [[127, 2, 4, -2]]


def test_int8_linear_compositions_brute_force():
    """The two dequantise-then-linear oracle functions against numpy loops that index every code,
    scale and minimum themselves: distinct per-row / per-group (scale, min) values, so that a
    swapped column, a transposed scale or a wrong group index changes the result."""
    rng = np.random.default_rng(7)
    n, k, gs = 3, 8, 4
    x = rng.standard_normal((2, k))
    bias, res = rng.standard_normal(n), rng.standard_normal((2, n))
    xt, bt, rt = torch.from_numpy(x), torch.from_numpy(bias), torch.from_numpy(res)
    # per-channel: y[t, r] = sum_j x[t, j] * q[r, j] * s[r] + bias[r] + res[t, r]
    q = rng.integers(-127, 128, size=(n, k)).astype(np.int8)
    s = np.array([2.0 ** -6, 3 * 2.0 ** -9, 5 * 2.0 ** -8], dtype=np.float16)  # exact products in fp16
    want = np.zeros((2, n))
    for t in range(2):
        for r in range(n):
            acc = 0.0
            for j in range(k):
                acc += x[t, j] * (float(q[r, j]) * float(s[r]))
            want[t, r] = acc + bias[r] + res[t, r]
    got = oracle.int8_channel_linear(xt, torch.from_numpy(q), torch.from_numpy(s), None, 0.0, bt, rt)
    # the per-channel oracle rounds q*s to fp16 (the dense dequantisation): exact for these scales
    assert np.abs(got.numpy() - want).max() < 1e-12
    same = oracle.linear(xt, torch.from_numpy(q).double() * torch.from_numpy(s).double()[:, None], None, 0.0, bt, rt)
    assert torch.allclose(got, same, atol=1e-12, rtol=0)
    # group format: row r, group g owns pair r * (k / gs) + g: w = code * scale + min, not rounded
    qu = rng.integers(0, 256, size=(n, k)).astype(np.uint8)
    smv = (rng.standard_normal((n * (k // gs), 2)) * 0.01).astype(np.float16)
    want = np.zeros((2, n))
    for t in range(2):
        for r in range(n):
            acc = 0.0
            for j in range(k):
                pair = smv[r * (k // gs) + j // gs]
                acc += x[t, j] * (float(qu[r, j]) * float(pair[0]) + float(pair[1]))
            want[t, r] = acc + bias[r] + res[t, r]
    got = oracle.int8_group_linear(xt, torch.from_numpy(qu), torch.from_numpy(smv), gs, None, 0.0, bt, rt)
    assert np.abs(got.numpy() - want).max() < 1e-12
    # and against the pinned dense dequantisation (fp32 result of the fma, before the 16-bit store)
    dq = oracle.rtn_dequantize_group(torch.from_numpy(qu), torch.from_numpy(smv), gs, torch.float32)
    via_dq = oracle.linear(xt, dq, None, 0.0, bt, rt)
    assert float((got - via_dq).abs().max()) < 1e-5
    # a fused norm goes in front of both, as in linear()
    gam = torch.from_numpy(rng.standard_normal(k))
    a = oracle.int8_channel_linear(xt, torch.from_numpy(q), torch.from_numpy(s), gam, 1e-5)
    b = oracle.linear(oracle.rmsnorm(xt, gam, 1e-5), torch.from_numpy(q).double() * torch.from_numpy(s).double()[:, None])
    assert torch.allclose(a, b, atol=1e-12, rtol=0)


def test_rounded_normalised_activations_mode():
    """rmsnorm(round_to=dtype) / norm_round: the exact gamma * x_hat rounded ONCE to the 16-bit type
    (what the reference's RMSNorm kernel stores, csrc/norm/rmsnorm_fp16_kernels.cu:111-115) -- closed
    forms that tell one rounding from none and from the fallback's two (rmsnorm.py:140-146)."""
    bf = torch.bfloat16
    x = torch.ones(1, 4)
    # x_hat = 1 (eps = 0): the result is gamma itself, rounded to bf16 (8 significant bits, ties to even)
    gam = torch.tensor([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, 1 + 2.0 ** -7, 0.7])
    y = oracle.rmsnorm(x, gam, 0.0, round_to=bf)
    assert y.dtype == torch.float64
    assert y[0].tolist() == [1.0, 1 + 2.0 ** -6, 1 + 2.0 ** -7, float(torch.tensor(0.7).to(bf))]
    assert oracle.rmsnorm(x, gam, 0.0)[0, 0].item() == 1 + 2.0 ** -8        # un-rounded mode untouched
    # one rounding, not the fallback's two
    g = torch.Generator().manual_seed(3)
    xr = torch.randn(64, 512, generator=g).to(bf)
    gr = (1 + 0.1 * torch.randn(512, generator=g)).to(bf)
    once = oracle.rmsnorm(xr, gr, 1e-5, round_to=bf)
    exact = oracle.rmsnorm(xr, gr, 1e-5)
    twice = oracle.rmsnorm(xr, gr, 1e-5, reference_path=True).double()
    assert torch.equal(once, exact.to(bf).double())
    assert float((once - exact).abs().max()) <= float(exact.abs().max()) * 2.0 ** -8
    assert not torch.equal(once, twice)
    assert float((twice - exact).abs().mean()) > float((once - exact).abs().mean())  # two roundings lose more
    # linear / gateup_silu / gateupdown_mlp with norm_round == the same functions fed the rounded activations
    w, wu, wd = torch.randn(24, 512, generator=g) * 0.05, torch.randn(24, 512, generator=g) * 0.05, torch.randn(512, 24, generator=g) * 0.05
    assert torch.equal(oracle.linear(xr, w, gr, 1e-5, norm_round=bf), oracle.linear(once, w))
    assert torch.equal(oracle.gateup_silu(xr, w, wu, gr, 1e-5, norm_round=bf), oracle.gateup_silu(once, w, wu))
    assert torch.equal(oracle.gateupdown_mlp(xr, w, wu, wd, gr, 1e-5, norm_round=bf), oracle.gateupdown_mlp(once, w, wu, wd))
    q, k, v = oracle.multilinear(xr, [w[:8], w[8:16], w[16:]], gr, 1e-5, norm_round=bf)
    assert torch.equal(torch.cat([q, k, v], -1), oracle.linear(once, w))


def test_bf16_gateup_elementwise_error_is_set_by_the_8_bit_operands():
    """Why the bf16 gate/up tests carry a second, wider elementwise assertion against the oracle
    with exact normalised activations: with gamma * x rounded to bf16 (once, as the RMSNorm kernel of
    the reference does; or twice, as its Python fallback does, rmsnorm.py:140-146) and everything
    else exact, single elements of silu(G x) * (U x) already sit more than 1e-2 * (|ref| + rms) away,
    while the error over max |ref| stays far below 1e-2."""
    g = torch.Generator().manual_seed(0)
    bf = torch.bfloat16
    x = torch.randn(16, 4096, generator=g).to(bf)
    gam = (1 + 0.1 * torch.randn(4096, generator=g)).to(bf)
    wg = (0.02 * torch.randn(2048, 4096, generator=g)).to(bf)
    wu = (0.02 * torch.randn(2048, 4096, generator=g)).to(bf)
    exact = oracle.gateup_silu(x, wg, wu, gam, 1e-5)
    rms = exact.pow(2).mean().sqrt()
    for rounded in (oracle.gateup_silu(x, wg, wu, gam, 1e-5, norm_round=bf),
                    oracle.gateup_silu(oracle.rmsnorm(x, gam, 1e-5, reference_path=True), wg, wu)):
        err = (rounded - exact).abs()
        assert float(err.max() / exact.abs().max()) < 5e-3
        assert 1e-2 < float((err / (exact.abs() + rms)).max()) < 4e-2


def test_rope_properties_and_brute_force():
    d = 8
    cos, sin = oracle.rope_tables(10000.0, d, 64)
    q, k = torch.randn(1, 2, 1, d), torch.randn(1, 2, 1, d)
    q0, k0 = oracle.apply_rope(q, k, cos, sin, torch.tensor([[0]]))
    assert torch.allclose(q0, q.double()) and torch.allclose(k0, k.double())
    # complex-rotation brute force: pairs (i, i + d/2) rotate by pos * theta^(-2i/d)
    pos = 13
    qr, _ = oracle.apply_rope(q, k, cos, sin, torch.tensor([[pos]]))
    for h in range(2):
        for i in range(d // 2):
            ang = np.float32(pos) * np.float32(1.0 / (10000.0 ** (2 * i / d)))
            z = complex(float(q[0, h, 0, i]), float(q[0, h, 0, i + d // 2])) * complex(math.cos(ang), math.sin(ang))
            assert abs(float(qr[0, h, 0, i]) - z.real) < 1e-5 and abs(float(qr[0, h, 0, i + d // 2]) - z.imag) < 1e-5
    # relative-position property
    def dot(m, n):
        a, _ = oracle.apply_rope(q, k, cos, sin, torch.tensor([[m]]))
        _, b = oracle.apply_rope(q, k, cos, sin, torch.tensor([[n]]))
        return (a * b).sum(-1)
    assert torch.allclose(dot(9, 4), dot(45, 40), atol=1e-4)
    assert not torch.allclose(dot(9, 4), dot(9, 5), atol=1e-3)


def test_static_cache_update_semantics():
    kc, vc = torch.zeros(1, 2, 8, 4), torch.zeros(1, 2, 8, 4)
    k1, v1 = torch.randn(1, 2, 3, 4), torch.randn(1, 2, 3, 4)
    kk, vv, seen = oracle.static_cache_update(kc, vc, k1, v1, torch.arange(3), 0)
    assert seen == 3 and torch.equal(kk, k1) and torch.equal(vv, v1)
    k2, v2 = torch.randn(1, 2, 1, 4), torch.randn(1, 2, 1, 4)
    kk, vv, seen = oracle.static_cache_update(kc, vc, k2, v2, torch.tensor([3]), seen)
    assert seen == 4 and torch.equal(kk, torch.cat([k1, k2], 2)) and not kc[:, :, 4:].any()
    assert oracle.next_pow2(288) == 512 and oracle.next_pow2(1) == 1


def test_attention_closed_forms_and_brute_force():
    rng = np.random.default_rng(2)
    b, hq, hkv, s, d = 1, 4, 2, 5, 6
    q = rng.standard_normal((b, hq, 1, d))
    k = rng.standard_normal((b, hkv, s, d))
    v = rng.standard_normal((b, hkv, s, d))
    ref = np.zeros((b, 1, hq * d))
    for h in range(hq):
        kv = h // (hq // hkv)
        sc = np.array([sum(q[0, h, 0, i] * k[0, kv, t, i] for i in range(d)) / math.sqrt(d) for t in range(s)])
        p = np.exp(sc - sc.max())
        p /= p.sum()
        for i in range(d):
            ref[0, 0, h * d + i] = sum(p[t] * v[0, kv, t, i] for t in range(s))
    T = torch.from_numpy
    got = oracle.decode_attention(T(q), T(k), T(v))
    assert np.allclose(got.numpy(), ref, atol=1e-12)
    # the grouped form equals the reference's repeat_kv form
    rk = oracle.repeat_kv(T(k), 2)
    assert rk.shape == (1, 4, 5, 6) and torch.equal(rk[:, 1], T(k)[:, 0]) and torch.equal(rk[:, 2], T(k)[:, 1])
    # S = 1 -> v0 ; identical keys -> mean of V
    out1 = oracle.decode_attention(T(q), T(k[:, :, :1]), T(v[:, :, :1]))
    assert np.allclose(out1.numpy().reshape(hq, d), np.repeat(v[0, :, 0], 2, axis=0))
    same = np.repeat(k[:, :, :1], s, axis=2)
    outm = oracle.decode_attention(T(q), T(same), T(v))
    assert np.allclose(outm.numpy().reshape(hq, d), np.repeat(v[0].mean(1), 2, axis=0))
    # an additive -inf mask removes keys
    m = torch.zeros(1, 1, 1, s, dtype=torch.float64)
    m[..., :2] = float("-inf")
    outk = oracle.decode_attention(T(q), T(k), T(v), m)
    assert torch.allclose(outk, oracle.decode_attention(T(q), T(k[:, :, 2:]), T(v[:, :, 2:])))


def test_rel_err_denominator():
    assert oracle.rel_err(torch.tensor([1.0, 2.0]), torch.tensor([1.0, 4.0])) == 0.5


def test_greedy_advance_rules():
    """Stop-check semantics (csrc/generation/generation.cu:29-113) on hand-made cases: the
    argmax must agree with torch.argmax, an eos token finishes its row, a finished row emits the
    pad token from then on, and the step budget finishes every row."""
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(4, 50, generator=g)
    logits[1, 7] = 100.0   # row 1 picks the eos token 7
    logits[2, 9] = 100.0   # row 2 is already finished: must emit pad, not 9
    unfinished = torch.tensor([1, 1, 0, 1])
    toks, unf = oracle.greedy_advance(logits, unfinished, [7, 11], pad_token_id=3, steps_done=0, max_steps=10)
    expect = logits.argmax(-1)
    assert toks[0] == expect[0] and toks[3] == expect[3]
    assert toks[1] == 7 and toks[2] == 3
    assert unf.tolist() == [1, 0, 0, 1]
    # last step of the budget finishes everything
    _, unf2 = oracle.greedy_advance(logits, unfinished, [7, 11], 3, steps_done=9, max_steps=10)
    assert unf2.tolist() == [0, 0, 0, 0]
    # without an eos criterion a finished row keeps its argmax
    toks3, _ = oracle.greedy_advance(logits, unfinished, None, 3, 0, 10)
    assert torch.equal(toks3, expect)
    # ties -> lowest index; all -inf -> 0
    t = torch.zeros(2, 6); t[0, 2] = t[0, 4] = 1.0; t[1, :] = float("-inf")
    toks4, _ = oracle.greedy_advance(t, None, None, 0, 0, 10)
    assert toks4.tolist() == [2, 0]


def test_philox_known_answers():
    """Known-answer vectors of Philox4x32-10 from the Random123 distribution (kat_vectors)."""
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
        ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
        ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
         [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
    ]
    for ctr, key, want in kat:
        assert oracle.philox4x32_10(ctr, key) == want


def test_sample_scores_distribution():
    """argmax of the oracle's scores is a draw from softmax(logits / T): frequencies over many
    (row, step) streams match the probabilities (a wrong sign or a missing log would not)."""
    logits = torch.tensor([2.0, 1.0, 0.0, -1.0, float("-inf"), 0.5])
    temp = 0.7
    probs = torch.softmax(logits.double() / temp, -1)
    counts = torch.zeros(6)
    n = 3000
    for i in range(n):
        counts[int(oracle.sample_scores(logits, temp, seed=1234, row=i % 7, step=i // 7).argmax())] += 1
    freq = counts / n
    assert counts[4] == 0
    assert (freq - probs.float()).abs().max() < 4 * float((probs * (1 - probs) / n).sqrt().max()) + 1e-3
