"""CPU tests of the host-side layer API (no GPU): replace()/copy/finalize protocol, dispatch
rules, fused-QKV slicing, static-cache bookkeeping, RTN quantisers, replacement table.
They follow the reference's own test recipes (tests/test_linear.py, test_multilinear.py,
test_gateupdownmlp.py, test_rmsnorm.py, test_static_kvcache.py there): build a torch/HF
layer with seeded weights, replace it, feed batch-4 inputs and compare with
allclose(rtol 1e-4, atol 1e-1) -- plus tighter checks, since on CPU fp32 both sides run the
same torch ops."""

import copy

import pytest
import torch
import torch.nn as nn

import oracle
from muillm_amd import _hf
from muillm_amd.engine import init_engine
from muillm_amd.engineconfig import MuiEngineConfig
from muillm_amd.modules.gateupdownmlp import MuiGateUpDownMLP, _MuiGateUpSiLUMethod
from muillm_amd.modules.kvcache.cache_utils import (MuiStaticCache, _next_pow2, create_static_cache,
                                                    grow_static_cache_if_needed)
from muillm_amd.modules.linear import MuiLinear
from muillm_amd.modules.models.llama.model import MuiDecoderConfig, MuiLlamaForCausalLM
from muillm_amd.modules.multilinear import MuiMultiLinear
from muillm_amd.modules.norm.rmsnorm import MuiRMSNorm
from muillm_amd.modules.quantized.int8gateupdownmlp import MuiInt8GateUpDownMLP
from muillm_amd.modules.quantized.int8linear import MuiInt8Linear
from muillm_amd.quantization.quantizationmethod import Int8WeightOnlyQuantizationMethod
from muillm_amd.quantization.rtnquantizer import ChannelRTNQuantizer, RTNQuantizer
from muillm_amd.replacement.replacementcontext import MuiReplacementContext
from muillm_amd.replacement.replacements import replace_layers
from tests.util import reference_allclose


@pytest.fixture(scope="module")
def ctx():
    cfg = MuiEngineConfig()
    return MuiReplacementContext(cfg, model=None, device="cpu")


def random_linear(in_features, out_features, bias=True, seed=0):
    torch.manual_seed(seed)
    lin = nn.Linear(in_features, out_features, bias=bias)
    lin.weight.data = torch.randn(out_features, in_features) * 0.05
    return lin


class TinyRMSNorm(nn.Module):
    """HF LlamaRMSNorm's definition, for when transformers is not importable."""

    def __init__(self, n, eps=1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(n))
        self.variance_epsilon = eps

    def forward(self, x):
        h = x.to(torch.float32)
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * h.to(x.dtype)


def make_norm(n, eps=1e-5, seed=0):
    torch.manual_seed(seed)
    if _hf.HAVE_TRANSFORMERS:
        m = _hf.LlamaRMSNorm(n, eps=eps)
    else:
        m = TinyRMSNorm(n, eps)
    m.weight.data = 1 + 0.1 * torch.randn(n)
    return m


def test_engine_config_rejects_tensor_parallelism():
    with pytest.raises(ValueError):
        MuiEngineConfig(tensor_parallelism=2)
    assert MuiEngineConfig().is_rank0()


@pytest.mark.parametrize("bias", [True, False])
def test_linear_replace_cpu_fp32(ctx, bias):
    lin = random_linear(256, 128, bias)
    mui = MuiLinear.replace(ctx, copy.deepcopy(lin))
    mui.finalize_init()
    x = torch.rand(4, 256)
    y, ref = mui(x), lin(x)
    assert reference_allclose(y, ref) and torch.allclose(y, ref, atol=1e-5)
    r = torch.rand(4, 128)
    assert torch.allclose(mui(x, residual=r), ref + r, atol=1e-5)
    assert MuiLinear.replace(ctx, mui) is mui  # idempotent


def test_linear_replace_with_norm_keeps_epsilon(ctx):
    lin, norm = random_linear(256, 128, False), make_norm(256, eps=1e-3)
    mui = MuiLinear.replace(ctx, copy.deepcopy(lin), prev_layernorm_module=copy.deepcopy(norm))
    mui.finalize_init()
    assert mui.normalize and mui.variance_epsilon == 1e-3  # the reference resets this to 0
    x = torch.rand(4, 256)
    assert torch.allclose(mui(x), lin(norm(x)), atol=1e-5)
    assert torch.allclose(mui(x).double(), oracle.linear(x, lin.weight.data, norm.weight.data, 1e-3), atol=1e-5)
    with pytest.raises(ValueError):
        MuiLinear.replace(ctx, mui, prev_layernorm_module=norm)  # norm given twice


def test_multilinear_matches_separate_linears(ctx):
    lins = [random_linear(256, n, False, seed=i) for i, n in enumerate((128, 64, 64))]
    norm = make_norm(256)
    mui = MuiMultiLinear.replace(ctx, [copy.deepcopy(l) for l in lins], prev_layernorm_module=copy.deepcopy(norm))
    mui.finalize_init()
    x = torch.rand(4, 256)
    outs = mui(x)
    assert [o.shape[-1] for o in outs] == [128, 64, 64]
    for o, l in zip(outs, lins):
        assert torch.allclose(o, l(norm(x)), atol=1e-5)
    back, nw = mui.replace_back()
    for b, l in zip(back, lins):
        assert torch.equal(b.weight, l.weight)
    assert torch.equal(nw, norm.weight)
    mixed = [random_linear(256, 8, True), random_linear(256, 8, False)]
    with pytest.raises(ValueError):
        MuiMultiLinear.replace(ctx, mixed)


def test_rmsnorm_replace(ctx):
    norm = make_norm(256, eps=1e-6)
    mui = MuiRMSNorm.replace(ctx, copy.deepcopy(norm))
    x = torch.rand(4, 256)
    assert torch.allclose(mui(x), norm(x), atol=1e-6)
    assert torch.allclose(mui(x).double(), oracle.rmsnorm(x, norm.weight.data, 1e-6), atol=1e-5)
    assert MuiRMSNorm.replace(ctx, mui) is mui


class TinyMLP(nn.Module):
    def __init__(self, hid, inter, seed=0):
        super().__init__()
        torch.manual_seed(seed)
        self.gate_proj = nn.Linear(hid, inter, bias=False)
        self.up_proj = nn.Linear(hid, inter, bias=False)
        self.down_proj = nn.Linear(inter, hid, bias=False)
        self.act_fn = nn.SiLU()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


@pytest.mark.parametrize("method", list(_MuiGateUpSiLUMethod))
def test_mlp_replace(ctx, method):
    mlp, norm = TinyMLP(128, 384), make_norm(128)
    mui = MuiGateUpDownMLP.replace(ctx, copy.deepcopy(mlp), prev_layernorm_module=copy.deepcopy(norm))
    mui.finalize_init()
    mui.method = method
    x, r = torch.rand(4, 128), torch.rand(4, 128)
    ref = mlp(norm(x)) + r
    assert torch.allclose(mui(x, residual=r), ref, atol=1e-5)
    assert torch.allclose(mui(x, residual=r).double(),
                          oracle.gateupdown_mlp(x, mlp.gate_proj.weight.data, mlp.up_proj.weight.data,
                                                mlp.down_proj.weight.data, norm.weight.data, 1e-5, r), atol=1e-5)


def test_next_pow2():
    assert [_next_pow2(x) for x in (0, 1, 2, 3, 64, 65, 288)] == [1, 1, 2, 4, 64, 128, 512]
    with pytest.raises(ValueError):
        _next_pow2(-1)


def test_static_cache_semantics_cpu():
    """tests/test_static_kvcache.py:28-112 of the reference on CPU tensors."""
    cfg = MuiDecoderConfig(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=2,
                           max_position_embeddings=256)
    cache = create_static_cache(MuiEngineConfig(), cfg, max_batch_size=2, seq_len=70, device="cpu", dtype=torch.float32)
    assert isinstance(cache, MuiStaticCache) and cache.get_max_length() == 128 and len(cache) == 2
    assert cache.key_cache[0].shape == (2, 1, 128, 128) and not cache.key_cache[0].any()
    ks, seen = [], 0
    for t in [64] + [1] * 16:
        cp = torch.arange(seen, seen + t)
        for layer in range(2):
            k, v = torch.randn(2, 1, t, 128), torch.randn(2, 1, t, 128)
            ko, vo = cache.update(k, v, layer, {"cache_position": cp})
            if layer == 0:
                ks.append(k)
                seen += t
                assert torch.equal(ko, torch.cat(ks, dim=2))
            assert ko.shape[2] == seen
        assert cache.get_seq_length() == seen
    grow_static_cache_if_needed(cache, 200, 256)
    assert cache.get_max_length() == 256 and torch.equal(cache.key_cache[0][:, :, :seen], torch.cat(ks, dim=2))
    assert not cache.key_cache[0][:, :, seen:].any()
    grow_static_cache_if_needed(cache, 1000, 256)  # capped at the model's maximum
    assert cache.get_max_length() == 256
    cache.reset()
    assert cache.get_seq_length() == 0 and not cache.key_cache[1].any()


# ------------------------------------------------------------------------------------
# quantisers
# ------------------------------------------------------------------------------------
def test_group_rtn_quantizer_matches_oracle_and_bounds():
    torch.manual_seed(0)
    w = (torch.randn(64, 512) * 0.02).half()
    q, smv = RTNQuantizer(groupsize=128).group_quantize_tensor(w)
    qo, smvo = oracle.rtn_quantize_group(w, 128)
    assert torch.equal(q, qo) and torch.equal(smv, smvo)
    assert q.dtype == torch.uint8 and smv.shape == (64 * 4, 2) and smv.dtype == torch.float16
    dq = RTNQuantizer(groupsize=128).group_dequantize_tensor(q, smv, torch.float16)
    err = (dq.float() - w.float()).abs().reshape(-1, 128)
    assert bool((err <= smv[:, :1].float() * 0.5 + 2e-4).all())  # half a step (+ fp16 rounding of scale/min)
    g = w.reshape(-1, 128).float()
    assert bool((q.reshape(-1, 128)[torch.arange(256), g.argmin(1)] == 0).all())
    assert bool((q.reshape(-1, 128)[torch.arange(256), g.argmax(1)] == 255).all())
    with pytest.raises(ValueError):
        RTNQuantizer(groupsize=100)
    with pytest.raises(ValueError):
        RTNQuantizer(groupsize=128).group_quantize_tensor(torch.zeros(4, 100))


def test_channel_rtn_quantizer():
    torch.manual_seed(1)
    w = (torch.randn(32, 256) * 0.02).half()
    w[3] = 0
    q, s = ChannelRTNQuantizer().quantize_tensor(w)
    qo, so = oracle.rtn_quantize_channel(w)
    assert torch.equal(q, qo) and torch.equal(s, so)
    assert q.dtype == torch.int8 and int(q.abs().max()) <= 127
    rows = torch.arange(32)
    amax_idx = w.float().abs().argmax(1)
    assert bool((q[rows, amax_idx].abs()[w.float().abs().amax(1) > 0] == 127).all())  # row max -> +-127
    dq = ChannelRTNQuantizer().dequantize_tensor(q, s)
    assert torch.equal(dq, oracle.rtn_dequantize_channel(q, s))
    # half a step, plus the fp16 rounding of the dequantised value and of the scale itself
    assert bool(((dq.float() - w.float()).abs() <= s.float()[:, None] * 0.5 + w.float().abs() * 2.0 ** -9 + 1e-7).all())
    assert not q[3].any()


def test_int8_modules_cpu(ctx):
    for gs in (0, 64):
        qm = Int8WeightOnlyQuantizationMethod(group_size=gs)
        qctx = MuiReplacementContext(MuiEngineConfig(qm), model=None, device="cpu")
        lin = random_linear(256, 128, True)
        ql = MuiInt8Linear.replace(qctx, MuiLinear.replace(ctx, copy.deepcopy(lin)))
        x = torch.rand(4, 256)
        assert oracle.rel_err(ql(x), lin(x).double()) < 2e-2
        mlp, norm = TinyMLP(128, 384), make_norm(128)
        mui = MuiGateUpDownMLP.replace(ctx, copy.deepcopy(mlp), prev_layernorm_module=copy.deepcopy(norm))
        qmlp = MuiInt8GateUpDownMLP.replace(qctx, mui)
        xx, r = torch.rand(4, 128), torch.rand(4, 128)
        assert oracle.rel_err(qmlp(xx, residual=r), (mlp(norm(xx)) + r).double()) < 2e-2
        assert qmlp.gate_up_weights.shape == (384, 2, 128)


# ------------------------------------------------------------------------------------
# replacement table / init_engine on a whole (tiny) HuggingFace model, CPU fp32
# ------------------------------------------------------------------------------------
@pytest.mark.skipif(not _hf.HAVE_TRANSFORMERS, reason="transformers not installed")
@pytest.mark.parametrize("family", ["llama", "mistral"])
def test_init_engine_on_hf_model_cpu(family):
    torch.manual_seed(0)
    kw = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
              num_key_value_heads=1, vocab_size=320, max_position_embeddings=128, rms_norm_eps=1e-5)
    if family == "llama":
        hf = _hf.LlamaForCausalLM(_hf.LlamaConfig(**kw))
    else:
        hf = _hf.MistralForCausalLM(_hf.MistralConfig(**kw, sliding_window=None))
    hf.eval()
    ids = torch.randint(0, 320, (2, 12))
    with torch.no_grad():
        ref = hf(input_ids=ids, use_cache=False).logits
    model = init_engine(copy.deepcopy(hf), device="cpu")
    assert isinstance(model, MuiLlamaForCausalLM)
    names = {type(m).__name__ for m in model.modules()}
    assert {"MuiDecoderLayer", "MuiMultiLinear", "MuiSdpaAttention", "MuiGateUpDownMLP", "MuiRMSNorm", "MuiLinear"} <= names
    assert not any(isinstance(m, (_hf.LlamaDecoderLayer, _hf.MistralDecoderLayer)) for m in model.modules())
    with torch.no_grad():
        out = model(input_ids=ids)
    assert torch.allclose(out.logits, ref, atol=2e-4, rtol=1e-4)
    # prefill + 3 single-token steps through the static cache equal the full forward
    with torch.no_grad():
        cache = model(input_ids=ids[:, :9]).past_key_values
        assert isinstance(cache, MuiStaticCache) and cache.get_seq_length() == 9
        for t in range(9, 12):
            step = model(input_ids=ids[:, t : t + 1], past_key_values=cache)
            assert torch.allclose(step.logits[:, 0], ref[:, t], atol=3e-4, rtol=1e-4)
        assert cache.get_seq_length() == 12


def test_replace_layers_leaves_unknown_modules(ctx):
    class Odd(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(16, 16)
            self.act = nn.GELU()
            self.keep = nn.Linear(16, 16)
            self.keep._muillm_no_further_replacement = True

    m = Odd()
    out = replace_layers(m, MuiReplacementContext(ctx.engine_config, m, "cpu"))
    assert isinstance(out.lin, MuiLinear) and isinstance(out.act, nn.GELU) and type(out.keep) is nn.Linear


# ------------------------------------------------------------------------------------
# guards of the decode loop (host logic; nothing here provokes an out-of-range read)
# ------------------------------------------------------------------------------------
def _tiny_lm(max_pos=32, **extra):
    cfg = MuiDecoderConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                           num_key_value_heads=1, vocab_size=64, max_position_embeddings=max_pos)
    for k, v in extra.items():
        setattr(cfg, k, v)
    return MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float32, device="cpu", seed=0,
                                           init_std=0.05)


def test_forward_refuses_positions_beyond_the_rotary_tables():
    lm = _tiny_lm(max_pos=32)
    ids = torch.randint(0, 64, (1, 30))
    with torch.no_grad():
        out = lm(input_ids=ids)
        lm(input_ids=ids[:, :2], past_key_values=out.past_key_values)      # 32 tokens: the last table row
        with pytest.raises(ValueError, match="rotary positions"):
            lm(input_ids=ids[:, :1], past_key_values=out.past_key_values)  # 33rd token
        with pytest.raises(ValueError, match="rotary positions"):
            lm(input_ids=torch.randint(0, 64, (1, 33)))


def test_forward_refuses_a_batch_larger_than_the_cache():
    lm = _tiny_lm()
    cache = create_static_cache(MuiEngineConfig(), lm.config, max_batch_size=1, seq_len=16, device="cpu",
                                dtype=torch.float32)
    with torch.no_grad(), pytest.raises(ValueError, match="max_batch_size"):
        lm(input_ids=torch.randint(0, 64, (2, 4)), past_key_values=cache)


@pytest.mark.skipif(not _hf.HAVE_TRANSFORMERS, reason="transformers not installed")
def test_sliding_window_matches_hf_mistral_and_the_oracle():
    """A Mistral config with sliding_window=8 on 20 tokens: the converted model's full forward (mask
    route) and its prefill + single-token steps across the window's edge give HuggingFace's logits;
    the oracle's sliding mask gives them too (which pins it for the GPU tests)."""
    torch.manual_seed(0)
    kw = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
              num_key_value_heads=1, vocab_size=320, max_position_embeddings=128, rms_norm_eps=1e-5)
    hf = _hf.MistralForCausalLM(_hf.MistralConfig(**kw, sliding_window=8)).eval()
    hf_full = _hf.MistralForCausalLM(_hf.MistralConfig(**kw, sliding_window=None)).eval()
    hf_full.load_state_dict(hf.state_dict())
    ids = torch.randint(0, 320, (2, 20))
    with torch.no_grad():
        ref = hf(input_ids=ids, use_cache=False).logits
        ref_full = hf_full(input_ids=ids, use_cache=False).logits
    assert float((ref - ref_full)[:, 8:].abs().max()) > 1e-3  # the window does change the result here
    assert torch.allclose(ref[:, :8], ref_full[:, :8], atol=1e-5)
    model = init_engine(copy.deepcopy(hf), device="cpu")
    with torch.no_grad():
        out = model(input_ids=ids)
        assert torch.allclose(out.logits, ref, atol=3e-4, rtol=1e-4)
        cache = model(input_ids=ids[:, :5]).past_key_values
        for t in range(5, 20):
            step = model(input_ids=ids[:, t : t + 1], past_key_values=cache)
            assert torch.allclose(step.logits[:, 0], ref[:, t], atol=3e-4, rtol=1e-4), t
    # the oracle with the same window
    sd = {k: v.double() for k, v in hf.state_dict().items()}
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
    cos, sin = oracle.rope_tables(_hf.rope_theta_of(hf.config), 128, 32)
    mk = lambda: [torch.zeros(2, 1, 32, 128, dtype=torch.float64) for _ in range(2)]
    kc, vc = mk(), mk()
    lg, seen = oracle.decoder_model_step(ids, params, kc, vc, cos, sin, 0, 2, 1, store_dtype=torch.float64, sliding_window=8)
    assert torch.allclose(lg, ref.double(), atol=2e-4)
    kc, vc = mk(), mk()
    lg, seen = oracle.decoder_model_step(ids[:, :5], params, kc, vc, cos, sin, 0, 2, 1, store_dtype=torch.float64, sliding_window=8)
    for t in range(5, 20):
        lg, seen = oracle.decoder_model_step(ids[:, t : t + 1], params, kc, vc, cos, sin, seen, 2, 1,
                                             store_dtype=torch.float64, sliding_window=8)
        assert torch.allclose(lg[:, 0], ref[:, t].double(), atol=2e-4), t


def test_reusable_cache_never_touches_a_callers_cache():
    """generate(ids, cache=mine) followed by generate(other_ids) must not reset or reuse `mine`: only a
    cache the decoder created itself is recycled."""
    from muillm_amd.modules.models.graphdecoder import MuiGraphDecoder

    lm = _tiny_lm(max_pos=64)
    dec = MuiGraphDecoder(lm, use_graph=False)
    mine = create_static_cache(MuiEngineConfig(), lm.config, max_batch_size=1, seq_len=16, device="cpu", dtype=torch.float32)
    ids = torch.randint(0, 64, (1, 4))
    dec.cache, dec.owns_cache = mine, False  # what prefill(ids, n, cache=mine) records
    assert MuiLlamaForCausalLM._reusable_cache(dec, None, ids) is None
    dec.owns_cache = True  # a cache prefill() created itself is recycled (emptied)
    mine._seen_tokens = 5
    assert MuiLlamaForCausalLM._reusable_cache(dec, None, ids) is mine and mine.get_seq_length() == 0
    other = create_static_cache(MuiEngineConfig(), lm.config, max_batch_size=1, seq_len=16, device="cpu", dtype=torch.float32)
    assert MuiLlamaForCausalLM._reusable_cache(dec, other, ids) is other


def test_graph_decoder_prefill_guards_and_capture_key():
    """MuiGraphDecoder.prefill refuses, before any kernel runs, what the rotary tables or the cache
    cannot hold; the key of a captured step changes when the cache is re-allocated. (The decode
    loop itself needs the GPU kernels: its continuation test lives in test_modules_gpu.py.)"""
    from muillm_amd.modules.models.graphdecoder import MuiGraphDecoder

    lm = _tiny_lm(max_pos=64)
    dec = MuiGraphDecoder(lm, use_graph=False)
    ids = torch.randint(0, 64, (1, 6))
    with pytest.raises(ValueError, match="rotary positions"):
        dec.prefill(ids, 60)
    cache = create_static_cache(MuiEngineConfig(), lm.config, max_batch_size=1, seq_len=8, device="cpu",
                                dtype=torch.float32)
    with pytest.raises(ValueError, match="max_batch_size"):
        dec.prefill(torch.randint(0, 64, (2, 6)), 4, cache=cache)
    with torch.no_grad():
        lm(input_ids=ids, past_key_values=cache)                            # the cache now holds 6 tokens
    with pytest.raises(ValueError, match="rotary positions"):
        dec.prefill(ids, 53, cache=cache)                                   # 6 + 6 + 53 > 64
    with pytest.raises(ValueError, match="empty cache"):
        dec.prefill(ids, 2, cache=cache, attention_mask=torch.tensor([[0, 1, 1, 1, 1, 1]]))
    dec.cache, dec._batch, dec.mask4d = cache, 1, None
    before = dec._capture_key()
    assert dec._capture_key() == before
    cache.grow_cache(20, 64)                                                # 8 -> 32 slots: new tensors
    after = dec._capture_key()
    assert after != before, "a re-allocated cache must invalidate a captured step"
    dec.mask4d = torch.zeros(1, 1, 1, 32)
    assert dec._capture_key() != after                                      # a padding mask is part of the step
    dec._batch = 2
    assert dec._capture_key()[1] == 2
