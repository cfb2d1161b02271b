"""GPU tests of the layer classes, decoder layer, whole-model harness, int8 quantisation and
the HIP-graph decode loop, against the CPU oracle and (where importable) HuggingFace's own
layers on the same device."""

import copy

import pytest
import torch
import torch.nn as nn

import oracle
from muillm_amd import _hf
from muillm_amd.engine import init_engine
from muillm_amd.engineconfig import MuiEngineConfig
from muillm_amd.modules.gateupdownmlp import MuiGateUpDownMLP
from muillm_amd.modules.kvcache.cache_utils import MuiStaticCache, create_static_cache
from muillm_amd.modules.linear import MuiLinear
from muillm_amd.modules.models.graphdecoder import MuiGraphDecoder
from muillm_amd.modules.models.llama.model import MuiDecoderConfig, MuiLlamaForCausalLM
from muillm_amd.modules.multilinear import MuiMultiLinear
from muillm_amd.modules.norm.rmsnorm import MuiRMSNorm
from muillm_amd.modules.quantized.int8gateupdownmlp import MuiInt8GateUpDownMLP
from muillm_amd.modules.quantized.int8linear import MuiInt8Linear
from muillm_amd.quantization.quantizationmethod import Int8WeightOnlyQuantizationMethod
from muillm_amd.replacement.replacementcontext import MuiReplacementContext
from tests.util import assert_parity, reference_allclose

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ctx():
    return MuiReplacementContext(MuiEngineConfig(), model=None, device=DEV)


def test_engine_reports_gfx950(ctx):
    info = ctx.engine_config.cpp_engine.info
    assert info["is_gfx950"] == 1 and info["wave_size"] == 64 and info["compute_units"] >= 64


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tokens", [1, 4, 32])
def test_linear_module(ctx, dtype, tokens):
    """tests/test_linear.py of the reference (batch 4) plus the single-token and prefill cases."""
    torch.manual_seed(0)
    lin = nn.Linear(2048, 1024, bias=True).to(dtype)
    lin.weight.data = (torch.randn(1024, 2048) * 0.05).to(dtype)
    mui = MuiLinear.replace(ctx, copy.deepcopy(lin))
    mui.finalize_init()
    x = torch.rand(tokens, 2048).to(dtype)
    r = torch.rand(tokens, 1024).to(dtype)
    y = mui(x.to(DEV), residual=r.to(DEV))
    ref = oracle.linear(x, lin.weight.data, bias=lin.bias.data, residual=r)
    assert reference_allclose(y, ref)
    assert_parity(y, ref, 1e-2, f"MuiLinear {dtype} b={tokens}")


def test_multilinear_and_mlp_modules(ctx):
    torch.manual_seed(1)
    hid, inter = 512, 1536
    norm_w = (1 + 0.1 * torch.randn(hid)).half()

    class Norm(nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = nn.Parameter(norm_w.clone())
            self.variance_epsilon = 1e-5

    lins = []
    for n in (512, 128, 128):
        l = nn.Linear(hid, n, bias=False).half()
        l.weight.data = (torch.randn(n, hid) * 0.02).half()
        lins.append(l)
    qkv = MuiMultiLinear.replace(ctx, [copy.deepcopy(l) for l in lins], prev_layernorm_module=Norm())
    qkv.finalize_init()
    x = torch.randn(1, 1, hid).half()
    q, k, v = qkv(x.to(DEV))
    refs = oracle.multilinear(x, [l.weight.data for l in lins], norm_w, 1e-5)
    for got, ref in zip((q, k, v), refs):
        assert_parity(got, ref, 1e-2, "fused QKV slice", tight=4e-3)
    assert q.shape == (1, 1, 512) and k.shape == (1, 1, 128) and not k.is_contiguous() or k.shape[-1] == 128

    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj = nn.Linear(hid, inter, bias=False).half()
            self.up_proj = nn.Linear(hid, inter, bias=False).half()
            self.down_proj = nn.Linear(inter, hid, bias=False).half()
            self.act_fn = nn.SiLU()
            for l in (self.gate_proj, self.up_proj, self.down_proj):
                l.weight.data = (torch.randn_like(l.weight.float()) * 0.02).half()

    mlp = MLP()
    wg, wu, wd = (mlp.gate_proj.weight.data.clone(), mlp.up_proj.weight.data.clone(), mlp.down_proj.weight.data.clone())
    mui = MuiGateUpDownMLP.replace(ctx, mlp, prev_layernorm_module=Norm())
    mui.finalize_init()
    # the repack aliases gate/up onto one interleaved buffer without changing their values
    assert mui.gate_up_packed.shape == (inter, 2, hid)
    assert mui.gate_proj.weight.data_ptr() == mui.gate_up_packed.data_ptr()
    assert mui.up_proj.weight.data_ptr() == mui.gate_up_packed.data_ptr() + hid * 2
    assert torch.equal(mui.gate_proj.weight.cpu(), wg) and torch.equal(mui.up_proj.weight.cpu(), wu)
    for tokens in (1, 4, 32):  # fused kernel, small batch, and the unfused prefill route
        xx = torch.randn(tokens, hid).half()
        rr = torch.randn(tokens, hid).half()
        out = mui(xx.to(DEV), residual=rr.to(DEV))
        assert_parity(out, oracle.gateupdown_mlp(xx, wg, wu, wd, norm_w, 1e-5, rr), 1e-2, f"MuiGateUpDownMLP b={tokens}")


@pytest.mark.parametrize("tokens", [17, 100])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mlp_module_long_prompt_route(ctx, tokens, dtype):
    """More tokens than the fused GEMV family takes: one matmul over the interleaved gate/up rows,
    the SiLU*mul kernel, residual in the down projection's epilogue."""
    torch.manual_seed(11)
    hid, inter = 256, 704
    mlp = MuiGateUpDownMLP(MuiEngineConfig(), hid, inter, torch.nn.SiLU(), variance_epsilon=1e-5, normalize=True,
                           device=DEV, dtype=dtype)
    with torch.no_grad():
        for lin in (mlp.gate_proj, mlp.up_proj, mlp.down_proj):
            lin.weight.copy_(torch.randn_like(lin.weight) * 0.05)
        mlp.norm_weights.copy_(1 + 0.1 * torch.randn_like(mlp.norm_weights))
    mlp.finalize_init()
    assert mlp.gate_up_packed is not None
    x = torch.randn(2, tokens, hid, device=DEV, dtype=dtype)
    r = torch.randn(2, tokens, hid, device=DEV, dtype=dtype)
    ref = oracle.gateupdown_mlp(x.cpu(), mlp.gate_proj.weight.detach().cpu(), mlp.up_proj.weight.detach().cpu(),
                     mlp.down_proj.weight.detach().cpu(), mlp.norm_weights.detach().cpu(), 1e-5, r.cpu())
    with torch.no_grad():
        y = mlp(x, residual=r)
    assert y.shape == x.shape
    assert_parity(y, ref, 1e-2, f"long-prompt MLP {tokens}")


def _small_config(layers=2):
    return MuiDecoderConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=layers,
                            num_attention_heads=4, num_key_value_heads=2, vocab_size=1024,
                            max_position_embeddings=256, rope_theta=500000.0, rms_norm_eps=1e-5)


def _oracle_params(lm):
    """Weights of a MuiLlamaForCausalLM as CPU tensors in the oracle's layout."""
    cfg = lm.config
    d = cfg.hidden_size // cfg.num_attention_heads
    hq, hkv = cfg.num_attention_heads, cfg.num_key_value_heads
    layers = []
    for layer in lm.model.layers:
        w = layer.qkv_proj.linear.weight.detach().cpu()
        layers.append(dict(
            ln1=layer.qkv_proj.linear.norm_weights.detach().cpu(), wq=w[: hq * d], wk=w[hq * d : (hq + hkv) * d],
            wv=w[(hq + hkv) * d :], wo=layer.self_attn.o_proj.weight.detach().cpu(),
            ln2=layer.mlp.norm_weights.detach().cpu(), wg=layer.mlp.gate_proj.weight.detach().cpu(),
            wu=layer.mlp.up_proj.weight.detach().cpu(), wd=layer.mlp.down_proj.weight.detach().cpu(),
            eps=cfg.rms_norm_eps))
    return dict(embed=lm.model.embed_tokens.weight.detach().cpu(), layers=layers,
                norm=lm.model.norm.weight.detach().cpu(), lm_head=lm.lm_head.weight.detach().cpu(),
                eps=cfg.rms_norm_eps)


def test_model_prefill_and_decode_vs_oracle():
    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=0,
                                         init_std=0.05)
    params = _oracle_params(lm)
    d = 128
    cos, sin = oracle.rope_tables(cfg.rope_theta, d, cfg.max_position_embeddings)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size, (2, 12), generator=g)
    cap = 64
    kcs = [torch.zeros(2, 2, cap, d, dtype=torch.float16) for _ in range(2)]
    vcs = [torch.zeros(2, 2, cap, d, dtype=torch.float16) for _ in range(2)]
    ref_logits, seen = oracle.decoder_model_step(ids, params, kcs, vcs, cos, sin, 0, 4, 2)
    with torch.no_grad():
        out = lm(input_ids=ids.to(DEV))
    assert out.logits.dtype == torch.float32 and out.logits.shape == (2, 12, cfg.vocab_size)
    assert_parity(out.logits, ref_logits, 1e-2, "prefill logits")
    cache = out.past_key_values
    assert isinstance(cache, MuiStaticCache) and cache.get_seq_length() == 12 and cache.get_max_length() == 16
    # greedy decode, one token at a time, against the oracle on its own growing cache
    nxt = ref_logits[:, -1].argmax(-1)
    for step in range(6):
        ref_logits, seen = oracle.decoder_model_step(nxt.unsqueeze(1), params, kcs, vcs, cos, sin, seen, 4, 2)
        with torch.no_grad():
            out = lm(input_ids=nxt.unsqueeze(1).to(DEV), past_key_values=cache)
        assert_parity(out.logits, ref_logits, 1e-2, f"decode step {step}")
        assert cache.get_seq_length() == seen
        nxt = ref_logits[:, -1].argmax(-1)
    assert cache.get_max_length() == 32  # grew by the power-of-two schedule


def test_model_three_query_heads_per_kv_head_and_chunked_prompt():
    """A 6 / 2-head decoder (ratio 3, as in Llama-3.2-3B) with a 17-token prompt (the fused linears
    run in two chunks): prefill and greedy decode against the oracle, through the layer modules and
    through the single-call stack."""
    cfg = MuiDecoderConfig(hidden_size=768, intermediate_size=1536, num_hidden_layers=2, num_attention_heads=6,
                           num_key_value_heads=2, vocab_size=512, max_position_embeddings=256,
                           rope_theta=500000.0, rms_norm_eps=1e-5)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=7,
                                         init_std=0.05)
    params = _oracle_params(lm)
    d = 128
    cos, sin = oracle.rope_tables(cfg.rope_theta, d, cfg.max_position_embeddings)
    ids = torch.randint(0, cfg.vocab_size, (1, 17), generator=torch.Generator().manual_seed(7))
    for use_stack in (False, True):
        lm.model.use_decoder_stack = use_stack
        kcs = [torch.zeros(1, 2, 64, d, dtype=torch.float16) for _ in range(2)]
        vcs = [torch.zeros(1, 2, 64, d, dtype=torch.float16) for _ in range(2)]
        ref_logits, seen = oracle.decoder_model_step(ids, params, kcs, vcs, cos, sin, 0, 6, 2)
        with torch.no_grad():
            out = lm(input_ids=ids.to(DEV))
        assert_parity(out.logits, ref_logits, 1e-2, "prefill logits (ratio 3)")
        cache = out.past_key_values
        nxt = ref_logits[:, -1].argmax(-1)
        for step in range(4):
            ref_logits, seen = oracle.decoder_model_step(nxt.unsqueeze(1), params, kcs, vcs, cos, sin, seen, 6, 2)
            with torch.no_grad():
                out = lm(input_ids=nxt.unsqueeze(1).to(DEV), past_key_values=cache)
            assert_parity(out.logits, ref_logits, 1e-2, f"decode step {step} (ratio 3, stack={use_stack})")
            nxt = ref_logits[:, -1].argmax(-1)
        assert (lm.model._stack is not None) == use_stack
    lm.model.use_decoder_stack = True


@pytest.mark.parametrize("batch", [1, 2])
def test_graph_decode_matches_eager(batch):
    cfg = _small_config(layers=3)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=1,
                                         init_std=0.05)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, cfg.vocab_size, (batch, 32), generator=g).to(DEV)
    n_new = 24
    eager, eager_logits = lm.generate_greedy(ids, n_new, use_graph=False, return_logits=True)
    dec = MuiGraphDecoder(lm, use_graph=True)
    graph, graph_logits = dec.generate(ids, n_new, return_logits=True)
    assert eager.shape == (batch, 32 + n_new)
    assert torch.equal(eager, graph), "graph replay and eager decode disagree"
    assert torch.equal(eager_logits, graph_logits)
    # a second generation on the same decoder re-uses the captured graph, with eager work and
    # synchronisations in between, and must reproduce the result exactly
    torch.cuda.synchronize()
    _ = lm(input_ids=ids[:, :5])
    torch.cuda.synchronize()
    dec.cache.reset()
    graph2 = dec.generate(ids, n_new, cache=dec.cache)
    assert torch.equal(graph2, eager)
    assert dec.cache.get_seq_length() == 32 + n_new - 1


@pytest.mark.parametrize("prompt_len", [8, 24])
def test_sliding_window_generation_both_launch_modes(prompt_len):
    """A Mistral-style config with sliding_window=16: generations that start inside the window and
    cross it (prompt 8) or start beyond it (prompt 24, whose prefill takes the masked route) give the
    oracle's windowed logits step by step, the same tokens and bit-identical logits from stream
    launches and from HIP-graph replay, and differ from the unwindowed model once the window is
    left (the reference's mistral/model.py:590-602)."""
    cfg = _small_config(layers=2)
    cfg.sliding_window = 16
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=11,
                                         init_std=0.05)
    params = _oracle_params(lm)
    d = 128
    cos, sin = oracle.rope_tables(cfg.rope_theta, d, cfg.max_position_embeddings)
    ids = torch.randint(0, cfg.vocab_size, (2, prompt_len), generator=torch.Generator().manual_seed(3))
    n_new = 20
    runs = []
    for use_graph in (False, True, None):
        dec = MuiGraphDecoder(lm, use_graph=use_graph)
        toks, logits = dec.generate(ids.to(DEV), n_new, return_logits=True)
        assert dec._window == 16 and dec.mask4d is not None
        runs.append((toks.cpu(), logits.cpu()))
    for toks, logits in runs[1:]:
        assert torch.equal(toks, runs[0][0]) and torch.equal(logits, runs[0][1])
    toks, logits = runs[0]
    # teacher-forced oracle over the generated sequence, with and without the window
    for window, must_match in ((16, True), (None, False)):
        kcs = [torch.zeros(2, 2, 64, d, dtype=torch.float16) for _ in range(2)]
        vcs = [torch.zeros(2, 2, 64, d, dtype=torch.float16) for _ in range(2)]
        ref, seen = oracle.decoder_model_step(toks[:, :prompt_len], params, kcs, vcs, cos, sin, 0, 4, 2, sliding_window=window)
        worst = oracle.rel_err(logits[:, 0], ref[:, -1])
        for step in range(1, n_new):
            ref, seen = oracle.decoder_model_step(toks[:, prompt_len + step - 1 : prompt_len + step], params, kcs, vcs,
                                                  cos, sin, seen, 4, 2, sliding_window=window)
            if must_match:
                assert_parity(logits[:, step], ref[:, 0], 1e-2, f"windowed decode step {step} (prompt {prompt_len})")
            worst = max(worst, oracle.rel_err(logits[:, step], ref[:, 0]))
        assert (worst <= 1e-2) == must_match, (window, worst)


def test_graph_decode_several_steps_per_replay():
    """decode() without stop checks or logits collection replays STEPS_PER_REPLAY steps per graph
    launch and finishes with single-step replays: tokens, the logits of the last step and the cache
    length must be those of the eager loop, for step counts on both sides of a multiple."""
    cfg = _small_config(layers=2)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=6,
                                         init_std=0.05)
    g = torch.Generator().manual_seed(7)
    ids = torch.randint(0, cfg.vocab_size, (2, 12), generator=g).to(DEV)
    k = MuiGraphDecoder.STEPS_PER_REPLAY
    for n_steps in (2 * k, 3 * k + 1, 2 * k - 1):
        results = []
        for use_graph in (False, True):
            dec = MuiGraphDecoder(lm, use_graph=use_graph)
            dec.prefill(ids, n_steps + 2)    # emits the first token
            dec.decode(1)
            dec.decode(n_steps)
            torch.cuda.synchronize()
            results.append((dec.out_tokens.clone(), dec.logits.clone(), dec.cache.get_seq_length(), dec))
        assert torch.equal(results[0][0], results[1][0]), n_steps
        assert torch.equal(results[0][1], results[1][1]), n_steps
        assert results[0][2] == results[1][2] == 12 + 1 + n_steps
        assert results[1][3].graph_multi is not None


def test_graph_decoder_reuse_after_cache_growth_and_multi_turn():
    """One decoder object, one cache object, a second generation that needs a larger cache: the
    cache tensors are re-allocated, so the captured step must be recorded again (a stale graph
    would read the old tensors). And a cache that already holds a first turn is continued, not
    overwritten: two turns == one generation over the concatenated prompt."""
    cfg = _small_config(layers=2)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=4,
                                         init_std=0.05)
    g = torch.Generator().manual_seed(5)
    short = torch.randint(0, cfg.vocab_size, (1, 8), generator=g).to(DEV)
    long_p = torch.randint(0, cfg.vocab_size, (1, 40), generator=g).to(DEV)
    dec = MuiGraphDecoder(lm, use_graph=True)
    first = dec.generate(short, 8)                          # capacity 16
    cache = dec.cache
    ptr = cache.key_cache[0].data_ptr()
    graph = dec.graph
    assert graph is not None
    cache.reset()
    second = dec.generate(long_p, 8, cache=cache)           # needs 48 slots: grows to 64, new tensors
    assert cache.key_cache[0].data_ptr() != ptr and cache.get_max_length() == 64
    assert dec.graph is not graph, "the graph captured on the old cache tensors was replayed"
    assert torch.equal(second, lm.generate_greedy(long_p, 8, use_graph=False))
    assert torch.equal(first, lm.generate_greedy(short, 8, use_graph=False))
    # same buffers again: the captured step is kept
    graph = dec.graph
    cache.reset()
    third = dec.generate(short, 8, cache=cache)
    assert dec.graph is graph and torch.equal(third, first)
    # multi-turn: the second prompt continues after the 8 + 8 - 1 tokens the cache holds
    turn2 = dec.generate(short, 6, cache=cache)
    assert cache.get_seq_length() == 15 + 8 + 6 - 1 and int(dec.cpos) == 15 + 8 + 6 - 1
    eager = MuiGraphDecoder(lm, use_graph=False)
    eager.generate(short, 8)                                # the same first turn, eagerly
    c2 = eager.cache
    with torch.no_grad():
        out = lm(input_ids=short, past_key_values=c2)       # second turn through plain forward calls
        toks = [out.logits[:, -1].argmax(-1)]
        for _ in range(5):
            out = lm(input_ids=toks[-1].unsqueeze(1), past_key_values=c2)
            toks.append(out.logits[:, -1].argmax(-1))
    assert torch.equal(turn2[:, 8:], torch.stack(toks, dim=1))
    # generate() keeps its decoder: the second call replays the first call's graph
    lm.generate(short, max_new_tokens=8)
    kept = lm._graph_decoder[1]
    g0 = kept.graph
    out = lm.generate(short, max_new_tokens=8)
    assert lm._graph_decoder[1] is kept and kept.graph is g0 and torch.equal(out, first)
    with pytest.raises(ValueError, match="rotary positions"):
        lm.generate(long_p, max_new_tokens=cfg.max_position_embeddings)


@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decoder_stack_call_matches_layer_modules(batch, dtype):
    """mui_decoder_stack_step (all layers in one C call) runs the same kernels in the same order
    as the layer modules: identical logits and cache contents, with and without padding masks,
    also after the cache has grown (the descriptor is rebuilt)."""
    cfg = _small_config(layers=3)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=dtype, device=DEV, seed=2, init_std=0.05)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, cfg.vocab_size, (batch, 11), generator=g).to(DEV)
    results = {}
    for use_stack in (False, True):
        lm.model.use_decoder_stack = use_stack
        out = lm(input_ids=ids)
        cache = out.past_key_values
        nxt = out.logits[:, -1].argmax(-1)
        logits = []
        for _ in range(9):  # crosses the 16 -> 32 capacity step
            out = lm(input_ids=nxt.unsqueeze(1), past_key_values=cache)
            logits.append(out.logits[:, -1].clone())
            nxt = out.logits[:, -1].argmax(-1)
        assert (lm.model._stack is not None) == use_stack or not use_stack
        results[use_stack] = (torch.stack(logits), [k.clone() for k in cache.key_cache],
                              [v.clone() for v in cache.value_cache], cache.get_seq_length())
    assert lm.model._stack is not None, "the single-call path did not engage"
    a, b2 = results[False], results[True]
    assert a[3] == b2[3] == 20
    assert torch.equal(a[0], b2[0])
    for x, y in zip(a[1] + a[2], b2[1] + b2[2]):
        assert torch.equal(x, y)
    # left-padded batch through generate(): same tokens with and without the single call
    if batch > 1:
        mask = torch.ones_like(ids)
        mask[0, :4] = 0
        toks = {}
        for use_stack in (False, True):
            lm.model.use_decoder_stack = use_stack
            toks[use_stack] = lm.generate(ids, attention_mask=mask, max_new_tokens=6, use_graph=False).cpu()
        assert torch.equal(toks[False], toks[True])
    lm.model.use_decoder_stack = True
    # a weight swapped after the descriptor was built is noticed (the descriptor is rebuilt)
    if batch == 1:
        out = lm(input_ids=ids)
        cache = out.past_key_values
        nxt = out.logits[:, -1].argmax(-1).unsqueeze(1)
        before = lm(input_ids=nxt, past_key_values=cache).logits.clone()
        old_stack = lm.model._stack
        mlp = lm.model.layers[1].mlp
        mlp.down_proj.weight = torch.nn.Parameter(torch.zeros_like(mlp.down_proj.weight), requires_grad=False)
        cache.reset()
        out = lm(input_ids=ids)
        after = lm(input_ids=nxt, past_key_values=out.past_key_values).logits
        assert lm.model._stack is not old_stack
        assert not torch.equal(before, after)
        lm.model.use_decoder_stack = False
        cache2 = lm(input_ids=ids).past_key_values
        ref = lm(input_ids=nxt, past_key_values=cache2).logits
        lm.model.use_decoder_stack = True
        assert torch.equal(after, ref)


@pytest.mark.parametrize("modules", [["qkv_proj", "o_proj", "mlp"], ["mlp"], ["o_proj"]])
@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("group_size", [0, 128])
def test_decoder_stack_call_int8_layers(modules, batch, group_size):
    """int8 projections -- per-channel (group_size 0) or the reference's group-wise (scale, min)
    format -- all of them, or only some (the rest stay fp16), go through the single call too: same
    logits and cache contents as the layer modules called one by one, and the same tokens from
    HIP-graph replay."""
    cfg = _small_config(layers=2)
    base = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=5,
                                           init_std=0.05, finalize=False)
    qm = Int8WeightOnlyQuantizationMethod(group_size=group_size, modules=modules)
    lm = init_engine(copy.deepcopy(base), device=DEV, engine_config=MuiEngineConfig(qm))
    g = torch.Generator().manual_seed(6)
    ids = torch.randint(0, cfg.vocab_size, (batch, 9), generator=g).to(DEV)
    results = {}
    with torch.no_grad():
        for use_stack in (False, True):
            lm.model.use_decoder_stack = use_stack
            out = lm(input_ids=ids)
            cache = out.past_key_values
            nxt = out.logits[:, -1].argmax(-1)
            logits = []
            for _ in range(5):
                out = lm(input_ids=nxt.unsqueeze(1), past_key_values=cache)
                logits.append(out.logits[:, -1].clone())
                nxt = out.logits[:, -1].argmax(-1)
            results[use_stack] = (torch.stack(logits), [k.clone() for k in cache.key_cache + cache.value_cache])
    assert lm.model._stack is not None, "the single-call path did not engage"
    assert torch.equal(results[False][0], results[True][0])
    for x, y in zip(results[False][1], results[True][1]):
        assert torch.equal(x, y)
    eager = lm.generate_greedy(ids, 6, use_graph=False)
    assert torch.equal(lm.generate_greedy(ids, 6, use_graph=True), eager)
    # a layer that mixes the two int8 formats keeps the per-layer calls (one descriptor, one format)
    if group_size and len(modules) == 3:
        mixed = init_engine(copy.deepcopy(base), device=DEV, engine_config=MuiEngineConfig(
            Int8WeightOnlyQuantizationMethod(group_size=0, modules=["o_proj"])))
        from muillm_amd.quantization.quantizedreplacements import quantize_layers
        mixed = quantize_layers(mixed, MuiEngineConfig(Int8WeightOnlyQuantizationMethod(group_size=128, modules=["mlp"])),
                                device=DEV)
        with torch.no_grad():
            out = mixed(input_ids=ids)
            mixed(input_ids=out.logits[:, -1].argmax(-1).unsqueeze(1), past_key_values=out.past_key_values)
        assert mixed.model._stack is None


def test_argmax_kernel():
    from muillm_amd import muillm_ext
    g = torch.Generator().manual_seed(2)
    for rows, v in ((1, 128256), (3, 1000), (2, 7), (1, 32000)):
        x = torch.randn(rows, v, generator=g).half().to(DEV)
        assert torch.equal(muillm_ext.mui_argmax(x).cpu(), x.float().argmax(-1).cpu())
    x = torch.zeros(2, 4096, dtype=torch.float16, device=DEV)
    x[0, 77] = x[0, 3000] = 5.0  # ties -> lowest index
    x[1, :] = float("-inf")
    out = muillm_ext.mui_argmax(x).cpu()
    assert out[0] == 77 and out[1] == 0
    xb = torch.randn(2, 5000, generator=g).bfloat16().to(DEV)[:, :4999]  # strided rows
    assert torch.equal(muillm_ext.mui_argmax(xb).cpu(), xb.float().argmax(-1).cpu())


def test_greedy_advance_kernel():
    """mui_greedy_advance against the oracle's restatement of argmax + stop check, over several
    consecutive steps on the same device-side state."""
    from muillm_amd import muillm_ext
    g = torch.Generator().manual_seed(3)
    B, V, max_steps = 5, 1000, 6
    eos = [17, 400]
    ids = torch.zeros(B, 1, dtype=torch.int64, device=DEV)
    pos = torch.full((B, 1), 40, dtype=torch.int64, device=DEV)
    cpos = torch.full((1,), 40, dtype=torch.int64, device=DEV)
    step = torch.zeros(B, dtype=torch.int64, device=DEV)
    toks = torch.full((B, max_steps), -1, dtype=torch.int64, device=DEV)
    unf = torch.ones(B, dtype=torch.int64, device=DEV)
    eos_t = torch.tensor(eos, dtype=torch.int64, device=DEV)
    ref_unf = torch.ones(B, dtype=torch.int64)
    for s_i in range(max_steps):
        logits = torch.randn(B, V, generator=g).half()
        if s_i == 1:
            logits[2, 17] = 50.0   # row 2 hits an eos token at step 1
        if s_i == 3:
            logits[4, 400] = 50.0  # row 4 at step 3
        muillm_ext.mui_greedy_advance(logits.to(DEV), ids, step, toks, position_ids=pos, cache_position=cpos,
                                      unfinished=unf, eos_token_ids=eos_t, pad_token_id=9)
        exp_tok, ref_unf = oracle.greedy_advance(logits, ref_unf, eos, 9, steps_done=s_i, max_steps=max_steps)
        assert torch.equal(toks[:, s_i].cpu(), exp_tok), s_i
        assert torch.equal(ids.cpu().view(-1), exp_tok)
        assert torch.equal(unf.cpu(), ref_unf), s_i
        assert int(cpos.item()) == 41 + s_i and torch.equal(pos.cpu().view(-1), torch.full((B,), 41 + s_i))
        assert torch.equal(step.cpu(), torch.full((B,), s_i + 1))
    assert toks[2, 2:].eq(9).all() and toks[4, 4:].eq(9).all()  # finished rows emit the pad token
    assert unf.sum().item() == 0                                   # the step budget finished the rest
    # one more call beyond the budget must not write outside tokens_out
    before = toks.clone()
    muillm_ext.mui_greedy_advance(torch.randn(B, V, generator=g).half().to(DEV), ids, step, toks)
    assert torch.equal(toks, before)
    # bf16, no optional state
    lg = torch.randn(2, 333, generator=g).bfloat16().to(DEV)
    ids2 = torch.zeros(2, dtype=torch.int64, device=DEV); st2 = torch.zeros(2, dtype=torch.int64, device=DEV)
    out2 = torch.zeros(2, 4, dtype=torch.int64, device=DEV)
    muillm_ext.mui_greedy_advance(lg, ids2, st2, out2)
    assert torch.equal(out2[:, 0].cpu(), lg.float().argmax(-1).cpu())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_greedy_advance_on_several_workgroups(dtype):
    """The workspace form (a long row scanned by several workgroups, candidates folded under a 64-bit
    atomic max) must choose the tokens of the plain form bit for bit -- ties to the lowest index also
    across workgroups, -0 equal to +0, NaN and -inf never chosen, rows without any candidate give
    token 0 -- step after step on one workspace, which every call leaves zero-filled."""
    from muillm_amd import muillm_ext
    g = torch.Generator().manual_seed(31)
    B, V, steps = 6, 128256, 4     # 16032 chunks: 16 workgroups per row
    ws = muillm_ext.greedy_workspace(B, DEV)
    assert ws.numel() == 16 * B and int(ws.sum()) == 0
    state = {}
    for name in ("plain", "ws"):
        state[name] = dict(ids=torch.zeros(B, 1, dtype=torch.int64, device=DEV), step=torch.zeros(B, dtype=torch.int64, device=DEV),
                           toks=torch.full((B, steps), -1, dtype=torch.int64, device=DEV),
                           pos=torch.full((B, 1), 7, dtype=torch.int64, device=DEV), cpos=torch.full((1,), 7, dtype=torch.int64, device=DEV),
                           unf=torch.ones(B, dtype=torch.int64, device=DEV))
    eos_t = torch.tensor([5], dtype=torch.int64, device=DEV)
    for s_i in range(steps):
        logits = torch.randn(B, V, generator=g).to(dtype)
        top = float(logits.float().max()) + 1.0
        logits[0, 100000] = top; logits[0, 2000] = top; logits[0, 70000] = top    # a tie across workgroups: 2000 wins
        logits[1] = float("-inf"); logits[1, 3] = float("nan")                      # nothing to choose: token 0
        logits[2] = float("nan"); logits[2, 127999] = -3.0                           # one candidate in the last workgroup
        logits[3] = -1.0; logits[3, 90000] = 0.0; logits[3, 40000] = -0.0            # -0 == +0: the lower index wins
        logits[4, 128255] = top                                                      # the very last element
        if s_i == 2:
            logits[5, 5] = top                                                       # row 5 stops on the eos token
        lg = logits.to(DEV)
        for name, w in (("plain", None), ("ws", ws)):
            st = state[name]
            muillm_ext.mui_greedy_advance(lg, st["ids"], st["step"], st["toks"], position_ids=st["pos"], cache_position=st["cpos"],
                                          unfinished=st["unf"], eos_token_ids=eos_t, pad_token_id=9, workspace=w)
        a, b = state["plain"], state["ws"]
        for key in a:
            assert torch.equal(a[key], b[key]), (key, s_i)
        tok = b["toks"][:, s_i].cpu()
        assert tok[0] == 2000 and tok[1] == 0 and tok[2] == 127999 and tok[3] == 40000 and tok[4] == 128255
        assert int(ws.sum()) == 0, "the workspace must be zero-filled again after every call"
    assert state["ws"]["unf"][5] == 0 and state["ws"]["toks"][5, 3] == 9
    # a short vocabulary, unaligned rows and a missing workspace fall back to one workgroup
    lg = torch.randn(2, 5000, generator=g).to(dtype).to(DEV)[:, :4999]
    ids2 = torch.zeros(2, dtype=torch.int64, device=DEV); st2 = torch.zeros(2, dtype=torch.int64, device=DEV)
    out2 = torch.zeros(2, 2, dtype=torch.int64, device=DEV)
    muillm_ext.mui_greedy_advance(lg, ids2, st2, out2, workspace=muillm_ext.greedy_workspace(2, DEV))
    assert torch.equal(out2[:, 0].cpu(), lg.float().argmax(-1).cpu())


def test_greedy_advance_leaves_the_embedding_row():
    """With an embedding table the launch that chooses the token also copies that token's row to
    embed_out (finished rows: the pad token's), in the single-workgroup form and in the workspace form."""
    from muillm_amd import muillm_ext
    g = torch.Generator().manual_seed(41)
    for dtype, V, H in ((torch.float16, 128256, 4096), (torch.bfloat16, 1000, 72), (torch.float16, 333, 13)):
        B = 3
        table = torch.randn(V, H, generator=g).to(dtype).to(DEV)
        logits = torch.randn(B, V, generator=g).to(dtype).to(DEV)
        logits[1, 7] = 100.0                                # row 1 chooses the eos token 7 ...
        for ws in (None, muillm_ext.greedy_workspace(B, DEV)):
            ids = torch.zeros(B, 1, dtype=torch.int64, device=DEV); step = torch.zeros(B, dtype=torch.int64, device=DEV)
            toks = torch.zeros(B, 2, dtype=torch.int64, device=DEV); unf = torch.ones(B, dtype=torch.int64, device=DEV)
            eos_t = torch.tensor([7], dtype=torch.int64, device=DEV)
            emb = torch.full((B, 1, H), 5.0, dtype=dtype, device=DEV)
            for s_i in range(2):
                muillm_ext.mui_greedy_advance(logits, ids, step, toks, unfinished=unf, eos_token_ids=eos_t, pad_token_id=2,
                                              workspace=ws, embed_table=table, embed_out=emb)
                assert torch.equal(emb[:, 0], table[ids.view(-1)]), (dtype, V, s_i)
            assert toks[1].tolist() == [7, 2]                # ... and emits the pad token (and its row) afterwards
            if ws is not None:
                assert int(ws.sum()) == 0
    with pytest.raises(RuntimeError):
        muillm_ext.mui_greedy_advance(logits, ids, step, toks, embed_table=table)


def test_generate_left_padded_batch_matches_single_runs():
    """Left-padded batch generation (static device-side mask + per-row rotary positions, graph
    replay) must give every row the tokens it gets when generated alone without padding."""
    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=8, init_std=0.08)
    g = torch.Generator().manual_seed(2)
    long_p = torch.randint(1, cfg.vocab_size, (1, 11), generator=g)
    short_p = torch.randint(1, cfg.vocab_size, (1, 6), generator=g)
    n_new = 10
    alone = [lm.generate(p.to(DEV), max_new_tokens=n_new)[0, p.shape[1]:].cpu() for p in (long_p, short_p)]
    batch = torch.zeros(2, 11, dtype=torch.int64)
    mask = torch.zeros(2, 11, dtype=torch.int64)
    batch[0], mask[0] = long_p[0], 1
    batch[1, 5:], mask[1, 5:] = short_p[0], 1
    for use_graph in (True, False):
        out = lm.generate(batch.to(DEV), attention_mask=mask.to(DEV), max_new_tokens=n_new, use_graph=use_graph).cpu()
        assert out.shape == (2, 11 + n_new)
        for r in range(2):
            got = out[r, 11:]
            # fp16 reduction order differs between batch sizes: allow a late divergence, not an early one
            agree = int((got == alone[r]).long().cumprod(0).sum())
            assert agree >= n_new - 2, (use_graph, r, got, alone[r])


def test_padded_prompt_runs_on_the_library_attention_kernel(monkeypatch):
    """A left-padded batch of prompts must not reach torch's scaled_dot_product_attention (the
    reference's route for masked prompts): the 2-D attention mask travels to the layers as a key
    padding mask and the library's prompt kernel applies it. Logits of the real tokens must match
    the rows run alone."""
    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=12, init_std=0.08)
    g = torch.Generator().manual_seed(4)
    long_p = torch.randint(1, cfg.vocab_size, (1, 40), generator=g)
    short_p = torch.randint(1, cfg.vocab_size, (1, 23), generator=g)
    with torch.no_grad():
        alone = [lm(input_ids=p.to(DEV)).logits[0, -1].float().cpu() for p in (long_p, short_p)]
    batch = torch.zeros(2, 40, dtype=torch.int64)
    mask = torch.zeros(2, 40, dtype=torch.int64)
    batch[0], mask[0] = long_p[0], 1
    batch[1, 17:], mask[1, 17:] = short_p[0], 1
    pos = (mask.cumsum(-1) - 1).clamp(min=0)

    def no_sdpa(*args, **kwargs):
        raise AssertionError("the padded prompt fell back to torch SDPA")

    monkeypatch.setattr(torch.nn.functional, "scaled_dot_product_attention", no_sdpa)
    with torch.no_grad():
        out = lm(input_ids=batch.to(DEV), attention_mask=mask.to(DEV), position_ids=pos.to(DEV)).logits[:, -1].float().cpu()
    assert torch.isfinite(out).all()
    for r in range(2):
        assert float((out[r] - alone[r]).abs().max()) <= 3e-2 * float(alone[r].abs().max()) + 1e-3


def test_hf_static_cache_as_input_cache():
    """A HuggingFace StaticCache handed to the model (the reference dispatches that type too,
    muillm/modules/attention/rotaryembedding.py:392-418): prefill and three decode steps must give
    the logits of the same run on a MuiStaticCache, and the HF object must end up holding the
    rotated keys."""
    transformers = pytest.importorskip("transformers")
    from transformers import LlamaConfig, StaticCache
    from muillm_amd.modules.kvcache.cache_utils import create_static_cache

    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=13, init_std=0.08)
    hf_cfg = LlamaConfig(hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                         num_hidden_layers=cfg.num_hidden_layers, num_attention_heads=cfg.num_attention_heads,
                         num_key_value_heads=cfg.num_key_value_heads, vocab_size=cfg.vocab_size,
                         max_position_embeddings=cfg.max_position_embeddings)
    try:
        hf_cache = StaticCache(config=hf_cfg, max_cache_len=64)
    except TypeError:
        pytest.skip("this transformers version builds StaticCache differently")
    mui_cache = create_static_cache(MuiEngineConfig(), cfg, 1, 64, DEV, torch.float16)
    ids = torch.randint(1, cfg.vocab_size, (1, 9), generator=torch.Generator().manual_seed(5)).to(DEV)

    def run(cache):
        outs = []
        with torch.no_grad():
            o = lm(input_ids=ids, past_key_values=cache, use_cache=True,
                   cache_position=torch.arange(9, device=DEV))
            outs.append(o.logits[0, -1].float().cpu())
            tok = o.logits[:, -1].argmax(-1, keepdim=True)
            for step in range(3):
                o = lm(input_ids=tok, past_key_values=cache, use_cache=True,
                       cache_position=torch.tensor([9 + step], device=DEV),
                       position_ids=torch.tensor([[9 + step]], device=DEV))
                outs.append(o.logits[0, -1].float().cpu())
                tok = o.logits[:, -1].argmax(-1, keepdim=True)
        return outs

    ref = run(mui_cache)
    got = run(hf_cache)
    for a, b in zip(got, ref):
        assert float((a - b).abs().max()) <= 2e-2 * float(b.abs().max()) + 1e-3
    layer0 = hf_cache.layers[0] if hasattr(hf_cache, "layers") else None
    keys = layer0.keys if layer0 is not None else hf_cache.key_cache[0]
    assert bool(keys[:, :, :12].abs().sum() > 0) and bool((keys[:, :, 12:] == 0).all())


def test_generate_stops_at_eos_and_pads():
    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=9, init_std=0.08)
    ids = torch.randint(1, cfg.vocab_size, (2, 7), generator=torch.Generator().manual_seed(3)).to(DEV)
    free = lm.generate(ids, max_new_tokens=8).cpu()
    eos = int(free[0, 7 + 3])                      # row 0 emits this at its 4th new token
    first_hit = [int((free[r, 7:] == eos).nonzero()[0]) if bool((free[r, 7:] == eos).any()) else None for r in range(2)]
    out = lm.generate(ids, max_new_tokens=8, eos_token_id=eos, pad_token_id=0).cpu()
    for r in range(2):
        h = first_hit[r]
        if h is None:
            assert torch.equal(out[r], free[r])
        else:
            assert torch.equal(out[r, : 7 + h + 1], free[r, : 7 + h + 1])   # identical up to and including eos
            assert bool((out[r, 7 + h + 1:] == 0).all())                      # pad afterwards
    with pytest.raises(NotImplementedError):
        lm.generate(ids, max_new_tokens=2, repetition_penalty=1.2)
    # top_k = 1 sampling is greedy decoding; top_p -> 0 as well
    k1 = lm.generate(ids, max_new_tokens=8, do_sample=True, top_k=1, seed=5).cpu()
    p0 = lm.generate(ids, max_new_tokens=8, do_sample=True, top_p=1e-6, seed=6).cpu()
    assert torch.equal(k1, free) and torch.equal(p0, free)


def test_generate_early_stop_without_host_sync():
    """When every row has hit an eos token the loop ends early (asynchronous stop check); what it
    emits is the free-running sequence up to each row's eos, then padding."""
    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=10, init_std=0.08)
    ids = torch.randint(1, cfg.vocab_size, (3, 5), generator=torch.Generator().manual_seed(4)).to(DEV)
    n_new = 96
    free = lm.generate(ids, max_new_tokens=n_new).cpu()
    eos = sorted({int(free[r, 5 + 2]) for r in range(3)})  # every row emits one of these by its 3rd token
    dec = MuiGraphDecoder(lm, use_graph=True, eos_token_ids=eos, pad_token_id=0)
    out = dec.generate(ids, n_new, stop_check_every=8).cpu()
    assert out.shape == free.shape
    for r in range(3):
        hits = [i for i in range(n_new) if int(free[r, 5 + i]) in eos]
        h = hits[0]
        assert h <= 2
        assert torch.equal(out[r, : 5 + h + 1], free[r, : 5 + h + 1]) and bool((out[r, 5 + h + 1:] == 0).all())
    assert dec.cache.get_seq_length() < 5 + n_new - 1   # the loop really stopped before the budget


def test_embedding_kernel():
    from muillm_amd.modules.embedding import MuiEmbedding
    g = torch.Generator().manual_seed(11)
    for dtype, vocab, dim in ((torch.float16, 1000, 4096), (torch.bfloat16, 77, 100)):
        emb = MuiEmbedding(MuiEngineConfig(), vocab, dim, device=DEV, dtype=dtype)
        emb.finalize_init()
        for idt in (torch.int64, torch.int32):
            ids = torch.randint(0, vocab, (3, 5), generator=g).to(idt).to(DEV)
            out = emb(ids)
            assert out.shape == (3, 5, dim)
            assert torch.equal(out, torch.nn.functional.embedding(ids.long(), emb.weight))
    # a strided view of a wider table (row pitch != dim) goes through the same kernel
    from muillm_amd import muillm_ext
    table = torch.randn(50, 256, generator=g).half().to(DEV)
    ids = torch.tensor([0, 49, 7], device=DEV)
    assert torch.equal(muillm_ext.muillm_embedding_forward(None, table[:, :128], ids), table[ids, :128])


def test_sample_advance_kernel_matches_oracle_draws():
    """Every draw of mui_sample_advance is the argmax of the oracle's scores for the same
    (seed, row, step) -- up to fp32 rounding of the scores -- and the bookkeeping is the greedy one."""
    from muillm_amd import muillm_ext
    g = torch.Generator().manual_seed(12)
    B, V, max_steps, seed, temp = 6, 203, 5, 0x1234567890ABCDEF, 0.8
    ids = torch.zeros(B, 1, dtype=torch.int64, device=DEV)
    step = torch.zeros(B, dtype=torch.int64, device=DEV)
    toks = torch.full((B, max_steps), -1, dtype=torch.int64, device=DEV)
    pos = torch.full((B, 1), 7, dtype=torch.int64, device=DEV)
    cpos = torch.full((1,), 7, dtype=torch.int64, device=DEV)
    for s_i in range(max_steps):
        logits = (2.0 * torch.randn(B, V, generator=g)).half()
        logits[:, 5] = float("-inf")  # a filtered token can never be drawn
        muillm_ext.mui_sample_advance(logits.to(DEV), ids, step, toks, temperature=temp, seed=seed,
                                      position_ids=pos, cache_position=cpos)
        got = toks[:, s_i].cpu()
        for b in range(B):
            sc = oracle.sample_scores(logits[b], temp, seed, b, s_i)
            assert got[b] != 5
            assert float(sc.max() - sc[got[b]]) <= 1e-4 * max(1.0, float(sc.max().abs())), (s_i, b)
        assert torch.equal(ids.cpu().view(-1), got) and int(cpos.item()) == 8 + s_i
        assert torch.equal(step.cpu(), torch.full((B,), s_i + 1))


def test_sample_advance_distribution_and_reproducibility():
    from muillm_amd import muillm_ext
    rows, V = 8192, 16
    logits = torch.linspace(-2.0, 2.0, V).half()
    probs = torch.softmax(logits.double() / 0.9, -1)
    lg = logits.unsqueeze(0).expand(rows, V).contiguous().to(DEV)

    def draw(seed, step0):
        ids = torch.zeros(rows, dtype=torch.int64, device=DEV)
        step = torch.full((rows,), step0, dtype=torch.int64, device=DEV)
        out = torch.zeros(rows, step0 + 1, dtype=torch.int64, device=DEV)
        muillm_ext.mui_sample_advance(lg, ids, step, out, temperature=0.9, seed=seed)
        return ids.cpu()

    a, a2, b, c = draw(1, 0), draw(1, 0), draw(2, 0), draw(1, 1)
    assert torch.equal(a, a2)                                  # same (seed, row, step) -> same draw
    assert not torch.equal(a, b) and not torch.equal(a, c)     # seed and step both matter
    freq = torch.bincount(torch.cat([a, b, c]), minlength=V).double() / (3 * rows)
    sigma = (probs * (1 - probs) / (3 * rows)).sqrt()
    assert ((freq - probs).abs() <= 5 * sigma + 1e-4).all(), (freq, probs)


def test_graph_decode_sampling_reproducible():
    cfg = _small_config()
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=5, init_std=0.05)
    ids = torch.randint(0, cfg.vocab_size, (2, 6), generator=torch.Generator().manual_seed(1)).to(DEV)
    outs = []
    for use_graph in (True, False, True):
        dec = MuiGraphDecoder(lm, use_graph=use_graph, do_sample=True, temperature=1.0, seed=99)
        outs.append(dec.generate(ids, 12).cpu())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])   # replayed == eager, run to run
    greedy = MuiGraphDecoder(lm, use_graph=True).generate(ids, 12).cpu()
    assert not torch.equal(outs[0], greedy)


@pytest.mark.skipif(not _hf.HAVE_TRANSFORMERS, reason="transformers not installed")
def test_init_engine_on_hf_llama_gpu_fp16():
    """Drop-in check: a HuggingFace Llama (fp16, GPU) before and after init_engine."""
    torch.manual_seed(0)
    cfg = _hf.LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                          num_key_value_heads=2, vocab_size=1024, max_position_embeddings=256, rms_norm_eps=1e-5,
                          rope_theta=500000.0)
    hf = _hf.LlamaForCausalLM(cfg).half().eval()
    ids = torch.randint(0, 1024, (2, 20))
    with torch.no_grad():
        ref = hf.float()(input_ids=ids, use_cache=False).logits.double()  # fp32 reference on CPU
    hf = hf.half()
    model = init_engine(copy.deepcopy(hf), device=DEV)
    with torch.no_grad():
        out = model(input_ids=ids[:, :16].to(DEV))
        assert_parity(out.logits, ref[:, :16], 1e-2, "HF prefill logits")
        cache = out.past_key_values
        for t in range(16, 20):
            step = model(input_ids=ids[:, t : t + 1].to(DEV), past_key_values=cache)
            assert_parity(step.logits[:, 0], ref[:, t], 1e-2, f"HF decode step {t}")


@pytest.mark.parametrize("group_size", [0, 128])
def test_int8_quantized_model(group_size):
    cfg = _small_config()
    base = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device=DEV, seed=3,
                                           init_std=0.05, finalize=False)
    qm = Int8WeightOnlyQuantizationMethod(group_size=group_size, modules=["qkv_proj", "o_proj", "mlp"])
    qmodel = init_engine(copy.deepcopy(base), device=DEV, engine_config=MuiEngineConfig(qm))
    fmodel = init_engine(base, device=DEV, engine_config=MuiEngineConfig())
    kinds = [type(m).__name__ for m in qmodel.modules()]
    assert kinds.count("MuiInt8GateUpDownMLP") == 2 and kinds.count("MuiInt8Linear") == 2 + 2 + 2  # qkv, o, down
    assert isinstance(qmodel.lm_head, MuiLinear)  # filtered out by name, stays 16-bit
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(0, cfg.vocab_size, (1, 10), generator=g).to(DEV)
    with torch.no_grad():
        fo, qo = fmodel(input_ids=ids), qmodel(input_ids=ids)
        assert oracle.rel_err(qo.logits.cpu(), fo.logits.cpu().double()) < 6e-2
        fc, qc = fo.past_key_values, qo.past_key_values
        tok = fo.logits[:, -1].argmax(-1, keepdim=True)
        f1 = fmodel(input_ids=tok, past_key_values=fc)   # single-token: the int8 GEMV kernels run here
        q1 = qmodel(input_ids=tok, past_key_values=qc)
        assert oracle.rel_err(q1.logits.cpu(), f1.logits.cpu().double()) < 6e-2
    # the quantised single-token layer equals the oracle on its own quantised weights
    layer = qmodel.model.layers[0]
    x = torch.randn(1, 1, cfg.hidden_size, generator=g).half()
    oproj = layer.self_attn.o_proj
    assert isinstance(oproj, MuiInt8Linear)
    y = oproj(x.to(DEV))
    if group_size == 0:
        ref = oracle.int8_channel_linear(x, oproj.weights_int8.cpu(), oproj.scales.cpu())
    else:
        ref = oracle.int8_group_linear(x, oproj.weights_uint8.cpu(), oproj.scales_min_vals.cpu(), group_size)
    assert_parity(y, ref, 1e-2, "int8 o_proj")
    assert isinstance(layer.mlp, MuiInt8GateUpDownMLP)
