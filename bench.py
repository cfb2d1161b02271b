#!/usr/bin/env python3
"""Benchmark of the decode hot path on one MI355X.

  python bench.py --gpus 1 --steps K --warmup W

A "step" is one greedy decode step (one token for one user) of a randomly initialised
Llama-3-8B-shaped fp16 decoder: 32 layers, hidden 4096, 32/8 heads x 128, MLP 14336, vocab
128256, static KV cache, 32-token random prompt, batch 1. The step (32 x
[fused norm+QKV GEMV, fused RoPE + cache write + flash decoding, o_proj GEMV + residual,
fused norm + gate/up + SiLU GEMV, down GEMV + residual], final norm + lm_head GEMV, token
choice, which also fetches the chosen token's embedding row for the next step)
runs the way the library's decoder chooses (`config.launch`: one library call per step that
enqueues the whole layer stack on the stream, or replay of the captured step from a HIP graph; the
`variants` force each); all inputs are resident in HBM before the timed region.

Prints ONE JSON line with the whole-job throughput (tokens/s/user), a `roofline` object for
the dominant kernel (the fused gate/up GEMV: half of all bytes streamed per token) timed
live with HIP events over cold (distinct) weight buffers, a `cpu_baseline` object (the
reference's PyTorch fallback path in fp16 on this box's host cores, bounded sample), and a
`kernels` table (GB/s per fused kernel family, informational).
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the gate/up GEMV at the Llama-3-8B shape, from two `rocprofv3 --pmc` runs of
# `bench.py --pmc-probe` (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same
# counter reads for the probe's elementwise copy of 234,881,024 B: FETCH_SIZE reads 114,706.4 for the copy
# (x1.99968 to KiB) and 114,783.9 for the GEMV; WRITE_SIZE reads 229,376.0 for the copy (x1.0) and 224.02
# for the GEMV. 235,039,678 B fetched + 229,396 B written.
GATEUP_TRAFFIC_BYTES = 235039678 + 229396
GATEUP_TRAFFIC_SOURCE = ("profiles/gateup_gemv_llama3_8b_pmc_traffic.md: rocprofv3 --pmc counter runs of 2026-11-26 on "
                         "commit 1a733c7 (counters need profiler runs of their own; not re-measured by this run)")
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 / bf16 matrix-core peak
BASELINE_TOKENS_PER_S = 210.0  # reference README: Llama-3-8B fp16 bs1 on 1x MI300X


def _progress(msg):
    """Stage marker on stderr (stdout carries the one JSON line): a long run stays visibly alive."""
    print("[bench %.0fs] %s" % (time.perf_counter() - _T0, msg), file=sys.stderr, flush=True)


_T0 = time.perf_counter()


def _event_time_us(fn, iters, warm):
    import torch

    for i in range(warm):
        fn(i)
    torch.cuda.synchronize()
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for i in range(iters):
        fn(i)
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 1e3 / iters


def bench_decode(lm, steps, warmup, prompt_len=32, use_graph=None, batch=1, windows=1):
    """`windows` timed generations, each the whole workload again: prompt prefill into the emptied
    cache, `warmup` untimed decode steps, then exactly `steps` timed ones between two device
    synchronisations. Returns the list of window times (seconds) and the decoder."""
    import torch

    from muillm_amd.modules.models.graphdecoder import MuiGraphDecoder

    dev = "cuda"
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, lm.config.vocab_size, (batch, prompt_len), generator=g).to(dev)
    dec = MuiGraphDecoder(lm, use_graph=use_graph)
    times = []
    for w in range(windows):
        if w:
            dec.cache.reset()
        dec.prefill(ids, steps + warmup + 1, cache=dec.cache if w else None)
        dec.decode(warmup)  # captures the graph on first use, then W untimed steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.decode(steps)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return (times if windows > 1 else times[0]), dec


def _median(vals):
    v = sorted(vals)
    n = len(v)
    return v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])


def _rate_summary(times, steps, per_step=1):
    """Median / min / max rate over timed windows, and which window was the fastest."""
    rates = [per_step * steps / t for t in times]
    return {"median": round(_median(rates), 2), "min": round(min(rates), 2), "max": round(max(rates), 2),
            "windows": [round(r, 2) for r in rates], "fastest_window": rates.index(max(rates))}


def bench_prefill(lm, tokens, iters=3):
    """Prefill of one `tokens`-token prompt (batch 1, last-token logits only): every linear layer on
    the library's prompt kernels (rmsnorm launch + tiled matrix-core GEMM), causal attention on its
    prompt attention kernel. Returns ms and the arithmetic rate over the dense fp16 MFMA peak."""
    import torch

    cfg = lm.config
    ids = torch.randint(0, cfg.vocab_size, (1, tokens), generator=torch.Generator().manual_seed(1)).to("cuda")
    with torch.no_grad():
        for _ in range(2):
            lm(input_ids=ids, num_logits_to_keep=1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            lm(input_ids=ids, num_logits_to_keep=1)
        torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / iters * 1e3
    hid, inter = cfg.hidden_size, cfg.intermediate_size
    hq, hkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, hid // cfg.num_attention_heads
    linear_flops = 2.0 * tokens * cfg.num_hidden_layers * ((hq + 2 * hkv) * d * hid + hid * hid + 3 * hid * inter)
    attn_flops = 4.0 * hq * d * tokens * tokens / 2 * cfg.num_hidden_layers
    tflops = (linear_flops + attn_flops) / ms / 1e9
    return {"ms": round(ms, 3), "tokens_per_s": round(tokens / ms * 1e3, 1), "TFLOP/s": round(tflops, 1),
            "mfma_peak_frac": round(tflops / MFMA_FP16_PEAK_TFLOPS, 4)}


def bench_int8_variant(config, steps, warmup, group_size=0):
    """The same decode benchmark with the decoder layers quantised to int8 (group_size 0: symmetric
    per output channel; else the reference's group-wise uint8 + (scale, min) format; lm_head stays
    16-bit, as the reference's module-name filter would leave it)."""
    import torch

    from muillm_amd.engine import init_engine
    from muillm_amd.engineconfig import MuiEngineConfig
    from muillm_amd.modules.models.llama.model import MuiLlamaForCausalLM
    from muillm_amd.quantization.quantizationmethod import Int8WeightOnlyQuantizationMethod

    qm = Int8WeightOnlyQuantizationMethod(group_size=group_size, modules=["qkv_proj", "o_proj", "mlp"])
    base = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), config, dtype=torch.float16, device="cuda", seed=0,
                                           finalize=False)
    lm8 = init_engine(base, device="cuda", engine_config=MuiEngineConfig(qm))
    torch.cuda.synchronize()
    t, dec = bench_decode(lm8, steps, warmup, windows=3)
    dt = _median(t)
    del dec
    t, dec = bench_decode(lm8, steps, warmup, use_graph=True, windows=3)
    dt_graph = _median(t)
    hid, inter, v = config.hidden_size, config.intermediate_size, config.vocab_size
    hq, hkv, d = config.num_attention_heads, config.num_key_value_heads, hid // config.num_attention_heads
    codes = config.num_hidden_layers * ((hq + 2 * hkv) * d * hid + hid * hid + 3 * hid * inter)
    # per-channel: one fp16 scale per row (negligible); group format: 4 bytes of (scale, min) per group
    wbytes = codes + (codes // group_size * 4 if group_size else 0) + 2 * v * hid
    del dec, lm8, base
    torch.cuda.empty_cache()
    return {"tokens_per_s": round(steps / dt, 2), "ms_per_step": round(dt / steps * 1e3, 4),
            "graph_replay_tokens_per_s": round(steps / dt_graph, 2),
            "weight_bytes_per_token": wbytes, "hbm_floor_ms": round(wbytes / (HBM_PEAK_GBPS * 1e9) * 1e3, 4),
            "format": ("uint8 + fp16 (scale, min) per group of %d inputs (the reference's RTN format); lm_head fp16" % group_size)
            if group_size else "int8 per output channel + fp16 scale; lm_head fp16"}


def bench_hf_dropin(config, steps, prompt_len=32, windows=3):
    """The drop-in path the reference's own number is taken on (examples/llama3_8b.py:98-106,148-167
    there): a HuggingFace LlamaForCausalLM -- here built at the 8B shape straight on the device with
    random weights, no checkpoint --, init_engine() on it, a short warm-up generate(), then timed
    model.generate(ids, max_new_tokens=steps) calls, prompt prefill included in the time."""
    import torch

    try:
        from transformers import LlamaConfig, LlamaForCausalLM
    except Exception as e:  # transformers is optional for this library
        return {"skipped": "transformers not importable: %r" % (e,)}
    from muillm_amd.engine import init_engine

    hf_cfg = LlamaConfig(hidden_size=config.hidden_size, intermediate_size=config.intermediate_size,
                         num_hidden_layers=config.num_hidden_layers, num_attention_heads=config.num_attention_heads,
                         num_key_value_heads=config.num_key_value_heads, vocab_size=config.vocab_size,
                         max_position_embeddings=config.max_position_embeddings, rms_norm_eps=config.rms_norm_eps,
                         rope_theta=500000.0, tie_word_embeddings=False)
    torch.manual_seed(0)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)
    try:
        with torch.device("cuda"):
            hf = LlamaForCausalLM(hf_cfg)
    finally:
        torch.set_default_dtype(prev)
    hf.eval()
    model = init_engine(hf, device="cuda")
    ids = torch.randint(0, config.vocab_size, (1, prompt_len), generator=torch.Generator().manual_seed(0)).to("cuda")
    model.generate(ids, max_new_tokens=10)  # the reference's example warms up the same way
    torch.cuda.synchronize()
    times = []
    for _ in range(windows):
        t0 = time.perf_counter()
        out = model.generate(ids, max_new_tokens=steps)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    assert out.shape == (1, prompt_len + steps)
    dt = _median(times)
    res = {"new_tokens_per_s": round(steps / dt, 2), "new_tokens_per_s_windows": [round(steps / t, 2) for t in times],
           "reference_formula_total_tokens_per_s": round((prompt_len + steps) / dt, 2),
           "what": "transformers.LlamaForCausalLM (random init at the 8B shape) -> init_engine -> model.generate("
                   "ids[1, %d], max_new_tokens=%d), greedy, timed over the whole call: prefill + %d decode steps; "
                   "reference_formula counts prompt + new tokens over the same time, as examples/llama3_8b.py does"
                   % (prompt_len, steps, steps)}
    del model, hf
    torch.cuda.empty_cache()
    return res


def measured_copy_ceiling():
    """Device-to-device copy rate (read + write bytes per second) of torch's copy over 1 GiB
    buffers, rotating over 3 source/destination pairs: a practical HBM ceiling to hold the
    8 TB/s datasheet figure against."""
    import torch

    n = 1 << 29  # fp16 elements = 1 GiB
    src = [torch.empty(n, device="cuda", dtype=torch.float16).fill_(1.0) for _ in range(3)]
    dst = [torch.empty(n, device="cuda", dtype=torch.float16) for _ in range(3)]
    us = _event_time_us(lambda i: dst[i % 3].copy_(src[i % 3]), iters=12, warm=3)
    return round(2 * n * 2 / us / 1e3, 1)


def measured_read_ceiling():
    """Read-only rate of the library's probe kernel (the GEMVs' access shape, nothing but loads)
    over 1 GiB buffers, rotating over 3 of them: what a kernel that only has to read can reach."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    n = 1 << 30
    src = [torch.empty(n, device="cuda", dtype=torch.uint8).fill_(1) for _ in range(3)]
    sink = torch.zeros(64, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    us = _event_time_us(lambda i: lib.mui_probe_read(stream, src[i % 3].data_ptr(), n, sink.data_ptr()), iters=12, warm=3)
    return round(n / us / 1e3, 1)


def gateup_roofline(lm):
    """Average launch duration of the fused gate/up+SiLU GEMV over the model's 32 distinct
    (cold) weight buffers, HIP events on the launch stream."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    layers = lm.model.layers
    hid, inter = lm.config.hidden_size, lm.config.intermediate_size
    x = torch.randn(hid, device="cuda", dtype=torch.float16)
    h = torch.empty(inter, device="cuda", dtype=torch.float16)
    stream = torch.cuda.current_stream().cuda_stream
    ptrs = [(l.mlp.gate_proj.weight.data_ptr(), l.mlp.up_proj.weight.data_ptr(), l.mlp.gate_proj.weight.stride(0),
             l.mlp.norm_weights.data_ptr()) for l in layers]

    def fn(i):
        gp, up, pitch, nw = ptrs[i % len(ptrs)]
        lib.mui_gateup_silu(stream, 0, gp, up, pitch, x.data_ptr(), nw, 1e-5, h.data_ptr(), inter, hid, 1)

    samples = [_event_time_us(fn, iters=8 * len(ptrs), warm=len(ptrs)) for _ in range(5)]
    us = _median(samples)
    alg_bytes = 2 * inter * hid * 2 + 2 * (hid + hid + inter)  # G and U once, x, gamma, h
    achieved = alg_bytes / us / 1e3
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": GATEUP_TRAFFIC_BYTES if (hid, inter) == (4096, 14336) else None,
            "traffic_source": GATEUP_TRAFFIC_SOURCE if (hid, inter) == (4096, 14336) else None,
            "kernel": "gemv_kernel<F16,R=4,CH=2,NORM,GATEUP> (fused RMSNorm + gate/up + SiLU*mul)",
            "avg_launch_us": round(us, 2), "avg_launch_us_min": round(min(samples), 2),
            "avg_launch_us_max": round(max(samples), 2),
            "samples": "median of 5 x (8 launches per layer's buffer, HIP events on the launch stream)",
            "algorithmic_bytes_per_launch": alg_bytes}


def pmc_probe(launches=6):
    """Counter probe for `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`: a few launches of the
    fused gate/up GEMV at the Llama-3-8B shape over distinct weight buffers, then the same number of
    launches of a plain elementwise copy kernel that reads and writes exactly as many bytes as one
    gate/up launch reads (the calibration for the counter's unit)."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    hid, inter = 4096, 14336
    f16 = dict(device="cuda", dtype=torch.float16)
    ws = [torch.randn(inter, 2, hid, **f16) * 0.02 for _ in range(launches)]
    x, gamma, h = torch.randn(hid, **f16), torch.ones(hid, **f16), torch.empty(inter, **f16)
    src = [torch.randn(inter * 2 * hid, **f16) for _ in range(2)]
    dst = torch.empty(inter * 2 * hid, **f16)
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    for w in ws:
        _lib.check(lib.mui_gateup_silu(stream, 0, w[:, 0].data_ptr(), w[:, 1].data_ptr(), 2 * hid, x.data_ptr(),
                                       gamma.data_ptr(), 1e-5, h.data_ptr(), inter, hid, 1), "mui_gateup_silu")
    torch.cuda.synchronize()
    for i in range(launches):
        torch.mul(src[i % 2], 1.0, out=dst)
    torch.cuda.synchronize()
    print(json.dumps({"pmc_probe": {"launches": launches, "gateup_algorithmic_bytes": 2 * inter * hid * 2 + 2 * (2 * hid + inter),
                                    "copy_bytes_read": dst.numel() * 2, "copy_bytes_written": dst.numel() * 2}}))


def pmc_probe_batched(launches=6, tokens=8):
    """Counter probe for the batched (matrix-core) MLP: a few launches of the fused gate/up and of
    the down projection at `tokens` tokens, Llama-3-8B shape, over distinct weight buffers
    (`rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F16 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES`,
    and `--pmc FETCH_SIZE` for the traffic)."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    hid, inter = 4096, 14336
    f16 = dict(device="cuda", dtype=torch.float16)
    gu = [torch.randn(inter, 2, hid, **f16) * 0.02 for _ in range(launches)]
    dn = [torch.randn(hid, inter, **f16) * 0.02 for _ in range(launches)]
    x, gamma = torch.randn(tokens, hid, **f16), torch.ones(hid, **f16)
    h, res, y = torch.empty(tokens, inter, **f16), torch.randn(tokens, hid, **f16), torch.empty(tokens, hid, **f16)
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    for w, d in zip(gu, dn):
        _lib.check(lib.mui_gateup_silu(stream, 0, w[:, 0].data_ptr(), w[:, 1].data_ptr(), 2 * hid, x.data_ptr(),
                                       gamma.data_ptr(), 1e-5, h.data_ptr(), inter, hid, tokens), "mui_gateup_silu")
        _lib.check(lib.mui_linear(stream, 0, d.data_ptr(), inter, h.data_ptr(), None, 0.0, None, None, res.data_ptr(),
                                  y.data_ptr(), hid, inter, tokens), "mui_linear")
    torch.cuda.synchronize()
    print(json.dumps({"pmc_probe_batched": {"launches": launches, "tokens": tokens,
                                            "gateup_flops": 4 * inter * hid * tokens, "down_flops": 2 * inter * hid * tokens,
                                            "gateup_weight_bytes": 4 * inter * hid, "down_weight_bytes": 2 * inter * hid}}))


def pmc_probe_int8(launches=4):
    """Counter probe for the int8 GEMVs of a Llama-3-8B layer (per-channel format): QKV, o_proj, down
    and gate/up at 1 and at 4 tokens, `launches` launches each over distinct weight buffers, then as
    many launches of an elementwise copy of 117,440,512 B for the counters' units
    (`rocprofv3 --pmc FETCH_SIZE`; `--pmc SQ_WAVES SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_VMEM_RD`;
    `--pmc SQ_BUSY_CU_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY GRBM_GUI_ACTIVE`)."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    hid, inter, n_qkv = 4096, 14336, 6144
    f16 = dict(device="cuda", dtype=torch.float16)
    stream = torch.cuda.current_stream().cuda_stream
    gamma = torch.ones(hid, **f16)
    X, RES, HM = torch.randn(4, hid, **f16), torch.randn(4, hid, **f16), torch.randn(4, inter, **f16)
    Y = torch.empty(4 * inter, **f16)
    shapes = (("qkv", n_qkv, hid, True, False), ("o_proj", hid, hid, False, True), ("down", hid, inter, False, True))
    info = {}
    for b in (1, 4):
        for name, n, k, norm, resid in shapes:
            ws = [(torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda"), torch.rand(n, **f16) * 1e-3 + 1e-4)
                  for _ in range(launches)]
            xin = X if k == hid else HM
            torch.cuda.synchronize()
            for q, sc in ws:
                _lib.check(lib.mui_int8_linear(stream, 0, q.data_ptr(), k, sc.data_ptr(), xin.data_ptr(),
                                               gamma.data_ptr() if norm else None, 1e-5, None,
                                               RES.data_ptr() if resid else None, Y.data_ptr(), n, k, b), "mui_int8_linear")
            torch.cuda.synchronize()
            info["%s_tokens%d" % (name, b)] = {"weight_bytes": n * k, "weights": n * k}
            del ws
        ws = [(torch.randint(-127, 128, (inter, 2, hid), dtype=torch.int8, device="cuda"),
               torch.rand(inter, 2, **f16) * 1e-3 + 1e-4) for _ in range(launches)]
        torch.cuda.synchronize()
        for q, sc in ws:
            _lib.check(lib.mui_int8_gateup_silu(stream, 0, q.data_ptr(), q.data_ptr() + hid, 2 * hid, sc.data_ptr(),
                                                sc.data_ptr() + 2, 2, X.data_ptr(), gamma.data_ptr(), 1e-5, Y.data_ptr(),
                                                inter, hid, b), "mui_int8_gateup_silu")
        torch.cuda.synchronize()
        info["gateup_tokens%d" % b] = {"weight_bytes": 2 * inter * hid, "weights": 2 * inter * hid}
        del ws
    src = [torch.randn(inter * hid, **f16) for _ in range(2)]
    dst = torch.empty(inter * hid, **f16)
    for i in range(launches):
        torch.mul(src[i % 2], 1.0, out=dst)
    torch.cuda.synchronize()
    info["copy"] = {"bytes_read": dst.numel() * 2, "bytes_written": dst.numel() * 2}
    print(json.dumps({"pmc_probe_int8": {"launches": launches, "order": "tokens 1: qkv, o_proj, down, gateup; tokens 4: same; copy",
                                         "calls": info}}))


def _graph_chain_us(launch, n=400, replays=10):
    """Average cost of one launch in a HIP graph of `n` copies of `launch(stream)` on one stream
    (every kernel waits for the one before it), over `replays` replays."""
    import torch

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = torch.cuda.current_stream().cuda_stream
        for _ in range(n):
            launch(st)
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(replays):
        graph.replay()
    b.record()
    torch.cuda.synchronize()
    return round(a.elapsed_time(b) * 1e3 / (replays * n), 3)


def probe_warm(lm, steps, warmup, decode_rate=False):
    """Cache warming by the idle workgroups of the short-context attention launch
    (mui_attn_decode_fused_warm): the pair [fused RoPE + cache write + attention at 64 cached tokens,
    o_proj GEMV + residual] over the model's 32 o_proj matrices, HIP-event timed, and the decode
    rate on stream launches, for a few settings of mui_tune_warm (workgroups, percent) in one process."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    f16 = dict(device="cuda", dtype=torch.float16)
    hq, hkv, d, S = 32, 8, 128, 64
    hid = lm.config.hidden_size
    layers = lm.model.layers
    op = [l.self_attn.o_proj.weight for l in layers]
    qs = (hq + 2 * hkv) * d
    qkvx = torch.randn(1, qs, **f16)
    caches = [(torch.randn(1, hkv, 512, d, **f16), torch.randn(1, hkv, 512, d, **f16)) for _ in layers]
    cos, sin = [t.cuda() for t in _rope_tables_f32(512, d)]
    pos = torch.full((1, 1), S - 1, dtype=torch.int64, device="cuda")
    cpos = torch.full((1,), S - 1, dtype=torch.int64, device="cuda")
    o = torch.empty(1, hq * d, **f16)
    res, y = torch.randn(hid, **f16), torch.empty(hid, **f16)
    slab = lib.mui_linear_row_group_bytes(16, hq * d, op[0].stride(0) * 2)

    def pair(i, attn_only=False, gemv_only=False):
        kc, vc = caches[i % len(caches)]
        w = op[i % len(op)]
        if not gemv_only:
            lib.mui_attn_decode_fused_warm(stream, 0, qkvx.data_ptr(), qs, qkvx.data_ptr() + 2 * hq * d, qs,
                                           qkvx.data_ptr() + 2 * (hq + hkv) * d, qs, cos.data_ptr(), sin.data_ptr(), d // 2,
                                           cos.shape[0], pos.data_ptr(), 1, cpos.data_ptr(), S, kc.data_ptr(), vc.data_ptr(),
                                           hkv * 512 * d, 512 * d, d, None, 0, None, None, 1, o.data_ptr(), 1, hq, hkv, d, 512,
                                           w.data_ptr(), w.numel() * 2, slab)
        if not attn_only:
            lib.mui_linear(stream, 0, w.data_ptr(), w.stride(0), o.data_ptr(), None, 0.0, None, None, res.data_ptr(),
                           y.data_ptr(), hid, hq * d, 1)

    out = {"slab_bytes": slab}
    settings = [("off", -1, 0, 0)]
    for wgs in (256, 512):
        for pct in (50, 75, 100):
            for delay in (0, 4, 6, 8, 10):
                settings.append(("wg%d_pct%d_delay%d" % (wgs, pct, delay), wgs, pct, delay))
    settings.append(("off_again", -1, 0, 0))
    for name, wgs, pct, delay in settings:
        _lib.check(lib.mui_tune_warm(wgs, pct, delay), "mui_tune_warm")
        row = {"attention+o_proj_us": round(_median([_event_time_us(pair, 320, 64) for _ in range(3)]), 2),
               "attention_us": round(_median([_event_time_us(lambda i: pair(i, attn_only=True), 320, 64) for _ in range(3)]), 2),
               "o_proj_alone_us": round(_median([_event_time_us(lambda i: pair(i, gemv_only=True), 320, 64) for _ in range(3)]), 2)}
        if decode_rate:
            times, dec = bench_decode(lm, steps, warmup, use_graph=False, windows=3)
            row["decode_tokens_per_s"] = _rate_summary(times, steps)
            del dec
        out[name] = row
        _progress("probe-warm %s: %s" % (name, row))
    _lib.check(lib.mui_tune_warm(0, 0, -1), "mui_tune_warm")
    print(json.dumps({"probe_warm": out}))


def probe_chain(n_mats=32, n_launches=64):
    """A chain of dependent 4096 x 4096 fp16 GEMVs over distinct matrices: ordinary launches against
    launches that overlap their predecessor's tail and take x through arrival counters in memory
    (mui_probe_gemv_chain). Reports microseconds per GEMV, whether a bounded wait ran out, and whether
    the chain's result is bit-identical to the ordinary launches'."""
    import ctypes

    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    n = 4096
    g = torch.Generator(device="cuda").manual_seed(0)
    mats = [(torch.randn(n, n, device="cuda", generator=g) / 64).half() for _ in range(n_mats)]
    ptrs = (ctypes.c_void_p * n_mats)(*[m.data_ptr() for m in mats])
    x0 = torch.randn(n, device="cuda", generator=g).half()
    xa, xb = torch.empty_like(x0), torch.empty_like(x0)
    flags = torch.zeros(lib.mui_probe_chain_flag_bytes(n_launches) // 4, dtype=torch.int32, device="cuda")
    err = torch.zeros(1, dtype=torch.int32, device="cuda")
    out = {}
    ref = None
    for name, mode, wgs in (("ordinary", 0, 0), ("overlapped_coherent_x", 1, 0), ("overlapped_cached_x", 2, 0),
                            ("ordinary_256wg", 0, 256), ("overlapped_coherent_x_256wg", 1, 256),
                            ("overlapped_coherent_x_1024wg", 1, 1024),
                            ("overlapped_poll_wave", 3, 0), ("overlapped_poll_wave_all_weights_first", 4, 0),
                            ("overlapped_poll_wave_256wg", 3, 256), ("overlapped_poll_wave_all_weights_first_256wg", 4, 256),
                            ("independent_ordinary", 6, 0), ("independent_free_to_overlap", 5, 0),
                            ("ordinary_again", 0, 0)):
        samples = []
        for rep in range(6):
            xa.copy_(x0)
            flags.zero_()
            err.zero_()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            _lib.check(lib.mui_probe_gemv_chain(stream, mode, ptrs, n_mats, n_launches, n, n, xa.data_ptr(), xb.data_ptr(),
                                                flags.data_ptr(), err.data_ptr(), wgs, 20000), "mui_probe_gemv_chain")
            b.record()
            torch.cuda.synchronize()
            if rep:
                samples.append(a.elapsed_time(b) * 1e3 / n_launches)
        res = (xa if n_launches % 2 == 0 else xb).clone()
        if mode in (5, 6):
            res = ref  # independent launches: timing only
        if ref is None:
            ref = res
        out[name] = {"us_per_gemv": round(_median(samples), 3), "min": round(min(samples), 3), "max": round(max(samples), 3),
                     "wait_ran_out": bool(err.item()), "bit_identical_to_ordinary": bool(torch.equal(res, ref)),
                     "finite": bool(torch.isfinite(res).all())}
        _progress("probe-chain %s: %s" % (name, out[name]))
    # the chain dealt alternately to two streams (two hardware queues)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    for name, mode, wgs in (("two_streams_independent", 0, 0), ("two_streams_handoff", 1, 0),
                            ("two_streams_poll_wave", 2, 0), ("two_streams_poll_wave_all_weights_first", 3, 0),
                            ("two_streams_handoff_256wg", 1, 256), ("two_streams_poll_wave_all_weights_first_256wg", 3, 256)):
        samples = []
        for rep in range(6):
            xa.copy_(x0)
            flags.zero_()
            err.zero_()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(sa)
            sb.wait_event(a)
            _lib.check(lib.mui_probe_gemv_chain2(sa.cuda_stream, sb.cuda_stream, mode, ptrs, n_mats, n_launches, n, n,
                                                 xa.data_ptr(), xb.data_ptr(), flags.data_ptr(), err.data_ptr(), wgs, 20000),
                       "mui_probe_gemv_chain2")
            done_b = torch.cuda.Event()
            done_b.record(sb)
            sa.wait_event(done_b)
            b.record(sa)
            torch.cuda.synchronize()
            if rep:
                samples.append(a.elapsed_time(b) * 1e3 / n_launches)
        res = (xa if n_launches % 2 == 0 else xb).clone()
        out[name] = {"us_per_gemv": round(_median(samples), 3), "min": round(min(samples), 3), "max": round(max(samples), 3),
                     "wait_ran_out": bool(err.item()),
                     "bit_identical_to_ordinary": None if mode == 0 else bool(torch.equal(res, ref))}
        _progress("probe-chain %s: %s" % (name, out[name]))
    print(json.dumps({"probe_chain": out}))


def probe_kernel_boundary():
    """What one dependent kernel costs inside a replayed HIP graph when it has next to nothing to do:
    the read probe over 16 B and over 64 KiB, and a 256 x 256 GEMV (alone, and two of them feeding each
    other). This is the part of every launch of a decode step that no kernel code can remove."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    f16 = dict(device="cuda", dtype=torch.float16)
    sink = torch.zeros(64, dtype=torch.int32, device="cuda")
    src = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    w, x, y = torch.randn(256, 256, **f16), torch.randn(256, **f16), torch.empty(256, **f16)

    def gemv(st, a, b):
        lib.mui_linear(st, 0, w.data_ptr(), 256, a.data_ptr(), None, 0.0, None, None, None, b.data_ptr(), 256, 256, 1)

    out = {
        "read_probe_16B_us": _graph_chain_us(lambda st: lib.mui_probe_read(st, src.data_ptr(), 16, sink.data_ptr())),
        "read_probe_64KiB_us": _graph_chain_us(lambda st: lib.mui_probe_read(st, src.data_ptr(), 65536, sink.data_ptr())),
        "gemv_256x256_us": _graph_chain_us(lambda st: gemv(st, x, y)),
        "gemv_256x256_feeding_each_other_us": _graph_chain_us(lambda st: (gemv(st, x, y), gemv(st, y, x)), n=200) / 2,
    }
    print(json.dumps({"probe_kernel_boundary": out}))


def probe_flash_splits():
    """Fused RoPE + cache write + flash decoding at batch 1 (32 / 8 heads x 128) over the number of
    sequence splits, 1k to 32k context, K/V rotated over distinct buffers (> 1 GB per ring)."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    f16 = dict(device="cuda", dtype=torch.float16)
    hq, hkv, d, B = 32, 8, 128, 1
    qs = (hq + 2 * hkv) * d
    table = {}
    for S in (1024, 4096, 16384, 32768):
        kvbytes = B * 2 * hkv * S * d * 2
        cnt = max(2, min(64, int(1.0e9 // kvbytes) + 1))
        caches = [(torch.randn(B, hkv, S, d, **f16), torch.randn(B, hkv, S, d, **f16)) for _ in range(cnt)]
        qkvx = torch.randn(B, qs, **f16)
        cos, sin = [t.cuda() for t in _rope_tables_f32(S, d)]
        pos = torch.full((B, 1), S - 1, dtype=torch.int64, device="cuda")
        cpos = torch.full((1,), S - 1, dtype=torch.int64, device="cuda")
        o = torch.empty(B, hq * d, **f16)
        row = {"kv_bytes": kvbytes, "auto_splits": lib.mui_flash_decode_splits(B, hq, hkv, S)}
        for ns in (1, 8, 16, 32, 48, 64, 128):
            if ns > 1 and S // ns < 32:
                continue
            scratch = torch.empty(max(lib.mui_flash_decode_scratch_bytes(B, hq, d, ns), 16), dtype=torch.uint8, device="cuda")

            def att(i):
                kc, vc = caches[i % len(caches)]
                _lib.check(lib.mui_attn_decode_fused(
                    stream, 0, qkvx.data_ptr(), qs, qkvx.data_ptr() + 2 * hq * d, qs, qkvx.data_ptr() + 2 * (hq + hkv) * d, qs,
                    cos.data_ptr(), sin.data_ptr(), d // 2, cos.shape[0], pos.data_ptr(), 1, cpos.data_ptr(), S,
                    kc.data_ptr(), vc.data_ptr(), hkv * S * d, S * d, d, None, 0, None, scratch.data_ptr(), ns, o.data_ptr(),
                    B, hq, hkv, d, S), "mui_attn_decode_fused")

            row["splits_%d_us" % ns] = round(_event_time_us(att, 10 * cnt, cnt), 2)
        table["context_%d" % S] = row
        del caches
        torch.cuda.empty_cache()
    print(json.dumps({"probe_flash_splits": table}))


_PROMPT_SHAPES = (("qkv", 6144, 4096, False), ("o_proj", 4096, 4096, False), ("gateup", 14336, 4096, True),
                  ("down", 4096, 14336, False))


def _prompt_gemm_call(lib, stream, w, x, y, n, k, tokens, gateup, ws=None):
    from muillm_amd import _lib

    if gateup:
        _lib.check(lib.mui_gateup_silu(stream, 0, w.data_ptr(), w.data_ptr() + 2 * k, 2 * k, x.data_ptr(), None, 0.0,
                                       y.data_ptr(), n, k, tokens), "mui_gateup_silu")
    else:
        _lib.check(lib.mui_linear_ws(stream, 0, w.data_ptr(), k, x.data_ptr(), None, 0.0, None, None, None, y.data_ptr(),
                                     n, k, tokens, None if ws is None else ws.data_ptr(),
                                     0 if ws is None else ws.numel()), "mui_linear_ws")


def probe_prompt(counters_only=False):
    """The prompt kernels at the Llama-3-8B shapes. Timing mode: every projection at 64 to 4096 tokens
    through the C ABI (weights rotated over > 1 GB) beside torch.matmul on the same operands, and causal
    attention at 512 to 8192 tokens beside repeat_kv + torch SDPA. Counter mode (for `rocprofv3 --pmc`):
    three launches of the gate/up projection at 2048 tokens and of attention at 4096 tokens."""
    import torch
    import torch.nn.functional as F

    from muillm_amd import _lib, muillm_ext

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    f16 = dict(device="cuda", dtype=torch.float16)
    hq, hkv, d = 32, 8, 128
    if counters_only:
        n, k, tokens = 14336, 4096, 2048
        w = torch.randn(2 * n, k, **f16) * 0.02
        x, y = torch.randn(tokens, k, **f16), torch.empty(tokens, n, **f16)
        q = torch.randn(1, hq, 4096, d, **f16)
        kk, vv = torch.randn(1, hkv, 4096, d, **f16), torch.randn(1, hkv, 4096, d, **f16)
        for _ in range(3):
            _prompt_gemm_call(lib, stream, w, x, y, n, k, tokens, True)
        for _ in range(3):
            muillm_ext.mui_prefill_attention(q, kk, vv)
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe_prompt": {"gateup_flops_per_launch": 2.0 * tokens * 2 * n * k,
                                               "attention_flops_per_launch": 4.0 * hq * d * 4096 * 4096 / 2}}))
        return
    out = {"linears": {}, "attention": {}}
    ws = torch.zeros(lib.mui_linear_workspace_bytes(), dtype=torch.uint8, device="cuda")  # as the host layer passes it
    for name, n, k, gateup in _PROMPT_SHAPES:
        rows = 2 * n if gateup else n
        ring = [torch.randn(rows, k, **f16) * 0.02 for _ in range(max(2, int(1e9 // (2 * rows * k)) + 1))]
        for tokens in (64, 128, 256, 512, 1024, 2048, 4096):
            x, y = torch.randn(tokens, k, **f16), torch.empty(tokens, n, **f16)
            yt = torch.empty(tokens, rows, **f16)
            us = _event_time_us(lambda i: _prompt_gemm_call(lib, stream, ring[i % len(ring)], x, y, n, k, tokens, gateup, ws), 20, 3)
            us_t = _event_time_us(lambda i: torch.matmul(x, ring[i % len(ring)].t(), out=yt), 20, 3)
            flops = 2.0 * tokens * rows * k
            out["linears"]["%s_tokens%d" % (name, tokens)] = {
                "us": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1),
                "mfma_peak_frac": round(flops / us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4), "torch_matmul_us": round(us_t, 1)}
        del ring
        torch.cuda.empty_cache()
    for tokens in (512, 1024, 2048, 4096, 8192):
        q = torch.randn(1, hq, tokens, d, **f16)
        kk, vv = torch.randn(1, hkv, tokens, d, **f16), torch.randn(1, hkv, tokens, d, **f16)

        def sdpa(i):
            ke = kk[:, :, None].expand(1, hkv, hq // hkv, tokens, d).reshape(1, hq, tokens, d)
            ve = vv[:, :, None].expand(1, hkv, hq // hkv, tokens, d).reshape(1, hq, tokens, d)
            return F.scaled_dot_product_attention(q, ke, ve, is_causal=True)

        us = _event_time_us(lambda i: muillm_ext.mui_prefill_attention(q, kk, vv), 10, 2)
        us_t = _event_time_us(sdpa, 10, 2)
        flops = 4.0 * hq * d * tokens * tokens / 2
        out["attention"]["tokens%d" % tokens] = {"us": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1),
                                                 "mfma_peak_frac": round(flops / us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 4),
                                                 "torch_repeat_kv_sdpa_us": round(us_t, 1)}
    out["whole_model_ms"] = _probe_prompt_whole_model()
    print(json.dumps({"probe_prompt": out}))


_PROMPT_SHAPES_OTHER = (("70b_qkv", 10240, 8192, False), ("70b_o_proj", 8192, 8192, False), ("70b_gateup", 28672, 8192, True),
                        ("70b_down", 8192, 28672, False), ("13b_qkv", 15360, 5120, False), ("13b_o_proj", 5120, 5120, False),
                        ("13b_gateup", 13824, 5120, True), ("13b_down", 5120, 13824, False))


def probe_prompt_other_shapes():
    """The prompt GEMM at the projections of a Llama-3-70B- and a Llama-2-13B-shaped layer, 512 to 4096
    tokens, beside torch.matmul on the same operands (for gate/up the matmul alone): the tile choice
    was calibrated on the 8B shapes and has to carry over."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    f16 = dict(device="cuda", dtype=torch.float16)
    ws = torch.zeros(lib.mui_linear_workspace_bytes(), dtype=torch.uint8, device="cuda")
    out = {}
    for name, n, k, gateup in _PROMPT_SHAPES_OTHER:
        rows = 2 * n if gateup else n
        ring = [torch.randn(rows, k, **f16) * 0.02 for _ in range(max(2, int(1e9 // (2 * rows * k)) + 1))]
        for tokens in (512, 1024, 2048, 4096):
            x, y = torch.randn(tokens, k, **f16), torch.empty(tokens, n, **f16)
            yt = torch.empty(tokens, rows, **f16)
            us = _event_time_us(lambda i: _prompt_gemm_call(lib, stream, ring[i % len(ring)], x, y, n, k, tokens, gateup, ws), 10, 2)
            us_t = _event_time_us(lambda i: torch.matmul(x, ring[i % len(ring)].t(), out=yt), 10, 2)
            out["%s_tokens%d" % (name, tokens)] = {"us": round(us, 1), "TFLOP/s": round(2.0 * tokens * rows * k / us / 1e6, 1),
                                                   "torch_matmul_us": round(us_t, 1)}
        del ring
        torch.cuda.empty_cache()
    print(json.dumps({"probe_prompt_other_shapes": out}))


def probe_prompt_int8():
    """Prefill of the 8B-shaped model with int8 decoder layers, per format and prompt length, on both
    routes the host layer has: the tiled GEMM that converts the codes on their way to LDS, and every
    matrix dequantised once per call followed by the GEMM on 16-bit weights (the reference's route).
    The host layer's thresholds choose between them; here each is forced in turn."""
    import torch

    from muillm_amd import muillm_ext
    from muillm_amd.engine import init_engine
    from muillm_amd.engineconfig import MuiEngineConfig
    from muillm_amd.modules.models.llama.model import MuiDecoderConfig, MuiLlamaForCausalLM
    from muillm_amd.quantization.quantizationmethod import Int8WeightOnlyQuantizationMethod

    config = MuiDecoderConfig.llama3_8b(max_position_embeddings=8192)
    out = {}
    for group_size, knob in ((0, "INT8_DEQUANT_MIN_TOKENS"), (128, "INT8_GROUP_DEQUANT_MIN_TOKENS")):
        qm = Int8WeightOnlyQuantizationMethod(group_size=group_size, modules=["qkv_proj", "o_proj", "mlp"])
        base = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), config, dtype=torch.float16, device="cuda", seed=0,
                                               finalize=False)
        lm8 = init_engine(base, device="cuda", engine_config=MuiEngineConfig(qm))
        torch.cuda.synchronize()
        default = getattr(muillm_ext, knob)
        name = "group128" if group_size else "per_channel"
        out[name] = {"dequantise_once_from_tokens": default}
        try:
            for tokens in (32, 64, 512, 1024, 1536, 2048, 4096):
                row = {}
                for route, thr in (("codes_converted_on_the_way_to_lds", 1 << 30), ("dequantise_once_then_16bit_gemm", 17)):
                    setattr(muillm_ext, knob, thr)
                    row[route + "_ms"] = bench_prefill(lm8, tokens)["ms"]
                out[name]["tokens%d" % tokens] = row
        finally:
            setattr(muillm_ext, knob, default)
        del lm8, base
        torch.cuda.empty_cache()
    print(json.dumps({"probe_prompt_int8": out}))


def trace_prefill(tokens, passes=3):
    """Prefill passes of the 8B-shaped fp16 model (embedding to last-token logits) for a kernel trace:
    two warm-up passes, then `passes` passes with a device synchronisation after each."""
    import torch

    from muillm_amd.engineconfig import MuiEngineConfig
    from muillm_amd.modules.models.llama.model import MuiDecoderConfig, MuiLlamaForCausalLM

    cfg = MuiDecoderConfig.llama3_8b(max_position_embeddings=16384)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device="cuda", seed=0)
    ids = torch.randint(0, cfg.vocab_size, (1, tokens), device="cuda")
    with torch.no_grad():
        for _ in range(2):
            lm(input_ids=ids, num_logits_to_keep=1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(passes):
            lm(input_ids=ids, num_logits_to_keep=1)
            torch.cuda.synchronize()
    print(json.dumps({"trace_prefill": {"tokens": tokens, "passes": passes,
                                        "ms_per_pass": round((time.perf_counter() - t0) / passes * 1e3, 3)}}))


def _probe_prompt_whole_model():
    """Prefill of the 8B-shaped model (embedding to last-token logits) on the library's prompt kernels,
    and with every linear layer of more than 32 tokens handed to torch instead (rmsnorm kernel +
    F.linear, the reference's route for multi-token inputs) -- attention on the library's kernel in
    both. Same process, alternating."""
    import torch

    from muillm_amd import muillm_ext
    from muillm_amd.engineconfig import MuiEngineConfig
    from muillm_amd.modules.models.llama.model import MuiDecoderConfig, MuiLlamaForCausalLM

    cfg = MuiDecoderConfig.llama3_8b(max_position_embeddings=16384)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), cfg, dtype=torch.float16, device="cuda", seed=0)
    dispatchable = muillm_ext.kernel_dispatchable

    def run(tokens, iters=3):
        ids = torch.randint(0, cfg.vocab_size, (1, tokens), device="cuda")
        with torch.no_grad():
            for _ in range(2):
                lm(input_ids=ids, num_logits_to_keep=1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(iters):
                lm(input_ids=ids, num_logits_to_keep=1)
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / iters * 1e3

    res = {}
    for tokens in (64, 128, 512, 1024, 2048, 4096, 8192):
        ours = run(tokens)
        muillm_ext.kernel_dispatchable = lambda x: dispatchable(x) and muillm_ext._num_tokens(x) <= 32
        try:
            theirs = run(tokens)
        finally:
            muillm_ext.kernel_dispatchable = dispatchable
        res["tokens%d" % tokens] = {"library_kernels": round(ours, 2), "torch_gemm_route": round(theirs, 2)}
    return res


def pmc_probe_attention(launches=3):
    """Counter probe for flash decoding (`rocprofv3 --pmc FETCH_SIZE`): fused RoPE + cache write +
    attention at 32k context, batch 8 and batch 1, over distinct caches."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    hq, hkv, d = 32, 8, 128
    f16 = dict(device="cuda", dtype=torch.float16)
    stream = torch.cuda.current_stream().cuda_stream
    info = {}
    for S, B in ((32768, 8), (32768, 1)):
        caches = [(torch.randn(B, hkv, S, d, **f16), torch.randn(B, hkv, S, d, **f16)) for _ in range(launches)]
        qkvx = torch.randn(B, (hq + 2 * hkv) * d, **f16)
        cos, sin = [t.cuda() for t in _rope_tables_f32(S, d)]
        pos = torch.full((B, 1), S - 1, dtype=torch.int64, device="cuda")
        cpos = torch.full((1,), S - 1, dtype=torch.int64, device="cuda")
        n_splits = lib.mui_flash_decode_splits(B, hq, hkv, S)
        scratch = torch.empty(max(lib.mui_flash_decode_scratch_bytes(B, hq, d, n_splits), 16), dtype=torch.uint8, device="cuda")
        o = torch.empty(B, hq * d, **f16)
        qs = (hq + 2 * hkv) * d
        torch.cuda.synchronize()
        for kc, vc in caches:
            _lib.check(lib.mui_attn_decode_fused(
                stream, 0, qkvx.data_ptr(), qs, qkvx.data_ptr() + 2 * hq * d, qs, qkvx.data_ptr() + 2 * (hq + hkv) * d, qs,
                cos.data_ptr(), sin.data_ptr(), d // 2, cos.shape[0], pos.data_ptr(), 1, cpos.data_ptr(), S, kc.data_ptr(), vc.data_ptr(),
                hkv * S * d, S * d, d, None, 0, None, scratch.data_ptr(), n_splits, o.data_ptr(), B, hq, hkv, d, S),
                "mui_attn_decode_fused")
        torch.cuda.synchronize()
        info["ctx%d_batch%d" % (S, B)] = {"kv_bytes": B * 2 * hkv * S * d * 2, "n_splits": n_splits}
        del caches
        torch.cuda.empty_cache()
    print(json.dumps({"pmc_probe_attention": info}))


def kernel_table(lm, int8_tokens=(1, 4)):
    """GB/s of each fused kernel family at the benchmark shapes, HIP-event timed through the C ABI
    with pre-allocated outputs. Weights rotate over distinct buffers totalling >= 0.9 GB (the model's
    32 layers, or a ring) so neither L2 nor the 256 MB Infinity Cache can serve them ("cold").
    Bytes are algorithmic: weights (+ scales) once plus the mandatory vectors. Informational; times
    of the few-microsecond kernels include the launch-to-launch gap of back-to-back launches."""
    import torch

    from muillm_amd import _lib

    lib = _lib.load()
    layers = lm.model.layers
    nl = len(layers)
    hid, inter, v = lm.config.hidden_size, lm.config.intermediate_size, lm.config.vocab_size
    stream = torch.cuda.current_stream().cuda_stream
    f16 = dict(device="cuda", dtype=torch.float16)
    gamma = (1 + 0.1 * torch.randn(hid)).half().cuda()
    X, RES = torch.randn(16, hid, **f16), torch.randn(16, hid, **f16)
    HMID = torch.randn(16, inter, **f16)
    Y = torch.empty(16 * max(v, inter), **f16)
    out = {}

    sink = torch.zeros(64, dtype=torch.int32, device="cuda")

    def add(name, fn, nbytes, ring, iters=10, reads=None):
        """reads: [(buffer pointers, bytes), ...] = the matrices the call streams; the read probe
        over the same buffers (one launch per matrix the call itself uses a launch for) gives the
        least time those bytes can take on this device, launch latency included."""
        us = _event_time_us(fn, iters=max(iters * ring, 40), warm=max(ring, 8))
        out[name] = {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                     "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3)}
        if reads:
            def probe(i):
                for ptrs, nb in reads:
                    lib.mui_probe_read(stream, ptrs[i % len(ptrs)], nb, sink.data_ptr())
            floor = _event_time_us(probe, iters=max(iters * ring, 40), warm=max(ring, 8))
            out[name]["read_floor_us"] = round(floor, 2)
            out[name]["vs_read_floor"] = round(floor / us, 3)

    def linear(w, xin, norm, resid, n, k, b=1):
        return lambda i: lib.mui_linear(stream, 0, w[i % len(w)], k, xin.data_ptr(), norm, 1e-5, None, None,
                                        resid, Y.data_ptr(), n, k, b)

    # ---- 16-bit GEMV family at the decoder's shapes (1 token)
    qkv = [l.qkv_proj.linear.weight.data_ptr() for l in layers]
    n_qkv = layers[0].qkv_proj.linear.weight.shape[0]
    op = [l.self_attn.o_proj.weight.data_ptr() for l in layers]
    dn = [l.mlp.down_proj.weight.data_ptr() for l in layers]
    add("C1_norm_linear_residual_%dx%d" % (hid, hid), linear(op, X, gamma.data_ptr(), RES.data_ptr(), hid, hid),
        2 * hid * hid + 2 * (4 * hid), nl, reads=[(op, 2 * hid * hid)])
    add("qkv_norm_gemv_%dx%d" % (n_qkv, hid), linear(qkv, X, gamma.data_ptr(), None, n_qkv, hid),
        2 * n_qkv * hid + 2 * (2 * hid + n_qkv), nl, reads=[(qkv, 2 * n_qkv * hid)])
    add("o_proj_gemv_residual_%dx%d" % (hid, hid), linear(op, X, None, RES.data_ptr(), hid, hid),
        2 * hid * hid + 2 * (3 * hid), nl, reads=[(op, 2 * hid * hid)])
    add("down_gemv_residual_%dx%d" % (hid, inter), linear(dn, HMID, None, RES.data_ptr(), hid, inter),
        2 * hid * inter + 2 * (inter + 2 * hid), nl, reads=[(dn, 2 * hid * inter)])
    add("lm_head_gemv_%dx%d" % (v, hid), linear([lm.lm_head.weight.data_ptr()], X, None, None, v, hid),
        2 * v * hid + 2 * (hid + v), 1, iters=40, reads=[([lm.lm_head.weight.data_ptr()], 2 * v * hid)])

    # ---- C2: the whole MLP (fused norm + gate/up + SiLU, then down + residual), 1..8 tokens
    gu = [(l.mlp.gate_proj.weight.data_ptr(), l.mlp.up_proj.weight.data_ptr(), l.mlp.gate_proj.weight.stride(0),
           l.mlp.norm_weights.data_ptr()) for l in layers]
    # gate and up rows interleave in one packed buffer per layer, gate row 0 first
    gu_base = [min(g[0], g[1]) for g in gu]
    assert all(abs(g[0] - g[1]) == 2 * hid and g[2] == 2 * hid for g in gu)
    hbuf = torch.empty(16, inter, **f16)
    for b in (1, 2, 4, 8, 16):
        def mlp(i, b=b):
            gp, up, pitch, nw = gu[i % nl]
            lib.mui_gateup_silu(stream, 0, gp, up, pitch, X.data_ptr(), nw, 1e-5, hbuf.data_ptr(), inter, hid, b)
            lib.mui_linear(stream, 0, dn[i % nl], inter, hbuf.data_ptr(), None, 0.0, None, None, RES.data_ptr(),
                           Y.data_ptr(), hid, inter, b)
        name = "C2_mlp_%dx%d_tokens%d" % (inter, hid, b)
        add(name, mlp, 3 * inter * hid * 2 + 2 * hid + b * (3 * hid * 2 + 2 * inter * 2), nl,
            reads=[(gu_base, 4 * inter * hid), (dn, 2 * hid * inter)])
        # arithmetic rate of the batched call; from 3 tokens on it runs on the matrix cores (padded
        # to 16 token columns), whose utilisation is this rate over the dense fp16 MFMA peak
        tflops = 6.0 * inter * hid * b / out[name]["us"] / 1e6
        out[name]["TFLOP/s"] = round(tflops, 1)
        out[name]["compute_unit"] = "MFMA v_mfma_f32_16x16x32_f16" if b >= 3 else "vector ALUs"
        if b >= 3:
            out[name]["mfma_peak_frac"] = round(tflops / MFMA_FP16_PEAK_TFLOPS, 4)
            out[name]["mfma_issued_frac"] = round(tflops * 16.0 / b / MFMA_FP16_PEAK_TFLOPS, 4)

    # ---- C3: int8 per-channel GEMVs (ring of random codes: speed does not depend on the values)
    def i8_ring(n, k):
        cnt = max(2, int(0.95e9 // (n * k)) + 1)
        return [(torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda"),
                 (torch.rand(n, **f16) * 1e-3 + 1e-4)) for _ in range(cnt)]

    for b in int8_tokens:
        for name, n, k, norm, resid in (("qkv", n_qkv, hid, True, False), ("o_proj", hid, hid, False, True),
                                        ("down", hid, inter, False, True)):
            ring = i8_ring(n, k)
            xin = X if k == hid else HMID

            def f(i, ring=ring, xin=xin, n=n, k=k, norm=norm, resid=resid, b=b):
                q, sc = ring[i % len(ring)]
                lib.mui_int8_linear(stream, 0, q.data_ptr(), k, sc.data_ptr(), xin.data_ptr(),
                                    gamma.data_ptr() if norm else None, 1e-5, None,
                                    RES.data_ptr() if resid else None, Y.data_ptr(), n, k, b)
            add("C3_int8_%s_%dx%d_tokens%d" % (name, n, k, b), f,
                n * k + 2 * n + 2 * hid * norm + b * 2 * (k + n + n * resid), len(ring),
                reads=[([q.data_ptr() for q, _ in ring], n * k)])
            del ring
        ring = [(torch.randint(-127, 128, (inter, 2, hid), dtype=torch.int8, device="cuda"),
                 torch.rand(inter, 2, **f16) * 1e-3 + 1e-4) for _ in range(9)]

        def g(i, ring=ring, b=b):
            q, sc = ring[i % len(ring)]
            lib.mui_int8_gateup_silu(stream, 0, q.data_ptr(), q.data_ptr() + hid, 2 * hid, sc.data_ptr(),
                                     sc.data_ptr() + 2, 2, X.data_ptr(), gamma.data_ptr(), 1e-5, hbuf.data_ptr(),
                                     inter, hid, b)
        add("C3_int8_gateup_silu_%dx%d_tokens%d" % (2 * inter, hid, b), g,
            2 * inter * hid + 4 * inter + 2 * hid + b * 2 * (hid + inter), len(ring),
            reads=[([q.data_ptr() for q, _ in ring], 2 * inter * hid)])
        del ring
    torch.cuda.empty_cache()

    # ---- C3g: the same GEMVs on the reference's own format (uint8 codes + fp16 (scale, min) per group
    # of 128 inputs, muillm/quantization/rtnquantizer.py:49-88)
    gshift, gsz = 7, 128

    def g_ring(n, k):
        cnt = max(2, int(0.95e9 // (n * k)) + 1)
        return [(torch.randint(0, 256, (n, k), dtype=torch.uint8, device="cuda"),
                 torch.rand(n * (k // gsz), 2, **f16) * 1e-3 + 1e-4) for _ in range(cnt)]

    for b in int8_tokens:
        for name, n, k, norm, resid in (("qkv", n_qkv, hid, True, False), ("o_proj", hid, hid, False, True),
                                        ("down", hid, inter, False, True)):
            ring = g_ring(n, k)
            xin = X if k == hid else HMID

            def fg(i, ring=ring, xin=xin, n=n, k=k, norm=norm, resid=resid, b=b):
                q, smv = ring[i % len(ring)]
                lib.mui_int8_group_linear(stream, 0, q.data_ptr(), k, smv.data_ptr(), gshift, xin.data_ptr(),
                                          gamma.data_ptr() if norm else None, 1e-5, None,
                                          RES.data_ptr() if resid else None, Y.data_ptr(), n, k, b)
            add("C3g_group128_%s_%dx%d_tokens%d" % (name, n, k, b), fg,
                n * k + 4 * n * (k // gsz) + 2 * hid * norm + b * 2 * (k + n + n * resid), len(ring),
                reads=[([q.data_ptr() for q, _ in ring], n * k)])
            del ring
        ring = [(torch.randint(0, 256, (inter, 2, hid), dtype=torch.uint8, device="cuda"),
                 torch.rand(inter, 2, hid // gsz, 2, **f16) * 1e-3 + 1e-4) for _ in range(9)]

        def gg(i, ring=ring, b=b):
            q, smv = ring[i % len(ring)]
            lib.mui_int8_group_gateup_silu(stream, 0, q.data_ptr(), q.data_ptr() + hid, 2 * hid, smv.data_ptr(),
                                           smv.data_ptr() + 2 * 2 * (hid // gsz), 4 * (hid // gsz), gshift,
                                           X.data_ptr(), gamma.data_ptr(), 1e-5, hbuf.data_ptr(), inter, hid, b)
        add("C3g_group128_gateup_silu_%dx%d_tokens%d" % (2 * inter, hid, b), gg,
            2 * inter * hid + 8 * inter * (hid // gsz) + 2 * hid + b * 2 * (hid + inter), len(ring),
            reads=[([q.data_ptr() for q, _ in ring], 2 * inter * hid)])
        del ring
    torch.cuda.empty_cache()

    # ---- C4: fused RoPE + cache write + flash decoding, GQA 32/8 x 128 (bytes = the K/V rows read)
    hq, hkv, d = 32, 8, 128
    for S, B in ((1024, 1), (4096, 1), (16384, 1), (32768, 1), (1024, 8), (4096, 8), (32768, 8)):
        kvbytes = B * 2 * hkv * S * d * 2
        cnt = max(2, min(64, int(1.0e9 // kvbytes) + 1))
        caches = [(torch.randn(B, hkv, S, d, **f16), torch.randn(B, hkv, S, d, **f16)) for _ in range(cnt)]
        qkvx = torch.randn(B, (hq + 2 * hkv) * d, **f16)
        cos, sin = [t.cuda() for t in _rope_tables_f32(S, d)]
        pos = torch.full((B, 1), S - 1, dtype=torch.int64, device="cuda")
        cpos = torch.full((1,), S - 1, dtype=torch.int64, device="cuda")
        n_splits = lib.mui_flash_decode_splits(B, hq, hkv, S)
        scratch = torch.empty(max(lib.mui_flash_decode_scratch_bytes(B, hq, d, n_splits), 16), dtype=torch.uint8, device="cuda")
        o = torch.empty(B, hq * d, **f16)

        qs = (hq + 2 * hkv) * d

        def att(i, caches=caches, B=B, S=S, n_splits=n_splits):
            kc, vc = caches[i % len(caches)]
            lib.mui_attn_decode_fused(stream, 0, qkvx.data_ptr(), qs, qkvx.data_ptr() + 2 * hq * d, qs,
                                      qkvx.data_ptr() + 2 * (hq + hkv) * d, qs, cos.data_ptr(), sin.data_ptr(), d // 2,
                                      cos.shape[0], pos.data_ptr(), 1, cpos.data_ptr(), S, kc.data_ptr(), vc.data_ptr(),
                                      hkv * S * d, S * d, d, None, 0, None, scratch.data_ptr(), n_splits, o.data_ptr(),
                                      B, hq, hkv, d, S)
        add("C4_rope_cachewrite_flashdecode_ctx%d_batch%d_splits%d" % (S, B, n_splits), att, kvbytes + 4 * B * hq * d, cnt)
        del caches
        torch.cuda.empty_cache()
    return out


def _rope_tables_f32(max_pos, d, theta=500000.0):
    import torch

    inv = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    ang = torch.outer(torch.arange(max_pos, dtype=torch.float64), inv)
    return ang.cos().float().contiguous(), ang.sin().float().contiguous()


def cpu_baseline(config, layers_sample=4, steps_sample=100, ctx_len=64):
    """The reference's PyTorch fallback path (fp16 tensors, CPU) for one decode step, on a
    bounded sample: `layers_sample` decoder layers x `steps_sample` steps + one lm_head call,
    extrapolated linearly to the full depth. Reported, not a target."""
    import torch

    import oracle

    torch.manual_seed(0)
    hid, inter, v = config.hidden_size, config.intermediate_size, config.vocab_size
    hq, hkv = config.num_attention_heads, config.num_key_value_heads
    d = hid // hq
    mk = lambda *s: (torch.randn(*s) * 0.02).half()
    layers = []
    for _ in range(layers_sample):
        layers.append(dict(ln1=torch.ones(hid).half(), wqkv=mk((hq + 2 * hkv) * d, hid), wo=mk(hid, hid),
                           ln2=torch.ones(hid).half(), wg=mk(inter, hid), wu=mk(inter, hid), wd=mk(hid, inter),
                           k=torch.randn(1, hkv, ctx_len, d).half(), v=torch.randn(1, hkv, ctx_len, d).half()))
    lm_head = mk(v, hid)
    cos, sin = oracle.rope_tables(500000.0, d, ctx_len + steps_sample + 1, dtype=torch.float16)
    h0 = torch.randn(1, 1, hid).half()

    def layer_step(p, h, pos):
        qkv = oracle.linear(h, p["wqkv"], p["ln1"], 1e-5, reference_path=True)
        q = qkv[..., : hq * d].view(1, 1, hq, d).transpose(1, 2)
        k = qkv[..., hq * d : (hq + hkv) * d].view(1, 1, hkv, d).transpose(1, 2)
        vv = qkv[..., (hq + hkv) * d :].view(1, 1, hkv, d).transpose(1, 2)
        q, k = oracle.apply_rope(q, k, cos, sin, torch.tensor([[pos]]), reference_path=True)
        kk = torch.cat([p["k"], k], dim=2)
        vv = torch.cat([p["v"], vv], dim=2)
        a = oracle.decode_attention(q, kk, vv, reference_path=True)
        h1 = oracle.linear(a, p["wo"], residual=h, reference_path=True)
        return oracle.gateupdown_mlp(h1, p["wg"], p["wu"], p["wd"], p["ln2"], 1e-5, h1, reference_path=True)

    with torch.no_grad():
        layer_step(layers[0], h0, ctx_len)  # warm-up
        t0 = time.perf_counter()
        for s in range(steps_sample):
            h = h0
            for p in layers:
                h = layer_step(p, h, ctx_len + s)
        t_layers = (time.perf_counter() - t0) / (steps_sample * layers_sample)
        ones = torch.ones(hid).half()
        oracle.linear(h0, lm_head, ones, 1e-5, reference_path=True)
        head_times = []
        for _ in range(11):  # median of 11 calls: a single call varies 2x from run to run
            t0 = time.perf_counter()
            oracle.linear(h0, lm_head, ones, 1e-5, reference_path=True)
            head_times.append(time.perf_counter() - t0)
        t_head = sorted(head_times)[len(head_times) // 2]
    per_token = t_layers * config.num_hidden_layers + t_head
    layer_bytes = 2 * ((hq + 2 * hkv) * d * hid + hid * hid + 3 * hid * inter)
    head_bytes = 2 * v * hid
    return {"value": round(1.0 / per_token, 4), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{layers_sample} decoder layers x {steps_sample} decode steps (ctx {ctx_len}) + median of 11 lm_head "
                      f"calls of the reference's PyTorch fallback path in fp16 on CPU, extrapolated to "
                      f"{config.num_hidden_layers} layers",
            "s_per_layer": round(t_layers, 5), "s_lm_head": round(t_head, 5),
            "s_lm_head_min_max": [round(min(head_times), 5), round(max(head_times), 5)],
            "layer_weight_GB/s": round(layer_bytes / t_layers / 1e9, 1),
            "lm_head_weight_GB/s": round(head_bytes / t_head / 1e9, 1),
            "cpu_model": _cpu_model(), "host_cpus": os.cpu_count()}


def _cpu_model():
    """The host CPU's model string (/proc/cpuinfo), for reading the baseline figure."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform

    return platform.processor() or platform.machine()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--windows", type=int, default=5,
                    help="timed windows of --steps steps (each a fresh generation); value = their median")
    ap.add_argument("--layers", type=int, default=32, help="decoder depth (32 = the Llama-3-8B shape; fewer is NOT the benchmark)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-table", action="store_true")
    ap.add_argument("--no-variants", action="store_true", help="skip the eager (no HIP graph) and int8 decode runs")
    ap.add_argument("--tune-attention", default=None, metavar="WAVES,MIN_TOKENS,DIRECT,MFMA",
                    help="experiment: mui_tune_attention(waves per workgroup, min tokens per split, "
                         "longest unsplit sequence (-1 disables the head-parallel unsplit mode), shortest sequence for "
                         "the matrix-core kernel (-1 disables it))")
    ap.add_argument("--tune-skinny", default=None, metavar="MIN_TOKENS,STREAM_B,MULTI_MAX_TOKENS",
                    help="experiment: mui_tune_skinny(...) before anything is timed (2,0,1 sends int8 weights at "
                         "2..4 tokens to the matrix-core kernel)")
    ap.add_argument("--tune-prefill", default=None, metavar="TILE,WIDE_MAX_TOKENS",
                    help="experiment: mui_tune_prefill(...) before anything is timed (100 + tile: operand tiles staged "
                         "through registers instead of loaded straight into LDS)")
    ap.add_argument("--tune-gemv", default=None, metavar="ROWS,WGS_PER_CU",
                    help="experiment: mui_tune_gemv(...) before anything is timed")
    ap.add_argument("--tune-int8-quad", default=None, metavar="ON,MIN_TOKENS,WGS_PER_CU,SETS",
                    help="experiment: mui_tune_int8_quad(...) before anything is timed")
    ap.add_argument("--table-int8-tokens", default="1,4", metavar="LIST",
                    help="token counts of the int8 rows of the kernel table (the baseline's configuration: 1,4)")
    ap.add_argument("--only-kernel-table", action="store_true",
                    help="only time the per-kernel table (for rocprofv3 kernel traces of the C1-C4 shapes)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="only launch the gate/up GEMV and a calibration copy a few times (for rocprofv3 --pmc runs)")
    ap.add_argument("--pmc-probe-batched", action="store_true",
                    help="launch the 8-token MLP kernels a few times and exit (for rocprofv3 --pmc)")
    ap.add_argument("--pmc-probe-int8", action="store_true",
                    help="launch the int8 GEMVs of a Llama-3-8B layer at 1 and 4 tokens a few times and exit (for rocprofv3 --pmc)")
    ap.add_argument("--pmc-probe-attention", action="store_true",
                    help="launch flash decoding at 32k context a few times and exit (for rocprofv3 --pmc)")
    ap.add_argument("--probe-kernel-boundary", action="store_true",
                    help="time chains of near-empty dependent kernels in a replayed HIP graph and exit")
    ap.add_argument("--probe-warm", action="store_true",
                    help="time attention + o_proj and the decode rate over cache-warming settings and exit")
    ap.add_argument("--probe-chain", action="store_true",
                    help="time a chain of dependent GEMVs as ordinary launches and as overlapped launches with a "
                         "hand-off through memory, and exit")
    ap.add_argument("--probe-flash-splits", action="store_true",
                    help="time fused flash decoding at batch 1 over the number of sequence splits and exit")
    ap.add_argument("--probe-prompt", action="store_true",
                    help="time the prompt GEMMs and prompt attention at the Llama-3-8B shapes beside torch and exit")
    ap.add_argument("--trace-prefill", type=int, default=0, metavar="TOKENS",
                    help="a few prefill passes of the 8B-shaped model at this prompt length (for rocprofv3 --kernel-trace)")
    ap.add_argument("--probe-prompt-int8", action="store_true",
                    help="time the int8 model's prefill on both routes (codes converted in the GEMM / matrices "
                         "dequantised first) in both formats and exit")
    ap.add_argument("--probe-prompt-other-shapes", action="store_true",
                    help="time the prompt GEMM at the 70B- and 13B-shaped projections beside torch.matmul and exit")
    ap.add_argument("--pmc-probe-prompt", action="store_true",
                    help="launch the gate/up prompt GEMM (2048 tokens) and prompt attention (4096) three times and exit "
                         "(for rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build drives exactly one GPU (no tensor parallelism, no collectives); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from muillm_amd.engineconfig import MuiEngineConfig
    from muillm_amd.modules.models.llama.model import MuiDecoderConfig, MuiLlamaForCausalLM

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.pmc_probe:
        pmc_probe()
        return
    if args.pmc_probe_batched:
        pmc_probe_batched()
        return
    if args.pmc_probe_int8:
        pmc_probe_int8()
        return
    if args.pmc_probe_attention:
        pmc_probe_attention()
        return
    if args.probe_kernel_boundary:
        probe_kernel_boundary()
        return
    if args.probe_chain:
        probe_chain()
        return
    if args.probe_flash_splits:
        probe_flash_splits()
        return
    if args.tune_prefill:
        from muillm_amd import _lib
        _lib.check(_lib.load().mui_tune_prefill(*(int(v) for v in args.tune_prefill.split(","))), "mui_tune_prefill")
    if args.probe_prompt_int8:
        probe_prompt_int8()
        return
    if args.probe_prompt_other_shapes:
        probe_prompt_other_shapes()
        return
    if args.probe_prompt or args.pmc_probe_prompt:
        probe_prompt(counters_only=args.pmc_probe_prompt)
        return
    if args.trace_prefill:
        trace_prefill(args.trace_prefill)
        return
    if args.tune_attention:
        from muillm_amd import _lib

        w, mt, dt, mf = (int(v) for v in args.tune_attention.split(","))
        _lib.check(_lib.load().mui_tune_attention(w, mt, dt, mf), "mui_tune_attention")
    if args.tune_gemv:
        from muillm_amd import _lib
        _lib.check(_lib.load().mui_tune_gemv(*(int(v) for v in args.tune_gemv.split(","))), "mui_tune_gemv")
    if args.tune_int8_quad:
        from muillm_amd import _lib
        _lib.check(_lib.load().mui_tune_int8_quad(*(int(v) for v in args.tune_int8_quad.split(","))), "mui_tune_int8_quad")
    if args.tune_skinny:
        from muillm_amd import _lib

        a, b, c = (int(v) for v in args.tune_skinny.split(","))
        _lib.check(_lib.load().mui_tune_skinny(a, b, c), "mui_tune_skinny")
    config = MuiDecoderConfig.llama3_8b(num_hidden_layers=args.layers, max_position_embeddings=8192)
    lm = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), config, dtype=torch.float16, device="cuda", seed=0)
    torch.cuda.synchronize()

    if args.only_kernel_table:
        print(json.dumps({"kernels": kernel_table(lm, tuple(int(v) for v in args.table_int8_tokens.split(",")))}))
        return
    if args.probe_warm:
        probe_warm(lm, args.steps, args.warmup)
        return
    _progress("model built; headline decode windows")
    times, dec = bench_decode(lm, args.steps, args.warmup, windows=args.windows)
    times = times if isinstance(times, list) else [times]
    head = _rate_summary(times, args.steps)
    dt = _median(times)
    tokens_per_s = args.steps / dt
    hid, inter, v = config.hidden_size, config.intermediate_size, config.vocab_size
    hq, hkv, d = config.num_attention_heads, config.num_key_value_heads, 128
    weight_bytes = config.num_hidden_layers * 2 * ((hq + 2 * hkv) * d * hid + hid * hid + 3 * hid * inter) + 2 * v * hid

    result = {
        "metric": "tokens/s/user, Llama-3-8B-shaped fp16 decode, batch 1",
        "value": round(tokens_per_s, 2),
        "value_min": head["min"], "value_max": head["max"], "value_windows": head["windows"],
        "value_is": "median of %d timed windows, each a fresh generation (prefill, %d warm-up steps, %d timed steps); "
                    "fastest window: #%d" % (args.windows, args.warmup, args.steps, head["fastest_window"]),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": round(tokens_per_s / BASELINE_TOKENS_PER_S, 3) if args.layers == 32 else None,
        "dtype": "fp16",
        "data": "synthetic",
        "config": {
            "workload": f"Llama-3-8B-shaped decoder, random init N(0,0.02): {config.num_hidden_layers} layers, hidden 4096, "
                        "32/8 heads x128, MLP 14336, vocab 128256, RMSNorm eps 1e-5; 32-token random prompt then greedy "
                        "decode at batch 1, static KV cache, the decoder's own choice of launch mode (`launch`)",
            "launch": ("HIP-graph replay, %d steps per replay" % dec.STEPS_PER_REPLAY) if dec.use_graph
                      else "stream launches: one library call per step enqueues the layer stack",
            "prompt_len": 32, "batch": 1, "cache_capacity": dec.cache.max_cache_len,
            "weight_bytes_per_token": weight_bytes,
            "hbm_floor_ms": round(weight_bytes / (HBM_PEAK_GBPS * 1e9) * 1e3, 4),
            "end_to_end_frac_of_hbm_floor": round(weight_bytes / (HBM_PEAK_GBPS * 1e9) / (dt / args.steps), 4),
        },
    }
    _progress("headline %.2f tokens/s; roofline" % tokens_per_s)
    result["roofline"] = gateup_roofline(lm)
    result["roofline"]["measured_copy_ceiling_GB/s"] = measured_copy_ceiling()
    result["roofline"]["measured_read_ceiling_GB/s"] = measured_read_ceiling()
    if not args.no_kernel_table:
        _progress("kernel table")
        result["kernels"] = kernel_table(lm)
    del dec
    if not args.no_variants:
        # the two launch modes, each forced, on the headline's step counts
        _progress("variants: launch modes")
        t_g, dec_g = bench_decode(lm, args.steps, args.warmup, use_graph=True, windows=args.windows)
        t_e, dec_e = bench_decode(lm, args.steps, args.warmup, use_graph=False, windows=args.windows)
        t_g, t_e = (t if isinstance(t, list) else [t] for t in (t_g, t_e))
        sg, se = _rate_summary(t_g, args.steps), _rate_summary(t_e, args.steps)
        result["variants"] = {"fp16_graph_replay_tokens_per_s": sg["median"], "fp16_graph_replay_windows": sg["windows"],
                              "fp16_stream_launches_tokens_per_s": se["median"],
                              "fp16_stream_launches_windows": se["windows"]}
        del dec_e, dec_g
        for ctx in (4096,):
            dt_c, dec_c = bench_decode(lm, 64, 8, prompt_len=ctx)
            result["variants"]["fp16_context%d_tokens_per_s" % ctx] = round(64 / dt_c, 2)
            del dec_c
            torch.cuda.empty_cache()
        _progress("variants: prefill")
        for ptoks in (512, 4096):
            result["variants"]["prefill_%d" % ptoks] = bench_prefill(lm, ptoks)
            torch.cuda.empty_cache()
        _progress("variants: batches")
        for bsz in (4, 8, 16):
            dt_b, dec_b = bench_decode(lm, min(args.steps, 128), min(args.warmup, 8), batch=bsz)
            result["variants"]["fp16_batch%d_aggregate_tokens_per_s" % bsz] = round(bsz * min(args.steps, 128) / dt_b, 1)
            result["variants"]["fp16_batch%d_ms_per_step" % bsz] = round(dt_b / min(args.steps, 128) * 1e3, 4)
            del dec_b
        del lm
        torch.cuda.empty_cache()
        _progress("variants: bf16")
        lm_bf = MuiLlamaForCausalLM.from_config(MuiEngineConfig(), config, dtype=torch.bfloat16, device="cuda", seed=0)
        t_bf, dec_bf = bench_decode(lm_bf, args.steps, args.warmup, windows=3)
        result["variants"]["bf16_tokens_per_s"] = _rate_summary(t_bf, args.steps)["median"]
        del dec_bf, lm_bf
        torch.cuda.empty_cache()
        _progress("variants: int8")
        result["variants"]["int8"] = bench_int8_variant(config, args.steps, args.warmup)
        _progress("variants: int8 group 128")
        result["variants"]["int8_group128"] = bench_int8_variant(config, args.steps, args.warmup, group_size=128)
        _progress("variants: HuggingFace drop-in generate()")
        result["variants"]["hf_dropin_generate"] = bench_hf_dropin(config, args.steps)
        if "new_tokens_per_s" in result["variants"]["hf_dropin_generate"]:
            result["variants"]["hf_dropin_generate_tokens_per_s"] = result["variants"]["hf_dropin_generate"]["new_tokens_per_s"]
    if not args.no_cpu_baseline:
        _progress("cpu baseline")
        result["cpu_baseline"] = cpu_baseline(config)
        result["cpu_baseline"]["gpu_over_cpu"] = round(tokens_per_s / result["cpu_baseline"]["value"], 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
