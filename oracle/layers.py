"""CPU restatement of the reference's layer semantics (test infrastructure only).

All functions take torch CPU tensors.  Unless `reference_path=True`, inputs are upcast to
float64 and the float64 result is returned un-rounded: this is the accumulate-in-high-
precision reference the stated tolerances are measured against.

Citations are into the reference tree (Epliz/muiLLM).
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

__all__ = [
    "greedy_advance",
    "philox4x32_10",
    "sample_scores",
    "rmsnorm",
    "linear",
    "multilinear",
    "gateupdown_mlp",
    "gateup_silu",
    "rtn_quantize_group",
    "rtn_dequantize_group",
    "rtn_quantize_channel",
    "rtn_dequantize_channel",
    "int8_channel_linear",
    "int8_group_linear",
    "rope_inv_freq",
    "rope_tables",
    "rotate_half",
    "apply_rope",
    "static_cache_update",
    "repeat_kv",
    "decode_attention",
    "decoder_layer",
    "decoder_model_step",
    "next_pow2",
    "rel_err",
]

_HI = torch.float64


def _hi(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.detach().to("cpu", _HI)


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max |got - ref| / max |ref|  (the denominator the parity gates use)."""
    ref = ref.to(_HI)
    return float((got.to(_HI) - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# --------------------------------------------------------------------------------------
# RMSNorm -- muillm/modules/norm/rmsnorm.py:138-146 (HF LlamaRMSNorm form)
# --------------------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, reference_path: bool = False,
            round_to: Optional[torch.dtype] = None):
    """y = weight * x * rsqrt(mean(x^2, -1) + eps).

    reference_path=True reproduces the fallback literally: fp32 upcast, the normalised
    activations rounded back to the input dtype BEFORE the multiply by weight
    (rmsnorm.py:140-146).
    round_to=dtype: the exact result rounded once to that 16-bit type and returned in float64 --
    what the reference's RMSNorm kernel stores (one rounding after the multiply by weight,
    csrc/norm/rmsnorm_fp16_kernels.cu:111-115 and its bf16 twin), which is the operand its matrix
    multiply then reads whenever the norm and the linear are separate launches (multi-token
    inputs, csrc/modules/linear_module.cpp:57-79)."""
    if reference_path:
        input_dtype = x.dtype
        h = x.to(torch.float32)
        variance = h.pow(2).mean(-1, keepdim=True)
        h = h * torch.rsqrt(variance + eps)
        return weight * h.to(input_dtype)
    xh, wh = _hi(x), _hi(weight)
    variance = xh.pow(2).mean(-1, keepdim=True)
    out = wh * (xh * torch.rsqrt(variance + eps))
    return out.to(round_to).to(_HI) if round_to is not None else out


# --------------------------------------------------------------------------------------
# Linear (+ fused input norm, bias, residual) -- muillm/modules/linear.py:324-333
# --------------------------------------------------------------------------------------
def linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    norm_weights: Optional[torch.Tensor] = None,
    eps: float = 0.0,
    bias: Optional[torch.Tensor] = None,
    residual: Optional[torch.Tensor] = None,
    mul_bias: Optional[torch.Tensor] = None,
    reference_path: bool = False,
    norm_round: Optional[torch.dtype] = None,
):
    """y = F.linear(rmsnorm(x) if norm_weights else x, weight, bias) (+ residual).

    norm_round=dtype: the normalised activations pass through that 16-bit type on their way into
    the product (rmsnorm(round_to=dtype)), accumulation still in float64.

    `mul_bias` follows the kernel-level form y = (W x) * mul_bias + bias + residual
    (csrc/linear/linear_fp16_kernels.cu:163-356); the Python layer always passes None."""
    if reference_path:
        if norm_weights is not None:
            x = rmsnorm(x, norm_weights, eps, reference_path=True)
        out = F.linear(x, weight, None)
        if mul_bias is not None:
            out = out * mul_bias
        if bias is not None:
            out = out + bias
        if residual is not None:
            out = out + residual
        return out
    xh = rmsnorm(x, norm_weights, eps, round_to=norm_round) if norm_weights is not None else _hi(x)
    out = xh @ _hi(weight).T
    if mul_bias is not None:
        out = out * _hi(mul_bias)
    if bias is not None:
        out = out + _hi(bias)
    if residual is not None:
        out = out + _hi(residual)
    return out


def multilinear(
    x: torch.Tensor,
    weights: Sequence[torch.Tensor],
    norm_weights: Optional[torch.Tensor] = None,
    eps: float = 0.0,
    biases: Optional[Sequence[torch.Tensor]] = None,
    norm_round: Optional[torch.dtype] = None,
) -> Tuple[torch.Tensor, ...]:
    """Fused QKV: one linear over the row-concatenated weights, returned as last-dim slices
    (muillm/modules/multilinear.py:56-66,186-237)."""
    w = torch.cat(list(weights), dim=0)
    b = torch.cat(list(biases), dim=0) if biases is not None else None
    out = linear(x, w, norm_weights, eps, b, norm_round=norm_round)
    outs, start = [], 0
    for wi in weights:
        outs.append(out[..., start : start + wi.shape[0]])
        start += wi.shape[0]
    return tuple(outs)


# --------------------------------------------------------------------------------------
# Gate/Up/Down MLP -- muillm/modules/gateupdownmlp.py:343-359
# --------------------------------------------------------------------------------------
def gateup_silu(x, gate_w, up_w, norm_weights=None, eps: float = 0.0, norm_round: Optional[torch.dtype] = None):
    """silu(G xn) * (U xn): the intermediate the fused kernel writes
    (csrc/ffn/gateup_fp16_kernels.cu:596-601). norm_round: as in linear()."""
    xh = rmsnorm(x, norm_weights, eps, round_to=norm_round) if norm_weights is not None else _hi(x)
    g = xh @ _hi(gate_w).T
    u = xh @ _hi(up_w).T
    return F.silu(g) * u


def gateupdown_mlp(
    x, gate_w, up_w, down_w, norm_weights=None, eps: float = 0.0, residual=None,
    reference_path: bool = False, round_intermediate: Optional[torch.dtype] = None,
    norm_round: Optional[torch.dtype] = None,
):
    """out = down(silu(gate(xn)) * up(xn)) + residual  (_forward_unfused, :343-359).

    round_intermediate=torch.float16 rounds the 14336-wide intermediate to 16 bits the way
    both the reference kernels and this build store it between the two GEMVs."""
    if reference_path:
        if norm_weights is not None:
            x = rmsnorm(x, norm_weights, eps, reference_path=True)
        g = F.linear(x, gate_w)
        u = F.linear(x, up_w)
        out = F.linear(F.silu(g) * u, down_w)
        if residual is not None:
            out = out + residual
        return out
    h = gateup_silu(x, gate_w, up_w, norm_weights, eps, norm_round=norm_round)
    if round_intermediate is not None:
        h = h.to(round_intermediate).to(_HI)
    out = h @ _hi(down_w).T
    if residual is not None:
        out = out + _hi(residual)
    return out


# --------------------------------------------------------------------------------------
# RTN quantisation
# --------------------------------------------------------------------------------------
def rtn_quantize_group(w: torch.Tensor, group_size: int = 128, f: float = 1.0):
    """The reference's asymmetric group-wise uint8 RTN
    (muillm/quantization/rtnquantizer.py:49-88): returns (uint8 [N,K], (scale,min) [N*G,2])
    with the pair stored in w's dtype."""
    if group_size <= 0 or (group_size & (group_size - 1)) != 0:
        raise ValueError("group size must be a power of two")
    if w.dim() != 2 or w.shape[-1] % group_size != 0:
        raise ValueError("group size must divide the last dimension of a 2-D weight")
    to_quant = w.reshape(-1, group_size).to(torch.float32)
    max_val = to_quant.amax(dim=1, keepdim=True)
    min_val = to_quant.amin(dim=1, keepdim=True)
    val_range = (f * (max_val - min_val)).clamp(min=1e-6)
    val_center = (min_val + max_val) * 0.5
    min_val = val_center - val_range * 0.5
    scales = val_range / 255
    q = to_quant.sub(min_val).div(scales).clamp(0, 255).round().to(torch.uint8).reshape_as(w)
    return q, torch.cat([scales, min_val], dim=-1).to(w.dtype)


def rtn_dequantize_group(q: torch.Tensor, scales_min_vals: torch.Tensor, group_size: int,
                         dtype: torch.dtype = torch.float16, kernel_form: bool = True):
    """kernel_form=True: half(float(q)*float(scale) + float(min)), one rounding
    (csrc/int8_dequantization_kernel.cu:50-59).  kernel_form=False: the Python fallback,
    multiply then add in the scale dtype, two roundings (rtnquantizer.py:91-102)."""
    qg = q.reshape(-1, group_size)
    scales = scales_min_vals[:, None, 0]
    mins = scales_min_vals[:, None, 1]
    if kernel_form:
        # q*scale+min is exact in float64; rounding it to fp32 reproduces the fp32 fma's
        # single rounding, the store then rounds fp32 -> 16 bit.
        dq = torch.addcmul(mins.to(_HI), qg.to(_HI), scales.to(_HI))
        return dq.to(torch.float32).reshape_as(q).to(dtype)
    return qg.mul(scales).add(mins).reshape_as(q).to(dtype)


def rtn_quantize_channel(w: torch.Tensor):
    """Symmetric per-output-channel int8 RTN (the on-device format of the int8 decode
    GEMVs): s[n] = half(max|w[n,:]| / 127), q = clamp(round_half_even(w / s), -127, 127).

    The divide is done in fp32 on the fp16-rounded scale so that quantise and dequantise
    agree on s.  An all-zero row gets the smallest positive fp16 as scale (q = 0)."""
    if w.dim() != 2:
        raise ValueError("only 2-D weights can be quantised")
    wf = w.to(torch.float32)
    amax = wf.abs().amax(dim=1)
    s = (amax / 127.0).to(torch.float16)
    tiny = torch.tensor(2.0 ** -24, dtype=torch.float16)
    s = torch.where(s > 0, s, tiny)
    q = torch.round(wf / s.to(torch.float32)[:, None]).clamp(-127, 127).to(torch.int8)
    return q, s


def rtn_dequantize_channel(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """w = half(float(q) * float(s)): an 8-bit integer times an 11-bit significand is exact
    in fp32, so this equals torch's q.half() * s[:, None] bit for bit."""
    return (q.to(torch.float32) * s.to(torch.float32)[:, None]).to(s.dtype)


def int8_channel_linear(x, q, s, norm_weights=None, eps=0.0, bias=None, residual=None):
    """Dequantise-then-linear (muillm/modules/quantized/int8linear.py:279-293) on the
    per-channel format, accumulated in float64."""
    return linear(x, rtn_dequantize_channel(q, s), norm_weights, eps, bias, residual)


def int8_group_linear(x, q, scales_min_vals, group_size, norm_weights=None, eps=0.0,
                      bias=None, residual=None):
    """Same for the reference's group format; the weights are the exact (un-rounded)
    q*scale+min values, which is what the reference int8 GEMV accumulates
    (csrc/int8_linear_kernels.cu:213-236)."""
    qg = q.reshape(-1, group_size).to(_HI)
    w = (qg * scales_min_vals[:, None, 0].to(_HI) + scales_min_vals[:, None, 1].to(_HI)).reshape(q.shape)
    return linear(x, w, norm_weights, eps, bias, residual)


# --------------------------------------------------------------------------------------
# RoPE -- muillm/modules/attention/rotaryembedding.py:23-64,313-351
# --------------------------------------------------------------------------------------
def rope_inv_freq(theta: float, dim: int) -> torch.Tensor:
    """HF 'default' rope init: 1 / theta^(2i/dim), computed in fp32."""
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).to(torch.float32) / dim))


def rope_tables(theta: float, dim: int, max_pos: int, dtype=torch.float32, attention_scaling=1.0):
    """cos/sin tables [max_pos, dim] with emb = cat(freqs, freqs) (:313-337).  The angle is
    formed in fp32 like the reference does."""
    inv_freq = rope_inv_freq(theta, dim)
    t = torch.arange(max_pos, dtype=torch.int64).type_as(inv_freq)
    freqs = torch.outer(t, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return (emb.cos() * attention_scaling).to(dtype), (emb.sin() * attention_scaling).to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2 :]
    return torch.cat((-x2, x1), dim=-1)


def apply_rope(q, k, cos, sin, position_ids, reference_path: bool = False):
    """q, k: [B, H, T, D]; cos, sin: tables [max_pos, D]; position_ids [B, T].
    q' = q*cos + rotate_half(q)*sin (:31-64)."""
    c = cos[position_ids].unsqueeze(1)  # [B,1,T,D]
    s = sin[position_ids].unsqueeze(1)
    if reference_path:
        c, s = c.to(q.dtype), s.to(q.dtype)
        return (q * c) + (rotate_half(q) * s), (k * c) + (rotate_half(k) * s)
    c, s, qh, kh = _hi(c), _hi(s), _hi(q), _hi(k)
    return (qh * c) + (rotate_half(qh) * s), (kh * c) + (rotate_half(kh) * s)


# --------------------------------------------------------------------------------------
# Static KV cache -- muillm/modules/kvcache/cache_utils.py:185-204,681-712
# --------------------------------------------------------------------------------------
def next_pow2(x: int) -> int:
    if x < 0:
        raise ValueError("x should be positive")
    p = 1
    while p < x:
        p *= 2
    return p


def static_cache_update(k_cache, v_cache, k_new, v_new, cache_position, seen_tokens: int):
    """Index-copy the new rows at cache_position along dim 2, then return views narrowed to
    the tokens seen so far (StaticCache.update + narrow, cache_utils.py:185-204).
    Caches are [B, Hkv, MAX_T, D] and are modified in place."""
    k_cache.index_copy_(2, cache_position, k_new.to(k_cache.dtype))
    v_cache.index_copy_(2, cache_position, v_new.to(v_cache.dtype))
    seen = seen_tokens + k_new.shape[-2]
    return k_cache.narrow(2, 0, seen), v_cache.narrow(2, 0, seen), seen


# --------------------------------------------------------------------------------------
# Decode attention -- muillm/modules/attention/baseattention.py:219-253, kvcache.py:3-12
# --------------------------------------------------------------------------------------
def repeat_kv(h: torch.Tensor, n_rep: int) -> torch.Tensor:
    b, hk, s, d = h.shape
    if n_rep == 1:
        return h
    return h[:, :, None, :, :].expand(b, hk, n_rep, s, d).reshape(b, hk * n_rep, s, d)


def decode_attention(q, k, v, mask=None, reference_path: bool = False):
    """q [B,Hq,T,D], k/v [B,Hkv,S,D], additive mask broadcastable to [B,1,T,S] or None.
    Returns [B, T, Hq*D].  softmax(q k^T / sqrt(D) + mask) v with GQA head h -> kv head
    h // (Hq/Hkv)."""
    b, hq, t, d = q.shape
    n_rep = hq // k.shape[1]
    if reference_path:
        kk, vv = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
        w = torch.matmul(q, kk.transpose(2, 3)) / math.sqrt(d)
        if mask is not None:
            w = w + mask
        w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
        o = torch.matmul(w, vv)
        return o.transpose(1, 2).contiguous().reshape(b, t, hq * d)
    # Same arithmetic without materialising the repeated K/V: query heads are grouped per
    # KV head ([Hkv, n_rep*T, D] x [Hkv, D, S]); one batch row at a time to bound memory.
    hkv, s = k.shape[1], k.shape[2]
    outs = []
    for bi in range(b):
        qh = _hi(q[bi]).reshape(hkv, n_rep * t, d)
        kh, vh = _hi(k[bi]), _hi(v[bi])
        w = torch.matmul(qh, kh.transpose(1, 2)) / math.sqrt(d)  # [Hkv, n_rep*T, S]
        if mask is not None:
            mb = _hi(mask[bi] if mask.shape[0] > 1 else mask[0])  # [1 or Hq, T, S]
            mb = mb.expand(hq, t, s).reshape(hkv, n_rep * t, s)
            w = w + mb
        w = F.softmax(w, dim=-1)
        o = torch.matmul(w, vh).reshape(hq, t, d)
        outs.append(o.transpose(0, 1).reshape(t, hq * d))
    return torch.stack(outs, dim=0)


# --------------------------------------------------------------------------------------
# Decoder layer -- muillm/modules/decoder/decoder.py:130-165
# --------------------------------------------------------------------------------------
def decoder_layer(
    h: torch.Tensor,            # [B, T, hidden]
    p: dict,                    # weights: ln1, wq, wk, wv, wo, ln2, wg, wu, wd (+ eps)
    k_cache: torch.Tensor,      # [B, Hkv, MAX_T, D]  (modified in place)
    v_cache: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    position_ids: torch.Tensor,  # [B, T]
    cache_position: torch.Tensor,  # [T]
    seen_tokens: int,
    n_heads: int,
    n_kv_heads: int,
    store_dtype: torch.dtype = torch.float16,
    sliding_window: Optional[int] = None,
    norm_round: Optional[torch.dtype] = None,
):
    """One decoder layer with the rounding points of the fused path: q/k/v, attention
    output, post-attention hidden state and MLP intermediate are stored in `store_dtype`
    between kernels; everything inside a kernel is float64 here (norm_round=dtype: except the
    normalised activations, which pass through that type as in linear()).
    Causal masking is applied for T > 1 (prefill). sliding_window=W hides, from the query in
    cache slot c, the keys at or before c - W (muillm/modules/models/mistral/model.py:590-602)."""
    b, t, hid = h.shape
    d = hid // n_heads
    eps = p["eps"]
    rnd = lambda z: z.to(store_dtype)
    q, k, v = multilinear(h, [p["wq"], p["wk"], p["wv"]], p["ln1"], eps, norm_round=norm_round)
    q = rnd(q).view(b, t, n_heads, d).transpose(1, 2)
    k = rnd(k).view(b, t, n_kv_heads, d).transpose(1, 2)
    v = rnd(v).view(b, t, n_kv_heads, d).transpose(1, 2)
    qr, kr = apply_rope(q, k, cos, sin, position_ids)
    qr, kr = rnd(qr), rnd(kr)
    kk, vv, seen = static_cache_update(k_cache, v_cache, kr, v, cache_position, seen_tokens)
    mask = None
    if t > 1 or (sliding_window is not None and kk.shape[2] > sliding_window):
        s = kk.shape[2]
        qpos = cache_position.view(t, 1)
        kpos = torch.arange(s).view(1, s)
        visible = kpos <= qpos
        if sliding_window is not None:
            visible = visible & (kpos > qpos - sliding_window)
        mask = torch.where(visible, 0.0, float("-inf")).to(_HI).view(1, 1, t, s)
    attn = rnd(decode_attention(qr, kk, vv, mask))
    h1 = rnd(linear(attn, p["wo"], residual=h))
    out = gateupdown_mlp(h1, p["wg"], p["wu"], p["wd"], p["ln2"], eps, residual=h1,
                         round_intermediate=store_dtype, norm_round=norm_round)
    return rnd(out), seen


# --------------------------------------------------------------------------------------
# Whole decoder -- muillm/modules/models/llama/model.py:298-322,360-406,778-785
# --------------------------------------------------------------------------------------
def decoder_model_step(ids, params, k_caches, v_caches, cos, sin, seen_tokens: int, n_heads: int,
                       n_kv_heads: int, store_dtype: torch.dtype = torch.float16,
                       sliding_window: Optional[int] = None, norm_round: Optional[torch.dtype] = None):
    """Embed -> layers -> final RMSNorm -> lm_head for `ids` [B, T] appended after
    `seen_tokens` cached tokens. params: {'embed', 'layers': [layer dicts], 'norm', 'lm_head',
    'eps'}. Returns (logits float64 [B, T, V], new seen_tokens). Hidden states between layers
    are stored in `store_dtype` like the fused path does."""
    b, t = ids.shape
    h = params["embed"][ids].to(store_dtype)
    pos = torch.arange(seen_tokens, seen_tokens + t).unsqueeze(0).expand(b, t)
    cpos = torch.arange(seen_tokens, seen_tokens + t)
    seen = seen_tokens
    for li, lp in enumerate(params["layers"]):
        h, seen = decoder_layer(h, lp, k_caches[li], v_caches[li], cos, sin, pos, cpos, seen_tokens,
                                n_heads, n_kv_heads, store_dtype, sliding_window, norm_round)
    hn = rmsnorm(h, params["norm"], params["eps"]).to(store_dtype)
    return linear(hn, params["lm_head"]), seen


# ---------------------------------------------------------------------------------------
# generation-loop helper
# ---------------------------------------------------------------------------------------
def greedy_advance(logits, unfinished, eos_token_ids, pad_token_id: int, steps_done: int, max_steps: int):
    """Greedy token choice plus the stop check of the reference's sampling loop:
    next_tokens = argmax(logits) (muillm/sampling/generation.py:330-335); rows that had already
    finished emit pad_token_id when an eos criterion exists; a row stays unfinished while its
    token is none of eos_token_ids and steps remain (muillm_add_tokens_check_finished_kernel,
    csrc/generation/generation.cu:29-113: `next_token = prev_unfinished ? next_token : pad`,
    `unfinished &= next_token != eos`, `unfinished &= T <= max_length`).
    logits [B, V]; unfinished [B] (0/1); steps_done = tokens already emitted per row.
    Returns (tokens [B] int64, unfinished [B] int64). Plain Python loops: test sizes only."""
    lg = logits.float()
    b = lg.shape[0]
    toks = torch.zeros(b, dtype=torch.int64)
    unf = torch.zeros(b, dtype=torch.int64)
    eos = [int(e) for e in eos_token_ids] if eos_token_ids is not None else []
    for r in range(b):
        row = lg[r]
        best, best_i = float("-inf"), None
        for i in range(row.shape[0]):  # lowest index wins ties; NaN never wins
            v = float(row[i])
            if v > best:
                best, best_i = v, i
        tok = 0 if best_i is None else best_i
        was = bool(unfinished[r]) if unfinished is not None else True
        if eos and not was:
            tok = int(pad_token_id)
        still = was and (steps_done + 1 < max_steps)
        for e in eos:
            still = still and tok != e
        toks[r] = tok
        unf[r] = 1 if still else 0
    return toks, unf


# ---------------------------------------------------------------------------------------
# sync-free sampling
# ---------------------------------------------------------------------------------------
def philox4x32_10(counter, key):
    """Philox4x32-10 block function (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
    as 1, 2, 3", SC'11; the generator behind torch's CUDA RNG as well). counter: 4 uint32, key: 2
    uint32 -> 4 uint32. Pinned by the known-answer vectors of the Random123 distribution."""
    m0, m1, w0, w1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
    c = [int(x) & 0xFFFFFFFF for x in counter]
    k = [int(x) & 0xFFFFFFFF for x in key]
    for _ in range(10):
        p0, p1 = m0 * c[0], m1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF, p1 & 0xFFFFFFFF,
             ((p0 >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF, p0 & 0xFFFFFFFF]
        k = [(k[0] + w0) & 0xFFFFFFFF, (k[1] + w1) & 0xFFFFFFFF]
    return c


def sample_scores(logits_row, temperature: float, seed: int, row: int, step: int):
    """Scores whose argmax is the sampled token: logit / temperature - log q with q = -log u ~ Exp(1),
    i.e. the draw argmax(softmax(logits / temperature) / q) of the reference's
    muillm_multinomial_sample_one_no_sync (muillm/sampling/multinomial.py:4-6) in log space.
    u for vocabulary entry v: Philox4x32-10 with key (seed low, seed high) and counter
    (v // 4, row, step mod 2^32, 0), lane v % 4, u = ((bits >> 8) + 1) * 2^-24. float64. Loops:
    small vocabularies only."""
    import math

    lg = logits_row.double()
    out = torch.empty_like(lg)
    blocks = {}
    for v in range(lg.shape[0]):
        c = v // 4
        if c not in blocks:
            blocks[c] = philox4x32_10([c, row, step & 0xFFFFFFFF, 0], [seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF])
        u = ((blocks[c][v % 4] >> 8) + 1) * 2.0 ** -24
        q = max(-math.log(u), 1e-30)
        out[v] = float(lg[v]) / temperature - math.log(q)
    return out
