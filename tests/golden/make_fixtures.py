#!/usr/bin/env python3
"""Writes tests/golden/hf_llama_small.npz: small input/output vectors produced by the
HuggingFace Transformers *library* (not by the reference repository, which has no data files
and cannot be imported here) for the layer definitions the reference swaps out:
LlamaRMSNorm, LlamaMLP, rotary tables + apply_rotary_pos_emb, eager_attention_forward
(GQA), the 'llama3' rope scaling, and a 2-layer LlamaForCausalLM. The CPU tests check the
oracle against these vectors, so the GPU box never needs transformers to pin the oracle.

Run from the repo root:  python tests/golden/make_fixtures.py
(seeded; transformers 5.15 / torch 2.10 wrote the committed file)."""
import os

import numpy as np
import torch
import transformers
from transformers.models.llama import modeling_llama as ml
from transformers.models.llama.configuration_llama import LlamaConfig


def main():
    torch.manual_seed(1234)
    out = {}
    cfg = LlamaConfig(hidden_size=128, intermediate_size=160, num_hidden_layers=2, num_attention_heads=2,
                      num_key_value_heads=1, vocab_size=300, max_position_embeddings=96, rms_norm_eps=1e-5,
                      rope_theta=500000.0, attention_bias=False, mlp_bias=False)
    cfg._attn_implementation = "eager"

    # RMSNorm (fp32)
    norm = ml.LlamaRMSNorm(128, eps=1e-5)
    norm.weight.data = 1 + 0.1 * torch.randn(128)
    x = torch.randn(3, 128)
    out["norm_w"], out["norm_x"], out["norm_y"] = norm.weight.data, x, norm(x)

    # MLP (fp32)
    mlp = ml.LlamaMLP(cfg)
    for p in mlp.parameters():
        p.data.normal_(0, 0.05)
    xm = torch.randn(3, 128)
    out["mlp_wg"], out["mlp_wu"], out["mlp_wd"] = mlp.gate_proj.weight.data, mlp.up_proj.weight.data, mlp.down_proj.weight.data
    out["mlp_x"], out["mlp_y"] = xm, mlp(xm)

    # rotary tables and application
    rot = ml.LlamaRotaryEmbedding(cfg)
    pos = torch.tensor([[0, 1, 5, 95], [7, 8, 9, 10]])
    q = torch.randn(2, 4, 4, 64)
    k = torch.randn(2, 2, 4, 64)
    cos, sin = rot(q, pos)
    qr, kr = ml.apply_rotary_pos_emb(q, k, cos, sin)
    out.update(rope_pos=pos, rope_q=q, rope_k=k, rope_cos=cos, rope_sin=sin, rope_qr=qr, rope_kr=kr,
               rope_inv_freq=rot.inv_freq)

    # llama3 rope scaling inverse frequencies
    cfg3 = LlamaConfig(hidden_size=512, num_attention_heads=4, max_position_embeddings=131072,
                       rope_parameters={"rope_type": "llama3", "rope_theta": 500000.0, "factor": 8.0,
                                        "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                        "original_max_position_embeddings": 8192})
    rot3 = ml.LlamaRotaryEmbedding(cfg3)
    out["llama3_inv_freq"] = rot3.inv_freq

    # eager GQA attention with an additive mask
    class _M:  # what eager_attention_forward reads from its module argument
        num_key_value_groups = 2
        training = False

    qa, ka, va = torch.randn(2, 4, 1, 64), torch.randn(2, 2, 9, 64), torch.randn(2, 2, 9, 64)
    mask = torch.zeros(2, 1, 1, 9)
    mask[0, 0, 0, :3] = torch.finfo(torch.float32).min
    ao, _ = ml.eager_attention_forward(_M(), qa, ka, va, mask, scaling=64 ** -0.5)
    out.update(attn_q=qa, attn_k=ka, attn_v=va, attn_mask=mask, attn_out=ao)  # ao: [B, T, H, D]

    # whole tiny model, fp32: logits for a 2 x 10 prompt
    small = LlamaConfig(hidden_size=128, intermediate_size=192, num_hidden_layers=2, num_attention_heads=2,
                        num_key_value_heads=1, vocab_size=64, max_position_embeddings=32, rms_norm_eps=1e-5,
                        rope_theta=500000.0, attention_bias=False, mlp_bias=False, tie_word_embeddings=False)
    small._attn_implementation = "eager"
    model = ml.LlamaForCausalLM(small).eval()
    for p in model.parameters():  # fp16-representable weights so the fixture can store them in 16 bits
        p.data = p.data.half().float()
    ids = torch.randint(0, 64, (2, 10))
    with torch.no_grad():
        logits = model(input_ids=ids, use_cache=False).logits
    out["model_ids"], out["model_logits"] = ids, logits
    sd = model.state_dict()
    for name, t in sd.items():
        out["sd." + name] = t.half()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hf_llama_small.npz")
    np.savez_compressed(path, **{k: v.detach().numpy() for k, v in out.items()},
                        versions=np.array([transformers.__version__, torch.__version__]))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
