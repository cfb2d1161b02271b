"""repeat_kv for the unfused attention routes (muillm/modules/attention/kvcache.py:3-12 in the
reference, HuggingFace's helper of the same name): every KV head repeated for the query heads that
share it. The decode and prompt kernels never call it -- they read each KV head once."""
import torch


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[batch, kv_heads, seq, dim] -> [batch, kv_heads * n_rep, seq, dim] with head h of the result
    being KV head h // n_rep (what torch.repeat_interleave(x, n_rep, dim=1) returns)."""
    if n_rep == 1:
        return hidden_states
    b, h, s, d = hidden_states.shape
    return hidden_states.unsqueeze(2).expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)
