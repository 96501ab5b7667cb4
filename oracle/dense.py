"""Oracle (test infrastructure): dense softmax attention, with and without a KV-cache write.

Follows wan/modules/attention.py:141-187 (`attention`, SDPA branch: non-causal
softmax(q k^T * d^-0.5) v on [B,L,H,D] tensors) and wan/modules/attn_patch.py:416-434
(`full_attention_with_kv_cache` / `attention_ref`: slice-assign new K/V into the
cache view, then attention over the whole view).
"""
import torch


def attention(q, k, v, sm_scale=None, dtype=torch.float64, return_lse=False):
    """q [B,Lq,H,D], k,v [B,Lk,H,D] -> [B,Lq,H,D] (and natural-log LSE [B,H,Lq])."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    B, Lq, H, D = q.shape
    out = torch.empty((B, Lq, H, D), dtype=dtype)
    lse = torch.empty((B, H, Lq), dtype=dtype)
    for b in range(B):
        for h in range(H):
            s = (q[b, :, h].to(dtype) @ k[b, :, h].to(dtype).T) * sm_scale
            lse[b, h] = torch.logsumexp(s, -1)
            out[b, :, h] = torch.exp(s - lse[b, h].unsqueeze(-1)) @ v[b, :, h].to(dtype)
    return (out, lse) if return_lse else out


def full_attention_with_kv_cache(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale=None,
                                 dtype=torch.float64):
    """Writes new_k/new_v into the cache views IN PLACE at [start_idx:end_idx], then dense attention."""
    if not (0 <= start_idx <= end_idx <= k_cache.shape[1]):
        raise ValueError("start_idx/end_idx out of range")
    k_cache[:, start_idx:end_idx] = new_k
    v_cache[:, start_idx:end_idx] = new_v
    return attention(q, k_cache, v_cache, sm_scale, dtype)


def dense_flops(B, H, D, Lq, Lk):
    return 4 * B * H * Lq * Lk * D
