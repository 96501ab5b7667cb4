"""Fused q/k prologue (RMSNorm + 3-D RoPE + KV-cache write) and the RoPE angle table.

Replaces, in CausalWanSelfAttention.forward (wan/modules/causal_model.py:801-807, 899-905) and the
Monarch op (wan/modules/monarch_attn.py:1783-1785, 1230-1231): norm_q / norm_k, causal_rope_apply
on q and k, the block-order rearrangement of new K/V and their slice-assignment into the cache.
"""
import ctypes as C
import math

import torch

from . import lib as _l
from .monarch_attn import _DT, _stream


def rope_table(head_dim, max_pos=1024, theta=10000.0, device=None):
    """float64 [max_pos, head_dim/2, 2] table of (cos, sin) of pos * theta^(-2m'/dim_axis), the three
    axis ladders concatenated as the reference builds them (model.py:421-428,
    causal_model.py:1350-1357): dims (d - 4(d//6), 2(d//6), 2(d//6))."""
    d = head_dim
    cols = []
    pos = torch.arange(max_pos, dtype=torch.float64)[:, None]
    for dim_axis in (d - 4 * (d // 6), 2 * (d // 6), 2 * (d // 6)):
        inv = 1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64),
                              torch.arange(0, dim_axis, 2, dtype=torch.float64) / dim_axis)
        cols.append(pos * inv[None, :])
    ang = torch.cat(cols, dim=1)
    tab = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).contiguous()
    return tab.to(device) if device is not None else tab


def qk_prologue(xq, xk, xv, wq, wk, num_heads, grid, start_frame, rope, k_cache, v_cache, start_idx,
                f_tied=1, h_reduce=1, w_reduce=1, eps=1e-6):
    """xq, xk, xv: [B, S, C] projections (S = F*h*w tokens of `grid` = (F, h, w)); wq, wk: [C] RMSNorm
    weights in the same dtype.  Returns roped q [B, S, H, D]; writes roped k and v into
    k_cache/v_cache[:, start_idx:start_idx+S] in Monarch block order, in place."""
    B, S, Cdim = xq.shape
    F, h, w = grid
    if Cdim % num_heads:
        raise ValueError("model dim is not a multiple of num_heads")
    D = Cdim // num_heads
    for name, t in (("xq", xq), ("xk", xk), ("xv", xv)):
        if t.shape != xq.shape or t.dtype != xq.dtype or not t.is_cuda or t.stride(2) != 1:
            raise ValueError(f"{name}: expected a [B, S, C] GPU tensor like xq with a contiguous last axis")
        if t.stride() != xq.stride():
            raise ValueError("xq, xk, xv must share strides")
    if wq.dtype != xq.dtype or wk.dtype != xq.dtype:
        raise ValueError("RMSNorm weights must have the activations' dtype")
    if rope.dtype != torch.float64 or rope.dim() != 3 or rope.shape[1] != D // 2 or not rope.is_contiguous():
        raise ValueError("rope must be the contiguous float64 [max_pos, D/2, 2] table of rope_table()")
    if k_cache.shape != v_cache.shape or k_cache.stride() != v_cache.stride() or k_cache.dtype != xq.dtype:
        raise ValueError("k_cache / v_cache mismatch")
    q_out = torch.empty((B, S, num_heads, D), dtype=xq.dtype, device=xq.device)
    d = _l.PrologueDesc()
    d.dtype = _DT[xq.dtype]
    d.B, d.S, d.H, d.D = B, S, num_heads, D
    d.F, d.h, d.w = F, h, w
    d.start_frame = start_frame
    d.eps = eps
    d.tiling = _l.Tiling(f_tied, h_reduce, w_reduce, h, w)
    d.x_stride = (C.c_int64 * 2)(xq.stride(0), xq.stride(1))
    d.q_stride = _l.strides3(q_out)
    d.cache_stride = _l.strides3(k_cache)
    d.cache_tokens = k_cache.shape[1]
    d.start_idx = start_idx
    with torch.cuda.device(xq.device):
        _l.check(_l.load().sfm_qk_prologue(
            C.byref(d), xq.data_ptr(), xk.data_ptr(), xv.data_ptr(), wq.contiguous().data_ptr(),
            wk.contiguous().data_ptr(), rope.data_ptr(), rope.shape[0], q_out.data_ptr(), k_cache.data_ptr(),
            v_cache.data_ptr(), _stream(xq)))
    return q_out
