"""Oracle (test infrastructure): q/k prologue = RMSNorm over the model dim + 3-D RoPE.

Follows
  * wan/modules/model.py:462-478          WanRMSNorm: x * rsqrt(mean(x^2) + eps) over the FULL model
                                          dim in fp32, cast back to x's dtype, times weight
  * wan/modules/model.py:421-428          rope_params: angle(pos, m) = pos * theta^(-2m/dim_axis)
  * wan/modules/causal_model.py:1350-1357 table = cat[axis0: d - 4(d//6), axis1: 2(d//6), axis2: 2(d//6)]
  * wan/modules/causal_model.py:687-715   causal_rope_apply: interleaved pairs (x[2m], x[2m+1]) rotated in
                                          float64 by the angle of (frame+start_frame | row | col), result
                                          cast back to x's dtype
  * wan/modules/causal_model.py:801-807, 899-905  order: Linear -> RMSNorm -> view heads -> RoPE

Pinned by the reference's own outputs (tests/golden/block_reference_vectors.npz: causal_rope_apply on three grids in
float64 and bfloat16, the complex table, WanRMSNorm in float32 and bfloat16) in tests/test_block_reference_vectors.py, and by
the closed forms and invariants of tests/test_oracle_dense_prologue.py.
"""
import math

import numpy as np
import torch


def rms_norm(x, weight, eps=1e-6):
    """x [..., C] (any float dtype), weight [C] -> same dtype as x*weight would have in torch."""
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return y.to(x.dtype) * weight


def rope_axis_pairs(head_dim):
    """Number of complex pairs given to (frame, row, col): [c - 2(c//3), c//3, c//3] with c = head_dim/2."""
    c = head_dim // 2
    return [c - 2 * (c // 3), c // 3, c // 3]


def rope_angles(max_pos, head_dim, theta=10000.0):
    """float64 array ang[pos, m] for the m-th pair of a head; every axis uses the SAME pos row
    index but its own frequency ladder theta^(-2m'/dim_axis), dim_axis = 2*pairs(axis)...
    except that the reference builds the three ladders with dims (d - 4(d//6), 2(d//6), 2(d//6))."""
    d = head_dim
    dims = [d - 4 * (d // 6), 2 * (d // 6), 2 * (d // 6)]
    cols = []
    pos = np.arange(max_pos, dtype=np.float64)[:, None]
    for dim_axis in dims:
        m = np.arange(0, dim_axis, 2, dtype=np.float64)
        inv = 1.0 / np.power(theta, m / dim_axis)
        cols.append(pos * inv[None, :])
    return np.concatenate(cols, axis=1)          # [max_pos, d/2]


def rope_apply(x, grid, start_frame=0, theta=10000.0, max_pos=1024):
    """x [B, S, H, D] with S = F*h*w tokens in (frame,row,col) order; grid = (F, h, w).
    Rotates in float64 and rounds back to x.dtype once."""
    F, h, w = grid
    B, S, H, D = x.shape
    assert S == F * h * w
    ang = rope_angles(max_pos, D, theta)
    n0, n1, n2 = rope_axis_pairs(D)
    fr = np.repeat(np.arange(F), h * w) + start_frame
    ro = np.tile(np.repeat(np.arange(h), w), F)
    co = np.tile(np.arange(w), F * h)
    tok_ang = np.concatenate([ang[fr, :n0], ang[ro, n0:n0 + n1], ang[co, n0 + n1:]], axis=1)   # [S, D/2]
    c = torch.from_numpy(np.cos(tok_ang))[None, :, None, :]
    s = torch.from_numpy(np.sin(tok_ang))[None, :, None, :]
    xd = x.to(torch.float64).reshape(B, S, H, D // 2, 2)
    re = xd[..., 0] * c - xd[..., 1] * s
    im = xd[..., 0] * s + xd[..., 1] * c
    return torch.stack([re, im], dim=-1).reshape(B, S, H, D).to(x.dtype)


def qk_prologue(xq, xk, xv, wq, wk, num_heads, grid, start_frame, eps=1e-6):
    """[B,S,C] projections -> roped q, roped k, v as [B,S,H,D] (token order)."""
    B, S, C = xq.shape
    D = C // num_heads
    q = rope_apply(rms_norm(xq, wq, eps).view(B, S, num_heads, D), grid, start_frame)
    k = rope_apply(rms_norm(xk, wk, eps).view(B, S, num_heads, D), grid, start_frame)
    return q, k, xv.view(B, S, num_heads, D)
