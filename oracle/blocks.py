"""Oracle (test infrastructure): token order <-> Monarch block order.

Follows wan/modules/monarch_attn.py:1696-1703 (`_get_rearrange_fns`).

Tokens arrive in (frame, row, col) order, S = F*h*w.  With tiling
(f_tied, h_reduce, w_reduce):

    frame = A*f_tied + ft          row = c*(h/h_reduce) + ii       col = e*(w/w_reduce) + j
    block-frame  a  = (A*h_reduce + c)*w_reduce + e
    block row    i  = ft*(h/h_reduce) + ii          (b1 = f_tied*h/h_reduce)
    block col    j                                   (b2 = w/w_reduce)

The permutation is written here as an explicit index table (numpy), not with
einops, so that it is an independent statement of the same mapping.
"""
import numpy as np
import torch


def block_dims(n_tokens, f_tied, h_reduce, w_reduce, h, w):
    """-> (n_block_frames, b1, b2).  Raises ValueError on sizes the tiling does not divide."""
    if h % h_reduce or w % w_reduce:
        raise ValueError("h_reduce / w_reduce must divide the frame grid")
    group = f_tied * h * w
    if n_tokens % group:
        raise ValueError(f"{n_tokens} tokens is not a multiple of f_tied*h*w = {group}")
    return (n_tokens // group) * h_reduce * w_reduce, f_tied * (h // h_reduce), w // w_reduce


def block_to_token_index(n_tokens, f_tied, h_reduce, w_reduce, h, w):
    """int64 array idx[a, i, j] = natural token index of block coordinate (a, i, j)."""
    na, b1, b2 = block_dims(n_tokens, f_tied, h_reduce, w_reduce, h, w)
    hh, ww = h // h_reduce, w // w_reduce
    idx = np.empty((na, b1, b2), dtype=np.int64)
    for a in range(na):
        e = a % w_reduce
        c = (a // w_reduce) % h_reduce
        A = a // (w_reduce * h_reduce)
        for i in range(b1):
            ft, ii = divmod(i, hh)
            frame = A * f_tied + ft
            row = c * hh + ii
            base = (frame * h + row) * w + e * ww
            idx[a, i, :] = base + np.arange(b2)
    return idx


def to_blocks(x, f_tied, h_reduce, w_reduce, h, w):
    """x [B, S, H, D] in token order -> [B, a, b1, b2, H, D] in Monarch block order."""
    idx = block_to_token_index(x.shape[1], f_tied, h_reduce, w_reduce, h, w)
    na, b1, b2 = idx.shape
    flat = torch.from_numpy(idx.reshape(-1))
    return x.index_select(1, flat).reshape(x.shape[0], na, b1, b2, x.shape[2], x.shape[3])


def from_blocks(xb, f_tied, h_reduce, w_reduce, h, w):
    """Inverse of to_blocks: [B, a, b1, b2, H, D] -> [B, S, H, D] in token order."""
    B, na, b1, b2, H, D = xb.shape
    n = na * b1 * b2
    idx = block_to_token_index(n, f_tied, h_reduce, w_reduce, h, w).reshape(-1)
    out = torch.empty((B, n, H, D), dtype=xb.dtype)
    out[:, torch.from_numpy(idx)] = xb.reshape(B, n, H, D)
    return out
