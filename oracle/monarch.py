"""Oracle (test infrastructure): Monarch-factored attention on the CPU.

Restates, in own code, the torch formulas of the reference:
  * one factor iteration          wan/modules/monarch_attn.py:1801-1830  (`monarch_attn_ref_op`)
  * several factor iterations     wan/modules/monarch_attn.py:1705-1751  (`monarch_attn_slow`)
  * op with KV cache              wan/modules/monarch_attn.py:1778-1796, 1860-1878
  * op without cache / causal     wan/modules/monarch_attn.py:1753-1776, 1832-1858
  * kernel-level quantities       wan/modules/monarch_attn.py:210-250 (step 1), 800-838 (step 2)

Notation (per batch element and head; s = sm_scale):
    Q[a, i, j, :]   queries of block-frame a, block row i, block col j
    K[f, k, l, :]   keys    of block-frame f, block row k, block col l   (V alike)

    S1[a,f,k,j,l] = s <Q[a,k,j], K[f,k,l]>          R = softmax_l S1      (right factor)
    Kbar[a,f,k,j] = sum_l R K[f,k,l]                 Y = sum_l R V[f,k,l]
    negH[a,f,k,j] = sum_l R log R
    S2[a,i,j,(f,k)] = s <Q[a,i,j], Kbar[a,f,k,j]> - negH[a,f,k,j]
    L = softmax_(f,k) S2                                                   (left factor)
    O[a,i,j] = sum_(f,k) L Y[a,f,k,j]

All arithmetic is done in `dtype` (float64 by default) from the inputs as
given; `round_to` optionally rounds the quantities the device kernels keep in
16-bit storage (P before the contractions, Kbar, Y) so that a test can tell
kernel rounding from kernel error.
"""
import math

import torch

from . import blocks


def _rnd(x, round_to):
    return x if round_to is None else x.to(round_to).to(x.dtype)


def _allowed(a_idx, f_idx, causal_block):
    """Block-causal visibility of KV block-frame f for query block-frame a
    (monarch_attn.py:139-141, 804-807): hidden when a // cbs < f // cbs."""
    if not causal_block:
        return True
    return (a_idx // causal_block) >= (f_idx // causal_block)


def step1_head(Q, K, V, s, round_to=None):
    """Right factor for one (batch, head).  Q [a,b1,b2,D]; K,V [f,b1,b2,D] (already in compute dtype).
    -> Kbar, Y [a,f,b1(k),b2(j),D], negH [a,f,k,j], lse1 [a,f,k,j]."""
    S1 = s * torch.einsum("akjd,fkld->afkjl", Q, K)
    lse1 = torch.logsumexp(S1, dim=-1)
    R = torch.exp(S1 - lse1.unsqueeze(-1))
    negH = (R * (S1 - lse1.unsqueeze(-1))).sum(-1)
    Rr = _rnd(R, round_to)
    Kbar = _rnd(torch.einsum("afkjl,fkld->afkjd", Rr, K), round_to)
    Y = _rnd(torch.einsum("afkjl,fkld->afkjd", Rr, V), round_to)
    return Kbar, Y, negH, lse1


def step2_head(Q, Kbar, Y, negH, s, causal_block=0, round_to=None):
    """Left factor and output for one (batch, head).  -> O [a,b1,b2,D], lse2 [a,i,j]."""
    na, nf = Kbar.shape[0], Kbar.shape[1]
    S2 = s * torch.einsum("aijd,afkjd->aijfk", Q, Kbar) - negH.permute(0, 3, 1, 2).unsqueeze(1)
    if causal_block:
        for a_idx in range(na):
            for f_idx in range(nf):
                if not _allowed(a_idx, f_idx, causal_block):
                    S2[a_idx, :, :, f_idx, :] = -math.inf
    flat = S2.flatten(3)
    lse2 = torch.logsumexp(flat, dim=-1)
    L = torch.exp(flat - lse2.unsqueeze(-1)).reshape(S2.shape)
    O = torch.einsum("aijfk,afkjd->aijd", _rnd(L, round_to), Y)
    return O, lse2


def monarch_1iter(Q, K, V, sm_scale, causal_block=0, dtype=torch.float64, round_to=None,
                  return_parts=False):
    """One-iteration Monarch attention (monarch_attn.py:1801-1830).

    Q [B,a,b1,b2,H,D]; K,V [B,f,b1,b2,H,D]  ->  [B,a,b1,b2,H,D] in `dtype`."""
    B, na, b1, b2, H, D = Q.shape
    out = torch.empty((B, na, b1, b2, H, D), dtype=dtype)
    parts = {}
    for b in range(B):
        for h in range(H):
            q = Q[b, :, :, :, h].to(dtype)
            k = K[b, :, :, :, h].to(dtype)
            v = V[b, :, :, :, h].to(dtype)
            Kbar, Y, negH, lse1 = step1_head(q, k, v, sm_scale, round_to)
            o, lse2 = step2_head(q, Kbar, Y, negH, sm_scale, causal_block, round_to)
            out[b, :, :, :, h] = o
            if return_parts:
                parts[(b, h)] = dict(Kbar=Kbar, Y=Y, negH=negH, lse1=lse1, lse2=lse2)
    return (out, parts) if return_parts else out


def implied_attention_matrix(Q, K, sm_scale, dtype=torch.float64):
    """Dense [a*b1*b2, f*b1*b2] matrix whose rows are the attention weights Monarch
    implies for one (batch, head): A[(a,i,j),(f,k,l)] = L[a,i,j,(f,k)] * R[a,f,k,j,l].
    Q [a,b1,b2,D], K [f,b1,b2,D].  Used by tests on tiny inputs only."""
    q, k = Q.to(dtype), K.to(dtype)
    na, b1, b2, _ = q.shape
    nf = k.shape[0]
    S1 = sm_scale * torch.einsum("akjd,fkld->afkjl", q, k)
    R = torch.softmax(S1, -1)
    negH = (R * torch.log_softmax(S1, -1)).sum(-1)
    Kbar = torch.einsum("afkjl,fkld->afkjd", R, k)
    S2 = sm_scale * torch.einsum("aijd,afkjd->aijfk", q, Kbar) - negH.permute(0, 3, 1, 2).unsqueeze(1)
    L = torch.softmax(S2.flatten(3), -1).reshape(S2.shape)
    A = torch.einsum("aijfk,afkjl->aijfkl", L, R)
    return A.reshape(na * b1 * b2, nf * b1 * b2)


def monarch_iter(Q, K, V, sm_scale, num_iters=1, dtype=torch.float64):
    """Alternating refinement with `num_iters` passes (monarch_attn.py:1705-1751).

    Each pass recomputes the right factor from per-block query representatives
        rep[a,f,k,j] = sum_i L[a,i,j,(f,k)] Q[a,i,j]  with weight  w = sum_i L
    (first pass: rep = Q[a,k,j], w = 1) using logits <rep, K> * min(1/(w+1e-6), 1e4),
    then the left factor as in `monarch_1iter`.  Pinned by golden vectors of the
    reference function for num_iters in {1, 2, 3, 8} (tests/test_oracle_golden.py)."""
    B, na, b1, b2, H, D = Q.shape
    nf = K.shape[1]
    out = torch.empty((B, na, b1, b2, H, D), dtype=dtype)
    rs = math.sqrt(sm_scale)
    for b in range(B):
        for h in range(H):
            q = Q[b, :, :, :, h].to(dtype) * rs
            k = K[b, :, :, :, h].to(dtype) * rs
            v = V[b, :, :, :, h].to(dtype)
            rep = q.unsqueeze(1).expand(na, nf, b1, b2, D)          # [a,f,k,j,D]
            w = torch.ones((na, nf, b1, b2), dtype=dtype)
            for it in range(num_iters):
                z = torch.einsum("afkjd,fkld->afkjl", rep, k)
                z = z * torch.clamp(1.0 / (w + 1e-6), max=1e4).unsqueeze(-1)
                logR = torch.log_softmax(z, -1)
                R = torch.exp(logR)
                Kbar = torch.einsum("afkjl,fkld->afkjd", R, k)
                negH = (R * logR).sum(-1)                            # [a,f,k,j]
                S2 = torch.einsum("aijd,afkjd->aijfk", q, Kbar) - negH.permute(0, 3, 1, 2).unsqueeze(1)
                L = torch.softmax(S2.flatten(3), -1).reshape(S2.shape)   # [a,i,j,f,k]
                if it + 1 < num_iters:
                    rep = torch.einsum("aijfk,aijd->afkjd", L, q)
                    w = L.sum(1).permute(0, 2, 3, 1)                 # [a,f,k,j]
            Y = torch.einsum("afkjl,fkld->afkjd", R, v)
            out[b, :, :, :, h] = torch.einsum("aijfk,afkjd->aijd", L, Y)
    return out


# --------------------------------------------------------------------------- public-op compositions

def monarch_attn(q, k, v, f_tied, h_reduce, w_reduce, h, w, sm_scale=None, block_causal_size=None,
                 num_iters=1, dtype=torch.float64, round_to=None):
    """No-cache op on token-ordered [B,S,H,D] tensors (monarch_attn.py:1753-1776)."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    qb = blocks.to_blocks(q, f_tied, h_reduce, w_reduce, h, w)
    kb = blocks.to_blocks(k, f_tied, h_reduce, w_reduce, h, w)
    vb = blocks.to_blocks(v, f_tied, h_reduce, w_reduce, h, w)
    cbs = 0
    if block_causal_size is not None:
        per_block = qb.shape[2] * qb.shape[3]
        if q.shape[1] % block_causal_size or k.shape[1] != q.shape[1] or block_causal_size % per_block:
            raise ValueError("block_causal_size must divide S, align with the Monarch block and S_kv == S_q")
        if num_iters != 1:
            raise ValueError("causal masking is defined for num_iters == 1 only")
        cbs = block_causal_size // per_block
    if num_iters == 1:
        ob = monarch_1iter(qb, kb, vb, sm_scale, cbs, dtype, round_to)
    else:
        ob = monarch_iter(qb, kb, vb, sm_scale, num_iters, dtype)
    return blocks.from_blocks(ob, f_tied, h_reduce, w_reduce, h, w)


def monarch_attn_with_kv_cache(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, f_tied, h_reduce,
                               w_reduce, h, w, sm_scale=None, num_iters=1, dtype=torch.float64,
                               round_to=None):
    """Cache write + Monarch over the whole cache view (monarch_attn.py:1778-1796, 1860-1878).

    new_k/new_v are written, in Monarch block order, to k_cache/v_cache[:, start_idx:end_idx]
    IN PLACE; the cache view [B,Skv,H,D] is then read as [B,f,b1,b2,H,D]."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    B, _, H, D = q.shape
    qb = blocks.to_blocks(q, f_tied, h_reduce, w_reduce, h, w)
    _, _, b1, b2, _, _ = qb.shape
    k_cache[:, start_idx:end_idx] = blocks.to_blocks(new_k, f_tied, h_reduce, w_reduce, h, w).reshape(B, -1, H, D)
    v_cache[:, start_idx:end_idx] = blocks.to_blocks(new_v, f_tied, h_reduce, w_reduce, h, w).reshape(B, -1, H, D)
    kb = k_cache.reshape(B, -1, b1, b2, H, D)
    vb = v_cache.reshape(B, -1, b1, b2, H, D)
    if num_iters == 1:
        ob = monarch_1iter(qb, kb, vb, sm_scale, 0, dtype, round_to)
    else:
        ob = monarch_iter(qb, kb, vb, sm_scale, num_iters, dtype)
    return blocks.from_blocks(ob, f_tied, h_reduce, w_reduce, h, w)


def monarch_attn_causal_chunked(q, k, v, f_tied, h_reduce, w_reduce, h, w, block_causal_size, sm_scale=None,
                                dtype=torch.float64):
    """Block-causal Monarch evaluated chunk by chunk over growing KV prefixes
    (monarch_attn.py:1832-1858) -- the independent statement the masked op must equal."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    qb = blocks.to_blocks(q, f_tied, h_reduce, w_reduce, h, w)
    kb = blocks.to_blocks(k, f_tied, h_reduce, w_reduce, h, w)
    vb = blocks.to_blocks(v, f_tied, h_reduce, w_reduce, h, w)
    cbs = block_causal_size // (qb.shape[2] * qb.shape[3])
    outs = []
    for a0 in range(0, qb.shape[1], cbs):
        outs.append(monarch_1iter(qb[:, a0:a0 + cbs], kb[:, :a0 + cbs], vb[:, :a0 + cbs], sm_scale, 0, dtype))
    return blocks.from_blocks(torch.cat(outs, 1), f_tied, h_reduce, w_reduce, h, w)


def monarch_flops(B, H, D, a, f, b1, b2):
    """Algorithmic forward FLOPs: step 1 (6 a f b1 b2^2 D) + step 2 (4 a b2 f b1^2 D) per head."""
    return B * H * (6 * a * f * b1 * b2 * b2 * D + 4 * a * b2 * f * b1 * b1 * D)
