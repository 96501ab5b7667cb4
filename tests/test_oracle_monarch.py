"""Pins for the Monarch oracle: each check is a fact the mathematics fixes independently of
the oracle's own formula (special cases that reduce to dense attention, scalar-loop
reconstruction of the implied attention matrix, invariances)."""
import math

import numpy as np
import pytest
import torch

from oracle import blocks, dense, monarch


def _rand(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float64)


def _dense_blocks(Q, K, V, s):
    """Dense softmax attention over all keys, on block-shaped tensors."""
    B, a, b1, b2, H, D = Q.shape
    q = Q.reshape(B, -1, H, D)
    k = K.reshape(B, -1, H, D)
    v = V.reshape(B, -1, H, D)
    return dense.attention(q, k, v, s).reshape(Q.shape)


def test_b2_equal_one_is_dense():
    Q, K, V = _rand((2, 3, 5, 1, 2, 8), 1), _rand((2, 4, 5, 1, 2, 8), 2), _rand((2, 4, 5, 1, 2, 8), 3)
    out = monarch.monarch_1iter(Q, K, V, 0.3)
    assert torch.allclose(out, _dense_blocks(Q, K, V, 0.3), atol=1e-12)


def test_single_row_single_frame_is_dense():
    Q, K, V = _rand((1, 3, 1, 7, 2, 8), 4), _rand((1, 1, 1, 7, 2, 8), 5), _rand((1, 1, 1, 7, 2, 8), 6)
    out = monarch.monarch_1iter(Q, K, V, 0.25)
    assert torch.allclose(out, _dense_blocks(Q, K, V, 0.25), atol=1e-12)


def _scalar_loop_matrix(Q, K, s):
    """Implied attention matrix for one head built with scalar Python loops from the
    definition (softmax within a key block row, entropy-corrected softmax over block rows)."""
    a_n, b1, b2, D = Q.shape
    f_n = K.shape[0]
    q, k = Q.numpy(), K.numpy()
    A = np.zeros((a_n, b1, b2, f_n, b1, b2))
    for a in range(a_n):
        for j in range(b2):
            R = np.zeros((f_n, b1, b2))
            kbar = np.zeros((f_n, b1, D))
            negH = np.zeros((f_n, b1))
            for f in range(f_n):
                for kk in range(b1):
                    logits = np.array([s * np.dot(q[a, kk, j], k[f, kk, l]) for l in range(b2)])
                    p = np.exp(logits - logits.max())
                    p /= p.sum()
                    R[f, kk] = p
                    kbar[f, kk] = sum(p[l] * k[f, kk, l] for l in range(b2))
                    negH[f, kk] = sum(p[l] * math.log(p[l]) for l in range(b2))
            for i in range(b1):
                lg = np.array([[s * np.dot(q[a, i, j], kbar[f, kk]) - negH[f, kk] for kk in range(b1)]
                               for f in range(f_n)])
                w = np.exp(lg - lg.max())
                w /= w.sum()
                for f in range(f_n):
                    for kk in range(b1):
                        A[a, i, j, f, kk] = w[f, kk] * R[f, kk]
    return A.reshape(a_n * b1 * b2, f_n * b1 * b2)


def test_implied_matrix_scalar_loops():
    Q, K, V = _rand((1, 2, 3, 4, 1, 5), 7), _rand((1, 3, 3, 4, 1, 5), 8), _rand((1, 3, 3, 4, 1, 5), 9)
    s = 0.4
    A = _scalar_loop_matrix(Q[0, :, :, :, 0], K[0, :, :, :, 0], s)
    assert np.allclose(A.sum(1), 1.0, atol=1e-12)
    ref = torch.from_numpy(A) @ V[0, :, :, :, 0].reshape(-1, 5)
    out = monarch.monarch_1iter(Q, K, V, s)[0, :, :, :, 0].reshape(-1, 5)
    assert torch.allclose(out, ref, atol=1e-12)
    A2 = monarch.implied_attention_matrix(Q[0, :, :, :, 0], K[0, :, :, :, 0], s)
    assert torch.allclose(A2, torch.from_numpy(A), atol=1e-12)


def test_constant_v_gives_constant_output():
    Q, K = _rand((1, 2, 3, 4, 2, 6), 10), _rand((1, 3, 3, 4, 2, 6), 11)
    V = torch.ones((1, 3, 3, 4, 2, 6), dtype=torch.float64) * 2.5
    assert torch.allclose(monarch.monarch_1iter(Q, K, V, 0.5), torch.full(Q.shape, 2.5, dtype=torch.float64), atol=1e-12)


def test_kv_frame_permutation_invariance():
    Q, K, V = _rand((1, 2, 3, 4, 2, 6), 12), _rand((1, 4, 3, 4, 2, 6), 13), _rand((1, 4, 3, 4, 2, 6), 14)
    perm = torch.tensor([2, 0, 3, 1])
    a = monarch.monarch_1iter(Q, K, V, 0.5)
    b = monarch.monarch_1iter(Q, K[:, perm], V[:, perm], 0.5)
    assert torch.allclose(a, b, atol=1e-12)


def test_kv_chunks_merge_by_lse():
    Q, K, V = _rand((1, 2, 3, 4, 1, 6), 15), _rand((1, 5, 3, 4, 1, 6), 16), _rand((1, 5, 3, 4, 1, 6), 17)
    full = monarch.monarch_1iter(Q, K, V, 0.5)
    o1, p1 = monarch.monarch_1iter(Q, K[:, :2], V[:, :2], 0.5, return_parts=True)
    o2, p2 = monarch.monarch_1iter(Q, K[:, 2:], V[:, 2:], 0.5, return_parts=True)
    l1, l2 = p1[(0, 0)]["lse2"], p2[(0, 0)]["lse2"]
    w1 = torch.exp(l1 - torch.logaddexp(l1, l2)).unsqueeze(-1)
    merged = w1 * o1[0, :, :, :, 0] + (1 - w1) * o2[0, :, :, :, 0]
    assert torch.allclose(merged, full[0, :, :, :, 0], atol=1e-12)


def test_gibbs_equality_on_diagonal():
    """For i == k the step-2 logit s<q,Kbar> + H(R) equals logsumexp_l(s<q,k_l>); for i != k it is a lower bound."""
    Q, K, V = _rand((1, 1, 3, 5, 1, 6), 18), _rand((1, 2, 3, 5, 1, 6), 19), _rand((1, 2, 3, 5, 1, 6), 20)
    s = 0.7
    _, parts = monarch.monarch_1iter(Q, K, V, s, return_parts=True)
    p = parts[(0, 0)]
    q, k = Q[0, :, :, :, 0], K[0, :, :, :, 0]
    for i in range(3):
        for kk in range(3):
            for j in range(5):
                for f in range(2):
                    logit = s * torch.dot(q[0, i, j], p["Kbar"][0, f, kk, j]) - p["negH"][0, f, kk, j]
                    true = torch.logsumexp(s * (k[f, kk] @ q[0, i, j]), 0)
                    if i == kk:
                        assert abs(logit - true) < 1e-12
                    else:
                        # Gibbs: the bound uses R built from q[kk], so it can only under-estimate
                        assert logit <= true + 1e-12


def test_rounding_hook_changes_little():
    Q, K, V = _rand((1, 2, 4, 6, 1, 16), 21), _rand((1, 3, 4, 6, 1, 16), 22), _rand((1, 3, 4, 6, 1, 16), 23)
    a = monarch.monarch_1iter(Q, K, V, 0.25)
    b = monarch.monarch_1iter(Q, K, V, 0.25, round_to=torch.bfloat16)
    assert 0 < (a - b).abs().max() < 2e-2


@pytest.mark.parametrize("num_iters", [1, 2, 4])
def test_iter_b2_one_is_dense(num_iters):
    Q, K, V = _rand((1, 2, 4, 1, 2, 8), 24), _rand((1, 3, 4, 1, 2, 8), 25), _rand((1, 3, 4, 1, 2, 8), 26)
    out = monarch.monarch_iter(Q, K, V, 0.3, num_iters)
    assert torch.allclose(out, _dense_blocks(Q, K, V, 0.3), atol=1e-9)


def test_iter_one_matches_single_pass():
    Q, K, V = _rand((1, 2, 3, 4, 2, 8), 27), _rand((1, 3, 3, 4, 2, 8), 28), _rand((1, 3, 3, 4, 2, 8), 29)
    a = monarch.monarch_iter(Q, K, V, 0.3, 1)
    b = monarch.monarch_1iter(Q, K, V, 0.3)
    assert torch.allclose(a, b, atol=1e-5) and not torch.equal(a, b)


def test_iter_more_passes_move_towards_dense():
    """Not a pin of the iterates (those stay unpinned) -- a sanity property: refinement does not
    leave the simplex (constant V stays constant)."""
    Q, K = _rand((1, 2, 3, 4, 1, 8), 30), _rand((1, 3, 3, 4, 1, 8), 31)
    V = torch.full((1, 3, 3, 4, 1, 8), -1.25, dtype=torch.float64)
    out = monarch.monarch_iter(Q, K, V, 0.3, 3)
    assert torch.allclose(out, torch.full(Q.shape, -1.25, dtype=torch.float64), atol=1e-9)


# ------------------------------------------------------------------ block order

@pytest.mark.parametrize("f_tied,h_reduce,w_reduce", [(1, 1, 1), (1, 2, 1), (3, 1, 1), (3, 2, 2), (1, 3, 4), (3, 6, 1)])
def test_block_order_formula_and_round_trip(f_tied, h_reduce, w_reduce):
    h, w, F = 6, 8, 3
    S = F * h * w
    x = torch.arange(S, dtype=torch.float64).reshape(1, S, 1, 1).repeat(2, 1, 3, 2)
    xb = blocks.to_blocks(x, f_tied, h_reduce, w_reduce, h, w)
    na, b1, b2 = blocks.block_dims(S, f_tied, h_reduce, w_reduce, h, w)
    assert xb.shape == (2, na, b1, b2, 3, 2)
    hh, ww = h // h_reduce, w // w_reduce
    for a in range(na):
        for i in range(b1):
            for j in range(b2):
                tok = int(xb[0, a, i, j, 0, 0])
                frame, rem = divmod(tok, h * w)
                row, col = divmod(rem, w)
                assert (frame // f_tied, row // hh, col // ww) == (a // (h_reduce * w_reduce), (a // w_reduce) % h_reduce, a % w_reduce)
                assert (frame % f_tied) * hh + row % hh == i and col % ww == j
    assert torch.equal(blocks.from_blocks(xb, f_tied, h_reduce, w_reduce, h, w), x)


def test_block_order_identity_in_memory():
    x = _rand((1, 2 * 4 * 6, 2, 4), 40)
    assert torch.equal(blocks.to_blocks(x, 1, 1, 1, 4, 6).reshape(x.shape), x)
    assert torch.equal(blocks.to_blocks(x, 1, 2, 1, 4, 6).reshape(x.shape), x)


def test_block_dims_rejects_bad_sizes():
    with pytest.raises(ValueError):
        blocks.block_dims(100, 1, 1, 1, 4, 6)
    with pytest.raises(ValueError):
        blocks.block_dims(48, 1, 3, 1, 4, 6)


# ------------------------------------------------------------------ op compositions

def test_kv_cache_op_writes_cache_and_matches_blocks():
    h, w, H, D = 3, 4, 2, 8
    q = _rand((1, 2 * h * w, H, D), 50)
    kc, vc = _rand((1, 5 * h * w, H, D), 51), _rand((1, 5 * h * w, H, D), 52)
    nk, nv = _rand((1, 2 * h * w, H, D), 53), _rand((1, 2 * h * w, H, D), 54)
    kc0 = kc.clone()
    out = monarch.monarch_attn_with_kv_cache(q, kc, vc, nk, nv, 3 * h * w, 5 * h * w, 1, 1, 1, h, w)
    assert torch.equal(kc[:, 3 * h * w:], nk) and torch.equal(kc[:, :3 * h * w], kc0[:, :3 * h * w])
    ref = monarch.monarch_1iter(q.reshape(1, 2, h, w, H, D), kc.reshape(1, 5, h, w, H, D),
                                vc.reshape(1, 5, h, w, H, D), D ** -0.5).reshape(q.shape)
    assert torch.allclose(out, ref, atol=1e-12)


def test_kv_cache_op_block_order_in_cache():
    """With w_reduce > 1 the cache holds tokens in block order, not token order."""
    h, w, H, D = 2, 4, 1, 4
    q = _rand((1, h * w, H, D), 55)
    kc, vc = torch.zeros((1, h * w, H, D), dtype=torch.float64), torch.zeros((1, h * w, H, D), dtype=torch.float64)
    nk, nv = _rand((1, h * w, H, D), 56), _rand((1, h * w, H, D), 57)
    monarch.monarch_attn_with_kv_cache(q, kc, vc, nk, nv, 0, h * w, 1, 1, 2, h, w)
    assert torch.equal(kc, blocks.to_blocks(nk, 1, 1, 2, h, w).reshape(kc.shape))
    assert not torch.equal(kc, nk)


def test_masked_causal_equals_chunked():
    h, w, H, D, F = 2, 3, 2, 8, 4
    q, k, v = _rand((1, F * h * w, H, D), 60), _rand((1, F * h * w, H, D), 61), _rand((1, F * h * w, H, D), 62)
    for bcs in (h * w, 2 * h * w):
        a = monarch.monarch_attn(q, k, v, 1, 1, 1, h, w, block_causal_size=bcs)
        b = monarch.monarch_attn_causal_chunked(q, k, v, 1, 1, 1, h, w, bcs)
        assert torch.allclose(a, b, atol=1e-12)


def test_c1_plumbing_case_against_brute_force():
    """B=1,H=2,D=64, 3 frames of 8x8 tokens, q,k,v drawn in this order from generator seed 0 (fp32)."""
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 192, 2, 64, generator=g)
    k = torch.randn(1, 192, 2, 64, generator=g)
    v = torch.randn(1, 192, 2, 64, generator=g)
    out = monarch.monarch_attn(q, k, v, 1, 1, 1, 8, 8, sm_scale=0.125)
    for hd in range(2):
        A = monarch.implied_attention_matrix(q[0, :, hd].reshape(3, 8, 8, 64), k[0, :, hd].reshape(3, 8, 8, 64), 0.125)
        assert torch.allclose(A.sum(1), torch.ones(192, dtype=torch.float64), atol=1e-12)
        assert (out[0, :, hd] - A @ v[0, :, hd].double()).abs().max() < 1e-5
    assert monarch.monarch_flops(1, 2, 64, 3, 3, 8, 8) == 5898240
