"""The oracle against golden vectors produced by the reference's own pure-torch formulas
(tests/golden/make_reference_vectors.py wrote them in the authoring container; inputs are regenerated
from the stored seeds).

Tolerance 2e-6: the reference formulas evaluate their softmaxes in float32 whatever the input dtype
(`bR.to(torch.float32)`, monarch_attn.py:1715, 1815), the oracle in float64; a wrong index, sign or
transposed operand shows up at 1e-1."""
import os

import numpy as np
import pytest
import torch

from oracle import blocks, monarch

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "monarch_reference_vectors.npz"))


def _inputs(ci):
    seed, B, a, f, b1, b2, H, D = (int(x) for x in GOLD[f"case{ci}_meta"])
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, a, b1, b2, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, f, b1, b2, H, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, f, b1, b2, H, D, generator=g, dtype=torch.float64)
    return q, k, v, float(GOLD[f"case{ci}_scale"])


@pytest.mark.parametrize("ci", [0, 1, 2])
def test_one_iteration_matches_reference_formula(ci):
    q, k, v, s = _inputs(ci)
    out = monarch.monarch_1iter(q, k, v, s)
    assert np.abs(out.numpy() - GOLD[f"case{ci}_ref_op"]).max() < 2e-6


@pytest.mark.parametrize("ci", [0, 1, 2])
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_iterated_refinement_matches_reference_formula(ci, n):
    q, k, v, s = _inputs(ci)
    out = monarch.monarch_iter(q, k, v, s, n)
    assert np.abs(out.numpy() - GOLD[f"case{ci}_slow{n}"]).max() < 2e-6


@pytest.mark.parametrize("tiling", [(1, 1, 1), (1, 2, 1), (3, 1, 1), (3, 2, 2), (1, 3, 4)])
def test_block_order_matches_reference_permutation(tiling):
    idx = blocks.block_to_token_index(3 * 6 * 8, *tiling, 6, 8)
    assert np.array_equal(idx, GOLD["order_%d_%d_%d" % tiling])


@pytest.mark.parametrize("ci", [0, 1, 2])
def test_gradients_match_autograd_of_the_reference_formula(ci):
    """dq, dk, dv of the one-iteration formula for a seeded cotangent: autograd through the oracle against autograd
    through the reference's `monarch_attn_ref_op` (float32 softmaxes there: 1e-5)."""
    q, k, v, s = _inputs(ci)
    seed = int(GOLD[f"case{ci}_meta"][0])
    cot = torch.randn(q.shape, generator=torch.Generator().manual_seed(seed + 1000), dtype=torch.float64)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    monarch.monarch_1iter(qa, ka, va, s).backward(cot)
    for name, t in (("dq", qa), ("dk", ka), ("dv", va)):
        ref = GOLD[f"case{ci}_{name}"]
        assert np.abs(t.grad.numpy() - ref).max() < 1e-5 * max(1.0, np.abs(ref).max()), name


@pytest.mark.parametrize("ci", [0, 1, 2])
@pytest.mark.parametrize("n", [2, 3])
def test_refinement_gradients_match_autograd_of_the_reference_formula(ci, n):
    """dq, dk, dv of the iterated refinement (the reference's `monarch_attn_slow` is plain differentiable torch): autograd
    through the oracle against autograd through the reference function, same cotangent as above."""
    q, k, v, s = _inputs(ci)
    seed = int(GOLD[f"case{ci}_meta"][0])
    cot = torch.randn(q.shape, generator=torch.Generator().manual_seed(seed + 1000), dtype=torch.float64)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    monarch.monarch_iter(qa, ka, va, s, n).backward(cot)
    for name, t in (("dq", qa), ("dk", ka), ("dv", va)):
        ref = GOLD[f"case{ci}_slow{n}_{name}"]
        assert np.abs(t.grad.numpy() - ref).max() < 1e-5 * max(1.0, np.abs(ref).max()), name
