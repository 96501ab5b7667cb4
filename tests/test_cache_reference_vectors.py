"""The product's `CausalWanSelfAttention` (cache state machine, eviction with sink frames, RoPE start frame, dispatch
between Monarch, dense first chunk, dense fallback and refinement passes, block-order cache rows) against what the
reference's own `CausalWanSelfAttention.forward` did, call by call, on the same scripted sequences
(tests/golden/cache_reference_vectors.npz, written by tests/golden/make_cache_reference_vectors.py; scenarios and seeds in
tests/golden/block_fixture.py).  CPU, float64, oracle operators."""
import os
import sys

import numpy as np
import pytest
import torch

import self_forcing_amd as sfa
from oracle.ops import OracleOps

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import block_fixture as fx  # noqa: E402

cm = sfa.causal_model
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cache_reference_vectors.npz"))


def _module(local, sink, cache_frames, flags):
    total = cache_frames * fx.A_FRAME if local == -1 else 7 * fx.A_FRAME
    m = cm.CausalWanSelfAttention(fx.A_DIM, fx.A_HEADS, local, sink, True, fx.EPS, 0, (fx.A_H, fx.A_W), total,
                                  cm.AttentionFlags(0, **flags), OracleOps(compute_dtype=torch.float64)).double().eval()
    with torch.no_grad():
        for k, p in m.named_parameters():
            p.copy_(fx.attn_parameter(k, tuple(p.shape)))
    return m


@pytest.mark.parametrize("ring", [False, True])
@pytest.mark.parametrize("scen", sorted(fx.A_SCENARIOS))
def test_cache_sequence_matches_the_reference_forward(scen, ring):
    """ring = False keeps the reference's row order in a windowed cache (shift-down eviction, causal_model.py:912-926):
    outputs, both counters and every cache row are compared.  ring = True (the default) overwrites the oldest chunk
    instead: the same rows sit elsewhere in the cache, so the outputs and the global counter are compared."""
    local, sink, cache_frames, flags, calls = fx.A_SCENARIOS[scen]
    m = _module(local, sink, cache_frames, dict(flags, ring_cache=ring))
    d = fx.A_DIM // fx.A_HEADS
    kv = {"k": torch.zeros(1, cache_frames * fx.A_FRAME, fx.A_HEADS, d, dtype=torch.float64),
          "v": torch.zeros(1, cache_frames * fx.A_FRAME, fx.A_HEADS, d, dtype=torch.float64),
          "global_end_index": torch.tensor([0], dtype=torch.long), "local_end_index": torch.tensor([0], dtype=torch.long)}
    wts = torch.arange(1, fx.A_HEADS * d + 1, dtype=torch.float64).view(1, 1, fx.A_HEADS, d)
    ringed = 0
    for i, (start_frame, frames) in enumerate(calls):
        with torch.no_grad():
            y = m(fx.attn_input(scen, i), (frames, fx.A_H, fx.A_W), kv, start_frame * fx.A_FRAME)
        # the reference's pure-torch Monarch formulas take their softmaxes in float32 (the dense paths do not)
        np.testing.assert_allclose(y.numpy(), GOLD[f"{scen}.{i}.out"], atol=1e-9 if flags.get("disable_monarch") else 5e-6, rtol=0,
                                   err_msg=f"output of call {i}")
        ends = (int(kv["global_end_index"].item()), int(kv["local_end_index"].item()))
        if kv.get("_ring"):
            assert ends[0] == int(GOLD[f"{scen}.{i}.ends"][0]), (i, ends)
            for key in ("k", "v"):          # the same set of rows as the reference's cache holds, in another order
                mine = np.sort((kv[key] * wts).sum(dim=(2, 3)).numpy().ravel())
                np.testing.assert_allclose(mine, np.sort(GOLD[f"{scen}.{i}.{key}_rows"].ravel()), atol=1e-9, rtol=0)
            ringed += 1
            continue
        assert ends == tuple(int(v) for v in GOLD[f"{scen}.{i}.ends"]), (i, ends)
        np.testing.assert_allclose((kv["k"] * wts).sum(dim=(2, 3)).numpy(), GOLD[f"{scen}.{i}.k_rows"], atol=1e-9, rtol=0,
                                   err_msg=f"K cache rows after call {i}")
        np.testing.assert_allclose((kv["v"] * wts).sum(dim=(2, 3)).numpy(), GOLD[f"{scen}.{i}.v_rows"], atol=1e-9, rtol=0,
                                   err_msg=f"V cache rows after call {i}")
    assert (ringed > 0) == (ring and local != -1)
    # window_sink ends with a two-frame chunk that would straddle its three-frame ring: the cache is rotated back into the
    # reference's order then, and from there on (and at the end) everything is compared again; dense_window stays a ring
    assert bool(kv.get("_ring")) == (ring and scen == "dense_window")
    if kv.get("_ring"):
        return
    np.testing.assert_allclose(kv["k"].numpy(), GOLD[f"{scen}.k"], atol=1e-10, rtol=0)
    np.testing.assert_allclose(kv["v"].numpy(), GOLD[f"{scen}.v"], atol=1e-10, rtol=0)


def test_a_wrong_sink_size_would_show():
    """Sensitivity of the pin: the windowed scenario with the sink frame ignored ends with different cache rows."""
    local, sink, cache_frames, flags, calls = fx.A_SCENARIOS["window_sink"]
    m = _module(local, 0, cache_frames, dict(flags, ring_cache=False))
    d = fx.A_DIM // fx.A_HEADS
    kv = {"k": torch.zeros(1, cache_frames * fx.A_FRAME, fx.A_HEADS, d, dtype=torch.float64),
          "v": torch.zeros(1, cache_frames * fx.A_FRAME, fx.A_HEADS, d, dtype=torch.float64),
          "global_end_index": torch.tensor([0], dtype=torch.long), "local_end_index": torch.tensor([0], dtype=torch.long)}
    for i, (start_frame, frames) in enumerate(calls):
        with torch.no_grad():
            m(fx.attn_input("window_sink", i), (frames, fx.A_H, fx.A_W), kv, start_frame * fx.A_FRAME)
    assert np.abs(kv["k"].numpy() - GOLD["window_sink.k"]).max() > 1e-2


def test_cross_attention_with_its_cache_matches_the_reference_forward():
    """model.py:733-768: the first call computes and keeps the text K/V, later calls read them whatever context they get."""
    m = cm.WanT2VCrossAttention(fx.A_DIM, fx.A_HEADS, fx.EPS, OracleOps(compute_dtype=torch.float64)).double().eval()
    with torch.no_grad():
        for k, p in m.named_parameters():
            p.copy_(fx.attn_parameter("cross." + k, tuple(p.shape)))
    cache = {"is_init": False, "k": None, "v": None}
    xs = [fx.randn(71, 1, 30, fx.A_DIM), fx.randn(72, 1, 18, fx.A_DIM)]
    ctx = [fx.randn(73, 1, 9, fx.A_DIM), fx.randn(74, 1, 9, fx.A_DIM)]
    with torch.no_grad():
        for i in range(2):
            np.testing.assert_allclose(m(xs[i], ctx[i], cache).numpy(), GOLD[f"cross.{i}.out"], atol=1e-9, rtol=0)
        np.testing.assert_allclose(m(xs[1], ctx[1], None).numpy(), GOLD["cross.nocache"], atol=1e-9, rtol=0)
    assert cache["is_init"]
    np.testing.assert_allclose(cache["k"].numpy(), GOLD["cross.k"], atol=1e-10, rtol=0)
