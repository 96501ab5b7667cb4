"""Pins for the dense-attention, RMSNorm, RoPE, KV-cache-state and schedule oracles."""
import math

import numpy as np
import pytest
import torch

from oracle import cache, dense, prologue, sched


def _rand(shape, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float64).to(dtype)


# ------------------------------------------------------------------ dense attention

@pytest.mark.parametrize("B,Lq,Lk,H,D", [(1, 17, 13, 1, 32), (2, 31, 29, 3, 64), (2, 64, 48, 4, 64)])
def test_dense_matches_library_sdpa(B, Lq, Lk, H, D):
    q, k, v = _rand((B, Lq, H, D), 1), _rand((B, Lk, H, D), 2), _rand((B, Lk, H, D), 3)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
    assert torch.allclose(dense.attention(q, k, v), ref.transpose(1, 2), atol=1e-12)


def test_dense_scalar_loops_and_lse():
    q, k, v = _rand((1, 3, 1, 4), 4), _rand((1, 5, 1, 4), 5), _rand((1, 5, 1, 4), 6)
    out, lse = dense.attention(q, k, v, sm_scale=0.3, return_lse=True)
    for i in range(3):
        w = [math.exp(0.3 * float(torch.dot(q[0, i, 0], k[0, j, 0]))) for j in range(5)]
        z = sum(w)
        ref = sum(w[j] / z * v[0, j, 0] for j in range(5))
        assert torch.allclose(out[0, i, 0], ref, atol=1e-12)
        assert abs(float(lse[0, 0, i]) - math.log(z)) < 1e-12


def test_dense_with_cache_writes_then_attends():
    q = _rand((2, 7, 2, 8), 7)
    kc, vc = _rand((2, 12, 2, 8), 8), _rand((2, 12, 2, 8), 9)
    nk, nv = _rand((2, 5, 2, 8), 10), _rand((2, 5, 2, 8), 11)
    k2, v2 = kc.clone(), vc.clone()
    k2[:, 7:12], v2[:, 7:12] = nk, nv
    out = dense.full_attention_with_kv_cache(q, kc, vc, nk, nv, 7, 12)
    assert torch.equal(kc, k2) and torch.equal(vc, v2)
    assert torch.allclose(out, dense.attention(q, k2, v2), atol=1e-12)
    with pytest.raises(ValueError):
        dense.full_attention_with_kv_cache(q, kc, vc, nk, nv, 9, 14)


# ------------------------------------------------------------------ RMSNorm / RoPE

def test_rms_norm_matches_library_routine():
    x = _rand((2, 5, 48), 12, torch.float32)
    w = _rand((48,), 13, torch.float32)
    ref = torch.nn.functional.rms_norm(x, (48,), w, eps=1e-6)
    assert torch.allclose(prologue.rms_norm(x, w, 1e-6), ref, atol=1e-6)
    # normalises over the whole model dim: unit weight gives unit mean square
    y = prologue.rms_norm(x, torch.ones(48), 1e-12)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(2, 5), atol=1e-5)


def test_rms_norm_rounding_points_bf16():
    x = _rand((1, 3, 64), 14, torch.bfloat16)
    w = _rand((64,), 15, torch.bfloat16)
    y = prologue.rms_norm(x, w)
    assert y.dtype == torch.bfloat16
    xf = x.float()
    n = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    assert torch.equal(y, (n.float() * w.float()).to(torch.bfloat16))


def test_rope_axis_split_and_frequencies():
    assert prologue.rope_axis_pairs(128) == [22, 21, 21]
    ang = prologue.rope_angles(8, 128)
    assert ang.shape == (8, 64)
    # pos 1: theta^(-2m/44) for the frame axis, theta^(-2m/42) for row and col
    assert np.allclose(ang[1, :22], 10000.0 ** (-np.arange(22) * 2 / 44))
    assert np.allclose(ang[1, 22:43], 10000.0 ** (-np.arange(21) * 2 / 42))
    assert np.allclose(ang[1, 43:], 10000.0 ** (-np.arange(21) * 2 / 42))
    assert np.allclose(ang[3], 3 * ang[1])


def test_rope_closed_form_per_token():
    F, h, w, H, D = 2, 3, 4, 2, 12
    x = _rand((1, F * h * w, H, D), 16)
    y = prologue.rope_apply(x, (F, h, w), start_frame=5)
    ang = prologue.rope_angles(64, D)
    n0, n1, _ = prologue.rope_axis_pairs(D)
    for tok in (0, 7, 23):
        fr, rem = divmod(tok, h * w)
        ro, co = divmod(rem, w)
        for m in range(D // 2):
            pos = fr + 5 if m < n0 else (ro if m < n0 + n1 else co)
            zc = complex(x[0, tok, 1, 2 * m], x[0, tok, 1, 2 * m + 1]) * complex(math.cos(ang[pos, m]), math.sin(ang[pos, m]))
            assert abs(float(y[0, tok, 1, 2 * m]) - zc.real) < 1e-12 and abs(float(y[0, tok, 1, 2 * m + 1]) - zc.imag) < 1e-12


def test_rope_preserves_pair_norms_and_shift_is_slicing():
    F, h, w, H, D = 4, 2, 3, 1, 16
    x = _rand((1, F * h * w, H, D), 17)
    y = prologue.rope_apply(x, (F, h, w))
    assert torch.allclose(x.reshape(-1, 2).norm(dim=1), y.reshape(-1, 2).norm(dim=1), atol=1e-12)
    tail = prologue.rope_apply(x[:, 2 * h * w:], (2, h, w), start_frame=2)
    assert torch.allclose(tail, y[:, 2 * h * w:], atol=1e-12)


def test_rope_relative_position_property():
    """<R_p q, R_p' k> depends on p - p' only (frame axis, same row/col)."""
    H, D = 1, 16
    q, k = _rand((1, 1, H, D), 18), _rand((1, 1, H, D), 19)

    def dot(pq, pk):
        a = prologue.rope_apply(q, (1, 1, 1), start_frame=pq)
        b = prologue.rope_apply(k, (1, 1, 1), start_frame=pk)
        return float((a * b).sum())

    assert abs(dot(5, 2) - dot(9, 6)) < 1e-10
    assert abs(dot(5, 2) - dot(5, 3)) > 1e-6


def test_qk_prologue_order_of_operations():
    B, F, h, w, H, D = 1, 2, 2, 3, 2, 12
    xq, xk, xv = (_rand((B, F * h * w, H * D), s, torch.float32) for s in (20, 21, 22))
    wq, wk = _rand((H * D,), 23, torch.float32), _rand((H * D,), 24, torch.float32)
    q, k, v = prologue.qk_prologue(xq, xk, xv, wq, wk, H, (F, h, w), 3)
    assert torch.equal(v, xv.view(B, -1, H, D))
    assert torch.allclose(q, prologue.rope_apply(prologue.rms_norm(xq, wq).view(B, -1, H, D), (F, h, w), 3))
    assert torch.allclose(k, prologue.rope_apply(prologue.rms_norm(xk, wk).view(B, -1, H, D), (F, h, w), 3))


# ------------------------------------------------------------------ KV-cache state machine

def test_cache_trace_seven_chunks_five_passes():
    """local_attn_size = -1, 3-frame chunks of 1560 tokens: chunk c writes [4680c, 4680(c+1)),
    re-runs of the same chunk overwrite the same slot, the view grows by one chunk."""
    st = cache.KVCacheState(32760, 32760, 1560)
    for c in range(7):
        for p in range(5):
            s = st.step(4680 * c, 4680)
            assert (s.cache_start, s.view_len, s.write_start, s.write_end) == (0, 4680 * (c + 1), 4680 * c, 4680 * (c + 1))
            assert s.roll_len == 0
            assert (st.global_end, st.local_end) == (4680 * (c + 1), 4680 * (c + 1))


def test_cache_trace_window_with_sink():
    """4-frame window of 10-token frames, 1 sink frame, 2-frame chunks (hand trace):
    chunk 0 -> [0,20); chunk 1 -> [20,40), cache full; chunk 2 evicts 20 tokens: tokens [30,40) move to
    [10,20) (sink [0,10) stays) and the new chunk lands at [20,40)."""
    st = cache.KVCacheState(40, 40, 10, local_attn_size=4, sink_frames=1)
    s = st.step(0, 20)
    assert (s.write_start, s.write_end, s.view_len, s.roll_len) == (0, 20, 20, 0)
    s = st.step(0, 20)                      # second denoising pass of chunk 0: same slot
    assert (s.write_start, s.write_end, s.roll_len) == (0, 20, 0)
    s = st.step(20, 20)
    assert (s.write_start, s.write_end, s.view_len, s.roll_len) == (20, 40, 40, 0)
    s = st.step(40, 20)
    assert (s.roll_src, s.roll_dst, s.roll_len) == (30, 10, 10)
    assert (s.write_start, s.write_end, s.view_len) == (20, 40, 40)
    s = st.step(40, 20)                     # re-run: no second eviction
    assert s.roll_len == 0 and (s.write_start, s.write_end) == (20, 40)
    assert st.global_end == 60 and st.local_end == 40


def test_cache_max_attention_clamp():
    st = cache.KVCacheState(60, 30, 10)
    st.step(0, 20)
    s = st.step(20, 20)
    assert (s.cache_start, s.view_len, s.write_start, s.write_end) == (10, 30, 10, 30)


# ------------------------------------------------------------------ schedule

def test_sigma_closed_form_and_warped_steps():
    sig, ts = sched.sigma_table(shift=5.0)
    assert len(sig) == 1000 and sig[0] == 1.0
    raw = 1.0 - 250 / 1000
    assert abs(sig[250] - 5 * raw / (1 + 4 * raw)) < 1e-12
    w = sched.warped_steps()
    assert [round(x, 2) for x in w] == [1000.0, 937.5, 833.33, 625.0]
    assert abs(sched.sigma_of(625.0) - 0.625) < 1e-9
