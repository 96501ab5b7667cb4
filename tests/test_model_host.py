"""Host logic of the causal DiT and the rollout pipeline, run on the CPU with oracle attention operators:
cache index state machine, dispatch flags, shapes, scheduler, determinism."""
import numpy as np
import pytest
import torch

import self_forcing_amd as sfa
from oracle import cache as ocache, sched as osched
from oracle.ops import OracleOps

cm, pl = sfa.causal_model, sfa.pipeline
TINY = dict(dim=64, ffn_dim=128, num_heads=2, num_layers=2, text_dim=32, text_len=8, frame_hw=(2, 3), total_seq_len=6 * 6)


def _tiny(ops, seed=0, **flags):
    torch.manual_seed(seed)
    m = cm.CausalWanModel(ops=ops, attention_flags=flags, **TINY)
    m.init_weights(zero_head=False)
    return pl.WanDiffusionWrapper(m.float().eval())


def test_scheduler_matches_closed_form():
    s = pl.FlowMatchScheduler(shift=5.0)
    sig, ts = osched.sigma_table(shift=5.0)
    assert np.allclose(s.sigmas.numpy(), sig, atol=1e-6) and np.allclose(s.timesteps.numpy(), ts, atol=1e-3)
    x0, eps = torch.randn(2, 3, 4, 4), torch.randn(2, 3, 4, 4)
    t = torch.tensor([625.0, 1000.0])
    got = s.add_noise(x0, eps, t)
    for i, tt in enumerate((625.0, 1000.0)):
        sg = osched.sigma_of(tt)
        assert torch.allclose(got[i], (1 - sg) * x0[i] + sg * eps[i], atol=1e-5)


def test_flow_to_x0_conversion():
    gen = _tiny(OracleOps())
    flow, xt = torch.randn(3, 16, 4, 6), torch.randn(3, 16, 4, 6)
    t = torch.tensor([1000.0, 937.5, 625.0])
    x0 = gen._convert_flow_pred_to_x0(flow, xt, t)
    for i, tt in enumerate(t.tolist()):
        assert torch.allclose(x0[i], xt[i] - osched.sigma_of(tt) * flow[i], atol=1e-5)


def test_cache_step_matches_oracle_state_machine():
    for local_attn, sink, max_attn in ((-1, 0, 36), (4, 1, 24), (3, 0, 18)):
        cache_len = 36 if local_attn == -1 else local_attn * 6
        kv = {"k": torch.zeros(1, cache_len, 1, 8), "global_end_index": torch.tensor([0]), "local_end_index": torch.tensor([0])}
        st = ocache.KVCacheState(cache_len, max_attn, 6, local_attn, sink)
        for cur in (0, 0, 12, 12, 24, 24, 24):
            roll, cs, ls, le, ce = cm.cache_step(kv, cur, 12, 6, local_attn, sink, max_attn)
            cm.cache_commit(kv, ce, le)
            o = st.step(cur, 12)
            assert roll == (o.roll_src, o.roll_dst, o.roll_len) or (roll[2] == 0 and o.roll_len == 0)
            assert (cs, ls, le) == (o.cache_start, o.write_start, o.write_end)
            assert int(kv["global_end_index"]) == st.global_end and int(kv["local_end_index"]) == st.local_end


@pytest.mark.parametrize("reset", ["replace", "in_place"])
def test_reference_style_reset_of_a_rolled_window_cache(reset):
    """The reference starts a new video by resetting only the two index tensors (pipeline/causal_inference.py:134-138).
    A windowed cache that has rolled (local end = cache length, global end beyond it) must then start again at 0: the
    host mirrors of the counters follow the tensors, whoever writes them."""
    local_attn, sink, frame = 4, 0, 6
    cache_len = local_attn * frame
    kv = {"k": torch.zeros(1, cache_len, 1, 8), "global_end_index": torch.tensor([0]), "local_end_index": torch.tensor([0])}
    for cur in (0, 12, 24, 36):
        roll, cs, ls, le, ce = cm.cache_step(kv, cur, 12, frame, local_attn, sink, cache_len)
        cm.cache_commit(kv, ce, le)
    assert (le, ce) == (cache_len, 48) and roll[2] > 0
    if reset == "replace":
        kv["global_end_index"] = torch.tensor([0])
        kv["local_end_index"] = torch.tensor([0])
    else:
        kv["global_end_index"].zero_()
        kv["local_end_index"].fill_(0)
    roll, cs, ls, le, ce = cm.cache_step(kv, 0, 12, frame, local_attn, sink, cache_len)
    assert (roll[2], cs, ls, le, ce) == (0, 0, 0, 12, 12)
    cm.cache_commit(kv, ce, le)
    # ... and a run of steps after the reset follows the oracle's state machine from scratch
    st = ocache.KVCacheState(cache_len, cache_len, frame, local_attn, sink)
    st.step(0, 12)
    for cur in (12, 12, 24):
        roll, cs, ls, le, ce = cm.cache_step(kv, cur, 12, frame, local_attn, sink, cache_len)
        cm.cache_commit(kv, ce, le)
        o = st.step(cur, 12)
        assert (cs, ls, le) == (o.cache_start, o.write_start, o.write_end)
    assert int(kv["global_end_index"]) == st.global_end and int(kv["local_end_index"]) == st.local_end


def test_pipeline_rollout_dispatch_and_cache_trace():
    ops = OracleOps()
    gen = _tiny(ops, use_framewise=True)
    pipe = pl.CausalInferencePipeline(gen, frame_hw=(2, 3), num_cache_frames=6)
    noise = torch.randn(1, 6, 16, 4, 6)
    ctx = torch.randn(1, 5, 32)
    out = pipe.inference(noise, ctx)
    assert out.shape == noise.shape and torch.isfinite(out).all() and out.abs().sum() > 0
    assert [round(float(t), 2) for t in pipe.denoising_step_list] == [1000.0, 937.5, 833.33, 625.0]
    # 2 chunks x (4 + 1) passes x 2 layers, Monarch over 3 then 6 cached frames
    mon = [c for c in ops.calls if c[0] == "monarch"]
    assert len(mon) == 20 and [c[1] for c in mon] == [18] * 10 + [36] * 10
    pro = [c for c in ops.calls if c[0] == "prologue"]
    assert [c[1] for c in pro] == [0] * 10 + [3] * 10 and [c[2] for c in pro] == [0] * 10 + [18] * 10
    # cross-attention K/V computed once per layer, then served from the cache
    assert all(c["is_init"] for c in pipe.crossattn_cache)
    assert sum(1 for c in ops.calls if c[0] == "dense") == 20
    assert pipe.kv_cache1[0]["_global_end"] == 36 and int(pipe.kv_cache1[0]["local_end_index"]) == 36
    # a second video resets the counters and gives the same result with the same seeds
    pipe._seed_count = 0
    out2 = pipe.inference(noise, ctx)
    assert torch.equal(out, out2)


def test_dense_init_and_disable_flags():
    ops = OracleOps()
    pipe = pl.CausalInferencePipeline(_tiny(ops, use_framewise=True, use_dense_init=True), frame_hw=(2, 3), num_cache_frames=6)
    pipe.inference(torch.randn(1, 6, 16, 4, 6), torch.randn(1, 5, 32))
    kinds = [c[0] for c in ops.calls if c[0] in ("monarch",) or (c[0] == "dense" and c[1] != 8)]
    assert kinds == ["dense"] * 10 + ["monarch"] * 10          # first chunk (3 cached frames) runs dense
    assert [c[3] for c in ops.calls if c[0] == "prologue"][:10] == [(1, 1, 1)] * 10
    ops2 = OracleOps()
    pipe2 = pl.CausalInferencePipeline(_tiny(ops2, disable_monarch=True), frame_hw=(2, 3), num_cache_frames=6)
    pipe2.inference(torch.randn(1, 3, 16, 4, 6), torch.randn(1, 5, 32))
    assert not any(c[0] == "monarch" for c in ops2.calls)


def test_env_flags_are_read_like_the_reference(monkeypatch):
    monkeypatch.setenv("MONARCH_ATTN_FRAMEWISE", "1")
    monkeypatch.setenv("MONARCH_ATTN_H_REDUCE", "2")
    monkeypatch.setenv("MONARCH_ATTN_DISABLE_LAYERS", "0,3")
    f0, f1 = cm.AttentionFlags(0), cm.AttentionFlags(1)
    assert f0.use_framewise and f0.h_reduce == 2 and f0.disable_monarch and not f1.disable_monarch
    monkeypatch.setenv("MONARCH_ATTN_NUM_ITERS", "8")
    assert cm.AttentionFlags(1).num_iters == 8


def test_patchify_equals_conv3d_and_unpatchify_inverts():
    m = _tiny(OracleOps()).model
    x = torch.randn(2, 16, 3, 4, 6)
    tok, grid = m._patchify(x)
    ref = m.patch_embedding(x).flatten(2).transpose(1, 2)
    assert grid == (3, 2, 3) and torch.allclose(tok, ref, atol=1e-5)
    y = torch.randn(2, 18, 64)
    u = m.unpatchify(y, grid)
    assert u.shape == (2, 16, 3, 4, 6)
    # token (f,h,w), patch offset (q,r), channel c lands at [c, f, 2h+q, 2w+r]
    assert u[1, 5, 2, 3, 4] == y[1, (2 * 2 + 1) * 3 + 2].view(1, 2, 2, 16)[0, 1, 0, 5]


@pytest.mark.parametrize("local_attn,sink,monarch", [(6, 0, True), (9, 3, True), (6, 0, False)])
def test_ring_cache_gives_the_windowed_rollout_of_the_shifting_cache(local_attn, sink, monarch):
    """5 chunks of 3 frames through a window of `local_attn` frames (the first `sink` pinned): the cache kept as a
    ring against the reference's shift-down eviction (causal_model.py:912-926).  Same rows, other order in the
    cache: results agree up to the order of float32 sums."""
    outs = []
    for ring in (False, True):
        flags = dict(use_framewise=True, ring_cache=ring) if monarch else dict(disable_monarch=True, ring_cache=ring)
        torch.manual_seed(0)
        m = cm.CausalWanModel(ops=OracleOps(), attention_flags=flags, local_attn_size=local_attn, sink_size=sink, **TINY)
        m.init_weights(zero_head=False)
        gen = pl.WanDiffusionWrapper(m.float().eval())
        pipe = pl.CausalInferencePipeline(gen, frame_hw=(2, 3), local_attn_size=local_attn)
        g = torch.Generator().manual_seed(3)
        noise = torch.randn(1, 15, 16, 4, 6, generator=g)
        ctx = torch.randn(1, 5, 32, generator=g)
        outs.append(pipe.inference(noise, ctx))
        assert pipe.kv_cache1[0].get("_ring", False) == ring
    assert torch.isfinite(outs[0]).all() and outs[0].abs().sum() > 0
    assert torch.allclose(outs[0], outs[1], atol=2e-5, rtol=1e-4)
    # the first two chunks fit the window; later ones differ from an unbounded cache, so eviction did happen
    assert not torch.allclose(outs[0][:, 9:], _unbounded(noise, ctx)[:, 9:], atol=1e-3)


def _unbounded(noise, ctx):
    torch.manual_seed(0)
    m = cm.CausalWanModel(ops=OracleOps(), attention_flags=dict(use_framewise=True), **{**TINY, "total_seq_len": 15 * 6})
    m.init_weights(zero_head=False)
    pipe = pl.CausalInferencePipeline(pl.WanDiffusionWrapper(m.float().eval()), frame_hw=(2, 3), num_cache_frames=15)
    return pipe.inference(noise, ctx)


def test_ring_cache_falls_back_when_chunks_would_straddle_the_ring():
    kv = {"k": torch.zeros(1, 4 * 6, 1, 8)}           # window of 4 frames, chunks of 3: 4 % 3 != 0
    assert cm.cache_step_ring(kv, 0, 18, 6, 0) == (0, 18, 18)
    assert cm.cache_step_ring(kv, 18, 18, 6, 0) is None
    kv = {"k": torch.zeros(1, 9 * 6, 1, 8)}           # 3 sink frames + ring of 6
    assert cm.cache_step_ring(kv, 54, 18, 6, 3) == (18, 54, 72)
    assert cm.cache_step_ring(kv, 72, 18, 6, 3) == (36, 54, 90)
    assert cm.cache_step_ring(kv, 90, 18, 6, 3) == (18, 54, 108)
    # chunk sizes may change as long as no chunk straddles: two frames at the start of the ring, then four to its end
    assert cm.cache_step_ring(kv, 108, 12, 6, 3) == (36, 54, 120)
    assert cm.cache_step_ring(kv, 120, 6, 6, 3) == (48, 54, 126)
    assert cm.cache_step_ring(kv, 126, 18, 6, 3) == (18, 54, 144)
    assert cm.cache_step_ring(kv, 144, 24, 6, 3) is None


def test_leaving_the_ring_restores_the_reference_row_order():
    """Window of 5 frames, one sink frame, chunks of 2, 2, 1 (fills), 2 (ring), then 3 (would straddle) and 1: the same
    rollout with the shifting cache from the start holds the same rows in the same places afterwards."""
    outs, caches = [], []
    for ring in (False, True):
        torch.manual_seed(0)
        att = cm.CausalWanSelfAttention(16, 2, 5, 1, True, 1e-6, 0, (2, 3), None,
                                        cm.AttentionFlags(0, disable_monarch=True, ring_cache=ring),
                                        OracleOps(compute_dtype=torch.float64)).double().eval()
        kv = {"k": torch.zeros(1, 30, 2, 8, dtype=torch.float64), "v": torch.zeros(1, 30, 2, 8, dtype=torch.float64),
              "global_end_index": torch.tensor([0]), "local_end_index": torch.tensor([0])}
        g = torch.Generator().manual_seed(1)
        ys, start = [], 0
        for frames in (2, 2, 1, 2, 3, 1):
            x = torch.randn(1, frames * 6, 16, generator=g, dtype=torch.float64)
            with torch.no_grad():
                ys.append(att(x, (frames, 2, 3), kv, start * 6))
            if frames == 2 and start >= 5:
                assert kv.get("_ring", False) == ring
            start += frames
        assert not kv.get("_ring", False)
        outs.append(torch.cat(ys, 1))
        caches.append((kv["k"].clone(), kv["v"].clone(), int(kv["global_end_index"]), int(kv["local_end_index"])))
    assert torch.allclose(outs[0], outs[1], atol=1e-12)
    assert torch.equal(caches[0][0], caches[1][0]) and torch.equal(caches[0][1], caches[1][1])
    assert caches[0][2:] == caches[1][2:]
