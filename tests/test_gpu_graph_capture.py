"""The KV-cache attention operators under HIP graph capture: the library allocates nothing and never synchronises, so a
call can be recorded once and replayed; every replay is checked against the eager result on the same inputs."""
import pytest
import torch

import self_forcing_amd as sfa

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
mattn = sfa.monarch_attn


@pytest.mark.parametrize("op", ["monarch", "dense"])
def test_kv_cache_op_replays_from_a_graph(op):
    A, F, b1, b2, H, D, new_f = 2, 5, 6, 52, 3, 128, 2
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(123)
    mk = lambda n: torch.randn(1, n * b1 * b2, H, D, generator=g).to(dtype).to(DEV)
    q, kc, vc, nk, nv = mk(A), mk(F), mk(F), mk(new_f), mk(new_f)
    start, end = (F - new_f) * b1 * b2, F * b1 * b2
    if op == "monarch":
        call, args = mattn.monarch_attn_with_kv_cache, (start, end, 1, 1, 1, b1, b2, D ** -0.5)
    else:
        call, args = sfa.attention.full_attention_with_kv_cache, (start, end, D ** -0.5)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up outside the capture
        call(q, kc, vc, nk, nv, *args)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call(q, kc, vc, nk, nv, *args)
    for it in range(4):
        for t in (q, nk, nv):
            t.copy_(torch.randn(t.shape, generator=g).to(dtype))      # new contents, same addresses
        kc[:, :start].copy_(torch.randn(kc[:, :start].shape, generator=g).to(dtype))
        vc[:, :start].copy_(torch.randn(vc[:, :start].shape, generator=g).to(dtype))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        kc2, vc2 = kc.clone(), vc.clone()
        want = call(q, kc2, vc2, nk, nv, *args)      # eager, between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {it}"
        assert torch.equal(kc, kc2) and torch.equal(vc, vc2)


def test_a_whole_model_pass_replays_from_a_graph():
    """One pass of the causal DiT (2 layers, every operator of the block, time embedding, head) recorded once and
    replayed with new latents and timesteps at the same addresses: every replay equals the eager pass on those inputs,
    with eager work and synchronisation between the replays.  Nothing in the pass copies from the host or waits for
    the device."""
    cm, pl = sfa.causal_model, sfa.pipeline
    torch.manual_seed(0)
    model = cm.CausalWanModel(attention_flags=dict(use_framewise=True), dim=256, ffn_dim=512, num_heads=2, num_layers=2,
                              text_dim=64, text_len=16, frame_hw=(6, 52), total_seq_len=6 * 6 * 52)
    model.init_weights(zero_head=False)
    gen = pl.WanDiffusionWrapper(model.to(torch.bfloat16).eval().to(DEV))
    g = torch.Generator().manual_seed(7)
    new_x = lambda: torch.randn(1, 3, 16, 12, 104, generator=g).to(torch.bfloat16).to(DEV)
    x, t = new_x(), torch.full((1, 3), 750, device=DEV, dtype=torch.int64)
    cond = {"prompt_embeds": torch.randn(1, 16, 64, generator=g).to(torch.bfloat16).to(DEV)}
    kv = [{"k": torch.zeros(1, 6 * 312, 2, 128, dtype=torch.bfloat16, device=DEV),
           "v": torch.zeros(1, 6 * 312, 2, 128, dtype=torch.bfloat16, device=DEV),
           "global_end_index": torch.tensor([0], device=DEV), "local_end_index": torch.tensor([0], device=DEV)} for _ in range(2)]
    ca = [{"k": None, "v": None, "is_init": False} for _ in range(2)]
    gen(new_x(), cond, t, kv, ca, 0)                                  # the first chunk, eager: fills the cache's first half
    call = lambda: gen(x, cond, t, kv, ca, 3 * 312)[1]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call()
    for it, step in enumerate((1000, 500, 250, 0)):
        x.copy_(new_x())
        t.fill_(step)
        graph.replay()
        torch.cuda.synchronize()
        got, k_got = out.clone(), [c["k"].clone() for c in kv]
        want = call()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {it}"
        assert all(torch.equal(a, c["k"]) for a, c in zip(k_got, kv))
