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
