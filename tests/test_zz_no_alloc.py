"""The entry point that allocates nothing (sfm_monarch_attn_with_kv_cache_static) against the entry point it is a
variant of (sfm_monarch_attn_with_kv_cache with a caller-owned workspace), through the C ABI: outputs and cache
contents bit for bit, on two calls in a row of which the second is smaller (the shared scratch keeps the first
call's contents)."""
import ctypes as C

import pytest
import torch

import self_forcing_amd as sfa
from self_forcing_amd import lib as L
from gpu_util import assert_close_16bit, randn
from oracle import monarch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call_pair(B, H, D, h, w, nq_frames, nc_frames, tiling, dtype, seed):
    """Runs both entry points on the same inputs; returns (static out, workspace out, caches of both, oracle inputs)."""
    f_tied, h_reduce, w_reduce = tiling
    nq, nc = nq_frames * h * w, nc_frames * h * w
    q, nk, nv = (randn((B, nq, H, D), seed + i, dtype).to(DEV) for i in range(3))
    kc0, vc0 = randn((B, nc, H, D), seed + 3, dtype).to(DEV), randn((B, nc, H, D), seed + 4, dtype).to(DEV)
    lib = L.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs, caches = [], []
    for static in (True, False):
        kc, vc = kc0.clone(), vc0.clone()
        out = torch.full_like(q, float("nan"))
        d = sfa.monarch_attn._desc(q, kc, vc, out, f_tied, h_reduce, w_reduce, h, w, D ** -0.5, 1, 0, 1)
        args = (C.byref(d), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), nk.data_ptr(), nv.data_ptr(), L.strides3(nk),
                nc - nq, nc, out.data_ptr())
        if static:
            L.check(lib.sfm_monarch_attn_with_kv_cache_static(*args, stream))
        else:
            n = sfa.monarch_attn.monarch_workspace_bytes(d)
            ws = torch.empty(n, dtype=torch.uint8, device=DEV)
            L.check(lib.sfm_monarch_attn_with_kv_cache(*args, ws.data_ptr(), n, stream))
        torch.cuda.synchronize()
        outs.append(out)
        caches.append((kc, vc))
    return outs, caches, (q, kc0, vc0, nk, nv)


def test_static_scratch_matches_workspace_entry_point_twice():
    dtype = torch.bfloat16
    # first call: 480p block shape, 2 heads, 9-frame cache; second call: smaller grid, fewer frames, another tiling
    for (B, H, D, h, w, nqf, ncf, tiling, seed) in ((1, 2, 128, 30, 52, 3, 9, (1, 1, 1), 700),
                                                    (1, 2, 128, 6, 52, 3, 6, (3, 1, 1), 710)):
        (o_static, o_ws), ((kc_s, vc_s), (kc_w, vc_w)), (q, kc0, vc0, nk, nv) = _call_pair(B, H, D, h, w, nqf, ncf, tiling,
                                                                                          dtype, seed)
        assert not torch.isnan(o_static.float()).any()
        assert torch.equal(o_static, o_ws)
        assert torch.equal(kc_s, kc_w) and torch.equal(vc_s, vc_w)
        nq, nc = nqf * h * w, ncf * h * w
        ref = monarch.monarch_attn_with_kv_cache(q.cpu(), kc0.cpu(), vc0.cpu(), nk.cpu(), nv.cpu(), nc - nq, nc, *tiling, h, w,
                                                 dtype=torch.float32)
        assert_close_16bit(o_static, ref, dtype)
