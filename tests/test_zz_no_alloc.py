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


def _call_pair(B, H, D, h, w, nq_frames, nc_frames, tiling, dtype, seed, num_iters=1):
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
        d = sfa.monarch_attn._desc(q, kc, vc, out, f_tied, h_reduce, w_reduce, h, w, D ** -0.5, 1, 0, num_iters)
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


@pytest.mark.parametrize("num_iters", [1, 2])
def test_static_scratch_splits_the_heads_over_several_passes(num_iters):
    """12 heads against a 21-frame cache of 30 x 52 tokens need 624 MB of scratch (1.2 GB with refinement), so the
    128 MiB array serves them in several passes; outputs and caches equal the caller-workspace entry point's, which
    runs one pass."""
    (o_static, o_ws), ((kc_s, vc_s), (kc_w, vc_w)), _ = _call_pair(1, 12, 128, 30, 52, 3, 21, (1, 1, 1), torch.bfloat16, 720,
                                                                  num_iters)
    assert not torch.isnan(o_static.float()).any()
    assert torch.equal(o_static, o_ws)
    assert torch.equal(kc_s, kc_w) and torch.equal(vc_s, vc_w)


def test_static_scratch_rejects_a_unit_that_does_not_fit():
    """One head of fp32 tensors at 30 x 52 with 21 frames and h_reduce = 2 needs 2 matrices of 6 x 52 x 640 rows x
    128 x 4 B = 204 MB > 128 MiB: refused with SFM_ERR_WORKSPACE before anything is written."""
    h, w, D = 30, 52, 128
    q = randn((1, 3 * h * w, 1, D), 730).to(DEV)
    kc, vc = randn((1, 21 * h * w, 1, D), 731).to(DEV), randn((1, 21 * h * w, 1, D), 732).to(DEV)
    kc0 = kc.clone()
    out = torch.zeros_like(q)
    d = sfa.monarch_attn._desc(q, kc, vc, out, 1, 2, 1, h, w, D ** -0.5, 1, 0, 1)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = L.load().sfm_monarch_attn_with_kv_cache_static(C.byref(d), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), q.data_ptr(),
                                                        q.data_ptr(), L.strides3(q), 18 * h * w, 21 * h * w, out.data_ptr(),
                                                        stream)
    torch.cuda.synchronize()
    assert L.ERR_NAMES[rc] == "SFM_ERR_WORKSPACE"
    assert torch.equal(kc, kc0) and not out.any()
