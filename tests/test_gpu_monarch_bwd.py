"""GPU parity of the Monarch backward (autograd Functions over sfm_monarch_bwd) against torch autograd through the
float64 CPU oracle.  Shapes follow the reference's harness (run_kv_cache_test / run_causal_test,
monarch_attn.py:1880-1957) at sizes the oracle finishes in seconds.

Tolerances: fp32 tensors <= 2e-4 of the gradient's max-abs (fp32 kernels, sums of ~10^3 terms); 16-bit tensors the
reference harness's own raw bar, atol = rtol = 1e-2 (bf16) / 1e-3 (fp16) on the unscaled gradients
(monarch_attn.py:1908-1920)."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import max_abs, randn
from oracle import blocks, monarch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
mattn = sfa.monarch_attn


def _leaf(t, dev=None):
    t = t.clone().detach()
    if dev:
        t = t.to(dev)
    return t.requires_grad_(True)


def _close(got, ref, dtype):
    got, ref = got.detach().float().cpu(), ref.detach().float()
    if dtype == torch.float32:
        assert (got - ref).abs().max() <= 2e-4 * max(1.0, ref.abs().max().item())
    else:
        # the reference harness's own bar (monarch_attn.py:1908-1920): raw atol = rtol = 1e-2 (bf16) / 1e-3 (fp16).
        # 16-bit gradients are rounded once at the end; accumulation is fp32
        tol = 1e-2 if dtype == torch.bfloat16 else 1e-3
        assert torch.allclose(got, ref, atol=tol, rtol=tol), ((got - ref).abs().max().item(), ref.abs().max().item())


@pytest.fixture
def switches():
    """Sets the library's process-wide implementation switches for one test and puts the old mask back."""
    lib = sfa.lib.load()
    old = lib.sfm_get_switches()
    yield lib.sfm_set_switches
    lib.sfm_set_switches(old)


@pytest.fixture(params=["gemm", "simt"])
def bwd_path(request, switches):
    """Both backward implementations behind sfm_monarch_bwd: batched library GEMMs + row kernels (default) and the
    fp32 SIMT kernels (the SFM_SW_BWD_SIMT switch, also what runs when rocBLAS cannot be loaded)."""
    switches(sfa.lib.SW_BWD_SIMT if request.param == "simt" else 0)
    assert sfa.lib.load().sfm_monarch_bwd_uses_gemm() == (1 if request.param == "gemm" else 0)
    return request.param


@pytest.mark.parametrize("tiling,h,w", [((1, 1, 1), 4, 8), ((1, 2, 1), 6, 8), ((3, 1, 1), 4, 6), ((1, 1, 2), 3, 8)])
def test_no_cache_fp32_gradients(tiling, h, w, bwd_path):
    F = 3
    q0 = randn((2, F * h * w, 2, 32), 100, torch.float32)
    k0, v0 = (randn((2, 2 * F * h * w, 2, 32), 101 + i, torch.float32) for i in range(2))
    do = randn((2, F * h * w, 2, 32), 103, torch.float32)
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, *tiling, h, w).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    out = mattn.monarch_attn(qd, kd, vd, *tiling, h, w)
    out.backward(do.to(DEV))
    _close(qd.grad, qr.grad, torch.float32)
    _close(kd.grad, kr.grad, torch.float32)
    _close(vd.grad, vr.grad, torch.float32)


@pytest.mark.parametrize("tiling,h,w", [((1, 1, 1), 4, 8), ((1, 2, 1), 6, 8), ((3, 1, 1), 4, 8), ((1, 1, 2), 3, 16), ((3, 2, 2), 4, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_no_cache_16bit_gradients_over_the_tilings(tiling, h, w, dtype):
    """Token-order k, v (no cache): the fused kernels read q, k, v rows through the tiling's index maps."""
    F, H, D = 3, 2, 64
    q0, do = (randn((1, F * h * w, H, D), 180 + i, dtype) for i in range(2))
    k0, v0 = (randn((1, 2 * F * h * w, H, D), 182 + i, dtype) for i in range(2))
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, *tiling, h, w).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    mattn.monarch_attn(qd, kd, vd, *tiling, h, w).backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(kd.grad, kr.grad, dtype)
    _close(vd.grad, vr.grad, dtype)


def test_block_causal_fp32_gradients(bwd_path):
    h, w, F = 3, 8, 4
    q0, k0, v0, do = (randn((1, F * h * w, 2, 64), 110 + i, torch.float32) for i in range(4))
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, 1, 1, 1, h, w, block_causal_size=2 * h * w).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    mattn.monarch_attn(qd, kd, vd, 1, 1, 1, h, w, block_causal_size=2 * h * w).backward(do.to(DEV))
    _close(qd.grad, qr.grad, torch.float32)
    _close(kd.grad, kr.grad, torch.float32)
    _close(vd.grad, vr.grad, torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("partial", [False, True])
def test_kv_cache_gradients_like_the_reference_harness(dtype, partial, bwd_path):
    """q of 2 frames, cache of 5 frames of which the last 2 arrive with the call; h_reduce = 2 so that block
    order differs from token order.  partial = grad_only_new_kv."""
    h, w, H, D = 6, 20, 2, 64
    tiling = (1, 2, 1)
    n_old, n_new = 3 * h * w, 2 * h * w
    q0 = randn((1, 2 * h * w, H, D), 120, dtype)
    k_old, v_old = (randn((1, n_old, H, D), 121 + i, dtype) for i in range(2))       # cache rows (block order)
    k_new, v_new = (randn((1, n_new, H, D), 123 + i, dtype) for i in range(2))       # token order
    do = randn((1, 2 * h * w, H, D), 125, dtype)

    # oracle: functional composition of the cache write, float64
    qr, kor, vor, knr, vnr = (_leaf(t.double()) for t in (q0, k_old, v_old, k_new, v_new))
    kfull = torch.cat([kor, blocks.to_blocks(knr, *tiling, h, w).reshape(1, n_new, H, D)], 1)
    vfull = torch.cat([vor, blocks.to_blocks(vnr, *tiling, h, w).reshape(1, n_new, H, D)], 1)
    qb = blocks.to_blocks(qr, *tiling, h, w)
    b1, b2 = qb.shape[2], qb.shape[3]
    ob = monarch.monarch_1iter(qb, kfull.reshape(1, -1, b1, b2, H, D), vfull.reshape(1, -1, b1, b2, H, D), D ** -0.5)
    blocks.from_blocks(ob, *tiling, h, w).backward(do.double())

    qd, knd, vnd = _leaf(q0, DEV), _leaf(k_new, DEV), _leaf(v_new, DEV)
    kc = torch.zeros(1, n_old + n_new, H, D, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    kc[:, :n_old], vc[:, :n_old] = k_old.to(DEV), v_old.to(DEV)
    kc.requires_grad_(not partial)
    vc.requires_grad_(not partial)
    out = mattn.monarch_attn_with_kv_cache(qd, kc, vc, knd, vnd, n_old, n_old + n_new, *tiling, h, w,
                                           grad_only_new_kv=partial)
    out.backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(knd.grad, knr.grad, dtype)
    _close(vnd.grad, vnr.grad, dtype)
    if not partial:
        _close(kc.grad[:, :n_old], kor.grad, dtype)
        _close(vc.grad[:, :n_old], vor.grad, dtype)
    else:
        assert kc.grad is None and vc.grad is None


def test_480p_block_shape_bf16_one_head(bwd_path):
    """b1 = 30, b2 = 52, D = 128 as in the 480p grid: 1 query frame against 3 cached frames, one head."""
    h, w, D = 30, 52, 128
    q0 = randn((1, h * w, 1, D), 130, torch.bfloat16)
    k0, v0 = (randn((1, 3 * h * w, 1, D), 131 + i, torch.bfloat16) for i in range(2))
    do = randn((1, h * w, 1, D), 133, torch.bfloat16)
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, 1, 1, 1, h, w).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    mattn.monarch_attn(qd, kd, vd, 1, 1, 1, h, w).backward(do.to(DEV))
    _close(qd.grad, qr.grad, torch.bfloat16)
    _close(kd.grad, kr.grad, torch.bfloat16)
    _close(vd.grad, vr.grad, torch.bfloat16)


@pytest.mark.parametrize("h,w,Fq,Fk,D,causal,dtype", [
    (4, 52, 3, 3, 128, True, torch.bfloat16),      # 156 (a, j) columns: every fused kernel, last column block partial
    (4, 52, 3, 5, 64, False, torch.float16),
    (4, 52, 4, 4, 64, True, torch.bfloat16),       # 208 columns: two passes of the right-factor kernel over each tile
    (4, 52, 7, 7, 128, False, torch.float16),      # 364 columns: three passes
    (5, 6, 2, 3, 64, False, torch.bfloat16),       # b2 = 6, not a multiple of 4: likewise
    (4, 20, 3, 9, 128, False, torch.bfloat16),     # 36 rows (f, k) per column: two chunks of the left factor, the second with 4 rows
    (8, 12, 2, 8, 64, False, torch.float16),       # 64 rows: two full chunks
    (6, 10, 6, 6, 128, True, torch.bfloat16),      # block-causal with two chunks: the visible rows end inside a chunk
    (40, 12, 2, 2, 128, False, torch.bfloat16),    # b1 = 40: two 32-row query tiles in the left factor (partial slabs summed)
    (90, 52, 1, 2, 128, False, torch.bfloat16),    # b1 = 90, b2 = 52: three frames of 30 x 52 tied per block, as the reference's default tiling
    (100, 8, 3, 3, 64, True, torch.float16),       # four tiles, block-causal
])
def test_16bit_gradients_across_the_fused_kernels_limits(h, w, Fq, Fk, D, causal, dtype):
    H = 2
    q0, do = (randn((1, Fq * h * w, H, D), 150 + i, dtype) for i in range(2))
    k0, v0 = (randn((1, Fk * h * w, H, D), 152 + i, dtype) for i in range(2))
    kw = {"block_causal_size": h * w} if causal else {}
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, 1, 1, 1, h, w, **kw).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    mattn.monarch_attn(qd, kd, vd, 1, 1, 1, h, w, **kw).backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(kd.grad, kr.grad, dtype)
    _close(vd.grad, vr.grad, dtype)


@pytest.mark.parametrize("causal", [False, True])
def test_backward_with_and_without_the_forwards_saved_tensors(causal):
    """sfm_monarch_bwd recomputes the left factor's row statistics; sfm_monarch_bwd_saved takes them (and the output)
    from sfm_monarch_fwd_stats.  Both against the float64 oracle, and the forward with statistics against the plain one."""
    h, w, F, H, D = 4, 52, 3, 3, 128
    dtype = torch.bfloat16
    q0, do = (randn((2, F * h * w, H, D), 160 + i, dtype) for i in range(2))
    k0, v0 = (randn((2, F * h * w, H, D), 162 + i, dtype) for i in range(2))
    kw = {"block_causal_size": h * w} if causal else {}
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, 1, 1, 1, h, w, **kw).backward(do.double())
    qd, kd, vd, dod = q0.to(DEV), k0.to(DEV), v0.to(DEV), do.to(DEV)
    tiling, cbf = (1, 1, 1, h, w), 1 if causal else 0
    out, stats = mattn._monarch_fwd_stats(qd, kd, vd, tiling, D ** -0.5, 0, cbf)
    assert stats is not None and stats.dtype == torch.float32
    assert torch.equal(out, mattn.monarch_attn(qd, kd, vd, *tiling, **kw))
    # the statistics do not depend on how many (batch, head) units a pass of the forward takes
    out4, stats4 = mattn._monarch_fwd_stats(qd, kd, vd, tiling, D ** -0.5, 0, cbf, heads_per_pass=4)
    # (one float per block row, rows padded to 32 per (unit, a, j): the padding is never written)
    valid = lambda st: st.view(2 * H, F * w, 32)[..., :h]
    assert torch.equal(out, out4) and torch.equal(valid(stats), valid(stats4))
    for kept in ({}, {"out": out, "stats": stats}, {"out": out, "stats": stats, "heads_per_pass": 4}):
        dq, dk, dv = mattn._monarch_bwd(qd, kd, vd, dod, tiling, D ** -0.5, 0, cbf, **kept)
        _close(dq, qr.grad, dtype)
        _close(dk, kr.grad, dtype)
        _close(dv, vr.grad, dtype)
    # fp32 tensors run the forward without statistics: the autograd path falls back to recomputing
    out32, stats32 = mattn._monarch_fwd_stats(qd.float(), kd.float(), vd.float(), tiling, D ** -0.5, 0, cbf)
    assert stats32 is None


@pytest.mark.parametrize("switch", ["SW_BWD_LEFT_GEMM", "SW_BWD_FWD_GEMM", "SW_BWD_DQA_GEMM", "SW_BWD_RIGHT_GEMM", "SW_BWD_DQK_GEMM"])
def test_each_fused_part_can_fall_back_to_the_library_chain(switch, switches):
    """The measurement switches that put one fused part back on the batched GEMMs + row kernels (what also runs for
    shapes a fused kernel does not take): same gradients, and the workspace query follows the switch."""
    switches(getattr(sfa.lib, switch))
    h, w, F, H, D = 4, 20, 2, 2, 64
    dtype = torch.bfloat16
    q0, do = (randn((1, F * h * w, H, D), 170 + i, dtype) for i in range(2))
    k0, v0 = (randn((1, 3 * h * w, H, D), 172 + i, dtype) for i in range(2))
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, 1, 1, 1, h, w).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    mattn.monarch_attn(qd, kd, vd, 1, 1, 1, h, w).backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(kd.grad, kr.grad, dtype)
    _close(vd.grad, vr.grad, dtype)


def test_480p_block_shape_new_frame_gradients_only():
    """b1 = 30, b2 = 52, D = 128: one query frame against a cache of three frames whose last one arrives with the call;
    grad_only_new_kv, so that the right-factor kernel skips the gradient products of two of the three block-frames."""
    h, w, H, D = 30, 52, 1, 128
    dtype = torch.bfloat16
    n = h * w
    q0, do = (randn((1, n, H, D), 190 + i, dtype) for i in range(2))
    k_old, v_old = (randn((1, 2 * n, H, D), 192 + i, dtype) for i in range(2))
    k_new, v_new = (randn((1, n, H, D), 194 + i, dtype) for i in range(2))
    qr, kor, vor, knr, vnr = (_leaf(t.double()) for t in (q0, k_old, v_old, k_new, v_new))
    monarch.monarch_attn(qr, torch.cat([kor, knr], 1), torch.cat([vor, vnr], 1), 1, 1, 1, h, w).backward(do.double())
    qd, knd, vnd = _leaf(q0, DEV), _leaf(k_new, DEV), _leaf(v_new, DEV)
    kc = torch.zeros(1, 3 * n, H, D, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    kc[:, :2 * n], vc[:, :2 * n] = k_old.to(DEV), v_old.to(DEV)
    out = mattn.monarch_attn_with_kv_cache(qd, kc, vc, knd, vnd, 2 * n, 3 * n, 1, 1, 1, h, w, grad_only_new_kv=True)
    out.backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(knd.grad, knr.grad, dtype)
    _close(vnd.grad, vnr.grad, dtype)


def test_fused_chain_runs_without_rocblas():
    """Where every part of the chain has a fused kernel no library product is called: a process that cannot load rocBLAS
    (SFM_NO_ROCBLAS) gets the same gradients, bit for bit, as this one."""
    import os
    import subprocess
    import sys
    h, w, F, H, D = 4, 20, 2, 2, 64
    code = f"""
import sys, torch
sys.path.insert(0, {os.path.dirname(os.path.abspath(__file__))!r}); sys.path.insert(0, {os.path.dirname(os.path.dirname(os.path.abspath(__file__)))!r})
import self_forcing_amd as sfa
from gpu_util import randn
assert sfa.lib.load().sfm_monarch_bwd_uses_gemm() == int(sys.argv[1])
q, do = (randn((1, {F * h * w}, {H}, {D}), 230 + i, torch.bfloat16).cuda() for i in range(2))
k, v = (randn((1, {3 * h * w}, {H}, {D}), 232 + i, torch.bfloat16).cuda() for i in range(2))
q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
sfa.monarch_attn.monarch_attn(q, k, v, 1, 1, 1, {h}, {w}).backward(do)
print("SUM", *(float(t.grad.double().abs().sum()) for t in (q, k, v)))
"""
    outs = []
    for no_blas in (False, True):
        env = dict(os.environ)
        env.pop("SFM_NO_ROCBLAS", None)
        if no_blas:
            env["SFM_NO_ROCBLAS"] = "1"
        r = subprocess.run([sys.executable, "-c", code, "0" if no_blas else "1"], env=env, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append([ln for ln in r.stdout.splitlines() if ln.startswith("SUM")][0])
    assert outs[0] == outs[1]


def test_descriptor_errors():
    q = randn((1, 64, 1, 32), 140, torch.float32).to(DEV).requires_grad_(True)
    with pytest.raises(ValueError):                        # block-causal masking is defined for one iteration only
        mattn.monarch_attn(q, q, q, 1, 1, 1, 4, 8, block_causal_size=32, num_iters=2)


@pytest.mark.parametrize("saved", [False, True])
def test_three_frames_tied_480p_blocks_on_the_fused_kernels(saved):
    """The reference's default tiling at 480p (f_tied = 3: b1 = 90, b2 = 52), 3 query frames against 6, through the tiling's
    index maps; with the forward's saved output and statistics and recomputing them.  The fused chain must be the one
    that runs: its workspace is smaller than the library chain's."""
    h, w, H, D = 30, 52, 1, 128
    dtype = torch.bfloat16
    q0, do = (randn((1, 3 * h * w, H, D), 180 + i, dtype) for i in range(2))
    k0, v0 = (randn((1, 6 * h * w, H, D), 182 + i, dtype) for i in range(2))
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    monarch.monarch_attn(qr, kr, vr, 3, 1, 1, h, w).backward(do.double())
    qd, kd, vd, dod = q0.to(DEV), k0.to(DEV), v0.to(DEV), do.to(DEV)
    tiling = (3, 1, 1, h, w)
    kept = {}
    if saved:
        out, stats = mattn._monarch_fwd_stats(qd, kd, vd, tiling, D ** -0.5, 0, 0)
        assert stats is not None
        kept = {"out": out, "stats": stats}
    dq, dk, dv = mattn._monarch_bwd(qd, kd, vd, dod, tiling, D ** -0.5, 0, 0, **kept)
    _close(dq, qr.grad, dtype)
    _close(dk, kr.grad, dtype)
    _close(dv, vr.grad, dtype)


@pytest.mark.parametrize("h,w,Fq,Fk,H,hpp", [
    (4, 52, 3, 5, 3, 0),        # one slab: every fused part, all heads in one pass
    (40, 12, 2, 3, 3, 2),       # b1 = 40: two query-row slices (two slabs of partial sums), a shorter last pass
    (90, 8, 1, 2, 2, 1),        # three slices, one head per pass
    (5, 6, 2, 3, 2, 0),         # b2 = 6: the right factor on the library chain, whose scratch is laid out differently
])
def test_backward_stays_inside_an_exactly_sized_workspace(h, w, Fq, Fk, H, hpp):
    """sfm_monarch_bwd with a workspace of exactly the queried size and canary bytes behind it; the gradients equal the
    autograd path's, which sizes its own scratch."""
    from gpu_util import monarch_bwd_exact_workspace
    dtype, D = torch.bfloat16, 64
    q0, do = (randn((1, Fq * h * w, H, D), 400 + i, dtype).to(DEV) for i in range(2))
    k0, v0 = (randn((1, Fk * h * w, H, D), 402 + i, dtype).to(DEV) for i in range(2))
    dq, dk, dv = monarch_bwd_exact_workspace(q0, k0, v0, do, (1, 1, 1, h, w), hpp)
    want = mattn._monarch_bwd(q0, k0, v0, do, (1, 1, 1, h, w), D ** -0.5, 0, 0)
    for got, ref in zip((dq, dk, dv), want):
        assert torch.equal(got, ref)
