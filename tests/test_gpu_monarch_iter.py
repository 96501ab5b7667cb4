"""GPU parity of the iterated-refinement Monarch path (num_iters > 1) through the C ABI, against the
reference's own golden vectors (monarch_attn_slow, tests/golden/) and the CPU oracle.

Tolerances: fp32 tensors <= 2e-5 max-abs (fp32 kernels against a float64 oracle, several chained
softmaxes); 16-bit tensors the reference's atol = rtol = 1e-2 (bf16) / 1e-3 (fp16)."""
import os

import numpy as np
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import assert_close_16bit, max_abs, monarch_fwd_exact_workspace, randn
from oracle import monarch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
mattn = sfa.monarch_attn
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "monarch_reference_vectors.npz"))


def _golden_inputs(ci):
    seed, B, a, f, b1, b2, H, D = (int(x) for x in GOLD[f"case{ci}_meta"])
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, a, b1, b2, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, f, b1, b2, H, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, f, b1, b2, H, D, generator=g, dtype=torch.float64)
    return q, k, v, float(GOLD[f"case{ci}_scale"]), (B, a, f, b1, b2, H, D)


@pytest.mark.parametrize("ci", [0, 1, 2])
@pytest.mark.parametrize("n", [2, 3, 8])
def test_golden_vectors_of_the_reference_refinement(ci, n):
    """With f_tied = h_reduce = w_reduce = 1 and h = b1, w = b2 token order is block order, so the stored
    blocked tensors are the token-order inputs reshaped."""
    q, k, v, s, (B, a, f, b1, b2, H, D) = _golden_inputs(ci)
    tok = lambda t: t.reshape(B, -1, H, D).float().to(DEV)
    out = mattn.monarch_attn(tok(q), tok(k), tok(v), 1, 1, 1, b1, b2, sm_scale=s, num_iters=n)
    gold = torch.from_numpy(GOLD[f"case{ci}_slow{n}"]).reshape(B, -1, H, D)
    assert max_abs(out, gold) < 2e-5


@pytest.mark.parametrize("tiling,h,w", [((1, 1, 1), 6, 20), ((1, 2, 1), 6, 20), ((3, 1, 1), 4, 12), ((1, 1, 2), 5, 8)])
@pytest.mark.parametrize("n", [2, 4])
def test_fp32_tilings_against_oracle(tiling, h, w, n):
    F = 3
    q = randn((2, F * h * w, 2, 64), 70, torch.float32)
    k, v = (randn((2, 2 * F * h * w, 2, 64), 71 + i, torch.float32) for i in range(2))
    ref = monarch.monarch_attn(q, k, v, *tiling, h, w, num_iters=n)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), *tiling, h, w, num_iters=n)
    assert max_abs(out, ref) < 2e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_16bit_inputs_and_cache_entry_point(dtype):
    """Cache holds 2 of 3 frames, the third arrives with the call; rows are in block order (h_reduce = 2)."""
    h, w, H, D = 6, 20, 3, 128
    q = randn((1, h * w, H, D), 80, dtype)
    k, v = (randn((1, 3 * h * w, H, D), 81 + i, dtype) for i in range(2))
    ref = monarch.monarch_attn(q, k, v, 1, 2, 1, h, w, num_iters=3, dtype=torch.float32)
    kc, vc = torch.zeros(1, 3 * h * w, H, D, dtype=dtype, device=DEV), torch.zeros(1, 3 * h * w, H, D, dtype=dtype, device=DEV)
    mattn.monarch_attn_with_kv_cache(q.to(DEV), kc, vc, k[:, :2 * h * w].to(DEV), v[:, :2 * h * w].to(DEV), 0, 2 * h * w,
                                     1, 2, 1, h, w)
    out = mattn.monarch_attn_with_kv_cache(q.to(DEV), kc, vc, k[:, 2 * h * w:].to(DEV), v[:, 2 * h * w:].to(DEV),
                                           2 * h * w, 3 * h * w, 1, 2, 1, h, w, num_iters=3)
    assert_close_16bit(out, ref, dtype)


def test_one_and_many_iterations_share_limits():
    """num_iters == 1 stays on the fast path (no 1/(1 + 1e-6) factor); the first refinement pass of the iterated
    path carries it, as the reference's pure-torch function does."""
    q, k, v = (randn((1, n * 4 * 16, 2, 64), 90 + i, torch.float32) for i, n in enumerate((2, 3, 3)))
    one = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, 4, 16, num_iters=1)
    ref1 = monarch.monarch_attn(q, k, v, 1, 1, 1, 4, 16)
    assert max_abs(one, ref1) < 1e-5
    with pytest.raises(ValueError):
        mattn.monarch_attn(q.to(DEV), q.to(DEV), q.to(DEV), 1, 1, 1, 4, 16, block_causal_size=64, num_iters=2)


@pytest.mark.parametrize("f_tied", [1, 3])
def test_c2_shape_two_iterations_bf16(f_tied):
    """Full 480p sizes (3 query frames, 21 cached frames of 30 x 52 tokens), 2 heads, frame-wise blocks
    (b1 = 30) and three frames tied per block (b1 = 90, query rows taken in chunks): against the oracle on
    head 0 and through the size-independent property that constant V gives constant output."""
    a, f, b1, b2, H, D = 3, 21, 30, 52, 2, 128
    q = randn((1, a * b1 * b2, H, D), 95, torch.bfloat16)
    k = randn((1, f * b1 * b2, H, D), 96, torch.bfloat16)
    v = randn((1, f * b1 * b2, H, D), 97, torch.bfloat16)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), f_tied, 1, 1, b1, b2, num_iters=2)
    ref = monarch.monarch_attn(q[:, :, :1], k[:, :, :1], v[:, :, :1], f_tied, 1, 1, b1, b2, num_iters=2, dtype=torch.float32)
    assert_close_16bit(out[:, :, :1], ref, torch.bfloat16)
    vc = torch.full_like(v, 0.75)
    outc = mattn.monarch_attn(q.to(DEV), k.to(DEV), vc.to(DEV), f_tied, 1, 1, b1, b2, num_iters=2)
    assert max_abs(outc, torch.full_like(q, 0.75)) < 4e-3


@pytest.fixture
def switches():
    lib = sfa.lib.load()
    old = lib.sfm_get_switches()
    yield lib.sfm_set_switches
    lib.sfm_set_switches(old)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("h,w,D,frames,n", [(6, 20, 128, (1, 3), 2), (8, 40, 64, (2, 3), 3), (30, 52, 128, (1, 2), 3),
                                             (5, 33, 64, (2, 2), 8), (32, 64, 128, (1, 2), 2), (4, 8, 128, (3, 5), 8),
                                             (40, 33, 128, (1, 2), 3),       # two 32-row query tiles
                                             (90, 20, 64, (1, 2), 2),        # three (b1 = 90: three 30-row frames tied)
                                             (100, 8, 128, (2, 1), 2),       # four
                                             (6, 80, 128, (2, 3), 2),        # 80 columns: three key tiles in step 1
                                             (5, 128, 64, (1, 2), 3),        # 128 columns
                                             (45, 80, 128, (1, 2), 2)])      # the 720p grid
def test_mfma_refinement_against_the_oracle_and_the_fp32_kernels(dtype, h, w, D, frames, n, switches):
    """16-bit tensors with b1 <= 128, b2 <= 128 run the refinement on the MFMA kernels (representatives kept in the
    tensor dtype); the same call with SFM_SW_ITER_SIMT runs the fp32 kernels.  Both against the fp32 oracle at the
    reference's 16-bit bar, and against each other."""
    H = 2
    fq, fk = frames
    q = randn((1, fq * h * w, H, D), 300, dtype)
    k, v = (randn((1, fk * h * w, H, D), 301 + i, dtype) for i in range(2))
    ref = monarch.monarch_attn(q, k, v, 1, 1, 1, h, w, num_iters=n, dtype=torch.float32)
    switches(0)
    fast = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, h, w, num_iters=n)
    switches(sfa.lib.SW_ITER_SIMT)
    slow = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, h, w, num_iters=n)
    assert_close_16bit(slow, ref, dtype)
    assert_close_16bit(fast, ref, dtype)
    assert_close_16bit(fast, slow.float(), dtype)


def test_mfma_refinement_golden_vectors_in_bf16():
    """The reference's own refinement outputs (float64 golden vectors), inputs rounded to bf16: D = 64 case of the
    fixture, num_iters 2, 3 and 8, on the MFMA kernels."""
    q, k, v, s, (B, a, f, b1, b2, H, D) = _golden_inputs(2)
    tok = lambda t: t.reshape(B, -1, H, D).to(torch.bfloat16).to(DEV)
    for n in (2, 3, 8):
        gold = torch.from_numpy(GOLD[f"case2_slow{n}"]).reshape(B, -1, H, D)
        out = mattn.monarch_attn(tok(q), tok(k), tok(v), 1, 1, 1, b1, b2, sm_scale=s, num_iters=n)
        # the golden output is that of the unrounded inputs: the input rounding alone moves it by ~1e-2
        assert max_abs(out, gold) < 4e-2
        ref = monarch.monarch_attn(tok(q).cpu(), tok(k).cpu(), tok(v).cpu(), 1, 1, 1, b1, b2, sm_scale=s, num_iters=n, dtype=torch.float32)
        assert_close_16bit(out, ref, torch.bfloat16)


@pytest.mark.parametrize("dtype,heads_per_pass", [(torch.bfloat16, 1), (torch.bfloat16, 2), (torch.float32, 1)])
def test_refinement_in_several_passes_stays_inside_its_workspace(dtype, heads_per_pass):
    """num_iters = 2 with fewer heads per pass than heads: every pass's scratch (the left factor's row statistics
    included) lies inside a workspace of exactly the queried size, and the passes give the bits of one pass."""
    h, w, H, D = 6, 20, 3, 128
    q = randn((1, 2 * h * w, H, D), 400, dtype).to(DEV)
    k, v = (randn((1, 3 * h * w, H, D), 401 + i, dtype).to(DEV) for i in range(2))
    part = monarch_fwd_exact_workspace(q, k, v, (1, 1, 1, h, w), heads_per_pass, num_iters=2)
    full = monarch_fwd_exact_workspace(q, k, v, (1, 1, 1, h, w), H, num_iters=2)
    assert torch.equal(part, full)
    ref = monarch.monarch_attn(q.cpu(), k.cpu(), v.cpu(), 1, 1, 1, h, w, num_iters=2, dtype=torch.float32)
    if dtype == torch.float32:
        assert max_abs(part, ref) < 2e-5
    else:
        assert_close_16bit(part, ref, dtype)


@pytest.mark.parametrize("ci", [0, 1, 2])
@pytest.mark.parametrize("n", [2, 3])
def test_refinement_gradients_against_the_reference_golden_gradients(ci, n):
    """dq, dk, dv of num_iters = 2, 3 under autograd (HIP forward, gradients from the torch restatement of the passes on
    the GPU) against the gradients autograd gives through the reference's own `monarch_attn_slow` for the same seeded
    cotangent (fp32 on the GPU against float64: 2e-4 of the gradient's max-abs)."""
    q, k, v, s, (B, a, f, b1, b2, H, D) = _golden_inputs(ci)
    seed = int(GOLD[f"case{ci}_meta"][0])
    cot = torch.randn(q.shape, generator=torch.Generator().manual_seed(seed + 1000), dtype=torch.float64)
    tok = lambda t: t.reshape(B, -1, H, D).float().to(DEV)
    qd, kd, vd = (tok(t).requires_grad_(True) for t in (q, k, v))
    out = mattn.monarch_attn(qd, kd, vd, 1, 1, 1, b1, b2, sm_scale=s, num_iters=n)
    assert max_abs(out, torch.from_numpy(GOLD[f"case{ci}_slow{n}"]).reshape(B, -1, H, D)) < 2e-5
    out.backward(tok(cot))
    for name, t in (("dq", qd), ("dk", kd), ("dv", vd)):
        ref = torch.from_numpy(GOLD[f"case{ci}_slow{n}_{name}"]).reshape(B, -1, H, D)
        assert max_abs(t.grad, ref) < 2e-4 * max(1.0, ref.abs().max().item()), name


@pytest.mark.parametrize("grad_only_new_kv", [False, True])
def test_refinement_gradients_through_the_cache_entry_point(grad_only_new_kv):
    """bf16, h_reduce = 2 (block order differs from token order), cache of 3 frames of which the last arrives with the
    call: gradients of q, of the new K / V (token order) and of the cache (block order) against autograd through the
    float64 oracle on the same rounded inputs; the reference's 16-bit bar."""
    h, w, H, D, n = 6, 20, 2, 64, 2
    tiling = (1, 2, 1)
    dtype = torch.bfloat16
    fr = h * w
    q = randn((1, fr, H, D), 500, dtype)
    kc, vc = randn((1, 3 * fr, H, D), 501, dtype), randn((1, 3 * fr, H, D), 502, dtype)
    nk, nv = randn((1, fr, H, D), 503, dtype), randn((1, fr, H, D), 504, dtype)
    cot = randn((1, fr, H, D), 505, dtype)
    # oracle: float64 leaves, the cache assembled from the old rows and the new chunk
    from oracle import blocks
    qo, nko, nvo = (t.double().requires_grad_(True) for t in (q, nk, nv))
    kco, vco = kc.double().requires_grad_(True), vc.double().requires_grad_(True)
    new_rows_k = blocks.to_blocks(nko, *tiling, h, w).reshape(1, -1, H, D)
    new_rows_v = blocks.to_blocks(nvo, *tiling, h, w).reshape(1, -1, H, D)
    kfull = torch.cat((kco[:, :2 * fr], new_rows_k), 1)
    vfull = torch.cat((vco[:, :2 * fr], new_rows_v), 1)
    b1, b2 = h // 2, w
    ob = monarch.monarch_iter(blocks.to_blocks(qo, *tiling, h, w), kfull.reshape(1, -1, b1, b2, H, D),
                              vfull.reshape(1, -1, b1, b2, H, D), D ** -0.5, n)
    blocks.from_blocks(ob, *tiling, h, w).backward(cot.double())
    # device
    qd, nkd, nvd = (t.to(DEV).requires_grad_(True) for t in (q, nk, nv))
    kcd, vcd = kc.to(DEV).requires_grad_(True), vc.to(DEV).requires_grad_(True)
    out = mattn.monarch_attn_with_kv_cache(qd, kcd, vcd, nkd, nvd, 2 * fr, 3 * fr, *tiling, h, w, num_iters=n,
                                           grad_only_new_kv=grad_only_new_kv)
    out.backward(cot.to(DEV))
    tol = 1e-2
    for got, ref in ((qd.grad, qo.grad), (nkd.grad, nko.grad), (nvd.grad, nvo.grad)):
        assert torch.allclose(got.float().cpu(), ref.float(), atol=tol, rtol=tol), max_abs(got, ref)
    if grad_only_new_kv:
        assert kcd.grad is None and vcd.grad is None
    else:
        for got, ref in ((kcd.grad, kco.grad), (vcd.grad, vco.grad)):
            assert torch.allclose(got[:, :2 * fr].float().cpu(), ref[:, :2 * fr].float(), atol=tol, rtol=tol)
