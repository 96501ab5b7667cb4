"""GPU parity of the Monarch attention kernels against the CPU oracle, through the C ABI.

Tolerances: fp32 path <= 1e-5 max-abs; 16-bit paths the reference's atol = rtol = 1e-2 (bf16) /
1e-3 (fp16) against the fp32 oracle, and max-abs < 2e-2 with per-head cosine > 0.999."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import assert_close_16bit, max_abs, monarch_fwd_exact_workspace, per_head_cosine, randn
from oracle import blocks, dense, monarch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
mattn = sfa.monarch_attn


def _tokens(F, h, w):
    return F * h * w


def test_c1_plumbing_fp32():
    """B=1, H=2, D=64, 3 frames of 8x8 tokens, q,k,v ~ N(0,1) drawn in this order from seed 0."""
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 192, 2, 64, generator=g) for _ in range(3))
    ref = monarch.monarch_attn(q, k, v, 1, 1, 1, 8, 8, sm_scale=0.125)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, 8, 8, sm_scale=0.125)
    assert max_abs(out, ref) < 1e-5
    # same case through the KV-cache entry point: cache holds frames 0-1, frame 2 arrives
    kc, vc = torch.zeros(1, 192, 2, 64, device=DEV), torch.zeros(1, 192, 2, 64, device=DEV)
    kc[:, :128], vc[:, :128] = k[:, :128].to(DEV), v[:, :128].to(DEV)
    out2 = mattn.monarch_attn_with_kv_cache(q.to(DEV), kc, vc, k[:, 128:].to(DEV), v[:, 128:].to(DEV), 128, 192,
                                            1, 1, 1, 8, 8, sm_scale=0.125)
    assert max_abs(out2, ref) < 1e-5
    assert torch.equal(kc.cpu(), k) and torch.equal(vc.cpu(), v)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,D,a,f,b1,b2", [
    (1, 1, 128, 1, 1, 2, 8),          # single wave tile, one row tile of keys
    (1, 2, 128, 3, 4, 6, 52),         # the 52-column block of the 480p grid
    (2, 2, 64, 2, 3, 5, 20),          # head_dim 64, ragged everything
    (1, 2, 128, 6, 6, 15, 52),        # reduce2xh-like: two query chunks per step-1 workgroup group
    (1, 1, 128, 2, 3, 40, 33),        # more than 32 block rows: two query-row tiles in step 2
    (1, 3, 64, 5, 2, 3, 64),          # full 64-wide key tile
    (1, 1, 128, 9, 2, 4, 32),         # 9 x 32 = 288 columns: query block-frames split across workgroups
    (1, 2, 64, 3, 4, 7, 52),          # head_dim 64 with two 32-row key tiles, five waves per group
    (1, 1, 128, 4, 3, 5, 40),         # 160 columns exactly; the second key tile is ragged (rows 40..63 masked)
    (1, 1, 64, 7, 2, 3, 24),          # one key tile, 168 columns: six waves in a single group
    (1, 1, 128, 2, 11, 3, 36),        # 33 scratch rows per (a, j): the last 32-row chunk of step 2 holds one valid row
    (1, 1, 128, 9, 1, 3, 52),         # one kv block-frame, three query chunks: consecutive tiles differ in (k, chunk) only
    (1, 2, 128, 9, 1, 2, 53),         # same with an odd column count
])
def test_mfma_path_small_shapes(dtype, B, H, D, a, f, b1, b2):
    q, k, v = (randn((B, n * b1 * b2, H, D), 10 + i, dtype) for i, n in enumerate((a, f, f)))
    ref = monarch.monarch_attn(q, k, v, 1, 1, 1, b1, b2, dtype=torch.float32)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, b1, b2)
    assert_close_16bit(out, ref, dtype)


@pytest.mark.parametrize("heads_per_pass", [1, 2, 5])
def test_head_passes_give_identical_results(heads_per_pass):
    """Passes over fewer heads give the same bits.  The one-kernel forward is the exception: the tile ranges of its
    workgroups, and with them the points where partial outputs are rounded and merged, depend on the units of a pass,
    so its passes agree to a rounding step of the output (and each with the oracle)."""
    q, k, v = (randn((1, n * 6 * 20, 5, 128), 20 + i, torch.bfloat16).to(DEV) for i, n in enumerate((2, 3, 3)))
    full = mattn.monarch_attn(q, k, v, 1, 1, 1, 6, 20, heads_per_pass=5)
    part = mattn.monarch_attn(q, k, v, 1, 1, 1, 6, 20, heads_per_pass=heads_per_pass)
    assert torch.equal(full, part)
    ref = monarch.monarch_attn(q.cpu(), k.cpu(), v.cpu(), 1, 1, 1, 6, 20, dtype=torch.float32)
    one = mattn.monarch_attn(q, k, v, 1, 1, 1, 6, 20, heads_per_pass=heads_per_pass, one_kernel=True)
    assert_close_16bit(one, ref, torch.bfloat16)
    assert max_abs(one, mattn.monarch_attn(q, k, v, 1, 1, 1, 6, 20, heads_per_pass=5, one_kernel=True)) <= 2 ** -6


@pytest.mark.parametrize("one_kernel", [False, True])
@pytest.mark.parametrize("shape,heads,heads_per_pass", [
    ((3, 3, 6, 20), 5, 3),         # last pass of 2 units: the one-kernel forward needs more slots for it than for 3
    ((3, 3, 6, 20), 5, 2),
    ((2, 4, 12, 16), 7, 4),
])
def test_shorter_last_pass_stays_inside_an_exactly_sized_workspace(one_kernel, shape, heads, heads_per_pass):
    """units % heads_per_pass != 0: the last pass is shorter.  The workspace is exactly what the query returns, with
    canary bytes behind it."""
    a, f, b1, b2 = shape
    q, k, v = (randn((1, n * b1 * b2, heads, 128), 120 + i, torch.bfloat16).to(DEV) for i, n in enumerate((a, f, f)))
    out = monarch_fwd_exact_workspace(q, k, v, (1, 1, 1, b1, b2), heads_per_pass, one_kernel=one_kernel)
    ref = monarch.monarch_attn(q.cpu(), k.cpu(), v.cpu(), 1, 1, 1, b1, b2, dtype=torch.float32)
    assert_close_16bit(out, ref, torch.bfloat16)
    if not one_kernel:
        assert torch.equal(out, mattn.monarch_attn(q, k, v, 1, 1, 1, b1, b2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,a,f,b1,b2", [
    (1, 1, 1, 1, 2, 8),            # two tiles in all
    (1, 2, 3, 4, 6, 52),           # the 52-column block of the 480p grid
    (2, 3, 2, 3, 5, 20),           # ragged everything, batch 2
    (1, 2, 6, 6, 15, 52),          # reduce2xh-like
    (1, 1, 2, 3, 32, 33),          # 32 block rows, odd column count (rows padded to 36 in LDS)
    (1, 3, 5, 2, 3, 64),           # full 64-wide key tile: 11 columns per workgroup
    (1, 1, 9, 2, 4, 32),           # 288 columns in 24 groups
    (1, 1, 2, 11, 3, 36),          # 33 tiles per unit: a left-factor pass over one parked row
    (1, 2, 1, 40, 30, 8),          # 1200 tiles per unit, 8 columns: many streams per unit, many slots to merge
    (1, 7, 3, 2, 17, 13),          # streams that cross unit boundaries
])
def test_two_kernel_and_one_kernel_forward_agree_with_the_oracle(dtype, B, H, a, f, b1, b2):
    q, k, v = (randn((B, n * b1 * b2, H, 128), 70 + i, dtype) for i, n in enumerate((a, f, f)))
    ref = monarch.monarch_attn(q, k, v, 1, 1, 1, b1, b2, dtype=torch.float32)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    one = mattn.monarch_attn(qd, kd, vd, 1, 1, 1, b1, b2, one_kernel=True)
    two = mattn.monarch_attn(qd, kd, vd, 1, 1, 1, b1, b2)
    assert_close_16bit(one, ref, dtype)
    assert_close_16bit(two, ref, dtype)


@pytest.mark.parametrize("f_tied,h_reduce,w_reduce", [(1, 1, 1), (1, 2, 1), (3, 1, 1), (1, 2, 2), (3, 3, 4), (1, 6, 13)])
def test_kv_cache_op_tilings(f_tied, h_reduce, w_reduce):
    """Every tiling: output vs oracle and the cache contents (block order) bit for bit."""
    h, w, H, D = 6, 52, 2, 128
    dtype = torch.bfloat16
    nq, nc = 3 * h * w, 9 * h * w
    q, nk, nv = (randn((1, nq, H, D), 30 + i, dtype) for i in range(3))
    kc, vc = randn((1, nc, H, D), 33, dtype), randn((1, nc, H, D), 34, dtype)
    kc_o, vc_o = kc.clone(), vc.clone()
    ref = monarch.monarch_attn_with_kv_cache(q, kc_o, vc_o, nk, nv, nc - nq, nc, f_tied, h_reduce, w_reduce, h, w,
                                             dtype=torch.float32)
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = mattn.monarch_attn_with_kv_cache(q.to(DEV), kd, vd, nk.to(DEV), nv.to(DEV), nc - nq, nc, f_tied, h_reduce,
                                           w_reduce, h, w)
    assert torch.equal(kd.cpu(), kc_o) and torch.equal(vd.cpu(), vc_o)
    assert_close_16bit(out, ref, dtype)


def test_kv_cache_view_with_batch_stride_and_prefix():
    """B=2, the op sees kv_cache[:, :local_end] of a longer allocation (batch stride = full cache)."""
    h, w, H, D = 4, 20, 2, 64
    dtype = torch.float16
    blk = h * w
    full_k, full_v = randn((2, 8 * blk, H, D), 40, dtype).to(DEV), randn((2, 8 * blk, H, D), 41, dtype).to(DEV)
    sentinel_k = full_k[:, 5 * blk:].clone()
    q, nk, nv = (randn((2, 2 * blk, H, D), 42 + i, dtype) for i in range(3))
    kc_o, vc_o = full_k[:, :5 * blk].cpu().clone(), full_v[:, :5 * blk].cpu().clone()
    ref = monarch.monarch_attn_with_kv_cache(q, kc_o, vc_o, nk, nv, 3 * blk, 5 * blk, 1, 1, 1, h, w, dtype=torch.float32)
    out = mattn.monarch_attn_with_kv_cache(q.to(DEV), full_k[:, :5 * blk], full_v[:, :5 * blk], nk.to(DEV), nv.to(DEV),
                                           3 * blk, 5 * blk, 1, 1, 1, h, w)
    assert_close_16bit(out, ref, dtype)
    assert torch.equal(full_k[:, :5 * blk].cpu(), kc_o)
    assert torch.equal(full_k[:, 5 * blk:], sentinel_k)          # nothing written past the view


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_block_causal_no_cache(dtype):
    h, w, H, D, F = 3, 20, 2, 64, 6
    q, k, v = (randn((1, F * h * w, H, D), 50 + i, dtype) for i in range(3))
    for bcs in (h * w, 3 * h * w):
        ref = monarch.monarch_attn_causal_chunked(q, k, v, 1, 1, 1, h, w, bcs, dtype=torch.float32)
        out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, h, w, block_causal_size=bcs)
        if dtype == torch.float32:
            assert max_abs(out, ref) < 1e-5
        else:
            assert_close_16bit(out, ref, dtype, atol_scale=2.0)      # the reference's causal bar is 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("a,f,b1,b2,D", [
    (2, 3, 3, 80, 128),            # 80 columns: three 32-row key tiles
    (3, 4, 45, 80, 128),           # the 720p grid (utils/resolution.py:14-27): 45 x 80 tokens per frame
    (2, 3, 67, 120, 128),          # the 1080p grid: 67 x 120, four key tiles, two query block-frames per workgroup
    (3, 2, 5, 128, 64),            # full 128-wide blocks, head_dim 64
    (1, 2, 4, 97, 128),            # odd width
    (3, 6, 90, 52, 128),           # the reference's default tiling at 480p: three frames tied, b1 = 90
])
def test_wide_and_tall_blocks_run_on_the_mfma_kernels(dtype, a, f, b1, b2, D):
    """b2 in (64, 128] (the reference's 720p / 1080p grids) and b1 > 32 (f_tied = 3) against the oracle; the fp32 path
    for the same 16-bit tensors (reached with fp32 copies) must agree as well."""
    q, k, v = (randn((1, n * b1 * b2, 2, D), 60 + i, dtype) for i, n in enumerate((a, f, f)))
    ref = monarch.monarch_attn(q, k, v, 1, 1, 1, b1, b2, dtype=torch.float32)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, b1, b2)
    assert_close_16bit(out, ref, dtype)


def test_720p_kv_cache_call_with_block_order_cache():
    """monarch_attn_with_kv_cache at 45 x 80 with h_reduce = 3 (b1 = 15, b2 = 80): cache rows bit-exact in block order."""
    h, w, H, D = 45, 80, 2, 128
    dtype = torch.bfloat16
    nq, nc = 3 * h * w, 6 * h * w
    q, nk, nv = (randn((1, nq, H, D), 130 + i, dtype) for i in range(3))
    kc, vc = randn((1, nc, H, D), 133, dtype), randn((1, nc, H, D), 134, dtype)
    kc_o, vc_o = kc.clone(), vc.clone()
    ref = monarch.monarch_attn_with_kv_cache(q, kc_o, vc_o, nk, nv, nc - nq, nc, 1, 3, 1, h, w, dtype=torch.float32)
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = mattn.monarch_attn_with_kv_cache(q.to(DEV), kd, vd, nk.to(DEV), nv.to(DEV), nc - nq, nc, 1, 3, 1, h, w)
    assert torch.equal(kd.cpu(), kc_o) and torch.equal(vd.cpu(), vc_o)
    assert_close_16bit(out, ref, dtype)


def test_generic_path_very_wide_blocks():
    """b2 = 144 is outside the MFMA kernels (b2 <= 128) and runs the fp32 generic kernels; b2 = 160 at head_dim 128 is
    past their LDS budget and is refused before anything runs."""
    q, k, v = (randn((1, n * 3 * 144, 2, 128), 60 + i, torch.bfloat16) for i, n in enumerate((2, 3, 3)))
    ref = monarch.monarch_attn(q, k, v, 1, 1, 1, 3, 144, dtype=torch.float32)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, 3, 144)
    assert_close_16bit(out, ref, torch.bfloat16)
    q, k, v = (randn((1, n * 3 * 160, 1, 128), 60 + i, torch.bfloat16).to(DEV) for i, n in enumerate((1, 1, 1)))
    with pytest.raises(sfa.lib.SfmError, match="SFM_ERR_UNSUPPORTED"):
        mattn.monarch_attn(q, k, v, 1, 1, 1, 3, 160)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B", [1, 2])
def test_reference_kv_cache_test_shape(dtype, B):
    """The reference's own harness shape (monarch_attn.py:1981-1984): A=3, F=21, 30x52, H=12, D=128, new_f=3.
    The oracle is evaluated on 3 of the 12 heads to keep the CPU side to seconds."""
    A, F, b1, b2, H, D, new_f = 3, 21, 30, 52, 12, 128, 3
    q = randn((B, A * b1 * b2, H, D), 70, dtype)
    kc, vc = randn((B, F * b1 * b2, H, D), 71, dtype), randn((B, F * b1 * b2, H, D), 72, dtype)
    nk, nv = randn((B, new_f * b1 * b2, H, D), 73, dtype), randn((B, new_f * b1 * b2, H, D), 74, dtype)
    start, end = (F - new_f) * b1 * b2, F * b1 * b2
    kd, vd = kc.to(DEV), vc.to(DEV)
    out = mattn.monarch_attn_with_kv_cache(q.to(DEV), kd, vd, nk.to(DEV), nv.to(DEV), start, end, 1, 1, 1, b1, b2,
                                           D ** -0.5)
    heads = [0, 5, 11]
    kc[:, start:end], vc[:, start:end] = nk, nv
    assert torch.equal(kd.cpu(), kc) and torch.equal(vd.cpu(), vc)
    ref = monarch.monarch_attn(q[:, :, heads], kc[:, :, heads], vc[:, :, heads], 1, 1, 1, b1, b2, dtype=torch.float32)
    assert_close_16bit(out[:, :, heads], ref, dtype)


@pytest.mark.parametrize("frames", [3, 6, 9, 12, 15, 18, 21])
def test_kv_length_sweep(frames):
    """Cache grows by one chunk per generated chunk: f in {3, ..., 21} at the 30 x 52 block."""
    b1, b2, H, D = 30, 52, 2, 128
    q = randn((1, 3 * b1 * b2, H, D), 80, torch.bfloat16)
    k, v = randn((1, frames * b1 * b2, H, D), 81, torch.bfloat16), randn((1, frames * b1 * b2, H, D), 82, torch.bfloat16)
    ref = monarch.monarch_attn(q[:, :, :1], k[:, :, :1], v[:, :, :1], 1, 1, 1, b1, b2, dtype=torch.float32)
    out = mattn.monarch_attn(q.to(DEV), k.to(DEV), v.to(DEV), 1, 1, 1, b1, b2)
    assert_close_16bit(out[:, :, :1], ref, torch.bfloat16)


def test_full_size_properties_c2():
    """Size-independent facts at the full C2 shape (H=12, 4680 queries vs 32760 keys):
    constant V gives constant output; permuting KV block-frames changes nothing (up to rounding)."""
    b1, b2, H, D = 30, 52, 12, 128
    q = randn((1, 3 * b1 * b2, H, D), 90, torch.bfloat16).to(DEV)
    k = randn((1, 21 * b1 * b2, H, D), 91, torch.bfloat16).to(DEV)
    v = randn((1, 21 * b1 * b2, H, D), 92, torch.bfloat16).to(DEV)
    const = torch.full_like(v, 1.5)
    out = mattn.monarch_attn(q, k, const, 1, 1, 1, b1, b2)
    assert (out.float() - 1.5).abs().max().item() <= 2 ** -6     # one bf16 ulp at 1.5
    base = mattn.monarch_attn(q, k, v, 1, 1, 1, b1, b2)
    perm = torch.randperm(21, generator=torch.Generator().manual_seed(1))
    kp = k.view(1, 21, b1 * b2, H, D)[:, perm].reshape(k.shape)
    vp = v.view(1, 21, b1 * b2, H, D)[:, perm].reshape(v.shape)
    other = mattn.monarch_attn(q, kp, vp, 1, 1, 1, b1, b2)
    assert max_abs(base, other) < 4e-3
    assert per_head_cosine(base, other) > 0.9999


def test_monarch_vs_dense_is_reported_not_asserted(capsys):
    """Monarch is an approximation of dense attention; the gap on random inputs is printed."""
    b1, b2, H, D = 30, 52, 2, 128
    q, k, v = (randn((1, n * b1 * b2, H, D), 95 + i, torch.bfloat16).to(DEV) for i, n in enumerate((3, 6, 6)))
    m = mattn.monarch_attn(q, k, v, 1, 1, 1, b1, b2)
    d = sfa.attention.attention(q, k, v)
    print(f"monarch vs dense: max-abs {max_abs(m, d):.3e}, per-head cosine {per_head_cosine(m, d):.4f}")


def test_host_argument_errors():
    q = randn((1, 60, 2, 64), 1, torch.bfloat16).to(DEV)
    kc = randn((1, 120, 2, 64), 2, torch.bfloat16).to(DEV)
    with pytest.raises(ValueError):
        mattn.monarch_attn_with_kv_cache(q, kc, kc.clone(), q, q, 50, 110, 1, 1, 1, 3, 20)   # start not block aligned
    with pytest.raises(ValueError):
        mattn.monarch_attn_with_kv_cache(q, kc, kc.clone(), q, q, 60, 120, 1, 1, 1, 4, 20)   # 60 tokens != k * 80
    with pytest.raises(ValueError):
        mattn.monarch_attn(q.cpu(), kc, kc, 1, 1, 1, 3, 20)
    with pytest.raises(ValueError):
        mattn.monarch_attn(q, kc, kc, 1, 1, 1, 3, 20, block_causal_size=60)                  # needs Skv == Sq


def test_wrappers_reuse_one_scratch_buffer_per_stream():
    """Steady-state calls allocate nothing: the workspace is a grow-only buffer per (device, stream); results do not
    depend on what an earlier, larger call left in it."""
    mattn = sfa.monarch_attn
    mattn.release_scratch()
    h, w, H, D = 6, 20, 2, 128
    q1, k1, v1 = (randn((1, n * h * w, H, D), 400 + i, torch.bfloat16).to(DEV) for i, n in enumerate((1, 3, 3)))
    q2, k2, v2 = (randn((1, n * h * w, H, D), 410 + i, torch.bfloat16).to(DEV) for i, n in enumerate((2, 5, 5)))
    small_first = mattn.monarch_attn(q1, k1, v1, 1, 1, 1, h, w)
    key = (0, torch.cuda.current_stream().cuda_stream)
    n_small = mattn._SCRATCH[key].numel()
    mattn.monarch_attn(q2, k2, v2, 1, 1, 1, h, w)
    buf = mattn._SCRATCH[key]
    assert buf.numel() > n_small
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    small_again = mattn.monarch_attn(q1, k1, v1, 1, 1, 1, h, w)
    assert mattn._SCRATCH[key] is buf                                   # no new workspace
    assert torch.cuda.memory_stats()["allocation.all.allocated"] - before == 1      # the output tensor only
    assert torch.equal(small_again, small_first)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        other = mattn.monarch_attn(q1, k1, v1, 1, 1, 1, h, w)
    side.synchronize()
    assert (0, side.cuda_stream) in mattn._SCRATCH and torch.equal(other, small_first)
    mattn.release_scratch()
    assert not mattn._SCRATCH
