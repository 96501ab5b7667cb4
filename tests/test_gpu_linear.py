"""GPU parity of the block's fused linear layers (`sfm_linear`) against fp32 `torch.matmul` followed by the eager
chain's rounding points (nn.Linear output rounded, GELU of it rounded; gated product rounded, residual sum rounded:
wan/modules/model.py:648-650, wan/modules/causal_model.py:1189-1204)."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
lin = sfa.linear


def _ref(x, w, b, dtype, epilogue, res=None, gate=None, rpf=1):
    y = x.float() @ w.float().t()
    if b is not None:
        y = y + b.float()
    y = y.to(dtype)
    if epilogue == "gelu_tanh":
        return torch.nn.functional.gelu(y.float(), approximate="tanh").to(dtype)
    if epilogue == "gate_residual":
        if gate is not None:
            g = gate.reshape(x.shape[0], -1, 1, w.shape[0]).float()
            y = (y.float().unflatten(1, (g.shape[1], rpf)) * g).flatten(1, 2).to(dtype)
        return (res.float() + y.float()).to(dtype)
    return y


def _assert_rounding_close(got, ref, dtype, frac=1e-2, steps=1, scale=None):
    """Equal up to the accumulation order of the fp32 sums: at most `steps` rounding steps of the result (one per
    rounding that follows the product), on a small fraction of the elements.  `scale`: the magnitude the steps are
    measured at where it is not the result's own (a sum of two rounded terms)."""
    got, ref = got.float(), ref.float()
    unit = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)          # largest relative spacing of the format
    err = (got - ref).abs()
    mag = (ref.abs() if scale is None else scale.float()).clamp_min(2.0 ** -6)
    assert (err <= steps * unit * mag).all(), (err.max().item(), (err / mag).max().item())
    assert (err > 0).sum().item() <= max(frac * err.numel(), 2), (err > 0).float().mean().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tile_rows", [0, 128, 256])
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (300, 264, 128), (1, 8, 64), (517, 1000, 192), (130, 520, 256), (640, 304, 320),
                                   (4680, 1536, 1536)])
def test_plain_linear(dtype, tile_rows, M, N, K):
    """K from one to 24 stages of 64 (the first, second-to-last and last stages of the load ring are separate code);
    both tile heights, and the library's own choice."""
    x, w, b = randn((1, M, K), 1, dtype).to(DEV), (randn((N, K), 2, dtype) * K ** -0.5).to(dtype).to(DEV), randn((N,), 3, dtype).to(DEV)
    out = lin.linear(x, w, b, tile_rows=tile_rows)
    _assert_rounding_close(out, _ref(x, w, b, dtype, "none"), dtype)
    out = lin.linear(x, w, None, tile_rows=tile_rows)
    _assert_rounding_close(out, _ref(x, w, None, dtype, "none"), dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_strided_rows_and_batches(dtype):
    """x as a column slice of a wider tensor (the fused q/k/v projection's output layout), two batch entries."""
    B, L, K, N = 2, 333, 128, 136
    wide = randn((B, L, 3 * K), 4, dtype).to(DEV)
    x = wide[..., K:2 * K]
    w, b = (randn((N, K), 5, dtype) * K ** -0.5).to(dtype).to(DEV), randn((N,), 6, dtype).to(DEV)
    out_wide = torch.zeros(B, L, 2 * N, dtype=dtype, device=DEV)
    out = lin.linear(x, w, b, out=out_wide[..., N:])
    assert out.data_ptr() == out_wide[..., N:].data_ptr() and not out_wide[..., :N].any()
    _assert_rounding_close(out, _ref(x, w, b, dtype, "none"), dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tile_rows", [128, 256])
@pytest.mark.parametrize("M,N,K", [(300, 264, 128), (4680, 8960, 1536)])
def test_gelu_tanh_epilogue(dtype, tile_rows, M, N, K):
    x, w, b = randn((1, M, K), 7, dtype).to(DEV), (randn((N, K), 8, dtype) * K ** -0.5).to(dtype).to(DEV), randn((N,), 9, dtype).to(DEV)
    out = lin.linear(x, w, b, epilogue="gelu_tanh", tile_rows=tile_rows)
    # a product that lands one rounding step away moves the result by |gelu'(y)| steps of y: in the left tail, where
    # the result itself is tiny, that is many steps of the result, so the steps are measured at |gelu(y)| + |y gelu'(y)|
    y = _ref(x, w, b, dtype, "none").float().requires_grad_(True)
    g = torch.nn.functional.gelu(y, approximate="tanh")
    g.sum().backward()
    mag = g.detach().abs() + (y.detach() * y.grad).abs()
    _assert_rounding_close(out, _ref(x, w, b, dtype, "gelu_tanh"), dtype, frac=3e-2, steps=2, scale=mag)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,F,rpf,N,K,gated", [(1, 3, 100, 264, 128, True), (2, 2, 60, 136, 192, True), (1, 3, 1560, 1536, 8960, True),
                                               (1, 1, 300, 264, 128, False)])
@pytest.mark.parametrize("tile_rows", [128, 256])
def test_gate_residual_epilogue(dtype, tile_rows, B, F, rpf, N, K, gated):
    L = F * rpf
    x, w, b = randn((B, L, K), 10, dtype).to(DEV), (randn((N, K), 11, dtype) * K ** -0.5).to(dtype).to(DEV), randn((N,), 12, dtype).to(DEV)
    res = randn((B, L, N), 13, dtype).to(DEV)
    gate = randn((B, F, 1, N), 14, dtype).to(DEV) if gated else None
    ref = _ref(x, w, b, dtype, "gate_residual", res, gate, rpf)
    mag = res.float().abs() + (ref.float() - res.float()).abs()        # |res| + |gated product|
    keep = res.clone()
    out = lin.linear(x, w, b, epilogue="gate_residual", res=res, gate=gate, tile_rows=tile_rows)
    assert out.data_ptr() == res.data_ptr()                     # in place, like `x = x + y * e`
    _assert_rounding_close(out, ref, dtype, frac=2e-2, steps=3, scale=mag)
    out2 = torch.empty_like(keep)
    lin.linear(x, w, b, epilogue="gate_residual", res=keep, gate=gate, out=out2, tile_rows=tile_rows)
    assert torch.equal(out2, out)


def test_the_fused_tail_equals_the_separate_kernels():
    """Same product, then the library's own gated-residual kernel: bit for bit what the epilogue writes."""
    dtype = torch.bfloat16
    B, F, rpf, N, K = 1, 3, 200, 520, 256
    x, w, b = randn((B, F * rpf, K), 20, dtype).to(DEV), (randn((N, K), 21, dtype) * K ** -0.5).to(dtype).to(DEV), randn((N,), 22, dtype).to(DEV)
    res, gate = randn((B, F * rpf, N), 23, dtype).to(DEV), randn((B, F, 1, N), 24, dtype).to(DEV)
    y = lin.linear(x, w, b)
    want = sfa.block_ops.gate_residual_(res.clone(), y, gate)
    got = lin.linear(x, w, b, epilogue="gate_residual", res=res.clone(), gate=gate)
    assert torch.equal(got, want)


def test_argument_errors():
    x, w = randn((1, 64, 64), 30, torch.bfloat16).to(DEV), randn((8, 64), 31, torch.bfloat16).to(DEV)
    with pytest.raises(ValueError):
        lin.linear(x.float(), w.float())
    with pytest.raises(ValueError):
        lin.linear(x, w.half())
    with pytest.raises(ValueError):
        lin.linear(x[..., :32], w[:, :32])                       # K not a multiple of 64
    with pytest.raises(ValueError):
        lin.linear(x, w, epilogue="gate_residual")               # no res
    with pytest.raises(ValueError):
        lin.linear(x, w, epilogue="relu")
    assert not lin.supported(x.float(), w.float()) and lin.supported(x, w)


def test_block_ffn_on_the_own_kernel_matches_the_library_path():
    """HipAttentionOps(own_gemm=True): the FFN half of the block (Linear + GELU, Linear + gated residual) on the own
    kernel against the default path (hipBLASLt with its GELU epilogue + the gated-residual kernel)."""
    cm = sfa.causal_model
    dtype = torch.bfloat16
    dim, ffn, F, rpf = 256, 640, 3, 120
    torch.manual_seed(3)
    up, down = torch.nn.Linear(dim, ffn), torch.nn.Linear(ffn, dim)
    torch.nn.init.normal_(up.bias, std=0.1)
    torch.nn.init.normal_(down.bias, std=0.1)
    up, down = up.to(DEV, dtype), down.to(DEV, dtype)
    x, xn = randn((1, F * rpf, dim), 40, dtype).to(DEV), randn((1, F * rpf, dim), 41, dtype).to(DEV)
    gate = randn((1, F, 1, dim), 42, dtype).to(DEV)
    with torch.no_grad():
        lib_ops, own_ops = cm.HipAttentionOps(), cm.HipAttentionOps(own_gemm=True)
        want = lib_ops.linear_gate_residual(x.clone(), lib_ops.linear_gelu(xn, up), down, gate)
        h = own_ops.linear_gelu(xn, up)
        got = own_ops.linear_gate_residual(x.clone(), h, down, gate)
    # hipBLASLt applies GELU to the unrounded product, the own kernel to the rounded one as the eager chain does
    assert (h.float() - lib_ops.linear_gelu(xn, up).float()).abs().max() <= 2.0 ** -6
    err = (got.float() - want.float()).abs()
    assert err.max() <= 2.0 ** -4 and err.mean() < 2e-3, (err.max().item(), err.mean().item())


def test_square_projection_on_the_own_kernel_matches_the_library():
    """HipAttentionOps(own_gemm="auto").linear: N, K <= 2048 run on sfm_linear, wider layers and the default stay on
    the library; same values up to the fp32 summation order."""
    cm = sfa.causal_model
    dtype = torch.bfloat16
    torch.manual_seed(5)
    sq, wide = torch.nn.Linear(512, 512).to(DEV, dtype), torch.nn.Linear(512, 2304).to(DEV, dtype)
    x = randn((1, 700, 512), 50, dtype).to(DEV)
    with torch.no_grad():
        auto, none = cm.HipAttentionOps(own_gemm="auto"), cm.HipAttentionOps()
        assert none.linear(x, wide).data_ptr() != 0 and not none.own_square and auto.own_square and not auto.own_gemm
        _assert_rounding_close(auto.linear(x, sq), sq(x), dtype)
        assert torch.equal(auto.linear(x, wide), wide(x))           # too wide for "auto": the library runs it
        assert torch.equal(none.linear(x, sq), sq(x))
