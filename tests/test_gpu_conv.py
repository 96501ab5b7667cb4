"""GPU parity of the channels-last convolution kernel (`sfm_conv3d_cl` through conv_ops.conv_cl) against torch's
fp32 convolution of the same 16-bit operands: the shapes of the streaming VAE decoder (causal 3x3x3 with and
without history, the (3,1,1) temporal convolution, the 3x3 convolution behind the nearest x2 upsampling, the
16-channel input and the 3-channel head), ragged tile edges, both 16-bit types."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from self_forcing_amd import conv_ops as co

pytestmark = pytest.mark.gpu

CASES = [
    # cin, cout, kt, k, T, H, W, up2x, history frames, dtype
    (96, 96, 3, 3, 2, 5, 7, False, 2, torch.bfloat16),
    (192, 192, 3, 3, 3, 6, 10, False, 1, torch.bfloat16),
    (192, 384, 3, 3, 1, 4, 9, False, 0, torch.bfloat16),
    (384, 768, 3, 1, 2, 5, 6, False, 2, torch.bfloat16),
    (16, 384, 3, 3, 1, 6, 8, False, 0, torch.bfloat16),
    (96, 3, 3, 3, 4, 9, 13, False, 2, torch.bfloat16),
    (384, 192, 1, 3, 2, 5, 6, True, 0, torch.bfloat16),
    (192, 96, 1, 3, 3, 4, 7, True, 0, torch.bfloat16),
    (96, 96, 3, 3, 3, 33, 41, False, 2, torch.float16),
    (64, 64, 3, 3, 1, 1, 1, False, 0, torch.float16),
    (96, 96, 3, 3, 2, 16, 16, False, 2, torch.bfloat16),          # 512 voxels: exactly two workgroup tiles
]


@pytest.mark.parametrize("cin,cout,kt,k,T,H,W,up2x,hist,dt", CASES)
def test_conv_cl_matches_fp32_convolution(cin, cout, kt, k, T, H, W, up2x, hist, dt):
    torch.manual_seed(cin * 7 + cout + T)
    conv = (nn.Conv2d(cin, cout, 3, padding=1) if kt == 1 else nn.Conv3d(cin, cout, (kt, k, k))).cuda().to(dt)
    x = torch.randn(T, H, W, cin, device="cuda").to(dt)
    h = torch.randn(hist, H, W, cin, device="cuda").to(dt) if hist else None
    y = co.conv_cl(x, conv, h, up2x)
    wf, bf = conv.weight.float(), conv.bias.float()
    if kt == 1:
        z = x.float().permute(0, 3, 1, 2)
        if up2x:
            z = F.interpolate(z, scale_factor=2.0, mode="nearest")
        ref = F.conv2d(z, wf, bf, padding=1).permute(0, 2, 3, 1)
    else:
        xf = x.float().permute(3, 0, 1, 2).unsqueeze(0)
        if h is not None:
            xf = torch.cat([h.float().permute(3, 0, 1, 2).unsqueeze(0), xf], 2)
        xf = F.pad(xf, (k // 2, k // 2, k // 2, k // 2, (kt - 1) - (xf.shape[2] - T), 0))
        ref = F.conv3d(xf, wf, bf)[0].permute(1, 2, 3, 0)
    assert y.shape == ref.shape
    # fp32 accumulation of 16-bit products, one rounding of the result
    tol = (2.0 ** -8 if dt == torch.bfloat16 else 2.0 ** -11) * max(1.0, ref.abs().max().item()) * 1.01
    assert (y.float() - ref).abs().max().item() <= tol


def test_conv_cl_rejects_bad_arguments():
    import ctypes as C
    from self_forcing_amd import lib as L
    lib = L.load()
    d = L.ConvDesc()
    d.dtype, d.T, d.H, d.W, d.Cin, d.Cout, d.Cout_pad, d.kt, d.kh, d.kw = L.SFM_BF16, 1, 4, 4, 48, 32, 32, 3, 3, 3
    buf = torch.zeros(1 << 16, dtype=torch.bfloat16, device="cuda")
    for i in range(3):
        d.x_stride[i] = d.y_stride[i] = 64
    assert lib.sfm_conv3d_cl(C.byref(d), buf.data_ptr(), buf.data_ptr(), None, None, buf.data_ptr(), None) == -3      # Cin % 32
    d.Cin = 64
    d.x_stride[2] = 60
    assert lib.sfm_conv3d_cl(C.byref(d), buf.data_ptr(), buf.data_ptr(), None, None, buf.data_ptr(), None) == -5      # stride
    d.x_stride[2] = 64
    assert lib.sfm_conv3d_cl(C.byref(d), None, buf.data_ptr(), None, None, buf.data_ptr(), None) == -1


@pytest.mark.parametrize("cout", [96, 3])
def test_conv_cl_adds_the_residual_input(cout):
    torch.manual_seed(cout)
    conv = nn.Conv3d(96, cout, 3).cuda().to(torch.bfloat16)
    x = torch.randn(2, 6, 9, 96, device="cuda").to(torch.bfloat16)
    res = torch.randn(2, 6, 9, cout, device="cuda").to(torch.bfloat16)
    y = co.conv_cl(x, conv, None, res=res)
    xf = F.pad(x.float().permute(3, 0, 1, 2).unsqueeze(0), (1, 1, 1, 1, 2, 0))
    ref = F.conv3d(xf, conv.weight.float(), conv.bias.float())[0].permute(1, 2, 3, 0) + res.float()
    assert (y.float() - ref).abs().max().item() <= 2.0 ** -8 * max(1.0, ref.abs().max().item()) * 1.01


@pytest.mark.parametrize("C_,act,dt", [(96, True, torch.bfloat16), (192, True, torch.bfloat16), (384, False, torch.bfloat16),
                                      (384, True, torch.float16), (32, False, torch.float16)])
def test_norm_act_matches_fp32(C_, act, dt):
    torch.manual_seed(C_)
    x = torch.randn(3, 5, 7, C_, device="cuda").to(dt)
    x[0, 0, 0] = 0                                                     # an all-zero voxel stays zero (clamped norm)
    gamma = (1.0 + 0.3 * torch.randn(C_, 1, 1, 1, device="cuda")).to(dt)
    big = torch.zeros(5, 7, 9, C_ + 32, device="cuda", dtype=dt)
    out = big[2:, 1:6, 1:8, :C_]                                       # a strided view, like a padded conv input
    co.norm_act(x, gamma, act, out=out)
    xf = x.float()
    ref = F.normalize(xf, dim=-1) * C_ ** 0.5 * gamma.float().view(-1)
    if act:
        ref = F.silu(ref)
    tol = (2.0 ** -8 if dt == torch.bfloat16 else 2.0 ** -11) * max(1.0, ref.abs().max().item()) * 1.01
    assert (out.float() - ref).abs().max().item() <= tol
    assert big[:2].abs().max() == 0 and big[:, 0].abs().max() == 0 and big[..., C_:].abs().max() == 0   # nothing outside the view


def test_conv_cl_reuses_its_padded_input_buffer_without_stale_values():
    """Calls of one padded shape share one zero-bordered buffer that is filled once.  A call without history after a
    call with history (a new stream after an old one), and a call with fewer real input channels in the same padded
    shape, must not see what the earlier call left there: each result equals the one from a fresh buffer, bit for bit."""
    torch.manual_seed(3)
    conv = nn.Conv3d(96, 96, 3).cuda().to(torch.bfloat16)
    conv16 = nn.Conv3d(80, 96, 3).cuda().to(torch.bfloat16)           # 80 real channels in the same 96-channel padded shape
    x = torch.randn(2, 9, 11, 96, device="cuda").to(torch.bfloat16)
    h = torch.randn(2, 9, 11, 96, device="cuda").to(torch.bfloat16)
    co.release_padded()
    fresh_none = co.conv_cl(x, conv, None)
    co.release_padded()
    fresh_one = co.conv_cl(x, conv, h[:1])
    co.release_padded()
    fresh_16 = co.conv_cl(x[..., :80].contiguous(), conv16, None)
    co.release_padded()
    with_h, tail = co.conv_cl(x, conv, h, want_tail=True)
    assert torch.equal(tail, x)                                        # the last two frames of (history + input)
    assert len(co._PADDED) == 1
    assert torch.equal(co.conv_cl(x, conv, h[:1]), fresh_one)          # one history frame: the other one is zero again
    assert torch.equal(co.conv_cl(x, conv, None), fresh_none)
    assert torch.equal(co.conv_cl(x[..., :80].contiguous(), conv16, None), fresh_16)
    assert len(co._PADDED) == 2                                        # fewer real channels: a buffer of its own
    assert not torch.equal(with_h, fresh_none)


def test_strided_padded_input_takes_the_general_kernel_with_the_same_result():
    """The 3x3 kernels run on a contiguous padded input as one run of rows per kernel row; a padded input that is a
    view into a wider buffer goes through the general kernel.  Same convolution: the two agree to the rounding of the
    result (the taps are summed in a different order)."""
    import ctypes as C
    from self_forcing_amd import lib as L
    torch.manual_seed(5)
    T, H, W, c = 3, 10, 13, 96
    conv = nn.Conv3d(c, c, 3).cuda().to(torch.bfloat16)
    x = torch.randn(T, H, W, c, device="cuda").to(torch.bfloat16)
    h = torch.randn(2, H, W, c, device="cuda").to(torch.bfloat16)
    want = co.conv_cl(x, conv, h)
    wt, bias, kt, k, cout, cin, cin_p, cout_p = co.prepared(conv, x.dtype, x.device)
    wide = torch.zeros(T + 2, H + 2, W + 6, c, device="cuda", dtype=torch.bfloat16)
    xp = wide[:, :, 2:2 + W + 2]                                   # the padded input, rows W + 6 columns apart
    xp[:2, 1:1 + H, 1:1 + W] = h
    xp[2:, 1:1 + H, 1:1 + W] = x
    y = torch.empty(T, H, W, c, device="cuda", dtype=torch.bfloat16)
    d = L.ConvDesc()
    d.dtype, d.T, d.H, d.W, d.Cin, d.Cout, d.Cout_pad, d.kt, d.kh, d.kw, d.up2x = L.SFM_BF16, T, H, W, c, c, cout_p, 3, 3, 3, 0
    for i in range(3):
        d.x_stride[i], d.y_stride[i] = xp.stride(i), y.stride(i)
    L.check(L.load().sfm_conv3d_cl(C.byref(d), xp.data_ptr(), wt.data_ptr(), bias.data_ptr(), None, y.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert (y.float() - want.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, want.float().abs().max().item())
    assert not torch.equal(y, torch.zeros_like(y))


@pytest.mark.parametrize("cin,cout,T,H,W", [(96, 96, 12, 480, 832), (192, 192, 12, 240, 416), (96, 3, 12, 480, 832)])
def test_conv_cl_at_the_decoders_full_sizes(cin, cout, T, H, W):
    """The decoder's largest convolutions (1.1 GB of padded input, 18 840 voxel tiles over the 8 XCDs, the 3-channel
    head) against torch's fp32 convolution of the same bf16 operands, every output element."""
    torch.manual_seed(cin + cout)
    conv = nn.Conv3d(cin, cout, 3).cuda().to(torch.bfloat16)
    x = torch.randn(T, H, W, cin, device="cuda").to(torch.bfloat16)
    h = torch.randn(2, H, W, cin, device="cuda").to(torch.bfloat16)
    y = co.conv_cl(x, conv, h)
    xf = torch.cat([h, x]).float().permute(3, 0, 1, 2).unsqueeze(0)
    ref = F.conv3d(F.pad(xf, (1, 1, 1, 1, 0, 0)), conv.weight.float(), conv.bias.float())[0].permute(1, 2, 3, 0)
    del xf
    assert y.shape == ref.shape
    tol = 2.0 ** -8 * max(1.0, ref.abs().max().item()) * 1.01
    worst = 0.0
    for t in range(T):                                  # frame by frame: no second full-size fp32 temporary
        worst = max(worst, (y[t].float() - ref[t]).abs().max().item())
    assert worst <= tol
    co.release_padded()
