"""GPU parity of the streaming VAE decoder (torch convolutions on the device) against the float64 CPU
restatement, and its streaming property at a larger size."""
import pytest
import torch

import self_forcing_amd as sfa
from oracle import vae as ov

vd = sfa.vae_decode
pytestmark = pytest.mark.gpu


def _decoder(dtype, dim=96, seed=0):
    torch.manual_seed(seed)
    m = vd.WanVAEDecoder(z_dim=16, dim=dim).eval()
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith("gamma"):
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
            elif name.endswith("proj.weight"):
                p.copy_(0.05 * torch.randn_like(p))            # zero-initialised in the reference; exercised here
    return m.to("cuda", dtype)


def test_fp32_decode_matches_oracle_full_width():
    m = _decoder(torch.float32)
    g = torch.Generator().manual_seed(1)
    lat = torch.randn(1, 3, 16, 4, 6, generator=g)
    want = ov.decode_to_pixel(lat, {k: v.cpu() for k, v in m.state_dict().items()})
    got = m.decode_to_pixel(lat.cuda()).cpu().double()
    assert got.shape == want.shape == (1, 9, 3, 32, 48)
    assert want.abs().max() > 0.05                              # not saturated, not trivially zero
    torch.testing.assert_close(got, want, atol=2e-4, rtol=0)


def test_bf16_decode_matches_oracle_within_16bit_error():
    m = _decoder(torch.bfloat16, seed=2)
    g = torch.Generator().manual_seed(3)
    lat = torch.randn(1, 2, 16, 4, 6, generator=g).to(torch.bfloat16)
    want = ov.decode_to_pixel(lat.double(), {k: v.cpu() for k, v in m.state_dict().items()})
    got = m.decode_to_pixel(lat.cuda()).cpu().double()
    err = (got - want).abs()
    # ~40 bf16 convolutions and norms in sequence; pixels live in [-1, 1]
    assert err.max() < 6e-2 and err.mean() < 8e-3, (err.max().item(), err.mean().item())


def test_chunked_stream_equals_one_shot_on_the_device():
    m = _decoder(torch.bfloat16, seed=4)
    g = torch.Generator().manual_seed(5)
    lat = torch.randn(1, 6, 16, 15, 26, generator=g).to(torch.bfloat16).cuda()
    whole = m.decode_to_pixel(lat)
    assert whole.shape == (1, 21, 3, 120, 208)
    st, outs = m.new_state(), []
    for t0 in (0, 3):
        outs.append(m.decode_to_pixel(lat[:, t0:t0 + 3], use_cache=True, state=st))
    got = torch.cat(outs, 1)
    # same arithmetic, but the convolutions see other batch shapes: equal up to the library's algorithm choice
    assert (got - whole).abs().max() < 1e-1
    assert (got - whole).abs().mean() < 4e-3


def test_torch_and_hip_convolution_paths_agree(monkeypatch):
    m = _decoder(torch.bfloat16, seed=6)
    g = torch.Generator().manual_seed(7)
    lat = torch.randn(1, 3, 16, 6, 8, generator=g).to(torch.bfloat16).cuda()
    st = m.new_state()
    fast = m.decode_to_pixel(lat, use_cache=True, state=st)
    assert st.layout == "cl"
    monkeypatch.setenv("SFM_VAE_TORCH_CONV", "1")
    st2 = m.new_state()
    slow = m.decode_to_pixel(lat, use_cache=True, state=st2)
    assert st2.layout == "ncthw"
    want = ov.decode_to_pixel(lat.double().cpu(), {k: v.cpu() for k, v in m.state_dict().items()})
    e_fast, e_slow = (fast.cpu().double() - want).abs(), (slow.cpu().double() - want).abs()
    # the HIP path is held to the error of the library path (both bf16 with fp32 accumulation)
    assert e_fast.max() < 6e-2 and e_fast.mean() < 8e-3, (e_fast.max().item(), e_fast.mean().item())
    assert e_fast.mean() < 2.0 * e_slow.mean() + 1e-3


def test_fp16_decode_streams_on_the_hip_path():
    """The demo runs its decoder in fp16 (demo.py:430)."""
    m = _decoder(torch.float16, seed=8)
    g = torch.Generator().manual_seed(9)
    lat = torch.randn(1, 4, 16, 5, 7, generator=g).to(torch.float16)
    want = ov.decode_to_pixel(lat.double(), {k: v.cpu() for k, v in m.state_dict().items()})
    st, outs = m.new_state(), []
    for t0, t1 in ((0, 1), (1, 4)):
        outs.append(m.decode_to_pixel(lat[:, t0:t1].cuda(), use_cache=True, state=st))
    assert st.layout == "cl"
    got = torch.cat(outs, 1).cpu().double()
    assert got.shape == want.shape == (1, 13, 3, 40, 56)
    err = (got - want).abs()
    assert err.max() < 1.5e-2 and err.mean() < 2e-3, (err.max().item(), err.mean().item())



def _reference_fixture(dtype):
    """The decoder at dim=32 with the fixture's seeded weights, the latent, and the output of the reference's own
    `decode` (clamped as its wrapper does): tests/golden/vae_reference_vectors.npz."""
    from test_vae_reference_vectors import reference_decoder
    m, lat, want = reference_decoder()
    return m.to("cuda", dtype), lat, want


def test_fp32_decode_reproduces_the_reference_output():
    m, lat, want = _reference_fixture(torch.float32)
    got = m.decode_to_pixel(lat.float().cuda()).cpu().double()
    torch.testing.assert_close(got, want, atol=2e-4, rtol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("split", [(5,), (2, 3)])
def test_hip_convolution_path_reproduces_the_reference_output(dtype, split):
    """The channels-last 16-bit path (own convolution kernels) whole and as the reference's `cached_decode` chunks."""
    m, lat, want = _reference_fixture(dtype)
    st, outs, t0 = m.new_state(), [], 0
    for n in split:
        outs.append(m.decode_to_pixel(lat[:, t0:t0 + n].to(dtype).cuda(), use_cache=True, state=st))
        t0 += n
    assert st.layout == "cl"
    err = (torch.cat(outs, 1).cpu().double() - want).abs()
    bar = (6e-2, 8e-3) if dtype == torch.bfloat16 else (1e-2, 1.5e-3)
    assert err.max() < bar[0] and err.mean() < bar[1], (err.max().item(), err.mean().item())
