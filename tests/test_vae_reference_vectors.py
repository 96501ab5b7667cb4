"""The reference's own VAE decode output (tests/golden/vae_reference_vectors.npz: `WanVAE_.decode` and
`.cached_decode` of wan/modules/vae.py:548-596 at dim=32 on weights seeded by name, written by
tests/golden/make_vae_reference_vectors.py) against oracle/vae.py and against the product module on the CPU.
Only the fixture is read here: the weights are regenerated from the seed and checked against the stored
per-parameter checksums."""
import os
import sys

import numpy as np
import pytest
import torch

import self_forcing_amd as sfa
from oracle import vae as ov

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import vae_fixture as fx  # noqa: E402

vd = sfa.vae_decode
FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vae_reference_vectors.npz")


def load_fixture():
    """-> (weights by reference state-dict name, latent [B,T,C,h,w], decode output [B,T',3,H,W] before the clamp,
    cached_decode output in chunks of 2 + 3 latent frames)."""
    z = np.load(FIX, allow_pickle=False)
    assert int(z["seed"]) == fx.SEED and int(z["dim"]) == fx.DIM
    shapes = {str(n): tuple(int(v) for v in str(s).split(",")) for n, s in zip(z["names"], z["shapes"])}
    W = fx.weights_for(shapes)
    for n, want in zip(z["names"], z["checksums"]):
        w = W[str(n)]
        got = float((w * torch.arange(1, w.numel() + 1, dtype=torch.float64).view(w.shape).remainder(7).add(1)).sum())
        assert abs(got - float(want)) <= 1e-9 * max(1.0, abs(float(want))), n
    to_btchw = lambda a: torch.from_numpy(a).permute(0, 2, 1, 3, 4).contiguous()
    return W, fx.latent(), to_btchw(z["decode"]), to_btchw(z["cached_decode_2_3"])


def test_fixture_is_the_reference_layout_at_dim_32():
    W, lat, whole, chunks = load_fixture()
    assert whole.shape == (1, 17, 3, 24, 32) and torch.equal(whole, chunks)
    assert W["decoder.conv1.weight"].shape == (128, 16, 3, 3, 3) and W["decoder.head.2.weight"].shape == (3, 32, 3, 3, 3)
    assert (whole.abs() > 1).double().mean() > 0.05                        # the clamp is exercised too


def test_oracle_reproduces_the_reference_decode():
    W, lat, whole, _ = load_fixture()
    got = ov.decode_frames(lat, W)
    # the reference upsamples through fp32 (vae.py:57-63: exact for a nearest-neighbour copy of values that were
    # rounded to fp32 on the way, which is the only fp32 step of a float64 run)
    torch.testing.assert_close(got, whole, atol=2e-6, rtol=0)
    torch.testing.assert_close(ov.decode_to_pixel(lat, W), whole.clamp(-1, 1), atol=2e-6, rtol=0)


@pytest.mark.parametrize("split", [(2, 3), (1, 1, 1, 1, 1), (4, 1)])
def test_oracle_stream_reproduces_the_reference_cached_decode(split):
    W, lat, _, chunks = load_fixture()
    st, outs, t0 = ov.Stream(), [], 0
    for n in split:
        outs.append(ov.decode_frames(lat[:, t0:t0 + n], W, st))
        t0 += n
    torch.testing.assert_close(torch.cat(outs, 1), chunks, atol=2e-6, rtol=0)


def reference_decoder(dtype=torch.float64):
    W, lat, whole, chunks = load_fixture()
    m = vd.WanVAEDecoder(z_dim=16, dim=fx.DIM).double().eval()
    assert set(m.state_dict()) == set(W)                                   # same names as the reference's conv2 / decoder
    m.load_reference_state_dict(W)
    return m.to(dtype), lat, whole.clamp(-1, 1)


def test_module_reproduces_the_reference_decode_on_the_cpu():
    m, lat, want = reference_decoder()
    torch.testing.assert_close(m.decode_to_pixel(lat).double(), want, atol=5e-6, rtol=0)
    for split in ((2, 3), (1, 4), (3, 1, 1)):
        st, outs, t0 = m.new_state(), [], 0
        for n in split:
            outs.append(m.decode_to_pixel(lat[:, t0:t0 + n], use_cache=True, state=st))
            t0 += n
        torch.testing.assert_close(torch.cat(outs, 1).double(), want, atol=5e-6, rtol=0)


def test_a_wrong_block_order_or_a_dropped_cache_would_show():
    """Sensitivity of the pin: swapping two residual blocks' weights, or restarting the stream in the middle, moves
    the output by far more than the tolerance."""
    W, lat, whole, _ = load_fixture()
    W2 = dict(W)
    for k in list(W):
        if k.startswith("decoder.upsamples.0."):
            W2[k] = W[k.replace("upsamples.0.", "upsamples.1.")]
    assert (ov.decode_frames(lat, W2) - whole).abs().max() > 1e-2
    restarted = torch.cat([ov.decode_frames(lat[:, :2], W), ov.decode_frames(lat[:, 2:], W)], 1)
    assert restarted.shape != whole.shape or (restarted - whole).abs().max() > 1e-2
