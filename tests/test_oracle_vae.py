"""Pins of the streaming VAE decode restatement (oracle/vae.py) and, on the CPU, of the product module
(self-forcing_amd/vae_decode.py) against it.  Nothing of the reference is imported; its checkpoint is not
available offline, so the composition of the pieces is compared between two independently written
implementations and each piece is pinned against brute force, a library routine or an invariant."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import self_forcing_amd as sfa
from oracle import vae as ov

vd = sfa.vae_decode
F64 = torch.float64


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=F64) * scale


def test_causal_conv_matches_a_triple_loop():
    x, w, b = _rand(1, 2, 4, 3, 3, seed=1), _rand(3, 2, 3, 3, 3, seed=2), _rand(3, seed=3)
    y = ov.causal_conv3d(x, w, b)
    assert y.shape == (1, 3, 4, 3, 3)
    ref = np.zeros((3, 4, 3, 3))
    xn, wn = x[0].numpy(), w.numpy()
    for o in range(3):
        for t in range(4):
            for i in range(3):
                for j in range(3):
                    acc = b[o].item()
                    for c in range(2):
                        for dt in range(3):
                            tt = t + dt - 2                      # taps reach two frames into the past, none ahead
                            for di in range(3):
                                for dj in range(3):
                                    ii, jj = i + di - 1, j + dj - 1
                                    if tt >= 0 and 0 <= ii < 3 and 0 <= jj < 3:
                                        acc += wn[o, c, dt, di, dj] * xn[c, tt, ii, jj]
                    ref[o, t, i, j] = acc
    np.testing.assert_allclose(y[0].numpy(), ref, atol=1e-12)


def test_cached_frames_equal_one_convolution_over_the_clip():
    x, w, b = _rand(1, 3, 7, 4, 5, seed=4), _rand(5, 3, 3, 3, 3, seed=5), _rand(5, seed=6)
    W = {"c.weight": w, "c.bias": b}
    whole = ov.causal_conv3d(x, w, b)
    for split in ([1] * 7, [1, 3, 3], [2, 1, 4]):
        st, outs, t0 = ov.Stream(), [], 0
        for n in split:
            outs.append(ov._cached_conv(x[:, :, t0:t0 + n], W, "c", st))
            t0 += n
        torch.testing.assert_close(torch.cat(outs, 2), whole, atol=1e-12, rtol=0)


def test_rms_norm_is_the_library_normalisation_with_unit_rms():
    x, g = _rand(2, 6, 3, 4, 5, seed=7), _rand(6, seed=8)
    y = ov.rms_norm(x, g)
    torch.testing.assert_close(y, F.normalize(x, dim=1) * 6 ** 0.5 * g.view(1, 6, 1, 1, 1), atol=1e-12, rtol=0)
    y1 = ov.rms_norm(x, torch.ones(6, dtype=F64))
    torch.testing.assert_close(y1.pow(2).mean(dim=1), torch.ones(2, 3, 4, 5, dtype=F64), atol=1e-12, rtol=0)


def test_attention_block_is_single_head_attention_per_frame():
    c = 4
    x = _rand(1, c, 2, 3, 3, seed=9)
    W = {"a.norm.gamma": torch.ones(c, 1, 1, dtype=F64), "a.to_qkv.weight": _rand(3 * c, c, 1, 1, seed=10),
         "a.to_qkv.bias": _rand(3 * c, seed=11), "a.proj.weight": _rand(c, c, 1, 1, seed=12), "a.proj.bias": _rand(c, seed=13)}
    y = ov.attention_block(x, W, "a")
    for t in range(2):                                           # frames do not see each other
        xt = x[:, :, t]
        n = F.normalize(xt, dim=1) * c ** 0.5
        qkv = F.conv2d(n, W["a.to_qkv.weight"], W["a.to_qkv.bias"]).reshape(1, 3, c, 9).transpose(2, 3)
        o = F.scaled_dot_product_attention(qkv[:, 0:1], qkv[:, 1:2], qkv[:, 2:3])[:, 0]
        o = F.conv2d(o.transpose(1, 2).reshape(1, c, 3, 3), W["a.proj.weight"], W["a.proj.bias"])
        torch.testing.assert_close(y[:, :, t], xt + o, atol=1e-10, rtol=0)


def test_temporal_upsampling_order_and_first_frame():
    """time_conv's first c output channels are the even output frames, the last c the odd ones; the first frame of a
    stream is not doubled and is not part of the second frame's history."""
    c = 2
    w = torch.zeros(2 * c, c, 3, 1, 1, dtype=F64)
    for ch in range(c):
        w[ch, ch, 2] = 1.0               # even frame = current input frame
        w[c + ch, ch, 1] = 10.0          # odd frame = 10 x previous input frame
    W = {"u.time_conv.weight": w, "u.time_conv.bias": torch.zeros(2 * c, dtype=F64),
         "u.resample.1.weight": torch.zeros(c // 2, c, 3, 3, dtype=F64), "u.resample.1.bias": torch.zeros(c // 2, dtype=F64)}
    W["u.resample.1.weight"][0, 0, 1, 1] = 1.0                   # pass channel 0 through
    st = ov.Stream()
    x = torch.arange(1, 4, dtype=F64).view(1, 1, 3, 1, 1).expand(1, c, 3, 2, 2).contiguous()     # frames valued 1, 2, 3
    y0 = ov.upsample(x[:, :, :1], W, "u", st, temporal=True)
    assert y0.shape == (1, 1, 1, 4, 4) and torch.all(y0 == 1.0)
    y1 = ov.upsample(x[:, :, 1:2], W, "u", st, temporal=True)
    assert y1.shape == (1, 1, 2, 4, 4)
    assert torch.all(y1[:, :, 0] == 2.0) and torch.all(y1[:, :, 1] == 0.0)      # history of frame 2 is zeros, not frame 1
    y2 = ov.upsample(x[:, :, 2:3], W, "u", st, temporal=True)
    assert torch.all(y2[:, :, 0] == 3.0) and torch.all(y2[:, :, 1] == 20.0)


def _tiny_decoder(seed=0, dim=8):
    torch.manual_seed(seed)
    m = vd.WanVAEDecoder(z_dim=16, dim=dim).double().eval()
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith("gamma"):
                p.copy_(1.0 + 0.2 * torch.randn_like(p))
            else:
                p.copy_(0.25 * torch.randn_like(p))
    return m


def test_module_matches_oracle_and_streams():
    m = _tiny_decoder()
    lat = _rand(1, 5, 16, 4, 6, seed=20)
    want = ov.decode_to_pixel(lat, m.state_dict())
    assert want.shape == (1, 1 + 4 * 4, 3, 32, 48)
    got = m.decode_to_pixel(lat)
    # the module upsamples in fp32 as the reference does (vae.py:57-63); everything else here is float64
    torch.testing.assert_close(got.double(), want, atol=5e-6, rtol=0)
    for split in ([1, 1, 1, 1, 1], [3, 2], [1, 4], [2, 3]):
        st, outs, t0 = m.new_state(), [], 0
        for n in split:
            outs.append(m.decode_to_pixel(lat[:, t0:t0 + n], use_cache=True, state=st))
            t0 += n
        torch.testing.assert_close(torch.cat(outs, 1).double(), want, atol=5e-6, rtol=0)
    # the oracle's own stream continues across calls as well
    st = ov.Stream()
    a = ov.decode_to_pixel(lat[:, :2], m.state_dict(), st)
    b = ov.decode_to_pixel(lat[:, 2:], m.state_dict(), st)
    torch.testing.assert_close(torch.cat([a, b], 1), want, atol=1e-12, rtol=0)


def test_decoder_is_causal():
    m = _tiny_decoder(seed=1)
    W = m.state_dict()
    lat = _rand(1, 4, 16, 3, 3, seed=21, scale=0.3)
    base = ov.decode_to_pixel(lat, W)
    lat2 = lat.clone()
    lat2[:, 2:] += 1.0                                            # change latent frames 2, 3
    moved = ov.decode_to_pixel(lat2, W)
    n_fixed = 1 + 4 * 1                                           # pixels of latent frames 0, 1
    torch.testing.assert_close(moved[:, :n_fixed], base[:, :n_fixed], atol=0, rtol=0)
    assert (moved[:, n_fixed:] - base[:, n_fixed:]).abs().max() > 1e-3


def test_parameter_names_follow_the_reference_layout():
    """Entries a reference checkpoint holds for the decode half (names from wan/modules/vae.py:369-421, :505-509)."""
    m = vd.WanVAEDecoder()
    keys = set(m.state_dict())
    for k in ("conv2.weight", "decoder.conv1.weight", "decoder.middle.0.residual.0.gamma", "decoder.middle.0.residual.2.weight",
              "decoder.middle.0.residual.6.bias", "decoder.middle.1.norm.gamma", "decoder.middle.1.to_qkv.weight",
              "decoder.middle.1.proj.bias", "decoder.upsamples.3.time_conv.weight", "decoder.upsamples.3.resample.1.weight",
              "decoder.upsamples.4.shortcut.weight", "decoder.upsamples.7.time_conv.bias", "decoder.upsamples.11.resample.1.bias",
              "decoder.upsamples.14.residual.6.weight", "decoder.head.0.gamma", "decoder.head.2.weight"):
        assert k in keys, k
    assert "decoder.upsamples.11.time_conv.weight" not in keys and "decoder.upsamples.15.residual.0.gamma" not in keys
    sd = m.state_dict()
    assert sd["decoder.conv1.weight"].shape == (384, 16, 3, 3, 3)
    assert sd["decoder.upsamples.3.time_conv.weight"].shape == (768, 384, 3, 1, 1)
    assert sd["decoder.upsamples.4.shortcut.weight"].shape == (384, 192, 1, 1, 1)
    assert sd["decoder.upsamples.11.resample.1.weight"].shape == (96, 192, 3, 3)
    assert sd["decoder.head.2.weight"].shape == (3, 96, 3, 3, 3)
    assert sd["decoder.middle.0.residual.0.gamma"].shape == (384, 1, 1, 1) and sd["decoder.middle.1.norm.gamma"].shape == (384, 1, 1)
    # an encoder's entries are ignored, a missing decoder entry is an error
    extra = dict(sd)
    extra["encoder.conv1.weight"] = torch.zeros(1)
    m.load_reference_state_dict(extra)
    del extra["decoder.head.2.weight"]
    with pytest.raises(KeyError):
        m.load_reference_state_dict(extra)
