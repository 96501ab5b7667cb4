"""TEST INFRASTRUCTURE ONLY - CPU restatement (float64) of the reference's streaming VAE decode.

Follows wan/modules/vae.py: causal convolution with a two-frame cache (:17-36), RMS norm (:39-54),
nearest x2 + 3x3 conv upsampling with the temporal doubling of 'upsample3d' (:66-134), residual block
(:186-220), single-head attention block (:223-262), `Decoder3d` (:369-472), one latent frame per decoder
call as in `decode` (:548-572), latent de-normalisation and clamp of utils/wan_wrapper.py:91-114.

It is a function of a flat dict of weights (the reference's state-dict names) and keeps the per-convolution
caches in a dict keyed by those names; it shares no code with the product module.

Pinned by tests/test_oracle_vae.py without importing the reference: the causal convolution against a
brute-force triple loop and, frame by frame with its cache, against one convolution over the whole
zero-front-padded clip; the norm against its closed form; the attention block against an explicit softmax;
causality of the whole decoder (pixels of frames <= 1 + 4 (t - 1) do not depend on latent frames > t); the
frame count 1 + 4 (T - 1).  The composition of these pieces into the full decoder (channel counts, order of
blocks, the chunked stream) is pinned by tests/golden/vae_reference_vectors.npz: the output of the reference's
own `decode` and `cached_decode` on seeded weights at dim=32 (tests/golden/make_vae_reference_vectors.py wrote
it in the authoring container), which decode_frames reproduces to 1e-6 (the reference rounds to fp32 at every upsampling, vae.py:57-63).
"""
import numpy as np
import torch
import torch.nn.functional as F

F64 = torch.float64
MEAN = (-0.7571, -0.7089, -0.9113, 0.1075, -0.1745, 0.9653, -0.1517, 1.5508,
        0.4134, -0.0715, 0.5517, -0.3632, -0.1922, -0.9497, 0.2503, -0.2921)
STD = (2.8184, 1.4541, 2.3275, 2.6558, 1.2196, 1.7708, 2.6052, 2.0743,
       3.2687, 2.1526, 2.8652, 1.5579, 1.6382, 1.1253, 2.8251, 1.9160)


def causal_conv3d(x, w, b, cache=None):
    """x [B,C,T,H,W]; kernel (kt,kh,kw); pads (kh//2, kw//2) in space, kt - 1 frames towards the past, of which
    the cache supplies its own length (vae.py:22-36)."""
    kt, kh, kw = w.shape[2:]
    past = kt - 1
    if cache is not None and past > 0:
        x = torch.cat([cache, x], dim=2)
        past -= cache.shape[2]
    x = F.pad(x, (kw // 2, kw // 2, kh // 2, kh // 2, past, 0))
    return F.conv3d(x, w, b)


def rms_norm(x, gamma):
    """vae.py:51-54: x / max(|x|_2, 1e-12) over channels, times sqrt(C) gamma."""
    n = x.pow(2).sum(dim=1, keepdim=True).sqrt().clamp_min(1e-12)
    return x / n * (x.shape[1] ** 0.5) * gamma.reshape(1, -1, *([1] * (x.dim() - 2)))


def silu(x):
    return x / (1.0 + torch.exp(-x))


class Stream:
    """Caches of one decode stream, keyed by convolution name."""

    def __init__(self):
        self.cache = {}
        self.frames = 0


def _cached_conv(x, W, name, st):
    """vae.py:205-217: remember the last two input frames, convolve with the previous cache."""
    prev = st.cache.get(name)
    keep = x[:, :, -2:].clone()
    if keep.shape[2] < 2 and prev is not None:
        keep = torch.cat([prev[:, :, -1:], keep], dim=2)
    y = causal_conv3d(x, W[name + ".weight"], W[name + ".bias"], prev)
    st.cache[name] = keep
    return y


def residual_block(x, W, name, st):
    h = x
    if name + ".shortcut.weight" in W:
        h = causal_conv3d(x, W[name + ".shortcut.weight"], W[name + ".shortcut.bias"])
    x = silu(rms_norm(x, W[name + ".residual.0.gamma"]))
    x = _cached_conv(x, W, name + ".residual.2", st)
    x = silu(rms_norm(x, W[name + ".residual.3.gamma"]))
    x = _cached_conv(x, W, name + ".residual.6", st)
    return x + h


def attention_block(x, W, name):
    b, c, t, h, w = x.shape
    y = x.permute(0, 2, 1, 3, 4).reshape(b * t, c, h, w)
    y = rms_norm(y, W[name + ".norm.gamma"])
    qkv = F.conv2d(y, W[name + ".to_qkv.weight"], W[name + ".to_qkv.bias"]).reshape(b * t, 3 * c, h * w)
    q, k, v = qkv[:, :c].transpose(1, 2), qkv[:, c:2 * c].transpose(1, 2), qkv[:, 2 * c:].transpose(1, 2)
    p = torch.softmax(q @ k.transpose(1, 2) / (c ** 0.5), dim=-1)
    o = (p @ v).transpose(1, 2).reshape(b * t, c, h, w)
    o = F.conv2d(o, W[name + ".proj.weight"], W[name + ".proj.bias"])
    return x + o.reshape(b, t, c, h, w).permute(0, 2, 1, 3, 4)


def upsample(x, W, name, st, temporal):
    b, c, t, h, w = x.shape
    if temporal:
        key = name + ".time_conv"
        prev = st.cache.get(key)
        if prev is None:
            st.cache[key] = "Rep"                                   # first frame: no doubling (vae.py:104-107)
        else:
            keep = x[:, :, -2:].clone()
            if keep.shape[2] < 2:
                head = torch.zeros_like(keep) if isinstance(prev, str) else prev[:, :, -1:]
                keep = torch.cat([head, keep], dim=2)
            y = causal_conv3d(x, W[key + ".weight"], W[key + ".bias"], None if isinstance(prev, str) else prev)
            st.cache[key] = keep
            x = torch.stack((y[:, :c], y[:, c:]), dim=3).reshape(b, c, 2 * t, h, w)
            t = 2 * t
    y = x.permute(0, 2, 1, 3, 4).reshape(b * t, c, h, w)
    y = y.repeat_interleave(2, dim=2).repeat_interleave(2, dim=3)   # nearest x2
    y = F.conv2d(y, W[name + ".resample.1.weight"], W[name + ".resample.1.bias"], padding=1)
    return y.reshape(b, t, -1, 2 * h, 2 * w).permute(0, 2, 1, 3, 4)


def decoder_layout(W):
    """Order and kind of the `decoder.upsamples.N` entries present in the weights."""
    n = 0
    layout = []
    while any(k.startswith(f"decoder.upsamples.{n}.") for k in W):
        p = f"decoder.upsamples.{n}"
        if p + ".resample.1.weight" in W:
            layout.append((p, "up3d" if p + ".time_conv.weight" in W else "up2d"))
        else:
            layout.append((p, "res"))
        n += 1
    return layout


def decode_frame(x, W, st):
    """One decoder call on the frames in x (the reference always passes one), vae.py:423-472."""
    x = _cached_conv(x, W, "decoder.conv1", st)
    x = residual_block(x, W, "decoder.middle.0", st)
    x = attention_block(x, W, "decoder.middle.1")
    x = residual_block(x, W, "decoder.middle.2", st)
    for name, kind in decoder_layout(W):
        if kind == "res":
            x = residual_block(x, W, name, st)
        else:
            x = upsample(x, W, name, st, temporal=(kind == "up3d"))
    x = silu(rms_norm(x, W["decoder.head.0.gamma"]))
    return _cached_conv(x, W, "decoder.head.2", st)


def decode_frames(latent, W, st=None):
    """latent [B,T,C,h,w] -> decoder output [B,T',3,8h,8w] (float64, before the wrapper's clamp), one latent
    frame per decoder call; pass the Stream of earlier chunks to continue it (vae.py:574-596)."""
    W = {k: torch.as_tensor(np.asarray(v.detach().cpu().double()) if isinstance(v, torch.Tensor) else v, dtype=F64) for k, v in W.items()}
    st = Stream() if st is None else st
    z = torch.as_tensor(latent, dtype=F64).permute(0, 2, 1, 3, 4)
    C = z.shape[1]
    z = z * torch.tensor(STD[:C], dtype=F64).view(1, C, 1, 1, 1) + torch.tensor(MEAN[:C], dtype=F64).view(1, C, 1, 1, 1)
    x = causal_conv3d(z, W["conv2.weight"], W["conv2.bias"])
    outs = [decode_frame(x[:, :, i:i + 1], W, st) for i in range(x.shape[2])]
    st.frames += x.shape[2]
    return torch.cat(outs, dim=2).permute(0, 2, 1, 3, 4)


def decode_to_pixel(latent, W, st=None):
    """decode_frames followed by the clamp to [-1, 1] of utils/wan_wrapper.py:109."""
    return decode_frames(latent, W, st).clamp(-1, 1)
