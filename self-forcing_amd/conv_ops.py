"""Channels-last convolutions of the streaming VAE decoder on the HIP library (`sfm_conv3d_cl`).

Activations are [T, H, W, C] tensors (one video; channels contiguous).  Weights are re-laid out once per module
as [kt, kh, kw, Cout_pad, Cin] and cached on it.  The reference's modules are nn.Conv3d / nn.Conv2d on
[B, C, T, H, W] (wan/modules/vae.py:17-36, :76-79)."""
import collections
import ctypes as C

import torch

from . import lib as L

_DT = {torch.bfloat16: L.SFM_BF16, torch.float16: L.SFM_F16}


def prepared(conv, dtype, device):
    """(wt [kt,kh,kw,Cout_pad,Cin_pad], bias fp32 or None, kt, k) of an nn.Conv3d / nn.Conv2d, cached on the module.
    Cin is padded with zero weights to a multiple of 32, Cout with zero rows to a multiple of 32."""
    key = (dtype, str(device), conv.weight._version, conv.weight.data_ptr())
    hit = getattr(conv, "_sfm_cl", None)
    if hit is not None and hit[0] == key:
        return hit[1]
    w = conv.weight.detach()
    if w.dim() == 4:                                   # Conv2d: one frame
        w = w.unsqueeze(2)
    cout, cin, kt, kh, kw = w.shape
    cin_p, cout_p = (cin + 31) // 32 * 32, (cout + 31) // 32 * 32
    wt = torch.zeros(kt, kh, kw, cout_p, cin_p, dtype=dtype, device=device)
    wt[:, :, :, :cout, :cin] = w.permute(2, 3, 4, 0, 1).to(device=device, dtype=dtype)
    bias = conv.bias.detach().to(device=device, dtype=torch.float32).contiguous() if conv.bias is not None else None
    out = (wt.contiguous(), bias, kt, kh, cout, cin, cin_p, cout_p)
    conv._sfm_cl = (key, out)
    return out


def norm_act(x, gamma, act, out=None):
    """RMS norm over the channels of x [T, H, W, C] (+ SiLU if act) on the HIP library; `out` may be a strided view
    (e.g. the interior of a padded convolution input)."""
    T, H, W, Cn = x.shape
    if out is None:
        out = torch.empty_like(x)
    g = gamma.detach().reshape(-1).to(device=x.device, dtype=x.dtype).contiguous()
    if x.stride(3) != 1 or out.stride(3) != 1:
        raise ValueError("norm_act: channels must be contiguous")
    S3 = C.c_int64 * 3
    lib = L.load()
    stream = torch.cuda.current_stream(x.device).cuda_stream
    L.check(lib.sfm_vae_norm_act(_DT[x.dtype], T, H, W, Cn, 1 if act else 0, x.data_ptr(), S3(*x.stride()[:3]), g.data_ptr(),
                                 out.data_ptr(), S3(*out.stride()[:3]), stream))
    return out


_PADDED = collections.OrderedDict()
PADDED_BUDGET_BYTES = 16 << 30      # one 480 x 832 decode stream keeps 29 buffers, 4.8 GB (the largest 1.0 GB)


def _padded(shape, cin, dtype, device):
    """A zero-bordered input buffer of `shape`, one per (device, stream, shape, real input channels, dtype): the kernel
    never writes its input, every call overwrites the interior, so border, channel padding and anything else a call does
    not write stay zero and no call after the first fills the buffer.  Calls that share a buffer are ordered by their
    stream.  The buffers are kept across calls up to PADDED_BUDGET_BYTES in all; past that the least recently used ones
    are dropped (another chunk length, resolution or stream brings its own set), and release_padded() drops them all.
    Returns (buffer, it is new)."""
    key = (device, torch.cuda.current_stream(device).cuda_stream, tuple(shape), cin, dtype)
    buf = _PADDED.get(key)
    if buf is not None:
        _PADDED.move_to_end(key)
        return buf, False
    buf = _PADDED[key] = torch.zeros(shape, dtype=dtype, device=device)
    total = sum(b.numel() * b.element_size() for b in _PADDED.values())
    while total > PADDED_BUDGET_BYTES and len(_PADDED) > 1:
        _, old = _PADDED.popitem(last=False)            # never the one just made: it is the newest
        total -= old.numel() * old.element_size()
    return buf, True


def release_padded():
    """Drop the cached padded input buffers (they are rebuilt on demand)."""
    _PADDED.clear()


def conv_cl(x, conv, history=None, up2x=False, norm=None, want_tail=False, res=None):
    """x [T, H, W, Cin] -> [T, H', W', Cout] for a causal Conv3d (kt - 1 frames of `history`, zeros where it is
    shorter) or a Conv2d applied per frame; with up2x the nearest x2 upsampling in front of a 3x3 Conv2d is folded
    into the convolution (H' = 2 H, W' = 2 W).  With norm = (gamma, act) the convolution's input is
    norm_act(x, gamma, act), written straight into the padded buffer.  `res` [T, H', W', Cout] is added to the result
    inside the kernel.  With want_tail the last two frames of the
    (history + input) sequence come back as well: what the next call of a stream passes as `history`."""
    if x.dtype not in _DT:
        raise TypeError(f"conv_cl: dtype {x.dtype} (bf16 or fp16 only)")
    wt, bias, kt, k, cout, cin, cin_p, cout_p = prepared(conv, x.dtype, x.device)
    T, H, W, _ = x.shape
    past = kt - 1
    pad = (k - 1) // 2
    if past == 0 and pad == 0 and cin_p == cin and x.is_contiguous() and norm is None:
        xp = x
    else:
        xp, new = _padded((T + past, H + 2 * pad, W + 2 * pad, cin_p), cin, x.dtype, x.device)
        n = min(history.shape[0], past) if history is not None else 0
        if n > 0:
            xp[past - n:past, pad:pad + H, pad:pad + W, :cin] = history[-n:]
        if n < past and not new:
            xp[:past - n].zero_()                   # no history yet: these frames hold an earlier call's
        inner = xp[past:, pad:pad + H, pad:pad + W, :cin]
        if norm is None:
            inner.copy_(x)
        else:
            norm_act(x, norm[0], norm[1], out=inner)
    Ho, Wo = (2 * H, 2 * W) if up2x else (H, W)
    y = torch.empty(T, Ho, Wo, cout, dtype=x.dtype, device=x.device)
    if res is not None and (res.shape != y.shape or res.dtype != y.dtype):
        raise ValueError(f"conv_cl: res {tuple(res.shape)} {res.dtype} does not match the output {tuple(y.shape)} {y.dtype}")
    if res is not None:
        res = res.contiguous()
    d = L.ConvDesc()
    d.dtype = _DT[x.dtype]
    d.T, d.H, d.W = T, Ho, Wo
    d.Cin, d.Cout, d.Cout_pad = cin_p, cout, cout_p
    d.kt, d.kh, d.kw = kt, k, k
    d.up2x = 1 if up2x else 0
    for i in range(3):
        d.x_stride[i] = xp.stride(i)
        d.y_stride[i] = y.stride(i)
    lib = L.load()
    stream = torch.cuda.current_stream(x.device).cuda_stream
    L.check(lib.sfm_conv3d_cl(C.byref(d), xp.data_ptr(), wt.data_ptr(), bias.data_ptr() if bias is not None else None,
                              res.data_ptr() if res is not None else None, y.data_ptr(), stream))
    if want_tail:
        n = min(2, T + past)
        return y, xp[T + past - n:, pad:pad + H, pad:pad + W, :cin].clone()
    return y
