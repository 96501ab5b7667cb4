"""Streaming Wan VAE decoder: latents [B, T, 16, h, w] -> pixels [B, 1 + 4 (T - 1), 3, 8 h, 8 w].

Host-side mirror of the decode half of the reference's VAE (wan/modules/vae.py:369-472 `Decoder3d`,
:548-596 `decode` / `cached_decode`, utils/wan_wrapper.py:91-114 `decode_to_pixel`) and of the demo's
chunk-by-chunk decode (demo.py:406-441).  Parameter names follow the reference's modules so that its
checkpoint's `conv2.*` and `decoder.*` entries load unchanged (`load_reference_state_dict`).

Every temporal convolution is causal and keeps the last two input frames of the previous call
(vae.py:28-36, :202-219), held here in an explicit `DecodeState` instead of module attributes, so one
decoder serves any number of independent streams.  The reference feeds the decoder one latent frame per
call; the convolutions are causal, so a call may carry any number of frames and give the same result, and
this decoder pushes a whole chunk through at once (only the very first frame of a stream goes alone: the
temporal upsamplers skip it, vae.py:104-107).

Two execution paths share the parameters and the stream logic.  On the GPU in bf16 / fp16 a stream of one video
runs channels-last ([T, H, W, C] activations): 3x3x3, (3,1,1) and upsampling convolutions go to the HIP
implicit-GEMM kernel (`conv_ops.conv_cl`, which folds the nearest x2 upsampling into the convolution), 1x1
convolutions are matrix products.  Anywhere else (CPU, fp32, batches, `SFM_VAE_TORCH_CONV=1`) the modules run as
torch convolutions on [B, C, T, H, W].  A DecodeState stays with the path that started it.
"""
import os

import torch
import torch.nn as nn
import torch.nn.functional as F

TAIL = 2                                    # frames every causal convolution remembers (vae.py:14)

LATENT_MEAN = (-0.7571, -0.7089, -0.9113, 0.1075, -0.1745, 0.9653, -0.1517, 1.5508,
               0.4134, -0.0715, 0.5517, -0.3632, -0.1922, -0.9497, 0.2503, -0.2921)
LATENT_STD = (2.8184, 1.4541, 2.3275, 2.6558, 1.2196, 1.7708, 2.6052, 2.0743,
              3.2687, 2.1526, 2.8652, 1.5579, 1.6382, 1.1253, 2.8251, 1.9160)


class DecodeState:
    """What a stream carries from one call to the next: per temporal convolution the last frames of its
    input (`tails[i]`, None before the first call), and for the temporal upsamplers the marker that the
    first frame has passed (`FIRST`, the reference's 'Rep')."""
    FIRST = "first-frame-passed"

    def __init__(self, n_convs):
        self.tails = [None] * n_convs
        self.cursor = 0
        self.frames_in = 0
        self.layout = None                  # "cl" (channels-last, HIP convolutions) or "ncthw" (torch), set by the first call

    def rewind(self):
        self.cursor = 0

    def take(self):
        i = self.cursor
        self.cursor += 1
        return i


def _next_tail(x, prev):
    """Last TAIL frames of the stream ending with `x` (vae.py:205-213)."""
    tail = x[:, :, -TAIL:].clone()
    if tail.shape[2] < TAIL and isinstance(prev, torch.Tensor):
        tail = torch.cat([prev[:, :, -1:].to(tail.device), tail], dim=2)
    return tail


class CausalConv3d(nn.Conv3d):
    """Conv3d padded only towards the past in time (vae.py:17-36)."""

    def __init__(self, cin, cout, kernel_size, stride=1, padding=0):
        super().__init__(cin, cout, kernel_size, stride=stride, padding=0)
        pt, ph, pw = (padding,) * 3 if isinstance(padding, int) else padding
        self.past = 2 * pt
        self.hw = (pw, pw, ph, ph)

    def forward(self, x, tail=None):
        past = self.past
        if tail is not None and past > 0:
            x = torch.cat([tail.to(x.device), x], dim=2)
            past -= tail.shape[2]
        return super().forward(F.pad(x, self.hw + (past, 0)))

    def stream(self, x, state):
        """Applies the convolution to the next frames of a stream and updates the stream's tail."""
        i = state.take()
        prev = state.tails[i]
        tail = _next_tail(x, prev)
        y = self(x, prev)
        state.tails[i] = tail
        return y

    def stream_cl(self, x, state, norm=None, res=None):
        """`stream` for channels-last activations [T, H, W, C]; with norm = (gamma, act) the convolution's input is
        the RMS norm (+ SiLU) of x and `res` is added to the result.  The tail kept is always two frames (a zero frame stands in before the stream
        has two), which the convolution treats exactly like the reference's shorter cache plus zero padding."""
        from . import conv_ops
        i = state.take()
        prev = state.tails[i]
        y, tail = conv_ops.conv_cl(x, self, prev if isinstance(prev, torch.Tensor) else None, norm=norm, want_tail=True, res=res)
        state.tails[i] = tail
        return y

    def pointwise_cl(self, x):
        """A 1x1x1 convolution of channels-last activations: a matrix product over the channels."""
        return F.linear(x, self.weight.view(self.out_channels, self.in_channels), self.bias)


class RMS_norm(nn.Module):
    """x / |x|_2 over channels * sqrt(C) * gamma (vae.py:39-54)."""

    def __init__(self, dim, images=True):
        super().__init__()
        self.scale = dim ** 0.5
        self.gamma = nn.Parameter(torch.ones((dim, 1, 1) if images else (dim, 1, 1, 1)))

    def forward(self, x):
        return F.normalize(x, dim=1) * self.scale * self.gamma

    def forward_cl(self, x, act=False):
        from . import conv_ops
        return conv_ops.norm_act(x.contiguous(), self.gamma, act)


class _Nearest2x(nn.Module):
    """Nearest-neighbour x2 in height and width, computed in fp32 (vae.py:57-63).  Sits at index 0 of
    `Resample.resample` like the reference's parameter-free Upsample."""

    def forward(self, x):
        return F.interpolate(x.float(), scale_factor=(2.0, 2.0), mode="nearest").type_as(x)


class Resample(nn.Module):
    """Spatial x2 upsampling, preceded for mode 'upsample3d' by a temporal x2 (vae.py:66-134)."""

    def __init__(self, dim, mode):
        super().__init__()
        assert mode in ("upsample2d", "upsample3d")
        self.mode = mode
        self.resample = nn.Sequential(_Nearest2x(), nn.Conv2d(dim, dim // 2, 3, padding=1))
        if mode == "upsample3d":
            self.time_conv = CausalConv3d(dim, dim * 2, (3, 1, 1), padding=(1, 0, 0))

    def forward(self, x, state):
        b, c, t, h, w = x.shape
        if self.mode == "upsample3d":
            i = state.take()
            prev = state.tails[i]
            if prev is None:
                # the first frame of a stream is not doubled and leaves no tail behind (vae.py:104-107)
                state.tails[i] = DecodeState.FIRST
            else:
                tail = x[:, :, -TAIL:].clone()
                if tail.shape[2] < TAIL:
                    # vae.py:110-124: after the first frame the missing history is zeros
                    head = prev[:, :, -1:].to(tail.device) if isinstance(prev, torch.Tensor) else torch.zeros_like(tail)
                    tail = torch.cat([head, tail], dim=2)
                y = self.time_conv(x, prev if isinstance(prev, torch.Tensor) else None)
                state.tails[i] = tail
                # channels [0, c) are the even output frames, [c, 2c) the odd ones (vae.py:131-134)
                x = torch.stack((y[:, :c], y[:, c:]), dim=3).reshape(b, c, 2 * t, h, w)
                t = 2 * t
        x = x.permute(0, 2, 1, 3, 4).reshape(b * t, c, h, w)
        x = self.resample(x)
        return x.reshape(b, t, x.shape[1], 2 * h, 2 * w).permute(0, 2, 1, 3, 4)


    def forward_cl(self, x, state):
        """`forward` for channels-last activations [T, H, W, C]."""
        from . import conv_ops
        t, h, w, c = x.shape
        if self.mode == "upsample3d":
            i = state.take()
            prev = state.tails[i]
            if prev is None:
                state.tails[i] = DecodeState.FIRST
            else:
                tail = x[-TAIL:].clone()
                if tail.shape[0] < TAIL:
                    head = prev[-1:] if isinstance(prev, torch.Tensor) else torch.zeros_like(tail)
                    tail = torch.cat([head, tail], dim=0)
                y = conv_ops.conv_cl(x, self.time_conv, prev if isinstance(prev, torch.Tensor) else None)
                state.tails[i] = tail
                x = torch.stack((y[..., :c], y[..., c:]), dim=1).reshape(2 * t, h, w, c)
        return conv_ops.conv_cl(x, self.resample[1], None, up2x=True)


class ResidualBlock(nn.Module):
    """norm, SiLU, conv, norm, SiLU, conv + shortcut (vae.py:186-220)."""

    def __init__(self, in_dim, out_dim):
        super().__init__()
        self.residual = nn.Sequential(
            RMS_norm(in_dim, images=False), nn.SiLU(), CausalConv3d(in_dim, out_dim, 3, padding=1),
            RMS_norm(out_dim, images=False), nn.SiLU(), nn.Dropout(0.0), CausalConv3d(out_dim, out_dim, 3, padding=1))
        self.shortcut = CausalConv3d(in_dim, out_dim, 1) if in_dim != out_dim else nn.Identity()

    def forward(self, x, state):
        skip = self.shortcut(x)
        for layer in self.residual:
            x = layer.stream(x, state) if isinstance(layer, CausalConv3d) else layer(x)
        return x + skip

    def forward_cl(self, x, state):
        skip = self.shortcut.pointwise_cl(x) if isinstance(self.shortcut, CausalConv3d) else x
        r = self.residual                       # norm, SiLU, conv, norm, SiLU, dropout(0), conv
        x = r[2].stream_cl(x, state, norm=(r[0].gamma, True))
        return r[6].stream_cl(x, state, norm=(r[3].gamma, True), res=skip)          # the residual sum happens in the kernel


class AttentionBlock(nn.Module):
    """Single-head self-attention over the pixels of each frame (vae.py:223-262)."""

    def __init__(self, dim):
        super().__init__()
        self.norm = RMS_norm(dim)
        self.to_qkv = nn.Conv2d(dim, dim * 3, 1)
        self.proj = nn.Conv2d(dim, dim, 1)
        nn.init.zeros_(self.proj.weight)

    def forward(self, x, state=None):
        b, c, t, h, w = x.shape
        y = x.permute(0, 2, 1, 3, 4).reshape(b * t, c, h, w)
        qkv = self.to_qkv(self.norm(y)).reshape(b * t, 3, c, h * w).transpose(2, 3)       # [bt, 3, hw, c]
        o = F.scaled_dot_product_attention(qkv[:, 0:1], qkv[:, 1:2], qkv[:, 2:3])          # one head
        o = self.proj(o[:, 0].transpose(1, 2).reshape(b * t, c, h, w))
        return x + o.reshape(b, t, c, h, w).permute(0, 2, 1, 3, 4)

    def forward_cl(self, x, state=None):
        t, h, w, c = x.shape
        qkv = F.linear(self.norm.forward_cl(x).reshape(t, h * w, c), self.to_qkv.weight.view(3 * c, c), self.to_qkv.bias)
        q, k, v = qkv.split(c, dim=-1)                                                     # [t, hw, c] each
        if x.is_cuda and x.dtype in (torch.bfloat16, torch.float16):
            # head_dim 384 is outside the fused attention kernels of the libraries: two plain matrix products with the
            # logits kept in fp32 (6240 x 6240 per frame) and the softmax between them
            p = torch.bmm(q, k.transpose(1, 2), out_dtype=torch.float32).mul_(c ** -0.5)
            o = torch.bmm(torch.softmax(p, dim=-1, out=p).to(x.dtype), v)
        else:
            o = F.scaled_dot_product_attention(q.unsqueeze(1), k.unsqueeze(1), v.unsqueeze(1))[:, 0]
        return x + F.linear(o, self.proj.weight.view(c, c), self.proj.bias).reshape(t, h, w, c)


class Decoder3d(nn.Module):
    """vae.py:369-472 with the reference's defaults for the Wan 2.1 VAE (vae.py:626-633): dim 96,
    multipliers (1, 2, 4, 4), two residual blocks (+1) per level, no attention outside the middle."""

    def __init__(self, dim=96, z_dim=16, dim_mult=(1, 2, 4, 4), num_res_blocks=2, temporal_upsample=(True, True, False)):
        super().__init__()
        dims = [dim * m for m in (dim_mult[-1],) + tuple(dim_mult[::-1])]
        self.conv1 = CausalConv3d(z_dim, dims[0], 3, padding=1)
        self.middle = nn.Sequential(ResidualBlock(dims[0], dims[0]), AttentionBlock(dims[0]), ResidualBlock(dims[0], dims[0]))
        ups = []
        for level, (cin, cout) in enumerate(zip(dims[:-1], dims[1:])):
            if level > 0:
                cin = cin // 2                      # the upsampler below halved the channels
            for _ in range(num_res_blocks + 1):
                ups.append(ResidualBlock(cin, cout))
                cin = cout
            if level != len(dim_mult) - 1:
                ups.append(Resample(cout, "upsample3d" if temporal_upsample[level] else "upsample2d"))
        self.upsamples = nn.Sequential(*ups)
        self.head = nn.Sequential(RMS_norm(dims[-1], images=False), nn.SiLU(), CausalConv3d(dims[-1], 3, 3, padding=1))

    def forward(self, x, state):
        state.rewind()
        x = self.conv1.stream(x, state)
        for layer in self.middle:
            x = layer(x, state)
        for layer in self.upsamples:
            x = layer(x, state)
        x = self.head[1](self.head[0](x))
        return self.head[2].stream(x, state)

    def forward_cl(self, x, state):
        state.rewind()
        x = self.conv1.stream_cl(x, state)
        for layer in self.middle:
            x = layer.forward_cl(x, state)
        for layer in self.upsamples:
            x = layer.forward_cl(x, state)
        return self.head[2].stream_cl(x, state, norm=(self.head[0].gamma, True))


class WanVAEDecoder(nn.Module):
    """`conv2` + `decoder` of the reference's WanVAE_ (vae.py:486-513) with the latent statistics of
    utils/wan_wrapper.py:58-67."""

    def __init__(self, z_dim=16, dim=96):
        super().__init__()
        self.z_dim = z_dim
        self.conv2 = CausalConv3d(z_dim, z_dim, 1)
        self.decoder = Decoder3d(dim=dim, z_dim=z_dim)
        self.register_buffer("mean", torch.tensor(LATENT_MEAN[:z_dim], dtype=torch.float32).view(1, z_dim, 1, 1, 1), persistent=False)
        self.register_buffer("std", torch.tensor(LATENT_STD[:z_dim], dtype=torch.float32).view(1, z_dim, 1, 1, 1), persistent=False)

    # ---- state ------------------------------------------------------------------------------------
    def new_state(self):
        n = sum(1 for m in self.decoder.modules() if isinstance(m, CausalConv3d) and m.past > 0)
        return DecodeState(n)

    def load_reference_state_dict(self, sd):
        """Loads the `conv2.*` and `decoder.*` entries of a reference VAE checkpoint (the encoder's are
        ignored).  The caller reads the file (`torch.load(..., weights_only=True)`)."""
        own = self.state_dict()
        picked = {k: v for k, v in sd.items() if k in own}
        missing = [k for k in own if k not in picked]
        if missing:
            raise KeyError(f"checkpoint lacks {len(missing)} decoder entries, e.g. {missing[:3]}")
        self.load_state_dict(picked, strict=True)

    # ---- decoding ---------------------------------------------------------------------------------
    def _channels_last(self, z, state):
        """Whether this call runs on the HIP convolution path; a stream keeps the path it started with."""
        if state.layout is None:
            ok = (z.is_cuda and z.shape[0] == 1 and z.dtype in (torch.bfloat16, torch.float16)
                  and os.environ.get("SFM_VAE_TORCH_CONV", "0") != "1")
            state.layout = "cl" if ok else "ncthw"
        if state.layout == "cl" and z.shape[0] != 1:
            raise ValueError("a channels-last decode stream carries one video")
        return state.layout == "cl"

    def _frames(self, z, state):
        """z: [B, C, t, h, w] un-normalised latents -> [B, 3, t', 8h, 8w]."""
        if self._channels_last(z, state):
            x = self.conv2.pointwise_cl(z[0].permute(1, 2, 3, 0))                  # [t, h, w, C]
            run, cat_dim = self.decoder.forward_cl, 0
            pick = lambda a, b: x[a:b]
        else:
            x = self.conv2(z)
            run, cat_dim = self.decoder, 2
            pick = lambda a, b: x[:, :, a:b]
        n = z.shape[2]
        outs = []
        start = 0
        if state.frames_in == 0:
            outs.append(run(pick(0, 1), state))
            start = 1
        if n > start:
            outs.append(run(pick(start, n), state))
        state.frames_in += n
        out = outs[0] if len(outs) == 1 else torch.cat(outs, dim=cat_dim)
        return out.permute(3, 0, 1, 2).unsqueeze(0) if state.layout == "cl" else out

    @torch.no_grad()
    def decode_stream(self, latent, state):
        """Next chunk of a stream.  latent: [B, T, C, h, w] (the generator's layout); returns pixels
        [B, T', 3, 8h, 8w] in fp32 clamped to [-1, 1] with T' = 4 T, or 4 T - 3 for the first chunk
        (demo.py:406-441: chunk-by-chunk decode; utils/wan_wrapper.py:91-114)."""
        z = latent.to(self.conv2.weight.dtype).permute(0, 2, 1, 3, 4)
        z = z * self.std.to(z.dtype) + self.mean.to(z.dtype)        # vae.py:551-555 with scale = (mean, 1 / std)
        out = self._frames(z, state)
        return out.float().clamp_(-1, 1).permute(0, 2, 1, 3, 4)

    @torch.no_grad()
    def decode_to_pixel(self, latent, use_cache=False, state=None):
        """utils/wan_wrapper.py:91-114.  Without `use_cache` a whole video is decoded from a fresh state
        (vae.py:548-572); with it the stream in `state` continues (vae.py:574-596; the reference keeps
        that state inside the module, here the caller owns it)."""
        if not use_cache:
            state = self.new_state()
        elif state is None:
            raise ValueError("use_cache=True needs the stream's DecodeState")
        return self.decode_stream(latent, state)
