"""Causal Wan DiT around the attention hot path (PyTorch-ROCm host, HIP attention kernels).

Counterpart of the reference's KV-cache inference path:
    CausalWanSelfAttention   wan/modules/causal_model.py:718-807, 899-1108
    WanT2VCrossAttention     wan/modules/model.py:733-768
    CausalWanAttentionBlock  wan/modules/causal_model.py:1111-1205
    CausalHead               wan/modules/causal_model.py:1208-1236
    CausalWanModel           wan/modules/causal_model.py:1250-1370, 1582-1720, 1896-1943
Module / parameter names follow the reference so that its state dicts load unchanged.

What differs from the reference, on purpose:
  * q/k RMSNorm, 3-D RoPE and the KV-cache write are one fused kernel (prologue.qk_prologue); the cache is
    written before the attention op, which then reads it (no rearranged copies of q, k, v);
  * the cache counters are mirrored as Python ints next to the reference's two int64 tensors, so no
    device->host sync happens per layer (the reference does >= 4 `.item()` calls per layer);
  * the patch embedding is a GEMM over unfolded 1x2x2 patches (same parameters as the Conv3d).
Forward only; training paths (flex-attention masks, teacher forcing) are not part of this build.
"""
import math
import os

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import attention as _attn
from . import block_ops as _blk
from . import linear as _lin
from . import monarch_attn as _mon
from . import prologue as _pro

FRAME_HEIGHT = 30          # utils/resolution.py:7-12 (480p)
FRAME_WIDTH = 52
TOTAL_SEQ_LEN = 21 * 30 * 52


class HipAttentionOps:
    """The HIP operators the model calls (attention, fused prologue, fused block element-wise ops).  Tests
    may pass another object with the same methods (e.g. one built on the CPU oracle and eager torch ops) to
    obtain a reference run of the same module code.

    own_gemm selects which linear layers run on the library's own matrix-product kernel (`linear.linear`) instead of
    hipBLASLt: False (default) none; "auto" the square projections of the block (attention output, cross-attention q
    and output: N, K <= 2048), where the own kernel's 128 x 256 tiles are level with hipBLASLt in isolation (26 vs
    25-29 us at 4680 x 1536 x 1536) and 0.5 % slower over a rollout; True additionally the FFN with the GELU and the
    gated residual update in the GEMM's epilogue (10-15 % slower than the tuned hipBLASLt kernels at those shapes)."""

    def __init__(self, own_gemm=False):
        self.own_gemm = own_gemm is True
        self.own_square = own_gemm is True or own_gemm == "auto"

    def linear(self, x, linear):
        """nn.Linear forward for inference: the own kernel for the block's square projections, else the library."""
        w = linear.weight
        if (self.own_square and not torch.is_grad_enabled() and w.shape[0] <= 2048 and w.shape[1] <= 2048 and x.dim() == 3
                and _lin.supported(x, w)):
            return _lin.linear(x, w, linear.bias)
        return linear(x)

    def rope_table(self, head_dim, device):
        return _pro.rope_table(head_dim, device=device)

    def qk_prologue(self, *args, **kwargs):
        return _pro.qk_prologue(*args, **kwargs)

    def monarch_cached(self, q, k_view, v_view, f_tied, h_reduce, w_reduce, h, w, num_iters=1):
        return _mon.monarch_attn(q, k_view, v_view, f_tied, h_reduce, w_reduce, h, w, kv_block_order=True,
                                 num_iters=num_iters)

    def dense(self, q, k, v):
        return _attn.attention(q, k, v, dtype=q.dtype)

    # fused element-wise operators of the block (block_ops.py)
    def ln_modulate(self, x, scale, shift, eps):
        return _blk.ln_modulate(x, scale, shift, eps)

    def ln_affine(self, x, weight, bias, eps):
        return _blk.ln_affine(x, weight, bias, eps)

    def gate_residual(self, x, y, gate=None):
        return _blk.gate_residual_(x, y if y.stride(2) == 1 else y.contiguous(), gate)

    def rms_norm(self, x, weight, eps):
        return _blk.rms_norm(x, weight, eps)

    def gate_residual_ln(self, x, y, gate, eps, scale=None, shift=None, weight=None, bias=None):
        """(x + y * gate, norm of that sum): residual update and the next sub-layer's LayerNorm in one kernel."""
        return _blk.gate_residual_ln_(x, y if y.stride(2) == 1 else y.contiguous(), gate, scale, shift, weight, bias, eps)

    def linear_gelu(self, x, linear):
        """GELU(tanh)(x W^T + b) with the activation applied in the GEMM's epilogue (hipBLASLt through
        torch's addmm-with-activation); the reference runs Linear and nn.GELU(approximate='tanh') apart
        (model.py:648-650)."""
        if self.own_gemm and _lin.supported(x, linear.weight):
            return _lin.linear(x, linear.weight, linear.bias, epilogue="gelu_tanh")
        out = torch._addmm_activation(linear.bias, x.reshape(-1, x.shape[-1]), linear.weight.t(), use_gelu=True)
        return out.view(*x.shape[:-1], out.shape[-1])

    def linear_gate_residual(self, x, h, linear, gate):
        """x + linear(h) * gate, in place into x (the FFN's second half and the block's last residual update,
        causal_model.py:1203-1204)."""
        if self.own_gemm and _lin.supported(h, linear.weight):
            return _lin.linear(h, linear.weight, linear.bias, epilogue="gate_residual", res=x, gate=gate)
        return self.gate_residual(x, linear(h), gate)


def _env_int(name, default):
    return int(os.getenv(name, str(default)))


class AttentionFlags:
    """The reference selects the attention kernel through process environment variables read in the module
    constructor (causal_model.py:739-766); the same names are honoured here, and every field can be
    overridden explicitly."""

    def __init__(self, block_num=None, **override):
        self.num_iters = _env_int("MONARCH_ATTN_NUM_ITERS", 1)
        self.use_dense_init = bool(_env_int("USE_DENSE_INIT", 0))
        self.h_reduce = _env_int("MONARCH_ATTN_H_REDUCE", 1)
        self.w_reduce = _env_int("MONARCH_ATTN_W_REDUCE", 1)
        self.use_framewise = bool(_env_int("MONARCH_ATTN_FRAMEWISE", 0))
        self.disable_monarch = bool(_env_int("DISABLE_MONARCH_ATTN", 0))
        # no counterpart in the reference: a windowed KV cache (local_attn_size != -1) is kept as a ring instead of
        # being shifted down on every eviction (cache_step_ring); 0 keeps the reference's row order in the cache
        self.ring_cache = bool(_env_int("SFM_RING_KV_CACHE", 1))
        layers = os.getenv("MONARCH_ATTN_DISABLE_LAYERS")
        if layers is not None and block_num is not None and block_num in [int(x) for x in layers.split(",")]:
            self.disable_monarch = True
        for k, v in override.items():
            if not hasattr(self, k):
                raise TypeError(f"unknown attention flag {k}")
            setattr(self, k, v)


class WanRMSNorm(nn.Module):
    """model.py:462-478: fp32 normalisation over the full model dim, cast back, times weight."""

    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + self.eps)).type_as(x) * self.weight


class WanLayerNorm(nn.LayerNorm):
    def __init__(self, dim, eps=1e-6, elementwise_affine=False):
        super().__init__(dim, elementwise_affine=elementwise_affine, eps=eps)

    def forward(self, x):
        return super().forward(x).type_as(x)


def sinusoidal_embedding_1d(dim, position):
    """model.py:407-417: cat[cos, sin] of position * 10000^(-m/half), float64."""
    half = dim // 2
    position = position.type(torch.float64)
    sinusoid = torch.outer(position, torch.pow(10000, -torch.arange(half, dtype=position.dtype, device=position.device).div(half)))
    return torch.cat([torch.cos(sinusoid), torch.sin(sinusoid)], dim=1)


def _sync_mirrors(kv_cache):
    """The host-integer mirrors `_global_end` / `_local_end` follow the two int64 tensors of the reference's cache
    dict: they are read back (one device sync) whenever a tensor is another object or has been written by anyone but
    cache_commit since the mirrors were taken, e.g. after the reference's own reset, which replaces the tensors
    (pipeline/causal_inference.py:134-138)."""
    g, l = kv_cache["global_end_index"], kv_cache["local_end_index"]
    src = kv_cache.get("_mirror_of")
    if src is None or src[0] is not g or src[1] != g._version or src[2] is not l or src[3] != l._version:
        kv_cache["_global_end"] = int(g.item())
        kv_cache["_local_end"] = int(l.item())
        kv_cache["_mirror_of"] = (g, g._version, l, l._version)
        kv_cache.pop("_written", None)
        kv_cache.pop("_ring", None)


def reset_cache_counters(kv_cache, device):
    """Start of a video (pipeline/causal_inference.py:134-138): fresh zero counters, K/V storage kept.  Sets the host
    mirrors along with the tensors, so that no device sync is needed to learn that they are zero."""
    g = kv_cache["global_end_index"] = torch.tensor([0], dtype=torch.long, device=device)
    l = kv_cache["local_end_index"] = torch.tensor([0], dtype=torch.long, device=device)
    kv_cache["_global_end"] = kv_cache["_local_end"] = 0
    kv_cache["_mirror_of"] = (g, g._version, l, l._version)
    kv_cache.pop("_written", None)
    kv_cache.pop("_ring", None)


def cache_step(kv_cache, current_start, num_new, frame_seqlen, local_attn_size, sink_size, max_attention_size):
    """Index arithmetic of one self-attention call (causal_model.py:907-938), on host integers.
    Returns (roll, cache_start, local_start, local_end) with local_* relative to cache_start and
    roll = (src, dst, len) of the window-eviction copy (len 0 = none)."""
    _sync_mirrors(kv_cache)
    g_end, l_end = kv_cache["_global_end"], kv_cache["_local_end"]
    current_end = current_start + num_new
    cache_len = kv_cache["k"].shape[1]
    sink_tokens = sink_size * frame_seqlen
    roll = (0, 0, 0)
    if local_attn_size != -1 and current_end > g_end and num_new + l_end > cache_len:
        evicted = num_new + l_end - cache_len
        rolled = l_end - evicted - sink_tokens
        roll = (sink_tokens + evicted, sink_tokens, rolled)
        local_end = l_end + current_end - g_end - evicted
    else:
        local_end = l_end + current_end - g_end
    local_start = local_end - num_new
    cache_start = max(0, local_end - max_attention_size)
    return roll, cache_start, local_start - cache_start, local_end - cache_start, current_end


def cache_step_ring(kv_cache, current_start, num_new, frame_seqlen, sink_size):
    """Windowed cache kept as a ring: the chunk at global tokens [current_start, current_start + num_new) is
    written over the oldest chunk after the sink frames instead of shifting the window down
    (causal_model.py:912-926 does the shift with a copy).  Attention over the cache is a sum over its rows, so
    the order in which block-frames sit in it does not change the result; the rotary phase is in the rows.
    Chunks must arrive in order (a re-run of the latest chunk lands in the same slot).
    Returns (write_start, view_len, current_end), or None when the chunk would straddle the end of the ring."""
    cache_len = kv_cache["k"].shape[1]
    sink = sink_size * frame_seqlen
    ring = cache_len - sink
    current_end = current_start + num_new
    if current_end <= cache_len:                       # still filling: positions are the global ones
        return current_start, current_end, current_end
    if ring <= 0 or current_start < sink:
        return None
    pos = sink + (current_start - sink) % ring
    if pos + num_new > cache_len:
        return None
    return pos, cache_len, current_end


def ring_to_window_order(kv_cache, sink_tokens):
    """Leave the ring: rotate the rows after the sink frames so that the oldest comes first, which is the order the
    reference's shift-down eviction keeps (causal_model.py:912-926), and set the local end as the reference has it for a
    full window.  One copy of the cache; needed when a chunk arrives that would straddle the end of the ring."""
    _sync_mirrors(kv_cache)
    cache_len = kv_cache["k"].shape[1]
    g_end = kv_cache["_global_end"]
    if g_end > cache_len:
        pos = sink_tokens + (g_end - sink_tokens) % (cache_len - sink_tokens)
        if pos != sink_tokens:
            for key in ("k", "v"):
                t = kv_cache[key]
                t[:, sink_tokens:] = torch.cat((t[:, pos:], t[:, sink_tokens:pos]), 1)
        kv_cache["_local_end"] = cache_len
        kv_cache.pop("_written", None)
    kv_cache["_ring"] = False


def cache_commit(kv_cache, current_end, local_end):
    """causal_model.py:1102-1103 (the reference stores the view-relative local end)."""
    kv_cache["_global_end"], kv_cache["_local_end"] = current_end, local_end
    if kv_cache.get("_written") != (current_end, local_end):     # unchanged when a chunk is re-run at another timestep
        g, l = kv_cache["global_end_index"], kv_cache["local_end_index"]
        g.fill_(current_end)
        l.fill_(local_end)
        kv_cache["_written"] = (current_end, local_end)
        kv_cache["_mirror_of"] = (g, g._version, l, l._version)


class CausalWanSelfAttention(nn.Module):

    def __init__(self, dim, num_heads, local_attn_size=-1, sink_size=0, qk_norm=True, eps=1e-6, block_num=None,
                 frame_hw=(FRAME_HEIGHT, FRAME_WIDTH), total_seq_len=None, flags=None, ops=None):
        assert dim % num_heads == 0
        super().__init__()
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.local_attn_size, self.sink_size, self.eps = local_attn_size, sink_size, eps
        self.frame_hw = frame_hw
        frame_tokens = frame_hw[0] * frame_hw[1]
        if total_seq_len is None:
            total_seq_len = 21 * frame_tokens
        self.max_attention_size = total_seq_len if local_attn_size == -1 else local_attn_size * frame_tokens
        self.flags = flags if flags is not None else AttentionFlags(block_num)
        self.ops = ops if ops is not None else HipAttentionOps()
        self.block_num = block_num
        if not qk_norm:
            raise NotImplementedError("the fused prologue always applies the q/k RMSNorm")
        self.q = nn.Linear(dim, dim)
        self.k = nn.Linear(dim, dim)
        self.v = nn.Linear(dim, dim)
        self.o = nn.Linear(dim, dim)
        self.norm_q = WanRMSNorm(dim, eps=eps)
        self.norm_k = WanRMSNorm(dim, eps=eps)
        self._rope = None
        self._qkv = None

    def _project_qkv(self, x):
        """q, k, v projections as one GEMM over the concatenated weights (the parameters stay the reference's
        three Linear layers; the concatenation is rebuilt when one of them changes).  The three results are
        column slices of one [B, S, 3C] tensor, which the prologue reads through its row stride."""
        ws = (self.q.weight, self.k.weight, self.v.weight)
        key = tuple((w.data_ptr(), w._version) for w in ws) + (x.dtype, x.device)
        if self._qkv is None or self._qkv[0] != key:
            with torch.no_grad():
                self._qkv = (key, torch.cat(ws, 0).contiguous(), torch.cat((self.q.bias, self.k.bias, self.v.bias), 0).contiguous())
        y = torch.nn.functional.linear(x, self._qkv[1], self._qkv[2])
        c = self.dim
        return y[..., :c], y[..., c:2 * c], y[..., 2 * c:]

    def forward(self, x, grid, kv_cache, current_start=0):
        """x [B, S, C] with S = F*h*w tokens of grid = (F, h, w); kv_cache: the reference's per-layer dict."""
        b, s = x.shape[:2]
        n, d = self.num_heads, self.head_dim
        F_, h, w = grid
        frame_seqlen = h * w
        fl = self.flags
        if self._rope is None or self._rope.device != x.device:
            self._rope = self.ops.rope_table(d, x.device)

        ring = None
        if fl.ring_cache and self.local_attn_size != -1 and "_ring" not in kv_cache:
            _sync_mirrors(kv_cache)
            if kv_cache["_global_end"] > kv_cache["k"].shape[1]:
                kv_cache["_ring"] = False       # filled past its window by a caller that shifts: keep that order
        if fl.ring_cache and self.local_attn_size != -1 and kv_cache.get("_ring", True):
            ring = cache_step_ring(kv_cache, current_start, s, frame_seqlen, self.sink_size)
            if ring is None and kv_cache.get("_ring"):
                ring_to_window_order(kv_cache, self.sink_size * frame_seqlen)
            kv_cache["_ring"] = ring is not None
        if ring is not None:
            write_start, view_len, current_end = ring
            cache_start, local_start, local_end = 0, write_start, write_start + s
        else:
            roll, cache_start, local_start, local_end, current_end = cache_step(
                kv_cache, current_start, s, frame_seqlen, self.local_attn_size, self.sink_size, self.max_attention_size)
            if roll[2] > 0:      # window eviction (causal_model.py:919-922)
                src, dst, ln = roll
                for key in ("k", "v"):
                    moved = kv_cache[key][:, src:src + ln]
                    # the ranges overlap when more rows stay than leave; only then is a temporary needed
                    kv_cache[key][:, dst:dst + ln] = moved.clone() if src - dst < ln else moved
            view_len = local_end
        is_init = fl.use_dense_init and view_len == 3 * frame_seqlen
        dense = fl.disable_monarch or is_init
        f_tied = 1 if fl.use_framewise else 3
        # dense attention keeps the cache in token order (causal_model.py:961-962), Monarch in block order
        tiling = (1, 1, 1) if dense else (f_tied, fl.h_reduce, fl.w_reduce)

        xq, xk, xv = self._project_qkv(x) if not torch.is_grad_enabled() else (self.q(x), self.k(x), self.v(x))
        q = self.ops.qk_prologue(xq, xk, xv, self.norm_q.weight, self.norm_k.weight, n, grid,
                                 current_start // frame_seqlen, self._rope, kv_cache["k"], kv_cache["v"],
                                 cache_start + local_start, *tiling, eps=self.eps)
        k_view = kv_cache["k"][:, cache_start:cache_start + view_len]
        v_view = kv_cache["v"][:, cache_start:cache_start + view_len]
        if dense:
            y = self.ops.dense(q, k_view, v_view)
        else:
            y = self.ops.monarch_cached(q, k_view, v_view, f_tied, fl.h_reduce, fl.w_reduce, h, w, fl.num_iters)
        cache_commit(kv_cache, current_end, local_end)
        return self.ops.linear(y.flatten(2), self.o)


class WanT2VCrossAttention(nn.Module):
    """Text cross-attention with K/V computed once per video and kept in `crossattn_cache`."""

    def __init__(self, dim, num_heads, eps=1e-6, ops=None):
        super().__init__()
        self.num_heads, self.head_dim = num_heads, dim // num_heads
        self.ops = ops if ops is not None else HipAttentionOps()
        self.q = nn.Linear(dim, dim)
        self.k = nn.Linear(dim, dim)
        self.v = nn.Linear(dim, dim)
        self.o = nn.Linear(dim, dim)
        self.norm_q = WanRMSNorm(dim, eps=eps)
        self.norm_k = WanRMSNorm(dim, eps=eps)

    def forward(self, x, context, crossattn_cache=None):
        b, n, d = x.size(0), self.num_heads, self.head_dim
        q = self.ops.rms_norm(self.ops.linear(x, self.q), self.norm_q.weight, self.norm_q.eps).view(b, -1, n, d)
        if crossattn_cache is not None and crossattn_cache["is_init"]:
            k, v = crossattn_cache["k"], crossattn_cache["v"]
        else:
            k = self.norm_k(self.k(context)).view(b, -1, n, d)
            v = self.v(context).view(b, -1, n, d)
            if crossattn_cache is not None:
                crossattn_cache["is_init"] = True
                crossattn_cache["k"], crossattn_cache["v"] = k, v
        return self.ops.linear(self.ops.dense(q, k, v).flatten(2), self.o)


class CausalWanAttentionBlock(nn.Module):

    def __init__(self, dim, ffn_dim, num_heads, local_attn_size=-1, sink_size=0, qk_norm=True, cross_attn_norm=True,
                 eps=1e-6, block_num=None, frame_hw=(FRAME_HEIGHT, FRAME_WIDTH), total_seq_len=None, flags=None,
                 ops=None):
        super().__init__()
        self.eps = eps
        self.ops = ops if ops is not None else HipAttentionOps()
        self.norm1 = WanLayerNorm(dim, eps)
        self.self_attn = CausalWanSelfAttention(dim, num_heads, local_attn_size, sink_size, qk_norm, eps, block_num,
                                                frame_hw, total_seq_len, flags, ops)
        self.norm3 = WanLayerNorm(dim, eps, elementwise_affine=True) if cross_attn_norm else nn.Identity()
        self.cross_attn = WanT2VCrossAttention(dim, num_heads, eps, ops)
        self.norm2 = WanLayerNorm(dim, eps)
        self.ffn = nn.Sequential(nn.Linear(dim, ffn_dim), nn.GELU(approximate='tanh'), nn.Linear(ffn_dim, dim))
        self.modulation = nn.Parameter(torch.randn(1, 6, dim) / dim ** 0.5)

    def forward(self, x, e, grid, context, kv_cache, crossattn_cache, current_start, e_summed=None, xn=None, next_mod=None):
        """x [B, L, C]; e [B, F, 6, C] per-frame modulation; e_summed: `modulation + e` where the caller has already
        formed it (the model does so for all blocks in one launch).  xn: norm1 + modulation of x where the block before
        has already produced it; next_mod = (scale, shift) of the block that follows: the block then returns
        (x, norm1 + modulation of x for that block), formed in the pass that adds the FFN's gated output (the same
        values with one read and one write of x fewer per layer)."""
        ops = self.ops
        e = (self.modulation.unsqueeze(1) + e if e_summed is None else e_summed).chunk(6, dim=2)
        y = self.self_attn(ops.ln_modulate(x, e[1], e[0], self.eps) if xn is None else xn, grid, kv_cache, current_start)
        if isinstance(self.norm3, nn.Identity):
            x = xn = ops.gate_residual(x, y, e[2])
        else:
            x, xn = ops.gate_residual_ln(x, y, e[2], self.eps, weight=self.norm3.weight, bias=self.norm3.bias)
        x, xn = ops.gate_residual_ln(x, self.cross_attn(xn, context, crossattn_cache), None, self.eps, scale=e[4], shift=e[3])
        h = ops.linear_gelu(xn, self.ffn[0])
        if next_mod is None:
            return ops.linear_gate_residual(x, h, self.ffn[2], e[5])
        if getattr(ops, "own_gemm", False):
            x = ops.linear_gate_residual(x, h, self.ffn[2], e[5])
            return x, ops.ln_modulate(x, next_mod[0], next_mod[1], self.eps)
        return ops.gate_residual_ln(x, self.ffn[2](h), e[5], self.eps, scale=next_mod[0], shift=next_mod[1])


class CausalHead(nn.Module):

    def __init__(self, dim, out_dim, patch_size, eps=1e-6):
        super().__init__()
        self.norm = WanLayerNorm(dim, eps)
        self.head = nn.Linear(dim, math.prod(patch_size) * out_dim)
        self.modulation = nn.Parameter(torch.randn(1, 2, dim) / dim ** 0.5)

    def forward(self, x, e):
        nf, fs = e.shape[1], x.shape[1] // e.shape[1]
        e = (self.modulation.unsqueeze(1) + e).chunk(2, dim=2)
        return self.head(self.norm(x).unflatten(1, (nf, fs)) * (1 + e[1]) + e[0])


WAN_CONFIGS = {
    # wan/configs/wan_t2v_1_3B.py:20-28, wan/configs/wan_t2v_14B.py:20-28
    "1.3B": dict(dim=1536, ffn_dim=8960, num_heads=12, num_layers=30),
    "14B": dict(dim=5120, ffn_dim=13824, num_heads=40, num_layers=40),
}


class CausalWanModel(nn.Module):
    fuse_next_norm = True     # block i also forms block i + 1's norm1 + modulation (same values, one pass over x fewer)

    def __init__(self, patch_size=(1, 2, 2), text_len=512, in_dim=16, dim=2048, ffn_dim=8192, freq_dim=256,
                 text_dim=4096, out_dim=16, num_heads=16, num_layers=32, local_attn_size=-1, sink_size=0, qk_norm=True,
                 cross_attn_norm=True, eps=1e-6, frame_hw=(FRAME_HEIGHT, FRAME_WIDTH), total_seq_len=None,
                 attention_flags=None, ops=None):
        super().__init__()
        if patch_size[0] != 1:
            raise NotImplementedError("temporal patching is not used by the causal generator")
        self.patch_size, self.text_len, self.in_dim, self.dim = patch_size, text_len, in_dim, dim
        self.freq_dim, self.out_dim, self.num_heads, self.num_layers = freq_dim, out_dim, num_heads, num_layers
        self.local_attn_size = local_attn_size
        self.patch_embedding = nn.Conv3d(in_dim, dim, kernel_size=patch_size, stride=patch_size)
        self.text_embedding = nn.Sequential(nn.Linear(text_dim, dim), nn.GELU(approximate='tanh'), nn.Linear(dim, dim))
        self.time_embedding = nn.Sequential(nn.Linear(freq_dim, dim), nn.SiLU(), nn.Linear(dim, dim))
        self.time_projection = nn.Sequential(nn.SiLU(), nn.Linear(dim, dim * 6))
        flags = attention_flags or {}
        self.blocks = nn.ModuleList([
            CausalWanAttentionBlock(dim, ffn_dim, num_heads, local_attn_size, sink_size, qk_norm, cross_attn_norm, eps, i,
                                    frame_hw, total_seq_len, AttentionFlags(i, **flags), ops)
            for i in range(num_layers)])
        self.head = CausalHead(dim, out_dim, patch_size, eps)
        self.init_weights()

    def init_weights(self, zero_head=True):
        """causal_model.py:1921-1943.  zero_head=False gives the output layer a Xavier init as well, which a
        random-weight end-to-end check needs (a zero head makes every latent 0)."""
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.xavier_uniform_(m.weight)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
        nn.init.xavier_uniform_(self.patch_embedding.weight.flatten(1))
        for seq in (self.text_embedding, self.time_embedding):
            for m in seq.modules():
                if isinstance(m, nn.Linear):
                    nn.init.normal_(m.weight, std=.02)
        if zero_head:
            nn.init.zeros_(self.head.head.weight)

    def _patchify(self, x):
        """[B, C, F, H, W] -> tokens [B, F*h*w, dim]; same arithmetic as the strided Conv3d."""
        B, C, Fr, H, W = x.shape
        _, ph, pw = self.patch_size
        h, w = H // ph, W // pw
        p = x.view(B, C, Fr, h, ph, w, pw).permute(0, 2, 3, 5, 1, 4, 6).reshape(B, Fr * h * w, C * ph * pw)
        wgt = self.patch_embedding.weight.view(self.dim, C * ph * pw)
        return F.linear(p, wgt, self.patch_embedding.bias), (Fr, h, w)

    def _summed_modulations(self, e0):
        """`block.modulation + e0` of every block as one [layers, B, F, 6, C] tensor (one launch per pass instead of one
        per block; the same sums).  The stacked parameters are rebuilt when one of them changes.  None where the blocks
        are not this module's own (tests plug in stand-ins) or gradients are wanted."""
        if torch.is_grad_enabled() or not all(isinstance(b, CausalWanAttentionBlock) for b in self.blocks):
            return None
        mods = [b.modulation for b in self.blocks]
        key = tuple((m.data_ptr(), m._version) for m in mods)
        if getattr(self, "_mod_stack", None) is None or self._mod_stack[0] != key:
            with torch.no_grad():
                self._mod_stack = (key, torch.stack([m.detach() for m in mods]).unsqueeze(2))     # [L, 1, 1, 6, C]
        return self._mod_stack[1] + e0.unsqueeze(0)

    def unpatchify(self, x, grid):
        """[B, L, prod(patch)*C_out] -> [B, C_out, F, H, W] (causal_model.py:1896-1919)."""
        Fr, h, w = grid
        c = self.out_dim
        u = x.view(x.shape[0], Fr, h, w, *self.patch_size, c)
        u = torch.einsum('bfhwpqrc->bcfphqwr', u)
        return u.reshape(x.shape[0], c, Fr * self.patch_size[0], h * self.patch_size[1], w * self.patch_size[2])

    @torch.no_grad()
    def forward(self, x, t, context, seq_len=None, kv_cache=None, crossattn_cache=None, current_start=0, cache_start=0):
        """x [B, C_in, F, H, W] latents of one chunk, t [B, F] timesteps, context [B, L_text, text_dim];
        kv_cache / crossattn_cache: per-layer lists of dicts (pipeline/causal_inference.py:288-322)."""
        if kv_cache is None:
            raise NotImplementedError("only the KV-cache inference path is built")
        x, grid = self._patchify(x)
        e = self.time_embedding(sinusoidal_embedding_1d(self.freq_dim, t.flatten()).type_as(x))
        e0 = self.time_projection(e).unflatten(1, (6, self.dim)).unflatten(0, t.shape)
        if context.shape[1] < self.text_len:
            context = torch.cat([context, context.new_zeros(context.shape[0], self.text_len - context.shape[1],
                                                            context.shape[2])], dim=1)
        context = self.text_embedding(context)
        e_all = self._summed_modulations(e0)
        if e_all is None:
            for i, block in enumerate(self.blocks):
                x = block(x, e0, grid, context, kv_cache[i], crossattn_cache[i] if crossattn_cache is not None else None,
                          current_start)
        else:
            # every block but the last also forms the next block's normalised, modulated input
            xn, last = None, len(self.blocks) - 1
            for i, block in enumerate(self.blocks):
                nxt = None if i == last or not self.fuse_next_norm else (e_all[i + 1][:, :, 1:2], e_all[i + 1][:, :, 0:1])
                r = block(x, e0, grid, context, kv_cache[i], crossattn_cache[i] if crossattn_cache is not None else None,
                          current_start, e_summed=e_all[i], xn=xn, next_mod=nxt)
                x, xn = r if nxt is not None else (r, None)
        x = self.head(x, e.unflatten(0, t.shape).unsqueeze(2))
        return self.unpatchify(x.flatten(1, 2) if x.dim() == 4 else x, grid)
