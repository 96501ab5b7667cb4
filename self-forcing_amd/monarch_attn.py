"""Monarch attention operators with the reference's call signatures.

    monarch_attn_with_kv_cache  <->  wan/modules/monarch_attn.py:1778-1796
    monarch_attn                <->  wan/modules/monarch_attn.py:1753-1776

Inputs are [B, S, H, D] CUDA tensors (bf16 / fp16 / fp32, head_dim contiguous) in token order;
the KV cache holds rows in Monarch block order and is updated in place.  Under autograd the operators
are torch.autograd.Functions whose backward runs the library's backward kernels (num_iters == 1).
num_iters > 1 runs the alternating refinement the reference implements in pure torch
(monarch_attn_slow, wan/modules/monarch_attn.py:1705-1751) as HIP kernels; under autograd its forward is still the HIP
kernels and its backward differentiates a torch restatement of the passes on the GPU (the reference's own refinement is
differentiable torch and has no backward kernels either).
"""
import ctypes as C

import torch

from . import lib as _l

_DT = {torch.bfloat16: _l.SFM_BF16, torch.float16: _l.SFM_F16, torch.float32: _l.SFM_F32}


def _check4(name, t, dtype=None, device=None):
    if not isinstance(t, torch.Tensor) or t.dim() != 4:
        raise ValueError(f"{name} must be a [B, S, H, D] tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    if t.stride(3) != 1:
        raise ValueError(f"{name}: head_dim must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name}: dtype {t.dtype} differs from q's {dtype}")
    if device is not None and t.device != device:
        raise ValueError(f"{name}: device {t.device} differs from q's {device}")


def _desc(q, k, v, out, f_tied, h_reduce, w_reduce, h, w, sm_scale, kv_block_order, causal_block_frames, num_iters=1,
          one_kernel=False):
    if q.dtype not in _DT:
        raise ValueError(f"unsupported dtype {q.dtype}")
    d = _l.MonarchDesc()
    d.dtype = _DT[q.dtype]
    d.B, d.q_tokens, d.H, d.D = q.shape
    d.kv_tokens = k.shape[1]
    d.tiling = _l.Tiling(f_tied, h_reduce, w_reduce, h, w)
    d.kv_block_order = kv_block_order
    d.causal_block_frames = causal_block_frames
    d.sm_scale = float(sm_scale)
    d.num_iters = int(num_iters)
    d.flags = _l.SFM_MONARCH_ONE_KERNEL if one_kernel else 0
    d.q_stride = _l.strides3(q)
    d.k_stride = _l.strides3(k)
    d.v_stride = _l.strides3(v)
    d.o_stride = _l.strides3(out)
    return d


_SCRATCH = {}


def scratch(nbytes, device):
    """The library's workspace for a call on `device`'s current stream: one grow-only byte buffer per (device, stream),
    so that steady-state calls allocate nothing (a caller recording a HIP graph warms the buffer up with one eager
    call first).  Calls on one stream are ordered, so they can share it; `release_scratch()` gives the memory back."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(device).cuda_stream)
    buf = _SCRATCH.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = _SCRATCH[key] = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)
    return buf


def release_scratch():
    _SCRATCH.clear()


def monarch_workspace_bytes(desc, heads_per_pass=0):
    n = C.c_size_t(0)
    _l.check(_l.load().sfm_monarch_workspace_bytes(C.byref(desc), heads_per_pass, C.byref(n)))
    return n.value


def _stream(t):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _from_block_order(x, f_tied, h_reduce, w_reduce, h, w):
    """Inverse of the reference's rearrangement (monarch_attn.py:1696-1703) on a [B, n, H, D] tensor."""
    if f_tied == 1 and h_reduce == 1 and w_reduce == 1:
        return x
    B, n, H, D = x.shape
    x = x.reshape(B, -1, h_reduce, w_reduce, f_tied, h // h_reduce, w // w_reduce, H, D)
    return x.permute(0, 1, 4, 2, 5, 3, 6, 7, 8).reshape(B, n, H, D)


def _causal_block_frames(q, k, tiling, block_causal_size, num_iters=1):
    """Block-causal size in tokens -> block-frames, with the reference's checks (monarch_attn.py:1485-1491)."""
    if block_causal_size is None:
        return 0
    f_tied, h_reduce, w_reduce, h, w = tiling
    per_block = f_tied * (h // h_reduce) * (w // w_reduce)
    if q.shape[1] % block_causal_size:
        raise ValueError(f"block_causal_size ({block_causal_size}) must divide sequence length ({q.shape[1]})")
    if k.shape[1] != q.shape[1]:
        raise ValueError("causal attention needs kv length equal to q length")
    if block_causal_size % per_block:
        raise ValueError("block_causal_size must align with Monarch block sizes")
    if num_iters != 1:
        raise ValueError("causal currently only supported for num_iters=1")
    return block_causal_size // per_block


def kv_cache_write(new_k, new_v, k_cache, v_cache, start_idx, end_idx, f_tied, h_reduce, w_reduce, h, w):
    """new_k / new_v (token order) into k_cache / v_cache[:, start_idx:end_idx] in Monarch block order
    (monarch_attn.py:1784-1785, 1230-1231)."""
    if new_k.stride() != new_v.stride():
        new_k, new_v = new_k.contiguous(), new_v.contiguous()
    if k_cache.stride() != v_cache.stride():
        raise ValueError("k_cache and v_cache must share their strides")
    B, _, H, D = new_k.shape
    with torch.cuda.device(new_k.device):
        _l.check(_l.load().sfm_kv_cache_write(_DT[new_k.dtype], B, H, D, C.byref(_l.Tiling(f_tied, h_reduce, w_reduce, h, w)),
                                              new_k.data_ptr(), new_v.data_ptr(), _l.strides3(new_k), k_cache.data_ptr(),
                                              v_cache.data_ptr(), _l.strides3(k_cache), k_cache.shape[1], start_idx, end_idx,
                                              _stream(new_k)))


def _monarch_fwd_stats(q, k, v, tiling, sm_scale, kv_block_order, cbf, heads_per_pass=0):
    """Forward for autograd: returns (out, stats) where stats is the opaque row-statistics tensor that
    sfm_monarch_bwd_saved takes, or None when the forward that runs for these tensors produces none (the
    reference's forward keeps z and z_lse the same way, monarch_attn.py:1309-1317)."""
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    d = _desc(q, k, v, out, *tiling, sm_scale, kv_block_order, cbf, 1)
    n = C.c_size_t(0)
    _l.check(_l.load().sfm_monarch_stats_bytes(C.byref(d), C.byref(n)))
    nbytes = monarch_workspace_bytes(d, heads_per_pass)
    ws = scratch(nbytes, q.device)
    stats = torch.empty(n.value // 4, dtype=torch.float32, device=q.device) if n.value else None
    with torch.cuda.device(q.device):
        if stats is None:
            _l.check(_l.load().sfm_monarch_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                               ws.data_ptr(), nbytes, _stream(q)))
        else:
            _l.check(_l.load().sfm_monarch_fwd_stats(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                     stats.data_ptr(), ws.data_ptr(), nbytes, _stream(q)))
    return out, stats


def _monarch_bwd(q, k, v, dout, tiling, sm_scale, kv_block_order, cbf, kv_f0=0, kv_f1=None, heads_per_pass=0, out=None,
                 stats=None):
    """Raw call of sfm_monarch_bwd (or sfm_monarch_bwd_saved when the forward's `out` and `stats` are given): returns
    (dq float32, dk, dv); dk, dv cover kv block-frames [kv_f0, kv_f1) in the row order of k."""
    f_tied, h_reduce, w_reduce, h, w = tiling
    per_frame = f_tied * (h // h_reduce) * (w // w_reduce)
    nf = k.shape[1] // per_frame
    if kv_f1 is None:
        kv_f1 = nf
    if dout.stride(3) != 1 or (out is not None and dout.stride() != out.stride()):
        dout = dout.contiguous()
    if out is not None and out.stride() != dout.stride():
        out = out.contiguous()
    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    dk = torch.empty((k.shape[0], (kv_f1 - kv_f0) * per_frame, k.shape[2], k.shape[3]), dtype=k.dtype, device=k.device)
    dv = torch.empty_like(dk)
    bd = _l.MonarchBwdDesc()
    bd.fwd = _desc(q, k, v, dout, f_tied, h_reduce, w_reduce, h, w, sm_scale, kv_block_order, cbf)
    bd.dq_stride = _l.strides3(dq)
    bd.dkv_stride = _l.strides3(dk)
    bd.kv_grad_frame_start, bd.kv_grad_frame_end = kv_f0, kv_f1
    n = C.c_size_t(0)
    _l.check(_l.load().sfm_monarch_bwd_workspace_bytes(C.byref(bd), heads_per_pass, C.byref(n)))
    ws = scratch(n.value, q.device)
    with torch.cuda.device(q.device):
        if out is None or stats is None:
            _l.check(_l.load().sfm_monarch_bwd(C.byref(bd), q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(),
                                               dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), n.value,
                                               _stream(q)))
        else:
            _l.check(_l.load().sfm_monarch_bwd_saved(C.byref(bd), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                     stats.data_ptr(), dout.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                                     dv.data_ptr(), ws.data_ptr(), n.value, _stream(q)))
    return dq, dk, dv


class _MonarchFn(torch.autograd.Function):
    """monarch_attn under autograd (_attention_no_cache, monarch_attn.py:1472-1693)."""

    @staticmethod
    def forward(ctx, q, k, v, tiling, sm_scale, block_causal_size, heads_per_pass, kv_block_order):
        cbf = _causal_block_frames(q, k, tiling, block_causal_size)
        _check4("q", q)
        _check4("k", k, q.dtype, q.device)
        _check4("v", v, q.dtype, q.device)
        if k.stride() != v.stride():
            k, v = k.contiguous(), v.contiguous()
        out, stats = _monarch_fwd_stats(q, k, v, tiling, sm_scale, 1 if kv_block_order else 0, cbf, heads_per_pass)
        ctx.has_stats = stats is not None
        if stats is not None:
            ctx.save_for_backward(q, k, v, out, stats)
        else:
            ctx.save_for_backward(q, k, v)
        ctx.cfg = (tiling, sm_scale, cbf, kv_block_order)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, *kept = ctx.saved_tensors
        out, stats = kept if ctx.has_stats else (None, None)
        tiling, sm_scale, cbf, kv_block_order = ctx.cfg
        dq, dk, dv = _monarch_bwd(q, k, v, dout, tiling, sm_scale, 1 if kv_block_order else 0, cbf, out=out, stats=stats)
        return dq.to(q.dtype), dk, dv, None, None, None, None, None


class _MonarchCacheFn(torch.autograd.Function):
    """monarch_attn_with_kv_cache under autograd (_attention_with_cache, monarch_attn.py:1225-1470): the caches
    are written in place in the forward and saved by reference, as the reference does; with grad_only_new_kv
    only the block-frames written by this call get K/V gradients (:1364-1374)."""

    @staticmethod
    def forward(ctx, q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, tiling, sm_scale, grad_only_new_kv,
                heads_per_pass):
        _check4("q", q)
        for name, t in (("k_cache", k_cache), ("v_cache", v_cache), ("new_k", new_k), ("new_v", new_v)):
            _check4(name, t, q.dtype, q.device)
        if k_cache.shape != v_cache.shape or new_k.shape != new_v.shape:
            raise ValueError("k/v shapes differ")
        if new_k.shape[1] != end_idx - start_idx:
            raise ValueError(f"new_k holds {new_k.shape[1]} tokens but end_idx - start_idx = {end_idx - start_idx}")
        kv_cache_write(new_k, new_v, k_cache, v_cache, start_idx, end_idx, *tiling)
        out, stats = _monarch_fwd_stats(q, k_cache, v_cache, tiling, sm_scale, 1, 0, heads_per_pass)
        ctx.has_stats = stats is not None
        if stats is not None:
            ctx.save_for_backward(q, k_cache, v_cache, out, stats)
        else:
            ctx.save_for_backward(q, k_cache, v_cache)
        ctx.cfg = (start_idx, end_idx, tiling, sm_scale, grad_only_new_kv)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k_cache, v_cache, *kept = ctx.saved_tensors
        out, stats = kept if ctx.has_stats else (None, None)
        start_idx, end_idx, tiling, sm_scale, grad_only_new_kv = ctx.cfg
        f_tied, h_reduce, w_reduce, h, w = tiling
        per_frame = f_tied * (h // h_reduce) * (w // w_reduce)
        if grad_only_new_kv:
            dq, dk, dv = _monarch_bwd(q, k_cache, v_cache, dout, tiling, sm_scale, 1, 0, start_idx // per_frame,
                                      end_idx // per_frame, out=out, stats=stats)
            dk_cache = dv_cache = None
            dk_new, dv_new = dk, dv
        else:
            dq, dk_cache, dv_cache = _monarch_bwd(q, k_cache, v_cache, dout, tiling, sm_scale, 1, 0, out=out, stats=stats)
            dk_new, dv_new = dk_cache[:, start_idx:end_idx], dv_cache[:, start_idx:end_idx]
        dk_new = _from_block_order(dk_new, *tiling)
        dv_new = _from_block_order(dv_new, *tiling)
        return dq.to(q.dtype), dk_cache, dv_cache, dk_new, dv_new, None, None, None, None, None, None


def _to_block_order(x, f_tied, h_reduce, w_reduce, h, w):
    """The reference's rearrangement (monarch_attn.py:1696-1703) of a token-order [B, n, H, D] tensor: rows in Monarch
    block order."""
    if f_tied == 1 and h_reduce == 1 and w_reduce == 1:
        return x
    B, n, H, D = x.shape
    x = x.reshape(B, -1, f_tied, h_reduce, h // h_reduce, w_reduce, w // w_reduce, H, D)
    return x.permute(0, 1, 3, 5, 2, 4, 6, 7, 8).reshape(B, n, H, D)


def _refinement_torch(qb, kb, vb, sm_scale, num_iters):
    """The refinement passes (monarch_attn.py:1705-1751) as differentiable torch ops on block-ordered tensors
    qb [B, a, b1, b2, H, D], kb / vb [B, f, b1, b2, H, D]; used for gradients only.  Pass p forms the right factor R from
    the per-block query representatives of pass p - 1 (first pass: the queries themselves, weight 1), then the left
    factor L; the last pass's factors are applied to V."""
    rs = float(sm_scale) ** 0.5
    q = qb.permute(0, 4, 1, 2, 3, 5) * rs                 # [B, H, a, i, j, D]
    k = kb.permute(0, 4, 1, 2, 3, 5) * rs                 # [B, H, f, k, l, D]
    v = vb.permute(0, 4, 1, 2, 3, 5)
    nf = k.shape[2]
    rep = q.unsqueeze(3).expand(-1, -1, -1, nf, -1, -1, -1)          # [B, H, a, f, k, j, D]: block row k of the queries
    inv_w = q.new_full((), 1.0 / (1.0 + 1e-6))
    for it in range(num_iters):
        z = torch.einsum("bhafkjd,bhfkld->bhafkjl", rep, k) * inv_w
        log_r = torch.log_softmax(z, -1)
        r = log_r.exp()
        kbar = torch.einsum("bhafkjl,bhfkld->bhafkjd", r, k)
        neg_h = (r * log_r).sum(-1)                                   # [B, H, a, f, k, j]
        s2 = torch.einsum("bhaijd,bhafkjd->bhaijfk", q, kbar) - neg_h.permute(0, 1, 2, 5, 3, 4).unsqueeze(3)
        left = torch.softmax(s2.flatten(5), -1).reshape(s2.shape)    # [B, H, a, i, j, f, k]
        if it + 1 < num_iters:
            rep = torch.einsum("bhaijfk,bhaijd->bhafkjd", left, q)
            inv_w = torch.clamp(1.0 / (left.sum(3).permute(0, 1, 2, 4, 5, 3) + 1e-6), max=1e4).unsqueeze(-1)
    y = torch.einsum("bhafkjl,bhfkld->bhafkjd", r, v)
    return torch.einsum("bhaijfk,bhafkjd->bhaijd", left, y).permute(0, 2, 3, 4, 1, 5)


def _refinement_grads(q, k, v, dout, tiling, sm_scale, num_iters, kv_block_order):
    """(dq, dk, dv) of the refinement for token-order q / dout and k, v in token order or (kv_block_order) block order;
    gradients come back in the same orders, float32."""
    f_tied, h_reduce, w_reduce, h, w = tiling
    b1, b2 = f_tied * (h // h_reduce), w // w_reduce
    with torch.enable_grad():
        q_, k_, v_ = (t.detach().float().requires_grad_(True) for t in (q, k, v))
        B, _, H, D = q.shape
        qb = _to_block_order(q_, *tiling).reshape(B, -1, b1, b2, H, D)
        kb = (k_ if kv_block_order else _to_block_order(k_, *tiling)).reshape(B, -1, b1, b2, H, D)
        vb = (v_ if kv_block_order else _to_block_order(v_, *tiling)).reshape(B, -1, b1, b2, H, D)
        ob = _refinement_torch(qb, kb, vb, sm_scale, num_iters)
        out = _from_block_order(ob.reshape(B, -1, H, D), *tiling)
        return torch.autograd.grad(out, (q_, k_, v_), dout.float())


class _MonarchIterFn(torch.autograd.Function):
    """monarch_attn with num_iters > 1 under autograd: HIP kernels forward, torch restatement for the gradients."""

    @staticmethod
    def forward(ctx, q, k, v, tiling, sm_scale, num_iters, heads_per_pass, kv_block_order):
        with torch.no_grad():
            out = monarch_attn(q, k, v, *tiling, sm_scale=sm_scale, num_iters=num_iters, heads_per_pass=heads_per_pass,
                               kv_block_order=kv_block_order)
        ctx.save_for_backward(q, k, v)
        ctx.cfg = (tiling, sm_scale, num_iters, kv_block_order)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v = ctx.saved_tensors
        tiling, sm_scale, num_iters, kv_block_order = ctx.cfg
        dq, dk, dv = _refinement_grads(q, k, v, dout, tiling, sm_scale, num_iters, kv_block_order)
        return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None, None, None, None, None


class _MonarchCacheIterFn(torch.autograd.Function):
    """monarch_attn_with_kv_cache with num_iters > 1 under autograd (cache written in place in the forward)."""

    @staticmethod
    def forward(ctx, q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, tiling, sm_scale, num_iters, grad_only_new_kv,
                heads_per_pass):
        with torch.no_grad():
            out = monarch_attn_with_kv_cache(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, *tiling, sm_scale=sm_scale,
                                             num_iters=num_iters, heads_per_pass=heads_per_pass)
        ctx.save_for_backward(q, k_cache, v_cache)
        ctx.cfg = (start_idx, end_idx, tiling, sm_scale, num_iters, grad_only_new_kv)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k_cache, v_cache = ctx.saved_tensors
        start_idx, end_idx, tiling, sm_scale, num_iters, grad_only_new_kv = ctx.cfg
        dq, dkc, dvc = _refinement_grads(q, k_cache, v_cache, dout, tiling, sm_scale, num_iters, True)
        dk_new = _from_block_order(dkc[:, start_idx:end_idx], *tiling).to(k_cache.dtype)
        dv_new = _from_block_order(dvc[:, start_idx:end_idx], *tiling).to(v_cache.dtype)
        if grad_only_new_kv:
            dkc = dvc = None
        else:
            dkc, dvc = dkc.to(k_cache.dtype), dvc.to(v_cache.dtype)
        return dq.to(q.dtype), dkc, dvc, dk_new, dv_new, None, None, None, None, None, None, None


def _needs_grad(*ts):
    return torch.is_grad_enabled() and any(t.requires_grad for t in ts)


def monarch_attn_with_kv_cache(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, f_tied, h_reduce, w_reduce, h, w,
                               sm_scale=None, num_iters=1, grad_only_new_kv=False, heads_per_pass=0, one_kernel=False):
    """Writes new_k/new_v into k_cache/v_cache[:, start_idx:end_idx] (block order, in place) and
    returns one-iteration Monarch attention of q against the whole cache view.  `heads_per_pass` and `one_kernel`
    (no counterparts in the reference) bound the scratch and select the forward that keeps its intermediates in LDS."""
    if _needs_grad(q, k_cache, v_cache, new_k, new_v):
        if sm_scale is None:
            sm_scale = q.shape[-1] ** -0.5
        if num_iters != 1:
            return _MonarchCacheIterFn.apply(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx,
                                             (f_tied, h_reduce, w_reduce, h, w), sm_scale, num_iters, grad_only_new_kv,
                                             heads_per_pass)
        return _MonarchCacheFn.apply(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx,
                                     (f_tied, h_reduce, w_reduce, h, w), sm_scale, grad_only_new_kv, heads_per_pass)
    _check4("q", q)
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache), ("new_k", new_k), ("new_v", new_v)):
        _check4(name, t, q.dtype, q.device)
    if k_cache.shape != v_cache.shape or new_k.shape != new_v.shape:
        raise ValueError("k/v shapes differ")
    if new_k.stride() != new_v.stride():
        new_v = new_v.contiguous()
        new_k = new_k.contiguous()
    if new_k.shape[1] != end_idx - start_idx:
        raise ValueError(f"new_k holds {new_k.shape[1]} tokens but end_idx - start_idx = {end_idx - start_idx}")
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    d = _desc(q, k_cache, v_cache, out, f_tied, h_reduce, w_reduce, h, w, sm_scale, 1, 0, num_iters, one_kernel)
    nbytes = monarch_workspace_bytes(d, heads_per_pass)
    ws = scratch(nbytes, q.device)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_monarch_attn_with_kv_cache(
            C.byref(d), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), new_k.data_ptr(), new_v.data_ptr(),
            _l.strides3(new_k), start_idx, end_idx, out.data_ptr(), ws.data_ptr(), nbytes, _stream(q)))
    return out


def monarch_attn_with_kv_cache_static(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, f_tied, h_reduce, w_reduce, h, w,
                                      sm_scale=None, num_iters=1, out=None):
    """monarch_attn_with_kv_cache for callers that cannot allocate (HIP graph capture, serving loops): the scratch
    is the library's own per-GPU array (lib.STATIC_SCRATCH_BYTES) instead of a fresh tensor, and with `out` given
    nothing is allocated at all.  No autograd.  Calls on one GPU share the scratch and must not overlap."""
    _check4("q", q)
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache), ("new_k", new_k), ("new_v", new_v)):
        _check4(name, t, q.dtype, q.device)
    if k_cache.shape != v_cache.shape or new_k.shape != new_v.shape or new_k.stride() != new_v.stride():
        raise ValueError("k/v shapes or strides differ")
    if new_k.shape[1] != end_idx - start_idx:
        raise ValueError(f"new_k holds {new_k.shape[1]} tokens but end_idx - start_idx = {end_idx - start_idx}")
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    else:
        _check4("out", out, q.dtype, q.device)
        if out.shape != q.shape:
            raise ValueError("out must have q's shape")
    d = _desc(q, k_cache, v_cache, out, f_tied, h_reduce, w_reduce, h, w, sm_scale, 1, 0, num_iters)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_monarch_attn_with_kv_cache_static(
            C.byref(d), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), new_k.data_ptr(), new_v.data_ptr(),
            _l.strides3(new_k), start_idx, end_idx, out.data_ptr(), _stream(q)))
    return out


def monarch_attn(q, k, v, f_tied, h_reduce, w_reduce, h, w, sm_scale=None, block_causal_size=None, num_iters=1,
                 heads_per_pass=0, kv_block_order=False, one_kernel=False):
    """One-iteration Monarch attention without a cache write; `block_causal_size` (tokens) masks
    block-frames of later causal blocks.  `kv_block_order=True` (no counterpart in the reference) says
    that k, v are a KV-cache view whose rows are already in Monarch block order, e.g. after
    prologue.qk_prologue wrote them."""
    if _needs_grad(q, k, v):
        if sm_scale is None:
            sm_scale = q.shape[-1] ** -0.5
        if num_iters != 1:
            if block_causal_size is not None:
                raise ValueError("causal currently only supported for num_iters=1")
            return _MonarchIterFn.apply(q, k, v, (f_tied, h_reduce, w_reduce, h, w), sm_scale, num_iters, heads_per_pass,
                                        kv_block_order)
        return _MonarchFn.apply(q, k, v, (f_tied, h_reduce, w_reduce, h, w), sm_scale, block_causal_size,
                                heads_per_pass, kv_block_order)
    _check4("q", q)
    _check4("k", k, q.dtype, q.device)
    _check4("v", v, q.dtype, q.device)
    if k.stride() != v.stride():
        k, v = k.contiguous(), v.contiguous()
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    cbf = _causal_block_frames(q, k, (f_tied, h_reduce, w_reduce, h, w), block_causal_size, num_iters)
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    d = _desc(q, k, v, out, f_tied, h_reduce, w_reduce, h, w, sm_scale, 1 if kv_block_order else 0, cbf, num_iters, one_kernel)
    nbytes = monarch_workspace_bytes(d, heads_per_pass)
    ws = scratch(nbytes, q.device)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_monarch_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                           ws.data_ptr(), nbytes, _stream(q)))
    return out
