"""Dense attention operators with the reference's call signatures.

    attention                     <->  wan/modules/attention.py:141-187
    full_attention_with_kv_cache  <->  wan/modules/attn_patch.py:416-419
"""
import ctypes as C
import warnings

import torch

from . import lib as _l
from .monarch_attn import _DT, _check4, _stream, scratch as _scratch


def _dense_desc(q, k, v, out, sm_scale):
    d = _l.DenseDesc()
    d.dtype = _DT[q.dtype]
    d.B, d.q_tokens, d.H, d.D = q.shape
    d.kv_tokens = k.shape[1]
    d.sm_scale = float(sm_scale)
    d.q_stride = _l.strides3(q)
    d.k_stride = _l.strides3(k)
    d.v_stride = _l.strides3(v)
    d.o_stride = _l.strides3(out)
    return d


def _dense_fwd(q, k, v, sm_scale, want_lse):
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty((q.shape[0], q.shape[2], q.shape[1]), dtype=torch.float32, device=q.device) if want_lse else None
    d = _dense_desc(q, k, v, out, sm_scale)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_dense_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                         lse.data_ptr() if want_lse else None, _stream(q)))
    return out, lse


def _dense_bwd(q, k, v, out, lse, dout, sm_scale, kv0=0, kv1=None):
    """Raw call of sfm_dense_bwd: (dq float32, dk, dv); dk, dv cover keys [kv0, kv1)."""
    if kv1 is None:
        kv1 = k.shape[1]
    if dout.stride() != out.stride():
        dout = dout.contiguous()
        out = out.contiguous()
    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    dk = torch.empty((k.shape[0], kv1 - kv0, k.shape[2], k.shape[3]), dtype=k.dtype, device=k.device)
    dv = torch.empty_like(dk)
    bd = _l.DenseBwdDesc()
    bd.fwd = _dense_desc(q, k, v, out, sm_scale)
    bd.dq_stride = _l.strides3(dq)
    bd.dkv_stride = _l.strides3(dk)
    bd.kv_grad_start, bd.kv_grad_end = kv0, kv1
    n = C.c_size_t(0)
    _l.check(_l.load().sfm_dense_bwd_workspace_bytes(C.byref(bd), C.byref(n)))
    ws = _scratch(n.value, q.device)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_dense_bwd(C.byref(bd), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                                         dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ws.data_ptr(), n.value,
                                         _stream(q)))
    return dq, dk, dv


class _DenseFn(torch.autograd.Function):
    """attention under autograd: keeps q, k, v, the output and its log-sum-exp, as `_attention.forward` does
    (attn_patch.py:346-351)."""

    @staticmethod
    def forward(ctx, q, k, v, sm_scale):
        out, lse = _dense_fwd(q, k, v, sm_scale, True)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.sm_scale = sm_scale
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        dq, dk, dv = _dense_bwd(q, k, v, out, lse, dout, ctx.sm_scale)
        return dq.to(q.dtype), dk, dv, None


class _DenseCacheFn(torch.autograd.Function):
    """full_attention_with_kv_cache under autograd (`_attention`, attn_patch.py:305-413): the caches are written in place
    and saved by reference; with grad_only_new_kv only the keys written by this call get gradients (:362-364)."""

    @staticmethod
    def forward(ctx, q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale, grad_only_new_kv):
        out, lse = _dense_cache_fwd(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale, True)
        ctx.save_for_backward(q, k_cache, v_cache, out, lse)
        ctx.cfg = (start_idx, end_idx, sm_scale, grad_only_new_kv)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k_cache, v_cache, out, lse = ctx.saved_tensors
        start_idx, end_idx, sm_scale, grad_only_new_kv = ctx.cfg
        if grad_only_new_kv:
            dq, dk_new, dv_new = _dense_bwd(q, k_cache, v_cache, out, lse, dout, sm_scale, start_idx, end_idx)
            dk_cache = dv_cache = None
        else:
            dq, dk_cache, dv_cache = _dense_bwd(q, k_cache, v_cache, out, lse, dout, sm_scale)
            dk_new, dv_new = dk_cache[:, start_idx:end_idx], dv_cache[:, start_idx:end_idx]
        return dq.to(q.dtype), dk_cache, dv_cache, dk_new, dv_new, None, None, None, None


def _needs_grad(*ts):
    return torch.is_grad_enabled() and any(t.requires_grad for t in ts)


def attention(q, k, v, q_lens=None, k_lens=None, dropout_p=0., softmax_scale=None, q_scale=None, causal=False,
              window_size=(-1, -1), deterministic=False, dtype=torch.bfloat16, fa_version=None, return_lse=False):
    """softmax(q k^T * scale) v on [B, L, H, D] tensors.  Dtypes as in the reference's flash path (attention.py:62-70,
    135-138): float16 / bfloat16 inputs are used as they are, anything else is cast to `dtype`, and the result comes
    back in q's original dtype.  dtype=torch.float32 (which the reference does not accept) keeps fp32 inputs on the
    fp32 kernel."""
    if causal or dropout_p != 0. or window_size != (-1, -1):
        raise NotImplementedError("only non-causal, dropout-free, full-window attention is built")
    if q_lens is not None or k_lens is not None:
        warnings.warn("q_lens / k_lens are ignored (as in the reference's SDPA branch)")
    _check4("q", q)
    _check4("k", k, None, q.device)
    _check4("v", v, None, q.device)
    half_dtypes = (torch.float16, torch.bfloat16)
    if dtype not in half_dtypes + (torch.float32,):
        raise ValueError("dtype must be float16, bfloat16 or float32")
    out_dtype = q.dtype
    if q_scale is not None:
        q = q * q_scale
    q = q if q.dtype in half_dtypes else q.to(dtype)
    k, v = k.to(q.dtype), v.to(q.dtype)
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** -0.5
    if _needs_grad(q, k, v):
        if return_lse:
            raise NotImplementedError("return_lse is not differentiable")
        return _DenseFn.apply(q, k, v, softmax_scale).to(out_dtype)
    out, lse = _dense_fwd(q, k, v, softmax_scale, return_lse)
    out = out.to(out_dtype)
    return (out, lse) if return_lse else out


def full_attention_with_kv_cache(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale=None,
                                 grad_only_new_kv=False):
    """k_cache/v_cache[:, start_idx:end_idx] = new_k/new_v (in place), then dense attention over the view."""
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    if _needs_grad(q, k_cache, v_cache, new_k, new_v):
        return _DenseCacheFn.apply(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale, grad_only_new_kv)
    return _dense_cache_fwd(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale, False)[0]


def _dense_cache_fwd(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale, want_lse):
    _check4("q", q)
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache), ("new_k", new_k), ("new_v", new_v)):
        _check4(name, t, q.dtype, q.device)
    if not (0 <= start_idx <= end_idx <= k_cache.shape[1]):
        raise ValueError("start_idx / end_idx out of range")
    if new_k.shape[1] != end_idx - start_idx:
        raise ValueError("new_k does not hold end_idx - start_idx tokens")
    if new_k.stride() != new_v.stride():
        new_k, new_v = new_k.contiguous(), new_v.contiguous()
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty((q.shape[0], q.shape[2], q.shape[1]), dtype=torch.float32, device=q.device) if want_lse else None
    d = _dense_desc(q, k_cache, v_cache, out, sm_scale)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_full_attention_with_kv_cache(
            C.byref(d), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), new_k.data_ptr(), new_v.data_ptr(),
            _l.strides3(new_k), start_idx, end_idx, out.data_ptr(), lse.data_ptr() if want_lse else None, _stream(q)))
    return out, lse
