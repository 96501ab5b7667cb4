"""Dense attention operators with the reference's call signatures.

    attention                     <->  wan/modules/attention.py:141-187
    full_attention_with_kv_cache  <->  wan/modules/attn_patch.py:416-419
"""
import ctypes as C
import warnings

import torch

from . import lib as _l
from .monarch_attn import _DT, _check4, _stream


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


def attention(q, k, v, q_lens=None, k_lens=None, dropout_p=0., softmax_scale=None, q_scale=None, causal=False,
              window_size=(-1, -1), deterministic=False, dtype=torch.bfloat16, fa_version=None, return_lse=False):
    """softmax(q k^T * scale) v on [B, L, H, D] tensors; inputs are cast to `dtype` like the reference does."""
    if causal or dropout_p != 0. or window_size != (-1, -1):
        raise NotImplementedError("only non-causal, dropout-free, full-window attention is built")
    if q_lens is not None or k_lens is not None:
        warnings.warn("q_lens / k_lens are ignored (as in the reference's SDPA branch)")
    _check4("q", q)
    _check4("k", k, None, q.device)
    _check4("v", v, None, q.device)
    if q_scale is not None:
        q = q * q_scale
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** -0.5
    out = torch.empty(q.shape, dtype=dtype, device=q.device)
    lse = torch.empty((q.shape[0], q.shape[2], q.shape[1]), dtype=torch.float32, device=q.device) if return_lse else None
    d = _dense_desc(q, k, v, out, softmax_scale)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_dense_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                         lse.data_ptr() if return_lse else None, _stream(q)))
    return (out, lse) if return_lse else out


def full_attention_with_kv_cache(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale=None,
                                 grad_only_new_kv=False):
    """k_cache/v_cache[:, start_idx:end_idx] = new_k/new_v (in place), then dense attention over the view."""
    if torch.is_grad_enabled() and (q.requires_grad or new_k.requires_grad or new_v.requires_grad):
        raise NotImplementedError("forward only: call under torch.no_grad()")
    _check4("q", q)
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache), ("new_k", new_k), ("new_v", new_v)):
        _check4(name, t, q.dtype, q.device)
    if not (0 <= start_idx <= end_idx <= k_cache.shape[1]):
        raise ValueError("start_idx / end_idx out of range")
    if new_k.shape[1] != end_idx - start_idx:
        raise ValueError("new_k does not hold end_idx - start_idx tokens")
    if new_k.stride() != new_v.stride():
        new_k, new_v = new_k.contiguous(), new_v.contiguous()
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    d = _dense_desc(q, k_cache, v_cache, out, sm_scale)
    with torch.cuda.device(q.device):
        _l.check(_l.load().sfm_full_attention_with_kv_cache(
            C.byref(d), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), new_k.data_ptr(), new_v.data_ptr(),
            _l.strides3(new_k), start_idx, end_idx, out.data_ptr(), None, _stream(q)))
    return out
