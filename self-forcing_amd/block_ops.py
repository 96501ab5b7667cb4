"""Fused element-wise operators of the causal Wan block (LayerNorm + adaLN modulation, gated residual,
RMSNorm); counterparts of the eager chains in wan/modules/causal_model.py:1176-1205 and
wan/modules/model.py:462-478.  [B, L, C] tensors, modulation rows [B, F, 1, C] (one per latent frame)."""
import torch

from . import lib as _l
from .monarch_attn import _DT, _stream


def _rows(x):
    if not x.is_cuda:
        raise ValueError("the block operators run on the GPU")
    if x.dtype not in _DT:
        raise ValueError(f"unsupported dtype {x.dtype}")
    if x.dim() != 3 or x.stride(2) != 1 or x.stride(0) != x.shape[1] * x.stride(1):
        raise ValueError("expected a [B, L, C] tensor with contiguous channels and evenly strided rows")
    return x.shape[0] * x.shape[1], x.shape[2], x.stride(1)


def _like(name, t, x):
    """The kernels read every operand in x's dtype: another dtype (or device) would be misread, not converted."""
    if t.dtype != x.dtype or t.device != x.device:
        raise ValueError(f"{name}: {t.dtype} on {t.device}, expected {x.dtype} on {x.device} like the activations")
    return t


def _vec(name, t, x):
    _like(name, t, x)
    if t.dim() != 1 or t.shape[0] != x.shape[2]:
        raise ValueError(f"{name}: expected a [C] vector")
    return t.contiguous()


def _mod(e, x):
    """[B, F, 1, C] (or [B, F, C]) modulation tensor -> (tensor, frame stride, rows per frame)."""
    B, L, C = x.shape
    _like("modulation", e, x)
    e = e.reshape(B, -1, C)
    if e.stride(2) != 1 or (B > 1 and e.stride(0) != e.shape[1] * e.stride(1)):
        e = e.contiguous()
    if L % e.shape[1]:
        raise ValueError("token count is not a multiple of the number of modulation frames")
    return e, e.stride(1), L // e.shape[1]


def ln_modulate(x, scale, shift, eps=1e-6):
    """LayerNorm(x) (no affine) * (1 + scale) + shift with per-frame scale/shift."""
    rows, C, xs = _rows(x)
    sc, ms, rpf = _mod(scale, x)
    sh, ms2, _ = _mod(shift, x)
    if ms2 != ms:
        sc, sh = sc.contiguous(), sh.contiguous()
        ms = sc.stride(1)
    y = torch.empty_like(x, memory_format=torch.contiguous_format)
    with torch.cuda.device(x.device):
        _l.check(_l.load().sfm_ln_modulate(_DT[x.dtype], rows, C, eps, x.data_ptr(), xs, y.data_ptr(), C, sc.data_ptr(),
                                           sh.data_ptr(), ms, rpf, None, None, _stream(x)))
    return y


def ln_affine(x, weight, bias, eps=1e-6):
    rows, C, xs = _rows(x)
    weight, bias = _vec("weight", weight, x), _vec("bias", bias, x)
    y = torch.empty_like(x, memory_format=torch.contiguous_format)
    with torch.cuda.device(x.device):
        _l.check(_l.load().sfm_ln_modulate(_DT[x.dtype], rows, C, eps, x.data_ptr(), xs, y.data_ptr(), C, None, None, 0, 1,
                                           weight.data_ptr(), bias.data_ptr(), _stream(x)))
    return y


def gate_residual_(x, y, gate=None):
    """x += y * gate (per-frame gate) in place; gate=None: x += y."""
    rows, C, xs = _rows(x)
    _, _, ys = _rows(_like("y", y, x))
    if y.shape != x.shape:
        raise ValueError("x and y must have the same shape")
    g, ms, rpf = (None, 0, 1) if gate is None else _mod(gate, x)
    with torch.cuda.device(x.device):
        _l.check(_l.load().sfm_gate_residual(_DT[x.dtype], rows, C, x.data_ptr(), xs, y.data_ptr(), ys,
                                             None if g is None else g.data_ptr(), ms, rpf, _stream(x)))
    return x


def gate_residual_ln_(x, y, gate=None, scale=None, shift=None, weight=None, bias=None, eps=1e-6):
    """x += y * gate in place (gate=None: x += y), then returns (x, LayerNorm(x) * (1 + scale) + shift), or the
    affine LayerNorm when weight / bias are given: one pass over the rows instead of two kernels."""
    rows, C, xs = _rows(x)
    _, _, ys = _rows(_like("y", y, x))
    if y.shape != x.shape:
        raise ValueError("x and y must have the same shape")
    g, gms, grpf = (None, 0, 1) if gate is None else _mod(gate, x)
    out = torch.empty_like(x, memory_format=torch.contiguous_format)
    if weight is None:
        sc, ms, rpf = _mod(scale, x)
        sh, ms2, _ = _mod(shift, x)
        if ms2 != ms:
            sc, sh = sc.contiguous(), sh.contiguous()
            ms = sc.stride(1)
        mod = (sc.data_ptr(), sh.data_ptr(), ms, rpf, None, None)
    else:
        weight, bias = _vec("weight", weight, x), _vec("bias", bias, x)
        mod = (None, None, 0, 1, weight.data_ptr(), bias.data_ptr())
    with torch.cuda.device(x.device):
        _l.check(_l.load().sfm_gate_residual_ln(_DT[x.dtype], rows, C, eps, x.data_ptr(), xs, y.data_ptr(), ys,
                                                None if g is None else g.data_ptr(), gms, grpf, out.data_ptr(), C, *mod,
                                                _stream(x)))
    return x, out


def rms_norm(x, weight, eps=1e-6):
    rows, C, xs = _rows(x)
    weight = _vec("weight", weight, x)
    y = torch.empty_like(x, memory_format=torch.contiguous_format)
    with torch.cuda.device(x.device):
        _l.check(_l.load().sfm_rms_norm(_DT[x.dtype], rows, C, eps, x.data_ptr(), xs, y.data_ptr(), C, weight.data_ptr(),
                                        _stream(x)))
    return y
