"""The block's linear layers with their element-wise tails fused into the matrix product (`sfm_linear`): counterparts
of nn.Linear + nn.GELU(approximate='tanh') (wan/modules/model.py:648-650) and of the gated residual updates
`x + y * e[i]` after the output projections (wan/modules/causal_model.py:1189, 1196, 1203-1204).  16-bit tensors."""
import torch

from . import lib as _l
from .block_ops import _like, _mod, _rows
from .monarch_attn import _DT, _stream

_EPI = {"none": _l.EPI_NONE, "gelu_tanh": _l.EPI_GELU_TANH, "gate_residual": _l.EPI_GATE_RESIDUAL}


def supported(x, weight):
    """Whether `linear` takes these operands (16-bit GPU tensors, K a multiple of 64, N of 8, below 4 GiB each)."""
    return (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and weight.dtype == x.dtype and x.dim() == 3
            and weight.shape[1] % 64 == 0 and weight.shape[0] % 8 == 0 and x.stride(2) == 1 and x.stride(1) % 8 == 0
            and x.stride(0) == x.shape[1] * x.stride(1) and weight.numel() * 2 < 2 ** 32
            and x.shape[0] * x.shape[1] * x.stride(1) * 2 < 2 ** 32)


def linear(x, weight, bias=None, epilogue="none", res=None, gate=None, out=None, tile_rows=0):
    """x: [B, L, K]; weight: [N, K]; bias: [N] or None.
    epilogue "none": x @ weight.T + bias; "gelu_tanh": GELU (tanh form) of that; "gate_residual": res + (that) * gate with
    gate a per-frame modulation tensor [B, F, 1, N] (None: res + that), written to `out` (default: in place into res).
    `tile_rows` (0, 128, 256) forces the output rows per workgroup; 0 lets the library choose from the shape."""
    if epilogue not in _EPI:
        raise ValueError(f"unknown epilogue {epilogue!r}")
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError("linear takes float16 / bfloat16 tensors")
    rows, K, xs = _rows(x)
    _like("weight", weight, x)
    if weight.dim() != 2 or weight.shape[1] != K:
        raise ValueError("weight must be [N, K]")
    weight = weight.contiguous()
    N = weight.shape[0]
    if bias is not None:
        _like("bias", bias, x)
        if bias.shape != (N,):
            raise ValueError("bias must be [N]")
        bias = bias.contiguous()
    B, L = x.shape[:2]
    d = _l.LinearDesc()
    d.dtype, d.epilogue, d.M, d.N, d.K, d.x_stride = _DT[x.dtype], _EPI[epilogue], rows, N, K, xs
    d.tile_rows = tile_rows
    g = None
    if epilogue == "gate_residual":
        if res is None:
            raise ValueError("the gated-residual epilogue needs res")
        _like("res", res, x)
        if res.shape != (B, L, N):
            raise ValueError("res must be [B, L, N]")
        _, _, rs = _rows(res)
        d.res_stride = rs
        out = res if out is None else out
        if gate is not None:
            g, d.gate_stride, d.rows_per_frame = _mod(gate, res)
    elif res is not None or gate is not None:
        raise ValueError("res / gate belong to the gate_residual epilogue")
    if out is None:
        out = torch.empty((B, L, N), dtype=x.dtype, device=x.device)
    _like("out", out, x)
    if out.shape != (B, L, N):
        raise ValueError("out must be [B, L, N]")
    _, _, d.out_stride = _rows(out)
    with torch.cuda.device(x.device):
        _l.check(_l.load().sfm_linear(d, x.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(),
                                      None if res is None else res.data_ptr(), None if g is None else g.data_ptr(),
                                      out.data_ptr(), _stream(x)))
    return out
