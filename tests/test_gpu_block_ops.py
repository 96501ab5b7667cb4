"""GPU parity of the fused block element-wise kernels against the reference's eager chains (run on the CPU in
the same dtype by oracle.ops.OracleOps).  The kernels keep the eager ops' rounding points; only the fp32
statistics are summed in another order, so results may differ by one rounding step on a small fraction."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import randn
from oracle.ops import OracleOps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
blk = sfa.block_ops
STEP = {torch.bfloat16: 2 ** -7, torch.float16: 2 ** -10, torch.float32: 2 ** -20}


def _check(got, ref, dtype, frac_limit=2e-3):
    g, r = got.float().cpu(), ref.float().cpu()
    diff = (g - r).abs()
    assert (diff / r.abs().clamp_min(1.0)).max().item() <= 2 * STEP[dtype]
    if dtype != torch.float32:
        assert (diff > 0).float().mean().item() < frac_limit


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,F,fs,C", [(1, 3, 40, 1536), (2, 2, 7, 256), (1, 1, 5, 5120)])
def test_ln_modulate_gate_residual_rms(dtype, B, F, fs, C):
    o = OracleOps()
    x, y = randn((B, F * fs, C), 1, dtype), randn((B, F * fs, C), 2, dtype)
    e = (0.3 * randn((B, F, 6, C), 3, torch.float32)).to(dtype)
    ch = e.chunk(6, dim=2)
    w, b = (1 + 0.1 * randn((C,), 4, torch.float32)).to(dtype), (0.1 * randn((C,), 5, torch.float32)).to(dtype)
    xd, yd, ed = x.to(DEV), y.to(DEV), e.to(DEV)
    chd = ed.chunk(6, dim=2)
    _check(blk.ln_modulate(xd, chd[1], chd[0], 1e-6), o.ln_modulate(x, ch[1], ch[0], 1e-6), dtype)
    _check(blk.ln_affine(xd, w.to(DEV), b.to(DEV), 1e-6), o.ln_affine(x, w, b, 1e-6), dtype)
    _check(blk.rms_norm(xd, w.to(DEV), 1e-6), o.rms_norm(x, w, 1e-6), dtype)
    ref = o.gate_residual(x, y, ch[2])
    got = blk.gate_residual_(xd.clone(), yd, chd[2])
    assert torch.equal(got.cpu(), ref)                     # no statistics involved: bit exact
    assert torch.equal(blk.gate_residual_(xd.clone(), yd).cpu(), x + y)
    # residual update + the next norm in one kernel: the updated rows bit exact, the norm as the separate kernels
    for gate, gate_d in ((ch[2], chd[2]), (None, None)):
        xr, nr = o.gate_residual_ln(x, y, gate, 1e-6, scale=ch[4], shift=ch[3])
        xg, ng = blk.gate_residual_ln_(xd.clone(), yd, gate_d, scale=chd[4], shift=chd[3], eps=1e-6)
        assert torch.equal(xg.cpu(), xr)
        _check(ng, nr, dtype)
    xr, nr = o.gate_residual_ln(x, y, ch[2], 1e-6, weight=w, bias=b)
    xg, ng = blk.gate_residual_ln_(xd.clone(), yd, chd[2], weight=w.to(DEV), bias=b.to(DEV), eps=1e-6)
    assert torch.equal(xg.cpu(), xr)
    _check(ng, nr, dtype)


def test_block_ops_reject_bad_layouts():
    x = randn((1, 8, 64), 1, torch.bfloat16).to(DEV)
    with pytest.raises(ValueError):
        blk.rms_norm(x.transpose(1, 2), torch.ones(8, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError):
        blk.ln_modulate(x, torch.zeros(1, 3, 1, 64, dtype=torch.bfloat16, device=DEV),
                        torch.zeros(1, 3, 1, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError):        # C not a multiple of 8
        blk.rms_norm(randn((1, 8, 12), 1, torch.bfloat16).to(DEV), torch.ones(12, dtype=torch.bfloat16, device=DEV))


def test_block_ops_reject_operands_of_another_dtype_or_device():
    """The kernels read every operand in the activations' dtype: fp32 modulation or norm weights next to bf16
    activations would be misread, so the wrappers refuse them (and host tensors)."""
    x = randn((1, 12, 64), 2, torch.bfloat16).to(DEV)
    m16 = torch.zeros(1, 3, 1, 64, dtype=torch.bfloat16, device=DEV)
    m32, w32 = m16.float(), torch.ones(64, device=DEV)
    w16 = w32.bfloat16()
    for call in (lambda: blk.ln_modulate(x, m32, m16), lambda: blk.ln_modulate(x, m16, m32),
                 lambda: blk.ln_affine(x, w32, w16), lambda: blk.ln_affine(x, w16, w32), lambda: blk.rms_norm(x, w32),
                 lambda: blk.rms_norm(x, w16.cpu()), lambda: blk.rms_norm(x.cpu(), w16.cpu()),
                 lambda: blk.gate_residual_(x.clone(), x.float()), lambda: blk.gate_residual_(x.clone(), x, m32),
                 lambda: blk.gate_residual_ln_(x.clone(), x, m16, weight=w32, bias=w16),
                 lambda: blk.gate_residual_ln_(x.clone(), x, m16, scale=m32, shift=m16),
                 lambda: blk.rms_norm(x, torch.ones(32, dtype=torch.bfloat16, device=DEV))):
        with pytest.raises(ValueError):
            call()
