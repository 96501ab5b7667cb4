"""Backward of the dense attention operators (sfm_dense_bwd through the autograd functions) against torch autograd
through the float64 oracle.  The oracle's dense attention is a plain softmax(q k^T s) v in torch (oracle/dense.py),
pinned by the golden vectors and closed forms of tests/test_oracle_dense_prologue.py; its autograd gradient is the
mathematical one."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import randn
from oracle import dense

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _leaf(t, dev=None):
    t = t.clone().detach()
    if dev:
        t = t.to(dev)
    return t.requires_grad_(True)


def _close(got, ref, dtype):
    got, ref = got.detach().float().cpu(), ref.detach().float()
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-3
    # 16-bit gradients are rounded once at the end; accumulation is fp32
    assert torch.allclose(got, ref, atol=tol * max(1.0, ref.abs().max().item()), rtol=tol)


@pytest.mark.parametrize("dtype,B,Lq,Lk,H,D", [
    (torch.bfloat16, 1, 128, 64, 1, 128),          # one workgroup of each kernel, one tile
    (torch.bfloat16, 2, 200, 333, 3, 128),         # ragged in both directions, several tiles
    (torch.float16, 1, 70, 130, 2, 64),
    (torch.bfloat16, 1, 1560, 4680, 2, 128),       # a frame of queries against three frames of keys (480p grid)
])
def test_dense_gradients(dtype, B, Lq, Lk, H, D):
    q0, do = (randn((B, Lq, H, D), 200 + i, dtype) for i in range(2))
    k0, v0 = (randn((B, Lk, H, D), 202 + i, dtype) for i in range(2))
    qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
    dense.attention(qr, kr, vr).backward(do.double())
    qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
    out = sfa.attention.attention(qd, kd, vd, dtype=dtype)
    out.backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(kd.grad, kr.grad, dtype)
    _close(vd.grad, vr.grad, dtype)


@pytest.mark.parametrize("partial", [False, True])
def test_dense_kv_cache_gradients(partial):
    """q against a cache of 5 x 48 keys of which keys 96..192 arrive with the call; partial = grad_only_new_kv."""
    dtype, H, D = torch.bfloat16, 2, 64
    q0, do = (randn((1, 100, H, D), 210 + i, dtype) for i in range(2))
    k_old, v_old = (randn((1, 240, H, D), 212 + i, dtype) for i in range(2))
    k_new, v_new = (randn((1, 96, H, D), 214 + i, dtype) for i in range(2))
    qr, kor, vor, knr, vnr = (_leaf(t.double()) for t in (q0, k_old, v_old, k_new, v_new))
    kfull = torch.cat([kor[:, :96], knr, kor[:, 192:]], 1)
    vfull = torch.cat([vor[:, :96], vnr, vor[:, 192:]], 1)
    dense.attention(qr, kfull, vfull).backward(do.double())

    qd, knd, vnd = _leaf(q0, DEV), _leaf(k_new, DEV), _leaf(v_new, DEV)
    kc, vc = k_old.to(DEV).clone(), v_old.to(DEV).clone()
    kc.requires_grad_(not partial)
    vc.requires_grad_(not partial)
    out = sfa.attention.full_attention_with_kv_cache(qd, kc, vc, knd, vnd, 96, 192, grad_only_new_kv=partial)
    out.backward(do.to(DEV))
    _close(qd.grad, qr.grad, dtype)
    _close(knd.grad, knr.grad, dtype)
    _close(vnd.grad, vnr.grad, dtype)
    if not partial:
        # rows 96..192 of the cache gradient belong to the keys written by the call
        keep = torch.ones(240, dtype=torch.bool)
        keep[96:192] = False
        _close(kc.grad[:, keep], kor.grad[:, keep], dtype)
        _close(vc.grad[:, keep], vor.grad[:, keep], dtype)
    else:
        assert kc.grad is None and vc.grad is None


def test_dense_backward_argument_checks():
    q = randn((1, 64, 1, 32), 220, torch.bfloat16).to(DEV).requires_grad_(True)      # head_dim 32: forward only
    out = sfa.attention.attention(q, q, q)
    with pytest.raises(Exception):
        out.sum().backward()
