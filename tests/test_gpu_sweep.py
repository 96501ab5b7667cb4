"""Seeded sweep of Monarch attention over drawn tilings, grids, lengths, head counts, dtypes and call kinds (plain,
block-causal, KV-cache write, refinement passes, one-kernel forward, gradients), each against the CPU oracle.  The
hand-picked shapes of the other files sit on the kernels' known limits; this file draws the shapes so that limits
nobody thought of get their turn (b1 from 1 to 126, b2 from 2 to 128, one to twelve block-frames on either side).

Tolerances are the files' own: forward as tests/test_gpu_monarch.py (fp32 <= 2e-5; 16-bit the reference's
atol = rtol = 1e-2 / 1e-3, twice that block-causal), gradients as tests/test_gpu_monarch_bwd.py."""
import random

import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import assert_close_16bit, max_abs, randn
from oracle import monarch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
mattn = sfa.monarch_attn

KINDS = ("plain", "causal", "cache", "iters", "one_kernel", "grad", "grad_causal", "grad_cache")


def _draw(seed):
    """One case: tiling (f_tied, h_reduce, w_reduce, h, w), query / key frame counts, batch, heads, head_dim, dtype."""
    r = random.Random(seed)
    kind = KINDS[seed % len(KINDS)]
    grad = kind.startswith("grad")
    f_tied, h_reduce, w_reduce = r.choice((1, 1, 2, 3)), r.choice((1, 1, 2, 3)), r.choice((1, 1, 2))
    budget = 1200 if grad else 2000                     # tokens per tied frame group: keeps the float64 oracle in seconds
    b2 = r.choice((r.randint(2, 24), r.randint(25, 64), r.randint(65, 128) if not grad else r.randint(33, 64), 52))
    tall = r.random() < 0.3                            # tall blocks: several 32-row query tiles per column
    if tall:
        b2, h_reduce, w_reduce = r.randint(2, 16), 1, 1
    rows = max(1, min(126 // f_tied, budget // (b2 * f_tied * h_reduce * w_reduce)))
    hb = r.randint(rows // 2 + 1, rows) if tall else r.randint(1, rows)          # block rows per frame
    h, w = hb * h_reduce, b2 * w_reduce
    group = f_tied * h * w                             # tokens of one query / key frame group
    nq = r.randint(1, max(1, min(4, 2 * budget // group)))
    nk = nq if "causal" in kind else r.randint(1, max(1, min(6, 4 * budget // group)))
    if kind in ("cache", "grad_cache"):
        nk = max(nk, nq + 1) if r.random() < 0.7 else max(nk, nq)
    dtype = r.choice((torch.bfloat16, torch.bfloat16, torch.float16, torch.float32))
    if kind == "one_kernel":
        dtype = r.choice((torch.bfloat16, torch.float16))
    return dict(kind=kind, tiling=(f_tied, h_reduce, w_reduce, h, w), Fq=nq * f_tied, Fk=nk * f_tied, B=r.choice((1, 1, 2)),
                H=r.choice((1, 2, 3)), D=r.choice((64, 128)), dtype=dtype, num_iters=r.choice((2, 3)), seed=seed)


def _leaf(t, dev=None):
    t = t.clone().detach()
    return (t.to(dev) if dev else t).requires_grad_(True)


def _fwd_close(out, ref, dtype, causal=False):
    if dtype == torch.float32:
        assert max_abs(out, ref) < 2e-5
    else:
        assert_close_16bit(out, ref, dtype, atol_scale=2.0 if causal else 1.0)


def _grad_close(got, ref, dtype):
    got, ref = got.detach().float().cpu(), ref.detach().float()
    if dtype == torch.float32:
        assert (got - ref).abs().max() <= 2e-4 * max(1.0, ref.abs().max().item())
    else:
        tol = 1e-2 if dtype == torch.bfloat16 else 1e-3
        assert torch.allclose(got, ref, atol=tol, rtol=tol), ((got - ref).abs().max().item(), ref.abs().max().item())


@pytest.mark.parametrize("seed", range(320))
def test_drawn_case_against_the_oracle(seed):
    c = _draw(seed)
    kind, tiling, dtype, B, H, D = c["kind"], c["tiling"], c["dtype"], c["B"], c["H"], c["D"]
    frame = tiling[3] * tiling[4]
    sq, skv = c["Fq"] * frame, c["Fk"] * frame
    print(c, flush=True)
    q0, k0, v0, do = (randn((B, n, H, D), 1000 * seed + i, dtype) for i, n in enumerate((sq, skv, skv, sq)))
    group = tiling[0] * frame

    if kind in ("plain", "causal", "iters", "one_kernel"):
        kw = {}
        if kind == "causal":
            kw["block_causal_size"] = group * random.Random(seed).choice([d for d in (1, 2, 3) if (c["Fq"] // tiling[0]) % d == 0])
        if kind == "iters":
            kw["num_iters"] = c["num_iters"]
        ref = monarch.monarch_attn(q0, k0, v0, *tiling, dtype=torch.float32 if kind != "iters" else torch.float64, **kw)
        out = mattn.monarch_attn(q0.to(DEV), k0.to(DEV), v0.to(DEV), *tiling, one_kernel=kind == "one_kernel", **kw)
        if kind == "iters" and dtype == torch.float32:
            assert max_abs(out, ref) < 1e-4            # refinement passes feed on each other: fp32 sums reorder
        else:
            _fwd_close(out, ref, dtype, causal=kind == "causal")
        if kind == "one_kernel":                        # where the one-kernel forward applies it still equals the oracle;
            two = mattn.monarch_attn(q0.to(DEV), k0.to(DEV), v0.to(DEV), *tiling)      # elsewhere it is the same kernels
            assert max_abs(out, two) < (2e-2 if dtype == torch.bfloat16 else 2e-3)
        return

    if kind == "cache":
        n_new = sq
        kc, vc = k0.clone(), v0.clone()
        nk, nv = (randn((B, n_new, H, D), 1000 * seed + 10 + i, dtype) for i in range(2))
        kc_o, vc_o = kc.clone(), vc.clone()
        ref = monarch.monarch_attn_with_kv_cache(q0, kc_o, vc_o, nk, nv, skv - n_new, skv, *tiling, dtype=torch.float32)
        kd, vd = kc.to(DEV), vc.to(DEV)
        out = mattn.monarch_attn_with_kv_cache(q0.to(DEV), kd, vd, nk.to(DEV), nv.to(DEV), skv - n_new, skv, *tiling)
        assert torch.equal(kd.cpu(), kc_o) and torch.equal(vd.cpu(), vc_o)
        _fwd_close(out, ref, dtype)
        return

    if kind in ("grad", "grad_causal"):
        kw = {"block_causal_size": group} if kind == "grad_causal" else {}
        qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
        monarch.monarch_attn(qr, kr, vr, *tiling, **kw).backward(do.double())
        qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
        mattn.monarch_attn(qd, kd, vd, *tiling, **kw).backward(do.to(DEV))
        for got, want in ((qd.grad, qr.grad), (kd.grad, kr.grad), (vd.grad, vr.grad)):
            _grad_close(got, want, dtype)
        return

    # grad_cache: the cache's old rows are block-ordered data, the new rows arrive in token order; gradients for both
    from oracle import blocks
    n_new = sq
    n_old = skv - n_new
    k_new, v_new = (randn((B, n_new, H, D), 1000 * seed + 10 + i, dtype) for i in range(2))
    qr, kor, vor, knr, vnr = (_leaf(t.double()) for t in (q0, k0[:, :n_old], v0[:, :n_old], k_new, v_new))
    t5 = tiling
    kfull = torch.cat([kor, blocks.to_blocks(knr, *t5).reshape(B, n_new, H, D)], 1)
    vfull = torch.cat([vor, blocks.to_blocks(vnr, *t5).reshape(B, n_new, H, D)], 1)
    qb = blocks.to_blocks(qr, *t5)
    b1, b2 = qb.shape[2], qb.shape[3]
    ob = monarch.monarch_1iter(qb, kfull.reshape(B, -1, b1, b2, H, D), vfull.reshape(B, -1, b1, b2, H, D), D ** -0.5)
    blocks.from_blocks(ob, *t5).backward(do.double())
    partial = bool(seed & 8)
    qd, knd, vnd = _leaf(q0, DEV), _leaf(k_new, DEV), _leaf(v_new, DEV)
    kc = torch.zeros(B, skv, H, D, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    kc[:, :n_old], vc[:, :n_old] = k0[:, :n_old].to(DEV), v0[:, :n_old].to(DEV)
    kc.requires_grad_(not partial)
    vc.requires_grad_(not partial)
    mattn.monarch_attn_with_kv_cache(qd, kc, vc, knd, vnd, n_old, skv, *tiling, grad_only_new_kv=partial).backward(do.to(DEV))
    for got, want in ((qd.grad, qr.grad), (knd.grad, knr.grad), (vnd.grad, vnr.grad)):
        _grad_close(got, want, dtype)
    if not partial and n_old:
        _grad_close(kc.grad[:, :n_old], kor.grad, dtype)
        _grad_close(vc.grad[:, :n_old], vor.grad, dtype)


# ---- the other operators of the path: dense attention (forward, gradients), the q/k prologue, the block's linear layers ----

OTHER = ("dense", "dense_grad", "prologue", "linear")


@pytest.mark.parametrize("seed", range(160))
def test_drawn_case_of_the_other_operators(seed):
    from oracle import blocks, dense, prologue
    r = random.Random(10_000 + seed)
    kind = OTHER[seed % len(OTHER)]
    if kind in ("dense", "dense_grad"):
        grad = kind == "dense_grad"
        B, H, D = r.choice((1, 1, 2)), r.choice((1, 2, 3, 5)), r.choice((64, 128)) if grad else r.choice((32, 64, 128))
        Lq = r.choice((r.randint(1, 130), r.randint(131, 700), r.randint(701, 2600 if not grad else 1200)))
        Lk = r.choice((r.randint(1, 70), r.randint(71, 600), r.randint(601, 3000 if not grad else 1500)))
        dtype = r.choice((torch.bfloat16, torch.float16)) if grad else r.choice((torch.bfloat16, torch.float16, torch.float32))
        print(dict(kind=kind, B=B, Lq=Lq, Lk=Lk, H=H, D=D, dtype=dtype), flush=True)
        q0, k0, v0, do = (randn((B, n, H, D), 2000 * seed + i, dtype) for i, n in enumerate((Lq, Lk, Lk, Lq)))
        if not grad:
            ref, lse_ref = dense.attention(q0, k0, v0, dtype=torch.float32, return_lse=True)
            out, lse = sfa.attention.attention(q0.to(DEV), k0.to(DEV), v0.to(DEV), dtype=dtype, return_lse=True)
            if dtype == torch.float32:
                assert max_abs(out, ref) < 1e-5
            else:
                assert_close_16bit(out, ref, dtype)
            assert max_abs(lse, lse_ref) < 1e-3
            return
        qr, kr, vr = _leaf(q0.double()), _leaf(k0.double()), _leaf(v0.double())
        dense.attention(qr, kr, vr).backward(do.double())
        qd, kd, vd = _leaf(q0, DEV), _leaf(k0, DEV), _leaf(v0, DEV)
        sfa.attention.attention(qd, kd, vd, dtype=dtype).backward(do.to(DEV))
        tol = 1e-2 if dtype == torch.bfloat16 else 1e-3
        for got, want in ((qd.grad, qr.grad), (kd.grad, kr.grad), (vd.grad, vr.grad)):
            got, want = got.float().cpu(), want.float()
            assert torch.allclose(got, want, atol=tol * max(1.0, want.abs().max().item()), rtol=tol)
        return

    if kind == "prologue":
        f_tied, h_reduce, w_reduce = r.choice((1, 1, 3)), r.choice((1, 2, 3)), r.choice((1, 1, 2, 4))
        h, w = h_reduce * r.randint(1, 12), w_reduce * r.randint(1, 20)
        F, H, D = f_tied * r.randint(1, 3), r.choice((1, 2, 5, 12)), r.choice((64, 128))
        B, dtype = r.choice((1, 2)), r.choice((torch.bfloat16, torch.float16, torch.float32))
        start_frame = r.randint(0, 40)
        print(dict(kind=kind, tiling=(f_tied, h_reduce, w_reduce, h, w), F=F, B=B, H=H, D=D, dtype=dtype, start=start_frame), flush=True)
        S, Cd = F * h * w, H * D
        xq, xk, xv = (randn((B, S, Cd), 3000 * seed + i, dtype) for i in range(3))
        wq, wk = ((1 + 0.1 * randn((Cd,), 3000 * seed + 3 + i, torch.float32)).to(dtype) for i in range(2))
        pre = f_tied * h * w * r.randint(0, 2)
        qr, kr, vr = prologue.qk_prologue(xq, xk, xv, wq, wk, H, (F, h, w), start_frame)
        kc = torch.zeros(B, pre + S + 7, H, D, dtype=dtype, device=DEV)
        vc = torch.zeros_like(kc)
        rope = sfa.prologue.rope_table(D, device=DEV)
        qo = sfa.prologue.qk_prologue(xq.to(DEV), xk.to(DEV), xv.to(DEV), wq.to(DEV), wk.to(DEV), H, (F, h, w), start_frame,
                                      rope, kc, vc, pre, f_tied, h_reduce, w_reduce)
        kref = blocks.to_blocks(kr, f_tied, h_reduce, w_reduce, h, w).reshape(B, S, H, D)
        vref = blocks.to_blocks(vr, f_tied, h_reduce, w_reduce, h, w).reshape(B, S, H, D)
        assert torch.equal(vc[:, pre:pre + S].cpu(), vref)
        assert (kc[:, :pre] == 0).all() and (kc[:, pre + S:] == 0).all() and (vc[:, pre + S:] == 0).all()
        one_step = {torch.bfloat16: 2 ** -7, torch.float16: 2 ** -10, torch.float32: 2 ** -21}[dtype]
        for got, ref in ((qo, qr), (kc[:, pre:pre + S], kref)):
            g, rf = got.float().cpu(), ref.float().cpu()
            assert ((g - rf).abs() / rf.abs().clamp_min(1.0)).max().item() <= 2 * one_step
        return

    # linear: out = epilogue(x W^T + b) against fp32 matmul followed by the eager chain's roundings
    dtype = r.choice((torch.bfloat16, torch.float16))
    M, N, K = r.choice((r.randint(1, 300), r.randint(301, 2000))), 8 * r.randint(1, 160), 64 * r.randint(1, 24)
    epi = r.choice(("none", "none", "gelu_tanh", "gate_residual"))
    tile_rows = r.choice((0, 128, 256))
    print(dict(kind=kind, M=M, N=N, K=K, dtype=dtype, epilogue=epi, tile_rows=tile_rows), flush=True)
    x = randn((1, M, K), 4000 * seed, dtype).to(DEV)
    wt = (randn((N, K), 4000 * seed + 1, dtype) * K ** -0.5).to(dtype).to(DEV)
    b = randn((N,), 4000 * seed + 2, dtype).to(DEV) if r.random() < 0.7 else None
    assert sfa.linear.supported(x, wt)
    y = x.float() @ wt.float().t()
    y = (y + b.float() if b is not None else y).to(dtype)
    kw = {}
    if epi == "gelu_tanh":
        ref = torch.nn.functional.gelu(y.float(), approximate="tanh").to(dtype)
        # a product one rounding step away moves the result by |gelu'(y)| steps of y, which in the left tail is many steps
        # of the tiny result: the steps are measured at |gelu(y)| + |y gelu'(y)| (as tests/test_gpu_linear.py does)
        yl = y.float().requires_grad_(True)
        gl = torch.nn.functional.gelu(yl, approximate="tanh")
        gl.sum().backward()
        scale = gl.detach().abs() + (yl.detach() * yl.grad).abs()
    elif epi == "gate_residual":
        res = randn((1, M, N), 4000 * seed + 3, dtype).to(DEV)
        gate = randn((1, 1, 1, N), 4000 * seed + 4, dtype).to(DEV)
        yg = (y.float() * gate.reshape(1, 1, N).float()).to(dtype)
        ref = (res.float() + yg.float()).to(dtype)
        scale = res.float().abs() + yg.float().abs()
        kw = dict(res=res.clone(), gate=gate)
    else:
        ref, scale = y, None
    out = sfa.linear.linear(x, wt, b, epilogue=epi, tile_rows=tile_rows, **kw)
    unit = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    err = (out.float() - ref.float()).abs()
    mag = (ref.float().abs() if scale is None else scale).clamp_min(2.0 ** -6)
    steps = {"none": 1, "gelu_tanh": 2, "gate_residual": 3}[epi]
    assert (err <= steps * unit * mag).all(), (err.max().item(), (err / mag).max().item())
