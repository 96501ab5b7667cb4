"""Helpers shared by the GPU parity tests."""
import torch


def randn(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def max_abs(a, b):
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


def per_head_cosine(a, b):
    """min over (batch, head) of the cosine between [B,S,H,D] tensors."""
    a, b = a.double().cpu(), b.double().cpu()
    B, S, H, D = a.shape
    x = a.permute(0, 2, 1, 3).reshape(B * H, -1)
    y = b.permute(0, 2, 1, 3).reshape(B * H, -1)
    return torch.nn.functional.cosine_similarity(x, y, dim=1).min().item()


def assert_close_16bit(got, ref, dtype, atol_scale=1.0):
    """The reference's own bar (atol = rtol = 1e-2 bf16, 1e-3 fp16; monarch_attn.py:1908-1909) against
    the fp32/fp64 oracle, plus the north-star bar: max-abs < 2e-2 and per-head cosine > 0.999."""
    tol = (1e-2 if dtype == torch.bfloat16 else 1e-3) * atol_scale
    g, r = got.double().cpu(), ref.double().cpu()
    assert not torch.isnan(g).any()
    bad = ((g - r).abs() > tol + tol * r.abs()).sum().item()
    assert bad == 0, f"{bad} of {g.numel()} elements outside atol=rtol={tol}; max-abs {max_abs(g, r):.3e}"
    assert max_abs(g, r) < 2e-2
    assert per_head_cosine(got, ref) > 0.999


def monarch_fwd_exact_workspace(q, k, v, tiling, heads_per_pass, num_iters=1, one_kernel=False, kv_block_order=0):
    """sfm_monarch_fwd through the C ABI with a workspace of exactly sfm_monarch_workspace_bytes(heads_per_pass) and
    64 KiB of canary bytes behind it; returns the output after checking that the canary is untouched."""
    import ctypes as C

    import self_forcing_amd as sfa
    from self_forcing_amd import lib as L

    f_tied, h_reduce, w_reduce, h, w = tiling
    out = torch.full_like(q, float("nan"))
    d = sfa.monarch_attn._desc(q, k, v, out, f_tied, h_reduce, w_reduce, h, w, q.shape[-1] ** -0.5, kv_block_order, 0,
                               num_iters, one_kernel)
    n = sfa.monarch_attn.monarch_workspace_bytes(d, heads_per_pass)
    pad = 64 * 1024
    buf = torch.full((n + pad,), 0xA5, dtype=torch.uint8, device=q.device)
    stream = C.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
    L.check(L.load().sfm_monarch_fwd(C.byref(d), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), buf.data_ptr(), n,
                                     stream))
    torch.cuda.synchronize()
    assert bool((buf[n:] == 0xA5).all()), "bytes behind the workspace were overwritten"
    return out


def monarch_bwd_exact_workspace(q, k, v, dout, tiling, heads_per_pass=0, cbf=0):
    """sfm_monarch_bwd through the C ABI with a workspace of exactly sfm_monarch_bwd_workspace_bytes(heads_per_pass) and
    64 KiB of canary bytes behind it; returns (dq, dk, dv) after checking that the canary is untouched."""
    import ctypes as C

    import self_forcing_amd as sfa
    from self_forcing_amd import lib as L

    f_tied, h_reduce, w_reduce, h, w = tiling
    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    dk, dv = torch.empty_like(k), torch.empty_like(v)
    bd = L.MonarchBwdDesc()
    bd.fwd = sfa.monarch_attn._desc(q, k, v, dout, f_tied, h_reduce, w_reduce, h, w, q.shape[-1] ** -0.5, 0, cbf)
    bd.dq_stride = L.strides3(dq)
    bd.dkv_stride = L.strides3(dk)
    per_frame = f_tied * (h // h_reduce) * (w // w_reduce)
    bd.kv_grad_frame_start, bd.kv_grad_frame_end = 0, k.shape[1] // per_frame
    n = C.c_size_t(0)
    L.check(L.load().sfm_monarch_bwd_workspace_bytes(C.byref(bd), heads_per_pass, C.byref(n)))
    pad = 64 * 1024
    buf = torch.full((n.value + pad,), 0xA5, dtype=torch.uint8, device=q.device)
    stream = C.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
    L.check(L.load().sfm_monarch_bwd(C.byref(bd), q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), dq.data_ptr(),
                                     dk.data_ptr(), dv.data_ptr(), buf.data_ptr(), n.value, stream))
    torch.cuda.synchronize()
    assert bool((buf[n.value:] == 0xA5).all()), "bytes behind the workspace were overwritten"
    return dq, dk, dv
