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
