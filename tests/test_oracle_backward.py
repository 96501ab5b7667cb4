"""The oracle's gradients (torch autograd through the float64 oracle forward, which the golden vectors pin)
against central finite differences and against the closed-form backward the HIP kernels implement."""
import torch

from oracle import monarch


def _rand(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float64)


def test_autograd_of_the_oracle_matches_finite_differences():
    q, k, v = _rand((1, 2, 3, 4, 1, 8), 1), _rand((1, 3, 3, 4, 1, 8), 2), _rand((1, 3, 3, 4, 1, 8), 3)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b, c: monarch.monarch_1iter(a, b, c, 0.4), (q, k, v), eps=1e-6, atol=1e-6)


def test_closed_form_backward_equals_autograd():
    """dS2 = L (dLm - sum L dLm), dKbar = s dS2^T q, dY = L^T dO, dc = -sum_i dS2, dR = dKbar.K + dY.V + dc ln R,
    dS1 = R (dR - sum R dR), dQ = s dS2 Kbar + s dS1 K, dK = R^T dKbar + s dS1^T q, dV = R^T dY."""
    s = 0.3
    q, k, v = _rand((2, 3, 4, 8), 4), _rand((3, 3, 4, 8), 5), _rand((3, 3, 4, 8), 6)       # [a,b1,b2,D], [f,b1,b2,D]
    dO = _rand((2, 3, 4, 8), 7)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = monarch.monarch_1iter(qa[None, :, :, :, None], ka[None, :, :, :, None], va[None, :, :, :, None], s)[0, :, :, :, 0]
    out.backward(dO)

    S1 = s * torch.einsum("akjd,fkld->afkjl", q, k)
    R = torch.softmax(S1, -1)
    lnR = torch.log_softmax(S1, -1)
    Kbar = torch.einsum("afkjl,fkld->afkjd", R, k)
    Y = torch.einsum("afkjl,fkld->afkjd", R, v)
    c = (R * lnR).sum(-1)
    S2 = s * torch.einsum("aijd,afkjd->aijfk", q, Kbar) - c.permute(0, 3, 1, 2).unsqueeze(1)
    L = torch.softmax(S2.flatten(3), -1).reshape(S2.shape)
    dLm = torch.einsum("aijd,afkjd->aijfk", dO, Y)
    dS2 = L * (dLm - (L * dLm).sum((3, 4), keepdim=True))
    dY = torch.einsum("aijfk,aijd->afkjd", L, dO)
    dKbar = s * torch.einsum("aijfk,aijd->afkjd", dS2, q)
    dc = -dS2.sum(1).permute(0, 2, 3, 1)                                        # [a,f,k,j]
    dR = torch.einsum("afkjd,fkld->afkjl", dKbar, k) + torch.einsum("afkjd,fkld->afkjl", dY, v) + dc.unsqueeze(-1) * lnR
    dS1 = R * (dR - (R * dR).sum(-1, keepdim=True))
    dq = s * torch.einsum("aijfk,afkjd->aijd", dS2, Kbar) + s * torch.einsum("afkjl,fkld->akjd", dS1, k)
    dk = torch.einsum("afkjl,afkjd->fkld", R, dKbar) + s * torch.einsum("afkjl,akjd->fkld", dS1, q)
    dv = torch.einsum("afkjl,afkjd->fkld", R, dY)
    assert (dq - qa.grad).abs().max() < 1e-12
    assert (dk - ka.grad).abs().max() < 1e-12
    assert (dv - va.grad).abs().max() < 1e-12
