"""Writes golden input/output vectors of the reference's pure-torch Monarch formulas.

Runs ONLY in the authoring container (needs /root/reference).  wan/modules/monarch_attn.py cannot be
imported as a module (it asserts a CUDA Triton back-end at import, line 15), so the two pure-torch
functions are located in its syntax tree and executed, from the reference file where it lies, against the
installed torch + einops on the CPU.  Nothing of the reference's text is written anywhere: the outputs are
the arrays in monarch_reference_vectors.npz (inputs are regenerated from the seeds stored with them).

    python tests/golden/make_reference_vectors.py
"""
import ast
import os

import numpy as np
import torch
from einops import rearrange

REF = "/root/reference/wan/modules/monarch_attn.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "monarch_reference_vectors.npz")
WANTED = ("monarch_attn_slow", "monarch_attn_ref_op", "_get_rearrange_fns")


def load_functions():
    tree = ast.parse(open(REF).read(), REF)
    ns = {"torch": torch, "rearrange": rearrange}
    for node in tree.body:
        if isinstance(node, ast.FunctionDef) and node.name in WANTED:
            code = compile(ast.Module(body=[node], type_ignores=[]), REF, "exec")
            exec(code, ns)
    return ns


def case_inputs(seed, B, a, f, b1, b2, H, D):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, a, b1, b2, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, f, b1, b2, H, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, f, b1, b2, H, D, generator=g, dtype=torch.float64)
    return q, k, v


CASES = [  # (seed, B, a, f, b1, b2, H, D, sm_scale)
    (0, 1, 2, 3, 3, 4, 2, 8, 0.35),
    (1, 2, 1, 2, 4, 5, 1, 16, 0.25),
    (2, 1, 3, 3, 8, 8, 2, 64, 0.125),
]
ITERS = (1, 2, 3, 8)
TILINGS = [(1, 1, 1), (1, 2, 1), (3, 1, 1), (3, 2, 2), (1, 3, 4)]


def main():
    fn = load_functions()
    out = {}
    for ci, (seed, B, a, f, b1, b2, H, D, s) in enumerate(CASES):
        q, k, v = case_inputs(seed, B, a, f, b1, b2, H, D)
        out[f"case{ci}_meta"] = np.array([seed, B, a, f, b1, b2, H, D], dtype=np.int64)
        out[f"case{ci}_scale"] = np.array(s)
        out[f"case{ci}_ref_op"] = fn["monarch_attn_ref_op"](q, k, v, s).numpy()
        for n in ITERS:
            out[f"case{ci}_slow{n}"] = fn["monarch_attn_slow"](q, k, v, s, num_iters=n).numpy()
        # gradients of the one-iteration formula by autograd, for the cotangent drawn from seed + 1000
        qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
        cot = torch.randn(q.shape, generator=torch.Generator().manual_seed(seed + 1000), dtype=torch.float64)
        fn["monarch_attn_ref_op"](qa, ka, va, s).backward(cot)
        out[f"case{ci}_dq"], out[f"case{ci}_dk"], out[f"case{ci}_dv"] = qa.grad.numpy(), ka.grad.numpy(), va.grad.numpy()
        # the refinement is plain differentiable torch in the reference: its gradients for the same cotangent
        for n in (2, 3):
            qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
            fn["monarch_attn_slow"](qa, ka, va, s, num_iters=n).backward(cot)
            out[f"case{ci}_slow{n}_dq"], out[f"case{ci}_slow{n}_dk"], out[f"case{ci}_slow{n}_dv"] = (
                qa.grad.numpy(), ka.grad.numpy(), va.grad.numpy())
    # block-order permutation: token ids through rearrange_fn for several tilings (h=6, w=8, 3 frames)
    h, w, F = 6, 8, 3
    x = torch.arange(F * h * w, dtype=torch.float64).reshape(1, -1, 1, 1)
    for (ft, hr, wr) in TILINGS:
        fwd, back = fn["_get_rearrange_fns"](x, ft, hr, wr, h, w)
        xb = fwd(x)
        assert torch.equal(back(xb), x)
        out[f"order_{ft}_{hr}_{wr}"] = xb.reshape(xb.shape[1], xb.shape[2], xb.shape[3]).numpy().astype(np.int64)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
