"""Writes the output of the reference's own `CausalWanModel._forward_inference` wiring (embeddings, time
projection, block loop, head, unpatchify: causal_model.py:1582-1720, 1896-1919, with `CausalHead.forward` :1227-1236
and `sinusoidal_embedding_1d` model.py:407-418) on seeded parameters and stand-in blocks.

Runs ONLY in the authoring container (needs /root/reference).  The methods are located in the file's syntax tree and
executed, from where they lie, as plain functions whose `self` carries torch modules built as the reference's
constructor builds them (causal_model.py:1326-1346) with the parameters of block_fixture.model_parameter, and the
fixture's stand-in for a block.  Only the output is written (model_wiring_reference_vectors.npz).

    python tests/golden/make_model_wiring_reference_vectors.py
"""
import ast
import math
import os
import sys
import types

import numpy as np
import torch
import torch.nn as nn

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import block_fixture as fx  # noqa: E402

REF = "/root/reference/wan/modules/causal_model.py"
OUT = os.path.join(HERE, "model_wiring_reference_vectors.npz")


def function(path, name, ns, cls=None):
    tree = ast.parse(open(path).read(), path)
    body = tree.body
    if cls is not None:
        body = [n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == cls][0].body
    node = [n for n in body if isinstance(n, ast.FunctionDef) and n.name == name][0]
    exec(compile(ast.Module(body=[node], type_ignores=[]), path, "exec"), ns)
    return ns[name]


def seeded(module, prefix):
    with torch.no_grad():
        for k, p in module.named_parameters():
            p.copy_(fx.model_parameter(f"{prefix}.{k}", tuple(p.shape)))
    return module.double()


def main():
    ns = {"torch": torch, "math": math}
    function("/root/reference/wan/modules/model.py", "sinusoidal_embedding_1d", ns)
    fwd = function(REF, "_forward_inference", ns, cls="CausalWanModel")
    unpatchify = function(REF, "unpatchify", ns, cls="CausalWanModel")
    head_fwd = function(REF, "forward", {"torch": torch}, cls="CausalHead")

    d = fx.M_DIM
    head = types.SimpleNamespace(modulation=fx.model_parameter("head.modulation", (1, 2, d)),
                                 norm=nn.LayerNorm(d, eps=fx.EPS, elementwise_affine=False),
                                 head=seeded(nn.Linear(d, math.prod(fx.M_PATCH) * fx.M_OUT).double(), "head.head"))
    m = types.SimpleNamespace(
        model_type="t2v", patch_size=fx.M_PATCH, text_len=fx.M_TEXT_LEN, dim=d, freq_dim=fx.M_FREQ, out_dim=fx.M_OUT,
        freqs=torch.zeros(1), block_mask=None, gradient_checkpointing=False,
        patch_embedding=seeded(nn.Conv3d(fx.M_IN, d, kernel_size=fx.M_PATCH, stride=fx.M_PATCH).double(), "patch_embedding"),
        text_embedding=seeded(nn.Sequential(nn.Linear(fx.M_TEXT, d), nn.GELU(approximate="tanh"), nn.Linear(d, d)).double(), "text_embedding"),
        time_embedding=seeded(nn.Sequential(nn.Linear(fx.M_FREQ, d), nn.SiLU(), nn.Linear(d, d)).double(), "time_embedding"),
        time_projection=seeded(nn.Sequential(nn.SiLU(), nn.Linear(d, d * 6)).double(), "time_projection"),
        head=lambda x, e: head_fwd(head, x, e))
    m.unpatchify = lambda x, g: unpatchify(m, x, g)

    def make_block(i):
        def block(x, e, seq_lens, grid_sizes, freqs, context, context_lens, block_mask, kv_cache=None, crossattn_cache=None,
                  current_start=0, cache_start=None, timestep=None):
            return fx.block_stand_in(x, e, context, i)
        return block
    m.blocks = [make_block(i) for i in range(fx.M_LAYERS)]

    X = fx.model_inputs()
    outs = {}
    with torch.no_grad():
        # the reference takes a tensor batch as an iterable of [C, F, H, W] videos and of [L, C] text embeddings; one
        # timestep per call (it asserts t == t[0, 0]): the batch rows are run one by one with their first timestep
        for b in range(X["x"].shape[0]):
            t = X["t"][b:b + 1, :1].expand(1, X["x"].shape[2]).contiguous()
            outs[f"out{b}"] = fwd(m, X["x"][b:b + 1], t, X["context"][b:b + 1], seq_len=10 ** 6,
                                  kv_cache=[None] * fx.M_LAYERS, crossattn_cache=[None] * fx.M_LAYERS, current_start=0).numpy()
    np.savez_compressed(OUT, **outs)
    print("wrote", OUT, os.path.getsize(OUT), "bytes;", {k: v.shape for k, v in outs.items()})


if __name__ == "__main__":
    main()
