"""Writes the output of the reference's own block and head wiring on seeded stand-in sub-layers.

Runs ONLY in the authoring container (needs /root/reference).  wan/modules/causal_model.py cannot be imported
(diffusers, flex-attention compiled at import), so `CausalWanAttentionBlock.forward` (causal_model.py:1152-1205)
and `CausalHead.forward` (:1227-1236) are located in the file's syntax tree and executed, from where they lie, as
plain functions whose `self` carries torch's own LayerNorm / Linear / GELU modules with the seeded parameters of
block_fixture.py and the fixture's stand-in attention sub-layers.  Only outputs are written
(wiring_reference_vectors.npz); inputs and parameters are regenerated from their seeds.

    python tests/golden/make_wiring_reference_vectors.py
"""
import ast
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
OUT = os.path.join(HERE, "wiring_reference_vectors.npz")


def method(cls, name):
    tree = ast.parse(open(REF).read(), REF)
    for node in tree.body:
        if isinstance(node, ast.ClassDef) and node.name == cls:
            for sub in node.body:
                if isinstance(sub, ast.FunctionDef) and sub.name == name:
                    ns = {"torch": torch}
                    exec(compile(ast.Module(body=[sub], type_ignores=[]), REF, "exec"), ns)
                    return ns[name]
    raise KeyError((cls, name))


def main():
    P, X = fx.parameters(), fx.inputs()
    sa, ca = fx.SelfAttnStandIn(), fx.CrossAttnStandIn()
    ffn = nn.Sequential(nn.Linear(fx.DIM, fx.FFN), nn.GELU(approximate="tanh"), nn.Linear(fx.FFN, fx.DIM)).double()
    norm3 = nn.LayerNorm(fx.DIM, eps=fx.EPS, elementwise_affine=True).double()
    with torch.no_grad():
        ffn[0].weight.copy_(P["ffn.0.weight"]); ffn[0].bias.copy_(P["ffn.0.bias"])
        ffn[2].weight.copy_(P["ffn.2.weight"]); ffn[2].bias.copy_(P["ffn.2.bias"])
        norm3.weight.copy_(P["norm3.weight"]); norm3.bias.copy_(P["norm3.bias"])
    plain_norm = nn.LayerNorm(fx.DIM, eps=fx.EPS, elementwise_affine=False)
    block = types.SimpleNamespace(
        modulation=P["modulation"], norm1=plain_norm, norm2=plain_norm, norm3=norm3, ffn=ffn,
        # the reference's call signatures (causal_model.py:1184-1187, 1194-1195)
        self_attn=lambda x, seq_lens, grid_sizes, freqs, block_mask, kv_cache, current_start, cache_start, timestep: sa.apply_to(x),
        cross_attn=lambda x, context, context_lens, crossattn_cache=None: ca.apply_to(x, context))
    fwd = method("CausalWanAttentionBlock", "forward")
    with torch.no_grad():
        y = fwd(block, X["x"], X["e"], None, None, None, X["context"], None, None)
        y_plain = fwd(types.SimpleNamespace(**{**vars(block), "norm3": nn.Identity()}), X["x"], X["e"], None, None, None,
                      X["context"], None, None)
    head_lin = nn.Linear(fx.DIM, 16).double()
    with torch.no_grad():
        head_lin.weight.copy_(P["head.head.weight"]); head_lin.bias.copy_(P["head.head.bias"])
    head = types.SimpleNamespace(modulation=P["head.modulation"], norm=plain_norm, head=head_lin)
    with torch.no_grad():
        z = method("CausalHead", "forward")(head, X["x"], X["e_head"])
    np.savez_compressed(OUT, block=y.numpy(), block_without_norm3=y_plain.numpy(), head=z.numpy())
    print("wrote", OUT, os.path.getsize(OUT), "bytes; block", tuple(y.shape), "head", tuple(z.shape))


if __name__ == "__main__":
    main()
