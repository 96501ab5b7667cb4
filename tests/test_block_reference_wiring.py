"""The product's block and head against the output of the reference's own `CausalWanAttentionBlock.forward` and
`CausalHead.forward` (tests/golden/wiring_reference_vectors.npz, written by
tests/golden/make_wiring_reference_vectors.py from the methods where they lie in causal_model.py:1152-1236) on the
same seeded parameters, inputs and stand-in attention sub-layers (tests/golden/block_fixture.py).  CPU, float64."""
import os
import sys

import numpy as np
import pytest
import torch
import torch.nn as nn

import self_forcing_amd as sfa
from oracle.ops import OracleOps

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import block_fixture as fx  # noqa: E402

cm = sfa.causal_model
GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "wiring_reference_vectors.npz"))


class _SelfAttn(nn.Module):
    def __init__(self):
        super().__init__()
        self.f = fx.SelfAttnStandIn()

    def forward(self, x, grid, kv_cache, current_start):
        return self.f.apply_to(x)


class _CrossAttn(nn.Module):
    def __init__(self):
        super().__init__()
        self.f = fx.CrossAttnStandIn()

    def forward(self, x, context, crossattn_cache):
        return self.f.apply_to(x, context)


def _block(cross_attn_norm=True, permute=None):
    P = fx.parameters()
    blk = cm.CausalWanAttentionBlock(fx.DIM, fx.FFN, 2, cross_attn_norm=cross_attn_norm, eps=fx.EPS, block_num=0, frame_hw=(2, 5),
                                     ops=OracleOps(), flags=cm.AttentionFlags(0)).double()
    blk.self_attn, blk.cross_attn = _SelfAttn(), _CrossAttn()
    with torch.no_grad():
        mod = P["modulation"] if permute is None else P["modulation"][:, permute]
        blk.modulation.copy_(mod)
        if cross_attn_norm:
            blk.norm3.weight.copy_(P["norm3.weight"]); blk.norm3.bias.copy_(P["norm3.bias"])
        blk.ffn[0].weight.copy_(P["ffn.0.weight"]); blk.ffn[0].bias.copy_(P["ffn.0.bias"])
        blk.ffn[2].weight.copy_(P["ffn.2.weight"]); blk.ffn[2].bias.copy_(P["ffn.2.bias"])
    return blk.eval()


def _run(blk, permute=None):
    X = fx.inputs()
    e = X["e"] if permute is None else X["e"][:, :, permute]
    with torch.no_grad():
        return blk(X["x"].clone(), e, (fx.FRAMES, 2, 5), X["context"], None, None, 0)


@pytest.mark.parametrize("cross_attn_norm,key", [(True, "block"), (False, "block_without_norm3")])
def test_block_wiring_is_the_reference_forward(cross_attn_norm, key):
    y = _run(_block(cross_attn_norm))
    np.testing.assert_allclose(y.numpy(), GOLD[key], atol=1e-10, rtol=0)


@pytest.mark.parametrize("perm", [[1, 0, 2, 3, 4, 5], [0, 1, 5, 3, 4, 2], [0, 1, 2, 4, 3, 5], [3, 4, 2, 0, 1, 5]])
def test_a_permuted_modulation_row_would_show(perm):
    """Sensitivity of the pin: feeding the six modulation rows in another order moves the output far beyond the bar."""
    y = _run(_block(permute=perm), permute=perm)
    assert np.abs(y.numpy() - GOLD["block"]).max() > 1e-2


def test_head_wiring_is_the_reference_forward():
    P, X = fx.parameters(), fx.inputs()
    head = cm.CausalHead(fx.DIM, 4, (1, 2, 2), eps=fx.EPS).double()
    with torch.no_grad():
        head.modulation.copy_(P["head.modulation"])
        head.head.weight.copy_(P["head.head.weight"]); head.head.bias.copy_(P["head.head.bias"])
        z = head(X["x"], X["e_head"])
    np.testing.assert_allclose(z.numpy().reshape(GOLD["head"].shape), GOLD["head"], atol=1e-10, rtol=0)


class _Block(nn.Module):
    def __init__(self, index):
        super().__init__()
        self.index = index

    def forward(self, x, e, grid, context, kv_cache, crossattn_cache, current_start):
        return fx.block_stand_in(x, e, context, self.index)


def test_model_wiring_is_the_reference_forward_inference():
    """Patch embedding, time embedding and projection (the six modulation rows in the reference's order), text
    embedding with padding to text_len, block loop, head and unpatchify against the reference's own
    `_forward_inference` (tests/golden/model_wiring_reference_vectors.npz) with stand-in blocks."""
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model_wiring_reference_vectors.npz"))
    m = cm.CausalWanModel(patch_size=fx.M_PATCH, text_len=fx.M_TEXT_LEN, in_dim=fx.M_IN, dim=fx.M_DIM, ffn_dim=64, freq_dim=fx.M_FREQ,
                          text_dim=fx.M_TEXT, out_dim=fx.M_OUT, num_heads=2, num_layers=fx.M_LAYERS, eps=fx.EPS, frame_hw=(2, 3),
                          ops=OracleOps()).double().eval()
    m.blocks = nn.ModuleList([_Block(i) for i in range(fx.M_LAYERS)])
    with torch.no_grad():
        for k, p in m.named_parameters():
            p.copy_(fx.model_parameter(k, tuple(p.shape)))
    X = fx.model_inputs()
    for b in range(2):
        t = X["t"][b:b + 1, :1].expand(1, 3).contiguous()
        out = m(X["x"][b:b + 1], t, X["context"][b:b + 1], kv_cache=[None] * fx.M_LAYERS, crossattn_cache=[None] * fx.M_LAYERS)
        np.testing.assert_allclose(out.numpy(), gold[f"out{b}"], atol=1e-10, rtol=0)
    # both videos in one batch (the reference runs them one by one): the same rows
    t = X["t"][:, :1].expand(2, 3).contiguous()
    out = m(X["x"], t, X["context"], kv_cache=[None] * fx.M_LAYERS, crossattn_cache=[None] * fx.M_LAYERS)
    np.testing.assert_allclose(out.numpy(), np.concatenate([gold["out0"], gold["out1"]]), atol=1e-10, rtol=0)
