"""Writes what the reference's own `CausalWanSelfAttention.forward` (KV-cache branch, causal_model.py:899-1108) does
to the cache and returns, call by call, for scripted sequences of chunks (block_fixture.A_SCENARIOS): whole-history and
windowed caches, sink frames, re-runs of a chunk, dense first chunk, Monarch disabled, refinement passes.

Runs ONLY in the authoring container (needs /root/reference).  The method is located in the file's syntax tree and
executed, from where it lies, as a plain function.  Its collaborators are the reference's own pure-torch functions,
extracted the same way: `causal_rope_apply`, `rope_params`, `WanRMSNorm` and, from monarch_attn.py,
`monarch_attn_with_kv_cache`, `_get_rearrange_fns`, `monarch_attn_slow`, `monarch_attn_ref_op`.  Two things are not
the reference's: the Triton function `_attention_with_cache` is replaced by the cache write it performs
(monarch_attn.py:1230-1231) followed by `monarch_attn_ref_op`, and `attention` (flash-attn) by a float64 softmax
attention.  Only results are written (cache_reference_vectors.npz); inputs and parameters come from seeds.

    python tests/golden/make_cache_reference_vectors.py
"""
import ast
import math
import os
import sys
import types

import numpy as np
import torch
import torch.nn as nn
from einops import rearrange

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import block_fixture as fx  # noqa: E402

REF = "/root/reference/wan/modules"
OUT = os.path.join(HERE, "cache_reference_vectors.npz")


def extract(path, names, ns, cls=None):
    tree = ast.parse(open(path).read(), path)
    body = tree.body
    if cls is not None:
        body = [n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == cls][0].body
    for node in body:
        if isinstance(node, (ast.FunctionDef, ast.ClassDef)) and node.name in names:
            exec(compile(ast.Module(body=[node], type_ignores=[]), path, "exec"), ns)
    missing = [n for n in names if n not in ns]
    assert not missing, missing


def softmax_attention(q, k, v):
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) * q.shape[-1] ** -0.5
    return torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, dim=-1), v)


def main():
    mon = {"torch": torch, "rearrange": rearrange}
    extract(f"{REF}/monarch_attn.py", ("monarch_attn_with_kv_cache", "_get_rearrange_fns", "monarch_attn_slow", "monarch_attn_ref_op"), mon)

    class CacheWriteThenRefOp:
        @staticmethod
        def apply(q, k_cache, v_cache, new_k, new_v, start_idx, end_idx, sm_scale, *unused):
            b, _, nh, d = new_k.shape
            k_cache[:, start_idx:end_idx, :, :] = new_k
            v_cache[:, start_idx:end_idx, :, :] = new_v
            kb = k_cache.reshape(b, -1, q.shape[2], q.shape[3], nh, d)
            vb = v_cache.reshape(b, -1, q.shape[2], q.shape[3], nh, d)
            return mon["monarch_attn_ref_op"](q, kb, vb, sm_scale)
    mon["_attention_with_cache"] = CacheWriteThenRefOp

    ns = {"torch": torch, "math": math, "nn": nn, "attention": softmax_attention,
          "monarch_attn_with_kv_cache": mon["monarch_attn_with_kv_cache"],
          "frame_height": fx.A_H, "frame_width": fx.A_W, "total_seq_len": None}
    extract(f"{REF}/model.py", ("rope_params", "WanRMSNorm"), ns)
    extract(f"{REF}/causal_model.py", ("causal_rope_apply",), ns)
    extract(f"{REF}/causal_model.py", ("forward",), ns, cls="CausalWanSelfAttention")
    fwd = ns["forward"]

    d = fx.A_DIM // fx.A_HEADS
    freqs = torch.cat([ns["rope_params"](1024, d - 4 * (d // 6)), ns["rope_params"](1024, 2 * (d // 6)),
                       ns["rope_params"](1024, 2 * (d // 6))], dim=1)

    def linear(name):
        m = nn.Linear(fx.A_DIM, fx.A_DIM).double()
        with torch.no_grad():
            m.weight.copy_(fx.attn_parameter(name + ".weight", (fx.A_DIM, fx.A_DIM)))
            m.bias.copy_(fx.attn_parameter(name + ".bias", (fx.A_DIM,)))
        return m

    def norm(name):
        m = ns["WanRMSNorm"](fx.A_DIM, eps=fx.EPS).double()
        with torch.no_grad():
            m.weight.copy_(fx.attn_parameter(name + ".weight", (fx.A_DIM,)))
        return m

    out = {}
    for scen, (local, sink, cache_frames, flags, calls) in fx.A_SCENARIOS.items():
        total = cache_frames * fx.A_FRAME if local == -1 else 7 * fx.A_FRAME
        me = types.SimpleNamespace(
            num_heads=fx.A_HEADS, head_dim=d, local_attn_size=local, sink_size=sink,
            max_attention_size=total if local == -1 else local * fx.A_FRAME,
            num_iters=flags.get("num_iters", 1), use_dense_init=flags.get("use_dense_init", False),
            h_reduce=flags.get("h_reduce", 1), w_reduce=flags.get("w_reduce", 1), use_framewise=flags.get("use_framewise", False),
            disable_monarch=flags.get("disable_monarch", False), topk=None, use_svg=False, use_radial_attn=False, use_hacks=False,
            block_num=0, q=linear("q"), k=linear("k"), v=linear("v"), o=linear("o"), norm_q=norm("norm_q"), norm_k=norm("norm_k"))
        kv = {"k": torch.zeros(1, cache_frames * fx.A_FRAME, fx.A_HEADS, d, dtype=torch.float64),
              "v": torch.zeros(1, cache_frames * fx.A_FRAME, fx.A_HEADS, d, dtype=torch.float64),
              "global_end_index": torch.tensor([0], dtype=torch.long), "local_end_index": torch.tensor([0], dtype=torch.long)}
        for i, (start_frame, frames) in enumerate(calls):
            x = fx.attn_input(scen, i)
            grid = torch.tensor([[frames, fx.A_H, fx.A_W]])
            with torch.no_grad():
                y = fwd(me, x, torch.tensor([x.shape[1]]), grid, freqs, None, kv_cache=kv, current_start=start_frame * fx.A_FRAME)
            out[f"{scen}.{i}.out"] = y.numpy()
            # per cache row: a weighted sum of its elements (every call), the cache itself after the last call
            wts = torch.arange(1, fx.A_HEADS * d + 1, dtype=torch.float64).view(1, 1, fx.A_HEADS, d)
            out[f"{scen}.{i}.k_rows"] = (kv["k"] * wts).sum(dim=(2, 3)).numpy()
            out[f"{scen}.{i}.v_rows"] = (kv["v"] * wts).sum(dim=(2, 3)).numpy()
            if i + 1 == len(calls):
                out[f"{scen}.k"] = kv["k"].numpy().copy()
                out[f"{scen}.v"] = kv["v"].numpy().copy()
            out[f"{scen}.{i}.ends"] = np.array([kv["global_end_index"].item(), kv["local_end_index"].item()])
        print(scen, "ok:", [tuple(out[f"{scen}.{i}.ends"]) for i in range(len(calls))])
    # ---- cross-attention with its cache (model.py:733-768): first call fills the cache, the second reads it (the context
    # it is given then is ignored)
    cns = {"torch": torch, "flash_attention": lambda q, k, v, k_lens=None: softmax_attention(q, k, v)}
    extract(f"{REF}/model.py", ("forward",), cns, cls="WanT2VCrossAttention")
    me = types.SimpleNamespace(num_heads=fx.A_HEADS, head_dim=d, q=linear("cross.q"), k=linear("cross.k"), v=linear("cross.v"),
                               o=linear("cross.o"), norm_q=norm("cross.norm_q"), norm_k=norm("cross.norm_k"))
    cache = {"is_init": False, "k": None, "v": None}
    xs = [fx.randn(71, 1, 30, fx.A_DIM), fx.randn(72, 1, 18, fx.A_DIM)]
    ctx = [fx.randn(73, 1, 9, fx.A_DIM), fx.randn(74, 1, 9, fx.A_DIM)]
    with torch.no_grad():
        for i in range(2):
            out[f"cross.{i}.out"] = cns["forward"](me, xs[i], ctx[i], None, crossattn_cache=cache).numpy()
        out["cross.nocache"] = cns["forward"](me, xs[1], ctx[1], None).numpy()
    out["cross.k"] = cache["k"].numpy()
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
