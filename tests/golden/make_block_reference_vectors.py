"""Writes golden vectors of the reference's small pure-torch pieces around the attention path.

Runs ONLY in the authoring container (needs /root/reference).  The modules that hold these pieces cannot be
imported here (wan/modules/__init__.py pulls in diffusers, flashinfer and a CUDA Triton back-end), so the functions
and classes are located in the files' syntax trees and executed, from where they lie, against the installed
torch; utils/scheduler.py has no such dependencies and is imported by path.  Nothing of the reference's text is
written: block_reference_vectors.npz holds outputs only, inputs are regenerated from the seeds stored with them.

  rope_params + the table of causal_model.py:1352-1357 + causal_rope_apply   (model.py:421-428, causal_model.py:687-715)
  WanRMSNorm.forward                                                          (model.py:462-478)
  sinusoidal_embedding_1d                                                     (model.py:407-418)
  attention_ref                                                               (attn_patch.py:423-434)
  FlowMatchScheduler tables, add_noise, and _convert_flow_pred_to_x0          (utils/scheduler.py:106-176, utils/wan_wrapper.py:172-196)

    python tests/golden/make_block_reference_vectors.py
"""
import ast
import importlib.util
import os
import types

import numpy as np
import torch
import torch.nn as nn

REF = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "block_reference_vectors.npz")


def extract(path, names, ns):
    tree = ast.parse(open(path).read(), path)
    for node in tree.body:
        if isinstance(node, (ast.FunctionDef, ast.ClassDef)) and node.name in names:
            exec(compile(ast.Module(body=[node], type_ignores=[]), path, "exec"), ns)
    missing = [n for n in names if n not in ns]
    assert not missing, missing
    return ns


def method(path, cls, name, ns):
    """A single method of a class, as a plain function."""
    tree = ast.parse(open(path).read(), path)
    for node in tree.body:
        if isinstance(node, ast.ClassDef) and node.name == cls:
            for sub in node.body:
                if isinstance(sub, ast.FunctionDef) and sub.name == name:
                    exec(compile(ast.Module(body=[sub], type_ignores=[]), path, "exec"), ns)
                    return ns[name]
    raise KeyError(name)


def randn(seed, *shape, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64).to(dtype)


def main():
    ns = {"torch": torch, "nn": nn}
    extract(f"{REF}/wan/modules/model.py", ("rope_params", "sinusoidal_embedding_1d", "WanRMSNorm"), ns)
    extract(f"{REF}/wan/modules/causal_model.py", ("causal_rope_apply",), ns)
    extract(f"{REF}/wan/modules/attn_patch.py", ("attention_ref",), ns)
    out = {}

    # ---- RoPE: head dim 128, grid (3, 4, 5), start frames 0 and 7; head dim 64 with another grid
    for tag, d, grid, start, H in (("a", 128, (3, 4, 5), 0, 2), ("b", 128, (3, 4, 5), 7, 2), ("c", 64, (2, 6, 3), 19, 3)):
        freqs = torch.cat([ns["rope_params"](1024, d - 4 * (d // 6)), ns["rope_params"](1024, 2 * (d // 6)),
                           ns["rope_params"](1024, 2 * (d // 6))], dim=1)
        S = grid[0] * grid[1] * grid[2]
        x = randn(100 + ord(tag), 1, S, H, d)
        y = ns["causal_rope_apply"](x, torch.tensor([list(grid)]), freqs, start_frame=start)
        out[f"rope_{tag}_meta"] = np.array([100 + ord(tag), d, *grid, start, H])
        out[f"rope_{tag}_out"] = y.numpy()
        out[f"rope_{tag}_out_bf16"] = ns["causal_rope_apply"](x.to(torch.bfloat16), torch.tensor([list(grid)]), freqs,
                                                                start_frame=start).float().numpy()
    table = torch.cat([ns["rope_params"](1024, 128 - 4 * (128 // 6)), ns["rope_params"](1024, 2 * (128 // 6)),
                       ns["rope_params"](1024, 2 * (128 // 6))], dim=1)
    out["rope_table_128"] = torch.view_as_real(table)[:40].numpy()            # [pos, pair, (cos, sin)]

    # ---- WanRMSNorm over the model dim, float32 and bfloat16 inputs
    norm = ns["WanRMSNorm"](384, eps=1e-6)
    with torch.no_grad():
        norm.weight.copy_(1 + 0.1 * randn(201, 384, dtype=torch.float32))
    x = randn(202, 2, 7, 384, dtype=torch.float32) * 3
    out["rms_f32"] = norm(x).detach().numpy()
    nb = ns["WanRMSNorm"](384, eps=1e-6).to(torch.bfloat16)
    with torch.no_grad():
        nb.weight.copy_(norm.weight.to(torch.bfloat16))
    out["rms_bf16"] = nb(x.to(torch.bfloat16)).detach().float().numpy()

    # ---- sinusoidal time embedding
    out["sinus"] = ns["sinusoidal_embedding_1d"](256, torch.tensor([1000.0, 937.5, 833.3333, 625.0, 0.0, 3.0])).numpy()

    # ---- dense attention with a cache write (float64)
    q, kc, vc = randn(301, 2, 5, 3, 16), randn(302, 2, 9, 3, 16), randn(303, 2, 9, 3, 16)
    nk, nv = randn(304, 2, 4, 3, 16), randn(305, 2, 4, 3, 16)
    kc2, vc2 = kc.clone(), vc.clone()
    out["attn_ref"] = ns["attention_ref"](q, kc2, vc2, nk, nv, 3, 7, sm_scale=0.3, grad_only_new_kv=True).numpy()
    out["attn_ref_kcache"] = kc2.numpy()

    # ---- scheduler as utils/wan_wrapper.py:139-142 builds it, the warped step list of pipeline/causal_inference.py:33-35
    spec = importlib.util.spec_from_file_location("reference_scheduler", f"{REF}/utils/scheduler.py")
    sm = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(sm)
    sch = sm.FlowMatchScheduler(shift=5.0, sigma_min=0.0, extra_one_step=True)
    sch.set_timesteps(1000, training=True)
    out["sched_sigmas"] = sch.sigmas.numpy()
    out["sched_timesteps"] = sch.timesteps.numpy()
    ts = torch.cat((sch.timesteps.cpu(), torch.tensor([0], dtype=torch.float32)))
    out["sched_warped"] = ts[1000 - torch.tensor([1000, 750, 500, 250])].numpy()
    x0, noise = randn(401, 4, 2, 3, 3, dtype=torch.float32), randn(402, 4, 2, 3, 3, dtype=torch.float32)
    tq = torch.tensor([1000.0, 937.5, 833.0, 1.0])
    out["sched_add_noise"] = sch.add_noise(x0, noise, tq).numpy()
    conv = method(f"{REF}/utils/wan_wrapper.py", "WanDiffusionWrapper", "_convert_flow_pred_to_x0", {"torch": torch})
    holder = types.SimpleNamespace(scheduler=sch)
    flow = randn(403, 4, 2, 3, 3, dtype=torch.bfloat16)
    xt = randn(404, 4, 2, 3, 3, dtype=torch.bfloat16)
    out["sched_x0"] = conv(holder, flow, xt, tq).float().numpy()

    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes;", len(out), "arrays")


if __name__ == "__main__":
    main()
