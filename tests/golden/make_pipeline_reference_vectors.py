"""Writes what the reference's own sampler loop (`CausalInferencePipeline.inference`, pipeline/causal_inference.py:
60-270, with `_initialize_kv_cache` / `_initialize_crossattn_cache` :288-322) produces and how it calls the generator,
on a stand-in generator (block_fixture.GeneratorStandIn), run twice in a row (the second run exercises the cache reset).

Runs ONLY in the authoring container (needs /root/reference).  The methods are located in the file's syntax tree and
executed, from where they lie, as plain functions; the scheduler is the reference's utils/scheduler.py imported by
path; the warped step list is computed by the lines of `__init__` that do it (:31-35), restated here in two lines.
Written: the output latents, the call log, and the entries of the reference's `rand_seeds` list that the runs consumed
(data; the product takes the seeds as a parameter).

    python tests/golden/make_pipeline_reference_vectors.py
"""
import ast
import importlib.util
import json
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import block_fixture as fx  # noqa: E402

REF = "/root/reference/pipeline/causal_inference.py"
OUT = os.path.join(HERE, "pipeline_reference_vectors.npz")


def main():
    tree = ast.parse(open(REF).read(), REF)
    from typing import List, Optional
    ns = {"torch": torch, "List": List, "Optional": Optional, "total_seq_len": 21 * fx.P_FRAME_TOKENS, "seed_count": 0}
    for node in tree.body:
        if isinstance(node, ast.Assign) and getattr(node.targets[0], "id", None) == "rand_seeds":
            ns["rand_seeds"] = ast.literal_eval(node.value)
    cls = [n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == "CausalInferencePipeline"][0]
    for sub in cls.body:
        if isinstance(sub, ast.FunctionDef) and sub.name in ("inference", "_initialize_kv_cache", "_initialize_crossattn_cache"):
            exec(compile(ast.Module(body=[sub], type_ignores=[]), REF, "exec"), ns)

    spec = importlib.util.spec_from_file_location("reference_scheduler", "/root/reference/utils/scheduler.py")
    sm = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(sm)
    sch = sm.FlowMatchScheduler(shift=5.0, sigma_min=0.0, extra_one_step=True)
    sch.set_timesteps(1000, training=True)
    gen = fx.GeneratorStandIn(sch)
    timesteps = torch.cat((sch.timesteps.cpu(), torch.tensor([0], dtype=torch.float32)))
    me = types.SimpleNamespace(
        generator=gen, scheduler=sch, text_encoder=lambda text_prompts: {"prompt_embeds": text_prompts},
        vae=types.SimpleNamespace(decode_to_pixel=lambda x, use_cache=False: x),
        denoising_step_list=timesteps[1000 - torch.tensor([1000, 750, 500, 250], dtype=torch.long)],
        num_transformer_blocks=2, frame_seq_length=fx.P_FRAME_TOKENS, kv_cache1=None, crossattn_cache=None,
        args=types.SimpleNamespace(context_noise=0), num_frame_per_block=3, independent_first_frame=False, local_attn_size=-1)
    me._initialize_kv_cache = lambda **kw: ns["_initialize_kv_cache"](me, **kw)
    me._initialize_crossattn_cache = lambda **kw: ns["_initialize_crossattn_cache"](me, **kw)
    X = fx.pipeline_inputs()
    outs = {}
    with torch.no_grad():
        for run in range(2):
            gen.calls.clear()
            _, lat = ns["inference"](me, X["noise"] + run, X["prompt"], return_latents=True)
            outs[f"latents{run}"] = lat.numpy()
            outs[f"calls{run}"] = np.array(json.dumps(gen.calls))
    outs["seeds"] = np.array(ns["rand_seeds"][:ns["seed_count"]])
    np.savez_compressed(OUT, **outs)
    print("wrote", OUT, os.path.getsize(OUT), "bytes;", ns["seed_count"], "seeds used;", len(gen.calls), "generator calls per run")


if __name__ == "__main__":
    main()
