"""The product's sampler loop (`pipeline.CausalInferencePipeline.inference`) against what the reference's own
`CausalInferencePipeline.inference` produced and how it called the generator
(tests/golden/pipeline_reference_vectors.npz, written by tests/golden/make_pipeline_reference_vectors.py) with the same
stand-in generator, inputs and seeds, two videos in a row (the second after the cache reset).  CPU."""
import json
import os
import sys

import numpy as np
import torch

import self_forcing_amd as sfa

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import block_fixture as fx  # noqa: E402

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pipeline_reference_vectors.npz"))


def test_sampler_loop_reproduces_the_reference_inference():
    sch = sfa.pipeline.FlowMatchScheduler(shift=5.0, sigma_min=0.0, extra_one_step=True)
    gen = fx.GeneratorStandIn(sch)
    pipe = sfa.pipeline.CausalInferencePipeline(gen, frame_hw=(2, 3), seeds=[int(s) for s in GOLD["seeds"]])
    X = fx.pipeline_inputs()
    for run in range(2):
        gen.calls.clear()
        lat = pipe.inference(X["noise"] + run, X["prompt"])
        calls = json.loads(str(GOLD[f"calls{run}"]))
        got = json.loads(json.dumps(gen.calls))
        assert len(got) == len(calls) == 10                  # 2 chunks x (4 denoising passes + 1 clean re-run)
        for i, (g, c) in enumerate(zip(got, calls)):
            assert g == c, (run, i, g, c)                     # shape, timesteps, start token, cache end seen, cross cache state
        np.testing.assert_allclose(lat.numpy(), GOLD[f"latents{run}"], atol=1e-6, rtol=0)
    assert pipe._seed_count == len(GOLD["seeds"]) == 12       # 2 videos x 2 chunks x 3 re-noising draws
