"""The reference's own outputs for the small pure-torch pieces around the attention path
(tests/golden/block_reference_vectors.npz, written by tests/golden/make_block_reference_vectors.py from the functions
where they lie in the reference) against the oracle and against the product's host-side counterparts.  CPU only."""
import os

import numpy as np
import pytest
import torch

import self_forcing_amd as sfa
from oracle import dense, prologue, sched

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "block_reference_vectors.npz"))


def randn(seed, *shape, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64).to(dtype)


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_rope_of_the_oracle_is_causal_rope_apply(tag):
    seed, d, F, h, w, start, H = (int(v) for v in GOLD[f"rope_{tag}_meta"])
    x = randn(seed, 1, F * h * w, H, d)
    got = prologue.rope_apply(x, (F, h, w), start_frame=start)
    np.testing.assert_allclose(got.numpy(), GOLD[f"rope_{tag}_out"], atol=1e-12, rtol=0)
    got16 = prologue.rope_apply(x.to(torch.bfloat16), (F, h, w), start_frame=start)
    assert np.array_equal(got16.float().numpy(), GOLD[f"rope_{tag}_out_bf16"])          # rotated in float64, rounded once


def test_rope_tables():
    """The oracle's angles and the table the product hands to the prologue kernel: cos / sin of the reference's complex
    table (rope_params + the three-way concatenation of causal_model.py:1352-1357)."""
    ref = GOLD["rope_table_128"]                                       # [40, 64, 2]
    ang = prologue.rope_angles(40, 128)
    np.testing.assert_allclose(np.cos(ang), ref[..., 0], atol=1e-12, rtol=0)
    np.testing.assert_allclose(np.sin(ang), ref[..., 1], atol=1e-12, rtol=0)
    table = sfa.prologue.rope_table(128, device="cpu")
    assert table.dtype == torch.float64 and table.shape[1:] == (64, 2)
    np.testing.assert_allclose(table[:40].numpy(), ref, atol=1e-12, rtol=0)


def test_rms_norm_is_wan_rms_norm():
    w = 1 + 0.1 * randn(201, 384, dtype=torch.float32)
    x = randn(202, 2, 7, 384, dtype=torch.float32) * 3
    assert np.array_equal(prologue.rms_norm(x, w, eps=1e-6).numpy(), GOLD["rms_f32"])
    xb, wb = x.to(torch.bfloat16), w.to(torch.bfloat16)
    assert np.array_equal(prologue.rms_norm(xb, wb, eps=1e-6).float().numpy(), GOLD["rms_bf16"])
    m = sfa.causal_model.WanRMSNorm(384, eps=1e-6)
    with torch.no_grad():
        m.weight.copy_(w)
    assert np.array_equal(m(x).detach().numpy(), GOLD["rms_f32"])
    assert np.array_equal(m.to(torch.bfloat16)(xb).detach().float().numpy(), GOLD["rms_bf16"])


def test_time_embedding():
    pos = torch.tensor([1000.0, 937.5, 833.3333, 625.0, 0.0, 3.0])
    got = sfa.causal_model.sinusoidal_embedding_1d(256, pos)
    assert got.dtype == torch.float64
    np.testing.assert_allclose(got.numpy(), GOLD["sinus"], atol=1e-12, rtol=0)


def test_dense_oracle_is_attention_ref():
    q, kc, vc = randn(301, 2, 5, 3, 16), randn(302, 2, 9, 3, 16), randn(303, 2, 9, 3, 16)
    nk, nv = randn(304, 2, 4, 3, 16), randn(305, 2, 4, 3, 16)
    out = dense.full_attention_with_kv_cache(q, kc, vc, nk, nv, 3, 7, sm_scale=0.3)
    np.testing.assert_allclose(out.numpy(), GOLD["attn_ref"], atol=1e-12, rtol=0)
    assert np.array_equal(kc.numpy(), GOLD["attn_ref_kcache"])          # the cache is written in place, rows 3..6


def test_scheduler_tables_and_conversions():
    sch = sfa.pipeline.FlowMatchScheduler(shift=5.0, sigma_min=0.0, extra_one_step=True)
    assert np.array_equal(sch.sigmas.numpy(), GOLD["sched_sigmas"]) and np.array_equal(sch.timesteps.numpy(), GOLD["sched_timesteps"])
    sig, ts = sched.sigma_table(shift=5.0)
    np.testing.assert_allclose(sig, GOLD["sched_sigmas"], atol=1e-6, rtol=0)        # the reference's table is float32
    np.testing.assert_allclose(ts, GOLD["sched_timesteps"], atol=1e-3, rtol=0)
    np.testing.assert_allclose(sched.warped_steps(), GOLD["sched_warped"], atol=1e-3, rtol=0)
    x0, noise = randn(401, 4, 2, 3, 3, dtype=torch.float32), randn(402, 4, 2, 3, 3, dtype=torch.float32)
    tq = torch.tensor([1000.0, 937.5, 833.0, 1.0])
    assert np.array_equal(sch.add_noise(x0, noise, tq).numpy(), GOLD["sched_add_noise"])
    wrap = sfa.pipeline.WanDiffusionWrapper.__new__(sfa.pipeline.WanDiffusionWrapper)
    torch.nn.Module.__init__(wrap)
    wrap.scheduler = sch
    flow, xt = randn(403, 4, 2, 3, 3, dtype=torch.bfloat16), randn(404, 4, 2, 3, 3, dtype=torch.bfloat16)
    assert np.array_equal(wrap._convert_flow_pred_to_x0(flow, xt, tq).float().numpy(), GOLD["sched_x0"])


def test_pipeline_warps_its_step_list_like_the_reference():
    """pipeline/causal_inference.py:33-35: timesteps[1000 - t] of the table extended by a trailing zero."""
    gen = sfa.pipeline.WanDiffusionWrapper.__new__(sfa.pipeline.WanDiffusionWrapper)
    torch.nn.Module.__init__(gen)
    gen.scheduler = sfa.pipeline.FlowMatchScheduler(shift=5.0)
    gen.model = torch.nn.Module()
    gen.model.num_layers, gen.model.num_heads, gen.model.dim, gen.model.local_attn_size = 1, 1, 128, -1
    pipe = sfa.pipeline.CausalInferencePipeline(gen)
    assert np.array_equal(torch.as_tensor(pipe.denoising_step_list).float().numpy(), GOLD["sched_warped"])
    plain = sfa.pipeline.CausalInferencePipeline(gen, warp_denoising_step=False)
    assert [int(t) for t in plain.denoising_step_list] == [1000, 750, 500, 250]
