"""End to end: the causal DiT + rollout on the GPU (HIP attention) against the SAME module code on the CPU
with oracle attention operators, same weights, same noise, same seeds."""
import pytest
import torch

import self_forcing_amd as sfa
from gpu_util import max_abs
from oracle.ops import OracleOps

pytestmark = pytest.mark.gpu
cm, pl = sfa.causal_model, sfa.pipeline
CFG = dict(dim=256, ffn_dim=512, num_heads=2, num_layers=2, text_dim=64, text_len=16, frame_hw=(6, 52),
           total_seq_len=6 * 6 * 52)


def _pair(**flags):
    torch.manual_seed(0)
    ref = cm.CausalWanModel(ops=OracleOps(), attention_flags=flags, **CFG)
    ref.init_weights(zero_head=False)
    ref = ref.to(torch.bfloat16).eval()
    dev = cm.CausalWanModel(attention_flags=flags, **CFG).to(torch.bfloat16).eval()
    dev.load_state_dict(ref.state_dict())
    return pl.WanDiffusionWrapper(ref), pl.WanDiffusionWrapper(dev.to("cuda:0"))


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.double().flatten().cpu(), b.double().flatten().cpu(), dim=0).item()


@pytest.mark.parametrize("flags", [dict(use_framewise=True), dict(use_framewise=True, h_reduce=2, use_dense_init=True),
                                   dict(disable_monarch=True), dict(use_framewise=True, num_iters=2),
                                   dict(),                                  # the reference's default tiling: f_tied = 3
                                   dict(w_reduce=2)])
def test_rollout_latents_match_oracle_model(flags):
    """2 chunks x (4 + 1) passes of a 2-layer model at the 52-column grid.  Tolerance: bf16 GEMMs differ in
    accumulation order between CPU and GPU, so latents are compared by cosine > 0.995 per chunk and
    max-abs < 5 % of the reference's range."""
    g = torch.Generator().manual_seed(0)
    noise = torch.randn(1, 6, 16, 12, 104, generator=g).to(torch.bfloat16)
    ctx = torch.randn(1, 16, 64, generator=g).to(torch.bfloat16)
    ref_gen, dev_gen = _pair(**flags)
    pipe_ref = pl.CausalInferencePipeline(ref_gen, frame_hw=(6, 52), num_cache_frames=6)
    ref = pipe_ref.inference(noise, ctx)
    pipe = pl.CausalInferencePipeline(dev_gen, frame_hw=(6, 52), num_cache_frames=6)
    out = pipe.inference(noise.to("cuda:0"), ctx.to("cuda:0"), profile=True)
    assert torch.isfinite(out).all() and len(pipe.last_chunk_ms) == 2
    for c in range(2):
        assert _cos(out[:, 3 * c:3 * c + 3], ref[:, 3 * c:3 * c + 3]) > 0.995
    assert max_abs(out, ref) < 0.05 * ref.float().abs().max().item()
    # the caches end up holding the same clean-chunk K/V, row for row (same block order), and the same counters
    for layer in range(2):
        for key in ("k", "v"):
            cd, cr = pipe.kv_cache1[layer][key], pipe_ref.kv_cache1[layer][key]
            assert _cos(cd, cr) > 0.999 and max_abs(cd, cr) < 0.05 * cr.float().abs().max().item()
        assert pipe.kv_cache1[layer]["_global_end"] == pipe_ref.kv_cache1[layer]["_global_end"] == 6 * 312
        assert int(pipe.kv_cache1[layer]["local_end_index"]) == int(pipe_ref.kv_cache1[layer]["local_end_index"]) == 6 * 312


def test_single_forward_matches_closely():
    ref_gen, dev_gen = _pair(use_framewise=True)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 3, 16, 12, 104, generator=g).to(torch.bfloat16)
    ctx = torch.randn(1, 16, 64, generator=g).to(torch.bfloat16)
    t = torch.full((1, 3), 937.5)

    def caches(device):
        kv = [{"k": torch.zeros(1, 6 * 312, 2, 128, dtype=torch.bfloat16, device=device),
               "v": torch.zeros(1, 6 * 312, 2, 128, dtype=torch.bfloat16, device=device),
               "global_end_index": torch.tensor([0], device=device), "local_end_index": torch.tensor([0], device=device)}
              for _ in range(2)]
        return kv, [{"k": None, "v": None, "is_init": False} for _ in range(2)]

    kv_r, ca_r = caches("cpu")
    kv_d, ca_d = caches("cuda:0")
    f_ref, x0_ref = ref_gen(x, {"prompt_embeds": ctx}, t, kv_r, ca_r, 0)
    f_dev, x0_dev = dev_gen(x.to("cuda:0"), {"prompt_embeds": ctx.to("cuda:0")}, t.to("cuda:0"), kv_d, ca_d, 0)
    assert _cos(f_dev, f_ref) > 0.999 and _cos(x0_dev, x0_ref) > 0.999
    # layer-0 cache rows (prologue output of the first layer) agree to one bf16 step
    assert max_abs(kv_d[0]["k"][:, :936], kv_r[0]["k"][:, :936]) <= 2 ** -5
    assert torch.equal(kv_d[0]["v"][:, 936:].cpu(), kv_r[0]["v"][:, 936:])


def test_windowed_rollout_with_ring_cache_matches_shifting_cache_on_cpu():
    """3 chunks through a 6-frame window: the GPU keeps the cache as a ring, the CPU reference run shifts it
    down as the reference does; the third chunk evicts the first."""
    torch.manual_seed(0)
    ref = cm.CausalWanModel(ops=OracleOps(), attention_flags=dict(use_framewise=True), local_attn_size=6, **CFG)
    ref.init_weights(zero_head=False)
    ref = ref.to(torch.bfloat16).eval()
    dev = cm.CausalWanModel(attention_flags=dict(use_framewise=True, ring_cache=True), local_attn_size=6, **CFG).to(torch.bfloat16).eval()
    dev.load_state_dict(ref.state_dict())
    g = torch.Generator().manual_seed(0)
    noise = torch.randn(1, 9, 16, 12, 104, generator=g).to(torch.bfloat16)
    ctx = torch.randn(1, 16, 64, generator=g).to(torch.bfloat16)
    out_ref = pl.CausalInferencePipeline(pl.WanDiffusionWrapper(ref), frame_hw=(6, 52), local_attn_size=6).inference(noise, ctx)
    pipe = pl.CausalInferencePipeline(pl.WanDiffusionWrapper(dev.to("cuda:0")), frame_hw=(6, 52), local_attn_size=6)
    out = pipe.inference(noise.to("cuda:0"), ctx.to("cuda:0"))
    assert pipe.kv_cache1[0]["_ring"] and pipe.kv_cache1[0]["_local_end"] == 3 * 312      # third chunk wrapped to the start
    for c in range(3):
        assert _cos(out[:, 3 * c:3 * c + 3], out_ref[:, 3 * c:3 * c + 3]) > 0.995


def test_pipeline_decodes_each_chunk_as_it_is_finished():
    """inference(vae=...) hands every clean chunk to one decode stream; the pixels equal decoding the finished latents in
    one go (pipeline/causal_inference.py:265) up to the convolution kernels' 16-bit rounding per call shape."""
    from self_forcing_amd import vae_decode as vd
    g = torch.Generator().manual_seed(0)
    noise = torch.randn(1, 6, 16, 12, 104, generator=g).to(torch.bfloat16).to("cuda:0")
    ctx = torch.randn(1, 16, 64, generator=g).to(torch.bfloat16).to("cuda:0")
    _, dev_gen = _pair(use_framewise=True)
    torch.manual_seed(3)
    vae = vd.WanVAEDecoder(dim=32).eval().to("cuda:0", torch.bfloat16)
    pipe = pl.CausalInferencePipeline(dev_gen, frame_hw=(6, 52), num_cache_frames=6)
    latents, video = pipe.inference(noise, ctx, vae=vae)
    assert video.shape == (1, 1 + 4 * 5, 3, 96, 832) and torch.isfinite(video).all()
    whole = vae.decode_to_pixel(latents)
    assert (video - whole).abs().max() < 5e-2 and (video - whole).abs().mean() < 3e-3
    seen = []
    pipe.inference(noise, ctx, vae=vae, on_pixels=lambda i, px: seen.append((i, px.shape[1])))
    assert seen == [(0, 9), (1, 12)]
    # the decoder on a stream of its own, beside the generator's next passes: same latents, same pixels
    pipe._seed_count = 0
    lat_a, vid_a = pipe.inference(noise, ctx, vae=vae)
    pipe._seed_count = 0
    lat_b, vid_b = pipe.inference(noise, ctx, vae=vae, decode_stream=torch.cuda.Stream())
    torch.cuda.synchronize()
    assert torch.equal(lat_a, lat_b) and torch.equal(vid_a, vid_b)


def test_next_blocks_input_formed_in_the_block_before_changes_nothing():
    """The model lets block i form block i + 1's normalised, modulated input in the pass that adds its FFN output.
    Same kernels' arithmetic on the same rounded rows: output and caches equal those of the per-block route, bit for bit."""
    _, dev_gen = _pair(use_framewise=True)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 3, 16, 12, 104, generator=g).to(torch.bfloat16).to("cuda:0")
    ctx = torch.randn(1, 16, 64, generator=g).to(torch.bfloat16).to("cuda:0")
    t = torch.full((1, 3), 500.0, device="cuda:0")

    def run():
        kv = [{"k": torch.zeros(1, 6 * 312, 2, 128, dtype=torch.bfloat16, device="cuda:0"),
               "v": torch.zeros(1, 6 * 312, 2, 128, dtype=torch.bfloat16, device="cuda:0"),
               "global_end_index": torch.tensor([0], device="cuda:0"), "local_end_index": torch.tensor([0], device="cuda:0")}
              for _ in range(2)]
        ca = [{"k": None, "v": None, "is_init": False} for _ in range(2)]
        return dev_gen(x, {"prompt_embeds": ctx}, t, kv, ca, 0)[0], kv

    fused, kv_f = run()
    dev_gen.model._summed_modulations = lambda e0: None
    plain, kv_p = run()
    assert torch.equal(fused, plain)
    for a, b in zip(kv_f, kv_p):
        assert torch.equal(a["k"], b["k"]) and torch.equal(a["v"], b["v"])
