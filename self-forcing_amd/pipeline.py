"""Few-step autoregressive rollout around the causal DiT: scheduler, x0 conversion, KV-cache ownership.

Counterpart of
    FlowMatchScheduler            utils/scheduler.py:106-176
    WanDiffusionWrapper           utils/wan_wrapper.py:117-143, 172-196, 221-292
    CausalInferencePipeline       pipeline/causal_inference.py:13-50, 51-322
Text encoder and VAE are outside this build: `inference` takes prompt embeddings and returns latents.
"""
import time

import torch
import torch.nn as nn

from .causal_model import FRAME_HEIGHT, FRAME_WIDTH, CausalWanModel, reset_cache_counters


class FlowMatchScheduler:
    """sigma ladder with shift; float32 like the reference's torch.linspace tables."""

    def __init__(self, num_inference_steps=1000, num_train_timesteps=1000, shift=5.0, sigma_max=1.0, sigma_min=0.0,
                 extra_one_step=True):
        self.num_train_timesteps, self.shift = num_train_timesteps, shift
        self.sigma_max, self.sigma_min, self.extra_one_step = sigma_max, sigma_min, extra_one_step
        self.set_timesteps(num_inference_steps)

    def set_timesteps(self, num_inference_steps):
        if self.extra_one_step:
            sig = torch.linspace(self.sigma_max, self.sigma_min, num_inference_steps + 1)[:-1]
        else:
            sig = torch.linspace(self.sigma_max, self.sigma_min, num_inference_steps)
        self.sigmas = self.shift * sig / (1 + (self.shift - 1) * sig)
        self.timesteps = self.sigmas * self.num_train_timesteps

    def _sigma(self, timestep, device):
        self.sigmas, self.timesteps = self.sigmas.to(device), self.timesteps.to(device)
        idx = torch.argmin((self.timesteps.unsqueeze(0) - timestep.unsqueeze(1)).abs(), dim=1)
        return self.sigmas[idx].reshape(-1, 1, 1, 1)

    def add_noise(self, original_samples, noise, timestep):
        """(1 - sigma_t) x0 + sigma_t noise on [B*T, C, H, W] with timestep [B*T]."""
        sigma = self._sigma(timestep.flatten(), noise.device)
        return ((1 - sigma) * original_samples + sigma * noise).type_as(noise)


class WanDiffusionWrapper(nn.Module):
    """Wraps the DiT: latents [B, F, C, H, W] in, (flow_pred, x0_pred) out."""

    def __init__(self, model, timestep_shift=5.0):
        super().__init__()
        self.model = model
        self.scheduler = FlowMatchScheduler(shift=timestep_shift, sigma_min=0.0, extra_one_step=True)

    def get_scheduler(self):
        return self.scheduler

    def _convert_flow_pred_to_x0(self, flow_pred, xt, timestep):
        """x0 = x_t - sigma_t * flow in float64 (wan_wrapper.py:172-196)."""
        dt, sch = flow_pred.dtype, self.scheduler
        tab = getattr(self, "_x0_tables", None)
        if tab is None or tab[0] is not sch.sigmas or tab[1] != flow_pred.device:
            # float64 copies of the tables on the device, made once: no host copy per pass
            self._x0_tables = tab = (sch.sigmas, flow_pred.device, sch.sigmas.double().to(flow_pred.device),
                                     sch.timesteps.double().to(flow_pred.device))
        sig, ts = tab[2], tab[3]
        idx = torch.argmin((ts.unsqueeze(0) - timestep.double().unsqueeze(1)).abs(), dim=1)
        return (xt.double() - sig[idx].reshape(-1, 1, 1, 1) * flow_pred.double()).to(dt)

    @torch.no_grad()
    def forward(self, noisy_image_or_video, conditional_dict, timestep, kv_cache=None, crossattn_cache=None,
                current_start=None):
        flow = self.model(noisy_image_or_video.permute(0, 2, 1, 3, 4), t=timestep,
                          context=conditional_dict["prompt_embeds"], kv_cache=kv_cache,
                          crossattn_cache=crossattn_cache, current_start=current_start).permute(0, 2, 1, 3, 4)
        x0 = self._convert_flow_pred_to_x0(flow.flatten(0, 1), noisy_image_or_video.flatten(0, 1),
                                           timestep.flatten(0, 1)).unflatten(0, flow.shape[:2])
        return flow, x0


class CausalInferencePipeline(nn.Module):
    """Chunk loop x denoising loop with per-layer KV caches (pipeline/causal_inference.py:182-254).

    denoising_step_list (1000, 750, 500, 250) is warped through the shifted sigma table when
    warp_denoising_step is set (`:33-35`); after the last step of a chunk the clean chunk is run once more
    at t = context_noise so that the cache holds K/V of the clean frames (`:236-245`).  The reference draws
    the re-noising randoms from a hard-coded seed list for eval consistency; here `seeds` is a parameter
    (any iterable of ints, cycled) and defaults to 0, 1, 2, ..."""

    def __init__(self, generator, denoising_step_list=(1000, 750, 500, 250), warp_denoising_step=True,
                 num_frame_per_block=3, context_noise=0, local_attn_size=-1, frame_hw=(FRAME_HEIGHT, FRAME_WIDTH),
                 num_cache_frames=21, seeds=None):
        super().__init__()
        self.generator = generator
        self.scheduler = generator.get_scheduler()
        steps = torch.tensor(denoising_step_list, dtype=torch.long)
        if warp_denoising_step:
            ts = torch.cat((self.scheduler.timesteps.cpu(), torch.tensor([0], dtype=torch.float32)))
            steps = ts[1000 - steps]
        self.denoising_step_list = steps
        self.num_frame_per_block = num_frame_per_block
        self.context_noise = context_noise
        self.local_attn_size = local_attn_size
        self.frame_seq_length = frame_hw[0] * frame_hw[1]
        self.num_cache_frames = num_cache_frames
        self.kv_cache1 = None
        self.crossattn_cache = None
        self.seeds = list(seeds) if seeds is not None else None
        self._seed_count = 0
        self.last_chunk_ms = []

    def _initialize_kv_cache(self, batch_size, dtype, device):
        m = self.generator.model
        frames = self.local_attn_size if self.local_attn_size != -1 else self.num_cache_frames
        size = frames * self.frame_seq_length
        self.kv_cache1 = [{
            "k": torch.zeros([batch_size, size, m.num_heads, m.dim // m.num_heads], dtype=dtype, device=device),
            "v": torch.zeros([batch_size, size, m.num_heads, m.dim // m.num_heads], dtype=dtype, device=device),
        } for _ in range(m.num_layers)]
        for c in self.kv_cache1:
            reset_cache_counters(c, device)

    def _initialize_crossattn_cache(self):
        self.crossattn_cache = [{"k": None, "v": None, "is_init": False} for _ in range(self.generator.model.num_layers)]

    def _reset_caches(self, device):
        for c in self.crossattn_cache:
            c["is_init"] = False
        for c in self.kv_cache1:       # only the counters are reset, not the K/V storage (`:129-138`)
            reset_cache_counters(c, device)

    def _next_seed(self):
        if self.seeds is None:
            s = self._seed_count
        else:
            s = self.seeds[self._seed_count % len(self.seeds)]
        self._seed_count += 1
        return s

    @torch.no_grad()
    def inference(self, noise, prompt_embeds, profile=False, vae=None, on_pixels=None, decode_stream=None):
        """noise [B, F, C, H, W]; prompt_embeds [B, L_text, text_dim].  Returns latents [B, F, C, H, W].

        With `vae` (a vae_decode.WanVAEDecoder) every chunk is decoded as soon as it is clean, continuing one
        decode stream (the demo's chunk-by-chunk decode, demo.py:406-441); the pixel chunks [B, T', 3, 8H, 8W]
        go to `on_pixels(chunk_index, pixels)` if given, else they are concatenated and returned as a second
        value.  The reference's offline pipeline decodes the finished video in one go instead
        (pipeline/causal_inference.py:265): call `vae.decode_to_pixel(latents)` on the result for that.
        With `decode_stream` (a torch.cuda.Stream of default priority) the decoder runs on that stream beside the
        generator's following passes (same results; 1.6 % more videos per second at 480 x 832); `on_pixels` then
        receives tensors that are complete on `decode_stream`, and the returned video is complete on the current one."""
        B, num_frames, C, H, W = noise.shape
        assert num_frames % self.num_frame_per_block == 0
        num_blocks = num_frames // self.num_frame_per_block
        cond = {"prompt_embeds": prompt_embeds}
        output = torch.zeros_like(noise)
        if self.kv_cache1 is None or self.kv_cache1[0]["k"].shape[0] != B:
            self._initialize_kv_cache(B, noise.dtype, noise.device)
            self._initialize_crossattn_cache()
        else:
            self._reset_caches(noise.device)
        self.last_chunk_ms = []
        start_frame = 0
        # The noise re-injected between denoising steps is drawn on the host, so that the same seeds give the same
        # video on any device.  All of a video's draws are made up front, in the order the steps consume the seeds,
        # into one pinned buffer that is uploaded once: a pageable upload inside the loop would wait for the GPU at
        # every step.
        n_draws = num_blocks * (len(self.denoising_step_list) - 1)
        eps_all = None
        if n_draws > 0:
            nf = self.num_frame_per_block
            host = torch.empty((n_draws, B * nf, C, H, W), dtype=noise.dtype, pin_memory=noise.is_cuda)
            for i in range(n_draws):
                g = torch.Generator().manual_seed(self._next_seed())
                host[i] = torch.randn((B * nf, C, H, W), generator=g, dtype=torch.float32)
            eps_all = host.to(noise.device, non_blocking=True)
        draw = 0
        decode_state = vae.new_state() if vae is not None else None
        pixels = []
        for block in range(num_blocks):
            nf = self.num_frame_per_block
            if profile:
                torch.cuda.synchronize(noise.device)
                t0 = time.perf_counter()
            noisy = noise[:, start_frame:start_frame + nf]
            cur = start_frame * self.frame_seq_length
            for index, cur_t in enumerate(self.denoising_step_list):
                timestep = torch.ones([B, nf], device=noise.device, dtype=torch.int64) * cur_t
                _, denoised = self.generator(noisy, cond, timestep, self.kv_cache1, self.crossattn_cache, cur)
                if index < len(self.denoising_step_list) - 1:
                    next_t = self.denoising_step_list[index + 1]
                    flat = denoised.flatten(0, 1)
                    eps = eps_all[draw]
                    draw += 1
                    noisy = self.scheduler.add_noise(
                        flat, eps, next_t * torch.ones([B * nf], device=noise.device, dtype=torch.long)
                    ).unflatten(0, denoised.shape[:2])
            output[:, start_frame:start_frame + nf] = denoised
            if vae is not None:
                if decode_stream is None:
                    px = vae.decode_to_pixel(denoised, use_cache=True, state=decode_state)
                else:
                    # the decoder runs beside the generator's next passes: it needs only this chunk's clean latents
                    decode_stream.wait_stream(torch.cuda.current_stream(noise.device))
                    with torch.cuda.stream(decode_stream):
                        px = vae.decode_to_pixel(denoised, use_cache=True, state=decode_state)
                    denoised.record_stream(decode_stream)
                if on_pixels is not None:
                    on_pixels(block, px)
                else:
                    pixels.append(px)
            ctx_t = torch.ones([B, nf], device=noise.device, dtype=torch.int64) * self.context_noise
            self.generator(denoised, cond, ctx_t, self.kv_cache1, self.crossattn_cache, cur)
            if profile:
                torch.cuda.synchronize(noise.device)
                self.last_chunk_ms.append((time.perf_counter() - t0) * 1e3)
            start_frame += nf
        if decode_stream is not None:
            torch.cuda.current_stream(noise.device).wait_stream(decode_stream)
        if vae is not None and on_pixels is None:
            return output, torch.cat(pixels, dim=1)
        return output


def use_tuned_gemms(filename=None, tune=True):
    """Lets PyTorch's TunableOp pick the hipBLASLt / rocBLAS solution of every GEMM shape around the attention
    operators (projections, FFN, embeddings).  Selections for the 1.3B shapes measured on gfx950 ship next to
    this file and are loaded first; with `tune` a shape that is not listed is timed once, on its first call.
    New selections go to a file in the temporary directory, never back into the package."""
    import os
    import tempfile
    import torch.cuda.tunable as tn
    if filename is None:
        filename = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_tuning_gfx950.csv")
    tn.enable(True)
    tn.tuning_enable(bool(tune))
    tn.set_max_tuning_duration(50)
    tn.set_max_tuning_iterations(30)
    tn.set_filename(os.path.join(tempfile.gettempdir(), f"sfm_gemm_tuning_{os.getpid()}.csv"))
    if os.path.exists(filename):
        tn.read_file(filename)


def build_generator(size="1.3B", dtype=torch.bfloat16, device="cuda:0", seed=0, zero_head=False, timestep_shift=5.0,
                    init_on_device=False, **model_overrides):
    """Random-init causal Wan generator of a named size (reference init, optionally with a non-zero head).
    `init_on_device` draws the weights on `device` instead of on the host (other values for the same seed; the 14B
    model's 56 GB of fp32 parameters take over a minute to draw on the host)."""
    from .causal_model import WAN_CONFIGS
    cfg = dict(WAN_CONFIGS[size]) if size in WAN_CONFIGS else {}
    cfg.update(model_overrides)
    torch.manual_seed(seed)
    if init_on_device:
        with torch.device(device):
            model = CausalWanModel(**cfg)
    else:
        model = CausalWanModel(**cfg)
    model.init_weights(zero_head=zero_head)
    model = model.to(dtype=dtype, device=device).eval()
    return WanDiffusionWrapper(model, timestep_shift=timestep_shift)
