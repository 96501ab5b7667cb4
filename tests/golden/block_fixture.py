"""Seeded sub-layers and inputs shared by make_wiring_reference_vectors.py (which plugs them into the reference's own
`CausalWanAttentionBlock.forward` / `CausalHead.forward`) and by tests/test_block_reference_wiring.py (which plugs
the same ones into the product's block and head).  The attention sub-layers are stand-ins: any deterministic
function of their inputs shows whether the wiring around them (which modulation row goes where, the `1 +`, the
residual sums) is the reference's."""
import torch
import torch.nn as nn

DIM, FFN, FRAMES, FRAME_TOKENS, CTX = 48, 112, 3, 10, 7
EPS = 1e-6


def randn(seed, *shape):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


class SelfAttnStandIn(nn.Module):
    """y = x W + (token index) * u: depends on every input channel and on the token's position."""

    def __init__(self):
        super().__init__()
        self.w = nn.Parameter(randn(11, DIM, DIM) / DIM ** 0.5)
        self.u = nn.Parameter(randn(12, DIM) * 0.01)

    def apply_to(self, x):
        pos = torch.arange(x.shape[1], dtype=x.dtype).view(1, -1, 1)
        return x @ self.w + pos * self.u


class CrossAttnStandIn(nn.Module):
    """y = tanh(x W) + mean over the context tokens of (context V)."""

    def __init__(self):
        super().__init__()
        self.w = nn.Parameter(randn(13, DIM, DIM) / DIM ** 0.5)
        self.v = nn.Parameter(randn(14, DIM, DIM) / DIM ** 0.5)

    def apply_to(self, x, context):
        return torch.tanh(x @ self.w) + (context @ self.v).mean(dim=1, keepdim=True)


def parameters():
    """name -> tensor for the block's and the head's own parameters."""
    return {
        "modulation": randn(21, 1, 6, DIM) / DIM ** 0.5,
        "norm3.weight": 1 + 0.2 * randn(22, DIM), "norm3.bias": 0.1 * randn(23, DIM),
        "ffn.0.weight": randn(24, FFN, DIM) / DIM ** 0.5, "ffn.0.bias": 0.1 * randn(25, FFN),
        "ffn.2.weight": randn(26, DIM, FFN) / FFN ** 0.5, "ffn.2.bias": 0.1 * randn(27, DIM),
        "head.modulation": randn(28, 1, 2, DIM) / DIM ** 0.5,
        "head.head.weight": randn(29, 16, DIM) / DIM ** 0.5, "head.head.bias": 0.1 * randn(30, 16),
    }


def inputs():
    L = FRAMES * FRAME_TOKENS
    return {"x": randn(31, 2, L, DIM), "e": 0.5 * randn(32, 2, FRAMES, 6, DIM), "context": randn(33, 2, CTX, DIM),
            "e_head": 0.5 * randn(34, 2, FRAMES, 1, DIM)}


# ---- whole-model wiring (embeddings -> blocks -> head -> unpatchify) -----------------------------------------------
M_DIM, M_IN, M_OUT, M_FREQ, M_TEXT, M_TEXT_LEN, M_LAYERS = 32, 4, 4, 16, 24, 6, 2
M_PATCH = (1, 2, 2)
M_LATENT = (2, M_IN, 3, 4, 6)            # [B, C, F, H, W] -> 3 frames of 2 x 3 tokens


def model_parameter(name, shape):
    import zlib
    t = randn(zlib.crc32(name.encode()) & 0x7FFFFFFF, *shape)
    if name.endswith(".bias"):
        return 0.1 * t
    fan_in = 1
    for s in shape[1:]:
        fan_in *= s
    return t / max(fan_in, 1) ** 0.5


def model_inputs():
    return {"x": randn(51, *M_LATENT), "t": torch.tensor([[1000.0, 937.5, 833.0], [625.0, 625.0, 3.0]], dtype=torch.float64),
            "context": randn(52, 2, 5, M_TEXT)}            # 5 text tokens: padded to M_TEXT_LEN by the model


def block_stand_in(x, e, context, index):
    """Stands in for a whole attention block: uses every one of the six modulation rows with its own weight, per frame,
    and the embedded context."""
    nf = e.shape[1]
    fs = x.shape[1] // nf
    coef = sum((r + 1) * e[:, :, r] for r in range(6))                        # [B, F, C]
    y = x + 0.1 * (index + 1) * (torch.tanh(x).unflatten(1, (nf, fs)) * coef.unsqueeze(2)).flatten(1, 2)
    return y + 0.01 * context.mean(dim=1, keepdim=True)


# ---- self-attention with the KV cache (cache state machine, RoPE start frame, dispatch) ---------------------------------
A_DIM, A_HEADS, A_H, A_W = 32, 2, 4, 6
A_FRAME = A_H * A_W

# name -> (local_attn_size, sink_size, cache frames, flags, [(current_start in frames, chunk frames), ...])
A_SCENARIOS = {
    # whole-history cache, framewise Monarch; every chunk is run twice (a denoising pass, then the clean re-run)
    "full_framewise": (-1, 0, 7, dict(use_framewise=True), [(0, 2), (0, 2), (2, 2), (2, 2), (4, 3), (4, 3)]),
    # three frames tied per block, h_reduce = 2, dense attention on the first chunk (USE_DENSE_INIT)
    "tied_reduce_init": (-1, 0, 6, dict(h_reduce=2, use_dense_init=True), [(0, 3), (0, 3), (3, 3), (3, 3)]),
    # window of 4 frames with one sink frame: evictions from the fifth frame on, re-runs after an eviction
    "window_sink": (4, 1, 4, dict(use_framewise=True), [(0, 1), (1, 1), (2, 1), (3, 1), (4, 1), (4, 1), (5, 1), (6, 2), (6, 2)]),
    # Monarch disabled: dense attention, cache in token order, window without sink
    "dense_window": (3, 0, 3, dict(disable_monarch=True), [(0, 1), (1, 2), (3, 1), (3, 1), (4, 2)]),
    # refinement passes
    "iters": (-1, 0, 4, dict(use_framewise=True, num_iters=3), [(0, 2), (2, 2), (2, 2)]),
}


def attn_parameter(name, shape):
    import zlib
    t = randn((zlib.crc32(("attn." + name).encode()) & 0x7FFFFFFF), *shape)
    if name.endswith(".bias"):
        return 0.1 * t
    if name.startswith("norm_"):
        return 1 + 0.2 * t
    return t / shape[-1] ** 0.5


def attn_input(scenario, call):
    import zlib
    _, _, _, _, calls = A_SCENARIOS[scenario]
    frames = calls[call][1]
    return randn(zlib.crc32(f"{scenario}.{call}".encode()) & 0x7FFFFFFF, 1, frames * A_FRAME, A_DIM)


# ---- the sampler's chunk loop (pipeline) ------------------------------------------------------------------------------
P_FRAMES, P_C, P_H, P_W, P_FRAME_TOKENS = 6, 2, 4, 6, 6            # latents [1, 6, 2, 4, 6]; 6 tokens per frame after patching


class GeneratorStandIn(nn.Module):
    """Stands in for the wrapped DiT: a deterministic function of the noisy latents, the timestep, the chunk's start
    token and the prompt, and a log of what it was called with."""

    def __init__(self, scheduler):
        super().__init__()
        self.scheduler = scheduler
        self.model = types_namespace(num_layers=2, num_heads=2, dim=8, local_attn_size=-1)
        self.calls = []

    def get_scheduler(self):
        return self.scheduler

    def forward(self, noisy_image_or_video, conditional_dict, timestep, kv_cache=None, crossattn_cache=None, current_start=None):
        t = timestep.float()
        self.calls.append((tuple(noisy_image_or_video.shape), [round(float(v), 3) for v in t.flatten().tolist()], int(current_start),
                           int(kv_cache[0]["global_end_index"].item()), bool(crossattn_cache[0]["is_init"])))
        for c in crossattn_cache:
            c["is_init"] = True
        for c in kv_cache:                                   # what the model's self-attention does to the counters
            c["global_end_index"].fill_(int(current_start) + noisy_image_or_video.shape[1] * P_FRAME_TOKENS)
        x0 = (0.8 * noisy_image_or_video + 0.1 * torch.sin(t / 100.0).view(*t.shape, 1, 1, 1) + 1e-3 * float(current_start)
              + 0.05 * conditional_dict["prompt_embeds"].mean())
        return -x0, x0


def types_namespace(**kw):
    import types
    return types.SimpleNamespace(**kw)


def pipeline_inputs():
    g = torch.Generator().manual_seed(61)
    return {"noise": torch.randn(1, P_FRAMES, P_C, P_H, P_W, generator=g), "prompt": torch.randn(1, 5, 4, generator=g)}
