"""MI355X (gfx950) Monarch / KV-cache attention for the causal Wan DiT.

Host-side mirror of the reference's attention operators; all compute runs in the HIP
library `libsfm_attn.so` built from `csrc/` (see `build.py`).  Sub-modules keep the
reference's module names:

    monarch_attn.monarch_attn_with_kv_cache / monarch_attn.monarch_attn
    attention.attention / attention.full_attention_with_kv_cache
    prologue.qk_prologue / prologue.rope_table
    causal_model.CausalWanModel (+ self-attention, block, head), pipeline.CausalInferencePipeline
    vae_decode.WanVAEDecoder (streaming latent -> pixel decode; channels-last HIP convolutions and norms, conv_ops)
"""
from . import lib, monarch_attn, attention, prologue, causal_model, pipeline, vae_decode, linear, block_ops  # noqa: F401

__all__ = ["lib", "monarch_attn", "attention", "prologue", "causal_model", "pipeline", "vae_decode", "linear"]
