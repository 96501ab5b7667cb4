"""Writes the golden output of the reference's streaming VAE decode on seeded random weights.

Runs ONLY in the authoring container (needs /root/reference).  wan/modules/vae.py is pure torch + einops
and is imported from where it lies; `WanVAE_` is built with the layout of `_video_vae` (vae.py:626-634) at
dim=32, its `conv2.*` / `decoder.*` parameters are overwritten with vae_fixture.weights_for (seeded by
name), and the two decode entry points are run in float64 on the CPU on a 5-frame latent:

  * `decode` (vae.py:548-572): the whole clip from a cleared cache,
  * `cached_decode` (vae.py:574-596): the same clip as a 2-frame chunk and a 3-frame chunk,

with scale = (mean, 1 / std) as utils/wan_wrapper.py:98-100 passes it.  Nothing of the reference's text is
written: vae_reference_vectors.npz holds the output pixels before the wrapper's clamp, the parameter names
with their shapes, and one checksum per parameter so that a test can tell that it regenerated the same
weights.

    python tests/golden/make_vae_reference_vectors.py
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import vae_fixture as fx  # noqa: E402

REF = "/root/reference/wan/modules/vae.py"
OUT = os.path.join(HERE, "vae_reference_vectors.npz")
MEAN = (-0.7571, -0.7089, -0.9113, 0.1075, -0.1745, 0.9653, -0.1517, 1.5508,
        0.4134, -0.0715, 0.5517, -0.3632, -0.1922, -0.9497, 0.2503, -0.2921)
STD = (2.8184, 1.4541, 2.3275, 2.6558, 1.2196, 1.7708, 2.6052, 2.0743,
       3.2687, 2.1526, 2.8652, 1.5579, 1.6382, 1.1253, 2.8251, 1.9160)


def main():
    spec = importlib.util.spec_from_file_location("reference_vae", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    model = mod.WanVAE_(dim=fx.DIM, z_dim=16, dim_mult=[1, 2, 4, 4], num_res_blocks=2, attn_scales=[],
                        temperal_downsample=[False, True, True], dropout=0.0).double().eval()
    sd = model.state_dict()
    names = [k for k in sd if k.startswith(("conv2.", "decoder."))]
    W = fx.weights_for({k: sd[k].shape for k in names})
    model.load_state_dict(W, strict=False)
    scale = [torch.tensor(MEAN, dtype=torch.float64), 1.0 / torch.tensor(STD, dtype=torch.float64)]
    z = fx.latent().permute(0, 2, 1, 3, 4)                # the wrapper's [B, C, T, h, w]
    with torch.no_grad():
        whole = model.decode(z, scale)
        model.clear_cache()
        chunks = torch.cat([model.cached_decode(z[:, :, :2], scale), model.cached_decode(z[:, :, 2:], scale)], 2)
    print("output", tuple(whole.shape), "abs max", whole.abs().max().item(), "fraction clamped",
          (whole.abs() > 1).double().mean().item(), "chunks - whole", (chunks - whole).abs().max().item())
    np.savez_compressed(
        OUT, seed=np.array(fx.SEED), dim=np.array(fx.DIM), names=np.array(names),
        shapes=np.array([",".join(map(str, sd[k].shape)) for k in names]),
        checksums=np.array([float((W[k] * torch.arange(1, W[k].numel() + 1, dtype=torch.float64).view(W[k].shape)
                                   .remainder(7).add(1)).sum()) for k in names]),
        decode=whole.numpy(), cached_decode_2_3=chunks.numpy())
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
