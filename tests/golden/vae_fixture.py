"""Seeded weights and latents shared by make_vae_reference_vectors.py (which feeds them to the reference's
decoder) and by the tests (which feed them to the oracle and to the product module).  Every tensor is drawn
from a generator seeded by its own state-dict name, so the values do not depend on the order in which an
implementation lists its parameters."""
import zlib

import torch

SEED = 20240611
LATENT_SHAPE = (1, 5, 16, 3, 4)          # [B, T, C, h, w], the generator's layout
DIM = 32


def tensor_for(name, shape, seed=SEED):
    g = torch.Generator().manual_seed((zlib.crc32(name.encode()) ^ seed) & 0x7FFFFFFF)
    t = torch.randn(*shape, generator=g, dtype=torch.float64)
    if name.endswith(".gamma"):
        return 1.0 + 0.2 * t
    if name.endswith(".bias"):
        return 0.1 * t
    fan_in = 1
    for s in shape[1:]:
        fan_in *= s
    return t * (1.25 / fan_in ** 0.5)


def weights_for(shapes, seed=SEED):
    """shapes: {state-dict name: shape} of the `conv2.*` and `decoder.*` entries."""
    return {k: tensor_for(k, tuple(s), seed) for k, s in shapes.items()}


def latent(seed=SEED):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*LATENT_SHAPE, generator=g, dtype=torch.float64)
