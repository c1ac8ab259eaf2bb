"""PolarQuantizer (reference turboquant_mlx/quantizer.py:47-132) on top of the HIP codec."""
from __future__ import annotations

import math

import torch

from . import ops
from .rotation import random_diagonal_sign

# quantizer.py:27-36 / cache.py:15-25
CODEBOOKS = {
    1: (-0.7979, 0.7979),
    2: (-1.5104, -0.4528, 0.4528, 1.5104),
    3: (-2.1520, -1.3440, -0.7560, -0.2451, 0.2451, 0.7560, 1.3440, 2.1520),
    4: (-2.7326, -2.0690, -1.6180, -1.2562, -0.9423, -0.6568, -0.3881, -0.1284,
        0.1284, 0.3881, 0.6568, 0.9423, 1.2562, 1.6180, 2.0690, 2.7326),
}


def gaussian_codebook(bits: int) -> torch.Tensor:
    """quantizer.py:18-38: Lloyd-Max N(0,1) centroids, float32 (host tensor)."""
    if bits not in CODEBOOKS:
        raise ValueError(f"Unsupported bit width: {bits}. Use 1-4.")
    return torch.tensor(CODEBOOKS[bits], dtype=torch.float32)


def gaussian_boundaries(centroids: torch.Tensor) -> torch.Tensor:
    """quantizer.py:41-44: float32 midpoints."""
    return (centroids[:-1] + centroids[1:]) / 2.0


class PolarQuantizer:
    """quantizer.py:47-132.  quantize -> (uint8 indices, float32 norms); dequantize inverts it.

    The tables live on the host (they reach the kernels by value); `signs` lives on `device`.
    """

    def __init__(self, dim: int, bits: int = 3, seed: int = 42, device=None):
        self.dim = dim
        self.bits = bits
        self.n_levels = 2 ** bits
        self.centroids = gaussian_codebook(bits)
        self.boundaries = gaussian_boundaries(self.centroids)
        self.scale = 1.0 / math.sqrt(dim)
        self.device = torch.device(device) if device is not None else torch.device("cuda")
        self.signs = random_diagonal_sign(dim, seed=seed, device=self.device)

    def quantize(self, x: torch.Tensor):
        lead = x.shape[:-1]
        packed, norms = ops.fused_quantize(x.reshape(-1, self.dim), self.signs, self.boundaries,
                                           self.dim, self.bits, variant="mlx")
        idx = ops.unpack_indices(packed, self.bits, self.dim)
        return idx.reshape(*lead, self.dim), norms.reshape(lead)

    def dequantize(self, indices: torch.Tensor, norms: torch.Tensor) -> torch.Tensor:
        lead = indices.shape[:-1]
        packed = ops.pack_indices(indices.reshape(-1, self.dim), self.bits)
        out = ops.packed_dequantize(packed, norms.reshape(-1), self.centroids, self.signs, self.dim, self.bits)
        return out.reshape(*lead, self.dim)
