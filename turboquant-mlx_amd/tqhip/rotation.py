"""Walsh-Hadamard rotation helpers (reference turboquant_mlx/rotation.py) on torch GPU tensors.

The butterfly itself runs in the HIP library (the query pre-rotation kernel with a
sign vector of ones); these wrappers add the normalisation and sign placement.
"""
from __future__ import annotations

import math

import torch

from . import ops

_MASK64 = 0xFFFFFFFFFFFFFFFF


def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    return z ^ (z >> 31)


def sign_pattern(d: int, seed: int) -> list:
    """The +-1 pattern for (d, seed) as python floats: +1 where the top bit of
    mix64(mix64(seed) + i) is set.  NOT the MLX PRNG stream of rotation.py:47-49 (that
    stream cannot be reproduced without MLX): a cache written by the reference is decodable
    here only if its sign vector is supplied explicitly."""
    base = _mix64(seed & _MASK64)
    return [1.0 if (_mix64((base + i) & _MASK64) >> 63) else -1.0 for i in range(d)]


def random_diagonal_sign(d: int, seed: int = 42, device=None) -> torch.Tensor:
    """rotation.py:37-49 surface: (d,) float32 tensor of +-1 (see sign_pattern for the generator)."""
    return torch.tensor(sign_pattern(d, seed), dtype=torch.float32, device=device)


def raw_butterfly(x: torch.Tensor) -> torch.Tensor:
    """Un-normalised butterfly over the last axis (stage order of rotation.py:22-32), float32."""
    d = x.shape[-1]
    assert d > 0 and (d & (d - 1)) == 0, f"Dimension must be power of 2, got {d}"
    flat = x.reshape(-1, d)
    ones = torch.ones(d, dtype=torch.float32, device=x.device)
    return ops.prerotate_query(flat, ones).reshape(x.shape)


def walsh_hadamard_transform(x: torch.Tensor) -> torch.Tensor:
    """rotation.py:7-34: butterfly then * float32(1/sqrt(d))."""
    d = x.shape[-1]
    return raw_butterfly(x) * (1.0 / math.sqrt(d))


def randomized_hadamard_transform(x: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """rotation.py:52-64: WHT(x * signs)."""
    d = x.shape[-1]
    flat = x.reshape(-1, d)
    return (ops.prerotate_query(flat, signs) * (1.0 / math.sqrt(d))).reshape(x.shape)


def inverse_randomized_hadamard(x: torch.Tensor, signs: torch.Tensor) -> torch.Tensor:
    """rotation.py:67-80: WHT(x) * signs."""
    return walsh_hadamard_transform(x) * signs.to(device=x.device, dtype=torch.float32)
