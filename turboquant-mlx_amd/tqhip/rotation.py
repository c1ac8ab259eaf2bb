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
    mix64(mix64(seed) + i) is set.  NOT the MLX PRNG stream of rotation.py:47-49: a cache written by the
    reference is decodable here only with its own sign vector, supplied explicitly (mlx_sign_pattern restates
    that stream, unverified)."""
    base = _mix64(seed & _MASK64)
    return [1.0 if (_mix64((base + i) & _MASK64) >> 63) else -1.0 for i in range(d)]


_ROT = ((13, 15, 26, 6), (17, 29, 16, 24))
_MASK32 = 0xFFFFFFFF


def threefry2x32(key: tuple, count: tuple) -> tuple:
    """Threefry-2x32, 20 rounds (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): the hash
    behind the counter-based generators of JAX and MLX.  key and count are pairs of 32-bit words."""
    ks = (key[0] & _MASK32, key[1] & _MASK32, (0x1BD11BDA ^ key[0] ^ key[1]) & _MASK32)
    x0 = (count[0] + ks[0]) & _MASK32
    x1 = (count[1] + ks[1]) & _MASK32
    for block in range(5):
        for r in _ROT[block & 1]:
            x0 = (x0 + x1) & _MASK32
            x1 = ((x1 << r) | (x1 >> (32 - r))) & _MASK32
            x1 ^= x0
        x0 = (x0 + ks[(block + 1) % 3]) & _MASK32
        x1 = (x1 + ks[(block + 2) % 3] + block + 1) & _MASK32
    return x0, x1


def mlx_sign_pattern(d: int, seed: int) -> list:
    """The +-1 pattern that rotation.py:47-49 draws -- `mx.random.key(seed)`, `mx.random.bernoulli(p=0.5,
    shape=(d,), key=key)`, True -> +1 -- restated from the published algorithm of MLX's generator (mlx >= 0.20, the
    reference's only pin, pyproject.toml:13): key = (seed >> 32, seed & 0xffffffff); the d 32-bit words come from
    threefry2x32(key, (i, i + ceil(d / 2))), first output word to element i, second to element i + ceil(d / 2)
    (for odd d the middle word is the first output of (floor(d / 2), 0)); uniform = float32(word) / float32(2^32 - 1),
    capped below 1; the mask is uniform < 0.5.  The hash is checked against its known-answer vectors; the rest
    follows MLX's source as published and CANNOT be checked without an MLX install: parity unpinned.  Use it to
    decode a cache the reference serialised (which stores only the seed); new caches keep sign_pattern."""
    import numpy as np
    key = ((seed >> 32) & _MASK32, seed & _MASK32)
    half, odd = d // 2, d & 1
    words = [0] * d
    for i in range(half):
        a, b = threefry2x32(key, (i, i + half + odd))
        words[i], words[i + half + odd] = a, b
    if odd:
        words[half] = threefry2x32(key, (half, 0))[0]
    f32 = np.float32
    u = np.asarray(words, dtype=np.uint32).astype(f32) / f32(4294967295.0)
    u = np.minimum(u, np.nextafter(f32(1.0), f32(0.0)))
    return [1.0 if x < f32(0.5) else -1.0 for x in u]


def random_diagonal_sign(d: int, seed: int = 42, device=None, stream: str = "native") -> torch.Tensor:
    """rotation.py:37-49 surface: (d,) float32 tensor of +-1.  stream="native": this library's generator
    (sign_pattern); stream="mlx": the restated MLX stream (mlx_sign_pattern, unverified)."""
    if stream not in ("native", "mlx"):
        raise ValueError(f"stream must be 'native' or 'mlx', got {stream!r}")
    pattern = sign_pattern(d, seed) if stream == "native" else mlx_sign_pattern(d, seed)
    return torch.tensor(pattern, dtype=torch.float32, device=device)


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
