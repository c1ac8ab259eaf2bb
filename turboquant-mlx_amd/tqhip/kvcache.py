"""Plain fp16 KV cache and the causal-mask helper.

The reference leans on two pieces of the third-party mlx-lm package that are not part of
its tree: `mlx_lm.models.cache.KVCache` (v_only_cache.py:19,42; adaptive.py:9,51) and
`mlx_lm.models.base.create_causal_mask` (cache.py:328).  This module provides the small
subset of their behaviour the PolarQuant caches rely on: step-256 growth, `offset`,
`update_and_fetch`, `state`, `trim`, `make_mask`.
"""
from __future__ import annotations

import torch


def create_causal_mask(N: int, offset: int = 0, window_size=None, device=None) -> torch.Tensor:
    """Boolean (N, offset + N) mask: query row i (absolute position offset + i) may attend key j
    when j <= offset + i, and, with a window, j > offset + i - window_size."""
    rinds = torch.arange(offset + N, device=device)
    linds = torch.arange(offset, offset + N, device=device)[:, None]
    mask = linds >= rinds[None]
    if window_size is not None:
        mask = mask & (linds < rinds[None] + window_size)
    return mask


def make_mask_for(offset: int, N: int, return_array: bool = False, window_size=None, device=None):
    """The mask contract of cache.py:314-334: None for single-token decode, the string "causal"
    for a multi-token forward without an explicit array, else an offset-aware array."""
    if N == 1:
        return None
    if return_array or (window_size is not None and N > window_size):
        return create_causal_mask(N, offset=offset, window_size=window_size, device=device)
    return "causal"


class KVCache:
    """Uncompressed cache: keys/values [B, H, T_alloc, D] grown in steps of 256."""

    step = 256

    def __init__(self):
        self.keys = None
        self.values = None
        self.offset = 0

    def reserve(self, B, H, S, k_dim, v_dim, k_dtype, v_dtype, device):
        """Make room for S more positions (growth in steps of 256, zero-filled) without inserting."""
        prev = self.offset
        if self.keys is None or prev + S > self.keys.shape[2]:
            n_steps = (self.step + S - 1) // self.step
            new_k = torch.zeros((B, H, n_steps * self.step, k_dim), dtype=k_dtype, device=device)
            new_v = torch.zeros((B, H, n_steps * self.step, v_dim), dtype=v_dtype, device=device)
            if self.keys is not None:
                if prev % self.step != 0:
                    self.keys = self.keys[..., :prev, :]
                    self.values = self.values[..., :prev, :]
                self.keys = torch.cat([self.keys, new_k], dim=2)
                self.values = torch.cat([self.values, new_v], dim=2)
            else:
                self.keys, self.values = new_k, new_v

    def reallocate(self, B, H, n, k_dim, v_dim, k_dtype, v_dtype, device):
        """Fresh contiguous storage of exactly n positions holding the first `offset` positions (a capacity
        chosen by the caller, for an owner that keeps this cache in step with a second storage)."""
        new_k = torch.zeros((B, H, n, k_dim), dtype=k_dtype, device=device)
        new_v = torch.zeros((B, H, n, v_dim), dtype=v_dtype, device=device)
        if self.keys is not None and self.offset > 0:
            new_k[..., :self.offset, :] = self.keys[..., :self.offset, :]
            new_v[..., :self.offset, :] = self.values[..., :self.offset, :]
        self.keys, self.values = new_k, new_v

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        prev = self.offset
        B, H, S, k_dim = keys.shape
        self.reserve(B, H, S, k_dim, values.shape[3], keys.dtype, values.dtype, keys.device)
        self.offset += S
        self.keys[..., prev:self.offset, :] = keys
        self.values[..., prev:self.offset, :] = values
        return self.keys[..., :self.offset, :], self.values[..., :self.offset, :]

    @property
    def state(self):
        if self.keys is None:
            return []
        if self.offset == self.keys.shape[2]:
            return [self.keys, self.values]
        return [self.keys[..., :self.offset, :], self.values[..., :self.offset, :]]

    @state.setter
    def state(self, v):
        if not v:
            return
        self.keys, self.values = v
        self.offset = self.keys.shape[2]

    @property
    def meta_state(self):
        return ""

    @meta_state.setter
    def meta_state(self, v):
        if v:
            raise ValueError("KVCache has no meta_state")

    @classmethod
    def from_state(cls, state, meta_state=""):
        obj = cls()
        obj.state = state
        return obj

    def is_trimmable(self):
        return True

    def trim(self, n):
        n = min(self.offset, n)
        self.offset -= n
        return n

    def size(self):
        return self.offset

    def empty(self):
        return self.keys is None

    def make_mask(self, N, return_array: bool = False, window_size=None):
        dev = self.keys.device if self.keys is not None else None
        return make_mask_for(self.offset, N, return_array, window_size, dev)

    @property
    def nbytes(self):
        if self.keys is None:
            return 0
        return self.keys.nbytes + self.values.nbytes
