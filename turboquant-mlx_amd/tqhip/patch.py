"""Attention dispatcher for models that keep PolarQuant caches (counterpart of patch.py:1-90).

The reference monkey-patches `mlx_lm.models.base.scaled_dot_product_attention(queries, keys,
values, cache, scale, mask)` so that a decode step on a fused TurboQuantKVCache reads the packed
storage instead of the placeholder K/V that `update_and_fetch` returned (patch.py:14-41).  There
is no mlx-lm here; the same dispatcher is offered as a plain function with that signature, and
`apply_patch(module, ...)` installs it over the `scaled_dot_product_attention` attribute of
whatever torch model modules the caller names (the reference walks `sys.modules` for mlx-lm's).

Beyond the reference: a multi-token step on a fused cache is served from the packed storage too
(the reference falls through to stock SDPA over its zero placeholders there), and a decode step on
a VOnlyTurboQuantCache skips the dequantised value buffer.
"""
from __future__ import annotations

import torch

from .attention import turboquant_attention, turboquant_prefill_attention, vonly_decode_attention
from .cache import TurboQuantKVCache
from .v_only_cache import VOnlyTurboQuantCache

_patched = {}          # id(module) -> (module, original attribute or _MISSING)
_MISSING = object()


def _stock_sdpa(queries, keys, values, scale, mask):
    if keys.dtype != queries.dtype:            # a V-only cache hands out float16 keys whatever the model's dtype
        keys = keys.to(queries.dtype)
    if values.dtype != queries.dtype:
        values = values.to(queries.dtype)
    n_rep = queries.shape[1] // keys.shape[1]
    if n_rep > 1:
        keys = keys.repeat_interleave(n_rep, dim=1)
        values = values.repeat_interleave(n_rep, dim=1)
    if isinstance(mask, str):
        if mask != "causal":
            raise ValueError(f"unknown mask {mask!r}")
        S, T = queries.shape[2], keys.shape[2]
        mask = torch.ones((S, T), dtype=torch.bool, device=queries.device).tril(T - S)
    return torch.nn.functional.scaled_dot_product_attention(queries, keys, values, attn_mask=mask, scale=scale)


def scaled_dot_product_attention(queries, keys, values, cache, scale, mask=None, sinks=None):
    """patch.py:14-41 on torch tensors.  queries (B, n_heads, S, dim); keys / values as returned by
    `cache.update_and_fetch`; mask None, "causal" or an array (the contract of cache.make_mask)."""
    if sinks is not None:
        raise ValueError("attention sinks are not supported")
    is_decode = queries.shape[2] == 1
    if isinstance(cache, TurboQuantKVCache) and not cache.v_only and cache.offset > 0 and cache.fused:
        if is_decode:
            # one library call either way; with a threshold, shapes outside the matrix-core kernels compose the ops
            return turboquant_attention(queries, cache, scale, mask, sparse_v_threshold=cache.sparse_v_threshold,
                                        fused=True)
        if mask is None or (isinstance(mask, str) and mask == "causal"):
            return turboquant_prefill_attention(queries, cache, scale, causal=mask is not None)
        raise ValueError("a fused TurboQuantKVCache holds no dequantised K/V: a multi-token step takes "
                         "mask=None or mask='causal' (cache.make_mask(N)), not an explicit array")
    if isinstance(cache, VOnlyTurboQuantCache) and cache.offset > 0:
        if is_decode:
            return vonly_decode_attention(queries, cache, scale, mask,
                                          sparse_v_threshold=getattr(cache, "sparse_v_threshold", None))
        if cache.fused:                    # the values handed in are a placeholder
            values = cache.dequantized_values(queries.dtype)
    return _stock_sdpa(queries, keys, values, scale, mask)


def apply_patch(*modules):
    """Install the dispatcher as `scaled_dot_product_attention` of each given module (or any object
    with attributes); idempotent.  patch.py:44-72."""
    for m in modules:
        if id(m) in _patched:
            continue
        _patched[id(m)] = (m, getattr(m, "scaled_dot_product_attention", _MISSING))
        m.scaled_dot_product_attention = scaled_dot_product_attention


def remove_patch():
    """Undo every apply_patch.  patch.py:75-90."""
    for m, orig in list(_patched.values()):
        if orig is _MISSING:
            delattr(m, "scaled_dot_product_attention")
        else:
            m.scaled_dot_product_attention = orig
    _patched.clear()
