"""Layer-adaptive cache list (reference turboquant_mlx/adaptive.py:13-57)."""
from __future__ import annotations

from .cache import TurboQuantKVCache
from .kvcache import KVCache


def make_adaptive_cache(num_layers: int, bits: int = 3, k_bits: int = None, v_bits: int = None,
                        fp16_layers: int = 4, seed: int = 42, fused: bool = False, model=None):
    """First and last `fp16_layers` layers keep an uncompressed KVCache, the rest get a
    TurboQuantKVCache.  k_bits / v_bits are accepted and ignored, as in the reference
    (adaptive.py:53-56)."""
    if model is not None and hasattr(model, "make_cache"):
        default_cache = model.make_cache()
        if default_cache and not isinstance(default_cache[0], KVCache):
            cache_type = type(default_cache[0]).__name__
            raise ValueError(
                f"[TurboQuant] Incompatible cache type: {cache_type}. "
                f"TurboQuant only works with standard multi-head attention "
                f"(KVCache). MLA, SSM, and hybrid architectures are not supported.")
    caches = []
    for i in range(num_layers):
        if i < fp16_layers or i >= num_layers - fp16_layers:
            caches.append(KVCache())
        else:
            caches.append(TurboQuantKVCache(bits=bits, seed=seed, fused=fused))
    return caches
