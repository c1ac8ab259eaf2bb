"""VOnlyTurboQuantCache (reference turboquant_mlx/v_only_cache.py:24-127): fp16 keys in a plain
KVCache, values PolarQuant-compressed in a TurboQuantKVCache(v_only=True)."""
from __future__ import annotations

import torch

from .cache import TurboQuantKVCache, _round_up
from .kvcache import KVCache


class VOnlyTurboQuantCache:
    """update_and_fetch stores K in fp16, compresses V and returns (K_fp16, V_dequantised).
    With no_v_buffer=True the fp16 V buffer is not kept: V is re-dequantised from the packed
    storage on every call (v_only_cache.py:41-49).

    fused=True (not in the reference, which relies on MLX never evaluating an unused dequant; same
    meaning as TurboQuantKVCache(fused=True), cache.py:162-165): V is only encoded, and the second
    return value is a stride-0 all-zero placeholder of the right shape.  For callers that read the
    packed values directly (vonly_decode_attention, tqhip.patch); `dequantized_values()` gives the
    fp16 values when a multi-token step needs them."""

    def __init__(self, bits: int = 3, seed: int = 42, no_v_buffer: bool = False, fused: bool = False, v_signs=None,
                 sign_stream: str = "native"):
        """v_signs ([dim] of +-1): the value rotation's sign vector, used instead of the one derived from
        `seed + 1` (cache.py:96); sign_stream ("native" | "mlx"): the generator that derives it otherwise, as for
        TurboQuantKVCache.  Everything else as the reference (v_only_cache.py:41-49) plus `fused`."""
        self._k_cache = KVCache()
        self._v_tq = TurboQuantKVCache(bits=bits, seed=seed, v_only=True, v_signs=v_signs, sign_stream=sign_stream)
        self._v_bits = bits
        self._no_v_buffer = no_v_buffer
        self.fused = fused
        self._zero, self._zero_key = None, None
        self._step, self._step_key = None, None

    def _encode_only(self, keys, values):
        tq = self._v_tq
        B, H, S, v_dim = values.shape
        tq._dtype = keys.dtype
        tq._ensure_quantizer(keys.shape[-1], v_dim, values.device)
        tq._ensure_storage(B, H, S, values.device)
        tq._encode(values, tq._v_q, tq.v_packed, tq.v_norms, B, H, S, v_dim, tq.offset)
        tq.offset += S

    def _align_storage(self, B, H, S, dim, v_dtype, device):
        """Room for S more positions with ONE capacity for the key cache and the packed values, both
        contiguous: the single-call decode step describes all four tensors by one t_alloc.  The two storages
        grow by different rules when they are filled through their own update_and_fetch (the key cache trims
        to its offset and appends whole steps, the packed storage rounds offset + S up to a step) or are
        restored from `state` slices, so they are brought to round_up(max(needed, either capacity), 256)
        here; nothing moves when they already agree and have room."""
        kc, tq = self._k_cache, self._v_tq
        need = kc.offset + S
        have_k = 0 if kc.keys is None else kc.keys.shape[2]
        have_v = 0 if tq.v_packed is None else tq.v_packed.shape[2]
        n = _round_up(max(need, have_k, have_v), tq.step)
        if (have_k != n or not kc.keys.is_contiguous() or not kc.values.is_contiguous()
                or kc.keys.dtype != torch.float16 or kc.values.dtype != v_dtype):
            if kc.keys is not None and (kc.keys.dtype != torch.float16 or kc.values.dtype != v_dtype):
                raise ValueError("the stored keys must be float16 and the stored values of the new values' dtype")
            kc.reallocate(B, H, n, dim, dim, torch.float16, v_dtype, device)
        if have_v != n or not tq.v_packed.is_contiguous() or not tq.v_norms.is_contiguous():
            tq._reallocate(B, H, n, device)

    # Decode-sized inserts of a fused cache go through one launch (key rows to float16, value rows
    # raw and encoded) instead of two slice assignments, a cast and the encoder.
    _FUSED_APPEND_MAX_TOKENS = 16

    def _append_fused(self, keys, values) -> bool:
        from . import ops
        kc, tq = self._k_cache, self._v_tq
        B, H, S, v_dim = values.shape
        if (S > self._FUSED_APPEND_MAX_TOKENS or keys.shape != values.shape or not values.is_cuda
                or (kc.values is not None and kc.values.dtype != values.dtype)
                or (kc.keys is not None and kc.keys.dtype != torch.float16)
                or kc.offset != tq.offset):
            return False
        tq._dtype = keys.dtype
        tq._ensure_quantizer(keys.shape[-1], v_dim, values.device)
        self._align_storage(B, H, S, v_dim, values.dtype, values.device)
        ops.vonly_append_into(keys, values, tq._v_q.signs, tq._v_q.boundaries, kc.keys, kc.values,
                              tq.v_packed, tq.v_norms, position=kc.offset, bits=tq.quant_bits,
                              variant=tq.encode_variant)
        kc.offset += S
        tq.offset += S
        return True

    def reserve(self, B: int, H: int, n_positions: int, dim: int, dtype=torch.float16, device="cuda"):
        """Allocate storage for `n_positions` more positions now, so that steps recorded in a HIP graph keep
        their addresses for that long (storage otherwise grows in steps of 256, which reallocates)."""
        kc, tq = self._k_cache, self._v_tq
        device = torch.device(device)
        tq._ensure_quantizer(dim, dim, device)
        if kc.offset != tq.offset:
            raise ValueError("keys and values hold different numbers of positions")
        self._align_storage(B, H, n_positions, dim, dtype if kc.values is None else kc.values.dtype, device)

    def set_offset(self, n: int):
        """Set the number of valid positions (keys and values alike): for a caller that replayed recorded steps
        with a device-side position and now tells the host-side bookkeeping how far the cache has got."""
        have_k = 0 if self._k_cache.keys is None else self._k_cache.keys.shape[2]
        have_v = 0 if self._v_tq.v_packed is None else self._v_tq.v_packed.shape[2]
        if not 0 <= n <= min(have_k, have_v):
            raise ValueError(f"offset {n} outside the storage")
        self._k_cache.offset = n
        self._v_tq.offset = n

    def decode_step(self, queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, attn_scale: float,
                    position: torch.Tensor | None = None, out: torch.Tensor | None = None):
        """Insert one token and attend in one library call: the result of `update_and_fetch(keys, values)`
        followed by `vonly_decode_attention(queries, self, attn_scale)` (no mask, no sparse-V threshold).
        queries (B, n_heads, 1, dim), keys / values (B, n_kv, 1, dim) -> (B, n_heads, 1, dim) in queries.dtype.
        Not in the reference, where the two halves are separate calls of the model's attention layer
        (v_only_cache.py:52-78, then SDPA).

        With `position` (one-element int64 GPU tensor holding the cache's current offset) the kernels read the
        insert position and the attended length from it when they run: the step can be recorded in a HIP graph
        once and replayed, the caller advancing the tensor by one after every step and calling `set_offset`
        when it is done replaying; `reserve` keeps the storage from moving meanwhile.  `out` (B, n_heads, dim)
        receives the result when given."""
        from . import attention, ops
        kc, tq = self._k_cache, self._v_tq
        B, n_q, S_q, dim = queries.shape
        H = values.shape[1]
        if (S_q != 1 or values.shape[2] != 1 or keys.shape != values.shape or n_q % H or not values.is_cuda
                or queries.dtype not in ops._DTYPES or keys.dtype not in ops._DTYPES or values.dtype not in ops._DTYPES
                or (kc.values is not None and kc.values.dtype != values.dtype)
                or (kc.keys is not None and kc.keys.dtype != torch.float16) or kc.offset != tq.offset):
            if position is not None:
                raise ValueError("a step with a device-side position needs one new token, float16/bfloat16/float32 "
                                 "queries and a cache whose stored values have the dtype of the new ones")
            self.update_and_fetch(keys, values)
            return attention.vonly_decode_attention(queries, self, attn_scale)
        tq._dtype = keys.dtype
        tq._ensure_quantizer(dim, dim, values.device)
        self._align_storage(B, H, 1, dim, values.dtype, values.device)
        key = (kc.keys.data_ptr(), kc.values.data_ptr(), tq.v_packed.data_ptr(), tq.v_norms.data_ptr(),
               kc.keys.shape[2], n_q)
        if self._step_key != key:
            try:
                self._step = ops.VOnlyStep(kc.keys, kc.values, tq.v_packed, tq.v_norms, tq._v_q.signs,
                                           tq._v_q.boundaries, tq._v_q.centroids, n_rep=n_q // H,
                                           bits=tq.quant_bits, variant=tq.encode_variant)
            except ValueError:                     # a shape the single call does not serve
                if position is not None:
                    raise
                self.update_and_fetch(keys, values)
                return attention.vonly_decode_attention(queries, self, attn_scale)
            self._step_key = key
        if position is not None and (position.dtype != torch.int64 or position.numel() != 1 or not position.is_cuda):
            raise ValueError("a device-side position must be a one-element int64 tensor on the GPU")
        sb, sh_, _, sd = self._step.shape
        if (sb, sh_, sd) != (B, H, dim) or values.shape[0] != B or not (queries.is_cuda and keys.is_cuda):
            raise ValueError(f"the cache stores {sb} x {sh_} groups of dim {sd} on the GPU; got queries {tuple(queries.shape)}, "
                             f"keys {tuple(keys.shape)} on {keys.device}")
        if out is None:
            res = torch.empty((B, n_q, 1, dim), dtype=queries.dtype, device=queries.device)
        elif out.numel() != B * n_q * dim or not out.is_contiguous() or not out.is_cuda or out.dtype not in ops._DTYPES:
            raise ValueError(f"out must be a contiguous GPU tensor of {B} x {n_q} x {dim} elements")
        else:
            res = out
        ops.step_call_unchecked(self._step, keys.contiguous(), values.contiguous(), queries.contiguous(),
                                kc.offset if position is None else position, attn_scale, res, packed=False)
        kc.offset += 1
        tq.offset += 1
        return res if res.dim() == 4 else res[:, :, None, :]

    def dequantized_values(self, dtype=None) -> torch.Tensor:
        """All cached values, dequantised: [B, H, offset, D]."""
        tq = self._v_tq
        B, H = tq.v_packed.shape[0], tq.v_packed.shape[1]
        return tq._full_dequant(tq.v_packed, tq.v_norms, tq._v_q, tq._v_dim, B, H, tq.offset, dtype or tq._dtype)

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        # The decode kernels read float16 keys: bf16 / float32 keys are stored as float16 (exact for bf16
        # values inside the float16 range, which keys are); the reference keeps whatever dtype it is
        # given (v_only_cache.py:41-47), so `state` then differs in the dtype of its first entry.
        if self.fused and self._append_fused(keys, values):
            k_out = self._k_cache.keys[..., :self._k_cache.offset, :]
        else:
            k16 = keys if keys.dtype == torch.float16 else keys.to(torch.float16)
            k_out, _ = self._k_cache.update_and_fetch(k16, values)
            if self.fused:
                self._encode_only(keys, values)
        if self.fused:
            B, H, _, v_dim = values.shape
            key = (values.dtype, values.device)
            if self._zero is None or self._zero_key != key:          # one element, made once
                self._zero, self._zero_key = torch.zeros((1, 1, 1, 1), dtype=values.dtype, device=values.device), key
            return k_out, self._zero.expand(B, H, self._v_tq.offset, v_dim)
        if self._no_v_buffer:                                    # v_only_cache.py:54-75
            tq = self._v_tq
            B, H, S, v_dim = values.shape
            tq._dtype = keys.dtype
            tq._ensure_quantizer(keys.shape[-1], v_dim, values.device)
            tq._ensure_storage(B, H, S, values.device)
            prev = tq.offset
            tq._encode(values, tq._v_q, tq.v_packed, tq.v_norms, B, H, S, v_dim, prev)
            tq.offset += S
            v_out = tq._full_dequant(tq.v_packed, tq.v_norms, tq._v_q, v_dim, B, H, tq.offset, values.dtype)
        else:
            _, v_out = self._v_tq.update_and_fetch(keys, values)
        return k_out, v_out

    @property
    def offset(self):
        return self._k_cache.offset

    @property
    def state(self):
        k_state = list(self._k_cache.state) if self._k_cache.state else []
        v_state = list(self._v_tq.state) if self._v_tq.state else []
        return k_state + v_state

    @property
    def meta_state(self):
        return f"VOnlyTQ,{self._v_bits},{self._v_tq.seed},{self._v_tq.meta_state}"

    @classmethod
    def from_state(cls, state, meta_state, v_signs=None, sign_stream: str = "native"):
        """v_only_cache.py:95-111.  The serialised cache carries its seed, not its sign vector: pass the
        v_signs the cache was written with when they were given explicitly (or come from the reference,
        whose seed-to-signs generator is MLX's), or sign_stream="mlx" to expand a reference-written cache's
        seed by the restated MLX stream."""
        parts = meta_state.split(",", 3)
        bits = int(parts[1])
        seed = int(parts[2])
        obj = cls(bits=bits, seed=seed, v_signs=v_signs, sign_stream=sign_stream)
        if len(state) >= 2:
            obj._k_cache.keys = state[0]
            obj._k_cache.values = state[1]
            obj._k_cache.offset = state[0].shape[2]
        if len(state) > 2:
            tq = obj._v_tq
            tq.state = state[2:]
            tq.meta_state = parts[3]
            tq._v_pdim = tq.v_packed.shape[-1]
            if tq._v_dim is not None:                     # usable at once (attention straight off the restored cache),
                tq._ensure_quantizer(tq._v_dim, tq._v_dim, tq.v_packed.device)   # not only after the next insert
        return obj

    @classmethod
    def from_kvcache(cls, kv, bits: int = 3, seed: int = 42, **kwargs):
        """Construct empty, then insert the valid prefix of an uncompressed cache (see
        TurboQuantKVCache.from_kvcache)."""
        obj = cls(bits=bits, seed=seed, **kwargs)
        if kv.keys is not None and kv.offset > 0:
            obj.update_and_fetch(kv.keys[..., :kv.offset, :], kv.values[..., :kv.offset, :])
        return obj

    def make_mask(self, *args, **kwargs):
        return self._k_cache.make_mask(*args, **kwargs)

    def empty(self):
        return self._k_cache.offset == 0

    def is_trimmable(self):
        return True

    def trim(self, n):
        self._k_cache.trim(n)
        return self._v_tq.trim(n)

    def size(self):
        return self._k_cache.offset

    @property
    def nbytes(self):
        ks = self._k_cache
        k_bytes = 0 if ks.keys is None else ks.keys[..., :ks.offset, :].numel() * ks.keys.element_size()
        return k_bytes + self._v_tq.nbytes
