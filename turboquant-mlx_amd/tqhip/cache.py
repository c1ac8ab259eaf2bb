"""TurboQuantKVCache: the reference's cache object (turboquant_mlx/cache.py:42-369) over the
HIP codec.  Storage layout, growth rule, fetch modes, serialisation strings and quirks follow
the reference member by member; new vectors are encoded by the GPU straight into the packed
storage (no staging copy) and prefill dequantises straight into the fp16 buffer.
"""
from __future__ import annotations

import torch

from . import ops
from .kvcache import make_mask_for
from .quantizer import gaussian_boundaries, gaussian_codebook
from .rotation import random_diagonal_sign


def _checked_signs(signs, dim, device) -> torch.Tensor:
    """A caller's sign vector as the kernels take it: float32 [dim] of +-1 on `device`."""
    t = torch.as_tensor(signs)
    if t.dim() != 1 or t.numel() != dim:
        raise ValueError(f"a sign vector must have shape ({dim},), got {tuple(t.shape)}")
    t = t.detach().to(device=device, dtype=torch.float32).contiguous()
    if not bool((t.abs() == 1.0).all()):
        raise ValueError("a sign vector holds +1 and -1 only")
    return t


def _check_sign_stream(sign_stream):
    if sign_stream not in ("native", "mlx"):
        raise ValueError(f"sign_stream must be 'native' or 'mlx', got {sign_stream!r}")


class _Quantizer:
    """cache.py:33-39: signs (device) + codebook tables (host).  `signs` overrides the vector that
    random_diagonal_sign derives from `seed` (whose generator is this package's own, not MLX's): the way to
    read a cache written by the reference, which stores only the seed (cache.py:286)."""

    def __init__(self, dim, bits, seed, device, signs=None, sign_stream="native"):
        self.dim = dim
        self.bits = bits
        self.signs = (random_diagonal_sign(dim, seed=seed, device=device, stream=sign_stream) if signs is None
                      else _checked_signs(signs, dim, device))
        self.centroids = gaussian_codebook(bits)
        self.boundaries = gaussian_boundaries(self.centroids)


def _round_up(n, step):
    return ((n + step - 1) // step) * step


def _group_stride(t: torch.Tensor, inner: int) -> int:
    """Rows between consecutive (b, h) groups of a [B, H, T, inner] (or [B, H, T] with inner=1)
    tensor whose rows are dense and whose batch stride is H head strides -- true for the cache's
    own allocations and for time-slices of them."""
    if inner == 1 and t.dim() == 3:
        ok = t.stride(2) == 1 and t.stride(0) == t.shape[1] * t.stride(1)
        gs = t.stride(1)
    else:
        ok = (t.stride(3) == 1 and t.stride(2) == inner and t.stride(1) % inner == 0
              and t.stride(0) == t.shape[1] * t.stride(1))
        gs = t.stride(1) // inner
    if not ok:
        raise ValueError("cache storage must be row-contiguous [B, H, T, *]; call .contiguous() first")
    return gs


class TurboQuantKVCache:
    """PolarQuant KV cache with packed uint32 indices + float32 norms (cache.py:42-51).

    update_and_fetch returns, like the reference:
      fused=True   zero placeholders (attention reads the packed storage directly);
      v_only=True  (zero K placeholder, dequantised V);
      default      dequantised (K, V) from an incrementally maintained fp16 buffer.
    """

    step = 256                                               # cache.py:52

    _DTYPE_MAP = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}
    _DTYPE_NAME = {v: k for k, v in _DTYPE_MAP.items()}

    def __init__(self, bits: int = 3, seed: int = 42, fused: bool = False,
                 sparse_v_threshold: float | None = None, v_only: bool = False,
                 encode_variant: str = "mlx", k_signs=None, v_signs=None, sign_stream: str = "native"):
        """k_signs / v_signs ([dim] of +-1, any tensor-like): the rotation's sign vectors, used instead of the ones
        derived from `seed` / `seed + 1` (cache.py:92,96).  sign_stream: which generator derives them when they
        are not given -- "native" (this package's) or "mlx" (the restated stream of rotation.py:47-49, for a
        cache the reference wrote with that seed).  Everything else as the reference (cache.py:54-61)."""
        _check_sign_stream(sign_stream)
        self.quant_bits = bits
        self.seed = seed
        self.offset = 0
        self.fused = fused
        self.sparse_v_threshold = sparse_v_threshold
        self.v_only = v_only
        # "mlx": packed bits equal to the pure-array quantiser (quantizer.py:85-106 + packing.py);
        # "metal": equal to the Metal encoder the reference cache calls (cache.py:140 -> metal.py:147).
        # The two differ only for values within an ulp of a decision boundary.
        self.encode_variant = encode_variant
        self._reset_fields()
        self._k_signs_given, self._v_signs_given = k_signs, v_signs
        self.sign_stream = sign_stream

    def _reset_fields(self):
        self.k_packed = None
        self.k_norms = None
        self.v_packed = None
        self.v_norms = None
        self._k_deq_buf = None
        self._v_deq_buf = None
        self._deq_offset = 0
        self._deq_alloc = 0
        self._k_q = None
        self._v_q = None
        self._k_dim = None
        self._v_dim = None
        self._k_pdim = None
        self._v_pdim = None
        self._dtype = None
        self._step, self._step_key = None, None
        self._k_signs_given, self._v_signs_given = None, None
        self.sign_stream = "native"

    # ---------------------------------------------------------------- setup (cache.py:90-123)
    def _device(self):
        for t in (self.v_packed, self.k_packed):
            if t is not None:
                return t.device
        return torch.device("cuda")

    def _ensure_quantizer(self, k_dim, v_dim, device=None):
        device = device if device is not None else self._device()
        if not self.v_only and self._k_q is None:
            self._k_q = _Quantizer(k_dim, self.quant_bits, self.seed, device, self._k_signs_given, self.sign_stream)
            self._k_dim = k_dim
            self._k_pdim = ops.packed_dim(k_dim, self.quant_bits)
        if self._v_q is None:
            self._v_q = _Quantizer(v_dim, self.quant_bits, self.seed + 1, device, self._v_signs_given, self.sign_stream)
            self._v_dim = v_dim
            self._v_pdim = ops.packed_dim(v_dim, self.quant_bits)

    def _grow(self, old_p, old_n, B, H, n, pdim, prev, device):
        new_p = torch.zeros((B, H, n, pdim), dtype=torch.uint32, device=device)
        new_n = torch.zeros((B, H, n), dtype=torch.float32, device=device)
        if old_p is not None and prev > 0:
            new_p[..., :prev, :] = old_p[..., :prev, :]
            new_n[..., :prev] = old_n[..., :prev]
        return new_p, new_n

    def _ensure_storage(self, B, H, num_new, device):
        prev = self.offset
        needed = prev + num_new
        if self.v_packed is None or needed > self.v_packed.shape[2]:
            self._reallocate(B, H, _round_up(needed, self.step), device)

    def _reallocate(self, B, H, n, device):
        """Fresh contiguous storage of n positions per (b, h) holding the first `offset` positions."""
        prev = self.offset
        if not self.v_only:
            self.k_packed, self.k_norms = self._grow(self.k_packed, self.k_norms, B, H, n,
                                                     self._k_pdim, prev, device)
        self.v_packed, self.v_norms = self._grow(self.v_packed, self.v_norms, B, H, n,
                                                 self._v_pdim, prev, device)

    # ---------------------------------------------------------------- codec calls
    def _encode(self, x, q, packed, norms, B, H, S, dim, prev):
        ops.encode_into(x.reshape(-1, dim), q.signs, q.boundaries, packed, norms,
                        n_groups=B * H, rows_per_group=S,
                        packed_group_stride=_group_stride(packed, packed.shape[3]),
                        norms_group_stride=_group_stride(norms, 1), dim=dim, bits=self.quant_bits,
                        variant=self.encode_variant, packed_row_offset=prev, norms_row_offset=prev)

    def _dequant_range(self, packed, norms, q, dim, buf, B, H, start, count):
        """Dequantise positions [start, start+count) of every (b, h) into buf[..., start:start+count, :]."""
        ops.dequant_into(packed, norms, q.centroids, q.signs, buf, n_groups=B * H, rows_per_group=count,
                         packed_group_stride=_group_stride(packed, packed.shape[3]),
                         norms_group_stride=_group_stride(norms, 1), out_group_stride=buf.shape[2], dim=dim, bits=self.quant_bits,
                         packed_row_offset=start, norms_row_offset=start, out_row_offset=start)

    def _full_dequant(self, packed, norms, q, dim, B, H, total, dtype):
        """cache.py:125-129: every stored position, as a fresh [B, H, total, dim] tensor."""
        out = torch.empty((B, H, total, dim), dtype=dtype, device=packed.device)
        ops.dequant_into(packed, norms, q.centroids, q.signs, out, n_groups=B * H, rows_per_group=total,
                         packed_group_stride=_group_stride(packed, packed.shape[3]),
                         norms_group_stride=_group_stride(norms, 1),
                         out_group_stride=total, dim=dim, bits=self.quant_bits)
        return out

    def _incremental(self, packed, norms, q, dim, buf, B, H, prev, total, dtype):
        """Decode step of cache.py:171-180 / 192-207: dequantise only the new rows, in half
        precision (dequant_fp16), cast to the cache dtype, into the persistent buffer."""
        if total > self._deq_alloc_for(buf):
            na = _round_up(total, self.step)
            grown = torch.zeros((B, H, na, dim), dtype=dtype, device=buf.device)
            grown[..., :self._deq_offset, :] = buf[..., :self._deq_offset, :]
            buf = grown
        if dtype == torch.float16:
            self._dequant_range(packed, norms, q, dim, buf, B, H, prev, total - prev)
        else:
            tmp = torch.empty((B, H, total - prev, dim), dtype=torch.float16, device=buf.device)
            ops.dequant_into(packed, norms, q.centroids, q.signs, tmp, n_groups=B * H,
                             rows_per_group=total - prev,
                             packed_group_stride=_group_stride(packed, packed.shape[3]),
                             norms_group_stride=_group_stride(norms, 1), out_group_stride=total - prev, dim=dim,
                             bits=self.quant_bits, packed_row_offset=prev, norms_row_offset=prev)
            buf[..., prev:total, :] = tmp.to(dtype)
        return buf

    @staticmethod
    def _deq_alloc_for(buf):
        return buf.shape[2]

    def _prefill_buffer(self, packed, norms, q, dim, B, H, total, dtype):
        """cache.py:182-188 / 208-218: full dequant into a fresh step-rounded buffer."""
        alloc = _round_up(total, self.step)
        buf = torch.zeros((B, H, alloc, dim), dtype=dtype, device=packed.device)
        self._dequant_range(packed, norms, q, dim, buf, B, H, 0, total)
        return buf, alloc

    # ---------------------------------------------------------------- cache.py:131-218
    def _zero_like(self, t: torch.Tensor) -> torch.Tensor:
        """A zero scalar of t's dtype on t's device, made once: the source of the stride-0 placeholders
        (a fresh one per step would cost a fill launch each)."""
        key = (t.dtype, t.device)
        z = self.__dict__.setdefault("_zero_scalars", {}).get(key)
        if z is None:
            z = self._zero_scalars[key] = t.new_zeros(())
        return z

    def reserve(self, B: int, H: int, n_positions: int, dim: int, device="cuda"):
        """Allocate storage for `n_positions` more positions now, so that steps recorded in a HIP graph keep
        their addresses for that long (storage otherwise grows in steps of 256, which reallocates)."""
        device = torch.device(device)
        self._ensure_quantizer(dim, dim, device)
        self._ensure_storage(B, H, n_positions, device)

    def decode_step(self, queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, attn_scale: float,
                    position: torch.Tensor | None = None, out: torch.Tensor | None = None):
        """Encode one token and attend in one library call: the result of `update_and_fetch(keys, values)`
        followed by `turboquant_attention(queries, self, attn_scale, fused=True)` (no mask, no threshold) on
        a cache with packed keys and values.  queries (B, n_heads, 1, dim), keys / values (B, n_kv, 1, dim)
        -> (B, n_heads, 1, dim) in queries.dtype.  Not in the reference, where the two halves are separate
        calls of the model's attention layer (cache.py:131-165, fused_attention.py:20-125).

        With `position` (one-element int64 GPU tensor holding the cache's current offset) the kernels read the
        insert position and the attended length from it when they run, so the step can be recorded in a HIP
        graph once and replayed while the caller advances the tensor; set `offset` afterwards.  `out`
        (B, n_heads, dim) receives the result when given."""
        from . import attention
        B, n_q, S_q, dim = queries.shape
        H = values.shape[1]
        ok = (not self.v_only and S_q == 1 and values.shape[2] == 1 and keys.shape == values.shape
              and keys.shape[3] == dim and n_q % H == 0 and values.is_cuda
              and queries.dtype in ops._DTYPES and keys.dtype in ops._DTYPES and values.dtype in ops._DTYPES
              and ops.vonly_sparse_supported(dim, self.quant_bits, n_q // H))
        if ok:
            self._dtype = keys.dtype
            self._ensure_quantizer(dim, dim, values.device)
            self._ensure_storage(B, H, 1, values.device)
            key = (self.k_packed.data_ptr(), self.k_norms.data_ptr(), self.v_packed.data_ptr(),
                   self.v_norms.data_ptr(), self.v_packed.shape[2], n_q)
            if self._step_key != key:
                try:
                    self._step = ops.PackedStep(self.k_packed, self.k_norms, self.v_packed, self.v_norms,
                                                self._k_q.signs, self._v_q.signs, self._v_q.boundaries,
                                                self._v_q.centroids, dim=dim, n_rep=n_q // H, bits=self.quant_bits,
                                                variant=self.encode_variant)
                    self._step_key = key
                except ValueError:                 # storage handed in through `state` as slices
                    ok = False
        if not ok:
            if position is not None:
                raise ValueError("a step with a device-side position needs one new token, dim 128, "
                                 "n_rep <= 16 and contiguous storage")
            self.update_and_fetch(keys, values)
            return attention.turboquant_attention(queries, self, attn_scale, fused=True)
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
                                self.offset if position is None else position, attn_scale, res, packed=True)
        self.offset += 1          # _deq_offset stays behind: the next unfused fetch dequantises the whole cache
        return res if res.dim() == 4 else res[:, :, None, :]

    def update_and_fetch(self, keys: torch.Tensor, values: torch.Tensor):
        B, H, S, k_dim = keys.shape
        v_dim = values.shape[3]
        device = values.device
        self._dtype = keys.dtype
        self._ensure_quantizer(k_dim, v_dim, device)
        self._ensure_storage(B, H, S, device)
        prev = self.offset

        self._encode(values, self._v_q, self.v_packed, self.v_norms, B, H, S, v_dim, prev)
        if not self.v_only:
            self._encode(keys, self._k_q, self.k_packed, self.k_norms, B, H, S, k_dim, prev)

        self.offset += S
        total = self.offset

        if self.fused:
            # zero placeholders of the right shape that own no memory (stride-0 views)
            return (self._zero_like(keys).expand(B, H, total, k_dim),
                    self._zero_like(values).expand(B, H, total, v_dim))

        incremental = S <= 4 and self._v_deq_buf is not None and self._deq_offset == prev

        if self.v_only:
            if incremental:
                self._v_deq_buf = self._incremental(self.v_packed, self.v_norms, self._v_q, v_dim,
                                                    self._v_deq_buf, B, H, prev, total, values.dtype)
                self._deq_alloc = self._v_deq_buf.shape[2]
            else:
                self._v_deq_buf, self._deq_alloc = self._prefill_buffer(
                    self.v_packed, self.v_norms, self._v_q, v_dim, B, H, total, values.dtype)
            self._deq_offset = total
            return self._zero_like(keys).expand(B, H, total, k_dim), self._v_deq_buf[..., :total, :]

        if incremental:
            self._k_deq_buf = self._incremental(self.k_packed, self.k_norms, self._k_q, k_dim,
                                                self._k_deq_buf, B, H, prev, total, keys.dtype)
            self._v_deq_buf = self._incremental(self.v_packed, self.v_norms, self._v_q, v_dim,
                                                self._v_deq_buf, B, H, prev, total, values.dtype)
            self._deq_alloc = self._v_deq_buf.shape[2]
        else:
            self._k_deq_buf, _ = self._prefill_buffer(self.k_packed, self.k_norms, self._k_q, k_dim,
                                                      B, H, total, keys.dtype)
            self._v_deq_buf, self._deq_alloc = self._prefill_buffer(
                self.v_packed, self.v_norms, self._v_q, v_dim, B, H, total, values.dtype)
        self._deq_offset = total
        return self._k_deq_buf[..., :total, :], self._v_deq_buf[..., :total, :]

    # ---------------------------------------------------------------- cache.py:220-247
    def empty(self):
        return self.v_packed is None if self.v_only else self.k_packed is None

    @property
    def nbytes(self):
        total = 0
        if self.k_packed is not None:
            B, H = self.k_packed.shape[:2]
            total += B * H * self.offset * (self.k_packed.shape[3] * 4 + 4)
        if self.v_packed is not None:
            B, H = self.v_packed.shape[:2]
            total += B * H * self.offset * (self.v_packed.shape[3] * 4 + 4)
        return total

    @property
    def compression_ratio(self) -> float:
        """FP16 bytes of the uncompressed K+V divided by packed + norm bytes (cache.py:234-247)."""
        total = self.nbytes
        if total == 0:
            return 1.0
        ref = self.v_packed if self.v_only else self.k_packed
        if ref is None:
            return 1.0
        B, H = ref.shape[0], ref.shape[1]
        fp16_bytes = B * H * self.offset * ((self._k_dim or 0) + (self._v_dim or 0)) * 2
        return fp16_bytes / total

    # ---------------------------------------------------------------- cache.py:249-297
    @property
    def state(self):
        if self.v_packed is None and self.k_packed is None:
            return []
        parts = []
        if self.k_packed is not None:
            parts += [self.k_packed[..., :self.offset, :], self.k_norms[..., :self.offset]]
        if self.v_packed is not None:
            parts += [self.v_packed[..., :self.offset, :], self.v_norms[..., :self.offset]]
        return parts

    @state.setter
    def state(self, v):
        if not v:
            return
        if len(v) == 4:
            self.k_packed, self.k_norms, self.v_packed, self.v_norms = v
            self.offset = self.k_packed.shape[2]
        elif len(v) == 2:
            self.v_packed, self.v_norms = v
            self.offset = self.v_packed.shape[2]
        else:
            raise ValueError(f"Expected 2 (v_only) or 4 arrays in state, got {len(v)}")

    @property
    def meta_state(self):
        dtype_str = self._DTYPE_NAME.get(self._dtype, "float16")
        return (f"{self.offset},{self.quant_bits},{self.seed},"
                f"{self._k_dim or 0},{self._v_dim or 0},{dtype_str}")

    @meta_state.setter
    def meta_state(self, v):
        parts = v.split(",")
        self.offset, self.quant_bits, self.seed = int(parts[0]), int(parts[1]), int(parts[2])
        self._k_dim = int(parts[3]) or None
        self._v_dim = int(parts[4]) or None
        self._dtype = self._DTYPE_MAP.get(parts[5], torch.float16) if len(parts) > 5 else torch.float16

    # ---------------------------------------------------------------- cache.py:299-334
    def is_trimmable(self):
        return True

    def trim(self, n):
        n = min(self.offset, n)
        self.offset -= n
        self._k_deq_buf = None
        self._v_deq_buf = None
        self._deq_offset = 0
        self._deq_alloc = 0
        return n

    def size(self):
        return self.offset

    def make_mask(self, N, return_array: bool = False, window_size=None):
        return make_mask_for(self.offset, N, return_array, window_size, self._device())

    # ---------------------------------------------------------------- cache.py:336-369
    @classmethod
    def from_state(cls, state, meta_state, k_signs=None, v_signs=None, sign_stream: str = "native"):
        """cache.py:336-369.  The serialised cache carries its seed, not its sign vectors (cache.py:286): a cache
        written with explicit signs -- or by the reference, whose seed-to-signs generator is MLX's -- restores
        correctly only with the same k_signs / v_signs given here, or, for a reference-written cache whose
        vectors were not kept, with sign_stream="mlx" (the seed is then expanded by the restated MLX stream)."""
        _check_sign_stream(sign_stream)
        obj = cls.__new__(cls)
        obj._reset_fields()
        obj._k_signs_given, obj._v_signs_given = k_signs, v_signs
        obj.sign_stream = sign_stream
        obj.fused = False
        obj.sparse_v_threshold = None
        obj.v_only = False
        obj.encode_variant = "mlx"
        obj.meta_state = meta_state
        obj.state = state
        if obj.k_packed is not None:
            obj._k_pdim = obj.k_packed.shape[-1]
        if obj.v_packed is not None:
            obj._v_pdim = obj.v_packed.shape[-1]
        if obj._k_dim is not None and obj._v_dim is not None:
            obj._ensure_quantizer(obj._k_dim, obj._v_dim)
        return obj

    # ---------------------------------------------------------------- from_kvcache
    @classmethod
    def from_kvcache(cls, kv, bits: int = 3, seed: int = 42, **kwargs):
        """Compress an existing uncompressed cache (anything with .keys/.values/.offset, layout
        [B, H, T, D]).  Defined as: construct an empty cache, then update_and_fetch with the valid
        prefix.  The reference tree has no such constructor; its README shows the name on the
        mixed-quant cache of its mlx-lm fork (README.md:41-46)."""
        obj = cls(bits=bits, seed=seed, **kwargs)
        if kv.keys is not None and kv.offset > 0:
            obj.update_and_fetch(kv.keys[..., :kv.offset, :], kv.values[..., :kv.offset, :])
        return obj
