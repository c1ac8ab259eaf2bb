"""Kernel wrappers: the reference's operator API on torch tensors.

Each function has the name, argument order and error behaviour of the reference
wrapper it stands in for (cited per function; paths relative to the reference's
turboquant_mlx/ package), takes `torch.Tensor` where the reference takes
`mx.array`, and launches the HIP kernel of libtqhip.so on torch's current stream.
Tensors must live on a GPU; there is no CPU implementation behind these calls.
"""
from __future__ import annotations

import ctypes as C
import math

import torch

from . import _lib
from ._lib import DecodeShape, TQ_BF16, TQ_F16, TQ_F32

VALS_PER_WORD = {1: 32, 2: 16, 3: 10, 4: 8}       # packing.py:16
BIT_MASK = {1: 0x1, 2: 0x3, 3: 0x7, 4: 0xF}       # packing.py:17

_DTYPES = {torch.float32: TQ_F32, torch.float16: TQ_F16, torch.bfloat16: TQ_BF16}
_TORCH_OF = {TQ_F32: torch.float32, TQ_F16: torch.float16, TQ_BF16: torch.bfloat16}


def packed_dim(dim: int, bits: int) -> int:
    """packing.py:20-23."""
    vpw = VALS_PER_WORD[bits]
    return (dim + vpw - 1) // vpw


# ------------------------------------------------------------------ helpers

def _need_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "tqhip kernels run on the GPU only: got a tensor on "
                f"{t.device}; there is no CPU fallback")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor):
    """Raw hipStream_t of torch's current stream on the tensor's device."""
    if _raw_stream is not None:                       # avoids building a torch.cuda.Stream object per call
        idx = t.device.index
        return C.c_void_p(_raw_stream(torch.cuda.current_device() if idx is None else idx))
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}; use float32, float16 or bfloat16") from None


def _host_table(x):
    """Small table (boundaries / centroids) as a ctypes float array.  Accepts tensors, lists."""
    if isinstance(x, torch.Tensor):
        key = (x.data_ptr(), x._version, x.numel())
        hit = _host_table.cache.get(key)
        if hit is None:
            hit = _lib.host_floats(x.detach().float().cpu().tolist())
            if len(_host_table.cache) > 256:
                _host_table.cache.clear()
            _host_table.cache[key] = hit
        return hit
    return _lib.host_floats(x)


_host_table.cache = {}


def _as_f32_dev(x, like: torch.Tensor) -> torch.Tensor:
    if isinstance(x, torch.Tensor) and x.dtype == torch.float32 and x.device == like.device and x.is_contiguous():
        return x
    if not isinstance(x, torch.Tensor):
        x = torch.tensor(list(x), dtype=torch.float32)
    return x.to(device=like.device, dtype=torch.float32).contiguous()


_workspaces = {}


def _workspace(device, stream_id: int, nbytes: int) -> torch.Tensor:
    """Per (device, stream) scratch buffer for tile partials, grown on demand."""
    key = (device, stream_id)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _u32(t: torch.Tensor) -> torch.Tensor:
    """View / convert an integer tensor of packed words as uint32."""
    if t.dtype == torch.uint32:
        return t
    if t.dtype == torch.int32:
        return t.view(torch.uint32)
    return (t.to(torch.int64) & 0xFFFFFFFF).to(torch.int32).view(torch.uint32)


def _rows_view(t: torch.Tensor, inner: int):
    """(head_stride_in_rows, ok) for a [H, T, inner] view whose rows are contiguous."""
    if t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != inner or t.stride(0) % inner:
        return None
    return t.stride(0) // inner


def _head_layout_3d(t: torch.Tensor, inner: int) -> tuple[torch.Tensor, int]:
    hs = _rows_view(t, inner)
    if hs is None:
        t = t.contiguous()
        hs = t.stride(0) // inner
    return t, hs


def _head_layout_2d(t: torch.Tensor) -> tuple[torch.Tensor, int]:
    if t.dim() != 2 or t.stride(1) != 1:
        t = t.contiguous()
    return t, t.stride(0)


# ------------------------------------------------------------------ packing (integer plumbing)

def pack_indices(indices: torch.Tensor, bits: int) -> torch.Tensor:
    """packing.py:26-56.  (..., dim) integer indices -> (..., packed_dim) uint32."""
    vpw = VALS_PER_WORD[bits]
    shape = indices.shape
    dim = shape[-1]
    pd = packed_dim(dim, bits)
    flat = indices.reshape(-1, dim).to(torch.int64)
    if dim % vpw:
        flat = torch.nn.functional.pad(flat, (0, pd * vpw - dim))
    flat = flat.reshape(-1, pd, vpw)
    shifts = torch.arange(vpw, device=flat.device, dtype=torch.int64) * bits
    words = (flat << shifts).sum(dim=-1)            # disjoint bit fields: sum == OR
    return words.to(torch.int32).view(torch.uint32).reshape(*shape[:-1], pd)


def unpack_indices(packed: torch.Tensor, bits: int, dim: int) -> torch.Tensor:
    """packing.py:59-87.  (..., packed_dim) uint32 -> (..., dim) uint8."""
    vpw = VALS_PER_WORD[bits]
    shape = packed.shape
    w = _u32(packed).contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(vpw, device=w.device, dtype=torch.int64) * bits
    vals = (w.unsqueeze(-1) >> shifts) & BIT_MASK[bits]
    vals = vals.reshape(*shape[:-1], shape[-1] * vpw)[..., :dim]
    return vals.to(torch.uint8)


# ------------------------------------------------------------------ encode / dequant

def encode_into(x: torch.Tensor, signs: torch.Tensor, boundaries, packed: torch.Tensor,
                norms: torch.Tensor, *, n_groups: int, rows_per_group: int,
                packed_group_stride: int, norms_group_stride: int, dim: int, bits: int,
                variant: str = "mlx", packed_row_offset: int = 0, norms_row_offset: int = 0) -> None:
    """Encode rows of `x` straight into caller-owned packed / norm storage (tq_encode)."""
    _need_gpu(x, signs, packed, norms)
    x = x.contiguous()
    pd = packed_dim(dim, bits)
    var = {"mlx": _lib.TQ_ENCODE_MLX, "metal": _lib.TQ_ENCODE_METAL}[variant]
    lib = _lib.load()
    _lib.check(lib.tq_encode(
        _ptr(x), _dt(x), _ptr(signs), _host_table(boundaries),
        C.c_void_p(packed.data_ptr() + packed_row_offset * pd * 4),
        C.c_void_p(norms.data_ptr() + norms_row_offset * 4),
        n_groups, rows_per_group, packed_group_stride, norms_group_stride,
        dim, bits, var, _stream(x)))


def vonly_append_into(keys: torch.Tensor, values: torch.Tensor, signs: torch.Tensor, boundaries,
                      k_f16: torch.Tensor, v_raw, v_packed: torch.Tensor, v_norms: torch.Tensor, *,
                      position, bits: int, variant: str = "mlx") -> None:
    """Insert the S new tokens `keys`, `values` [B, H, S, D] at time index `position` of a cache with
    float16 keys `k_f16` [B, H, T_alloc, D], optional unencoded values `v_raw` (same dtype as
    `values`, or None) and packed values `v_packed` [B, H, T_alloc, pdim] / `v_norms` [B, H, T_alloc]
    in one launch (tq_vonly_append).  Same result as the slice assignments + encode_into of
    VOnlyTurboQuantCache.update_and_fetch (v_only_cache.py:52-53)."""
    _need_gpu(keys, values, signs, k_f16, v_packed, v_norms)
    B, H, S, D = values.shape
    on_device = isinstance(position, torch.Tensor)
    if on_device:
        # tq_vonly_append_at: the position is read on the GPU when the kernel runs (one-element int64 tensor); all
        # four tensors must then hold the same number of positions, and rows past the storage are dropped
        if position.dtype != torch.int64 or position.numel() != 1 or not position.is_cuda:
            raise ValueError("a device-side position must be a one-element int64 tensor on the GPU")
        pos_dev, position = position, 0
        if len({k_f16.shape[2], v_packed.shape[2], v_norms.shape[2]} | ({v_raw.shape[2]} if v_raw is not None else set())) != 1:
            raise ValueError("a device-side position needs key, value, packed and norm storage of one length")
    if keys.shape != values.shape:
        raise ValueError(f"keys {tuple(keys.shape)} and values {tuple(values.shape)} must have one shape")
    if k_f16.dtype != torch.float16 or not k_f16.is_contiguous():
        raise ValueError("k_f16 must be a contiguous float16 tensor")
    for name, t in (("k_f16", k_f16), ("v_packed", v_packed), ("v_norms", v_norms)) + ((("v_raw", v_raw),) if v_raw is not None else ()):
        if tuple(t.shape[:2]) != (B, H) or t.shape[2] < position + S:
            raise ValueError(f"{name} {tuple(t.shape)} cannot hold positions {position}..{position + S} of {B} x {H} groups")
    if v_raw is not None and (v_raw.dtype != values.dtype or not v_raw.is_contiguous()):
        raise ValueError("v_raw must be contiguous and of the dtype of values")
    if (v_packed.dtype not in (torch.uint32, torch.int32) or v_norms.dtype != torch.float32
            or not v_packed.is_contiguous() or not v_norms.is_contiguous()):
        raise ValueError("v_packed must be contiguous uint32 and v_norms contiguous float32")
    signs = _as_f32_dev(signs, values)
    keys, values = keys.contiguous(), values.contiguous()
    pd = packed_dim(D, bits)
    var = {"mlx": _lib.TQ_ENCODE_MLX, "metal": _lib.TQ_ENCODE_METAL}[variant]
    lib = _lib.load()
    if on_device:
        _lib.check(lib.tq_vonly_append_at(
            _ptr(keys), _dt(keys), _ptr(values), _dt(values), _ptr(signs), _host_table(boundaries),
            _ptr(k_f16), _ptr(v_raw), _ptr(v_packed), _ptr(v_norms), B * H, S, k_f16.shape[2], D, bits, var,
            _ptr(pos_dev), _stream(values)))
        return
    _lib.check(lib.tq_vonly_append(
        _ptr(keys), _dt(keys), _ptr(values), _dt(values), _ptr(signs), _host_table(boundaries),
        C.c_void_p(k_f16.data_ptr() + position * D * 2),
        None if v_raw is None else C.c_void_p(v_raw.data_ptr() + position * D * v_raw.element_size()),
        C.c_void_p(v_packed.data_ptr() + position * pd * 4), C.c_void_p(v_norms.data_ptr() + position * 4),
        B * H, S, k_f16.shape[2], 0 if v_raw is None else v_raw.shape[2], v_packed.shape[2], v_norms.shape[2],
        D, bits, var, _stream(values)))


def fused_quantize(vectors: torch.Tensor, signs: torch.Tensor, boundaries, dim: int, bits: int,
                   variant: str = "mlx"):
    """metal.py:147-196.  (n_vecs, dim) fp16/bf16/fp32 -> packed (n_vecs, pdim) uint32, norms (n_vecs,) f32.

    variant="mlx" reproduces the bits of PolarQuantizer.quantize + pack_indices
    (quantizer.py:85-106); variant="metal" those of the Metal encoder (metal.py:66-77).
    """
    if bits not in VALS_PER_WORD:
        raise KeyError(bits)                                    # packing.py:22 via metal.py:177
    _need_gpu(vectors)
    n_vecs = vectors.shape[0]
    vectors = vectors.reshape(n_vecs, dim)
    signs = _as_f32_dev(signs, vectors)
    pd = packed_dim(dim, bits)
    packed = torch.empty((n_vecs, pd), dtype=torch.uint32, device=vectors.device)
    norms = torch.empty((n_vecs,), dtype=torch.float32, device=vectors.device)
    encode_into(vectors, signs, boundaries, packed, norms, n_groups=1, rows_per_group=n_vecs,
                packed_group_stride=0, norms_group_stride=0, dim=dim, bits=bits, variant=variant)
    return packed, norms


def dequant_into(packed: torch.Tensor, norms: torch.Tensor, centroids, signs: torch.Tensor,
                 out: torch.Tensor, *, n_groups: int, rows_per_group: int, packed_group_stride: int,
                 norms_group_stride: int, out_group_stride: int, dim: int, bits: int,
                 packed_row_offset: int = 0, norms_row_offset: int = 0, out_row_offset: int = 0) -> None:
    """Dequantise rows of caller-owned packed storage into caller-owned `out` (tq_dequant)."""
    _need_gpu(packed, norms, signs, out)
    pd = packed_dim(dim, bits)
    lib = _lib.load()
    _lib.check(lib.tq_dequant(
        C.c_void_p(packed.data_ptr() + packed_row_offset * pd * 4),
        C.c_void_p(norms.data_ptr() + norms_row_offset * 4),
        _host_table(centroids), _ptr(signs),
        C.c_void_p(out.data_ptr() + out_row_offset * dim * out.element_size()), _dt(out),
        n_groups, rows_per_group, packed_group_stride, norms_group_stride, out_group_stride,
        dim, bits, _stream(out)))


def _dequant(packed, norms, centroids, signs, dim, bits, dtype):
    _need_gpu(packed, norms)
    seq_len = norms.shape[0]
    packed = _u32(packed).reshape(seq_len, -1).contiguous()
    norms = norms.to(torch.float32).contiguous()
    signs = _as_f32_dev(signs, packed)
    out = torch.empty((seq_len, dim), dtype=dtype, device=packed.device)
    dequant_into(packed, norms, centroids, signs, out, n_groups=1, rows_per_group=seq_len,
                 packed_group_stride=0, norms_group_stride=0, out_group_stride=0, dim=dim, bits=bits)
    return out


def packed_dequantize(packed, norms, centroids, signs, dim: int, bits: int) -> torch.Tensor:
    """kernels.py:123-155.  (seq, pdim) uint32 + (seq,) -> (seq, dim) float32."""
    return _dequant(packed, norms, centroids, signs, dim, bits, torch.float32)


prerot_packed_dequantize = packed_dequantize      # metal_kernels_v4.py:27


def dequant_fp16(packed, norms, centroids, signs, dim: int, bits: int) -> torch.Tensor:
    """metal.py:199-232.  Same arithmetic, half-precision output."""
    return _dequant(packed, norms, centroids, signs, dim, bits, torch.float16)


# ------------------------------------------------------------------ scores

def prerotate_query(q: torch.Tensor, signs) -> torch.Tensor:
    """metal_kernels_v4.py:119-150.  (n_heads, dim) -> raw butterfly of signs*q, float32."""
    if q.dim() != 2:
        raise ValueError(f"prerotate_query expects (n_heads, dim), got {tuple(q.shape)}")
    _need_gpu(q)
    n_heads, dim = q.shape
    if q.dtype not in _DTYPES:
        q = q.float()
    q = q.contiguous()
    signs = _as_f32_dev(signs, q)
    out = torch.empty((n_heads, dim), dtype=torch.float32, device=q.device)
    _lib.check(_lib.load().tq_prerotate_query(_ptr(q), _dt(q), _ptr(signs), _ptr(out), n_heads, dim, _stream(q)))
    return out


def _check_gqa(n_q: int, n_kv: int, n_rep: int):
    if n_q != n_kv * n_rep:
        raise ValueError(f"n_q_heads ({n_q}) must equal n_kv_heads ({n_kv}) * n_rep ({n_rep})")


def _mma_flag(precision: str) -> int:
    if precision not in ("fp32", "fp16"):
        raise ValueError(f"precision must be 'fp32' or 'fp16', got {precision!r}")
    return 1 if precision == "fp16" else 0


def _mma_mode(precision) -> int:
    """allow_mma of the two reference-named wrappers: None = float32 fidelity on the fastest kernel
    (split operands on the matrix cores where the shape allows), "fp32" = the float32 vector kernels,
    "fp16" = fp16 operands."""
    if precision is None:
        return _lib.TQ_MMA_SPLIT
    return _lib.TQ_MMA_FP16 if _mma_flag(precision) else _lib.TQ_MMA_OFF


def prerot_fused_qk_scores(q_rot: torch.Tensor, k_packed: torch.Tensor, k_norms: torch.Tensor,
                           centroids, dim: int, bits: int, n_rep: int = 1,
                           precision=None) -> torch.Tensor:
    """metal_kernels_v4.py:153-221.  Scores of pre-rotated queries against packed K, GQA-aware.

    q_rot (n_q, dim); k_packed (n_kv, seq, pdim); k_norms (n_kv, seq) -> (n_q, seq) float32.
    precision=None (default): float32 fidelity -- at d = 128 and n_rep <= 16 on the matrix cores with
    every operand as an fp16 value plus the fp16 remainder of its rounding (products exact in float32,
    ~1e-6 relative; the reference's bar is 1e-4 absolute, tests/test_prerot.py:90-95), other shapes on
    the float32 vector kernels.  "fp32": the float32 vector kernels for every shape (the reference's
    operation order).  "fp16": q_rot and the centroids rounded to half on the matrix cores (~3e-4
    relative).
    """
    _need_gpu(q_rot, k_packed, k_norms)
    n_q = q_rot.shape[0]
    n_kv, seq_len = k_norms.shape
    _check_gqa(n_q, n_kv, n_rep)
    pd = packed_dim(dim, bits)
    q_rot = q_rot.to(torch.float32).contiguous()
    k_packed, phs = _head_layout_3d(_u32(k_packed), pd)
    k_norms, nhs = _head_layout_2d(k_norms.to(torch.float32))
    out = torch.empty((n_q, seq_len), dtype=torch.float32, device=q_rot.device)
    _lib.check(_lib.load().tq_prerot_qk_scores(
        _ptr(q_rot), _ptr(k_packed), _ptr(k_norms), _host_table(centroids), _ptr(out),
        n_kv, n_rep, seq_len, phs, nhs, dim, bits, _mma_mode(precision), _stream(q_rot)))
    return out


def packed_fused_qk_scores(query: torch.Tensor, k_packed: torch.Tensor, k_norms: torch.Tensor,
                           centroids, signs, dim: int, bits: int) -> torch.Tensor:
    """kernels.py:158-196.  One butterfly per K row, MHA only: (H, D), (H, S, pdim), (H, S) -> (H, S)."""
    _need_gpu(query, k_packed, k_norms)
    n_heads, seq_len = k_norms.shape
    pd = packed_dim(dim, bits)
    query = query.to(torch.float32).contiguous()
    k_packed, phs = _head_layout_3d(_u32(k_packed), pd)
    k_norms, nhs = _head_layout_2d(k_norms.to(torch.float32))
    signs = _as_f32_dev(signs, query)
    out = torch.empty((n_heads, seq_len), dtype=torch.float32, device=query.device)
    _lib.check(_lib.load().tq_packed_qk_scores(
        _ptr(query), _ptr(k_packed), _ptr(k_norms), _host_table(centroids), _ptr(signs), _ptr(out),
        n_heads, seq_len, phs, nhs, dim, bits, _stream(query)))
    return out


def dense_qk_scores(q: torch.Tensor, k: torch.Tensor, scale: float, n_rep: int = 1) -> torch.Tensor:
    """<q[h], K[h // n_rep, p]> * scale for fp16 keys: (n_q, D), (n_kv, T, D) fp16 -> (n_q, T) f32."""
    _need_gpu(q, k)
    n_q, dim = q.shape
    n_kv, seq_len, _ = k.shape
    _check_gqa(n_q, n_kv, n_rep)
    if k.dtype != torch.float16:
        raise ValueError(f"dense keys must be float16, got {k.dtype}")
    if q.dtype not in _DTYPES:
        q = q.float()
    q = q.contiguous()
    k, khs = _head_layout_3d(k, dim)
    out = torch.empty((n_q, seq_len), dtype=torch.float32, device=q.device)
    _lib.check(_lib.load().tq_dense_qk_scores(_ptr(q), _dt(q), _ptr(k), _ptr(out), n_kv, n_rep, seq_len,
                                               khs, dim, float(scale), _stream(q)))
    return out


def softmax_rows(scores: torch.Tensor, scale: float = 1.0, mask: torch.Tensor | None = None) -> torch.Tensor:
    """softmax(scores * scale + mask) along the last axis of a (rows, T) float32 tensor
    (fused_attention.py:78-94).  mask: (T,), (1, T) or (rows, T)."""
    _need_gpu(scores, mask)
    scores = scores.to(torch.float32).contiguous()
    n_rows, seq_len = scores.shape
    mrs = 0
    if mask is not None:
        mask = mask.to(torch.float32)
        if mask.dim() == 1:
            mask = mask.reshape(1, -1)
        if mask.shape[-1] != seq_len or mask.shape[0] not in (1, n_rows):
            raise ValueError(f"mask shape {tuple(mask.shape)} does not match scores {tuple(scores.shape)}")
        mask = mask.contiguous()
        mrs = seq_len if mask.shape[0] == n_rows and n_rows > 1 else 0
    out = torch.empty_like(scores)
    _lib.check(_lib.load().tq_softmax_rows(_ptr(scores), _ptr(mask), mrs, _ptr(out), n_rows, seq_len,
                                            float(scale), _stream(scores)))
    return out


# ------------------------------------------------------------------ sparse V

def sparse_v_matvec(weights: torch.Tensor, v_packed: torch.Tensor, v_norms: torch.Tensor, centroids,
                    signs, dim: int, bits: int, threshold: float = 1e-5, n_rep: int = 1,
                    precision=None) -> torch.Tensor:
    """sparse_v.py:94-186.  Weighted sum of dequantised V rows with the butterfly pulled out of
    the position loop; positions with weight < threshold are skipped; threshold <= 0 is dense.

    weights (n_q, seq); v_packed (n_kv, seq, pdim); v_norms (n_kv, seq) -> (n_q, dim) float32.
    precision as in prerot_fused_qk_scores (None: weights * norm and centroids as value + remainder on
    the matrix cores, within the reference's 1e-5 of the largest output, tests/test_sparse_v.py:70-75;
    "fp16": both rounded to half).
    """
    if dim & (dim - 1):
        raise ValueError(f"dim must be a power of 2, got {dim}")
    if dim > 256:
        raise ValueError(f"dim > 256 not supported by threadgroup layout, got {dim}")
    _need_gpu(weights, v_packed, v_norms)
    n_q, seq_len = weights.shape
    n_kv = v_packed.shape[0]
    _check_gqa(n_q, n_kv, n_rep)
    pd = packed_dim(dim, bits)
    weights = weights.to(torch.float32).contiguous()
    v_packed, phs = _head_layout_3d(_u32(v_packed), pd)
    v_norms, nhs = _head_layout_2d(v_norms.to(torch.float32))
    signs = _as_f32_dev(signs, weights)
    out = torch.empty((n_q, dim), dtype=torch.float32, device=weights.device)
    lib = _lib.load()
    need = lib.tq_workspace_bytes(_lib.TQ_OP_SPARSE_V, 1, n_q, seq_len, dim)
    stream = _stream(weights)
    ws = _workspace(weights.device, stream.value or 0, need)
    _lib.check(lib.tq_sparse_v_matvec(
        _ptr(weights), _ptr(v_packed), _ptr(v_norms), _host_table(centroids), _ptr(signs), _ptr(out),
        _ptr(ws), ws.numel(), n_kv, n_rep, seq_len, phs, nhs, dim, bits, float(max(threshold, 0.0)),
        _mma_mode(precision), stream))
    return out


def count_active_positions(weights: torch.Tensor, threshold: float = 1e-5) -> int:
    """sparse_v.py:189-191 (diagnostics only)."""
    return int((weights > threshold).sum().item())


# ------------------------------------------------------------------ fused decode attention

def _decode_shape(*, n_seq, n_kv, n_rep, dim, bits, block_size, seq_len, seq_offsets, k_strides, kn_strides,
                  v_strides, vn_strides, mask, mask_strides, attn_scale, out_dtype,
                  allow_mma: bool = True) -> DecodeShape:
    sh = DecodeShape()
    sh.n_seq, sh.n_kv_heads, sh.n_rep, sh.dim, sh.bits, sh.block_size = n_seq, n_kv, n_rep, dim, bits, block_size
    sh.seq_len = seq_len
    sh.seq_offsets = seq_offsets.data_ptr() if seq_offsets is not None else None
    sh.k_seq_stride, sh.k_head_stride = k_strides
    sh.kn_seq_stride, sh.kn_head_stride = kn_strides
    sh.v_seq_stride, sh.v_head_stride = v_strides
    sh.vn_seq_stride, sh.vn_head_stride = vn_strides
    sh.mask = mask.data_ptr() if mask is not None else None
    sh.mask_seq_stride, sh.mask_head_stride = mask_strides
    sh.attn_scale = float(attn_scale)
    sh.out_dtype = _DTYPES[out_dtype]
    sh.allow_mma = 1 if allow_mma else 0
    return sh


def _check_rows(T: int, ragged: bool, n_seq: int, **tensors):
    """The kernels trust the attended length: refuse one that exceeds what the tensors hold (cache layout: rows
    per (sequence, head); ragged batch: the rows of all sequences together) before anything is launched."""
    for name, t in tensors.items():
        rows = t.shape[-2] if name in ("k", "k_packed", "v_packed") else t.shape[-1]
        if T > rows:
            raise ValueError(f"attended length {T} exceeds the {rows} rows of {name}")
        if not ragged and t.dim() >= 3 + (name in ("k", "k_packed", "v_packed")) and t.shape[0] != n_seq:
            raise ValueError(f"{name} holds {t.shape[0]} sequences, the query {n_seq}")


def _check_offsets(seq_offsets: torch.Tensor, n_seq: int, validate: bool, **tensors) -> None:
    """The kernels read seq_offsets as n_seq + 1 int32 values and trust them: sequence s occupies rows
    seq_offsets[s] .. seq_offsets[s + 1] - 1 of the ragged tensors.  Dtype, count and layout are checked here
    (an int64 tensor, torch.cumsum's default, would be read as int32 pairs: zero or negative lengths and
    silently wrong outputs).  That the offsets start at >= 0, never decrease and end inside the tensors is the
    caller's contract; validate=True checks it too, at the price of one device-to-host synchronisation."""
    if (seq_offsets.dtype != torch.int32 or seq_offsets.dim() != 1 or seq_offsets.numel() != n_seq + 1
            or not seq_offsets.is_contiguous()):
        raise ValueError(f"seq_offsets must be a contiguous int32 tensor with n_seq + 1 = {n_seq + 1} entries, got "
                         f"{seq_offsets.dtype} {tuple(seq_offsets.shape)}")
    if validate:
        off = seq_offsets.cpu().tolist()
        if off[0] < 0 or any(b < a for a, b in zip(off, off[1:])):
            raise ValueError("seq_offsets must start at >= 0 and never decrease")
        for name, t in tensors.items():
            rows = t.shape[-2] if name in ("k", "k_packed", "v_packed") else t.shape[-1]
            if off[-1] > rows:
                raise ValueError(f"seq_offsets end at row {off[-1]}, {name} holds {rows}")


def _kv_layout(t: torch.Tensor, inner: int, ragged: bool):
    """Strides in rows for KV addressing.  Accepts [H, T, inner] (one sequence or ragged batch) or
    [B, H, T, inner] (cache layout); the last two axes must be row-contiguous."""
    if t.dim() == 3:
        t, hs = _head_layout_3d(t, inner)
        return t, (0, hs)
    if t.dim() != 4:
        raise ValueError(f"expected a 3-D or 4-D KV tensor, got shape {tuple(t.shape)}")
    if t.stride(3) != 1 or t.stride(2) != inner or t.stride(1) % inner or t.stride(0) % inner:
        t = t.contiguous()
    return t, (t.stride(0) // inner, t.stride(1) // inner)


def _norm_layout(t: torch.Tensor):
    if t.dim() == 2:
        t, hs = _head_layout_2d(t)
        return t, (0, hs)
    if t.dim() != 3:
        raise ValueError(f"expected a 2-D or 3-D norm tensor, got shape {tuple(t.shape)}")
    if t.stride(2) != 1:
        t = t.contiguous()
    return t, (t.stride(0), t.stride(1))


def _mask_layout(mask, n_seq: int, n_q: int, seq_len: int, device):
    """Additive float mask broadcastable to (n_seq, n_q, seq_len) -> (tensor, (seq_stride, head_stride))."""
    if mask is None:
        return None, (0, 0)
    m = mask.to(device=device, dtype=torch.float32)
    while m.dim() < 3:
        m = m.unsqueeze(0)
    if m.shape[-1] != seq_len or m.shape[0] not in (1, n_seq) or m.shape[1] not in (1, n_q):
        raise ValueError(f"mask shape {tuple(mask.shape)} not broadcastable to ({n_seq}, {n_q}, {seq_len})")
    m = m.contiguous()
    ss = m.shape[1] * seq_len if m.shape[0] == n_seq and n_seq > 1 else 0
    hs = seq_len if m.shape[1] == n_q and n_q > 1 else 0
    return m, (ss, hs)


def flash_decode(q_rot: torch.Tensor, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids,
                 v_signs, dim: int, bits: int, attn_scale: float, *, n_rep: int = 1, block_size: int = 16,
                 seq_len: int | None = None, seq_offsets: torch.Tensor | None = None,
                 max_seq_len: int | None = None, mask=None, out_dtype=torch.float32,
                 precision: str = "fp16", sparse_v_threshold: float = 0.0,
                 validate_offsets: bool = False) -> torch.Tensor:
    """Batched form of flash_attention_turboquant (tq_flash_decode).

    sparse_v_threshold > 0: softmax weights below it are dropped from the value sum (the threshold of
    sparse_v.py:59-65 on the final weights, as turboquant_attention applies it, fused_attention.py:109-121)
    -- tq_flash_sparse_decode, matrix-core shape only (see vonly_sparse_supported).

    precision="fp16" (default): matrix-core kernels where the shape allows (d = 128, any width,
    n_rep <= 16), operands rounded to half, float32 accumulation; "fp32": float32 kernels.

    q_rot (n_seq, n_q, dim) float32.  K/V either cache layout [n_seq, n_kv, T_alloc, *] with the
    uniform valid length `seq_len`, or ragged [n_kv, sum(L), *] with int32 `seq_offsets`
    (n_seq + 1 entries on the GPU, non-decreasing, ending inside the tensors: the caller's contract, checked
    only with validate_offsets=True, which synchronises once) and `max_seq_len`.  Returns (n_seq, n_q, dim)
    `out_dtype`.
    """
    _need_gpu(q_rot, k_packed, k_norms, v_packed, v_norms, seq_offsets)
    if dim > 128 or dim & (dim - 1):
        raise ValueError(f"dim must be a power of 2 and <= 128, got {dim}")
    if block_size < 1 or block_size > 32:
        raise ValueError(f"block_size must be in 1..32, got {block_size}")
    n_seq, n_q, _ = q_rot.shape
    ragged = seq_offsets is not None
    n_kv = k_norms.shape[-2]
    _check_gqa(n_q, n_kv, n_rep)
    pd = packed_dim(dim, bits)
    q_rot = q_rot.to(torch.float32).contiguous()
    k_packed, ks = _kv_layout(_u32(k_packed), pd, ragged)
    v_packed, vs = _kv_layout(_u32(v_packed), pd, ragged)
    k_norms, kns = _norm_layout(k_norms if k_norms.dtype == torch.float32 else k_norms.to(torch.float32))
    v_norms, vns = _norm_layout(v_norms if v_norms.dtype == torch.float32 else v_norms.to(torch.float32))
    if ragged:
        if max_seq_len is None:
            raise ValueError("max_seq_len is required with seq_offsets")
        _check_offsets(seq_offsets, n_seq, validate_offsets, k_packed=k_packed, k_norms=k_norms, v_packed=v_packed,
                       v_norms=v_norms)
        T = int(max_seq_len)
    else:
        T = int(seq_len if seq_len is not None else k_norms.shape[-1])
    _check_rows(T, ragged, n_seq, k_packed=k_packed, k_norms=k_norms, v_packed=v_packed, v_norms=v_norms)
    v_signs = _as_f32_dev(v_signs, q_rot)
    mask, ms = _mask_layout(mask, n_seq, n_q, T, q_rot.device)
    out = torch.empty((n_seq, n_q, dim), dtype=out_dtype, device=q_rot.device)
    sh = _decode_shape(n_seq=n_seq, n_kv=n_kv, n_rep=n_rep, dim=dim, bits=bits, block_size=block_size,
                       seq_len=T, seq_offsets=seq_offsets, k_strides=ks, kn_strides=kns, v_strides=vs,
                       vn_strides=vns, mask=mask, mask_strides=ms, attn_scale=attn_scale, out_dtype=out_dtype,
                       allow_mma=bool(_mma_flag(precision)))
    lib = _lib.load()
    stream = _stream(q_rot)
    if sparse_v_threshold and sparse_v_threshold > 0.0:
        if not (vonly_sparse_supported(dim, bits, n_rep) and T > 0):
            raise ValueError("thresholded flash decode needs dim 128, n_rep <= 16 and a non-empty cache; "
                             "compose prerot_fused_qk_scores, softmax_rows and sparse_v_matvec for other shapes")
        need = lib.tq_vonly_sparse_workspace_bytes(n_seq, n_q, T)
        ws = _workspace(q_rot.device, stream.value or 0, need)
        _lib.check(lib.tq_flash_sparse_decode(
            _ptr(q_rot), _ptr(k_packed), _ptr(k_norms), _ptr(v_packed), _ptr(v_norms),
            _host_table(k_centroids), _host_table(v_centroids), _ptr(v_signs), float(sparse_v_threshold), _ptr(out),
            _ptr(ws), ws.numel(), C.byref(sh), stream))
        return out
    need = lib.tq_workspace_bytes(_lib.TQ_OP_FLASH_DECODE, n_seq, n_q, T, dim)
    ws = _workspace(q_rot.device, stream.value or 0, need)
    _lib.check(lib.tq_flash_decode(
        _ptr(q_rot), _ptr(k_packed), _ptr(k_norms), _ptr(v_packed), _ptr(v_norms),
        _host_table(k_centroids), _host_table(v_centroids), _ptr(v_signs), _ptr(out),
        _ptr(ws), ws.numel(), C.byref(sh), stream))
    return out


def flash_decode_from_q(q: torch.Tensor, k_signs, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids,
                        v_signs, dim: int, bits: int, attn_scale: float, *, n_rep: int = 1,
                        seq_len: int | None = None, seq_offsets: torch.Tensor | None = None,
                        max_seq_len: int | None = None, mask=None, out_dtype=torch.float32,
                        sparse_v_threshold: float = 0.0, validate_offsets: bool = False) -> torch.Tensor:
    """The decode step of turboquant_attention (fused_attention.py:56-121) in ONE library call from the query
    itself: the pre-rotation of prerotate_query happens inside the attention kernels (tq_flash_decode_from_q).
    q (n_seq, n_q, dim) fp16 / bf16 / float32; other arguments as flash_decode.  Matrix-core shapes only
    (vonly_sparse_supported); callers fall back to prerotate_query + flash_decode otherwise."""
    _need_gpu(q, k_packed, k_norms, v_packed, v_norms, seq_offsets)
    n_seq, n_q, _ = q.shape
    ragged = seq_offsets is not None
    n_kv = k_norms.shape[-2]
    _check_gqa(n_q, n_kv, n_rep)
    if not vonly_sparse_supported(dim, bits, n_rep):
        raise ValueError("flash_decode_from_q needs dim 128 and n_rep <= 16; use prerotate_query + flash_decode")
    pd = packed_dim(dim, bits)
    if q.dtype not in _DTYPES:
        q = q.float()
    q = q.contiguous()
    k_packed, ks = _kv_layout(_u32(k_packed), pd, ragged)
    v_packed, vs = _kv_layout(_u32(v_packed), pd, ragged)
    k_norms, kns = _norm_layout(k_norms if k_norms.dtype == torch.float32 else k_norms.to(torch.float32))
    v_norms, vns = _norm_layout(v_norms if v_norms.dtype == torch.float32 else v_norms.to(torch.float32))
    if ragged:
        if max_seq_len is None:
            raise ValueError("max_seq_len is required with seq_offsets")
        _check_offsets(seq_offsets, n_seq, validate_offsets, k_packed=k_packed, k_norms=k_norms, v_packed=v_packed,
                       v_norms=v_norms)
        T = int(max_seq_len)
    else:
        T = int(seq_len if seq_len is not None else k_norms.shape[-1])
    if T <= 0:
        raise ValueError("flash_decode_from_q needs a non-empty cache")
    _check_rows(T, ragged, n_seq, k_packed=k_packed, k_norms=k_norms, v_packed=v_packed, v_norms=v_norms)
    k_signs = _as_f32_dev(k_signs, q)
    v_signs = _as_f32_dev(v_signs, q)
    mask, ms = _mask_layout(mask, n_seq, n_q, T, q.device)
    out = torch.empty((n_seq, n_q, dim), dtype=out_dtype, device=q.device)
    sh = _decode_shape(n_seq=n_seq, n_kv=n_kv, n_rep=n_rep, dim=dim, bits=bits, block_size=16,
                       seq_len=T, seq_offsets=seq_offsets, k_strides=ks, kn_strides=kns, v_strides=vs,
                       vn_strides=vns, mask=mask, mask_strides=ms, attn_scale=attn_scale, out_dtype=out_dtype,
                       allow_mma=True)
    lib = _lib.load()
    stream = _stream(q)
    thr = float(sparse_v_threshold) if sparse_v_threshold and sparse_v_threshold > 0.0 else 0.0
    need = (lib.tq_vonly_sparse_workspace_bytes(n_seq, n_q, T) if thr > 0.0
            else lib.tq_workspace_bytes(_lib.TQ_OP_FLASH_DECODE, n_seq, n_q, T, dim))
    ws = _workspace(q.device, stream.value or 0, need)
    _lib.check(lib.tq_flash_decode_from_q(
        _ptr(q), _dt(q), _ptr(k_signs), _ptr(k_packed), _ptr(k_norms), _ptr(v_packed), _ptr(v_norms),
        _host_table(k_centroids), _host_table(v_centroids), _ptr(v_signs), thr, _ptr(out),
        _ptr(ws), ws.numel(), C.byref(sh), stream))
    return out


def flash_attention_turboquant(q_rot, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids,
                               v_signs, dim: int, bits: int, attn_scale: float, block_size: int = 16,
                               n_rep: int = 1, precision: str = "fp16") -> torch.Tensor:
    """flash_attention.py:168-274.  One sequence: q_rot (n_q, dim); K/V (n_kv, seq, pdim) + (n_kv, seq)
    -> (n_q, dim) float32 = softmax(QK * scale) @ V over the packed cache."""
    out = flash_decode(q_rot.unsqueeze(0), k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids,
                       v_signs, dim, bits, attn_scale, n_rep=n_rep, block_size=block_size, precision=precision)
    return out[0]


def vonly_sparse_supported(dim: int, bits: int, n_rep: int) -> bool:
    """Shapes the one-call steps over PACKED keys cover (the matrix-core kernels: flash decode from the raw query,
    its thresholded form, the packed cache's decode_step): d = 128 at every width."""
    return dim == 128 and 1 <= bits <= 4 and 1 <= n_rep <= 16


def vonly_threshold_supported(dim: int, bits: int, n_rep: int) -> bool:
    """Shapes the thresholded one-call V-only decode step covers: fp16 keys, packed values of any width."""
    return dim == 128 and 1 <= bits <= 4 and 1 <= n_rep <= 16


def vonly_decode(q: torch.Tensor, k: torch.Tensor, v_packed, v_norms, v_centroids, v_signs, dim: int,
                 bits: int, attn_scale: float, *, n_rep: int = 1, seq_len: int | None = None,
                 seq_offsets: torch.Tensor | None = None, max_seq_len: int | None = None, mask=None,
                 out_dtype=torch.float32, precision: str = "fp16", sparse_v_threshold: float = 0.0,
                 out: torch.Tensor | None = None, static_scratch: bool = False,
                 validate_offsets: bool = False) -> torch.Tensor:
    """Dense-softmax decode attention over fp16 keys and packed values (tq_vonly_decode_attn).
    precision as in flash_decode (on the matrix-core path fp16 queries enter as they are, bf16 converted to
    fp16, float32 as an fp16 value plus the fp16 remainder of that rounding).

    sparse_v_threshold > 0: softmax weights below it are dropped from the value sum (threshold rule of
    sparse_v.py:59-65 on the final weights, as in hybrid_attention.py:52-88) -- tq_vonly_sparse_decode_attn,
    matrix-core shape only (see vonly_sparse_supported).

    out: a contiguous (n_seq, n_q, dim) tensor to write into (its dtype is the output dtype) instead of a new one.
    static_scratch=True takes tq_vonly_decode_attn_static: the per-tile partial sums go to an array inside the
    library instead of a torch workspace, so with `out` given and inputs already in the kernel's layout the call
    allocates no device memory (for callers under HIP-graph capture or in loops that must not allocate); shapes
    whose partial sums exceed that array raise, and calls that overlap on one GPU would race on it.

    q (n_seq, n_q, dim) fp16/bf16/fp32; k [n_seq, n_kv, T_alloc, dim] or ragged [n_kv, sum(L), dim] fp16;
    V as in flash_decode.  Returns (n_seq, n_q, dim) `out_dtype`.
    """
    _need_gpu(q, k, v_packed, v_norms, seq_offsets)
    if k.dtype != torch.float16:
        raise ValueError(f"dense keys must be float16, got {k.dtype}")
    n_seq, n_q, _ = q.shape
    ragged = seq_offsets is not None
    n_kv = v_norms.shape[-2]
    _check_gqa(n_q, n_kv, n_rep)
    pd = packed_dim(dim, bits)
    if q.dtype not in _DTYPES:
        q = q.float()
    q = q.contiguous()
    k, ks = _kv_layout(k, dim, ragged)
    v_packed, vs = _kv_layout(_u32(v_packed), pd, ragged)
    v_norms, vns = _norm_layout(v_norms if v_norms.dtype == torch.float32 else v_norms.to(torch.float32))
    if ragged:
        if max_seq_len is None:
            raise ValueError("max_seq_len is required with seq_offsets")
        _check_offsets(seq_offsets, n_seq, validate_offsets, k=k, v_packed=v_packed, v_norms=v_norms)
        T = int(max_seq_len)
    else:
        T = int(seq_len if seq_len is not None else v_norms.shape[-1])
    _check_rows(T, ragged, n_seq, k=k, v_packed=v_packed, v_norms=v_norms)
    v_signs = _as_f32_dev(v_signs, q)
    mask, ms = _mask_layout(mask, n_seq, n_q, T, q.device)
    if out is None:
        out = torch.empty((n_seq, n_q, dim), dtype=out_dtype, device=q.device)
    else:
        _need_gpu(out)
        if tuple(out.shape) != (n_seq, n_q, dim) or not out.is_contiguous() or out.dtype not in _DTYPES:
            raise ValueError(f"out must be a contiguous ({n_seq}, {n_q}, {dim}) float32/float16/bfloat16 tensor")
        out_dtype = out.dtype
    sh = _decode_shape(n_seq=n_seq, n_kv=n_kv, n_rep=n_rep, dim=dim, bits=bits, block_size=16, seq_len=T,
                       seq_offsets=seq_offsets, k_strides=ks, kn_strides=(0, 0), v_strides=vs, vn_strides=vns,
                       mask=mask, mask_strides=ms, attn_scale=attn_scale, out_dtype=out_dtype,
                       allow_mma=bool(_mma_flag(precision)))
    lib = _lib.load()
    stream = _stream(q)
    if static_scratch:
        if sparse_v_threshold and sparse_v_threshold > 0.0:
            raise ValueError("static_scratch serves the dense step only (sparse_v_threshold = 0)")
        _lib.check(lib.tq_vonly_decode_attn_static(
            _ptr(q), _dt(q), _ptr(k), _ptr(v_packed), _ptr(v_norms), _host_table(v_centroids), _ptr(v_signs),
            _ptr(out), C.byref(sh), stream))
        return out
    if sparse_v_threshold and sparse_v_threshold > 0.0:
        if not (vonly_threshold_supported(dim, bits, n_rep) and T > 0):
            raise ValueError("thresholded V-only decode needs dim 128, n_rep <= 16 and a non-empty cache; "
                             "compose dense_qk_scores, softmax_rows and sparse_v_matvec for other shapes")
        need = lib.tq_vonly_sparse_workspace_bytes(n_seq, n_q, T)
        ws = _workspace(q.device, stream.value or 0, need)
        _lib.check(lib.tq_vonly_sparse_decode_attn(
            _ptr(q), _dt(q), _ptr(k), _ptr(v_packed), _ptr(v_norms), _host_table(v_centroids), _ptr(v_signs),
            float(sparse_v_threshold), _ptr(out), _ptr(ws), ws.numel(), C.byref(sh), stream))
        return out
    need = lib.tq_workspace_bytes(_lib.TQ_OP_VONLY_DECODE, n_seq, n_q, T, dim)
    ws = _workspace(q.device, stream.value or 0, need)
    _lib.check(lib.tq_vonly_decode_attn(
        _ptr(q), _dt(q), _ptr(k), _ptr(v_packed), _ptr(v_norms), _host_table(v_centroids), _ptr(v_signs),
        _ptr(out), _ptr(ws), ws.numel(), C.byref(sh), stream))
    return out


class VOnlyStep:
    """The storage of a V-only cache as tq_vonly_decode_step takes it (struct tq_vonly_cache_desc), filled in
    once and reused until the storage is reallocated.  Keeps the tensors it points into alive."""

    def __init__(self, k_f16: torch.Tensor, v_raw, v_packed: torch.Tensor, v_norms: torch.Tensor, signs: torch.Tensor,
                 boundaries, centroids, *, n_rep: int, bits: int, variant: str = "mlx", precision: str = "fp16"):
        _need_gpu(k_f16, v_raw, v_packed, v_norms, signs)
        B, H, T, D = k_f16.shape
        pd = packed_dim(D, bits)
        if k_f16.dtype != torch.float16:
            raise ValueError("k_f16 must be float16")
        shapes = [("k_f16", k_f16, (B, H, T, D)), ("v_packed", v_packed, (B, H, T, pd)), ("v_norms", v_norms, (B, H, T))]
        if v_raw is not None:
            shapes.append(("v_raw", v_raw, (B, H, T, D)))
        for name, t, want in shapes:
            if tuple(t.shape) != want or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous {want} tensor, got {tuple(t.shape)}")
        if v_norms.dtype != torch.float32:
            raise ValueError("v_norms must be float32")
        if v_packed.dtype not in (torch.uint32, torch.int32):
            raise ValueError("v_packed must be uint32 (or its int32 view)")
        if n_rep < 1:
            raise ValueError(f"n_rep must be >= 1, got {n_rep}")
        self._keep = (k_f16, v_raw, v_packed, v_norms, signs)
        self.v_dtype = None if v_raw is None else v_raw.dtype
        self.shape = (B, H, T, D)
        self.n_rep = n_rep
        d = _lib.VOnlyCacheDesc()
        d.k_f16, d.v_packed, d.v_norms, d.v_signs = k_f16.data_ptr(), v_packed.data_ptr(), v_norms.data_ptr(), signs.data_ptr()
        d.v_raw = None if v_raw is None else v_raw.data_ptr()
        b = [float(x) for x in (boundaries.tolist() if isinstance(boundaries, torch.Tensor) else boundaries)]
        c = [float(x) for x in (centroids.tolist() if isinstance(centroids, torch.Tensor) else centroids)]
        if len(b) != (1 << bits) - 1 or len(c) != 1 << bits:
            raise ValueError(f"{bits}-bit tables need {(1 << bits) - 1} boundaries and {1 << bits} centroids")
        for i, x in enumerate(b):
            d.boundaries[i] = x
        for i, x in enumerate(c):
            d.centroids[i] = x
        d.t_alloc, d.n_seq, d.n_kv_heads, d.n_rep, d.dim, d.bits = T, B, H, n_rep, D, bits
        d.variant = {"mlx": _lib.TQ_ENCODE_MLX, "metal": _lib.TQ_ENCODE_METAL}[variant]
        d.allow_mma = _mma_flag(precision)
        self.desc = d
        self._ref = C.byref(d)
        self._need = _lib.load().tq_workspace_bytes(_lib.TQ_OP_VONLY_DECODE, B, H * n_rep, T, D)
        self._ws, self._ws_refs = None, []


def vonly_decode_step(step: VOnlyStep, keys: torch.Tensor, values: torch.Tensor, q: torch.Tensor, position,
                      attn_scale: float, out_dtype=None, out: torch.Tensor | None = None) -> torch.Tensor:
    """One decode step of a V-only cache in one library call (tq_vonly_decode_step): insert the new token
    keys / values (B, n_kv, dim) at time index `position`, then attend with q (B, n_kv * n_rep, dim) over
    positions 0 .. position.  Same result as vonly_append_into followed by vonly_decode.  Returns
    (B, n_q, dim) in out_dtype (default q.dtype), written into `out` when one is given.

    `position` may be a one-element int64 tensor on the GPU (tq_vonly_decode_step_at): the kernels then read
    the position when they run, so the launches can be recorded once in a HIP graph and replayed while the
    caller advances the counter (`position.add_(1)` on the same stream, after the step); the grids cover the
    whole storage, which costs a few idle workgroups, and an insert past the storage is dropped."""
    _need_gpu(keys, values, q, out)
    B, H, T, D = step.shape
    n_q = H * step.n_rep
    if tuple(keys.shape) != (B, H, D) or tuple(values.shape) != (B, H, D) or tuple(q.shape) != (B, n_q, D):
        raise ValueError(f"expected keys / values {(B, H, D)} and q {(B, n_q, D)}, got {tuple(keys.shape)}, "
                         f"{tuple(values.shape)}, {tuple(q.shape)}")
    if step.v_dtype is not None and values.dtype != step.v_dtype:
        raise ValueError(f"values are {values.dtype}, the cache keeps {step.v_dtype}")
    on_device = isinstance(position, torch.Tensor)
    if on_device:
        if position.dtype != torch.int64 or position.numel() != 1 or not position.is_cuda:
            raise ValueError("a device-side position must be a one-element int64 tensor on the GPU")
    elif not 0 <= position < T:
        raise ValueError(f"position {position} outside the storage of {T} positions")
    keys, values, q = keys.contiguous(), values.contiguous(), q.contiguous()
    if out is None:
        out = torch.empty((B, n_q, D), dtype=out_dtype or q.dtype, device=q.device)
    elif tuple(out.shape) != (B, n_q, D) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous {(B, n_q, D)} tensor")
    stream = _stream(q)
    _step_workspace(step, q.device, stream.value or 0)
    lib = _lib.load()
    if on_device:
        _lib.check(lib.tq_vonly_decode_step_at(
            step._ref, _ptr(keys), _dt(keys), _ptr(values), _dt(values), _ptr(q), _dt(q), _ptr(out), _dt(out),
            _ptr(position), attn_scale, stream))
    else:
        _lib.check(lib.tq_vonly_decode_step(
            step._ref, _ptr(keys), _dt(keys), _ptr(values), _dt(values), _ptr(q), _dt(q), _ptr(out), _dt(out),
            position, attn_scale, stream))
    return out


def _step_workspace(step, device, stream_id: int) -> None:
    """Point the descriptor at the (device, stream) workspace.  The descriptor keeps every buffer it has ever
    handed to the library alive: a call recorded in a HIP graph has the address baked in, and the shared
    buffer is replaced (not grown in place) when a later, larger op needs more."""
    ws = _workspace(device, stream_id, step._need)
    if step._ws is not ws:
        step._ws_refs.append(ws)
        step._ws = ws
        step.desc.workspace, step.desc.workspace_bytes = ws.data_ptr(), ws.numel()


def step_call_unchecked(step, keys: torch.Tensor, values: torch.Tensor, q: torch.Tensor, position, attn_scale: float,
                        out: torch.Tensor, packed: bool) -> None:
    """The library call of vonly_decode_step / packed_decode_step without their argument checks, for the cache
    objects, which have established shapes, dtypes and devices themselves: keys / values / q / out are contiguous
    and hold (B, heads, dim) elements in any view of that memory (a (B, heads, 1, dim) tensor qualifies)."""
    stream = _stream(q)
    _step_workspace(step, q.device, stream.value or 0)
    lib = _lib.load()
    if isinstance(position, torch.Tensor):
        fn = lib.tq_packed_decode_step_at if packed else lib.tq_vonly_decode_step_at
        pos = C.c_void_p(position.data_ptr())
    else:
        fn = lib.tq_packed_decode_step if packed else lib.tq_vonly_decode_step
        pos = position
    _lib.check(fn(step._ref, keys.data_ptr(), _DTYPES[keys.dtype], values.data_ptr(), _DTYPES[values.dtype],
                  q.data_ptr(), _DTYPES[q.dtype], out.data_ptr(), _DTYPES[out.dtype], pos, attn_scale, stream))


def _fill_table(dst, values, n, what):
    vals = [float(x) for x in (values.tolist() if isinstance(values, torch.Tensor) else values)]
    if len(vals) != n:
        raise ValueError(f"expected {n} {what}, got {len(vals)}")
    for i, x in enumerate(vals):
        dst[i] = x


class PackedStep:
    """The storage of a cache with packed keys and values as tq_packed_decode_step takes it (struct
    tq_packed_cache_desc), filled in once and reused until the storage is reallocated.  Keeps the tensors
    it points into alive."""

    def __init__(self, k_packed: torch.Tensor, k_norms: torch.Tensor, v_packed: torch.Tensor, v_norms: torch.Tensor,
                 k_signs: torch.Tensor, v_signs: torch.Tensor, boundaries, centroids, *, dim: int, n_rep: int,
                 bits: int, variant: str = "mlx"):
        _need_gpu(k_packed, k_norms, v_packed, v_norms, k_signs, v_signs)
        B, H, T = k_norms.shape
        pd = packed_dim(dim, bits)
        for name, t, want, dts in (("k_packed", k_packed, (B, H, T, pd), (torch.uint32, torch.int32)),
                                   ("v_packed", v_packed, (B, H, T, pd), (torch.uint32, torch.int32)),
                                   ("k_norms", k_norms, (B, H, T), (torch.float32,)),
                                   ("v_norms", v_norms, (B, H, T), (torch.float32,))):
            if tuple(t.shape) != want or not t.is_contiguous() or t.dtype not in dts:
                raise ValueError(f"{name} must be a contiguous {want} tensor of {dts[0]}, got {tuple(t.shape)} {t.dtype}")
        for name, t in (("k_signs", k_signs), ("v_signs", v_signs)):
            if t.dtype != torch.float32 or t.numel() != dim or not t.is_contiguous():
                raise ValueError(f"{name} must be {dim} contiguous float32 values")
        if n_rep < 1:
            raise ValueError(f"n_rep must be >= 1, got {n_rep}")
        self._keep = (k_packed, k_norms, v_packed, v_norms, k_signs, v_signs)
        self.shape = (B, H, T, dim)
        self.n_rep = n_rep
        d = _lib.PackedCacheDesc()
        d.k_packed, d.k_norms, d.v_packed, d.v_norms = k_packed.data_ptr(), k_norms.data_ptr(), v_packed.data_ptr(), v_norms.data_ptr()
        d.k_signs, d.v_signs = k_signs.data_ptr(), v_signs.data_ptr()
        _fill_table(d.boundaries, boundaries, (1 << bits) - 1, "boundaries")
        _fill_table(d.centroids, centroids, 1 << bits, "centroids")
        d.t_alloc, d.n_seq, d.n_kv_heads, d.n_rep, d.dim, d.bits = T, B, H, n_rep, dim, bits
        d.variant = {"mlx": _lib.TQ_ENCODE_MLX, "metal": _lib.TQ_ENCODE_METAL}[variant]
        self.desc = d
        self._ref = C.byref(d)
        self._need = _lib.load().tq_workspace_bytes(_lib.TQ_OP_FLASH_DECODE, B, H * n_rep, T, dim)
        self._ws, self._ws_refs = None, []


def packed_decode_step(step: PackedStep, keys: torch.Tensor, values: torch.Tensor, q: torch.Tensor, position,
                       attn_scale: float, out_dtype=None, out: torch.Tensor | None = None) -> torch.Tensor:
    """One decode step of a packed cache in one library call (tq_packed_decode_step): encode the new token
    keys / values (B, n_kv, dim) at time index `position`, then attend with q (B, n_kv * n_rep, dim; not
    pre-rotated) over positions 0 .. position.  Same result as two encode_into calls followed by
    flash_decode_from_q.  Returns (B, n_q, dim) in out_dtype (default q.dtype), written into `out` when given.
    `position` may be a one-element int64 GPU tensor (tq_packed_decode_step_at), as in vonly_decode_step."""
    _need_gpu(keys, values, q, out)
    B, H, T, D = step.shape
    n_q = H * step.n_rep
    if tuple(keys.shape) != (B, H, D) or tuple(values.shape) != (B, H, D) or tuple(q.shape) != (B, n_q, D):
        raise ValueError(f"expected keys / values {(B, H, D)} and q {(B, n_q, D)}, got {tuple(keys.shape)}, "
                         f"{tuple(values.shape)}, {tuple(q.shape)}")
    on_device = isinstance(position, torch.Tensor)
    if on_device:
        if position.dtype != torch.int64 or position.numel() != 1 or not position.is_cuda:
            raise ValueError("a device-side position must be a one-element int64 tensor on the GPU")
    elif not 0 <= position < T:
        raise ValueError(f"position {position} outside the storage of {T} positions")
    keys, values, q = keys.contiguous(), values.contiguous(), q.contiguous()
    if out is None:
        out = torch.empty((B, n_q, D), dtype=out_dtype or q.dtype, device=q.device)
    elif tuple(out.shape) != (B, n_q, D) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous {(B, n_q, D)} tensor")
    stream = _stream(q)
    _step_workspace(step, q.device, stream.value or 0)
    lib = _lib.load()
    fn = lib.tq_packed_decode_step_at if on_device else lib.tq_packed_decode_step
    _lib.check(fn(step._ref, _ptr(keys), _dt(keys), _ptr(values), _dt(values), _ptr(q), _dt(q), _ptr(out), _dt(out),
                  _ptr(position) if on_device else position, attn_scale, stream))
    return out


def prefill_attention(q: torch.Tensor, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids,
                      k_signs, v_signs, dim: int, bits: int, attn_scale: float, *, n_rep: int = 1,
                      kv_len: int | None = None, q_pos0: int | None = None, causal: bool = True,
                      out_dtype=None, fp16_query: bool = False) -> torch.Tensor:
    """Chunked-prefill attention over packed K and V on the matrix cores (tq_prefill_attn).

    The reference dequantises the whole cache and calls stock SDPA for this step (cache.py:125-129,
    209-210); here the packed rows are decoded tile by tile in LDS and never written back.

    q (n_q, n_rows, dim) fp16/bf16/fp32, not pre-rotated; k_packed / v_packed (n_kv, T_alloc, pdim) uint32,
    k_norms / v_norms (n_kv, T_alloc) fp32; the first kv_len positions are attended (default T_alloc).
    q_pos0 is the cache position of query row 0 (default kv_len - n_rows: the chunk is the cache's
    tail).  Returns (n_q, n_rows, dim) in out_dtype (default q.dtype).
    fp16_query=True drops the fp16 remainder of the rotated query (a third fewer matrix instructions):
    fine on data without outlier channels, up to 1e-2 of an output row with them -- off by default.
    """
    _need_gpu(q, k_packed, k_norms, v_packed, v_norms)
    n_q, n_rows, _ = q.shape
    n_kv = k_norms.shape[0]
    _check_gqa(n_q, n_kv, n_rep)
    pd = packed_dim(dim, bits)
    if q.dtype not in _DTYPES:
        q = q.float()
    q = q.contiguous()
    k_packed = _u32(k_packed)
    v_packed = _u32(v_packed)
    if k_packed.stride(-1) != 1 or k_packed.stride(-2) != pd or v_packed.stride(-1) != 1 or v_packed.stride(-2) != pd:
        k_packed, v_packed = k_packed.contiguous(), v_packed.contiguous()
    k_norms = k_norms.to(torch.float32)
    v_norms = v_norms.to(torch.float32)
    if k_norms.stride(-1) != 1 or v_norms.stride(-1) != 1:
        k_norms, v_norms = k_norms.contiguous(), v_norms.contiguous()
    T = int(kv_len if kv_len is not None else k_norms.shape[-1])
    _check_rows(T, True, 1, k_packed=k_packed, k_norms=k_norms, v_packed=v_packed, v_norms=v_norms)
    pos0 = int(q_pos0 if q_pos0 is not None else T - n_rows)
    out_dtype = out_dtype or q.dtype
    out = torch.empty((n_q, n_rows, dim), dtype=out_dtype, device=q.device)
    if n_rows == 0:
        return out
    k_signs = _as_f32_dev(k_signs, q)
    v_signs = _as_f32_dev(v_signs, q)
    lib = _lib.load()
    need = lib.tq_prefill_workspace_bytes(n_q, n_rows, T, dim)
    stream = _stream(q)
    ws = _workspace(q.device, stream.value or 0, max(need, 256))
    _lib.check(lib.tq_prefill_attn(
        _ptr(q), _dt(q), _ptr(k_packed), _ptr(k_norms), _ptr(v_packed), _ptr(v_norms),
        _host_table(k_centroids), _host_table(v_centroids), _ptr(k_signs), _ptr(v_signs),
        _ptr(out), _dt(out), _ptr(ws), ws.numel(), n_kv, n_rep, n_rows, T, pos0,
        k_packed.stride(0) // pd, k_norms.stride(0), v_packed.stride(0) // pd, v_norms.stride(0),
        dim, bits, float(attn_scale), (1 if causal else 0) | (2 if fp16_query else 0), stream))
    return out
