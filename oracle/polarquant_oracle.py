"""CPU oracle for the PolarQuant KV-cache hot path.  TEST INFRASTRUCTURE ONLY.

This module is a numpy restatement of the reference's algorithm; it exists to
check the HIP kernels and to serve as the timed CPU baseline.  Nothing in the
shipped package may import it: only tests, the smoke check and the bench's
cpu_baseline leg do.

Every function cites the reference file:line it follows (paths relative to the
reference tree).  Arithmetic that decides packed bits is done in float32 with
numpy (IEEE, no FMA contraction), one rounding per reference operation.

Parity status
-------------
pinned (closed forms / invariants / brute force, see tests/test_oracle_*.py):
  raw_butterfly, walsh_hadamard_transform, codebook tables and boundaries,
  quantize, pack_indices / unpack_indices, dequantize, prerotate_query,
  prerot_fused_qk_scores, packed_fused_qk_scores, sparse_v_matvec,
  flash_attention_turboquant, turboquant_attention.
parity unpinned (only an MLX install could pin them):
  * random_diagonal_sign: the reference draws the +-1 pattern from MLX's
    PRNG stream (rotation.py:47-49); MLX is not available, so this module
    uses its own documented generator.  Every function takes `signs`
    explicitly, so the rest of the path is independent of the generator.
    mlx_random_diagonal_sign restates MLX's stream from its published
    algorithm: its hash (threefry2x32) is pinned by the Random123
    known-answer vectors, the word layout and the float conversion are not.
  * the float32 summation order inside mx.linalg.norm (quantizer.py:89) is
    backend-defined; this oracle fixes it to the only order the reference
    specifies, the stride-halving tree of its Metal encoder (metal.py:33-38).
"""

from __future__ import annotations

import math

import numpy as np

F32 = np.float32

# packing.py:16-17
VALS_PER_WORD = {1: 32, 2: 16, 3: 10, 4: 8}
BIT_MASK = {1: 0x1, 2: 0x3, 3: 0x7, 4: 0xF}

# quantizer.py:27-36 (duplicated at cache.py:15-25)
_CODEBOOKS = {
    1: [-0.7979, 0.7979],
    2: [-1.5104, -0.4528, 0.4528, 1.5104],
    3: [-2.1520, -1.3440, -0.7560, -0.2451, 0.2451, 0.7560, 1.3440, 2.1520],
    4: [-2.7326, -2.0690, -1.6180, -1.2562, -0.9423, -0.6568, -0.3881, -0.1284,
        0.1284, 0.3881, 0.6568, 0.9423, 1.2562, 1.6180, 2.0690, 2.7326],
}


# --------------------------------------------------------------------------
# rotation.py
# --------------------------------------------------------------------------

def raw_butterfly(x: np.ndarray) -> np.ndarray:
    """Un-normalised Walsh-Hadamard butterfly on the last axis, float32.

    Stage order h = 1, 2, ..., d/2; at each stage the pair (j, j+h) with bit h
    of j clear becomes (a+b, a-b).  rotation.py:22-32; the same data flow is
    the in-kernel loop at metal.py:51-64.
    """
    x = np.array(x, dtype=F32, copy=True)
    d = x.shape[-1]
    if d <= 0 or d & (d - 1):
        raise AssertionError(f"Dimension must be power of 2, got {d}")
    lead = x.shape[:-1]
    h = 1
    while h < d:
        v = x.reshape(*lead, d // (2 * h), 2, h)
        a = v[..., 0, :]
        b = v[..., 1, :]
        x = np.stack([a + b, a - b], axis=-2).reshape(*lead, d)
        h *= 2
    return x


def wht_scale(d: int) -> np.float32:
    """float32 value of the python scalar 1/sqrt(d) (rotation.py:34, quantizer.py:73)."""
    return F32(1.0 / math.sqrt(d))


def walsh_hadamard_transform(x: np.ndarray) -> np.ndarray:
    """rotation.py:7-34: raw butterfly then one multiply by float32(1/sqrt(d))."""
    return raw_butterfly(x) * wht_scale(x.shape[-1])


def _splitmix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & 0xFFFFFFFFFFFFFFFF
    return z ^ (z >> 31)


def random_diagonal_sign(d: int, seed: int = 42) -> np.ndarray:
    """(d,) float32 vector of +-1.  PARITY UNPINNED versus rotation.py:37-49.

    The reference takes the pattern from MLX's PRNG, which cannot be reproduced
    offline.  Generator used here: element i is +1 when the top bit of
    splitmix64(splitmix64(seed) + i) is set, else -1.
    """
    base = _splitmix64(seed & 0xFFFFFFFFFFFFFFFF)
    out = np.empty(d, dtype=F32)
    for i in range(d):
        out[i] = 1.0 if (_splitmix64((base + i) & 0xFFFFFFFFFFFFFFFF) >> 63) else -1.0
    return out


def threefry2x32(key0, key1, x0, x1):
    """Threefry-2x32-20 (Salmon et al., SC'11) on uint32 arrays: the counter-based hash of MLX's `mx.random`
    (third-party, mlx >= 0.20, pyproject.toml:13; absent here).  Pinned by the Random123 known-answer vectors."""
    u32 = np.uint32
    key0, key1 = u32(key0), u32(key1)
    ks = (key0, key1, u32(0x1BD11BDA) ^ key0 ^ key1)
    x0 = np.asarray(x0, dtype=u32).copy()
    x1 = np.asarray(x1, dtype=u32).copy()
    rot = ((13, 15, 26, 6), (17, 29, 16, 24))
    with np.errstate(over="ignore"):
        x0 += ks[0]
        x1 += ks[1]
        for block in range(5):
            for r in rot[block & 1]:
                x0 += x1
                x1 = (x1 << u32(r)) | (x1 >> u32(32 - r))
                x1 ^= x0
            x0 += ks[(block + 1) % 3]
            x1 += ks[(block + 2) % 3] + u32(block + 1)
    return x0, x1


def mlx_random_diagonal_sign(d: int, seed: int = 42) -> np.ndarray:
    """rotation.py:47-49 with MLX's generator restated from its published source: key (seed >> 32, seed & 2^32-1);
    word i and word i + ceil(d/2) are the two outputs of threefry2x32(key, (i, i + ceil(d/2))) (odd d: the middle
    word is the first output of (floor(d/2), 0)); uniform = float32(word) / float32(2^32 - 1), capped below 1;
    +1 where uniform < 0.5.  PARITY UNPINNED beyond the hash: only an MLX install could confirm the layout."""
    half, odd = d // 2, d & 1
    i = np.arange(half, dtype=np.uint32)
    a, b = threefry2x32((seed >> 32) & 0xFFFFFFFF, seed & 0xFFFFFFFF, i, i + np.uint32(half + odd))
    words = np.empty(d, dtype=np.uint32)
    words[:half] = a
    words[half + odd:] = b
    if odd:
        words[half] = threefry2x32((seed >> 32) & 0xFFFFFFFF, seed & 0xFFFFFFFF, [half], [0])[0][0]
    u = np.minimum(words.astype(F32) / F32(4294967295.0), np.nextafter(F32(1.0), F32(0.0)))
    return np.where(u < F32(0.5), F32(1.0), F32(-1.0)).astype(F32)


def randomized_hadamard_transform(x: np.ndarray, signs: np.ndarray) -> np.ndarray:
    """rotation.py:52-64: WHT(x * signs)."""
    return walsh_hadamard_transform(np.asarray(x, dtype=F32) * np.asarray(signs, dtype=F32))


def inverse_randomized_hadamard(x: np.ndarray, signs: np.ndarray) -> np.ndarray:
    """rotation.py:67-80: WHT(x) * signs."""
    return walsh_hadamard_transform(x) * np.asarray(signs, dtype=F32)


# --------------------------------------------------------------------------
# quantizer.py
# --------------------------------------------------------------------------

def gaussian_codebook(bits: int) -> np.ndarray:
    """quantizer.py:18-38: literal Lloyd-Max N(0,1) centroid tables as float32."""
    if bits not in _CODEBOOKS:
        raise ValueError(f"Unsupported bit width: {bits}. Use 1-4.")
    return np.array(_CODEBOOKS[bits], dtype=F32)


def gaussian_boundaries(centroids: np.ndarray) -> np.ndarray:
    """quantizer.py:41-44: float32 midpoints (c[i] + c[i+1]) / 2."""
    c = np.asarray(centroids, dtype=F32)
    return (c[:-1] + c[1:]) / F32(2.0)


def sumsq_tree(x32: np.ndarray) -> np.ndarray:
    """Sum of squares over the last axis in the stride-halving order of metal.py:33-38.

    ns[e] = x[e]*x[e]; for stride = d/2, d/4, ..., 1: ns[e] += ns[e+stride] for
    e < stride; the result is ns[0].  Each product and each add rounds to float32.
    """
    ns = x32 * x32
    d = ns.shape[-1]
    stride = d // 2
    while stride > 0:
        ns = ns[..., :stride] + ns[..., stride:2 * stride]
        stride //= 2
    return ns[..., 0]


def quantize(x: np.ndarray, signs: np.ndarray, boundaries: np.ndarray,
             variant: str = "mlx"):
    """PolarQuant encode of (..., d) vectors -> (idx uint8 (..., d), norms f32 (...)).

    variant="mlx" follows PolarQuantizer.quantize, quantizer.py:85-106:
      float32 upcast; n = ||x||; u = x / max(n, 1e-8); y = WHT(u * signs)
      (raw butterfly then * float32(1/sqrt d), rotation.py:34,64);
      z = y / float32(1/sqrt d) (quantizer.py:97); idx = #{b : z > b} strict.
    variant="metal" follows the fused Metal encoder, metal.py:29-77: same up to
      the raw butterfly, then compares the raw butterfly output directly
      (metal.py:66-69) -- no multiply/divide by the scale.
    The returned norm is the un-clamped n (quantizer.py:106, metal.py:98-100).
    """
    x32 = np.asarray(x).astype(F32)
    signs = np.asarray(signs, dtype=F32)
    boundaries = np.asarray(boundaries, dtype=F32)
    d = x32.shape[-1]
    n = np.sqrt(sumsq_tree(x32)).astype(F32)
    safe = np.maximum(n, F32(1e-8))
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        u = x32 / safe[..., None]
        w = raw_butterfly(u * signs)
        if variant == "mlx":
            s = wht_scale(d)
            z = (w * s) / s
        elif variant == "metal":
            z = w
        else:
            raise ValueError(f"unknown variant {variant!r}")
        idx = np.zeros(z.shape, dtype=np.uint8)
        for b in boundaries.tolist():
            idx = idx + (z > F32(b)).astype(np.uint8)
    return idx, n


def dequantize(idx: np.ndarray, norms: np.ndarray, centroids: np.ndarray,
               signs: np.ndarray) -> np.ndarray:
    """quantizer.py:108-132: ((raw_butterfly(c[idx]*s) * s) * signs) * norm, float32.

    The Metal decoders use the identical operation order (kernels.py:30,53;
    metal.py:118,139).
    """
    c = np.asarray(centroids, dtype=F32)
    signs = np.asarray(signs, dtype=F32)
    d = idx.shape[-1]
    s = wht_scale(d)
    y = c[np.asarray(idx).astype(np.int64)] * s
    x_unit = (raw_butterfly(y) * s) * signs
    return x_unit * np.asarray(norms, dtype=F32)[..., None]


# --------------------------------------------------------------------------
# packing.py
# --------------------------------------------------------------------------

def packed_dim(dim: int, bits: int) -> int:
    """packing.py:20-23."""
    vpw = VALS_PER_WORD[bits]
    return (dim + vpw - 1) // vpw


def pack_indices(indices: np.ndarray, bits: int) -> np.ndarray:
    """packing.py:26-56: element e goes to word e // vpw, bit offset (e % vpw) * bits."""
    vpw = VALS_PER_WORD[bits]
    idx = np.asarray(indices)
    dim = idx.shape[-1]
    flat = idx.reshape(-1, dim).astype(np.uint32)
    pd = packed_dim(dim, bits)
    padded = np.zeros((flat.shape[0], pd * vpw), dtype=np.uint32)
    padded[:, :dim] = flat
    padded = padded.reshape(-1, pd, vpw)
    out = np.zeros((flat.shape[0], pd), dtype=np.uint32)
    for i in range(vpw):
        out |= padded[:, :, i] << np.uint32(i * bits)
    return out.reshape(*idx.shape[:-1], pd)


def unpack_indices(packed: np.ndarray, bits: int, dim: int) -> np.ndarray:
    """packing.py:59-87."""
    vpw = VALS_PER_WORD[bits]
    mask = np.uint32(BIT_MASK[bits])
    p = np.asarray(packed, dtype=np.uint32)
    pd = p.shape[-1]
    flat = p.reshape(-1, pd)
    vals = np.stack([(flat >> np.uint32(i * bits)) & mask for i in range(vpw)], axis=-1)
    vals = vals.reshape(flat.shape[0], pd * vpw)[:, :dim]
    return vals.reshape(*p.shape[:-1], dim).astype(np.uint8)


def fused_quantize(vectors: np.ndarray, signs: np.ndarray, boundaries: np.ndarray,
                   dim: int, bits: int, variant: str = "mlx"):
    """metal.py:147-196 surface: (n_vecs, dim) -> packed (n_vecs, pdim) u32, norms (n_vecs,) f32."""
    idx, norms = quantize(np.asarray(vectors).reshape(-1, dim), signs, boundaries, variant)
    return pack_indices(idx, bits), norms


def packed_dequantize(packed: np.ndarray, norms: np.ndarray, centroids: np.ndarray,
                      signs: np.ndarray, dim: int, bits: int) -> np.ndarray:
    """kernels.py:123-155 surface: (seq, pdim) u32 + (seq,) -> (seq, dim) float32."""
    return dequantize(unpack_indices(packed, bits, dim), norms, centroids, signs)


def dequant_fp16(packed, norms, centroids, signs, dim: int, bits: int) -> np.ndarray:
    """metal.py:199-232: same arithmetic, result cast to half."""
    return packed_dequantize(packed, norms, centroids, signs, dim, bits).astype(np.float16)


# --------------------------------------------------------------------------
# kernels.py / metal_kernels_v4.py
# --------------------------------------------------------------------------

def prerotate_query(q: np.ndarray, signs: np.ndarray) -> np.ndarray:
    """metal_kernels_v4.py:37-62: raw_butterfly(q * signs), no 1/sqrt(d)."""
    q = np.asarray(q)
    if q.ndim != 2:
        raise ValueError(f"prerotate_query expects (n_heads, dim), got {q.shape}")
    return raw_butterfly(q.astype(F32) * np.asarray(signs, dtype=F32))


def packed_fused_qk_scores(query, k_packed, k_norms, centroids, signs, dim: int, bits: int):
    """kernels.py:58-117: score[h,p] = sum_e dequant(K[h,p])[e] * q[h,e]  (MHA only)."""
    kd = packed_dequantize(k_packed, k_norms, centroids, signs, dim, bits)  # (H,S,D)
    q = np.asarray(query).astype(F32)
    return np.einsum("hsd,hd->hs", kd.astype(np.float64), q.astype(np.float64)).astype(F32)


def prerot_fused_qk_scores(q_rot, k_packed, k_norms, centroids, dim: int, bits: int,
                           n_rep: int = 1) -> np.ndarray:
    """metal_kernels_v4.py:71-113,153-221.

    score[h,p] = (sum_e c[idx[h//n_rep,p,e]] * q_rot[h,e]) * norm[h//n_rep,p] * (1/dim).
    """
    q_rot = np.asarray(q_rot, dtype=F32)
    k_norms = np.asarray(k_norms, dtype=F32)
    n_q = q_rot.shape[0]
    n_kv, seq = k_norms.shape
    if n_q != n_kv * n_rep:
        raise ValueError(
            f"n_q_heads ({n_q}) must equal n_kv_heads ({n_kv}) * n_rep ({n_rep})")
    c = np.asarray(centroids, dtype=F32)
    idx = unpack_indices(k_packed, bits, dim).astype(np.int64)      # (n_kv, seq, dim)
    cv = c[idx].astype(np.float64)
    qg = q_rot.reshape(n_kv, n_rep, dim).astype(np.float64)
    dots = np.matmul(qg, cv.transpose(0, 2, 1))                      # (n_kv, n_rep, seq)
    out = dots.astype(F32) * k_norms[:, None, :] * F32(1.0 / dim)
    return out.reshape(n_q, seq).astype(F32)


# --------------------------------------------------------------------------
# sparse_v.py
# --------------------------------------------------------------------------

def sparse_v_matvec(weights, v_packed, v_norms, centroids, signs, dim: int, bits: int,
                    threshold: float = 1e-5, n_rep: int = 1) -> np.ndarray:
    """sparse_v.py:32-88,94-186.

    S[h,e] = sum over p with not (w[h,p] < thr) of w[h,p] * norm[h//n_rep,p] * c[idx[h//n_rep,p,e]];
    out[h] = raw_butterfly(S[h]) * signs * (1/dim); thr = float32(max(threshold, 0)).
    """
    if dim & (dim - 1):
        raise ValueError(f"dim must be a power of 2, got {dim}")
    if dim > 256:
        raise ValueError(f"dim > 256 not supported by threadgroup layout, got {dim}")
    w = np.asarray(weights).astype(F32)
    n_q, seq = w.shape
    n_kv = np.asarray(v_packed).shape[0]
    if n_q != n_kv * n_rep:
        raise ValueError(
            f"n_q_heads ({n_q}) must equal n_kv_heads ({n_kv}) * n_rep ({n_rep})")
    thr = F32(max(threshold, 0.0))
    c = np.asarray(centroids, dtype=F32)
    idx = unpack_indices(v_packed, bits, dim).astype(np.int64)
    cv = c[idx].astype(np.float64)                                   # (n_kv, seq, dim)
    wn = np.where(w < thr, F32(0), w).reshape(n_kv, n_rep, seq).astype(np.float64)
    wn = wn * np.asarray(v_norms, dtype=F32).astype(np.float64)[:, None, :]
    S = np.matmul(wn, cv).reshape(n_q, dim).astype(F32)
    return raw_butterfly(S) * np.asarray(signs, dtype=F32) * F32(1.0 / dim)


def count_active_positions(weights, threshold: float = 1e-5) -> int:
    """sparse_v.py:189-191."""
    return int((np.asarray(weights) > threshold).sum())


# --------------------------------------------------------------------------
# flash_attention.py / fused_attention.py
# --------------------------------------------------------------------------

def _softmax64(s: np.ndarray) -> np.ndarray:
    s = s.astype(np.float64)
    m = s.max(axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - m)
    return e / e.sum(axis=-1, keepdims=True)


def flash_attention_turboquant(q_rot, k_packed, k_norms, v_packed, v_norms, k_centroids,
                               v_centroids, v_signs, dim: int, bits: int, attn_scale: float,
                               block_size: int = 16, n_rep: int = 1) -> np.ndarray:
    """flash_attention.py:36-163,168-274, evaluated in float64 (the blocked online
    softmax is mathematically the plain softmax; block_size only validates).

    out[h] = signs_v * raw_butterfly(sum_p softmax_p(s[h,:]) * v_norm * c_v[idx_v]) / dim,
    s[h,p] = (sum_e c_k[idx_k] * q_rot[h,e]) * k_norm * (1/dim) * attn_scale.
    """
    if dim > 128 or dim & (dim - 1):
        raise ValueError(f"dim must be a power of 2 and <= 128, got {dim}")
    if block_size < 1 or block_size > 32:
        raise ValueError(f"block_size must be in 1..32, got {block_size}")
    s = prerot_fused_qk_scores(q_rot, k_packed, k_norms, k_centroids, dim, bits, n_rep)
    w = _softmax64(s.astype(np.float64) * float(attn_scale))
    return sparse_v_matvec(w.astype(F32), v_packed, v_norms, v_centroids, v_signs, dim, bits,
                           threshold=0.0, n_rep=n_rep)


def turboquant_attention_single(q, k_packed, k_norms, v_packed, v_norms, k_centroids, k_signs,
                                v_centroids, v_signs, dim: int, bits: int, attn_scale: float,
                                mask=None, sparse_v_threshold=None) -> np.ndarray:
    """One batch element of fused_attention.py:56-121: prerotate -> scores -> *scale -> +mask
    -> softmax -> sparse_v_matvec.  q: (n_q, dim); packed K/V: (n_kv, T, pdim)."""
    n_q = q.shape[0]
    n_kv = k_packed.shape[0]
    n_rep = n_q // n_kv
    q_rot = prerotate_query(q, k_signs)
    s = prerot_fused_qk_scores(q_rot, k_packed, k_norms, k_centroids, dim, bits, n_rep)
    s = s * F32(attn_scale)
    if mask is not None:
        s = s + np.asarray(mask, dtype=F32)
    w = _softmax64(s).astype(F32)
    thr = sparse_v_threshold if (sparse_v_threshold is not None and sparse_v_threshold >= 0.0) else 0.0
    return sparse_v_matvec(w, v_packed, v_norms, v_centroids, v_signs, dim, bits,
                           threshold=thr, n_rep=n_rep)


def vonly_decode_attention(q, k, v_packed, v_norms, v_centroids, v_signs, dim: int, bits: int,
                           attn_scale: float, threshold: float = 0.0, mask=None) -> np.ndarray:
    """Dense-K scores -> softmax -> sparse_v_matvec for a V-only cache: the composition of
    hybrid_attention.py:52-88 with fp16 keys (v_only_cache.py:24-38) in place of the
    affine-quantised ones.  q: (n_q, dim); k: (n_kv, T, dim) fp16; returns (n_q, dim) f32."""
    q = np.asarray(q)
    k = np.asarray(k)
    n_q = q.shape[0]
    n_kv, T, _ = k.shape
    n_rep = n_q // n_kv
    if n_q != n_kv * n_rep:
        raise ValueError(
            f"n_q_heads ({n_q}) must equal n_kv_heads ({n_kv}) * n_rep ({n_rep})")
    qg = q.reshape(n_kv, n_rep, dim).astype(np.float64)
    s = np.matmul(qg, k.astype(np.float64).transpose(0, 2, 1)).reshape(n_q, T) * float(attn_scale)
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64)
    w = _softmax64(s).astype(F32)
    return sparse_v_matvec(w, v_packed, v_norms, v_centroids, v_signs, dim, bits,
                           threshold=threshold, n_rep=n_rep)


def dense_attention(q, k, v, attn_scale: float, mask=None) -> np.ndarray:
    """Plain softmax(q k^T * scale + mask) v in float64 with GQA head grouping.
    q: (n_q, S_q, d); k, v: (n_kv, T, d); mask broadcastable to (n_q, S_q, T)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    n_q, S_q, d = q.shape
    n_kv, T, _ = k.shape
    n_rep = n_q // n_kv
    qg = q.reshape(n_kv, n_rep, S_q, d)
    s = np.einsum("grqd,gtd->grqt", qg, k) * float(attn_scale)
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64).reshape(n_kv, n_rep, S_q, T) \
            if np.asarray(mask).ndim == 3 else s + np.asarray(mask, dtype=np.float64)
    w = _softmax64(s)
    return np.einsum("grqt,gtd->grqd", w, v).reshape(n_q, S_q, v.shape[-1])


def prefill_attention(q, k_packed, k_norms, v_packed, v_norms, k_centroids, v_centroids, k_signs,
                      v_signs, dim: int, bits: int, attn_scale: float, q_pos0: int, n_rep: int = 1,
                      causal: bool = True) -> np.ndarray:
    """Chunk of query rows against a packed cache, as the reference's prefill computes it:
    dequantise K and V (cache.py:125-129, 209-210 -> quantizer.py:108-132) and run plain
    softmax attention with the causal rule "row i sees positions <= q_pos0 + i"
    (cache.py:314-334 builds that mask with mlx-lm's create_causal_mask(N, offset)).

    q: (n_q, n_rows, dim); k_packed/v_packed: (n_kv, T, pdim); norms (n_kv, T).  float64 result
    (n_q, n_rows, dim)."""
    q = np.asarray(q)
    n_q, n_rows, _ = q.shape
    n_kv, T = np.asarray(k_norms).shape
    if n_q != n_kv * n_rep:
        raise ValueError(
            f"n_q_heads ({n_q}) must equal n_kv_heads ({n_kv}) * n_rep ({n_rep})")
    pd = packed_dim(dim, bits)
    k = packed_dequantize(np.asarray(k_packed).reshape(-1, pd), np.asarray(k_norms).reshape(-1),
                          k_centroids, k_signs, dim, bits).reshape(n_kv, T, dim)
    v = packed_dequantize(np.asarray(v_packed).reshape(-1, pd), np.asarray(v_norms).reshape(-1),
                          v_centroids, v_signs, dim, bits).reshape(n_kv, T, dim)
    mask = None
    if causal:
        pos = np.arange(T)[None, :]
        row = np.arange(n_rows)[:, None] + int(q_pos0)
        mask = np.where(pos <= row, 0.0, -np.inf)                      # (n_rows, T), broadcast over heads
    return dense_attention(q.astype(np.float64), k, v, attn_scale, mask)
