"""Decode-step attention over PolarQuant caches.

`turboquant_attention` is the reference composition (fused_attention.py:20-125): pre-rotate the
query, score it against the packed keys, scale, mask, softmax, then the butterfly-pulled-out
weighted sum over packed values.  `vonly_decode_attention` is the same for a V-only cache, whose
keys are fp16.  Both can run as ONE fused launch per step when no positive sparse-V threshold is
asked for; the threshold is defined on final softmax weights, so with one the scores of the whole
sequence are produced first (for a V-only cache inside one library call, otherwise as separate ops).
"""
from __future__ import annotations

import torch

from . import ops


def _mask_rows(mask, b: int, n_q: int, total: int):
    """The mask rank cases of fused_attention.py:81-92, returning a (rows, total) float tensor."""
    m = mask
    if m.dim() == 4:
        m = m[min(b, m.shape[0] - 1)]
        m = m[:, 0, :]
        if m.shape[0] == 1:
            m = m.expand(n_q, total)
    elif m.dim() == 3:
        m = m[min(b, m.shape[0] - 1), 0, :].reshape(1, -1).expand(n_q, total)
    elif m.dim() == 1:
        m = m.reshape(1, -1)
    if m.dtype == torch.bool:
        m = torch.zeros(m.shape, dtype=torch.float32, device=m.device).masked_fill_(~m, float("-inf"))
    return m


def turboquant_attention(queries: torch.Tensor, cache, attn_scale: float, mask=None, v_buffer=None,
                         sparse_v_threshold: float | None = None, fused: bool = False) -> torch.Tensor:
    """fused_attention.py:20-125.  queries (B, n_heads, 1, dim) against a TurboQuantKVCache holding
    packed K and V; returns (B, n_heads, 1, dim) in queries.dtype.

    fused=True runs the whole step as one library call (pre-rotation aside) when no v_buffer is given: one
    launch + merge without a sparse-V threshold, three passes with one (d = 128 / n_rep <= 16; other
    shapes compose the separate ops); the result is the same up to summation order and operand rounding.
    """
    B, n_q, S_q, dim = queries.shape
    if S_q != 1:
        raise ValueError(f"turboquant_attention is a decode step: expected one query token, got {S_q}")
    total = cache.offset
    n_kv = cache.k_packed.shape[1]
    n_rep = n_q // n_kv
    bits = cache.quant_bits
    kq, vq = cache._k_q, cache._v_q
    thr = sparse_v_threshold if (sparse_v_threshold is not None and sparse_v_threshold >= 0.0) else 0.0

    one_call_thr = thr > 0.0 and ops.vonly_sparse_supported(dim, bits, n_rep) and total > 0 and dim == cache._v_dim
    if fused and v_buffer is None and (thr == 0.0 or one_call_thr):
        m = None
        if mask is not None:
            m = torch.stack([_mask_rows(mask, b, n_q, total).expand(n_q, total) for b in range(B)])
        od = queries.dtype if queries.dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.float32
        if ops.vonly_sparse_supported(dim, bits, n_rep) and total > 0 and dim == cache._v_dim:
            # one call: the kernels rotate the query themselves
            out = ops.flash_decode_from_q(queries[:, :, 0, :], kq.signs, cache.k_packed, cache.k_norms, cache.v_packed,
                                          cache.v_norms, kq.centroids, vq.centroids, vq.signs, dim, bits, attn_scale,
                                          n_rep=n_rep, seq_len=total, mask=m, out_dtype=od, sparse_v_threshold=thr)
        else:
            q_rot = ops.prerotate_query(queries.reshape(B * n_q, dim), kq.signs).reshape(B, n_q, dim)
            out = ops.flash_decode(q_rot, cache.k_packed, cache.k_norms, cache.v_packed, cache.v_norms,
                                   kq.centroids, vq.centroids, vq.signs, dim, bits, attn_scale, n_rep=n_rep,
                                   seq_len=total, mask=m, out_dtype=od, sparse_v_threshold=thr)
        out = out[:, :, None, :]
        return out if out.dtype == queries.dtype else out.to(queries.dtype)

    outputs = []
    for b in range(B):
        kp = cache.k_packed[b, :, :total, :]
        kn = cache.k_norms[b, :, :total]
        q_rot = ops.prerotate_query(queries[b, :, 0, :], kq.signs)
        scores = ops.prerot_fused_qk_scores(q_rot, kp, kn, kq.centroids, dim, bits, n_rep=n_rep)
        m = _mask_rows(mask, b, n_q, total) if mask is not None else None
        weights = ops.softmax_rows(scores, attn_scale, m)
        if v_buffer is not None:
            v_deq = v_buffer[b]
            if n_rep > 1:
                v_deq = v_deq.repeat_interleave(n_rep, dim=0)
            out = weights[:, None, :].to(queries.dtype) @ v_deq.to(queries.dtype)
        else:
            vp = cache.v_packed[b, :, :total, :]
            vn = cache.v_norms[b, :, :total]
            mv = ops.sparse_v_matvec(weights, vp, vn, vq.centroids, vq.signs, cache._v_dim, bits,
                                     threshold=thr, n_rep=n_rep)
            out = mv[:, None, :].to(queries.dtype)
        outputs.append(out)
    return torch.stack(outputs, dim=0)


def vonly_decode_attention(queries: torch.Tensor, cache, attn_scale: float, mask=None,
                           sparse_v_threshold: float | None = None) -> torch.Tensor:
    """Decode attention straight off a VOnlyTurboQuantCache: softmax(q K^T * scale + mask) over the
    fp16 keys, then the weighted sum over the packed values without ever dequantising them
    (the dense-K-scores -> softmax -> sparse_v_matvec shape of hybrid_attention.py:52-88).

    queries (B, n_heads, 1, dim) -> (B, n_heads, 1, dim) in queries.dtype.  With no positive
    threshold the step is one fused launch; with one it is one call of three passes (scores, weights
    and values, merge) so that the threshold applies to the final weights (sparse_v.py:60-61); shapes
    outside the matrix-core kernels (dim != 128, more than 16 query heads per kv head) run scores, softmax and sparse-V separately.
    """
    B, n_q, S_q, dim = queries.shape
    if S_q != 1:
        raise ValueError(f"vonly_decode_attention is a decode step: expected one query token, got {S_q}")
    kc, tq = cache._k_cache, cache._v_tq
    total = kc.offset
    n_kv = kc.keys.shape[1]
    n_rep = n_q // n_kv
    vq = tq._v_q
    bits = tq.quant_bits
    thr = sparse_v_threshold if (sparse_v_threshold is not None and sparse_v_threshold >= 0.0) else 0.0
    if thr == 0.0 or (ops.vonly_threshold_supported(dim, bits, n_rep) and total > 0):
        m = None
        if mask is not None:
            m = torch.stack([_mask_rows(mask, b, n_q, total).expand(n_q, total) for b in range(B)])
        od = queries.dtype if queries.dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.float32
        out = ops.vonly_decode(queries[:, :, 0, :], kc.keys, tq.v_packed, tq.v_norms, vq.centroids, vq.signs,
                               dim, bits, attn_scale, n_rep=n_rep, seq_len=total, mask=m, out_dtype=od,
                               sparse_v_threshold=thr)
        out = out[:, :, None, :]                           # written in the query dtype by the merge pass
        return out if out.dtype == queries.dtype else out.to(queries.dtype)
    outputs = []
    for b in range(B):
        scores = ops.dense_qk_scores(queries[b, :, 0, :], kc.keys[b, :, :total, :], 1.0, n_rep=n_rep)
        m = _mask_rows(mask, b, n_q, total) if mask is not None else None
        weights = ops.softmax_rows(scores, attn_scale, m)
        mv = ops.sparse_v_matvec(weights, tq.v_packed[b, :, :total, :], tq.v_norms[b, :, :total],
                                 vq.centroids, vq.signs, tq._v_dim, bits, threshold=thr, n_rep=n_rep)
        outputs.append(mv[:, None, :].to(queries.dtype))
    return torch.stack(outputs, dim=0)


def turboquant_prefill_attention(queries: torch.Tensor, cache, attn_scale: float, causal: bool = True) -> torch.Tensor:
    """Multi-token forward (prompt chunk) straight off the packed K and V of a TurboQuantKVCache,
    after `cache.update_and_fetch` has encoded the chunk: the last S of the cache's `offset`
    positions are the chunk's own, and query row i attends positions <= offset - S + i.

    The reference has no such path: its prefill dequantises the whole cache (cache.py:209-218) and
    hands fp16 K/V to stock SDPA, and with fused=True it returns zero placeholders (cache.py:162-165)
    that only a decode step knows how to bypass.  queries (B, n_heads, S, dim) -> same shape and dtype.
    """
    B, n_q, S, dim = queries.shape
    total = cache.offset
    if S > total:
        raise ValueError(f"the cache holds {total} positions, fewer than the {S} query rows")
    n_kv = cache.k_packed.shape[1]
    n_rep = n_q // n_kv
    kq, vq = cache._k_q, cache._v_q
    outs = [ops.prefill_attention(queries[b], cache.k_packed[b], cache.k_norms[b], cache.v_packed[b],
                                  cache.v_norms[b], kq.centroids, vq.centroids, kq.signs, vq.signs, dim,
                                  cache.quant_bits, attn_scale, n_rep=n_rep, kv_len=total, q_pos0=total - S,
                                  causal=causal)
            for b in range(B)]
    return torch.stack(outs, dim=0)
