"""Per-kernel micro-benchmarks at the shapes of the reference's configurations.

Methodology of the reference's scripts/bench_sparse_v.py:49-57 (warm-up, then a timed loop with a
sync at the end), adapted to a GPU with large caches: HIP events on the launch stream, many
back-to-back launches, and rotation over several independent input sets so that the 256 MB
Infinity Cache cannot serve the reads.  Prints one line per case: us per call, GB/s of algorithmic
bytes and the fraction of 8 TB/s.

    python -m tqhip.bench_kernels [--iters 200] [--cases encode,scores,flash,flash_long,sparse_v,sparse_v_grid,vonly,vonly_batch,vonly_lengths,widths,packed_widths,codec_widths,prefill,step]
"""
from __future__ import annotations

import argparse
import math

import numpy as np

import torch

import tqhip
from tqhip.quantizer import gaussian_boundaries, gaussian_codebook

PEAK = 8000.0


def timeit(fns, iters, warmup=10):
    """fns: list of zero-arg callables (one per input set), called round-robin."""
    for i in range(warmup):
        fns[i % len(fns)]()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        fns[i % len(fns)]()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def report(name, us, nbytes):
    gbs = nbytes / us / 1e3
    print(f"{name:58s} {us:10.2f} us  {gbs:8.1f} GB/s  {100 * gbs / PEAK:5.1f} % of 8 TB/s", flush=True)


def n_sets_for(nbytes):
    return max(2, min(16, int(math.ceil(420e6 / max(nbytes, 1)))))


def bench_encode(iters, dev):
    cb = gaussian_codebook(3)
    bd = gaussian_boundaries(cb)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    for n_vecs, label in ((4096, "config 1: 4096 vectors"), (131072 * 8, "config 5: 1 048 576 vectors")):
        nbytes = n_vecs * (256 + 56)
        xs = [torch.randn((n_vecs, 128), device=dev, dtype=torch.float16) for _ in range(n_sets_for(nbytes))]
        if "config 5" in label:
            for x in xs:
                x[:, 17] *= 20                          # 1 % outlier channels scaled x20
        fns = [(lambda x=x: tqhip.fused_quantize(x, signs, bd, 128, 3)) for x in xs]
        report(f"encode d=128 3-bit, {label}", timeit(fns, iters), nbytes)
        p, n = tqhip.fused_quantize(xs[0], signs, bd, 128, 3)
        fns = [(lambda: tqhip.dequant_fp16(p, n, cb, signs, 128, 3))]
        report(f"dequant_fp16 d=128 3-bit, {n_vecs} vectors (cache-warm)", timeit(fns, iters), n_vecs * (56 + 256))
        fns = [(lambda: tqhip.packed_dequantize(p, n, cb, signs, 128, 3))]
        report(f"packed_dequantize (float32 out), {n_vecs} vectors", timeit(fns, iters), n_vecs * (56 + 512))


def packed_sets(n_kv, T, dev, n_sets, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    sets = []
    for _ in range(n_sets):
        p = torch.randint(0, 2 ** 30, (n_kv, T, 13), generator=g, device=dev, dtype=torch.int32).view(torch.uint32)
        n = torch.rand((n_kv, T), generator=g, device=dev) + 0.1
        sets.append((p, n))
    return sets


def bench_scores(iters, dev):
    cb = gaussian_codebook(3)
    for T in (4096, 16384, 65536):
        nbytes = 224 * T + 112 * T + 14336
        sets = packed_sets(4, T, dev, n_sets_for(nbytes), 3)
        q_rot = torch.randn((28, 128), device=dev)
        for prec, label in ((None, "default (split operands, float32 fidelity)"), ("fp32", "float32 vector kernels"),
                            ("fp16", "fp16 operands")):
            fns = [(lambda p=p, n=n: tqhip.prerot_fused_qk_scores(q_rot, p, n, cb, 128, 3, n_rep=7, precision=prec))
                   for p, n in sets]
            report(f"config 3: prerot scores 28/4 heads, T={T}, {label}", timeit_graph(fns, iters), nbytes)


def bench_sparse_v(iters, dev):
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    for T in (8192, 32768):
        nbytes = 28 * T * 4 + 4 * T * 56 + 28 * 128 * 4
        sets = packed_sets(4, T, dev, n_sets_for(nbytes), 4)
        w = torch.softmax(torch.randn((28, T), device=dev) * 5, dim=-1)
        for thr, prec, label in ((0.0, None, "default (split operands)"), (1e-5, None, "default (split operands)"),
                                 (1e-5, "fp32", "float32 vector kernels"), (1e-5, "fp16", "fp16 operands")):
            fns = [(lambda p=p, n=n: tqhip.sparse_v_matvec(w, p, n, cb, signs, 128, 3, threshold=thr, n_rep=7,
                                                           precision=prec)) for p, n in sets]
            report(f"sparse_v_matvec 28/4 heads, T={T}, thr={thr:g}, {label}", timeit_graph(fns, iters), nbytes)


def bench_sparse_v_grid(iters, dev):
    """The reference's micro-benchmark grid (scripts/bench_sparse_v.py:148-171): dense (packed_dequantize, then
    weights x V) against sparse_v_matvec over sequence lengths x thresholds; 32 heads (MHA), d = 128, 3-bit,
    weights = softmax(5 * N(0,1)).  Same columns as the script's table: ms, speed-up over dense, active positions,
    cosine against dense.  HIP-graph replays (GPU time of the calls, no host gaps)."""
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    H = 32
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    print("| seq_len | dense us | thr | sparse_v us | speed-up | active % | cosine |")
    print("|---|---|---|---|---|---|---|")
    for S in (512, 2048, 8192, 16384):
        n_sets = n_sets_for(H * S * 56)
        sets = packed_sets(H, S, dev, n_sets, 100 + S)
        w = torch.softmax(torch.randn((H, S), generator=g, device=dev) * 5, dim=-1)

        def dense(p, n):
            v = tqhip.packed_dequantize(p.reshape(H * S, -1), n.reshape(-1), cb, signs, 128, 3).reshape(H, S, 128)
            return torch.einsum("hs,hsd->hd", w, v)
        d_us = timeit_graph([(lambda p=p, n=n: dense(p, n)) for p, n in sets], iters)
        d_out = dense(*sets[0])
        for thr in (0.0, 1e-5, 1e-4):
            fns = [(lambda p=p, n=n: tqhip.sparse_v_matvec(w, p, n, cb, signs, 128, 3, threshold=thr)) for p, n in sets]
            us = timeit_graph(fns, iters)
            out = tqhip.sparse_v_matvec(w, sets[0][0], sets[0][1], cb, signs, 128, 3, threshold=thr)
            cosine = float((out * d_out).sum() / (out.norm() * d_out.norm() + 1e-8))
            active = tqhip.count_active_positions(w, thr)
            print(f"| {S} | {d_us:.1f} | {thr:g} | {us:.1f} | {d_us / us:.2f}x | {100.0 * active / (H * S):.1f} | {cosine:.6f} |",
                  flush=True)


def bench_flash(iters, dev):
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    g = torch.Generator()
    g.manual_seed(4)
    lens = torch.randint(4096, 32769, (16,), generator=g)
    offs = torch.cat([torch.zeros(1, dtype=torch.int64), lens.cumsum(0)]).to(torch.int32).to(dev)
    total = int(lens.sum())
    nbytes = 896 * total + 262144
    k = packed_sets(8, total, dev, 2, 5)
    v = packed_sets(8, total, dev, 2, 6)
    q_rot = torch.randn((16, 32, 128), device=dev)
    fns = [(lambda i=i: tqhip.flash_decode(q_rot, k[i][0], k[i][1], v[i][0], v[i][1], cb, cb, signs, 128, 3,
                                           1 / math.sqrt(128), n_rep=4, seq_offsets=offs,
                                           max_seq_len=int(lens.max()), out_dtype=torch.float16)) for i in range(2)]
    report(f"config 4: flash decode 32/8 heads, 16 seqs, sum L={total}", timeit(fns, max(20, iters // 10)), nbytes)
    fns = [(lambda i=i: tqhip.flash_decode(q_rot, k[i][0], k[i][1], v[i][0], v[i][1], cb, cb, signs, 128, 3,
                                           1 / math.sqrt(128), n_rep=4, seq_offsets=offs,
                                           max_seq_len=int(lens.max()), out_dtype=torch.float16,
                                           sparse_v_threshold=1e-5)) for i in range(2)]
    report(f"config 4, threshold 1e-5: thresholded flash decode (scores, weights + values, merge), one call",
           timeit(fns, max(20, iters // 10)), nbytes)


def bench_flash_long(iters, dev):
    """Flash decode of ONE long sequence (cache layout), packed K and V: the streaming pass at its
    longest step count."""
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    for n_q, n_kv, T in ((32, 8, 32768), (32, 8, 131072), (28, 4, 131072)):
        nbytes = n_kv * T * 112 + 2 * n_q * 512
        n_sets = max(2, n_sets_for(nbytes))
        ks, vs = packed_sets(n_kv, T, dev, n_sets, 5), packed_sets(n_kv, T, dev, n_sets, 6)
        q_rot = torch.randn((1, n_q, 128), device=dev)
        fns = [(lambda i=i: tqhip.flash_decode(q_rot, ks[i][0], ks[i][1], vs[i][0], vs[i][1], cb, cb, signs, 128, 3,
                                               1 / math.sqrt(128), n_rep=n_q // n_kv, out_dtype=torch.float16))
               for i in range(n_sets)]
        report(f"flash decode, one sequence, {n_q}/{n_kv} heads, T={T}", timeit(fns, max(20, iters // 4)), nbytes)


def bench_vonly(iters, dev):
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    for T in (4096, 32768, 131072):
        nbytes = 4 * T * 312 + 28 * 256 * 2
        sets = packed_sets(4, T, dev, n_sets_for(nbytes), 7)
        ks = [torch.randn((4, T, 128), device=dev, dtype=torch.float16) for _ in sets]
        q = torch.randn((1, 28, 128), device=dev, dtype=torch.float16)
        fns = [(lambda k=k, p=p, n=n: tqhip.vonly_decode(q, k, p, n, cb, signs, 128, 3, 1 / math.sqrt(128), n_rep=7))
               for k, (p, n) in zip(ks, sets)]
        report(f"config 2 shape: V-only decode 28/4 heads, T={T} (python-call launch)", timeit(fns, iters), nbytes)
        if T == 32768:
            # sparse-V threshold 1e-5 on the final weights: one call (scores pass, weights-and-values pass, merge) ...
            fns = [(lambda k=k, p=p, n=n: tqhip.vonly_decode(q, k, p, n, cb, signs, 128, 3, 1 / math.sqrt(128), n_rep=7,
                                                             sparse_v_threshold=1e-5)) for k, (p, n) in zip(ks, sets)]
            report(f"config 2 shape, threshold 1e-5: thresholded V-only decode, T={T}, one call", timeit(fns, iters), nbytes)

            # ... against the composition of the three separate ops it replaces
            def composed(k, p, n):
                sc = tqhip.dense_qk_scores(q[0], k, 1.0, n_rep=7)
                w = tqhip.softmax_rows(sc, 1 / math.sqrt(128))
                return tqhip.sparse_v_matvec(w, p, n, cb, signs, 128, 3, threshold=1e-5, n_rep=7, precision="fp16")
            fns = [(lambda k=k, p=p, n=n: composed(k, p, n)) for k, (p, n) in zip(ks, sets)]
            report(f"config 2 shape, threshold 1e-5: dense scores + softmax + sparse-V as three ops, T={T}",
                   timeit(fns, iters), nbytes)


def timeit_graph(fns, iters):
    """Like timeit, but the calls are recorded once into a HIP graph (one round over the input sets) and the
    graph is replayed: kernel time without the cost of the Python calls."""
    for f in fns:
        f()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for f in fns:
            f()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for f in fns:
                f()
    reps = max(3, iters // len(fns))
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * len(fns))


def bench_vonly_lengths(iters, dev):
    """The decode step of configuration 2's heads (28 query / 4 kv, 3-bit values) over cache lengths from 4 096 to
    131 072 positions, multiples of the tile and not: which launch shape the host picks changes along the way (four- or
    eight-wave tiles, the streaming pass).  HIP-graph replay over 8 buffer sets, tile pass + merge pass."""
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    lengths = (4096, 8192, 16384, 20000, 30000, 32768, 32769, 40000, 49152, 50000, 65536, 65537, 100000, 131071, 131072)
    t_max = max(lengths) + 8
    sets = packed_sets(4, t_max, dev, 8, 7)
    ks = [torch.randn((1, 4, t_max, 128), device=dev, dtype=torch.float16) for _ in sets]
    q = torch.randn((1, 28, 128), device=dev, dtype=torch.float16)
    for T in lengths:
        fns = [(lambda k=k, p=p, n=n: tqhip.vonly_decode(q, k, p[None], n[None], cb, signs, 128, 3, 1 / math.sqrt(128),
                                                         n_rep=7, seq_len=T)) for k, (p, n) in zip(ks, sets)]
        report(f"V-only decode 28/4 heads, T={T} (graph)", timeit_graph(fns, max(iters, 160)), 4 * T * 312 + 28 * 256 * 2)


def bench_widths(iters, dev):
    """V-only decode at the other value widths (1, 2 and 4 bits): the matrix-core tile pass against the
    float32 kernels that served these widths before it (precision="fp32"), HIP-graph replay."""
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(8)
    for bits in (1, 2, 3, 4):
        cb = gaussian_codebook(bits)
        pd = tqhip.packed_dim(128, bits)
        for T in (32768, 131072):
            nbytes = 4 * T * (256 + 4 * pd + 4) + 28 * 256 * 2
            n_sets = n_sets_for(nbytes)
            ks = [torch.randn((4, T, 128), device=dev, dtype=torch.float16) for _ in range(n_sets)]
            codes = [torch.randint(0, 2 ** bits, (4 * T, 128), generator=g, device=dev, dtype=torch.uint8) for _ in range(n_sets)]
            ps = [tqhip.pack_indices(c, bits).reshape(4, T, pd) for c in codes]
            ns = [torch.rand((4, T), generator=g, device=dev) + 0.1 for _ in range(n_sets)]
            q = torch.randn((1, 28, 128), device=dev, dtype=torch.float16)
            for prec in ("fp16", "fp32"):
                fns = [(lambda k=k, p=p, n=n: tqhip.vonly_decode(q, k, p, n, cb, signs, 128, bits, 1 / math.sqrt(128),
                                                                 n_rep=7, precision=prec)) for k, p, n in zip(ks, ps, ns)]
                kind = "matrix cores" if prec == "fp16" else "float32 kernels"
                report(f"V-only decode 28/4 heads, {bits}-bit values, T={T}, {kind} (graph)", timeit_graph(fns, iters), nbytes)


def bench_vonly_batch(iters, dev):
    """V-only decode over batches (28/4 heads, 3-bit values, HIP-graph replay): cache layout with one length, and
    ragged batches (seq_offsets) with lengths drawn uniformly from a range, as a serving loop holds them."""
    cb = gaussian_codebook(3)
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    sc = 1 / math.sqrt(128)

    def make(shape):
        n = int(np.prod(shape))
        K = torch.randn(shape + (128,), device=dev, dtype=torch.float16)
        codes = torch.randint(0, 8, (n, 128), generator=g, device=dev, dtype=torch.uint8)
        return K, tqhip.pack_indices(codes, 3).reshape(*shape, 13), torch.rand(shape, generator=g, device=dev) + 0.5

    for n_seq, T in ((16, 8192), (16, 16384), (8, 32768), (64, 2048)):
        nbytes = n_seq * 4 * T * 312
        sets = [make((n_seq, 4, T)) for _ in range(n_sets_for(nbytes))]
        q = torch.randn((n_seq, 28, 128), device=dev, dtype=torch.float16)
        fns = [(lambda K=K, p=p, n=n: tqhip.vonly_decode(q, K, p, n, cb, signs, 128, 3, sc, n_rep=7, seq_len=T)) for K, p, n in sets]
        report(f"V-only decode 28/4 heads, {n_seq} sequences x {T} (graph)", timeit_graph(fns, iters), nbytes)
        del sets
    for seed, n_seq, lo, hi in ((4, 16, 4096, 32768), (5, 32, 1024, 8192), (6, 8, 16384, 65536), (7, 64, 256, 4096)):
        lens = np.random.default_rng(seed).integers(lo, hi + 1, size=n_seq)
        offs = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=dev)
        tot = int(lens.sum())
        nbytes = tot * 4 * 312
        sets = [make((4, tot)) for _ in range(n_sets_for(nbytes))]
        q = torch.randn((n_seq, 28, 128), device=dev, dtype=torch.float16)
        fns = [(lambda K=K, p=p, n=n: tqhip.vonly_decode(q, K, p, n, cb, signs, 128, 3, sc, n_rep=7, seq_offsets=offs,
                                                         max_seq_len=int(lens.max()))) for K, p, n in sets]
        report(f"V-only decode 28/4 heads, ragged batch of {n_seq}, L ~ U({lo}, {hi}), sum L={tot} (graph)",
               timeit_graph(fns, iters), nbytes)
        del sets


def bench_packed_widths(iters, dev):
    """The steps over PACKED keys at every width (32/8 heads): scores, flash decode (single sequence, HIP-graph
    replay) and a 512-row prefill chunk, matrix cores against the float32 kernels (none for prefill)."""
    ks_ = tqhip.random_diagonal_sign(128, 42, device=dev)
    vs_ = tqhip.random_diagonal_sign(128, 43, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    sc = 1 / math.sqrt(128)
    for bits in (1, 2, 3, 4):
        cb = gaussian_codebook(bits)
        pd = tqhip.packed_dim(128, bits)
        row = 4 * pd + 4
        for T in (32768, 131072):
            n_sets = n_sets_for(2 * 8 * T * row)

            def packed():
                codes = torch.randint(0, 2 ** bits, (8 * T, 128), generator=g, device=dev, dtype=torch.uint8)
                return tqhip.pack_indices(codes, bits).reshape(8, T, pd), torch.rand((8, T), generator=g, device=dev) + 0.5
            sets = [(packed(), packed()) for _ in range(n_sets)]
            q_rot = torch.randn((1, 32, 128), device=dev)
            for prec in ("fp16", "fp32"):
                kind = "matrix cores" if prec == "fp16" else "float32 kernels"
                fns = [(lambda k=k: tqhip.prerot_fused_qk_scores(q_rot[0], k[0], k[1], cb, 128, bits, n_rep=4, precision=prec))
                       for k, _ in sets]
                report(f"scores 32/8 heads, {bits}-bit keys, T={T}, {kind} (graph)", timeit_graph(fns, iters),
                       8 * T * row + 32 * T * 4)
                fns = [(lambda k=k, v=v: tqhip.flash_decode(q_rot, k[0][None], k[1][None], v[0][None], v[1][None], cb, cb, vs_,
                                                            128, bits, sc, n_rep=4, seq_len=T, precision=prec))
                       for k, v in sets]
                report(f"flash decode 32/8 heads, {bits}-bit, T={T}, {kind} (graph)", timeit_graph(fns, iters), 2 * 8 * T * row)
        T, n_rows = 32768, 512
        (kp, kn), (vp, vn) = sets[0][0], sets[0][1]
        kp, kn, vp, vn = kp[:, :T], kn[:, :T], vp[:, :T], vn[:, :T]
        q = torch.randn((32, n_rows, 128), device=dev, dtype=torch.float16)
        us = timeit([lambda: tqhip.prefill_attention(q, kp, kn, vp, vn, cb, cb, ks_, vs_, 128, bits, sc, n_rep=4)],
                    max(5, iters // 20), warmup=2)
        flops = 4.0 * 32 * 128 * sum(T - n_rows + i + 1 for i in range(n_rows))
        print(f"prefill chunk 512 rows x 32/8 heads, {bits}-bit, T={T:<7d} {us:10.1f} us  {flops / us / 1e6:8.1f} TFLOP/s  "
              f"{100 * flops / us / 1e6 / 2500:5.1f} % of 2.5 PFLOP/s", flush=True)


def bench_codec_widths(iters, dev):
    """Encode / dequantise 1 048 576 vectors at every width: the streaming kernels (row count a multiple of 16)
    against the generic one-wavefront-per-vector kernels (one row fewer)."""
    signs = tqhip.random_diagonal_sign(128, 43, device=dev)
    n = 131072 * 8
    xs = [torch.randn((n, 128), device=dev, dtype=torch.float16) for _ in range(2)]
    for bits in (1, 2, 3, 4):
        cb = gaussian_codebook(bits)
        bd = gaussian_boundaries(cb)
        pd = tqhip.packed_dim(128, bits)
        for rows, kind in ((n, "streaming kernel"), (n - 1, "generic kernel")):
            fns = [(lambda x=x: tqhip.fused_quantize(x[:rows], signs, bd, 128, bits)) for x in xs]
            report(f"encode d=128 {bits}-bit, {rows} vectors, {kind}", timeit(fns, max(10, iters // 4)), rows * (256 + 4 * pd + 4))
            p, nr = tqhip.fused_quantize(xs[0][:rows], signs, bd, 128, bits)
            fns = [(lambda: tqhip.dequant_fp16(p, nr, cb, signs, 128, bits))]
            report(f"dequant_fp16 d=128 {bits}-bit, {rows} vectors, {kind}", timeit(fns, max(10, iters // 4)), rows * (256 + 4 * pd + 4))


def bench_prefill(iters, dev):
    """benchmark configuration 5, attention half: a chunk of 512 query rows x 32 heads at the end of a
    131072-position packed cache (8 kv heads), causal.  Matrix-core bound: reported in TFLOP/s of
    the 4 * rows * heads * d * visible-positions useful flops against the 2.5 PFLOP/s fp16 peak."""
    cb = gaussian_codebook(3)
    ks = tqhip.random_diagonal_sign(128, 42, device=dev)
    vs = tqhip.random_diagonal_sign(128, 43, device=dev)
    n_rows = 512
    for T in (8192, 32768, 131072):
        (kp, kn), (vp, vn) = packed_sets(8, T, dev, 1, 8)[0], packed_sets(8, T, dev, 1, 9)[0]
        q = torch.randn((32, n_rows, 128), device=dev, dtype=torch.float16)
        visible = sum(T - n_rows + i + 1 for i in range(n_rows))
        flops = 4.0 * 32 * 128 * visible
        nbytes = 8 * T * 112 + 2 * 32 * n_rows * 256
        for flag, label in ((False, "value + remainder query (default)"), (True, "fp16_query=True")):
            fn = lambda: tqhip.prefill_attention(q, kp, kn, vp, vn, cb, cb, ks, vs, 128, 3, 1 / math.sqrt(128), n_rep=4,
                                                 fp16_query=flag)
            us = timeit([fn], max(5, iters // 20), warmup=2)
            print(f"config 5: prefill chunk 512 rows x 32/8 heads, T={T:<7d} {label}: {us:10.1f} us  "
                  f"{flops / us / 1e6:8.1f} TFLOP/s  {100 * flops / us / 1e6 / 2500:5.1f} % of 2.5 PFLOP/s  "
                  f"({nbytes / us / 1e3:6.1f} GB/s of packed cache)", flush=True)


def bench_step(iters, dev):
    """Wall time of a whole layer step (insert one token + attention) through the cache objects: the two calls
    of the reference's surface, the single library call, and 28 layers recorded in a HIP graph with the position
    in device memory.  Wall clock (perf_counter around a synchronised loop): host cost is the point."""
    import time
    D, L = 128, 28
    sc = 1 / math.sqrt(D)

    def wall(fn, n):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    n = max(20, iters // 2)
    for T in (4096, 30720):
        for kind, n_q, n_kv in (("V-only cache", 28, 4), ("packed cache", 32, 8)):
            mk = (lambda: tqhip.VOnlyTurboQuantCache(bits=3, fused=True)) if kind == "V-only cache" else \
                 (lambda: tqhip.TurboQuantKVCache(bits=3, fused=True))
            k0 = torch.randn((1, n_kv, T, D), device=dev, dtype=torch.float16)
            v0 = torch.randn((1, n_kv, T, D), device=dev, dtype=torch.float16)
            k1, v1 = torch.randn((1, n_kv, 1, D), device=dev, dtype=torch.float16), torch.randn((1, n_kv, 1, D), device=dev, dtype=torch.float16)
            q = torch.randn((1, n_q, 1, D), device=dev, dtype=torch.float16)
            c = mk()
            c.update_and_fetch(k0, v0)
            attend = tqhip.vonly_decode_attention if kind == "V-only cache" else \
                (lambda qq, cc, s: tqhip.turboquant_attention(qq, cc, s, fused=True))

            def two_calls():
                c.update_and_fetch(k1, v1)
                return attend(q, c, sc)
            us2 = wall(two_calls, n)
            c = mk()
            c.update_and_fetch(k0, v0)
            us1 = wall(lambda: c.decode_step(q, k1, v1, sc), n)
            print(f"layer step, {kind}, {n_q}/{n_kv} heads, T~{T}: update_and_fetch + attention {us2:6.1f} us wall, "
                  f"decode_step {us1:6.1f} us wall", flush=True)
            del c
        for kind, n_q, n_kv in (("V-only cache", 28, 4), ("packed cache", 32, 8), ("V-only cache, 4-bit values", 28, 4),
                                ("V-only cache, 2-bit values", 28, 4)):
            vb = 4 if "4-bit" in kind else 2 if "2-bit" in kind else 3
            mk = (lambda: tqhip.VOnlyTurboQuantCache(bits=vb, fused=True)) if kind.startswith("V-only cache") else \
                 (lambda: tqhip.TurboQuantKVCache(bits=3, fused=True))
            caches = [mk() for _ in range(L)]
            k0 = torch.randn((1, n_kv, T, D), device=dev, dtype=torch.float16)
            for c in caches:
                c.reserve(1, n_kv, T + 2048, D)
                c.update_and_fetch(k0, k0)
            k1 = torch.randn((1, n_kv, 1, D), device=dev, dtype=torch.float16)
            q = torch.randn((1, n_q, 1, D), device=dev, dtype=torch.float16)
            outs = [torch.empty((1, n_q, D), device=dev, dtype=torch.float16) for _ in range(L)]
            pos = torch.tensor([T], dtype=torch.int64, device=dev)

            def token():
                for i, c in enumerate(caches):
                    c.decode_step(q, k1, k1, sc, position=pos, out=outs[i])
                pos.add_(1)
            token()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                token()
            us = wall(g.replay, n) / L
            print(f"layer step, {kind}, {n_q}/{n_kv} heads, T~{T}: {L} layers recorded in a HIP graph, position in "
                  f"device memory: {us:6.1f} us per layer step", flush=True)
            del g, caches


CASES = {"vonly_lengths": bench_vonly_lengths, "step": bench_step, "prefill": bench_prefill, "encode": bench_encode, "scores": bench_scores, "sparse_v": bench_sparse_v, "flash": bench_flash,
         "flash_long": bench_flash_long, "vonly": bench_vonly, "widths": bench_widths, "codec_widths": bench_codec_widths,
         "packed_widths": bench_packed_widths, "vonly_batch": bench_vonly_batch, "sparse_v_grid": bench_sparse_v_grid}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=200)
    ap.add_argument("--cases", default=",".join(c for c in CASES if c != "step"),
                    help="comma-separated; `step` (wall time of whole layer steps) runs only when named")
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    for c in args.cases.split(","):
        CASES[c](args.iters, dev)


if __name__ == "__main__":
    main()
