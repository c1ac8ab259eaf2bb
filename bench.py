#!/usr/bin/env python3
"""Headline benchmark: V-only decode attention at the Qwen2.5-7B GQA shape, 32K context.

One step = one layer's decode attention: q[28,128] fp16 against fp16 K[4,32768,128] and 3-bit
packed V[4,32768,13]+norms[4,32768], dense softmax, out[28,128] -- the fused tq_vonly_decode_attn
entry point of libtqhip.so, called through the C ABI.  Inputs are resident in HBM before the timed
region; the steps rotate over N_SETS independent (q, K, V) sets totalling > 400 MB so that neither
the L2s nor the 256 MB Infinity Cache can serve the reads.  The K timed steps are captured once
into a HIP graph (back-to-back launches, no host gaps) and the graph is replayed until at least
MIN_TIMED_MS of GPU time has passed, with a HIP event on the launch stream after every MIN_SAMPLE_MS
worth of replays: `ms_per_step` is the MEDIAN sample divided by its steps (a single replay of 20
steps is a 0.3 ms sample, and an event record per replay would add 0.2 us to each of its steps),
the fastest and slowest sample are reported beside it.

Prints ONE JSON line (see the fields below).  `roofline.achieved` = algorithmic bytes per step
(40 908 800 B: q 7 168 + K 33 554 432 + V packed 6 815 744 + V norms 524 288 + out 7 168)
divided by the measured time per step.  `cpu_baseline` times the numpy oracle on the same
workload on this host's cores.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "turboquant-mlx_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

N_Q, N_KV, N_REP, D, BITS, T = 28, 4, 7, 128, 3, 32768
PDIM = 13
ALGO_BYTES = N_Q * D * 2 + N_KV * T * D * 2 + N_KV * T * PDIM * 4 + N_KV * T * 4 + N_Q * D * 2
HBM_PEAK_GBS = 8000.0
N_SETS = 10
MIN_TIMED_MS = 50.0       # GPU time every timed quantity is measured over (at least 5 replays)
MIN_SAMPLE_MS = 2.0      # GPU time between two event records of the timed region
READ_WGS = 2048           # workgroups of the plain-read probe (8 per CU)
THRESHOLD = 1e-5          # sparse-V threshold of the secondary figure: the reference's default (sparse_v.py:102)

# HBM bytes per launch of the dominant kernel (the tile pass), from two rocprofv3 --pmc runs of
# `python bench.py --steps 60 --warmup 6 --no-cpu --no-graph --no-ceiling` (FETCH_SIZE, then WRITE_SIZE), each
# scaled by what the same counter reads for `python bench.py --calibrate-copy --steps 40`, a plain
# copy of ALGO_BYTES bytes (FETCH_SIZE reads 19986.6 for 39950 KiB -> factor 1.9988; WRITE_SIZE
# reads 39950.0 -> factor 1.0000).  Tile pass: FETCH_SIZE 20071.2 -> 40119 KiB, WRITE_SIZE 916.0
# -> 916 KiB (run to run the fetch figure moves by a few KiB).  Summary: profiles/vonly_decode_c2_pmc_traffic.md.
MEASURED_TRAFFIC_BYTES = 42019784  # (20071.2 * 39950.0 / 19986.6 + 916.0) KiB, from the unrounded averages


def make_sets(torch, tqhip, dev):
    from tqhip.quantizer import gaussian_boundaries, gaussian_codebook
    cb = gaussian_codebook(BITS)
    bd = gaussian_boundaries(cb)
    signs = tqhip.random_diagonal_sign(D, 43, device=dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    sets = []
    for _ in range(N_SETS):
        q = torch.randn((1, N_Q, D), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
        k = torch.randn((N_KV, T, D), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
        v = torch.randn((N_KV * T, D), generator=gen, device=dev, dtype=torch.float32).to(torch.float16)
        vp, vn = tqhip.fused_quantize(v, signs, bd, D, BITS)
        del v
        sets.append((q, k, vp.reshape(N_KV, T, PDIM), vn.reshape(N_KV, T)))
    return sets, cb, signs


def cpu_baseline(torch, sets, cb, signs, budget_s=12.0):
    """The numpy oracle on set 0 at full size, timed on the host."""
    import numpy as np
    from oracle import polarquant_oracle as orc
    q, k, vp, vn = [t.cpu().numpy() for t in sets[0]]
    cbn, sg = cb.numpy(), signs.cpu().numpy()
    sc = 1.0 / math.sqrt(D)

    def run():
        return orc.vonly_decode_attention(q[0], k, vp, vn, cbn, sg, D, BITS, sc)
    ref = run()                       # warm-up, and the reference output for the check below
    ref_thr = orc.vonly_decode_attention(q[0], k, vp, vn, cbn, sg, D, BITS, sc, threshold=THRESHOLD)
    t0 = time.perf_counter()
    n = 0
    while True:
        run()
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 120:
            break
    per = el / n
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = 1
    return ref, ref_thr, {
        "value": round(ALGO_BYTES / per / 1e9, 3), "unit": "GB/s", "us_per_layer": round(per * 1e6, 1),
        "cores": threads, "kind": "port",
        "sample": f"{n} full-size steps (28/4 heads, d=128, T=32768) of the numpy oracle; its matmuls run "
                  f"on {threads} BLAS threads, unpack/gather/softmax on one (host reports {os.cpu_count()} cpus)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the plain-read probe (`read_ceiling` of the line)")
    ap.add_argument("--calibrate-read", action="store_true",
                    help="instead of the benchmark, time tq_probe_read: one launch that only streams the K / packed-V / "
                         "norm bytes of a step (and an empty launch), with the benchmark's rotation and launch pattern")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="instead of the benchmark, run --steps plain device copies of ALGO_BYTES bytes each "
                         "(known traffic: ALGO_BYTES read + ALGO_BYTES written) to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the hot path shards by kv head "
              "with no communication). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import tqhip
    from tqhip import _lib, ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        srcs = [torch.full((ALGO_BYTES,), i + 1, dtype=torch.uint8, device=dev) for i in range(N_SETS)]
        dst = torch.empty(ALGO_BYTES, dtype=torch.uint8, device=dev)
        for i in range(args.steps):
            dst.copy_(srcs[i % N_SETS])
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy": True, "copies": args.steps, "bytes_read_each": ALGO_BYTES,
                          "bytes_written_each": ALGO_BYTES}))
        return
    sets, cb, signs = make_sets(torch, tqhip, dev)
    sc = 1.0 / math.sqrt(D)
    lib = _lib.load()

    # Pre-bound C-ABI calls: one argument tuple per buffer set, so a step is a single ctypes call.
    outs = [torch.empty((1, N_Q, D), dtype=torch.float32, device=dev) for _ in range(N_SETS)]
    ws_bytes = lib.tq_workspace_bytes(_lib.TQ_OP_VONLY_DECODE, 1, N_Q, T, D)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    cb_host = _lib.host_floats(cb.tolist())
    shape = ops._decode_shape(n_seq=1, n_kv=N_KV, n_rep=N_REP, dim=D, bits=BITS, block_size=16, seq_len=T,
                              seq_offsets=None, k_strides=(0, T), kn_strides=(0, 0), v_strides=(0, T),
                              vn_strides=(0, T), mask=None, mask_strides=(0, 0), attn_scale=sc,
                              out_dtype=torch.float32)

    def bound(i, stream):
        q, k, vp, vn = sets[i]
        return (C.c_void_p(q.data_ptr()), _lib.TQ_F16, C.c_void_p(k.data_ptr()), C.c_void_p(vp.data_ptr()),
                C.c_void_p(vn.data_ptr()), cb_host, C.c_void_p(signs.data_ptr()), C.c_void_p(outs[i].data_ptr()),
                C.c_void_p(ws.data_ptr()), ws.numel(), C.byref(shape), C.c_void_p(stream))

    def step(i, argsets, phases=3, rot=N_SETS):
        a = argsets[i % rot]
        rc = lib.tq_vonly_decode_attn_phases(*a[:-1], phases, a[-1])
        if rc != 0:
            _lib.check(rc)

    # correctness of what is being timed: set 0 against the oracle
    cur = torch.cuda.current_stream(dev)
    eager_args = [bound(i, cur.cuda_stream) for i in range(N_SETS)]
    step(0, eager_args)
    torch.cuda.synchronize()
    checked = outs[0].clone()

    # secondary: the same step with the reference's default sparse-V threshold on the FINAL softmax weights
    # (tq_vonly_sparse_decode_attn: scores pass, weights + values pass, merge pass)
    thr_ws_bytes = lib.tq_vonly_sparse_workspace_bytes(1, N_Q, T)
    thr_ws = torch.zeros(thr_ws_bytes, dtype=torch.uint8, device=dev)
    thr_out = torch.empty((1, N_Q, D), dtype=torch.float32, device=dev)

    def thr_step(i, stream):
        q, k, vp, vn = sets[i % N_SETS]
        rc = lib.tq_vonly_sparse_decode_attn(
            C.c_void_p(q.data_ptr()), _lib.TQ_F16, C.c_void_p(k.data_ptr()), C.c_void_p(vp.data_ptr()),
            C.c_void_p(vn.data_ptr()), cb_host, C.c_void_p(signs.data_ptr()), C.c_float(THRESHOLD),
            C.c_void_p(thr_out.data_ptr()), C.c_void_p(thr_ws.data_ptr()), thr_ws.numel(), C.byref(shape),
            C.c_void_p(stream))
        if rc != 0:
            _lib.check(rc)
    thr_step(0, cur.cuda_stream)
    torch.cuda.synchronize()
    thr_checked = thr_out.clone()
    cpu = None
    if not args.no_cpu and not args.calibrate_read:
        ref, ref_thr, cpu = cpu_baseline(torch, sets, cb, signs)
        err = np.abs(outs[0][0].cpu().numpy() - ref)
        if not np.all(err <= 1e-3 + 2e-3 * np.abs(ref)):
            print(f"bench: GPU output disagrees with the oracle (max err {err.max():.3e})", file=sys.stderr)
            sys.exit(1)
        err = np.abs(thr_checked[0].cpu().numpy() - ref_thr)
        if not np.all(err <= 1e-3 + 2e-3 * np.abs(ref_thr)):
            print(f"bench: thresholded GPU output disagrees with the oracle (max err {err.max():.3e})", file=sys.stderr)
            sys.exit(1)

    side = torch.cuda.Stream(device=dev)

    def timed(one_step):
        """(median, min, max, replays): ms per step of `one_step(i, stream)` over samples of replays of a HIP graph of
        `args.steps` back-to-back steps (eager launches once with --no-graph), HIP events on the launch stream."""
        with torch.cuda.stream(side):
            for i in range(args.warmup):
                one_step(i, side.cuda_stream)
            side.synchronize()
            if args.no_graph:
                ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                ev0.record(side)
                for i in range(args.steps):
                    one_step(i, side.cuda_stream)
                ev1.record(side)
                side.synchronize()
                per = ev0.elapsed_time(ev1) / args.steps
                return per, per, per, 1
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                g_stream = torch.cuda.current_stream(dev).cuda_stream
                for i in range(args.steps):
                    one_step(i, g_stream)
            graph.replay()                      # untimed: instantiation, page-in
            side.synchronize()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
            ev[0].record(side)
            graph.replay()
            ev[1].record(side)
            side.synchronize()
            est = max(ev[0].elapsed_time(ev[1]), 1e-3)
            # a sample = `per_sample` replays between two event records (at least MIN_SAMPLE_MS of GPU time, so that
            # the records themselves, a few microseconds each, do not show in a short graph's figure)
            per_sample = int(max(1, math.ceil(MIN_SAMPLE_MS / est)))
            n_rep = int(min(max(5, math.ceil(MIN_TIMED_MS / (est * per_sample))), 4000))
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep + 1)]
            ev[0].record(side)
            for r in range(n_rep):
                for _ in range(per_sample):
                    graph.replay()
                ev[r + 1].record(side)
            side.synchronize()
        torch.cuda.synchronize()
        per = sorted(ev[r].elapsed_time(ev[r + 1]) / (args.steps * per_sample) for r in range(n_rep))
        return per[n_rep // 2], per[0], per[-1], n_rep * per_sample

    arg_cache = {}

    def decode_step(phases, rot=N_SETS):
        def one(i, stream):
            if stream not in arg_cache:
                arg_cache[stream] = [bound(j, stream) for j in range(N_SETS)]
            step(i, arg_cache[stream], phases, rot)
        return one

    def read_ceiling():
        """One launch that only streams the K, packed-V and norm bytes of a step (tq_probe_read, rotating over
        copies of the buffer sets), the same with the launch shape of the tile pass (256 workgroups) with and
        without a 3.5 KB store per workgroup at the end, and an empty launch -- all timed like the decode step."""
        part = N_REP * (D + 2) * 4 // 16 * 16               # bytes of one workgroup's partial result
        sink = torch.zeros(16 + READ_WGS * part, dtype=torch.uint8, device=dev)
        srcs = [torch.cat([k.reshape(-1).view(torch.uint8), vp.reshape(-1).view(torch.uint8),
                           vn.reshape(-1).view(torch.uint8)]) for (_, k, vp, vn) in sets]
        nbytes = srcs[0].numel() // 16 * 16

        def read_step(nb, wgs=READ_WGS, store=0):
            def one(i, stream):
                rc = lib.tq_probe_read(C.c_void_p(srcs[i % N_SETS].data_ptr()), nb, C.c_void_p(sink.data_ptr()),
                                       wgs, store, C.c_void_p(stream))
                if rc != 0:
                    _lib.check(rc)
            return one
        r_med, r_min, r_max, r_n = timed(read_step(nbytes))
        t_med = timed(read_step(nbytes, 256))[0]
        s_med = timed(read_step(nbytes, 256, part))[0]
        e_med, e_min, e_max, _ = timed(read_step(0))
        return {
            "bytes_per_launch": nbytes, "workgroups": READ_WGS,
            "us_per_launch": round(r_med * 1e3, 3), "min": round(r_min * 1e3, 3), "max": round(r_max * 1e3, 3),
            "replays": r_n, "GB/s": round(nbytes / (r_med * 1e-3) / 1e9, 1),
            "frac_of_peak": round(nbytes / (r_med * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "us_256_workgroups": round(t_med * 1e3, 3),
            "us_256_workgroups_storing_a_partial_each": round(s_med * 1e3, 3), "partial_bytes": part,
            "empty_launch_us": round(e_med * 1e3, 3), "empty_launch_min": round(e_min * 1e3, 3),
            "empty_launch_max": round(e_max * 1e3, 3),
            "note": "one launch that only reads the K, packed-V and norm bytes of a step (rotating buffer sets, the "
                    "benchmark's launch pattern): the practical ceiling for a launch of this size on this box; the "
                    "256-workgroup figures use the grid of the tile pass, the second one ends every workgroup with "
                    "the store of a partial result"}

    if args.calibrate_read:
        print(json.dumps({"calibrate_read": True, "buffer_sets": N_SETS, "steps": args.steps, "warmup": args.warmup,
                          "launch": "eager" if args.no_graph else "hipgraph", "read": read_ceiling()}))
        return

    mode = "eager" if args.no_graph else "hipgraph"
    ms_per_step, ms_min, ms_max, n_replays = timed(decode_step(3))    # whole step: tile pass + merge pass
    ms_tile, tile_min, tile_max, _ = timed(decode_step(1))            # dominant kernel alone, same launch pattern
    ms_warm = timed(decode_step(3, rot=1))[0]   # one buffer set over and over: its 41 MB stay in the 256 MB Infinity Cache
    ms_thr, thr_min, thr_max, _ = timed(thr_step)
    gbs = ALGO_BYTES / (ms_per_step * 1e-3) / 1e9
    gbs_tile = ALGO_BYTES / (ms_tile * 1e-3) / 1e9
    ceiling = None if args.no_ceiling else read_ceiling()
    if ceiling is not None:
        ceiling["frac_of_step"] = round(ceiling["us_per_launch"] / (ms_per_step * 1e3), 4)
    thr_step(0, cur.cuda_stream)
    torch.cuda.synchronize()
    if not torch.equal(thr_out, thr_checked):
        print("bench: the timed thresholded steps left a result that differs from the checked one", file=sys.stderr)
        sys.exit(1)
    step(0, eager_args)                         # leave outs[0] = the full result of set 0
    torch.cuda.synchronize()

    # the timed steps must have produced the same result as the checked eager step
    if not torch.equal(outs[0], checked):
        print("bench: the timed steps left a result that differs from the checked one", file=sys.stderr)
        sys.exit(1)

    line = {
        "metric": "sparse-V decode attn us/layer & HBM GB/s (% peak), 7B GQA shape, 32K ctx",
        "value": round(gbs, 1), "unit": "GB/s",
        "us_per_layer": round(ms_per_step * 1e3, 3), "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 in, f32 accumulate",
        "data": "synthetic (seeded N(0,1) fp16 q/K; V = 3-bit PolarQuant of seeded N(0,1) fp16)",
        "config": {"workload": "config 2: V-only decode attention, 28 q / 4 kv heads (n_rep 7), d=128, "
                               "batch 1, 1 query token, 32768 cached positions, dense softmax (threshold 0)",
                   "launch": mode, "buffer_sets": N_SETS, "algorithmic_bytes_per_step": ALGO_BYTES},
        "roofline": {"bound": "hbm", "achieved": round(gbs_tile, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs_tile / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": "tqm::vonly_tile_mfma_kernel", "us_per_launch": round(ms_tile * 1e3, 3),
                     "note": "algorithmic bytes / event-timed launch period of the tile pass alone; "
                             "`value` covers the whole step (tile pass + merge pass)"},
        "cpu_baseline": cpu,
        "read_ceiling": ceiling,
        "timing": {"method": "median over samples of back-to-back HIP-graph replays of `steps` steps each (>= %g ms of GPU "
                             "time per sample, >= %d ms in all)" % (MIN_SAMPLE_MS, int(MIN_TIMED_MS))
                   if not args.no_graph else "one pass of eager launches",
                   "replays": n_replays, "us_per_layer_min": round(ms_min * 1e3, 3), "us_per_layer_max": round(ms_max * 1e3, 3),
                   "tile_us_min": round(tile_min * 1e3, 3), "tile_us_max": round(tile_max * 1e3, 3)},
        "threshold_1e-5": {"us_per_layer": round(ms_thr * 1e3, 3), "min": round(thr_min * 1e3, 3), "max": round(thr_max * 1e3, 3),
                           "value": round(ALGO_BYTES / (ms_thr * 1e-3) / 1e9, 1), "unit": "GB/s",
                           "pct_hbm_peak": round(100 * ALGO_BYTES / (ms_thr * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
                           "note": "the same step with the reference's default sparse-V threshold (sparse_v.py:102) applied to "
                                   "the final softmax weights: tq_vonly_sparse_decode_attn (scores pass, weights + values "
                                   "pass, merge pass), timed like `value`, checked against the oracle; algorithmic bytes as for "
                                   "the dense step (the scores written and re-read between the passes are not counted)"},
        "warm_cache": {"us_per_layer": round(ms_warm * 1e3, 3), "value": round(ALGO_BYTES / (ms_warm * 1e-3) / 1e9, 1),
                       "unit": "GB/s", "note": "same step on ONE buffer set (inputs served from the Infinity Cache); "
                                               "reported beside `value`, never as it"},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
