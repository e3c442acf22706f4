#!/usr/bin/env python3
"""Search-throughput benchmark of the HIP path: queries/s and achieved HBM GB/s.

Workload (the headline metric): TurboQuantIndex 10,000,000 x 1536, 4-bit,
k=10, no filter.  One step = one batch search (default 1024 queries) over the
whole index, with the index, the queries and the result buffers already
resident in HBM when the timed region starts.  A batch-1 figure is measured in
the same run and reported beside it.  The index is synthetic: L2-normalised
i.i.d. Gaussian rows (seed 0) generated on the device and encoded there by the
library's own ingest kernel, in 100k-row chunks.

Prints ONE JSON line.  `roofline` prices the dominant kernel (the code scan) by
its mean launch duration, measured with HIP events on the library's own stream
inside the timed region.  A 1024-query chunk of this workload is one launch of
the wide permute-dot kernel, which reads the codes once for all 1024 queries and
is bound by the matrix unit: algorithmic operations per launch = 2 * queries *
vectors * dim int8 multiply-adds (reported in the TFLOP/s field; they are
integer operations, peak 5.0 POP/s dense).  The HBM side of the same launch is
reported beside it under `hbm`; the batch-1 scan is HBM-bound and carries its
own figures under `batch1`.  Algorithmic bytes per launch = codes + per-vector
scales.  `cpu_baseline` times the CPU oracle (a C port
of the reference's search, not the reference binary) on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


# HBM bytes one launch of the dominant kernel moves (reads + writes), from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this same command, each scaled by the copy-probe factor (see profiles/).
MEASURED_TRAFFIC = {
    ("k_scan_p4_wide", 10_000_000, 1536, 4): 7.7826e9,    # 3,775,910 x 2 KiB fetched + 48,384 KiB written
    ("k_scan_p4_multi", 10_000_000, 1536, 4): 7.7359e9,   # 3,775,570 x 2 KiB fetched + 3,451 KiB written
    ("k_scan_p4", 10_000_000, 1536, 4): 7.7208e9,         # 3,769,800 x 2 KiB fetched + 265 KiB written
    ("k_scan_lut_bt", 10_000_000, 1536, 2): 3.8802e9,     # 1,894,650 x 2 KiB fetched
    ("k_scan_lut16", 10_000_000, 1536, 2): 3.8830e9,      # 1,895,400 x 2 KiB fetched + 1,189 KiB written
    ("k_scan_lut", 10_000_000, 1536, 2): 3.8809e9,        # 1,894,970 x 2 KiB fetched
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--n", type=int, default=10_000_000)
    ap.add_argument("--dim", type=int, default=1536)
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--k", type=int, default=10)
    ap.add_argument("--batch", type=int, default=1024)
    ap.add_argument("--score-mode", choices=["auto", "lut"], default="auto",
                    help="auto = what the reference runs on a VNNI/dotprod host (int8 permute-dot at 4-bit); "
                         "lut = the classic u8-LUT kernel's floats")
    ap.add_argument("--tile-groups", action="store_true",
                    help="keep large batches on the tile-group kernel (96 queries per pass over the codes) "
                         "instead of the all-queries-per-pass one")
    ap.add_argument("--cpu-sample", type=int, default=2_000_000, help="vectors in the CPU-baseline sample (0 = skip)")
    ap.add_argument("--cpu-threads", type=int, default=16)
    ap.add_argument("--no-config3", action="store_true",
                    help="skip the extra keys: configuration 3 (10M x 1536 2-bit, k=100, batches 1 and 1024) and the "
                         "adversarial insertion orders")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run the plain copy kernel over a 4 GiB buffer (counter calibration) and exit")
    return ap.parse_args()


def cpu_baseline(args):
    """The reference's search restated in C (oracle/), timed on the host cores: where the host has
    AVX-512 VNNI, the reference's own production kernel for 4-bit (vpshufb + vpdpbusd over the
    vector-major layout, eight queries per pass, the reference's tiling); otherwise, and for other
    bit widths, the portable loop.  On a bounded sample of the workload, scaled to the full index."""
    import numpy as np
    from oracle import oracle as O
    n_s, dim, bits = args.cpu_sample, args.dim, args.bits
    threads = max(1, min(args.cpu_threads, os.cpu_count() or 1))
    vnni = bits == 4 and O.have_vnni() and (dim // 2) % 4 == 0

    def make_index(n_rows, seed):
        rng = np.random.default_rng(seed)
        rot = O.Rotation(dim)
        packed_parts, scale_parts = [], []
        for c0 in range(0, n_rows, 100_000):          # encode in 100k-row pieces to bound host memory
            v = rng.standard_normal((min(100_000, n_rows - c0), dim), dtype=np.float32)
            v /= np.linalg.norm(v, axis=1, keepdims=True)
            p, s = O.encode(rot, v, bits)
            packed_parts.append(p)
            scale_parts.append(s)
        packed, scales = np.concatenate(packed_parts), np.concatenate(scale_parts)
        seq = O.repack_seq(packed, n_rows, bits, dim)
        codes = O.seq_to_vector_major(seq, n_rows, bits, dim) if vnni else seq     # the layout kept at rest
        return rng, rot, codes, scales

    def search(rot, codes, scales, q, k, n_rows):
        if vnni:
            return O.search_vnni(rot, codes, scales, q, k, dim, n_rows, n_threads=threads)
        return O.search_fast(rot, codes, scales, q, k, bits, dim, n_rows, n_threads=threads)

    rng, rot, codes, scales = make_index(n_s, 0)
    q = rng.standard_normal((args.batch, dim), dtype=np.float32)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    search(rot, codes, scales, q[:8], args.k, n_s)   # warm
    ts = []
    for _ in range(5):
        t0 = time.perf_counter()
        search(rot, codes, scales, q, args.k, n_s)
        ts.append(time.perf_counter() - t0)
    dt = float(np.median(ts))
    pairs_per_s = args.batch * n_s / dt
    what = ("C restatement of the reference's AVX-512 VNNI permute-dot kernel and tiling (search.rs:1392-1567)"
            if vnni else "portable C loop over the reference's arithmetic (host without AVX-512 VNNI)"
            if bits == 4 else "portable C loop over the reference's u8-LUT arithmetic")
    out = {
        "value": pairs_per_s / args.n,     # queries/s this rate sustains over the full index
        "unit": "queries/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{args.batch} queries x {n_s} of {args.n} vectors ({dim}-dim, {bits}-bit, k={args.k}), "
                  f"median of 5 runs {dt:.2f} s, scaled by {n_s}/{args.n}; {what}, not the reference binary",
    }
    del codes, scales
    if vnni and dim == 1536:
        # The cell the reference publishes (README speed table, benchmarks/results/
        # speed_d1536_4bit_x86_mt.json: 0.185 ms per query on an 8-vCPU Sapphire Rapids VM):
        # 100K vectors, 1000 queries, k=64, one warm-up query, median of 5.
        rng, rot, codes, scales = make_index(100_000, 0)
        q = rng.standard_normal((1000, dim), dtype=np.float32)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
        search(rot, codes, scales, q[:1], 64, 100_000)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            search(rot, codes, scales, q, 64, 100_000)
            ts.append(time.perf_counter() - t0)
        out["reference_cell"] = {
            "workload": "100000 x 1536 4-bit, 1000 queries, k=64 (synthetic unit Gaussian rows)",
            "ms_per_query": float(np.median(ts)) / 1000 * 1e3, "cores": threads,
            "published_ms_per_query": 0.185, "published_on": "8 vCPU Xeon Platinum 8481C (c3-standard-8), "
            "OpenAI DBpedia embeddings"}
    return out


def config3_extra(T, torch, build_index, run, args):
    """Configuration 3 beside the headline: 10M x 1536 2-bit, k=100 (u8 LUT, u32 epilogue), batches 1
    and 1024, each with the HBM roofline of its scan launch (algorithmic bytes = codes + row scales)."""
    n, dim, bits, k = 10_000_000, 1536, 2, 100
    ix = build_index(dim, bits, n)
    alg = ((n + 31) // 32) * (dim // 4) * 32 + 4 * n
    res = {"workload": f"TurboQuantIndex {n}x{dim} {bits}-bit, k={k}, no filter", "dtype": "u8",
           "algorithmic_bytes_per_launch": alg}
    for nq, steps in ((1024, max(3, args.steps // 2)), (1, max(args.steps, 15))):
        dt, scan_ms, launches, q_full = run(nq, steps, 1, ix=ix, k=k, dim=dim)
        launch_s = scan_ms * 1e-3 / max(launches, 1)
        # byte tables serve single queries; sixteen queries per pass stream their tables through LDS
        kern = "k_scan_lut_bt" if q_full == 1 else "k_scan_lut16" if q_full > 8 else "k_scan_lut"
        res[f"batch{nq}"] = {"queries_per_s": nq * steps / dt, "ms_per_step": dt / steps * 1e3,
                             "queries_per_launch": q_full, "scan_launch_ms": launch_s * 1e3,
                             "roofline": {"bound": "hbm", "achieved": alg / launch_s / 1e9, "peak": 8000.0,
                                          "unit": "GB/s", "frac": alg / launch_s / 1e9 / 8000.0,
                                          "traffic": MEASURED_TRAFFIC.get((kern, n, dim, bits)), "kernel": kern}}
    res["overflow_redos"] = ix.overflow_redos()
    ix.close()
    return res


def adversarial_extra(T, torch, run, args, normal_ms, ladder):
    """What the candidate-overflow handling costs at full size (10M x 1536 4-bit, k=10, 1024 queries) on
    insertion orders chosen against it.  (1) a 1000-cluster mixture inserted cluster by cluster,
    queries next to database rows: every query has thousands of near neighbours in a few hundred
    consecutive blocks.  (2) an index laid out against the sampler itself, with the strides the
    library reports for this search (tv_debug_sampling_plan): every block any sampling level of the
    first pass reads holds rows pointing away from the queries, every other block rows pointing
    towards them, so the full scan starts from a floor far too low, every query overflows, and the
    batch is scanned again from raised floors (ladder shifted half a stride).  (3) the same with only
    the first level's blocks poisoned: the second level then lets everything through, overflows, and
    is repeated on the device from the floor taken from what fitted; the full scan runs once."""
    dev = torch.device("cuda:0")
    n, dim, k, nq = 10_000_000, 1536, 10, 1024
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    strides, offsets = ladder
    out = {"normal_ms_per_step": normal_ms, "ladder_block_strides": [int(x) for x in strides],
           "repeated_pass_block_offsets": [int(x) for x in offsets]}

    def timed(ix, q, steps=4):
        torch.cuda.synchronize()
        os_ = torch.empty(nq, k, device=dev)
        oi = torch.empty(nq, k, dtype=torch.int64, device=dev)
        ix.level_repeats(track=1)
        t1 = time.perf_counter()
        ix.search_dev(q.data_ptr(), nq, k, os_.data_ptr(), oi.data_ptr())
        first_ms, first_redos = (time.perf_counter() - t1) * 1e3, ix.overflow_redos()
        r0, e0, l0 = ix.overflow_redos(), ix.exact_redos(), ix.level_repeats()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        each = []
        for _ in range(steps):
            t1 = time.perf_counter()
            ix.search_dev(q.data_ptr(), nq, k, os_.data_ptr(), oi.data_ptr())   # returns with its results complete
            each.append(round((time.perf_counter() - t1) * 1e3, 3))
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / steps * 1e3
        # (the library changes ladders when one fails for many queries, so the steps need not cost the same)
        return {"ms_per_step": ms, "vs_normal": ms / normal_ms, "ms_each_step": each,
                # the index's first search on this layout (untimed above; it also pays first-use set-up):
                # where a ladder fails for the first time and the library switches
                "first_search_ms": round(first_ms, 3), "first_search_queries_repeated": first_redos,
                "queries_repeated_per_step": (ix.overflow_redos() - r0) / steps,
                "queries_on_exact_path_per_step": (ix.exact_redos() - e0) / steps,
                "sampling_levels_repeated_per_step": (ix.level_repeats() - l0) / steps}

    # (1) clustered, cluster by cluster
    centres = torch.randn(1000, dim, device=dev, generator=gen)
    ix = T.NativeIndex(dim, 4)
    keep = None
    for c0 in range(0, n, 100_000):
        cid = torch.arange(c0, c0 + 100_000, device=dev) // 10_000
        v = centres[cid] + 0.3 * torch.randn(100_000, dim, device=dev, generator=gen)
        v = (v / v.norm(dim=1, keepdim=True)).contiguous()
        if keep is None:
            keep = v[:: 100_000 // nq][:nq].clone()
        torch.cuda.synchronize()
        ix.add_dev(v.data_ptr(), v.shape[0])
    q = keep + 0.05 * torch.randn(nq, dim, device=dev, generator=gen) / dim ** 0.5
    q = (q / q.norm(dim=1, keepdim=True)).contiguous()
    out["clustered_inserted_cluster_by_cluster"] = timed(ix, q)
    ix.close()
    del ix, v, centres
    torch.cuda.empty_cache()

    # (2), (3) against the sampler
    u = torch.randn(dim, device=dev, generator=gen)
    u = u / u.norm()
    q = u + 0.5 * torch.randn(nq, dim, device=dev, generator=gen) / dim ** 0.5
    q = (q / q.norm(dim=1, keepdim=True)).contiguous()
    layouts = [("every_sampling_level_poisoned", strides[:-1])]
    if len(strides) > 2:      # with one sampling level only, the two layouts are the same
        layouts.append(("first_sampling_level_poisoned", strides[:1]))
    for key, poisoned in layouts:
        ix = T.NativeIndex(dim, 4)
        for c0 in range(0, n, 100_000):
            blocks = torch.arange(c0, c0 + 100_000, device=dev) // 32
            sampled = torch.zeros_like(blocks, dtype=torch.bool)
            for st in poisoned:
                sampled |= blocks % int(st) == 0
            sign = torch.where(sampled, -1.0, 1.0).unsqueeze(1)
            v = sign * 0.3 * u + torch.randn(100_000, dim, device=dev, generator=gen) / dim ** 0.5
            v = (v / v.norm(dim=1, keepdim=True)).contiguous()
            torch.cuda.synchronize()
            ix.add_dev(v.data_ptr(), v.shape[0])
        assert [int(x) for x in ix.sampling_plan(nq, k)[0]] == [int(x) for x in strides], "laid out against another ladder"
        out[key] = timed(ix, q)
        ix.close()
        del ix, v
        torch.cuda.empty_cache()
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path, so --gpus {args.gpus} is not run "
              f"(value would be the single GPU's throughput).", file=sys.stderr)
        sys.exit(2)
    import torch
    from turbovec_amd import _lib as T

    dev = torch.device("cuda:0")
    if args.copy_probe:
        nbytes = 4 << 30
        src = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        dst = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        ix = T.NativeIndex(64, 4)
        ms = ix.stream_probe(src.data_ptr(), dst.data_ptr(), nbytes, reps=3)
        print(json.dumps({"copy_probe_bytes_read": nbytes, "copy_probe_bytes_written": nbytes, "ms": ms,
                          "GBps_read_plus_write": 2 * nbytes / (ms * 1e-3) / 1e9}))
        return
    n, dim, bits, k = args.n, args.dim, args.bits, args.k
    G = dim // (8 // bits)
    n_blocks = (n + 31) // 32
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)

    def build_index(dim, bits, n):
        # 100k-row chunks of unit Gaussian rows, generated and encoded on the device (tv_index_add_dev)
        ix = T.NativeIndex(dim, bits)
        for c0 in range(0, n, 100_000):
            v = torch.randn(min(100_000, n - c0), dim, device=dev, generator=gen)
            v = (v / v.norm(dim=1, keepdim=True)).contiguous()
            torch.cuda.synchronize()
            ix.add_dev(v.data_ptr(), v.shape[0])
        del v
        torch.cuda.empty_cache()
        return ix

    ix = build_index(dim, bits, n)
    if args.tile_groups:
        ix.set_path(4)
    if args.score_mode == "lut":
        ix.set_score_mode(T.SCORE_L_CLASSIC)
    mode_p = bits == 4 and args.score_mode == "auto"

    def make_queries(nq, dim=dim):
        q = torch.randn(nq, dim, device=dev, generator=gen)
        return q / q.norm(dim=1, keepdim=True)

    def run(nq, steps, warmup, ix=ix, k=k, dim=dim):
        q = make_queries(nq, dim)
        # the library works on its own stream: buffers handed to a _dev entry point must be complete
        torch.cuda.synchronize()
        out_s = torch.empty(nq, k, device=dev)
        out_i = torch.empty(nq, k, dtype=torch.int64, device=dev)
        for _ in range(warmup):
            ix.search_dev(q.data_ptr(), nq, k, out_s.data_ptr(), out_i.data_ptr())
        torch.cuda.synchronize()
        scan_ms, launches = 0.0, 0
        t0 = time.perf_counter()
        for _ in range(steps):
            ix.search_dev(q.data_ptr(), nq, k, out_s.data_ptr(), out_i.data_ptr())
            ms, nl = ix.last_scan_ms()
            scan_ms += ms
            launches += nl
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        return dt, scan_ms, launches, ix.queries_per_launch()

    ladder = ix.sampling_plan(args.batch, k)       # block strides of the sampling levels of a batch search here
    alg_bytes = n_blocks * G * 32 + 4 * n          # codes + per-vector scales, one pass
    d_codes, _, code_bytes = ix.device_ptrs()
    read_ms = ix.stream_probe(d_codes, None, code_bytes, reps=5)   # pure read of the same buffer
    read_probe = code_bytes / (read_ms * 1e-3) / 1e9
    mfma_probe = ix.mfma_probe(iters=2000, reps=3) / 1e12 if mode_p else None   # TOP/s of the bare MFMA loop
    dt, scan_ms, launches, q_full = run(args.batch, args.steps, args.warmup)
    # a step is ceil(batch / q_full) full-scan launches; the last may serve fewer queries
    q_per_launch = args.batch / max(1, -(-args.batch // max(q_full, 1)))
    value = args.batch * args.steps / dt
    launch_s = scan_ms * 1e-3 / max(launches, 1)
    achieved = alg_bytes / launch_s / 1e9
    dt1, scan1_ms, launches1, _ = run(1, max(args.steps, 15), args.warmup)
    b1_steps = max(args.steps, 15)
    b1_launch_s = scan1_ms * 1e-3 / max(launches1, 1)
    # configuration 2's middle batch: 64 queries are one pass of the tile-group kernel
    dt64, scan64_ms, launches64, q64_full = run(64, max(args.steps, 10), args.warmup)
    b64_steps = max(args.steps, 10)
    b64_launch_s = scan64_ms * 1e-3 / max(launches64, 1)

    # End-to-end rate when the boundary hands over host buffers (queries up, results down over PCIe).
    import numpy as np
    # Protocol of the reference's own cell harness: warm-up, then the median of >= 5 (batch) and
    # >= 15 (single query) timed calls, each including the copies.
    def median_host_call(qh, reps):
        ix.search(qh, k)
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            ix.search(qh, k)
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    q_host = make_queries(args.batch).cpu().numpy()
    host_batch_s = median_host_call(q_host, 5)
    host_single_s = median_host_call(q_host[:1], 15)
    host_qps = args.batch / host_batch_s
    # one call of four chunks (the reference's Python sends 4096-row calls): the chunks are enqueued
    # back to back and their overflow flags read once
    q_host4 = make_queries(4 * args.batch).cpu().numpy()
    host_batch4_s = median_host_call(q_host4, 5)
    del q_host4

    # Eight caller threads, one query per call (the reference's search is &self and scales with
    # caller threads): calls that arrive while the index is busy are merged into the next launch.
    import threading
    def threads_single(n_threads, calls):
        qs = [q_host[t:t + 1].copy() for t in range(n_threads)]
        m0 = ix.merged_calls()
        def work(t):
            for _ in range(calls):
                ix.search(qs[t], k)
        ths = [threading.Thread(target=work, args=(t,)) for t in range(n_threads)]
        t0 = time.perf_counter()
        for th in ths:
            th.start()
        for th in ths:
            th.join()
        dt_t = time.perf_counter() - t0
        return n_threads * calls / dt_t, (ix.merged_calls() - m0) / (n_threads * calls)
    threads_single(8, 3)
    t8_qps, t8_merged = threads_single(8, 40)

    if mode_p:
        kernel = "k_scan_p4_wide" if q_full >= 256 else "k_scan_p4_multi" if q_full > 32 else "k_scan_p4"
    else:
        kernel = "k_scan_lut_bt" if q_full == 1 else "k_scan_lut16" if q_full > 8 else "k_scan_lut"
    traffic = MEASURED_TRAFFIC.get((kernel, n, dim, bits))
    int8_ops = 2.0 * q_per_launch * n * dim        # multiply-adds x2 of one launch, permute-dot mode

    out = {
        "metric": "queries/sec, 10Mx1536 4-bit, k=10, batch 1024, inputs and outputs resident in HBM (tv_search_dev); "
                  "host_buffers = the boundary call tv_search with PCIe copies, median of 5; batch1 beside it",
        "value": value,
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if mode_p else "u8",
        "data": "synthetic",
        "config": {"workload": f"TurboQuantIndex {n}x{dim} {bits}-bit, k={k}, no filter, batch {args.batch}",
                   "score_mode": "permute-dot (int8 weights x int8 codebook levels, i32 accumulate)" if mode_p
                   else "u8 LUT, integer accumulate", "n": n, "dim": dim, "bits": bits, "k": k, "batch": args.batch},
        "batch1": {"queries_per_s": b1_steps / dt1, "ms_per_query": dt1 / b1_steps * 1e3,
                   "scan_kernel_ms": b1_launch_s * 1e3, "achieved_GBps": alg_bytes / b1_launch_s / 1e9,
                   "frac_of_hbm_peak": alg_bytes / b1_launch_s / 1e9 / 8000.0,
                   "frac_of_achievable": alg_bytes / b1_launch_s / 1e9 / read_probe,
                   "outside_scan_us": (dt1 / b1_steps - b1_launch_s) * 1e6,
                   "end_to_end_frac_of_hbm_peak": alg_bytes / (dt1 / b1_steps) / 1e9 / 8000.0},
        "batch64": {"queries_per_s": 64 * b64_steps / dt64, "ms_per_step": dt64 / b64_steps * 1e3,
                    "queries_per_launch": q64_full, "scan_launch_ms": b64_launch_s * 1e3,
                    "roofline": {"bound": "hbm", "achieved": alg_bytes / b64_launch_s / 1e9, "peak": 8000.0, "unit": "GB/s",
                                 "frac": alg_bytes / b64_launch_s / 1e9 / 8000.0,
                                 "traffic": MEASURED_TRAFFIC.get(("k_scan_p4_multi", n, dim, bits)),
                                 "kernel": "k_scan_p4_multi" if mode_p else "k_scan_lut",
                                 "int8_TOPs": 2.0 * min(64, q64_full) * n * dim / b64_launch_s / 1e12 if mode_p else None}},
        "threads8_batch1": {"queries_per_s": t8_qps, "one_thread_queries_per_s": 1.0 / host_single_s,
                            "vs_one_thread": t8_qps * host_single_s, "calls_served_by_another_callers_launch": t8_merged,
                            "note": "8 threads x 40 single-query tv_search calls (host buffers); waiting calls "
                                    "with the same k and mask are merged into the next launch"},
        "host_buffers": {"queries_per_s": host_qps, "batch_median_ms": host_batch_s * 1e3,
                         "single_query_median_ms": host_single_s * 1e3,
                         "batch_x4_queries_per_s": 4 * args.batch / host_batch4_s,
                         "batch_x4_median_ms": host_batch4_s * 1e3,
                         "batch_x4_vs_batch": (4 * args.batch / host_batch4_s) / host_qps,
                         "note": "tv_search with host query/result buffers (PCIe both ways): median of 5 batch "
                                 "calls and of 15 single-query calls after a warm-up"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": 8000.0, "unit": "GB/s",
                     "frac": achieved / 8000.0, "traffic": traffic,
                     "kernel": kernel,
                     "achievable_read_GBps": read_probe, "frac_of_achievable": achieved / read_probe,
                     "algorithmic_bytes_per_launch": alg_bytes, "launches_timed": launches,
                     "mean_launch_ms": launch_s * 1e3, "queries_per_launch": q_per_launch,
                     "queries_per_full_launch": q_full},
    }
    if mode_p:
        mfma = {"achieved": int8_ops / launch_s / 1e12, "peak": 5000.0, "unit": "TFLOP/s",
                "frac": int8_ops / launch_s / 1e12 / 5000.0,
                "achievable": mfma_probe, "frac_of_achievable": int8_ops / launch_s / 1e12 / mfma_probe,
                "note": "int8 operations (2 per multiply-add) of the queries one launch scores, over the same "
                        "launch time; peak = 5.0 POP/s dense int8; achievable = the same MFMA loop alone "
                        "(registers x LDS, pseudo-random bytes, no HBM) timed in this run"}
        if kernel == "k_scan_p4_wide":
            # one launch serves the whole chunk: the matrix unit bounds it, the HBM read is paid once
            hbm = out["roofline"]
            out["roofline"] = {"bound": "mfma", **mfma, "traffic": traffic, "kernel": kernel,
                               "algorithmic_ops_per_launch": int8_ops, "launches_timed": launches,
                               "mean_launch_ms": launch_s * 1e3, "queries_per_launch": q_per_launch,
                               "queries_per_full_launch": q_full}
            out["hbm"] = {k: hbm[k] for k in ("achieved", "peak", "unit", "frac", "traffic",
                                              "algorithmic_bytes_per_launch", "achievable_read_GBps")}
        else:
            out["mfma"] = mfma
    # queries of the timed steps that left the sampled path for the exact one (candidate overflow);
    # Gaussian rows never do, and a non-zero count would mean the timed steps include that path's cost
    out["overflow_redos"] = ix.overflow_redos()
    out["exact_redos"] = ix.exact_redos()
    if not args.no_config3 and (n, dim, bits) == (10_000_000, 1536, 4) and not args.tile_groups:
        ix.close()
        del ix
        torch.cuda.empty_cache()
        out["config3"] = config3_extra(T, torch, build_index, run, args)
        torch.cuda.empty_cache()
        out["adversarial"] = adversarial_extra(T, torch, run, args, out["ms_per_step"], ladder)
    if args.cpu_sample > 0:
        out["cpu_baseline"] = cpu_baseline(args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
