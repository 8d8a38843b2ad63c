#!/usr/bin/env python3
"""Throughput of the column-vector-sparse SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (named in `config.workload`): the ResNet-50 3x3-conv-shaped single SpMM the metric
is quoted on - A is 512 x 4608 with V = 8 column vectors at 90 % sparsity (binomial row
lengths), B is 4608 x 256 fp16 row-major, fp16 output with fp32 accumulate.  All operands are
resident in HBM before the timed region.  A step is one operator call through the C ABI
(`vs_wmma_spmm_f16`).  The K timed steps are captured once into a HIP graph and replayed, so
the host's per-call launch cost (about 10 us from Python) does not hide a 5 us kernel; the
eager per-call figure is reported next to it.

Prints one JSON line: effective TFLOP/s = 2 * nnz * N / time, the HBM roofline of the kernel
(algorithmic bytes / average launch duration from HIP events on the launch stream / 8 TB/s) and
the CPU baseline (the C restatement of the reference's host loop, timed on this box's cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def spmm_algorithmic_bytes(pat, n_dense):
    """Bytes one launch must move at least once: values, column indices, row offsets, row swizzle,
    every referenced row of B once, and C once."""
    import numpy as np
    k_ref = int(np.unique(pat.column_indices[:pat.nnz_vec]).size)
    return (2 * pat.nnz + 4 * pat.nnz_vec + 4 * (pat.m_vec + 1) + 4 * pat.m_vec
            + 2 * k_ref * n_dense + 2 * pat.m * n_dense)


def sddmm_algorithmic_bytes(pat, k):
    import numpy as np
    n_ref = int(np.unique(pat.column_indices[:pat.nnz_vec]).size)
    return (2 * pat.m * k + 2 * n_ref * k + 4 * pat.nnz_vec + 4 * (pat.m_vec + 1) + 4 * pat.m_vec
            + 2 * pat.nnz)


def time_graph(torch, fn, steps, warmup, replays=7):
    """Capture `steps` calls of fn into a HIP graph and replay it `replays` times; return the medians of
    (wall ms/step, event ms/step).  One replay now and then runs at twice its usual time (clock ramp after an
    idle gap) and a single replay of a short graph carries its fixed start-up cost, so no single replay is used."""
    for _ in range(max(warmup, 1)):
        fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(steps):
            fn()
    graph.replay()  # untimed: first replay uploads the graph
    torch.cuda.synchronize()
    walls, events = [], []
    # wall clock and device events in replays of their own: the two event records are packets of their own in the
    # stream and cost a short graph 0.4 us per step of wall time (20 steps: 4.6 against 4.2 us)
    for _ in range(max(1, replays)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        walls.append((t1 - t0) * 1e3 / steps)
    for _ in range(max(1, replays)):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        events.append(e0.elapsed_time(e1) / steps)
    walls.sort()
    events.sort()
    return walls[len(walls) // 2], events[len(events) // 2]


def kernel_source_tag(*names):
    """First 16 hex digits of the SHA-256 of the kernel sources a counter summary belongs to."""
    import hashlib
    h = hashlib.sha256()
    for name in names:
        with open(os.path.join(ROOT, "vectorsparse_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


SPMM_SOURCES = ("spmm_mfma.hip", "spmm_mfma_step.hpp", "vs_common.hpp")
SDDMM_SOURCES = ("sddmm_mfma.hip", "vs_common.hpp")


def measured_traffic(path, sources):
    """(HBM-side bytes per launch, note) of a kernel from the committed rocprofv3 --pmc summary (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the same counter reads for a copy of known size).  The summary names the
    kernel sources it was measured on (`kernel_source_tag`); when they have changed since, the figure is stale
    and None is returned with a note saying so."""
    value, tag = None, None
    try:
        with open(path) as f:
            for ln in f:
                if ln.startswith("traffic_bytes_per_launch"):
                    value = float(ln.split()[1])
                elif ln.startswith("kernel_source_tag"):
                    tag = ln.split()[1]
    except OSError:
        return None, "no counter summary at %s" % os.path.relpath(path, ROOT)
    now = kernel_source_tag(*sources)
    if value is None:
        return None, "no traffic figure in %s" % os.path.relpath(path, ROOT)
    if tag != now:
        return None, "%s was measured on kernel sources %s, the sources are now %s: stale, not reported" % (
            os.path.relpath(path, ROOT), tag, now)
    return value, "from %s (kernel sources %s)" % (os.path.relpath(path, ROOT), now)


def time_eager(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


def cpu_baseline(pat, B, n_dense, flops, budget_s=12.0):
    """The oracle (a port of spmm_benchmark.cpp:66-86) on one host core, as the reference runs it,
    plus an all-cores OpenMP figure; same inputs as the GPU run."""
    from oracle import c_oracle as co

    def one(threads):
        t0 = time.perf_counter()
        co.spmm_host_ref_f32(pat.m_vec, pat.vec_length, n_dense, pat.n, pat.row_offsets, pat.column_indices,
                             pat.values, B, threads=threads)
        return time.perf_counter() - t0

    one(1)
    times = []
    t_start = time.perf_counter()
    while time.perf_counter() - t_start < budget_s and len(times) < 200:
        times.append(one(1))
    times.sort()
    med = times[len(times) // 2]
    cores = min(co.max_threads(), 16)
    mt = sorted(one(cores) for _ in range(7))[3] if cores > 1 else med
    return {
        "value": flops / med * 1e-12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": "%d full passes of the same workload (median), single thread as in the reference" % len(times),
        "ms": med * 1e3,
        "all_cores": {"value": flops / mt * 1e-12, "unit": "TFLOP/s", "cores": cores, "ms": mt * 1e3},
    }


PMC_MODES = ["spmm", "spmm_largest", "spmm_slab_50", "spmm_slab_90", "spmm_valu_v1", "sddmm_valu_v1", "sddmm_k128", "spmm_dma", "spmm_split_rows", "spmm_row_parts", "sddmm", "attention",
             "attention_window"]


def largest_sweep_point(cv):
    """The largest single-GPU point of the ResNet-50-shaped sweep: M = 2048, K = 4608, N = 256, V = 8, 90 %."""
    pat = cv.random_values(cv.uniform_pattern(2048 // 8, 4608, 0.9, seed=3, vec_length=8), seed=4)
    return pat, cv.dense_uniform(4608, 256, seed=5)


COLD_KERNELS = (("spmm_config2", "spmm_mfma_kernelILi8ELi4E"), ("spmm_largest", "spmm_mfma_kernelILi8ELi8E"),
                ("sddmm_config4", "sddmm_mfma_kernel"), ("dense_gemm_config2", "Cijk_"), ("empty_kernel", "floor_probe_kernel"))
COLD_PROFILE = os.path.join(ROOT, "profiles", "cold_cache_kernel_stats.txt")


def cold_summary(stats_csv):
    """Text of profiles/cold_cache_kernel_stats.txt from the kernel_stats.csv of
    `rocprofv3 --kernel-trace --stats ... -- python3 bench.py --cold`."""
    import csv
    found = {}
    with open(stats_csv) as f:
        for r in csv.DictReader(f):
            for key, needle in COLD_KERNELS:
                if needle in r["Name"]:
                    calls, total = found.get(key, (0, 0.0))
                    found[key] = (calls + int(r["Calls"]), total + float(r["TotalDurationNs"]))
    lines = ["Flushed-cache durations by the kernels' own timestamps (how the reference measures: Nsight --cache-control all,",
             "ncu_profile.py:91): every timed launch follows a 1 GiB fill that evicts the L2s and the Infinity Cache.",
             "",
             "commands (`cd /tmp && export TMPDIR=/tmp` first, then from the repository root):",
             "  rocprofv3 --kernel-trace --stats --output-format csv -d OUT -o t -- python3 bench.py --cold",
             "  python3 bench.py --cold-summary OUT/t_kernel_stats.csv > profiles/cold_cache_kernel_stats.txt",
             "",
             "kernel_source_tag_spmm %s" % kernel_source_tag(*SPMM_SOURCES),
             "kernel_source_tag_sddmm %s" % kernel_source_tag(*SDDMM_SOURCES),
             "",
             "mean kernel duration over the launches of the run (each right behind a fill), microseconds:"]
    for key, _ in COLD_KERNELS:
        if key in found:
            calls, total = found[key]
            lines.append("cold_us %-20s %8.2f   (%d launches)" % (key, total / calls * 1e-3, calls))
    return "\n".join(lines)


def read_cold_profile():
    """({name: microseconds}, note) from the committed summary of a `--cold` run; figures of kernels whose sources
    have changed since are dropped (the dense GEMM and the empty kernel are not ours and stay)."""
    values, tags = {}, {}
    try:
        with open(COLD_PROFILE) as f:
            for ln in f:
                w = ln.split()
                if len(w) >= 3 and w[0] == "cold_us":
                    values[w[1]] = float(w[2])
                elif len(w) == 2 and w[0].startswith("kernel_source_tag_"):
                    tags[w[0][len("kernel_source_tag_"):]] = w[1]
    except OSError:
        return {}, "no summary at %s" % os.path.relpath(COLD_PROFILE, ROOT)
    stale = []
    if tags.get("spmm") != kernel_source_tag(*SPMM_SOURCES):
        stale += [k for k in ("spmm_config2", "spmm_largest") if values.pop(k, None) is not None]
    if tags.get("sddmm") != kernel_source_tag(*SDDMM_SOURCES):
        stale += [k for k in ("sddmm_config4",) if values.pop(k, None) is not None]
    note = "from %s" % os.path.relpath(COLD_PROFILE, ROOT)
    if stale:
        note += "; dropped as stale (kernel sources changed since the run): " + ", ".join(stale)
    return values, note


def fine_grained_spmm_point(cv):
    """Where the fine-grained SpMM path is at home: V = 1, M = 2048, K = 4608, N = 256 at 90 % sparsity."""
    pat = cv.random_values(cv.uniform_pattern(2048, 4608, 0.9, seed=13, vec_length=1), seed=14)
    return pat, cv.dense_uniform(4608, 256, seed=15)


def fine_grained_sddmm_mask(cv):
    """The same for SDDMM: a 2048 x 2048 mask of single elements (V = 1) at 90 % sparsity (K = 64)."""
    return cv.uniform_pattern(2048, 2048, 0.9, seed=16, vec_length=1)


def sweep_v8(torch, cv, ops, iters=30):
    """The north-star comparison on the ResNet-50-shaped grid: every (M, K) of the sweep at N = 256, V = 8, at 80 % and
    90 % sparsity, through the reference-shaped entry point, each point verified (float64 product on a sample of rows,
    as the sweep driver does) and timed beside hipBLASLt's dense fp16 product of the same shape (the comparison of
    the reference's plot_spmm.py:43-58, per sparsity bucket)."""
    import numpy as np
    from vectorsparse_amd import sweep
    from vectorsparse_amd.benchmark_common import time_launches
    dense_us, dense_in, out_by_m, B_by_k = {}, {}, {}, {}
    buckets = {}
    unverified = 0
    for s in (0.8, 0.9):
        rows = []
        for M in sweep.MS:
            for K in sweep.KS:
                pat = sweep.spmm_grid_pattern(M, K, s, 8)
                if K not in B_by_k:
                    host = cv.dense_uniform(K, sweep.N_DENSE, seed=11)
                    B_by_k[K] = (host, torch.from_numpy(host).cuda())
                B_host, B = B_by_k[K]
                out = out_by_m.setdefault(M, torch.empty((M, sweep.N_DENSE), dtype=torch.float16, device="cuda"))
                prob = ops.DeviceProblem(pat, sort=True)
                out.fill_(float("nan"))
                prob.spmm(B, kernel="wmma", out=out)
                torch.cuda.synchronize()
                ok, rel = sweep.verify_spmm(pat, B_host, out.cpu().numpy())
                unverified += 0 if ok else 1
                us = time_launches(torch, lambda: prob.spmm(B, kernel="wmma", out=out), iters, warmup=2, replays=3)
                if (M, K) not in dense_us:
                    A = torch.randn((M, K), dtype=torch.float16, device="cuda")
                    dense_us[(M, K)] = time_launches(torch, lambda: torch.matmul(A, B, out=out), iters, warmup=2, replays=3)
                    del A
                rows.append({"M": M, "K": K, "us": us, "dense_us": dense_us[(M, K)], "speedup": dense_us[(M, K)] / us,
                             "frac": sweep.spmm_bytes(pat, sweep.N_DENSE) / (us * 1e-6) * 1e-9 / HBM_PEAK_GBS,
                             "max_rel_err": rel, "verified": ok})
        worst = min(rows, key=lambda r: r["speedup"])
        best = max(rows, key=lambda r: r["frac"])
        fracs = sorted(r["frac"] for r in rows)
        buckets["%g" % s] = {
            "points": len(rows), "verified": sum(1 for r in rows if r["verified"]),
            "geomean_speedup_vs_dense": sweep.geomean([r["speedup"] for r in rows]),
            "worst_speedup_vs_dense": worst["speedup"], "worst_point": "M=%d K=%d" % (worst["M"], worst["K"]),
            "points_slower_than_dense": sum(1 for r in rows if r["speedup"] < 1.0),
            "max_frac": best["frac"], "max_frac_point": "M=%d K=%d (%.2f us)" % (best["M"], best["K"], best["us"]),
            "median_frac": fracs[len(fracs) // 2],
            "max_rel_err": max(r["max_rel_err"] for r in rows)}
    if unverified:
        raise SystemExit("sweep_v8: %d point(s) failed verification" % unverified)
    return {"workload": "config 3 at V=8, N=256: M in %s x K in %s, uniform rows, vs_wmma_spmm_f16 with the sorted swizzle; "
                        "frac = algorithmic bytes / launch time / 8 TB/s" % (list(sweep.MS), list(sweep.KS)),
            "launches_per_replay": iters, "by_sparsity": buckets}


def skewed_point(cv, np):
    """Pareto-distributed row lengths (mean about 280 vectors, the longest row dense), 1024 vector rows x 4608."""
    rng = np.random.default_rng(0)
    m_vec, K = 1024, 4608
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 150, K).astype(np.int64)
    lengths = lengths[rng.permutation(m_vec)]
    ro, ci = cv._pattern_from_lengths(rng, m_vec, K, lengths)
    return cv.random_values(cv.ColVecCSR(m_vec, K, 8, ro, ci), 1), cv.dense_uniform(K, 256, seed=2)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--pmc", nargs="?", const="spmm", default=None, choices=PMC_MODES,
                    help="counter-collection mode for `rocprofv3 --pmc`: a 64 MiB device copy of known size "
                         "(calibration), then ten eager launches of one kernel and nothing else: the headline SpMM "
                         "(config 2), the largest sweep point (2048 x 4608 at 90 %%), the LDS-staged schedule on that shape at 50 %% and 90 %%, config 2 on the LDS-DMA gather "
                         "variant, the split-row SpMM and the SpMM with rows in parts on Pareto-distributed rows, the config-4 SDDMM, the config-5 "
                         "attention layer with its plan, or that layer with a plain 513-wide window mask")
    ap.add_argument("--cold", action="store_true",
                    help="flushed-cache mode for `rocprofv3 --kernel-trace --stats`: ten rounds of (1 GiB fill, ONE launch) "
                         "for each of the config-2 SpMM, the largest sweep point, the config-4 SDDMM, the dense GEMM of "
                         "config 2 and a kernel that does nothing; the kernels' own timestamps are the cold durations")
    ap.add_argument("--cold-summary", metavar="KERNEL_STATS_CSV", default=None,
                    help="turn the kernel_stats.csv of such a run into the text of profiles/cold_cache_kernel_stats.txt "
                         "(printed; no GPU needed)")
    args = ap.parse_args()
    if args.cold_summary:
        print(cold_summary(args.cold_summary))
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: the SpMM/SDDMM path has no multi-GPU leg (rows shard with no "
              "exchange step); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from vectorsparse_amd import _lib
    from vectorsparse_amd import colvec_csr as cv
    from vectorsparse_amd import ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)

    # ---- headline workload: config 2
    M, K, N, V, sparsity = 512, 4608, 256, 8, 0.9
    pat = cv.random_values(cv.binomial_pattern(M // V, K, sparsity, seed=1, vec_length=V), seed=101)
    B = cv.dense_uniform(K, N, seed=201)
    prob = ops.DeviceProblem(pat, sort=True)
    Bd = torch.from_numpy(B).cuda()
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    flops = 2.0 * pat.nnz * N
    alg_bytes = spmm_algorithmic_bytes(pat, N)

    def step():
        prob.spmm(Bd, kernel="wmma", out=out)

    # ---- SDDMM companion point (config 4: M = N = 2048, K = 64, V = 8, 90 %)
    mask = cv.uniform_pattern(2048 // 8, 2048, 0.9, seed=4, vec_length=8)
    lhs = torch.from_numpy(cv.dense_normal(2048, 64, seed=14)).cuda()
    rhs = torch.from_numpy(cv.dense_normal(2048, 64, seed=24)).cuda()
    sprob = ops.DeviceProblem(mask)
    sout = torch.empty((mask.nnz_vec, 8), dtype=torch.float16, device="cuda")

    def sddmm_step():
        sprob.sddmm(lhs, rhs, kernel="wmma", out=sout)

    if args.cold:
        import ctypes
        probe_lib = ctypes.CDLL(os.path.join(ROOT, "vectorsparse_amd", "libvsprobe.so"))
        probe_lib.vsprobe_empty_launch.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        lpat, lB = largest_sweep_point(cv)
        lprob = ops.DeviceProblem(lpat, sort=True)
        lBd = torch.from_numpy(lB).cuda()
        lout = torch.empty((lpat.m, 256), dtype=torch.float16, device="cuda")
        Ad = torch.randn((M, K), dtype=torch.float16, device="cuda")
        dense_out = torch.empty((M, N), dtype=torch.float16, device="cuda")
        launches = (step, lambda: lprob.spmm(lBd, kernel="wmma", out=lout), sddmm_step,
                    lambda: torch.matmul(Ad, Bd, out=dense_out),
                    lambda: probe_lib.vsprobe_empty_launch(256, 512, torch.cuda.current_stream().cuda_stream))
        thrash = torch.empty(512 * 1024 * 1024, dtype=torch.float16, device="cuda")
        for i in range(10):
            for fn in launches:
                thrash.fill_(float(i))
                fn()
            torch.cuda.synchronize()
        print(json.dumps({"cold_mode": "10 rounds of (1 GiB fill, one launch) for %d kernels" % len(launches)}))
        return

    if args.pmc:
        src = torch.zeros(32 * 1024 * 1024, dtype=torch.float16, device="cuda")   # 64 MiB read + 64 MiB written
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        info = {"pmc_mode": args.pmc, "copy_bytes_each_way": src.numel() * 2}
        if args.pmc in ("spmm", "spmm_dma"):
            if args.pmc == "spmm_dma":
                _lib.set_option("spmm_gather", 2)
            for _ in range(10):
                step()
            info["algorithmic_bytes"] = alg_bytes
            info["kernel_source_tag"] = kernel_source_tag(*SPMM_SOURCES)
        elif args.pmc == "spmm_largest":
            lpat, lB = largest_sweep_point(cv)
            lprob = ops.DeviceProblem(lpat, sort=True)
            lBd = torch.from_numpy(lB).cuda()
            lout = torch.empty((lpat.m, 256), dtype=torch.float16, device="cuda")
            for _ in range(10):
                lprob.spmm(lBd, kernel="wmma", out=lout)
            info["algorithmic_bytes"] = spmm_algorithmic_bytes(lpat, 256)
            info["nonzero_vectors"] = int(lpat.nnz_vec)
            info["kernel_source_tag"] = kernel_source_tag(*SPMM_SOURCES)
        elif args.pmc in ("spmm_slab_50", "spmm_slab_90"):
            # the LDS-staged schedule (vs_wmma_spmm_f16_slab) on 2048 x 4608 x 256 at 50 % / 90 %, ten launches
            lpat = cv.random_values(cv.uniform_pattern(2048 // 8, 4608, 0.5 if args.pmc.endswith("50") else 0.9,
                                                       seed=3, vec_length=8), seed=4)
            lprob = ops.DeviceProblem(lpat, sort=True)
            lBd = torch.from_numpy(cv.dense_uniform(4608, 256, seed=5)).cuda()
            lout = torch.empty((lpat.m, 256), dtype=torch.float16, device="cuda")
            ws = torch.empty(max(16, ops.spmm_slab_workspace_bytes(lpat.m_vec, 8, 256, 4608)), dtype=torch.uint8, device="cuda")
            for _ in range(10):
                ops.spmm_slab(lpat.m_vec, 8, 256, 4608, lprob.row_indices, lprob.row_offsets, lprob.column_indices,
                              lprob.values, lBd, lout, ws)
            info["algorithmic_bytes"] = spmm_algorithmic_bytes(lpat, 256)
            info["nonzero_vectors"] = int(lpat.nnz_vec)
            info["kernel_source_tag"] = kernel_source_tag("spmm_mfma_slab.hip", "spmm_mfma_step.hpp", "vs_common.hpp")
        elif args.pmc == "spmm_valu_v1":
            # the fine-grained SpMM on the shape it exists for: V = 1 (2048 x 4608 x 256 at 90 %)
            vpat, vB = fine_grained_spmm_point(cv)
            vprob = ops.DeviceProblem(vpat, sort=True)
            vBd = torch.from_numpy(vB).cuda()
            vout = torch.empty((vpat.m, 256), dtype=torch.float16, device="cuda")
            for _ in range(10):
                vprob.spmm(vBd, kernel="cuda", out=vout)
            info["algorithmic_bytes"] = spmm_algorithmic_bytes(vpat, 256)
            info["nonzero_vectors"] = int(vpat.nnz_vec)
            info["kernel_source_tag"] = kernel_source_tag("spmm_valu.hip", "vs_common.hpp")
        elif args.pmc == "sddmm_valu_v1":
            # the fine-grained SDDMM at V = 1 (2048 x 2048 mask at 90 %, K = 64)
            vmask = fine_grained_sddmm_mask(cv)
            vsprob = ops.DeviceProblem(vmask)
            vsout = torch.empty((vmask.nnz_vec, 1), dtype=torch.float16, device="cuda")
            for _ in range(10):
                vsprob.sddmm(lhs, rhs, kernel="cuda", out=vsout)
            info["algorithmic_bytes"] = sddmm_algorithmic_bytes(vmask, 64)
            info["nonzero_vectors"] = int(vmask.nnz_vec)
            info["kernel_source_tag"] = kernel_source_tag("sddmm_valu.hip", "vs_common.hpp")
        elif args.pmc == "sddmm_k128":
            lhs128 = torch.from_numpy(cv.dense_normal(2048, 128, seed=15)).cuda()
            rhs128 = torch.from_numpy(cv.dense_normal(2048, 128, seed=25)).cuda()
            for _ in range(10):
                sprob.sddmm(lhs128, rhs128, kernel="wmma", out=sout)
            info["algorithmic_bytes"] = sddmm_algorithmic_bytes(mask, 128)
            info["kernel_source_tag"] = kernel_source_tag(*SDDMM_SOURCES)
        elif args.pmc == "spmm_split_rows":
            kpat, kB = skewed_point(cv, np)
            kprob = ops.DeviceProblem(kpat, sort=True)
            kBd = torch.from_numpy(kB).cuda()
            kout = torch.empty((kpat.m, 256), dtype=torch.float16, device="cuda")
            for _ in range(10):
                kprob.spmm(kBd, kernel="wmma", out=kout, split_rows=True)
            info["algorithmic_bytes"] = spmm_algorithmic_bytes(kpat, 256)
            info["nonzero_vectors"] = int(kpat.nnz_vec)
        elif args.pmc == "spmm_row_parts":
            kpat, kB = skewed_point(cv, np)
            kprob = ops.DeviceProblem(kpat, sort=True)
            kBd = torch.from_numpy(kB).cuda()
            kout = torch.empty((kpat.m, 256), dtype=torch.float16, device="cuda")
            for _ in range(10):
                kprob.spmm_row_parts(kBd, out=kout)
            info["algorithmic_bytes"] = spmm_algorithmic_bytes(kpat, 256)
            info["nonzero_vectors"] = int(kpat.nnz_vec)
            info["kernel_source_tag"] = kernel_source_tag(*SPMM_SOURCES)
        elif args.pmc == "sddmm":
            for _ in range(10):
                sddmm_step()
            info["algorithmic_bytes"] = sddmm_algorithmic_bytes(mask, 64)
            info["kernel_source_tag"] = kernel_source_tag(*SDDMM_SOURCES)
        else:
            heads, seq, dim = 16, 4096, 64
            if args.pmc == "attention_window":
                amask = cv.band_strided_pattern(seq, 8, band_half_width=256, stride=seq)
            else:
                amask = cv.band_strided_pattern(seq, 8, band_half_width=128, stride=128)
            layer = ops.SparseAttention(amask)
            gen = torch.Generator(device="cuda").manual_seed(5)
            q, kk_, vv = (torch.randn((heads, seq, dim), device="cuda", generator=gen).half() for _ in range(3))
            ctx = torch.empty((heads, seq, dim), dtype=torch.float16, device="cuda")
            for _ in range(10):
                layer.forward(q, kk_, vv, out=ctx)
            info["algorithmic_bytes"] = 4 * heads * seq * dim * 2      # q, k, v read once, out written once
            info["rows_per_workgroup"] = layer.union_rows(dim, dim, heads)
            info["nonzero_vectors"] = int(amask.nnz_vec)
        torch.cuda.synchronize()
        print(json.dumps(info))
        return

    wall_ms, ev_ms = time_graph(torch, step, args.steps, args.warmup)
    # A replay takes about 11 us of device time to get going, whatever its length (20 launches between two events
    # read 3.9 us each, 200 read 3.35 us, also right behind another replay): the kernel's average launch duration -
    # `roofline` and every device-side figure under `extra` - is therefore taken over at least 200 launches per
    # replay, while `value` and `ms_per_step` stay the wall clock of exactly --steps steps.
    dev_steps = max(args.steps, 200)
    if dev_steps != args.steps:
        _, ev_ms = time_graph(torch, step, dev_steps, args.warmup)
    eager_wall_ms, _ = time_eager(torch, step, args.steps, args.warmup)
    # the same problem through the batched entry point, which also takes the pattern's nonzero count
    _, hinted_ms = time_graph(torch, lambda: prob.spmm(Bd, kernel="wmma", out=out, row_length_hint=True),
                              dev_steps, args.warmup)
    step()

    # correctness of what was just timed (reference criterion and 1e-2 relative)
    from oracle import c_oracle as co
    ref = co.spmm_host_ref_f32(pat.m_vec, V, N, K, pat.row_offsets, pat.column_indices, pat.values, B)
    got = out.cpu().numpy().astype(np.float64)
    floor = 1e-2 * float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    max_rel = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))
    errors = int(np.sum(np.abs(got - ref) > 0.5))

    # ---- the dispatch floor of the headline launch: a kernel that does nothing on the same grid.  No kernel of
    # that shape finishes sooner, so algorithmic bytes / this time is the ceiling of `roofline.frac` on config 2.
    import ctypes
    probe_path = os.path.join(ROOT, "vectorsparse_amd", "libvsprobe.so")
    if not os.path.exists(probe_path):
        raise SystemExit("%s not found: build it with `python -m vectorsparse_amd.build`" % probe_path)
    floor_lib = ctypes.CDLL(probe_path)
    floor_lib.vsprobe_empty_launch.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p]

    def probe(threads):  # on whatever stream is current at the call (the capture stream inside time_graph)
        return lambda: floor_lib.vsprobe_empty_launch(256, threads, torch.cuda.current_stream().cuda_stream)

    _, floor_ms = time_graph(torch, probe(1024), dev_steps, args.warmup)
    _, floor_small_ms = time_graph(torch, probe(64), dev_steps, args.warmup)

    # ---- dense fp16 GEMM (hipBLASLt through torch) on the same M x K x N, same timing method
    Ad = torch.randn((M, K), dtype=torch.float16, device="cuda")
    dense_out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    _, dense_ms = time_graph(torch, lambda: torch.matmul(Ad, Bd, out=dense_out), dev_steps, args.warmup)

    # ---- the largest single-GPU point of the sweep (2048 x 4608 x 256, 90 %): the end where the roofline counts
    lpat, lB = largest_sweep_point(cv)
    lprob = ops.DeviceProblem(lpat, sort=True)
    lBd = torch.from_numpy(lB).cuda()
    lout = torch.empty((lpat.m, 256), dtype=torch.float16, device="cuda")
    _, large_ms = time_graph(torch, lambda: lprob.spmm(lBd, kernel="wmma", out=lout), dev_steps, args.warmup)
    large_bytes = spmm_algorithmic_bytes(lpat, 256)
    lA = torch.randn((lpat.m, 4608), dtype=torch.float16, device="cuda")
    _, large_dense_ms = time_graph(torch, lambda: torch.matmul(lA, lBd, out=lout), dev_steps, args.warmup)

    # ---- skewed rows: reference-shaped entry, batched entry with the row-length hints, split-row schedule, rows in parts
    kpat, kB = skewed_point(cv, np)
    kprob = ops.DeviceProblem(kpat, sort=True)
    kBd = torch.from_numpy(kB).cuda()
    kout = torch.empty((kpat.m, 256), dtype=torch.float16, device="cuda")
    skew_steps = max(20, dev_steps // 4)
    _, skew_plain_ms = time_graph(torch, lambda: kprob.spmm(kBd, out=kout), skew_steps, 3)
    _, skew_hint_ms = time_graph(torch, lambda: kprob.spmm(kBd, out=kout, row_length_hint=True), skew_steps, 3)
    _, skew_split_ms = time_graph(torch, lambda: kprob.spmm(kBd, out=kout, split_rows=True), skew_steps, 3)
    kref = kout.clone()
    _, skew_parts_ms = time_graph(torch, lambda: kprob.spmm_row_parts(kBd, out=kout), skew_steps, 3)
    torch.cuda.synchronize()
    # (rows in parts add a split row's nonzeros in another order than the split-row schedule: equal up to fp32 rounding
    # of sums of a few thousand terms, then both rounded to fp16)
    skew_parts_diff = float((kout.float() - kref.float()).abs().max() / kref.float().abs().max())
    if not skew_parts_diff < 2e-3:
        raise SystemExit("rows in parts and split rows disagree on the skewed point: %g" % skew_parts_diff)
    kparts = kprob.row_parts(0)[0]
    upat = cv.random_values(cv.uniform_pattern(kpat.m_vec, kpat.n, 1 - kpat.nnz_vec / (kpat.m_vec * kpat.n), 1, 8), 1)
    uprob = ops.DeviceProblem(upat, sort=True)
    _, skew_uniform_ms = time_graph(torch, lambda: uprob.spmm(kBd, out=kout), skew_steps, 3)
    _, skew_uniform_hint_ms = time_graph(torch, lambda: uprob.spmm(kBd, out=kout, row_length_hint=True), skew_steps, 3)

    # ---- SDDMM on the same skewed pattern as a mask (K = 64): row kernel, nonzero-range schedule, rows in parts
    kg = torch.Generator(device="cuda").manual_seed(11)
    klhs = torch.randn((kpat.m, 64), device="cuda", generator=kg).half()
    krhs = torch.randn((kpat.n, 64), device="cuda", generator=kg).half()
    ksout = torch.empty((kpat.nnz_vec, 8), dtype=torch.float16, device="cuda")
    _, sk_sd_row_ms = time_graph(torch, lambda: kprob.sddmm(klhs, krhs, out=ksout, algorithm=1), skew_steps, 3)
    _, sk_sd_flat_ms = time_graph(torch, lambda: kprob.sddmm(klhs, krhs, out=ksout, algorithm=2), skew_steps, 3)
    ksref = ksout.clone()
    _, sk_sd_parts_ms = time_graph(torch, lambda: kprob.sddmm_row_parts(klhs, krhs, out=ksout), skew_steps, 3)
    torch.cuda.synchronize()
    if not torch.equal(ksout, ksref):   # (the same arithmetic per output on every schedule)
        raise SystemExit("SDDMM with rows in parts and on the nonzero-range schedule disagree on the skewed point")
    _, sk_sd_uniform_ms = time_graph(torch, lambda: uprob.sddmm(klhs, krhs, out=ksout[:upat.nnz_vec], algorithm=1),
                                     skew_steps, 3)

    # ---- SDDMM config 4
    _, sddmm_ms = time_graph(torch, sddmm_step, dev_steps, args.warmup)
    sddmm_flops = 2.0 * mask.nnz * 64
    sddmm_bytes = sddmm_algorithmic_bytes(mask, 64)
    # the fine-grained paths (cudaSpmm / cudaSddmm of the reference) on the same two workloads
    _, valu_spmm_ms = time_graph(torch, lambda: prob.spmm(Bd, kernel="cuda", out=out), dev_steps, args.warmup)
    _, valu_sddmm_ms = time_graph(torch, lambda: sprob.sddmm(lhs, rhs, kernel="cuda", out=sout), dev_steps, args.warmup)
    full = torch.empty((2048, 2048), dtype=torch.float16, device="cuda")
    _, sddmm_dense_ms = time_graph(torch, lambda: torch.matmul(lhs, rhs.t(), out=full), dev_steps, args.warmup)

    # ---- fixed-mask sparse attention layer (config 5: 16 heads, seq 4096, d 64, V = 8 band + strided mask)
    heads, seq, dim = 16, 4096, 64
    amask = cv.band_strided_pattern(seq, 8, band_half_width=128, stride=128)
    layer = ops.SparseAttention(amask)
    gen = torch.Generator(device="cuda").manual_seed(5)
    q, kk_, vv = (torch.randn((heads, seq, dim), device="cuda", generator=gen).half() for _ in range(3))
    scores = torch.empty((heads, amask.nnz_vec, 8), dtype=torch.float16, device="cuda")
    ctx = torch.empty((heads, seq, dim), dtype=torch.float16, device="cuda")
    attn_steps = max(5, dev_steps // 10)
    _, attn_ms = time_graph(torch, lambda: layer.forward(q, kk_, vv, scores=scores, out=ctx), attn_steps, 3)

    def dense_attention():
        s_ = torch.matmul(q, kk_.transpose(1, 2))
        return torch.matmul(torch.softmax(s_ * 0.125, dim=-1), vv)

    _, dense_attn_ms = time_graph(torch, dense_attention, 5, 2, replays=3)
    attn_flops = 2.0 * amask.nnz * heads * dim * 2
    # the same layer with a plain 513-wide window (unions of up to 634 columns per 16 vector rows)
    wmask = cv.band_strided_pattern(seq, 8, band_half_width=256, stride=seq)
    wlayer = ops.SparseAttention(wmask)
    _, window_ms = time_graph(torch, lambda: wlayer.forward(q, kk_, vv, out=ctx), attn_steps, 3)

    # a +-64 band with 64 global tokens (eight vector rows that attend to everything, 64 columns everybody attends
    # to): rows far longer than the rest, which the layer runs as three operators on a dispatch list of row parts
    grows = []
    for i in range(seq // 8):
        c = 8 * i + 4
        grows.append(np.arange(seq) if i < 8 else np.union1d(np.arange(max(0, c - 64), min(seq, c + 64)), np.arange(64)))
    gmask = cv.ColVecCSR(seq // 8, seq, 8, np.concatenate([[0], np.cumsum([len(r) for r in grows])]).astype(np.int32),
                         np.concatenate(grows).astype(np.int32))
    glayer = ops.SparseAttention(gmask)
    gscores = torch.empty((heads, gmask.nnz_vec, 8), dtype=torch.float16, device="cuda")
    _, global_ms = time_graph(torch, lambda: glayer.forward(q, kk_, vv, scores=gscores, out=ctx), attn_steps, 3)
    gref = ctx.clone()
    _, global_whole_rows_ms = time_graph(torch, lambda: glayer.forward(q, kk_, vv, scores=gscores, out=ctx, fused=True),
                                         attn_steps, 3)
    torch.cuda.synchronize()
    global_diff = float((ctx.float() - gref.float()).abs().max())
    if not global_diff < 2e-2:
        raise SystemExit("attention with global tokens: rows in parts and whole rows disagree: %g" % global_diff)

    # ---- cold caches (how the reference measures: Nsight --cache-control all): the kernels' own timestamps from a
    # `rocprofv3 --kernel-trace` run of `bench.py --cold`, committed under profiles/ (HIP events round a single eager
    # launch read 6 us for a kernel that does nothing, so they are not used for this)
    cold, cold_note = read_cold_profile()

    # ---- the fine-grained paths where they are at home: V = 1
    vpat, vB = fine_grained_spmm_point(cv)
    vprob = ops.DeviceProblem(vpat, sort=True)
    vBd = torch.from_numpy(vB).cuda()
    vout = torch.empty((vpat.m, 256), dtype=torch.float16, device="cuda")
    fine_steps = max(20, dev_steps // 4)
    _, v1_spmm_valu_ms = time_graph(torch, lambda: vprob.spmm(vBd, kernel="cuda", out=vout), fine_steps, 3)
    _, v1_spmm_mfma_ms = time_graph(torch, lambda: vprob.spmm(vBd, kernel="wmma", out=vout), fine_steps, 3)
    v1_spmm_bytes, v1_spmm_flops = spmm_algorithmic_bytes(vpat, 256), 2.0 * vpat.nnz * 256
    vA = torch.randn((vpat.m, 4608), dtype=torch.float16, device="cuda")
    _, v1_dense_ms = time_graph(torch, lambda: torch.matmul(vA, vBd, out=vout), fine_steps, 3)
    vmask = fine_grained_sddmm_mask(cv)
    vsprob = ops.DeviceProblem(vmask)
    vsout = torch.empty((vmask.nnz_vec, 1), dtype=torch.float16, device="cuda")
    _, v1_sddmm_valu_ms = time_graph(torch, lambda: vsprob.sddmm(lhs, rhs, kernel="cuda", out=vsout), fine_steps, 3)
    _, v1_sddmm_mfma_ms = time_graph(torch, lambda: vsprob.sddmm(lhs, rhs, kernel="wmma", out=vsout, algorithm=1), fine_steps, 3)
    v1_sddmm_bytes, v1_sddmm_flops = sddmm_algorithmic_bytes(vmask, 64), 2.0 * vmask.nnz * 64

    # ---- config 4's other three points (K = 128, and 95 % sparsity)
    sddmm_more = {}
    for kk, sp, seed in ((128, 0.9, 4), (64, 0.95, 6), (128, 0.95, 6)):
        m4 = mask if sp == 0.9 else cv.uniform_pattern(2048 // 8, 2048, sp, seed=seed, vec_length=8)
        p4 = sprob if sp == 0.9 else ops.DeviceProblem(m4)
        l4 = torch.from_numpy(cv.dense_normal(2048, kk, seed=14 + kk)).cuda()
        r4 = torch.from_numpy(cv.dense_normal(2048, kk, seed=24 + kk)).cuda()
        o4 = torch.empty((m4.nnz_vec, 8), dtype=torch.float16, device="cuda")
        _, ms4 = time_graph(torch, lambda: p4.sddmm(l4, r4, kernel="wmma", out=o4), dev_steps, 3)
        f4 = torch.empty((2048, 2048), dtype=torch.float16, device="cuda")
        _, dense4 = time_graph(torch, lambda: torch.matmul(l4, r4.t(), out=f4), fine_steps, 3)
        sddmm_more["k%d_s%g" % (kk, sp)] = (sddmm_algorithmic_bytes(m4, kk), ms4, 2.0 * m4.nnz * kk, dense4)

    # ---- the sweep's V = 8 points at 80 % and 90 % beside hipBLASLt
    sweep_block = sweep_v8(torch, cv, ops)

    achieved = alg_bytes / (ev_ms * 1e-3) * 1e-9
    traffic, traffic_note = measured_traffic(os.path.join(ROOT, "profiles", "spmm_mfma_config2_pmc.txt"), SPMM_SOURCES)
    large_traffic, _ = measured_traffic(os.path.join(ROOT, "profiles", "spmm_mfma_largest_pmc.txt"), SPMM_SOURCES)
    sddmm_traffic, sddmm_note = measured_traffic(os.path.join(ROOT, "profiles", "sddmm_mfma_config4_pmc.txt"), SDDMM_SOURCES)

    def hbm(nbytes, ms, traffic_bytes=None, **more):
        gbs = nbytes / (ms * 1e-3) * 1e-9
        d = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
             "traffic": traffic_bytes, "algorithmic_bytes": nbytes, "avg_launch_us": ms * 1e3}
        d.update(more)
        return d

    line = {
        "metric": "SpMM effective TFLOP/s (2*nnz*N), fp16 V=8, 90% sparse",
        "value": flops / (wall_ms * 1e-3) * 1e-12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "config2: single SpMM M=512 K=4608 N=256 V=8 sparsity=0.9 (binomial rows), "
                               "sorted row swizzle, fp16 out / fp32 accumulate",
                   "nnz_vec": pat.nnz_vec,
                   "launch": "HIP graph of `steps` operator calls, median of 7 replays (wall clock); device-side "
                             "figures from replays of %d launches" % dev_steps},
        "roofline": hbm(alg_bytes, ev_ms, traffic, kernel="spmm_mfma_kernel<V=8>", traffic_note=traffic_note,
                        caches="warm: the 3.2 MB working set stays in the Infinity Cache between launches (the L2s "
                               "start every launch cold); see extra.cold_cache",
                        frac_cold=(alg_bytes / (cold["spmm_config2"] * 1e-6) * 1e-9 / HBM_PEAK_GBS
                                   if "spmm_config2" in cold else None),
                        frac_cold_note="from extra.cold_cache.kernel_us.spmm_config2 (kernel timestamps of a launch "
                                       "behind a 1 GiB fill; " + cold_note + ")",
                        ceiling_frac=alg_bytes / (floor_ms * 1e-3) * 1e-9 / HBM_PEAK_GBS,
                        ceiling_note="a kernel that does nothing on this launch's grid (256 workgroups of up to 1024 threads) "
                                     "takes extra.launch_floor.empty_grid_us: the HBM-roofline time of config 2 "
                                     "(0.40 us) is a quarter of it, so frac cannot exceed ceiling_frac on this config"),
        "parity": {"max_rel_err": max_rel, "errors_gt_0.5": errors},
        "extra": {
            "eager_ms_per_step": eager_wall_ms,
            "batched_entry_with_nonzero_count_ms": hinted_ms,
            "dense_gemm_ms": dense_ms,
            "speedup_vs_dense_gemm": dense_ms / ev_ms,
            "launch_floor": {"empty_grid_us": floor_ms * 1e3, "empty_grid_one_wave_per_workgroup_us": floor_small_ms * 1e3,
                             "frac_of_floor": floor_ms / ev_ms},
            "cold_cache": {"method": "mean kernel duration by the kernels' own timestamps (rocprofv3 --kernel-trace --stats of "
                                     "`bench.py --cold`: every launch right behind a 1 GiB fill), read from the committed "
                                     "summary; null where the kernel sources have changed since",
                           "source": cold_note, "kernel_us": cold,
                           "speedup_vs_dense_gemm_config2": (cold["dense_gemm_config2"] / cold["spmm_config2"]
                                                             if "dense_gemm_config2" in cold and "spmm_config2" in cold else None)},
            "sweep_v8": sweep_block,
            "spmm_largest_sweep_point": dict(
                hbm(large_bytes, large_ms, large_traffic),
                workload="M=2048 K=4608 N=256 V=8 sparsity=0.9", tflops=2.0 * lpat.nnz * 256 / (large_ms * 1e-3) * 1e-12,
                gather_tbs=lpat.nnz_vec * 512 / (large_ms * 1e-3) * 1e-12, dense_gemm_us=large_dense_ms * 1e3,
                speedup_vs_dense_gemm=large_dense_ms / large_ms),
            "spmm_skewed_rows": {"workload": "1024 vector rows x 4608, Pareto row lengths (mean %.0f, longest %d), N=256"
                                             % (kpat.nnz_vec / kpat.m_vec, int(np.diff(kpat.row_offsets).max())),
                                 "reference_entry_us": skew_plain_ms * 1e3, "hinted_batched_entry_us": skew_hint_ms * 1e3,
                                 "split_rows_entry_us": skew_split_ms * 1e3,
                                 "row_parts_entry_us": skew_parts_ms * 1e3,
                                 "row_parts": "%d rows in up to %d parts" % (kparts.n_split, kparts.parts_max),
                                 "uniform_rows_same_nonzeros_us": skew_uniform_ms * 1e3,
                                 "uniform_rows_same_nonzeros_hinted_us": skew_uniform_hint_ms * 1e3,
                                 "row_parts_over_uniform_hinted": skew_parts_ms / skew_uniform_hint_ms},
            "sddmm_skewed_rows": {"workload": "the same pattern as a mask, K=64", "row_kernel_us": sk_sd_row_ms * 1e3,
                                  "nonzero_range_schedule_us": sk_sd_flat_ms * 1e3, "row_parts_entry_us": sk_sd_parts_ms * 1e3,
                                  "uniform_rows_same_nonzeros_us": sk_sd_uniform_ms * 1e3,
                                  "row_parts_over_uniform": sk_sd_parts_ms / sk_sd_uniform_ms},
            "sddmm_config4_k64": dict(
                hbm(sddmm_bytes, sddmm_ms, sddmm_traffic, traffic_note=sddmm_note, kernel="sddmm_mfma_kernel<V=8>"),
                ms=sddmm_ms, tflops=sddmm_flops / (sddmm_ms * 1e-3) * 1e-12, dense_product_us=sddmm_dense_ms * 1e3,
                speedup_vs_dense=sddmm_dense_ms / sddmm_ms),
            "sddmm_config4_other_points": {
                name: dict(hbm(nb, ms4, kernel="sddmm_mfma_kernel<V=8>"), tflops=fl / (ms4 * 1e-3) * 1e-12,
                           dense_product_us=d4 * 1e3, speedup_vs_dense=d4 / ms4)
                for name, (nb, ms4, fl, d4) in sddmm_more.items()},
            "fine_grained_paths": {
                "spmm_v1_2048x4608x256_s90": {
                    "cuda_path": dict(hbm(v1_spmm_bytes, v1_spmm_valu_ms, kernel="spmm_valu_kernel<V=1>"),
                                      tflops=v1_spmm_flops / (v1_spmm_valu_ms * 1e-3) * 1e-12),
                    "wmma_path": dict(hbm(v1_spmm_bytes, v1_spmm_mfma_ms, kernel="spmm_mfma_kernel<V=1>"),
                                      tflops=v1_spmm_flops / (v1_spmm_mfma_ms * 1e-3) * 1e-12),
                    "dense_gemm_us": v1_dense_ms * 1e3, "cuda_over_wmma": v1_spmm_mfma_ms / v1_spmm_valu_ms},
                "sddmm_v1_2048x2048_k64_s90": {
                    "cuda_path": dict(hbm(v1_sddmm_bytes, v1_sddmm_valu_ms, kernel="sddmm_valu_kernel<V=1>"),
                                      tflops=v1_sddmm_flops / (v1_sddmm_valu_ms * 1e-3) * 1e-12),
                    "wmma_path": dict(hbm(v1_sddmm_bytes, v1_sddmm_mfma_ms, kernel="sddmm_mfma_kernel<V=1>"),
                                      tflops=v1_sddmm_flops / (v1_sddmm_mfma_ms * 1e-3) * 1e-12),
                    "cuda_over_wmma": v1_sddmm_mfma_ms / v1_sddmm_valu_ms},
                "spmm_config2": dict(hbm(alg_bytes, valu_spmm_ms, kernel="spmm_valu_kernel<V=8>"),
                                     tflops=flops / (valu_spmm_ms * 1e-3) * 1e-12, speedup_vs_dense_gemm=dense_ms / valu_spmm_ms),
                "sddmm_config4_k64": dict(hbm(sddmm_bytes, valu_sddmm_ms, kernel="sddmm_valu_kernel<V=8>"),
                                          tflops=sddmm_flops / (valu_sddmm_ms * 1e-3) * 1e-12,
                                          speedup_vs_dense=sddmm_dense_ms / valu_sddmm_ms)},
            "attention_window513": {"layer_ms": window_ms, "density": 1.0 - wmask.sparsity,
                                    "tflops": 2.0 * wmask.nnz * heads * dim * 2 / (window_ms * 1e-3) * 1e-12},
            "attention_global_tokens": {"workload": "16 heads x 4096 x 64, +-64 band with 64 global tokens",
                                        "density": 1.0 - gmask.sparsity, "layer_ms": global_ms,
                                        "whole_rows_sddmm_softmax_spmm_ms": global_whole_rows_ms,
                                        "speedup": global_whole_rows_ms / global_ms},
            "attention_config5": {"layer_ms": attn_ms, "density": 1.0 - amask.sparsity,
                                  "tflops": attn_flops / (attn_ms * 1e-3) * 1e-12,
                                  "dense_masked_attention_ms": dense_attn_ms,
                                  "speedup_vs_dense": dense_attn_ms / attn_ms},
        },
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(pat, B, N, flops)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
