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


def time_cold(torch, fn, samples=20):
    """Device time of single launches with the caches thrashed in between: a 1 GiB fill evicts the 256 MB
    Infinity Cache and the L2s before every timed launch (the reference measures with Nsight's
    --cache-control all, i.e. flushed caches)."""
    thrash = torch.empty(512 * 1024 * 1024, dtype=torch.float16, device="cuda")
    times = []
    for i in range(samples):
        thrash.fill_(float(i))
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    del thrash
    times.sort()
    return times[len(times) // 2]


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


PMC_MODES = ["spmm", "spmm_largest", "spmm_slab_50", "spmm_slab_90", "spmm_dma", "spmm_split_rows", "spmm_row_parts", "sddmm", "attention",
             "attention_window"]


def largest_sweep_point(cv):
    """The largest single-GPU point of the ResNet-50-shaped sweep: M = 2048, K = 4608, N = 256, V = 8, 90 %."""
    pat = cv.random_values(cv.uniform_pattern(2048 // 8, 4608, 0.9, seed=3, vec_length=8), seed=4)
    return pat, cv.dense_uniform(4608, 256, seed=5)


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
    args = ap.parse_args()
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

    # ---- cold caches (how the reference measures: Nsight --cache-control all)
    cold_ms = time_cold(torch, step)
    cold_floor_ms = time_cold(torch, probe(512))  # what the same method reads for a kernel that does nothing
    cold_dense_ms = time_cold(torch, lambda: torch.matmul(Ad, Bd, out=dense_out))
    cold_large_ms = time_cold(torch, lambda: lprob.spmm(lBd, kernel="wmma", out=lout), samples=10)
    cold_sddmm_ms = time_cold(torch, sddmm_step, samples=10)
    cold_attn_ms = time_cold(torch, lambda: layer.forward(q, kk_, vv, scores=scores, out=ctx), samples=10)

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
                        frac_cold=alg_bytes / (cold_ms * 1e-3) * 1e-9 / HBM_PEAK_GBS,
                        frac_cold_note="from extra.cold_cache.spmm_config2_us, which contains the %.1f us the same "
                                       "method reads for an empty kernel" % (cold_floor_ms * 1e3),
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
            "cold_cache": {"method": "HIP events round one eager launch that follows a 1 GiB fill; the same method reads "
                                     "empty_kernel_us for a kernel that does nothing on config 2's grid, so only the "
                                     "differences to it are kernel time",
                           "empty_kernel_us": cold_floor_ms * 1e3,
                           "spmm_config2_us": cold_ms * 1e3, "dense_gemm_config2_us": cold_dense_ms * 1e3,
                           "spmm_largest_us": cold_large_ms * 1e3, "sddmm_config4_us": cold_sddmm_ms * 1e3,
                           "attention_config5_us": cold_attn_ms * 1e3},
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
            "fine_grained_paths": {
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
