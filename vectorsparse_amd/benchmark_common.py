"""Shared pieces of the two benchmark command lines."""
import os
import time

import numpy as np

from . import colvec_csr as cv


def load_pattern(bm, vec_length):
    """`bm` is a .smtx path, or `synthetic:M,K,sparsity,seed` (M scalar rows, uniform rows)."""
    if bm.startswith("synthetic:"):
        m, k, sparsity, seed = bm[len("synthetic:"):].split(",")
        m, k, sparsity, seed = int(m), int(k), float(sparsity), int(seed)
        if m % vec_length:
            raise SystemExit("synthetic M must be a multiple of v")
        return cv.uniform_pattern(m // vec_length, k, sparsity, seed, vec_length)
    if not os.path.exists(bm):
        raise SystemExit("benchmark file not found: %s" % bm)
    return cv.read_smtx(bm, vec_length)


def time_launches(torch, fn, iters=50, warmup=5, replays=5):
    """Device time of one call in microseconds: HIP events on the launch stream around `iters` calls
    replayed from a HIP graph (host launch cost is not part of it); the median of `replays` replays, because
    a single replay now and then runs at twice its usual time (clock ramp after an idle gap)."""
    for _ in range(warmup):
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
        for _ in range(iters):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(max(1, replays)):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) * 1e3 / iters)
    times.sort()
    return times[len(times) // 2]


def verdict(name, got, ref):
    """The reference's acceptance test (|diff| > 0.5 counted, spmm_benchmark.cpp:206-225) plus the
    max relative error with the denominator floored at 1e-2 * rms(ref)."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    errors = int(np.sum(np.abs(got - ref) > 0.5))
    floor = 1e-2 * float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    rel = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), max(floor, 1e-30)))) if ref.size else 0.0
    if errors > 0:
        print("%s does not agree with SEQUENTIAL! %d errors!" % (name, errors))
    else:
        print("Results verified: they agree.")
    print("max relative error %.3e (%s 1e-2)" % (rel, "<=" if rel <= 1e-2 else ">"))
    return errors == 0 and rel <= 1e-2


_SDDMM_ALGORITHMS = {0: "wmma", 1: "mma_reg", 2: "mma_shfl", 3: "mma_arch"}


def duration_csv_path(root, bm, dim_k, dim_v, kernel, job, sort=True, precision="half", sddmm_alg=1):
    """Path of the per-run duration file for one (benchmark, k, v, kernel) point, laid out the way the
    reference's plot scripts look it up (file_name_server.py:6-45): `<root>/<job>/<bm>_<kernel>_<precision>
    [_sort][_<sddmm algorithm>]_k<k>_v<v>.csv`, where `bm` is the benchmark's name below the data set root
    without its extension and `kernel` is "wmma", "cuda" or "dense"."""
    if kernel not in ("wmma", "cuda", "dense"):
        raise ValueError("kernel must be wmma, cuda or dense")
    if job not in ("spmm", "sddmm"):
        raise ValueError("job must be spmm or sddmm")
    name = bm[:-len(".smtx")] if bm.endswith(".smtx") else bm
    name += "_%s_%s" % (kernel, "half" if precision == "half" else "single")
    if sort:
        name += "_sort"
    if job == "sddmm" and kernel == "wmma":
        name += "_" + _SDDMM_ALGORITHMS.get(sddmm_alg, "mma_reg")
    return os.path.join(root, job, "%s_k%d_v%d.csv" % (name, dim_k, dim_v))


def write_duration_csv(path, kernel_name, duration_us, process="vectorsparse_amd"):
    """One profiler-style record per kernel launch of the run: the reference's reader
    (file_name_server.py:57-81) sums, over the rows of the file, the value in the next-to-last field of every
    row whose fourth field from the end contains "Duration", with the unit ("nsecond") in between."""
    os.makedirs(os.path.dirname(path), exist_ok=True)
    header = ["ID", "Process ID", "Process Name", "Host Name", "Kernel Name", "Kernel Time", "Context", "Stream",
              "Section Name", "Metric Name", "Metric Unit", "Metric Value", "Rule Name"]
    stamp = time.strftime("%Y-%b-%d %H:%M:%S")
    with open(path, "w") as f:
        f.write(",".join('"%s"' % h for h in header) + "\n")
        row = ["0", str(os.getpid()), process, "127.0.0.1", kernel_name, stamp, "1", "0", "GPU Speed Of Light",
               "Duration", "nsecond", "%.0f" % (duration_us * 1e3), ""]
        f.write(",".join('"%s"' % x for x in row[:-1]) + ",\n")
