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
