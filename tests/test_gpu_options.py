"""Launch-shape options: per-thread overrides do not leak between threads or calls, and the automatic launch
shapes stay close to the best hand-picked ones on the headline configurations."""
import threading

import numpy as np
import pytest
import torch

from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from vectorsparse_amd.benchmark_common import time_launches

pytestmark = pytest.mark.gpu


def _long_rows():
    # rows of about 2000 vectors and an fp32 output: the number of waves per row changes the order of the fp32
    # summation, which shows in the low bits of the result and so tells which launch shape a call really used
    pat = cv.random_values(cv.binomial_pattern(8, 4096, 0.5, seed=3, vec_length=8), seed=4)
    return pat, cv.dense_uniform(4096, 128, seed=5)


def test_thread_options_do_not_leak_between_threads_and_streams(gpu):
    pat, B = _long_rows()
    prob = ops.DeviceProblem(pat)
    Bd = torch.from_numpy(B).cuda()

    def run(stream=None):
        out = torch.empty((pat.m, 128), dtype=torch.float32, device="cuda")
        prob.spmm(Bd, out=out, stream=stream)
        return out

    expect = {}
    for waves in (1, 16):
        with _lib.thread_options(spmm_waves=waves):
            expect[waves] = run().clone()
    torch.cuda.synchronize()
    assert not torch.equal(expect[1], expect[16]), "the two shapes must be distinguishable by their bits"
    base = run().clone()                           # outside the blocks the automatic shape is back
    torch.cuda.synchronize()

    failures = []

    def worker(waves):
        stream = torch.cuda.Stream()
        with _lib.thread_options(spmm_waves=waves):
            for _ in range(200):
                got = run(stream)
                stream.synchronize()
                if not torch.equal(got, expect[waves]):
                    failures.append(waves)
                    return

    threads = [threading.Thread(target=worker, args=(w,)) for w in (1, 16)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, "a thread saw another thread's launch shape: %s" % failures

    # one thread, two streams, the option changed between the calls: every call uses what was set last
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(20):
        with _lib.thread_options(spmm_waves=1):
            a = run(s1)
        with _lib.thread_options(spmm_waves=16):
            b = run(s2)
        c = run(s1)
        torch.cuda.synchronize()
        assert torch.equal(a, expect[1]) and torch.equal(b, expect[16]) and torch.equal(c, base)
    # the process-wide default is what threads without overrides see
    try:
        _lib.set_option("spmm_waves", 16)
        torch.cuda.synchronize()
        assert torch.equal(run(), expect[16])
        with _lib.thread_options(spmm_waves=1):
            assert torch.equal(run(), expect[1])
    finally:
        _lib.set_option("spmm_waves", 0)
    with pytest.raises(_lib.VSparseError):
        with _lib.thread_options(spmm_waves=99):
            pass


def _best_of(fn, settings):
    """(time of the automatic shape, best time over hand-picked shapes), each the minimum of three medians."""
    def t():
        return min(time_launches(torch, fn, iters=100) for _ in range(3))
    auto = t()
    best = auto
    for kw in settings:
        with _lib.thread_options(**kw):
            best = min(best, t())
    return auto, best


def test_automatic_launch_shapes_are_close_to_the_best_on_the_headline_configs(gpu):
    """Config 2 (SpMM) and config 4 (SDDMM): the shape the library picks by itself must be within 10 % of the best
    of the hand-picked shapes, so that a regression of the launch heuristics does not pass silently."""
    pat = cv.random_values(cv.binomial_pattern(64, 4608, 0.9, seed=1, vec_length=8), seed=101)
    Bd = torch.from_numpy(cv.dense_uniform(4608, 256, seed=201)).cuda()
    prob = ops.DeviceProblem(pat, sort=True)
    out = torch.empty((512, 256), dtype=torch.float16, device="cuda")
    auto, best = _best_of(lambda: prob.spmm(Bd, out=out),
                          [dict(spmm_cols_per_lane=c, spmm_waves=w, spmm_pipe=p) for c in (4, 8) for w in (4, 8, 16)
                           for p in (1, 2)])
    print("config 2 SpMM: automatic %.2f us, best override %.2f us" % (auto, best))
    assert auto <= 1.10 * best

    # the largest point of the sweep at the headline sparsity, reference-shaped and hinted entry
    big = cv.random_values(cv.uniform_pattern(256, 4608, 0.9, seed=3, vec_length=8), seed=102)
    bprob = ops.DeviceProblem(big)
    bout = torch.empty((2048, 256), dtype=torch.float16, device="cuda")
    for hint in (False, True):
        auto, best = _best_of(lambda: bprob.spmm(Bd, out=bout, row_length_hint=hint),
                              [dict(spmm_cols_per_lane=8, spmm_waves=w, spmm_steps=st, spmm_pipe=p)
                               for w in (2, 4, 8) for st, p in ((2, 1), (2, 2), (4, 1))])
        print("2048 x 4608 at 90 %%, hints %d: automatic %.2f us, best override %.2f us" % (hint, auto, best))
        assert auto <= 1.10 * best

    for K, s in ((64, 0.9), (128, 0.9), (64, 0.95), (128, 0.95)):
        mask = cv.uniform_pattern(256, 2048, s, seed=4, vec_length=8)
        lhs = torch.from_numpy(cv.dense_normal(2048, K, seed=14)).cuda()
        rhs = torch.from_numpy(cv.dense_normal(2048, K, seed=24)).cuda()
        sprob = ops.DeviceProblem(mask)
        sout = torch.empty((mask.nnz_vec, 8), dtype=torch.float16, device="cuda")
        auto, best = _best_of(lambda: sprob.sddmm(lhs, rhs, out=sout, algorithm=1),
                              [dict(sddmm_group=g, sddmm_slots=sl) for g in (1, 2, 4) for sl in (4, 8, 16)])
        print("config 4 SDDMM K=%d s=%g: automatic %.2f us, best override %.2f us" % (K, s, auto, best))
        assert auto <= 1.10 * best
