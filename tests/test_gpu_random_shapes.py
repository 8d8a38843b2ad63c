"""Randomised differential parity: many small random shapes, every kernel path, against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity, retired_variants_built

pytestmark = pytest.mark.gpu


def _random_pattern(rng, V):
    m_vec = int(rng.integers(1, 70))
    n = int(rng.integers(1, 700))
    kind = rng.integers(0, 4)
    if kind == 0:      # uniform density
        lengths = rng.binomial(n, rng.uniform(0.02, 0.6), size=m_vec)
    elif kind == 1:    # heavy tail
        lengths = np.minimum((rng.pareto(1.2, m_vec) + 0.1) * n * 0.05, n).astype(np.int64)
    elif kind == 2:    # many empty rows
        lengths = np.where(rng.random(m_vec) < 0.6, 0, rng.integers(1, n + 1, m_vec))
    else:              # dense rows
        lengths = np.full(m_vec, n)
    ro, ci = cv._pattern_from_lengths(rng, m_vec, n, lengths.astype(np.int64))
    return cv.ColVecCSR(m_vec, n, V, ro, ci).validate()


@pytest.mark.parametrize("seed", range(40))
def test_spmm_random(gpu, seed):
    rng = np.random.default_rng(1000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    pat = cv.random_values(_random_pattern(rng, V), seed=seed)
    N = int(rng.choice([4, 8, 16, 40, 64, 96, 128, 200, 256, 264, 384, 520]))
    B = cv.dense_uniform(pat.n, N, seed=seed + 1)
    ref = co.spmm_host_ref_f32(pat.m_vec, V, N, pat.n, pat.row_offsets, pat.column_indices, pat.values, B)
    prob = ops.DeviceProblem(pat, sort=bool(seed % 2))
    Bd = torch.from_numpy(B).cuda()
    what = "seed %d V%d m_vec%d n%d N%d nnz_vec%d" % (seed, V, pat.m_vec, pat.n, N, pat.nnz_vec)
    print(what, flush=True)
    assert_parity(prob.spmm(Bd, kernel="wmma").cpu().numpy(), ref, "wmma " + what)
    if N % 8 == 0:
        assert_parity(prob.spmm(Bd, kernel="cuda").cpu().numpy(), ref, "cuda " + what)


@pytest.mark.parametrize("seed", range(60))
def test_spmm_random_launch_shapes(gpu, seed):
    """Random patterns under random launch-shape overrides (waves, columns per lane, steps in flight, pipelined or
    plain walk, guard waves, blocks per wave, team mapping) through the reference-shaped entry and through the
    hinted batched one: every combination the options allow computes the same function."""
    from vectorsparse_amd import _lib
    rng = np.random.default_rng(5000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    pat = _random_pattern(rng, V)
    if seed % 3 == 0:   # long rows, so that waves walk several blocks
        n = int(rng.integers(700, 3000))
        lengths = np.minimum((rng.pareto(1.2, pat.m_vec) + 0.05) * n * 0.2, n).astype(np.int64)
        ro, ci = cv._pattern_from_lengths(rng, pat.m_vec, n, lengths)
        pat = cv.ColVecCSR(pat.m_vec, n, V, ro, ci).validate()
    pat = cv.random_values(pat, seed=seed)
    N = int(rng.choice([8, 64, 128, 136, 256, 264]))
    B = cv.dense_uniform(pat.n, N, seed=seed + 1)
    ref = co.spmm_host_ref_f32(pat.m_vec, V, N, pat.n, pat.row_offsets, pat.column_indices, pat.values, B)
    Bd = torch.from_numpy(B).cuda()
    prob = ops.DeviceProblem(pat, sort=bool(seed % 2))
    # (four steps in flight exist only in a library built with VS_RETIRED_VARIANTS=1; the draw is made either way,
    # so that the other options of a seed do not depend on the build)
    step_choice = (lambda x: x) if retired_variants_built() else (lambda x: 2 if x == 4 else x)
    for trial in range(4):
        opts = dict(spmm_waves=int(rng.choice([0, 0, 1, 2, 3, 4, 8, 16])), spmm_cols_per_lane=int(rng.choice([0, 4, 8])),
                    spmm_steps=step_choice(int(rng.choice([0, 1, 2, 2, 4]))), spmm_pipe=int(rng.choice([0, 1, 2, 2])),
                    spmm_guard_waves=int(rng.choice([0, 1, 2, 4, 8])),
                    spmm_blocks_per_wave=int(rng.choice([0, 1, 2, 8, 64])), spmm_teams=int(rng.choice([0, 1, 2])))
        hint = bool(rng.integers(0, 2))
        what = "seed %d trial %d V%d m_vec%d n%d N%d nnz_vec%d hint %d %s" % (seed, trial, V, pat.m_vec, pat.n, N,
                                                                              pat.nnz_vec, hint, opts)
        print(what, flush=True)
        with _lib.thread_options(**opts):
            got = prob.spmm(Bd, kernel="wmma", row_length_hint=hint)
        torch.cuda.synchronize()
        assert_parity(got.cpu().numpy(), ref, what)


@pytest.mark.parametrize("seed", range(40))
def test_sddmm_random(gpu, seed):
    rng = np.random.default_rng(2000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    pat = _random_pattern(rng, V)
    K = int(rng.choice([8, 16, 24, 32, 40, 64, 96, 128, 136, 256, 264, 520]))
    A = cv.dense_normal(pat.m, K, seed=seed + 1)
    B = cv.dense_normal(pat.n, K, seed=seed + 2)
    ref = co.sddmm_host_ref_f32(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B)
    prob = ops.DeviceProblem(pat, sort=bool(seed % 2))
    Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    what = "seed %d V%d m_vec%d n%d K%d nnz_vec%d" % (seed, V, pat.m_vec, pat.n, K, pat.nnz_vec)
    print(what, flush=True)
    for kernel in ("wmma", "cuda"):
        got = prob.sddmm(Ad, Bd, kernel=kernel).cpu().numpy().reshape(-1)
        assert_parity(got, ref, kernel + " " + what)
    if seed % 4 == 0:       # the cross-lane path with a contraction length that is not a multiple of 8
        K2 = K + int(rng.integers(1, 8))
        A2 = cv.dense_normal(pat.m, K2, seed=seed + 3)
        B2 = cv.dense_normal(pat.n, K2, seed=seed + 4)
        ref2 = co.sddmm_host_ref_f32(pat.m_vec, K2, V, pat.row_offsets, pat.column_indices, A2, B2)
        got = prob.sddmm(torch.from_numpy(A2).cuda(), torch.from_numpy(B2).cuda(), kernel="cuda")
        assert_parity(got.cpu().numpy().reshape(-1), ref2, "cuda K%d " % K2 + what)


def test_concurrent_streams_do_not_interfere(gpu):
    """The library keeps no per-call state: different problems launched back to back on two streams (no
    synchronisation between them) give the same bits as when each runs alone."""
    import torch
    from vectorsparse_amd import ops
    rng = np.random.default_rng(99)
    probs = []
    for i, (m_vec, n, V, k) in enumerate(((64, 4608, 8, 256), (300, 512, 2, 64), (128, 1024, 4, 128))):
        pat = cv.random_values(cv.binomial_pattern(m_vec, n, 0.9, seed=i, vec_length=V), seed=50 + i)
        B = torch.from_numpy(cv.dense_uniform(n, k, seed=60 + i)).cuda()
        A = torch.from_numpy(cv.dense_normal(pat.m, k, seed=70 + i)).cuda()
        R = torch.from_numpy(cv.dense_normal(n, k, seed=80 + i)).cuda()
        probs.append((ops.DeviceProblem(pat, sort=True), B, A, R))
    alone = []
    for prob, B, A, R in probs:
        alone.append((prob.spmm(B).clone(), prob.sddmm(A, R).clone()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = []
    for rep in range(20):
        for i, (prob, B, A, R) in enumerate(probs):
            s = streams[(i + rep) % 2]
            with torch.cuda.stream(s):
                outs.append((i, prob.spmm(B, stream=s), prob.sddmm(A, R, stream=s)))
    torch.cuda.synchronize()
    for i, c, d in outs:
        assert torch.equal(c, alone[i][0]) and torch.equal(d, alone[i][1])


def test_hip_graph_replays_equal_eager(gpu):
    """Every entry point is capturable (no allocation, no memset, no synchronisation inside): a captured
    SDDMM -> softmax -> SpMM chain plus the single-launch layer, replayed several times with eager work and
    synchronisations in between and fresh inputs each time, equals the eager result every time."""
    import torch
    from vectorsparse_amd import ops
    V, heads, seq, d = 8, 4, 512, 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=48, stride=64)
    layer = ops.SparseAttention(mask)
    layer.plan(d, d)                     # built outside the capture
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = (torch.randn((heads, seq, d), device="cuda", generator=g).half() for _ in range(3))
    scores = torch.empty((heads, mask.nnz_vec, V), dtype=torch.float16, device="cuda")
    out_chain = torch.empty((heads, seq, d), dtype=torch.float16, device="cuda")
    out_layer = torch.empty((heads, seq, d), dtype=torch.float16, device="cuda")

    def work():
        layer.forward(q, k, v, scores=scores, out=out_chain, fused=False)
        layer.forward(q, k, v, out=out_layer, fused="layer")

    work()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    for rep in range(4):
        for t in (q, k, v):
            t.copy_(torch.randn(t.shape, device="cuda", generator=g).half())   # new inputs, same buffers
        work()
        torch.cuda.synchronize()
        want_chain, want_layer = out_chain.clone(), out_layer.clone()
        out_chain.zero_()
        out_layer.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_chain, want_chain), "replay %d: chain" % rep
        assert torch.equal(out_layer, want_layer), "replay %d: layer" % rep
