"""SpMM parity on the GPU: HIP kernels through the C ABI vs the CPU oracle (same seeded inputs).

Tolerance (written in tests/util.py): max relative error <= 1e-2 with the denominator floored at
1e-2*rms(ref), and zero elements beyond the reference's own 0.5 absolute criterion.  Pattern
arrays must come back byte-identical.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity, retired_variants_built

pytestmark = pytest.mark.gpu


def _run(pat, B, kernel, sort=False, out_dtype=torch.float16, device="cuda"):
    prob = ops.DeviceProblem(pat, sort=sort, device=device)
    Bd = torch.from_numpy(B).to(device)
    k = B.shape[1]
    # canary rows either side of the output catch out-of-range writes
    pad = 64
    buf = torch.full((pat.m + 2 * pad, k), 12345.0, dtype=out_dtype, device=device)
    out = buf[pad:pad + pat.m]
    prob.spmm(Bd, kernel=kernel, out=out)
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert np.all(host[:pad] == 12345.0) and np.all(host[pad + pat.m:] == 12345.0), "wrote outside the output"
    assert np.array_equal(prob.row_offsets.cpu().numpy(), pat.row_offsets)
    assert np.array_equal(prob.column_indices.cpu().numpy(), pat.column_indices)
    return host[pad:pad + pat.m]


def _oracle(pat, B):
    return co.spmm_host_ref_f32(pat.m_vec, pat.vec_length, B.shape[1], pat.n, pat.row_offsets,
                                pat.column_indices, pat.values, B)


def _kernels(V):
    return ["wmma", "cuda"]


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_config1_oracle_case(gpu, kernel):
    # M=256, K=256, V=4, N=128, 90 % sparse, exactly 26 vectors per row
    pat = cv.random_values(cv.uniform_pattern(64, 256, 0.9, seed=0, vec_length=4), seed=100)
    B = cv.dense_uniform(256, 128, seed=200)
    assert_parity(_run(pat, B, kernel), _oracle(pat, B), "config1/" + kernel)


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
@pytest.mark.parametrize("sort", [False, True])
def test_config2_resnet_shape(gpu, kernel, sort):
    # M=512, K=4608, V=8, N=256, 90 % sparse, binomial row lengths
    pat = cv.random_values(cv.binomial_pattern(64, 4608, 0.9, seed=1, vec_length=8), seed=101)
    B = cv.dense_uniform(4608, 256, seed=201)
    assert_parity(_run(pat, B, kernel, sort=sort), _oracle(pat, B), "config2/%s/sort=%d" % (kernel, sort))


SWEEP = [
    # (M, K, sparsity) subset of the ResNet-50-like grid, N = 256
    (64, 64, 0.5), (128, 147, 0.7), (256, 576, 0.8), (1024, 1152, 0.95), (2048, 2304, 0.98), (2048, 4608, 0.9),
]


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("shape", SWEEP, ids=lambda s: "M%d_K%d_s%g" % s)
def test_config3_sweep_points(gpu, V, shape):
    M, K, s = shape
    seed = (M * 31 + K * 7 + int(s * 100) * 3 + V) % 100000
    pat = cv.random_values(cv.uniform_pattern(M // V, K, s, seed=seed, vec_length=V), seed=seed + 1)
    B = cv.dense_uniform(K, 256, seed=seed + 2)
    ref = _oracle(pat, B)
    for kernel in _kernels(V):
        assert_parity(_run(pat, B, kernel), ref, "sweep M%d K%d s%g V%d %s" % (M, K, s, V, kernel))


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_ragged_rows_and_empty_rows(gpu, V, kernel):
    # lengths 0, 1, 15, 16, 17, 31, 33, 300 ... exercise the padded tail of every tile size
    lengths = np.array([0, 1, 15, 16, 17, 0, 31, 33, 64, 65, 300, 2, 0, 128, 7, 0], dtype=np.int64)
    n = 320
    rng = np.random.default_rng(5)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    pat = cv.random_values(cv.ColVecCSR(len(lengths), n, V, ro, ci).validate(), seed=6)
    B = cv.dense_uniform(n, 192, seed=7)
    got = _run(pat, B, kernel)
    assert_parity(got, _oracle(pat, B), "ragged V%d %s" % (V, kernel))
    for i in np.nonzero(lengths == 0)[0]:
        assert not got[i * V:(i + 1) * V].any(), "empty vector row %d must be written as zeros" % i


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("steps", [1, 2, 4])
@pytest.mark.parametrize("cpl", [4, 8])
def test_steps_in_flight_variants_keep_parity(gpu, V, steps, cpl):
    """The MFMA kernel with one, two or four 32-vector steps of gathered rows in flight per wave: rows that end
    inside a block (1, 33, 65, 127, 129 vectors), empty rows, rows of many blocks, and every wave count - including
    more waves than a row has blocks."""
    if steps == 4 and not retired_variants_built():
        pytest.skip("four steps in flight are compiled only with VS_RETIRED_VARIANTS=1")
    lengths = np.array([0, 1, 33, 64, 65, 0, 127, 128, 129, 300, 2, 0, 700, 7, 96, 0], dtype=np.int64)
    n = 768
    rng = np.random.default_rng(50 + V)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    pat = cv.random_values(cv.ColVecCSR(len(lengths), n, V, ro, ci).validate(), seed=51)
    for N in (64, 136, 256):
        B = cv.dense_uniform(n, N, seed=N)
        ref = _oracle(pat, B)
        for waves in (0, 1, 3, 8, 16):
            with _lib.thread_options(spmm_steps=steps, spmm_cols_per_lane=cpl, spmm_waves=waves):
                got = _run(pat, B, "wmma")
                got32 = _run(pat, B, "wmma", out_dtype=torch.float32) if waves in (0, 3) else None
            assert_parity(got, ref, "steps=%d cpl=%d waves=%d N=%d" % (steps, cpl, waves, N))
            if got32 is not None:
                assert_parity(got32, ref, "fp32 out, steps=%d cpl=%d waves=%d N=%d" % (steps, cpl, waves, N))
            if steps == 2:
                # the walk that pipelines successive blocks of a row and the plain one multiply and add in the same
                # order: same bits
                for pipe in (1, 2):
                    with _lib.thread_options(spmm_steps=steps, spmm_cols_per_lane=cpl, spmm_waves=waves, spmm_pipe=pipe):
                        other = _run(pat, B, "wmma")
                    assert_parity(other, ref, "pipe=%d cpl=%d waves=%d N=%d" % (pipe, cpl, waves, N))
                    if pipe == 1:
                        plain = other
                assert np.array_equal(plain, other), "pipelined and plain walks differ, cpl=%d waves=%d N=%d" % (cpl, waves, N)


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
@pytest.mark.parametrize("V", [1, 8])
def test_columns_in_any_order_within_a_row(gpu, kernel, V):
    """The format does not promise ascending columns within a row (the reference's loops take them as they come,
    spmm_benchmark.cpp:66-86): rows shuffled in place, long and short ones."""
    rng = np.random.default_rng(70 + V)
    lengths = np.array([0, 5, 64, 65, 700, 33, 1500, 128], dtype=np.int64)
    n = 1600
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    ci = ci.copy()
    for i in range(len(lengths)):
        rng.shuffle(ci[ro[i]:ro[i + 1]])
    pat = cv.random_values(cv.ColVecCSR(len(lengths), n, V, ro, ci), seed=71)
    B = cv.dense_uniform(n, 136, seed=72)
    assert_parity(_run(pat, B, kernel), _oracle(pat, B), "shuffled columns V%d %s" % (V, kernel))


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_all_rows_empty(gpu, kernel):
    pat = cv.ColVecCSR(8, 64, 8, np.zeros(9, np.int32), np.zeros(0, np.int32), np.zeros((0, 8), np.float16))
    B = cv.dense_uniform(64, 64, seed=1)
    got = _run(pat, B, kernel)
    assert got.shape == (64, 64) and not got.any()


@pytest.mark.parametrize("N", [1, 3, 4, 8, 12, 24, 30, 64, 66, 72, 136, 147, 512, 1000, 1001])
@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_dense_width_edges(gpu, N, kernel):
    # any dense width on both paths (the reference has no bounds check at all, src/wmma_spmm.cu:362-384): widths
    # that are not a multiple of 4 (MFMA) / 8 (fine-grained) take the kernels that move the operands half by half;
    # odd widths make every row of B and of the output start at an odd half
    pat = cv.random_values(cv.binomial_pattern(24, 200, 0.8, seed=N, vec_length=8), seed=N + 1)
    B = cv.dense_uniform(200, N, seed=N + 2)
    ref = _oracle(pat, B)
    assert_parity(_run(pat, B, kernel), ref, "N=%d %s" % (N, kernel))
    if N in (3, 30, 147, 1001):
        assert_parity(_run(pat, B, kernel, out_dtype=torch.float32, sort=True), ref, "N=%d %s fp32 out" % (N, kernel))


@pytest.mark.parametrize("V", [1, 2, 4])
@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_odd_dense_widths_every_vector_length(gpu, V, kernel):
    lengths = np.array([0, 1, 15, 33, 64, 65, 300, 2, 0, 7], dtype=np.int64)
    rng = np.random.default_rng(5)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), 320, lengths)
    pat = cv.random_values(cv.ColVecCSR(len(lengths), 320, V, ro, ci).validate(), seed=6)
    for N in (5, 66, 131):
        B = cv.dense_uniform(320, N, seed=N)
        assert_parity(_run(pat, B, kernel), _oracle(pat, B), "V%d N=%d %s" % (V, N, kernel))


def test_dense_width_multiple_of_4_on_mfma_path(gpu):
    pat = cv.random_values(cv.binomial_pattern(24, 100, 0.7, seed=3, vec_length=4), seed=4)
    for N in (4, 12, 68, 132, 2, 6, 70):
        B = cv.dense_uniform(100, N, seed=N)
        assert_parity(_run(pat, B, "wmma"), _oracle(pat, B), "N=%d wmma" % N)


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_skewed_rows_and_swizzle_invariance(gpu, kernel):
    # one very long row among short ones; the result must not depend on the row swizzle at all
    lengths = np.full(40, 20, dtype=np.int64)
    lengths[17] = 1500
    lengths[3] = 700
    rng = np.random.default_rng(11)
    ro, ci = cv._pattern_from_lengths(rng, 40, 2048, lengths)
    pat = cv.random_values(cv.ColVecCSR(40, 2048, 8, ro, ci), seed=12)
    B = cv.dense_uniform(2048, 256, seed=13)
    a = _run(pat, B, kernel, sort=False)
    b = _run(pat, B, kernel, sort=True)
    assert_parity(a, _oracle(pat, B), "skew " + kernel)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), "row swizzle changed the bits"


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_fp32_output_overload(gpu, kernel):
    pat = cv.random_values(cv.binomial_pattern(32, 512, 0.9, seed=21, vec_length=8), seed=22)
    B = cv.dense_uniform(512, 128, seed=23)
    got = _run(pat, B, kernel, out_dtype=torch.float32)
    assert got.dtype == np.float32
    assert_parity(got, _oracle(pat, B), "fp32 out " + kernel)


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_subnormal_values_keep_exact_products(gpu, kernel, V):
    """fp16 subnormals times large rhs entries: every product is exact in fp32 (the host loop's arithmetic,
    spmm_benchmark.cpp:79-81), so the fp32 output equals the count of nonzeros times 2^-10 exactly - on MFMA,
    on v_fma_mix_f32 (V = 1) and on v_dot2_f32_f16 (V >= 2) alike; a path that flushed them would return zeros."""
    pat = cv.uniform_pattern(16, 96, 0.5, seed=41, vec_length=V)
    vals = np.full((pat.nnz_vec, V), 2.0 ** -20, dtype=np.float16)
    pat = cv.ColVecCSR(pat.m_vec, pat.n, V, pat.row_offsets, pat.column_indices, vals)
    B = np.full((96, 64), 1024.0, dtype=np.float16)
    got = _run(pat, B, kernel, out_dtype=torch.float32)
    want = np.repeat(np.diff(pat.row_offsets), V).astype(np.float32)[:, None] * np.float32(2.0 ** -10)
    assert np.array_equal(got, np.broadcast_to(want, got.shape))
    assert np.array_equal(_oracle(pat, B), got)


def test_launch_shape_overrides_keep_parity(gpu):
    pat = cv.random_values(cv.binomial_pattern(16, 1024, 0.8, seed=31, vec_length=8), seed=32)
    B = cv.dense_uniform(1024, 256, seed=33)
    ref = _oracle(pat, B)
    try:
        for cpl in (4, 8):
            for waves in (1, 2, 3, 8, 16):
                _lib.set_option("spmm_cols_per_lane", cpl)
                _lib.set_option("spmm_waves", waves)
                assert_parity(_run(pat, B, "wmma"), ref, "cpl=%d waves=%d" % (cpl, waves))
        for waves in (1, 2, 4):
            _lib.set_option("spmm_waves", waves)
            assert_parity(_run(pat, B, "cuda"), ref, "cuda waves=%d" % waves)
    finally:
        _lib.set_option("spmm_cols_per_lane", 0)
        _lib.set_option("spmm_waves", 0)


def test_deterministic_and_linear(gpu):
    pat = cv.random_values(cv.binomial_pattern(64, 4608, 0.9, seed=1, vec_length=8), seed=101)
    B = cv.dense_uniform(4608, 256, seed=201)
    a = _run(pat, B, "wmma")
    b = _run(pat, B, "wmma")
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    # scaling the values by a power of two scales the result exactly
    doubled = pat.with_values(pat.values * np.float16(2))
    c = _run(doubled, B, "wmma")
    normal = np.abs(a) >= 2.0 ** -13      # doubling commutes with fp16 rounding outside the subnormal range
    assert np.array_equal(c[normal], (a * np.float16(2))[normal])


def test_wrong_dtype_and_host_tensor_are_rejected(gpu):
    pat = cv.random_values(cv.uniform_pattern(4, 32, 0.5, seed=1, vec_length=4), seed=2)
    prob = ops.DeviceProblem(pat)
    B = torch.ones((32, 64), dtype=torch.float32, device="cuda")
    with pytest.raises(TypeError):
        prob.spmm(B)
    with pytest.raises(ValueError):
        prob.spmm(torch.ones((32, 64), dtype=torch.float16))


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_row_length_hint_changes_the_launch_shape_not_the_result(gpu, kernel):
    # the batched entry point takes the pattern's nonzero count: any value (right, wrong, absent) must give
    # parity, and the right one the same bits as the reference-shaped entry point up to summation order
    for (m_vec, n, s, V) in ((64, 4608, 0.9, 8), (256, 1152, 0.98, 8), (96, 2304, 0.5, 2), (40, 640, 0.95, 1)):
        pat = cv.random_values(cv.binomial_pattern(m_vec, n, s, seed=m_vec, vec_length=V), seed=9)
        B = cv.dense_uniform(n, 128, seed=10)
        ref = _oracle(pat, B)
        prob = ops.DeviceProblem(pat, sort=True)
        Bd = torch.from_numpy(B).cuda()
        for hint in (pat.nnz_vec, -1, 0, 1, 50 * pat.nnz_vec):
            out = torch.empty((1, pat.m, 128), dtype=torch.float16, device="cuda")
            ops.spmm_batched(pat.m_vec, V, 128, n, prob.row_indices, prob.row_offsets, prob.column_indices,
                             prob.values, Bd, out, kernel=kernel, nonzeros_vec=hint)
            torch.cuda.synchronize()
            assert_parity(out[0].cpu().numpy(), ref, "hint %d on %s" % (hint, (m_vec, n, s, V)))
            for longest in (int(np.diff(pat.row_offsets).max()), 0, 1 << 30):
                ops.spmm_batched(pat.m_vec, V, 128, n, prob.row_indices, prob.row_offsets, prob.column_indices,
                                 prob.values, Bd, out, kernel=kernel, nonzeros_vec=hint, longest_row_vec=longest)
                torch.cuda.synchronize()
                assert_parity(out[0].cpu().numpy(), ref, "hints %d, %d on %s" % (hint, longest, (m_vec, n, s, V)))
        hinted = prob.spmm(Bd, kernel=kernel, row_length_hint=True)
        torch.cuda.synchronize()
        assert_parity(hinted.cpu().numpy(), ref, "DeviceProblem hinted")


def test_longest_row_hint_on_heavy_tailed_rows(gpu):
    """A few rows far longer than the mean (one of them dense): the hinted launch gives the long rows more
    waves; parity with the oracle either way and with every wave count forced by hand."""
    rng = np.random.default_rng(5)
    m_vec, n, V, N = 192, 2048, 8, 128
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 40, n).astype(np.int64)
    lengths[7] = n
    lengths[100] = 0
    ro, ci = cv._pattern_from_lengths(rng, m_vec, n, lengths)
    pat = cv.random_values(cv.ColVecCSR(m_vec, n, V, ro, ci), seed=6)
    assert lengths.max() > 4 * lengths.mean()
    B = cv.dense_uniform(n, N, seed=7)
    ref = _oracle(pat, B)
    Bd = torch.from_numpy(B).cuda()
    for sort in (False, True):
        prob = ops.DeviceProblem(pat, sort=sort)
        assert prob.longest_row_vec == n
        plain = prob.spmm(Bd)
        hinted = prob.spmm(Bd, row_length_hint=True)
        torch.cuda.synchronize()
        assert_parity(plain.cpu().numpy(), ref, "heavy tail, reference-shaped entry")
        assert_parity(hinted.cpu().numpy(), ref, "heavy tail, hinted")


@pytest.mark.parametrize("V,m_vec", [(8, 1100), (1, 2500)])
@pytest.mark.parametrize("N", [64, 256])
def test_skewed_rows_on_a_grid_that_fills_the_chip(gpu, V, m_vec, N):
    """More workgroups than the chip holds at once: the launches keep a few waves per workgroup for rows far longer
    than expected and let a wave take several 64-vector blocks of a row (reference-shaped entry: lengths unknown;
    batched entry: mean and longest known).  Pareto lengths with a dense row, empty rows and rows that end inside
    a block, every guard setting, identity and sorted order."""
    rng = np.random.default_rng(90 + V)
    n = 2304
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.05) * 60, n).astype(np.int64)
    lengths[3] = n
    lengths[m_vec // 2] = n - 1
    lengths[10:14] = 0
    lengths[20:26] = [1, 63, 64, 65, 127, 129]
    ro, ci = cv._pattern_from_lengths(rng, m_vec, n, lengths)
    pat = cv.random_values(cv.ColVecCSR(m_vec, n, V, ro, ci).validate(), seed=91)
    B = cv.dense_uniform(n, N, seed=92)
    ref = _oracle(pat, B)
    Bd = torch.from_numpy(B).cuda()
    for sort in (False, True):
        prob = ops.DeviceProblem(pat, sort=sort)
        for guard, pipe in [(0, 0), (1, 0), (2, 0), (8, 0), (0, 1), (0, 2), (2, 2), (8, 2)]:
            with _lib.thread_options(spmm_guard_waves=guard, spmm_pipe=pipe):
                plain = prob.spmm(Bd)
            torch.cuda.synchronize()
            assert_parity(plain.cpu().numpy(), ref, "full grid, V%d N%d sort %d guard %d pipe %d" % (V, N, sort, guard, pipe))
        hinted = prob.spmm(Bd, row_length_hint=True)
        torch.cuda.synchronize()
        assert_parity(hinted.cpu().numpy(), ref, "full grid, hinted, V%d N%d sort %d" % (V, N, sort))
        # the long-row count of the sorted entry point is a hint: any count, in any order of the rows, gives the
        # same result (teams of waves for the first `long_rows` entries, one wave per row behind them)
        # (spmm_teams = 2: on every launch, not only where the library expects the team mapping to pay)
        for teams, long_rows, pipe in ([(2, x, 0) for x in (0, 1, 5, 64, m_vec - 1, m_vec, m_vec + 9)] +
                                       [(0, 1, 0), (0, 64, 0), (2, 5, 1), (2, 5, 2), (2, m_vec, 2), (1, 5, 2)]):
            out = torch.full((1, pat.m, N), 3.0, dtype=torch.float16, device="cuda")
            with _lib.thread_options(spmm_teams=teams, spmm_pipe=pipe):
                ops.spmm_batched(pat.m_vec, V, N, n, prob.row_indices, prob.row_offsets, prob.column_indices,
                                 prob.values, Bd, out, nonzeros_vec=pat.nnz_vec, longest_row_vec=n, long_rows=long_rows)
            torch.cuda.synchronize()
            assert_parity(out[0].cpu().numpy(), ref,
                          "full grid, %d long rows said (teams %d), V%d N%d sort %d" % (long_rows, teams, V, N, sort))
        with _lib.thread_options(spmm_teams=1):
            assert_parity(prob.spmm(Bd, row_length_hint=True).cpu().numpy(), ref, "teams for every row")


@pytest.mark.parametrize("V", [1, 2, 4, 8])
def test_lds_dma_gather_variant_keeps_parity(gpu, V):
    """The variant of the MFMA kernel whose gathered rows go global -> LDS directly and reach the MFMA through
    transposing LDS reads (option spmm_gather = 2): same contract, every wave count, ragged rows, dense-width
    edges, and the same bits for any row swizzle."""
    if not retired_variants_built():
        pytest.skip("the LDS-DMA gather is compiled only with VS_RETIRED_VARIANTS=1")
    lengths = np.array([0, 1, 15, 16, 17, 0, 31, 33, 64, 65, 300, 2, 0, 128, 7, 0], dtype=np.int64)
    rng = np.random.default_rng(5)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), 320, lengths)
    ragged = cv.random_values(cv.ColVecCSR(len(lengths), 320, V, ro, ci).validate(), seed=6)
    big = cv.random_values(cv.binomial_pattern(512 // V, 4608, 0.9, seed=1, vec_length=V), seed=101)
    try:
        _lib.set_option("spmm_gather", 2)
        for N in (8, 72, 128, 192, 1000):
            B = cv.dense_uniform(320, N, seed=N)
            ref = _oracle(ragged, B)
            for waves in (0, 1, 3, 16):
                _lib.set_option("spmm_waves", waves)
                got = _run(ragged, B, "wmma")
                assert_parity(got, ref, "dma gather V%d N%d waves %d" % (V, N, waves))
        _lib.set_option("spmm_waves", 0)
        B = cv.dense_uniform(4608, 256, seed=201)
        a = _run(big, B, "wmma", sort=False)
        b = _run(big, B, "wmma", sort=True)
        assert_parity(a, _oracle(big, B), "dma gather config-2 shape V%d" % V)
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), "row swizzle changed the bits"
        assert_parity(_run(big, B, "wmma", out_dtype=torch.float32), _oracle(big, B), "dma gather fp32 out")
    finally:
        _lib.set_option("spmm_gather", 0)
        _lib.set_option("spmm_waves", 0)
