"""SDDMM parity on the GPU: HIP kernels through the C ABI vs the CPU oracle (same seeded inputs)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


def _run(pat, A, B, kernel, sort=False, out_dtype=torch.float16, algorithm=1, device="cuda"):
    prob = ops.DeviceProblem(pat, sort=sort, device=device)
    Ad = torch.from_numpy(A).to(device)
    Bd = torch.from_numpy(B).to(device)
    V = pat.vec_length
    pad = 128
    buf = torch.full((pat.nnz_vec + 2 * pad, V), 777.0, dtype=out_dtype, device=device)
    out = buf[pad:pad + pat.nnz_vec]
    prob.sddmm(Ad, Bd, kernel=kernel, out=out, algorithm=algorithm)
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert np.all(host[:pad] == 777.0) and np.all(host[pad + pat.nnz_vec:] == 777.0), "wrote outside the output"
    assert np.array_equal(prob.row_offsets.cpu().numpy(), pat.row_offsets)
    assert np.array_equal(prob.column_indices.cpu().numpy(), pat.column_indices)
    return host[pad:pad + pat.nnz_vec].reshape(-1)


def _oracle(pat, A, B):
    # fp32 flavour of the host loop: the comparison tolerance covers the final fp16 rounding
    return co.sddmm_host_ref_f32(pat.m_vec, A.shape[1], pat.vec_length, pat.row_offsets, pat.column_indices, A, B)


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
@pytest.mark.parametrize("K", [64, 128])
@pytest.mark.parametrize("sparsity", [0.9, 0.95])
def test_config4(gpu, kernel, K, sparsity):
    # M = N = 2048, V = 8, uniform mask
    seed = 4 + (K == 128) + 2 * (sparsity == 0.95)
    pat = cv.uniform_pattern(256, 2048, sparsity, seed=seed, vec_length=8)
    A = cv.dense_normal(2048, K, seed=seed + 10)
    B = cv.dense_normal(2048, K, seed=seed + 20)
    got = _run(pat, A, B, kernel)
    assert_parity(got, _oracle(pat, A, B), "config4 K%d s%g %s" % (K, sparsity, kernel))
    # the fp16 host loop itself (rounded output) agrees to within one rounding step
    ref16 = co.sddmm_host_ref_f16(pat.m_vec, K, 8, pat.row_offsets, pat.column_indices, A, B)
    assert_parity(got, ref16.astype(np.float32), "config4 vs fp16 host loop")


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("K", [8, 32, 64, 72, 128, 256, 320, 512, 1024])
def test_vec_lengths_and_contraction_sizes(gpu, V, K):
    pat = cv.binomial_pattern(96 // V, 300, 0.85, seed=V * 1000 + K, vec_length=V)
    A = cv.dense_normal(pat.m, K, seed=1)
    B = cv.dense_normal(300, K, seed=2)
    ref = _oracle(pat, A, B)
    for kernel in ("wmma", "cuda"):
        assert_parity(_run(pat, A, B, kernel), ref, "V%d K%d %s" % (V, K, kernel))


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("K", [1, 7, 12, 50, 100, 130])
def test_both_paths_take_any_k(gpu, V, K):
    """Contraction lengths off a multiple of 8 on both entry points and under every algorithm of the MFMA one (the
    whole of K is contracted; the reference's MMA kernels drop K % 64, src/wmma_sddmm.cu:88-120)."""
    pat = cv.binomial_pattern(48 // V, 100, 0.8, seed=V * 100 + K, vec_length=V)
    A = cv.dense_normal(pat.m, K, seed=3)
    B = cv.dense_normal(100, K, seed=4)
    ref = _oracle(pat, A, B)
    assert_parity(_run(pat, A, B, "cuda"), ref, "cuda V%d K%d" % (V, K))
    for algorithm in (0, 1, 2):
        assert_parity(_run(pat, A, B, "wmma", algorithm=algorithm), ref, "wmma V%d K%d algorithm %d" % (V, K, algorithm))
    assert_parity(_run(pat, A, B, "wmma", out_dtype=torch.float32), ref, "wmma f32 out V%d K%d" % (V, K))


@pytest.mark.parametrize("V", [1, 8])
@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_columns_in_any_order_within_a_row(gpu, V, kernel):
    """Mask rows shuffled in place: outputs stay aligned with the CSR positions (include/bm_test_utils.h:171-193
    takes the columns as they come)."""
    rng = np.random.default_rng(80 + V)
    lengths = np.array([0, 5, 64, 65, 300, 33, 17, 128], dtype=np.int64)
    n = 320
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    ci = ci.copy()
    for i in range(len(lengths)):
        rng.shuffle(ci[ro[i]:ro[i + 1]])
    pat = cv.ColVecCSR(len(lengths), n, V, ro, ci)
    A = cv.dense_normal(pat.m, 72, seed=81)
    B = cv.dense_normal(n, 72, seed=82)
    ref = _oracle(pat, A, B)
    for algorithm in ((0, 1, 2) if kernel == "wmma" else (1,)):
        assert_parity(_run(pat, A, B, kernel, algorithm=algorithm), ref, "shuffled columns V%d %s alg %d" % (V, kernel, algorithm))


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_ragged_and_empty_rows(gpu, V, kernel):
    lengths = np.array([0, 1, 15, 16, 17, 0, 31, 33, 64, 65, 300, 2, 0, 128, 7, 0], dtype=np.int64)
    rng = np.random.default_rng(5)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), 320, lengths)
    pat = cv.ColVecCSR(len(lengths), 320, V, ro, ci).validate()
    A = cv.dense_normal(pat.m, 64, seed=8)
    B = cv.dense_normal(320, 64, seed=9)
    assert_parity(_run(pat, A, B, kernel), _oracle(pat, A, B), "ragged V%d %s" % (V, kernel))


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_skew_swizzle_invariance_and_slots(gpu, kernel):
    lengths = np.full(40, 20, dtype=np.int64)
    lengths[17] = 1500
    lengths[3] = 700
    rng = np.random.default_rng(11)
    ro, ci = cv._pattern_from_lengths(rng, 40, 2048, lengths)
    pat = cv.ColVecCSR(40, 2048, 8, ro, ci)
    A = cv.dense_normal(pat.m, 128, seed=12)
    B = cv.dense_normal(2048, 128, seed=13)
    ref = _oracle(pat, A, B)
    a = _run(pat, A, B, kernel, sort=False)
    b = _run(pat, A, B, kernel, sort=True)
    assert_parity(a, ref, "skew " + kernel)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    try:
        for slots in (1, 2, 7, 64, 200):
            _lib.set_option("sddmm_slots", slots)
            c = _run(pat, A, B, kernel)
            assert np.array_equal(a.view(np.uint16), c.view(np.uint16)), "slots=%d changed the bits" % slots
    finally:
        _lib.set_option("sddmm_slots", 0)


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_fp32_output_overload(gpu, kernel):
    pat = cv.uniform_pattern(32, 512, 0.9, seed=21, vec_length=4)
    A = cv.dense_normal(pat.m, 64, seed=22)
    B = cv.dense_normal(512, 64, seed=23)
    got = _run(pat, A, B, kernel, out_dtype=torch.float32)
    assert got.dtype == np.float32
    assert_parity(got, _oracle(pat, A, B), "fp32 out " + kernel)


def test_algorithm_argument(gpu):
    pat = cv.uniform_pattern(16, 256, 0.9, seed=1, vec_length=8)
    A = cv.dense_normal(pat.m, 64, seed=2)
    B = cv.dense_normal(256, 64, seed=3)
    ref = _oracle(pat, A, B)
    outs = [_run(pat, A, B, "wmma", algorithm=alg) for alg in (0, 1, 2)]
    for o in outs:
        assert_parity(o, ref, "algorithm")
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])
    with pytest.raises(_lib.VSparseError):
        _run(pat, A, B, "wmma", algorithm=3)


@pytest.mark.parametrize("V", [1, 2, 4])
def test_automatic_algorithm_takes_the_fine_grained_kernel_on_small_masks_of_short_vectors(gpu, V):
    """algorithm 0 of the MFMA entry point: vectors of 1 to 4 rows fill at most a quarter of a matrix-core tile, so
    a mask of few nonzeros goes to the fine-grained kernel (the bits of cudaSddmm), a large one stays on MFMA
    (the bits of algorithm 1); both hold the oracle's tolerance."""
    small = cv.uniform_pattern(64 // V, 512, 0.95, seed=40 + V, vec_length=V)
    A = cv.dense_normal(small.m, 256, seed=41)
    B = cv.dense_normal(512, 256, seed=42)
    auto = _run(small, A, B, "wmma", algorithm=0)
    assert_parity(auto, _oracle(small, A, B), "algorithm 0, small mask, V%d" % V)
    assert np.array_equal(auto.view(np.uint16), _run(small, A, B, "cuda").view(np.uint16))
    large = cv.uniform_pattern(2048 // V, 2048, 0.5, seed=43 + V, vec_length=V)   # beyond every limit
    A = cv.dense_normal(large.m, 64, seed=44)
    B = cv.dense_normal(2048, 64, seed=45)
    auto = _run(large, A, B, "wmma", algorithm=0)
    assert np.array_equal(auto.view(np.uint16), _run(large, A, B, "wmma", algorithm=1).view(np.uint16))


def test_full_mask_equals_dense_product(gpu):
    V, m_vec, n, K = 8, 8, 96, 64
    ro = (np.arange(m_vec + 1) * n).astype(np.int32)
    ci = np.tile(np.arange(n, dtype=np.int32), m_vec)
    pat = cv.ColVecCSR(m_vec, n, V, ro, ci)
    A = cv.dense_normal(m_vec * V, K, seed=3)
    B = cv.dense_normal(n, K, seed=4)
    got = _run(pat, A, B, "wmma").reshape(m_vec, n, V).transpose(0, 2, 1).reshape(m_vec * V, n)
    dense = A.astype(np.float64) @ B.astype(np.float64).T
    assert_parity(got, dense, "full mask")


def test_sddmm_output_chains_into_spmm(gpu):
    # the [nnz_vec][V] output layout is exactly the `values` layout of SpMM
    V, K, N = 8, 64, 64
    pat = cv.band_strided_pattern(512, V, band_half_width=64, stride=64)
    Q = cv.dense_normal(512, K, seed=1)
    Kmat = cv.dense_normal(512, K, seed=2)
    W = cv.dense_uniform(512, N, seed=3)
    prob = ops.DeviceProblem(pat)
    scores = prob.sddmm(torch.from_numpy(Q).cuda(), torch.from_numpy(Kmat).cuda())
    prob.values = scores
    out = prob.spmm(torch.from_numpy(W).cuda())
    torch.cuda.synchronize()
    vals = scores.cpu().numpy()
    assert_parity(vals.reshape(-1), _oracle(pat, Q, Kmat), "chain sddmm")
    ref = co.spmm_host_ref_f32(pat.m_vec, V, N, 512, pat.row_offsets, pat.column_indices, vals, W)
    assert_parity(out.cpu().numpy(), ref, "chain spmm")


@pytest.mark.parametrize("V", [1, 2, 4, 8])
def test_algorithm_2_splits_the_nonzero_range_same_bits(gpu, V):
    """algorithm = 2 of wmmaSddmm (waves own ranges of nonzeros, not rows) gives the same bits as the row-slot
    schedule on uniform, ragged, heavily skewed and mostly empty patterns, for every contraction length class."""
    rng = np.random.default_rng(70 + V)
    n = 700
    patterns = {
        "uniform": cv.uniform_pattern(96, n, 0.9, seed=1, vec_length=V),
        "short rows": cv.uniform_pattern(300, n, 0.995, seed=2, vec_length=V),
    }
    lengths = np.minimum((rng.pareto(1.2, 150) + 0.05) * 40, n).astype(np.int64)
    lengths[::7] = 0
    lengths[3] = n
    ro, ci = cv._pattern_from_lengths(rng, 150, n, lengths)
    patterns["skewed with empty rows"] = cv.ColVecCSR(150, n, V, ro, ci)
    lengths = np.zeros(130, dtype=np.int64)
    lengths[[0, 64, 65, 129]] = [5, 1, 300, 17]
    ro, ci = cv._pattern_from_lengths(rng, 130, n, lengths)
    patterns["long runs of empty rows"] = cv.ColVecCSR(130, n, V, ro, ci)
    for name, mask in patterns.items():
        prob = ops.DeviceProblem(mask, sort=True)
        for K in (8, 40, 64, 104, 128, 200, 256):
            A = torch.from_numpy(cv.dense_normal(mask.m, K, seed=K)).cuda()
            B = torch.from_numpy(cv.dense_normal(n, K, seed=K + 1)).cuda()
            for dtype in (torch.float16, torch.float32):
                slot = prob.sddmm(A, B, kernel="wmma", out_dtype=dtype, algorithm=1)
                pad = torch.full((mask.nnz_vec + 32, V), 7.0, dtype=dtype, device="cuda")
                flat = pad[16:16 + mask.nnz_vec]
                prob.sddmm(A, B, kernel="wmma", out=flat, algorithm=2)
                torch.cuda.synchronize()
                assert torch.equal(slot, flat), "%s V%d K%d %s" % (name, V, K, dtype)
                assert bool((pad[:16] == 7.0).all()) and bool((pad[16 + mask.nnz_vec:] == 7.0).all())
        ref = co.sddmm_host_ref_f32(mask.m_vec, 64, V, mask.row_offsets, mask.column_indices,
                                    cv.dense_normal(mask.m, 64, seed=64), cv.dense_normal(n, 64, seed=65))
        got = prob.sddmm(torch.from_numpy(cv.dense_normal(mask.m, 64, seed=64)).cuda(),
                         torch.from_numpy(cv.dense_normal(n, 64, seed=65)).cuda(), kernel="wmma", algorithm=2)
        torch.cuda.synchronize()
        assert_parity(got.cpu().numpy().reshape(-1), ref, name)


def test_algorithm_2_batched_equals_unbatched(gpu):
    V, heads, n, K = 8, 3, 640, 64
    rng = np.random.default_rng(5)
    lengths = np.minimum((rng.pareto(1.3, 90) + 0.1) * 30, n).astype(np.int64)
    ro, ci = cv._pattern_from_lengths(rng, 90, n, lengths)
    mask = cv.ColVecCSR(90, n, V, ro, ci)
    prob = ops.DeviceProblem(mask)
    g = torch.Generator(device="cuda").manual_seed(1)
    A = torch.randn((heads, mask.m, K), device="cuda", generator=g).half()
    B = torch.randn((heads, n, K), device="cuda", generator=g).half()
    out = torch.empty((heads, mask.nnz_vec, V), dtype=torch.float16, device="cuda")
    ops.sddmm_batched(mask.m_vec, K, n, mask.nnz_vec, prob.row_indices, prob.row_offsets, prob.column_indices, A, B, out,
                      V, algorithm=2)
    torch.cuda.synchronize()
    for h in range(heads):
        one = prob.sddmm(A[h], B[h], algorithm=1)
        torch.cuda.synchronize()
        assert torch.equal(out[h], one), "head %d" % h


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_empty_contraction_writes_zeros(gpu, kernel, out_dtype):
    # k == 0: every sampled output is an empty sum (Host_sddmm, include/bm_test_utils.h:171-193, leaves 0)
    pat = cv.binomial_pattern(12, 80, 0.7, seed=3, vec_length=4)
    A = np.zeros((pat.m, 0), dtype=np.float16)
    B = np.zeros((80, 0), dtype=np.float16)
    got = _run(pat, A, B, kernel, out_dtype=out_dtype)
    assert got.shape == (pat.nnz,) and not got.any()
    ref = co.sddmm_host_ref_f32(pat.m_vec, 0, 4, pat.row_offsets, pat.column_indices, A, B)
    assert np.array_equal(ref, got.astype(np.float32))
