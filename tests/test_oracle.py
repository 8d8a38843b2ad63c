"""Pins the CPU oracle (C and numpy restatements) without any GPU."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

from oracle import c_oracle as co
from oracle import numpy_oracle as no
from vectorsparse_amd import colvec_csr as cv

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _problem(m_vec, n, V, sparsity, seed, skew=False):
    make = cv.binomial_pattern if skew else cv.uniform_pattern
    return cv.random_values(make(m_vec, n, sparsity, seed, V), seed + 1)


# ------------------------------------------------------------------ fp16 conversions

def test_half_to_float_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([co.half_to_float(int(b)) for b in bits], dtype=np.float32)
    finite = ~np.isnan(ref)
    assert np.array_equal(ref.view(np.uint32)[finite], got.view(np.uint32)[finite])
    assert np.isnan(got[~finite]).all()


def test_float_to_half_matches_ieee_rne():
    rng = np.random.default_rng(0)
    # random bit patterns concentrated on the half range, plus every half value, its neighbours
    # and the exact midpoints between consecutive halves (ties-to-even cases)
    halves = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    samples = np.concatenate([
        halves, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
        rng.uniform(-70000, 70000, 20000).astype(np.float32),
        (rng.standard_normal(20000) * 1e-6).astype(np.float32),
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 65504, 65519.99, 65520, 65536, 2 ** -24, 2 ** -25,
                  np.nextafter(np.float32(2 ** -25), np.float32(1)), 2 ** -14, 6.0975552e-05], dtype=np.float32),
    ])
    samples = np.concatenate([samples, -samples])
    with np.errstate(over="ignore", invalid="ignore"):
        ref = samples.astype(np.float16).view(np.uint16)
    got = np.array([co.float_to_half(x) for x in samples], dtype=np.uint16)
    nan = np.isnan(samples)
    assert np.array_equal(ref[~nan], got[~nan])
    assert np.all((got[nan] & 0x7c00) == 0x7c00) and np.all((got[nan] & 0x3ff) != 0)


# ------------------------------------------------------------------ operand generator

def test_generator_known_answers_from_libstdcxx():
    with open(os.path.join(GOLDEN, "minstd_uniform.json")) as f:
        gold = json.load(f)
    assert gold["engine_min"] == 1 and gold["engine_max"] == 2147483646
    head = np.array(gold["head_f32_bits"], dtype=np.uint32)
    got = co.make_dense_matrix_f32(gold["total"])
    assert np.array_equal(got[:head.size].view(np.uint32), head)
    bits = got.view(np.uint32)
    assert int(np.bitwise_xor.reduce(bits)) == gold["xor_f32_bits"]
    assert int(bits.astype(np.uint64).sum()) == gold["sum_f32_bits_mod_2_64"]
    assert int(bits[-1]) == gold["last_f32_bits"]
    # numpy restatement and the `skip` argument agree with the C one
    assert np.array_equal(no.make_dense_matrix_f32(300).view(np.uint32), bits[:300])
    assert np.array_equal(co.make_dense_matrix_f32(100, skip=777).view(np.uint32), bits[777:877])


def test_generator_first_six_values():
    # the first draws, as decimal literals
    expect32 = [-0.999984324, -0.73692441, 0.51121068, -0.0826997161, 0.0655344725, -0.562081635]
    expect16 = [-1.0, -0.736816406, 0.511230469, -0.0827026367, 0.0655517578, -0.562011719]
    np.testing.assert_allclose(co.make_dense_matrix_f32(6), expect32, rtol=1e-7)
    np.testing.assert_allclose(co.make_dense_matrix_f16(6).astype(np.float64), expect16, rtol=1e-7)
    assert np.array_equal(co.make_dense_matrix_f16(64).view(np.uint16),
                          co.make_dense_matrix_f32(64).astype(np.float16).view(np.uint16))


# ------------------------------------------------------------------ SpMM oracle

@pytest.mark.parametrize("V", [1, 2, 4, 8])
def test_spmm_c_equals_numpy_bitwise_and_float64_brute_force(V):
    p = _problem(16, 96, V, 0.8, seed=10 + V, skew=True)
    B = cv.dense_uniform(96, 40, seed=3)
    c = co.spmm_host_ref_f32(p.m_vec, V, 40, p.n, p.row_offsets, p.column_indices, p.values, B)
    n_ = no.spmm_host_ref_f32(p.m_vec, V, 40, p.n, p.row_offsets, p.column_indices, p.values, B)
    assert np.array_equal(c.view(np.uint32), n_.view(np.uint32))
    brute = p.to_dense() @ B.astype(np.float64)
    np.testing.assert_allclose(c, brute, rtol=1e-5, atol=1e-5)
    mt = co.spmm_host_ref_f32(p.m_vec, V, 40, p.n, p.row_offsets, p.column_indices, p.values, B, threads=4)
    assert np.array_equal(c.view(np.uint32), mt.view(np.uint32))


def test_spmm_v1_is_textbook_csr():
    p = _problem(40, 64, 1, 0.7, seed=5)
    B = cv.dense_uniform(64, 24, seed=6)
    A = sp.csr_matrix((p.values.reshape(-1).astype(np.float64), p.column_indices, p.row_offsets), shape=(40, 64))
    ref = A @ B.astype(np.float64)
    got = co.spmm_host_ref_f32(40, 1, 24, 64, p.row_offsets, p.column_indices, p.values, B)
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)


def test_spmm_closed_forms():
    V, n, k = 4, 32, 16
    pat = cv.binomial_pattern(12, n, 0.6, seed=2, vec_length=V)
    ones = pat.with_values(np.ones((pat.nnz_vec, V), np.float16))
    out = co.spmm_host_ref_f32(12, V, k, n, pat.row_offsets, pat.column_indices, ones.values,
                               np.ones((n, k), np.float16))
    # all-ones operands: every element of vector row i equals the row's length
    expect = np.repeat(pat.row_lengths(), V)[:, None] * np.ones((1, k))
    assert np.array_equal(out, expect.astype(np.float32))
    # a single nonzero vector: each output row is value * B[col]
    ro = np.array([0, 0, 1, 1], np.int32)
    ci = np.array([5], np.int32)
    vals = np.array([[0.5, -2.0, 3.0, 0.25]], np.float16)
    B = cv.dense_uniform(n, k, seed=9)
    out = co.spmm_host_ref_f32(3, V, k, n, ro, ci, vals, B)
    assert np.all(out[:4] == 0) and np.all(out[8:] == 0)          # empty vector rows are zero
    assert np.array_equal(out[4:8], vals[0].astype(np.float32)[:, None] * B[5].astype(np.float32)[None, :])
    # identity-like pattern col_j = j with one vector per row: row scaling of B
    m_vec = 8
    ro = np.arange(m_vec + 1, dtype=np.int32)
    ci = np.arange(m_vec, dtype=np.int32)
    vals = cv.dense_normal(m_vec, V, seed=1)
    out = co.spmm_host_ref_f32(m_vec, V, k, n, ro, ci, vals, B)
    expect = vals.astype(np.float32).reshape(-1, 1) * np.repeat(B[:m_vec].astype(np.float32), V, axis=0)
    assert np.array_equal(out, expect)


def test_spmm_accumulates_in_csr_order_fp32():
    # 1 + 2^-24 terms: sequential fp32 addition in ascending j loses the small terms one by one,
    # any re-association (pairwise, reversed) gives a different, larger result
    V, k = 1, 1
    n = 4097
    ro = np.array([0, n], np.int32)
    ci = np.arange(n, dtype=np.int32)
    vals = np.full((n, 1), 2.0 ** -13, np.float16)
    vals[0, 0] = 2048.0
    B = np.ones((n, 1), np.float16)
    out = co.spmm_host_ref_f32(1, V, k, n, ro, ci, vals, B)
    assert out[0, 0] == np.float32(2048.0)          # each 2^-13 is below half an ulp of 2048 (ulp = 2^-12)
    rev = co.spmm_host_ref_f32(1, V, k, n, ro, ci, vals[::-1].copy(), B)
    assert rev[0, 0] == np.float32(2048.5)          # small terms first: 4096 * 2^-13 = 0.5 survives


# ------------------------------------------------------------------ SDDMM oracle

@pytest.mark.parametrize("V", [1, 2, 4, 8])
def test_sddmm_c_equals_numpy_bitwise_and_float64_brute_force(V):
    K = 72
    pat = cv.binomial_pattern(10, 48, 0.7, seed=20 + V, vec_length=V)
    A = cv.dense_normal(pat.m, K, seed=1)
    B = cv.dense_normal(48, K, seed=2)
    c = co.sddmm_host_ref_f16(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B)
    n_ = no.sddmm_host_ref(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B)
    assert np.array_equal(c.view(np.uint16), n_.view(np.uint16))
    c32 = co.sddmm_host_ref_f32(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B)
    assert np.array_equal(c32.astype(np.float16).view(np.uint16), c.view(np.uint16))
    full = A.astype(np.float64) @ B.astype(np.float64).T
    rows = np.repeat(np.arange(pat.m_vec), pat.row_lengths())
    expect = np.stack([full[rows * V + v, pat.column_indices] for v in range(V)], axis=1).reshape(-1)
    np.testing.assert_allclose(c32, expect, rtol=1e-5, atol=1e-5)
    mt = co.sddmm_host_ref_f16(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B, threads=3)
    assert np.array_equal(c.view(np.uint16), mt.view(np.uint16))


def test_sddmm_accumulates_along_k_in_ascending_order_fp32():
    # Host_sddmm adds the products of one output in ascending l, in fp32 (include/bm_test_utils.h:181-186):
    # 2048 followed by 4096 terms of 2^-13 loses every small term (each is below half an ulp of 2048), the same
    # terms in descending l keep their sum 0.5.  A pairwise or reversed accumulation fails one of the two.
    K = 4097
    A = np.full((1, K), 2.0 ** -13, np.float16)
    A[0, 0] = 2048.0
    B = np.ones((1, K), np.float16)
    ro = np.array([0, 1], np.int32)
    ci = np.array([0], np.int32)
    out = co.sddmm_host_ref_f32(1, K, 1, ro, ci, A, B)
    assert out[0] == np.float32(2048.0)
    rev = co.sddmm_host_ref_f32(1, K, 1, ro, ci, A[:, ::-1].copy(), B)
    assert rev[0] == np.float32(2048.5)
    # the fp16 flavour rounds that fp32 sum once
    assert co.sddmm_host_ref_f16(1, K, 1, ro, ci, A[:, ::-1].copy(), B)[0] == np.float16(2048.0)   # 2048.5 -> even
    assert no.sddmm_host_ref(1, K, 1, ro, ci, A, B)[0] == np.float16(2048.0)


def test_sddmm_full_mask_is_dense_product_and_layout():
    V, m_vec, n, K = 2, 3, 5, 8
    ro = (np.arange(m_vec + 1) * n).astype(np.int32)
    ci = np.tile(np.arange(n, dtype=np.int32), m_vec)
    A = cv.dense_normal(m_vec * V, K, seed=3)
    B = cv.dense_normal(n, K, seed=4)
    out = co.sddmm_host_ref_f32(m_vec, K, V, ro, ci, A, B).reshape(m_vec, n, V)
    dense = (A.astype(np.float64) @ B.astype(np.float64).T).reshape(m_vec, V, n)
    np.testing.assert_allclose(out, dense.transpose(0, 2, 1), rtol=1e-6, atol=1e-6)


def test_sddmm_feeds_spmm():
    # (mask o A B^T) * W  through the two oracles equals the dense float64 computation
    V, K, N = 4, 16, 8
    pat = cv.uniform_pattern(6, 24, 0.5, seed=7, vec_length=V)
    A = cv.dense_normal(pat.m, K, seed=1)
    B = cv.dense_normal(24, K, seed=2)
    W = cv.dense_uniform(24, N, seed=3)
    vals = co.sddmm_host_ref_f16(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B)
    out = co.spmm_host_ref_f32(pat.m_vec, V, N, 24, pat.row_offsets, pat.column_indices, vals, W)
    dense = pat.with_values(vals.reshape(-1, V)).to_dense() @ W.astype(np.float64)
    np.testing.assert_allclose(out, dense, rtol=1e-5, atol=1e-4)


def test_empty_inputs():
    ro = np.zeros(5, np.int32)
    out = co.spmm_host_ref_f32(4, 8, 16, 32, ro, np.zeros(0, np.int32), np.zeros((0, 8), np.float16),
                               np.ones((32, 16), np.float16))
    assert out.shape == (32, 16) and not out.any()
    out = co.sddmm_host_ref_f16(4, 16, 8, ro, np.zeros(0, np.int32), np.ones((32, 16), np.float16),
                                np.ones((32, 16), np.float16))
    assert out.size == 0


# ------------------------------------------------------------------ row swizzles

def test_row_swizzles():
    rng = np.random.default_rng(0)
    lengths = rng.integers(0, 6, 200)
    ro = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    ident = co.identity_row_swizzle(200)
    assert np.array_equal(ident, np.arange(200))
    srt = co.sorted_row_swizzle(200, ro)
    assert np.array_equal(np.sort(srt), np.arange(200))              # a permutation
    assert np.all(np.diff(lengths[srt]) <= 0)                         # longest first
    assert np.array_equal(srt, no.sorted_row_swizzle(200, ro))        # same tie rule in both restatements
    for L in np.unique(lengths):                                      # ties keep ascending row order
        assert np.all(np.diff(srt[lengths[srt] == L]) > 0)


# ------------------------------------------------------------------ sparse softmax (attention middle step)

def test_sparse_softmax_oracle_vs_dense_masked_softmax():
    from scipy.special import softmax
    V = 4
    pat = cv.random_values(cv.binomial_pattern(6, 40, 0.6, seed=3, vec_length=V), seed=4)
    scale = 0.37
    got = no.sparse_softmax_ref(pat.m_vec, V, pat.row_offsets, pat.values, scale)
    dense = np.full((pat.m, pat.n), -np.inf)
    for i in range(pat.m_vec):
        for j in range(pat.row_offsets[i], pat.row_offsets[i + 1]):
            dense[i * V:(i + 1) * V, pat.column_indices[j]] = pat.values[j].astype(np.float64) * scale
    full = softmax(dense, axis=1)
    for i in range(pat.m_vec):
        for j in range(pat.row_offsets[i], pat.row_offsets[i + 1]):
            np.testing.assert_allclose(got[j], full[i * V:(i + 1) * V, pat.column_indices[j]], rtol=1e-12)
    # every scalar row sums to one; uniform inputs give 1 / row length
    for i in range(pat.m_vec):
        blk = got[pat.row_offsets[i]:pat.row_offsets[i + 1]]
        if blk.size:
            np.testing.assert_allclose(blk.sum(axis=0), 1.0, rtol=1e-12)
    ones = no.sparse_softmax_ref(pat.m_vec, V, pat.row_offsets, np.ones_like(pat.values), 5.0)
    L = np.repeat(pat.row_lengths(), pat.row_lengths())
    np.testing.assert_allclose(ones, (1.0 / L)[:, None] * np.ones((1, V)), rtol=1e-12)
