"""SpMM with the dense operand staged in LDS per block of vector rows (`vs_wmma_spmm_f16_slab`): the same contract
as the reference-shaped entry point (tests/util.py), checked against the CPU oracle through the C ABI - every vector
length, every number of parts of the contraction, dense widths that cut the last tile, swizzled and ragged rows, and
columns that are not sorted (which the schedule serves from memory instead of LDS)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


def _oracle(pat, B):
    return co.spmm_host_ref_f32(pat.m_vec, pat.vec_length, B.shape[1], pat.n, pat.row_offsets,
                                pat.column_indices, pat.values, B)


def _run(pat, B, parts=0, sort=False):
    """One call (twice: the second finds the workspace as the first left it) with canaries round the output and the
    workspace; returns the host copy of the output."""
    prob = ops.DeviceProblem(pat, sort=sort)
    Bd = torch.from_numpy(B).cuda()
    k = B.shape[1]
    pad = 64
    buf = torch.full((pat.m + 2 * pad, k), 12345.0, dtype=torch.float16, device="cuda")
    out = buf[pad:pad + pat.m]
    try:
        _lib.set_option("spmm_slab_parts", parts)
        need = ops.spmm_slab_workspace_bytes(pat.m_vec, pat.vec_length, k, pat.n)
        guard = 4096
        ws_buf = torch.full((need + 2 * guard,), 0x5A, dtype=torch.uint8, device="cuda")  # (never cleared: by contract)
        ws = ws_buf[guard:guard + need] if need else None
        for _ in range(2):
            out.fill_(777.0)
            ops.spmm_slab(pat.m_vec, pat.vec_length, k, pat.n, prob.row_indices, prob.row_offsets, prob.column_indices,
                          prob.values, Bd, out, ws)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("spmm_slab_parts", 0)
    host = buf.cpu().numpy()
    assert np.all(host[:pad] == 12345.0) and np.all(host[pad + pat.m:] == 12345.0), "wrote outside the output"
    wsh = ws_buf.cpu().numpy()
    assert np.all(wsh[:guard] == 0x5A) and np.all(wsh[guard + need:] == 0x5A), "wrote outside the workspace"
    assert np.array_equal(prob.row_offsets.cpu().numpy(), pat.row_offsets)
    assert np.array_equal(prob.column_indices.cpu().numpy(), pat.column_indices)
    return host[pad:pad + pat.m]


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("parts", [1, 2, 3, 7])
def test_every_vector_length_and_part_count(V, parts):
    pat = cv.random_values(cv.uniform_pattern(40, 900, 0.6, seed=V, vec_length=V), seed=10 + V)
    B = cv.dense_uniform(900, 128, seed=3)
    assert_parity(_run(pat, B, parts), _oracle(pat, B), "slab V=%d parts=%d" % (V, parts))


@pytest.mark.parametrize("k", [8, 72, 136, 264])
def test_dense_widths_that_cut_the_last_tile(k):
    pat = cv.random_values(cv.binomial_pattern(24, 640, 0.7, seed=5, vec_length=8), seed=6)
    B = cv.dense_uniform(640, k, seed=7)
    assert_parity(_run(pat, B, 2, sort=True), _oracle(pat, B), "slab k=%d" % k)


@pytest.mark.parametrize("sparsity", [0.5, 0.9, 0.98])
def test_sweep_shaped_points(sparsity):
    pat = cv.random_values(cv.uniform_pattern(128, 2304, sparsity, seed=8, vec_length=8), seed=9)
    B = cv.dense_uniform(2304, 256, seed=10)
    assert_parity(_run(pat, B), _oracle(pat, B), "slab 1024 x 2304 x 256 at %.2f" % sparsity)


def test_ragged_and_empty_rows_and_swizzle_invariance():
    rng = np.random.default_rng(3)
    lengths = rng.integers(0, 300, 50)
    lengths[[0, 7, 49]] = 0
    lengths[11] = 1000
    ro, ci = cv._pattern_from_lengths(rng, 50, 1000, lengths)
    pat = cv.random_values(cv.ColVecCSR(50, 1000, 4, ro, ci), 4)
    B = cv.dense_uniform(1000, 64, seed=5)
    plain = _run(pat, B, 3, sort=False)
    assert_parity(plain, _oracle(pat, B), "slab ragged rows")
    # a row's sum does not depend on which rows share its workgroup: same bits under any swizzle
    assert np.array_equal(plain, _run(pat, B, 3, sort=True))


def test_columns_out_of_order():
    pat = cv.random_values(cv.uniform_pattern(32, 700, 0.7, seed=9, vec_length=4), seed=10)
    ci = pat.column_indices.copy()
    va = pat.values.reshape(-1, 4).copy()
    rng = np.random.default_rng(0)
    for r in range(pat.m_vec):
        a, b = pat.row_offsets[r], pat.row_offsets[r + 1]
        perm = rng.permutation(b - a) if r % 2 else np.arange(b - a)[::-1]
        ci[a:b] = ci[a:b][perm]
        va[a:b] = va[a:b][perm]
    shuffled = cv.ColVecCSR(pat.m_vec, pat.n, 4, pat.row_offsets, ci).with_values(va)
    B = cv.dense_uniform(700, 64, seed=11)
    for parts in (1, 2):
        assert_parity(_run(shuffled, B, parts), _oracle(shuffled, B), "slab with unsorted columns, %d parts" % parts)


def test_rejects_what_it_cannot_take():
    pat = cv.random_values(cv.uniform_pattern(8, 64, 0.5, seed=1, vec_length=8), seed=2)
    prob = ops.DeviceProblem(pat)
    B = torch.zeros((64, 12), dtype=torch.float16, device="cuda")
    out = torch.empty((pat.m, 12), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.VSparseError) as e:
        ops.spmm_slab(pat.m_vec, 8, 12, 64, prob.row_indices, prob.row_offsets, prob.column_indices, prob.values, B, out)
    assert e.value.status == 801
