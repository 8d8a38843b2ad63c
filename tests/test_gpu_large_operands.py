"""Operands beyond 2^31 elements (4 GiB of fp16): every kernel must index them with 64-bit offsets.

The dense operand is generated on the device (it never exists on the host); the oracle runs on the host
over the few rows the pattern references, re-indexed densely, which is the same arithmetic in the same
order.  Where the output itself is the large array, a pattern with one nonzero vector per row makes every
output a single fp16 product, whose correctly rounded value torch computes on the device: bit-exact.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu

BIG_ROWS = (1 << 20) + 4096      # x 2048 columns = 2^31 + 2^23 elements, 4.03 GiB
WIDTH = 2048


@pytest.fixture(scope="module")
def big_matrix(gpu):
    g = torch.Generator(device="cuda").manual_seed(11)
    big = torch.empty((BIG_ROWS, WIDTH), dtype=torch.float16, device="cuda")
    big.normal_(generator=g)
    yield big
    del big
    torch.cuda.empty_cache()


def _pattern_into_the_far_end(V, m_vec, per_row, seed):
    """Columns spread over the whole operand, a third of them in the rows past the 2^31-element mark."""
    rng = np.random.default_rng(seed)
    first_far = (1 << 31) // WIDTH
    offsets = np.arange(m_vec + 1, dtype=np.int32) * per_row
    cols = np.empty(m_vec * per_row, dtype=np.int32)
    for i in range(m_vec):
        near = rng.choice(first_far, per_row - per_row // 3, replace=False)
        far = first_far + rng.choice(BIG_ROWS - first_far, per_row // 3, replace=False)
        cols[i * per_row:(i + 1) * per_row] = np.sort(np.concatenate([near, far]))
    cols[-1] = BIG_ROWS - 1          # the very last row of the operand
    return cv.ColVecCSR(m_vec, BIG_ROWS, V, offsets, cols)


def _compact(pat, big):
    """The referenced rows on the host and the same pattern re-indexed into them."""
    used, inverse = np.unique(pat.column_indices, return_inverse=True)
    rows = big[torch.from_numpy(used.astype(np.int64)).cuda()].cpu().numpy()
    small = cv.ColVecCSR(pat.m_vec, len(used), pat.vec_length, pat.row_offsets, inverse.astype(np.int32), pat.values)
    return small, rows


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
@pytest.mark.parametrize("V", [1, 8])
def test_spmm_gathers_beyond_4gib(big_matrix, kernel, V):
    pat = cv.random_values(_pattern_into_the_far_end(V, 24, 45, seed=V), seed=3)
    small, rows = _compact(pat, big_matrix)
    ref = co.spmm_host_ref_f32(small.m_vec, V, WIDTH, small.n, small.row_offsets, small.column_indices,
                               small.values, rows)
    out = ops.DeviceProblem(pat).spmm(big_matrix, kernel=kernel)
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy(), ref, "spmm %s V%d, rhs of %d elements" % (kernel, V, big_matrix.numel()))


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
@pytest.mark.parametrize("V", [2, 8])
def test_sddmm_gathers_beyond_4gib(big_matrix, kernel, V):
    pat = _pattern_into_the_far_end(V, 16, 33, seed=10 + V)
    small, rows = _compact(pat, big_matrix)
    lhs = cv.dense_normal(pat.m, WIDTH, seed=5)
    ref = co.sddmm_host_ref_f16(small.m_vec, WIDTH, V, small.row_offsets, small.column_indices, lhs, rows)
    out = ops.DeviceProblem(pat).sddmm(torch.from_numpy(lhs).cuda(), big_matrix, kernel=kernel)
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy().reshape(-1), ref, "sddmm %s V%d, rhs of %d elements" % (kernel, V, big_matrix.numel()))


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_spmm_output_beyond_4gib(gpu, kernel):
    # one nonzero vector per row: out[i*V + v, :] = values[i, v] * B[col_i, :], one rounding each
    V, n = 8, 96
    m_vec = BIG_ROWS // V
    rng = np.random.default_rng(17)
    cols = rng.integers(0, n, m_vec).astype(np.int32)
    pat = cv.ColVecCSR(m_vec, n, V, np.arange(m_vec + 1, dtype=np.int32), cols)
    pat = cv.random_values(pat, seed=18)
    B = torch.from_numpy(cv.dense_uniform(n, WIDTH, seed=19)).cuda()
    out = ops.DeviceProblem(pat).spmm(B, kernel=kernel)
    torch.cuda.synchronize()
    assert out.numel() > (1 << 31)
    values = torch.from_numpy(pat.values).cuda()
    cols_d = torch.from_numpy(cols.astype(np.int64)).cuda()
    block = 8192                      # vector rows per comparison block: bounded temporaries
    for start in range(0, m_vec, block):
        stop = min(start + block, m_vec)
        a = values[start:stop].float().reshape(-1, V, 1)
        b = B[cols_d[start:stop]].float().reshape(-1, 1, WIDTH)
        expect = (a * b).half().reshape(-1, WIDTH)
        assert torch.equal(out[start * V:stop * V], expect), "rows %d..%d" % (start * V, stop * V)
