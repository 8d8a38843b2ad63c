"""numpy restatement of the reference's host verification loops.

TEST INFRASTRUCTURE ONLY (see the package docstring).

fp16 x fp16 products are exact in fp32, so each function below is fully
determined by the order of its fp32 additions, which is kept as in the
reference: ascending nonzero index for SpMM, ascending contraction index for
SDDMM.  The vectorisation is only over output elements, never over the
summation index.
"""
import numpy as np


def spmm_host_ref_f32(m_vec, vec_length, k, n, row_offsets, column_indices, values, rhs_matrix):
    """spmm_benchmark.cpp:66-86.  `k` = dense width, `n` = columns of the sparse matrix.

    values: fp16 [nnz_vec * vec_length]; rhs_matrix: fp16 [n * k] row-major.
    Returns fp32 [m_vec * vec_length, k].
    """
    row_offsets = np.asarray(row_offsets)
    column_indices = np.asarray(column_indices)
    vals = np.asarray(values, dtype=np.float16).reshape(-1, vec_length).astype(np.float32)
    rhs = np.asarray(rhs_matrix, dtype=np.float16).reshape(n, k).astype(np.float32)
    out = np.zeros((m_vec * vec_length, k), dtype=np.float32)
    for i in range(m_vec):
        block = out[i * vec_length:(i + 1) * vec_length]
        for j in range(int(row_offsets[i]), int(row_offsets[i + 1])):
            block += vals[j][:, None] * rhs[int(column_indices[j])][None, :]
    return out


def sddmm_host_ref(m_vec, k, vec_length, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                   out_dtype=np.float16):
    """include/bm_test_utils.h:171-193 (Host_sddmm).

    lhs_matrix: fp16 [m_vec*vec_length, k]; rhs_matrix: fp16 [n, k].
    Returns out_dtype [nnz_vec * vec_length], element j*V+v.
    """
    row_offsets = np.asarray(row_offsets)
    col_indices = np.asarray(col_indices)
    lhs = np.asarray(lhs_matrix, dtype=np.float16).reshape(m_vec * vec_length, k).astype(np.float32)
    rhs = np.asarray(rhs_matrix, dtype=np.float16).reshape(-1, k).astype(np.float32)
    nnz_vec = int(row_offsets[m_vec])
    lengths = np.diff(row_offsets[:m_vec + 1])
    row_of = np.repeat(np.arange(m_vec), lengths)                      # [nnz_vec]
    lhs_rows = row_of[:, None] * vec_length + np.arange(vec_length)    # [nnz_vec, V]
    acc = np.zeros((nnz_vec, vec_length), dtype=np.float32)
    cols = col_indices[:nnz_vec]
    for l in range(k):
        acc += lhs[lhs_rows, l] * rhs[cols, l][:, None]
    return acc.astype(out_dtype).reshape(-1)


def sparse_softmax_ref(m_vec, vec_length, row_offsets, values, scale=1.0):
    """Row-wise softmax over the nonzeros of every scalar row, [nnz_vec, V] layout, in float64.

    The reference does not ship this operator (it includes Sputnik's sparse_softmax.h,
    include/sputnik.h:22, from an external library that is not in its tree), so this is the textbook
    definition: out = exp(s*x - max) / sum(exp(s*x - max)) over the row's stored elements.
    """
    row_offsets = np.asarray(row_offsets)
    x = np.asarray(values, dtype=np.float64).reshape(-1, vec_length) * float(scale)
    out = np.empty_like(x)
    for i in range(m_vec):
        lo, hi = int(row_offsets[i]), int(row_offsets[i + 1])
        if hi > lo:
            blk = x[lo:hi]
            e = np.exp(blk - blk.max(axis=0, keepdims=True))
            out[lo:hi] = e / e.sum(axis=0, keepdims=True)
    return out


def identity_row_swizzle(rows):
    """include/bm_test_utils.h:196-198."""
    return np.arange(rows, dtype=np.int32)


def sorted_row_swizzle(rows, row_offsets):
    """include/bm_test_utils.h:200-215; ties broken by ascending row index."""
    lengths = np.diff(np.asarray(row_offsets)[:rows + 1])
    return np.argsort(-lengths, kind="stable").astype(np.int32)


def make_dense_matrix_f32(count, skip=0):
    """include/bm_test_utils.h:130-142 with libstdc++'s default engine (minstd_rand0, seed 1)."""
    out = np.empty(count, dtype=np.float32)
    x = 1
    two = np.float32(2.0)
    neg1 = np.float32(-1.0)
    denom = np.float32(2147483648.0)
    for i in range(skip + count):
        x = (x * 16807) % 2147483647
        if i < skip:
            continue
        c = np.float32(x - 1) / denom
        if c >= np.float32(1.0):
            c = np.nextafter(np.float32(1.0), np.float32(0.0))
        out[i - skip] = c * two + neg1
    return out


def make_dense_matrix_f16(count, skip=0):
    return make_dense_matrix_f32(count, skip).astype(np.float16)
