"""Column-vector CSR: the sparse format of the SpMM / SDDMM path.

A matrix of ``m = m_vec * V`` rows is stored as ``m_vec`` *vector rows*; each
stored nonzero is a V x 1 column vector, so one ``column_indices`` entry
covers V scalar rows.  Layout (reference: spmm_benchmark.cpp:21-54 and
:79-81; sddmm_benchmark.cpp:172-206):

    row_offsets    int32 [m_vec + 1]
    column_indices int32 [nnz_vec]           column of vector j, in [0, n)
    values         fp16  [nnz_vec, V]        element (i*V + v, column_indices[j]) = values[j, v]

The ``.smtx`` text form holds only the pattern: ``m_vec, n, nnz_vec`` on the
first line, the offsets on the second, the column indices on the third; the
reader expands every file nonzero into a V-vector exactly as the reference
benchmarks do (``m = m_vec * V``, ``nnz = nnz_vec * V``).
"""
from dataclasses import dataclass
from typing import Optional

import numpy as np

VEC_LENGTHS = (1, 2, 4, 8)


@dataclass
class ColVecCSR:
    m_vec: int
    n: int                       # columns of the sparse matrix
    vec_length: int
    row_offsets: np.ndarray      # int32 [m_vec + 1]
    column_indices: np.ndarray   # int32 [nnz_vec]
    values: Optional[np.ndarray] = None   # fp16 [nnz_vec, V] (None for a pure mask)

    @property
    def m(self):
        return self.m_vec * self.vec_length

    @property
    def nnz_vec(self):
        return int(self.row_offsets[self.m_vec])

    @property
    def nnz(self):
        return self.nnz_vec * self.vec_length

    @property
    def sparsity(self):
        return 1.0 - self.nnz_vec / float(max(1, self.m_vec * self.n))

    def validate(self):
        """Raise ValueError unless the arrays describe a well-formed pattern."""
        if self.vec_length not in VEC_LENGTHS:
            raise ValueError("vec_length must be one of %s" % (VEC_LENGTHS,))
        ro, ci = self.row_offsets, self.column_indices
        if ro.dtype != np.int32 or ci.dtype != np.int32:
            raise ValueError("row_offsets / column_indices must be int32")
        if ro.shape != (self.m_vec + 1,):
            raise ValueError("row_offsets must have m_vec + 1 entries")
        if ro[0] != 0 or np.any(np.diff(ro) < 0):
            raise ValueError("row_offsets must start at 0 and be non-decreasing")
        if ci.shape[0] < self.nnz_vec:
            raise ValueError("column_indices shorter than row_offsets[m_vec]")
        if self.nnz_vec and (ci[:self.nnz_vec].min() < 0 or ci[:self.nnz_vec].max() >= self.n):
            raise ValueError("column index out of range")
        if self.values is not None and self.values.shape != (self.nnz_vec, self.vec_length):
            raise ValueError("values must be [nnz_vec, V]")
        return self

    def row_lengths(self):
        return np.diff(self.row_offsets)

    def to_dense(self, dtype=np.float64):
        """Expand to a dense (m, n) array (test helper; duplicates accumulate)."""
        out = np.zeros((self.m, self.n), dtype=dtype)
        V = self.vec_length
        vals = self.values.astype(dtype)
        for i in range(self.m_vec):
            for j in range(int(self.row_offsets[i]), int(self.row_offsets[i + 1])):
                out[i * V:(i + 1) * V, int(self.column_indices[j])] += vals[j]
        return out

    def with_values(self, values):
        values = np.ascontiguousarray(values, dtype=np.float16).reshape(self.nnz_vec, self.vec_length)
        return ColVecCSR(self.m_vec, self.n, self.vec_length, self.row_offsets, self.column_indices, values)


# --------------------------------------------------------------------------- .smtx

def write_smtx(path, m_vec, n, row_offsets, column_indices):
    """Write a pattern in the text form the reference benchmarks parse."""
    row_offsets = np.asarray(row_offsets)
    nnz_vec = int(row_offsets[m_vec])
    with open(path, "w") as f:
        f.write("%d, %d, %d\n" % (m_vec, n, nnz_vec))
        f.write(" ".join(str(int(x)) for x in row_offsets[:m_vec + 1]) + "\n")
        f.write(" ".join(str(int(x)) for x in np.asarray(column_indices)[:nnz_vec]) + "\n")


def read_smtx(path, vec_length):
    """Parse ``path`` and expand each nonzero to a V-vector (values left unset).

    Same field order and separators as spmm_benchmark.cpp:25-54: header split on
    commas, offsets and indices split on blanks.
    """
    with open(path, "r") as f:
        header = f.readline()
        m_vec, n, nnz_vec = (int(t) for t in header.split(","))
        offsets = np.array(f.readline().split(), dtype=np.int64)
        indices = np.array(f.readline().split(), dtype=np.int64)
    if offsets.shape[0] != m_vec + 1:
        raise ValueError("%s: expected %d row offsets, found %d" % (path, m_vec + 1, offsets.shape[0]))
    if indices.shape[0] != nnz_vec:
        raise ValueError("%s: expected %d column indices, found %d" % (path, nnz_vec, indices.shape[0]))
    return ColVecCSR(m_vec, n, vec_length, offsets.astype(np.int32), indices.astype(np.int32)).validate()


# --------------------------------------------------------------------------- synthetic patterns

def _pattern_from_lengths(rng, m_vec, n, lengths):
    row_offsets = np.zeros(m_vec + 1, dtype=np.int32)
    row_offsets[1:] = np.cumsum(lengths)
    cols = np.empty(int(row_offsets[-1]), dtype=np.int32)
    for i in range(m_vec):
        L = int(lengths[i])
        if L:
            cols[row_offsets[i]:row_offsets[i + 1]] = np.sort(rng.choice(n, L, replace=False))
    return row_offsets, cols


def uniform_pattern(m_vec, n, sparsity, seed, vec_length=1):
    """Exactly round((1 - sparsity) * n) distinct, sorted columns in every vector row."""
    rng = np.random.default_rng(seed)
    per_row = int(round((1.0 - sparsity) * n))
    per_row = max(0, min(n, per_row))
    ro, ci = _pattern_from_lengths(rng, m_vec, n, np.full(m_vec, per_row, dtype=np.int64))
    return ColVecCSR(m_vec, n, vec_length, ro, ci)


def binomial_pattern(m_vec, n, sparsity, seed, vec_length=1):
    """Row length ~ Binomial(n, 1 - sparsity): mildly skewed rows, columns uniform and sorted."""
    rng = np.random.default_rng(seed)
    lengths = rng.binomial(n, 1.0 - sparsity, size=m_vec)
    ro, ci = _pattern_from_lengths(rng, m_vec, n, lengths)
    return ColVecCSR(m_vec, n, vec_length, ro, ci)


def band_strided_pattern(seq_len, vec_length, band_half_width=128, stride=128):
    """Fixed sparse-attention mask: local band around the diagonal plus a strided column.

    Vector row i keeps the columns c with |c - (V*i + V/2)| <= band_half_width,
    clipped to [0, seq_len), and every column with c % stride == stride - 1.
    """
    m_vec = seq_len // vec_length
    rows = []
    strided = np.arange(stride - 1, seq_len, stride)
    for i in range(m_vec):
        centre = i * vec_length + vec_length // 2
        lo = max(0, centre - band_half_width)
        hi = min(seq_len - 1, centre + band_half_width)
        rows.append(np.union1d(np.arange(lo, hi + 1), strided))
    lengths = np.array([r.shape[0] for r in rows], dtype=np.int64)
    ro = np.zeros(m_vec + 1, dtype=np.int32)
    ro[1:] = np.cumsum(lengths)
    ci = np.concatenate(rows).astype(np.int32) if rows else np.zeros(0, np.int32)
    return ColVecCSR(m_vec, seq_len, vec_length, ro, ci)


def random_values(pattern, seed, scale=1.0):
    """fp16 ~ N(0, scale) values for every stored vector element."""
    rng = np.random.default_rng(seed)
    vals = (rng.standard_normal((pattern.nnz_vec, pattern.vec_length)) * scale).astype(np.float16)
    return pattern.with_values(vals)


def dense_uniform(rows, cols, seed):
    """fp16 ~ U(-1, 1), row-major."""
    rng = np.random.default_rng(seed)
    return rng.uniform(-1.0, 1.0, size=(rows, cols)).astype(np.float16)


def dense_normal(rows, cols, seed):
    """fp16 ~ N(0, 1), row-major."""
    rng = np.random.default_rng(seed)
    return rng.standard_normal((rows, cols)).astype(np.float16)


# --------------------------------------------------------------------------- row swizzles (host mirror)

def identity_row_swizzle(rows):
    """include/bm_test_utils.h:196-198."""
    return np.arange(rows, dtype=np.int32)


def sorted_row_swizzle(row_offsets):
    """Rows ordered by descending length (include/bm_test_utils.h:200-215).

    Ties keep ascending row order (a stable sort), one of the orders the
    reference's unstable std::sort may produce.
    """
    lengths = np.diff(np.asarray(row_offsets))
    return np.argsort(-lengths, kind="stable").astype(np.int32)
