"""Host-side mirror of the reference's operator API over the C ABI.

The four device operators keep the reference's names, argument order and
dimension letters (include/wmma_spmm.cuh:15-21, include/cuda_spmm.cuh:15-21,
include/wmma_sddmm.cuh:17-24, include/cuda_sddmm.cuh:16-23).  Arguments are
torch tensors on the GPU (used only as owners of device memory) or raw device
addresses; the output dtype of ``output_matrix`` / ``output_values`` (fp16 or
fp32) picks the overload, as C++ overload resolution does in the reference.
Every call is asynchronous on ``stream`` (default: torch's current stream).
"""
import numpy as np
import torch

from . import _lib


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


def _stream(stream):
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def _expect(t, dtype, name):
    if isinstance(t, torch.Tensor):
        if t.dtype != dtype:
            raise TypeError("%s must be %s, got %s" % (name, dtype, t.dtype))
        if not t.is_cuda:
            raise ValueError("%s must live in device memory" % name)
        if not t.is_contiguous():
            raise ValueError("%s must be contiguous" % name)


def _spmm(entry, m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
          output_matrix, stream):
    for t, nm in ((row_indices, "row_indices"), (row_offsets, "row_offsets"), (column_indices, "column_indices")):
        _expect(t, torch.int32, nm)
    _expect(values, torch.float16, "values")
    _expect(rhs_matrix, torch.float16, "rhs_matrix")
    f32 = isinstance(output_matrix, torch.Tensor) and output_matrix.dtype == torch.float32
    if not f32:
        _expect(output_matrix, torch.float16, "output_matrix")
    fn = getattr(_lib.lib(), entry + ("_f32out" if f32 else ""))
    st = fn(m_vec, vec_length, k, n, _ptr(row_indices), _ptr(row_offsets), _ptr(column_indices), _ptr(values),
            _ptr(rhs_matrix), _ptr(output_matrix), _stream(stream))
    _lib.check(st, entry)
    return output_matrix


def _sddmm(entry, m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
           output_values, vec_length, stream, algorithm=None):
    for t, nm in ((row_indices, "row_indices"), (row_offsets, "row_offsets"), (col_indices, "col_indices")):
        _expect(t, torch.int32, nm)
    _expect(lhs_matrix, torch.float16, "lhs_matrix")
    _expect(rhs_matrix, torch.float16, "rhs_matrix")
    f32 = isinstance(output_values, torch.Tensor) and output_values.dtype == torch.float32
    if not f32:
        _expect(output_values, torch.float16, "output_values")
    fn = getattr(_lib.lib(), entry + ("_f32out" if f32 else ""))
    args = [m_vec, k, n, nonzeros_vec, _ptr(row_indices), _ptr(row_offsets), _ptr(col_indices), _ptr(lhs_matrix),
            _ptr(rhs_matrix), _ptr(output_values), vec_length, _stream(stream)]
    if algorithm is not None:
        args.append(algorithm)
    _lib.check(fn(*args), entry)
    return output_values


class spmm:
    """Namespace ``spmm`` of the reference: C[m x k] = A[m x n] (column-vector CSR) * B[n x k]."""

    @staticmethod
    def wmmaSpmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                 output_matrix, stream=None):
        """MFMA path (reference: tensor-core path, src/wmma_spmm.cu:400-409)."""
        return _spmm("vs_wmma_spmm_f16", m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                     values, rhs_matrix, output_matrix, stream)

    @staticmethod
    def cudaSpmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                 output_matrix, stream=None):
        """Fine-grained packed-fp16 VALU path (reference: src/cuda_spmm.cu:316-325)."""
        return _spmm("vs_cuda_spmm_f16", m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                     values, rhs_matrix, output_matrix, stream)


class sddmm:
    """Namespace ``sddmm`` of the reference: D = (A[m x k] * B[n x k]^T) sampled on a column-vector CSR mask."""

    @staticmethod
    def wmmaSddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                  output_values, vec_length, stream=None, algorithm=1):
        """MFMA path (reference: src/wmma_sddmm.cu:3190-3202)."""
        return _sddmm("vs_wmma_sddmm_f16", m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                      lhs_matrix, rhs_matrix, output_values, vec_length, stream, algorithm)

    @staticmethod
    def cudaSddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                  output_values, vec_length, stream=None):
        """Cross-lane dot-product path (reference: src/cuda_sddmm.cu:1295-1331)."""
        return _sddmm("vs_cuda_sddmm_f16", m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                      lhs_matrix, rhs_matrix, output_values, vec_length, stream)


def IdentityRowSwizzle(rows):
    """include/bm_test_utils.h:196-198 through the C ABI (host arrays)."""
    out = np.empty(rows, dtype=np.int32)
    _lib.lib().vs_identity_row_swizzle(rows, out.ctypes.data)
    return out


def SortedRowSwizzle(rows, row_offsets):
    """include/bm_test_utils.h:200-215 through the C ABI (host arrays)."""
    ro = np.ascontiguousarray(row_offsets, dtype=np.int32)
    out = np.empty(rows, dtype=np.int32)
    _lib.lib().vs_sorted_row_swizzle(rows, ro.ctypes.data, out.ctypes.data)
    return out


class DeviceProblem:
    """Device-resident operands of one SpMM / SDDMM problem (caller-owned buffers, as in BmFN)."""

    def __init__(self, pattern, sort=False, device="cuda"):
        self.pattern = pattern
        self.m_vec = pattern.m_vec
        self.vec_length = pattern.vec_length
        self.n = pattern.n
        self.nnz_vec = pattern.nnz_vec
        swz = SortedRowSwizzle(pattern.m_vec, pattern.row_offsets) if sort else IdentityRowSwizzle(pattern.m_vec)
        self.row_indices = torch.from_numpy(swz).to(device)
        self.row_offsets = torch.from_numpy(np.ascontiguousarray(pattern.row_offsets)).to(device)
        self.column_indices = torch.from_numpy(np.ascontiguousarray(pattern.column_indices)).to(device)
        self.values = None
        if pattern.values is not None:
            self.values = torch.from_numpy(np.ascontiguousarray(pattern.values)).to(device)

    def spmm(self, rhs_matrix, kernel="wmma", out_dtype=torch.float16, out=None, stream=None):
        k = rhs_matrix.shape[1]
        if out is None:
            out = torch.empty((self.m_vec * self.vec_length, k), dtype=out_dtype, device=rhs_matrix.device)
        fn = spmm.wmmaSpmm if kernel == "wmma" else spmm.cudaSpmm
        return fn(self.m_vec, self.vec_length, k, self.n, self.row_indices, self.row_offsets,
                  self.column_indices, self.values, rhs_matrix, out, stream)

    def sddmm(self, lhs_matrix, rhs_matrix, kernel="wmma", out_dtype=torch.float16, out=None, stream=None,
              algorithm=1):
        k = lhs_matrix.shape[1]
        if out is None:
            out = torch.empty((self.nnz_vec, self.vec_length), dtype=out_dtype, device=lhs_matrix.device)
        if kernel == "wmma":
            return sddmm.wmmaSddmm(self.m_vec, k, self.n, self.nnz_vec, self.row_indices, self.row_offsets,
                                   self.column_indices, lhs_matrix, rhs_matrix, out, self.vec_length, stream,
                                   algorithm)
        return sddmm.cudaSddmm(self.m_vec, k, self.n, self.nnz_vec, self.row_indices, self.row_offsets,
                               self.column_indices, lhs_matrix, rhs_matrix, out, self.vec_length, stream)
