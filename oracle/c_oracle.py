"""ctypes front-end of libvsoracle.so (built from vs_oracle.c by oracle/Makefile).

TEST INFRASTRUCTURE ONLY (see the package docstring).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvsoracle.so")
_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_f32p = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile vs_oracle.c with gcc (make)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])
    else:
        subprocess.check_call(["make", "-C", _HERE, "-s"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.vso_half_to_float.restype = ctypes.c_float
        L.vso_half_to_float.argtypes = [ctypes.c_uint16]
        L.vso_float_to_half.restype = ctypes.c_uint16
        L.vso_float_to_half.argtypes = [ctypes.c_float]
        L.vso_spmm_host_ref_f32.restype = None
        L.vso_spmm_host_ref_f32.argtypes = [ctypes.c_int] * 4 + [_i32p, _i32p, _u16p, _u16p, _f32p]
        L.vso_spmm_host_ref_f32_mt.restype = None
        L.vso_spmm_host_ref_f32_mt.argtypes = [ctypes.c_int] * 4 + [_i32p, _i32p, _u16p, _u16p, _f32p, ctypes.c_int]
        L.vso_sddmm_host_ref_f16.restype = None
        L.vso_sddmm_host_ref_f16.argtypes = [ctypes.c_int] * 3 + [_i32p, _i32p, _u16p, _u16p, _u16p]
        L.vso_sddmm_host_ref_f16_mt.restype = None
        L.vso_sddmm_host_ref_f16_mt.argtypes = [ctypes.c_int] * 3 + [_i32p, _i32p, _u16p, _u16p, _u16p, ctypes.c_int]
        L.vso_sddmm_host_ref_f32.restype = None
        L.vso_sddmm_host_ref_f32.argtypes = [ctypes.c_int] * 3 + [_i32p, _i32p, _u16p, _u16p, _f32p]
        L.vso_identity_row_swizzle.restype = None
        L.vso_identity_row_swizzle.argtypes = [ctypes.c_int, _i32p]
        L.vso_sorted_row_swizzle.restype = None
        L.vso_sorted_row_swizzle.argtypes = [ctypes.c_int, _i32p, _i32p]
        L.vso_make_dense_matrix_f32.restype = None
        L.vso_make_dense_matrix_f32.argtypes = [ctypes.c_int64, ctypes.c_int64, _f32p]
        L.vso_make_dense_matrix_f16.restype = None
        L.vso_make_dense_matrix_f16.argtypes = [ctypes.c_int64, ctypes.c_int64, _u16p]
        L.vso_max_threads.restype = ctypes.c_int
        L.vso_max_threads.argtypes = []
        _lib = L
    return _lib


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f16(a):
    return np.ascontiguousarray(a, dtype=np.float16)


def _ptr(a, ctype):
    return a.ctypes.data_as(ctypes.POINTER(ctype))


def half_to_float(bits):
    return float(lib().vso_half_to_float(int(bits)))


def float_to_half(x):
    return int(lib().vso_float_to_half(float(np.float32(x))))


def spmm_host_ref_f32(m_vec, vec_length, k, n, row_offsets, column_indices, values, rhs_matrix, threads=1):
    ro, ci, va, rhs = _i32(row_offsets), _i32(column_indices), _f16(values), _f16(rhs_matrix)
    out = np.empty((m_vec * vec_length, k), dtype=np.float32)
    args = (m_vec, vec_length, k, n, _ptr(ro, ctypes.c_int32), _ptr(ci, ctypes.c_int32),
            _ptr(va.view(np.uint16), ctypes.c_uint16), _ptr(rhs.view(np.uint16), ctypes.c_uint16),
            _ptr(out, ctypes.c_float))
    if threads == 1:
        lib().vso_spmm_host_ref_f32(*args)
    else:
        lib().vso_spmm_host_ref_f32_mt(*args, threads)
    return out


def sddmm_host_ref_f16(m_vec, k, vec_length, row_offsets, col_indices, lhs_matrix, rhs_matrix, threads=1):
    ro, ci, lhs, rhs = _i32(row_offsets), _i32(col_indices), _f16(lhs_matrix), _f16(rhs_matrix)
    nnz = int(ro[m_vec]) * vec_length
    out = np.empty(nnz, dtype=np.float16)
    args = (m_vec, k, vec_length, _ptr(ro, ctypes.c_int32), _ptr(ci, ctypes.c_int32),
            _ptr(lhs.view(np.uint16), ctypes.c_uint16), _ptr(rhs.view(np.uint16), ctypes.c_uint16),
            _ptr(out.view(np.uint16), ctypes.c_uint16))
    if threads == 1:
        lib().vso_sddmm_host_ref_f16(*args)
    else:
        lib().vso_sddmm_host_ref_f16_mt(*args, threads)
    return out


def sddmm_host_ref_f32(m_vec, k, vec_length, row_offsets, col_indices, lhs_matrix, rhs_matrix):
    ro, ci, lhs, rhs = _i32(row_offsets), _i32(col_indices), _f16(lhs_matrix), _f16(rhs_matrix)
    nnz = int(ro[m_vec]) * vec_length
    out = np.empty(nnz, dtype=np.float32)
    lib().vso_sddmm_host_ref_f32(m_vec, k, vec_length, _ptr(ro, ctypes.c_int32), _ptr(ci, ctypes.c_int32),
                                 _ptr(lhs.view(np.uint16), ctypes.c_uint16),
                                 _ptr(rhs.view(np.uint16), ctypes.c_uint16), _ptr(out, ctypes.c_float))
    return out


def identity_row_swizzle(rows):
    out = np.empty(rows, dtype=np.int32)
    lib().vso_identity_row_swizzle(rows, _ptr(out, ctypes.c_int32))
    return out


def sorted_row_swizzle(rows, row_offsets):
    ro = _i32(row_offsets)
    out = np.empty(rows, dtype=np.int32)
    lib().vso_sorted_row_swizzle(rows, _ptr(ro, ctypes.c_int32), _ptr(out, ctypes.c_int32))
    return out


def make_dense_matrix_f32(count, skip=0):
    out = np.empty(count, dtype=np.float32)
    lib().vso_make_dense_matrix_f32(count, skip, _ptr(out, ctypes.c_float))
    return out


def make_dense_matrix_f16(count, skip=0):
    out = np.empty(count, dtype=np.float16)
    lib().vso_make_dense_matrix_f16(count, skip, _ptr(out.view(np.uint16), ctypes.c_uint16))
    return out


def max_threads():
    return int(lib().vso_max_threads())
