/*
 * vsparse_shim.hpp - the reference's C++ operator names on top of the C ABI of vsparse.h.
 *
 * Same namespaces, function names, overload sets and argument order as the reference's operator
 * headers (include/wmma_spmm.cuh:7-29, include/cuda_spmm.cuh:7-29, include/wmma_sddmm.cuh:7-33,
 * include/cuda_sddmm.cuh:7-32), so its call sites (spmm_benchmark.cpp:127,131 and
 * sddmm_benchmark.cpp:257,262) compile unchanged against this header and link with -lvsparse.
 * Header-only; needs a HIP compiler for hipError_t, hipStream_t and half.
 *
 * The fp32-operand overloads exist in the reference only to print that they are unsupported
 * (src/wmma_spmm.cu:413-422) and return success; here they return hipErrorNotSupported.
 * SpMM has no stream argument in the reference: those overloads launch on the null stream.
 */
#ifndef VSPARSE_SHIM_HPP_
#define VSPARSE_SHIM_HPP_

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "vsparse.h"

namespace spmm {

inline hipError_t wmmaSpmm(int m_vec, int vec_length, int k, int n, const int* row_indices, const int* row_offsets,
    const int* column_indices, const half* values, const half* rhs_matrix, half* output_matrix) {
  return static_cast<hipError_t>(vs_wmma_spmm_f16(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
      values, rhs_matrix, output_matrix, /*stream=*/nullptr));
}

inline hipError_t wmmaSpmm(int m_vec, int vec_length, int k, int n, const int* row_indices, const int* row_offsets,
    const int* column_indices, const half* values, const half* rhs_matrix, float* output_matrix) {
  return static_cast<hipError_t>(vs_wmma_spmm_f16_f32out(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
      values, rhs_matrix, output_matrix, /*stream=*/nullptr));
}

inline hipError_t wmmaSpmm(int, int, int, int, const int*, const int*, const int*, const float*, const float*, float*) {
  return hipErrorNotSupported;
}

inline hipError_t cudaSpmm(int m_vec, int vec_length, int k, int n, const int* row_indices, const int* row_offsets,
    const int* column_indices, const half* values, const half* rhs_matrix, half* output_matrix) {
  return static_cast<hipError_t>(vs_cuda_spmm_f16(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
      values, rhs_matrix, output_matrix, /*stream=*/nullptr));
}

inline hipError_t cudaSpmm(int m_vec, int vec_length, int k, int n, const int* row_indices, const int* row_offsets,
    const int* column_indices, const half* values, const half* rhs_matrix, float* output_matrix) {
  return static_cast<hipError_t>(vs_cuda_spmm_f16_f32out(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
      values, rhs_matrix, output_matrix, /*stream=*/nullptr));
}

inline hipError_t cudaSpmm(int, int, int, int, const int*, const int*, const int*, const float*, const float*, float*) {
  return hipErrorNotSupported;
}

}  // namespace spmm

namespace sddmm {

inline hipError_t wmmaSddmm(int m_vec, int k, int n, int nonzeros_vec, const int* row_indices, const int* row_offsets,
    const int* col_indices, const half* lhs_matrix, const half* rhs_matrix, half* output_values,
    int vec_length, hipStream_t stream, int algorithm) {
  return static_cast<hipError_t>(vs_wmma_sddmm_f16(m_vec, k, n, nonzeros_vec, row_indices, row_offsets,
      col_indices, lhs_matrix, rhs_matrix, output_values, vec_length, stream, algorithm));
}

inline hipError_t wmmaSddmm(int m_vec, int k, int n, int nonzeros_vec, const int* row_indices, const int* row_offsets,
    const int* col_indices, const half* lhs_matrix, const half* rhs_matrix, float* output_values,
    int vec_length, hipStream_t stream, int algorithm) {
  return static_cast<hipError_t>(vs_wmma_sddmm_f16_f32out(m_vec, k, n, nonzeros_vec, row_indices, row_offsets,
      col_indices, lhs_matrix, rhs_matrix, output_values, vec_length, stream, algorithm));
}

inline hipError_t wmmaSddmm(int, int, int, int, const int*, const int*, const int*, const float*, const float*, float*,
    int, hipStream_t, int) {
  return hipErrorNotSupported;
}

inline hipError_t cudaSddmm(int m_vec, int k, int n, int nonzeros_vec, const int* row_indices, const int* row_offsets,
    const int* col_indices, const half* lhs_matrix, const half* rhs_matrix, half* output_values,
    int vec_length, hipStream_t stream) {
  return static_cast<hipError_t>(vs_cuda_sddmm_f16(m_vec, k, n, nonzeros_vec, row_indices, row_offsets,
      col_indices, lhs_matrix, rhs_matrix, output_values, vec_length, stream));
}

inline hipError_t cudaSddmm(int m_vec, int k, int n, int nonzeros_vec, const int* row_indices, const int* row_offsets,
    const int* col_indices, const half* lhs_matrix, const half* rhs_matrix, float* output_values,
    int vec_length, hipStream_t stream) {
  return static_cast<hipError_t>(vs_cuda_sddmm_f16_f32out(m_vec, k, n, nonzeros_vec, row_indices, row_offsets,
      col_indices, lhs_matrix, rhs_matrix, output_values, vec_length, stream));
}

inline hipError_t cudaSddmm(int, int, int, int, const int*, const int*, const int*, const float*, const float*, float*,
    int, hipStream_t) {
  return hipErrorNotSupported;
}

}  // namespace sddmm

#endif  // VSPARSE_SHIM_HPP_
