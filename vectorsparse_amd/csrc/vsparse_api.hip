// C ABI of the library: argument validation and dispatch to the kernel launchers.
#include "../../include/vsparse.h"

#include <algorithm>
#include <cstring>
#include <numeric>
#include <vector>

#include "vs_common.hpp"

namespace vs {
// Launch-shape overrides: a process-wide default, and a per-thread copy that replaces it for the calls a thread
// makes once that thread has set one of its own (launch shapes are decided on the host inside the call, so two
// threads - or one thread between two calls - never see each other's choices).
static Options g_options;
static thread_local Options t_options;
static thread_local bool t_options_active = false;

const Options &options() { return t_options_active ? t_options : g_options; }
}  // namespace vs

namespace vs {

// Zeros for `bytes` bytes (whole 32-bit words, then the odd bytes) of each of gridDim.y buffers.
__global__ void zero_fill_kernel(unsigned char *out, long long bytes, long long stride_bytes)
{
    unsigned char *dst = out + (long long)blockIdx.y * stride_bytes;
    const long long words = bytes >> 2;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (long long)gridDim.x * blockDim.x)
        reinterpret_cast<uint32_t *>(dst)[i] = 0u;
    if (blockIdx.x == 0 && threadIdx.x < (bytes & 3)) dst[(words << 2) + threadIdx.x] = 0;
}

int launch_zero_fill(void *out, long long bytes, long long stride_bytes, int batch, hipStream_t stream)
{
    if (batch > 65535) return hipErrorNotSupported;
    if (bytes <= 0 || batch <= 0) return hipSuccess;
    long long blocks = (bytes / 4 + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
    hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)blocks, (unsigned)batch), dim3(256), 0, stream,
                       static_cast<unsigned char *>(out), bytes, stride_bytes);
    return (int)hipGetLastError();
}

}  // namespace vs

namespace {

using vs::half_t;

// The contraction is empty (k == 0): every sampled output of SDDMM is an empty sum.
int sddmm_zero_outputs(void *out, long long nonzeros_vec, int vec_length, size_t out_elem, int batch,
                       long long stride_out_elems, hipStream_t stream)
{
    return vs::launch_zero_fill(out, nonzeros_vec * vec_length * (long long)out_elem,
                                stride_out_elems * (long long)out_elem, batch, stream);
}

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

bool vec_ok(int v) { return v == 1 || v == 2 || v == 4 || v == 8; }

int check_spmm(int m_vec, int vec_length, int k, int n, const int *row_indices, const int *row_offsets,
               const int *column_indices, const void *values, const void *rhs, const void *out, size_t out_elem)
{
    if (m_vec < 0 || k < 0 || n < 0 || !vec_ok(vec_length)) return VS_ERROR_INVALID_VALUE;
    if (m_vec == 0 || k == 0) return VS_SUCCESS;
    if (!row_indices || !row_offsets || !out) return VS_ERROR_INVALID_VALUE;
    // column_indices / values may be null when the pattern has no nonzero at all (an empty device
    // allocation); the host cannot see the pattern, so only the dense operand is required here.
    (void)column_indices;
    if (n > 0 && !rhs) return VS_ERROR_INVALID_VALUE;
    (void)out_elem;
    if (!aligned(values, 2 * (size_t)vec_length) || !aligned(rhs, 16) || !aligned(out, 16))
        return VS_ERROR_INVALID_VALUE;
    return VS_SUCCESS;
}

int check_sddmm(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                const int *col_indices, const void *lhs, const void *rhs, const void *out, int vec_length,
                size_t out_elem)
{
    if (m_vec < 0 || k < 0 || n < 0 || nonzeros_vec < 0 || !vec_ok(vec_length)) return VS_ERROR_INVALID_VALUE;
    if (m_vec == 0 || nonzeros_vec == 0) return VS_SUCCESS;
    if (!row_indices || !row_offsets || !col_indices || !out) return VS_ERROR_INVALID_VALUE;
    if (k > 0 && (!lhs || !rhs)) return VS_ERROR_INVALID_VALUE;  // k == 0: the dense operands are empty
    if (!aligned(out, out_elem * (size_t)vec_length)) return VS_ERROR_INVALID_VALUE;
    if (k % 8 == 0 && (!aligned(lhs, 16) || !aligned(rhs, 16))) return VS_ERROR_INVALID_VALUE;
    return VS_SUCCESS;
}

}  // namespace

// the library is compiled with hidden visibility: what follows is its whole exported surface
#pragma GCC visibility push(default)
extern "C" {

int vs_version(void) { return 100; }

const char *vs_status_string(int status)
{
    switch (status) {
    case VS_SUCCESS: return "success";
    case VS_ERROR_INVALID_VALUE: return "invalid value (null pointer, negative size, misaligned operand, or unsupported vec_length/algorithm)";
    case VS_ERROR_NOT_SUPPORTED: return "shape not supported by the selected path (or beyond the size limit of an entry point that allocates nothing)";
    default: return hipGetErrorString(static_cast<hipError_t>(status));
    }
}

int vs_wmma_spmm_f16(int m_vec, int vec_length, int k, int n, const int *row_indices, const int *row_offsets,
                     const int *column_indices, const void *values, const void *rhs_matrix, void *output_matrix,
                     void *stream)
{
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_mfma<half_t>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                        static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                        static_cast<half_t *>(output_matrix), static_cast<hipStream_t>(stream));
}

int vs_wmma_spmm_f16_f32out(int m_vec, int vec_length, int k, int n, const int *row_indices,
                            const int *row_offsets, const int *column_indices, const void *values,
                            const void *rhs_matrix, float *output_matrix, void *stream)
{
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(float));
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_mfma<float>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                       static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                       output_matrix, static_cast<hipStream_t>(stream));
}

long long vs_wmma_spmm_workspace_bytes(int m_vec, int vec_length, int k, int n, int nonzeros_vec)
{
    (void)n;
    if (m_vec < 0 || k < 0 || nonzeros_vec < 0 || !vec_ok(vec_length)) return 0;
    return vs::spmm_flat_workspace_bytes(vec_length, k, nonzeros_vec);
}

static int check_spmm_ws(int nonzeros_vec, const int *column_indices, const void *values, const void *workspace,
                         long long workspace_bytes)
{
    if (nonzeros_vec < 0 || workspace_bytes < 0) return VS_ERROR_INVALID_VALUE;
    if (nonzeros_vec > 0 && (!column_indices || !values)) return VS_ERROR_INVALID_VALUE;
    if (workspace_bytes > 0 && (!workspace || !aligned(workspace, 16))) return VS_ERROR_INVALID_VALUE;
    return VS_SUCCESS;
}

int vs_wmma_spmm_f16_ws(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_indices,
                        const int *row_offsets, const int *column_indices, const void *values,
                        const void *rhs_matrix, void *output_matrix, void *workspace, long long workspace_bytes,
                        void *stream)
{
    static const int identity[1] = {0};  // the swizzle is not used by this schedule; only its presence was checked
    int st = check_spmm(m_vec, vec_length, k, n, row_indices ? row_indices : identity, row_offsets, column_indices,
                        values, rhs_matrix, output_matrix, sizeof(half_t));
    if (st == VS_SUCCESS) st = check_spmm_ws(nonzeros_vec, column_indices, values, workspace, workspace_bytes);
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_mfma_flat<half_t>(m_vec, vec_length, k, n, nonzeros_vec, row_offsets, column_indices,
                                             static_cast<const half_t *>(values),
                                             static_cast<const half_t *>(rhs_matrix),
                                             static_cast<half_t *>(output_matrix), static_cast<float *>(workspace),
                                             workspace_bytes, static_cast<hipStream_t>(stream));
}

int vs_wmma_spmm_f16_noalloc(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_indices,
                             const int *row_offsets, const int *column_indices, const void *values,
                             const void *rhs_matrix, void *output_matrix, void *stream)
{
    static const int identity[1] = {0};
    int st = check_spmm(m_vec, vec_length, k, n, row_indices ? row_indices : identity, row_offsets, column_indices,
                        values, rhs_matrix, output_matrix, sizeof(half_t));
    if (st == VS_SUCCESS) st = check_spmm_ws(nonzeros_vec, column_indices, values, nullptr, 0);
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_mfma_flat_static(m_vec, vec_length, k, n, nonzeros_vec, row_offsets, column_indices,
                                            static_cast<const half_t *>(values),
                                            static_cast<const half_t *>(rhs_matrix),
                                            static_cast<half_t *>(output_matrix), static_cast<hipStream_t>(stream));
}

long long vs_wmma_spmm_noalloc_scratch_bytes(void) { return vs::spmm_flat_scratch_bytes(); }

int vs_wmma_spmm_noalloc_reset(void *stream) { return vs::spmm_flat_scratch_reset(static_cast<hipStream_t>(stream)); }

int vs_wmma_spmm_f16_f32out_ws(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_indices,
                               const int *row_offsets, const int *column_indices, const void *values,
                               const void *rhs_matrix, float *output_matrix, void *workspace,
                               long long workspace_bytes, void *stream)
{
    static const int identity[1] = {0};
    int st = check_spmm(m_vec, vec_length, k, n, row_indices ? row_indices : identity, row_offsets, column_indices,
                        values, rhs_matrix, output_matrix, sizeof(float));
    if (st == VS_SUCCESS) st = check_spmm_ws(nonzeros_vec, column_indices, values, workspace, workspace_bytes);
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_mfma_flat<float>(m_vec, vec_length, k, n, nonzeros_vec, row_offsets, column_indices,
                                            static_cast<const half_t *>(values),
                                            static_cast<const half_t *>(rhs_matrix), output_matrix,
                                            static_cast<float *>(workspace), workspace_bytes,
                                            static_cast<hipStream_t>(stream));
}

long long vs_wmma_spmm_slab_workspace_bytes(int m_vec, int vec_length, int k, int n)
{
    if (m_vec < 0 || k < 0 || n < 0 || !vec_ok(vec_length)) return 0;
    return vs::spmm_slab_workspace_bytes(m_vec, vec_length, k, vs::choose_spmm_slab_parts(m_vec, k, n));
}

int vs_wmma_spmm_f16_slab(int m_vec, int vec_length, int k, int n, const int *row_indices, const int *row_offsets,
                          const int *column_indices, const void *values, const void *rhs_matrix, void *output_matrix,
                          void *workspace, long long workspace_bytes, void *stream)
{
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (workspace_bytes < 0 || (workspace_bytes > 0 && (!workspace || !aligned(workspace, 16)))) return VS_ERROR_INVALID_VALUE;
    return vs::launch_spmm_mfma_slab(m_vec, vec_length, k, n, vs::choose_spmm_slab_parts(m_vec, k, n), row_indices,
                                     row_offsets, column_indices, static_cast<const half_t *>(values),
                                     static_cast<const half_t *>(rhs_matrix), static_cast<half_t *>(output_matrix),
                                     workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int vs_cuda_spmm_f16(int m_vec, int vec_length, int k, int n, const int *row_indices, const int *row_offsets,
                     const int *column_indices, const void *values, const void *rhs_matrix, void *output_matrix,
                     void *stream)
{
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_valu<half_t>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                        static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                        static_cast<half_t *>(output_matrix), static_cast<hipStream_t>(stream));
}

int vs_cuda_spmm_f16_f32out(int m_vec, int vec_length, int k, int n, const int *row_indices,
                            const int *row_offsets, const int *column_indices, const void *values,
                            const void *rhs_matrix, float *output_matrix, void *stream)
{
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(float));
    if (st != VS_SUCCESS) return st;
    return vs::launch_spmm_valu<float>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                       static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                       output_matrix, static_cast<hipStream_t>(stream));
}

int vs_wmma_sddmm_f16(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const void *lhs_matrix, const void *rhs_matrix, void *output_values,
                      int vec_length, void *stream, int algorithm)
{
    if (algorithm < 0 || algorithm > 2) return VS_ERROR_INVALID_VALUE;
    int st = check_sddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                         output_values, vec_length, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (k == 0 && m_vec > 0)
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(half_t), 1, 0, static_cast<hipStream_t>(stream));
    vs::Batch one;
    one.algorithm = algorithm;
    return vs::launch_sddmm_mfma<half_t>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                                         static_cast<const half_t *>(lhs_matrix),
                                         static_cast<const half_t *>(rhs_matrix),
                                         static_cast<half_t *>(output_values), vec_length,
                                         static_cast<hipStream_t>(stream), one);
}

int vs_wmma_sddmm_f16_f32out(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                             const int *row_offsets, const int *col_indices, const void *lhs_matrix,
                             const void *rhs_matrix, float *output_values, int vec_length, void *stream,
                             int algorithm)
{
    if (algorithm < 0 || algorithm > 2) return VS_ERROR_INVALID_VALUE;
    int st = check_sddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                         output_values, vec_length, sizeof(float));
    if (st != VS_SUCCESS) return st;
    if (k == 0 && m_vec > 0)
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(float), 1, 0, static_cast<hipStream_t>(stream));
    vs::Batch one;
    one.algorithm = algorithm;
    return vs::launch_sddmm_mfma<float>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                                        static_cast<const half_t *>(lhs_matrix),
                                        static_cast<const half_t *>(rhs_matrix), output_values, vec_length,
                                        static_cast<hipStream_t>(stream), one);
}

int vs_cuda_sddmm_f16(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const void *lhs_matrix, const void *rhs_matrix, void *output_values,
                      int vec_length, void *stream)
{
    int st = check_sddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                         output_values, vec_length, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (k == 0 && m_vec > 0)
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(half_t), 1, 0, static_cast<hipStream_t>(stream));
    return vs::launch_sddmm_valu<half_t>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                                         static_cast<const half_t *>(lhs_matrix),
                                         static_cast<const half_t *>(rhs_matrix),
                                         static_cast<half_t *>(output_values), vec_length,
                                         static_cast<hipStream_t>(stream));
}

int vs_cuda_sddmm_f16_f32out(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                             const int *row_offsets, const int *col_indices, const void *lhs_matrix,
                             const void *rhs_matrix, float *output_values, int vec_length, void *stream)
{
    int st = check_sddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                         output_values, vec_length, sizeof(float));
    if (st != VS_SUCCESS) return st;
    if (k == 0 && m_vec > 0)
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(float), 1, 0, static_cast<hipStream_t>(stream));
    return vs::launch_sddmm_valu<float>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                                        static_cast<const half_t *>(lhs_matrix),
                                        static_cast<const half_t *>(rhs_matrix), output_values, vec_length,
                                        static_cast<hipStream_t>(stream));
}

static vs::Batch make_batch(int batch, long long a, long long b, long long out, int nonzeros_vec = -1,
                            int longest_row_vec = -1, int long_rows = -1)
{
    vs::Batch x;
    x.count = batch;
    x.stride_a = a;
    x.stride_b = b;
    x.stride_out = out;
    x.nonzeros_vec = nonzeros_vec;
    x.longest_row_vec = longest_row_vec;
    x.long_rows = long_rows;
    return x;
}

// Strides keep every problem's operand as aligned as the first one.
static bool stride_ok(long long stride, long long multiple) { return stride >= 0 && stride % multiple == 0; }

int vs_wmma_spmm_f16_batched(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                             int longest_row_vec, const int *row_indices,
                             const int *row_offsets, const int *column_indices, const void *values,
                             long long stride_values, const void *rhs_matrix, long long stride_rhs,
                             void *output_matrix, long long stride_output, void *stream)
{
    if (batch < 0) return VS_ERROR_INVALID_VALUE;
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (!stride_ok(stride_values, vec_length) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, 8))
        return VS_ERROR_INVALID_VALUE;
    return vs::launch_spmm_mfma<half_t>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                        static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                        static_cast<half_t *>(output_matrix), static_cast<hipStream_t>(stream),
                                        make_batch(batch, stride_values, stride_rhs, stride_output, nonzeros_vec, longest_row_vec));
}

int vs_wmma_spmm_f16_batched_sorted(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                                    int longest_row_vec, int long_rows, const int *row_indices, const int *row_offsets,
                                    const int *column_indices, const void *values, long long stride_values,
                                    const void *rhs_matrix, long long stride_rhs, void *output_matrix,
                                    long long stride_output, void *stream)
{
    if (batch < 0) return VS_ERROR_INVALID_VALUE;
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (!stride_ok(stride_values, vec_length) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, 8))
        return VS_ERROR_INVALID_VALUE;
    return vs::launch_spmm_mfma<half_t>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                        static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                        static_cast<half_t *>(output_matrix), static_cast<hipStream_t>(stream),
                                        make_batch(batch, stride_values, stride_rhs, stride_output, nonzeros_vec,
                                                   longest_row_vec, long_rows < 0 ? -1 : long_rows));
}

int vs_wmma_spmm_launch_shape(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                              int longest_row_vec, int long_rows, int shape[8])
{
    if (shape == nullptr || batch < 1 || batch > 65535 || m_vec < 1 || k < 1 || n < 0) return VS_ERROR_INVALID_VALUE;
    if (vec_length != 1 && vec_length != 2 && vec_length != 4 && vec_length != 8) return VS_ERROR_INVALID_VALUE;
    const vs::SpmmShape chosen = vs::choose_spmm_shape(
        false, m_vec, vec_length, k, n, make_batch(batch, 0, 0, 0, nonzeros_vec, longest_row_vec, long_rows < 0 ? -1 : long_rows));
    shape[0] = chosen.cols_per_lane;
    shape[1] = chosen.steps_in_flight;
    shape[2] = chosen.waves;
    shape[3] = chosen.blocks_per_wave;
    shape[4] = chosen.team_slots;
    shape[5] = chosen.ragged ? 1 : 0;
    shape[6] = chosen.dma ? 1 : 0;
    shape[7] = chosen.pipelined ? 1 : 0;
    return VS_SUCCESS;
}

int vs_cuda_spmm_f16_batched(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                             int longest_row_vec, const int *row_indices,
                             const int *row_offsets, const int *column_indices, const void *values,
                             long long stride_values, const void *rhs_matrix, long long stride_rhs,
                             void *output_matrix, long long stride_output, void *stream)
{
    if (batch < 0) return VS_ERROR_INVALID_VALUE;
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (!stride_ok(stride_values, vec_length) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, 8))
        return VS_ERROR_INVALID_VALUE;
    return vs::launch_spmm_valu<half_t>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                        static_cast<const half_t *>(values), static_cast<const half_t *>(rhs_matrix),
                                        static_cast<half_t *>(output_matrix), static_cast<hipStream_t>(stream),
                                        make_batch(batch, stride_values, stride_rhs, stride_output, nonzeros_vec, longest_row_vec));
}

int vs_wmma_sddmm_f16_batched(int batch, int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                              const int *row_offsets, const int *col_indices, const void *lhs_matrix,
                              long long stride_lhs, const void *rhs_matrix, long long stride_rhs,
                              void *output_values, long long stride_output, int vec_length, void *stream,
                              int algorithm)
{
    if (batch < 0 || algorithm < 0 || algorithm > 2) return VS_ERROR_INVALID_VALUE;
    int st = check_sddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                         output_values, vec_length, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (k == 0 && m_vec > 0) {
        if (!stride_ok(stride_output, vec_length)) return VS_ERROR_INVALID_VALUE;
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(half_t), batch, stride_output, static_cast<hipStream_t>(stream));
    }
    if (!stride_ok(stride_lhs, 8) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, vec_length))
        return VS_ERROR_INVALID_VALUE;
    vs::Batch many = make_batch(batch, stride_lhs, stride_rhs, stride_output);
    many.algorithm = algorithm;
    return vs::launch_sddmm_mfma<half_t>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                                         static_cast<const half_t *>(lhs_matrix),
                                         static_cast<const half_t *>(rhs_matrix),
                                         static_cast<half_t *>(output_values), vec_length,
                                         static_cast<hipStream_t>(stream), many);
}

int vs_cuda_sddmm_f16_batched(int batch, int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                              const int *row_offsets, const int *col_indices, const void *lhs_matrix,
                              long long stride_lhs, const void *rhs_matrix, long long stride_rhs,
                              void *output_values, long long stride_output, int vec_length, void *stream)
{
    if (batch < 0) return VS_ERROR_INVALID_VALUE;
    int st = check_sddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                         output_values, vec_length, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (k == 0 && m_vec > 0) {
        if (!stride_ok(stride_output, vec_length)) return VS_ERROR_INVALID_VALUE;
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(half_t), batch, stride_output, static_cast<hipStream_t>(stream));
    }
    const long long in_mult = (k % 8 == 0) ? 8 : 1;
    if (!stride_ok(stride_lhs, in_mult) || !stride_ok(stride_rhs, in_mult) || !stride_ok(stride_output, vec_length))
        return VS_ERROR_INVALID_VALUE;
    return vs::launch_sddmm_valu<half_t>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                                         static_cast<const half_t *>(lhs_matrix),
                                         static_cast<const half_t *>(rhs_matrix),
                                         static_cast<half_t *>(output_values), vec_length,
                                         static_cast<hipStream_t>(stream),
                                         make_batch(batch, stride_lhs, stride_rhs, stride_output));
}

int vs_wmma_spmm_softmax_f16_batched(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                             int longest_row_vec, const int *row_indices,
                                     const int *row_offsets, const int *column_indices, const void *scores,
                                     long long stride_scores, const void *rhs_matrix, long long stride_rhs,
                                     void *output_matrix, long long stride_output, float scale, void *stream)
{
    if (batch < 0) return VS_ERROR_INVALID_VALUE;
    int st = check_spmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, scores, rhs_matrix,
                        output_matrix, sizeof(half_t));
    if (st != VS_SUCCESS) return st;
    if (!stride_ok(stride_scores, vec_length) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, 8))
        return VS_ERROR_INVALID_VALUE;
    return vs::launch_spmm_softmax_mfma(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                                        static_cast<const half_t *>(scores), static_cast<const half_t *>(rhs_matrix),
                                        static_cast<half_t *>(output_matrix), scale,
                                        static_cast<hipStream_t>(stream),
                                        make_batch(batch, stride_scores, stride_rhs, stride_output, nonzeros_vec, longest_row_vec));
}

int vs_sparse_attention_f16(int batch, int m_vec, int vec_length, int n, int d_qk, int d_v, const int *row_indices,
                            const int *row_offsets, const int *col_indices, const void *q, long long stride_q,
                            const void *k, long long stride_k, const void *v, long long stride_v, void *out,
                            long long stride_out, float scale, int rows_per_workgroup, const void *plan,
                            long long plan_bytes, void *stream)
{
    if (batch < 0 || m_vec < 0 || n < 0 || d_qk < 0 || d_v < 0 || !vec_ok(vec_length)) return VS_ERROR_INVALID_VALUE;
    if (rows_per_workgroup < 0 || rows_per_workgroup > 128) return VS_ERROR_INVALID_VALUE;
    if (plan && (rows_per_workgroup < 2 || !aligned(plan, 16))) return VS_ERROR_INVALID_VALUE;
    // the kernels read the plan at offsets that follow from THIS launch's shape before they know whether it is
    // theirs: a buffer too small for this shape is rejected here, whatever it holds
    if (plan && (d_qk <= 0 || d_v <= 0 ||
                 plan_bytes < vs::sparse_attention_plan_bytes(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup) ||
                 vs::sparse_attention_plan_bytes(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup) <= 0))
        return VS_ERROR_INVALID_VALUE;
    if (batch == 0 || m_vec == 0 || d_v == 0) return VS_SUCCESS;
    if (!row_indices || !row_offsets || !q || !out) return VS_ERROR_INVALID_VALUE;
    if (n > 0 && (!k || !v)) return VS_ERROR_INVALID_VALUE;
    if (!aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || !aligned(out, 16)) return VS_ERROR_INVALID_VALUE;
    if (!stride_ok(stride_q, 8) || !stride_ok(stride_k, 8) || !stride_ok(stride_v, 8) || !stride_ok(stride_out, 8))
        return VS_ERROR_INVALID_VALUE;
    if (rows_per_workgroup > 1)  // union-gather kernel: pays off when neighbouring rows share columns
        return vs::launch_sparse_attention_union(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup, row_offsets,
                                                 col_indices, static_cast<const int *>(plan), static_cast<const half_t *>(q), static_cast<const half_t *>(k),
                                                 static_cast<const half_t *>(v), static_cast<half_t *>(out), scale,
                                                 static_cast<hipStream_t>(stream),
                                                 make_batch(batch, stride_q, stride_k, stride_out), stride_v);
    return vs::launch_sparse_attention(m_vec, vec_length, d_qk, d_v, row_indices, row_offsets, col_indices,
                                       static_cast<const half_t *>(q), static_cast<const half_t *>(k),
                                       static_cast<const half_t *>(v), static_cast<half_t *>(out), scale,
                                       static_cast<hipStream_t>(stream), make_batch(batch, stride_q, stride_k, stride_out),
                                       stride_v);
}

long long vs_sparse_attention_plan_bytes(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows_per_workgroup)
{
    if (m_vec < 0 || n < 0 || !vec_ok(vec_length) || rows_per_workgroup < 2 || rows_per_workgroup > 128) return 0;
    return vs::sparse_attention_plan_bytes(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup);
}

int vs_sparse_attention_plan(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows_per_workgroup,
                             const int *row_offsets, const int *col_indices, void *plan, long long plan_bytes,
                             void *stream)
{
    if (m_vec < 0 || n < 0 || !vec_ok(vec_length) || rows_per_workgroup < 2 || rows_per_workgroup > 128)
        return VS_ERROR_INVALID_VALUE;
    if (!plan || !aligned(plan, 16) || (m_vec > 0 && !row_offsets)) return VS_ERROR_INVALID_VALUE;
    return vs::launch_sparse_attention_plan(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup, row_offsets,
                                            col_indices, static_cast<int *>(plan), plan_bytes,
                                            static_cast<hipStream_t>(stream));
}

int vs_sparse_attention_union_capacity(int vec_length, int n, int d_qk, int d_v, int rows_per_workgroup, int with_plan,
                                       int *rows_used)
{
    if (!vec_ok(vec_length) || n < 0 || rows_per_workgroup < 2 || rows_per_workgroup > 128) return 0;
    return vs::sparse_attention_union_capacity(vec_length, n, d_qk, d_v, rows_per_workgroup, with_plan != 0, rows_used);
}

int vs_sparse_softmax_f16(int batch, int m_vec, int vec_length, const int *row_indices, const int *row_offsets,
                          const void *values_in, long long stride_in, void *values_out, long long stride_out,
                          float scale, void *stream)
{
    if (batch < 0 || m_vec < 0 || !vec_ok(vec_length)) return VS_ERROR_INVALID_VALUE;
    if (batch == 0 || m_vec == 0) return VS_SUCCESS;
    if (!row_indices || !row_offsets) return VS_ERROR_INVALID_VALUE;
    if (!aligned(values_in, 2 * (size_t)vec_length) || !aligned(values_out, 2 * (size_t)vec_length))
        return VS_ERROR_INVALID_VALUE;
    if (!stride_ok(stride_in, vec_length) || !stride_ok(stride_out, vec_length)) return VS_ERROR_INVALID_VALUE;
    return vs::launch_sparse_softmax(m_vec, vec_length, row_indices, row_offsets,
                                     static_cast<const half_t *>(values_in), static_cast<half_t *>(values_out),
                                     scale, static_cast<hipStream_t>(stream),
                                     make_batch(batch, stride_in, 0, stride_out));
}

long long vs_sparse_softmax_row_parts_workspace_bytes(int batch, int vec_length, int n_split, int parts_max)
{
    if (!vec_ok(vec_length)) return 0;
    return vs::sparse_softmax_row_parts_workspace_bytes(batch, vec_length, n_split, parts_max);
}

int vs_sparse_softmax_f16_row_parts(int batch, int vec_length, int n_slots, const int *slots, int n_split, int parts_max,
                                    const void *values_in, long long stride_in, void *values_out, long long stride_out,
                                    float scale, void *workspace, long long workspace_bytes, void *stream)
{
    if (batch < 0 || n_slots < 0 || n_split < 0 || parts_max < 0 || workspace_bytes < 0 || !vec_ok(vec_length))
        return VS_ERROR_INVALID_VALUE;
    if (batch == 0 || n_slots == 0) return VS_SUCCESS;
    if (!slots || !aligned(slots, 16)) return VS_ERROR_INVALID_VALUE;
    if (!aligned(values_in, 2 * (size_t)vec_length) || !aligned(values_out, 2 * (size_t)vec_length))
        return VS_ERROR_INVALID_VALUE;
    if (!stride_ok(stride_in, vec_length) || !stride_ok(stride_out, vec_length)) return VS_ERROR_INVALID_VALUE;
    if (workspace_bytes > 0 && (!workspace || !aligned(workspace, 8))) return VS_ERROR_INVALID_VALUE;
    return vs::launch_sparse_softmax_row_parts(vec_length, n_slots, slots, n_split, parts_max,
                                               static_cast<const half_t *>(values_in), static_cast<half_t *>(values_out),
                                               scale, workspace, workspace_bytes, static_cast<hipStream_t>(stream),
                                               make_batch(batch, stride_in, 0, stride_out));
}

void vs_identity_row_swizzle(int rows, int *row_indices)
{
    if (rows <= 0 || !row_indices) return;
    std::iota(row_indices, row_indices + rows, 0);
}

void vs_sorted_row_swizzle(int rows, const int *row_offsets, int *row_indices)
{
    if (rows <= 0 || !row_offsets || !row_indices) return;
    std::iota(row_indices, row_indices + rows, 0);
    // Longest rows first so they are dispatched first; a stable sort keeps equal-length rows in
    // ascending order, which makes the swizzle reproducible.
    std::stable_sort(row_indices, row_indices + rows, [row_offsets](int a, int b) {
        return row_offsets[a + 1] - row_offsets[a] > row_offsets[b + 1] - row_offsets[b];
    });
}

int vs_spmm_row_parts(int m_vec, const int *row_offsets, int limit_vec, int *slots, int max_slots, int *n_slots,
                      int *n_split, int *parts_max, int *longest_part_vec)
{
    if (m_vec < 0 || !row_offsets || !n_slots || !n_split || !parts_max || !longest_part_vec || max_slots < 0 ||
        (max_slots > 0 && !slots) || limit_vec < 0)
        return VS_ERROR_INVALID_VALUE;
    // Default: rows of more than 1152 vectors and of more than four mean lengths - a matrix of uniformly long rows
    // has no tail to cut (256 rows of 2304 vectors, N = 256: 14.6 us whole, 17.1 us in halves).
    long long limit = limit_vec;
    if (limit <= 0) {
        const long long mean = m_vec > 0 ? ((long long)row_offsets[m_vec] - row_offsets[0]) / m_vec : 0;
        limit = 4 * mean > 1152 ? 4 * mean : 1152;
    }
    limit = (limit + 63) / 64 * 64;  // whole blocks of two 32-vector steps
    struct Part {
        int row, beg, end, info;
    };
    std::vector<Part> parts;
    parts.reserve((size_t)m_vec + 64);
    int split = 0, most = 0, longest = 0;
    for (int row = 0; row < m_vec; ++row) {
        const int beg = row_offsets[row], end = row_offsets[row + 1];
        if (end < beg) return VS_ERROR_INVALID_VALUE;
        const long long len = (long long)end - beg;
        if (len <= limit) {
            parts.push_back({row, beg, end, 0});
            longest = len > longest ? (int)len : longest;
            continue;
        }
        // equal parts, each a whole number of blocks, no more of them than the limit asks for
        long long count = (len + limit - 1) / limit;
        if (count > 255) count = 255;
        const long long per = ((len + count - 1) / count + 63) / 64 * 64;
        count = (len + per - 1) / per;
        // (rounding the part up to whole blocks may take the whole row; a split row's number has 15 bits in the
        // part info: past 32767 split rows the others stay whole - slower to finish, the same result)
        if (count < 2 || split >= 32767) {
            parts.push_back({row, beg, end, 0});
            longest = len > longest ? (int)len : longest;
            continue;
        }
        for (long long p = 0; p < count; ++p) {
            const long long from = beg + p * per;
            const long long to = from + per < end ? from + per : end;
            parts.push_back({row, (int)from, (int)to, (int)count | (int)(p << 8) | (split << 16)});
        }
        longest = per > longest ? (int)per : longest;
        most = count > most ? (int)count : most;
        ++split;
    }
    // Longest first, as the sorted swizzle dispatches whole rows (include/bm_test_utils.h:200-215 of the
    // reference); a stable sort keeps the list reproducible and the parts of a row in ascending order.
    std::stable_sort(parts.begin(), parts.end(),
                     [](const Part &a, const Part &b) { return a.end - a.beg > b.end - b.beg; });
    *n_slots = (int)parts.size();
    *n_split = split;
    *parts_max = most;
    *longest_part_vec = longest;
    if ((long long)parts.size() + split > max_slots) return VS_ERROR_NOT_SUPPORTED;  // the counts say what the list needs
    for (size_t i = 0; i < parts.size(); ++i) {
        slots[4 * i] = parts[i].row;
        slots[4 * i + 1] = parts[i].beg;
        slots[4 * i + 2] = parts[i].end;
        slots[4 * i + 3] = parts[i].info;
        if (parts[i].info != 0 && ((parts[i].info >> 8) & 255) == 0) {  // behind the list: {row, parts} per split row
            int *entry = slots + 4 * (parts.size() + (size_t)(parts[i].info >> 16));
            entry[0] = parts[i].row;
            entry[1] = parts[i].info & 255;
            entry[2] = entry[3] = 0;
        }
    }
    return VS_SUCCESS;
}

long long vs_wmma_spmm_row_parts_workspace_bytes(int batch, int vec_length, int k, int n_split, int parts_max)
{
    if (!vec_ok(vec_length)) return 0;
    return vs::spmm_row_parts_workspace_bytes(batch, vec_length, k, n_split, parts_max);
}

int vs_wmma_spmm_f16_row_parts(int batch, int vec_length, int k, int n, int n_slots, const int *slots, int n_split,
                               int parts_max, int nonzeros_vec, int longest_part_vec, const int *column_indices,
                               const void *values, long long stride_values, const void *rhs_matrix, long long stride_rhs,
                               void *output_matrix, long long stride_output, void *workspace, long long workspace_bytes,
                               void *stream)
{
    if (!vec_ok(vec_length) || batch < 0 || k < 0 || n < 0 || n_slots < 0 || n_split < 0 || parts_max < 0 ||
        nonzeros_vec < 0 || longest_part_vec < 0 || workspace_bytes < 0)
        return VS_ERROR_INVALID_VALUE;
    if (n_slots > 0 && (!slots || !aligned(slots, 16))) return VS_ERROR_INVALID_VALUE;
    if (n_slots > 0 && k > 0 && (!rhs_matrix || !output_matrix)) return VS_ERROR_INVALID_VALUE;
    if (nonzeros_vec > 0 && (!column_indices || !values)) return VS_ERROR_INVALID_VALUE;
    if (!aligned(values, 2 * vec_length) || !aligned(rhs_matrix, 16) || !aligned(output_matrix, 16))
        return VS_ERROR_INVALID_VALUE;
    // every problem of the batch keeps the alignment of the first (as the other batched entry points ask)
    if (!stride_ok(stride_values, vec_length) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, 8))
        return VS_ERROR_INVALID_VALUE;
    if (workspace_bytes > 0 && (!workspace || !aligned(workspace, 16))) return VS_ERROR_INVALID_VALUE;
    return vs::launch_spmm_mfma_row_parts(vec_length, k, n, n_slots, slots, n_split, parts_max, nonzeros_vec,
                                          longest_part_vec, column_indices, static_cast<const half_t *>(values),
                                          static_cast<const half_t *>(rhs_matrix), static_cast<half_t *>(output_matrix),
                                          workspace, workspace_bytes, static_cast<hipStream_t>(stream),
                                          make_batch(batch, stride_values, stride_rhs, stride_output));
}

int vs_wmma_sddmm_f16_row_parts(int batch, int k, int n, int n_slots, const int *slots, int nonzeros_vec,
                                const int *col_indices, const void *lhs_matrix, long long stride_lhs,
                                const void *rhs_matrix, long long stride_rhs, void *output_values, long long stride_output,
                                int vec_length, void *stream)
{
    if (!vec_ok(vec_length) || batch < 0 || k < 0 || n < 0 || n_slots < 0 || nonzeros_vec < 0)
        return VS_ERROR_INVALID_VALUE;
    if (batch == 0 || n_slots == 0 || nonzeros_vec == 0) return VS_SUCCESS;
    if (!slots || !aligned(slots, 16) || !col_indices || !output_values) return VS_ERROR_INVALID_VALUE;
    if (k > 0 && (!lhs_matrix || !rhs_matrix)) return VS_ERROR_INVALID_VALUE;
    if (!aligned(output_values, sizeof(half_t) * (size_t)vec_length)) return VS_ERROR_INVALID_VALUE;
    if (!stride_ok(stride_lhs, 8) || !stride_ok(stride_rhs, 8) || !stride_ok(stride_output, vec_length))
        return VS_ERROR_INVALID_VALUE;
    if (k == 0)
        return sddmm_zero_outputs(output_values, nonzeros_vec, vec_length, sizeof(half_t), batch, stride_output,
                                  static_cast<hipStream_t>(stream));
    if (k % 8 != 0) return VS_ERROR_NOT_SUPPORTED;
    if (!aligned(lhs_matrix, 16) || !aligned(rhs_matrix, 16)) return VS_ERROR_INVALID_VALUE;
    vs::Batch b = make_batch(batch, stride_lhs, stride_rhs, stride_output);
    b.algorithm = 1;
    b.row_parts = true;
    return vs::launch_sddmm_mfma<half_t>(n_slots, k, n, nonzeros_vec, slots, nullptr, col_indices,
                                         static_cast<const half_t *>(lhs_matrix), static_cast<const half_t *>(rhs_matrix),
                                         static_cast<half_t *>(output_values), vec_length,
                                         static_cast<hipStream_t>(stream), b);
}

static int set_option_field(vs::Options &o, const char *name, int value)
{
    if (!name || value < 0) return VS_ERROR_INVALID_VALUE;
    if (std::strcmp(name, "spmm_waves") == 0) {
        if (value > 16) return VS_ERROR_INVALID_VALUE;
        o.spmm_waves = value;
    } else if (std::strcmp(name, "spmm_cols_per_lane") == 0) {
        if (value != 0 && value != 4 && value != 8) return VS_ERROR_INVALID_VALUE;
        o.spmm_cols_per_lane = value;
    } else if (std::strcmp(name, "spmm_teams") == 0) {
        if (value > 2) return VS_ERROR_INVALID_VALUE;
        o.spmm_teams = value;
    } else if (std::strcmp(name, "spmm_blocks_per_wave") == 0) {
        if (value > 64 || (value & (value - 1)) != 0) return VS_ERROR_INVALID_VALUE;
        o.spmm_blocks_per_wave = value;
    } else if (std::strcmp(name, "spmm_pipe") == 0) {
        if (value > 2) return VS_ERROR_INVALID_VALUE;
        o.spmm_pipe = value;
    } else if (std::strcmp(name, "spmm_guard_waves") == 0) {
        if (value > 16) return VS_ERROR_INVALID_VALUE;
        o.spmm_guard_waves = value;
    } else if (std::strcmp(name, "spmm_steps") == 0) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return VS_ERROR_INVALID_VALUE;
#ifndef VS_RETIRED_VARIANTS
        if (value == 4) return VS_ERROR_NOT_SUPPORTED;  // four steps in flight: compiled only with VS_RETIRED_VARIANTS
#endif
        o.spmm_steps = value;
    } else if (std::strcmp(name, "spmm_gather") == 0) {
        if (value > 2) return VS_ERROR_INVALID_VALUE;
#ifndef VS_RETIRED_VARIANTS
        if (value == 2) return VS_ERROR_NOT_SUPPORTED;  // the LDS-DMA gather: compiled only with VS_RETIRED_VARIANTS
#endif
        o.spmm_gather = value;
    } else if (std::strcmp(name, "spmm_slab_parts") == 0) {
        if (value > 64) return VS_ERROR_INVALID_VALUE;
        o.spmm_slab_parts = value;
    } else if (std::strcmp(name, "spmm_flat_piece") == 0) {
        o.spmm_flat_piece = value;
    } else if (std::strcmp(name, "spmm_flat_launches") == 0) {
        if (value > 2) return VS_ERROR_INVALID_VALUE;
        o.spmm_flat_launches = value;
    } else if (std::strcmp(name, "spmm_parts_launches") == 0) {
        if (value > 2) return VS_ERROR_INVALID_VALUE;
        o.spmm_parts_launches = value;
    } else if (std::strcmp(name, "spmm_flat_shared") == 0) {
        if (value > 2) return VS_ERROR_INVALID_VALUE;
        o.spmm_flat_shared = value;
    } else if (std::strcmp(name, "spmm_flat_waves") == 0) {
        if (value > 16) return VS_ERROR_INVALID_VALUE;
        o.spmm_flat_waves = value;
    } else if (std::strcmp(name, "sddmm_slots") == 0) {
        o.sddmm_slots = value;
    } else if (std::strcmp(name, "sddmm_flat_supers") == 0) {
        if (value > 16) return VS_ERROR_INVALID_VALUE;
        o.sddmm_flat_supers = value;
    } else if (std::strcmp(name, "sddmm_group") == 0) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return VS_ERROR_INVALID_VALUE;
        o.sddmm_group = value;
    } else if (std::strcmp(name, "sddmm_block_waves") == 0) {
        if (value > 16) return VS_ERROR_INVALID_VALUE;
        o.sddmm_block_waves = value;
    } else if (std::strcmp(name, "attention_waves") == 0) {
        if (value > 8) return VS_ERROR_INVALID_VALUE;
        o.attention_waves = value;
    } else if (std::strcmp(name, "attention_chunk") == 0) {
        o.attention_chunk = value;
    } else {
        return VS_ERROR_INVALID_VALUE;
    }
    return VS_SUCCESS;
}

int vs_set_option(const char *name, int value) { return set_option_field(vs::g_options, name, value); }

int vs_set_thread_option(const char *name, int value)
{
    if (!vs::t_options_active) {
        vs::t_options = vs::g_options;  // starts from the process-wide values as they are now
        vs::t_options_active = true;
    }
    return set_option_field(vs::t_options, name, value);
}

void vs_clear_thread_options(void) { vs::t_options_active = false; }

}  // extern "C"
#pragma GCC visibility pop
