// SDDMM on fp16 MFMA for a column-vector CSR mask (replaces src/wmma_sddmm.cu of the reference).
//
// out[j*V + v] = sum_l lhs[(i*V + v)*K + l] * rhs[col_j*K + l]   for every nonzero vector j of vector row i.
//
// Both operands are contiguous along the contraction index, which is exactly the per-lane layout
// v_mfma_f32_16x16x32_f16 wants (8 consecutive k per lane), so operands go from global memory
// straight into MFMA registers with 128-bit loads; there is no LDS stage and no barrier.
// Lane = (c = lane % 16, g = lane / 16).  One wave step covers 16 nonzero vectors of a row:
//   A operand: lhs row i*V + c (zero for c >= V), k slice [32*kk + 8g, +8)
//   B operand: rhs row col_{j0 + c},               same k slice
//   D[v][c]  : lane (c, g), register e  ->  out[(j0 + c)*V + 4g + e]   (4 consecutive outputs per lane)
// A wave owns (vector row, slot s) and walks the row's 16-vector groups s, s + slots, ...; the lhs
// slices of the vector row stay in registers across groups when K <= 256.
#include "vs_common.hpp"

namespace vs {

template <int V, typename OutT>
__device__ __forceinline__ void store_group(OutT *out, int j, int g, const float4_t &acc)
{
    const float tmp[4] = {acc[0], acc[1], acc[2], acc[3]};
    if constexpr (V >= 4) {
        if (4 * g < V) store_converted<OutT, 4>(out + (size_t)j * V + 4 * g, tmp);
    } else if constexpr (V == 2) {
        if (g == 0) store_converted<OutT, 2>(out + (size_t)j * 2, tmp);
    } else {
        if (g == 0) store_converted<OutT, 1>(out + (size_t)j, tmp);
    }
}

// KS > 0: K <= 32*KS, lhs slices preloaded; KS == 0: any K % 8 == 0, lhs re-read per group.
template <int V, int KS, typename OutT>
__global__ void __launch_bounds__(256)
sddmm_mfma_kernel(int m_vec, int K, int slots, const int *__restrict__ row_indices,
                  const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                  const half_t *__restrict__ lhs, const half_t *__restrict__ rhs, OutT *__restrict__ out,
                  long long stride_lhs, long long stride_rhs, long long stride_out)
{
    lhs += blockIdx.y * stride_lhs;  // batch: shared mask, per-problem operands
    rhs += blockIdx.y * stride_rhs;
    out += blockIdx.y * stride_out;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const long long wg = (long long)blockIdx.x * (blockDim.x >> 6) + wave;
    if (wg >= (long long)m_vec * slots) return;
    const int slot = (int)(wg / slots);
    const int s = (int)(wg % slots);
    const int row = row_indices[slot];
    const int beg = row_offsets[row];
    const int end = row_offsets[row + 1];
    const int n_groups = (end - beg + 15) >> 4;
    if (s >= n_groups) return;
    const int c = lane & 15;
    const int g = lane >> 4;
    const bool a_row_ok = c < V;
    const half_t *lhs_row = lhs + ((size_t)row * V + (a_row_ok ? c : 0)) * K;
    const half8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    if constexpr (KS > 0) {
        half8_t a[KS];
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            const int off = 32 * kk + 8 * g;
            a[kk] = zero8;
            if (a_row_ok && off < K) a[kk] = *reinterpret_cast<const half8_t *>(lhs_row + off);
        }
        for (int grp = s; grp < n_groups; grp += slots) {
            const int j = beg + 16 * grp + c;
            const bool valid = j < end;
            const int jc = valid ? j : end - 1;  // in-bounds gather for the padded slots; result discarded
            const half_t *rhs_row = rhs + (size_t)col_indices[jc] * K;
            half8_t b[KS];
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                const int off = 32 * kk + 8 * g;
                b[kk] = zero8;
                if (off < K) b[kk] = *reinterpret_cast<const half8_t *>(rhs_row + off);
            }
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KS; ++kk)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[kk], b[kk], acc, 0, 0, 0);
            if (valid) store_group<V, OutT>(out, j, g, acc);
        }
    } else {
        const int k_steps = (K + 31) >> 5;
        for (int grp = s; grp < n_groups; grp += slots) {
            const int j = beg + 16 * grp + c;
            const bool valid = j < end;
            const int jc = valid ? j : end - 1;
            const half_t *rhs_row = rhs + (size_t)col_indices[jc] * K;
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
            for (int kk = 0; kk < k_steps; ++kk) {
                const int off = 32 * kk + 8 * g;
                half8_t a = zero8, b = zero8;
                if (off < K) {
                    b = *reinterpret_cast<const half8_t *>(rhs_row + off);
                    if (a_row_ok) a = *reinterpret_cast<const half8_t *>(lhs_row + off);
                }
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
            }
            if (valid) store_group<V, OutT>(out, j, g, acc);
        }
    }
}

template <int V, int KS, typename OutT>
static int launch_one(int m_vec, int k, int slots, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
    constexpr int kWavesPerBlock = 4;
    const long long waves = (long long)m_vec * slots;
    const long long blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    hipLaunchKernelGGL((sddmm_mfma_kernel<V, KS, OutT>), dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * kWavesPerBlock), 0, stream,
                       m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out,
                       batch.stride_a, batch.stride_b, batch.stride_out);
    return (int)hipGetLastError();
}

template <int V, typename OutT>
static int launch_ks(int m_vec, int k, int slots, const int *row_indices, const int *row_offsets,
                     const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
    if (k <= 32) return launch_one<V, 1, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    if (k <= 64) return launch_one<V, 2, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    if (k <= 128) return launch_one<V, 4, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    if (k <= 256) return launch_one<V, 8, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    return launch_one<V, 0, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
}

// Workgroups per vector row: enough waves to fill the chip, at most one per 16-vector group of an
// average row (longer rows loop).
int sddmm_auto_slots(int m_vec, int nonzeros_vec, int group)
{
    int slots = options().sddmm_slots;
    if (slots > 0) return slots;
    const long long avg = ((long long)nonzeros_vec + m_vec - 1) / (m_vec > 0 ? m_vec : 1);
    const int avg_groups = (int)((avg + group - 1) / group);
    const int want = ceil_div(8192, m_vec > 0 ? m_vec : 1);
    slots = avg_groups < want ? avg_groups : want;
    return slots < 1 ? 1 : slots;
}

template <typename OutT>
int launch_sddmm_mfma(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                      const int *row_offsets, const int *col_indices, const half_t *lhs,
                      const half_t *rhs, OutT *out, int vec_length, hipStream_t stream, const Batch &batch)
{
    (void)n;
    if (m_vec == 0 || nonzeros_vec == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (k <= 0 || k % 8 != 0) return hipErrorNotSupported;
    const int slots = sddmm_auto_slots(m_vec * batch.count, nonzeros_vec * batch.count, 16);
    switch (vec_length) {
    case 1: return launch_ks<1, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 2: return launch_ks<2, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 4: return launch_ks<4, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 8: return launch_ks<8, OutT>(m_vec, k, slots, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

template int launch_sddmm_mfma<half_t>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                       const half_t *, half_t *, int, hipStream_t, const Batch &);
template int launch_sddmm_mfma<float>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                      const half_t *, float *, int, hipStream_t, const Batch &);

}  // namespace vs
