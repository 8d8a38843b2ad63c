// Fixed-mask sparse attention for one vector row per workgroup, in ONE launch:
//     out = softmax_row(scale * (Q K^T) sampled on the mask) V
// The mask is a column-vector CSR pattern (every stored column applies to the V consecutive query rows
// of a vector row).  This is the SDDMM -> softmax -> SpMM chain of the two operator kernels with the
// scores and probabilities kept in LDS instead of HBM, organised like flash attention so that rows of
// any length fit a fixed LDS budget:
//
//   for each chunk of <= `chunk` nonzero vectors of the row (one chunk for ordinary rows):
//     A  scores: the waves split the chunk's 16-vector groups; K rows are gathered with row-major
//        128-bit loads, moved to MFMA lane order with ds_bpermute, contracted with the row's Q slices
//        on v_mfma_f32_16x16x32_f16; raw fp32 scores go to LDS as sc[v][j].
//     B  softmax statistics: wave w owns scalar rows v = w, w + W, ...: chunk maximum, new running
//        maximum m, rescale factor exp2(m_old - m) for what was accumulated so far, running sum l,
//        and p[v][j] = exp2(s*score - m) stored to LDS as fp16 in the layout the next phase reads.
//     C  context: every wave rescales its accumulators, then the waves split the chunk's 32-vector
//        steps: A operand = p from LDS, V rows gathered and transposed in registers (as in the SpMM
//        kernel), v_mfma_f32_16x16x32_f16.
//   finally the waves' partial tiles are summed through LDS in a fixed order, divided by l and stored.
#include "vs_common.hpp"

namespace vs {

// V: vector length; KS: d_qk <= 32*KS; CPL: d_v <= 16*CPL.
template <int V, int KS, int CPL>
__global__ void __launch_bounds__(512)
sparse_attention_kernel(int d_qk, int d_v, int chunk, const int *__restrict__ row_indices,
                        const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                        const half_t *__restrict__ q, const half_t *__restrict__ k,
                        const half_t *__restrict__ v, half_t *__restrict__ out, long long stride_q,
                        long long stride_k, long long stride_v, long long stride_out, float scale)
{
    q += blockIdx.y * stride_q;
    k += blockIdx.y * stride_k;
    v += blockIdx.y * stride_v;
    out += blockIdx.y * stride_out;
    constexpr int TN = 16 * CPL;
    extern __shared__ __align__(16) unsigned char smem[];
    float *sc = reinterpret_cast<float *>(smem);                         // [V][chunk] raw scores
    half_t *pr = reinterpret_cast<half_t *>(sc + (size_t)V * chunk);      // [V][chunk] exp2 values
    int *idx = reinterpret_cast<int *>(pr + (size_t)V * chunk);           // [chunk] column indices
    float *m_run = reinterpret_cast<float *>(idx + chunk);                // [V] running maximum (base 2)
    float *l_run = m_run + V;                                             // [V] running sum
    float *factor = l_run + V;                                            // [V] rescale of this chunk
    float *partial = sc;                                                  // [W][V][TN], after the last chunk

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n_waves = blockDim.x >> 6;
    const int row = row_indices[blockIdx.x];
    const int beg = row_offsets[row];
    const int end = row_offsets[row + 1];
    const int c = lane & 15;   // MFMA order: column slot / sparse row v
    const int g = lane >> 4;   //             k group
    const int r = lane >> 2;   // load order for phase A: row within a group of 16
    const int qs = lane & 3;   //                          16-byte slice within a 64-byte k step
    const int src = (4 * c + g) << 2;
    const float s2 = scale * kLog2e;
    const int col0 = c * CPL;
    const bool col_ok = col0 < d_v;
    const half_t *v_col = v + (col_ok ? col0 : 0);

    if (tid < V) {
        m_run[tid] = -__builtin_inff();
        l_run[tid] = 0.f;
    }

    // Q slices of this vector row as the MFMA A operand (rows >= V are zero)
    half8_t qa[KS];
    {
        const bool ok = r < V;
        const half_t *q_row = q + ((size_t)row * V + (ok ? r : 0)) * d_qk;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) qa[kk] = to_mfma_order(load_slice16(q_row, kk, qs, d_qk, ok), src);
    }

    float4_t acc[CPL];
#pragma unroll
    for (int cc = 0; cc < CPL; ++cc) acc[cc] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int c0 = beg; c0 < end; c0 += chunk) {
        const int len = (end - c0) < chunk ? (end - c0) : chunk;
        const int padded = (len + 31) & ~31;
        // column indices of the chunk; the padding repeats the last valid vector (in-bounds gathers, p = 0)
        for (int t = tid; t < padded; t += blockDim.x) idx[t] = col_indices[c0 + (t < len ? t : len - 1)];

        // ---- phase A: raw scores of the chunk
        for (int grp = wave; grp < padded / 16; grp += n_waves) {
            const int jl = 16 * grp + r;
            const half_t *k_row = k + (size_t)col_indices[c0 + (jl < len ? jl : len - 1)] * d_qk;
            uint4_t raw[KS];
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) raw[kk] = load_slice16(k_row, kk, qs, d_qk, true);
            float4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KS; ++kk)
                s = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[kk], to_mfma_order(raw[kk], src), s, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int vv = 4 * g + e;
                if (vv < V) sc[(size_t)vv * chunk + 16 * grp + c] = s[e];
            }
        }
        __syncthreads();

        // ---- phase B: softmax statistics and exponentials, one scalar row per wave at a time
        for (int vv = wave; vv < V; vv += n_waves) {
            const float *srow = sc + (size_t)vv * chunk;
            float mx = -__builtin_inff();
            for (int j = lane; j < len; j += 64) mx = fmaxf(mx, srow[j] * s2);
            mx = wave_max(mx);
            const float m_old = m_run[vv];
            const float m_new = fmaxf(m_old, mx);
            float sum = 0.f;
            half_t *prow = pr + (size_t)vv * chunk;
            for (int j = lane; j < padded; j += 64) {
                float p = 0.f;
                if (j < len) p = __builtin_amdgcn_exp2f(srow[j] * s2 - m_new);
                sum += p;
                prow[j] = (half_t)p;
            }
            sum = wave_sum(sum);
            if (lane == 0) {
                const float f = __builtin_amdgcn_exp2f(m_old - m_new);  // 0 on the first chunk (m_old = -inf)
                factor[vv] = f;
                l_run[vv] = l_run[vv] * f + sum;
                m_run[vv] = m_new;
            }
        }
        __syncthreads();

        // ---- phase C: accumulate p * V rows
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int vv = 4 * g + e;
            const float f = vv < V ? factor[vv] : 0.f;
#pragma unroll
            for (int cc = 0; cc < CPL; ++cc) acc[cc][e] *= f;
        }
        for (int st = wave; st < padded / 32; st += n_waves) {
            const int4_t i_lo = *reinterpret_cast<const int4_t *>(idx + 32 * st + 8 * g);
            const int4_t i_hi = *reinterpret_cast<const int4_t *>(idx + 32 * st + 8 * g + 4);
            half8_t a = {0, 0, 0, 0, 0, 0, 0, 0};
            if (c < V) a = *reinterpret_cast<const half8_t *>(pr + (size_t)c * chunk + 32 * st + 8 * g);
            RowChunk<CPL> rows[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int col = e < 4 ? i_lo[e] : i_hi[e - 4];
                rows[e].load(v_col + (size_t)col * d_v);
            }
#pragma unroll
            for (int p = 0; p < CPL / 2; ++p) {
                uint4_t even, odd;
#pragma unroll
                for (int qq = 0; qq < 4; ++qq) {
                    even[qq] = pack_lo(rows[2 * qq].dword(p), rows[2 * qq + 1].dword(p));
                    odd[qq] = pack_hi(rows[2 * qq].dword(p), rows[2 * qq + 1].dword(p));
                }
                acc[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8_t, even), acc[2 * p], 0, 0, 0);
                acc[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8_t, odd), acc[2 * p + 1], 0, 0, 0);
            }
        }
        __syncthreads();  // the next chunk (or the reduction below) overwrites sc / pr / idx
    }

    // ---- sum the waves' partial tiles in a fixed order, normalise, store
    float *mine = partial + (size_t)wave * V * TN;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int vv = 4 * g + e;
        if (vv < V) {
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                float4_t t = {acc[4 * c4][e], acc[4 * c4 + 1][e], acc[4 * c4 + 2][e], acc[4 * c4 + 3][e]};
                *reinterpret_cast<float4_t *>(mine + vv * TN + c * CPL + 4 * c4) = t;
            }
        }
    }
    __syncthreads();
    for (int item = tid; item < V * 16; item += blockDim.x) {
        const int vv = item >> 4;
        const int cs2 = item & 15;
        const int col = cs2 * CPL;
        if (col >= d_v) continue;
        float sum[CPL];
#pragma unroll
        for (int cc = 0; cc < CPL; ++cc) sum[cc] = 0.f;
        for (int w = 0; w < n_waves; ++w) {
            const float *p = partial + (size_t)w * V * TN + vv * TN + cs2 * CPL;
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                const float4_t x = *reinterpret_cast<const float4_t *>(p + 4 * c4);
                sum[4 * c4] += x[0];
                sum[4 * c4 + 1] += x[1];
                sum[4 * c4 + 2] += x[2];
                sum[4 * c4 + 3] += x[3];
            }
        }
        const float norm = end > beg ? 1.f / l_run[vv] : 0.f;  // an empty row attends to nothing: zeros
#pragma unroll
        for (int cc = 0; cc < CPL; ++cc) sum[cc] *= norm;
        store_converted<half_t, CPL>(out + ((size_t)row * V + vv) * d_v + col, sum);
    }
}

template <int V, int KS, int CPL>
static int launch_one(int m_vec, int d_qk, int d_v, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const half_t *q, const half_t *k, const half_t *v, half_t *out,
                      float scale, hipStream_t stream, const Batch &batch, long long stride_v)
{
    constexpr int TN = 16 * CPL;
    int waves = options().attention_waves > 0 ? options().attention_waves : 4;
    if (waves > 8) waves = 8;
    int chunk = options().attention_chunk > 0 ? options().attention_chunk : 512;
    chunk = (chunk + 31) & ~31;
    // the partial tiles reuse the score buffer
    while ((size_t)chunk < (size_t)waves * TN) chunk += 32;
    const size_t lds = (size_t)chunk * (V * (sizeof(float) + sizeof(half_t)) + sizeof(int)) + 3 * V * sizeof(float);
    if (lds > 150 * 1024) return hipErrorNotSupported;
    auto kernel = sparse_attention_kernel<V, KS, CPL>;
    static std::atomic<unsigned long long> lds_allowed{0};
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 150 * 1024, lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(kernel, dim3((unsigned)m_vec, (unsigned)batch.count), dim3(64 * waves), lds, stream, d_qk, d_v,
                       chunk, row_indices, row_offsets, col_indices, q, k, v, out, batch.stride_a, batch.stride_b,
                       stride_v, batch.stride_out, scale);
    return (int)hipGetLastError();
}

template <int V>
static int launch_shape(int m_vec, int d_qk, int d_v, const int *row_indices, const int *row_offsets,
                        const int *col_indices, const half_t *q, const half_t *k, const half_t *v, half_t *out,
                        float scale, hipStream_t stream, const Batch &batch, long long stride_v)
{
#define VS_ATT(KS, CPL) \
    return launch_one<V, KS, CPL>(m_vec, d_qk, d_v, row_indices, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v)
    if (d_v <= 64) {
        if (d_qk <= 32) VS_ATT(1, 4);
        if (d_qk <= 64) VS_ATT(2, 4);
        VS_ATT(4, 4);
    }
    if (d_qk <= 32) VS_ATT(1, 8);
    if (d_qk <= 64) VS_ATT(2, 8);
    VS_ATT(4, 8);
#undef VS_ATT
}

int launch_sparse_attention(int m_vec, int vec_length, int d_qk, int d_v, const int *row_indices,
                            const int *row_offsets, const int *col_indices, const half_t *q, const half_t *k,
                            const half_t *v, half_t *out, float scale, hipStream_t stream, const Batch &batch,
                            long long stride_v)
{
    if (m_vec == 0 || batch.count == 0 || d_v == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (d_qk <= 0 || d_qk % 8 != 0 || d_qk > 128) return hipErrorNotSupported;
    if (d_v % 4 != 0 || d_v > 128 || (d_v > 64 && d_v % 8 != 0)) return hipErrorNotSupported;
    switch (vec_length) {
    case 1: return launch_shape<1>(m_vec, d_qk, d_v, row_indices, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    case 2: return launch_shape<2>(m_vec, d_qk, d_v, row_indices, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    case 4: return launch_shape<4>(m_vec, d_qk, d_v, row_indices, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    case 8: return launch_shape<8>(m_vec, d_qk, d_v, row_indices, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace vs
