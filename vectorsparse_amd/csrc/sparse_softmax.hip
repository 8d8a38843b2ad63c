// Row-wise softmax over the nonzeros of a column-vector CSR matrix, in the [nnz_vec][V] value layout
// that SDDMM writes and SpMM reads (the middle step of sparse attention: SDDMM -> softmax -> SpMM).
//
//   out[j*V + v] = exp(scale*x[j*V + v] - m_v) / sum_{j' in row i} exp(scale*x[j'*V + v] - m_v),
//   m_v = max_{j' in row i} scale*x[j'*V + v],          for every nonzero vector j of vector row i.
//
// One wave per vector row: lane t owns the nonzero vectors t, t + 64, ... (one V-wide load each, the
// row's block of values is contiguous), keeps V running maxima / sums in fp32 and combines them across
// the 64 lanes with DPP / ds_swizzle / ds_bpermute butterflies.  Rows of up to 512 vectors are held in
// registers between the passes; longer rows are read twice (running maximum and sum, then the normalisation).
// in == out is allowed.
#include "vs_common.hpp"

namespace vs {

template <int V>
struct VecIO;
template <>
struct VecIO<8> {
    typedef half8_t type;
};
template <>
struct VecIO<4> {
    typedef half4_t type;
};
template <>
struct VecIO<2> {
    typedef half2_t type;
};

template <int V>
__device__ __forceinline__ void load_scaled(float (&dst)[V], const half_t *p, float scale)
{
    if constexpr (V == 1) {
        dst[0] = (float)p[0] * scale;
    } else {
        const typename VecIO<V>::type t = *reinterpret_cast<const typename VecIO<V>::type *>(p);
#pragma unroll
        for (int v = 0; v < V; ++v) dst[v] = (float)t[v] * scale;
    }
}

template <int V>
__device__ __forceinline__ void store_vec(half_t *p, const float (&src)[V])
{
    store_converted<half_t, V>(p, src);
}

constexpr int kCached = 8;  // vectors per lane kept in registers: rows of up to 64 * 8 vectors

template <int V>
__global__ void __launch_bounds__(256)
sparse_softmax_kernel(int m_vec, const int *__restrict__ row_indices, const int *__restrict__ row_offsets,
                      const half_t *in, half_t *out, float scale, long long stride_in, long long stride_out)
{
    in += blockIdx.y * stride_in;
    out += blockIdx.y * stride_out;
    const int lane = threadIdx.x & 63;
    const int slot = blockIdx.x * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform
    if (slot >= m_vec) return;
    const int row = row_indices[slot];
    const int beg = row_offsets[row];
    const int end = row_offsets[row + 1];
    const int len = end - beg;
    if (len <= 0) return;
    const float s2 = scale * kLog2e;  // work in base 2: exp(y) = exp2(y * log2 e)

    float mx[V], sum[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        mx[v] = -__builtin_inff();
        sum[v] = 0.f;
    }

    if (len <= 64 * kCached) {
        float x[kCached][V];
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = beg + lane + 64 * c;
            if (j < end) {
                load_scaled<V>(x[c], in + (size_t)j * V, s2);
#pragma unroll
                for (int v = 0; v < V; ++v) mx[v] = fmaxf(mx[v], x[c][v]);
            }
        }
#pragma unroll
        for (int v = 0; v < V; ++v) mx[v] = wave_max(mx[v]);
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = beg + lane + 64 * c;
            if (j < end) {
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    x[c][v] = __builtin_amdgcn_exp2f(x[c][v] - mx[v]);
                    sum[v] += x[c][v];
                }
            }
        }
#pragma unroll
        for (int v = 0; v < V; ++v) sum[v] = 1.0f / wave_sum(sum[v]);
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = beg + lane + 64 * c;
            if (j < end) {
                float y[V];
#pragma unroll
                for (int v = 0; v < V; ++v) y[v] = x[c][v] * sum[v];
                store_vec<V>(out + (size_t)j * V, y);
            }
        }
        return;
    }

    // Longer rows: two passes over the row, each in chunks of kCached vectors per lane whose loads are all requested
    // before the first is used - a lane that asks for one vector at a time pays a memory round trip per 64 vectors
    // of the row (a dense row of 4096 vectors: 192 of them one after the other).  The first pass keeps a running
    // maximum and a sum relative to it per lane (rescaled once per chunk when the maximum moves), combined across
    // the lanes at the end; the second normalises.  The loads are made whether or not the vector exists (past the
    // row's end a lane re-reads the row's last vector): a load behind a branch makes every wait after it count for
    // the path without it.
    constexpr int kChunk = 64 * kCached;
    const int last = end - 1;
    for (int j0 = beg + lane; j0 < end; j0 += kChunk) {
        float x[kCached][V];
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = j0 + 64 * c;
            load_scaled<V>(x[c], in + (size_t)(j < end ? j : last) * V, s2);
        }
        float top[V];
#pragma unroll
        for (int v = 0; v < V; ++v) top[v] = mx[v];
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
#pragma unroll
            for (int v = 0; v < V; ++v) top[v] = fmaxf(top[v], x[c][v]);  // (a repeated vector changes no maximum)
        }
#pragma unroll
        for (int v = 0; v < V; ++v) {
            sum[v] *= __builtin_amdgcn_exp2f(mx[v] - top[v]);  // (0 on the first chunk: its maximum was -inf)
            mx[v] = top[v];
        }
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const bool exists = j0 + 64 * c < end;
#pragma unroll
            for (int v = 0; v < V; ++v) sum[v] += exists ? __builtin_amdgcn_exp2f(x[c][v] - mx[v]) : 0.f;
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float all = wave_max(mx[v]);  // every lane has seen at least one vector of a row this long
        sum[v] = 1.0f / wave_sum(sum[v] * __builtin_amdgcn_exp2f(mx[v] - all));
        mx[v] = all;
    }
    for (int j0 = beg + lane; j0 < end; j0 += kChunk) {
        float x[kCached][V];
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = j0 + 64 * c;
            load_scaled<V>(x[c], in + (size_t)(j < end ? j : last) * V, s2);
        }
        // (in == out: every load of the chunk is in registers before its first store; the vector that lanes past
        // the row's end re-read is not used)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = j0 + 64 * c;
            if (j < end) {
                float y[V];
#pragma unroll
                for (int v = 0; v < V; ++v) y[v] = __builtin_amdgcn_exp2f(x[c][v] - mx[v]) * sum[v];
                store_vec<V>(out + (size_t)j * V, y);
            }
        }
    }
}

template <int V>
static int launch_one(int m_vec, const int *row_indices, const int *row_offsets, const half_t *in, half_t *out,
                      float scale, hipStream_t stream, const Batch &batch)
{
    constexpr int kWavesPerBlock = 4;
    const int blocks = ceil_div(m_vec, kWavesPerBlock);
    hipLaunchKernelGGL((sparse_softmax_kernel<V>), dim3((unsigned)blocks, (unsigned)batch.count),
                       dim3(64 * kWavesPerBlock), 0, stream, m_vec, row_indices, row_offsets, in, out, scale,
                       batch.stride_a, batch.stride_out);
    return (int)hipGetLastError();
}

int launch_sparse_softmax(int m_vec, int vec_length, const int *row_indices, const int *row_offsets,
                          const half_t *values_in, half_t *values_out, float scale, hipStream_t stream,
                          const Batch &batch)
{
    if (m_vec == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    switch (vec_length) {
    case 1: return launch_one<1>(m_vec, row_indices, row_offsets, values_in, values_out, scale, stream, batch);
    case 2: return launch_one<2>(m_vec, row_indices, row_offsets, values_in, values_out, scale, stream, batch);
    case 4: return launch_one<4>(m_vec, row_indices, row_offsets, values_in, values_out, scale, stream, batch);
    case 8: return launch_one<8>(m_vec, row_indices, row_offsets, values_in, values_out, scale, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace vs
