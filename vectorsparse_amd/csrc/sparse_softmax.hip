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

// The softmax of the nonzero vectors [beg, end) of one vector row, by one wave (s2 = scale * log2 e).
template <int V>
__device__ __forceinline__ void softmax_row(const half_t *in, half_t *out, int beg, int end, float s2, int lane)
{
    const int len = end - beg;
    if (len <= 0) return;

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
    softmax_row<V>(in, out, row_offsets[row], row_offsets[row + 1], scale * kLog2e, lane);  // base 2: exp(y) = exp2(y log2 e)
}

// Rows in parts (the dispatch list of vs_spmm_row_parts: four ints per slot, {vector row, first nonzero, end, part
// info}): a slot that is a whole row is done by its wave as above; the parts of a split row each leave their maximum
// and their sum relative to it ([problem][split row][part][v] pairs of floats), and a second launch combines a row's
// pairs in ascending order of the parts - the same numbers in every part's wave - and normalises the part.  A row of
// thousands of vectors so takes as many waves as it has parts instead of one.
template <int V>
__global__ void __launch_bounds__(256)
sparse_softmax_parts_kernel(int n_slots, const int *__restrict__ slots, int n_split, int parts_max, const half_t *in,
                            half_t *out, float scale, long long stride_in, long long stride_out, float2_t *stats,
                            int second)
{
    in += blockIdx.y * stride_in;
    out += blockIdx.y * stride_out;
    const int lane = threadIdx.x & 63;
    const int slot = blockIdx.x * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform
    if (slot >= n_slots) return;
    const int4_t d = reinterpret_cast<const int4_t *>(slots)[slot];
    const int beg = d[1], end = d[2], info = d[3];
    const float s2 = scale * kLog2e;
    if (info == 0) {
        if (!second) softmax_row<V>(in, out, beg, end, s2, lane);
        return;
    }
    float2_t *mine = stats + ((size_t)(blockIdx.y * n_split + (info >> 16)) * parts_max) * V;  // [part][v]
    const int last = end - 1;
    constexpr int kChunk = 64 * kCached;
    if (!second) {
        float mx[V], sum[V];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            mx[v] = -__builtin_inff();
            sum[v] = 0.f;
        }
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
                for (int v = 0; v < V; ++v) top[v] = fmaxf(top[v], x[c][v]);
            }
#pragma unroll
            for (int v = 0; v < V; ++v) {
                // (a lane's first chunk: nothing summed yet - and no exp2 of -inf minus -inf when the part gives
                // the lane no vector at all)
                sum[v] = mx[v] == -__builtin_inff() ? 0.f : sum[v] * __builtin_amdgcn_exp2f(mx[v] - top[v]);
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
            const float all = wave_max(mx[v]);  // finite: a part holds at least one vector
            const float rel = mx[v] == -__builtin_inff() ? 0.f : sum[v] * __builtin_amdgcn_exp2f(mx[v] - all);
            const float total = wave_sum(rel);
            if (lane == 0) mine[((info >> 8) & 255) * V + v] = float2_t{all, total};
        }
        return;
    }
    // The row's pairs, one per lane and turn (pair i belongs to scalar row i % V, and 64 % V == 0, so a lane only
    // meets pairs of scalar row lane % V), then one maximum and one sum per scalar row across the wave: every
    // part's wave computes the same two numbers, with one round trip to memory instead of one per pair.
    const int count = info & 255;
    float m_lane = -__builtin_inff(), t_lane = 0.f;
    for (int i = lane; i < count * V; i += 64) {
        const float2_t e = mine[i];
        const float top = fmaxf(m_lane, e[0]);
        t_lane = (m_lane == top ? t_lane : t_lane * __builtin_amdgcn_exp2f(m_lane - top)) +
                 (e[0] == top ? e[1] : e[1] * __builtin_amdgcn_exp2f(e[0] - top));  // (no exp2 of -inf minus -inf)
        m_lane = top;
    }
    float mx[V], inv[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const bool mine_v = (lane & (V - 1)) == v;
        const float all = wave_max(mine_v ? m_lane : -__builtin_inff());  // finite: lane v holds part 0's pair
        const float rel = mine_v && m_lane != -__builtin_inff() ? t_lane * __builtin_amdgcn_exp2f(m_lane - all) : 0.f;
        mx[v] = all;
        inv[v] = 1.0f / wave_sum(rel);
    }
    for (int j0 = beg + lane; j0 < end; j0 += kChunk) {
        float x[kCached][V];
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = j0 + 64 * c;
            load_scaled<V>(x[c], in + (size_t)(j < end ? j : last) * V, s2);
        }
        asm volatile("" ::: "memory");  // (in == out: the chunk is in registers before its first store)
#pragma unroll
        for (int c = 0; c < kCached; ++c) {
            const int j = j0 + 64 * c;
            if (j < end) {
                float y[V];
#pragma unroll
                for (int v = 0; v < V; ++v) y[v] = __builtin_amdgcn_exp2f(x[c][v] - mx[v]) * inv[v];
                store_vec<V>(out + (size_t)j * V, y);
            }
        }
    }
}

template <int V>
static int launch_parts(int n_slots, const int *slots, int n_split, int parts_max, const half_t *in, half_t *out,
                        float scale, hipStream_t stream, const Batch &batch, float2_t *stats)
{
    constexpr int kWavesPerBlock = 4;
    const int blocks = ceil_div(n_slots, kWavesPerBlock);
    for (int second = 0; second < (n_split > 0 ? 2 : 1); ++second) {
        hipLaunchKernelGGL((sparse_softmax_parts_kernel<V>), dim3((unsigned)blocks, (unsigned)batch.count),
                           dim3(64 * kWavesPerBlock), 0, stream, n_slots, slots, n_split, parts_max, in, out, scale,
                           batch.stride_a, batch.stride_out, stats, second);
        const hipError_t st = hipGetLastError();
        if (st != hipSuccess) return (int)st;
    }
    return hipSuccess;
}

long long sparse_softmax_row_parts_workspace_bytes(int batch, int vec_length, int n_split, int parts_max)
{
    if (batch <= 0 || n_split <= 0 || parts_max <= 0) return 0;
    return (long long)batch * n_split * parts_max * vec_length * (long long)sizeof(float2_t);
}

int launch_sparse_softmax_row_parts(int vec_length, int n_slots, const int *slots, int n_split, int parts_max,
                                    const half_t *values_in, half_t *values_out, float scale, void *workspace,
                                    long long workspace_bytes, hipStream_t stream, const Batch &batch)
{
    if (n_slots == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535 || n_split > 32767 || parts_max > 255) return hipErrorNotSupported;
    if (sparse_softmax_row_parts_workspace_bytes(batch.count, vec_length, n_split, parts_max) > workspace_bytes)
        return hipErrorNotSupported;
    float2_t *stats = static_cast<float2_t *>(workspace);
    switch (vec_length) {
    case 1: return launch_parts<1>(n_slots, slots, n_split, parts_max, values_in, values_out, scale, stream, batch, stats);
    case 2: return launch_parts<2>(n_slots, slots, n_split, parts_max, values_in, values_out, scale, stream, batch, stats);
    case 4: return launch_parts<4>(n_slots, slots, n_split, parts_max, values_in, values_out, scale, stream, batch, stats);
    case 8: return launch_parts<8>(n_slots, slots, n_split, parts_max, values_in, values_out, scale, stream, batch, stats);
    default: return hipErrorInvalidValue;
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
