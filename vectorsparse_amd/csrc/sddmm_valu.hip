// Fine-grained SDDMM with per-lane slices of the contraction and a cross-lane reduction
// (replaces src/cuda_sddmm.cu of the reference).
//
// A wave is G = 64/LK groups of LK lanes; a group owns one nonzero vector j per step and lane
// cl of the group owns the slice k in [chunk*LK*VEC + cl*VEC, +VEC) of both operand rows
// (VEC = 8 halves: one 128-bit load; VEC = 1 for K % 8 != 0).  Each lane forms the V partial dot
// products of its slice with v_dot2_f32_f16 (packed fp16 pairs, exact products, fp32 sum; the
// reference rounds each product to fp16 first, src/cuda_sddmm.cu:382, which by itself exceeds the
// 1e-2 relative-error budget against the host loop on near-zero outputs and is not reproduced),
// then the LK lanes of a group combine them with a reduce-scatter butterfly: at every stage a lane keeps half of its values and adds the
// partner's copy of that half, so after log2(V) stages each output sits in exactly one lane.
// Partners are reached with DPP (quad_perm, row_half_mirror, row_mirror) inside a 16-lane row,
// ds_swizzle across rows and ds_bpermute across the two 32-lane halves.
#include <type_traits>

#include "vs_common.hpp"

namespace vs {

// One butterfly stage over `vals[0..NV)`.  Returns through vals[0..max(NV/2,1)).
template <int STRIDE, int NV>
__device__ __forceinline__ void reduce_stage(float *vals, int cl)
{
    if constexpr (NV > 1) {
        const bool upper = (cl & STRIDE) != 0;
#pragma unroll
        for (int i = 0; i < NV / 2; ++i) {
            const float send = upper ? vals[i] : vals[i + NV / 2];
            const float keep = upper ? vals[i + NV / 2] : vals[i];
            vals[i] = keep + partner<STRIDE>(send);
        }
    } else {
        vals[0] += partner<STRIDE>(vals[0]);
    }
}

template <int LK, int NV>
__device__ __forceinline__ void reduce_group(float *vals, int cl)
{
    if constexpr (LK > 1) {
        reduce_stage<LK / 2, NV>(vals, cl);
        reduce_group<LK / 2, (NV > 1 ? NV / 2 : 1)>(vals, cl);
    }
}

template <int VEC>
__device__ __forceinline__ void load_slice(half_t (&dst)[VEC], const half_t *p, bool ok)
{
    if constexpr (VEC == 8) {
        half8_t t = {0, 0, 0, 0, 0, 0, 0, 0};
        if (ok) t = *reinterpret_cast<const half8_t *>(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) dst[i] = t[i];
    } else {
        dst[0] = ok ? p[0] : (half_t)0.f;
    }
}

template <int V, int VEC>
__device__ __forceinline__ void slice_dot(float (&acc)[V], const half_t (&a)[V][VEC], const half_t (&b)[VEC])
{
#pragma unroll
    for (int v = 0; v < V; ++v) {
        if constexpr (VEC == 8) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const half2_t aa = {a[v][2 * i], a[v][2 * i + 1]};
                const half2_t bb = {b[2 * i], b[2 * i + 1]};
                acc[v] = __builtin_amdgcn_fdot2(aa, bb, acc[v], false);  // v_dot2_f32_f16
            }
        } else {
            acc[v] = __builtin_fmaf((float)a[v][0], (float)b[0], acc[v]);
        }
    }
}

// SINGLE: the whole of K fits one chunk (K <= LK*VEC) and the lhs slices stay in registers.
template <int V, int LK, int VEC, bool SINGLE, typename OutT>
__global__ void __launch_bounds__(256)
sddmm_valu_kernel(int m_vec, int K, int slots, int waves_per_block, const int *__restrict__ row_indices,
                  const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                  const half_t *__restrict__ lhs, const half_t *__restrict__ rhs, OutT *__restrict__ out,
                  long long stride_lhs, long long stride_rhs, long long stride_out)
{
    if (blockIdx.y != 0) {  // batch: shared mask, per-problem operands (the strides are not loaded for problem 0)
        lhs += blockIdx.y * stride_lhs;
        rhs += blockIdx.y * stride_rhs;
        out += blockIdx.y * stride_out;
    }
    constexpr int G = 64 / LK;
    constexpr int CHUNK = LK * VEC;
    const int lane = threadIdx.x & 63;
    // wave-uniform 32-bit arithmetic (the launcher keeps m_vec * slots below 2^32): a 64-bit division per lane
    // here cost 0.15 us per launch
    // (the waves per workgroup come as an argument, which sits in scalar registers when the wave starts: the
    // workgroup size would be a load from the hidden arguments)
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned wg = blockIdx.x * (unsigned)waves_per_block + wave;
    if (wg >= (unsigned)m_vec * (unsigned)slots) return;
    const int slot = (int)(wg / (unsigned)slots);
    const int s = (int)(wg % (unsigned)slots);
    // the row's extent is requested for the identity order together with the swizzle entry, and again only if
    // the entry names another row
    const int row = row_indices[slot];
    int beg = row_offsets[slot];
    int end = row_offsets[slot + 1];
    asm volatile("" : "+s"(beg), "+s"(end));  // keeps these two requests apart from the dependent ones below
    if (row != slot) {
        beg = row_offsets[row];
        end = row_offsets[row + 1];
    }
    const int n_groups = (end - beg + G - 1) / G;
    if (s >= n_groups) return;
    const int cl = lane % LK;
    const int g = lane / LK;
    const half_t *lhs_rows = lhs + (size_t)row * V * K;
    const int n_chunks = SINGLE ? 1 : (K + CHUNK - 1) / CHUNK;

    half_t a0[V][VEC];
    if constexpr (SINGLE) {
        const int off = cl * VEC;
#pragma unroll
        for (int v = 0; v < V; ++v) load_slice<VEC>(a0[v], lhs_rows + (size_t)v * K + off, off < K);
    }

    // Every lane of the wave runs the same number of steps so the cross-lane exchanges below
    // always see all partners; padded slots gather the row's last vector and skip the store.
    // A wave takes the groups s, s + slots, ... of its row, U of them per turn while it has that many left: their
    // column indices are requested together and then their rhs rows, so that U gathered rows are in flight per lane
    // instead of one; what is left goes one group per turn (no padded requests: each would take the CU's address
    // path as long as a real one).
    constexpr int U = SINGLE ? (V <= 2 ? 4 : 2) : 1;
    auto turn = [&](auto count, int grp) {
        constexpr int N = decltype(count)::value;
        int j[N];
        bool valid[N];
        const half_t *rhs_row[N];
#pragma unroll
        for (int u = 0; u < N; ++u) {
            j[u] = beg + (grp + u * slots) * G + g;
            valid[u] = j[u] < end;
            const int jc = valid[u] ? j[u] : end - 1;
            rhs_row[u] = rhs + (size_t)col_indices[jc] * K;
        }
        float acc[N][V];
#pragma unroll
        for (int u = 0; u < N; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) acc[u][v] = 0.f;
        if constexpr (SINGLE) {
            const int off = cl * VEC;
            half_t b[N][VEC];
#pragma unroll
            for (int u = 0; u < N; ++u) load_slice<VEC>(b[u], rhs_row[u] + off, off < K);
#pragma unroll
            for (int u = 0; u < N; ++u) slice_dot<V, VEC>(acc[u], a0, b[u]);
        } else {
            for (int ch = 0; ch < n_chunks; ++ch) {
                const int off = ch * CHUNK + cl * VEC;
                const bool ok = off < K;
                half_t a[V][VEC];
                half_t b[VEC];
#pragma unroll
                for (int v = 0; v < V; ++v) load_slice<VEC>(a[v], lhs_rows + (size_t)v * K + off, ok);
                load_slice<VEC>(b, rhs_row[0] + off, ok);
                slice_dot<V, VEC>(acc[0], a, b);
            }
        }
#pragma unroll
        for (int u = 0; u < N; ++u) {
            reduce_group<LK, V>(acc[u], cl);
            // After the butterfly: V >= LK -> lane cl holds outputs v = cl*(V/LK) + i, i < V/LK;
            //                      V <  LK -> lanes with cl % (LK/V) == 0 hold output v = cl / (LK/V).
            if (valid[u]) {
                if constexpr (V >= LK) {
                    constexpr int PER = V / LK;
                    store_converted<OutT, PER>(out + (size_t)j[u] * V + cl * PER, acc[u]);
                } else {
                    constexpr int REP = LK / V;
                    if (cl % REP == 0) store_converted<OutT, 1>(out + (size_t)j[u] * V + cl / REP, acc[u]);
                }
            }
        }
    };
    int grp = s;
    if constexpr (U > 1) {
        for (; grp + (U - 1) * slots < n_groups; grp += U * slots) turn(std::integral_constant<int, U>(), grp);
    }
    for (; grp < n_groups; grp += slots) turn(std::integral_constant<int, 1>(), grp);
}

template <int V, int LK, int VEC, bool SINGLE, typename OutT>
static int launch_one(int m_vec, int k, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
    constexpr int kWavesPerBlock = 4;
    const int slots = sddmm_auto_slots((long long)m_vec * batch.count, (long long)nonzeros_vec * batch.count, 64 / LK, false);
    const long long waves = (long long)m_vec * slots;
    const long long blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL || blocks * kWavesPerBlock > 0xffffffffLL) return hipErrorNotSupported;
    hipLaunchKernelGGL((sddmm_valu_kernel<V, LK, VEC, SINGLE, OutT>), dim3((unsigned)blocks, (unsigned)batch.count),
                       dim3(64 * kWavesPerBlock), 0, stream, m_vec, k, slots, kWavesPerBlock, row_indices, row_offsets,
                       col_indices, lhs, rhs, out,
                       batch.stride_a, batch.stride_b, batch.stride_out);
    return (int)hipGetLastError();
}

template <int V, typename OutT>
static int launch_shape(int m_vec, int k, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                        const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
#define VS_GO(LK, VEC, SINGLE) \
    return launch_one<V, LK, VEC, SINGLE, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch)
    if (k % 8 == 0) {
        if (k <= 32) VS_GO(4, 8, true);
        if (k <= 64) VS_GO(8, 8, true);
        if (k <= 128) VS_GO(16, 8, true);
        if (k <= 256) VS_GO(32, 8, true);
        if (k <= 512) VS_GO(64, 8, true);
        VS_GO(64, 8, false);
    }
    if (k <= 16) VS_GO(16, 1, true);
    VS_GO(64, 1, false);
#undef VS_GO
}

template <typename OutT>
int launch_sddmm_valu(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                      const int *row_offsets, const int *col_indices, const half_t *lhs,
                      const half_t *rhs, OutT *out, int vec_length, hipStream_t stream, const Batch &batch)
{
    (void)n;
    if (m_vec == 0 || nonzeros_vec == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (k <= 0) return hipErrorNotSupported;
    switch (vec_length) {
    case 1: return launch_shape<1, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 2: return launch_shape<2, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 4: return launch_shape<4, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 8: return launch_shape<8, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

template int launch_sddmm_valu<half_t>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                       const half_t *, half_t *, int, hipStream_t, const Batch &);
template int launch_sddmm_valu<float>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                      const half_t *, float *, int, hipStream_t, const Batch &);

}  // namespace vs
