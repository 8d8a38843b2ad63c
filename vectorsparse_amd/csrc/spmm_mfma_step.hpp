// One 32-vector step of the SpMM tile loop on fp16 MFMA, shared by the row-per-workgroup kernel and the
// kernel that splits the nonzero range (src/wmma_spmm.cu:77-90 of the reference is the loop this replaces).
#pragma once
#include "vs_common.hpp"

namespace vs {

constexpr int kStep = 32;  // nonzero vectors per MFMA step

// Wave-private staging slot in LDS: 32 column indices, then the 32 vectors transposed to [v][nonzero].
template <int V>
constexpr int stage_bytes()
{
    return kStep * (int)sizeof(int) + V * kStep * (int)sizeof(half_t);
}

// The V halves of one nonzero vector, fetched with one load.
template <int V>
__device__ __forceinline__ void load_vector(half_t (&dst)[V], const half_t *p)
{
    if constexpr (V == 8) {
        const half8_t t = *reinterpret_cast<const half8_t *>(p);
#pragma unroll
        for (int v = 0; v < 8; ++v) dst[v] = t[v];
    } else if constexpr (V == 4) {
        const half4_t t = *reinterpret_cast<const half4_t *>(p);
#pragma unroll
        for (int v = 0; v < 4; ++v) dst[v] = t[v];
    } else if constexpr (V == 2) {
        const half2_t t = *reinterpret_cast<const half2_t *>(p);
        dst[0] = t[0];
        dst[1] = t[1];
    } else {
        dst[0] = p[0];
    }
}

// The same vector kept as loaded (one register per two halves) until its halves are needed.
template <int V>
struct PackedVector {
    typedef half_t vec_t __attribute__((ext_vector_type(V)));
    vec_t d;
    __device__ __forceinline__ void load(const half_t *p) { d = *reinterpret_cast<const vec_t *>(p); }
    __device__ __forceinline__ void store(half_t *p) const { *reinterpret_cast<vec_t *>(p) = d; }
    __device__ __forceinline__ void clear() { d = vec_t(0); }
    __device__ __forceinline__ half_t at(int v) const { return d[v]; }
    __device__ __forceinline__ float first() const { return (float)d[0]; }
};
template <>
struct PackedVector<1> {
    half_t d;
    __device__ __forceinline__ void load(const half_t *p) { d = p[0]; }
    __device__ __forceinline__ void store(half_t *p) const { p[0] = d; }
    __device__ __forceinline__ void clear() { d = (half_t)0.f; }
    __device__ __forceinline__ half_t at(int) const { return d; }
    __device__ __forceinline__ float first() const { return (float)d; }
};

__device__ __forceinline__ void wave_lds_fence()
{
    // LDS operations of one wave execute in order; this only stops the compiler from moving
    // LDS accesses of different lanes' data across the hand-off point.
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Consumes the staged step: lane (cs = lane % 16, g = lane / 16) reads its eight column indices and its
// slice of the transposed vectors from the wave's slot, gathers CPL consecutive halves of the eight rhs rows
// at column offset `col_off` (element offset of the lane's first column inside a row), calls `prefetch()`
// with those loads in flight, transposes the CPL x 8 block with v_perm_b32 and issues CPL MFMAs:
// acc[c][e] += sum_j vec[4g + e][j] * rhs[col_j][col_off + c].
// RAGGED: the dense width is not a multiple of CPL; `valid` (0..CPL) halves of the lane's chunk exist.
// PITCH: halves between the staged vectors' rows (the slot may be laid out for a block of several steps).
template <int V, int CPL, bool IDX32, bool RAGGED = false, int PITCH = kStep, typename Prefetch>
__device__ __forceinline__ void spmm_mfma_step(const int *idx_s, const half_t *vec_s, const half_t *rhs, int n_cols,
                                               uint32_t col_off, int cs, int g, float4_t (&acc)[CPL],
                                               Prefetch &&prefetch, int valid = CPL)
{
    const int4_t i_lo = *reinterpret_cast<const int4_t *>(idx_s + 8 * g);
    const int4_t i_hi = *reinterpret_cast<const int4_t *>(idx_s + 8 * g + 4);
    half8_t a = {0, 0, 0, 0, 0, 0, 0, 0};
    if (cs < V) a = *reinterpret_cast<const half8_t *>(vec_s + cs * PITCH + 8 * g);
    wave_lds_fence();

    RowChunk<CPL> chunk[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int col = e < 4 ? i_lo[e] : i_hi[e - 4];
        if constexpr (RAGGED) {
            load_ragged<CPL>(chunk[e], rhs + ((size_t)col * n_cols + col_off), valid);
        } else if constexpr (IDX32) {
            // rhs has fewer than 2^31 elements: 32-bit offsets from a uniform base
            chunk[e].load(rhs + ((uint32_t)col * (uint32_t)n_cols + col_off));
        } else {
            chunk[e].load(rhs + ((size_t)col * n_cols + col_off));
        }
    }
    prefetch();
#pragma unroll
    for (int p = 0; p < CPL / 2; ++p) {
        uint4_t even, odd;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            even[q] = pack_lo(chunk[2 * q].dword(p), chunk[2 * q + 1].dword(p));
            odd[q] = pack_hi(chunk[2 * q].dword(p), chunk[2 * q + 1].dword(p));
        }
        const half8_t b_even = __builtin_bit_cast(half8_t, even);
        const half8_t b_odd = __builtin_bit_cast(half8_t, odd);
        acc[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_even, acc[2 * p], 0, 0, 0);
        acc[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_odd, acc[2 * p + 1], 0, 0, 0);
    }
}

// A step shared by up to 16 / V consecutive vector rows: MFMA row `cs` carries scalar row cs % V of the vector row in
// group cs / V, which owns the staged slots [lo, hi) (per lane; the other slots read as zero for that row), so the
// accumulator rows of group p add up that row's nonzeros only.  Otherwise as spmm_mfma_step.
template <int V, int CPL, bool IDX32, typename Prefetch>
__device__ __forceinline__ void spmm_mfma_step_shared(const int *idx_s, const half_t *vec_s, const half_t *rhs,
                                                      int n_cols, uint32_t col_off, int cs, int g, float4_t (&acc)[CPL],
                                                      int lo, int hi, Prefetch &&prefetch)
{
    const int4_t i_lo = *reinterpret_cast<const int4_t *>(idx_s + 8 * g);
    const int4_t i_hi = *reinterpret_cast<const int4_t *>(idx_s + 8 * g + 4);
    uint4_t a_bits = *reinterpret_cast<const uint4_t *>(vec_s + (cs % V) * kStep + 8 * g);
    wave_lds_fence();
    const uint32_t span = hi > lo ? (uint32_t)(hi - lo) : 0u;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t first = (uint32_t)(8 * g + 2 * d - lo);  // wraps to a large value below lo
        const uint32_t keep = (first < span ? 0x0000ffffu : 0u) | (first + 1u < span ? 0xffff0000u : 0u);
        a_bits[d] &= keep;
    }
    const half8_t a = __builtin_bit_cast(half8_t, a_bits);

    RowChunk<CPL> chunk[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int col = e < 4 ? i_lo[e] : i_hi[e - 4];
        if constexpr (IDX32)
            chunk[e].load(rhs + ((uint32_t)col * (uint32_t)n_cols + col_off));
        else
            chunk[e].load(rhs + ((size_t)col * n_cols + col_off));
    }
    prefetch();
#pragma unroll
    for (int p = 0; p < CPL / 2; ++p) {
        uint4_t even, odd;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            even[q] = pack_lo(chunk[2 * q].dword(p), chunk[2 * q + 1].dword(p));
            odd[q] = pack_hi(chunk[2 * q].dword(p), chunk[2 * q + 1].dword(p));
        }
        const half8_t b_even = __builtin_bit_cast(half8_t, even);
        const half8_t b_odd = __builtin_bit_cast(half8_t, odd);
        acc[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_even, acc[2 * p], 0, 0, 0);
        acc[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_odd, acc[2 * p + 1], 0, 0, 0);
    }
}

// S steps at once: the staged slot holds S * 32 column indices and the vectors as [v][S * 32]; all 8 * S row segments
// of the lane are requested before the first MFMA, so the wave pays one memory round trip for S steps (at 2 * CPL / 4
// registers per segment in flight).  Otherwise as spmm_mfma_step.
template <int V, int CPL, int S, bool IDX32, int PITCH = S * kStep, typename Prefetch>
__device__ __forceinline__ void spmm_mfma_block(const int *idx_s, const half_t *vec_s, const half_t *rhs, int n_cols,
                                                uint32_t col_off, int cs, int g, float4_t (&acc)[CPL],
                                                Prefetch &&prefetch)
{
    int4_t i_lo[S], i_hi[S];
    half8_t a[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        i_lo[s] = *reinterpret_cast<const int4_t *>(idx_s + s * kStep + 8 * g);
        i_hi[s] = *reinterpret_cast<const int4_t *>(idx_s + s * kStep + 8 * g + 4);
        a[s] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (cs < V) a[s] = *reinterpret_cast<const half8_t *>(vec_s + cs * PITCH + s * kStep + 8 * g);
    }
    wave_lds_fence();

    RowChunk<CPL> chunk[S][8];
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int col = e < 4 ? i_lo[s][e] : i_hi[s][e - 4];
            if constexpr (IDX32)
                chunk[s][e].load(rhs + ((uint32_t)col * (uint32_t)n_cols + col_off));
            else
                chunk[s][e].load(rhs + ((size_t)col * n_cols + col_off));
        }
    }
    prefetch();
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int p = 0; p < CPL / 2; ++p) {
            uint4_t even, odd;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                even[q] = pack_lo(chunk[s][2 * q].dword(p), chunk[s][2 * q + 1].dword(p));
                odd[q] = pack_hi(chunk[s][2 * q].dword(p), chunk[s][2 * q + 1].dword(p));
            }
            const half8_t b_even = __builtin_bit_cast(half8_t, even);
            const half8_t b_odd = __builtin_bit_cast(half8_t, odd);
            acc[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s], b_even, acc[2 * p], 0, 0, 0);
            acc[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s], b_odd, acc[2 * p + 1], 0, 0, 0);
        }
    }
}

// The two halves of a step for a wave that keeps steps of successive blocks in flight: what a lane reads of a
// staged step (its eight column indices and its slice of the transposed vectors), the requests for the eight row
// segments, and - later, when they have returned - the transposition and the MFMAs.
struct StagedStep {
    int4_t i_lo, i_hi;
    half8_t a;
};

template <int V, int PITCH>
__device__ __forceinline__ void read_staged_step(StagedStep &st, const int *idx_s, const half_t *vec_s, int s, int cs, int g)
{
    st.i_lo = *reinterpret_cast<const int4_t *>(idx_s + s * kStep + 8 * g);
    st.i_hi = *reinterpret_cast<const int4_t *>(idx_s + s * kStep + 8 * g + 4);
    st.a = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (cs < V) st.a = *reinterpret_cast<const half8_t *>(vec_s + cs * PITCH + s * kStep + 8 * g);
}

template <int CPL>
__device__ __forceinline__ void request_step(RowChunk<CPL> (&chunk)[8], const StagedStep &st, const half_t *rhs,
                                             int n_cols, uint32_t col_off)
{
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int col = e < 4 ? st.i_lo[e] : st.i_hi[e - 4];
        chunk[e].load(rhs + ((uint32_t)col * (uint32_t)n_cols + col_off));  // rhs has fewer than 2^31 elements
    }
}

template <int CPL>
__device__ __forceinline__ void multiply_step(const RowChunk<CPL> (&chunk)[8], const half8_t &a, float4_t (&acc)[CPL])
{
#pragma unroll
    for (int p = 0; p < CPL / 2; ++p) {
        uint4_t even, odd;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            even[q] = pack_lo(chunk[2 * q].dword(p), chunk[2 * q + 1].dword(p));
            odd[q] = pack_hi(chunk[2 * q].dword(p), chunk[2 * q + 1].dword(p));
        }
        const half8_t b_even = __builtin_bit_cast(half8_t, even);
        const half8_t b_odd = __builtin_bit_cast(half8_t, odd);
        acc[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_even, acc[2 * p], 0, 0, 0);
        acc[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b_odd, acc[2 * p + 1], 0, 0, 0);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Meeting of partial tiles across workgroups within one launch (rows in parts, split rows).
//
// The parts of a row are computed by workgroups on different CUs - and different XCDs, whose L2s are not coherent
// with each other inside a launch.  Each part leaves an fp32 tile in a workspace and counts itself in on the row's
// arrival counter; whoever brings the count to the number of parts adds all tiles in ascending order, writes the row
// and puts the counter back to zero.  Nobody waits for anybody, and the sum is the same whoever arrives last.
//
// What makes the last arriver read the other parts' data, in this order and with nothing else (an L2-wide write-back
// and invalidate - __threadfence() - round the counter costs 60 us per launch instead of 1):
//   1. store_part(): the tile is stored with the device-coherence bits of the cache policy (sc0 sc1) set: the store
//      is written through the issuing CU's vector cache and its XCD's L2 to memory;
//   2. publish(): s_waitcnt vmcnt(0) - the wave does not go on until every such store has been acknowledged by the
//      memory side, i.e. is visible to any later access that bypasses the caches.  (The workgroup-scope release fence in
//      front of it only keeps the compiler from moving the stores below this point.)  When several waves of the
//      workgroup have stored, a workgroup barrier follows, so that all of them have passed their own publish();
//   3. arrive(): one lane adds 1 to the counter with a relaxed agent-scope atomic, which is carried out at the memory
//      side (L2 atomics of one address are ordered there, whichever XCD they come from): it is issued after the
//      acknowledgements of step 2, so a workgroup that observes count == parts - 1 knows every other part's stores
//      were acknowledged before its own add was performed;
//   4. collect(): a workgroup-scope acquire fence (compiler ordering only: the loads below are issued after the
//      atomic has returned its value), then load_part() reads every tile with sc0 sc1 set: past the vector cache and
//      the L2, from the memory side that acknowledged the stores of step 2;
//   5. rearm(): the counter goes back to zero with a relaxed agent-scope store; the next launch on the stream (a kernel
//      boundary) finds it so.  Launches that overlap on one workspace race - the caller's contract.
// The workspace area is addressed through a buffer descriptor (below 2^31 bytes, offsets in bytes).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

struct PartMeeting {
    static constexpr int kCoherent = 1 | 16;  // cache policy bits: sc0, sc1

    static __device__ __forceinline__ __amdgpu_buffer_rsrc_t area(float *base)
    {
        return __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7fffffff, 0x00020000);
    }
    static __device__ __forceinline__ void store_part(__amdgpu_buffer_rsrc_t tiles, uint32_t byte_offset, const float4_t &x)
    {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, x), tiles, byte_offset, 0, kCoherent);
    }
    // (a store that the NEXT launch reads: an ordinary one, the kernel boundary makes it visible)
    static __device__ __forceinline__ void store_plain(__amdgpu_buffer_rsrc_t tiles, uint32_t byte_offset, const float4_t &x)
    {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, x), tiles, byte_offset, 0, 0);
    }
    static __device__ __forceinline__ float4_t load_part(__amdgpu_buffer_rsrc_t tiles, uint32_t byte_offset)
    {
        return __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(tiles, byte_offset, 0, kCoherent));
    }
    static __device__ __forceinline__ void publish()
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
    }
    // every lane of the wave gets the number of parts that had arrived before this one
    static __device__ __forceinline__ int arrive(int *counter, int lane)
    {
        int arrived = 0;
        if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return __builtin_amdgcn_readfirstlane(arrived);
    }
    static __device__ __forceinline__ void collect() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup"); }
    static __device__ __forceinline__ void rearm(int *counter, int lane)
    {
        if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
};

// Last index i in [0, rows] with offsets[i] <= pos (of equal offsets, i.e. empty rows, the last one): the row
// that holds nonzero `pos` when pos < offsets[rows].  64-ary search, one probe per lane and round (two dependent
// loads for up to 4095 rows); every lane of the wave must be active and gets the same answer.
__device__ __forceinline__ int find_row_of(const int *__restrict__ offsets, int rows, int pos, int lane)
{
    int lo = 0, span = rows + 1;
    do {
        const int step = (span + 63) >> 6;
        const int idx = lo + lane * step;
        const int probe = idx < lo + span ? offsets[idx] : 0x7fffffff;
        const int below = __builtin_popcountll(__builtin_amdgcn_ballot_w64(probe <= pos));  // a prefix of the lanes
        const int k = below > 0 ? below - 1 : 0;
        lo += k * step;
        span = span - k * step < step ? span - k * step : step;
    } while (span > 1);
    return lo;
}

// The same search, returning the probes of its last round as a window over the offsets: on return lane l holds
// offsets[base + l] (0x7fffffff past offsets[rows]) and the row found is base + first, so that the caller can walk
// on from there (row base + i runs from lane i to lane i + 1) without another load.
__device__ __forceinline__ int find_row_window(const int *__restrict__ offsets, int rows, int pos, int lane,
                                               int &base, int &first)
{
    int lo = 0, span = rows + 1;
    for (;;) {
        const int step = (span + 63) >> 6;
        // the last round (step 1) probes 64 consecutive offsets whatever is left of the span: the offsets are
        // ascending, so the entries past the span are greater than pos and do not change the count
        const int idx = lo + lane * step;
        const bool inside = step == 1 ? idx <= rows : idx < lo + span;
        const int probe = inside ? offsets[idx] : 0x7fffffff;
        const int below = __builtin_popcountll(__builtin_amdgcn_ballot_w64(probe <= pos));  // a prefix of the lanes
        const int k = below > 0 ? below - 1 : 0;
        if (step == 1) {
            base = lo;
            first = k;
            return probe;
        }
        lo += k * step;
        span = span - k * step < step ? span - k * step : step;
    }
}

}  // namespace vs
