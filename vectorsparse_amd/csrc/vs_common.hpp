// Shared device/host helpers for the gfx950 SpMM / SDDMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace vs {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef int32_t int4_t __attribute__((ext_vector_type(4)));
// 4-byte aligned vector views: row starts inside the CSR arrays are only int-aligned.
typedef int32_t int4_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kWave = 64;

// v_perm_b32 selectors: pick the low (high) halves of two dwords, first operand in the low half.
constexpr uint32_t kPermLoLo = 0x05040100u;
constexpr uint32_t kPermHiHi = 0x07060302u;

__device__ __forceinline__ uint32_t pack_lo(uint32_t first, uint32_t second)
{
    return __builtin_amdgcn_perm(second, first, kPermLoLo);
}
__device__ __forceinline__ uint32_t pack_hi(uint32_t first, uint32_t second)
{
    return __builtin_amdgcn_perm(second, first, kPermHiHi);
}

template <typename T>
__device__ __forceinline__ T bit_cast_u32x2(uint32_t a, uint32_t b)
{
    uint2_t u = {a, b};
    return __builtin_bit_cast(T, u);
}

// Value held by the lane's partner in the opposite half of an aligned block of 2*STRIDE lanes.
template <int STRIDE>
__device__ __forceinline__ float partner(float x)
{
    const int xi = __builtin_bit_cast(int, x);
    int r;
    if constexpr (STRIDE == 1) {
        r = __builtin_amdgcn_update_dpp(0, xi, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    } else if constexpr (STRIDE == 2) {
        r = __builtin_amdgcn_update_dpp(0, xi, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    } else if constexpr (STRIDE == 4) {
        r = __builtin_amdgcn_update_dpp(0, xi, 0x141, 0xF, 0xF, true);  // row_half_mirror: i <-> 7 - i
    } else if constexpr (STRIDE == 8) {
        r = __builtin_amdgcn_update_dpp(0, xi, 0x140, 0xF, 0xF, true);  // row_mirror: i <-> 15 - i
    } else if constexpr (STRIDE == 16) {
        r = __builtin_amdgcn_ds_swizzle(xi, 0x401F);                    // bit mode, xor 16
    } else {
        const int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        r = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, xi);
    }
    return __builtin_bit_cast(float, r);
}


// CPL consecutive halves of one gathered row, fetched with one load (CPL = 8: 128 bits, 4: 64 bits).
template <int CPL>
struct RowChunk;
template <>
struct RowChunk<8> {
    uint4_t d;
    __device__ __forceinline__ void load(const half_t *p) { d = *reinterpret_cast<const uint4_t *>(p); }
    __device__ __forceinline__ uint32_t dword(int i) const { return d[i]; }
};
template <>
struct RowChunk<4> {
    uint2_t d;
    __device__ __forceinline__ void load(const half_t *p) { d = *reinterpret_cast<const uint2_t *>(p); }
    __device__ __forceinline__ uint32_t dword(int i) const { return d[i]; }
};

// The same chunk when the dense width is not a multiple of the chunk: rows then start at any 2-byte boundary and
// the last chunk of a row is cut, so the halves are fetched one by one and those at or past `valid` read as zero.
template <int CPL>
__device__ __forceinline__ void load_ragged(RowChunk<CPL> &chunk, const half_t *p, int valid)
{
    const uint16_t *h = reinterpret_cast<const uint16_t *>(p);
#pragma unroll
    for (int i = 0; i < CPL / 2; ++i) {
        const uint32_t lo = 2 * i < valid ? h[2 * i] : 0u;
        const uint32_t hi = 2 * i + 1 < valid ? h[2 * i + 1] : 0u;
        chunk.d[i] = lo | (hi << 16);
    }
}

// Row-major lane order -> MFMA lane order for a 16-row x 64-byte block: lane (c = lane % 16, g = lane / 16)
// takes the four registers of lane 4c + g (`src_lane_bytes` = (4c + g) * 4) through the LDS crossbar.
__device__ __forceinline__ half8_t to_mfma_order(const uint4_t &x, int src_lane_bytes)
{
    uint4_t y;
#pragma unroll
    for (int i = 0; i < 4; ++i) y[i] = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane_bytes, (int)x[i]);
    return __builtin_bit_cast(half8_t, y);
}

// Slice q (8 halves at k = 32*kk + 8q) of `row`, zero past K or when !ok.  Branch-free: a slice that
// does not exist is read at offset 0 (always valid) and replaced by zeros, so the load can be
// scheduled with its neighbours instead of sitting in its own exec-masked block.
__device__ __forceinline__ uint4_t load_slice16(const half_t *row, int kk, int q, int K, bool ok)
{
    const int off = 32 * kk + 8 * q;
    const bool take = ok && off < K;
    const uint4_t x = *reinterpret_cast<const uint4_t *>(row + (take ? off : 0));
    const uint4_t zero = {0u, 0u, 0u, 0u};
    return take ? x : zero;
}

// All-lane max / sum over the 64 lanes of a wave (every lane must be active).
__device__ __forceinline__ float wave_max(float x)
{
    x = fmaxf(x, partner<1>(x));
    x = fmaxf(x, partner<2>(x));
    x = fmaxf(x, partner<4>(x));
    x = fmaxf(x, partner<8>(x));
    x = fmaxf(x, partner<16>(x));
    x = fmaxf(x, partner<32>(x));
    return x;
}

__device__ __forceinline__ float wave_sum(float x)
{
    x += partner<1>(x);
    x += partner<2>(x);
    x += partner<4>(x);
    x += partner<8>(x);
    x += partner<16>(x);
    x += partner<32>(x);
    return x;
}

constexpr float kLog2e = 1.4426950408889634f;
// Store `Count` consecutive outputs converted from fp32 (Count in {1,2,4,8}).
template <typename OutT, int Count>
__device__ __forceinline__ void store_converted(OutT *dst, const float *src);

template <>
__device__ __forceinline__ void store_converted<half_t, 8>(half_t *dst, const float *src)
{
    half8_t h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (half_t)src[i];
    *reinterpret_cast<half8_t *>(dst) = h;
}
template <>
__device__ __forceinline__ void store_converted<half_t, 4>(half_t *dst, const float *src)
{
    half4_t h;
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = (half_t)src[i];
    *reinterpret_cast<half4_t *>(dst) = h;
}
template <>
__device__ __forceinline__ void store_converted<half_t, 2>(half_t *dst, const float *src)
{
    half2_t h = {(half_t)src[0], (half_t)src[1]};
    *reinterpret_cast<half2_t *>(dst) = h;
}
template <>
__device__ __forceinline__ void store_converted<half_t, 1>(half_t *dst, const float *src)
{
    *dst = (half_t)src[0];
}
template <>
__device__ __forceinline__ void store_converted<float, 8>(float *dst, const float *src)
{
    float4_t a = {src[0], src[1], src[2], src[3]};
    float4_t b = {src[4], src[5], src[6], src[7]};
    reinterpret_cast<float4_t *>(dst)[0] = a;
    reinterpret_cast<float4_t *>(dst)[1] = b;
}
template <>
__device__ __forceinline__ void store_converted<float, 4>(float *dst, const float *src)
{
    float4_t a = {src[0], src[1], src[2], src[3]};
    *reinterpret_cast<float4_t *>(dst) = a;
}
template <>
__device__ __forceinline__ void store_converted<float, 2>(float *dst, const float *src)
{
    dst[0] = src[0];
    dst[1] = src[1];
}
template <>
__device__ __forceinline__ void store_converted<float, 1>(float *dst, const float *src)
{
    dst[0] = src[0];
}

// The first `valid` of Count consecutive outputs, converted and stored one by one (no alignment assumed).
template <typename OutT, int Count>
__device__ __forceinline__ void store_ragged(OutT *dst, const float *src, int valid)
{
#pragma unroll
    for (int i = 0; i < Count; ++i)
        if (i < valid) dst[i] = (OutT)src[i];
}

// Launch-shape overrides (0 = automatic).
struct Options {
    int spmm_waves = 0;
    int spmm_cols_per_lane = 0;
    int spmm_steps = 0;         // MFMA SpMM: 32-vector steps a wave keeps in flight (1, 2, 4), 0 = automatic
    int spmm_teams = 0;         // MFMA SpMM with the long-row count known: 1 = every row gets a team of waves, 2 = only the long rows do, 0 = automatic
    int spmm_pipe = 0;          // MFMA SpMM, two steps in flight: 2 = waves pipeline successive blocks, 1 = never, 0 = automatic
    int spmm_blocks_per_wave = 0;  // ... blocks of a row a wave takes before another of the kept waves joins in (power of two), 0 = automatic
    int spmm_guard_waves = 0;   // MFMA SpMM, row lengths unknown, full grid: waves per workgroup kept for rows longer than expected
    int spmm_gather = 0;        // 1 = gathered rows through registers, 2 = through LDS-DMA loads, 0 = automatic
    int spmm_slab_parts = 0;    // SpMM with the dense operand staged in LDS (vs_wmma_spmm_f16_slab): parts of the contraction a block of rows is spread over (1..64), 0 = automatic
    int spmm_flat_piece = 0;    // split-row SpMM: nonzero vectors per wave (rounded up to 32), 0 = automatic
    int spmm_flat_launches = 0; // split-row SpMM: 1 = parts added inside the launch, 2 = by a second launch, 0 = automatic
    int spmm_flat_waves = 0;    // split-row SpMM: waves per workgroup, 0 = automatic
    int spmm_parts_launches = 0;  // rows in parts: 1 = the parts of a split row meet inside the launch, 2 = a second launch adds them, 0 = automatic
    int spmm_flat_shared = 0;   // split-row SpMM: 1 = every row segment starts its own step, 2 = rows share steps, 0 = automatic
    int sddmm_slots = 0;
    int sddmm_block_waves = 0;
    int sddmm_group = 0;        // MFMA SDDMM: 16-vector groups per wave step (1, 2, 4), 0 = automatic
    int sddmm_flat_supers = 0;  // flat MFMA SDDMM (algorithm 2): super-groups per wave, 0 = automatic
    int attention_waves = 0;
    int attention_chunk = 0;
};
const Options &options();  // the calling thread's overrides if it has set any, else the process-wide ones

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Raise a kernel's dynamic LDS limit above the 64 KB default.  The attribute belongs to the current device, so
// it is set once per (kernel, device): `done` is the call site's own mask of the devices already served.
inline hipError_t allow_large_lds(const void *kernel, int bytes, std::atomic<unsigned long long> &done)
{
    int device = 0;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) return status;
    const unsigned long long bit = 1ull << (device & 63);
    if (device < 64 && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
    status = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (status == hipSuccess && device < 64) done.fetch_or(bit, std::memory_order_release);
    return status;
}

// Waves per vector row for the SDDMM kernels; `group` = nonzero vectors a wave covers per step.
int sddmm_auto_slots(long long m_vec, long long nonzeros_vec, int group, bool mfma);  // rows and nonzero vectors of the whole batch

// Batched launches: problem b of `count` uses operand pointers advanced by b * stride (in elements);
// the sparsity pattern (row_indices, row_offsets, column indices) is shared by the whole batch.
struct Batch {
    int count = 1;
    long long stride_a = 0;    // SpMM: values        SDDMM: lhs_matrix
    long long stride_b = 0;    // SpMM: rhs_matrix    SDDMM: rhs_matrix
    long long stride_out = 0;  // SpMM: output_matrix SDDMM: output_values
    int nonzeros_vec = -1;     // SpMM: nonzero vectors of the pattern when the caller knows them (launch-shape hint)
    int longest_row_vec = -1;  // SpMM: nonzero vectors of the longest row when the caller knows them (same)
    int long_rows = -1;        // SpMM, rows ordered by length: leading entries of row_indices with more than 512 vectors
    int algorithm = 0;         // SDDMM on MFMA: 2 = waves split the nonzero range, else (row, slot) per wave
    bool row_parts = false;    // SDDMM on MFMA: row_indices is a dispatch list of row parts, m_vec counts its slots
};

// Launch shape of the MFMA SpMM (spmm_mfma.hip), chosen on the host.
struct SpmmShape {
    int cols_per_lane = 4;     // dense columns per lane: tiles of 16 x this many columns, 64- or 128-bit row segments
    int steps_in_flight = 1;   // 32-vector steps whose gathered rows a wave requests before its first MFMA (1, 2, 4)
    int waves = 1;             // waves per workgroup
    int blocks_per_wave = 1;   // blocks of a row a wave takes before another wave of the workgroup joins in
    int team_slots = -1;       // >= 0: only that many leading entries of row_indices get the workgroup as a team
    bool pipelined = false;    // waves keep steps of successive blocks of a row in flight (two-step blocks only)
    bool ragged = false;       // dense width not a multiple of 4: the half-by-half variant
    bool dma = false;          // the variant that gathers through LDS-DMA loads (option spmm_gather = 2)
};
SpmmShape choose_spmm_shape(bool softmax, int m_vec, int vec_length, int k, int n, const Batch &batch);

// Launchers (one per kernel family); return a hipError_t-valued int.
template <typename OutT>
int launch_spmm_mfma(int m_vec, int vec_length, int k, int n, const int *row_indices,
                     const int *row_offsets, const int *column_indices, const half_t *values,
                     const half_t *rhs, OutT *out, hipStream_t stream, const Batch &batch = Batch());
template <typename OutT>
int launch_spmm_mfma_dma(int m_vec, int vec_length, int k, int n, int waves, const int *row_indices,
                         const int *row_offsets, const int *column_indices, const half_t *values, const half_t *rhs,
                         OutT *out, hipStream_t stream, const Batch &batch);
template <typename OutT>
int launch_spmm_valu(int m_vec, int vec_length, int k, int n, const int *row_indices,
                     const int *row_offsets, const int *column_indices, const half_t *values,
                     const half_t *rhs, OutT *out, hipStream_t stream, const Batch &batch = Batch());
template <typename OutT>
int launch_sddmm_mfma(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                      const int *row_offsets, const int *col_indices, const half_t *lhs,
                      const half_t *rhs, OutT *out, int vec_length, hipStream_t stream,
                      const Batch &batch = Batch());
template <typename OutT>
int launch_sddmm_valu(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                      const int *row_offsets, const int *col_indices, const half_t *lhs,
                      const half_t *rhs, OutT *out, int vec_length, hipStream_t stream,
                      const Batch &batch = Batch());

// Writes `bytes` zero bytes to each of `batch` buffers `stride_bytes` apart (a kernel, not a memset node, so that
// callers may capture the call into a HIP graph).
int launch_zero_fill(void *out, long long bytes, long long stride_bytes, int batch, hipStream_t stream);

// Workspaces of fp32 partial tiles with arrival counters in front (split-row SpMM, rows in parts).  The counters'
// area depends on the size of the workspace alone, not on the problem: a caller may use one workspace for
// problems of different shapes, every call leaves the counters it has used at zero, and no call may find another
// shape's tiles where it looks for its counters.  A counter takes 4 bytes and stands for at least 512 bytes of
// partial tiles (two tiles of 64 floats for V = 1), so 1/128 of the workspace holds the counters of whatever
// fits the rest.
inline long long partial_tile_counter_bytes(long long workspace_bytes)
{
    return (workspace_bytes / 128 + 255) / 256 * 256;
}
// Workspace that holds `tile_bytes` of partial tiles and the counters' area that goes with its size.
inline long long partial_tile_workspace_for(long long tile_bytes)
{
    return tile_bytes + (tile_bytes / 127 + 255) / 256 * 256 + 512;
}

// Rows in parts keep every arrival counter in a cache line of its own: counters that share a line queue up
// behind each other at the memory side, where device-scope atomics are carried out.  A counter then takes 128
// bytes and stands for at least 512 bytes of partial tiles, so a fifth of the workspace holds the counters of
// whatever fits the rest.
constexpr int kPartCounterStride = 32;  // ints
inline long long row_parts_counter_bytes(long long workspace_bytes)
{
    return (workspace_bytes / 5 + 255) / 256 * 256;
}
inline long long row_parts_workspace_for(long long tile_bytes)
{
    return tile_bytes + (tile_bytes / 4 + 255) / 256 * 256 + 512;
}

// Rows in parts (csrc/spmm_mfma.hip, the kernel's PARTS variant): `slots` = the dispatch list of
// vs_spmm_row_parts in device memory, four ints per workgroup slot.
int launch_spmm_mfma_row_parts(int vec_length, int k, int n, int n_slots, const int *slots, int n_split, int parts_max,
                               int nonzeros_vec, int longest_part_vec, const int *column_indices, const half_t *values,
                               const half_t *rhs, half_t *out, void *workspace, long long workspace_bytes,
                               hipStream_t stream, const Batch &batch);
long long spmm_row_parts_workspace_bytes(int batch, int vec_length, int k, int n_split, int parts_max);

// SpMM with the dense operand staged in LDS once per block of sixteen vector rows (csrc/spmm_mfma_slab.hip):
// k % 8 == 0, n * k < 2^31, fp16 output; `workspace` holds the fp32 tiles of the parts.
int launch_spmm_mfma_slab(int m_vec, int vec_length, int k, int n, int ksplit, const int *row_indices,
                          const int *row_offsets, const int *column_indices, const half_t *values, const half_t *rhs,
                          half_t *out, void *workspace, long long workspace_bytes, hipStream_t stream);
long long spmm_slab_workspace_bytes(int m_vec, int vec_length, int k, int ksplit);
int choose_spmm_slab_parts(int m_vec, int k, int n);

// Split-row SpMM (csrc/spmm_mfma_flat.hip): `workspace` holds the fp32 partial tiles of rows longer than a piece.
template <typename OutT>
int launch_spmm_mfma_flat(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_offsets,
                          const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                          float *workspace, long long workspace_bytes, hipStream_t stream);
long long spmm_flat_workspace_bytes(int vec_length, int k, int nonzeros_vec);
// The same schedule with the workspace in a library-owned static device array (no allocation anywhere).
int launch_spmm_mfma_flat_static(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_offsets,
                                 const int *column_indices, const half_t *values, const half_t *rhs, half_t *out,
                                 hipStream_t stream);
long long spmm_flat_scratch_bytes();
int spmm_flat_scratch_reset(hipStream_t stream);

int launch_spmm_softmax_mfma(int m_vec, int vec_length, int k, int n, const int *row_indices,
                             const int *row_offsets, const int *column_indices, const half_t *scores,
                             const half_t *rhs, half_t *out, float scale, hipStream_t stream,
                             const Batch &batch = Batch());
int launch_sparse_attention(int m_vec, int vec_length, int d_qk, int d_v, const int *row_indices,
                            const int *row_offsets, const int *col_indices, const half_t *q, const half_t *k,
                            const half_t *v, half_t *out, float scale, hipStream_t stream, const Batch &batch,
                            long long stride_v);
int launch_sparse_attention_union(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows, const int *row_offsets,
                                  const int *col_indices, const int *plan, const half_t *q, const half_t *k,
                                  const half_t *v, half_t *out, float scale, hipStream_t stream, const Batch &batch,
                                  long long stride_v);
long long sparse_attention_plan_bytes(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows);
int launch_sparse_attention_plan(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows, const int *row_offsets,
                                 const int *col_indices, int *plan, long long plan_bytes, hipStream_t stream);
int sparse_attention_union_capacity(int vec_length, int n, int d_qk, int d_v, int rows, bool with_plan, int *rows_used);
int launch_sparse_softmax(int m_vec, int vec_length, const int *row_indices, const int *row_offsets,
                          const half_t *values_in, half_t *values_out, float scale, hipStream_t stream,
                          const Batch &batch = Batch());
// The softmax driven by a dispatch list of row parts: `workspace` takes a (maximum, sum) pair per part and scalar row.
int launch_sparse_softmax_row_parts(int vec_length, int n_slots, const int *slots, int n_split, int parts_max,
                                    const half_t *values_in, half_t *values_out, float scale, void *workspace,
                                    long long workspace_bytes, hipStream_t stream, const Batch &batch);
long long sparse_softmax_row_parts_workspace_bytes(int batch, int vec_length, int n_split, int parts_max);

}  // namespace vs
