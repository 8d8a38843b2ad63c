// Fine-grained SpMM on the fp16 vector ALU (replaces src/cuda_spmm.cu of the reference).
//
// A V x 1 vector times a gathered rhs row is a rank-1 update, not a dense contraction, so
// this path keeps it on the vector ALU: mixed-precision multiply-adds with fp16 operands, exact
// products and fp32 accumulation - v_fma_mix_f32 for V = 1, v_dot2_f32_f16 over pairs of
// nonzeros for V >= 2 (half the instructions per multiply-add).  The reference rounds every product to fp16
// first (src/spmm_utils/compute_utils.h:45); that rounding alone costs up to ~9e-2 of the
// 1e-2 relative-error budget against the host loop on near-zero outputs, so it is not
// reproduced.  Work item = (vector row, tile of TN = 8*LR dense columns); a wave is G = 64/LR groups
// of LR lanes, every lane owns 8 consecutive columns (one 128-bit load per gathered row, U = 8 rows in flight per
// lane, 4 for V = 8).  A wave fetches a block of up to 64 nonzeros with one coalesced load of indices and one of
// values per lane and parks them in LDS, from where its groups take U nonzeros each per turn; rows short enough
// for the workgroup's groups to take in one go, four nonzeros each, skip that hop.  The partial tiles (one per
// wave for V <= 2, whose groups are summed across the lanes first; one per group else) are summed through LDS in
// a fixed order.
#include <type_traits>

#include "vs_common.hpp"

namespace vs {

// The V halves of one nonzero vector as 32-bit words, two halves per word (V = 1: the low half of one word).
template <int V>
__device__ __forceinline__ void load_values(uint32_t (&dst)[V > 1 ? V / 2 : 1], const half_t *p)
{
    if constexpr (V == 8) {
        const uint4_t t = *reinterpret_cast<const uint4_t *>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = t[i];
    } else if constexpr (V == 4) {
        const uint2_t t = *reinterpret_cast<const uint2_t *>(p);
        dst[0] = t[0];
        dst[1] = t[1];
    } else if constexpr (V == 2) {
        dst[0] = *reinterpret_cast<const uint32_t *>(p);
    } else {
        dst[0] = *reinterpret_cast<const uint16_t *>(p);
    }
}

// Sum of x over the 64 / LR lanes of a wave that hold the same columns (lane = group * LR + column lane): a butterfly
// over the lane bits above LR; every lane ends up with the total.
template <int LR>
__device__ __forceinline__ float sum_over_groups(float x)
{
    if constexpr (LR <= 8) {
        const int xi = __builtin_bit_cast(int, x);
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, xi, 0x128, 0xF, 0xF, true));  // row_ror:8 = lane ^ 8
    }
    if constexpr (LR <= 16) x += partner<16>(x);
    if constexpr (LR <= 32) x += partner<32>(x);
    return x;
}

// RAGGED: the dense width is not a multiple of 8 (rows of the dense operand and of the output start at any 2-byte
// boundary, the last chunk of a row is cut): chunks are fetched and stored half by half.
// The second launch bound (waves per SIMD) is there for the launches of short rows: left to itself the compiler takes
// 86 (V = 1) and 102 (V = 2) registers where 60 and 72 do without a spill, and a launch of short rows - waves that live for
// one chain of round trips, three in four of them ending at once - then needs two rounds to seat its waves where one
// would do (2048 rows of 1 to 6 nonzeros, N = 256, V = 2: 3.24 against 2.95 us).
template <int V, int LR, typename OutT, bool RAGGED = false>
__global__ void __launch_bounds__(1024, RAGGED ? 4 : (V == 1 ? 8 : (V == 2 ? 7 : 4)))
spmm_valu_kernel(int n_cols, int n_tiles, int n_waves, uint32_t inv_waves, const int *__restrict__ row_indices,
                 const int *__restrict__ row_offsets, const int *__restrict__ column_indices,
                 const half_t *__restrict__ values, const half_t *__restrict__ rhs,
                 OutT *__restrict__ out, long long stride_values, long long stride_rhs, long long stride_out)
{
    if (blockIdx.y != 0) {  // batch: shared pattern, per-problem operands (the strides are not loaded for problem 0)
        values += blockIdx.y * stride_values;
        rhs += blockIdx.y * stride_rhs;
        out += blockIdx.y * stride_out;
    }
    extern __shared__ float partial[];  // [W * kTiles][V][TN] partial tiles, then the waves' staging slots
    constexpr int G = 64 / LR;
    constexpr int TN = 8 * LR;
    // Short vectors: the groups of a wave add their partial sums up across the lanes (below) and the wave leaves one
    // tile; V = 4 and 8 hold 32 and 64 accumulators per lane, for which that butterfly costs more than it saves
    // (V = 8, 64 rows x 4608: 5.3 -> 6.3 us), so every group leaves a tile of its own.
    constexpr bool kLaneSum = V <= 2;
    constexpr int kTiles = kLaneSum ? 1 : G;  // partial tiles per wave
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = blockIdx.x % n_tiles;
    const int slot = blockIdx.x / n_tiles;
    // the row's extent is requested for the identity order together with the swizzle entry, and again only if
    // the entry names another row: one dependent load less in the common case
    const int row = row_indices[slot];
    int beg = row_offsets[slot];
    int end = row_offsets[slot + 1];
    asm volatile("" : "+s"(beg), "+s"(end));  // keeps these two requests apart from the dependent ones below
    if (row != slot) {
        beg = row_offsets[row];
        end = row_offsets[row + 1];
    }
    constexpr int U = V <= 4 ? 8 : 4;  // nonzero vectors per group and turn: U gathered rows in flight per lane
    constexpr int kBlock = 64;   // nonzero vectors a wave fetches at once, at most: one column index and one vector per lane
    constexpr int kWords = V > 1 ? V / 2 : 1;
    // Wave w takes the blocks w, w + n_waves, .. of the row; inside a block group g takes the nonzeros
    // (t * G + g) * U .. + U - 1 of turn t.  A block is 64 nonzeros, or fewer (whole turns) when the row is short
    // enough for every wave to get one: a row of 115 nonzeros is eight blocks of 16 for eight waves, not two of 64.
    // Waves that have neither a block nor a share of the final sum (V * LR items, one per thread) end here: a
    // workgroup barrier waits only for the waves that still run.
    constexpr int kSumWaves = (V * LR + 63) / 64;
    constexpr int kTurn = G * U < kBlock ? G * U : kBlock;  // nonzeros of a turn (a power of two)
    // (inv_waves = 2^32 / n_waves + 1: the row's share per wave without a division, which costs a launch of
    // short rows 0.5 us; an inexact quotient only moves the block size, any size gives the same coverage)
    const int per_wave = (int)(((unsigned long long)(uint32_t)(end - beg + n_waves - 1) * inv_waves) >> 32);
    int block = (per_wave + kTurn - 1) / kTurn * kTurn;
    // (two turns a wave at least where the row has them: 512 rows of 115 nonzeros, V = 1, N = 256, eight waves launched:
    // 4.1 us with a turn each, 3.7 us with four of them taking two turns and the others ending at once)
    constexpr int kLeast = 2 * kTurn < kBlock ? 2 * kTurn : kBlock;
    block = block < kLeast ? kLeast : (block > kBlock ? kBlock : block);
    // waves with a block: all of them unless the blocks are at their smallest (a wave without one adds zeros)
    int alive_waves = block == kLeast ? (end - beg + kLeast - 1) / kLeast : n_waves;
    // A row short enough for every group of the workgroup to take its nonzeros in one go, kDirect each, does so
    // without the staging slot: one chain of two round trips (index, gathered row) on as many waves as the row has
    // groups of kDirect nonzeros.  (One wave with eight nonzeros per group instead measured 11-28 % slower over the
    // rows of 1 to 60 nonzeros of the sweep: every request of a wave, padded or not, takes the CU's address path
    // 16 cycles, and eight workgroups per CU queue there.)
    constexpr int kDirect = 4;
    const bool direct = end - beg <= n_waves * G * kDirect;
    if (direct) {
        const int groups = (end - beg + kDirect - 1) / kDirect;
        alive_waves = (groups + G - 1) / G;
    }
    alive_waves = alive_waves < kSumWaves ? kSumWaves : alive_waves;
    alive_waves = alive_waves < n_waves ? alive_waves : n_waves;
    if (wave >= alive_waves) return;
    const int cl = lane % LR;
    const int g = lane / LR;
    const int col0 = tile * TN + cl * 8;
    const bool col_ok = col0 < n_cols;  // n_cols % 8 == 0 unless RAGGED
    const half_t *rhs_col = rhs + (col_ok ? col0 : 0);
    const int valid = !col_ok ? 0 : (n_cols - col0 < 8 ? n_cols - col0 : 8);  // RAGGED: halves of the chunk that exist

    float acc[V][8];
#pragma unroll
    for (int v = 0; v < V; ++v)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[v][c] = 0.f;

    // The wave's staging slot: 64 column indices, then the 64 vectors.  Every lane fetches one nonzero of the block - two coalesced
    // requests per 64 nonzeros, the next block's under the current block's gathers - and the groups pick their
    // U nonzeros of a turn from the slot with a few LDS reads, where a request per nonzero and lane group
    // (eight for a turn of two groups, each serving two distinct addresses) kept the address path as busy with
    // indices as with gathered rows: large V = 1 problems ran at 19-21 TB/s of gather against the 24-28 TB/s of
    // the MFMA kernel, whose waves have always fetched their indices this way.
    constexpr int kSlotBytes = kBlock * (int)sizeof(int) + kBlock * V * (int)sizeof(half_t);
    // (with a tile per group the slot lies in the wave's own tiles, 2048 V bytes that are written after its last block;
    // a single tile of short vectors can be smaller than the slot, which then has room of its own behind the tiles)
    unsigned char *slot_s = kLaneSum
        ? reinterpret_cast<unsigned char *>(partial + (size_t)n_waves * V * TN) + (size_t)wave * kSlotBytes
        : reinterpret_cast<unsigned char *>(partial + (size_t)wave * G * V * TN);
    int *idx_s = reinterpret_cast<int *>(slot_s);
    uint32_t *val_s = reinterpret_cast<uint32_t *>(slot_s + kBlock * sizeof(int));  // [64][V] halves
    const int stride = n_waves * block;
    int j0 = beg + wave * block;
    int next_idx = 0;
    uint32_t next_val[kWords];
    auto fetch = [&](int from) {
        const int j = from + lane;
        const bool have = j < end && lane < block;
        const int jc = have ? j : end - 1;  // slots past the row's end repeat its last vector with zero values
        next_idx = column_indices[jc];
        load_values<V>(next_val, values + (size_t)jc * V);
        if (!have) {
#pragma unroll
            for (int i = 0; i < kWords; ++i) next_val[i] = 0u;
        }
    };
    // U nonzeros of a group: gather their rows (all U requests before the first use), multiply and add.
    auto consume = [&](auto count, const int (&col)[U], const uint32_t (&a)[U][kWords]) {
        constexpr int N = decltype(count)::value;  // nonzeros taken: the first N entries of col and a
        uint4_t b[N];
#pragma unroll
        for (int u = 0; u < N; ++u) {
            if constexpr (RAGGED) {
                RowChunk<8> chunk;
                load_ragged<8>(chunk, rhs_col + (size_t)col[u] * n_cols, valid);
                b[u] = chunk.d;
            } else {
                b[u] = *reinterpret_cast<const uint4_t *>(rhs_col + (size_t)col[u] * n_cols);
            }
        }
        if constexpr (V == 1) {
            // one multiply-add per column and nonzero: nothing to pair up
#pragma unroll
            for (int u = 0; u < N; ++u) {
                const float av = (float)__builtin_bit_cast(half2_t, a[u][0])[0];
                const half8_t bu = __builtin_bit_cast(half8_t, b[u]);
#pragma unroll
                for (int c = 0; c < 8; ++c) acc[0][c] = __builtin_fmaf(av, (float)bu[c], acc[0][c]);
            }
        } else {
            // Two nonzeros at a time on v_dot2_f32_f16 (two exact products and the accumulator summed in fp32 by
            // one instruction): the values of the two vectors and the two gathered rows are interleaved with
            // v_perm_b32 first - V + 8 shuffles buy 8 V instructions instead of 16 V.
#pragma unroll
            for (int u = 0; u < N; u += 2) {
                half2_t av[V], bv[8];
#pragma unroll
                for (int i = 0; i < V / 2; ++i) {
                    av[2 * i] = __builtin_bit_cast(half2_t, pack_lo(a[u][i], a[u + 1][i]));
                    av[2 * i + 1] = __builtin_bit_cast(half2_t, pack_hi(a[u][i], a[u + 1][i]));
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    bv[2 * i] = __builtin_bit_cast(half2_t, pack_lo(b[u][i], b[u + 1][i]));
                    bv[2 * i + 1] = __builtin_bit_cast(half2_t, pack_hi(b[u][i], b[u + 1][i]));
                }
#pragma unroll
                for (int v = 0; v < V; ++v)
#pragma unroll
                    for (int c = 0; c < 8; ++c) acc[v][c] = __builtin_amdgcn_fdot2(av[v], bv[c], acc[v][c], false);
            }
        }
    };
    // (a lambda, expanded at both of its calls: the short row's whole path then lies in one straight piece of code)
    auto finish = [&](bool one_group) __attribute__((always_inline)) {
    // The groups of a wave hold partial sums of the same V x TN tile: added up across the lanes first (a butterfly
    // of 64 / LR - 1 steps per accumulator), so that the workgroup sums one tile per wave through LDS instead of
    // one per group - with eight groups of eight lanes (the narrow tiles of small problems) that was a chain of
    // 64 tiles read by eight threads.
    if (G > 1 && kLaneSum && !one_group) {  // (a row of one group's nonzeros: the other groups hold zeros)
#pragma unroll
        for (int v = 0; v < V; ++v)
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[v][c] = sum_over_groups<LR>(acc[v][c]);
    }
    if (n_waves * kTiles == 1) {  // (deciding this by the row's length at run time instead measured 0.5 us slower)
        if (col_ok && g == 0) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                if constexpr (RAGGED)
                    store_ragged<OutT, 8>(out + ((size_t)row * V + v) * n_cols + col0, acc[v], valid);
                else
                    store_converted<OutT, 8>(out + ((size_t)row * V + v) * n_cols + col0, acc[v]);
            }
        }
        return;
    }

    // the tiles of the waves that are still running are written and summed (a wave without nonzeros writes zeros)
    if (g < kTiles) {
        float *mine = partial + (size_t)(wave * kTiles + g) * V * TN;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float4_t lo = {acc[v][0], acc[v][1], acc[v][2], acc[v][3]};
            float4_t hi = {acc[v][4], acc[v][5], acc[v][6], acc[v][7]};
            *reinterpret_cast<float4_t *>(mine + v * TN + cl * 8) = lo;
            *reinterpret_cast<float4_t *>(mine + v * TN + cl * 8 + 4) = hi;
        }
    }
    __syncthreads();
    for (int item = threadIdx.x; item < V * LR; item += 64 * alive_waves) {
        const int v = item / LR;
        const int cl2 = item % LR;
        const int col = tile * TN + cl2 * 8;
        if (col >= n_cols) continue;
        float sum[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) sum[c] = 0.f;
        for (int p = 0; p < alive_waves * kTiles; ++p) {
            const float *src = partial + (size_t)p * V * TN + v * TN + cl2 * 8;
            const float4_t x = *reinterpret_cast<const float4_t *>(src);
            const float4_t y = *reinterpret_cast<const float4_t *>(src + 4);
            sum[0] += x[0]; sum[1] += x[1]; sum[2] += x[2]; sum[3] += x[3];
            sum[4] += y[0]; sum[5] += y[1]; sum[6] += y[2]; sum[7] += y[3];
        }
        if constexpr (RAGGED)
            store_ragged<OutT, 8>(out + ((size_t)row * V + v) * n_cols + col, sum, n_cols - col);
        else
            store_converted<OutT, 8>(out + ((size_t)row * V + v) * n_cols + col, sum);
    }
    };
    // (the short row's code comes first and runs straight through: the instruction cache starts every launch cold, and
    // a jump across the staged loop's code costs a launch of short rows 0.2-0.4 us)
    if (__builtin_expect(direct, 1)) {
        const int first = beg + (wave * G + g) * kDirect;
        if (first < end) {
            int col[U];
            uint32_t a[U][kWords];
#pragma unroll
            for (int u = 0; u < kDirect; ++u) {
                const bool have = first + u < end;
                const int jc = have ? first + u : end - 1;  // padded slots repeat the last vector with zero values
                col[u] = column_indices[jc];
                load_values<V>(a[u], values + (size_t)jc * V);
                if (!have) {
#pragma unroll
                    for (int i = 0; i < kWords; ++i) a[u][i] = 0u;
                }
            }
            consume(std::integral_constant<int, kDirect>(), col, a);
        }
        finish(end - beg <= kDirect);
        return;
    }
    {
    if (j0 < end) fetch(j0);
    for (; j0 < end; j0 += stride) {
        idx_s[lane] = next_idx;
        if constexpr (V == 1) {
            reinterpret_cast<uint16_t *>(val_s)[lane] = (uint16_t)next_val[0];
        } else {
#pragma unroll
            for (int i = 0; i < kWords; ++i) val_s[lane * kWords + i] = next_val[i];
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (j0 + stride < end) fetch(j0 + stride);
        const int count = end - j0 < block ? end - j0 : block;
        const int turns = (count + kTurn - 1) / kTurn;
        for (int t = 0; t < turns; ++t) {
            const int first = (t * G + g) * U;  // the group's nonzeros of this turn: first .. first + U - 1 of the block
            if (first >= count) continue;       // (the last turn of a row: groups past its end have nothing to add)
            int col[U];
#pragma unroll
            for (int u4 = 0; u4 < U / 4; ++u4) {
                const int4_t c4 = *reinterpret_cast<const int4_t *>(idx_s + first + 4 * u4);
#pragma unroll
                for (int u = 0; u < 4; ++u) col[4 * u4 + u] = c4[u];
            }
            uint32_t a[U][kWords];  // the vectors' halves, two per word (V = 1: one half in the low bits)
            if constexpr (V == 1) {
#pragma unroll
                for (int u2 = 0; u2 < U / 2; ++u2) {
                    const uint32_t w = val_s[first / 2 + u2];  // (first is a multiple of U)
                    a[2 * u2][0] = w & 0xffffu;
                    a[2 * u2 + 1][0] = w >> 16;
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int i = 0; i < kWords; ++i) a[u][i] = val_s[(first + u) * kWords + i];
            }
            consume(std::integral_constant<int, U>(), col, a);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");  // the slot is read out before the next block lands in it
        __builtin_amdgcn_wave_barrier();
    }
    }

    finish(false);
}

template <int V, int LR, typename OutT, bool RAGGED = false>
static int launch_one(int m_vec, int k, int waves, const int *row_indices, const int *row_offsets,
                      const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                      hipStream_t stream, const Batch &batch)
{
    constexpr int G = 64 / LR;
    constexpr int TN = 8 * LR;
    const int n_tiles = ceil_div(k, TN);
    const long long blocks = (long long)m_vec * n_tiles;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    // LDS per wave: one partial tile of V x TN floats and the staging slot (64 indices, 64 vectors) for V <= 2, a tile
    // per group (the slot lies inside them) for V = 4 and 8; within 64 KiB.
    constexpr int kPerWave = V <= 2 ? V * TN * (int)sizeof(float) + 64 * (int)sizeof(int) + 64 * V * (int)sizeof(half_t)
                                    : G * V * TN * (int)sizeof(float);
    const int max_waves = (64 * 1024) / kPerWave;
    if (waves > max_waves) waves = max_waves;
    if (waves < 1) waves = 1;
    const size_t lds = (size_t)waves * kPerWave;
    hipLaunchKernelGGL((spmm_valu_kernel<V, LR, OutT, RAGGED>), dim3((unsigned)blocks, (unsigned)batch.count),
                       dim3(64 * waves), lds, stream, k, n_tiles, waves, (uint32_t)((1ull << 32) / (unsigned)waves + 1u), row_indices, row_offsets, column_indices, values,
                       rhs, out, batch.stride_a, batch.stride_b, batch.stride_out);
    return (int)hipGetLastError();
}

// Lanes per column tile: as wide as the dense matrix allows (one group covers a whole row of it), narrower
// while that leaves the chip without a workgroup per CU - narrow tiles put more groups on every nonzero range.
static int valu_tile_lanes(int m_vec, int k, int batch)
{
    int lr = k <= 64 ? 8 : (k <= 128 ? 16 : (k <= 256 ? 32 : 64));
    while (lr > 8 && (long long)m_vec * ceil_div(k, 8 * lr) * batch < 256) lr >>= 1;
    return lr;
}

template <int V, typename OutT>
static int launch_lr(int m_vec, int k, int waves, const int *row_indices, const int *row_offsets,
                     const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                     hipStream_t stream, const Batch &batch)
{
    if (k % 8 != 0)  // any dense width: the half-by-half variant, 16 lanes (128 columns) per tile
        return launch_one<V, 16, OutT, true>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    const int lr = valu_tile_lanes(m_vec, k, batch.count);
    if (lr == 8) return launch_one<V, 8, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    if (lr == 16) return launch_one<V, 16, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    if (lr == 32) return launch_one<V, 32, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    return launch_one<V, 64, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
}

template <typename OutT>
int launch_spmm_valu(int m_vec, int vec_length, int k, int n, const int *row_indices,
                     const int *row_offsets, const int *column_indices, const half_t *values,
                     const half_t *rhs, OutT *out, hipStream_t stream, const Batch &batch)
{
    if (m_vec == 0 || k == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    int waves = options().spmm_waves;
    if (waves <= 0) {
        const int lr = valu_tile_lanes(m_vec, k, batch.count);
        const long long blocks = (long long)m_vec * ceil_div(k, 8 * lr) * batch.count;
        waves = 2;
        while (waves < 8 && blocks * waves < 8192) waves <<= 1;
        // A wave is worth launching per 24 x groups / V nonzeros of a row (48 at V = 1 and 32 lanes per tile): measured over
        // M = 128 .. 2048, K = 64 .. 4608, 50 .. 98 % at N = 256, rows of up to 30 nonzeros of one or two rows' height are
        // 8-24 % faster on one wave than on the four to eight the grid alone would give them, rows of 58 to 128 are best
        // on two to four, and vectors of eight need about eight times the waves per nonzero.  The row length is the
        // mean where it is known (batched entry points), else a quarter of n.
        const int groups = 64 / lr;
        const long long row_estimate = batch.nonzeros_vec >= 0 ? ceil_div(batch.nonzeros_vec, m_vec) : n / 4;
        const long long want = ceil_div((int)((row_estimate * vec_length < 1 ? 1 : row_estimate * vec_length)), 24 * groups);
        int by_rows = 1;
        while (by_rows < want && by_rows < 16) by_rows <<= 1;
        if (waves > by_rows) waves = by_rows;
    }
    if (waves > 16) waves = 16;
    switch (vec_length) {
    case 1: return launch_lr<1, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    case 2: return launch_lr<2, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    case 4: return launch_lr<4, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    case 8: return launch_lr<8, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

template int launch_spmm_valu<half_t>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                      const half_t *, half_t *, hipStream_t, const Batch &);
template int launch_spmm_valu<float>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                     const half_t *, float *, hipStream_t, const Batch &);

}  // namespace vs
