// SDDMM on fp16 MFMA for a column-vector CSR mask (replaces src/wmma_sddmm.cu of the reference).
//
// out[j*V + v] = sum_l lhs[(i*V + v)*K + l] * rhs[col_j*K + l]   for every nonzero vector j of vector row i.
//
// Both operands are contiguous along the contraction index, which is the per-lane layout
// v_mfma_f32_16x16x32_f16 wants (8 consecutive k per lane).  One wave step covers 16 nonzero vectors:
//   A operand: lhs row i*V + c (zero for c >= V), k slice [32*kk + 8g, +8)        lane = (c = lane % 16,
//   B operand: rhs row col_{j0 + c},               same k slice                           g = lane / 16)
//   D[v][c]  : lane (c, g), register e  ->  out[(j0 + c)*V + 4g + e]   (4 consecutive outputs per lane)
// Loading in that layout would make the four lanes of every quad touch four different rows (four cache
// lines for 64 bytes), which caps the gather at a quarter of the L1 rate.  So the 128-bit loads are issued
// in the row-major lane order instead - lane n reads slice n % 4 of row n / 4, a quad reads 64 contiguous
// bytes - and the registers are moved to the MFMA lane order with ds_bpermute (LDS crossbar only, no LDS
// storage, no barrier).  A wave owns (vector row, slot s) and walks super-groups of GRP*16 vectors
// s, s + slots, ... with all GRP*KS loads of a super-group in flight together; the lhs slices of the
// vector row stay in registers across super-groups when K <= 256.
#include <type_traits>

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

// KS > 0: K <= 32*KS, lhs slices preloaded; KS == 0: any K % 8 == 0, lhs re-read per super-group.
// PARTS: `row_indices` is a dispatch list of row parts (vs_spmm_row_parts: four ints per slot, {vector row, first
// nonzero, end, part info}; row_offsets is not read, m_vec counts the slots): rows far longer than the rest are
// served as several slots, each by its own waves.  The outputs of a part are the part's nonzeros - nothing to add up.
template <int V, int KS, int GRP, typename OutT, bool PARTS = false>
__global__ void __launch_bounds__(1024)
sddmm_mfma_kernel(int m_vec, int K, int slots, int waves_per_block, const int *__restrict__ row_indices,
                  const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                  const half_t *__restrict__ lhs, const half_t *__restrict__ rhs, OutT *__restrict__ out,
                  long long stride_lhs, long long stride_rhs, long long stride_out)
{
    if (blockIdx.y != 0) {  // batch: shared mask, per-problem operands (the strides are not loaded for problem 0)
        lhs += blockIdx.y * stride_lhs;
        rhs += blockIdx.y * stride_rhs;
        out += blockIdx.y * stride_out;
    }
    constexpr int SUPER = 16 * GRP;
    const int lane = threadIdx.x & 63;
    // (row slot, slot within the row) from the wave's number in the launch: wave-uniform 32-bit arithmetic (the
    // launcher keeps m_vec * slots below 2^32).  The waves per workgroup come as an argument, which sits in
    // scalar registers when the wave starts: the workgroup size would be a load from the hidden arguments, in
    // front of everything else.
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned wg = blockIdx.x * (unsigned)waves_per_block + wave;
    if (wg >= (unsigned)m_vec * (unsigned)slots) return;
    const int slot = (int)(wg / (unsigned)slots);
    const int s = (int)(wg % (unsigned)slots);
    // the row's extent is requested for the identity order together with the swizzle entry, and again only if
    // the entry names another row: one dependent load less in the common case
    int row, beg, end;
    if constexpr (PARTS) {
        const int4_t d = reinterpret_cast<const int4_t *>(row_indices)[slot];  // one request for everything
        row = d[0];
        beg = d[1];
        end = d[2];
    } else {
        row = row_indices[slot];
        beg = row_offsets[slot];
        end = row_offsets[slot + 1];
        asm volatile("" : "+s"(beg), "+s"(end));  // keeps these two requests apart from the dependent ones below
        if (row != slot) {
            beg = row_offsets[row];
            end = row_offsets[row + 1];
        }
    }
    const int n_super = (end - beg + SUPER - 1) / SUPER;
    if (s >= n_super) return;
    const int c = lane & 15;        // MFMA order: column (nonzero vector) index
    const int g = lane >> 4;        //             k group
    const int r = lane >> 2;        // load order: row within the group of 16
    const int q = lane & 3;         //             16-byte slice within a 64-byte k step
    const int src = (4 * c + g) << 2;
    const bool a_row_ok = r < V;
    const half_t *lhs_row = lhs + ((size_t)row * V + (a_row_ok ? r : 0)) * K;

    if constexpr (KS > 0) {
        half8_t a[KS];
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) a[kk] = to_mfma_order(load_slice16(lhs_row, kk, q, K, a_row_ok), src);
        // the column indices of the next super-group are fetched while this one's rows are in flight
        int col[GRP];
        auto fetch = [&](int sg) {
#pragma unroll
            for (int u = 0; u < GRP; ++u) {
                const int jl = beg + SUPER * sg + 16 * u + r;
                // slots past the row's end gather its last vector (in bounds); their results are dropped
                col[u] = col_indices[jl < end ? jl : end - 1];
            }
        };
        fetch(s);
        for (int sg = s; sg < n_super; sg += slots) {
            const int j0 = beg + SUPER * sg;
            uint4_t raw[GRP][KS];
#pragma unroll
            for (int u = 0; u < GRP; ++u) {
                const half_t *rhs_row = rhs + (size_t)col[u] * K;
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) raw[u][kk] = load_slice16(rhs_row, kk, q, K, true);
            }
            if (sg + slots < n_super) fetch(sg + slots);
#pragma unroll
            for (int u = 0; u < GRP; ++u) {
                float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < KS; ++kk)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[kk], to_mfma_order(raw[u][kk], src), acc, 0, 0, 0);
                const int j = j0 + 16 * u + c;
                if (j < end) store_group<V, OutT>(out, j, g, acc);
            }
        }
    } else {
        const int k_steps = (K + 31) >> 5;
        for (int sg = s; sg < n_super; sg += slots) {
            const int j0 = beg + SUPER * sg;
            const half_t *rhs_row[GRP];
            float4_t acc[GRP];
#pragma unroll
            for (int u = 0; u < GRP; ++u) {
                const int jl = j0 + 16 * u + r;
                rhs_row[u] = rhs + (size_t)col_indices[jl < end ? jl : end - 1] * K;
                acc[u] = float4_t{0.f, 0.f, 0.f, 0.f};
            }
            for (int kk = 0; kk < k_steps; ++kk) {
                const half8_t a = to_mfma_order(load_slice16(lhs_row, kk, q, K, a_row_ok), src);
                uint4_t raw[GRP];
#pragma unroll
                for (int u = 0; u < GRP; ++u) raw[u] = load_slice16(rhs_row[u], kk, q, K, true);
#pragma unroll
                for (int u = 0; u < GRP; ++u)
                    acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, to_mfma_order(raw[u], src), acc[u], 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < GRP; ++u) {
                const int j = j0 + 16 * u + c;
                if (j < end) store_group<V, OutT>(out, j, g, acc[u]);
            }
        }
    }
}

// Flat variant (K <= 256): the waves split the NONZERO range instead of the rows.  Wave w owns `supers`
// consecutive super-groups of 16*GRP nonzero vectors of the CSR arrays, whatever rows they belong to, so
// every wave has the same amount of work however skewed the row lengths are, none is launched idle, and
// the row swizzle is not needed.  The wave requests the column indices and rhs rows of its first
// super-group at once (they do not depend on the rows), finds the row of its first nonzero meanwhile with a
// 64-ary search over row_offsets (one probe per lane and round: two dependent loads for up to 4095 vector
// rows), then walks the row segments inside each super-group: the lhs slices are fetched when the row
// changes and stay in registers while it lasts, one MFMA pass over the touched 16-vector groups per
// segment.  The arithmetic of an output is the same as in the row-slot kernel (same operands, same MFMA
// order): same bits.
constexpr int kFlatWaves = 8;  // waves per workgroup of the flat kernel

template <int V, int KS, int GRP, typename OutT>
__global__ void __launch_bounds__(64 * kFlatWaves)
sddmm_mfma_flat_kernel(int m_vec, int K, int nonzeros_vec, int supers, const int *__restrict__ row_offsets,
                       const int *__restrict__ col_indices, const half_t *__restrict__ lhs,
                       const half_t *__restrict__ rhs, OutT *__restrict__ out, long long stride_lhs,
                       long long stride_rhs, long long stride_out)
{
    if (blockIdx.y != 0) {
        lhs += blockIdx.y * stride_lhs;
        rhs += blockIdx.y * stride_rhs;
        out += blockIdx.y * stride_out;
    }
    constexpr int SUPER = 16 * GRP;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long long first = ((long long)blockIdx.x * kFlatWaves + wave) * supers * SUPER;
    if (first >= nonzeros_vec) return;
    const int range_begin = (int)first;
    const int range_end = first + (long long)supers * SUPER < nonzeros_vec ? range_begin + supers * SUPER : nonzeros_vec;
    const int c = lane & 15;        // MFMA order: column (nonzero vector) index
    const int g = lane >> 4;        //             k group
    const int r = lane >> 2;        // load order: row within the group of 16
    const int q = lane & 3;         //             16-byte slice within a 64-byte k step
    const int src = (4 * c + g) << 2;
    const bool a_row_ok = r < V;

    // column indices of a super-group, one group of 16 per register; slots past the range's end repeat its
    // last vector (in bounds), their results are dropped
    int col[GRP];
    auto fetch_cols = [&](int j0) {
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
            const int jl = j0 + 16 * u + r;
            col[u] = col_indices[jl < range_end ? jl : range_end - 1];
        }
    };
    fetch_cols(range_begin);

    // The last row index i in [0, m_vec] with row_offsets[i] <= range_begin (skips empty rows that start
    // there).  The final round probes consecutive offsets, which are also the row ends the walk below needs:
    // they are shifted into place (lane l: end of row base_row + l) instead of being loaded again.
    int lo = 0, span = m_vec + 1;
    int probe = 0, k = 0, step = 1;
    do {
        step = (span + 63) >> 6;
        const int idx = lo + lane * step;
        probe = idx < lo + span ? row_offsets[idx] : 0x7fffffff;
        const int below = __builtin_popcountll(__builtin_amdgcn_ballot_w64(probe <= range_begin));  // a prefix of the lanes
        k = below > 0 ? below - 1 : 0;
        lo += k * step;
        span = span - k * step < step ? span - k * step : step;
    } while (span > 1);
    int base_row = lo;
    if (base_row >= m_vec) return;  // nonzeros_vec exceeds row_offsets[m_vec]: nothing of the pattern is here
    int ends;  // lane l: end of row base_row + l (row_offsets[base_row + 1 + l], clamped to the last offset)
    if (step == 1) {
        // probe of lane l is row_offsets[base_row - k + l] (0x7fffffff past the array): take lane l + k + 1
        const int shifted = __builtin_amdgcn_ds_bpermute(((lane + k + 1) & 63) << 2, probe);
        const bool have = lane + k + 1 < 64 && shifted != 0x7fffffff;
        ends = have ? shifted : row_offsets[base_row + 1 + lane <= m_vec ? base_row + 1 + lane : m_vec];
    } else {
        ends = row_offsets[base_row + 1 + lane <= m_vec ? base_row + 1 + lane : m_vec];
    }
    int ri = 0;        // row base_row + ri is the candidate for the next nonzero
    int cur_row = -1;  // row whose lhs slices are in `a`
    half8_t a[KS];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) a[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};

    for (int j0 = range_begin; j0 < range_end; j0 += SUPER) {
        const int jend = j0 + SUPER < range_end ? j0 + SUPER : range_end;
        uint4_t raw[GRP][KS];
#pragma unroll
        for (int u = 0; u < GRP; ++u) {
            const half_t *rhs_row = rhs + (size_t)col[u] * K;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) raw[u][kk] = load_slice16(rhs_row, kk, q, K, true);
        }
        if (j0 + SUPER < range_end) fetch_cols(j0 + SUPER);  // under the rhs rows in flight
        int j = j0;
        while (j < jend) {
            if (ri == 64) {
                base_row += 64;
                ri = 0;
                if (base_row >= m_vec) return;
                ends = row_offsets[base_row + 1 + lane <= m_vec ? base_row + 1 + lane : m_vec];
            }
            const int row = base_row + ri;
            if (row >= m_vec) return;
            const int row_end = __builtin_amdgcn_readlane(ends, ri);
            if (row_end <= j) {  // the row ended (or is empty): next one
                ++ri;
                continue;
            }
            const int seg_end = row_end < jend ? row_end : jend;
            if (row != cur_row) {
                const half_t *lhs_row = lhs + ((size_t)row * V + (a_row_ok ? r : 0)) * K;
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) a[kk] = to_mfma_order(load_slice16(lhs_row, kk, q, K, a_row_ok), src);
                cur_row = row;
            }
#pragma unroll
            for (int u = 0; u < GRP; ++u) {
                const int g0 = j0 + 16 * u;
                if (g0 < seg_end && g0 + 16 > j) {  // the group holds nonzeros of this row segment
                    float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kk = 0; kk < KS; ++kk)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[kk], to_mfma_order(raw[u][kk], src), acc, 0, 0, 0);
                    const int jj = g0 + c;
                    if (jj >= j && jj < seg_end) store_group<V, OutT>(out, jj, g, acc);
                }
            }
            j = seg_end;
        }
    }
}

template <int V, int KS, int GRP, typename OutT>
static int launch_one(int m_vec, int k, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
    if constexpr (KS > 0) {
        if (batch.algorithm == 2 && !batch.row_parts) {
            // super-groups per wave: enough waves to fill the chip (~8192), at least `min_supers` of them per
            // wave so that the lhs slices and the row search are amortised, at most 16
            const long long n_supers = ((long long)nonzeros_vec + 16 * GRP - 1) / (16 * GRP);
            long long supers = (n_supers * batch.count + 8191) / 8192;
            const int min_supers = options().sddmm_flat_supers > 0 ? options().sddmm_flat_supers : (KS >= 8 ? 4 : (KS >= 4 ? 2 : 1));
            if (supers < min_supers) supers = min_supers;
            if (supers > 16) supers = 16;
            const long long flat_waves = (n_supers + supers - 1) / supers;
            const long long flat_blocks = (flat_waves + kFlatWaves - 1) / kFlatWaves;
            if (flat_blocks > 0x7fffffffLL) return hipErrorNotSupported;
            hipLaunchKernelGGL((sddmm_mfma_flat_kernel<V, KS, GRP, OutT>), dim3((unsigned)flat_blocks, (unsigned)batch.count),
                               dim3(64 * kFlatWaves), 0, stream, m_vec, k, nonzeros_vec, (int)supers, row_offsets, col_indices, lhs, rhs,
                               out, batch.stride_a, batch.stride_b, batch.stride_out);
            return (int)hipGetLastError();
        }
    }
    const int slots = sddmm_auto_slots((long long)m_vec * batch.count, (long long)nonzeros_vec * batch.count, 16 * GRP, true);
    const long long waves = (long long)m_vec * slots;
    // Waves per workgroup: eight on launches that fill the chip, fewer on smaller ones so that the launch still has two
    // workgroups per CU - a wave's lhs slices and rhs rows then do not queue behind seven other waves' on one CU's
    // address path while other CUs idle.  Measured (V = 8, K = 256, 512 / 1024 / 2048 rows at 98 %): 3.46 -> 2.38,
    // 3.59 -> 2.41, 3.69 -> 2.69 us with one wave per workgroup; K = 128, 512 rows at 90 %: 2.57 -> 2.20 us; launches of 4096
    // waves and more are the same or up to 8 % slower with narrow workgroups and keep eight.
    int kWavesPerBlock = options().sddmm_block_waves;
    if (kWavesPerBlock <= 0) {
        kWavesPerBlock = 1;
        while (kWavesPerBlock < 8 && waves * batch.count >= 512LL * 2 * kWavesPerBlock) kWavesPerBlock <<= 1;
    }
    const long long blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 0x7fffffffLL || blocks * kWavesPerBlock > 0xffffffffLL) return hipErrorNotSupported;
    if (batch.row_parts) {  // m_vec counts the slots of the dispatch list that row_indices points to
        if constexpr (std::is_same<OutT, half_t>::value) {
            hipLaunchKernelGGL((sddmm_mfma_kernel<V, KS, GRP, OutT, true>), dim3((unsigned)blocks, (unsigned)batch.count),
                               dim3(64 * kWavesPerBlock), 0, stream, m_vec, k, slots, kWavesPerBlock, row_indices, row_offsets,
                               col_indices, lhs, rhs, out, batch.stride_a, batch.stride_b, batch.stride_out);
            return (int)hipGetLastError();
        } else {
            return hipErrorNotSupported;
        }
    }
    hipLaunchKernelGGL((sddmm_mfma_kernel<V, KS, GRP, OutT>), dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * kWavesPerBlock), 0, stream,
                       m_vec, k, slots, kWavesPerBlock, row_indices, row_offsets, col_indices, lhs, rhs, out,
                       batch.stride_a, batch.stride_b, batch.stride_out);
    return (int)hipGetLastError();
}

// Vectors per wave step (16 * GRP): as many as the registers allow for the contraction length while the mask is
// large enough to fill the chip with such waves, fewer on small masks so that the launch has about 4096 working
// waves (a wave's time is one chain of dependent loads whatever its step holds, so on a small mask more, lighter
// waves finish sooner).
static int sddmm_group(int k, long long nonzeros_vec)
{
    const int forced = options().sddmm_group;
    int grp = k <= 64 ? 4 : (k <= 128 ? 2 : 1);
    if (forced == 1 || forced == 2 || forced == 4) return forced < grp ? forced : grp;
    while (grp > 1 && nonzeros_vec / (16 * grp) < 4096) grp >>= 1;
    return grp;
}

template <int V, int KS, typename OutT>
static int launch_grp(int grp, int m_vec, int k, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                      const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
    if constexpr (KS <= 2) {
        if (grp == 4) return launch_one<V, KS, 4, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    }
    if constexpr (KS <= 4) {
        if (grp >= 2) return launch_one<V, KS, 2, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    }
    return launch_one<V, KS, 1, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
}

template <int V, typename OutT>
static int launch_ks(int m_vec, int k, int nonzeros_vec, const int *row_indices, const int *row_offsets,
                     const int *col_indices, const half_t *lhs, const half_t *rhs, OutT *out, hipStream_t stream,
                      const Batch &batch)
{
    const int grp = sddmm_group(k, (long long)nonzeros_vec * batch.count);
    if (k <= 32) return launch_grp<V, 1, OutT>(grp, m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    if (k <= 64) return launch_grp<V, 2, OutT>(grp, m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    if (k <= 128) return launch_grp<V, 4, OutT>(grp, m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    if (k <= 256) return launch_one<V, 8, 1, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    return launch_one<V, 0, 4, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
}

// Waves per vector row.  Waves are independent (no reduction).  A wave that finds no super-group of its own exits
// after two scalar loads; what it costs is its share of a workgroup dispatch, which is why workgroups are eight
// waves wide.  Rows with more super-groups than waves loop.
// MFMA kernel: one wave per super-group of an average row, capped so that the launch has about 2048 to 4096 waves
// (eight per row up to 512 rows; measured on masks of 512 to 4096 rows and columns, K = 64 and 128, 70 to 95 %
// sparse: within 5 % of the best choice, where the rule below was 10 to 30 % off because half of its waves found
// nothing to do).
// Fine-grained kernel: twice as many as an average row has super-groups, so that a row twice the average still
// gets one super-group per wave, capped near the number of wave slots of the chip (it gains from up to 32 waves
// per row on the denser masks: 2048 x 2048 at 70 %, K = 128, 9.1 us against 12.1 us with eight).
int sddmm_auto_slots(long long m_vec, long long nonzeros_vec, int group, bool mfma)
{
    int slots = options().sddmm_slots;
    if (slots > 0) return slots;
    if (m_vec < 1) m_vec = 1;
    const long long avg = (nonzeros_vec + m_vec - 1) / m_vec;
    const long long avg_groups = (avg + group - 1) / group;
    long long pick;
    if (mfma) {
        long long cap = m_vec <= 1024 ? 2048 / m_vec : 8192 / m_vec;
        if (m_vec <= 1024 && cap < 8) cap = 8;
        pick = avg_groups < cap ? avg_groups : cap;
    } else {
        const long long want = (8192 + m_vec - 1) / m_vec;
        pick = 2 * avg_groups < want ? 2 * avg_groups : want;
    }
    return pick < 1 ? 1 : (int)pick;
}

template <typename OutT>
int launch_sddmm_mfma(int m_vec, int k, int n, int nonzeros_vec, const int *row_indices,
                      const int *row_offsets, const int *col_indices, const half_t *lhs,
                      const half_t *rhs, OutT *out, int vec_length, hipStream_t stream, const Batch &batch)
{
    (void)n;
    if (m_vec == 0 || nonzeros_vec == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (k <= 0) return hipErrorNotSupported;
    // Contraction lengths off a multiple of 8 (rows of the dense operands then start at any 2-byte boundary, out of
    // reach of 128-bit loads) run on the fine-grained kernel's scalar-load variant, whatever the algorithm: the
    // whole of k is contracted on both paths (the reference's MMA kernels drop k % 64, src/wmma_sddmm.cu:88-120).
    if (k % 8 != 0) {
        if (batch.row_parts) return hipErrorNotSupported;  // (the fine-grained kernel takes no dispatch list)
        return launch_sddmm_valu<OutT>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out,
                                       vec_length, stream, batch);
    }
    // algorithm 0 (automatic): vectors of 1, 2 or 4 rows fill 1/16 to 4/16 of an MFMA tile, and on masks of few
    // nonzeros the fine-grained kernel (dot products on the vector ALU, reduced across lanes with DPP) is ahead:
    // over the M = N = 512..4096, K = 64..256 grid by 5-40 % below these nonzero counts, behind above them.
    if (batch.algorithm == 0 && vec_length <= 4 && !batch.row_parts) {
        const long long total = (long long)nonzeros_vec * batch.count;
        long long limit = 0;
        if (vec_length == 1) limit = 800000;
        else if (vec_length == 2) limit = k >= 256 ? 200000 : (k >= 128 ? 16000 : 0);
        else limit = k >= 256 ? 16000 : (k >= 128 ? 8000 : 0);
        if (total <= limit)
            return launch_sddmm_valu<OutT>(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out,
                                           vec_length, stream, batch);
    }
    switch (vec_length) {
    case 1: return launch_ks<1, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 2: return launch_ks<2, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 4: return launch_ks<4, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    case 8: return launch_ks<8, OutT>(m_vec, k, nonzeros_vec, row_indices, row_offsets, col_indices, lhs, rhs, out, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

template int launch_sddmm_mfma<half_t>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                       const half_t *, half_t *, int, hipStream_t, const Batch &);
template int launch_sddmm_mfma<float>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                      const half_t *, float *, int, hipStream_t, const Batch &);

}  // namespace vs
