// Fixed-mask sparse attention for a block of R consecutive vector rows per workgroup: the K and V rows
// those rows need are gathered ONCE into LDS ("union gather") and the block is then computed as a dense
// tile against that union, with a per-row bit mask deciding which scores exist.
//
// Structured masks (local band, block-diagonal, strided columns) make neighbouring rows share almost all
// of their columns: with a band of 257 columns, 16 consecutive vector rows of length 8 touch ~410 distinct
// columns, not 16 x 283.  Computing every row against the whole union wastes a little arithmetic on
// masked-out pairs, but it fills all 16 rows of the MFMA tile (one vector row alone fills V of them),
// needs no per-nonzero address arithmetic (the union's rows sit in LDS in rank order, every address is
// lane base + immediate) and reads every K / V row from memory once per block.  Random masks have no
// overlap: when the union does not fit the LDS budget the workgroup falls back to per-row gathers from
// global memory (the caller should pick the one-row-per-workgroup kernel for such masks).
//
// Workgroup steps (W waves, 16 scalar rows = 16 / V vector rows per wave, K and V share ONE LDS buffer so
// that two workgroups fit a CU):
//   1  bitmap of the block's columns in LDS (atomic or), exclusive prefix of its word popcounts:
//      rank(col) = prefix[col / 32] + popcount(bitmap[col / 32] below bit col % 32) is the position of a
//      column in the sorted union; U = total popcount.
//   2  every nonzero writes its column at the column's rank (the list of the union) and sets its bit in
//      its vector row's mask over ranks (bit r set: the row holds the column of rank r).  Steps 1 and 2
//      depend only on the mask: a plan (sparse_attention_plan_kernel) holds their result for every
//      workgroup, and launches that are given one read it instead.  Copy the K rows of the union to LDS (128-bit loads, rows padded by 16 bytes
//      against bank conflicts, rows U.. of the last 32-rank step zero-filled).
//   A  per wave and 32-rank step: S^T = K_union Q^T on v_mfma_f32_16x16x32_f16 with the K rows as the A
//      operand and the wave's 16 Q rows as the B operand: lane (c, g) receives the scores of scalar row
//      c for ranks 4g..4g+3 of both 16-rank halves.  Steps in which none of the wave's rows holds a
//      column are skipped.  Run twice: the first pass keeps only the row maximum, the second recomputes
//      the scores (LDS reads and MFMA are cheap, registers are not) and keeps p = exp2(s - max) as packed
//      fp16, masked-out pairs as exact zeros.  The maximum of scalar row c combines the four lanes (c, *).
//   3  barrier, copy the V rows of the union over the K rows, barrier.
//   C  per wave and step: P V on the same MFMA with P as the A operand.  The contraction index of an MFMA
//      can be numbered freely as long as both operands agree, so k-slot (g, e) is DEFINED as the rank the
//      lane already holds: e < 4 -> rank 4g + e of the step's first half, e >= 4 -> 4g + e - 4 of its
//      second half.  P therefore goes from the score registers into the A operand with no data movement,
//      and the V rows (transposed in registers with v_perm_b32, as in the SpMM kernel) are read in that
//      same order.  One more MFMA per step with an all-ones B operand yields the row sums of the rounded
//      p in exactly the accumulator layout, so normalising needs no cross-lane traffic.
// Planned launches of eight waves do not hold the union at once: sparse_attention_stream_kernel below runs
// steps 2 (the copy) to C per sub-round of 128 ranks, the next sub-round's rows on their way meanwhile, with
// the V rows transposed while they are copied (one transposition per workgroup instead of one per wave).
#include "vs_common.hpp"

namespace vs {

constexpr int kMaxSteps = 10;   // fallback: 32-vector steps of a row whose scores are held in registers at once
constexpr int kUnionSteps = 16; // 32-rank steps of the union whose probabilities are held in registers at once

// Value of `x` held by lane `src_lane` (all lanes active).
__device__ __forceinline__ float from_lane(float x, int src_lane)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, x)));
}

// The K or V rows of a vector row's nonzeros, read from global memory by column (per-row path).
struct RowSource {
    const half_t *base;      // the global operand
    int pitch;               // halves between consecutive rows of `base`
    const int *col_indices;  // column of nonzero j
    __device__ __forceinline__ const half_t *row_of(int j, int end) const
    {
        const int jc = j < end ? j : end - 1;  // slots past the row's end repeat its last vector
        return base + (size_t)col_indices[jc] * pitch;
    }
};

// Scores of the 64 nonzeros [j0, j0 + 64) of a row against the row's Q slices.
// out[u][e]: group u (16 vectors), register e -> nonzero j0 + 16u + 4g + e, base-2 units, -inf past `end`.
template <int KS>
__device__ __forceinline__ void scores64(float (&out)[4][4], const RowSource &ksrc, int j0, int end, int d_qk,
                                         const half8_t (&qb)[KS], float s2, int c, int g)
{
    half8_t a[4][KS];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const half_t *k_row = ksrc.row_of(j0 + 16 * u + c, end);
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) a[u][kk] = __builtin_bit_cast(half8_t, load_slice16(k_row, kk, g, d_qk, true));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        float4_t sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][kk], qb[kk], sacc, 0, 0, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = j0 + 16 * u + 4 * g + e;
            out[u][e] = j < end ? sacc[e] * s2 : -__builtin_inff();
        }
    }
}

// Phase A for the nonzeros [c0, cend) of a row (at most 32*kMaxSteps of them): maximum `mx` of the
// base-2 scores joined with `m_floor`, then p = exp2(s - mx) as packed fp16 in MFMA k-slot order and
// the sum of the p.  Two passes over K: the first keeps only the maximum, the second recomputes the
// scores (LDS / cache reads and MFMA are cheap, registers are not).
template <int KS>
__device__ __forceinline__ void softmax_chunk(half8_t (&p)[kMaxSteps], float &mx, float &sum, float m_floor,
                                              const RowSource &ksrc, int c0, int cend, int d_qk,
                                              const half8_t (&qb)[KS], float s2, int c, int g)
{
    const int n_steps = (cend - c0 + 31) >> 5;
    mx = m_floor;
#pragma unroll
    for (int ss = 0; ss < kMaxSteps / 2; ++ss) {
        if (2 * ss < n_steps) {
            float sc[4][4];
            scores64<KS>(sc, ksrc, c0 + 64 * ss, cend, d_qk, qb, s2, c, g);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) mx = fmaxf(mx, sc[u][e]);
        }
    }
    mx = fmaxf(mx, partner<16>(mx));  // scalar row v = c lives in the four lanes (c, g = 0..3)
    mx = fmaxf(mx, partner<32>(mx));
    sum = 0.f;
#pragma unroll
    for (int ss = 0; ss < kMaxSteps / 2; ++ss) {
        p[2 * ss] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        p[2 * ss + 1] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (2 * ss < n_steps) {
            float sc[4][4];
            scores64<KS>(sc, ksrc, c0 + 64 * ss, cend, d_qk, qb, s2, c, g);
            // k-slot (g, e) of step t: e < 4 -> nonzero 4g + e of group 2t, e >= 4 -> 4g + e - 4 of group 2t + 1
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float pe = __builtin_amdgcn_exp2f(sc[u][e] - mx);  // exp2(-inf) = 0 past the row's end
                    sum += pe;
                    p[2 * ss + (u >> 1)][4 * (u & 1) + e] = (half_t)pe;
                }
            }
        }
    }
    sum += partner<16>(sum);
    sum += partner<32>(sum);
}

// Phase C for the same nonzeros: acc += P V with the gathered V rows transposed in registers.
template <int CPL>
__device__ __forceinline__ void accumulate_chunk(float4_t (&acc)[CPL], const half8_t (&p)[kMaxSteps],
                                                 const RowSource &vsrc, int c0, int cend, int col_off, int g)
{
    const int n_steps = (cend - c0 + 31) >> 5;
#pragma unroll
    for (int ss = 0; ss < kMaxSteps / 2; ++ss) {
        if (2 * ss < n_steps) {
            RowChunk<CPL> rows[2][8];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int j = c0 + 32 * (2 * ss + t) + (e < 4 ? 4 * g + e : 16 + 4 * g + (e - 4));
                    rows[t][e].load(vsrc.row_of(j, cend) + col_off);
                }
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int pp = 0; pp < CPL / 2; ++pp) {
                    uint4_t even, odd;
#pragma unroll
                    for (int qq = 0; qq < 4; ++qq) {
                        even[qq] = pack_lo(rows[t][2 * qq].dword(pp), rows[t][2 * qq + 1].dword(pp));
                        odd[qq] = pack_hi(rows[t][2 * qq].dword(pp), rows[t][2 * qq + 1].dword(pp));
                    }
                    acc[2 * pp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p[2 * ss + t], __builtin_bit_cast(half8_t, even), acc[2 * pp], 0, 0, 0);
                    acc[2 * pp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p[2 * ss + t], __builtin_bit_cast(half8_t, odd), acc[2 * pp + 1], 0, 0, 0);
                }
            }
        }
    }
}

// Divide the accumulated tile of a vector row by its softmax sums and store it.
template <int V, int CPL>
__device__ __forceinline__ void store_row(half_t *out, int row, int d_v, const float4_t (&acc)[CPL], float l_sum,
                                          bool empty, int c, int g)
{
    const int col0 = c * CPL;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int vv = 4 * g + e;
        const float le = from_lane(l_sum, vv & 15);  // the sum of scalar row vv lives in the lanes with c = vv
        if (vv < V && col0 < d_v) {
            const float norm = empty ? 0.f : 1.f / le;  // an empty row attends to nothing: zeros
            float tmp[CPL];
#pragma unroll
            for (int cc = 0; cc < CPL; ++cc) tmp[cc] = acc[cc][e] * norm;
            store_converted<half_t, CPL>(out + ((size_t)row * V + vv) * d_v + col0, tmp);
        }
    }
}

// Q^T of a vector row as the MFMA B operand: lane (v = c, g) holds Q[row*V + v][32kk + 8g .. +8).
template <int V, int KS>
__device__ __forceinline__ void load_q(half8_t (&qb)[KS], const half_t *q, int row, int d_qk, int c, int g)
{
    const bool ok = c < V;
    const half_t *q_row = q + ((size_t)row * V + (ok ? c : 0)) * d_qk;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) qb[kk] = __builtin_bit_cast(half8_t, load_slice16(q_row, kk, g, d_qk, ok));
}

// 16 consecutive scalar rows of Q as the MFMA B operand: lane (c, g) holds Q[first + c][32kk + 8g .. +8),
// zeros for rows at or past `limit`.
template <int KS>
__device__ __forceinline__ void load_q16(half8_t (&qb)[KS], const half_t *q, long long first, long long limit,
                                         int d_qk, int c, int g)
{
    const bool ok = first + c < limit;
    const half_t *q_row = q + (size_t)(ok ? first + c : 0) * d_qk;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) qb[kk] = __builtin_bit_cast(half8_t, load_slice16(q_row, kk, g, d_qk, ok));
}

// `x` where bit `bit` of `word` is set, `other` elsewhere (v_bfe_i32 + v_bfi_b32).
__device__ __forceinline__ float select_bit(unsigned word, int bit, float x, float other)
{
    const unsigned m = (unsigned)__builtin_amdgcn_sbfe((int)word, bit, 1);  // 0 or ~0
    return __builtin_bit_cast(float, (__builtin_bit_cast(unsigned, x) & m) | (__builtin_bit_cast(unsigned, other) & ~m));
}

// Halves between consecutive rows of the LDS copy: room for every slice either phase reads, plus
// 16 bytes so that consecutive ranks start 4 banks apart.
constexpr int union_pitch(int ks, int cpl)
{
    return (32 * ks > 16 * cpl ? 32 * ks : 16 * cpl) + 8;
}

// Head widths above 64 on either side (128 halves per K or V row).
constexpr bool union_wide(int ks, int cpl) { return ks == 4 || cpl == 8; }

// The K rows of one 32-rank step as MFMA A operands: a[u][kk] = row 32t + 16u + c, halves 32kk + 8g .. +8.
template <int KS, int PITCH>
__device__ __forceinline__ void load_k_step(half8_t (&a)[2][KS], const half_t *k_lane, int t)
{
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)
            a[u][kk] = *reinterpret_cast<const half8_t *>(k_lane + (32 * t + 16 * u) * PITCH + 32 * kk);
}

// S^T of one 32-rank step: sacc[u][e] = score of the lane's scalar row against rank 32t + 16u + 4g + e.
template <int KS>
__device__ __forceinline__ void scores_step(float4_t (&sacc)[2], const half8_t (&a)[2][KS], const half8_t (&qb)[KS])
{
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        sacc[u] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) sacc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][kk], qb[kk], sacc[u], 0, 0, 0);
    }
}

// The per-row path for the vector rows [row_first, row_last) of a workgroup: one vector row per wave at a time
// with the K / V rows read from global memory by column; no barrier, long rows in chunks with a running
// maximum and sum.
template <int V, int KS, int CPL>
__device__ __forceinline__ void per_row_block(int row_first, int row_last, int wave, int n_waves,
                                              const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                                              const half_t *__restrict__ q, const half_t *__restrict__ k,
                                              const half_t *__restrict__ v, half_t *__restrict__ out, int d_qk, int d_v,
                                              float s2, int c, int g, int col_off)
{
    const RowSource ksrc = {k, d_qk, col_indices};
    const RowSource vsrc = {v, d_v, col_indices};
    for (int row = row_first + wave; row < row_last; row += n_waves) {
        const int beg = row_offsets[row];
        const int end = row_offsets[row + 1];
        half8_t qb[KS];
        load_q<V, KS>(qb, q, row, d_qk, c, g);
        float m_run = -__builtin_inff(), l_run = 0.f;
        float4_t acc[CPL];
#pragma unroll
        for (int cc = 0; cc < CPL; ++cc) acc[cc] = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int c0 = beg; c0 < end; c0 += 32 * kMaxSteps) {
            const int cend = (c0 + 32 * kMaxSteps) < end ? (c0 + 32 * kMaxSteps) : end;
            half8_t p[kMaxSteps];
            float m_new, sum;
            softmax_chunk<KS>(p, m_new, sum, m_run, ksrc, c0, cend, d_qk, qb, s2, c, g);
            const float f = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first chunk (m_run = -inf)
            l_run = l_run * f + sum;
            m_run = m_new;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float fe = from_lane(f, (4 * g + e) & 15);  // accumulator row 4g + e belongs to scalar row 4g + e
#pragma unroll
                for (int cc = 0; cc < CPL; ++cc) acc[cc][e] *= fe;
            }
            accumulate_chunk<CPL>(acc, p, vsrc, c0, cend, col_off, g);
        }
        store_row<V, CPL>(out, row, d_v, acc, l_run, end == beg, c, g);
    }
}

// LDS arrays that describe the union of a block of rows.
struct UnionLds {
    unsigned *bitmap;   // [n_words] columns present in the block
    unsigned *prefix;   // [n_words] exclusive prefix of the bitmap's word popcounts
    int *wave_tot;      // [16] scan scratch, [15] = number of distinct columns
    unsigned *rowmask;  // [rounds][rows][steps] ranks each row holds, u_max = 32 * steps ranks per round at most
    int *ucols;         // [rounds * u_max] columns of the union in ascending order
};

// Steps 1 and 2 of the header comment for rows [row_first, row_last), by the whole workgroup: returns the
// number U of distinct columns; rowmask ([rounds][mask_words]) and ucols are complete (and visible to every
// thread) on return when U <= rounds * u_max, otherwise only U is meaningful.
__device__ __forceinline__ int build_union(const UnionLds &l, int n_words, int mask_words, int u_max, int rounds,
                                           int steps, int row_first, int row_last, const int *__restrict__ row_offsets,
                                           const int *__restrict__ col_indices)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_waves = blockDim.x >> 6;
    const int n_threads = blockDim.x;
    for (int w = tid; w < n_words; w += n_threads) l.bitmap[w] = 0u;
    for (int w = tid; w < rounds * mask_words; w += n_threads) l.rowmask[w] = 0u;
    __syncthreads();
    const int nz_first = row_offsets[row_first];
    const int nz_last = row_offsets[row_last];
    for (int j0 = nz_first + tid; j0 < nz_last; j0 += 4 * n_threads) {
        int col[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int j = j0 + i * n_threads;
            col[i] = j < nz_last ? col_indices[j] : -1;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (col[i] >= 0) atomicOr(&l.bitmap[col[i] >> 5], 1u << (col[i] & 31));
    }
    __syncthreads();
    if (n_words <= 1024) {
        // exclusive prefix of the word popcounts by one wave: a contiguous run of words per lane (one
        // barrier and no cross-wave step; the other waves only wait)
        if (wave == 0) {
            const int per = (n_words + 63) >> 6;
            const int w0 = lane * per;
            int local = 0;
            for (int w = w0; w < w0 + per && w < n_words; ++w) local += __builtin_popcount(l.bitmap[w]);
            int incl = local;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int up = __builtin_amdgcn_ds_bpermute(((lane - d) & 63) << 2, incl);
                if (lane >= d) incl += up;
            }
            int run = incl - local;
            for (int w = w0; w < w0 + per && w < n_words; ++w) {
                l.prefix[w] = (unsigned)run;
                run += __builtin_popcount(l.bitmap[w]);
            }
            if (lane == 63) l.wave_tot[15] = incl;
        }
        __syncthreads();
    } else {
        // the same with every thread taking a run of words: per-thread totals scanned inside each wave,
        // then the wave totals added up
        const int per = (n_words + n_threads - 1) / n_threads;
        const int w0 = tid * per;
        int local = 0;
        for (int w = w0; w < w0 + per && w < n_words; ++w) local += __builtin_popcount(l.bitmap[w]);
        int incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __builtin_amdgcn_ds_bpermute(((lane - d) & 63) << 2, incl);
            if (lane >= d) incl += up;
        }
        if (lane == 63) l.wave_tot[wave] = incl;
        __syncthreads();
        int base = 0;
        for (int w = 0; w < wave; ++w) base += l.wave_tot[w];
        int run = base + incl - local;
        for (int w = w0; w < w0 + per && w < n_words; ++w) {
            l.prefix[w] = (unsigned)run;
            run += __builtin_popcount(l.bitmap[w]);
        }
        if (tid == n_threads - 1) l.wave_tot[15] = run;
        __syncthreads();
    }
    const int n_union = l.wave_tot[15];
    if (n_union > rounds * u_max) return n_union;
    // every nonzero sets its bit in its row's mask and writes its column at the column's rank (all writers
    // of one rank write the same value), which lists the union without a pass over the bitmap; ranks
    // [i * u_max, (i + 1) * u_max) belong to round i, whose masks follow those of round i - 1
    auto mask_bit = [&](int r, int rank) {
        int word = r * steps;
        if (rounds > 1) {
            const int round = rank / u_max;
            rank -= round * u_max;
            word += round * mask_words;
        }
        atomicOr(&l.rowmask[word + (rank >> 5)], 1u << (rank & 31));
    };
    for (int r = wave; r < row_last - row_first; r += n_waves) {
        const int beg = row_offsets[row_first + r];
        const int end = row_offsets[row_first + r + 1];
        for (int j0 = beg + lane; j0 < end; j0 += 128) {
            const int j1 = j0 + 64;
            const int col_a = col_indices[j0];
            const int col_b = col_indices[j1 < end ? j1 : j0];
            const int rank_a = (int)l.prefix[col_a >> 5] + __builtin_popcount(l.bitmap[col_a >> 5] & ((1u << (col_a & 31)) - 1u));
            const int rank_b = (int)l.prefix[col_b >> 5] + __builtin_popcount(l.bitmap[col_b >> 5] & ((1u << (col_b & 31)) - 1u));
            mask_bit(r, rank_a);
            mask_bit(r, rank_b);
            l.ucols[rank_a] = col_a;
            l.ucols[rank_b] = col_b;
        }
    }
    __syncthreads();
    return n_union;
}

// A plan holds what build_union computes for every workgroup of a launch shape, so that launches on the
// same mask (every head, layer and step) read it instead of rebuilding it.  Layout, in 32-bit words:
// header [magic, m_vec, V, n, rows per workgroup, u_max, record stride, workgroups, rounds, steps, 0...]
// (16 words), then one record per workgroup: [U, 0, 0, 0], rowmask [rounds][rows][steps] (each round padded
// to 4 words), ucols [rounds * u_max].  Workgroups of eight waves stream the union through LDS
// (sparse_attention_stream_kernel): kStreamRounds rounds of kStreamRanks ranks.  Smaller workgroups hold the
// whole union in LDS at once: one round of up to 32 * kUnionSteps ranks.
constexpr int kPlanMagic = 0x56535041;
constexpr int kPlanHeader = 16;
constexpr int kStreamSteps = 4;
constexpr int kStreamRanks = 32 * kStreamSteps;
constexpr int kStreamRounds = 16;

__global__ void __launch_bounds__(256)
sparse_attention_plan_kernel(int m_vec, int vec_length, int n, int rows_per_block, int u_max, int rounds, int steps,
                             const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                             int *__restrict__ plan)
{
    const int n_words = (n + 31) >> 5;
    const int n_words_al = (n_words + 3) & ~3;
    const int mask_words = (rows_per_block * steps + 3) & ~3;
    extern __shared__ __align__(16) unsigned char smem[];
    UnionLds l;
    l.bitmap = reinterpret_cast<unsigned *>(smem);
    l.prefix = l.bitmap + n_words_al;
    l.wave_tot = reinterpret_cast<int *>(l.prefix + n_words_al);
    l.rowmask = reinterpret_cast<unsigned *>(l.wave_tot + 16);
    l.ucols = reinterpret_cast<int *>(l.rowmask + rounds * mask_words);
    const int cap = rounds * u_max;
    const int stride = 4 + rounds * mask_words + cap;
    const int tid = threadIdx.x;
    if (blockIdx.x == 0 && tid < kPlanHeader) {
        const int header[kPlanHeader] = {kPlanMagic, m_vec, vec_length, n, rows_per_block, u_max, stride,
                                         (int)gridDim.x, rounds, steps, 0, 0, 0, 0, 0, 0};
        int value = 0;
#pragma unroll
        for (int i = 0; i < kPlanHeader; ++i) value = (i == tid) ? header[i] : value;
        plan[tid] = value;
    }
    const int row_first = blockIdx.x * rows_per_block;
    const int row_last = (row_first + rows_per_block) < m_vec ? (row_first + rows_per_block) : m_vec;
    const int n_union = build_union(l, n_words, mask_words, u_max, rounds, steps, row_first, row_last,
                                    row_offsets, col_indices);
    int *rec = plan + kPlanHeader + (size_t)blockIdx.x * stride;
    if (tid < 4) rec[tid] = tid == 0 ? n_union : 0;
    if (n_union > cap) return;  // this workgroup's rows take the per-row path at every launch
    for (int w = tid; w < rounds * mask_words; w += blockDim.x) rec[4 + w] = (int)l.rowmask[w];
    for (int u = tid; u < cap; u += blockDim.x) rec[4 + rounds * mask_words + u] = u < n_union ? l.ucols[u] : 0;
}

// V: vector length; KS: d_qk <= 32*KS; CPL: d_v <= 16*CPL.
// PLANNED: the union and the row masks come from a plan of one round (sparse_attention_plan_kernel) instead
// of being rebuilt; a plan made for another mask shape or launch shape sends every workgroup to the per-row
// path.
template <int V, int KS, int CPL, bool PLANNED>
// Heads up to 64 wide: four waves per SIMD (128 registers), two eight-wave workgroups per CU.  Wider heads
// hold twice the Q / K / V slices per lane and 272-byte rows in LDS: two waves per SIMD (256 registers), one
// workgroup per CU with all of its LDS.
__global__ void __launch_bounds__(512, union_wide(KS, CPL) ? 2 : 4)
sparse_attention_union_kernel(int m_vec, int n, int d_qk, int d_v, int u_max,
                              const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                              const int *__restrict__ plan,
                              const half_t *__restrict__ q, const half_t *__restrict__ k,
                              const half_t *__restrict__ v, half_t *__restrict__ out, long long stride_q,
                              long long stride_k, long long stride_v, long long stride_out, float scale)
{
    q += blockIdx.y * stride_q;
    k += blockIdx.y * stride_k;
    v += blockIdx.y * stride_v;
    out += blockIdx.y * stride_out;
    constexpr int RPW = 16 / V;  // vector rows per wave: 16 scalar rows fill the MFMA tile
    constexpr int PITCH = union_pitch(KS, CPL);
    const int n_words = (n + 31) >> 5;
    const int n_words_al = (n_words + 3) & ~3;  // keeps the arrays behind the bitmap 16-byte aligned

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: row bounds stay in scalar registers
    const int n_waves = blockDim.x >> 6;
    const int n_threads = blockDim.x;
    const int rows_per_block = n_waves * RPW;
    const int mask_words = (rows_per_block * kUnionSteps + 3) & ~3;

    extern __shared__ __align__(16) unsigned char smem[];
    UnionLds l;
    half_t *buf;  // [u_max][PITCH]: K rows, later V rows
    if constexpr (PLANNED) {
        l.bitmap = l.prefix = nullptr;
        l.wave_tot = nullptr;
        l.rowmask = reinterpret_cast<unsigned *>(smem);
        buf = reinterpret_cast<half_t *>(l.rowmask + mask_words);
        l.ucols = nullptr;
    } else {
        l.bitmap = reinterpret_cast<unsigned *>(smem);
        l.prefix = l.bitmap + n_words_al;
        l.wave_tot = reinterpret_cast<int *>(l.prefix + n_words_al);
        l.rowmask = reinterpret_cast<unsigned *>(l.wave_tot + 16);
        buf = reinterpret_cast<half_t *>(l.rowmask + mask_words);
        l.ucols = reinterpret_cast<int *>(buf + (size_t)u_max * PITCH);
    }
    const unsigned *rowmask = l.rowmask;

    // Consecutive workgroups go to different XCDs (each with its own L2); neighbouring row blocks share
    // most of their K / V rows, so every XCD takes a contiguous run of row blocks instead.
    int bx = blockIdx.x;
    if ((gridDim.x & 7) == 0) bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);
    const int row_first = bx * rows_per_block;
    const int row_last = (row_first + rows_per_block) < m_vec ? (row_first + rows_per_block) : m_vec;
    const int c = lane & 15;
    const int g = lane >> 4;
    const float s2 = scale * kLog2e;
    const int col0 = c * CPL;
    const bool col_ok = col0 < d_v;
    const int col_off = col_ok ? col0 : 0;

    // ---- 1, 2. the union's columns and every row's mask over ranks: built here or read from the plan
    int n_union;
    const int *cols;  // columns of the union: LDS (built) or the plan's record (global)
    if constexpr (PLANNED) {
        const int stride = 4 + mask_words + u_max;
        const bool plan_ok = plan[0] == kPlanMagic && plan[1] == m_vec && plan[2] == V && plan[3] == n &&
                             plan[4] == rows_per_block && plan[5] == u_max && plan[6] == stride &&
                             plan[7] == (int)gridDim.x && plan[8] == 1 && plan[9] == kUnionSteps;
        const int *rec = plan + kPlanHeader + (size_t)(plan_ok ? bx : 0) * stride;
        n_union = plan_ok ? rec[0] : 0x7fffffff;
        cols = rec + 4 + mask_words;
        if (n_union <= u_max)
            for (int w = tid; w < mask_words; w += n_threads) l.rowmask[w] = (unsigned)rec[4 + w];
        // visible to the other waves after the barrier that follows the K gather
    } else {
        n_union = build_union(l, n_words, mask_words, u_max, 1, kUnionSteps, row_first, row_last, row_offsets,
                              col_indices);
        cols = l.ucols;
    }
    const bool use_lds = n_union <= u_max && (d_v % 8 == 0);
    if (!use_lds) {
        per_row_block<V, KS, CPL>(row_first, row_last, wave, n_waves, row_offsets, col_indices, q, k, v, out, d_qk, d_v,
                                  s2, c, g, col_off);
        return;
    }

    // ---- 2b .. C
    // Copy one operand's rows of ranks [u_first, u_first + n_here) into buf: 16 bytes per thread and slice,
    // kBatch slices in flight; rows past the round's ranks (the last step's padding) and slices past `d` are
    // written as zeros, so the arithmetic below never meets stale bits.
    auto gather = [&](const half_t *src, int d, int slice_shift, int u_first, int n_here, int n_steps) {
        constexpr int kBatch = 8;
        const int slices = d >> 3;
        const int total = (32 * n_steps) << slice_shift;
        for (int s0 = tid; s0 < total; s0 += kBatch * n_threads) {
            uint4_t data[kBatch];
            int dst[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int sidx = s0 + i * n_threads;
                dst[i] = -1;
                if (sidx < total) {
                    const int u = sidx >> slice_shift, sl = sidx & ((1 << slice_shift) - 1);
                    const bool real = u < n_here && sl < slices;
                    const int at = real ? u_first + u : 0;
                    const int col = PLANNED ? cols[at] : l.ucols[at];  // two address spaces
                    const uint4_t x = *reinterpret_cast<const uint4_t *>(src + (size_t)col * d + (real ? 8 * sl : 0));
                    const uint4_t zero = {0u, 0u, 0u, 0u};
                    data[i] = real ? x : zero;
                    dst[i] = u * PITCH + 8 * sl;
                }
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i)
                if (dst[i] >= 0) *reinterpret_cast<uint4_t *>(buf + dst[i]) = data[i];
        }
    };
    constexpr int kShiftK = KS == 1 ? 2 : (KS == 2 ? 3 : 4);  // 4 * KS slices of 8 halves per K row
    constexpr int kShiftV = CPL == 4 ? 3 : 4;                 // 2 * CPL slices per V row
    const int q_first = 16 * wave;                                 // first scalar row of the wave inside the block
    const long long q_global = (long long)row_first * V + q_first;  // the same in the whole operand
    const long long q_limit = (long long)row_last * V;
    half8_t qb[KS];  // requested before the K rows so that the first MFMA does not wait for it
    load_q16<KS>(qb, q, q_global, q_limit, d_qk, c, g);
    // The maximum is tracked on the raw dot products, so the scale must be non-negative: a negative one
    // moves its sign into Q.
    const float s2a = __builtin_fabsf(s2);
    if (s2 < 0.f) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            uint4_t bits = __builtin_bit_cast(uint4_t, qb[kk]);
#pragma unroll
            for (int i = 0; i < 4; ++i) bits[i] ^= 0x80008000u;
            qb[kk] = __builtin_bit_cast(half8_t, bits);
        }
    }
    const unsigned *mrow = rowmask + ((q_first + c) / V) * kUnionSteps;  // mask of the lane's vector row
    const half_t *k_lane = buf + c * PITCH + 8 * g;
    const half_t *v_lane = buf + 4 * g * PITCH + col_off;
    const float neg_inf = -__builtin_inff();

    // ---- A. per wave: 16 scalar rows against the n_steps steps of ranks in buf; maximum, then masked
    // exponentials; act = steps in which at least one row of the wave holds a column (uniform).
    auto scores = [&](int n_steps, half8_t (&p)[kUnionSteps], unsigned &act) {
        constexpr unsigned kLaneBits = 0x000F000Fu;  // after the shift by 4g: the lane's 4 + 4 ranks of a step
        unsigned full = 0;  // steps in which every lane's rows hold all of the lane's ranks: no masking needed
        float mx_raw = neg_inf;
        act = 0;
#pragma unroll
        for (int t = 0; t < kUnionSteps; ++t) {
            if (t < n_steps) {
                const unsigned word = mrow[t];
                if (__builtin_amdgcn_ballot_w64(word != 0u) != 0ull) {
                    act |= 1u << t;
                    const unsigned wg = word >> (4 * g);
                    half8_t a[2][KS];
                    load_k_step<KS, PITCH>(a, k_lane, t);
                    float4_t sacc[2];
                    scores_step<KS>(sacc, a, qb);
                    if (__builtin_amdgcn_ballot_w64((wg & kLaneBits) != kLaneBits) == 0ull) {
                        full |= 1u << t;
#pragma unroll
                        for (int u = 0; u < 2; ++u)
                            mx_raw = fmaxf(fmaxf(mx_raw, fmaxf(sacc[u][0], sacc[u][1])), fmaxf(sacc[u][2], sacc[u][3]));
                    } else {
#pragma unroll
                        for (int u = 0; u < 2; ++u)
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                mx_raw = fmaxf(mx_raw, select_bit(wg, 16 * u + e, sacc[u][e], neg_inf));
                    }
                }
            }
        }
        act = __builtin_amdgcn_readfirstlane(act);
        full = __builtin_amdgcn_readfirstlane(full);
        mx_raw = fmaxf(mx_raw, partner<16>(mx_raw));  // scalar row c lives in the four lanes (c, g = 0..3)
        mx_raw = fmaxf(mx_raw, partner<32>(mx_raw));
        const float neg_mx = mx_raw == neg_inf ? 0.f : -(mx_raw * s2a);  // a row with no column: every exponent stays -inf
#pragma unroll
        for (int t = 0; t < kUnionSteps; ++t) {
            p[t] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            if ((act >> t) & 1u) {
                half8_t a[2][KS];
                load_k_step<KS, PITCH>(a, k_lane, t);
                float4_t sacc[2];
                scores_step<KS>(sacc, a, qb);
                // k-slot (g, e) of step t: e < 4 -> rank 4g + e of the first half, e >= 4 -> 4g + e - 4 of the second
                if ((full >> t) & 1u) {
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            p[t][4 * u + e] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf(sacc[u][e], s2a, neg_mx));
                } else {
                    const unsigned wg = mrow[t] >> (4 * g);
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float bias = select_bit(wg, 16 * u + e, neg_mx, neg_inf);
                            p[t][4 * u + e] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf(sacc[u][e], s2a, bias));
                        }
                }
            }
        }
    };

    // ---- C. P V and the row sums against the V rows in buf (one wave owns its rows: nothing to reduce)
    float4_t acc[CPL];
    float4_t lacc;
    auto weighted_sum = [&](const half8_t (&p)[kUnionSteps], unsigned act) {
        const half8_t ones = {1, 1, 1, 1, 1, 1, 1, 1};
#pragma unroll
        for (int t = 0; t < kUnionSteps; ++t) {
            if ((act >> t) & 1u) {
                RowChunk<CPL> rows[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) rows[e].load(v_lane + (32 * t + (e < 4 ? e : 12 + e)) * PITCH);
#pragma unroll
                for (int pp = 0; pp < CPL / 2; ++pp) {
                    uint4_t even, odd;
#pragma unroll
                    for (int qq = 0; qq < 4; ++qq) {
                        even[qq] = pack_lo(rows[2 * qq].dword(pp), rows[2 * qq + 1].dword(pp));
                        odd[qq] = pack_hi(rows[2 * qq].dword(pp), rows[2 * qq + 1].dword(pp));
                    }
                    acc[2 * pp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p[t], __builtin_bit_cast(half8_t, even), acc[2 * pp], 0, 0, 0);
                    acc[2 * pp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p[t], __builtin_bit_cast(half8_t, odd), acc[2 * pp + 1], 0, 0, 0);
                }
                lacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(p[t], ones, lacc, 0, 0, 0);  // row sums, in accumulator layout
            }
        }
    };
    auto clear_sums = [&]() {
#pragma unroll
        for (int cc = 0; cc < CPL; ++cc) acc[cc] = float4_t{0.f, 0.f, 0.f, 0.f};
        lacc = float4_t{0.f, 0.f, 0.f, 0.f};
    };

    {
        // the accumulators come to life only after the exponentials are packed
        const int n_steps = (n_union + 31) >> 5;  // <= kUnionSteps because u_max <= 32 * kUnionSteps
        gather(k, d_qk, kShiftK, 0, n_union, n_steps);
        __syncthreads();
        half8_t p[kUnionSteps];
        unsigned act;
        scores(n_steps, p, act);
        __syncthreads();
        gather(v, d_v, kShiftV, 0, n_union, n_steps);  // V rows over the K rows
        __syncthreads();
        clear_sums();
        weighted_sum(p, act);
    }
    // normalise and store
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const long long row = q_global + 4 * g + e;  // accumulator register e of lane (c, g) is scalar row 4g + e
        if (row < q_limit && col_ok) {
            const float norm = lacc[e] > 0.f ? 1.f / lacc[e] : 0.f;  // a row with no column attends to nothing: zeros
            float tmp[CPL];
#pragma unroll
            for (int cc = 0; cc < CPL; ++cc) tmp[cc] = acc[cc][e] * norm;
            store_converted<half_t, CPL>(out + (size_t)row * d_v + col0, tmp);
        }
    }
}

// Planned launches of eight waves stream the union through LDS in sub-rounds of kStreamRanks ranks, K rows
// and V columns side by side: the rows, row masks and column numbers of the NEXT sub-round are requested
// before the current one is computed and parked in registers meanwhile, so after the first sub-round no wave
// waits for a gather.  A sub-round is short enough to keep its raw scores in registers: the K rows are read
// and multiplied once, not twice.  Maximum and sums run across the sub-rounds as in flash attention, so a
// workgroup takes unions of up to kStreamRounds * kStreamRanks columns.
//
// The kernel is bound by vector-ALU instructions (softmax arithmetic and operand shuffles), so two things
// are kept out of the waves' inner loop.  The V rows of a sub-round go to LDS transposed, in the order the
// P V MFMA wants its B operand - the transposition is done once per workgroup while the rows are written, not
// once per wave while they are read.  And the mask enters the scores as the accumulators' start value (0 or
// -inf), so neither the maximum nor the exponentials look at it again.
constexpr int kStreamVPitch = kStreamRanks + 8;  // halves between consecutive V columns in LDS
typedef int int2_t __attribute__((ext_vector_type(2)));

// Where rank r of a sub-round sits inside a V column: lane (c, g) multiplies ranks 16u + 4g + e (u < 2,
// e < 4) of a 32-rank step, which this order puts into 16 consecutive bytes.
__device__ __forceinline__ int stream_v_slot(int r) { return (r & ~31) | (((r >> 2) & 3) << 3) | (((r >> 4) & 1) << 2) | (r & 3); }

// First rank of pair `pair` (0 .. kStreamRanks / 2) in the order the threads take them: consecutive pairs differ
// in the bits that choose the 32-bit word inside a 16-byte chunk (e bit 1, then u), so the 32 lanes of a
// transposed write hit 32 different banks.
__device__ __forceinline__ int stream_v_pair_rank(int pair)
{
    return ((pair & 1) << 1) | (((pair >> 1) & 1) << 4) | (((pair >> 2) & 3) << 2) | ((pair >> 4) << 5);
}

// Offset in halves of 8-rank chunk `chunk` of V column `col`; chunks are permuted by column so that neither
// the transposed writes (lanes of a quad: columns 8 apart) nor the reads (lanes: columns CPL apart) collide.
__device__ __forceinline__ int stream_v_offset(int col, int chunk) { return col * kStreamVPitch + ((chunk ^ ((col >> 3) & 7)) << 3); }

// The per-row path as a function of its own: inlined into the streamed kernel it takes every register the launch
// bounds leave, and the allocator then parks values of the streamed path in scratch memory around it.
template <int V, int KS, int CPL>
__device__ __noinline__ void per_row_block_call(int row_first, int row_last, int wave, int n_waves,
                                                const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                                                const half_t *__restrict__ q, const half_t *__restrict__ k,
                                                const half_t *__restrict__ v, half_t *__restrict__ out, int d_qk,
                                                int d_v, float s2, int c, int g, int col_off)
{
    per_row_block<V, KS, CPL>(row_first, row_last, wave, n_waves, row_offsets, col_indices, q, k, v, out, d_qk, d_v, s2,
                              c, g, col_off);
}

template <int V, int KS, int CPL>
__global__ void __launch_bounds__(512, union_wide(KS, CPL) ? 2 : 4)
sparse_attention_stream_kernel(int m_vec, int n, int d_qk, int d_v,
                               const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                               const int *__restrict__ plan,
                               const half_t *__restrict__ q, const half_t *__restrict__ k,
                               const half_t *__restrict__ v, half_t *__restrict__ out, long long stride_q,
                               long long stride_k, long long stride_v, long long stride_out, float scale)
{
    q += blockIdx.y * stride_q;
    k += blockIdx.y * stride_k;
    v += blockIdx.y * stride_v;
    out += blockIdx.y * stride_out;
    constexpr int RPW = 16 / V;
    constexpr int PITCH = 32 * KS + 8;                              // halves between consecutive K rows in LDS
    constexpr int SS = kStreamSteps;
    constexpr int SR = kStreamRanks;
    constexpr int kThreads = 512;
    constexpr int kRows = 8 * RPW;                                  // vector rows per workgroup
    constexpr int kMaskWords = (kRows * SS + 3) & ~3;               // the plan's words per round: [kRows][SS]
    constexpr int kShiftK = KS == 1 ? 2 : (KS == 2 ? 3 : 4);        // 4 * KS slices of 8 halves per K row
    constexpr int kShiftV = CPL == 4 ? 3 : 4;                       // 2 * CPL slices per V row
    constexpr int NK = (SR << kShiftK) / kThreads;                  // 16-byte slices per thread and sub-round
    constexpr int NV = ((SR / 2) << kShiftV) / kThreads;            // pairs of V slices (two consecutive ranks)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned *maskbuf = reinterpret_cast<unsigned *>(smem);        // [kRows][SS] masks of the sub-round in LDS
    half_t *kbuf = reinterpret_cast<half_t *>(maskbuf + kRows * SS);  // [SR][PITCH]
    half_t *vbuf = kbuf + SR * PITCH;                                 // [16 * CPL columns][kStreamVPitch]

    int bx = blockIdx.x;
    if ((gridDim.x & 7) == 0) bx = (bx & 7) * (gridDim.x >> 3) + (bx >> 3);  // a run of row blocks per XCD
    const int row_first = bx * kRows;
    const int row_last = (row_first + kRows) < m_vec ? (row_first + kRows) : m_vec;
    const int c = lane & 15;
    const int g = lane >> 4;
    float s2 = scale * kLog2e;
    const int col0 = c * CPL;
    const bool col_ok = col0 < d_v;
    const int col_off = col_ok ? col0 : 0;

    constexpr int u_cap = kStreamRounds * SR;
    constexpr int stride = 4 + kStreamRounds * kMaskWords + u_cap;
    const bool plan_ok = plan[0] == kPlanMagic && plan[1] == m_vec && plan[2] == V && plan[3] == n &&
                         plan[4] == kRows && plan[5] == SR && plan[6] == stride && plan[7] == (int)gridDim.x &&
                         plan[8] == kStreamRounds && plan[9] == SS;
    const int *rec = plan + kPlanHeader + (size_t)(plan_ok ? bx : 0) * stride;
    const int n_union = plan_ok ? rec[0] : 0x7fffffff;
    // The record, the K rows and the V rows are read through buffer descriptors: a scalar base and one 32-bit byte
    // offset per thread and load, where a 64-bit pointer per thread and load used to take the registers that the
    // launch bounds do not leave (n <= 2^20 columns of at most 128 halves: every offset is below 2^28).
    const __amdgpu_buffer_rsrc_t rec_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<int *>(rec), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(k), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(v), 0, 0x7fffffff, 0x00020000);
    constexpr unsigned kMasksAt = 4u * 4u;                                        // byte offsets inside the record
    constexpr unsigned kColsAt = 4u * (4u + kStreamRounds * kMaskWords);

    // What a thread fetches per sub-round: NK slices of K rows (thread t takes slices t, t + 512, ...:
    // consecutive threads read consecutive 16 bytes of a row), NV times the same slice of the V rows of two
    // consecutive ranks, and one mask word.
    int col_k[NK];
    int2_t col_v[NV];
    uint4_t stage_k[NK], stage_v[NV][2];
    unsigned stage_m = 0;
    // column numbers of sub-round `round` < kStreamRounds (the plan lists 0 past the union: row 0, unused), which
    // do not wait for the union's size
    auto fetch_cols = [&](int round) {
        const unsigned at = kColsAt + 4u * (unsigned)(round * SR);  // (uniform)
#pragma unroll
        for (int i = 0; i < NK; ++i)
            col_k[i] = (int)__builtin_amdgcn_raw_buffer_load_b32(rec_rsrc, 4u * ((unsigned)(tid + i * kThreads) >> kShiftK), at, 0);
#pragma unroll
        for (int i = 0; i < NV; ++i)
            col_v[i] = __builtin_bit_cast(int2_t, __builtin_amdgcn_raw_buffer_load_b64(
                rec_rsrc, 4u * (unsigned)stream_v_pair_rank((tid + i * kThreads) >> kShiftV), at, 0));
    };
    // Requests only: nothing here reads what the loads return, so the wave goes on to the arithmetic at once.
    // Slices past the union or past d read the start of a valid row and are replaced by zeros in commit().
    auto fetch_rows = [&](int round) {  // needs col_k / col_v of the same sub-round
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int sidx = tid + i * kThreads;
            const int u = round * SR + (sidx >> kShiftK), sl = sidx & ((1 << kShiftK) - 1);
            const bool real = u < n_union && 8 * sl < d_qk;
            stage_k[i] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, 2u * ((unsigned)col_k[i] * (unsigned)d_qk + (real ? 8u * sl : 0u)), 0, 0);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int sidx = tid + i * kThreads;
            const int u = round * SR + stream_v_pair_rank(sidx >> kShiftV), sl = sidx & ((1 << kShiftV) - 1);
            const unsigned off = (u < n_union && 8 * sl < d_v) ? 8u * sl : 0u;
            stage_v[i][0] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, 2u * ((unsigned)col_v[i][0] * (unsigned)d_v + off), 0, 0);
            stage_v[i][1] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, 2u * ((unsigned)col_v[i][1] * (unsigned)d_v + off), 0, 0);
        }
        if (tid < kRows * SS) {
            // (the offset is made anew in every sub-round: kept across the loop it is the one value the register
            // allocator parks in scratch memory, and its reload waits for every gather requested just above)
            unsigned word = (unsigned)tid;
            asm volatile("" : "+v"(word));
            stage_m = __builtin_amdgcn_raw_buffer_load_b32(rec_rsrc, 4u * word, kMasksAt + 4u * (unsigned)(round * kMaskWords), 0);
        }
    };
    // The parked sub-round `round` into LDS; rows past the union and slices past d as zeros, so the arithmetic
    // never meets stale bits.  V goes in transposed: a thread holds 8 columns of two consecutive ranks and
    // writes, per column, the two ranks as one 32-bit word.
    auto commit = [&](int round) {
        const uint4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int sidx = tid + i * kThreads;
            const int u = sidx >> kShiftK, sl = sidx & ((1 << kShiftK) - 1);
            const bool real = round * SR + u < n_union && 8 * sl < d_qk;
            *reinterpret_cast<uint4_t *>(kbuf + u * PITCH + 8 * sl) = real ? stage_k[i] : zero;
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int sidx = tid + i * kThreads;
            const int r0 = stream_v_pair_rank(sidx >> kShiftV), sl = sidx & ((1 << kShiftV) - 1);
            const bool wide_enough = 8 * sl < d_v;
            const uint4_t first = (wide_enough && round * SR + r0 < n_union) ? stage_v[i][0] : zero;
            const uint4_t second = (wide_enough && round * SR + r0 + 1 < n_union) ? stage_v[i][1] : zero;
            const int slot = stream_v_slot(r0);
            half_t *dst = vbuf + stream_v_offset(8 * sl, slot >> 3) + (slot & 7);  // columns 8 sl .. 8 sl + 7 share their chunk order
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                *reinterpret_cast<uint32_t *>(dst + (2 * jj) * kStreamVPitch) = pack_lo(first[jj], second[jj]);
                *reinterpret_cast<uint32_t *>(dst + (2 * jj + 1) * kStreamVPitch) = pack_hi(first[jj], second[jj]);
            }
        }
        if (tid < kRows * SS) maskbuf[tid] = stage_m;
    };

    fetch_cols(0);  // requested together with the union's size
    if (n_union > u_cap || d_v % 8 != 0) {
        per_row_block_call<V, KS, CPL>(row_first, row_last, wave, 8, row_offsets, col_indices, q, k, v, out, d_qk, d_v,
                                       s2, c, g, col_off);
        return;
    }
    const int n_rounds = (n_union + SR - 1) / SR;
    const int q_first = 16 * wave;
    const long long q_global = (long long)row_first * V + q_first;
    const long long q_limit = (long long)row_last * V;
    half8_t qb[KS];
    load_q16<KS>(qb, q, q_global, q_limit, d_qk, c, g);
    if (n_rounds > 0) fetch_rows(0);
    if (n_rounds > 1) fetch_cols(1);
    // The maximum is tracked on raw dot products and masked-out pairs are -inf before the scale is applied, so
    // the scale the exponentials see must be positive: a negative one moves into Q, a zero one becomes Q = 0
    // (every pair of the mask then weighs the same, which is what a zero scale means).
    if (s2 == 0.f) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) qb[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        s2 = 1.f;
    }
    const float s2a = __builtin_fabsf(s2);
    if (s2 < 0.f) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            uint4_t bits = __builtin_bit_cast(uint4_t, qb[kk]);
#pragma unroll
            for (int i = 0; i < 4; ++i) bits[i] ^= 0x80008000u;
            qb[kk] = __builtin_bit_cast(half8_t, bits);
        }
    }
    const unsigned *mrow = maskbuf + ((q_first + c) / V) * SS;
    const half_t *k_lane = kbuf + c * PITCH + 8 * g;
    const float neg_inf = -__builtin_inff();
    constexpr unsigned kLaneBits = 0x000F000Fu;
    const half8_t ones = {1, 1, 1, 1, 1, 1, 1, 1};
    float4_t acc[CPL];
#pragma unroll
    for (int cc = 0; cc < CPL; ++cc) acc[cc] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t lacc = {0.f, 0.f, 0.f, 0.f};
    float mx_run = neg_inf;

    for (int round = 0; round < n_rounds; ++round) {
        if (round > 0) __syncthreads();  // every wave is done with the previous sub-round's rows and masks
        commit(round);
        __syncthreads();
        if (round + 1 < n_rounds) fetch_rows(round + 1);  // in flight during the arithmetic below
        if (round + 2 < n_rounds) fetch_cols(round + 2);
        const int n_here = (n_union - round * SR) < SR ? (n_union - round * SR) : SR;
        const int n_steps = (n_here + 31) >> 5;

        // scores of the sub-round, kept raw, masked-out pairs -inf; their maximum
        float4_t sacc[SS][2];
        unsigned act = 0;
        float mx_raw = neg_inf;
#pragma unroll
        for (int t = 0; t < SS; ++t) {
            sacc[t][0] = sacc[t][1] = float4_t{0.f, 0.f, 0.f, 0.f};
            if (t < n_steps) {
                const unsigned word = mrow[t];
                if (__builtin_amdgcn_ballot_w64(word != 0u) != 0ull) {
                    act |= 1u << t;
                    const unsigned wg = word >> (4 * g);
                    half8_t a[2][KS];
                    load_k_step<KS, PITCH>(a, k_lane, t);
                    if (__builtin_amdgcn_ballot_w64((wg & kLaneBits) != kLaneBits) != 0ull) {
#pragma unroll
                        for (int u = 0; u < 2; ++u)
#pragma unroll
                            for (int e = 0; e < 4; ++e) sacc[t][u][e] = select_bit(wg, 16 * u + e, 0.f, neg_inf);
                    }
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
#pragma unroll
                        for (int kk = 0; kk < KS; ++kk)
                            sacc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][kk], qb[kk], sacc[t][u], 0, 0, 0);
                        mx_raw = fmaxf(fmaxf(mx_raw, fmaxf(sacc[t][u][0], sacc[t][u][1])), fmaxf(sacc[t][u][2], sacc[t][u][3]));
                    }
                }
            }
        }
        act = __builtin_amdgcn_readfirstlane(act);
        mx_raw = fmaxf(mx_raw, partner<16>(mx_raw));  // scalar row c lives in the four lanes (c, g = 0..3)
        mx_raw = fmaxf(mx_raw, partner<32>(mx_raw));
        const float mx_new = fmaxf(mx_run, mx_raw);
        const float neg_mx = mx_new == neg_inf ? 0.f : -(mx_new * s2a);
        if (round > 0) {
            // bring what the earlier sub-rounds accumulated to the new maximum, unless no row's maximum moved
            const float f = mx_new == neg_inf ? 1.f
                            : (mx_run == neg_inf ? 0.f : __builtin_amdgcn_exp2f((mx_run - mx_new) * s2a));
            if (__builtin_amdgcn_ballot_w64(f != 1.f) != 0ull) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float fe = from_lane(f, (4 * g + e) & 15);  // accumulator register e of lane (c, g) is scalar row 4g + e
                    lacc[e] *= fe;
#pragma unroll
                    for (int cc = 0; cc < CPL; ++cc) acc[cc][e] *= fe;
                }
            }
        }
        mx_run = mx_new;

        // probabilities (exp2(-inf) = 0 for masked-out pairs), then P V and the row sums
#pragma unroll
        for (int t = 0; t < SS; ++t) {
            if ((act >> t) & 1u) {
                half8_t p;
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        p[4 * u + e] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf(sacc[t][u][e], s2a, neg_mx));
#pragma unroll
                for (int cc = 0; cc < CPL; ++cc) {
                    const half8_t b = *reinterpret_cast<const half8_t *>(vbuf + stream_v_offset(col_off + cc, 4 * t + g));
                    acc[cc] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p, b, acc[cc], 0, 0, 0);
                }
                lacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(p, ones, lacc, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const long long row = q_global + 4 * g + e;
        if (row < q_limit && col_ok) {
            const float norm = lacc[e] > 0.f ? 1.f / lacc[e] : 0.f;  // a row with no column attends to nothing: zeros
            float tmp[CPL];
#pragma unroll
            for (int cc = 0; cc < CPL; ++cc) tmp[cc] = acc[cc][e] * norm;
            store_converted<half_t, CPL>(out + (size_t)row * d_v + col0, tmp);
        }
    }
}

// 32-bit words of one round of row masks of a workgroup: `rows` vector rows x `steps` words, padded to 16 bytes.
static int union_mask_words(int rows, int steps) { return (rows * steps + 3) & ~3; }

// Launch shape of the union kernels for a request of `rows` vector rows per workgroup.
struct UnionShape {
    int waves;    // 16 scalar rows each
    int rows;     // vector rows per workgroup actually used
    bool stream;  // planned launch of eight waves: the streamed kernel
    int u_max;    // ranks of the union in LDS at once
    int rounds;   // rounds of u_max ranks a workgroup can take (1 unless streamed)
    int steps;    // mask words per vector row and round
    size_t lds;
    size_t plan_lds;  // LDS of the plan kernel for this shape
};

static bool union_shape(UnionShape &s, int vec_length, int n, int d_qk, int d_v, int rows, bool planned)
{
    const int rpw = 16 / vec_length;
    s.waves = ceil_div(rows < 1 ? 1 : rows, rpw);
    if (s.waves > 8) s.waves = 8;
    s.rows = s.waves * rpw;
    s.stream = planned && s.waves == 8;
    const int ks = d_qk <= 32 ? 1 : (d_qk <= 64 ? 2 : 4);
    const int cpl = d_v <= 64 ? 4 : 8;
    const size_t row_bytes = (size_t)union_pitch(ks, cpl) * sizeof(half_t);
    const int n_words = (((n + 31) / 32) + 3) & ~3;
    const size_t bitmaps = 2 * (size_t)n_words * sizeof(unsigned) + 16 * sizeof(int);  // what build_union adds
    if (s.stream) {
        s.u_max = kStreamRanks;
        s.rounds = kStreamRounds;
        s.steps = kStreamSteps;
        const size_t mask = (size_t)union_mask_words(s.rows, s.steps) * sizeof(unsigned);
        // masks of one sub-round, its K rows and its V columns (transposed) side by side
        s.lds = mask + (size_t)s.u_max * (32 * ks + 8) * sizeof(half_t) + (size_t)16 * cpl * kStreamVPitch * sizeof(half_t);
        s.plan_lds = bitmaps + s.rounds * (mask + (size_t)s.u_max * sizeof(int));
        return s.plan_lds <= 160 * 1024;
    }
    // Half of a CU's LDS per workgroup, so that two workgroups overlap each other's memory phases (wide heads:
    // one workgroup per CU, all of it).  With a plan the column bitmap, its prefix sums and the column list
    // stay out of the attention kernel's LDS.
    s.rounds = 1;
    s.steps = kUnionSteps;
    const size_t budget = (union_wide(ks, cpl) ? 152 : (planned ? 80 : 72)) * 1024;
    const size_t mask = (size_t)union_mask_words(s.rows, s.steps) * sizeof(unsigned);
    const size_t fixed = planned ? mask : bitmaps + mask;
    const size_t per_union_row = row_bytes + (planned ? 0 : sizeof(int));
    if (fixed + 32 * per_union_row > budget) return false;  // the column bitmap alone fills the budget
    s.u_max = (int)((budget - fixed) / per_union_row) & ~31;
    if (s.u_max > 32 * kUnionSteps) s.u_max = 32 * kUnionSteps;
    s.lds = fixed + (size_t)s.u_max * per_union_row;
    s.plan_lds = planned ? bitmaps + mask + (size_t)s.u_max * sizeof(int) : 0;
    return s.plan_lds <= 160 * 1024;
}

static bool union_dims_ok(int d_qk, int d_v)
{
    if (d_qk <= 0 || d_qk % 8 != 0 || d_qk > 128) return false;
    if (d_v <= 0 || d_v % 4 != 0 || d_v > 128 || (d_v > 64 && d_v % 8 != 0)) return false;
    return true;
}

struct UnionLaunch {
    int m_vec, n, d_qk, d_v, rows;
    const int *row_offsets, *col_indices, *plan;
    const half_t *q, *k, *v;
    half_t *out;
    float scale;
    hipStream_t stream;
    const Batch *batch;
    long long stride_v;
};

template <int V, int KS, int CPL, bool PLANNED>
static int launch_one(const UnionLaunch &a)
{
    UnionShape s;
    if (!union_shape(s, V, a.n, a.d_qk, a.d_v, a.rows, PLANNED)) return hipErrorNotSupported;
    static std::atomic<unsigned long long> lds_allowed{0}, stream_lds_allowed{0};
    const dim3 grid((unsigned)ceil_div(a.m_vec, s.rows), (unsigned)a.batch->count);
    if (PLANNED && s.stream) {
        auto kernel = sparse_attention_stream_kernel<V, KS, CPL>;
        const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 160 * 1024, stream_lds_allowed);
        if (attr != hipSuccess) return (int)attr;
        hipLaunchKernelGGL(kernel, grid, dim3(512), s.lds, a.stream, a.m_vec, a.n, a.d_qk, a.d_v, a.row_offsets,
                           a.col_indices, a.plan, a.q, a.k, a.v, a.out, a.batch->stride_a, a.batch->stride_b,
                           a.stride_v, a.batch->stride_out, a.scale);
        return (int)hipGetLastError();
    }
    auto kernel = sparse_attention_union_kernel<V, KS, CPL, PLANNED>;
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 160 * 1024, lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(kernel, grid, dim3(64 * s.waves), s.lds, a.stream, a.m_vec, a.n, a.d_qk, a.d_v, s.u_max,
                       a.row_offsets, a.col_indices, a.plan, a.q, a.k, a.v, a.out, a.batch->stride_a,
                       a.batch->stride_b, a.stride_v, a.batch->stride_out, a.scale);
    return (int)hipGetLastError();
}

template <int V, bool PLANNED>
static int launch_shape(const UnionLaunch &a)
{
    if (a.d_v <= 64) {
        if (a.d_qk <= 32) return launch_one<V, 1, 4, PLANNED>(a);
        if (a.d_qk <= 64) return launch_one<V, 2, 4, PLANNED>(a);
        return launch_one<V, 4, 4, PLANNED>(a);
    }
    if (a.d_qk <= 32) return launch_one<V, 1, 8, PLANNED>(a);
    if (a.d_qk <= 64) return launch_one<V, 2, 8, PLANNED>(a);
    return launch_one<V, 4, 8, PLANNED>(a);
}

template <bool PLANNED>
static int launch_v(int vec_length, const UnionLaunch &a)
{
    switch (vec_length) {
    case 1: return launch_shape<1, PLANNED>(a);
    case 2: return launch_shape<2, PLANNED>(a);
    case 4: return launch_shape<4, PLANNED>(a);
    case 8: return launch_shape<8, PLANNED>(a);
    default: return hipErrorInvalidValue;
    }
}

static bool union_supported(int vec_length, int n, int d_qk, int d_v)
{
    if (vec_length != 1 && vec_length != 2 && vec_length != 4 && vec_length != 8) return false;
    return n >= 0 && n <= 1024 * 1024 && union_dims_ok(d_qk, d_v);  // the column bitmap lives in LDS
}

int sparse_attention_union_capacity(int vec_length, int n, int d_qk, int d_v, int rows, bool with_plan, int *rows_used)
{
    UnionShape s;
    if (!union_supported(vec_length, n, d_qk, d_v) || d_v % 8 != 0) return 0;
    if (!union_shape(s, vec_length, n, d_qk, d_v, rows, with_plan)) return 0;
    if (rows_used) *rows_used = s.rows;
    return s.rounds * s.u_max;
}

long long sparse_attention_plan_bytes(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows)
{
    UnionShape s;
    if (m_vec < 0 || !union_supported(vec_length, n, d_qk, d_v)) return 0;
    if (!union_shape(s, vec_length, n, d_qk, d_v, rows, true)) return 0;
    const long long stride = 4 + s.rounds * ((long long)union_mask_words(s.rows, s.steps) + s.u_max);
    return (long long)sizeof(int) * (kPlanHeader + stride * ceil_div(m_vec, s.rows));
}

int launch_sparse_attention_plan(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows, const int *row_offsets,
                                 const int *col_indices, int *plan, long long plan_bytes, hipStream_t stream)
{
    UnionShape s;
    if (!union_supported(vec_length, n, d_qk, d_v)) return hipErrorNotSupported;
    if (!union_shape(s, vec_length, n, d_qk, d_v, rows, true)) return hipErrorNotSupported;
    const long long need = sparse_attention_plan_bytes(m_vec, vec_length, n, d_qk, d_v, rows);
    if (plan_bytes < need) return hipErrorInvalidValue;
    if (m_vec == 0) return hipSuccess;
    static std::atomic<unsigned long long> lds_allowed{0};
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(sparse_attention_plan_kernel), 160 * 1024,
                                            lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(sparse_attention_plan_kernel, dim3((unsigned)ceil_div(m_vec, s.rows)), dim3(256), s.plan_lds,
                       stream, m_vec, vec_length, n, s.rows, s.u_max, s.rounds, s.steps, row_offsets, col_indices, plan);
    return (int)hipGetLastError();
}

int launch_sparse_attention_union(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows, const int *row_offsets,
                                  const int *col_indices, const int *plan, const half_t *q, const half_t *k,
                                  const half_t *v, half_t *out, float scale, hipStream_t stream, const Batch &batch,
                                  long long stride_v)
{
    if (m_vec == 0 || batch.count == 0 || d_v == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (!union_supported(vec_length, n, d_qk, d_v)) return hipErrorNotSupported;
    const UnionLaunch a = {m_vec, n, d_qk, d_v, rows, row_offsets, col_indices, plan, q, k, v, out,
                           scale, stream, &batch, stride_v};
    if (plan) return launch_v<true>(vec_length, a);
    return launch_v<false>(vec_length, a);
}

}  // namespace vs
