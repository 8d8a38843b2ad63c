// Fixed-mask sparse attention for a block of R consecutive vector rows per workgroup, with the K and V
// rows those R rows need gathered ONCE into LDS ("union gather"), and one wave per vector row.
//
// Structured masks (local band, block-diagonal, strided columns) make neighbouring rows share almost all
// of their columns: with a band of 257 columns, 8 consecutive vector rows touch ~345 distinct columns,
// not 8 x 283.  Gathering each row's K / V rows separately (sparse_attention.hip) makes the L2 -> CU
// gather the bound; gathering the union once and serving every row of the block from LDS removes most
// of that traffic.  Random masks have no overlap: when the union does not fit the LDS budget the
// workgroup falls back to gathers from global memory, with the same arithmetic.
//
// Workgroup steps (R <= 8 rows, one wave per row, K and V share ONE LDS buffer so that two workgroups
// fit a CU and one's memory phases overlap the other's arithmetic):
//   1  bitmap of the block's columns in LDS (atomic or), exclusive prefix of its word popcounts:
//      rank(col) = prefix[col / 32] + popcount(bitmap[col / 32] below bit col % 32) is the position of a
//      column in the sorted union; U = total popcount.
//   2  list the union's columns, store the rank of every nonzero of the block (16 bits), copy the K rows
//      of the union to LDS (row-major 128-bit loads, rows padded by 16 bytes against bank conflicts).
//   A  per wave: S^T = K_gathered Q^T on v_mfma_f32_16x16x32_f16 with the gathered K rows as the A
//      operand and the row's Q slices as the B operand: lane (v, g) receives the scores of scalar row v
//      for nonzeros 4g..4g+3 of every 16-vector group.  Run twice: the first pass keeps only the row
//      maximum, the second recomputes the scores (LDS reads and MFMA are cheap, registers are not) and
//      keeps p = exp2(s - max) as packed fp16 plus the row sum.  Statistics of scalar row v combine the
//      four lanes that hold the same v (ds_swizzle xor 16, ds_bpermute xor 32).
//   3  barrier, copy the V rows of the union over the K rows, barrier.
//   C  per wave: P V on the same MFMA with P as the A operand.  The contraction index of an MFMA can be numbered
//      freely as long as both operands agree, so k-slot (g, e) is DEFINED as the nonzero the lane
//      already holds: e < 4 -> nonzero 4g + e of the step's first group, e >= 4 -> nonzero 4g + e - 4 of
//      its second group.  P therefore goes from the score registers into the A operand with no data
//      movement, and the gathered V rows (transposed in registers with v_perm_b32, as in the SpMM
//      kernel) are fetched in that same order.
// Blocks whose union, nonzero count or longest row exceed the LDS / register budget take the fallback.
#include "vs_common.hpp"

namespace vs {

constexpr int kMaxSteps = 10;  // 32-vector steps of a row whose scores are held in registers at once

// Value of `x` held by lane `src_lane` (all lanes active).
__device__ __forceinline__ float from_lane(float x, int src_lane)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, x)));
}

// Where the K / V rows of a block come from.  LDS = true: the workgroup's LDS copy, indexed by the rank
// of a nonzero's column in the union; LDS = false: global memory, indexed by the column itself.
template <bool LDS>
struct RowSource {
    const half_t *base;            // LDS copy (K rows, later V rows) or the global operand
    int pitch;                     // halves between consecutive rows of `base`
    const unsigned short *rkb;     // LDS: rank of nonzero j at rkb[j - nz_first]
    const int *col_indices;        // global: column of nonzero j
    int nz_first;
    __device__ __forceinline__ const half_t *row_of(int j, int end) const
    {
        const int jc = j < end ? j : end - 1;  // slots past the row's end repeat its last vector
        if constexpr (LDS) return base + (size_t)rkb[jc - nz_first] * pitch;
        else return base + (size_t)col_indices[jc] * pitch;
    }
};

// Scores of the 64 nonzeros [j0, j0 + 64) of a row against the row's Q slices.
// out[u][e]: group u (16 vectors), register e -> nonzero j0 + 16u + 4g + e, base-2 units, -inf past `end`.
template <int KS, bool LDS>
__device__ __forceinline__ void scores64(float (&out)[4][4], const RowSource<LDS> &ksrc, int j0, int end, int d_qk,
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
template <int KS, bool LDS>
__device__ __forceinline__ void softmax_chunk(half8_t (&p)[kMaxSteps], float &mx, float &sum, float m_floor,
                                              const RowSource<LDS> &ksrc, int c0, int cend, int d_qk,
                                              const half8_t (&qb)[KS], float s2, int c, int g)
{
    const int n_steps = (cend - c0 + 31) >> 5;
    mx = m_floor;
#pragma unroll
    for (int ss = 0; ss < kMaxSteps / 2; ++ss) {
        if (2 * ss < n_steps) {
            float sc[4][4];
            scores64<KS, LDS>(sc, ksrc, c0 + 64 * ss, cend, d_qk, qb, s2, c, g);
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
            scores64<KS, LDS>(sc, ksrc, c0 + 64 * ss, cend, d_qk, qb, s2, c, g);
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
template <int CPL, bool LDS>
__device__ __forceinline__ void accumulate_chunk(float4_t (&acc)[CPL], const half8_t (&p)[kMaxSteps],
                                                 const RowSource<LDS> &vsrc, int c0, int cend, int col_off, int g)
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

// V: vector length; KS: d_qk <= 32*KS; CPL: d_v <= 16*CPL.
template <int V, int KS, int CPL>
// four waves per SIMD: two eight-wave workgroups per CU
__global__ void __launch_bounds__(512, 4)
sparse_attention_union_kernel(int m_vec, int n, int d_qk, int d_v, int rows_per_block, int u_max, int rk_cap,
                              const int *__restrict__ row_offsets, const int *__restrict__ col_indices,
                              const half_t *__restrict__ q, const half_t *__restrict__ k,
                              const half_t *__restrict__ v, half_t *__restrict__ out, long long stride_q,
                              long long stride_k, long long stride_v, long long stride_out, float scale)
{
    q += blockIdx.y * stride_q;
    k += blockIdx.y * stride_k;
    v += blockIdx.y * stride_v;
    out += blockIdx.y * stride_out;
    const int n_words = (n + 31) >> 5;
    const int n_words_al = (n_words + 3) & ~3;  // keeps the arrays behind the bitmap 16-byte aligned
    const int pitch = (d_qk > d_v ? d_qk : d_v) + 8;  // halves; +16 bytes: consecutive ranks start 4 banks apart

    extern __shared__ __align__(16) unsigned char smem[];
    unsigned *bitmap = reinterpret_cast<unsigned *>(smem);
    unsigned *prefix = bitmap + n_words_al;                                // [n_words] exclusive popcount prefix
    int *wave_tot = reinterpret_cast<int *>(prefix + n_words_al);          // [16]: scan scratch, [14] longest row, [15] U
    half_t *buf = reinterpret_cast<half_t *>(wave_tot + 16);               // [u_max][pitch]: K rows, later V rows
    int *ucols = reinterpret_cast<int *>(buf + (size_t)u_max * pitch);     // [u_max] columns of the union
    unsigned short *rkb = reinterpret_cast<unsigned short *>(ucols + u_max);  // [rk_cap] rank of each nonzero

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: row bounds stay in scalar registers
    const int n_waves = blockDim.x >> 6;
    const int n_threads = blockDim.x;
    const int row_first = blockIdx.x * rows_per_block;
    const int row_last = (row_first + rows_per_block) < m_vec ? (row_first + rows_per_block) : m_vec;
    const int c = lane & 15;
    const int g = lane >> 4;
    const float s2 = scale * kLog2e;
    const int col0 = c * CPL;
    const bool col_ok = col0 < d_v;
    const int col_off = col_ok ? col0 : 0;

    // ---- 1. bitmap and rank prefix of the block's columns, longest row of the block
    for (int w = tid; w < n_words; w += n_threads) bitmap[w] = 0u;
    if (tid == 0) wave_tot[14] = 0;
    __syncthreads();
    const int nz_first = row_offsets[row_first];
    const int nz_last = row_offsets[row_last];
    if (row_first + tid < row_last) atomicMax(&wave_tot[14], row_offsets[row_first + tid + 1] - row_offsets[row_first + tid]);
    // Every thread keeps up to kOwn of the block's column indices in registers (all loads in flight at
    // once, reused for the ranks below); blocks with more nonzeros than that take the fallback.
    constexpr int kOwn = 8;
    int own_col[kOwn];
#pragma unroll
    for (int i = 0; i < kOwn; ++i) {
        const int j = nz_first + tid + i * n_threads;
        own_col[i] = j < nz_last ? col_indices[j] : -1;
    }
#pragma unroll
    for (int i = 0; i < kOwn; ++i)
        if (own_col[i] >= 0) atomicOr(&bitmap[own_col[i] >> 5], 1u << (own_col[i] & 31));
    for (int j = nz_first + tid + kOwn * n_threads; j < nz_last; j += n_threads) {
        const int col = col_indices[j];
        atomicOr(&bitmap[col >> 5], 1u << (col & 31));
    }
    __syncthreads();
    {
        // exclusive prefix of popcounts: every thread takes a contiguous run of words, the per-thread
        // totals are scanned inside each wave and the wave totals added up
        const int per = (n_words + n_threads - 1) / n_threads;
        const int w0 = tid * per;
        int local = 0;
        for (int w = w0; w < w0 + per && w < n_words; ++w) local += __builtin_popcount(bitmap[w]);
        int incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __builtin_amdgcn_ds_bpermute(((lane - d) & 63) << 2, incl);
            if (lane >= d) incl += up;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int base = 0;
        for (int w = 0; w < wave; ++w) base += wave_tot[w];
        int run = base + incl - local;
        for (int w = w0; w < w0 + per && w < n_words; ++w) {
            prefix[w] = (unsigned)run;
            run += __builtin_popcount(bitmap[w]);
        }
        if (tid == n_threads - 1) wave_tot[15] = run;
        __syncthreads();
    }
    const int n_union = wave_tot[15];
    const int nz_block = nz_last - nz_first;
    const bool use_lds = n_union <= u_max && n_union < 65536 && nz_block <= rk_cap && nz_block <= kOwn * n_threads &&
                         wave_tot[14] <= 32 * kMaxSteps && (row_last - row_first) <= n_waves && (d_v % 8 == 0);
    if (!use_lds) {
        // Fallback: same arithmetic with the K / V rows read from global memory by column; no barrier, so
        // every wave walks its rows on its own, long rows in chunks with a running maximum and sum.
        const RowSource<false> ksrc = {k, d_qk, nullptr, col_indices, nz_first};
        const RowSource<false> vsrc = {v, d_v, nullptr, col_indices, nz_first};
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
                softmax_chunk<KS, false>(p, m_new, sum, m_run, ksrc, c0, cend, d_qk, qb, s2, c, g);
                const float f = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first chunk (m_run = -inf)
                l_run = l_run * f + sum;
                m_run = m_new;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float fe = from_lane(f, (4 * g + e) & 15);  // accumulator row 4g + e belongs to scalar row 4g + e
#pragma unroll
                    for (int cc = 0; cc < CPL; ++cc) acc[cc][e] *= fe;
                }
                accumulate_chunk<CPL, false>(acc, p, vsrc, c0, cend, col_off, g);
            }
            store_row<V, CPL>(out, row, d_v, acc, l_run, end == beg, c, g);
        }
        return;
    }

    // ---- 2. the union's columns, the rank of every nonzero, the K rows of the union
    for (int w = tid; w < n_words; w += n_threads) {
        unsigned bits = bitmap[w];
        int pos = (int)prefix[w];
        while (bits) {
            const int b = __builtin_ctz(bits);
            ucols[pos++] = (w << 5) + b;
            bits &= bits - 1;
        }
    }
#pragma unroll
    for (int i = 0; i < kOwn; ++i) {
        if (own_col[i] >= 0) {
            const int col = own_col[i];
            const unsigned word = bitmap[col >> 5];
            rkb[tid + i * n_threads] =
                (unsigned short)(prefix[col >> 5] + __builtin_popcount(word & ((1u << (col & 31)) - 1u)));
        }
    }
    __syncthreads();
    // copy one operand's rows of the union into buf: 16 bytes per thread and slice, kBatch slices in flight
    auto gather = [&](const half_t *src, int d) {
        constexpr int kBatch = 8;
        const int slices = d >> 3;
        const int total = n_union * slices;
        for (int s0 = tid; s0 < total; s0 += kBatch * n_threads) {
            uint4_t data[kBatch];
            int dst[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int sidx = s0 + i * n_threads;
                dst[i] = -1;
                if (sidx < total) {
                    const int u = sidx / slices, sl = sidx - u * slices;
                    data[i] = *reinterpret_cast<const uint4_t *>(src + (size_t)ucols[u] * d + 8 * sl);
                    dst[i] = u * pitch + 8 * sl;
                }
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i)
                if (dst[i] >= 0) *reinterpret_cast<uint4_t *>(buf + dst[i]) = data[i];
        }
    };
    gather(k, d_qk);
    __syncthreads();

    // ---- A. one wave per vector row: maximum, then exponentials (packed fp16) and their sum
    const int row = row_first + wave;
    const bool has_row = row < row_last;
    const int beg = has_row ? row_offsets[row] : 0;
    const int end = has_row ? row_offsets[row + 1] : 0;
    const RowSource<true> src = {buf, pitch, rkb, nullptr, nz_first};  // K rows now, V rows after step 3
    half8_t p[kMaxSteps];
    float l_sum = 0.f;
    if (end > beg) {
        half8_t qb[KS];
        load_q<V, KS>(qb, q, row, d_qk, c, g);
        float mx;
        softmax_chunk<KS, true>(p, mx, l_sum, -__builtin_inff(), src, beg, end, d_qk, qb, s2, c, g);
    }

    // ---- 3. V rows of the union over the K rows
    __syncthreads();
    gather(v, d_v);
    __syncthreads();

    // ---- C. P V, normalise, store (one wave owns the whole row: nothing to reduce)
    if (!has_row) return;
    float4_t acc[CPL];
#pragma unroll
    for (int cc = 0; cc < CPL; ++cc) acc[cc] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (end > beg) accumulate_chunk<CPL, true>(acc, p, src, beg, end, col_off, g);
    store_row<V, CPL>(out, row, d_v, acc, l_sum, end == beg, c, g);
}

template <int V, int KS, int CPL>
static int launch_one(int m_vec, int n, int d_qk, int d_v, int rows, const int *row_offsets, const int *col_indices,
                      const half_t *q, const half_t *k, const half_t *v, half_t *out, float scale,
                      hipStream_t stream, const Batch &batch, long long stride_v)
{
    // Half of a CU's LDS per workgroup, so that two workgroups overlap each other's memory phases.
    constexpr size_t kLdsBudget = 72 * 1024;
    const int waves = 8;
    if (rows > waves) rows = waves;  // one wave per row
    if (rows < 1) rows = 1;
    const int n_words = (((n + 31) / 32) + 3) & ~3;
    const size_t fixed = 2 * (size_t)n_words * sizeof(unsigned) + 16 * sizeof(int);
    const int rk_cap = rows * 32 * kMaxSteps;  // ranks of the block's nonzeros, 16 bits each
    if (fixed + (size_t)rk_cap * 2 + 16 * 1024 > kLdsBudget) return hipErrorNotSupported;
    const int pitch = (d_qk > d_v ? d_qk : d_v) + 8;
    const size_t per_union_row = (size_t)pitch * sizeof(half_t) + sizeof(int);
    int u_max = (int)((kLdsBudget - fixed - (size_t)rk_cap * 2 - 64) / per_union_row);
    u_max &= ~7;
    const size_t lds = fixed + (size_t)rk_cap * 2 + (size_t)u_max * per_union_row;
    auto kernel = sparse_attention_union_kernel<V, KS, CPL>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess) return (int)attr;
    const int blocks = ceil_div(m_vec, rows);
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * waves), lds, stream, m_vec, n,
                       d_qk, d_v, rows, u_max, rk_cap, row_offsets, col_indices, q, k, v, out, batch.stride_a,
                       batch.stride_b, stride_v, batch.stride_out, scale);
    return (int)hipGetLastError();
}

template <int V>
static int launch_shape(int m_vec, int n, int d_qk, int d_v, int rows, const int *row_offsets, const int *col_indices,
                        const half_t *q, const half_t *k, const half_t *v, half_t *out, float scale,
                        hipStream_t stream, const Batch &batch, long long stride_v)
{
#define VS_ATT(KS, CPL) \
    return launch_one<V, KS, CPL>(m_vec, n, d_qk, d_v, rows, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v)
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

int launch_sparse_attention_union(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows, const int *row_offsets,
                                  const int *col_indices, const half_t *q, const half_t *k, const half_t *v,
                                  half_t *out, float scale, hipStream_t stream, const Batch &batch,
                                  long long stride_v)
{
    if (m_vec == 0 || batch.count == 0 || d_v == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (d_qk <= 0 || d_qk % 8 != 0 || d_qk > 128) return hipErrorNotSupported;
    if (d_v % 4 != 0 || d_v > 128 || (d_v > 64 && d_v % 8 != 0)) return hipErrorNotSupported;
    if (n > 1024 * 1024) return hipErrorNotSupported;  // the column bitmap lives in LDS
    switch (vec_length) {
    case 1: return launch_shape<1>(m_vec, n, d_qk, d_v, rows, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    case 2: return launch_shape<2>(m_vec, n, d_qk, d_v, rows, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    case 4: return launch_shape<4>(m_vec, n, d_qk, d_v, rows, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    case 8: return launch_shape<8>(m_vec, n, d_qk, d_v, rows, row_offsets, col_indices, q, k, v, out, scale, stream, batch, stride_v);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace vs
