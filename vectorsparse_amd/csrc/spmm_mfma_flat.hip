// SpMM on fp16 MFMA with the work split along the NONZERO range instead of the rows, for patterns whose row
// lengths are skewed (the reference only reorders the dispatch of whole rows, include/bm_test_utils.h:200-215;
// here a row that is far longer than the rest is shared by many waves on many CUs).
//
// The CSR arrays are cut into runs of `sub` nonzero vectors (a multiple of 32).  One wave owns (run, tile of 16*CPL
// dense columns); a workgroup of W waves owns W consecutive runs (a piece of P = W*sub vectors) of one tile.  A wave
// walks the row segments inside its run - a row that crosses a run boundary is cut there - so every wave has `sub`
// vectors of work whatever the row lengths are.  A segment that is a whole row is written to the output from the
// accumulators.  The other segments are summed in two levels, both in ascending order of the nonzeros, so the
// result does not depend on timing and no atomics touch the output:
//   * inside a workgroup through LDS: a wave parks the partial tile of a row that started before its run in its
//     slot F[w]; the wave in whose run a row starts keeps that segment in its accumulators and, after the one
//     barrier, adds the slots F[w+1], F[w+2], ... of the runs the row covers;
//   * across workgroups through the workspace: the part of a row that a piece holds goes to slot T[c] (the row
//     starts inside piece c) or F[c] (it started earlier), fp32.  A row that starts in piece c0 and ends in piece c1
//     has c1 - c0 + 1 parts, added as T[c0] + F[c0+1] + ... + F[c1] in one of two ways:
//     ONE_LAUNCH (default): every wave that has written a part counts itself in on the row's arrival counter (the
//     one of piece c0: at most one row starts in a piece and leaves it) and the wave that arrives last adds the
//     parts, writes the output rows and puts the counter back to zero.  Nobody waits for anybody and the sum is
//     the same whoever arrives last.  How the parts reach the wave that adds them: PartMeeting in
//     spmm_mfma_step.hpp (buffer accesses with the device-coherence bits set, tracked by the compiler; the same
//     accesses as inline assembly lost their data registers to reuse before the stores had read them).
//     Two launches: a second launch adds the parts; 1.5 to 2.5 us slower, no counters, and the route taken when
//     the tiles would not fit 32-bit buffer offsets.
// The zero rows of empty vector rows, which no wave's walk visits, are written by extra workgroups at the end of
// the grid (ONE_LAUNCH) or by the second launch (writing them from the walk costs the tile loop 24 registers and
// with them its occupancy).
// The arithmetic of a step is the row-per-workgroup kernel's (spmm_mfma_step).  row_indices is not needed.
#include "spmm_mfma_step.hpp"
#include "vs_common.hpp"

namespace vs {

// Accumulator layout <-> [v][column] tile of fp32: lane (cs, g), register e of acc[c] is row 4g + e, column cs*CPL + c.
// `p`: which group of V accumulator rows holds the vector row (rows p*V .. p*V + V - 1; 0 unless steps are shared).
template <int V, int CPL>
__device__ __forceinline__ void tile_store(float *tile_base, int pitch, int cs, int g, const float4_t (&acc)[CPL],
                                           int p = 0)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e - p * V;
        if (v >= 0 && v < V) {
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                float4_t t = {acc[4 * c4][e], acc[4 * c4 + 1][e], acc[4 * c4 + 2][e], acc[4 * c4 + 3][e]};
                *reinterpret_cast<float4_t *>(tile_base + (size_t)v * pitch + cs * CPL + 4 * c4) = t;
            }
        }
    }
}

template <int V, int CPL>
__device__ __forceinline__ void tile_add(const float *tile_base, int pitch, int cs, int g, float4_t (&acc)[CPL],
                                         int p = 0)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e - p * V;
        if (v >= 0 && v < V) {
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                const float4_t t = *reinterpret_cast<const float4_t *>(tile_base + (size_t)v * pitch + cs * CPL + 4 * c4);
                acc[4 * c4][e] += t[0];
                acc[4 * c4 + 1][e] += t[1];
                acc[4 * c4 + 2][e] += t[2];
                acc[4 * c4 + 3][e] += t[3];
            }
        }
    }
}

// The same two for tiles in the workspace that waves on other CUs - and other XCDs, whose L2 is a different one -
// read within the same launch: 128-bit buffer stores and loads with the device-coherence bits of the cache policy
// set (sc0 sc1: written through to memory, read past the caches), so that no cache-wide write-back or invalidate
// is needed around the arrival counter.  `tiles` is a buffer descriptor over the tile area of the workspace
// (below 2^31 bytes), offsets are in bytes.
template <int V, int CPL>
__device__ __forceinline__ void tile_store_coherent(__amdgpu_buffer_rsrc_t tiles, uint32_t tile_bytes, int pitch, int cs,
                                                    int g, const float4_t (&acc)[CPL], int p = 0)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e - p * V;
        if (v >= 0 && v < V) {
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                const float4_t t = {acc[4 * c4][e], acc[4 * c4 + 1][e], acc[4 * c4 + 2][e], acc[4 * c4 + 3][e]};
                PartMeeting::store_part(tiles, tile_bytes + 4u * (uint32_t)(v * pitch + cs * CPL + 4 * c4), t);
            }
        }
    }
}

// adds the lane's part of a tile (rows 4g..4g+3 below V, its CPL columns) to acc
template <int V, int CPL>
__device__ __forceinline__ void tile_add_coherent(__amdgpu_buffer_rsrc_t tiles, uint32_t tile_bytes, int pitch, int cs,
                                                  int g, float4_t (&acc)[CPL])
{
    float4_t part[4][CPL / 4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e;
#pragma unroll
        for (int c4 = 0; c4 < CPL / 4; ++c4) {
            part[e][c4] = float4_t{0.f, 0.f, 0.f, 0.f};
            if (v < V)
                part[e][c4] = PartMeeting::load_part(tiles, tile_bytes + 4u * (uint32_t)(v * pitch + cs * CPL + 4 * c4));
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int c4 = 0; c4 < CPL / 4; ++c4) {
            acc[4 * c4][e] += part[e][c4][0];
            acc[4 * c4 + 1][e] += part[e][c4][1];
            acc[4 * c4 + 2][e] += part[e][c4][2];
            acc[4 * c4 + 3][e] += part[e][c4][3];
        }
}

// The lane's CPL outputs of the V scalar rows of vector row `row`, converted and stored.
template <int V, int CPL, typename OutT>
__device__ __forceinline__ void tile_to_output(OutT *out, int row, int n_cols, int col0, bool col_ok, int g,
                                               const float4_t (&acc)[CPL], int p = 0)
{
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e - p * V;
        if (v >= 0 && v < V && col_ok) {
            float tmp[CPL];
#pragma unroll
            for (int q = 0; q < CPL; ++q) tmp[q] = acc[q][e];
            store_converted<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col0, tmp);
        }
    }
}

// ONE_LAUNCH: the parts of rows that cross workgroups are added inside this launch by whichever wave brings a
// row's last part (arrival counters at the start of the workspace, which every launch leaves at zero), and the
// workgroups past `main_blocks` write the zero rows of empty vector rows; there is no second launch.
// SHARED: a 32-vector step takes the next 32 nonzeros of the run whatever rows they belong to, as far as they lie
// in 16 / V consecutive vector rows: row r uses the V accumulator rows of group r % (16 / V), the MFMA's sparse
// operand holds every row's values in its own group of rows and zeros elsewhere, and a row's group is written out
// (or parked, for a row that started before the run) and cleared after the step in which the row ends.  A run
// then takes sub / 32 steps however short its rows are; without it every row segment starts a step of its own.
template <int V, int CPL, bool IDX32, bool ONE_LAUNCH, typename OutT, bool SHARED = false>
__global__ void __launch_bounds__(1024)
spmm_mfma_flat_kernel(int m_vec, int n_cols, int n_tiles, int nonzeros_vec, int sub, int main_blocks, int *counters,
                      const int *__restrict__ row_offsets, const int *__restrict__ column_indices,
                      const half_t *__restrict__ values, const half_t *__restrict__ rhs, OutT *__restrict__ out,
                      float *__restrict__ ws_base, int ws_pitch)
{
    constexpr int TN = 16 * CPL;
    constexpr int kStage = stage_bytes<V>();
    extern __shared__ __align__(16) unsigned char smem[];  // [W] staging slots, then [W] F tiles of V x TN fp32
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    if constexpr (ONE_LAUNCH) {
        if ((int)blockIdx.x >= main_blocks) {  // four vector rows per wave: zeros for the empty ones
            const int first = (((int)blockIdx.x - main_blocks) * n_waves + wave) * 4;
            const int quads = n_cols >> 2;  // n_cols % 4 == 0
            for (int row = first; row < first + 4 && row < m_vec; ++row) {
                if (row_offsets[row + 1] != row_offsets[row]) continue;
                const float zeros[4] = {0.f, 0.f, 0.f, 0.f};
                for (int item = lane; item < V * quads; item += 64)
                    store_converted<OutT, 4>(out + (size_t)row * V * n_cols + 4 * (size_t)item, zeros);
            }
            return;
        }
    }
    const int tile = blockIdx.x % n_tiles;
    const int c = blockIdx.x / n_tiles;  // piece
    const long long piece = (long long)n_waves * sub;
    const long long cb = c * piece;
    const long long ce = cb + piece;
    const long long sb_ll = cb + (long long)wave * sub;
    const int cs = lane & 15;
    const int g = lane >> 4;
    const int col0 = tile * TN + cs * CPL;
    const bool col_ok = col0 < n_cols;  // n_cols % CPL == 0: a lane's chunk is all in or all out
    const uint32_t col_off = col_ok ? col0 : 0;
    int *idx_s = reinterpret_cast<int *>(smem + (size_t)wave * kStage);
    half_t *vec_s = reinterpret_cast<half_t *>(idx_s + kStep);  // [V][kStep]
    float *f_tiles = reinterpret_cast<float *>(smem + (size_t)n_waves * kStage);
    float *f_mine = f_tiles + (size_t)wave * V * TN;
    float *ws = ws_base + tile * TN;
    const size_t ws_tile = (size_t)V * ws_pitch;  // floats per workspace tile; piece c: F at 2c, T at 2c + 1

    float4_t acc[CPL];
#pragma unroll
    for (int q = 0; q < CPL; ++q) acc[q] = float4_t{0.f, 0.f, 0.f, 0.f};
    bool has_t = false;   // the accumulators hold the first segment of a row that goes on past this run
    bool has_f = false;   // this run starts inside a row (its partial tile is in F[wave])
    int t_row = 0, t_row_end = 0, f_row = 0, f_row_beg = 0, f_row_end = 0;
    int t_pos = 0;        // SHARED: the group of accumulator rows that holds the row that goes on

    if (sb_ll < nonzeros_vec) {
        const int sb = (int)sb_ll;
        const int se = sb + sub < nonzeros_vec ? sb + sub : nonzeros_vec;
        int next_idx = 0;
        half_t next_vec[V];
#pragma unroll
        for (int v = 0; v < V; ++v) next_vec[v] = (half_t)0.f;
        // column index and vector of slot `lane` of the step that starts at nonzero `pos`; which of the 32 slots
        // belong to the segment is decided when the step is staged
        auto fetch = [&](int pos) {
            if (lane < kStep) {
                const int j = pos + lane < nonzeros_vec ? pos + lane : nonzeros_vec - 1;
                next_idx = column_indices[j];
                load_vector<V>(next_vec, values + (size_t)j * V);
            }
        };
        fetch(sb);  // the segments of a run follow each other without gaps from sb to se, whatever the rows are
        // offsets window: lane l holds row_offsets[base_row + l], so row base_row + i, i < 63, runs from lane i to
        // lane i + 1; the search leaves the window that holds the row of nonzero sb
        int base_row, ri;
        int offs = find_row_window(row_offsets, m_vec, sb, lane, base_row, ri);

        if constexpr (SHARED) {
            constexpr int R = 16 / V;                // vector rows that can share a step
            constexpr int PPL = V >= 4 ? 1 : 4 / V;  // row groups among a lane's four accumulator rows
            constexpr int EPP = 4 / PPL;             // accumulator rows per group and lane
            // ri = window lane of the row that holds nonzero `pos` (equal offsets, i.e. empty rows, are passed);
            // the window moves on until that row and the R - 1 after it have both their ends in it
            auto settle = [&](int pos) {
                for (;;) {
                    ri = __builtin_popcountll(__builtin_amdgcn_ballot_w64(offs <= pos)) - 1;
                    if (ri + R <= 62) break;
                    base_row += ri;
                    const int idx = base_row + lane;
                    offs = idx <= m_vec ? row_offsets[idx] : 0x7fffffff;
                }
            };
            settle(sb);
            {
                const int row0_beg = __builtin_amdgcn_readlane(offs, ri);
                if (row0_beg < sb) {  // the run starts inside a row
                    has_f = true;
                    f_row = base_row + ri;
                    f_row_beg = row0_beg;
                    f_row_end = __builtin_amdgcn_readlane(offs, ri + 1);
                }
            }
            int base = sb;
            while (base < se) {
                settle(base);
                const int r0 = base_row + ri;
                const int limit = __builtin_amdgcn_readlane(offs, ri + R);  // where row r0 + R starts
                int count = se - base < kStep ? se - base : kStep;
                count = limit - base < count ? limit - base : count;
                // slots >= count repeat the step's last column (in bounds) with a zero value
                const int last_idx = __builtin_amdgcn_readlane(next_idx, count - 1);
                if (lane < kStep) {
                    const bool valid = lane < count;
                    idx_s[lane] = valid ? next_idx : last_idx;
#pragma unroll
                    for (int v = 0; v < V; ++v) vec_s[v * kStep + lane] = valid ? next_vec[v] : (half_t)0.f;
                }
                wave_lds_fence();
                // MFMA row cs belongs to the vector row of group cs / V among r0 .. r0 + R - 1: its slots
                const int a_lane = ri + (((cs / V) - r0) & (R - 1));
                const int a_beg = __builtin_amdgcn_ds_bpermute(a_lane << 2, offs) - base;
                const int a_end = __builtin_amdgcn_ds_bpermute((a_lane + 1) << 2, offs) - base;
                const int step_end = base + count;
                spmm_mfma_step_shared<V, CPL, IDX32>(idx_s, vec_s, rhs, n_cols, col_off, cs, g, acc,
                                                     a_beg > 0 ? a_beg : 0, a_end < count ? a_end : count, [&] {
                                                         if (step_end < se) fetch(step_end);
                                                     });
                // rows that end inside the step leave the accumulators (the first row of the step ends first)
                if (__builtin_amdgcn_readlane(offs, ri + 1) <= step_end) {
#pragma unroll
                    for (int i = 0; i < PPL; ++i) {
                        const int grp = (4 * g + i * EPP) / V;
                        const int w_lane = ri + ((grp - r0) & (R - 1));
                        const int row = base_row + w_lane;
                        const int rb = __builtin_amdgcn_ds_bpermute(w_lane << 2, offs);
                        const int re = __builtin_amdgcn_ds_bpermute((w_lane + 1) << 2, offs);
                        if (re > base && re <= step_end) {
                            if (rb >= sb)  // the whole row lies in this run
                                tile_to_output<V, CPL, OutT>(out, row, n_cols, col0, col_ok, g, acc, grp);
                            else           // it started in an earlier run: its part goes to F[wave]
                                tile_store<V, CPL>(f_mine, TN, cs, g, acc, grp);
#pragma unroll
                            for (int e = i * EPP; e < (i + 1) * EPP; ++e)
#pragma unroll
                                for (int q = 0; q < CPL; ++q) acc[q][e] = 0.f;
                        }
                    }
                }
                base = step_end;
            }
            // the row that goes on past the run, if any: its group stays in the accumulators (it starts here) or
            // goes to F[wave] (it started earlier and covers the whole run)
            const int li = __builtin_popcountll(__builtin_amdgcn_ballot_w64(offs <= se - 1)) - 1;
            const int l_end = __builtin_amdgcn_readlane(offs, li + 1);
            if (l_end > se && l_end != 0x7fffffff) {
                const int l_row = base_row + li;
                const int grp = l_row & (R - 1);
                if (__builtin_amdgcn_readlane(offs, li) >= sb) {
                    has_t = true;
                    t_row = l_row;
                    t_row_end = l_end;
                    t_pos = grp;
                } else {
                    tile_store<V, CPL>(f_mine, TN, cs, g, acc, grp);
                }
            }
        } else
        for (;;) {
            if (ri == 63) {
                base_row += 63;
                ri = 0;
                if (base_row >= m_vec) break;
                offs = row_offsets[base_row + lane <= m_vec ? base_row + lane : m_vec];
            }
            const int row = base_row + ri;
            if (row >= m_vec) break;  // also when nonzeros_vec exceeds row_offsets[m_vec]: nothing of the pattern is here
            const int row_beg = __builtin_amdgcn_readlane(offs, ri);
            const int row_end = __builtin_amdgcn_readlane(offs, ri + 1);
            if (row_beg >= se) break;  // rows that start at or after the run's end belong to later runs
            ++ri;
            if (row_end == row_beg) continue;  // empty: the second launch writes its zeros
            const int seg_beg = row_beg > sb ? row_beg : sb;
            const int seg_end = row_end < se ? row_end : se;

            for (int base = seg_beg; base < seg_end; base += kStep) {
                const int count = seg_end - base;  // slots >= count are past the segment
                // their gathers repeat the segment's last column (in bounds, and a column the row really has) with
                // a zero value, so they contribute nothing
                const int last_idx = __builtin_amdgcn_readlane(next_idx, count < kStep ? count - 1 : kStep - 1);
                if (lane < kStep) {
                    const bool valid = lane < count;
                    idx_s[lane] = valid ? next_idx : last_idx;
#pragma unroll
                    for (int v = 0; v < V; ++v) vec_s[v * kStep + lane] = valid ? next_vec[v] : (half_t)0.f;
                }
                wave_lds_fence();
                // the next step starts where this one ends: inside the segment, or at the first nonzero of the
                // next row (CSR rows are contiguous)
                const int next_pos = base + kStep < seg_end ? base + kStep : seg_end;
                spmm_mfma_step<V, CPL, IDX32>(idx_s, vec_s, rhs, n_cols, col_off, cs, g, acc, [&] {
                    if (next_pos < se) fetch(next_pos);
                });
            }

            if (row_beg >= sb && row_end <= se) {  // a whole row
                tile_to_output<V, CPL, OutT>(out, row, n_cols, col0, col_ok, g, acc);
            } else if (row_beg < sb) {  // started in an earlier run (and may go on past this one)
                tile_store<V, CPL>(f_mine, TN, cs, g, acc);
                has_f = true;
                f_row = row;
                f_row_beg = row_beg;
                f_row_end = row_end;
            } else {  // starts here and goes on: the run's last segment, kept in the accumulators
                has_t = true;
                t_row = row;
                t_row_end = row_end;
                break;
            }
#pragma unroll
            for (int q = 0; q < CPL; ++q) acc[q] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
    }
    __syncthreads();

    // Parts of rows that leave the piece go to the workspace.  ONE_LAUNCH: `pending` = this wave has written one and
    // counts itself in on the row's counter (the counter of the piece the row starts in; at most one row starts
    // in a piece and leaves it).
    bool pending = false;
    int p_row = 0, p_first = 0, p_last = 0;  // the row, the piece it starts in, the piece it ends in
    if (has_t) {
        const long long stop = t_row_end < ce ? t_row_end : ce;
        const int last = (int)((stop - 1 - cb) / sub);  // the last run of this piece that holds nonzeros of the row
        for (int w = wave + 1; w <= last; ++w) tile_add<V, CPL>(f_tiles + (size_t)w * V * TN, TN, cs, g, acc, t_pos);
        if (t_row_end <= ce) {  // the row ends inside the piece: this is all of it
            tile_to_output<V, CPL, OutT>(out, t_row, n_cols, col0, col_ok, g, acc, t_pos);
        } else if constexpr (ONE_LAUNCH) {
            tile_store_coherent<V, CPL>(PartMeeting::area(ws_base), (uint32_t)(((size_t)2 * c + 1) * ws_tile + tile * TN) * 4u, ws_pitch,
                                        cs, g, acc, t_pos);
            pending = true;
            p_row = t_row;
            p_first = c;
            // (a row that row_offsets lets end past nonzeros_vec - an inconsistent call - has no parts beyond the last
            // launched piece: counting only those that exist leaves the counter at zero whatever the caller passed)
            p_last = (int)(((t_row_end < nonzeros_vec ? t_row_end : (long long)nonzeros_vec) - 1) / piece);
        } else {
            tile_store<V, CPL>(ws + ((size_t)2 * c + 1) * ws_tile, ws_pitch, cs, g, acc, t_pos);
        }
    }
    for (int round = 0; round < 2; ++round) {
        if (round == 1) {
            // the piece starts inside a row: its part of that row goes to F[c] (wave 0, after its own T part)
            pending = false;
            if (wave == 0 && has_f) {
                float4_t sum[CPL];
#pragma unroll
                for (int q = 0; q < CPL; ++q) sum[q] = float4_t{0.f, 0.f, 0.f, 0.f};
                const long long stop = f_row_end < ce ? f_row_end : ce;
                const int last = (int)((stop - 1 - cb) / sub);
                for (int w = 0; w <= last; ++w) tile_add<V, CPL>(f_tiles + (size_t)w * V * TN, TN, cs, g, sum);
                if constexpr (ONE_LAUNCH) {
                    tile_store_coherent<V, CPL>(PartMeeting::area(ws_base), (uint32_t)((size_t)2 * c * ws_tile + tile * TN) * 4u, ws_pitch,
                                                cs, g, sum);
                    pending = true;
                    p_row = f_row;
                    p_first = (int)(f_row_beg / piece);
                    p_last = (int)(((f_row_end < nonzeros_vec ? f_row_end : (long long)nonzeros_vec) - 1) / piece);
                } else {
                    tile_store<V, CPL>(ws + (size_t)2 * c * ws_tile, ws_pitch, cs, g, sum);
                }
            }
        }
        if constexpr (ONE_LAUNCH) {
            if (!pending) continue;
            int *counter = counters + (size_t)p_first * n_tiles + tile;
            PartMeeting::publish();
            if (PartMeeting::arrive(counter, lane) != p_last - p_first) continue;  // parts are still to come: whoever brings the last adds up
            PartMeeting::collect();
            float4_t total[CPL];
#pragma unroll
            for (int q = 0; q < CPL; ++q) total[q] = float4_t{0.f, 0.f, 0.f, 0.f};
            // T of the first piece, then F of the others, in ascending order
            for (int pc = p_first; pc <= p_last; ++pc)
                tile_add_coherent<V, CPL>(PartMeeting::area(ws_base),
                                          (uint32_t)(((size_t)2 * pc + (pc == p_first ? 1 : 0)) * ws_tile + tile * TN) * 4u,
                                          ws_pitch, cs, g, total);
            tile_to_output<V, CPL, OutT>(out, p_row, n_cols, col0, col_ok, g, total);
            PartMeeting::rearm(counter, lane);  // ready for the next launch
        }
    }
}

// Second launch.  Workgroups [0, n_pieces - 1), one per piece boundary p = (b + 1) * piece: when p falls strictly
// inside a row and is the first piece boundary inside that row, the workgroup adds the row's parts in ascending
// order and writes the row.  The remaining workgroups take four vector rows each (one per wave) and write zeros
// for the empty ones.
template <int V, typename OutT>
__global__ void __launch_bounds__(256)
spmm_flat_fixup_kernel(int m_vec, int n_cols, long long piece, int n_pieces, const int *__restrict__ row_offsets,
                       const float *__restrict__ ws, int ws_pitch, OutT *__restrict__ out)
{
    const int lane = threadIdx.x & 63;
    const int quads = n_cols >> 2;  // n_cols % 4 == 0
    if ((int)blockIdx.x >= n_pieces - 1) {
        const int row = ((int)blockIdx.x - (n_pieces - 1)) * 4 + (threadIdx.x >> 6);
        if (row >= m_vec) return;
        if (row_offsets[row + 1] != row_offsets[row]) return;
        const float zeros[4] = {0.f, 0.f, 0.f, 0.f};
        for (int item = lane; item < V * quads; item += 64)
            store_converted<OutT, 4>(out + (size_t)row * V * n_cols + 4 * (size_t)item, zeros);
        return;
    }
    const int b = blockIdx.x;
    const long long p = (b + 1) * piece;  // < nonzeros_vec < 2^31
    int base, first;
    const int offs = find_row_window(row_offsets, m_vec, (int)p, lane, base, first);  // every wave searches: no barrier
    const int row = base + first;
    if (row >= m_vec) return;
    const int row_beg = __builtin_amdgcn_readlane(offs, first);
    int row_end;
    if (first < 63)
        row_end = __builtin_amdgcn_readlane(offs, first + 1);
    else
        row_end = row_offsets[row + 1];  // the window ends with this row's start
    if (row_beg >= p || row_beg < p - piece) return;  // a row starts at the boundary / not its first boundary
    const float *first_part = ws + ((size_t)2 * b + 1) * V * ws_pitch;  // T[b]: the part that starts inside piece b
    for (int item = threadIdx.x; item < V * quads; item += 256) {
        const int v = item / quads;
        const int q = item - v * quads;
        const size_t at = (size_t)v * ws_pitch + 4 * (size_t)q;
        float4_t sum = *reinterpret_cast<const float4_t *>(first_part + at);
        for (int c = b + 1; c * piece < row_end; ++c) {
            const float4_t x = *reinterpret_cast<const float4_t *>(ws + (size_t)2 * c * V * ws_pitch + at);  // F[c]
            sum[0] += x[0];
            sum[1] += x[1];
            sum[2] += x[2];
            sum[3] += x[3];
        }
        const float tmp[4] = {sum[0], sum[1], sum[2], sum[3]};
        store_converted<OutT, 4>(out + ((size_t)row * V + v) * n_cols + 4 * (size_t)q, tmp);
    }
}

namespace {

// The workspace starts with the arrival counters, one per (piece, column tile), followed by the tiles F and T of
// every piece (partial_tile_counter_bytes: the counters' area follows the workspace's size, not the problem's shape).
struct FlatShape {
    bool one_launch;  // cross-workgroup parts added inside the launch (arrival counters) instead of by a second one
    bool shared;      // steps shared by consecutive rows
    int cpl;       // columns per lane (tile of 16*cpl dense columns)
    int waves;     // runs (= waves) per piece (= workgroup)
    int sub;       // nonzero vectors per run
    int n_pieces;
    int ws_pitch;  // floats per row of a workspace tile: the dense width rounded up to whole tiles
    long long counter_bytes;  // the counters' area at the start of the workspace (0 without a workspace)
};

// Launch shape: eight runs per piece, runs of four to eight steps sized so that the launch holds about 3600
// waves (measured on Pareto-distributed rows of mean 280, 256 to 4096 vector rows x 4608, N = 256: four steps
// best at 256 rows, five at 1024, eight at 4096; twelve thousand waves of two steps cost 1.6 times as much,
// because every wave pays its row search before its first gather; sixteen runs per piece 0 to 15 % behind eight);
// longer runs (fewer, larger pieces) when the workspace cannot hold two partial tiles per piece.
bool flat_shape(int vec_length, int k, int nonzeros_vec, long long workspace_bytes, FlatShape &s)
{
    const Options &o = options();
    int cpl = o.spmm_cols_per_lane;
    if (cpl != 4 && cpl != 8) {
        const long long steps = (nonzeros_vec + kStep - 1) / kStep;
        cpl = (k % 8 == 0 && k > 64 && steps * ceil_div(k, 128) >= 3584) ? 8 : 4;
    }
    if (cpl == 8 && k % 8 != 0) cpl = 4;
    const int n_tiles = ceil_div(k, 16 * cpl);
    s.cpl = cpl;
    s.ws_pitch = n_tiles * 16 * cpl;
    s.waves = o.spmm_flat_waves > 0 ? o.spmm_flat_waves : 8;
    s.one_launch = o.spmm_flat_launches != 2;  // (and the tile area below 2 GiB: 32-bit buffer offsets, see below)
    s.shared = o.spmm_flat_shared == 2;  // the launcher turns it on for short rows, which it knows the count of
    long long sub = o.spmm_flat_piece > 0 ? o.spmm_flat_piece : ((long long)nonzeros_vec * n_tiles + 3583) / 3584;
    sub = (sub + kStep - 1) / kStep * kStep;
    if (o.spmm_flat_piece <= 0) {
        if (sub < 4 * kStep) sub = 4 * kStep;
        if (sub > 8 * kStep) sub = 8 * kStep;
    }
    const long long slot_bytes = 2LL * vec_length * s.ws_pitch * (long long)sizeof(float);  // T and F of one piece
    // (a size query passes "no limit": the counters' area then follows from the tiles, see flat_workspace_for)
    const bool unlimited = workspace_bytes == 0x7fffffffffffffffLL;
    s.counter_bytes = unlimited || workspace_bytes <= 0 ? 0 : partial_tile_counter_bytes(workspace_bytes);
    for (;;) {
        const long long piece = sub * s.waves;
        const long long n_pieces = ((long long)nonzeros_vec + piece - 1) / piece;
        if (n_pieces <= 1 || unlimited || s.counter_bytes + n_pieces * slot_bytes <= workspace_bytes) {
            s.sub = (int)sub;
            s.n_pieces = (int)n_pieces;
            if (n_pieces * slot_bytes >= (1LL << 31)) s.one_launch = false;
            return true;
        }
        if (sub >= (1LL << 30)) return false;
        const long long fit = (workspace_bytes - s.counter_bytes) / slot_bytes;  // pieces the workspace can hold
        long long grown = fit > 1 ? ((long long)nonzeros_vec + fit - 1) / fit : (long long)nonzeros_vec;
        grown = ((grown + s.waves - 1) / s.waves + kStep - 1) / kStep * kStep;
        sub = grown > sub ? grown : sub + kStep;
    }
}

template <int V, int CPL, bool IDX32, bool ONE_LAUNCH, typename OutT, bool SHARED = false>
int launch_flat_kernel(int m_vec, int k, int nonzeros_vec, const FlatShape &s, const int *row_offsets,
                       const int *column_indices, const half_t *values, const half_t *rhs, OutT *out, float *workspace,
                       hipStream_t stream)
{
    const int n_tiles = ceil_div(k, 16 * CPL);
    const long long main_blocks = (long long)s.n_pieces * n_tiles;
    const long long zero_blocks = ONE_LAUNCH ? ceil_div(m_vec, 4 * s.waves) : 0;
    if (main_blocks + zero_blocks > 0x7fffffffLL) return hipErrorNotSupported;
    int *counters = reinterpret_cast<int *>(workspace);
    float *tiles = reinterpret_cast<float *>(reinterpret_cast<unsigned char *>(workspace) +
                                             (s.n_pieces > 1 ? s.counter_bytes : 0));
    const size_t lds = (size_t)s.waves * (stage_bytes<V>() + (size_t)V * 16 * CPL * sizeof(float));
    auto kernel = spmm_mfma_flat_kernel<V, CPL, IDX32, ONE_LAUNCH, OutT, SHARED>;
    static std::atomic<unsigned long long> lds_allowed{0};
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 96 * 1024, lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(main_blocks + zero_blocks)), dim3(64 * s.waves), lds, stream, m_vec, k,
                       n_tiles, nonzeros_vec, s.sub, (int)main_blocks, counters, row_offsets, column_indices, values, rhs,
                       out, tiles, s.ws_pitch);
    const hipError_t st = hipGetLastError();
    if (st != hipSuccess || ONE_LAUNCH) return (int)st;
    const long long fix_blocks = (long long)(s.n_pieces - 1) + ceil_div(m_vec, 4);
    if (fix_blocks > 0x7fffffffLL) return hipErrorNotSupported;
    hipLaunchKernelGGL((spmm_flat_fixup_kernel<V, OutT>), dim3((unsigned)fix_blocks), dim3(256), 0, stream, m_vec, k,
                       (long long)s.sub * s.waves, s.n_pieces, row_offsets, tiles, s.ws_pitch, out);
    return (int)hipGetLastError();
}

template <int V, int CPL, bool IDX32, typename OutT>
int launch_flat_idx(int m_vec, int k, int nonzeros_vec, const FlatShape &s, const int *row_offsets,
                    const int *column_indices, const half_t *values, const half_t *rhs, OutT *out, float *ws,
                    hipStream_t stream)
{
    if constexpr (IDX32) {
        if (s.shared && s.one_launch)
            return launch_flat_kernel<V, CPL, IDX32, true, OutT, true>(m_vec, k, nonzeros_vec, s, row_offsets,
                                                                       column_indices, values, rhs, out, ws, stream);
        if (s.shared)
            return launch_flat_kernel<V, CPL, IDX32, false, OutT, true>(m_vec, k, nonzeros_vec, s, row_offsets,
                                                                        column_indices, values, rhs, out, ws, stream);
    }
    if (s.one_launch)
        return launch_flat_kernel<V, CPL, IDX32, true, OutT>(m_vec, k, nonzeros_vec, s, row_offsets, column_indices, values,
                                                             rhs, out, ws, stream);
    return launch_flat_kernel<V, CPL, IDX32, false, OutT>(m_vec, k, nonzeros_vec, s, row_offsets, column_indices, values,
                                                          rhs, out, ws, stream);
}

template <int V, typename OutT>
int launch_flat_v(int m_vec, int k, int n, int nonzeros_vec, const FlatShape &s, const int *row_offsets,
                  const int *column_indices, const half_t *values, const half_t *rhs, OutT *out, float *ws,
                  hipStream_t stream)
{
    const bool idx32 = (long long)n * k < (1LL << 31);
    if (s.cpl == 8) {
        if (idx32) return launch_flat_idx<V, 8, true, OutT>(m_vec, k, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, ws, stream);
        return launch_flat_idx<V, 8, false, OutT>(m_vec, k, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, ws, stream);
    }
    if (idx32) return launch_flat_idx<V, 4, true, OutT>(m_vec, k, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, ws, stream);
    return launch_flat_idx<V, 4, false, OutT>(m_vec, k, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, ws, stream);
}

}  // namespace

long long spmm_flat_workspace_bytes(int vec_length, int k, int nonzeros_vec)
{
    if (k <= 0 || nonzeros_vec <= 0) return 0;
    FlatShape s;
    if (!flat_shape(vec_length, k, nonzeros_vec, 0x7fffffffffffffffLL, s)) return 0;
    if (s.n_pieces <= 1) return 0;
    return partial_tile_workspace_for(2LL * s.n_pieces * vec_length * s.ws_pitch * (long long)sizeof(float));
}

template <typename OutT>
int launch_spmm_mfma_flat(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_offsets,
                          const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                          float *workspace, long long workspace_bytes, hipStream_t stream)
{
    if (m_vec == 0 || k == 0) return hipSuccess;
    if (k % 4 != 0) return hipErrorNotSupported;
    if (nonzeros_vec == 0)  // no wave would visit any row: every output row is an empty sum
        return launch_zero_fill(out, (long long)m_vec * vec_length * k * (long long)sizeof(OutT), 0, 1, stream);
    FlatShape s;
    if (!flat_shape(vec_length, k, nonzeros_vec, workspace ? workspace_bytes : 0, s)) return hipErrorNotSupported;
    // Rows that share steps: 14 % faster on 4096 rows of 20 vectors and 7 % on 2048 rows of 50 (N = 256, V = 8),
    // where a step per row segment runs half empty; within 7 % either way on rows of a hundred vectors and more.
    if (options().spmm_flat_shared == 0 && nonzeros_vec / m_vec < 64) s.shared = true;
    switch (vec_length) {
    case 1: return launch_flat_v<1, OutT>(m_vec, k, n, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, workspace, stream);
    case 2: return launch_flat_v<2, OutT>(m_vec, k, n, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, workspace, stream);
    case 4: return launch_flat_v<4, OutT>(m_vec, k, n, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, workspace, stream);
    case 8: return launch_flat_v<8, OutT>(m_vec, k, n, nonzeros_vec, s, row_offsets, column_indices, values, rhs, out, workspace, stream);
    default: return hipErrorInvalidValue;
    }
}

// Library-owned scratch for the entry point that allocates nothing: the workspace of the split-row schedule in a
// static device array (every GPU the library runs on holds its own copy at its own address until the process
// ends).  Host code must not use the array's name as an address: it is resolved once per device.
constexpr long long kScratchBytes = 16LL << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static std::atomic<void *> scratch_of_device[64];

// The current device's copy of `scratch` (resolved on the first call on that device, with it current).
static int scratch_address(float **address)
{
    int device = 0;
    hipError_t st = hipGetDevice(&device);
    if (st != hipSuccess) return (int)st;
    if (device < 0 || device >= 64) return hipErrorNotSupported;
    void *p = scratch_of_device[device].load(std::memory_order_acquire);
    if (!p) {
        st = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (st != hipSuccess) return (int)st;
        if (!p) return hipErrorInvalidSymbol;
        scratch_of_device[device].store(p, std::memory_order_release);
    }
    *address = static_cast<float *>(p);
    return hipSuccess;
}

// Also resolves the current device's copy of the array, so that a caller who asks for the size before capturing a HIP
// graph has the symbol lookup outside the capture.
long long spmm_flat_scratch_bytes()
{
    float *unused = nullptr;
    (void)scratch_address(&unused);
    return kScratchBytes;
}

// Zeros for the arrival counters of the static array (a kernel, not a memset node: the call may be captured).
int spmm_flat_scratch_reset(hipStream_t stream)
{
    float *ws = nullptr;
    const int st = scratch_address(&ws);
    if (st != hipSuccess) return st;
    return launch_zero_fill(ws, partial_tile_counter_bytes(kScratchBytes), 0, 1, stream);
}

int launch_spmm_mfma_flat_static(int m_vec, int vec_length, int k, int n, int nonzeros_vec, const int *row_offsets,
                                 const int *column_indices, const half_t *values, const half_t *rhs, half_t *out,
                                 hipStream_t stream)
{
    if (m_vec == 0 || k == 0) return hipSuccess;
    if (k % 4 != 0) return hipErrorNotSupported;
    // the scratch must hold the partial tiles of some sixty pieces beside its counters, or the schedule degenerates
    const long long k_pad = (long long)ceil_div(k, 128) * 128;
    if (64LL * 2 * vec_length * k_pad * (long long)sizeof(float) > kScratchBytes) return hipErrorNotSupported;
    float *ws = nullptr;
    const int st = scratch_address(&ws);
    if (st != hipSuccess) return st;
    return launch_spmm_mfma_flat<half_t>(m_vec, vec_length, k, n, nonzeros_vec, row_offsets, column_indices, values, rhs,
                                         out, ws, kScratchBytes, stream);
}

template int launch_spmm_mfma_flat<half_t>(int, int, int, int, int, const int *, const int *, const half_t *,
                                           const half_t *, half_t *, float *, long long, hipStream_t);
template int launch_spmm_mfma_flat<float>(int, int, int, int, int, const int *, const int *, const half_t *,
                                          const half_t *, float *, float *, long long, hipStream_t);

}  // namespace vs
