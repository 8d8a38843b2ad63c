// SpMM on fp16 MFMA for column-vector CSR (replaces src/wmma_spmm.cu of the reference).
//
// Work item = (vector row, tile of TN = 16*CPL dense columns), one workgroup of W waves.
// The waves of a workgroup split the row's nonzero vectors in interleaved steps of 32 and
// their fp32 partial tiles are summed through LDS in a fixed order, so the result does not
// depend on timing and no cross-workgroup reduction is needed for the fp16 output.
//
// One step (32 nonzero vectors x TN columns) in a wave, lane = (cs = lane % 16, g = lane / 16):
//   * lanes 0..31 fetch one column index and one V-vector each (coalesced) and park them in a
//     wave-private LDS slot, the vectors transposed to [v][nonzero]; no workgroup barrier;
//   * every lane then issues eight loads of CPL consecutive halves, one per gathered rhs row
//     j = base + 8g + e, e = 0..7, at columns tile*TN + cs*CPL.. : for each e the 16 lanes of a
//     group read one contiguous 2*TN-byte segment (128-bit loads for CPL = 8), 8 rows in flight;
//   * v_mfma_f32_16x16x32_f16 wants, per lane, 8 consecutive k for ONE column, so the CPL x 8
//     block a lane holds is transposed in registers with v_perm_b32 (the dense operand never
//     goes through LDS);
//   * MFMA number c (c < CPL) computes D[v][cs] += sum_k a[v][j(k)] * B[col_j(k)][tile*TN + cs*CPL + c]
//     with the sparse vectors as the 16 x 32 A operand (rows v >= V are zero).
//   The accumulator of lane (cs, g), register e, MFMA c is out[4g + e][tile*TN + cs*CPL + c], i.e.
//   CPL consecutive outputs per (lane, e): one vector store each.
#include "spmm_mfma_step.hpp"
#include "vs_common.hpp"

namespace vs {

// SOFTMAX: the sparse values are raw scores and the kernel multiplies by softmax_row(scale * values)
// instead: a pre-pass finds each scalar row's maximum, the staging step turns every score into
// exp2(s*x - max) (and sums them), and the accumulated tile is divided by the row sum at the end.
// RAGGED: the dense width is not a multiple of CPL (rows of the dense operand and of the output start at any 2-byte
// boundary, the last chunk of a row is cut): chunks are fetched and stored half by half.
// S: 32-vector steps a wave keeps in flight at once (1, 2 or 4): its unit of work is a block of S steps whose 8 * S
// row segments per lane are all requested before the first MFMA.
// TEAMS: rows ordered by length; only the first team_slots entries of row_indices get the workgroup's waves as a
// team, behind them every wave takes a row of its own (below).
// PIPE (S = 2): a wave that takes several blocks of a row one after the other requests each step of the next block
// as soon as the same step of the current one is multiplied, so that it always has one or two steps in flight
// instead of two while it waits and none while it multiplies; the next block's indices and vectors are requested a
// block earlier for that, ahead of the current block's row segments (loads return in order).
// PARTS: the dispatch list names parts of rows instead of rows - `row_indices` holds four ints per workgroup slot,
// {vector row, first nonzero, end, part info} (vs_spmm_row_parts makes the list; row_offsets is not read) - so that
// a row far longer than the rest is served by several workgroups, each taking a run of its nonzeros.  Part info 0:
// the slot is a whole row and everything is as without the list.  Otherwise (parts | part << 8 | split row << 16)
// the workgroup's fp32 tile goes to the workspace (`part_tiles`, tile of (split row, part, column tile)) and the
// workgroup counts itself in on the row's arrival counter; the one that arrives last adds the parts in ascending
// order - same bits whoever it is - writes the row and puts the counter back to zero.  Nobody waits for anybody.
// How the parts reach the workgroup that adds them: PartMeeting in spmm_mfma_step.hpp.
template <int V, int CPL, bool SOFTMAX, bool IDX32, typename OutT, bool RAGGED = false, int S = 1, bool TEAMS = false,
          bool PIPE = false, bool PARTS = false>
__global__ void __launch_bounds__(S * CPL >= 32 ? 256 : (S * CPL >= 16 ? 512 : 1024))
spmm_mfma_kernel(int n_cols, int n_tiles, int shape, const int *__restrict__ row_indices,
                 const int *__restrict__ row_offsets, const int *__restrict__ column_indices,
                 const half_t *__restrict__ values, const half_t *__restrict__ rhs,
                 OutT *__restrict__ out, long long stride_values, long long stride_rhs, long long stride_out,
                 float scale, int team_slots, int n_slots,  // (the first sixteen dwords arrive preloaded in registers)
                 int *part_counters, float *part_tiles, int parts_max)
{
    static_assert(!PARTS || (!SOFTMAX && !RAGGED && !TEAMS), "row parts exist for the plain operator on whole chunks");
    // `shape` packs what the prologue needs into one of the kernel arguments that arrive in registers: bits 0-7
    // log2 of the blocks a wave takes of a row, bits 8-15 the waves per workgroup, bit 16 "the grid has 512
    // workgroups or more" - the workgroup size and the grid size would otherwise be loads from the hidden arguments.
    const int per_wave_log2 = shape & 255;
    const int n_waves = (shape >> 8) & 255;
    const bool full_grid = (shape >> 16) & 1;
    const bool parts_meet_later = (shape >> 17) & 1;  // PARTS: a second launch adds the parts of split rows
    if (blockIdx.y != 0) {  // batch: shared pattern, per-problem operands (the strides are not loaded for problem 0)
        values += blockIdx.y * stride_values;
        rhs += blockIdx.y * stride_rhs;
        out += blockIdx.y * stride_out;
    }
    extern __shared__ __align__(16) unsigned char smem[];  // [W] staging slots, then [W][V][TN] partials
    constexpr int TN = 16 * CPL;
    constexpr int kStage = S * stage_bytes<V>();
    constexpr int kBlock = S * kStep;       // nonzero vectors per block
    constexpr int F = (S + 1) / 2;          // vectors a lane fetches per block (lanes 0..31 only when S = 1)
    const int lane = threadIdx.x & 63;
    const int slot_wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the wave's LDS slot
    // Workgroup -> rows.  A team: the workgroup's waves share one row (team_slots < 0: every workgroup is one).
    // With rows ordered by length (team_slots >= 0) only the first team_slots entries of row_indices - the long
    // rows - get a team; behind them a workgroup takes n_waves consecutive entries, one row per wave, which then
    // needs neither barrier nor LDS for its result and leaves no wave without work.
    int tile = blockIdx.x % n_tiles;  // (a grid of (tile, slot, batch) without this division measured 1 % slower)
    int slot = blockIdx.x / n_tiles;
    int wave = slot_wave;  // the wave's place in its row's team
    bool solo = false;
    if constexpr (TEAMS) {
        if (slot >= team_slots) {
            const int b = blockIdx.x - team_slots * n_tiles;
            tile = b % n_tiles;
            slot = team_slots + (b / n_tiles) * n_waves + slot_wave;
            wave = 0;
            solo = true;
            if (slot >= n_slots) return;
        }
    }
    // The row's extent is requested for the identity order together with the swizzle entry itself, and again
    // only if the entry names another row: one dependent load less in the common case.
    int row, beg, end, part_info = 0;
    if constexpr (PARTS) {
        const int4_t d = reinterpret_cast<const int4_t *>(row_indices)[slot];  // one request for everything
        row = d[0];
        beg = d[1];
        end = d[2];
        part_info = d[3];
    } else {
        row = row_indices[slot];
        beg = row_offsets[slot];
        end = row_offsets[slot + 1];
        // (the empty statement keeps the two requests above: the compiler otherwise folds them into the dependent
        // ones below by selecting the index)
        asm volatile("" : "+s"(beg), "+s"(end));
        if (row != slot) {
            beg = row_offsets[row];
            end = row_offsets[row + 1];
        }
    }
    const int cs = lane & 15;
    const int g = lane >> 4;
    const int col0 = tile * TN + cs * CPL;
    const bool col_ok = col0 < n_cols;  // n_cols % CPL == 0 unless RAGGED: a lane's chunk is all in or all out
    const uint32_t col_off = col_ok ? col0 : 0;
    const int valid = !col_ok ? 0 : (n_cols - col0 < CPL ? n_cols - col0 : CPL);  // RAGGED: halves of the chunk that exist

    int *idx_s = reinterpret_cast<int *>(smem + (size_t)slot_wave * kStage);
    half_t *vec_s = reinterpret_cast<half_t *>(idx_s + kBlock);  // [V][kBlock]
    float *partial = reinterpret_cast<float *>(smem + (size_t)n_waves * kStage);
    float *sums_s = partial + (size_t)n_waves * V * TN;  // [W][V] softmax denominators (SOFTMAX only)

    // Short rows do not need every wave: with fewer than two steps per wave the partial-tile reduction costs
    // more than the split saves (S = 1); with S steps in flight a block is one round trip whatever its size, so
    // every block gets its own wave - except that the barrier and the sum through LDS cost more than a second
    // round trip, so a row of two blocks stays with one wave when the grid alone fills the chip (512 workgroups
    // and more: 3.23 against 3.35 us on 256 rows of 102 vectors, N = 256; with 256 workgroups 2.78 against 2.64).
    // The other waves end here: a workgroup barrier waits only for the waves that are still running, and a row
    // of a single active wave needs neither barrier nor LDS for its result.
    const int steps = (end - beg + kStep - 1) / kStep;
    // per_wave_log2 > 0 (the grid alone fills the chip): a wave takes 2^per_wave_log2 blocks of a row one after the
    // other, so that a row of the expected length keeps to the waves the chip has room for and only a row far longer
    // than expected spreads over the rest of its workgroup.
    int active = S == 1 ? (steps + 1) >> 1 : (steps + S - 1) / S;
    if (S > 1 && active == 2 && full_grid) active = 1;
    if (S > 1) active = (active + (1 << per_wave_log2) - 1) >> per_wave_log2;
    active = active < 1 ? 1 : (active > n_waves ? n_waves : active);
    if (solo) active = 1;
    if (wave >= active) return;

    const float s2 = scale * kLog2e;
    float row_max[V], row_sum[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        row_max[v] = -__builtin_inff();
        row_sum[v] = 0.f;
    }
    if constexpr (SOFTMAX) {
        for (int j = beg + lane; j < end; j += 64) {
            half_t x[V];
            load_vector<V>(x, values + (size_t)j * V);
#pragma unroll
            for (int v = 0; v < V; ++v) row_max[v] = fmaxf(row_max[v], (float)x[v] * s2);
        }
#pragma unroll
        for (int v = 0; v < V; ++v) row_max[v] = wave_max(row_max[v]);
    }

    float4_t acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = float4_t{0.f, 0.f, 0.f, 0.f};

    // The column index and the vector of the NEXT step are fetched into registers while the gathered
    // rows of the current step are in flight, so a wave pays one memory round trip per step, not two.
    const int stride = kBlock * active;
    int base = beg + kBlock * wave;
    const bool has_work = base < end;
    int next_idx[F];
    bool next_valid[F];
    PackedVector<V> next_vec[F];  // as loaded: the halves are taken apart when the block is staged
#pragma unroll
    for (int i = 0; i < F; ++i) {
        next_idx[i] = 0;
        next_valid[i] = false;
        next_vec[i].clear();
    }
    auto fetch = [&](int b) {
#pragma unroll
        for (int i = 0; i < F; ++i) {
            if (64 * i + lane < kBlock) {
                const int j = b + 64 * i + lane;
                next_valid[i] = j < end;
                // Slots past the row's end repeat its last vector with a zero value: the gather stays
                // in bounds and contributes nothing.
                const int jc = next_valid[i] ? j : end - 1;
                next_idx[i] = column_indices[jc];
                next_vec[i].load(values + (size_t)jc * V);
            }
        }
    };
    if (has_work) fetch(base);

    auto stage = [&]() {  // the fetched block into the wave's LDS slot
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const int at = 64 * i + lane;
            if (at < kBlock) {
                idx_s[at] = next_idx[i];
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    half_t staged = next_valid[i] ? next_vec[i].at(v) : (half_t)0.f;
                    if constexpr (SOFTMAX) {
                        const float p =
                            next_valid[i] ? __builtin_amdgcn_exp2f((float)next_vec[i].at(v) * s2 - row_max[v]) : 0.f;
                        row_sum[v] += p;
                        staged = (half_t)p;
                    }
                    vec_s[v * kBlock + at] = staged;
                }
            }
        }
        wave_lds_fence();
    };
    // the row's tile straight from the accumulators of the one wave that worked on it
    auto store_alone = [&]() {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int v = 4 * g + e;
            if (v < V && col_ok) {
                float norm = 1.f;
                if constexpr (SOFTMAX) {
                    float total = 1.f;
#pragma unroll
                    for (int vv = 0; vv < V; ++vv) total = (vv == v) ? row_sum[vv] : total;
                    norm = end > beg ? 1.f / total : 0.f;
                }
                float tmp[CPL];
#pragma unroll
                for (int c = 0; c < CPL; ++c) tmp[c] = acc[c][e] * norm;
                if constexpr (RAGGED)
                    store_ragged<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col0, tmp, valid);
                else
                    store_converted<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col0, tmp);
            }
        }
    };
    // PARTS, a slot that is a part of a row: where its tile lies in the workspace (byte offset), how a thread puts
    // its CPL sums of scalar row v there, and what the wave that has counted the workgroup in does when it is the
    // last of the row's parts.
    const int part_count = part_info & 255;
    const uint32_t part_tile_bytes = (uint32_t)V * TN * (uint32_t)sizeof(float);
    // (the launcher passes the number of split rows where the team mapping has its count: problem b of a batch has
    // its tiles and counters behind those of problems 0 .. b - 1)
    const int part_split = (int)blockIdx.y * team_slots + (part_info >> 16);
    const uint32_t part_row_base =
        (uint32_t)((part_split * parts_max) * n_tiles + tile) * part_tile_bytes;  // part 0 of the row, this tile
    auto park = [&](int v, int cs_at, const float (&vals)[CPL]) {
        const uint32_t at = part_row_base + (uint32_t)(((part_info >> 8) & 255) * n_tiles) * part_tile_bytes +
                            4u * (uint32_t)(v * TN + cs_at * CPL);
#pragma unroll
        for (int c4 = 0; c4 < CPL / 4; ++c4) {
            const float4_t t = {vals[4 * c4], vals[4 * c4 + 1], vals[4 * c4 + 2], vals[4 * c4 + 3]};
            if (parts_meet_later)  // read by the next launch
                PartMeeting::store_plain(PartMeeting::area(part_tiles), at + 16u * c4, t);
            else
                PartMeeting::store_part(PartMeeting::area(part_tiles), at + 16u * c4, t);
        }
    };
    auto arrive_and_finish = [&]() {  // one wave, all of its lanes; the workgroup's stores have completed
        int *counter = part_counters + ((size_t)part_split * n_tiles + tile) * kPartCounterStride;
        if (PartMeeting::arrive(counter, lane) != part_count - 1) return;  // parts are still to come: whoever brings the last adds up
        PartMeeting::collect();
        for (int item = lane; item < V * 16; item += 64) {
            const int v = item >> 4;
            const int cs_at = item & 15;
            const int col = tile * TN + cs_at * CPL;
            float total[CPL];
#pragma unroll
            for (int c = 0; c < CPL; ++c) total[c] = 0.f;
            for (int p = 0; p < part_count; ++p) {
                const uint32_t at = part_row_base + (uint32_t)(p * n_tiles) * part_tile_bytes +
                                    4u * (uint32_t)(v * TN + cs_at * CPL);
#pragma unroll
                for (int c4 = 0; c4 < CPL / 4; ++c4) {
                    const float4_t x = PartMeeting::load_part(PartMeeting::area(part_tiles), at + 16u * c4);
                    total[4 * c4] += x[0];
                    total[4 * c4 + 1] += x[1];
                    total[4 * c4 + 2] += x[2];
                    total[4 * c4 + 3] += x[3];
                }
            }
            if (col < n_cols) store_converted<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col, total);
        }
        PartMeeting::rearm(counter, lane);  // ready for the next launch
    };
    if constexpr (PIPE) {
        static_assert(S == 2 && IDX32 && !SOFTMAX && !RAGGED, "the pipelined walk exists for blocks of two steps");
        // (expected: the compiler then lays the walk's code out behind the epilogue, out of the short row's way -
        // the instruction cache starts every launch cold)
        if (__builtin_expect(has_work && base + stride >= end, 1)) {  // a single block: nothing to overlap it with
            stage();
            spmm_mfma_block<V, CPL, S, IDX32>(idx_s, vec_s, rhs, n_cols, col_off, cs, g, acc, [] {});
        } else if (has_work) {
            StagedStep now[2], then[2];
            RowChunk<CPL> first[8], second[8];
            stage();
            read_staged_step<V, kBlock>(now[0], idx_s, vec_s, 0, cs, g);
            read_staged_step<V, kBlock>(now[1], idx_s, vec_s, 1, cs, g);
            wave_lds_fence();
            // (fetched whether or not the block exists - past the row's end the lanes re-read its last vector - so
            // that the number of loads in flight is the same on every path and the waits below count exactly)
            fetch(base + stride);  // ahead of the row segments below
            __builtin_amdgcn_sched_barrier(0);
            request_step<CPL>(first, now[0], rhs, n_cols, col_off);
            request_step<CPL>(second, now[1], rhs, n_cols, col_off);
            __builtin_amdgcn_sched_barrier(0);
            for (;;) {
                base += stride;
                if (base >= end) break;
                stage();  // waits for the indices and vectors only: they were requested before the segments
                read_staged_step<V, kBlock>(then[0], idx_s, vec_s, 0, cs, g);
                read_staged_step<V, kBlock>(then[1], idx_s, vec_s, 1, cs, g);
                wave_lds_fence();
                fetch(base + stride);
                // (the scheduler otherwise waits for both steps, transposes both and only then requests the next
                // two: the barriers keep each step's requests right behind its multiplication)
                __builtin_amdgcn_sched_barrier(0);
                multiply_step<CPL>(first, now[0].a, acc);
                __builtin_amdgcn_sched_barrier(0);
                request_step<CPL>(first, then[0], rhs, n_cols, col_off);
                __builtin_amdgcn_sched_barrier(0);
                multiply_step<CPL>(second, now[1].a, acc);
                __builtin_amdgcn_sched_barrier(0);
                request_step<CPL>(second, then[1], rhs, n_cols, col_off);
                __builtin_amdgcn_sched_barrier(0);
                now[0] = then[0];
                now[1] = then[1];
            }
            multiply_step<CPL>(first, now[0].a, acc);
            multiply_step<CPL>(second, now[1].a, acc);
            // (a use of the last fetch on this path too: with uses only inside the loop the compiler moves the first
            // fetch behind the loop test, i.e. behind the row segments, and every wait for it becomes a wait for them)
#pragma unroll
            for (int i = 0; i < F; ++i) asm volatile("" ::"v"(next_idx[i]), "v"(next_vec[i].first()));
        }
    }
    for (; !PIPE && has_work && base < end; base += stride) {
        stage();
        if constexpr (S == 1) {
            spmm_mfma_step<V, CPL, IDX32, RAGGED>(idx_s, vec_s, rhs, n_cols, col_off, cs, g, acc, [&] {
                if (base + stride < end) fetch(base + stride);
            }, valid);
        } else {
            // A block that the row fills only in part still requests all its steps (the padding repeats one row
            // segment, which stays in the L1): asking for fewer steps behind a uniform branch measured 5 % slower
            // on short rows (the three code paths) and 4 % faster on long ones.
            spmm_mfma_block<V, CPL, S, IDX32>(idx_s, vec_s, rhs, n_cols, col_off, cs, g, acc, [&] {
                if (base + stride < end) fetch(base + stride);
            });
        }
    }

    if constexpr (SOFTMAX) {
#pragma unroll
        for (int v = 0; v < V; ++v) row_sum[v] = wave_sum(row_sum[v]);
    }

    if (active == 1) {
        if constexpr (PARTS) {
            if (part_info != 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int v = 4 * g + e;
                    if (v < V) {
                        float tmp[CPL];
#pragma unroll
                        for (int c = 0; c < CPL; ++c) tmp[c] = acc[c][e];
                        park(v, cs, tmp);
                    }
                }
                if (parts_meet_later) return;
                PartMeeting::publish();
                arrive_and_finish();
                return;
            }
        }
        store_alone();
        return;
    }

    float *mine = partial + (size_t)wave * V * TN;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e;
        if (v < V) {
#pragma unroll
            for (int c4 = 0; c4 < CPL / 4; ++c4) {
                float4_t t = {acc[4 * c4][e], acc[4 * c4 + 1][e], acc[4 * c4 + 2][e], acc[4 * c4 + 3][e]};
                *reinterpret_cast<float4_t *>(mine + v * TN + cs * CPL + 4 * c4) = t;
            }
        }
    }
    if constexpr (SOFTMAX) {
        if (lane < V) {
            float mine_sum = 0.f;
#pragma unroll
            for (int v = 0; v < V; ++v) mine_sum = (v == lane) ? row_sum[v] : mine_sum;
            sums_s[wave * V + lane] = mine_sum;
        }
    }
    __syncthreads();
    const int t = threadIdx.x;  // V * 16 <= 128 threads add: waves 0 and 1, both among the active ones here
    if (t < V * 16) {
        const int v = t >> 4;
        const int cs2 = t & 15;
        const int col = tile * TN + cs2 * CPL;
        if (col < n_cols) {
            float sum[CPL];
#pragma unroll
            for (int c = 0; c < CPL; ++c) sum[c] = 0.f;
            // added in wave order; the compiler unrolls this by eight with all sixteen LDS reads in flight, which
            // measured 2-7 % faster end to end than hand-made batches of four tiles with a select per term
            for (int w = 0; w < active; ++w) {
                const float *src = partial + (size_t)w * V * TN + v * TN + cs2 * CPL;
#pragma unroll
                for (int c4 = 0; c4 < CPL / 4; ++c4) {
                    const float4_t x = *reinterpret_cast<const float4_t *>(src + 4 * c4);
                    sum[4 * c4] += x[0];
                    sum[4 * c4 + 1] += x[1];
                    sum[4 * c4 + 2] += x[2];
                    sum[4 * c4 + 3] += x[3];
                }
            }
            if constexpr (SOFTMAX) {
                float total = 0.f;
                for (int w = 0; w < active; ++w) total += sums_s[w * V + v];
                const float norm = end > beg ? 1.f / total : 0.f;
#pragma unroll
                for (int c = 0; c < CPL; ++c) sum[c] *= norm;
            }
            if constexpr (PARTS) {
                if (part_info != 0)
                    park(v, cs2, sum);
                else
                    store_converted<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col, sum);
            } else if constexpr (RAGGED)
                store_ragged<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col, sum, n_cols - col);
            else
                store_converted<OutT, CPL>(out + ((size_t)row * V + v) * n_cols + col, sum);
        }
    }
    if constexpr (PARTS) {
        if (part_info != 0 && !parts_meet_later) {  // (uniform over the workgroup; idle waves have left)
            PartMeeting::publish();
            if (V * 16 > 64) __syncthreads();  // the adding threads span two waves: both have stored
            if (wave == 0) arrive_and_finish();
        }
    }
}

// Second launch of the rows in parts (when the parts do not meet inside the first): one workgroup per (split row,
// column tile) adds the row's partial tiles in ascending order - the same sum as the workgroup that arrives last
// computes in the one-launch form - and writes the row.  `split_rows`: four ints per split row, {vector row, parts}.
template <int V, int CPL>
__global__ void __launch_bounds__(V * 16 < 64 ? 64 : V * 16)
spmm_row_parts_sum_kernel(int n_cols, int n_tiles, const int *__restrict__ split_rows, int n_split, int parts_max,
                          const float *__restrict__ tiles, half_t *__restrict__ out, long long stride_out)
{
    constexpr int TN = 16 * CPL;
    const int tile = blockIdx.x % n_tiles;
    const int split_in_problem = blockIdx.x / n_tiles;
    const int row = split_rows[4 * split_in_problem];
    const int parts = split_rows[4 * split_in_problem + 1];
    const int split = (int)blockIdx.y * n_split + split_in_problem;  // batch: problem b's tiles behind those before it
    out += blockIdx.y * stride_out;
    const int item = threadIdx.x;
    if (item >= V * 16) return;
    const int v = item >> 4;
    const int cs = item & 15;
    const int col = tile * TN + cs * CPL;
    if (col >= n_cols) return;
    float total[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) total[c] = 0.f;
    const float *src = tiles + ((size_t)split * parts_max * n_tiles + tile) * V * TN + v * TN + cs * CPL;
    for (int p = 0; p < parts; ++p) {
#pragma unroll
        for (int c4 = 0; c4 < CPL / 4; ++c4) {
            const float4_t x = *reinterpret_cast<const float4_t *>(src + (size_t)p * n_tiles * V * TN + 4 * c4);
            total[4 * c4] += x[0];
            total[4 * c4 + 1] += x[1];
            total[4 * c4 + 2] += x[2];
            total[4 * c4 + 3] += x[3];
        }
    }
    store_converted<half_t, CPL>(out + ((size_t)row * V + v) * n_cols + col, total);
}

static int next_pow2(int x)
{
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

template <int V, int CPL, bool SOFTMAX, bool IDX32, typename OutT, int S = 1, bool TEAMS = false, bool PIPE = false>
static int launch_idx(int m_vec, int k, int n, int waves, const int *row_indices, const int *row_offsets,
                      const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                      hipStream_t stream, const Batch &batch, float scale, int per_wave = 1, int team_slots = -1)
{
    (void)n;
    int per_wave_log2 = 0;
    while ((2 << per_wave_log2) <= per_wave) ++per_wave_log2;
    constexpr int TN = 16 * CPL;
    const int n_tiles = ceil_div(k, TN);
    if (team_slots > m_vec) team_slots = m_vec;
    const long long blocks = team_slots < 0 ? (long long)m_vec * n_tiles
                                            : ((long long)team_slots + ceil_div(m_vec - team_slots, waves)) * n_tiles;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    const size_t lds = (size_t)waves * S * stage_bytes<V>() +
                       (waves > 1 ? (size_t)waves * V * (TN + 1) * sizeof(float) : 0);
    auto kernel = spmm_mfma_kernel<V, CPL, SOFTMAX, IDX32, OutT, false, S, TEAMS, PIPE>;
    static std::atomic<unsigned long long> lds_allowed{0};
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 96 * 1024, lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * waves), lds, stream,
                       k, n_tiles, per_wave_log2 | (waves << 8) | (blocks * batch.count >= 512 ? 1 << 16 : 0), row_indices,
                       row_offsets, column_indices, values, rhs, out, batch.stride_a, batch.stride_b, batch.stride_out, scale,
                       team_slots, m_vec, static_cast<int *>(nullptr), static_cast<float *>(nullptr), 0);
    return (int)hipGetLastError();
}

// Dense widths that are not a multiple of 4: the half-by-half variant of the 64-column-tile kernel.
template <int V, typename OutT>
static int launch_ragged(int m_vec, int k, int waves, const int *row_indices, const int *row_offsets,
                         const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                         hipStream_t stream, const Batch &batch)
{
    constexpr int TN = 64;
    const int n_tiles = ceil_div(k, TN);
    const long long blocks = (long long)m_vec * n_tiles;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    const size_t lds = (size_t)waves * stage_bytes<V>() + (waves > 1 ? (size_t)waves * V * (TN + 1) * sizeof(float) : 0);
    hipLaunchKernelGGL((spmm_mfma_kernel<V, 4, false, false, OutT, true>), dim3((unsigned)blocks, (unsigned)batch.count),
                       dim3(64 * waves), lds, stream, k, n_tiles, waves << 8, row_indices, row_offsets, column_indices, values, rhs,
                       out, batch.stride_a, batch.stride_b, batch.stride_out, 1.f, -1, m_vec, static_cast<int *>(nullptr),
                       static_cast<float *>(nullptr), 0);
    return (int)hipGetLastError();
}

// The kernel variant a launch shape names (blocks of several steps exist for offsets that fit 32 bits only).
template <int V, int CPL, bool SOFTMAX, typename OutT>
static int launch_one(const SpmmShape &shape, int m_vec, int k, int n, const int *row_indices, const int *row_offsets,
                      const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                      hipStream_t stream, const Batch &batch, float scale)
{
    const int waves = shape.waves;
    const int per_wave = shape.blocks_per_wave;
#define VS_SPMM_VARIANT(...)                                                                                          \
    launch_idx<V, CPL, SOFTMAX, __VA_ARGS__>(m_vec, k, n, waves, row_indices, row_offsets, column_indices, values, rhs, \
                                             out, stream, batch, scale,
    if ((long long)n * k >= (1LL << 31)) return VS_SPMM_VARIANT(false, OutT) 1, -1);
    if constexpr (SOFTMAX) {
        if (shape.steps_in_flight >= 2) return VS_SPMM_VARIANT(true, OutT, 2) per_wave, -1);
    } else {
#ifdef VS_RETIRED_VARIANTS
        if (shape.steps_in_flight == 4) return VS_SPMM_VARIANT(true, OutT, 4) per_wave, -1);
#endif
        if (shape.steps_in_flight >= 2) {
            // (only the two-step variants have the team mapping and the pipelined walk)
            if (shape.team_slots >= 0)
                return shape.pipelined ? VS_SPMM_VARIANT(true, OutT, 2, true, true) per_wave, shape.team_slots)
                                       : VS_SPMM_VARIANT(true, OutT, 2, true, false) per_wave, shape.team_slots);
            return shape.pipelined ? VS_SPMM_VARIANT(true, OutT, 2, false, true) per_wave, -1)
                                   : VS_SPMM_VARIANT(true, OutT, 2, false, false) per_wave, -1);
        }
    }
    return VS_SPMM_VARIANT(true, OutT) 1, -1);
#undef VS_SPMM_VARIANT
}

template <int CPL, bool SOFTMAX, typename OutT>
static int launch_v(const SpmmShape &shape, int vec_length, int m_vec, int k, int n, const int *row_indices,
                    const int *row_offsets, const int *column_indices, const half_t *values, const half_t *rhs,
                    OutT *out, hipStream_t stream, const Batch &batch, float scale)
{
    switch (vec_length) {
    case 1: return launch_one<1, CPL, SOFTMAX, OutT>(shape, m_vec, k, n, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch, scale);
    case 2: return launch_one<2, CPL, SOFTMAX, OutT>(shape, m_vec, k, n, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch, scale);
    case 4: return launch_one<4, CPL, SOFTMAX, OutT>(shape, m_vec, k, n, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch, scale);
    case 8: return launch_one<8, CPL, SOFTMAX, OutT>(shape, m_vec, k, n, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch, scale);
    default: return hipErrorInvalidValue;
    }
}

// The launch shape of an MFMA SpMM, chosen on the host from what the entry point knows of the problem (the row
// lengths only through the hints of the batched entry points) and from the calling thread's options.
SpmmShape choose_spmm_shape(bool softmax, int m_vec, int vec_length, int k, int n, const Batch &batch)
{
    SpmmShape shape;
    constexpr int kTargetBlocks = 256;   // one workgroup per CU at least
    constexpr int kTargetWaves = 4096;
    int cpl = options().spmm_cols_per_lane;
#ifdef VS_RETIRED_VARIANTS
    const bool use_dma = !softmax && options().spmm_gather == 2 && k % 8 == 0;
#else
    const bool use_dma = false;  // (the LDS-DMA gather and four steps in flight are compiled only with VS_RETIRED_VARIANTS)
#endif
    if (use_dma) cpl = 8;
    const bool hinted = batch.nonzeros_vec >= 0;
    int mean_steps = hinted ? ceil_div(ceil_div(batch.nonzeros_vec, m_vec), kStep) : ceil_div(n, 4 * kStep);
    const int longest_steps = ceil_div(batch.longest_row_vec > 0 ? batch.longest_row_vec : 0, kStep);
    // a few rows far longer than the mean (known only to the batched entry points)
    const bool skewed = hinted && longest_steps > 4 * mean_steps && longest_steps > 16;
    if (cpl != 4 && cpl != 8) {
        const long long blocks128 = (long long)m_vec * ceil_div(k, 128) * batch.count;
        // Skewed rows keep the narrow tile until the grid is four workgroups per CU: the long rows then spread over
        // twice the workgroups (256 rows, Pareto or one dense row among short ones, N = 256: 12.4 -> 11.4 us).
        const long long enough = skewed ? 4 * kTargetBlocks : kTargetBlocks;
        cpl = (k % 8 == 0 && k > 64 && blocks128 >= enough) ? 8 : 4;  // k <= 64 fits one 64-column tile
    }
    if (cpl == 8 && k % 8 != 0) cpl = 4;
    const bool ragged = k % 4 != 0;
    if (ragged) cpl = 4;
    const long long blocks = (long long)m_vec * ceil_div(k, 16 * cpl) * batch.count;
    // Row lengths unknown on a grid of at most a workgroup per CU: the rows are taken to hold half of n rather than a
    // quarter - there a wave that a shorter row leaves idle costs next to nothing, and a row of two blocks served by
    // one wave 9 % (128 rows x 147 at 50 %, N = 256: 2.66 us with one wave, 2.44 us with two).
    if (!hinted && blocks <= kTargetBlocks) mean_steps = ceil_div(n, 2 * kStep);
    // Steps of gathered rows a wave keeps in flight.  Two pay as soon as rows hold more than one step: the wave
    // waits once for 64 vectors instead of twice (ResNet-shaped grid, 16 to 2304 vectors per row, N = 64 and 256:
    // 5-20 % faster than one step at the best wave count of each; 3 % slower on rows of under 32 vectors).  Four
    // pay 2-4 % more on large problems with 128-bit segments and cost up to 14 % on rows of one or two steps, so
    // they are chosen only when the row lengths are known.  The unhinted entry takes the rows to hold a quarter of
    // n: the kernel leaves the waves that a shorter row does not need idle at little cost (1.5 % per doubling
    // of the workgroup beyond four waves), while too few waves for denser rows cost 10-18 %.
    // while the chip has room the workgroup of the longest row ends last, so that row sets the size
    const int row_steps = longest_steps > mean_steps ? longest_steps : mean_steps;
    const bool blocks_exist = !ragged && !use_dma && (long long)n * k < (1LL << 31);
    int in_flight = options().spmm_steps;
#ifndef VS_RETIRED_VARIANTS
    if (in_flight == 4) in_flight = 0;
#endif
    if (in_flight != 1 && in_flight != 2 && in_flight != 4) {
        in_flight = row_steps >= 2 ? 2 : 1;
        // Many heads of a large mask with vectors of one or two rows (16384 workgroups and more, every one a single
        // wave): such a launch is bound by its gather requests, and a row's last block of 64 is half padding on
        // average - 16 requested slots per row that a walk in steps of 32 does not issue.  16 heads x 4096 rows, N = 64,
        // V = 1: rows of 82 / 205 / 410 vectors 62.4 -> 50.0, 120.9 -> 109.8, 208.6 -> 201.1 us; V = 2, 205: 63.2 ->
        // 58.5; V = 4 and 8 are the other way round (rows of 102, V = 4: 11.8 against 12.8 us).
        if (hinted && vec_length <= 2 && blocks >= 16384 && mean_steps <= 16) in_flight = 1;
        // (rows of unequal length end in half-empty blocks of 128: on log-normal and Pareto lengths four steps in
        // flight were 10-25 % behind two)
#ifdef VS_RETIRED_VARIANTS
        if (options().spmm_pipe == 1 && hinted && cpl == 8 && blocks >= 512 && mean_steps >= 8 &&
            2 * longest_steps <= 3 * mean_steps)
            in_flight = 4;  // (only without the pipelined walk, which is 5-15 % ahead of it on the same shapes)
#endif
    }
    if (!blocks_exist) in_flight = 1;
    // The softmax-fused kernel has the two-step blocks only, and gains from them on rows of more than two blocks
    // of vectors of four or eight (16 heads x 4096, d = 64: band + strided mask 37.2 -> 31.0 us, uniform 90 % 44.5 ->
    // 39.2 us; rows of 82 vectors 15.8 -> 16.4 us, V = 1 at 95 % 114 -> 125 us).
    if (softmax && in_flight == 4) in_flight = 2;
    if (softmax && options().spmm_steps == 0 && (vec_length < 4 || row_steps <= 4)) in_flight = 1;
    int per_wave = 1;
    int team_slots = -1;
    int waves = options().spmm_waves;
    if (waves <= 0 && in_flight > 1) {
        // One wave per block of the (estimated) row, as far as the launch stays resident at once; waves that a
        // shorter row leaves without a block end at once.
        const int row_blocks = ceil_div(row_steps, in_flight);
        int want = row_blocks <= 1 ? 1 : next_pow2(row_blocks);
        // Eight waves at most: with pipelined walks eight waves that take two blocks and more each are ahead of
        // sixteen with one each also where the rows are known to fill all sixteen (64 rows x 4608, N = 256, rows of
        // 922 / 2304 vectors: 4.2 against 4.7 and 7.2 against 7.6 us), and sixteen-wave workgroups cost 3.5 % on rows
        // that fill eight or fewer.  (The skewed launches below size theirs themselves.)
        if (want > 8) want = 8;
        const int registers = in_flight * cpl;                                 // in flight per lane, of 32 bits / 2
        const int resident = (registers >= 32 ? 2 : registers >= 16 ? 3 : 5) * 1024;   // waves the chip holds at once
        int room = 1;
        while (2LL * room * blocks <= resident) room <<= 1;
        // Three and a half to four workgroups per CU: with one wave each every SIMD holds one wave and the launch is
        // a single even round, which a second wave per row (and the sum through LDS it brings) only slows down - rows
        // of 230 / 461 / 922 vectors, N = 256, on 896 and 1024 workgroups: V = 1 and 2 one wave 9-13 % ahead of two,
        // V = 4 3-12 %, V = 8 2-7 %; from 1152 to 1536 workgroups two waves are 1-3 % ahead again.
        if (blocks > 800 && blocks <= 1024) room = 1;
        waves = want < room ? want : room;
        // Row lengths unknown and the grid alone fills the chip: the workgroups still get a few waves, of which a
        // row of the expected length uses `room` (a wave takes want / room of its blocks); a row far longer than
        // expected spreads over all of them instead of holding one wave for the whole launch (1024 Pareto rows x
        // 4608, N = 256: 39 -> 15 us with four waves, 23 us with two; one dense row among 1023 short ones 39 -> 14 us).
        // The waves a row does not need end after reading the row's extent, but hold a wave slot until then:
        // 0.3-0.5 us per thousand of them.  Four waves against two, N = 256, K = 4608: on 2048 workgroups uniform rows
        // 4-16 % slower and Pareto / log-normal / one dense row 18-43 % faster; on 4096 workgroups uniform rows 0-4 %
        // slower, the skewed ones 8-39 % faster; on 8192 workgroups uniform rows up to 15 % slower and only the single
        // dense row faster - so grids beyond 4096 workgroups get two.
        int guard = options().spmm_guard_waves;
        if (guard <= 0) guard = blocks <= 4096 ? 4 : 2;
        // A wave takes half the blocks the estimate gives a row before a second one joins (four, for the eight the
        // cap allows on a full chip): with pipelined walks a second wave pays from there, the idle ones cost more
        // than the sum through LDS (N = 256, K = 4608, 1024 / 2048 rows; 2 / 4 / 8 / 16 blocks per wave: uniform rows at
        // 90 % 14.2 / 14.6 / 15.4 / 15.4 and 25.9 / 26.4 / 26.4 / 26.2 us, log-normal 13.8 / 13.5 / 13.4 / 15.5 and 26.3 /
        // 25.7 / 25.0 / 25.2, Pareto 14.9 / 14.8 / 14.5 / 15.1 and 19.1 / 19.0 / 18.5 / 19.8; 98 % and 50 % the same within
        // 1 %).  Matrices too narrow for a row of more than twelve blocks need no guard at all.
        if (!hinted && want > room && guard > room && ceil_div(ceil_div(n, kStep), in_flight) > 12) {
            const int launched = want < guard ? want : guard;
            per_wave = options().spmm_blocks_per_wave > 0 ? options().spmm_blocks_per_wave : (want >= 4 * room ? want / (2 * room) : 1);
            waves = launched;
        }
        // A few rows far longer than the mean (lengths known): the average row keeps to the waves the chip has room
        // for - a wave takes several of its blocks when the grid is full - and the longest row spreads over as many
        // waves as its blocks ask for at that rate, within a budget of launched waves (the waves a row does not
        // need end after reading its extent, at 0.3 us per thousand; where the average row itself fills more than
        // six waves the budget is half - log-normal lengths, 1024 rows: 17.4 us with four waves, 20.5 us with eight).
        if (skewed) {
            const int mean_blocks = ceil_div(mean_steps, in_flight);
            const int typical = mean_blocks <= 1 ? 1 : next_pow2(mean_blocks);
            const int base = typical < room ? typical : room;
            per_wave = typical / base;
            const long long budget = mean_blocks <= 6 ? 16384 : 8192;
            int cap = 16;
            while (cap > 4 && blocks * cap > budget) cap >>= 1;
            int for_longest = next_pow2(ceil_div(ceil_div(longest_steps, in_flight), per_wave));
            if (for_longest > cap) for_longest = cap;
            waves = base > for_longest ? base : for_longest;
        }
        // Rows ordered by length and the count of long ones known (batch.long_rows: the leading entries of
        // row_indices whose rows hold more than 512 vectors), on a grid of sixteen workgroups per CU or more whose
        // other rows are short: only the long rows get a team of waves - the longest at about eight blocks per
        // wave - and every other row one wave of a workgroup that takes as many rows as it has waves.  No wave is
        // launched without work (the launches above hand every row the team that only the long ones need, at
        // 0.3 us per thousand waves that end at once), but a lone wave walks its row's blocks one after the other.
        // Measured, N = 256, V = 8, 1 to 5 % of the rows between 1500 and 4608 vectors long among rows of 50 to 400:
        // 2048 rows of 50 to 150 vectors 4-18 % faster, 4096 rows of 50 to 100 vectors 5-12 % faster while the
        // long rows are 1 % or fewer; slower where the other rows are longer (200 to 300 vectors: 5-15 %), on
        // 4096 rows with 5 % long ones (8 %) and on smaller grids (512 rows of 100: 6.2 -> 7.6 us; 1024 rows: the
        // same within 3 %).  The other rows' mean length is bounded from what the hints say: every long row holds
        // 513 vectors at least.
        bool teams_pay = false;
        if (skewed && batch.long_rows > 0 && batch.long_rows < m_vec && blocks >= 4096) {
            const long long in_long = 513LL * batch.long_rows + (batch.longest_row_vec > 513 ? batch.longest_row_vec - 513 : 0);
            const long long others = batch.nonzeros_vec > in_long ? batch.nonzeros_vec - in_long : 0;
            const int others_mean = (int)(others / (m_vec - batch.long_rows));
            const int others_blocks = ceil_div(ceil_div(others_mean, kStep), 2);
            teams_pay = blocks < 8192 ? others_blocks <= 3 : (others_blocks <= 2 && 100LL * batch.long_rows <= m_vec);
        }
        if (batch.long_rows > 0 && options().spmm_teams != 1 && (teams_pay || options().spmm_teams == 2)) {
            team_slots = batch.long_rows < m_vec ? batch.long_rows : m_vec;
            per_wave = 1;
            if (in_flight == 4) in_flight = 2;
            int team = team_slots > 0 ? next_pow2(ceil_div(ceil_div(longest_steps, in_flight), 8)) : 4;
            waves = team < 4 ? 4 : (team > 16 ? 16 : team);
        }
    }
    if (waves <= 0) {
        waves = next_pow2((int)((kTargetWaves + blocks - 1) / blocks));
        if (hinted) {
            // Row lengths known: a wave is worth launching for about three 32-vector steps (measured over
            // the ResNet-shaped grid: within 0.4 % of the best power of two, 7 % better than sizing by n).
            const int by_rows = next_pow2(ceil_div(row_steps > 0 ? row_steps : 1, 3));
            if (waves > by_rows) waves = by_rows;
            // a second wave per row pays on a full chip from about ten steps per row (256 to 2048 vector rows,
            // N = 256 to 1024: one wave 3-8 % ahead at 4 to 8 steps, two waves 3-10 % ahead at 12 and more)
            if (waves < 2 && mean_steps >= 10) waves = 2;
            // A few rows far longer than the mean: a wave takes about half a microsecond per step of a lone
            // long row, so that row gets at most sixteen steps per wave - as far as the idle waves this hands
            // to every short row stay cheap (16384 waves per launch, or four per row).  Measured on 1024
            // Pareto-distributed rows (mean 280, longest 4608 vectors, N = 256): 40 us with two waves per row,
            // 15.8 us with the eight chosen here, 9.7 us for uniform rows.
            if (skewed) {
                int cap = 16;
                while (cap > 4 && blocks * cap > 16384) cap >>= 1;
                int for_longest = next_pow2(ceil_div(longest_steps, 16));
                if (for_longest > cap) for_longest = cap;
                if (waves < for_longest) waves = for_longest;
            }
        } else {
            const int max_useful = next_pow2(ceil_div(n > 0 ? n : 1, kStep));  // a row holds at most n vectors
            if (waves > max_useful) waves = max_useful;
            // On a full chip a second wave per row pays from about ten steps per row (see above); the row
            // lengths are unknown here, so they are taken to be a tenth of n (90 % sparsity).
            if (waves < 2 && n >= 100 * kStep) waves = 2;
        }
    }
    if (waves < 1) waves = 1;
    if (waves > 16) waves = 16;
    // launch bounds of the variants with 64 / 128 registers of row segments in flight
    if (in_flight * cpl >= 16 && waves > 8) waves = 8;
    if (in_flight * cpl >= 32 && waves > 4) waves = 4;
    if (ragged && waves > 8) waves = 8;  // 8 x 2.7 KB of LDS stay below the default limit of dynamic LDS
    shape.cols_per_lane = cpl;
    shape.steps_in_flight = in_flight;
    shape.waves = waves;
    shape.blocks_per_wave = per_wave;
    shape.team_slots = team_slots;
    // The pipelined walk (two-step blocks): a wave that takes several blocks of a row one after the other requests
    // the next block's segments step by step behind the multiplications instead of after them - 10-20 % on waves that
    // walk many blocks where the launch is not at the gather ceiling anyway, at 26 more registers.  Measured over
    // the ResNet-shaped grid (geometric means by grid size and row length, against the plain walk): with the row
    // lengths known 2-4 % faster on rows of two to eight blocks and 7-14 % on longer ones from 512 workgroups on,
    // the same within 1 % on rows of one block, 1-3 % slower only on rows of two blocks across 4096 workgroups;
    // without hints 1.5-2.5 % faster up to 2048 workgroups (rows of 230 vectors and more on 2048 workgroups 6-12 %)
    // and 2.5 % slower on 4096, where one guard wave walks each row at the gather ceiling - taken there too, for the
    // rows that the guard waves exist for: 1024 to 4096 Pareto rows are 4-11 % faster hinted, 12-19 % without hints.  It also outruns four steps in flight (5-15 % on the
    // shapes that used to take them), which the automatic choice therefore no longer takes.
    bool pipelined = false;
    if (in_flight == 2 && blocks_exist && !softmax && options().spmm_pipe != 1) {
        if (options().spmm_pipe == 2) {
            pipelined = true;
        } else if (hinted) {
            const int longest_blocks = ceil_div(row_steps, in_flight);
            pipelined = longest_blocks >= 3 || blocks < 4096;  // (its single-block path is the plain one)
        } else {
            pipelined = true;  // (on 4096 workgroups: uniform rows 2.5 % slower, Pareto rows 12-19 % faster)
        }
    }
    shape.pipelined = pipelined;
    shape.ragged = ragged;
    shape.dma = use_dma && !ragged;
    return shape;
}

template <bool SOFTMAX, typename OutT>
static int launch_any(int m_vec, int vec_length, int k, int n, const int *row_indices,
                      const int *row_offsets, const int *column_indices, const half_t *values,
                      const half_t *rhs, OutT *out, hipStream_t stream, const Batch &batch, float scale)
{
    if (m_vec == 0 || k == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535) return hipErrorNotSupported;
    if (SOFTMAX && k % 4 != 0) return hipErrorNotSupported;
    const SpmmShape shape = choose_spmm_shape(SOFTMAX, m_vec, vec_length, k, n, batch);
    const int waves = shape.waves;
    if constexpr (!SOFTMAX) {
        if (shape.ragged) {
            switch (vec_length) {
            case 1: return launch_ragged<1, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
            case 2: return launch_ragged<2, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
            case 4: return launch_ragged<4, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
            case 8: return launch_ragged<8, OutT>(m_vec, k, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
            default: return hipErrorInvalidValue;
            }
        }
#ifdef VS_RETIRED_VARIANTS
        if (shape.dma)
            return launch_spmm_mfma_dma<OutT>(m_vec, vec_length, k, n, waves, row_indices, row_offsets, column_indices,
                                              values, rhs, out, stream, batch);
#endif
    }
    if (shape.cols_per_lane == 8)
        return launch_v<8, SOFTMAX, OutT>(shape, vec_length, m_vec, k, n, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch, scale);
    return launch_v<4, SOFTMAX, OutT>(shape, vec_length, m_vec, k, n, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch, scale);
}

template <typename OutT>
int launch_spmm_mfma(int m_vec, int vec_length, int k, int n, const int *row_indices,
                     const int *row_offsets, const int *column_indices, const half_t *values,
                     const half_t *rhs, OutT *out, hipStream_t stream, const Batch &batch)
{
    return launch_any<false, OutT>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs,
                                   out, stream, batch, 1.f);
}

int launch_spmm_softmax_mfma(int m_vec, int vec_length, int k, int n, const int *row_indices,
                             const int *row_offsets, const int *column_indices, const half_t *scores,
                             const half_t *rhs, half_t *out, float scale, hipStream_t stream, const Batch &batch)
{
    return launch_any<true, half_t>(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, scores, rhs,
                                    out, stream, batch, scale);
}

// Rows in parts (the kernel's PARTS variant): `slots` is the dispatch list of vs_spmm_row_parts in device memory,
// the workspace holds the arrival counters of the split rows and their fp32 partial tiles.
namespace {

template <int V, int CPL, bool PIPE>
int launch_parts_kernel(int k, int n_slots, int n_split, bool two_launches, int waves, int per_wave, const int *slots,
                        int parts_max, const int *column_indices, const half_t *values, const half_t *rhs, half_t *out,
                        int *counters, float *tiles, hipStream_t stream, const Batch &batch)
{
    int per_wave_log2 = 0;
    while ((2 << per_wave_log2) <= per_wave) ++per_wave_log2;
    constexpr int TN = 16 * CPL;
    const int n_tiles = ceil_div(k, TN);
    const long long blocks = (long long)n_slots * n_tiles;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    const size_t lds = (size_t)waves * 2 * stage_bytes<V>() + (waves > 1 ? (size_t)waves * V * (TN + 1) * sizeof(float) : 0);
    auto kernel = spmm_mfma_kernel<V, CPL, false, true, half_t, false, 2, false, PIPE, true>;
    static std::atomic<unsigned long long> lds_allowed{0};
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 96 * 1024, lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * waves), lds, stream, k, n_tiles,
                       per_wave_log2 | (waves << 8) | (blocks * batch.count >= 512 ? 1 << 16 : 0) | (two_launches ? 1 << 17 : 0),
                       slots, static_cast<const int *>(nullptr), column_indices, values, rhs, out, batch.stride_a, batch.stride_b,
                       batch.stride_out, 1.f, n_split, n_slots, counters, tiles, parts_max);
    const hipError_t st = hipGetLastError();
    if (st != hipSuccess || !two_launches || n_split == 0) return (int)st;
    hipLaunchKernelGGL((spmm_row_parts_sum_kernel<V, CPL>), dim3((unsigned)(n_split * n_tiles), (unsigned)batch.count),
                       dim3(V * 16 < 64 ? 64 : V * 16), 0, stream, k, n_tiles, slots + 4 * (size_t)n_slots, n_split, parts_max,
                       tiles, out, batch.stride_out);
    return (int)hipGetLastError();
}

template <int V>
int launch_parts_v(const SpmmShape &shape, int k, int n_slots, int n_split, bool two_launches, const int *slots,
                   int parts_max, const int *column_indices, const half_t *values, const half_t *rhs, half_t *out,
                   int *counters, float *tiles, hipStream_t stream, const Batch &batch)
{
#define VS_PARTS_VARIANT(CPL, PIPE)                                                                                \
    launch_parts_kernel<V, CPL, PIPE>(k, n_slots, n_split, two_launches, shape.waves, shape.blocks_per_wave, slots, \
                                      parts_max, column_indices, values, rhs, out, counters, tiles, stream, batch)
    if (shape.cols_per_lane == 8) return shape.pipelined ? VS_PARTS_VARIANT(8, true) : VS_PARTS_VARIANT(8, false);
    return shape.pipelined ? VS_PARTS_VARIANT(4, true) : VS_PARTS_VARIANT(4, false);
#undef VS_PARTS_VARIANT
}

}  // namespace

long long spmm_row_parts_workspace_bytes(int batch, int vec_length, int k, int n_split, int parts_max)
{
    if (batch <= 0 || n_split <= 0 || parts_max <= 0 || k <= 0) return 0;
    const long long k_pad = (long long)ceil_div(k, 128) * 128;  // whole tiles of either width
    return row_parts_workspace_for((long long)batch * n_split * parts_max * vec_length * k_pad * (long long)sizeof(float));
}

int launch_spmm_mfma_row_parts(int vec_length, int k, int n, int n_slots, const int *slots, int n_split, int parts_max,
                               int nonzeros_vec, int longest_part_vec, const int *column_indices, const half_t *values,
                               const half_t *rhs, half_t *out, void *workspace, long long workspace_bytes,
                               hipStream_t stream, const Batch &batch)
{
    if (n_slots == 0 || k == 0 || batch.count == 0) return hipSuccess;
    if (batch.count > 65535 || (long long)batch.count * n_split > 0x7fffffffLL / 256) return hipErrorNotSupported;
    if (k % 4 != 0 || (long long)n * k >= (1LL << 31)) return hipErrorNotSupported;  // whole chunks, 32-bit offsets
    if (n_split > 32767 || parts_max > 255 || (n_split > 0 && parts_max < 2)) return hipErrorInvalidValue;
    const long long need = spmm_row_parts_workspace_bytes(batch.count, vec_length, k, n_split, parts_max);
    if (need > workspace_bytes || need - row_parts_counter_bytes(need) >= (1LL << 31)) return hipErrorNotSupported;
    Batch hints = batch;
    hints.nonzeros_vec = nonzeros_vec;
    hints.longest_row_vec = longest_part_vec;
    hints.long_rows = -1;
    SpmmShape shape = choose_spmm_shape(false, n_slots, vec_length, k, n, hints);
    if (shape.ragged || shape.dma) return hipErrorNotSupported;
    if (k % 8 != 0) shape.cols_per_lane = 4;
    if (shape.steps_in_flight != 2) {  // the variant exists for blocks of two steps
        shape.steps_in_flight = 2;
        shape.pipelined = false;
        shape.blocks_per_wave = 1;
    }
    // A list with split rows is cut off at the limit, which the rules for whole rows misread (they size the
    // workgroups by the mean row or by how far the longest row stands out).  Measured at N = 256, V = 8, K = 4608,
    // limits of 768-1536 vectors, 64 to 2048 rows of Pareto or log-normal lengths or with one dense row (2 / 4 / 8
    // waves, us): 39 K-214 K block steps of work 9.4-12.0 / 8.2-9.6 / 7.8-8.8; 418 K-933 K 12.6-15.1 / 10.2-14.8 /
    // 14.4-21.3; 1.18 M 17.7 / 19.9 / 29.6 - the waves that short slots leave idle cost what the long ones gain
    // once the launch holds enough work.
    if (n_split > 0 && options().spmm_waves == 0) {
        const long long work = (long long)nonzeros_vec * ceil_div(k, 128) * batch.count;
        shape.waves = work <= (256LL << 10) ? 8 : work <= (1LL << 20) ? 4 : 2;
        shape.blocks_per_wave = options().spmm_blocks_per_wave > 0 ? options().spmm_blocks_per_wave : 1;
        shape.pipelined = options().spmm_pipe != 1;
    }
    // The meeting inside the launch costs the last part of a row three memory round trips, a second launch costs a
    // launch: small problems are ahead with the second launch (64 / 256 Pareto rows 6.8 / 7.9 against 7.7 / 8.6 us, a
    // dense row among 63 / 255 short ones 6.8 / 7.0 against 7.8 / 7.8), from about 200 K block steps on the one launch
    // is (a dense row among 1023: 8.8 against 10.7 us; 1024 Pareto rows 11.0 against 13.1).
    const bool two_launches =
        options().spmm_parts_launches == 2 ||
        (options().spmm_parts_launches == 0 && n_split > 0 &&
         (long long)nonzeros_vec * ceil_div(k, 128) * batch.count <= 160 * 1024);
    int *counters = static_cast<int *>(workspace);
    float *tiles = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) +
                                             (n_split > 0 ? row_parts_counter_bytes(workspace_bytes) : 0));
    switch (vec_length) {
    case 1: return launch_parts_v<1>(shape, k, n_slots, n_split, two_launches, slots, parts_max, column_indices, values, rhs, out, counters, tiles, stream, batch);
    case 2: return launch_parts_v<2>(shape, k, n_slots, n_split, two_launches, slots, parts_max, column_indices, values, rhs, out, counters, tiles, stream, batch);
    case 4: return launch_parts_v<4>(shape, k, n_slots, n_split, two_launches, slots, parts_max, column_indices, values, rhs, out, counters, tiles, stream, batch);
    case 8: return launch_parts_v<8>(shape, k, n_slots, n_split, two_launches, slots, parts_max, column_indices, values, rhs, out, counters, tiles, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

template int launch_spmm_mfma<half_t>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                      const half_t *, half_t *, hipStream_t, const Batch &);
template int launch_spmm_mfma<float>(int, int, int, int, const int *, const int *, const int *, const half_t *,
                                     const half_t *, float *, hipStream_t, const Batch &);

}  // namespace vs
