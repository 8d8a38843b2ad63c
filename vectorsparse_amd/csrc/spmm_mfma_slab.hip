// SpMM on fp16 MFMA with the dense operand staged in LDS once per block of vector rows (the reference's tile loop,
// src/wmma_spmm.cu:77-90 with src/spmm_utils/sparse_tile.h:259-272 and dense_tile.h:255-259, fetches every
// nonzero's rhs row from memory; so does spmm_mfma_kernel, one L2 request per nonzero and lane group).
//
// Work item = (block of R = 8 vector rows, tile of 128 dense columns, part ks of the contraction); one workgroup of
// R waves, one vector row per wave.  Part ks of a row is positions [len * ks / ksplit, len * (ks + 1) / ksplit)
// of its nonzeros: with sorted columns the parts of the R rows cover about the same rows of the dense operand,
// and the workgroup walks that range in windows of 128 rhs rows:
//   * the window's 128 x 128 halves are loaded dense and coalesced (128-bit loads, every rhs row segment once per
//     workgroup instead of once per nonzero), held in registers while the previous windows are worked on, and
//     written to LDS row-major with a pitch of 256 bytes (two windows resident, rhs row r at slot r % 256);
//   * each wave walks its own row's nonzeros.  A step takes the next 32 of them when all their rhs rows are
//     resident - steps cross window borders - and fewer (the slots past them zeroed) only when the oldest resident
//     window is about to be replaced; lane (cs, g) reads the 16 bytes at columns 8 cs.. of rows 8 g .. 8 g + 7 of
//     the step from LDS (the sixteen lanes of a group read one 256-byte row: every bank once), transposes the 8 x 8
//     block with v_perm_b32 and issues eight v_mfma_f32_16x16x32_f16, exactly as spmm_mfma_step does with rows it
//     fetched from memory;
//   * column indices and value vectors come through a wave-private ring in LDS (three chunks of 64 nonzeros, fetched
//     a window ahead), read by the steps at any alignment.
// The sum over a row's nonzeros is taken in CSR order whatever the columns are.  Columns need not be sorted: a step
// whose first nonzero lies in a window that has already left LDS (never the case for sorted columns) fetches its rows
// from memory instead, and so does whatever is left when the last window is done.
// ksplit > 1: every workgroup leaves its rows' fp32 tiles in a workspace and a second launch adds the parts of a row in
// ascending order, converts and writes the row (nothing in the workspace has to be cleared, before or after).
//
// Measured and NOT chosen by any other entry point (vs_wmma_spmm_f16_slab runs it): on 2048 x 4608 x 256, V = 8, at 50 % sparsity the
// launch takes 31 us against 15.6 us for spmm_mfma_kernel - see the notes on the launcher below.
#include <type_traits>

#include "spmm_mfma_step.hpp"
#include "vs_common.hpp"

namespace vs {

constexpr int kSlabRows = 8;                               // vector rows (= waves) per workgroup
constexpr int kSlabTile = 128;                             // dense columns per workgroup
constexpr int kSlabWindow = 128;                           // rhs rows per window
constexpr int kSlabRowBytes = kSlabTile * 2;               // LDS pitch of a resident rhs row
constexpr int kSlabBytes = 2 * kSlabWindow * kSlabRowBytes;  // two resident windows
constexpr int kRingChunk = 64;                             // nonzeros per fetch of a wave
constexpr int kRingChunks = 3;
constexpr int kRingSlots = kRingChunks * kRingChunk + kStep;  // the first 32 slots are repeated behind the last

template <int V>
constexpr int slab_ring_bytes()
{
    return kRingSlots * (4 + 2 * V);
}
template <int V, int R>
constexpr int slab_lds_bytes()
{
    return kSlabBytes + R * slab_ring_bytes<V>() + 16;
}

// R: vector rows (= waves) per workgroup.
template <int V, int R>
__global__ void __launch_bounds__(64 * R)
spmm_mfma_slab_kernel(int n_cols, int n_tiles, int m_vec, int ksplit, int n_rows, const int *__restrict__ row_indices,
                      const int *__restrict__ row_offsets, const int *__restrict__ column_indices,
                      const half_t *__restrict__ values, const half_t *__restrict__ rhs, half_t *__restrict__ out,
                      float *tiles)
{
    extern __shared__ __align__(16) unsigned char smem[];  // resident windows, then the waves' rings, then 4 ints
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cs = lane & 15;
    const int g = lane >> 4;
    // consecutive workgroups (which the dispatcher deals round-robin to the eight XCDs) take different parts of the
    // contraction: a multiple of eight parts keeps each part's rhs rows in one XCD's L2
    const int ks = blockIdx.x % ksplit;
    const int tile = (blockIdx.x / ksplit) % n_tiles;
    const int rb = (blockIdx.x / ksplit) / n_tiles;
    int *ring_idx = reinterpret_cast<int *>(smem + kSlabBytes + wave * slab_ring_bytes<V>());
    half_t *ring_vec = reinterpret_cast<half_t *>(ring_idx + kRingSlots);
    int *shared = reinterpret_cast<int *>(smem + kSlabBytes + R * slab_ring_bytes<V>());
    if (threadIdx.x == 0) {
        shared[0] = 0x7fffffff;  // first rhs row any wave of the workgroup needs
        shared[1] = -1;          // last one
    }
    const int slot = rb * R + wave;
    const bool has_row = slot < m_vec;
    int row = 0, beg = 0, end = 0;
    if (has_row) {
        row = row_indices[slot];
        beg = row_offsets[row];
        end = row_offsets[row + 1];
    }
    __syncthreads();
    // this part of the row: positions [lo, hi)
    const uint32_t len = (uint32_t)(end - beg);
    const uint32_t per = len / (uint32_t)ksplit, extra = len % (uint32_t)ksplit;
    const int lo = beg + (int)(per * ks + ((uint32_t)ks < extra ? (uint32_t)ks : extra));
    const int hi = lo + (int)per + ((uint32_t)ks < extra ? 1 : 0);
    const int n_chunks = (hi - lo + kRingChunk - 1) / kRingChunk;

    struct Cand {
        int idx;
        PackedVector<V> vec;
    };
    // (requested whether or not the chunk exists - past the part's end the lanes re-read its last nonzero, an empty part
    // reads position 0 - so that every turn has the same number of loads in flight and the waits count exactly)
    auto load_chunk = [&](int c, Cand &r) {
        int j = lo + kRingChunk * c + lane;
        j = j < hi ? j : hi - 1;
        j = j < 0 ? 0 : j;
        r.idx = column_indices[j];
        r.vec.load(values + (size_t)j * V);
    };
    auto write_chunk = [&](int c, const Cand &r) {
        const int at = (c % kRingChunks) * kRingChunk + lane;
        ring_idx[at] = r.idx;
        r.vec.store(ring_vec + at * V);
        if (c % kRingChunks == 0 && lane < kStep) {  // the copy that lets a step read 32 slots in a row from any slot
            ring_idx[kRingChunks * kRingChunk + lane] = r.idx;
            r.vec.store(ring_vec + (kRingChunks * kRingChunk + lane) * V);
        }
        wave_lds_fence();
    };
    int loaded = 0;  // chunks in the ring so far
    {
        Cand c0, c1;
        int last_col = -1;
        load_chunk(0, c0);
        load_chunk(1, c1);
        if (hi > lo) last_col = column_indices[hi - 1];
        if (n_chunks > 0) {
            write_chunk(0, c0);
            loaded = 1;
            const int first_col = __builtin_amdgcn_readfirstlane(c0.idx);
            if (lane == 0) {
                atomicMin(&shared[0], first_col);
                atomicMax(&shared[1], last_col);
            }
        }
        if (n_chunks > 1) {
            write_chunk(1, c1);
            loaded = 2;
        }
    }
    __syncthreads();
    const int k_min = shared[0];
    const int k_max = shared[1] < n_rows ? shared[1] : n_rows - 1;

    const int col0 = tile * kSlabTile + cs * 8;  // the lane's 16 bytes of a row, and its 8 output columns
    const bool col_ok = col0 < n_cols;           // n_cols % 8 == 0: all in or all out
    const uint32_t col_off = col_ok ? col0 : 0;
    // a window is 128 rows x 16 pieces of 16 bytes; thread x takes pieces x, x + 64 R, .. (piece q: row q / 16, the
    // lane's own 8 columns); the last turn is cut for R = 12 (wave-uniformly: 64 R is a multiple of 64)
    constexpr int kPieces = kSlabWindow * 16;
    constexpr int kFill = (kPieces + 64 * R - 1) / (64 * R);
    auto load_window = [&](int t, uint4_t (&f)[kFill]) {
#pragma unroll
        for (int i = 0; i < kFill; ++i) {
            const int q = (int)threadIdx.x + i * 64 * R;
            int r = t * kSlabWindow + ((q >> 4) & (kSlabWindow - 1));
            r = r < n_rows ? r : n_rows - 1;
            f[i] = *reinterpret_cast<const uint4_t *>(rhs + ((uint32_t)r * (uint32_t)n_cols + col_off));
        }
    };
    auto write_window = [&](int t, const uint4_t (&f)[kFill]) {
#pragma unroll
        for (int i = 0; i < kFill; ++i) {
            const int q = (int)threadIdx.x + i * 64 * R;
            if (kPieces % (64 * R) == 0 || i + 1 < kFill || q < kPieces)
                *reinterpret_cast<uint4_t *>(smem + (((t & 1) * kSlabWindow + (q >> 4)) * kSlabRowBytes) + cs * 16) = f[i];
        }
    };

    float4_t acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = float4_t{0.f, 0.f, 0.f, 0.f};

    int p = lo;  // next position of the row
    int rp = 0;  // its slot in the ring
    auto advance = [&](int n) {
        p += n;
        rp += n;
        if (rp >= kRingChunks * kRingChunk) rp -= kRingChunks * kRingChunk;
    };
    // One step of n <= 32 nonzeros from ring slot rp on.  FULL: n == 32.  RESIDENT: their rhs rows are in LDS.
    // Slots past n read as zero vectors at the step's first column.
    auto step = [&](auto full_tag, auto resident_tag, int n, int first_col) {
        constexpr bool FULL = decltype(full_tag)::value;
        constexpr bool RESIDENT = decltype(resident_tag)::value;
        int cols[8];
        half8_t a = {0, 0, 0, 0, 0, 0, 0, 0};
        const int *ip = ring_idx + rp + 8 * g;
#pragma unroll
        for (int e = 0; e < 8; ++e) cols[e] = ip[e];
        if (cs < V) {
            const half_t *vp = ring_vec + (rp + 8 * g) * V + cs;
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = vp[e * V];
        }
        if constexpr (!FULL) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const bool keep = 8 * g + e < n;
                cols[e] = keep ? cols[e] : first_col;
                a[e] = keep ? a[e] : (half_t)0.f;
            }
        }
        RowChunk<8> chunk[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if constexpr (RESIDENT)
                chunk[e].d = *reinterpret_cast<const uint4_t *>(smem + (((uint32_t)cols[e] & 255u) << 8) + cs * 16);
            else
                chunk[e].load(rhs + ((uint32_t)cols[e] * (uint32_t)n_cols + col_off));
        }
        multiply_step<8>(chunk, a, acc);
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;
    // the next 32 positions (fewer at the end of the part or of what the ring holds): each lane's column
    auto candidates = [&](int &cnt) -> int {
        int avail = loaded * kRingChunk - (p - lo);
        avail = hi - p < avail ? hi - p : avail;
        cnt = avail < kStep ? avail : kStep;
        return ring_idx[rp + (lane & 31)];
    };

    if (k_min <= k_max) {
        const int t0 = k_min / kSlabWindow, t1 = k_max / kSlabWindow;
        uint4_t f[kFill];
        load_window(t0, f);
        write_window(t0, f);
        __syncthreads();
        for (int t = t0; t <= t1; ++t) {
            // resident: windows t - 1 (from the second turn on) and t; window t - 1 leaves after this turn
            const int res_lo = (t > t0 ? t - 1 : t0) * kSlabWindow;
            const uint32_t res_span = (uint32_t)((t + 1) * kSlabWindow - res_lo);
            const int next_lo = t == t1 ? 0x7fffffff : t * kSlabWindow;
            // requested now, used at the end of the turn: the next chunks of the row, then the next window
            Cand pend0, pend1;
            int n_pending = 0;
            {
                const int consumed = (p - lo) / kRingChunk;
                if (loaded < n_chunks && loaded - consumed < kRingChunks) {
                    n_pending = 1;
                    if (loaded + 1 < n_chunks && loaded + 1 - consumed < kRingChunks) n_pending = 2;
                }
            }
            load_chunk(loaded, pend0);
            load_chunk(loaded + 1, pend1);
            load_window(t + 1, f);
            for (;;) {
                int cnt;
                const int col = candidates(cnt);
                if (cnt <= 0) {
                    if (p >= hi) break;
                    // the ring has run dry inside a turn (rows denser than a chunk per window)
                    if (n_pending > 0) {
                        write_chunk(loaded, pend0);
                        ++loaded;
                        if (n_pending > 1) {
                            write_chunk(loaded, pend1);
                            ++loaded;
                        }
                        n_pending = 0;
                    } else {
                        Cand now;
                        load_chunk(loaded, now);
                        write_chunk(loaded, now);
                        ++loaded;
                    }
                    continue;
                }
                const bool mine = (lane & 31) < cnt;
                const bool in = mine && (uint32_t)(col - res_lo) < res_span;
                const uint32_t m_in = (uint32_t)__builtin_amdgcn_ballot_w64(in);
                const int n_in = m_in == 0xffffffffu ? 32 : __builtin_ctz(~m_in);
                const int first_col = __builtin_amdgcn_readfirstlane(col);
                if (n_in == 0) {
                    if (first_col >= res_lo) break;  // not resident yet: a later turn
                    step(no(), no(), cnt, first_col);  // its window has left: from memory
                    advance(cnt);
                    continue;
                }
                const uint32_t m_leaving = (uint32_t)__builtin_amdgcn_ballot_w64(in && col < next_lo);
                int n = cnt;
                if (n_in == cnt) {
                    // (fewer than 32 because the ring holds no more, not because the part ends: wait for the ring
                    // unless a row among them is about to leave)
                    if (cnt < kStep && p + cnt < hi && m_leaving == 0) break;
                } else {
                    const int blocker = __builtin_amdgcn_readlane(col, n_in);
                    const bool leaving = (m_leaving & ((1u << n_in) - 1u)) != 0;
                    if (!leaving && blocker >= res_lo) break;  // the step can still fill up in a later turn
                    n = n_in;
                }
                if (n == kStep)
                    step(yes(), yes(), n, first_col);
                else
                    step(no(), yes(), n, first_col);
                advance(n);
            }
            if (n_pending > 0) {
                write_chunk(loaded, pend0);
                ++loaded;
            }
            if (n_pending > 1) {
                write_chunk(loaded, pend1);
                ++loaded;
            }
            if (t < t1) {
                __syncthreads();  // every wave is done with window t - 1
                write_window(t + 1, f);
                __syncthreads();
            }
        }
    }
    // what the windows did not serve (columns out of order only): from memory
    while (p < hi) {
        int cnt;
        const int col = candidates(cnt);
        if (cnt <= 0) {
            Cand now;
            load_chunk(loaded, now);
            write_chunk(loaded, now);
            ++loaded;
            continue;
        }
        step(no(), no(), cnt, __builtin_amdgcn_readfirstlane(col));
        advance(cnt);
    }

    half_t *out_row = out + ((size_t)row * V) * n_cols + col0;
    if (ksplit == 1) {
        if (has_row && col_ok) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = 4 * g + e;
                if (v < V) {
                    float tmp[8];
#pragma unroll
                    for (int c = 0; c < 8; ++c) tmp[c] = acc[c][e];
                    store_converted<half_t, 8>(out_row + (size_t)v * n_cols, tmp);
                }
            }
        }
        return;
    }
    // this part's tile to the workspace; the next launch adds the parts up
    if (!has_row) return;
    constexpr uint32_t kTileFloats = (uint32_t)V * kSlabTile;
    float *mine = tiles + (((size_t)(rb * n_tiles + tile) * ksplit + ks) * R + wave) * kTileFloats;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int v = 4 * g + e;
        if (v < V) {
#pragma unroll
            for (int c4 = 0; c4 < 2; ++c4) {
                const float4_t x = {acc[4 * c4][e], acc[4 * c4 + 1][e], acc[4 * c4 + 2][e], acc[4 * c4 + 3][e]};
                *reinterpret_cast<float4_t *>(mine + v * kSlabTile + cs * 8 + 4 * c4) = x;
            }
        }
    }
}

// Second launch: one wave per (row block, column tile, row of the block) adds that row's tiles in ascending order of the
// parts and writes the row.
template <int V, int R>
__global__ void __launch_bounds__(256)
spmm_slab_sum_kernel(int n_cols, int n_tiles, int m_vec, int ksplit, const int *__restrict__ row_indices,
                     const float *__restrict__ tiles, half_t *__restrict__ out)
{
    const int lane = threadIdx.x & 63;
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);  // (group, row of the block)
    const int group = unit / R, wave = unit % R;
    const int tile = group % n_tiles, rb = group / n_tiles;
    const int slot = rb * R + wave;
    if (slot >= m_vec) return;
    const int row = row_indices[slot];
    constexpr int kTileFloats = V * kSlabTile;
    const float *base = tiles + ((size_t)group * ksplit * R + wave) * kTileFloats;
    constexpr int kItems = V * 32;
#pragma unroll
    for (int item = lane; item < kItems; item += 64) {
        float4_t total = {0.f, 0.f, 0.f, 0.f};
        for (int part0 = 0; part0 < ksplit; part0 += 8) {
            float4_t x[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int part = part0 + i < ksplit ? part0 + i : ksplit - 1;
                x[i] = *reinterpret_cast<const float4_t *>(base + (size_t)part * R * kTileFloats + 4 * item);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (part0 + i < ksplit) total += x[i];
        }
        const int v = item >> 5;
        const int col = tile * kSlabTile + (item & 31) * 4;
        if (col < n_cols) {
            const float tmp[4] = {total[0], total[1], total[2], total[3]};
            store_converted<half_t, 4>(out + ((size_t)row * V + v) * n_cols + col, tmp);
        }
    }
}

// What a launch needs: `ksplit` parts of the contraction (1 = no workspace) and the fp32 tiles that go with them.
long long spmm_slab_workspace_bytes(int m_vec, int vec_length, int k, int ksplit)
{
    if (ksplit <= 1) return 0;
    const long long groups = (long long)ceil_div(m_vec, kSlabRows) * ceil_div(k, kSlabTile);
    return groups * ksplit * kSlabRows * vec_length * kSlabTile * (long long)sizeof(float);
}

int choose_spmm_slab_parts(int m_vec, int k, int n)
{
    if (options().spmm_slab_parts > 0) return options().spmm_slab_parts;
    const int groups = ceil_div(m_vec, kSlabRows) * ceil_div(k, kSlabTile);
    int parts = 256 / groups;                        // a workgroup per CU at most
    const int most = n / (2 * kSlabWindow);          // a part walks two windows at least
    parts = parts > most ? most : parts;
    if (parts >= 8) parts = parts / 8 * 8;           // each part's rhs rows in one XCD's L2
    return parts < 1 ? 1 : (parts > 64 ? 64 : parts);
}

namespace {

template <int V>
int launch_slab_v(int m_vec, int k, int n, int ksplit, const int *row_indices, const int *row_offsets,
                  const int *column_indices, const half_t *values, const half_t *rhs, half_t *out, float *tiles,
                  hipStream_t stream)
{
    constexpr int R = kSlabRows;
    const int n_tiles = ceil_div(k, kSlabTile);
    const long long blocks = (long long)ceil_div(m_vec, R) * n_tiles * ksplit;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    auto kernel = spmm_mfma_slab_kernel<V, R>;
    static std::atomic<unsigned long long> lds_allowed{0};
    const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 160 * 1024, lds_allowed);
    if (attr != hipSuccess) return (int)attr;
    constexpr int kLds = slab_lds_bytes<V, R>();
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(64 * R), kLds, stream, k, n_tiles, m_vec, ksplit, n,
                       row_indices, row_offsets, column_indices, values, rhs, out, tiles);
    const hipError_t st = hipGetLastError();
    if (st != hipSuccess || ksplit == 1) return (int)st;
    const int units = ceil_div(m_vec, R) * n_tiles * R;
    hipLaunchKernelGGL((spmm_slab_sum_kernel<V, R>), dim3((unsigned)ceil_div(units, 4)), dim3(256), 0, stream, k, n_tiles,
                       m_vec, ksplit, row_indices, tiles, out);
    return (int)hipGetLastError();
}

}  // namespace

// k % 8 == 0, n * k < 2^31, fp16 output; workspace of spmm_slab_workspace_bytes(.., ksplit) bytes, contents undefined
// before and after.
//
// Where the time of this schedule goes, measured on one MI355X (2048 x 4608 x 256, V = 8, 50 % sparsity, four parts:
// 256 workgroups of eight waves, each walking nine windows; rocprofv3 counters and timing-only variants): launch,
// prologue (row extent -> first chunks -> first / last column -> first window, four dependent round trips) and the
// store of the partial tiles 4.5 us; the nine turns with nothing computed 7.8 us (0.87 us a turn: every launch starts
// with cold L2s, the window requested at the start of a turn is first touched by all workgroups at once, and the
// 160 KB of LDS hold two windows beside the rings - one turn of lookahead); the steps 19 us - 170 vector-ALU
// instructions a step (the 32 v_perm_b32 of the transposition, addresses, masks, the choice of the step's size)
// make the launch's 6.2 M vector-ALU instructions a floor of 10 us by themselves, on two waves per SIMD that hide
// nothing of each other's LDS round trips (46 % of the wave cycles waiting); the second launch 4.8 us.  31 us in all
// against 15.6 us for spmm_mfma_kernel, which issues about as many vector-ALU instructions but spreads them over
// 16 K short-lived waves whose phases overlap.  Sixteen waves per workgroup spill (146 registers wanted, 128 allowed).
int launch_spmm_mfma_slab(int m_vec, int vec_length, int k, int n, int ksplit, const int *row_indices,
                          const int *row_offsets, const int *column_indices, const half_t *values, const half_t *rhs,
                          half_t *out, void *workspace, long long workspace_bytes, hipStream_t stream)
{
    if (m_vec == 0 || k == 0) return hipSuccess;
    if (k % 8 != 0 || (long long)n * k >= (1LL << 31) || n < 1) return hipErrorNotSupported;
    if (ksplit < 1 || ksplit > 64) return hipErrorInvalidValue;
    const long long need = spmm_slab_workspace_bytes(m_vec, vec_length, k, ksplit);
    if (need > workspace_bytes) return hipErrorNotSupported;
    float *tiles = static_cast<float *>(workspace);
    switch (vec_length) {
    case 1: return launch_slab_v<1>(m_vec, k, n, ksplit, row_indices, row_offsets, column_indices, values, rhs, out, tiles, stream);
    case 2: return launch_slab_v<2>(m_vec, k, n, ksplit, row_indices, row_offsets, column_indices, values, rhs, out, tiles, stream);
    case 4: return launch_slab_v<4>(m_vec, k, n, ksplit, row_indices, row_offsets, column_indices, values, rhs, out, tiles, stream);
    case 8: return launch_slab_v<8>(m_vec, k, n, ksplit, row_indices, row_offsets, column_indices, values, rhs, out, tiles, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace vs
