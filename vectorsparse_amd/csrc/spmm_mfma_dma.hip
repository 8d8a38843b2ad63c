// SpMM on fp16 MFMA with the gathered rows of the dense operand going global -> LDS without passing through
// registers (global_load_lds_dwordx4) and the MFMA B operand fetched with the transposing LDS read
// (ds_read_b64_tr_b16); the counterpart of the reference's dense tile loader (src/spmm_utils/dense_tile.h:217-267)
// and tile loop (src/wmma_spmm.cu:77-90).  Same work split as spmm_mfma_kernel (one workgroup per vector row and
// tile of 128 dense columns, the waves take interleaved 32-vector steps, fixed-order reduction through LDS).
//
// One step in a wave, lane = (cs = lane % 16, g = lane / 16):
//   * lanes 0..31 park one column index and one V-vector each in the wave's staging slot (as spmm_mfma_kernel);
//   * eight LDS-DMA loads: load i brings, for every lane, the 16 bytes at columns tile*128 + 8*cs.. of gathered
//     row j = 8g + i.  The hardware writes lane l's 16 bytes at LDS base_i + 16*l, so load i leaves the 256-byte
//     segments of rows i, 8 + i, 16 + i, 24 + i side by side; base_i = i * (1024 + 32);
//   * MFMA c (16 dense columns 16c..16c+15) wants, in lane (cs, g), rows 8g..8g+7 of column 16c + cs.
//     ds_read_b64_tr_b16 serves a 16-lane group a 4 x 16 block: lane n passes the address of 4 halves
//     (row n / 4, columns 4 * (n % 4)..) and receives column n of the four rows.  Two such reads (rows 8g..8g+3 from
//     loads 0..3, rows 8g+4..8g+7 from loads 4..7) make the operand.  The 32 bytes of padding per load put the four
//     rows a group reads at once in different banks.
//   The accumulator of lane (cs, g), register e, MFMA c is out[4g + e][tile*128 + 16c + cs].
#include "spmm_mfma_step.hpp"
#include "vs_common.hpp"

namespace vs {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
#define VS_LDS(p) ((__attribute__((address_space(3))) unsigned char *)(p))

constexpr int kDmaTile = 128;            // dense columns per workgroup
constexpr int kDmaLoad = 1024 + 32;      // LDS bytes per LDS-DMA load: 64 lanes x 16 bytes, plus padding
constexpr int kDmaBuf = 8 * kDmaLoad;    // one step: 32 gathered rows x 256 bytes

template <int V>
constexpr int dma_wave_bytes()
{
    return stage_bytes<V>() + kDmaBuf;
}

template <int V, bool IDX32, typename OutT>
__global__ void __launch_bounds__(1024)
spmm_mfma_dma_kernel(int n_cols, int n_tiles, const int *__restrict__ row_indices,
                     const int *__restrict__ row_offsets, const int *__restrict__ column_indices,
                     const half_t *__restrict__ values, const half_t *__restrict__ rhs, OutT *__restrict__ out,
                     long long stride_values, long long stride_rhs, long long stride_out)
{
    values += blockIdx.y * stride_values;  // batch: shared pattern, per-problem operands
    rhs += blockIdx.y * stride_rhs;
    out += blockIdx.y * stride_out;
    extern __shared__ __align__(16) unsigned char smem[];  // per wave: staging slot, then the gather buffer
    constexpr int TN = kDmaTile;
    constexpr int kWaveBytes = dma_wave_bytes<V>();
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int tile = blockIdx.x % n_tiles;
    const int slot = blockIdx.x / n_tiles;
    const int row = row_indices[slot];
    const int beg = row_offsets[row];
    const int end = row_offsets[row + 1];
    const int cs = lane & 15;
    const int g = lane >> 4;
    const int col0 = tile * TN + cs * 8;   // the lane's 16-byte chunk of a gathered row
    const bool col_ok = col0 < n_cols;     // n_cols % 8 == 0: a chunk is all in or all out
    const uint32_t col_off = col_ok ? col0 : 0;

    unsigned char *mine = smem + (size_t)wave * kWaveBytes;
    int *idx_s = reinterpret_cast<int *>(mine);
    half_t *vec_s = reinterpret_cast<half_t *>(idx_s + kStep);  // [V][kStep]
    unsigned char *buf = mine + stage_bytes<V>();
    // the lane's corner of the 4 x 16 blocks it reads for MFMA 0: row cs / 4 of its k group, columns 4 * (cs % 4)..
    const unsigned char *tr_base = buf + (cs >> 2) * kDmaLoad + g * 256 + 8 * (cs & 3);

    float4_t acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int steps = (end - beg + kStep - 1) / kStep;
    int active = (steps + 1) >> 1;  // short rows do not need every wave (see spmm_mfma_kernel)
    active = active < 1 ? 1 : (active > n_waves ? n_waves : active);
    const int stride = kStep * active;
    int base = beg + kStep * wave;
    const bool has_work = wave < active && base < end;
    int next_idx = 0;
    bool next_valid = false;
    half_t next_vec[V];
#pragma unroll
    for (int v = 0; v < V; ++v) next_vec[v] = (half_t)0.f;
    auto fetch = [&](int b) {
        if (lane < kStep) {
            const int j = b + lane;
            next_valid = j < end;
            // slots past the row's end repeat its last vector with a zero value: in bounds, contributes nothing
            const int jc = next_valid ? j : end - 1;
            next_idx = column_indices[jc];
            load_vector<V>(next_vec, values + (size_t)jc * V);
        }
    };
    if (has_work) fetch(base);

    for (; has_work && base < end; base += stride) {
        if (lane < kStep) {
            idx_s[lane] = next_idx;
#pragma unroll
            for (int v = 0; v < V; ++v) vec_s[v * kStep + lane] = next_valid ? next_vec[v] : (half_t)0.f;
        }
        wave_lds_fence();
        const int4_t i_lo = *reinterpret_cast<const int4_t *>(idx_s + 8 * g);
        const int4_t i_hi = *reinterpret_cast<const int4_t *>(idx_s + 8 * g + 4);
        half8_t a = {0, 0, 0, 0, 0, 0, 0, 0};
        if (cs < V) a = *reinterpret_cast<const half8_t *>(vec_s + cs * kStep + 8 * g);
        wave_lds_fence();
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int col = i < 4 ? i_lo[i] : i_hi[i - 4];
            const half_t *src;
            if constexpr (IDX32)
                src = rhs + ((uint32_t)col * (uint32_t)n_cols + col_off);
            else
                src = rhs + ((size_t)col * n_cols + col_off);
            __builtin_amdgcn_global_load_lds(src, VS_LDS(buf + i * kDmaLoad), 16, 0, 0);
        }
        if (base + stride < end) fetch(base + stride);
        // the gathered rows are in LDS (and the next step's index and vector in registers) from here on
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) short4_t *)VS_LDS(tr_base + 32 * c));
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) short4_t *)VS_LDS(tr_base + 32 * c + 4 * kDmaLoad));
            const short8_t both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8_t, both), acc[c], 0, 0, 0);
        }
        wave_lds_fence();  // the buffer is read out before the next step's loads land in it
    }

    // partial tiles [v][128] fp32 in the (now idle) gather buffers, summed in wave order
    float *partial = reinterpret_cast<float *>(buf);
    if (wave < active) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int v = 4 * g + e;
            if (v < V) {
#pragma unroll
                for (int c = 0; c < 8; ++c) partial[v * TN + 16 * c + cs] = acc[c][e];
            }
        }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < V * 16; t += blockDim.x) {  // a single wave takes two turns for V = 8
        const int v = t >> 4;
        const int cs2 = t & 15;
        const int col = tile * TN + cs2 * 8;
        if (col < n_cols) {
            float sum[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) sum[c] = 0.f;
            // four partial tiles are requested at once (a wave past `active` contributes an exact zero) and added
            // in wave order: one LDS round trip per four waves instead of one per wave
            for (int w0 = 0; w0 < active; w0 += 4) {
                float4_t x[4][2];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int w = w0 + i < active ? w0 + i : active - 1;
                    const float *src = reinterpret_cast<const float *>(smem + (size_t)w * kWaveBytes + stage_bytes<V>()) +
                                       v * TN + cs2 * 8;
                    x[i][0] = *reinterpret_cast<const float4_t *>(src);
                    x[i][1] = *reinterpret_cast<const float4_t *>(src + 4);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool keep = w0 + i < active;
#pragma unroll
                    for (int c = 0; c < 8; ++c) sum[c] += keep ? x[i][c >> 2][c & 3] : 0.f;
                }
            }
            store_converted<OutT, 8>(out + ((size_t)row * V + v) * n_cols + col, sum);
        }
    }
}

template <int V, typename OutT>
static int launch_dma_v(int m_vec, int k, int n, int waves, const int *row_indices, const int *row_offsets,
                        const int *column_indices, const half_t *values, const half_t *rhs, OutT *out,
                        hipStream_t stream, const Batch &batch)
{
    const int n_tiles = ceil_div(k, kDmaTile);
    const long long blocks = (long long)m_vec * n_tiles;
    if (blocks > 0x7fffffffLL) return hipErrorNotSupported;
    const size_t lds = (size_t)waves * dma_wave_bytes<V>();
    static std::atomic<unsigned long long> allowed32{0}, allowed64{0};
    if ((long long)n * k < (1LL << 31)) {
        auto kernel = spmm_mfma_dma_kernel<V, true, OutT>;
        const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 160 * 1024, allowed32);
        if (attr != hipSuccess) return (int)attr;
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * waves), lds, stream, k, n_tiles,
                           row_indices, row_offsets, column_indices, values, rhs, out, batch.stride_a, batch.stride_b,
                           batch.stride_out);
    } else {
        auto kernel = spmm_mfma_dma_kernel<V, false, OutT>;
        const hipError_t attr = allow_large_lds(reinterpret_cast<const void *>(kernel), 160 * 1024, allowed64);
        if (attr != hipSuccess) return (int)attr;
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks, (unsigned)batch.count), dim3(64 * waves), lds, stream, k, n_tiles,
                           row_indices, row_offsets, column_indices, values, rhs, out, batch.stride_a, batch.stride_b,
                           batch.stride_out);
    }
    return (int)hipGetLastError();
}

// k % 8 == 0; waves <= 16 (16 waves x 9.1 KB of LDS fit the 160 KB of a CU once)
template <typename OutT>
int launch_spmm_mfma_dma(int m_vec, int vec_length, int k, int n, int waves, const int *row_indices,
                         const int *row_offsets, const int *column_indices, const half_t *values, const half_t *rhs,
                         OutT *out, hipStream_t stream, const Batch &batch)
{
    if (k % 8 != 0) return hipErrorNotSupported;
    switch (vec_length) {
    case 1: return launch_dma_v<1, OutT>(m_vec, k, n, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    case 2: return launch_dma_v<2, OutT>(m_vec, k, n, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    case 4: return launch_dma_v<4, OutT>(m_vec, k, n, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    case 8: return launch_dma_v<8, OutT>(m_vec, k, n, waves, row_indices, row_offsets, column_indices, values, rhs, out, stream, batch);
    default: return hipErrorInvalidValue;
    }
}

template int launch_spmm_mfma_dma<half_t>(int, int, int, int, int, const int *, const int *, const int *, const half_t *,
                                          const half_t *, half_t *, hipStream_t, const Batch &);
template int launch_spmm_mfma_dma<float>(int, int, int, int, int, const int *, const int *, const int *, const half_t *,
                                         const half_t *, float *, hipStream_t, const Batch &);

}  // namespace vs
