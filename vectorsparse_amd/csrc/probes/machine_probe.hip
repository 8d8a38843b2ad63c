// Machine probe for the floors the SpMM / SDDMM kernels are measured against on one GPU:
//   1. what a launch costs before any work (a kernel that does nothing, back to back inside a HIP graph);
//   2. what a chain of dependent loads costs right after a launch (the row swizzle -> offsets -> indices ->
//      gathered rows chain of the kernels);
//   3. how fast random 256-byte segments of an L2-resident matrix can be gathered into the CUs, through
//      registers, through global -> LDS loads, or both, with 4 to 32 segments in flight per 16-lane group;
//   4. what a launch costs that only writes its output (every lane one 16-byte store, no loads): the time a kernel
//      waits for its last stores to be acknowledged.
// Prints a short text report; times are medians of 7 replays of a graph of 100 launches.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <functional>
#include <random>
#include <vector>

typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
#define LDSP(p) ((__attribute__((address_space(3))) unsigned char *)(p))
#define CHECK(x)                                                                     \
    do {                                                                             \
        hipError_t e_ = (x);                                                         \
        if (e_ != hipSuccess) {                                                      \
            printf("%s failed: %s\n", #x, hipGetErrorString(e_));                    \
            return 1;                                                                \
        }                                                                            \
    } while (0)

__global__ void empty_kernel() {}

// One lane per wave (or all 64) follows L dependent loads through an 8 MiB table.
template <int L, int LANES>
__global__ void __launch_bounds__(1024) chain_kernel(const int *__restrict__ table, int mask, int *__restrict__ out)
{
    int idx = (blockIdx.x * 1024 + threadIdx.x) * 97;
    if ((threadIdx.x & 63) < LANES) {
#pragma unroll
        for (int l = 0; l < L; ++l) idx = table[(idx + l * 1237) & mask];
        if (idx == 0x7fffffff || threadIdx.x == 0) out[blockIdx.x] = idx;
    }
}

// Every lane stores 16 bytes, nothing is loaded.
__global__ void __launch_bounds__(1024) store_kernel(uint4_t *__restrict__ out)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    out[i] = uint4_t{(unsigned)i, 1u, 2u, 3u};
}

// REG segments per 16-lane group through registers plus DMA segments through LDS per iteration.
template <int REG, int DMA>
__global__ void __launch_bounds__(256)
gather_kernel(const int *__restrict__ idx, const uint4_t *__restrict__ rows, int row_u4, int n_idx, uint4_t *out)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & 63, g = lane >> 4, cs = lane & 15;
    const int wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int n_waves = (gridDim.x * blockDim.x) >> 6;
    constexpr int U = REG + DMA;
    unsigned char *buf = smem + (size_t)wave_in_block * (DMA > 0 ? DMA : 1) * 1024;
    uint4_t acc = {0, 0, 0, 0};
    for (int base = wave * 4 * U; base + 4 * U <= n_idx; base += n_waves * 4 * U) {
        int c[U];
#pragma unroll
        for (int u = 0; u < U; ++u) c[u] = idx[base + g * U + u];
        uint4_t v[REG > 0 ? REG : 1];
#pragma unroll
        for (int u = 0; u < REG; ++u) v[u] = rows[(size_t)c[u] * row_u4 + cs];
#pragma unroll
        for (int u = 0; u < DMA; ++u)
            __builtin_amdgcn_global_load_lds(&rows[(size_t)c[REG + u] * row_u4 + cs], LDSP(buf + u * 1024), 16, 0, 0);
#pragma unroll
        for (int u = 0; u < REG; ++u) acc ^= v[u];
        if (DMA > 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int u = 0; u < DMA; ++u) acc ^= *reinterpret_cast<const uint4_t *>(buf + u * 1024 + lane * 16);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
    }
    if (acc[0] == 0x12345678u) out[threadIdx.x] = acc;
}

// Median microseconds per launch: `launch` captured `count` times into a graph, replayed 7 times.
static double graph_us(hipStream_t stream, const std::function<void(hipStream_t)> &launch, int count = 100)
{
    hipGraph_t graph;
    hipGraphExec_t exec;
    launch(stream);
    if (hipStreamSynchronize(stream) != hipSuccess) return -1;
    if (hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) return -1;
    for (int i = 0; i < count; ++i) launch(stream);
    if (hipStreamEndCapture(stream, &graph) != hipSuccess) return -1;
    if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess) return -1;
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    hipGraphLaunch(exec, stream);
    hipStreamSynchronize(stream);
    std::vector<double> us;
    for (int r = 0; r < 7; ++r) {
        hipEventRecord(e0, stream);
        hipGraphLaunch(exec, stream);
        hipEventRecord(e1, stream);
        hipEventSynchronize(e1);
        float ms = 0;
        hipEventElapsedTime(&ms, e0, e1);
        us.push_back(ms * 1e3 / count);
    }
    hipGraphExecDestroy(exec);
    hipGraphDestroy(graph);
    std::sort(us.begin(), us.end());
    return us[us.size() / 2];
}

template <int REG, int DMA>
static void gather_row(const char *name, hipStream_t stream, const int *idx, const uint4_t *rows, int row_u4, int n_idx,
                       uint4_t *out)
{
    const size_t lds = (size_t)4 * DMA * 1024;
    if (lds > 65536)
        (void)hipFuncSetAttribute((const void *)gather_kernel<REG, DMA>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    printf("  %-28s", name);
    for (int blocks : {512, 1024, 2048, 4096}) {
        const double us = graph_us(stream, [&](hipStream_t s) {
            hipLaunchKernelGGL((gather_kernel<REG, DMA>), dim3(blocks), dim3(256), lds, s, idx, rows, row_u4, n_idx, out);
        }, 20);
        const double bytes = (double)(n_idx / (4 * (REG + DMA)) * (4 * (REG + DMA))) * 256;
        printf("  %5.2f TB/s", bytes / us * 1e-6);
    }
    printf("\n");
    fflush(stdout);
}

int main()
{
    hipStream_t stream;
    CHECK(hipStreamCreate(&stream));
    printf("machine probe (one GPU; medians of 7 replays of a HIP graph of back-to-back launches)\n\n");

    printf("1. a kernel that does nothing, microseconds per launch\n");
    for (int threads : {64, 256, 1024})
        for (int blocks : {1, 256, 2048}) {
            const double us = graph_us(stream, [&](hipStream_t s) { hipLaunchKernelGGL(empty_kernel, dim3(blocks), dim3(threads), 0, s); });
            printf("  %5d workgroups x %4d threads: %.2f us\n", blocks, threads, us);
        }

    printf("\n2. dependent loads after a launch (256 workgroups x 1024 threads, 8 MiB table), microseconds per launch\n");
    const int n = 1 << 21;
    int *table, *sink;
    CHECK(hipMalloc(&table, n * 4));
    CHECK(hipMalloc(&sink, 256 * 1024 * 4));
    {
        std::vector<int> h(n);
        for (int i = 0; i < n; ++i) h[i] = int((i * 2654435761u) >> 9);
        CHECK(hipMemcpy(table, h.data(), n * 4, hipMemcpyHostToDevice));
    }
#define CHAIN(L, LANES)                                                                                                   \
    printf("  %d dependent load(s), %2d lane(s) per wave: %.2f us\n", L, LANES, graph_us(stream, [&](hipStream_t s) {         \
               hipLaunchKernelGGL((chain_kernel<L, LANES>), dim3(256), dim3(1024), 0, s, table, n - 1, sink);             \
           }))
    CHAIN(0, 1);
    CHAIN(1, 1);
    CHAIN(2, 1);
    CHAIN(3, 1);
    CHAIN(4, 1);
    CHAIN(8, 1);
    CHAIN(4, 64);

    printf("\n3. gather of random 256-byte segments of a 4608 x 256 fp16 matrix (2.4 MB), TB/s at 512 / 1024 / 2048 / 4096\n"
           "   workgroups of 4 waves; `reg n` = n segments in flight per 16-lane group through registers, `dma n` = through\n"
           "   global -> LDS loads\n");
    const int K = 4608, N = 256, row_u4 = N * 2 / 16, n_idx = 3 << 18;
    uint4_t *rows, *out;
    int *idx;
    CHECK(hipMalloc(&rows, (size_t)K * N * 2));
    CHECK(hipMemset(rows, 1, (size_t)K * N * 2));
    CHECK(hipMalloc(&out, 4096));
    CHECK(hipMalloc(&idx, n_idx * 4));
    {
        std::vector<int> h(n_idx);
        std::mt19937 r(1);
        for (auto &x : h) x = r() % K;
        CHECK(hipMemcpy(idx, h.data(), n_idx * 4, hipMemcpyHostToDevice));
    }
    gather_row<4, 0>("reg 4", stream, idx, rows, row_u4, n_idx, out);
    gather_row<8, 0>("reg 8", stream, idx, rows, row_u4, n_idx, out);
    gather_row<16, 0>("reg 16", stream, idx, rows, row_u4, n_idx, out);
    gather_row<32, 0>("reg 32", stream, idx, rows, row_u4, n_idx, out);
    gather_row<0, 4>("dma 4", stream, idx, rows, row_u4, n_idx, out);
    gather_row<0, 8>("dma 8", stream, idx, rows, row_u4, n_idx, out);
    gather_row<0, 16>("dma 16", stream, idx, rows, row_u4, n_idx, out);
    gather_row<8, 8>("reg 8 + dma 8", stream, idx, rows, row_u4, n_idx, out);
    gather_row<16, 16>("reg 16 + dma 16", stream, idx, rows, row_u4, n_idx, out);
    printf("\n4. a kernel that only stores 16 bytes per lane, microseconds per launch\n");
    {
        uint4_t *dst;
        CHECK(hipMalloc(&dst, (size_t)4096 * 1024 * 16));
        for (int threads : {64, 256})
            for (int blocks : {256, 1024, 4096}) {
                const double us = graph_us(stream, [&](hipStream_t s) { hipLaunchKernelGGL(store_kernel, dim3(blocks), dim3(threads), 0, s, dst); });
                printf("  %5d workgroups x %4d threads (%7.0f KB written): %.2f us\n", blocks, threads, blocks * threads * 16 / 1e3, us);
            }
        CHECK(hipFree(dst));
    }
    CHECK(hipDeviceSynchronize());
    printf("\ndone\n");
    return 0;
}
