// Measurement aid, not part of libvsparse.so: a kernel that does nothing, launched on a grid of the caller's choice.
// Timing it prices the dispatch floor of a launch shape, below which no kernel of that shape can finish
// (bench.py reports it beside the headline launch).  Built as libvsprobe.so.
#include <hip/hip_runtime.h>

__global__ void floor_probe_kernel() {}

extern "C" __attribute__((visibility("default"))) int vsprobe_empty_launch(int blocks, int threads_per_block, void *stream)
{
    if (blocks < 1 || threads_per_block < 1 || threads_per_block > 1024) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(floor_probe_kernel, dim3((unsigned)blocks), dim3((unsigned)threads_per_block), 0,
                       static_cast<hipStream_t>(stream));
    return (int)hipGetLastError();
}
