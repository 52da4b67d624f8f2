// Streaming probe for the benchmark harness (libdsx_probe.so, NOT part of libdsx.so): what plain
// kernels of the per-Gaussian kernels' access shape (one 16-byte element per thread, non-temporal)
// reach on this device, and a kernel of known traffic against which HBM byte counters are scaled.
#include "dsx_probe.h"

#include <hip/hip_runtime.h>

namespace
{
typedef float probe_f4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void stream_probe_kernel(const probe_f4* __restrict__ src, probe_f4* __restrict__ dst,
                                                           int64_t count, int mode, float* sink)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= count)
        return;
    if(mode == 1)
    {
        const probe_f4 v = {1.f, 2.f, 3.f, 4.f};
        __builtin_nontemporal_store(v, dst + i);
        return;
    }
    const probe_f4 v = __builtin_nontemporal_load(src + i);
    if(mode == 2)
        __builtin_nontemporal_store(v, dst + i);
    else if(v.x + v.y + v.z + v.w == 12345.678f) // never true for the probe's data: keeps the load alive
        *sink = 1.f;
}

// many streams per thread: kReads arrays read and kWrites arrays written, 16 bytes of each
template <int kReads, int kWrites>
__global__ __launch_bounds__(256) void stream_probe_mixed_kernel(const probe_f4* __restrict__ src,
                                                                 probe_f4* __restrict__ dst, int64_t count)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= count)
        return;
    probe_f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for(int r = 0; r < kReads; ++r)
        acc += __builtin_nontemporal_load(src + r * count + i);
#pragma unroll
    for(int w = 0; w < kWrites; ++w)
        __builtin_nontemporal_store(acc, dst + w * count + i);
}
} // namespace

extern "C" int dsxp_stream_probe(const void* src, void* dst, size_t bytes, int mode, void* stream, float* milliseconds)
{
    if(mode < 0 || mode > 4 || (bytes & 15) != 0 || (mode != 1 && !src) || (mode != 0 && !dst))
        return -1;
    if(mode == 0 && !dst)
        dst = const_cast<void*>(src); // the sink is never written
    int64_t count = (int64_t)(bytes / 16);
    if(mode >= 3)
        count /= mode == 3 ? 28 : 14; // `bytes` is everything the launch moves
    if(milliseconds)
        *milliseconds = 0.f;
    if(count == 0)
        return 0;
    if(count >= (1ll << 39))
        return -4;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t start = nullptr, stop = nullptr;
    if(milliseconds && (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess))
        return -3;
    if(milliseconds)
        (void)hipEventRecord(start, s);
    const dim3 grid((unsigned)((count + 255) / 256));
    if(mode == 3)
        hipLaunchKernelGGL((stream_probe_mixed_kernel<10, 18>), grid, dim3(256), 0, s, static_cast<const probe_f4*>(src),
                           static_cast<probe_f4*>(dst), count);
    else if(mode == 4)
        hipLaunchKernelGGL((stream_probe_mixed_kernel<5, 9>), grid, dim3(256), 0, s, static_cast<const probe_f4*>(src),
                           static_cast<probe_f4*>(dst), count);
    else
        hipLaunchKernelGGL(stream_probe_kernel, grid, dim3(256), 0, s, static_cast<const probe_f4*>(src),
                           static_cast<probe_f4*>(dst), count, mode, static_cast<float*>(dst));
    int rc = hipGetLastError() == hipSuccess ? 0 : -2;
    if(milliseconds)
    {
        (void)hipEventRecord(stop, s);
        if(hipEventSynchronize(stop) != hipSuccess || hipEventElapsedTime(milliseconds, start, stop) != hipSuccess)
            rc = rc ? rc : -3;
        (void)hipEventDestroy(start);
        (void)hipEventDestroy(stop);
    }
    return rc;
}
