// Measurement aids (librptc_bench_aids.so): what the machine does with no decode at all, for the
// same bytes and the same launch pattern as the mat-vec.  bench.py times them beside the kernel it
// grades, so that the roofline figure can be read against the floor of this workload size: the time
// of an empty launch, and the time of a kernel that only reads the stream.  A library of its own:
// nothing here is part of the product path or of its header.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

__global__ __launch_bounds__(1024) void probe_empty_kernel() {}

// Every thread requests kPerThread 16-byte non-temporal loads before it uses any; the XOR of what
// it read is stored only if it equals a value the data cannot produce by design, so the loads
// cannot be removed and nothing is written.
constexpr int kPerThread = 3;

__global__ __launch_bounds__(1024) void probe_read_kernel(const uint32_t *__restrict__ data, uint32_t *sink, size_t total16)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const size_t base = (size_t)blockIdx.x * blockDim.x * kPerThread + threadIdx.x;
    u32x4 v[kPerThread];
#pragma unroll
    for (int k = 0; k < kPerThread; k++) {
        const size_t i = base + (size_t)k * blockDim.x;
        v[k] = u32x4{0u, 0u, 0u, 0u};
        if (i < total16) v[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(data) + i);
    }
    uint32_t s = 0;
#pragma unroll
    for (int k = 0; k < kPerThread; k++) s ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
    if (s == 0x9E3779B9u && sink) sink[0] = s;
}

}  // namespace

// one empty 1024-thread workgroup per workgroup of the mat-vec's grid
extern "C" int rptc_probe_empty(int workgroups, void *stream)
{
    if (workgroups < 1) return -2;
    hipLaunchKernelGGL(probe_empty_kernel, dim3(workgroups), dim3(1024), 0, static_cast<hipStream_t>(stream));
    return (int)hipGetLastError();
}

// reads `bytes` (a multiple of 16, 16-byte aligned) with non-temporal 16-byte loads and writes nothing
extern "C" int rptc_probe_read(const void *data, int64_t bytes, void *sink, void *stream)
{
    if (!data) return -1;
    if (bytes < 16 || bytes % 16 != 0) return -2;
    if (reinterpret_cast<uintptr_t>(data) & 15u) return -3;
    const size_t total16 = (size_t)bytes / 16;
    const size_t per_block = (size_t)1024 * kPerThread;
    const size_t grid = (total16 + per_block - 1) / per_block;
    if (grid >= ((size_t)1 << 31)) return -5;
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)grid), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint32_t *>(data), static_cast<uint32_t *>(sink), total16);
    return (int)hipGetLastError();
}
