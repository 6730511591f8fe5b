// Measurement aids (librptc_bench_aids.so): what the machine does with no decode at all, for the
// same bytes and the same launch pattern as the mat-vec.  bench.py times them beside the kernel it
// grades, so that the roofline figure can be read against the floor of this workload size: the time
// of an empty launch, and the time of a kernel that only reads the stream.  A library of its own:
// nothing here is part of the product path or of its header.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../csrc/decode_asm.hpp"

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

// Issue rate of the vector instructions the decode is made of: every wave runs `iters` rounds of 32 instructions of
// one kind on eight independent registers (a chain of eight never waits for its own result), one 1024-thread
// workgroup per compute unit, i.e. four waves a SIMD as in the mat-vec.  Nothing is read; the result is stored only
// if it equals a value it cannot take.
#define RPTC_PROBE_8(TEXT)                                                                                            \
    asm volatile(TEXT(%0) TEXT(%1) TEXT(%2) TEXT(%3) TEXT(%4) TEXT(%5) TEXT(%6) TEXT(%7)                              \
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7])   \
                 : "v"(a), "v"(b), "s"(sel))
#define RPTC_I_DOT2C(R) "v_dot2c_f32_f16 " #R ", %8, %9\n"
#define RPTC_I_PKMAD(R) "v_pk_mad_u16 " #R ", %8, %8, " #R "\n"
#define RPTC_I_PERM(R) "v_perm_b32 " #R ", " #R ", %9, %10\n"
#define RPTC_I_ALIGN(R) "v_alignbit_b32 " #R ", " #R ", %8, 7\n"
#define RPTC_I_ANDOR(R) "v_and_or_b32 " #R ", " #R ", %10, %9\n"
#define RPTC_I_FMA(R) "v_fma_f32 " #R ", %8, %9, " #R "\n"
// v_dot2c_f32_f16 on four sums in turn, as the decode block has them (a sum is added to every fourth instruction)
#define RPTC_PROBE_4X2(TEXT)                                                                                          \
    asm volatile(TEXT(%0) TEXT(%1) TEXT(%2) TEXT(%3) TEXT(%0) TEXT(%1) TEXT(%2) TEXT(%3)                              \
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7])   \
                 : "v"(a), "v"(b), "s"(sel))

template <int KIND>
__global__ __launch_bounds__(1024) void probe_valu_kernel(int iters, uint32_t seed, uint32_t *sink)
{
    uint32_t r[8];
#pragma unroll
    for (int i = 0; i < 8; i++) r[i] = seed + threadIdx.x * 8u + i;
    const uint32_t a = 0x3C003800u ^ (threadIdx.x << 3), b = 0x38003C00u + blockIdx.x;
    const uint32_t sel = 0x0C0C0500u;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (KIND == 0) RPTC_PROBE_8(RPTC_I_DOT2C);
            else if (KIND == 1) RPTC_PROBE_8(RPTC_I_PKMAD);
            else if (KIND == 2) RPTC_PROBE_8(RPTC_I_PERM);
            else if (KIND == 3) RPTC_PROBE_8(RPTC_I_ALIGN);
            else if (KIND == 4) RPTC_PROBE_8(RPTC_I_ANDOR);
            else if (KIND == 5) RPTC_PROBE_8(RPTC_I_FMA);
            else RPTC_PROBE_4X2(RPTC_I_DOT2C);
        }
    }
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) x ^= r[i];
    if (x == 0x9E3779B9u && sink) sink[0] = x;
}

// The decode block of the mat-vec by itself: every wave decodes `iters` stream elements that it makes up from
// registers (no global memory, the 64 KiB table in LDS as in the kernels), so the time per element and SIMD is what the
// block costs at that number of waves a SIMD with nothing else in the way.
__global__ void probe_decode_kernel(int iters, uint32_t seed, uint32_t *sink)
{
    extern __shared__ uint32_t probe_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < 16384; i += blockDim.x) probe_lds[i] = 0x3C003800u + (uint32_t)(i >> 6);
    __syncthreads();
    const uint32_t lane4 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(probe_lds)) + lane * 4;
    uint32_t xr[32];
#pragma unroll
    for (int q = 0; q < 32; q++) xr[q] = 0x38003C00u + (uint32_t)q;
    uint4 e = make_uint4(seed + tid, seed * 3u + tid, seed * 5u + tid, seed * 7u + tid);
    const uint64_t first_lanes = 0x0000000100000001ull;
    float acc = 0.f;
    for (int it = 0; it < iters; it++) {
        float a0, a1, a2, a3;
        rptc::decode_element_asm(e, e.w, first_lanes, lane4, xr, a0, a1, a2, a3);
        acc += (a0 + a1) + (a2 + a3);
        e.x += 0x9E3779B9u;          // the next element (a scalar-cheap change; the block does not depend on the last one)
        e.z ^= e.x;
    }
    if (__builtin_bit_cast(uint32_t, acc) == 0x9E3779B9u && sink) sink[0] = 1u;
}

}  // namespace

// `iters` elements decoded by every wave of `workgroups` workgroups of `threads` threads (64..1024: 1 to 4 waves a SIMD)
extern "C" int rptc_probe_decode(int iters, int threads, int workgroups, void *sink, void *stream)
{
    if (iters < 1 || threads < 64 || threads > 1024 || threads % 64 || workgroups < 1) return -2;
    static bool allowed = false;
    if (!allowed) {
        int rc = (int)hipFuncSetAttribute(reinterpret_cast<const void *>(probe_decode_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (rc) return rc;
        allowed = true;
    }
    // 150 KiB of LDS: one workgroup per compute unit, as the mat-vec has it
    hipLaunchKernelGGL(probe_decode_kernel, dim3(workgroups), dim3(threads), 150 * 1024, static_cast<hipStream_t>(stream), iters, 12345u,
                       static_cast<uint32_t *>(sink));
    return (int)hipGetLastError();
}

// `iters` rounds of 32 vector instructions of one kind in every wave of `workgroups` 1024-thread workgroups;
// kind: 0 v_dot2c_f32_f16, 1 v_pk_mad_u16, 2 v_perm_b32, 3 v_alignbit_b32, 4 v_and_or_b32, 5 v_fma_f32,
// 6 v_dot2c_f32_f16 on four sums in turn instead of eight
extern "C" int rptc_probe_valu(int kind, int iters, int workgroups, void *sink, void *stream)
{
    if (kind < 0 || kind > 6 || iters < 1 || workgroups < 1) return -2;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t *out = static_cast<uint32_t *>(sink);
#define RPTC_PROBE_GO(K) hipLaunchKernelGGL(probe_valu_kernel<K>, dim3(workgroups), dim3(1024), 0, s, iters, 12345u, out)
    switch (kind) {
    case 0: RPTC_PROBE_GO(0); break;
    case 1: RPTC_PROBE_GO(1); break;
    case 2: RPTC_PROBE_GO(2); break;
    case 3: RPTC_PROBE_GO(3); break;
    case 4: RPTC_PROBE_GO(4); break;
    case 5: RPTC_PROBE_GO(5); break;
    default: RPTC_PROBE_GO(6); break;
    }
#undef RPTC_PROBE_GO
    return (int)hipGetLastError();
}

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
