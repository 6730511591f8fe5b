// Measurement aids (librptc_bench_aids.so): what the machine does with no decode at all, for the
// same bytes and the same launch pattern as the mat-vec.  bench.py times them beside the kernel it
// grades, so that the roofline figure can be read against the floor of this workload size: the time
// of an empty launch, the time of a kernel that only reads the stream (one launch per layer, and as
// one persistent launch over all layers, the chain's pattern), and the issue rates of the vector and
// LDS instructions the decode is made of.  A library of its own, built beside bench.py: nothing here
// is part of the product path or of its header.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../let-it-slide_amd/csrc/decode_asm.hpp"

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

// The chain's read pattern with nothing decoded: one 1024-thread workgroup per compute unit stays for all `layers`;
// workgroup b reads its 1/grid share of every layer (16-byte non-temporal loads, a wave's request 1 KiB contiguous),
// the next layer's requests issued before the current layer's data is used, as the chain kernels do.
__global__ __launch_bounds__(1024) void probe_read_chain_kernel(const uint64_t *__restrict__ layer_ptrs, int copies, int layers,
                                                                 int per_group16, uint32_t *sink)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int tid = threadIdx.x;
    uint32_t acc = 0;
    u32x4 v[kPerThread], nv[kPerThread];
    auto issue = [&](int k, u32x4 (&dst)[kPerThread]) {
        const u32x4 *base = reinterpret_cast<const u32x4 *>(layer_ptrs[k % copies]) + (size_t)blockIdx.x * per_group16;
#pragma unroll
        for (int u = 0; u < kPerThread; u++) {
            const int i = tid + u * 1024;
            dst[u] = __builtin_nontemporal_load(base + (i < per_group16 ? i : 0));      // a thread past the share repeats element 0
        }
    };
    issue(0, v);
    for (int k = 0; k < layers; k++) {
        if (k + 1 < layers) issue(k + 1, nv);
#pragma unroll
        for (int u = 0; u < kPerThread; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
#pragma unroll
        for (int u = 0; u < kPerThread; u++) v[u] = nv[u];
    }
    if (acc == 0x9E3779B9u && sink) sink[0] = acc;
}

// LDS read instructions, sixteen waves of a workgroup issuing eight of a kind and waiting, `iters` times.
// KIND 0: ds_read_b32, every lane its own column of a row (the decode's gather); 1: ds_read2st64_b32 (two dwords
// 256 bytes apart: the reload of the activation registers in the chain kernel); 2: ds_read_b64; 3: ds_read_b128
template <int KIND>
__global__ __launch_bounds__(1024) void probe_lds_kernel(int iters, uint32_t seed, uint32_t *sink)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    extern __shared__ uint32_t probe_lds[];
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 16384; i += 1024) probe_lds[i] = (uint32_t)i * 64u;
    __syncthreads();
    const uint32_t base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(probe_lds));
    const uint32_t addr = base + lane * (KIND == 2 ? 8 : KIND == 3 ? 16 : 4);
    uint32_t acc = seed;
    for (int it = 0; it < iters; it++) {
        if (KIND == 0) {
            uint32_t t0, t1, t2, t3, t4, t5, t6, t7;
            asm volatile(
                "ds_read_b32 %0, %8 offset:0\n ds_read_b32 %1, %8 offset:256\n ds_read_b32 %2, %8 offset:512\n"
                "ds_read_b32 %3, %8 offset:768\n ds_read_b32 %4, %8 offset:1024\n ds_read_b32 %5, %8 offset:1280\n"
                "ds_read_b32 %6, %8 offset:1536\n ds_read_b32 %7, %8 offset:1792\n s_waitcnt lgkmcnt(0)\n"
                : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7) : "v"(addr) : "memory");
            acc ^= t0 ^ t1 ^ t2 ^ t3 ^ t4 ^ t5 ^ t6 ^ t7;
        } else if (KIND == 1 || KIND == 2) {
            u32x2 t0, t1, t2, t3, t4, t5, t6, t7;
            if (KIND == 1)
                asm volatile(
                    "ds_read2st64_b32 %0, %8 offset0:0 offset1:1\n ds_read2st64_b32 %1, %8 offset0:2 offset1:3\n"
                    "ds_read2st64_b32 %2, %8 offset0:4 offset1:5\n ds_read2st64_b32 %3, %8 offset0:6 offset1:7\n"
                    "ds_read2st64_b32 %4, %8 offset0:8 offset1:9\n ds_read2st64_b32 %5, %8 offset0:10 offset1:11\n"
                    "ds_read2st64_b32 %6, %8 offset0:12 offset1:13\n ds_read2st64_b32 %7, %8 offset0:14 offset1:15\n s_waitcnt lgkmcnt(0)\n"
                    : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7) : "v"(addr) : "memory");
            else
                asm volatile(
                    "ds_read_b64 %0, %8 offset:0\n ds_read_b64 %1, %8 offset:512\n ds_read_b64 %2, %8 offset:1024\n"
                    "ds_read_b64 %3, %8 offset:1536\n ds_read_b64 %4, %8 offset:2048\n ds_read_b64 %5, %8 offset:2560\n"
                    "ds_read_b64 %6, %8 offset:3072\n ds_read_b64 %7, %8 offset:3584\n s_waitcnt lgkmcnt(0)\n"
                    : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7) : "v"(addr) : "memory");
            acc ^= t0.x ^ t1.y ^ t2.x ^ t3.y ^ t4.x ^ t5.y ^ t6.x ^ t7.y;
        } else {
            u32x4 t0, t1, t2, t3, t4, t5, t6, t7;
            asm volatile(
                "ds_read_b128 %0, %8 offset:0\n ds_read_b128 %1, %8 offset:1024\n ds_read_b128 %2, %8 offset:2048\n"
                "ds_read_b128 %3, %8 offset:3072\n ds_read_b128 %4, %8 offset:4096\n ds_read_b128 %5, %8 offset:5120\n"
                "ds_read_b128 %6, %8 offset:6144\n ds_read_b128 %7, %8 offset:7168\n s_waitcnt lgkmcnt(0)\n"
                : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7) : "v"(addr) : "memory");
            acc ^= t0.x ^ t1.y ^ t2.z ^ t3.w ^ t4.x ^ t5.y ^ t6.z ^ t7.w;
        }
    }
    if (acc == 0x9E3779B9u && sink) sink[0] = acc;
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

// `layers` layers of `layer_bytes` each (a multiple of 16 * workgroups; layer k is layer_ptrs[k % copies], device pointers
// in device memory), read by `workgroups` resident workgroups in one launch; nothing is written
extern "C" int rptc_probe_read_chain(const void *layer_ptrs, int copies, int layers, int64_t layer_bytes, int workgroups, void *sink,
                                     void *stream)
{
    if (!layer_ptrs) return -1;
    if (copies < 1 || layers < 1 || workgroups < 1 || layer_bytes < 16 || layer_bytes % (16 * (int64_t)workgroups) != 0) return -2;
    const int64_t per_group16 = layer_bytes / 16 / workgroups;
    if (per_group16 > 1024 * kPerThread) return -5;
    hipLaunchKernelGGL(probe_read_chain_kernel, dim3(workgroups), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint64_t *>(layer_ptrs), copies, layers, (int)per_group16, static_cast<uint32_t *>(sink));
    return (int)hipGetLastError();
}

// `iters` rounds of 8 LDS read instructions of one kind in every wave of `workgroups` 1024-thread workgroups;
// kind: 0 ds_read_b32, 1 ds_read2st64_b32, 2 ds_read_b64, 3 ds_read_b128
extern "C" int rptc_probe_lds(int kind, int iters, int workgroups, void *sink, void *stream)
{
    if (kind < 0 || kind > 3 || iters < 1 || workgroups < 1) return -2;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t *out = static_cast<uint32_t *>(sink);
    static bool allowed = false;
    if (!allowed) {
        int rc = 0;
        rc = rc ? rc : (int)hipFuncSetAttribute(reinterpret_cast<const void *>(probe_lds_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        rc = rc ? rc : (int)hipFuncSetAttribute(reinterpret_cast<const void *>(probe_lds_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        rc = rc ? rc : (int)hipFuncSetAttribute(reinterpret_cast<const void *>(probe_lds_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        rc = rc ? rc : (int)hipFuncSetAttribute(reinterpret_cast<const void *>(probe_lds_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (rc) return rc;
        allowed = true;
    }
#define RPTC_PROBE_GO(K) hipLaunchKernelGGL(probe_lds_kernel<K>, dim3(workgroups), dim3(1024), 100 * 1024, s, iters, 12345u, out)
    switch (kind) {
    case 0: RPTC_PROBE_GO(0); break;
    case 1: RPTC_PROBE_GO(1); break;
    case 2: RPTC_PROBE_GO(2); break;
    default: RPTC_PROBE_GO(3); break;
    }
#undef RPTC_PROBE_GO
    return (int)hipGetLastError();
}
