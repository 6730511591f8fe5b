// Library-wide pieces of the C ABI: per-device state, status text, version.
#include <mutex>
#include <string.h>

#include "rptc_common.hpp"

namespace rptc {

int prepare_decompress();
int prepare_matvec();
int prepare_matvec_loop();
int prepare_matvec_steady();
int prepare_matvec_t(int device);
int prepare_matmul(int device);
int prepare_hadamard();
int prepare_decode_glue(int device);
int prepare_viterbi();
void matmul_counters(int device, uint32_t **counters, int *count);
void matvec_t_counters(int device, uint32_t **counters, int *count);
void attn_counters(int device, uint32_t **counters, int *count);

constexpr int kMaxDevices = 64;
static DeviceInfo g_devices[kMaxDevices];
static bool g_ready[kMaxDevices];
static std::mutex g_mutex;

int device_info(DeviceInfo **out)
{
    int dev = -1;
    int rc = (int)hipGetDevice(&dev);
    if (rc) return rc;
    if (dev < 0 || dev >= kMaxDevices) return RPTC_EDEVICE;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_ready[dev]) {
        hipDeviceProp_t prop;
        rc = (int)hipGetDeviceProperties(&prop, dev);
        if (rc) return rc;
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return RPTC_EDEVICE;
        DeviceInfo &d = g_devices[dev];
        d.device = dev;
        d.cus = prop.multiProcessorCount;
        if ((rc = (int)hipEventCreate(&d.ev_start))) return rc;
        if ((rc = (int)hipEventCreate(&d.ev_stop))) return rc;
        if ((rc = prepare_decompress())) return rc;
        if ((rc = prepare_matvec())) return rc;
        if ((rc = prepare_matvec_loop())) return rc;
        if ((rc = prepare_matvec_steady())) return rc;
        if ((rc = prepare_matvec_t(dev))) return rc;
        if ((rc = prepare_matmul(dev))) return rc;
        if ((rc = prepare_hadamard())) return rc;
        if ((rc = prepare_decode_glue(dev))) return rc;
        if ((rc = prepare_viterbi())) return rc;
        g_ready[dev] = true;
    }
    *out = &g_devices[dev];
    return 0;
}

// Counts the arrival counters that are not zero, and clears them when asked to.
static __device__ __align__(256) uint32_t g_check_result[64];

__global__ void scratch_check_clear_kernel(uint32_t *result) { *result = 0u; }

__global__ __launch_bounds__(256) void scratch_check_kernel(uint32_t *counters, int count, int reset, uint32_t *result)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    if (__hip_atomic_load(&counters[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
        atomicAdd(result, 1u);
        if (reset) __hip_atomic_store(&counters[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace rptc

extern "C" int rptc_scratch_check(int reset, int *nonzero, void *stream)
{
    using namespace rptc;
    if (!nonzero) return RPTC_ENULL;
    DeviceInfo *d;
    int rc = device_info(&d);
    if (rc) return rc;
    uint32_t *result;
    if ((rc = (int)hipGetSymbolAddress(reinterpret_cast<void **>(&result), HIP_SYMBOL(g_check_result)))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(scratch_check_clear_kernel, dim3(1), dim3(1), 0, s, result);
    void (*const sets[3])(int, uint32_t **, int *) = {matmul_counters, matvec_t_counters, attn_counters};
    for (auto get : sets) {
        uint32_t *counters;
        int count;
        get(d->device, &counters, &count);
        hipLaunchKernelGGL(scratch_check_kernel, dim3((count + 255) / 256), dim3(256), 0, s, counters, count, reset, result);
    }
    if ((rc = (int)hipGetLastError())) return rc;
    uint32_t host = 0;
    if ((rc = (int)hipMemcpyAsync(&host, result, sizeof(uint32_t), hipMemcpyDeviceToHost, s))) return rc;
    if ((rc = (int)hipStreamSynchronize(s))) return rc;
    *nonzero = (int)host;
    return 0;
}

extern "C" int rptc_version(void) { return 200; }

extern "C" int rptc_init(void)
{
    rptc::DeviceInfo *d;
    return rptc::device_info(&d);
}

extern "C" const char *rptc_status_string(int status)
{
    switch (status) {
    case RPTC_OK: return "success";
    case RPTC_ENULL: return "a required pointer is NULL";
    case RPTC_ESHAPE: return "a size breaks the op's shape rule";
    case RPTC_EALIGN: return "a pointer is not 16-byte aligned";
    case RPTC_EMODE: return "carry_mode must be RPTC_AS_WRITTEN (0) or RPTC_CONTINUOUS (1)";
    case RPTC_ELIMIT: return "a size exceeds what the kernel supports";
    case RPTC_EDEVICE: return "the current device is not a gfx950 GPU";
    case RPTC_EALIAS: return "an output buffer aliases an input the op still reads";
    case RPTC_EDEPEND: return "a layer of the chain reads or overwrites what a layer of the chain writes: run such layers as separate launches";
    default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown rptc status";
}
