// Library-wide pieces of the C ABI: per-device state, status text, version.
#include <mutex>
#include <string.h>

#include "rptc_common.hpp"

namespace rptc {

int prepare_decompress();
int prepare_matvec();
int prepare_matvec_t(int device);
int prepare_matmul(int device);
int prepare_hadamard();
int prepare_decode_glue(int device);
int prepare_viterbi();

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

}  // namespace rptc

extern "C" int rptc_version(void) { return 100; }

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
    default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown rptc status";
}
