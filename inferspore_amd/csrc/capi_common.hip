// Library-wide pieces of the C ABI: status strings, launch-error bookkeeping, device check.
#include <string.h>

#include <atomic>

#include "isp_common.h"

namespace isp {

static thread_local int t_last_hip_error = 0;

int note_launch(hipError_t e) {
    if (e == hipSuccess) return ISP_OK;
    t_last_hip_error = (int)e;
    return ISP_ERR_LAUNCH;
}

// Process-wide launch-heuristic overrides.  Relaxed atomics: a launcher reads each knob once per call,
// so a thread that sets a knob while others launch changes which variant later launches pick (never
// their results), without a data race.
static std::atomic<int> g_tuning[ISP_TUNE_COUNT];

int resident_waves() {
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cached[kMaxDevices];  // every thread stores the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256 * 32;
    int waves = cached[dev].load(std::memory_order_relaxed);
    if (waves == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        waves = cus * 32;  // 4 SIMDs x 8 wavefronts per compute unit
        cached[dev].store(waves, std::memory_order_relaxed);
    }
    return waves;
}

int tuning(int knob) {
    return (knob >= 0 && knob < ISP_TUNE_COUNT) ? g_tuning[knob].load(std::memory_order_relaxed) : 0;
}

}  // namespace isp

extern "C" {

int isp_tuning_set(int knob, int value) {
    if (knob < 0 || knob >= ISP_TUNE_COUNT) return ISP_ERR_BAD_SHAPE;
    return isp::g_tuning[knob].exchange(value, std::memory_order_relaxed);
}

const char* isp_version(void) { return "inferspore_amd 0.1 (gfx950)"; }

const char* isp_strerror(int status) {
    switch (status) {
        case ISP_OK: return "ok";
        case ISP_ERR_NULL_POINTER: return "a required pointer is NULL";
        case ISP_ERR_BAD_SHAPE: return "negative or inconsistent extents";
        case ISP_ERR_UNSUPPORTED: return "extents outside what the kernels implement";
        case ISP_ERR_LAUNCH: return "HIP reported an error at kernel launch";
        case ISP_ERR_DEVICE: return "no usable gfx950 device";
        default: return "unknown status";
    }
}

int isp_last_hip_error(void) { return isp::t_last_hip_error; }

int isp_init(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return ISP_ERR_DEVICE;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return ISP_ERR_DEVICE;
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return ISP_ERR_DEVICE;
    return ISP_OK;
}

}  // extern "C"
