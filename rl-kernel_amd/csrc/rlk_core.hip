// Error reporting, version and device query of the librlk_hip C ABI.
#include "rlk_common.hpp"

#include <string.h>

namespace {
thread_local char g_last_error[256] = "";
}

int rlk_fail(int code, const char* msg)
{
    strncpy(g_last_error, msg ? msg : "", sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return code;
}

extern "C" {

int rlk_version(void) { return 101; }

const char* rlk_last_error(void) { return g_last_error; }

int rlk_device_info(int32_t device, int32_t* compute_units, int32_t* max_clock_khz)
{
    if (!compute_units || !max_clock_khz) return rlk_fail(RLK_ERR_ARG, "rlk_device_info: null output pointer");
    int cu = 0, khz = 0;
    hipError_t e = hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, device);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, device);
    if (e != hipSuccess) return rlk_fail(RLK_ERR_ARG, hipGetErrorString(e));
    *compute_units = cu;
    *max_clock_khz = khz;
    return 0;
}

}  // extern "C"
