// Library-level C entry points: error text, version, device check.
#include "common.h"
#include "infllmv2_hip.h"
#include <string.h>

namespace infllmv2 {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

}  // namespace infllmv2

extern "C" const char* infllmv2_last_error(void) { return infllmv2::g_error; }

extern "C" int infllmv2_abi_version(void) { return INFLLMV2_ABI_VERSION; }

// Replaces the sm80/sm90 capability gate of flash_api.cpp:546-550: the code objects in this
// library exist for gfx950 only.
extern "C" int infllmv2_check_device(int device) {
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) {
        infllmv2::set_error("hipGetDeviceProperties(%d) failed: %s", device, hipGetErrorString(e));
        return 2;
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        infllmv2::set_error("this build only supports AMD gfx950 (MI355X); device %d is %s", device, prop.gcnArchName);
        return 1;
    }
    return 0;
}
