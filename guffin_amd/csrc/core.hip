// Library-wide host plumbing: error reporting, device binding, LDS limits.
#include "common.hpp"

#include <cstdio>
#include <cstring>

namespace guffin {

namespace {
thread_local char g_error[512] = "";
}

void set_last_error(const char* message) {
    std::snprintf(g_error, sizeof(g_error), "%s", message ? message : "");
}

int fail(int code, const char* message) {
    set_last_error(message);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return GUFFIN_OK;
    char buf[400];
    std::snprintf(buf, sizeof(buf), "%s: %s", what, hipGetErrorString(e));
    return fail(GUFFIN_E_HIP, buf);
}

int gemv_init(int cu_count);
int ops_init(int cu_count);
int gemv_packed_init(int device, int cu_count);
int head_init();

}  // namespace guffin

using namespace guffin;

extern "C" const char* guffin_hip_last_error(void) { return g_error; }

extern "C" const char* guffin_hip_arch(void) { return "gfx950"; }

extern "C" int guffin_hip_init(int device) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0)
        return fail(GUFFIN_E_HIP, "init: no HIP device is visible; this library has no CPU path");
    if (device < 0 || device >= count) return fail(GUFFIN_E_ARG, "init: device index out of range");
    if (hipSetDevice(device) != hipSuccess) return fail(GUFFIN_E_HIP, "init: hipSetDevice failed");
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return fail(GUFFIN_E_HIP, "init: cannot query the device");
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        char buf[200];
        std::snprintf(buf, sizeof(buf), "init: code object is gfx950 only, device is %s", prop.gcnArchName);
        return fail(GUFFIN_E_HIP, buf);
    }
    if (gemv_init(prop.multiProcessorCount) != 0 || ops_init(prop.multiProcessorCount) != 0 || head_init() != 0)
        return fail(GUFFIN_E_HIP, "init: could not raise a kernel's dynamic LDS limit");
    if (gemv_packed_init(device, prop.multiProcessorCount) != 0)
        return fail(GUFFIN_E_HIP, "init: could not take the address of the static scratch array on this device");
    return GUFFIN_OK;
}
