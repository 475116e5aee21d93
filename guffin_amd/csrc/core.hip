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
    resident_init(prop.multiProcessorCount);
    if (gemv_packed_init(device, prop.multiProcessorCount) != 0)
        return fail(GUFFIN_E_HIP, "init: could not take the address of the static scratch array on this device");
    return GUFFIN_OK;
}

extern "C" int guffin_vocab_map_invert(const int32_t* draft_to_target, uint32_t draft_vocab, uint32_t target_vocab,
                                       int32_t* target_to_draft, uint32_t* mapped_count) {
    if (!draft_to_target || !target_to_draft) return fail(GUFFIN_E_ARG, "vocab_map_invert: null pointer");
    if (draft_vocab == 0 || target_vocab == 0) return fail(GUFFIN_E_SHAPE, "vocab_map_invert: empty vocabulary");
    for (uint32_t t = 0; t < target_vocab; ++t) target_to_draft[t] = -1;
    uint32_t mapped = 0;
    for (uint32_t d = 0; d < draft_vocab; ++d) {
        const int32_t t = draft_to_target[d];
        if (t < -1 || (t >= 0 && static_cast<uint32_t>(t) >= target_vocab))
            return fail(GUFFIN_E_ARG, "vocab_map_invert: map token is out of bounds");
        if (t < 0) continue;
        if (target_to_draft[t] != -1) return fail(GUFFIN_E_ARG, "vocab_map_invert: map is not injective");
        target_to_draft[t] = static_cast<int32_t>(d);
        ++mapped;
    }
    if (mapped == 0) return fail(GUFFIN_E_ARG, "vocab_map_invert: intersection is empty");
    if (mapped_count) *mapped_count = mapped;
    return GUFFIN_OK;
}
