// Host-side plumbing shared by every entry point: thread-local error text,
// launch-status checks and cached device properties.
#include "pt_common.h"

#include <mutex>

namespace pt {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) {
    g_last_error = msg;
}

int fail(int code, const std::string &msg) {
    g_last_error = msg;
    return code;
}

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(PT_ERR_LAUNCH, std::string(what) + ": " + hipGetErrorString(e));
    return PT_OK;
}

int device_cu_count() {
    constexpr int     MAX_DEV = 64;
    static int        cached[MAX_DEV];
    static std::mutex mu;
    int               dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV)
        return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            n <= 0)
            n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

} // namespace pt

extern "C" {

const char *pt_last_error(void) {
    return pt::g_last_error.c_str();
}

int pt_abi_version(void) {
    return 2;
}

int pt_device_cu_count(void) {
    return pt::device_cu_count();
}

} // extern "C"
