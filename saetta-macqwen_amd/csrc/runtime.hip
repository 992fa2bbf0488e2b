// Error plumbing and device check of the C ABI.
#include "common.hpp"

#include <cstring>
#include <mutex>

namespace saetta {

char *error_buffer() {
    static thread_local char buf[512] = "";
    return buf;
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

int ensure_device() {
    static std::once_flag once;
    static int status = SAETTA_OK;
    static char why[256] = "";
    std::call_once(once, [] {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        hipDeviceProp_t prop;
        if (e == hipSuccess) e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) {
            status = SAETTA_E_DEVICE;
            snprintf(why, sizeof why, "no HIP device: %s", hipGetErrorString(e));
            (void)hipGetLastError();
            return;
        }
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
            status = SAETTA_E_DEVICE;
            snprintf(why, sizeof why, "device is %s; this library is built for gfx950 only",
                     prop.gcnArchName);
            return;
        }
        int (*const setups[])() = {setup_kv_quant, setup_prep, setup_deltanet, setup_decode, setup_prefill};
        for (auto setup : setups) {
            if (int rc = setup()) {
                status = SAETTA_E_DEVICE;
                snprintf(why, sizeof why, "kernels do not load: %s", hipGetErrorString(hipError_t(rc)));
                (void)hipGetLastError();
                return;
            }
        }
    });
    if (status != SAETTA_OK) return fail(status, "%s", why);
    return SAETTA_OK;
}

int launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return SAETTA_OK;
    return fail(int(e), "%s: %s", what, hipGetErrorString(e));
}

}  // namespace saetta

extern "C" int saetta_init(void) { return saetta::ensure_device(); }

extern "C" const char *saetta_last_error(void) { return saetta::error_buffer(); }
