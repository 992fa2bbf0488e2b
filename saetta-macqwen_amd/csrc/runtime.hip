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

// The set-up of a device (its architecture checked, the code objects loaded, the kernels' LDS
// limits raised) runs once per device, the first time a call finds that device current.
namespace {
constexpr int MAX_DEVICES = 64;
struct DeviceSetup {
    std::once_flag once;
    int status = SAETTA_OK;
    char why[256] = "";
};
DeviceSetup g_devices[MAX_DEVICES];
}  // namespace

int ensure_device() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(SAETTA_E_DEVICE, "no HIP device: %s", hipGetErrorString(e));
    }
    if (dev < 0 || dev >= MAX_DEVICES) return fail(SAETTA_E_DEVICE, "device index %d (up to %d)", dev, MAX_DEVICES - 1);
    DeviceSetup &d = g_devices[dev];
    std::call_once(d.once, [&d, dev] {
        hipDeviceProp_t prop;
        hipError_t e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) {
            d.status = SAETTA_E_DEVICE;
            snprintf(d.why, sizeof d.why, "no HIP device: %s", hipGetErrorString(e));
            (void)hipGetLastError();
            return;
        }
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
            d.status = SAETTA_E_DEVICE;
            snprintf(d.why, sizeof d.why, "device is %s; this library is built for gfx950 only", prop.gcnArchName);
            return;
        }
        int (*const setups[])() = {setup_kv_quant, setup_prep, setup_deltanet, setup_decode, setup_prefill};
        for (auto setup : setups) {
            if (int rc = setup()) {
                d.status = SAETTA_E_DEVICE;
                snprintf(d.why, sizeof d.why, "kernels do not load: %s", hipGetErrorString(hipError_t(rc)));
                (void)hipGetLastError();
                return;
            }
        }
    });
    if (d.status != SAETTA_OK) return fail(d.status, "%s", d.why);
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
