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
    // The device's sticky status word: pinned host memory that the kernels see through status_dev.  A
    // kernel whose bounded wait ran out stores a code there (one plain store by one lane); the host
    // reads it without synchronising.
    volatile uint32_t *status_host = nullptr;
    uint32_t *status_dev = nullptr;
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
        {
            void *host = nullptr, *devp = nullptr;
            e = hipHostMalloc(&host, 64, hipHostMallocMapped);
            if (e == hipSuccess) e = hipHostGetDevicePointer(&devp, host, 0);
            if (e != hipSuccess) {
                d.status = SAETTA_E_DEVICE;
                snprintf(d.why, sizeof d.why, "no pinned status word: %s", hipGetErrorString(e));
                (void)hipGetLastError();
                return;
            }
            memset(host, 0, 64);
            d.status_host = static_cast<volatile uint32_t *>(host);
            d.status_dev = static_cast<uint32_t *>(devp);
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

namespace {
DeviceSetup *current_setup() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return dev >= 0 && dev < MAX_DEVICES ? &g_devices[dev] : nullptr;
}
}  // namespace

uint32_t *device_status_word() {
    DeviceSetup *d = current_setup();
    return d ? d->status_dev : nullptr;
}

int launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(int(e), "%s: %s", what, hipGetErrorString(e));
    // A kernel of an EARLIER launch on this device that gave up a bounded wait has left its code in
    // the status word (this call's own launches have not run yet, as a rule): every call fails from
    // then on, until saetta_device_status(1) has cleared the word.
    DeviceSetup *d = current_setup();
    if (d && d->status_host) {
        if (const uint32_t code = *d->status_host) {
            return fail(SAETTA_E_WAIT,
                        "%s: a kernel launched earlier on this device gave up a bounded wait (status 0x%x); the "
                        "partial results of that launch are marked NaN; saetta_device_status(1) clears the status",
                        what, code);
        }
    }
    return SAETTA_OK;
}

}  // namespace saetta

extern "C" int saetta_init(void) { return saetta::ensure_device(); }

extern "C" const char *saetta_last_error(void) { return saetta::error_buffer(); }

extern "C" uint32_t saetta_device_status(int clear) {
    if (saetta::ensure_device() != SAETTA_OK) return 0;
    saetta::DeviceSetup *d = saetta::current_setup();
    if (!d || !d->status_host) return 0;
    const uint32_t code = *d->status_host;
    if (clear) *d->status_host = 0;
    return code;
}
