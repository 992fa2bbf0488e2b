// Shared by the kernel files of the gfx950 attention path: error plumbing for
// the C ABI and a few device helpers.  HIP/CDNA4 only.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/saetta_hip.h"

namespace saetta {

// Per-thread text of the last failure, returned by saetta_last_error().
char *error_buffer();
int fail(int code, const char *fmt, ...);
// Checks the device once per process; 0 or SAETTA_E_DEVICE.
int ensure_device();
// Turns the status of the launches since the last call into a return code; SAETTA_E_WAIT once a
// kernel on this device has left a code in the device's status word.
int launch_status(const char *what);
// Device address of the current device's sticky status word (pinned host memory): a kernel whose
// bounded wait runs out stores a non-zero code there.  nullptr before the device's set-up.
uint32_t *device_status_word();

// One-time set-up of a source file's kernels on the current device: loads their code object and
// raises their dynamic LDS limits, so that a first launch under stream capture has nothing left to
// do.  Called from ensure_device(); each returns a hipError_t as int.
int setup_kv_quant();
int setup_prep();
int setup_deltanet();
int setup_deltanet_chunk();
int setup_decode();
int setup_prefill();
// The chunked delta rule (deltanet_chunk.hip): the workspace a call needs (0: the call keeps to the
// token-by-token kernels), and the call itself (the delta rule only; the gated norm follows as for the
// token-by-token kernels) with a workspace of the caller's.
size_t deltanet_chunk_workspace_bytes(const saetta_rows_step_params &p);
int run_deltanet_chunk(hipStream_t stream, const float *mixed, const float *a, const float *b, const float *a_log,
                       const float *dt_bias, float *state, float *o, const saetta_rows_step_params &p, uint32_t channels,
                       void *workspace);
// Loads the code object `kernel` lives in.
inline int load_kernel(const void *kernel) {
    hipFuncAttributes attr;
    return int(hipFuncGetAttributes(&attr, kernel));
}

inline hipStream_t as_stream(saetta_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace saetta

#define SAETTA_REQUIRE(cond, code, ...)                       \
    do {                                                      \
        if (!(cond)) return saetta::fail((code), __VA_ARGS__); \
    } while (0)
