// A plain streaming read, for calibration only: how fast ONE launch of `workgroups` workgroups can
// pull `bytes` bytes from HBM when it computes nothing.  It is what bench.py holds the decode
// kernel's launch time against (a launch that streams 35 MB lasts only a few microseconds, and the
// launch itself and the ramp of the memory system are a fixed part of that).  Built into its own
// library (libsaetta_calib.so): not part of the product, not declared in include/saetta_hip.h.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Workgroup w reads the w-th of `gridDim.x` equal contiguous shares, 16 bytes per lane and load,
// UNROLL loads of a lane in flight at once, the whole workgroup striding through the share.
template <int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void calib_read_kernel(const u32x4 *src, size_t n16, uint32_t *sink) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t begin = per * blockIdx.x, end = begin + per < n16 ? begin + per : n16;
    u32x4 acc = {0, 0, 0, 0};
    size_t i = begin + threadIdx.x;
    for (; i + size_t(UNROLL - 1) * THREADS < end; i += size_t(UNROLL) * THREADS) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = __builtin_nontemporal_load(src + i + size_t(u) * THREADS);
#pragma unroll
        for (int u = 0; u < UNROLL; u++) acc ^= v[u];
    }
    for (; i < end; i += THREADS) acc ^= __builtin_nontemporal_load(src + i);
    // never true for the data bench.py fills in (all ones), but the compiler cannot know
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[blockIdx.x] = acc.x;
}
}  // namespace

// variant: 0 = 256 threads x 8 loads in flight, 1 = 512 x 4, 2 = 1024 x 4, 3 = 1024 x 2
extern "C" int saetta_calib_read(void *stream, const void *src, size_t bytes, uint32_t workgroups, uint32_t variant,
                                 void *sink) {
    if (!src || !sink || bytes % 16 || !workgroups || (reinterpret_cast<uintptr_t>(src) & 15)) return -1;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const u32x4 *p = static_cast<const u32x4 *>(src);
    uint32_t *k = static_cast<uint32_t *>(sink);
    const size_t n16 = bytes / 16;
    switch (variant) {
        case 0: calib_read_kernel<256, 8><<<workgroups, 256, 0, s>>>(p, n16, k); break;
        case 1: calib_read_kernel<512, 4><<<workgroups, 512, 0, s>>>(p, n16, k); break;
        case 2: calib_read_kernel<1024, 4><<<workgroups, 1024, 0, s>>>(p, n16, k); break;
        case 3: calib_read_kernel<1024, 2><<<workgroups, 1024, 0, s>>>(p, n16, k); break;
        default: return -1;
    }
    return int(hipGetLastError());
}
