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

// The same read through the path the decode kernel uses: workgroup w brings its share into LDS
// with global_load_lds_dwordx4 (1 KB per instruction, no registers), WAVES waves each issuing
// every WAVES-th instruction of the share back to back, then waiting for all of them.  The share
// must fit the 160 KB of LDS (it does for 256 workgroups and one layer's 35 MB).
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void calib_dma_kernel(const unsigned char *src, size_t bytes, uint32_t *sink) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const size_t per = (bytes / 1024 + gridDim.x - 1) / gridDim.x;  // instructions per workgroup
    const size_t begin = per * blockIdx.x * 1024;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(lds_raw));
    const unsigned char *base = src + begin;
    const size_t last = bytes - begin >= 16 ? bytes - begin - 16 : 0;  // loads past the buffer's end read its last 16 bytes
    if (begin >= bytes) return;
    for (uint32_t i = wave; i < per; i += WAVES) {
        size_t off = size_t(i) * 1024 + lane * 16;
        off = off < last ? off : last;
        asm volatile("s_mov_b32 m0, %0\n"
                     "s_nop 0\n"
                     "global_load_lds_dwordx4 %1, %2\n"
                     :
                     : "s"(lds0 + i * 1024), "v"(uint32_t(off)), "s"(base)
                     : "memory", "m0");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const uint32_t v = *reinterpret_cast<const uint32_t *>(lds_raw + threadIdx.x * 4);
    if (v == 0x9e3779b9u) sink[blockIdx.x] = v;
}
}  // namespace

// variant: 0 = 256 threads x 8 loads in flight, 1 = 512 x 4, 2 = 1024 x 4, 3 = 1024 x 2; 4..7 = to LDS with 4, 8, 12, 16 waves
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
        case 4: case 5: case 6: case 7: {
            // LDS-DMA readers: 4, 8, 12, 16 waves
            const size_t lds = ((bytes / 1024 + workgroups - 1) / workgroups) * 1024;
            if (lds > 160 * 1024) return -2;
            const unsigned char *b = static_cast<const unsigned char *>(src);
            void (*kern)(const unsigned char *, size_t, uint32_t *) =
                variant == 4 ? calib_dma_kernel<4> : variant == 5 ? calib_dma_kernel<8> : variant == 6 ? calib_dma_kernel<12> : calib_dma_kernel<16>;
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)) return -3;
            const int waves = variant == 4 ? 4 : variant == 5 ? 8 : variant == 6 ? 12 : 16;
            kern<<<workgroups, waves * 64, lds < 4096 ? 4096 : lds, s>>>(b, bytes, k);
            break;
        }
        default: return -1;
    }
    return int(hipGetLastError());
}
