// The matrix-core side of bench.py's calibration: what rate of v_mfma_f32_32x32x16_f16 ONE launch of the prefill
// attention kernel's shape (one workgroup of 8 waves per CU, two waves per SIMD) sustains when it does nothing but
// the multiplications, and at what shader clock.  Three kernels:
//   0  MFMAs back to back on operands that never change (what the matrix cores issue at best),
//   1  MFMAs back to back on operands that change with every instruction (8 + 8 registers of random data):
//      the same instruction count, but the multipliers' inputs toggle as they do on real keys and queries,
//   2  the prefill kernel's own inner loop without its softmax: per step and wave one stream_block (32 MFMAs whose
//      A operands are fresh 1 KB fragment reads from LDS, the wave's 8 KB share of the global -> LDS copies in
//      between), then the wait for the copies and the workgroup barrier.
// The chip holds a power limit by lowering the shader clock, so the three differ in clock, not in cycles: the
// clock (cycle counter over the 100 MHz counter, wave 0 of every workgroup) is reported beside the rate.
// Built into libsaetta_calib.so: not part of the product, not declared in include/saetta_hip.h.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#include "prefill_stream.hpp"

constexpr int WAVES = 8, THREADS = 64 * WAVES;
constexpr int PART_BYTES = 16384;           // a K or V^T part of a block of 32 keys, as the prefill kernel stages them
constexpr int LDS_BYTES = 8 * PART_BYTES;   // its ring: four K parts, four V^T parts

__device__ __forceinline__ void stamp(unsigned long long *out, unsigned long long c0, unsigned long long r0) {
    const unsigned long long c1 = clock64(), r1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) out[2 * blockIdx.x] = c1 - c0, out[2 * blockIdx.x + 1] = r1 - r0;
}

// 16-byte piece i of this lane from the operand buffer (any data will do; the pieces differ from lane to lane).
__device__ __forceinline__ half8 piece(const unsigned char *operands, uint32_t i) {
    return __builtin_bit_cast(half8, *reinterpret_cast<const u32x4 *>(operands + (size_t(i) * THREADS + threadIdx.x) * 16));
}

template <bool FRESH>
__global__ __launch_bounds__(THREADS, 2) void calib_mfma_registers_kernel(const unsigned char *operands, uint32_t steps,
                                                                          unsigned long long *out, float *sink) {
    half8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) a[i] = piece(operands, FRESH ? i : 0), b[i] = piece(operands, FRESH ? 8 + i : 8);
    floatx16 o[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] = 0.0f;
    }
    const unsigned long long c0 = clock64(), r0 = __builtin_amdgcn_s_memrealtime();
    for (uint32_t step = 0; step < steps; step++) {
#pragma unroll
        for (int i = 0; i < 32; i++)
            o[i & 7] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[FRESH ? i & 7 : 0], b[FRESH ? (i * 5 + 3) & 7 : 0], o[i & 7], 0, 0, 0);
    }
    stamp(out, c0, r0);
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) acc += o[i][0] + o[i][15];
    if (acc == 12345.678f) sink[blockIdx.x] = acc;  // (keeps the products alive)
}

__global__ __launch_bounds__(THREADS, 2) void calib_mfma_stream_kernel(const unsigned char *operands, uint32_t parts, uint32_t steps,
                                                                       unsigned long long *out, float *sink) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char tiles[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(tiles)), lane16 = lane * 16;
    half8 q[16], p[2];
#pragma unroll
    for (int i = 0; i < 16; i++) q[i] = piece(operands, i);
    p[0] = piece(operands, 16), p[1] = piece(operands, 17);
    floatx16 o[8], s;
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] = 0.0f;
    }
    // the ring's first contents: every wave brings in two halves of parts
    uint32_t at = (blockIdx.x * 61u) % parts;  // the part of the buffer this workgroup reads next (they walk it apart from each other)
    for (int h = 0; h < 2; h++) {
        Copy cp;
        cp.src = reinterpret_cast<uint64_t>(operands) + uint64_t(at) * PART_BYTES + (wave & 1) * 8192;
        cp.dst = lds0 + ((wave >> 1) + 4 * h) * PART_BYTES + (wave & 1) * 8192;
        copy_plain(cp, lane16);
        at = at + 1 < parts ? at + 1 : 0;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const unsigned long long c0 = clock64(), r0 = __builtin_amdgcn_s_memrealtime();
    for (uint32_t step = 0; step < steps; step++) {
        // as in the prefill kernel: the workgroup copies four parts per step, wave w half (w % 2) of part w / 2 of them,
        // and reads one K part and one V^T part per wave (the two waves of a SIMD different ones)
        const uint32_t slot = (2 * step + (wave >> 2)) & 3;
        Copy cp;
        cp.src = reinterpret_cast<uint64_t>(operands) + uint64_t((at + (wave >> 1)) % parts) * PART_BYTES + (wave & 1) * 8192;
        cp.dst = lds0 + ((((wave >> 1) & 1) * 4) + ((2 * step + 2 + (wave >> 2)) & 3)) * PART_BYTES + (wave & 1) * 8192;
        stream_block(s, o, q, p, lds0 + slot * PART_BYTES + lane16, lds0 + (4 + slot) * PART_BYTES + lane16, cp, lane16);
        at = at + 4 < parts ? at + 4 : at + 4 - parts;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    stamp(out, c0, r0);
    float acc = s[0];
#pragma unroll
    for (int i = 0; i < 8; i++) acc += o[i][0] + o[i][15];
    if (acc == 12345.678f) sink[blockIdx.x] = acc;
}
}  // namespace

// `steps` times 32 MFMAs per wave in `workgroups` workgroups of 8 waves.  operands: `bytes` of any f16 data (at least
// 1 MiB, a multiple of 16 KiB, 16-byte aligned; variant 2 walks all of it, so its size decides where the copies come
// from).  out: 2 x workgroups 64-bit words (shader cycles, 100 MHz ticks of each workgroup's loop); sink: workgroups floats.
extern "C" int saetta_calib_mfma(void *stream, uint32_t variant, uint32_t steps, uint32_t workgroups, const void *operands,
                                 size_t bytes, void *out, void *sink) {
    if (!operands || !out || !sink || !workgroups || !steps || bytes < (1u << 20) || bytes % PART_BYTES ||
        (reinterpret_cast<uintptr_t>(operands) & 15))
        return -1;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const unsigned char *src = static_cast<const unsigned char *>(operands);
    unsigned long long *o = static_cast<unsigned long long *>(out);
    float *k = static_cast<float *>(sink);
    switch (variant) {
        case 0: calib_mfma_registers_kernel<false><<<workgroups, THREADS, 0, st>>>(src, steps, o, k); break;
        case 1: calib_mfma_registers_kernel<true><<<workgroups, THREADS, 0, st>>>(src, steps, o, k); break;
        case 2:
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(calib_mfma_stream_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES))
                return -3;
            calib_mfma_stream_kernel<<<workgroups, THREADS, LDS_BYTES, st>>>(src, uint32_t(bytes / PART_BYTES), steps, o, k);
            break;
        default: return -1;
    }
    return int(hipGetLastError());
}
