// The group arithmetic of the KV-cache quantizer, shared by the kernels that produce codes.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdint>

#include "../../include/saetta_hip.h"

namespace saetta {

// A lane holds the 32 / BITS neighbouring values that make one u32 of codes; the group of 64 is
// SAETTA_QUANT_GROUP * BITS / 32 neighbouring lanes of the wavefront (all of them must call this
// together).  Returns the lane's word, lowest bits first, and the group's scale and bias.
// Semantics: quantize() of the reference's CPU code (src/kv_quant.rs:54-87), bit for bit: every
// float operation that decides a bit is spelled with a rounding intrinsic, so the compiler can
// neither fuse nor reassociate:
//   s   = half_rn((hi - lo) / levels)      IEEE divide
//   z   = half_rn(lo)
//   inv = s > 0 ? 1 / f32(s) : 0           IEEE divide
//   q   = clamp(rint((v - f32(z)) * inv), 0, levels), NaN -> 0
template <int BITS>
__device__ __forceinline__ uint32_t quantize_lane(const float (&v)[32 / BITS], __half &s, __half &z) {
    constexpr int VPL = 32 / BITS;
    constexpr int LANES = SAETTA_QUANT_GROUP / VPL;
    constexpr float LEVELS = float((1u << BITS) - 1);
    // fminf/fmaxf return the other operand when one is NaN, as f32::min/max do.
    float lo = INFINITY, hi = -INFINITY;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        lo = fminf(lo, v[i]);
        hi = fmaxf(hi, v[i]);
    }
#pragma unroll
    for (int step = 1; step < LANES; step *= 2) {
        lo = fminf(lo, __shfl_xor(lo, step));
        hi = fmaxf(hi, __shfl_xor(hi, step));
    }
    s = __float2half_rn(__fdiv_rn(__fsub_rn(hi, lo), LEVELS));
    z = __float2half_rn(lo);
    const float sf = __half2float(s), zf = __half2float(z);
    const float inv = sf > 0.0f ? __fdiv_rn(1.0f, sf) : 0.0f;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        float r = rintf(__fmul_rn(__fsub_rn(v[i], zf), inv));
        // NaN fails both comparisons of the clamp in Rust and casts to 0.
        uint32_t q = (r != r) ? 0u : uint32_t(fminf(fmaxf(r, 0.0f), LEVELS));
        packed |= q << (i * BITS);
    }
    return packed;
}

}  // namespace saetta
