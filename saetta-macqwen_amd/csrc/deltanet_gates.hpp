// Shared by the Gated DeltaNet kernel files: the gates of a token and head.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace saetta {

// From this many tokens on (without snapshots) saetta_deltanet_rows runs the chunked form of the
// delta rule on the matrix cores (deltanet_chunk.hip); below it the token-by-token kernels.
constexpr uint32_t DELTANET_CHUNK_FROM = 128;

// g = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b), with the hardware's exp2 and log2
// (the library routines are some 150 instructions, and in the kernels the gates sit in one wave's
// path): log1p(e) as e - e^2 / 2 below 2^-10 and log(1 + e) above; the errors stay near 1e-7.
// log_g, if asked for, is the exponent itself.
__device__ __forceinline__ void fast_gates(float a_plus_bias, float exp_a_log, float b, float &g, float &beta,
                                           float *log_g = nullptr) {
    const float e = __expf(-fabsf(a_plus_bias));
    const float log1p_e = e < 0x1p-10f ? e * (1.0f - 0.5f * e) : __logf(1.0f + e);
    const float softplus = fmaxf(a_plus_bias, 0.0f) + log1p_e;
    const float lg = -exp_a_log * softplus;
    if (log_g) *log_g = lg;
    g = __expf(lg);
    beta = __builtin_amdgcn_rcpf(1.0f + __expf(-b));
}

}  // namespace saetta
