// Gated DeltaNet (linear attention), one token: the conv and the step after it.
//
// Reference: kernels deltanet_conv and deltanet_step (kernels/layers.metal:198-226,290-357),
// recorded by GpuDeltaNet (src/gpu_layers.rs:573-1000); CPU definition src/cpu/deltanet.rs:69-155:
//   conv:  out[c] = silu(sum_t w[c][t] * past[t][c] + w[c][K-1] * x[c]); x shifts into the state
//   step, per value head h (key head h / (v_heads / k_heads)), key dim 128:
//     q, k L2-normalised (eps inside the root), q also times 1 / sqrt(128)
//     g = exp(-exp(A_log[h]) * softplus(a[h] + dt_bias[h])),  beta = sigmoid(b[h])
//     per state row i:  S_i <- g S_i;  d = (v[i] - S_i . k) beta;  S_i += d k;  o[i] = S_i . q
//     y = o / sqrt(mean(o^2) + eps) * norm_w * silu(z)
//
// The step is a stream over the recurrent state: 32 heads x 128 x 128 f32 = 2 MB read and 2 MB
// written per layer and token, everything else is small.  One workgroup of 1024 threads per value
// head; a state row is 128 floats = 32 lanes x float4, so a wavefront takes two rows at a time
// (whole 512-byte rows per half wave: reads and writes are full cache lines), all of a wave's
// rows are requested before the first is used, and the dot products are reductions over 32 lanes
// by DPP moves (no LDS).
#include "common.hpp"
#include "lanes.hpp"

namespace saetta {
namespace {

constexpr int K_DIM = 128;
constexpr int STEP_THREADS = 1024;
constexpr int MAX_ROWS_PER_LANE = 8;  // v_dim up to 256

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }
__device__ __forceinline__ float dot4(float4 a, float4 b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

__global__ __launch_bounds__(256) void deltanet_conv_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                            float *__restrict__ state, float *__restrict__ out,
                                                            saetta_conv_params p) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const uint32_t past = p.kernel_size - 1;
    const float *wc = w + size_t(c) * p.kernel_size;
    const float xc = x[c];
    // the CPU adds the stored inputs oldest first and the new one last (src/cpu/deltanet.rs:122-126)
    float old = 0.0f;
    for (uint32_t t = 0; t < past; t++) old += wc[t] * state[size_t(t) * p.channels + c];
    for (uint32_t t = 0; t + 1 < past; t++) state[size_t(t) * p.channels + c] = state[size_t(t + 1) * p.channels + c];
    state[size_t(past - 1) * p.channels + c] = xc;
    out[c] = silu_f(old + wc[past] * xc);
}

struct StepArgs {
    const float *q, *k, *v, *a, *b, *a_log, *dt_bias;
    float *state;
    const float *z, *norm_w;
    float *y;
    saetta_step_params p;
};

__global__ __launch_bounds__(STEP_THREADS) void deltanet_step_kernel(StepArgs a) {
    __shared__ float o_lds[MAX_ROWS_PER_LANE * 32];
    __shared__ float partial[STEP_THREADS / 64];
    const uint32_t h = blockIdx.x, tid = threadIdx.x;
    const uint32_t lane32 = tid & 31, half_wave = tid >> 5;  // 32 half waves, one state row each at a time
    const uint32_t v_dim = a.p.v_dim;
    const uint32_t kh = h / (a.p.v_heads / a.p.k_heads);

    // the state rows of this half wave: i = half_wave, half_wave + 32, ... all requested up front
    float4 s[MAX_ROWS_PER_LANE];
    float *rows = a.state + size_t(h) * v_dim * K_DIM;
#pragma unroll
    for (int r = 0; r < MAX_ROWS_PER_LANE; r++) {
        const uint32_t i = half_wave + 32 * r;
        if (i < v_dim) s[r] = reinterpret_cast<const float4 *>(rows + size_t(i) * K_DIM)[lane32];
    }
    float4 qv = reinterpret_cast<const float4 *>(a.q + size_t(kh) * K_DIM)[lane32];
    float4 kv = reinterpret_cast<const float4 *>(a.k + size_t(kh) * K_DIM)[lane32];
    // normalize_qk (src/cpu/deltanet.rs:133-146): x * (scale / sqrt(x . x + eps))
    const float qi = (1.0f / sqrtf(float(K_DIM))) / sqrtf(group_reduce<32>(dot4(qv, qv), SumOp()) + a.p.eps);
    const float ki = 1.0f / sqrtf(group_reduce<32>(dot4(kv, kv), SumOp()) + a.p.eps);
    qv.x *= qi, qv.y *= qi, qv.z *= qi, qv.w *= qi;
    kv.x *= ki, kv.y *= ki, kv.z *= ki, kv.w *= ki;

    const float xg = a.a[h] + a.dt_bias[h];
    const float softplus = fmaxf(xg, 0.0f) + log1pf(expf(-fabsf(xg)));
    const float g = expf(-expf(a.a_log[h]) * softplus);
    const float beta = sigmoid_f(a.b[h]);
    const float *vh = a.v + size_t(h) * v_dim;

#pragma unroll
    for (int r = 0; r < MAX_ROWS_PER_LANE; r++) {
        const uint32_t i = half_wave + 32 * r;
        if (i < v_dim) {  // the same for the 32 lanes of a row
            float4 x = s[r];
            x.x *= g, x.y *= g, x.z *= g, x.w *= g;
            const float delta = (vh[i] - group_reduce<32>(dot4(x, kv), SumOp())) * beta;
            x.x += kv.x * delta, x.y += kv.y * delta, x.z += kv.z * delta, x.w += kv.w * delta;
            reinterpret_cast<float4 *>(rows + size_t(i) * K_DIM)[lane32] = x;
            const float o = group_reduce<32>(dot4(x, qv), SumOp());
            if (lane32 == 0) o_lds[i] = o;
        }
    }
    __syncthreads();

    // gated RMSNorm over the head's v_dim outputs, times silu(z)
    const float o = tid < v_dim ? o_lds[tid] : 0.0f;
    const float sq = group_reduce<64>(o * o, SumOp());
    if ((tid & 63) == 0) partial[tid >> 6] = sq;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < STEP_THREADS / 64; w++) total += partial[w];
    const float inv = 1.0f / sqrtf(total / float(v_dim) + a.p.eps);
    if (tid < v_dim) {
        const size_t nidx = size_t(h) * v_dim + tid;
        a.y[nidx] = o * (inv * a.norm_w[tid]) * silu_f(a.z[nidx]);
    }
}

}  // namespace
}  // namespace saetta

using namespace saetta;

extern "C" int saetta_deltanet_conv(saetta_stream_t stream, const float *x, const float *w, float *state, float *out,
                                    saetta_conv_params p) {
    SAETTA_REQUIRE(x && w && state && out, SAETTA_E_NULL, "deltanet_conv: null buffer");
    // (a kernel of one tap has no state; the reference's conv_step cannot run it either)
    SAETTA_REQUIRE(p.kernel_size >= 2 && p.kernel_size <= 16, SAETTA_E_SHAPE, "deltanet_conv: kernel size %u (2..16)",
                   p.kernel_size);
    if (int rc = ensure_device()) return rc;
    if (p.channels == 0) return SAETTA_OK;
    deltanet_conv_kernel<<<(p.channels + 255) / 256, 256, 0, as_stream(stream)>>>(x, w, state, out, p);
    return launch_status("deltanet_conv");
}

extern "C" int saetta_deltanet_step(saetta_stream_t stream, const float *q, const float *k, const float *v,
                                    const float *a, const float *b, const float *a_log, const float *dt_bias,
                                    float *state, const float *z, const float *norm_w, float *y,
                                    saetta_step_params p) {
    SAETTA_REQUIRE(q && k && v && a && b && a_log && dt_bias && state && z && norm_w && y, SAETTA_E_NULL,
                   "deltanet_step: null buffer");
    SAETTA_REQUIRE(p.k_heads > 0 && p.v_heads > 0 && p.v_heads % p.k_heads == 0, SAETTA_E_SHAPE,
                   "deltanet_step: %u value heads over %u key heads", p.v_heads, p.k_heads);
    SAETTA_REQUIRE(p.v_dim >= 1 && p.v_dim <= 32 * MAX_ROWS_PER_LANE, SAETTA_E_SHAPE,
                   "deltanet_step: value dim %u (1..256); the key dim is 128", p.v_dim);
    SAETTA_REQUIRE(aligned(q, 16) && aligned(k, 16) && aligned(state, 16), SAETTA_E_ALIGN,
                   "deltanet_step: q, k and the state must be 16-byte aligned");
    if (int rc = ensure_device()) return rc;
    StepArgs args{q, k, v, a, b, a_log, dt_bias, state, z, norm_w, y, p};
    deltanet_step_kernel<<<p.v_heads, STEP_THREADS, 0, as_stream(stream)>>>(args);
    return launch_status("deltanet_step");
}
