// Gated DeltaNet (linear attention): the conv and the step after it, for one token, for up to 8
// rows of a verify step, and for the tokens of a prefill chunk in order.
//
// Kernels:
//   deltanet_conv_kernel, deltanet_step_kernel          one token, the reference's two ops
//   deltanet_conv_rows_kernel, deltanet_conv_state_kernel,
//   deltanet_rows_kernel, deltanet_gated_norm_rows_kernel   any number of tokens in order (prefill chunks)
//   deltanet_rows_small_kernel, deltanet_rows_small_tail_kernel
//                                                       conv and step together for 1..8 tokens
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
#include "deltanet_gates.hpp"
#include "lanes.hpp"

#include <type_traits>

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


// ---- several tokens in one launch: verify rows and prefill chunks ------------------------------
//
// Reference: conv_rows2 + conv_state, delta_prep + delta_rows3 and the gated norm after them
// (kernels/prefill.metal:734-1116, recorded by src/prefill.rs:1433-1578), and for verify rows
// deltanet_conv_rows + deltanet_step_rows (kernels/layers.metal:510-635, src/gpu_layers.rs:686-786).
// Token t + 1 sees the state token t left, exactly as t single-token calls would.

// One thread per (channel, tile of CONV_TILE tokens).  Input i of the window of token t is
// x[i] for i >= 0 and the stored state row i + kernel_size - 1 before that; the taps are added
// oldest first, as the single-token kernel does.  The window slides in registers (KS taps known
// at compile time for the common sizes), so every x is loaded once per tile.
constexpr uint32_t CONV_TILE = 32;

__device__ __forceinline__ float conv_input(const float *x, const float *state, int i, uint32_t c,
                                            const saetta_conv_rows_params &p) {
    return i >= 0 ? x[size_t(i) * p.channels + c] : state[size_t(i + int(p.kernel_size) - 1) * p.channels + c];
}

// The same for four channels a thread (16-byte loads and stores, eight tokens' loads in flight), four taps:
// every channel's sums are taken in the same order as above, so the results are the same bit for bit.
constexpr uint32_t CONV4_AHEAD = 8;
static_assert(CONV_TILE % CONV4_AHEAD == 0, "whole groups of tokens in a tile");
__global__ __launch_bounds__(256) void deltanet_conv_rows4_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                                  const float *__restrict__ state, float *__restrict__ out,
                                                                  float *__restrict__ snaps, saetta_conv_rows_params p) {
    constexpr int KS = 4;
    const uint32_t c4 = blockIdx.x * 256 + threadIdx.x, quads = p.channels / 4;
    if (c4 >= quads) return;
    const float4 *x4 = reinterpret_cast<const float4 *>(x), *s4 = reinterpret_cast<const float4 *>(state);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    // taps[j] holds tap j of the four channels (w is [channel][4]: the thread's 16 floats lie in a row)
    float4 taps[KS];
    {
        const float4 *w4 = reinterpret_cast<const float4 *>(w) + size_t(c4) * 4;
        const float4 a = w4[0], b = w4[1], c = w4[2], d = w4[3];
        taps[0] = make_float4(a.x, b.x, c.x, d.x), taps[1] = make_float4(a.y, b.y, c.y, d.y);
        taps[2] = make_float4(a.z, b.z, c.z, d.z), taps[3] = make_float4(a.w, b.w, c.w, d.w);
    }
    const uint32_t t_begin = blockIdx.y * CONV_TILE, t_end = min(p.tokens, t_begin + CONV_TILE);
    float4 win[KS - 1];
#pragma unroll
    for (int j = 0; j < KS - 1; j++) {
        const int i = int(t_begin) - (KS - 1) + j;
        win[j] = i >= 0 ? x4[size_t(i) * quads + c4] : s4[size_t(i + KS - 1) * quads + c4];
    }
    for (uint32_t t0 = t_begin; t0 < t_end; t0 += CONV4_AHEAD) {
        float4 xt[CONV4_AHEAD];
#pragma unroll
        for (uint32_t u = 0; u < CONV4_AHEAD; u++) xt[u] = x4[size_t(min(t0 + u, p.tokens - 1)) * quads + c4];
#pragma unroll
        for (uint32_t u = 0; u < CONV4_AHEAD; u++) {
            const uint32_t t = t0 + u;
            if (t >= t_end) break;
            float4 acc = make_float4(0, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < KS - 1; j++) {
                acc.x += taps[j].x * win[j].x, acc.y += taps[j].y * win[j].y, acc.z += taps[j].z * win[j].z, acc.w += taps[j].w * win[j].w;
            }
            o4[size_t(t) * quads + c4] = make_float4(silu_f(acc.x + taps[KS - 1].x * xt[u].x), silu_f(acc.y + taps[KS - 1].y * xt[u].y),
                                                     silu_f(acc.z + taps[KS - 1].z * xt[u].z), silu_f(acc.w + taps[KS - 1].w * xt[u].w));
#pragma unroll
            for (int j = 0; j + 1 < KS - 1; j++) win[j] = win[j + 1];
            win[KS - 2] = xt[u];
            if (p.snapshots) {
                float4 *snap = reinterpret_cast<float4 *>(snaps) + size_t(t) * (KS - 1) * quads;
#pragma unroll
                for (int j = 0; j < KS - 1; j++) snap[size_t(j) * quads + c4] = win[j];
            }
        }
    }
}

template <int KS>  // taps; 0: any number (read from p), the window is re-read from memory
__global__ __launch_bounds__(256) void deltanet_conv_rows_kernel(const float *__restrict__ x,
                                                                 const float *__restrict__ w,
                                                                 const float *__restrict__ state,
                                                                 float *__restrict__ out, float *__restrict__ snaps,
                                                                 saetta_conv_rows_params p) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const int past = int(p.kernel_size) - 1;
    const float *wc = w + size_t(c) * p.kernel_size;
    const uint32_t t_begin = blockIdx.y * CONV_TILE, t_end = min(p.tokens, t_begin + CONV_TILE);
    if constexpr (KS > 0) {
        float taps[KS], win[KS - 1];
#pragma unroll
        for (int j = 0; j < KS; j++) taps[j] = wc[j];
#pragma unroll
        for (int j = 0; j < KS - 1; j++) win[j] = conv_input(x, state, int(t_begin) - (KS - 1) + j, c, p);
        for (uint32_t t = t_begin; t < t_end; t++) {
            const float xt = x[size_t(t) * p.channels + c];
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < KS - 1; j++) acc += taps[j] * win[j];
            out[size_t(t) * p.channels + c] = silu_f(acc + taps[KS - 1] * xt);
#pragma unroll
            for (int j = 0; j + 1 < KS - 1; j++) win[j] = win[j + 1];
            win[KS - 2] = xt;
            if (p.snapshots) {
                float *snap = snaps + size_t(t) * (KS - 1) * p.channels;
#pragma unroll
                for (int j = 0; j < KS - 1; j++) snap[size_t(j) * p.channels + c] = win[j];
            }
        }
    } else {
        for (uint32_t t = t_begin; t < t_end; t++) {
            float acc = 0.0f;
            for (int j = 0; j < past; j++) acc += wc[j] * conv_input(x, state, int(t) - past + j, c, p);
            out[size_t(t) * p.channels + c] = silu_f(acc + wc[past] * x[size_t(t) * p.channels + c]);
            if (p.snapshots) {
                float *snap = snaps + size_t(t) * past * p.channels;
                for (int j = 0; j < past; j++) {
                    snap[size_t(j) * p.channels + c] = conv_input(x, state, int(t) - past + 1 + j, c, p);
                }
            }
        }
    }
}

// After the outputs: the last kernel_size - 1 inputs become the state.  Rows are written in
// ascending order and row j only reads rows above it (or x), so the shift is safe in place.
__global__ __launch_bounds__(256) void deltanet_conv_state_kernel(const float *__restrict__ x, float *state,
                                                                  saetta_conv_rows_params p) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= p.channels) return;
    const int past = int(p.kernel_size) - 1;
    for (int j = 0; j < past; j++) {
        state[size_t(j) * p.channels + c] = conv_input(x, state, int(p.tokens) - past + j, c, p);
    }
}

// The delta rule over the tokens, in order.  A workgroup owns a few rows of one value head's state
// for the whole launch: LANES lanes per row, 128 / LANES state values per lane in registers.  The
// chain from one token to the next (decay, S_i . k, its sum over the row's lanes, delta, update)
// cannot be shortened, so the rows are spread as wide as the chip: 32 lanes per row make the 4096
// rows of 32 heads two wavefronts on every SIMD, one running while the other waits on its chain.
// The q and k of the head's key head are the same for all its rows: they are staged per block of 16
// tokens in LDS (double buffered; the next block's loads are in flight while this one runs),
// normalised on the way in; g, beta and v of a block sit in the lanes (lane p of each 16 holds
// token p's) and reach the others by DPP row broadcasts.
constexpr int ROWS_TB = 16;  // tokens per staged block
#ifndef ROWS_LANES_PER_ROW
#define ROWS_LANES_PER_ROW 16
#endif

struct RowsArgs {
    const float *mixed, *a, *b, *a_log, *dt_bias;
    float *state;
    float *o;      // [tokens][v_heads][v_dim], before the gated norm
    float *snaps;  // [tokens] copies of the state, or unused
    saetta_rows_step_params p;
    uint32_t channels;
};

template <int I>
__device__ __forceinline__ float row_lane(float x) {
    // value of lane I of every row of 16 lanes
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x150 + I, 0xf, 0xf, true));
}

template <int I>
struct TokenLoop {
    template <class F>
    static __device__ __forceinline__ void run(F &&f) {
        f(std::integral_constant<int, I>{});
        if constexpr (I + 1 < ROWS_TB) TokenLoop<I + 1>::run(f);
    }
};

// sum of N float4 products as a tree (N = 1 or 2): two or three dependent additions after the products
template <int N>
__device__ __forceinline__ float dot_tree(const float4 (&a)[N], const float4 (&b)[N]) {
    float sum = (a[0].x * b[0].x + a[0].y * b[0].y) + (a[0].z * b[0].z + a[0].w * b[0].w);
    if constexpr (N == 2) sum += (a[1].x * b[1].x + a[1].y * b[1].y) + (a[1].z * b[1].z + a[1].w * b[1].w);
    return sum;
}

template <bool SNAPS, int LANES>
__global__ __launch_bounds__(256) void deltanet_rows_kernel(RowsArgs a) {
    constexpr int PER_LANE = K_DIM / LANES;  // state values per lane: 8 or 4
    constexpr int F4 = PER_LANE / 4;         // as float4s
    constexpr int ROWS_PER_WG = 256 / LANES;
    static_assert(LANES == 16 || LANES == 32, "a row is one or two DPP rows");
    // a token's q and k: [q | k][float4 of the lane][lane][4] floats, so that the lanes of a row read
    // contiguous bytes
    __shared__ __attribute__((aligned(16))) float qk_lds[2][ROWS_TB][2 * K_DIM];
    __shared__ float gb_lds[2][ROWS_TB][2];
    __shared__ float o_lds[ROWS_TB][ROWS_PER_WG];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t h = blockIdx.y, part = tid % LANES, row_in_wg = tid / LANES;
    const uint32_t tok_lane = tid & 15;  // the token of a block whose g, beta and v this lane holds
    const uint32_t row = blockIdx.x * ROWS_PER_WG + row_in_wg;
    const uint32_t v_dim = a.p.v_dim, v_heads = a.p.v_heads, tokens = a.p.tokens;
    const bool live = row < v_dim;
    const uint32_t kh = h / (v_heads / a.p.k_heads);
    const uint32_t key_size = a.p.k_heads * K_DIM;
    const size_t value_size = size_t(v_heads) * v_dim;

    float4 st[F4];
    float *sp = a.state + (size_t(h) * v_dim + (live ? row : 0)) * K_DIM + part * PER_LANE;
#pragma unroll
    for (int c = 0; c < F4; c++) st[c] = live ? reinterpret_cast<const float4 *>(sp)[c] : make_float4(0, 0, 0, 0);

    const float exp_a = expf(a.a_log[h]);
    const float bias = a.dt_bias[h];
    const float q_scale = 1.0f / sqrtf(float(K_DIM));

    // ---- one block's inputs, as loaded (registers) --------------------------------------------
    // thread -> float4 `lane` of token wave + 4 j of the block: lanes 0-31 are q, 32-63 are k
    float4 raw[ROWS_TB / 4];
    float ga = 0.0f, gbv = 0.0f;  // a and b of token `tid` (threads 0-15)
    bool g_real = false;          // that token exists
    float nv = 0.0f;              // v of token `tok_lane`, this thread's row
    auto load_block = [&](uint32_t t0) {
        const uint32_t off = (lane < 32 ? 0 : key_size) + kh * K_DIM + 4 * (lane & 31);
#pragma unroll
        for (int j = 0; j < ROWS_TB / 4; j++) {
            const uint32_t t = t0 + wave + 4 * j;
            raw[j] = make_float4(0, 0, 0, 0);
            if (t < tokens) raw[j] = *reinterpret_cast<const float4 *>(a.mixed + size_t(t) * a.channels + off);
        }
        g_real = t0 + tid < tokens;
        if (tid < ROWS_TB && g_real) {
            ga = a.a[size_t(t0 + tid) * v_heads + h];
            gbv = a.b[size_t(t0 + tid) * v_heads + h];
        }
        nv = 0.0f;
        if (live && t0 + tok_lane < tokens) {
            nv = a.mixed[size_t(t0 + tok_lane) * a.channels + 2 * key_size + h * v_dim + row];
        }
    };
    // normalise (src/cpu/deltanet.rs:133-146), compute the gates, and put the block into buffer `buf`
    auto store_block = [&](int buf) {
#pragma unroll
        for (int j = 0; j < ROWS_TB / 4; j++) {
            const float4 x = raw[j];
            const float ss = group_reduce<32>(dot4(x, x), SumOp());
            const float inv = (lane < 32 ? q_scale : 1.0f) * __builtin_amdgcn_rsqf(ss + a.p.eps);
            const uint32_t f = lane & 31;  // float4 f of the vector belongs to lane f / F4, its float4 f % F4
            float *dst = &qk_lds[buf][wave + 4 * j][(lane < 32 ? 0 : K_DIM) + (f % F4) * (LANES * 4) + (f / F4) * 4];
            *reinterpret_cast<float4 *>(dst) = make_float4(x.x * inv, x.y * inv, x.z * inv, x.w * inv);
        }
        if (tid < ROWS_TB) {
            float g, beta;
            fast_gates(ga + bias, exp_a, gbv, g, beta);
            gb_lds[buf][tid][0] = g_real ? g : 1.0f;
            gb_lds[buf][tid][1] = g_real ? beta : 0.0f;
        }
    };

    load_block(0);
    store_block(0);
    float v_cur = nv;
    __syncthreads();

    int cur = 0;
    for (uint32_t t0 = 0; t0 < tokens; t0 += ROWS_TB) {
        const bool more = t0 + ROWS_TB < tokens;
        if (more) load_block(t0 + ROWS_TB);
        const float g_mine = gb_lds[cur][tok_lane][0], b_mine = gb_lds[cur][tok_lane][1];
        const float v_mine = v_cur;

        // Tokens past the end of a ragged last block are staged as q = k = 0, g = 1, beta = 0: they
        // leave the state as it is, so the 16 steps run without a branch between them, and token
        // I + 1's q and k are read from LDS while token I is computed.
        float4 q_next[F4], k_next[F4];
        auto read_qk = [&](int i) {
            const float *qk = qk_lds[cur][i];
#pragma unroll
            for (int c = 0; c < F4; c++) {
                q_next[c] = *reinterpret_cast<const float4 *>(qk + c * (LANES * 4) + part * 4);
                k_next[c] = *reinterpret_cast<const float4 *>(qk + K_DIM + c * (LANES * 4) + part * 4);
            }
        };
        read_qk(0);
        float out_mine = 0.0f;  // lane `tok_lane` keeps the output of that token
        float out_part = 0.0f;  // this lane's share of the previous token's output: its sum over the
                                // row is not needed by the next token, so it runs beside that token's chain
        auto token = [&](auto index) {
            constexpr int I = decltype(index)::value;
            float4 q[F4], k[F4];
#pragma unroll
            for (int c = 0; c < F4; c++) q[c] = q_next[c], k[c] = k_next[c];
            if constexpr (I + 1 < ROWS_TB) read_qk(I + 1);
            __builtin_amdgcn_sched_barrier(0);  // the reads stay here, a token ahead of their use
            if constexpr (I > 0) {
                const float out = group_reduce<LANES>(out_part, SumOp());
                out_mine = tok_lane == I - 1 ? out : out_mine;
            }
            const float gt = row_lane<I>(g_mine), bt = row_lane<I>(b_mine), vt = row_lane<I>(v_mine);
#pragma unroll
            for (int c = 0; c < F4; c++) st[c].x *= gt, st[c].y *= gt, st[c].z *= gt, st[c].w *= gt;
            const float mem = group_reduce<LANES>(dot_tree<F4>(st, k), SumOp());
            const float delta = (vt - mem) * bt;
#pragma unroll
            for (int c = 0; c < F4; c++) {
                st[c].x += k[c].x * delta, st[c].y += k[c].y * delta, st[c].z += k[c].z * delta, st[c].w += k[c].w * delta;
            }
            out_part = dot_tree<F4>(st, q);
            if constexpr (SNAPS) {
                if (live && t0 + I < tokens) {
                    float *snap = a.snaps + size_t(t0 + I) * v_heads * v_dim * K_DIM +
                                  (size_t(h) * v_dim + row) * K_DIM + part * PER_LANE;
#pragma unroll
                    for (int c = 0; c < F4; c++) reinterpret_cast<float4 *>(snap)[c] = st[c];
                }
            }
        };
        TokenLoop<0>::run(token);
        {
            const float out = group_reduce<LANES>(out_part, SumOp());
            out_mine = tok_lane == ROWS_TB - 1 ? out : out_mine;
        }
        if (part < ROWS_TB) o_lds[part][row_in_wg] = out_mine;

        if (more) {
            store_block(cur ^ 1);
            v_cur = nv;
        }
        __syncthreads();  // the block's outputs are in o_lds; the next block is staged
        if (tid < ROWS_TB * ROWS_PER_WG) {
            // thread -> (token, row): the rows of a token are contiguous
            const uint32_t ti = tid / ROWS_PER_WG, ri = tid % ROWS_PER_WG;
            const uint32_t t = t0 + ti, r = blockIdx.x * ROWS_PER_WG + ri;
            if (t < tokens && r < v_dim) a.o[size_t(t) * value_size + size_t(h) * v_dim + r] = o_lds[ti][ri];
        }
        __syncthreads();  // o_lds is free again
        cur ^= 1;
    }
    if (live) {
#pragma unroll
        for (int c = 0; c < F4; c++) reinterpret_cast<float4 *>(sp)[c] = st[c];
    }
}

// The same for the chunks of a prefill, which are held to a tolerance and not to the single-token kernels'
// bits: LP = v_dim / 4 lanes per pair, four values each (16-byte loads and stores, two pairs per wavefront at
// the model's 128), the sum of squares over the LP lanes.
template <int LP>
__global__ __launch_bounds__(256) void deltanet_gated_norm_wide_kernel(float *y, const float *__restrict__ z,
                                                                       const float *__restrict__ norm_w, uint32_t pairs, float eps) {
    const uint32_t at = blockIdx.x * 256 + threadIdx.x, pair = at / LP, part = at % LP;
    if (pair >= pairs) return;  // (whole groups of LP lanes: 256 is a multiple of LP)
    float4 *yp = reinterpret_cast<float4 *>(y) + size_t(pair) * LP + part;
    const float4 o = *yp, g = reinterpret_cast<const float4 *>(z)[size_t(pair) * LP + part], w = reinterpret_cast<const float4 *>(norm_w)[part];
    const float total = group_reduce<LP>(o.x * o.x + o.y * o.y + o.z * o.z + o.w * o.w, SumOp());
    const float inv = 1.0f / sqrtf(total / float(4 * LP) + eps);
    *yp = make_float4(o.x * (inv * w.x) * silu_f(g.x), o.y * (inv * w.y) * silu_f(g.y), o.z * (inv * w.z) * silu_f(g.z), o.w * (inv * w.w) * silu_f(g.w));
}

// y = o / sqrt(mean(o^2) + eps) * norm_w * silu(z) per (token, value head), in place on y:
// one wavefront per pair, v_dim up to 256.
__global__ __launch_bounds__(256) void deltanet_gated_norm_rows_kernel(float *y, const float *__restrict__ z,
                                                                       const float *__restrict__ norm_w,
                                                                       uint32_t pairs, uint32_t v_dim, float eps) {
    const uint32_t pair = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (pair >= pairs) return;
    float *yp = y + size_t(pair) * v_dim;
    const float *zp = z + size_t(pair) * v_dim;
    float o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t d = lane + 64 * i;
        o[i] = d < v_dim ? yp[d] : 0.0f;
    }
    // the single-token kernel sums 64-lane partials in the same order: lanes first, then the groups of 64
    float total = 0.0f;
    {
        float part_sum[4];
#pragma unroll
        for (int i = 0; i < 4; i++) part_sum[i] = group_reduce<64>(o[i] * o[i], SumOp());
#pragma unroll
        for (int i = 0; i < 4; i++) total += part_sum[i];
    }
    const float inv = 1.0f / sqrtf(total / float(v_dim) + eps);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t d = lane + 64 * i;
        if (d < v_dim) yp[d] = o[i] * (inv * norm_w[d]) * silu_f(zp[d]);
    }
}


// ---- up to 8 tokens, conv and step together (the verify step) -----------------------------------
//
// Reference: kernel deltanet_rows (kernels/layers.metal, recorded by GpuDeltaNet::record_rows with
// DN_SIMDS = 0, src/gpu_layers.rs:737-757): conv, q/k norm, gates, delta rule, gated norm for m rows
// in one op, with the states after every row to the snapshot buffers; with one row, what
// GpuDeltaNet::record does (src/gpu_layers.rs:633-684).  The separate conv and step kernels above
// cost a launch each and the step runs on 32 workgroups.  Here a workgroup takes 16 rows of one value
// head's state (grid 8 x 32 at the model's shape), computes the conv outputs it needs itself for all
// the tokens (q and k of its key head, v of its rows: the conv state is only read) and walks the
// tokens; what needs the whole head or the whole layer is a small second launch: the gated norm over
// a head's outputs, the new conv state and the conv snapshots.
constexpr int SMALL_ROWS_MAX = 8;

struct SmallRowsArgs {
    const float *x, *w;
    float *conv_state;
    const float *a, *b, *a_log, *dt_bias;
    float *state;
    const float *z, *norm_w;
    float *y, *conv_snaps, *state_snaps;
    saetta_rows_fused_params p;
    uint32_t channels;
};

// out[t] of channel c for t < tokens.  The stored inputs and the new ones are one sequence in
// registers, the stored ones ending at index 14, x[t] at 15 + t; the taps are right-aligned the same
// way (the newest at 15), so that out[t] = sum_k taps[k] * seq[t + k] with constant indices: the
// unused leading taps are zeros, which leaves the sum (oldest first, the new input last, as the
// single-token kernel adds them) unchanged.  Every load is requested before the first is used.
template <typename F>
__device__ __forceinline__ void conv_small(const SmallRowsArgs &a, uint32_t c, F &&emit) {
    const uint32_t past = a.p.kernel_size - 1, tokens = a.p.rows;
    const float *wc = a.w + size_t(c) * a.p.kernel_size;
    float taps[16], seq[15 + SMALL_ROWS_MAX];
#pragma unroll
    for (uint32_t k = 0; k < 16; k++) taps[k] = k + past >= 15 ? wc[k + past - 15] : 0.0f;
#pragma unroll
    for (uint32_t k = 0; k < 15; k++) seq[k] = k + past >= 15 ? a.conv_state[size_t(k + past - 15) * a.channels + c] : 0.0f;
#pragma unroll
    for (uint32_t t = 0; t < SMALL_ROWS_MAX; t++) seq[15 + t] = t < tokens ? a.x[size_t(t) * a.channels + c] : 0.0f;
#pragma unroll
    for (uint32_t t = 0; t < SMALL_ROWS_MAX; t++) {
        if (t < tokens) {
            float acc = 0.0f;
#pragma unroll
            for (uint32_t k = 0; k < 15; k++) acc += taps[k] * seq[t + k];
            emit(t, silu_f(acc + taps[15] * seq[t + 15]));
        }
    }
}

// Waves 0-3 hold the 16 state rows (16 lanes a row) and compute the conv of the key head's q and k
// channels; wave 4 computes the conv of the 16 value channels and wave 5 the gates, so that no wave
// waits for memory twice before the first barrier.  Then the q/k norms of every token at once (one
// group of 16 lanes per token and vector), and the tokens in order with the next token's operands
// fetched from LDS while the current one's chain of sums runs.
constexpr int SMALL_THREADS = 384;

template <bool SNAPS>
__global__ __launch_bounds__(SMALL_THREADS) void deltanet_rows_small_kernel(SmallRowsArgs a) {
    __shared__ __attribute__((aligned(16))) float qk_lds[SMALL_ROWS_MAX][2 * K_DIM];  // per token: q then k, as [half][part][4]
    __shared__ float v_lds[SMALL_ROWS_MAX][16];
    __shared__ float gb_lds[SMALL_ROWS_MAX][2];   // decay, beta
    __shared__ float inv_lds[SMALL_ROWS_MAX][2];  // what q and k are multiplied by
    const uint32_t tid = threadIdx.x, part = tid & 15, row_in_wg = (tid >> 4) & 15;
    const uint32_t h = blockIdx.y, r0 = blockIdx.x * 16, row = r0 + row_in_wg;
    const uint32_t v_dim = a.p.v_dim, v_heads = a.p.v_heads, tokens = a.p.rows;
    const uint32_t kh = h / (v_heads / a.p.k_heads), key_size = a.p.k_heads * K_DIM;
    const bool live = tid < 256 && row < v_dim;
    float *sp = a.state + (size_t(h) * v_dim + (live ? row : 0)) * K_DIM + part * 8;
    float4 st[2];
    st[0] = live ? reinterpret_cast<const float4 *>(sp)[0] : make_float4(0, 0, 0, 0);
    st[1] = live ? reinterpret_cast<const float4 *>(sp)[1] : make_float4(0, 0, 0, 0);
    if (tid < 256) {
        const uint32_t e = tid & 127;
        const uint32_t slot = (tid < 128 ? 0 : K_DIM) + ((e & 7) >> 2) * 64 + (e >> 3) * 4 + (e & 3);
        conv_small(a, (tid < 128 ? 0 : key_size) + kh * K_DIM + e, [&](uint32_t t, float v) { qk_lds[t][slot] = v; });
    } else if (tid < 320) {
        const uint32_t i = tid - 256;
        if (i < 16 && r0 + i < v_dim) {
            conv_small(a, 2 * key_size + h * v_dim + r0 + i, [&](uint32_t t, float v) { v_lds[t][i] = v; });
        }
    } else {
        const uint32_t t = tid - 320;
        if (t < tokens) {
            fast_gates(a.a[size_t(t) * v_heads + h] + a.dt_bias[h], __expf(a.a_log[h]), a.b[size_t(t) * v_heads + h],
                       gb_lds[t][0], gb_lds[t][1]);
        }
    }
    __syncthreads();
    if (tid < 256) {
        // normalize_qk (src/cpu/deltanet.rs:133-146): group (tid / 16) takes token (group % 8), q or k
        const uint32_t t = row_in_wg & 7, which = row_in_wg >> 3;
        if (t < tokens) {
            const float4 lo = *reinterpret_cast<const float4 *>(qk_lds[t] + which * K_DIM + part * 4);
            const float4 hi = *reinterpret_cast<const float4 *>(qk_lds[t] + which * K_DIM + 64 + part * 4);
            const float sum = group_reduce<16>(dot4(lo, lo) + dot4(hi, hi), SumOp());
            const float scale = which == 0 ? 1.0f / sqrtf(float(K_DIM)) : 1.0f;
            if (part == 0) inv_lds[t][which] = scale * __builtin_amdgcn_rsqf(sum + a.p.eps);
        }
    }
    __syncthreads();
    if (tid >= 256) return;
    const size_t value_size = size_t(v_heads) * v_dim;
    float4 qn[2], kn[2];
    float gn, bn, vn, qin, kin;
    auto fetch = [&](uint32_t t) {
        qn[0] = *reinterpret_cast<const float4 *>(qk_lds[t] + part * 4);
        qn[1] = *reinterpret_cast<const float4 *>(qk_lds[t] + 64 + part * 4);
        kn[0] = *reinterpret_cast<const float4 *>(qk_lds[t] + K_DIM + part * 4);
        kn[1] = *reinterpret_cast<const float4 *>(qk_lds[t] + K_DIM + 64 + part * 4);
        gn = gb_lds[t][0], bn = gb_lds[t][1], vn = v_lds[t][row_in_wg];
        qin = inv_lds[t][0], kin = inv_lds[t][1];
    };
    fetch(0);
    for (uint32_t t = 0; t < tokens; t++) {
        float4 q[2], k[2];
        const float g = gn, beta = bn, v = vn, qi = qin, ki = kin;
#pragma unroll
        for (int c = 0; c < 2; c++) q[c] = qn[c], k[c] = kn[c];
        if (t + 1 < tokens) fetch(t + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 2; c++) {
            q[c].x *= qi, q[c].y *= qi, q[c].z *= qi, q[c].w *= qi;
            k[c].x *= ki, k[c].y *= ki, k[c].z *= ki, k[c].w *= ki;
            st[c].x *= g, st[c].y *= g, st[c].z *= g, st[c].w *= g;
        }
        const float mem = group_reduce<16>(dot4(st[0], k[0]) + dot4(st[1], k[1]), SumOp());
        const float delta = (v - mem) * beta;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            st[c].x += k[c].x * delta, st[c].y += k[c].y * delta, st[c].z += k[c].z * delta, st[c].w += k[c].w * delta;
        }
        const float o = group_reduce<16>(dot4(st[0], q[0]) + dot4(st[1], q[1]), SumOp());
        if (live) {
            if (part == 0) a.y[size_t(t) * value_size + size_t(h) * v_dim + row] = o;  // before the norm
            if constexpr (SNAPS) {
                float *snap = a.state_snaps + size_t(t) * v_heads * v_dim * K_DIM + (size_t(h) * v_dim + row) * K_DIM + part * 8;
                reinterpret_cast<float4 *>(snap)[0] = st[0];
                reinterpret_cast<float4 *>(snap)[1] = st[1];
            }
        }
    }
    if (live) reinterpret_cast<float4 *>(sp)[0] = st[0], reinterpret_cast<float4 *>(sp)[1] = st[1];
}

// After it.  Block b owns 16 channels of the conv: entry j of the conv state after token t is place
// t + 1 + j of (stored inputs, new inputs); the snapshots are written first, then, past a barrier
// (the entries are moved in place), the state after the last token.  The first blocks also norm the
// (token, head) pairs, one wave each, in place on y.
constexpr int TAIL_CHANNELS = 16;

__global__ __launch_bounds__(256) void deltanet_rows_small_tail_kernel(SmallRowsArgs a) {
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t v_dim = a.p.v_dim, tokens = a.p.rows, past = a.p.kernel_size - 1, channels = a.channels;
    const uint32_t pair = blockIdx.x * 4 + (tid >> 6), pairs = tokens * a.p.v_heads;
    const bool has_pair = pair < pairs;
    float o[4];
    if (has_pair) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t d = lane + 64 * i;
            o[i] = d < v_dim ? a.y[size_t(pair) * v_dim + d] : 0.0f;
        }
    }
    const uint32_t c = blockIdx.x * TAIL_CHANNELS + (tid & 15);
    const float *stored = a.conv_state, *fresh = a.x;
    auto place = [&](uint32_t at) {  // `at` in (stored inputs, new inputs)
        return at < past ? stored[size_t(at) * channels + c] : fresh[size_t(at - past) * channels + c];
    };
    if (c < channels) {
        if (a.p.snapshots) {
            float *__restrict__ snaps = a.conv_snaps;
#pragma unroll 2
            for (uint32_t e = tid >> 4; e < tokens * past; e += 16) {  // e = t * past + j
                snaps[size_t(e) * channels + c] = place(e / past + 1 + e % past);
            }
        }
    }
    const uint32_t j = tid >> 4;  // past <= 15 < 16 entries a block can move at once
    const bool moves = c < channels && j < past;
    const float moved = moves ? place(tokens + j) : 0.0f;
    __syncthreads();
    if (moves) a.conv_state[size_t(j) * channels + c] = moved;
    if (has_pair) {
        float *yp = a.y + size_t(pair) * v_dim;
        const float *zp = a.z + size_t(pair) * v_dim;
        float total = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) total += group_reduce<64>(o[i] * o[i], SumOp());
        const float inv = 1.0f / sqrtf(total / float(v_dim) + a.p.eps);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t d = lane + 64 * i;
            if (d < v_dim) yp[d] = o[i] * (inv * a.norm_w[d]) * silu_f(zp[d]);
        }
    }
}

void launch_small_rows(const SmallRowsArgs &args, hipStream_t stream) {
    const saetta_rows_fused_params &p = args.p;
    const dim3 grid((p.v_dim + 15) / 16, p.v_heads);
    if (p.snapshots) {
        deltanet_rows_small_kernel<true><<<grid, SMALL_THREADS, 0, stream>>>(args);
    } else {
        deltanet_rows_small_kernel<false><<<grid, SMALL_THREADS, 0, stream>>>(args);
    }
    const uint32_t pair_blocks = (p.rows * p.v_heads + 3) / 4, chan_blocks = (args.channels + TAIL_CHANNELS - 1) / TAIL_CHANNELS;
    deltanet_rows_small_tail_kernel<<<pair_blocks > chan_blocks ? pair_blocks : chan_blocks, 256, 0, stream>>>(args);
}

}  // namespace

int setup_deltanet() {
    if (int rc = load_kernel(reinterpret_cast<const void *>(deltanet_step_kernel))) return rc;
    return setup_deltanet_chunk();
}
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
    // q, k and v as the conv leaves them (one array, q | k | v: what the reference's layer passes,
    // src/cpu/deltanet.rs:80-83) take the kernels of saetta_deltanet_rows with one token: 8 workgroups
    // per value head instead of one.  deltanet_step_kernel is kept for vectors that lie apart.
    const size_t key_size = size_t(p.k_heads) * K_DIM;
    if (k == q + key_size && v == k + key_size && p.v_dim % 4 == 0) {
        const saetta_rows_step_params rp{p.k_heads, p.v_heads, p.v_dim, 1, p.eps, 0};
        return saetta_deltanet_rows(stream, q, a, b, a_log, dt_bias, state, z, norm_w, y, nullptr, rp);
    }
    StepArgs args{q, k, v, a, b, a_log, dt_bias, state, z, norm_w, y, p};
    deltanet_step_kernel<<<p.v_heads, STEP_THREADS, 0, as_stream(stream)>>>(args);
    return launch_status("deltanet_step");
}

extern "C" int saetta_deltanet_conv_rows(saetta_stream_t stream, const float *x, const float *w, float *state,
                                         float *out, float *snaps, saetta_conv_rows_params p) {
    SAETTA_REQUIRE(x && w && state && out, SAETTA_E_NULL, "deltanet_conv_rows: null buffer");
    SAETTA_REQUIRE(!p.snapshots || snaps, SAETTA_E_NULL, "deltanet_conv_rows: snapshots asked for, no buffer");
    SAETTA_REQUIRE(p.kernel_size >= 2 && p.kernel_size <= 16, SAETTA_E_SHAPE,
                   "deltanet_conv_rows: kernel size %u (2..16)", p.kernel_size);
    SAETTA_REQUIRE(p.tokens <= (1u << 20), SAETTA_E_SHAPE, "deltanet_conv_rows: %u tokens", p.tokens);
    if (int rc = ensure_device()) return rc;
    if (p.channels == 0 || p.tokens == 0) return SAETTA_OK;
    const dim3 grid((p.channels + 255) / 256, (p.tokens + CONV_TILE - 1) / CONV_TILE);
    // (four channels a thread pays from a tile of tokens up: a verify step's few rows want the workgroups)
    const bool by_four = p.tokens >= CONV_TILE && p.channels % 4 == 0 && aligned(x, 16) && aligned(w, 16) && aligned(state, 16) && aligned(out, 16) &&
                         (!p.snapshots || aligned(snaps, 16));
    if (p.kernel_size == 4 && by_four) {
        deltanet_conv_rows4_kernel<<<dim3((p.channels / 4 + 255) / 256, grid.y), 256, 0, as_stream(stream)>>>(x, w, state, out, snaps, p);
    } else if (p.kernel_size == 4) {
        deltanet_conv_rows_kernel<4><<<grid, 256, 0, as_stream(stream)>>>(x, w, state, out, snaps, p);
    } else if (p.kernel_size == 2) {
        deltanet_conv_rows_kernel<2><<<grid, 256, 0, as_stream(stream)>>>(x, w, state, out, snaps, p);
    } else {
        deltanet_conv_rows_kernel<0><<<grid, 256, 0, as_stream(stream)>>>(x, w, state, out, snaps, p);
    }
    deltanet_conv_state_kernel<<<grid.x, 256, 0, as_stream(stream)>>>(x, state, p);
    return launch_status("deltanet_conv_rows");
}

extern "C" size_t saetta_deltanet_rows_workspace_bytes(saetta_rows_step_params p) { return deltanet_chunk_workspace_bytes(p); }

extern "C" int saetta_deltanet_rows(saetta_stream_t stream, const float *mixed, const float *a, const float *b,
                                    const float *a_log, const float *dt_bias, float *state, const float *z,
                                    const float *norm_w, float *y, float *snaps, saetta_rows_step_params p) {
    return saetta_deltanet_rows_ws(stream, mixed, a, b, a_log, dt_bias, state, z, norm_w, y, snaps, p, nullptr, 0);
}

extern "C" int saetta_deltanet_rows_ws(saetta_stream_t stream, const float *mixed, const float *a, const float *b,
                                       const float *a_log, const float *dt_bias, float *state, const float *z,
                                       const float *norm_w, float *y, float *snaps, saetta_rows_step_params p,
                                       void *workspace, size_t workspace_size) {
    SAETTA_REQUIRE(mixed && a && b && a_log && dt_bias && state && z && norm_w && y, SAETTA_E_NULL,
                   "deltanet_rows: null buffer");
    SAETTA_REQUIRE(!p.snapshots || snaps, SAETTA_E_NULL, "deltanet_rows: snapshots asked for, no buffer");
    SAETTA_REQUIRE(p.k_heads > 0 && p.v_heads > 0 && p.v_heads % p.k_heads == 0, SAETTA_E_SHAPE,
                   "deltanet_rows: %u value heads over %u key heads", p.v_heads, p.k_heads);
    SAETTA_REQUIRE(p.v_dim >= 1 && p.v_dim <= 256 && p.v_dim % 4 == 0, SAETTA_E_SHAPE,
                   "deltanet_rows: value dim %u (a multiple of 4 up to 256); the key dim is 128", p.v_dim);
    SAETTA_REQUIRE(p.tokens <= (1u << 20), SAETTA_E_SHAPE, "deltanet_rows: %u tokens", p.tokens);
    SAETTA_REQUIRE(aligned(mixed, 16) && aligned(state, 16) && (!p.snapshots || aligned(snaps, 16)), SAETTA_E_ALIGN,
                   "deltanet_rows: mixed, the state and the snapshots must be 16-byte aligned");
    if (int rc = ensure_device()) return rc;
    if (p.tokens == 0) return SAETTA_OK;
    const uint32_t channels = 2 * p.k_heads * K_DIM + p.v_heads * p.v_dim;
    // A prefill chunk (128 tokens and more, no snapshots) whose caller brings a workspace: the delta rule in
    // blocks of 64 tokens on the matrix cores.  Without a workspace the call keeps to the token-by-token
    // kernels: the library holds no buffer of its own here, so calls on different streams share nothing.
    const size_t need = deltanet_chunk_workspace_bytes(p);
    const bool blocks = need > 0 && workspace != nullptr;
    if (blocks) {
        SAETTA_REQUIRE(workspace_size >= need && aligned(workspace, 16), SAETTA_E_SCRATCH,
                       "deltanet_rows: workspace of %zu bytes, %zu needed (16-byte aligned)", workspace_size, need);
        if (int rc = run_deltanet_chunk(as_stream(stream), mixed, a, b, a_log, dt_bias, state, y, p, channels, workspace)) return rc;
    } else {
        RowsArgs args{mixed, a, b, a_log, dt_bias, state, y, snaps, p, channels};
        constexpr int LANES = ROWS_LANES_PER_ROW, ROWS_PER_WG = 256 / LANES;
        const dim3 grid((p.v_dim + ROWS_PER_WG - 1) / ROWS_PER_WG, p.v_heads);
        if (p.snapshots) {
            deltanet_rows_kernel<true, LANES><<<grid, 256, 0, as_stream(stream)>>>(args);
        } else {
            deltanet_rows_kernel<false, LANES><<<grid, 256, 0, as_stream(stream)>>>(args);
        }
    }
    const uint32_t pairs = p.tokens * p.v_heads;
    const bool wide = blocks && aligned(y, 16) && aligned(z, 16) && aligned(norm_w, 16);
    if (wide && p.v_dim == 128) {
        deltanet_gated_norm_wide_kernel<32><<<(pairs * 32 + 255) / 256, 256, 0, as_stream(stream)>>>(y, z, norm_w, pairs, p.eps);
    } else if (wide && p.v_dim == 64) {
        deltanet_gated_norm_wide_kernel<16><<<(pairs * 16 + 255) / 256, 256, 0, as_stream(stream)>>>(y, z, norm_w, pairs, p.eps);
    } else if (wide && p.v_dim == 256) {
        deltanet_gated_norm_wide_kernel<64><<<(pairs * 64 + 255) / 256, 256, 0, as_stream(stream)>>>(y, z, norm_w, pairs, p.eps);
    } else {
        deltanet_gated_norm_rows_kernel<<<(pairs + 3) / 4, 256, 0, as_stream(stream)>>>(y, z, norm_w, pairs, p.v_dim, p.eps);
    }
    return launch_status("deltanet_rows");
}

extern "C" int saetta_deltanet_token(saetta_stream_t stream, const float *x, const float *w, float *conv_state,
                                     const float *a, const float *b, const float *a_log, const float *dt_bias,
                                     float *state, const float *z, const float *norm_w, float *y,
                                     saetta_conv_params cp, saetta_step_params sp) {
    SAETTA_REQUIRE(x && w && conv_state && a && b && a_log && dt_bias && state && z && norm_w && y, SAETTA_E_NULL,
                   "deltanet_token: null buffer");
    SAETTA_REQUIRE(cp.kernel_size >= 2 && cp.kernel_size <= 16, SAETTA_E_SHAPE, "deltanet_token: kernel size %u (2..16)",
                   cp.kernel_size);
    SAETTA_REQUIRE(sp.k_heads > 0 && sp.v_heads > 0 && sp.v_heads % sp.k_heads == 0, SAETTA_E_SHAPE,
                   "deltanet_token: %u value heads over %u key heads", sp.v_heads, sp.k_heads);
    SAETTA_REQUIRE(sp.v_dim >= 1 && sp.v_dim <= 256, SAETTA_E_SHAPE, "deltanet_token: value dim %u (1..256); the key dim is 128",
                   sp.v_dim);
    SAETTA_REQUIRE(cp.channels == 2 * sp.k_heads * K_DIM + sp.v_heads * sp.v_dim, SAETTA_E_SHAPE,
                   "deltanet_token: %u channels, the heads make %u", cp.channels, 2 * sp.k_heads * K_DIM + sp.v_heads * sp.v_dim);
    SAETTA_REQUIRE(aligned(state, 16), SAETTA_E_ALIGN, "deltanet_token: the state must be 16-byte aligned");
    if (int rc = ensure_device()) return rc;
    const saetta_rows_fused_params p{sp.k_heads, sp.v_heads, sp.v_dim, cp.kernel_size, sp.eps, 1, 0};
    SmallRowsArgs args{x, w, conv_state, a, b, a_log, dt_bias, state, z, norm_w, y, nullptr, nullptr, p, cp.channels};
    launch_small_rows(args, as_stream(stream));
    return launch_status("deltanet_token");
}

extern "C" int saetta_deltanet_rows_fused(saetta_stream_t stream, const float *x, const float *w, float *conv_state,
                                          const float *a, const float *b, const float *a_log, const float *dt_bias,
                                          float *state, const float *z, const float *norm_w, float *y,
                                          float *conv_snaps, float *state_snaps, saetta_rows_fused_params p) {
    SAETTA_REQUIRE(x && w && conv_state && a && b && a_log && dt_bias && state && z && norm_w && y, SAETTA_E_NULL,
                   "deltanet_rows_fused: null buffer");
    SAETTA_REQUIRE(!p.snapshots || (conv_snaps && state_snaps), SAETTA_E_NULL,
                   "deltanet_rows_fused: snapshots asked for, no buffers");
    SAETTA_REQUIRE(p.rows <= SMALL_ROWS_MAX, SAETTA_E_SHAPE, "deltanet_rows_fused: %u rows (up to 8)", p.rows);
    SAETTA_REQUIRE(p.kernel_size >= 2 && p.kernel_size <= 16, SAETTA_E_SHAPE,
                   "deltanet_rows_fused: kernel size %u (2..16)", p.kernel_size);
    SAETTA_REQUIRE(p.k_heads > 0 && p.v_heads > 0 && p.v_heads % p.k_heads == 0, SAETTA_E_SHAPE,
                   "deltanet_rows_fused: %u value heads over %u key heads", p.v_heads, p.k_heads);
    SAETTA_REQUIRE(p.v_dim >= 1 && p.v_dim <= 256, SAETTA_E_SHAPE,
                   "deltanet_rows_fused: value dim %u (1..256); the key dim is 128", p.v_dim);
    SAETTA_REQUIRE(aligned(state, 16) && (!p.snapshots || aligned(state_snaps, 16)), SAETTA_E_ALIGN,
                   "deltanet_rows_fused: the state and its snapshots must be 16-byte aligned");
    if (int rc = ensure_device()) return rc;
    if (p.rows == 0) return SAETTA_OK;
    const uint32_t channels = 2 * p.k_heads * K_DIM + p.v_heads * p.v_dim;
    SmallRowsArgs args{x, w, conv_state, a, b, a_log, dt_bias, state, z, norm_w, y, conv_snaps, state_snaps, p, channels};
    launch_small_rows(args, as_stream(stream));
    return launch_status("deltanet_rows_fused");
}
