// Attention before the scores, and the token's key and value into the cache, in one launch.
//
// Reference: GpuAttention::record_store (src/gpu_layers.rs:370-411) records attention_prep or
// attention_prep_float (kernels/layers.metal:637-702) and, for a quantized cache, two more
// dispatches of kv_quantize (src/kv_quant.rs:192-221).  Here the three are one kernel:
//   q head:  q = rope(rms_norm(q_and_gate[head][0..dim]) * q_norm)            -> q_out
//   k head:  k = rope(rms_norm(k[head]) * k_norm)  -> the key cache slot of the token
//   v head:  v                                       -> the value cache slot of the token
// and "the cache slot" is a half row, or the 8/4-bit codes, scales and biases of the row, made
// with the arithmetic of the quantizer kernel (kv_quant_device.hpp), so a key that goes through
// this kernel gets the codes that kv_quantize would have given the same f32 values.
// CPU definition: src/cpu/attention.rs:120-138 with rms_norm and rope of src/cpu/ops.rs:17-36,61-74:
// rms_norm: x * (1 / sqrt(mean(x^2) + eps)) * w; rope on the first 2 * half_dims values, value i
// paired with value i + half_dims (non-interleaved), angle = position * theta^(-i / half_dims).
// The angle and its sine and cosine are computed in f64, as on the CPU (the Metal kernel's f32
// angle loses bits at long positions).
//
// One workgroup of 256 threads (= head dim) per (head, row); row r of a verify step is the token
// at position + r.  The position comes from TokenParams in device memory when the kernel runs.
#include "common.hpp"
#include "kv_quant_device.hpp"
#include "lanes.hpp"

namespace saetta {
namespace {

constexpr int DIM = SAETTA_HEAD_DIM;

struct PrepArgs {
    const float *q_and_gate;  // [row][heads][2 * dim]
    const float *k, *v;       // [row][kv_heads][dim]
    const float *q_norm, *k_norm;
    float *q_out;             // [row][heads][dim]
    uint16_t *keys_half, *values_half;  // half cache [capacity][kv_heads][dim], or null
    saetta_quant_rows kq, vq;           // quantized cache (BITS 8 or 4)
    float *k_back;                      // [row][kv_heads][dim]: the normed, rotated key in f32, or null
    saetta_prep_params p;
    const saetta_token_params *tp;
    uint32_t capacity;
};

template <int BITS>
__global__ __launch_bounds__(256) void attention_prep_store_kernel(PrepArgs a) {
    __shared__ float head[DIM];
    __shared__ float partial[4];
    const uint32_t g = blockIdx.x, row = blockIdx.y, i = threadIdx.x;
    const uint32_t heads = a.p.heads, kvh = a.p.kv_heads, half = a.p.half_dims;
    const bool is_q = g < heads, is_k = !is_q && g < heads + kvh;
    const uint32_t j = is_q ? g : (is_k ? g - heads : g - heads - kvh);
    const uint32_t position = a.tp->position + row;

    float x = is_q   ? a.q_and_gate[(size_t(row) * heads + j) * 2 * DIM + i]
              : is_k ? a.k[(size_t(row) * kvh + j) * DIM + i]
                     : a.v[(size_t(row) * kvh + j) * DIM + i];
    if (is_q || is_k) {
        // x * (1 / sqrt(mean(x^2) + eps)) * w, the product taken as x * (scale * w) like the CPU does
        const float sq = group_reduce<64>(x * x, SumOp());
        if ((i & 63) == 0) partial[i >> 6] = sq;
        __syncthreads();
        const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
        const float scale = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(total, float(DIM)), a.p.eps)));
        x = __fmul_rn(x, __fmul_rn(scale, is_q ? a.q_norm[i] : a.k_norm[i]));
        head[i] = x;
        __syncthreads();
        if (i < 2 * half) {
            const uint32_t r = i < half ? i : i - half;
            const double freq = exp2(-double(r) / double(half) * double(a.p.log2_theta));
            const double angle = double(position) * freq;
            const float s = float(sin(angle)), c = float(cos(angle));
            const float u = head[r], w = head[r + half];
            x = i < half ? __fsub_rn(__fmul_rn(u, c), __fmul_rn(w, s)) : __fadd_rn(__fmul_rn(u, s), __fmul_rn(w, c));
        }
        if (is_q) {
            a.q_out[(size_t(row) * heads + j) * DIM + i] = x;
            return;
        }
        if (a.k_back) a.k_back[(size_t(row) * kvh + j) * DIM + i] = x;
    }
    if (position >= a.capacity) return;  // no slot: the caller's cache is full (every thread of the workgroup agrees)
    if constexpr (BITS == 16) {
        uint16_t *dst = (is_k ? a.keys_half : a.values_half) + (size_t(position) * kvh + j) * DIM;
        dst[i] = __half_as_ushort(__float2half_rn(x));
    } else {
        // The quantizer wants 32 / BITS neighbouring values per lane: through LDS.
        constexpr int VPL = 32 / BITS, LANES = SAETTA_QUANT_GROUP / VPL;
        __syncthreads();  // (the rotation above still reads head[])
        head[i] = x;
        __syncthreads();
        if (i < DIM / VPL) {  // whole wavefronts: 64 lanes at 8 bits, 32 at 4
            float v[VPL];
#pragma unroll
            for (int e = 0; e < VPL; e++) v[e] = head[i * VPL + e];
            __half s, z;
            const uint32_t word = quantize_lane<BITS>(v, s, z);
            const saetta_quant_rows rows = is_k ? a.kq : a.vq;
            const size_t group0 = (size_t(position) * kvh + j) * (DIM / SAETTA_QUANT_GROUP);  // of this head
            rows.data[group0 * LANES + i] = word;
            if (i % LANES == 0) {
                rows.scales[group0 + i / LANES] = __half_as_ushort(s);
                rows.biases[group0 + i / LANES] = __half_as_ushort(z);
            }
        }
    }
}

}  // namespace

int setup_prep() { return load_kernel(reinterpret_cast<const void *>(attention_prep_store_kernel<8>)); }
}  // namespace saetta

using namespace saetta;

extern "C" int saetta_attn_prep_store(saetta_stream_t stream, int bits, const float *q_and_gate, const float *k,
                                      const float *v, const float *q_norm, const float *k_norm, float *q_out,
                                      uint16_t *keys_half, uint16_t *values_half, saetta_quant_rows keys,
                                      saetta_quant_rows values, float *k_back, saetta_prep_params p, uint32_t rows,
                                      uint32_t capacity, const saetta_token_params *d_tp) {
    SAETTA_REQUIRE(bits == 16 || bits == 8 || bits == 4, SAETTA_E_BITS, "attn_prep_store: bits %d", bits);
    SAETTA_REQUIRE(p.dim == SAETTA_HEAD_DIM && p.kv_heads > 0 && p.heads > 0 && 2 * p.half_dims <= p.dim, SAETTA_E_SHAPE,
                   "attn_prep_store is written for head dim 256 (dim %u, rotary dims %u)", p.dim, 2 * p.half_dims);
    SAETTA_REQUIRE(rows >= 1 && rows <= SAETTA_MAX_ROWS, SAETTA_E_SHAPE, "attn_prep_store: %u rows (1..8)", rows);
    SAETTA_REQUIRE(q_and_gate && k && v && q_norm && k_norm && q_out && d_tp, SAETTA_E_NULL, "attn_prep_store: null buffer");
    if (bits == 16) {
        SAETTA_REQUIRE(keys_half && values_half, SAETTA_E_NULL, "attn_prep_store: null half cache");
    } else {
        SAETTA_REQUIRE(keys.data && keys.scales && keys.biases && values.data && values.scales && values.biases,
                       SAETTA_E_NULL, "attn_prep_store: null quantized cache");
    }
    if (int rc = ensure_device()) return rc;
    PrepArgs a{q_and_gate, k, v, q_norm, k_norm, q_out, keys_half, values_half, keys, values, k_back, p, d_tp, capacity};
    const dim3 grid(p.heads + 2 * p.kv_heads, rows);
    if (bits == 8) {
        attention_prep_store_kernel<8><<<grid, 256, 0, as_stream(stream)>>>(a);
    } else if (bits == 4) {
        attention_prep_store_kernel<4><<<grid, 256, 0, as_stream(stream)>>>(a);
    } else {
        attention_prep_store_kernel<16><<<grid, 256, 0, as_stream(stream)>>>(a);
    }
    return launch_status("attn_prep_store");
}
