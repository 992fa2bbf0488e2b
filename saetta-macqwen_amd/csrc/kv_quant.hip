// KV-cache quantizer for gfx950: 8- and 4-bit group-affine codes, groups of 64
// values with an f16 scale and bias, x ~ s * q + z.
//
// Semantics follow the reference's CPU quantize()/dequantize()
// (src/kv_quant.rs:54-105) bit for bit; the Metal kernels they stand in for
// are kv_quantize_{8,4} and kv_dequantize_{8,4} (kernels/kv_quant.metal:15-82).
//
// Layout in HBM (src/kv_quant.rs:156-180): token p's groups start at group
// p * per_token; the codes of group G are u32 words 2*bits*G .. , lowest bits
// first; scales[G], biases[G] are halves.
//
// Mapping: a lane owns the 32/bits values that make one u32 of codes (4 at
// 8 bits, 8 at 4 bits), so a group is 16 or 8 neighbouring lanes of a
// wavefront and its min/max are two short butterfly reductions.  Loads are
// float4 per lane, contiguous across the wavefront; every lane stores one
// dword of codes, contiguous as well.
#include "common.hpp"
#include "kv_quant_device.hpp"

namespace saetta {
namespace {

// The arithmetic of a group is quantize_lane (kv_quant_device.hpp).
template <int BITS>
__global__ __launch_bounds__(256) void kv_quantize_kernel(const float *__restrict__ x,
                                                          uint32_t *__restrict__ data,
                                                          uint16_t *__restrict__ scales,
                                                          uint16_t *__restrict__ biases,
                                                          saetta_kv_quant_params p,
                                                          const saetta_token_params *__restrict__ d_tp,
                                                          uint32_t pos_arg) {
    constexpr int VPL = 32 / BITS;               // values per lane = codes per word
    constexpr int LANES = SAETTA_QUANT_GROUP / VPL;  // lanes per group
    const uint32_t word = blockIdx.x * 256u + threadIdx.x;  // word index from x[0]
    const uint32_t g = word / LANES;
    const bool live = g < p.groups;
    // Lanes past the end still take part in the shuffles of their (dead) group.
    float v[VPL];
    if (live) {
        const float4 *src = reinterpret_cast<const float4 *>(x) + size_t(word) * (VPL / 4);
#pragma unroll
        for (int i = 0; i < VPL / 4; i++) {
            float4 f = src[i];
            v[4 * i] = f.x;
            v[4 * i + 1] = f.y;
            v[4 * i + 2] = f.z;
            v[4 * i + 3] = f.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < VPL; i++) v[i] = 0.0f;
    }
    __half s, z;
    const uint32_t packed = quantize_lane<BITS>(v, s, z);
    if (!live) return;
    const uint32_t pos = d_tp ? d_tp->position : pos_arg;
    const size_t first = size_t(pos) * p.per_token;  // destination group of g = 0
    data[first * LANES + word] = packed;
    if (word % LANES == 0) {
        scales[first + g] = __half_as_ushort(s);
        biases[first + g] = __half_as_ushort(z);
    }
}

// One lane per word of codes: 32/bits halves out, out[i] = half(f32(s)*q + f32(z)).
// s*q is exact in f32 (11 x 8 significant bits), so one rounding happens in
// the add and one in the conversion, as in the CPU version followed by
// f16::from_f32 (tests/kv_quant.rs:113-124).
template <int BITS>
__global__ __launch_bounds__(256) void kv_dequantize_kernel(const uint32_t *__restrict__ data,
                                                            const uint16_t *__restrict__ scales,
                                                            const uint16_t *__restrict__ biases,
                                                            uint16_t *__restrict__ out,
                                                            saetta_kv_quant_params p) {
    constexpr int VPL = 32 / BITS;
    constexpr int LANES = SAETTA_QUANT_GROUP / VPL;
    const uint32_t word = blockIdx.x * 256u + threadIdx.x;
    const uint32_t g = word / LANES;
    if (g >= p.groups) return;
    const uint32_t w = data[word];
    const float s = __half2float(__ushort_as_half(scales[g]));
    const float z = __half2float(__ushort_as_half(biases[g]));
    uint32_t o[VPL / 2];
#pragma unroll
    for (int i = 0; i < VPL; i += 2) {
        float a = __fadd_rn(__fmul_rn(s, float((w >> (i * BITS)) & ((1u << BITS) - 1))), z);
        float b = __fadd_rn(__fmul_rn(s, float((w >> ((i + 1) * BITS)) & ((1u << BITS) - 1))), z);
        o[i / 2] = uint32_t(__half_as_ushort(__float2half_rn(a))) |
                   (uint32_t(__half_as_ushort(__float2half_rn(b))) << 16);
    }
    uint32_t *dst = reinterpret_cast<uint32_t *>(out) + size_t(word) * (VPL / 2);
    if constexpr (VPL == 4) {
        *reinterpret_cast<uint2 *>(dst) = make_uint2(o[0], o[1]);
    } else {
        *reinterpret_cast<uint4 *>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// s * q + z in f32 (one rounding in the multiply, which is exact, and one in the add): what
// dequantize() returns on the CPU (src/kv_quant.rs:90-105), i.e. round_trip of the input.
template <int BITS>
__global__ __launch_bounds__(256) void kv_dequantize_f32_kernel(const uint32_t *__restrict__ data,
                                                                const uint16_t *__restrict__ scales,
                                                                const uint16_t *__restrict__ biases,
                                                                float *__restrict__ out, saetta_kv_quant_params p) {
    constexpr int VPL = 32 / BITS;
    constexpr int LANES = SAETTA_QUANT_GROUP / VPL;
    const uint32_t word = blockIdx.x * 256u + threadIdx.x;
    const uint32_t g = word / LANES;
    if (g >= p.groups) return;
    const uint32_t w = data[word];
    const float s = __half2float(__ushort_as_half(scales[g]));
    const float z = __half2float(__ushort_as_half(biases[g]));
    float4 *dst = reinterpret_cast<float4 *>(out) + size_t(word) * (VPL / 4);
#pragma unroll
    for (int i = 0; i < VPL; i += 4) {
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            o[e] = __fadd_rn(__fmul_rn(s, float((w >> ((i + e) * BITS)) & ((1u << BITS) - 1))), z);
        }
        dst[i / 4] = make_float4(o[0], o[1], o[2], o[3]);
    }
}

// f32 -> f16, four values per lane.
__global__ __launch_bounds__(256) void to_half_kernel(const float *__restrict__ x,
                                                      uint16_t *__restrict__ out, size_t n) {
    size_t i = (size_t(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i + 4 <= n) {
        float4 f = *reinterpret_cast<const float4 *>(x + i);
        uint32_t a = uint32_t(__half_as_ushort(__float2half_rn(f.x))) |
                     (uint32_t(__half_as_ushort(__float2half_rn(f.y))) << 16);
        uint32_t b = uint32_t(__half_as_ushort(__float2half_rn(f.z))) |
                     (uint32_t(__half_as_ushort(__float2half_rn(f.w))) << 16);
        *reinterpret_cast<uint2 *>(out + i) = make_uint2(a, b);
    } else {
        for (; i < n; i++) out[i] = __half_as_ushort(__float2half_rn(x[i]));
    }
}

}  // namespace

int setup_kv_quant() { return load_kernel(reinterpret_cast<const void *>(kv_quantize_kernel<8>)); }
}  // namespace saetta

using namespace saetta;

extern "C" int saetta_kv_quantize(saetta_stream_t stream, int bits, const float *x,
                                  saetta_quant_rows rows, saetta_kv_quant_params p,
                                  const saetta_token_params *d_tp, uint32_t pos) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "kv_quantize: bits %d (8 or 4)", bits);
    SAETTA_REQUIRE(x && rows.data && rows.scales && rows.biases, SAETTA_E_NULL,
                   "kv_quantize: null buffer");
    SAETTA_REQUIRE(aligned(x, 16), SAETTA_E_ALIGN, "kv_quantize: x must be 16-byte aligned");
    SAETTA_REQUIRE(p.per_token > 0, SAETTA_E_SHAPE, "kv_quantize: per_token 0");
    if (int rc = ensure_device()) return rc;
    if (p.groups == 0) return SAETTA_OK;
    const uint32_t lanes = bits == 8 ? 16 : 8;
    const uint32_t blocks = (p.groups * lanes + 255) / 256;
    if (bits == 8) {
        kv_quantize_kernel<8><<<blocks, 256, 0, as_stream(stream)>>>(x, rows.data, rows.scales,
                                                                     rows.biases, p, d_tp, pos);
    } else {
        kv_quantize_kernel<4><<<blocks, 256, 0, as_stream(stream)>>>(x, rows.data, rows.scales,
                                                                     rows.biases, p, d_tp, pos);
    }
    return launch_status("kv_quantize");
}

extern "C" int saetta_kv_dequantize(saetta_stream_t stream, int bits, saetta_quant_rows rows,
                                    uint16_t *out_f16, saetta_kv_quant_params p) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "kv_dequantize: bits %d (8 or 4)", bits);
    SAETTA_REQUIRE(out_f16 && rows.data && rows.scales && rows.biases, SAETTA_E_NULL,
                   "kv_dequantize: null buffer");
    SAETTA_REQUIRE(aligned(out_f16, 16), SAETTA_E_ALIGN, "kv_dequantize: out must be 16-byte aligned");
    if (int rc = ensure_device()) return rc;
    if (p.groups == 0) return SAETTA_OK;
    const uint32_t lanes = bits == 8 ? 16 : 8;
    const uint32_t blocks = (p.groups * lanes + 255) / 256;
    if (bits == 8) {
        kv_dequantize_kernel<8><<<blocks, 256, 0, as_stream(stream)>>>(rows.data, rows.scales,
                                                                       rows.biases, out_f16, p);
    } else {
        kv_dequantize_kernel<4><<<blocks, 256, 0, as_stream(stream)>>>(rows.data, rows.scales,
                                                                       rows.biases, out_f16, p);
    }
    return launch_status("kv_dequantize");
}

extern "C" int saetta_kv_dequantize_f32(saetta_stream_t stream, int bits, saetta_quant_rows rows, float *out,
                                        saetta_kv_quant_params p) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "kv_dequantize_f32: bits %d (8 or 4)", bits);
    SAETTA_REQUIRE(out && rows.data && rows.scales && rows.biases, SAETTA_E_NULL, "kv_dequantize_f32: null buffer");
    SAETTA_REQUIRE(aligned(out, 16), SAETTA_E_ALIGN, "kv_dequantize_f32: out must be 16-byte aligned");
    if (int rc = ensure_device()) return rc;
    if (p.groups == 0) return SAETTA_OK;
    const uint32_t lanes = bits == 8 ? 16 : 8;
    const uint32_t blocks = (p.groups * lanes + 255) / 256;
    if (bits == 8) {
        kv_dequantize_f32_kernel<8><<<blocks, 256, 0, as_stream(stream)>>>(rows.data, rows.scales, rows.biases, out, p);
    } else {
        kv_dequantize_f32_kernel<4><<<blocks, 256, 0, as_stream(stream)>>>(rows.data, rows.scales, rows.biases, out, p);
    }
    return launch_status("kv_dequantize_f32");
}

extern "C" int saetta_to_half(saetta_stream_t stream, const float *x, uint16_t *out_f16, size_t n) {
    SAETTA_REQUIRE(x && out_f16, SAETTA_E_NULL, "to_half: null buffer");
    SAETTA_REQUIRE(aligned(x, 16) && aligned(out_f16, 8), SAETTA_E_ALIGN,
                   "to_half: x must be 16-byte and out 8-byte aligned");
    if (int rc = ensure_device()) return rc;
    if (n == 0) return SAETTA_OK;
    const size_t blocks = (n + 1023) / 1024;
    to_half_kernel<<<dim3(uint32_t(blocks)), 256, 0, as_stream(stream)>>>(x, out_f16, n);
    return launch_status("to_half");
}
