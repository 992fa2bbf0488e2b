// Split-K decode / verify attention over the KV cache for gfx950 (MI355X).
//
// What it computes (reference: DecodeAttention::record{,_quant}
// src/attention.rs:73-135, AttentionRows::record{,_quant} src/rows.rs:369-493;
// CPU definition src/cpu/attention.rs:141-181): for each of m query rows and
// each of the 16 q heads,
//     out = softmax(q K^T * scale) V * sigmoid(gate)
// over the first len_r cached tokens, 8 q heads sharing one kv head, head dim
// 256.  The cache is f16 or 8/4-bit group-affine codes (groups of 64 dims,
// f16 scale and bias, x = s*q + z; layout in kv_quant.hip).
//
// Shape of the work: 2 kv heads only, so all parallelism comes from splitting
// the context.  Workgroup (split, kv head) walks the 128-token chunks split,
// split + nsplits, ... and keeps an online softmax per query row; it writes
// one unnormalised partial (o, m, l) per (row, q head) and a second kernel
// merges the partials and applies the gate.
//
// Inside a chunk the two contractions run on the matrix cores
// (v_mfma_f32_16x16x32_f16), because at 15-28 FLOP per cache byte a vector-ALU
// dot product cannot keep up with HBM:
//   phase A  S^T = K Q^T   wave w takes tokens 32w..32w+31 (two 16-token
//            blocks); A operand = key codes of 16 tokens, B operand = the
//            query rows.
//   phase B  online softmax per row over the chunk's 128 scores (in LDS).
//   phase C  O += P V      wave w takes dims 64w..64w+63, which is exactly
//            one quantization group, for all 128 tokens.
// Codes are never dequantized element by element.  A code byte c is placed in
// the low mantissa bits of an f16 with a zero exponent, i.e. the subnormal
// c * 2^-24, with one v_perm_b32 per two codes; the matrix cores take
// subnormal inputs at full precision.  Scale and bias of a group are applied
// to the 64-dim partial dot product (keys) or folded into the probability
// operand (values):
//   q.k   = sum_g  s_g * (q_g . c_g) + z_g * sum(q_g)
//   P V_g = (P * s_g) C_g + (P . z_g)
// The value operand needs (token, token+1) pairs per dim while memory holds
// (dim, dim+1) pairs per token; the same v_perm_b32 that widens the bytes
// picks them from two tokens' words, so the transposition costs nothing.
// q and P are split into f16 hi + lo parts (two MFMAs into one accumulator,
// or for a single row the hi and lo parts share one 16-row tile), which keeps
// the result within ~1e-6 of an f32 evaluation.
#include "common.hpp"

namespace saetta {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int DIM = SAETTA_HEAD_DIM;
constexpr int CHUNK = SAETTA_CHUNK;
constexpr int THREADS = 256;
constexpr int SC_STRIDE = CHUNK + 4;  // floats; keeps rows on different LDS banks
constexpr float NO_SCORE = -1e30f;    // finite "minus infinity" of the running max

// q is multiplied by scale * log2(e) * Q_UP before the hi/lo split so that
// the lo part stays a normal f16; probabilities by P_UP for the same reason.
constexpr float Q_UP = 16.0f;
constexpr float P_UP = 256.0f;
// A code byte b is fed to the matrix cores as the f16 subnormal b * 2^-24.
// 4-bit codes sit in the HIGH nibble of that byte (16c * 2^-24): the adders
// align products by exponent field, so leading zero bits of a subnormal
// mantissa are lost precision, and the high nibble loses four fewer.
template <int BITS>
constexpr float code_up() {
    return BITS == 8 ? 16777216.0f : BITS == 4 ? 1048576.0f : 1.0f;
}

struct PartialArgs {
    const float *q;
    const void *kdata;
    const void *vdata;
    const uint16_t *kscales, *kbiases, *vscales, *vbiases;
    float *part_o;
    float *part_ml;
    uint32_t heads, kv_heads, capacity;
    float scale;
    uint32_t rows, nsplits;
    const saetta_token_params *tp;
    uint32_t decode_len;  // 1: every row sees min(kv_len, capacity); 0: row r sees position + r + 1
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

__device__ __forceinline__ half8 as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = {a, b, c, d};
    return __builtin_bit_cast(half8, v);
}

// ---- key codes: 16 dims of one token per lane and group ----------------------
template <int BITS>
struct KeyRegs;
template <>
struct KeyRegs<8> {
    uint4 w;
};
template <>
struct KeyRegs<4> {
    uint2 w;
};
template <>
struct KeyRegs<16> {
    uint4 w[2];
};

// Lane (t, j): dims 64g + 16j .. +15 of `token`, kv head kv.
template <int BITS>
__device__ __forceinline__ KeyRegs<BITS> load_key(const void *data, uint32_t token, uint32_t kv_heads,
                                                  uint32_t kv, int g, int j) {
    KeyRegs<BITS> r;
    if constexpr (BITS == 8) {
        const uint4 *p = reinterpret_cast<const uint4 *>(data);
        r.w = p[(size_t(token) * kv_heads + kv) * 16 + g * 4 + j];
    } else if constexpr (BITS == 4) {
        const uint2 *p = reinterpret_cast<const uint2 *>(data);
        r.w = p[(size_t(token) * kv_heads + kv) * 16 + g * 4 + j];
    } else {
        const uint4 *p = reinterpret_cast<const uint4 *>(data);
        size_t i = (size_t(token) * kv_heads + kv) * 32 + g * 8 + j * 2;
        r.w[0] = p[i];
        r.w[1] = p[i + 1];
    }
    return r;
}

// The A operand of k-step `ab` (0: the lane's first 8 dims, 1: the next 8).
template <int BITS>
__device__ __forceinline__ half8 key_operand(const KeyRegs<BITS> &r, int ab) {
    if constexpr (BITS == 8) {
        uint32_t w0 = ab ? r.w.z : r.w.x, w1 = ab ? r.w.w : r.w.y;
        return as_half8(perm(0, w0, 0x0c010c00u), perm(0, w0, 0x0c030c02u), perm(0, w1, 0x0c010c00u),
                        perm(0, w1, 0x0c030c02u));
    } else if constexpr (BITS == 4) {
        uint32_t w = ab ? r.w.y : r.w.x;
        uint32_t x = (w << 4) & 0xf0f0f0f0u, y = w & 0xf0f0f0f0u;
        // slots: dims 0,2 | 4,6 | 1,3 | 5,7
        return as_half8(perm(0, x, 0x0c010c00u), perm(0, x, 0x0c030c02u), perm(0, y, 0x0c010c00u),
                        perm(0, y, 0x0c030c02u));
    } else {
        const uint4 &v = r.w[ab];
        return as_half8(v.x, v.y, v.z, v.w);
    }
}

template <int BITS>
__device__ __forceinline__ constexpr int key_slot_dim(int e) {
    if (BITS == 4) {
        constexpr int order[8] = {0, 2, 4, 6, 1, 3, 5, 7};
        return order[e];
    }
    return e;
}

// ---- value codes: one dword per token, 8 tokens per lane and k-step -----------
// 8-bit: the dword holds dims 4n..4n+3 of the wave's group; 4-bit: lanes 2i and
// 2i+1 load the same dword (8 dims) and use its low / high 16 bits; f16: two
// dwords, dims 2n, 2n+1 and 32+2n, 32+2n+1 of the wave's 64.
template <int BITS>
struct ValRegs {
    uint32_t w[BITS == 16 ? 16 : 8];
};

template <int BITS>
__device__ __forceinline__ uint32_t load_val_word(const void *data, uint32_t token, uint32_t kv_heads,
                                                  uint32_t kv, int wave, int n, int set) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(data);
    if constexpr (BITS == 8) {
        return p[((size_t(token) * kv_heads + kv) * 4 + wave) * 16 + n];
    } else if constexpr (BITS == 4) {
        return p[((size_t(token) * kv_heads + kv) * 4 + wave) * 8 + (n >> 1)];
    } else {
        return p[(size_t(token) * kv_heads + kv) * 128 + wave * 32 + set * 16 + n];
    }
}

// B operand of output tile `tile` (0..3) from the 8 tokens' words of a k-step.
// Tile e covers dims 4n + e (8/4-bit) or 32*(e/2) + 2n + e%2 (f16) of the wave's 64.
template <int BITS>
__device__ __forceinline__ half8 val_operand(const ValRegs<BITS> &r, int tile, int n) {
    uint32_t o[4];
    if constexpr (BITS == 8) {
        const uint32_t sel = 0x0c000c00u | (uint32_t(4 + tile) << 16) | uint32_t(tile);
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = perm(r.w[2 * i + 1], r.w[2 * i], sel);
    } else if constexpr (BITS == 4) {
        const uint32_t byte = uint32_t(tile >> 1);
        const uint32_t sel = 0x0c000c00u | ((4 + byte) << 16) | byte;
        const uint32_t sh = (n & 1) * 16, up = (tile & 1) ? 0 : 4;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t a = ((r.w[2 * i] >> sh) << up) & 0xf0f0u, b = ((r.w[2 * i + 1] >> sh) << up) & 0xf0f0u;
            o[i] = perm(b, a, sel);
        }
    } else {
        const int set = tile >> 1;
        const uint32_t sel = (tile & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = perm(r.w[set * 8 + 2 * i + 1], r.w[set * 8 + 2 * i], sel);
    }
    return as_half8(o[0], o[1], o[2], o[3]);
}

// f32 -> f16 hi part and f16 lo part with hi + lo = x to ~2^-22.  hi is x with
// the low 13 mantissa bits cleared, which an f16 holds exactly whatever way
// the conversion rounds; a conversion-based split breaks at ties when the
// compiler fuses one of the two conversions with the multiply that made x.
__device__ __forceinline__ void split_hi_lo(float x, _Float16 &hi, _Float16 &lo) {
    const float h = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x) & 0xffffe000u);
    hi = (_Float16)h;
    lo = (_Float16)(x - h);
}

// TILES: 16-row tiles of query rows (rows * 8 heads, rounded up).  PACKED: one
// verify row; its 8 heads' hi parts are operand rows 0-7 and lo parts rows 8-15
// of a single tile.  Otherwise hi and lo are two MFMAs into one accumulator.
template <int BITS, int TILES, bool PACKED>
struct Shape {
    static constexpr int S_ROWS = 16 * TILES;               // rows of the score buffer
    static constexpr int SOFT_ROWS = PACKED ? 8 : 16 * TILES;  // rows phase B walks
    static constexpr int TPR = THREADS / SOFT_ROWS;          // threads per row in phase B
    static constexpr int TPT = CHUNK / TPR;                  // tokens per thread in phase B
    static constexpr int PARTS = PACKED ? 1 : 2;
    static constexpr int Q_BYTES = TILES * PARTS * 8 * 64 * 16;
    static constexpr int S_BYTES = S_ROWS * SC_STRIDE * 4;
    static constexpr int SCALE_BYTES = (BITS == 16) ? 0 : 4 * 4 * CHUNK * 4;
    static constexpr int MISC_BYTES = (S_ROWS /*alpha*/ + TILES * 4 * 16 /*qsum*/ + 4 * S_ROWS /*zsum*/) * 4;
    static constexpr int LDS_BYTES = Q_BYTES + S_BYTES + SCALE_BYTES + MISC_BYTES;
};

template <int BITS, int TILES, bool PACKED>
__global__ __launch_bounds__(THREADS) void attention_partial_kernel(PartialArgs a) {
    using Sh = Shape<BITS, TILES, PACKED>;
    constexpr bool QUANT = BITS != 16;
    constexpr int PARTS = Sh::PARTS;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    half8 *q_lds = reinterpret_cast<half8 *>(lds_raw);                       // [tile][part][step][lane]
    float *s_lds = reinterpret_cast<float *>(lds_raw + Sh::Q_BYTES);         // [S_ROWS][SC_STRIDE]
    float *sc_lds = reinterpret_cast<float *>(lds_raw + Sh::Q_BYTES + Sh::S_BYTES);
    float *ks_lds = sc_lds, *kz_lds = sc_lds + 4 * CHUNK, *vs_lds = sc_lds + 8 * CHUNK,
          *vz_lds = sc_lds + 12 * CHUNK;                                      // [g][token]
    float *misc = reinterpret_cast<float *>(lds_raw + Sh::Q_BYTES + Sh::S_BYTES + Sh::SCALE_BYTES);
    float *alpha_lds = misc;                   // [S_ROWS]
    float *qsum_lds = misc + Sh::S_ROWS;        // [tile][g][16]
    float *zsum_lds = qsum_lds + TILES * 64;    // [wave][S_ROWS]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, j = lane >> 4;
    const uint32_t split = blockIdx.x, kv = blockIdx.y;
    const uint32_t kvh = a.kv_heads;

    const uint32_t position = a.tp->position;
    // Tokens the last row sees; the longest context of the launch.
    const uint32_t max_len =
        min(a.decode_len ? a.tp->kv_len : position + a.rows, a.capacity);
    if (split * CHUNK >= max_len) return;
    const uint32_t real_rows = a.rows * 8;  // (row, head) pairs of this kv head

    // ---- prologue: query operands ------------------------------------------------
    // Operand row `orow` of tile t: PACKED -> head orow & 7, part orow >> 3;
    // else (row, head) pair 16t + orow, both parts.
    {
        const float qmul = a.scale * 1.4426950408889634f * Q_UP;
        for (int item = tid; item < TILES * 8 * 64; item += THREADS) {
            const int t = item / 512, step = (item / 64) & 7, l = item & 63;
            const int on = l & 15, oj = l >> 4;
            const int g = step >> 1, ab = step & 1;
            const int pair = PACKED ? (on & 7) : 16 * t + on;
            float v[8];
            if (pair < int(real_rows)) {
                const int row = pair >> 3, head = pair & 7;
                const float *src = a.q + (size_t(row) * a.heads + kv * 8 + head) * DIM + 64 * g +
                                   16 * oj + 8 * ab;
                const float4 f0 = *reinterpret_cast<const float4 *>(src);
                const float4 f1 = *reinterpret_cast<const float4 *>(src + 4);
                v[0] = f0.x, v[1] = f0.y, v[2] = f0.z, v[3] = f0.w;
                v[4] = f1.x, v[5] = f1.y, v[6] = f1.z, v[7] = f1.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = 0.0f;
            }
            half8 hi, lo;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                _Float16 h, lw;
                split_hi_lo(v[key_slot_dim<BITS>(e)] * qmul, h, lw);
                hi[e] = h;
                lo[e] = lw;
            }
            if constexpr (PACKED) {
                q_lds[step * 64 + l] = (on < 8) ? hi : lo;
            } else {
                q_lds[((t * 2 + 0) * 8 + step) * 64 + l] = hi;
                q_lds[((t * 2 + 1) * 8 + step) * 64 + l] = lo;
            }
        }
    }
    __syncthreads();
    // Sum of each operand row's values per 64-dim group, for the key bias term.
    if constexpr (QUANT) {
        for (int item = tid; item < TILES * 4 * 16; item += THREADS) {
            const int t = item / 64, g = (item / 16) & 3, on = item & 15;
            float sum = 0.0f;
            for (int part = 0; part < PARTS; part++) {
                for (int ab = 0; ab < 2; ab++) {
                    for (int oj = 0; oj < 4; oj++) {
                        half8 h = q_lds[((t * PARTS + part) * 8 + g * 2 + ab) * 64 + oj * 16 + on];
#pragma unroll
                        for (int e = 0; e < 8; e++) sum += (float)h[e];
                    }
                }
            }
            qsum_lds[item] = sum;
        }
    }
    __syncthreads();

    // Query operands of a single tile live in registers for the whole kernel.
    half8 q_reg[TILES == 1 ? PARTS * 8 : 1];
    float qsum_reg[TILES == 1 ? 4 : 1];
    if constexpr (TILES == 1) {
#pragma unroll
        for (int i = 0; i < PARTS * 8; i++) q_reg[i] = q_lds[i * 64 + lane];
        if constexpr (QUANT) {
#pragma unroll
            for (int g = 0; g < 4; g++) qsum_reg[g] = qsum_lds[g * 16 + n];
        }
    }

    // ---- running state -------------------------------------------------------------
    // Phase B: thread (row, part) of SOFT_ROWS x TPR.
    const int b_row = tid / Sh::TPR, b_part = tid % Sh::TPR;
    uint32_t b_len;  // tokens row b_row sees
    {
        const int vrow = PACKED ? 0 : b_row >> 3;
        const bool real = PACKED || b_row < int(real_rows);
        const uint32_t len = a.decode_len ? a.tp->kv_len : position + vrow + 1;
        b_len = real ? min(len, a.capacity) : 0;
    }
    float m_run = NO_SCORE, l_part = 0.0f;
    // Phase C: accumulators of this wave's 64 dims, per tile 4 output tiles of 16 dims.
    floatx4 acc[TILES][4];
    float zacc[TILES];
#pragma unroll
    for (int t = 0; t < TILES; t++) {
        zacc[t] = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; e++) acc[t][e] = floatx4{0, 0, 0, 0};
    }

    for (uint32_t chunk = split; chunk * CHUNK < max_len; chunk += a.nsplits) {
        const uint32_t base = chunk * CHUNK;
        const uint32_t last = a.capacity - 1;  // clamp for addresses past the cache

        // ---- loads of the whole chunk, issued up front ---------------------------
        KeyRegs<BITS> kreg[2][4];
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const uint32_t token = min(base + 32 * wave + 16 * b + n, last);
#pragma unroll
            for (int g = 0; g < 4; g++) kreg[b][g] = load_key<BITS>(a.kdata, token, kvh, kv, g, j);
        }
        ValRegs<BITS> vreg[4];
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t tok = base + 32 * ks + 8 * j + e;
                const uint32_t token = min(tok, last);
                vreg[ks].w[e] = load_val_word<BITS>(a.vdata, token, kvh, kv, wave, n, 0);
                if constexpr (BITS == 16) {
                    vreg[ks].w[8 + e] = load_val_word<BITS>(a.vdata, token, kvh, kv, wave, n, 1);
                    // Rows past the context may hold anything, NaN included: 0 * NaN must not reach O.
                    if (tok >= max_len) vreg[ks].w[e] = 0, vreg[ks].w[8 + e] = 0;
                }
            }
        }
        // Scales and biases of the chunk: thread -> (array, token), 4 groups each.
        if constexpr (QUANT) {
            const int arr = tid >> 7, tok = tid & 127;  // 0: keys, 1: values
            const uint32_t token = min(base + tok, last);
            const bool live = base + tok < max_len;
            const size_t gi = (size_t(token) * kvh + kv) * 4;
            const uint2 sraw = *reinterpret_cast<const uint2 *>((arr ? a.vscales : a.kscales) + gi);
            const uint2 zraw = *reinterpret_cast<const uint2 *>((arr ? a.vbiases : a.kbiases) + gi);
            const float smul = arr ? P_UP : code_up<BITS>() / Q_UP;
            const float zmul = arr ? 1.0f : 1.0f / Q_UP;
            float *sdst = arr ? vs_lds : ks_lds, *zdst = arr ? vz_lds : kz_lds;
            const uint32_t sw[2] = {sraw.x, sraw.y}, zw[2] = {zraw.x, zraw.y};
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const __half s = __ushort_as_half(uint16_t(sw[g >> 1] >> (16 * (g & 1))));
                const __half z = __ushort_as_half(uint16_t(zw[g >> 1] >> (16 * (g & 1))));
                // Tokens past the context get 0 so that whatever their rows hold stays out.
                sdst[g * CHUNK + tok] = live ? __half2float(s) * smul : 0.0f;
                zdst[g * CHUNK + tok] = live ? __half2float(z) * zmul : 0.0f;
            }
        }
        __syncthreads();  // scales visible; also orders the previous chunk's phase C before new S

        // ---- phase A: scores -------------------------------------------------------
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            half8 qt[PARTS * 8];
            float qs[4];
            if constexpr (TILES == 1) {
#pragma unroll
                for (int i = 0; i < PARTS * 8; i++) qt[i] = q_reg[i];
#pragma unroll
                for (int g = 0; g < 4; g++) qs[g] = QUANT ? qsum_reg[g] : 0.0f;
            } else {
#pragma unroll
                for (int i = 0; i < PARTS * 8; i++) qt[i] = q_lds[(t * PARTS * 8 + i) * 64 + lane];
#pragma unroll
                for (int g = 0; g < 4; g++) qs[g] = QUANT ? qsum_lds[(t * 4 + g) * 16 + n] : 0.0f;
            }
#pragma unroll
            for (int b = 0; b < 2; b++) {
                floatx4 s = {0, 0, 0, 0};
                const int tok0 = 32 * wave + 16 * b + 4 * j;  // this lane's 4 tokens in C layout
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    floatx4 r = {0, 0, 0, 0};
#pragma unroll
                    for (int ab = 0; ab < 2; ab++) {
                        const half8 kop = key_operand<BITS>(kreg[b][g], ab);
#pragma unroll
                        for (int part = 0; part < PARTS; part++) {
                            r = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop, qt[part * 8 + g * 2 + ab], r, 0,
                                                                       0, 0);
                        }
                    }
                    if constexpr (QUANT) {
                        const floatx4 sc = *reinterpret_cast<const floatx4 *>(ks_lds + g * CHUNK + tok0);
                        const floatx4 zc = *reinterpret_cast<const floatx4 *>(kz_lds + g * CHUNK + tok0);
#pragma unroll
                        for (int i = 0; i < 4; i++) s[i] += sc[i] * r[i] + zc[i] * qs[g];
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; i++) s[i] += r[i] * (1.0f / Q_UP);
                    }
                }
                *reinterpret_cast<floatx4 *>(s_lds + (16 * t + n) * SC_STRIDE + tok0) = s;
            }
        }
        __syncthreads();

        // ---- phase B: online softmax per row ---------------------------------------
        {
            float sv[Sh::TPT];
            float *row = s_lds + b_row * SC_STRIDE + b_part * Sh::TPT;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i += 4) {
                floatx4 v = *reinterpret_cast<const floatx4 *>(row + i);
                if constexpr (PACKED) {
                    const floatx4 w = *reinterpret_cast<const floatx4 *>(row + 8 * SC_STRIDE + i);
                    v += w;
                }
                sv[i] = v[0], sv[i + 1] = v[1], sv[i + 2] = v[2], sv[i + 3] = v[3];
            }
            const uint32_t tok0 = base + b_part * Sh::TPT;
            float cm = NO_SCORE;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i++) cm = (tok0 + i < b_len) ? fmaxf(cm, sv[i]) : cm;
#pragma unroll
            for (int step = 1; step < Sh::TPR; step *= 2) cm = fmaxf(cm, __shfl_xor(cm, step));
            const float nm = fmaxf(m_run, cm);
            const float al = exp2f(m_run - nm);
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i++) {
                sv[i] = (tok0 + i < b_len) ? exp2f(sv[i] - nm) : 0.0f;
                sum += sv[i];
            }
            l_part = l_part * al + sum;
            m_run = nm;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i += 4) {
                *reinterpret_cast<floatx4 *>(row + i) = floatx4{sv[i], sv[i + 1], sv[i + 2], sv[i + 3]};
            }
            if (b_part == 0) alpha_lds[b_row] = al;
        }
        __syncthreads();

        // ---- phase C: O += P V for this wave's group -------------------------------
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            // Rescale what was summed so far.  Accumulator rows (C layout) are 4j..4j+3.
            {
                const int arow = PACKED ? ((4 * j) & 7) : 16 * t + 4 * j;
                const floatx4 al = *reinterpret_cast<const floatx4 *>(alpha_lds + arow);
#pragma unroll
                for (int e = 0; e < 4; e++) acc[t][e] *= al;
                zacc[t] *= alpha_lds[PACKED ? (n & 7) : 16 * t + n];
            }
            const float *prow = s_lds + (PACKED ? (n & 7) : 16 * t + n) * SC_STRIDE;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const int tk = 32 * ks + 8 * j;
                const floatx4 p0 = *reinterpret_cast<const floatx4 *>(prow + tk);
                const floatx4 p1 = *reinterpret_cast<const floatx4 *>(prow + tk + 4);
                float pv[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
                if constexpr (QUANT) {
                    const floatx4 s0 = *reinterpret_cast<const floatx4 *>(vs_lds + wave * CHUNK + tk);
                    const floatx4 s1 = *reinterpret_cast<const floatx4 *>(vs_lds + wave * CHUNK + tk + 4);
                    const floatx4 z0 = *reinterpret_cast<const floatx4 *>(vz_lds + wave * CHUNK + tk);
                    const floatx4 z1 = *reinterpret_cast<const floatx4 *>(vz_lds + wave * CHUNK + tk + 4);
                    const float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
                    const float zc[8] = {z0[0], z0[1], z0[2], z0[3], z1[0], z1[1], z1[2], z1[3]};
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        zacc[t] += pv[e] * zc[e];
                        pv[e] *= sc[e];
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) pv[e] *= P_UP;
                }
                half8 phi, plo;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    _Float16 h, lw;
                    split_hi_lo(pv[e], h, lw);
                    phi[e] = h;
                    plo[e] = lw;
                }
                if constexpr (PACKED) {
                    if (n >= 8) phi = plo;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const half8 vop = val_operand<BITS>(vreg[ks], e, n);
                    acc[t][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(phi, vop, acc[t][e], 0, 0, 0);
                    if constexpr (!PACKED) {
                        acc[t][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(plo, vop, acc[t][e], 0, 0, 0);
                    }
                }
            }
        }
        // The next chunk's first barrier (after its loads) keeps its writes to the
        // scale arrays behind this phase; S is rewritten only after that barrier too.
        if (chunk + a.nsplits < (max_len + CHUNK - 1) / CHUNK) __syncthreads();
    }

    // ---- epilogue: one partial per (row, head) ------------------------------------
    // m and l from the phase B threads.
#pragma unroll
    for (int step = 1; step < Sh::TPR; step *= 2) l_part += __shfl_xor(l_part, step);
    const bool b_has = split * CHUNK < b_len;  // this row has tokens in this split
    if (b_part == 0 && b_has) {
        const int vrow = PACKED ? 0 : b_row >> 3, head = b_row & 7;
        const size_t slot = (size_t(vrow) * a.nsplits + split) * a.heads + kv * 8 + head;
        a.part_ml[2 * slot] = m_run;
        a.part_ml[2 * slot + 1] = l_part;
    }
    // Bias sums: reduce over the 4 lane groups, hand to the C-layout lanes through LDS.
    if constexpr (QUANT) {
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            float z = zacc[t];
            z += __shfl_xor(z, 16);
            z += __shfl_xor(z, 32);
            // One copy per wave: the sum of wave w's group lives at [w][row].
            if (j == 0 && (!PACKED || n < 8)) zsum_lds[wave * Sh::S_ROWS + 16 * t + n] = z;
        }
        __syncthreads();
    }
    const float unscale = code_up<BITS>() / P_UP;
#pragma unroll
    for (int t = 0; t < TILES; t++) {
        floatx4 o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            o[e] = acc[t][e];
            if constexpr (PACKED) {
                // rows 8-15 hold the lo part of rows 0-7: lanes j and j + 2.
#pragma unroll
                for (int i = 0; i < 4; i++) o[e][i] += __shfl_xor(o[e][i], 32);
            }
        }
        if (PACKED && j >= 2) continue;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pair = 16 * t + 4 * j + i;  // (row, head) pair of this accumulator row
            if (pair >= int(real_rows)) continue;
            const int vrow = pair >> 3, head = pair & 7;
            const uint32_t len = min(a.decode_len ? a.tp->kv_len : position + vrow + 1, a.capacity);
            if (split * CHUNK >= len) continue;
            const float zb = QUANT ? zsum_lds[wave * Sh::S_ROWS + pair] : 0.0f;
            const size_t slot = (size_t(vrow) * a.nsplits + split) * a.heads + kv * 8 + head;
            float *dst = a.part_o + slot * DIM + 64 * wave;
            if constexpr (BITS == 16) {
                // tile e: dims 32*(e/2) + 2n + e%2
                *reinterpret_cast<float2 *>(dst + 2 * n) =
                    make_float2(o[0][i] * unscale, o[1][i] * unscale);
                *reinterpret_cast<float2 *>(dst + 32 + 2 * n) =
                    make_float2(o[2][i] * unscale, o[3][i] * unscale);
            } else {
                *reinterpret_cast<float4 *>(dst + 4 * n) =
                    make_float4(o[0][i] * unscale + zb, o[1][i] * unscale + zb, o[2][i] * unscale + zb,
                                o[3][i] * unscale + zb);
            }
        }
    }
}

// Merges the splits of one (q head, row): weights 2^(m_c - M), then the gate.
// 1024 threads = 4 slices x 256 dims, slice s takes splits s, s+4, ...
// (reference: attention_reduce / attention_reduce_rows,
// kernels/attention.metal:367-409, kernels/attention_rows.metal:296-342).
struct ReduceArgs {
    const float *part_o;
    const float *part_ml;
    const float *q_and_gate;
    float *out;
    uint32_t heads, capacity, nsplits;
    const saetta_token_params *tp;
    uint32_t decode_len;
};

__global__ __launch_bounds__(1024) void attention_reduce_kernel(ReduceArgs a) {
    __shared__ float slice_m[4], slice_l[4];
    __shared__ float slice_o[4][DIM];
    const uint32_t h = blockIdx.x, row = blockIdx.y;
    const uint32_t d = threadIdx.x & 255, s = threadIdx.x >> 8;
    const uint32_t len = min(a.decode_len ? a.tp->kv_len : a.tp->position + row + 1, a.capacity);
    const uint32_t parts = min(a.nsplits, (len + CHUNK - 1) / CHUNK);
    const float *ml = a.part_ml + size_t(2) * row * a.nsplits * a.heads;
    const float *po = a.part_o + size_t(row) * a.nsplits * a.heads * DIM;
    float m = NO_SCORE;
    for (uint32_t c = s; c < parts; c += 4) m = fmaxf(m, ml[2 * (size_t(c) * a.heads + h)]);
    if (d == 0) slice_m[s] = m;
    __syncthreads();
    m = fmaxf(fmaxf(slice_m[0], slice_m[1]), fmaxf(slice_m[2], slice_m[3]));
    float l = 0.0f, acc = 0.0f;
    for (uint32_t c = s; c < parts; c += 4) {
        const size_t i = size_t(c) * a.heads + h;
        const float w = exp2f(ml[2 * i] - m);
        l += w * ml[2 * i + 1];
        acc += w * po[i * DIM + d];
    }
    slice_o[s][d] = acc;
    if (d == 0) slice_l[s] = l;
    __syncthreads();
    if (s == 0) {
        const float o = slice_o[0][d] + slice_o[1][d] + slice_o[2][d] + slice_o[3][d];
        const float total = slice_l[0] + slice_l[1] + slice_l[2] + slice_l[3];
        const size_t qh = size_t(row) * a.heads + h;
        const float g = a.q_and_gate[qh * 2 * DIM + DIM + d];
        a.out[qh * DIM + d] = o / total * (1.0f / (1.0f + expf(-g)));
    }
}

// Most workgroups per kv head.  A split costs one 8 KB partial per row and
// kv head, so few is better; 512 keeps one chunk per workgroup up to 64k tokens.
constexpr uint32_t MAX_SPLITS = 512;

uint32_t splits_for(uint32_t capacity, uint32_t wanted) {
    uint32_t chunks = (capacity + CHUNK - 1) / CHUNK;
    uint32_t s = chunks < MAX_SPLITS ? chunks : MAX_SPLITS;
    if (wanted && wanted < s) s = wanted;
    return s ? s : 1;
}

template <int BITS, int TILES, bool PACKED>
void launch_partial(hipStream_t stream, const PartialArgs &a) {
    using Sh = Shape<BITS, TILES, PACKED>;
    auto kernel = attention_partial_kernel<BITS, TILES, PACKED>;
    static bool attr_set = false;
    if (!attr_set && Sh::LDS_BYTES > 48 * 1024) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, Sh::LDS_BYTES);
        attr_set = true;
    }
    kernel<<<dim3(a.nsplits, a.kv_heads), THREADS, Sh::LDS_BYTES, stream>>>(a);
}

template <int BITS>
void launch_partial_rows(hipStream_t stream, const PartialArgs &a) {
    if (a.rows == 1) {
        launch_partial<BITS, 1, true>(stream, a);
    } else if (a.rows == 2) {
        launch_partial<BITS, 1, false>(stream, a);
    } else if (a.rows <= 4) {
        launch_partial<BITS, 2, false>(stream, a);
    } else {
        launch_partial<BITS, 4, false>(stream, a);
    }
}

int run_attention(hipStream_t stream, int bits, const float *q, const void *kdata, const void *vdata,
                  const uint16_t *ks, const uint16_t *kz, const uint16_t *vs, const uint16_t *vz,
                  float *part_o, float *part_ml, const float *q_and_gate, float *out, uint32_t heads,
                  uint32_t kv_heads, uint32_t capacity, float scale, uint32_t rows, uint32_t wanted_splits,
                  const saetta_token_params *d_tp, bool decode_len, uint32_t stages, const char *what) {
    SAETTA_REQUIRE(bits == 16 || bits == 8 || bits == 4, SAETTA_E_BITS, "%s: bits %d", what, bits);
    SAETTA_REQUIRE(kv_heads > 0 && heads == kv_heads * SAETTA_GQA_GROUP, SAETTA_E_SHAPE,
                   "%s needs 8 q heads per kv head (heads %u, kv heads %u)", what, heads, kv_heads);
    SAETTA_REQUIRE(rows >= 1 && rows <= SAETTA_MAX_ROWS, SAETTA_E_SHAPE, "%s: %u rows (1..8)", what, rows);
    SAETTA_REQUIRE(capacity > 0, SAETTA_E_SHAPE, "%s: capacity 0", what);
    SAETTA_REQUIRE(q && kdata && vdata && part_o && part_ml && q_and_gate && out && d_tp, SAETTA_E_NULL,
                   "%s: null buffer", what);
    SAETTA_REQUIRE(bits == 16 || (ks && kz && vs && vz), SAETTA_E_NULL, "%s: null scales or biases", what);
    SAETTA_REQUIRE(aligned(q, 16) && aligned(kdata, 16) && aligned(vdata, 16) && aligned(part_o, 16) &&
                       aligned(part_ml, 8),
                   SAETTA_E_ALIGN, "%s: q, cache and scratch must be 16-byte aligned", what);
    SAETTA_REQUIRE(bits == 16 || (aligned(ks, 8) && aligned(kz, 8) && aligned(vs, 8) && aligned(vz, 8)),
                   SAETTA_E_ALIGN, "%s: scales and biases must be 8-byte aligned", what);
    if (int rc = ensure_device()) return rc;
    const uint32_t nsplits = splits_for(capacity, wanted_splits);
    if (stages & SAETTA_STAGE_PARTIAL) {
        PartialArgs a{q,        kdata,  vdata, ks,    kz,      vs,   vz,   part_o, part_ml,
                      heads,    kv_heads, capacity, scale, rows, nsplits, d_tp, decode_len ? 1u : 0u};
        if (bits == 8) {
            launch_partial_rows<8>(stream, a);
        } else if (bits == 4) {
            launch_partial_rows<4>(stream, a);
        } else {
            launch_partial_rows<16>(stream, a);
        }
    }
    if (stages & SAETTA_STAGE_REDUCE) {
        ReduceArgs r{part_o, part_ml, q_and_gate, out, heads, capacity, nsplits, d_tp, decode_len ? 1u : 0u};
        attention_reduce_kernel<<<dim3(heads, rows), 1024, 0, stream>>>(r);
    }
    return launch_status(what);
}

}  // namespace
}  // namespace saetta

using namespace saetta;

extern "C" size_t saetta_part_o_bytes(uint32_t heads, uint32_t capacity, uint32_t rows) {
    return size_t(rows) * splits_for(capacity, 0) * heads * DIM * sizeof(float);
}

extern "C" size_t saetta_part_ml_bytes(uint32_t heads, uint32_t capacity, uint32_t rows) {
    return size_t(rows) * splits_for(capacity, 0) * heads * 2 * sizeof(float);
}

extern "C" int saetta_attn_decode(saetta_stream_t stream, const float *q, const uint16_t *keys,
                                  const uint16_t *values, float *part_o, float *part_ml,
                                  const float *q_and_gate, float *out, saetta_decode_params p,
                                  const saetta_token_params *d_tp, uint32_t stages) {
    return run_attention(as_stream(stream), 16, q, keys, values, nullptr, nullptr, nullptr, nullptr, part_o,
                         part_ml, q_and_gate, out, p.heads, p.kv_heads, p.capacity, p.scale, 1, 0, d_tp,
                         true, stages, "attn_decode");
}

extern "C" int saetta_attn_decode_quant(saetta_stream_t stream, int bits, const float *q,
                                        saetta_quant_rows keys, saetta_quant_rows values, float *part_o,
                                        float *part_ml, const float *q_and_gate, float *out,
                                        saetta_decode_params p, const saetta_token_params *d_tp,
                                        uint32_t stages) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "attn_decode_quant: bits %d (8 or 4)", bits);
    return run_attention(as_stream(stream), bits, q, keys.data, values.data, keys.scales, keys.biases,
                         values.scales, values.biases, part_o, part_ml, q_and_gate, out, p.heads,
                         p.kv_heads, p.capacity, p.scale, 1, 0, d_tp, true, stages, "attn_decode_quant");
}

extern "C" int saetta_attn_rows(saetta_stream_t stream, const float *q, const uint16_t *keys,
                                const uint16_t *values, float *part_o, float *part_ml,
                                const float *q_and_gate, float *out, saetta_rows_params p,
                                const saetta_token_params *d_tp, uint32_t stages) {
    return run_attention(as_stream(stream), 16, q, keys, values, nullptr, nullptr, nullptr, nullptr, part_o,
                         part_ml, q_and_gate, out, p.heads, p.kv_heads, p.capacity, p.scale, p.rows,
                         p.splits, d_tp, false, stages, "attn_rows");
}

extern "C" int saetta_attn_rows_quant(saetta_stream_t stream, int bits, const float *q,
                                      saetta_quant_rows keys, saetta_quant_rows values, float *part_o,
                                      float *part_ml, const float *q_and_gate, float *out,
                                      saetta_rows_params p, const saetta_token_params *d_tp,
                                      uint32_t stages) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "attn_rows_quant: bits %d (8 or 4)", bits);
    return run_attention(as_stream(stream), bits, q, keys.data, values.data, keys.scales, keys.biases,
                         values.scales, values.biases, part_o, part_ml, q_and_gate, out, p.heads,
                         p.kv_heads, p.capacity, p.scale, p.rows, p.splits, d_tp, false, stages,
                         "attn_rows_quant");
}
