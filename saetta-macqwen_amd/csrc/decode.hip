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
// the context.  The context actually in use (read from TokenParams in device
// memory when the kernel runs) is cut into 16-token blocks and the blocks are
// dealt evenly to the `nsplits` workgroups of each kv head, so every
// workgroup streams the same number of bytes whatever the position is.  A
// workgroup walks its range in iterations of 64 to 192 tokens, keeps an
// online softmax per query row, and writes one unnormalised partial (o, m, l)
// per (row, q head); a second kernel merges the partials and applies the gate.
//
// Inside an iteration the two contractions run on the matrix cores
// (v_mfma_f32_16x16x32_f16), because at 15-28 FLOP per cache byte a vector-ALU
// dot product cannot keep up with HBM:
//   phase A  S^T = K Q^T   wave w takes the 16-token blocks w, w+4, w+8;
//            A operand = key codes of 16 tokens, B operand = the query rows.
//   phase B  online softmax per row over the iteration's scores (in LDS).
//   phase C  O += P V      wave w takes dims 64w..64w+63, which is exactly
//            one quantization group, for all tokens of the iteration.
// Codes are never dequantized element by element.  A code byte c is placed in
// the low mantissa bits of an f16 with a zero exponent, i.e. the subnormal
// c * 2^-24, with one v_perm_b32 per two codes; the matrix cores take
// subnormal inputs.  Scale and bias of a group are applied to the 64-dim
// partial dot product (keys) or folded into the probability operand (values):
//   q.k   = sum_g  s_g * (q_g . c_g)  +  sum_g z_g * sum(q_g)
//   P V_g = (P * s_g) C_g + (P . z_g)
// and the key bias term sum_g z_g * sum(q_g) is itself one small MFMA.
// The value operand needs (token, token+1) pairs per dim while memory holds
// (dim, dim+1) pairs per token; the same v_perm_b32 that widens the bytes
// picks them from two tokens' words, so the transposition costs nothing.
// q and P are split into f16 hi + lo parts (two MFMAs into one accumulator,
// or for a single row the hi and lo parts share one 16-row tile), which keeps
// the result within ~1e-6 of an f32 evaluation.
//
// All cache reads of the register kernels are buffer loads with the cache's
// size as the bound: rows past the capacity read as 0 instead of faulting, and
// the per-lane address is one 32-bit offset plus scalar and immediate parts.
//
// Kernels (one body, attention_partial_body, behind template switches):
//   attention_partial_kernel_p   one query row, one workgroup per CU (all registers)
//   attention_partial_kernel_1   one query row over codes, two workgroups per CU (long 4-bit caches)
//   attention_partial_kernel_n   2 rows (1 tile), 3-4 rows (2 tiles), 5-8 rows (4 tiles)
//   attention_partial_kernel_s   one to four query rows over codes in large caches: four more waves
//                                move the codes into LDS (global_load_lds), a whole share at once
//                                with the keys requested first (longer shares: rounds in alternate
//                                halves of LDS), the waves meeting through counters in LDS
//   attention_reduce_kernel      the merge of the splits and the gate
// Which one runs is decided in run_attention from the launch arguments alone, so that the partial
// and the reduce stage of a step agree on the number of splits.
#include "common.hpp"
#include "lanes.hpp"

namespace saetta {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int DIM = SAETTA_HEAD_DIM;
constexpr int THREADS = 256;
constexpr int BLOCK = 16;                     // tokens per MFMA block
// A buffer offset past any cache (their sizes stay below 2^31): the load returns 0 and touches no
// memory.  With UNCOND, loads that an iteration does not need are issued with it instead of being
// branched around, so that the number of loads in flight at every wait is known when the kernel is
// compiled: loads return in order, and a wait whose count is not known has to wait for all of them.
// (Measured per kernel: it pays for one and two query rows, not for the larger tiles.)
constexpr int OOB = int(0x80000000u);
// s_waitcnt operand that waits for the vector memory counter only (gfx9 encoding: vmcnt in bits
// 3:0 and 15:14, the other counters at their maxima).
constexpr int vmcnt_only(int n) {
    return (n & 15) | 0x70 | 0xf00 | ((n >> 4) << 14);
}
constexpr float NO_SCORE = -1e30f;            // finite "minus infinity" of the running max

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
// Bytes of one (token, kv head) of keys or values.
template <int BITS>
constexpr int row_bytes() {
    return BITS == 16 ? 512 : BITS * 32;
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
    uint32_t *status;     // the device's sticky status word (pinned host memory)
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

__device__ __forceinline__ half8 as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    u32x4 v = {a, b, c, d};
    return __builtin_bit_cast(half8, v);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, int(bytes), 0x00020000);
}

// ---- key codes: 16 dims of one token per lane and group ----------------------
template <int BITS>
struct KeyRegs {
    uint32_t w[BITS == 16 ? 8 : BITS / 2];  // 32 B (f16), 16 B (8-bit), 8 B (4-bit)
};

// Lane (t, j) reads dims 64g + 16j .. +15 of its token: `voff` is the lane's
// byte offset of (token, kv head, j), `soff` the scalar part (block), g is an immediate.
template <int BITS>
__device__ __forceinline__ KeyRegs<BITS> load_key(__amdgpu_buffer_rsrc_t rsrc, int voff, int soff, int g) {
    KeyRegs<BITS> r;
    if constexpr (BITS == 8) {
        u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + g * 64, soff, 0);
        r.w[0] = v.x, r.w[1] = v.y, r.w[2] = v.z, r.w[3] = v.w;
    } else if constexpr (BITS == 4) {
        u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff + g * 32, soff, 0);
        r.w[0] = v.x, r.w[1] = v.y;
    } else {
        u32x4 v0 = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + g * 128, soff, 0);
        u32x4 v1 = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + g * 128 + 16, soff, 0);
        r.w[0] = v0.x, r.w[1] = v0.y, r.w[2] = v0.z, r.w[3] = v0.w;
        r.w[4] = v1.x, r.w[5] = v1.y, r.w[6] = v1.z, r.w[7] = v1.w;
    }
    return r;
}

// Bytes of the lane's 16 dims inside a group.
template <int BITS>
constexpr int key_piece() {
    return BITS == 16 ? 32 : BITS * 2;
}

// The A operand of k-step `ab` (0: the lane's first 8 dims, 1: the next 8).
template <int BITS>
__device__ __forceinline__ half8 key_operand(const KeyRegs<BITS> &r, int ab) {
    if constexpr (BITS == 8) {
        const uint32_t w0 = r.w[2 * ab], w1 = r.w[2 * ab + 1];
        return as_half8(perm(0, w0, 0x0c010c00u), perm(0, w0, 0x0c030c02u), perm(0, w1, 0x0c010c00u),
                        perm(0, w1, 0x0c030c02u));
    } else if constexpr (BITS == 4) {
        const uint32_t w = r.w[ab];
        const uint32_t x = (w << 4) & 0xf0f0f0f0u, y = w & 0xf0f0f0f0u;
        // slots: dims 0,2 | 4,6 | 1,3 | 5,7
        return as_half8(perm(0, x, 0x0c010c00u), perm(0, x, 0x0c030c02u), perm(0, y, 0x0c010c00u),
                        perm(0, y, 0x0c030c02u));
    } else {
        return as_half8(r.w[4 * ab], r.w[4 * ab + 1], r.w[4 * ab + 2], r.w[4 * ab + 3]);
    }
}

// Which of the lane's 8 dims of a k-step sits in MFMA slot e.
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

// Byte offset of the lane's dword inside a (token, kv head) row.
template <int BITS>
__device__ __forceinline__ int val_lane_offset(int wave, int n) {
    if constexpr (BITS == 8) return wave * 64 + n * 4;
    if constexpr (BITS == 4) return wave * 32 + (n >> 1) * 4;
    return wave * 128 + n * 4;
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
            const uint32_t a = ((r.w[2 * i] >> sh) << up) & 0xf0f0u, b = ((r.w[2 * i + 1] >> sh) << up) & 0xf0f0u;
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

__device__ __forceinline__ float half_bits_to_float(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, uint16_t(bits16));
}

// TILES: 16-row tiles of query rows (rows * 8 heads, rounded up).  PACKED: one
// verify row; its 8 heads' hi parts are operand rows 0-7 and lo parts rows 8-15
// of a single tile.  Otherwise hi and lo are two MFMAs into one accumulator.
// ITB: blocks per iteration of a workgroup (a multiple of 4: one block per wave and round).
template <int BITS, int TILES, bool PACKED, int ITB>
struct Shape {
    static constexpr int IT_BLOCKS = ITB;
    static constexpr int IT_TOKENS = BLOCK * ITB;
    static constexpr int SC_STRIDE = IT_TOKENS + 4;  // floats; keeps rows on different LDS banks
    static constexpr bool QUANT = BITS != 16;
    static constexpr int S_ROWS = 16 * TILES;                  // rows of the score buffer
    static constexpr int SOFT_ROWS = PACKED ? 8 : 16 * TILES;  // rows phase B walks
    static constexpr int TPR = THREADS / SOFT_ROWS;            // threads per row in phase B
    static constexpr int TPT = IT_TOKENS / TPR;                // tokens per thread in phase B
    static constexpr int PARTS = PACKED ? 1 : 2;
    // LDS map, in bytes
    static constexpr int Q_OFF = 0;
    static constexpr int Q_BYTES = TILES * PARTS * 8 * 64 * 16;  // [tile][part][step][lane] half8
    static constexpr int S_OFF = Q_OFF + Q_BYTES;
    static constexpr int S_BYTES = S_ROWS * SC_STRIDE * 4;  // [row][token] f32
    static constexpr int KS_OFF = S_OFF + S_BYTES;          // [token][4] f16
    static constexpr int KZ_OFF = KS_OFF + (QUANT ? IT_TOKENS * 8 : 0);
    static constexpr int VS_OFF = KZ_OFF + (QUANT ? IT_TOKENS * 8 : 0);  // [4][token] f16
    static constexpr int VZ_OFF = VS_OFF + (QUANT ? IT_TOKENS * 8 : 0);
    static constexpr int ALPHA_OFF = VZ_OFF + (QUANT ? IT_TOKENS * 8 : 0);  // [S_ROWS] f32
    static constexpr int QZ_OFF = ALPHA_OFF + S_ROWS * 4;                   // [tile][hi, lo][lane] half8
    static constexpr int ZSUM_OFF = QZ_OFF + TILES * 2 * 64 * 16;           // [wave][S_ROWS] f32
    static constexpr int LDS_BYTES = ZSUM_OFF + 4 * S_ROWS * 4;
};

template <int BITS, int TILES, bool PACKED, int ITB, bool UNCOND>
__device__ __forceinline__ void attention_partial_body(const PartialArgs &a) {
    using Sh = Shape<BITS, TILES, PACKED, ITB>;
    constexpr int IT_BLOCKS = ITB, IT_TOKENS = Sh::IT_TOKENS, SC_STRIDE = Sh::SC_STRIDE;
    constexpr int KROUNDS = ITB / 4, KSTEPS = ITB / 2;
    constexpr bool QUANT = Sh::QUANT;
    constexpr int PARTS = Sh::PARTS;
    constexpr int RB = row_bytes<BITS>();
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = int(threadIdx.x), lane = tid & 63, wave = tid >> 6;
    half8 *q_lds = reinterpret_cast<half8 *>(lds_raw + Sh::Q_OFF);
    float *s_lds = reinterpret_cast<float *>(lds_raw + Sh::S_OFF);
    uint16_t *ks_lds = reinterpret_cast<uint16_t *>(lds_raw + Sh::KS_OFF);
    uint16_t *kz_lds = reinterpret_cast<uint16_t *>(lds_raw + Sh::KZ_OFF);
    uint16_t *vs_lds = reinterpret_cast<uint16_t *>(lds_raw + Sh::VS_OFF);
    uint16_t *vz_lds = reinterpret_cast<uint16_t *>(lds_raw + Sh::VZ_OFF);
    float *alpha_lds = reinterpret_cast<float *>(lds_raw + Sh::ALPHA_OFF);
    _Float16 *qz_lds = reinterpret_cast<_Float16 *>(lds_raw + Sh::QZ_OFF);
    float *zsum_lds = reinterpret_cast<float *>(lds_raw + Sh::ZSUM_OFF);

    const int n = lane & 15, j = lane >> 4;
    const uint32_t split = blockIdx.x, kv = blockIdx.y;
    const uint32_t kvh = a.kv_heads;
    const uint32_t real_rows = a.rows * 8;  // (row, head) pairs of this kv head

    // ---- query values: requested first, so that nothing they wait for is behind the cache ----
    // Item (tile t, k-step, lane l) is the 8 values that lane l feeds to the MFMA k-step;
    // operand row `on` of tile t: PACKED -> head on & 7, part on >> 3; else (row, head)
    // pair 16t + on, both parts.
    auto load_q_item = [&](int item, float (&v)[8]) {
        const int t = item / 512, step = (item / 64) & 7, l = item & 63;
        const int on = l & 15, oj = l >> 4;
        const int g = step >> 1, ab = step & 1;
        const int pair = PACKED ? (on & 7) : 16 * t + on;
        if (PACKED || pair < int(real_rows)) {  // (a single row always has its 8 heads)
            const int row = pair >> 3, head = pair & 7;
            const float *src = a.q + (size_t(row) * a.heads + kv * 8 + head) * DIM + 64 * g + 16 * oj + 8 * ab;
            const float4 f0 = *reinterpret_cast<const float4 *>(src);
            const float4 f1 = *reinterpret_cast<const float4 *>(src + 4);
            v[0] = f0.x, v[1] = f0.y, v[2] = f0.z, v[3] = f0.w;
            v[4] = f1.x, v[5] = f1.y, v[6] = f1.z, v[7] = f1.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = 0.0f;
        }
    };
    float q_early[TILES == 1 ? 2 : 1][8];
    if constexpr (TILES == 1) {
        load_q_item(tid, q_early[0]);
        load_q_item(tid + THREADS, q_early[1]);
    }

    // ---- the context and this workgroup's share of it -----------------------------
    const uint32_t position = a.tp->position;
    const uint32_t kv_len = a.tp->kv_len;
    // Tokens the last row sees; the longest context of the launch.
    const uint32_t max_len = min(a.decode_len ? kv_len : position + a.rows, a.capacity);
    const uint32_t nblocks = (max_len + BLOCK - 1) / BLOCK;
    uint32_t blk_begin, blk_end;
    if (nblocks <= a.nsplits) {
        blk_begin = split;
        blk_end = split + 1;
        if (split >= nblocks) return;
    } else {
        // (split + 1) * nblocks < 2^32: at most 256 splits and 2^27 blocks (32-bit cache offsets)
        blk_begin = split * nblocks / a.nsplits;
        blk_end = (split + 1) * nblocks / a.nsplits;
    }
    const uint32_t range = blk_end - blk_begin;
    const uint32_t n_it = (range + IT_BLOCKS - 1) / IT_BLOCKS;
    const uint32_t per_it = (range + n_it - 1) / n_it;
    const uint32_t n_rounds = n_it;

    const uint32_t cap_rows = a.capacity * kvh;
    const __amdgpu_buffer_rsrc_t k_rsrc = make_rsrc(a.kdata, cap_rows * RB);
    const __amdgpu_buffer_rsrc_t v_rsrc = make_rsrc(a.vdata, cap_rows * RB);
    const __amdgpu_buffer_rsrc_t ks_rsrc = make_rsrc(a.kscales, QUANT ? cap_rows * 8 : 0);
    const __amdgpu_buffer_rsrc_t kz_rsrc = make_rsrc(a.kbiases, QUANT ? cap_rows * 8 : 0);
    const __amdgpu_buffer_rsrc_t vs_rsrc = make_rsrc(a.vscales, QUANT ? cap_rows * 8 : 0);
    const __amdgpu_buffer_rsrc_t vz_rsrc = make_rsrc(a.vbiases, QUANT ? cap_rows * 8 : 0);
    const int tok_stride = int(kvh) * RB;  // bytes between tokens of one kv head

    // ---- the loads of one iteration ------------------------------------------------
    // Everything an iteration reads is requested before anything is computed: keys first
    // (phase A needs them first), then the small scale/bias rows, then the values.
    KeyRegs<BITS> kreg[KROUNDS][4];
    ValRegs<BITS> vreg[KSTEPS];
    u32x2 ksr = {0, 0}, kzr = {0, 0}, vsr = {0, 0}, vzr = {0, 0};
    auto blocks_of = [&](uint32_t it) { return it < n_it ? min(per_it, blk_end - (blk_begin + it * per_it)) : 0u; };
    auto load_keys = [&](uint32_t it) {
        const uint32_t base = (blk_begin + it * per_it) * BLOCK, nb = blocks_of(it);
        const int voff = int((base + BLOCK * wave + n) * kvh + kv) * RB + j * key_piece<BITS>();
#pragma unroll
        for (int i = 0; i < KROUNDS; i++) {
            const bool need = uint32_t(wave + 4 * i) < nb;
            if (UNCOND || need) {
                const int off = need ? voff : OOB;
#pragma unroll
                for (int g = 0; g < 4; g++) kreg[i][g] = load_key<BITS>(k_rsrc, off, i * 64 * tok_stride, g);
            }
        }
    };
    auto load_scales = [&](uint32_t it) {
        if constexpr (QUANT) {
            const uint32_t base = (blk_begin + it * per_it) * BLOCK;
            const bool need = uint32_t(tid) < blocks_of(it) * BLOCK;
            if (UNCOND || need) {
                const int voff = need ? int((base + tid) * kvh + kv) * 8 : OOB;
                ksr = __builtin_amdgcn_raw_buffer_load_b64(ks_rsrc, voff, 0, 0);
                kzr = __builtin_amdgcn_raw_buffer_load_b64(kz_rsrc, voff, 0, 0);
                vsr = __builtin_amdgcn_raw_buffer_load_b64(vs_rsrc, voff, 0, 0);
                vzr = __builtin_amdgcn_raw_buffer_load_b64(vz_rsrc, voff, 0, 0);
            }
        }
    };
    auto load_values = [&](uint32_t it) {
        const uint32_t base = (blk_begin + it * per_it) * BLOCK, ksteps = (blocks_of(it) + 1) / 2;
        const int voff = int((base + 8 * j) * kvh + kv) * RB + val_lane_offset<BITS>(wave, n);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            const bool need = uint32_t(ks) < ksteps;
            if (UNCOND || need) {
                const int off = need ? voff : OOB;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int soff = (32 * ks + e) * tok_stride;
                    vreg[ks].w[e] = __builtin_amdgcn_raw_buffer_load_b32(v_rsrc, off, soff, 0);
                    if constexpr (BITS == 16) {
                        vreg[ks].w[8 + e] = __builtin_amdgcn_raw_buffer_load_b32(v_rsrc, off + 64, soff, 0);
                    }
                }
            }
        }
    };
    load_scales(0);  // first: loads return in order, and the barrier that publishes the scales must not wait for the keys
    load_keys(0);
    load_values(0);

    // ---- prologue: query rows to f16 hi/lo operands in LDS ------------------------
    // (while the first iteration's keys are in flight; the values are requested after it)
    {
        const float qmul = a.scale * 1.4426950408889634f * Q_UP;
#pragma unroll
        for (int k = 0; k < TILES * 2; k++) {
            const int item = tid + k * THREADS;
            const int t = item / 512, step = (item / 64) & 7, l = item & 63;
            const int on = l & 15;
            float v[8];
            if constexpr (TILES == 1) {
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = q_early[k][e];
            } else {
                load_q_item(item, v);
            }
            half8 hi, lo;
            float sum_hi = 0.0f, sum_lo = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                _Float16 h, lw;
                split_hi_lo(v[key_slot_dim<BITS>(e)] * qmul, h, lw);
                hi[e] = h;
                lo[e] = lw;
                sum_hi += (float)h;
                sum_lo += (float)lw;
            }
            float sum;
            if constexpr (PACKED) {
                q_lds[step * 64 + l] = (on < 8) ? hi : lo;
                sum = (on < 8) ? sum_hi : sum_lo;
            } else {
                q_lds[((t * 2 + 0) * 8 + step) * 64 + l] = hi;
                q_lds[((t * 2 + 1) * 8 + step) * 64 + l] = lo;
                sum = sum_hi + sum_lo;
            }
            // The key bias term sum_g z_g * sum_{d in g} q_d is one more MFMA over the same 32
            // (lane group, slot) pairs: its B operand holds, in lane l and slot `step`, the sum of
            // the 8 operand values this item made (divided by Q_UP, as hi and lo halves), and its
            // A operand holds z_g of the step's group.
            if constexpr (QUANT) {
                _Float16 h, lw;
                split_hi_lo(sum * (1.0f / Q_UP), h, lw);
                qz_lds[((t * 2 + 0) * 64 + l) * 8 + step] = h;
                qz_lds[((t * 2 + 1) * 64 + l) * 8 + step] = lw;
            }
        }
    }
    __syncthreads();

    // Query operands of a single tile live in registers for the whole kernel.
    half8 q_reg[TILES == 1 ? PARTS * 8 : 1];
    half8 qz_reg[2] = {{0, 0, 0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0, 0, 0}};
    if constexpr (TILES == 1) {
#pragma unroll
        for (int i = 0; i < PARTS * 8; i++) q_reg[i] = q_lds[i * 64 + lane];
        if constexpr (QUANT) {
            qz_reg[0] = *reinterpret_cast<const half8 *>(qz_lds + lane * 8);
            qz_reg[1] = *reinterpret_cast<const half8 *>(qz_lds + (64 + lane) * 8);
        }
    }

    // ---- running state -------------------------------------------------------------
    // Phase B: thread (row, part) of SOFT_ROWS x TPR.
    const int b_row = tid / Sh::TPR, b_part = tid % Sh::TPR;
    uint32_t b_len;  // tokens row b_row sees
    {
        const int vrow = PACKED ? 0 : b_row >> 3;
        const bool real = PACKED || b_row < int(real_rows);
        const uint32_t len = a.decode_len ? kv_len : position + vrow + 1;
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

    for (uint32_t round = 0; round < n_rounds; round++) {
        const uint32_t it = round;
        const uint32_t blk0 = blk_begin + it * per_it;
        const uint32_t nb = blocks_of(it);  // blocks of this iteration, 0..ITB
        const uint32_t base = blk0 * BLOCK;
        const uint32_t it_tokens = nb * BLOCK;
        const uint32_t ksteps = (nb + 1) / 2;

        // Scales and biases of the iteration's tokens to LDS: thread = token, 4 groups each.  The key
        // ones before the barrier (phase A reads them); the value ones after it: a wave may still be
        // reading the previous iteration's in its phase C until every wave has arrived here.
        if constexpr (QUANT) {
            if (tid < IT_TOKENS) {
                *reinterpret_cast<u32x2 *>(ks_lds + 4 * tid) = ksr;
                *reinterpret_cast<u32x2 *>(kz_lds + 4 * tid) = kzr;
            }
        }
        __syncthreads();  // key scales visible; the previous iteration's phase C is over
        if constexpr (QUANT) {
            if (tid < IT_TOKENS) {
                // Tokens past the context or the iteration get value scale 0 and bias 0, so that
                // whatever their rows hold stays out of O (their probabilities are 0 as well).
                if (uint32_t(tid) >= it_tokens || base + tid >= max_len) vsr = u32x2{0, 0}, vzr = u32x2{0, 0};
                vs_lds[0 * IT_TOKENS + tid] = uint16_t(vsr.x), vs_lds[1 * IT_TOKENS + tid] = uint16_t(vsr.x >> 16);
                vs_lds[2 * IT_TOKENS + tid] = uint16_t(vsr.y), vs_lds[3 * IT_TOKENS + tid] = uint16_t(vsr.y >> 16);
                vz_lds[0 * IT_TOKENS + tid] = uint16_t(vzr.x), vz_lds[1 * IT_TOKENS + tid] = uint16_t(vzr.x >> 16);
                vz_lds[2 * IT_TOKENS + tid] = uint16_t(vzr.y), vz_lds[3 * IT_TOKENS + tid] = uint16_t(vzr.y >> 16);
            }
        }
        // ---- phase A: scores -------------------------------------------------------
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            half8 qt[PARTS * 8];
            half8 qz[2] = {qz_reg[0], qz_reg[1]};
            if constexpr (TILES == 1) {
#pragma unroll
                for (int i = 0; i < PARTS * 8; i++) qt[i] = q_reg[i];
            } else {
#pragma unroll
                for (int i = 0; i < PARTS * 8; i++) qt[i] = q_lds[(t * PARTS * 8 + i) * 64 + lane];
                if constexpr (QUANT) {
                    qz[0] = *reinterpret_cast<const half8 *>(qz_lds + ((t * 2 + 0) * 64 + lane) * 8);
                    qz[1] = *reinterpret_cast<const half8 *>(qz_lds + ((t * 2 + 1) * 64 + lane) * 8);
                }
            }
#pragma unroll
            for (int i = 0; i < KROUNDS; i++) {
                const int blk = wave + 4 * i;
                if (uint32_t(blk) >= nb) break;
                const int tok0 = BLOCK * blk + 4 * j;  // this lane's 4 tokens in C layout
                floatx4 s = {0, 0, 0, 0};
                if constexpr (QUANT) {
                    // bias term: slot e of every lane group belongs to group e / 2 of token n
                    const u32x2 zr = *reinterpret_cast<const u32x2 *>(kz_lds + 4 * (BLOCK * blk + n));
                    const half8 zop = as_half8(perm(0, zr.x, 0x01000100u), perm(0, zr.x, 0x03020302u),
                                               perm(0, zr.y, 0x01000100u), perm(0, zr.y, 0x03020302u));
                    s = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz[0], s, 0, 0, 0);
                    s = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz[1], s, 0, 0, 0);
                }
                floatx4 r[4];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    r[g] = floatx4{0, 0, 0, 0};
#pragma unroll
                    for (int ab = 0; ab < 2; ab++) {
                        const half8 kop = key_operand<BITS>(kreg[i][g], ab);
#pragma unroll
                        for (int part = 0; part < PARTS; part++) {
                            r[g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop, qt[part * 8 + g * 2 + ab], r[g], 0,
                                                                          0, 0);
                        }
                    }
                }
                if constexpr (QUANT) {
                    // scales of tokens tok0..tok0+3, 4 groups each: 32 contiguous bytes
                    const u32x4 s01 = *reinterpret_cast<const u32x4 *>(ks_lds + 4 * tok0);
                    const u32x4 s23 = *reinterpret_cast<const u32x4 *>(ks_lds + 4 * tok0 + 8);
                    const uint32_t sw[8] = {s01.x, s01.y, s01.z, s01.w, s23.x, s23.y, s23.z, s23.w};
                    constexpr float C1 = code_up<BITS>() / Q_UP;
#pragma unroll
                    for (int tk = 0; tk < 4; tk++) {
                        float d = 0.0f;
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            d += half_bits_to_float(sw[2 * tk + (g >> 1)] >> (16 * (g & 1))) * r[g][tk];
                        }
                        s[tk] += d * C1;
                    }
                } else {
#pragma unroll
                    for (int tk = 0; tk < 4; tk++) s[tk] = (r[0][tk] + r[1][tk] + r[2][tk] + r[3][tk]) * (1.0f / Q_UP);
                }
                *reinterpret_cast<floatx4 *>(s_lds + (16 * t + n) * SC_STRIDE + tok0) = s;
            }
        }
        // The key registers and the scale registers are free: request the next iteration's.
        if (it + 1 < n_it) {
            load_scales(it + 1);
            load_keys(it + 1);
        }
        __syncthreads();

        // ---- phase B: online softmax per row ---------------------------------------
        // Writes P * P_UP over the scores; l sums the plain P.
        {
            float sv[Sh::TPT];
            float *row = s_lds + b_row * SC_STRIDE + b_part * Sh::TPT;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i += 2) {
                floatx2 v = *reinterpret_cast<const floatx2 *>(row + i);
                if constexpr (PACKED) {
                    v += *reinterpret_cast<const floatx2 *>(row + 8 * SC_STRIDE + i);
                }
                sv[i] = v[0], sv[i + 1] = v[1];
            }
            const uint32_t tok0 = b_part * Sh::TPT;
            // tokens of this row in this iteration: inside the iteration and inside the row's context
            const uint32_t lim = b_len > base ? min(b_len - base, it_tokens) : 0;
            float cm = NO_SCORE;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i++) cm = (tok0 + i < lim) ? fmaxf(cm, sv[i]) : cm;
            cm = group_reduce<Sh::TPR>(cm, MaxOp());
            const float nm = fmaxf(m_run, cm);
            const float al = __builtin_amdgcn_exp2f(m_run - nm);
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i++) {
                sv[i] = (tok0 + i < lim) ? __builtin_amdgcn_exp2f(sv[i] - nm) : 0.0f;
                sum += sv[i];
            }
            l_part = l_part * al + sum;
            m_run = nm;
#pragma unroll
            for (int i = 0; i < Sh::TPT; i += 2) {
                *reinterpret_cast<floatx2 *>(row + i) = floatx2{sv[i] * P_UP, sv[i + 1] * P_UP};
            }
            if (b_part == 0) alpha_lds[b_row] = al;
        }
        __syncthreads();

        // ---- phase C: O += P V for this wave's group -------------------------------
        // The probability operands need only P and the value scales, so they are all built
        // before the first value code is touched: what is left to do once the (large,
        // last-requested) value loads land is the byte permutes and the MFMAs.
        auto build_p = [&](int t, int ks, half8 &phi, half8 &plo) {
            const float *prow = s_lds + (PACKED ? (n & 7) : 16 * t + n) * SC_STRIDE;
            const int tk = 32 * ks + 8 * j;
            const floatx4 p0 = *reinterpret_cast<const floatx4 *>(prow + tk);
            const floatx4 p1 = *reinterpret_cast<const floatx4 *>(prow + tk + 4);
            float pv[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
            if constexpr (QUANT) {
                const u32x4 sr = *reinterpret_cast<const u32x4 *>(vs_lds + wave * IT_TOKENS + tk);
                const u32x4 zr = *reinterpret_cast<const u32x4 *>(vz_lds + wave * IT_TOKENS + tk);
                const uint32_t sw[4] = {sr.x, sr.y, sr.z, sr.w}, zw[4] = {zr.x, zr.y, zr.z, zr.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    zacc[t] += pv[e] * half_bits_to_float(zw[e >> 1] >> (16 * (e & 1)));
                    pv[e] *= half_bits_to_float(sw[e >> 1] >> (16 * (e & 1)));
                }
            }
            if constexpr (PACKED) {
                // hi lanes (n < 8) keep x and let the conversion truncate it to its hi part;
                // lo lanes subtract the hi part first.
                const uint32_t lo_mask = (n >= 8) ? 0xffffe000u : 0u;
                uint32_t o[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float x0 = pv[e] - __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, pv[e]) & lo_mask);
                    const float x1 =
                        pv[e + 1] - __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, pv[e + 1]) & lo_mask);
                    // round toward zero: exact truncation to the hi part in hi lanes
                    o[e / 2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x0, x1));
                }
                phi = as_half8(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    _Float16 h, lw;
                    split_hi_lo(pv[e], h, lw);
                    phi[e] = h;
                    plo[e] = lw;
                }
            }
        };
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            // Rescale what was summed so far.  Accumulator rows (C layout) are 4j..4j+3.
            if (round > 0) {
                const int arow = PACKED ? ((4 * j) & 7) : 16 * t + 4 * j;
                const floatx4 al = *reinterpret_cast<const floatx4 *>(alpha_lds + arow);
#pragma unroll
                for (int e = 0; e < 4; e++) acc[t][e] *= al;
                zacc[t] *= alpha_lds[PACKED ? (n & 7) : 16 * t + n];
            }
            if constexpr (PACKED) {
                half8 phi[KSTEPS], plo[KSTEPS];
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ks++) {
                    if (uint32_t(ks) < ksteps) build_p(t, ks, phi[ks], plo[ks]);
                }
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ks++) {
                    if (uint32_t(ks) >= ksteps) break;
                    if constexpr (BITS == 16) {
                        // Rows past the context may hold anything, NaN included: 0 * NaN must not reach O.
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            if (base + 32 * ks + 8 * j + e >= max_len) vreg[ks].w[e] = 0, vreg[ks].w[8 + e] = 0;
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const half8 vop = val_operand<BITS>(vreg[ks], e, n);
                        acc[t][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(phi[ks], vop, acc[t][e], 0, 0, 0);
                        if constexpr (!PACKED) {
                            acc[t][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(plo[ks], vop, acc[t][e], 0, 0, 0);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ks++) {
                    if (uint32_t(ks) >= ksteps) break;
                    half8 phi, plo;
                    build_p(t, ks, phi, plo);
                    if constexpr (BITS == 16) {
                        if (t == 0) {
#pragma unroll
                            for (int e = 0; e < 8; e++) {
                                if (base + 32 * ks + 8 * j + e >= max_len) vreg[ks].w[e] = 0, vreg[ks].w[8 + e] = 0;
                            }
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const half8 vop = val_operand<BITS>(vreg[ks], e, n);
                        acc[t][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(phi, vop, acc[t][e], 0, 0, 0);
                        acc[t][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(plo, vop, acc[t][e], 0, 0, 0);
                    }
                }
            }
        }
        if (it + 1 < n_it) load_values(it + 1);
    }

    // ---- epilogue: one partial per (row, head) ------------------------------------
    // m and l from the phase B threads.
    l_part = group_reduce<Sh::TPR>(l_part, SumOp());
    if (b_part == 0 && (PACKED || b_row < int(real_rows))) {
        const int vrow = PACKED ? 0 : b_row >> 3, head = b_row & 7;
        const size_t slot = (size_t(vrow) * a.nsplits + split) * a.heads + kv * 8 + head;
        *reinterpret_cast<floatx2 *>(a.part_ml + 2 * slot) = floatx2{m_run, l_part};
    }
    // Bias sums: reduce over the 4 lane groups, hand to the C-layout lanes through LDS.
    if constexpr (QUANT) {
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            float z = zacc[t];
            z = across_rows<16, 64>(z, SumOp());
            // One copy per wave: the sum of wave w's group lives at [w][row].
            if (j == 0 && (!PACKED || n < 8)) zsum_lds[wave * Sh::S_ROWS + 16 * t + n] = z;
        }
        // written and read by lanes of the same wave: no workgroup barrier
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    constexpr float unscale = code_up<BITS>() / P_UP;
#pragma unroll
    for (int t = 0; t < TILES; t++) {
        floatx4 o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            o[e] = acc[t][e];
            if constexpr (PACKED) {
                // rows 8-15 hold the lo part of rows 0-7: lanes j and j + 2.
#pragma unroll
                for (int i = 0; i < 4; i++) o[e][i] = across_rows<32, 64>(o[e][i], SumOp());
            }
        }
        if (PACKED && j >= 2) continue;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pair = 16 * t + 4 * j + i;  // (row, head) pair of this accumulator row
            if (pair >= int(real_rows)) continue;
            const int vrow = pair >> 3, head = pair & 7;
            const float zb = QUANT ? zsum_lds[wave * Sh::S_ROWS + pair] * (1.0f / P_UP) : 0.0f;
            const size_t slot = (size_t(vrow) * a.nsplits + split) * a.heads + kv * 8 + head;
            float *dst = a.part_o + slot * DIM + 64 * wave;
            if constexpr (BITS == 16) {
                // tile e: dims 32*(e/2) + 2n + e%2
                *reinterpret_cast<float2 *>(dst + 2 * n) = make_float2(o[0][i] * unscale, o[1][i] * unscale);
                *reinterpret_cast<float2 *>(dst + 32 + 2 * n) = make_float2(o[2][i] * unscale, o[3][i] * unscale);
            } else {
                *reinterpret_cast<float4 *>(dst + 4 * n) =
                    make_float4(o[0][i] * unscale + zb, o[1][i] * unscale + zb, o[2][i] * unscale + zb,
                                o[3][i] * unscale + zb);
            }
        }
    }
}

// One query row over codes (a single packed tile) fits two waves per SIMD, i.e. two workgroups
// per CU (attention_partial_kernel_1, for long contexts); the others take the whole register file
// and run one workgroup per CU.  Which one runs is decided in run_attention.
// Blocks per iteration of each kernel.
constexpr int ITB_TWO_PER_CU = 12, ITB_ONE_PER_CU = 8;
template <int TILES>
constexpr int itb_rows() {
    return TILES == 1 ? 8 : 12;
}

template <int BITS>
__global__ __launch_bounds__(THREADS, 2) void attention_partial_kernel_1(PartialArgs a) {
    attention_partial_body<BITS, 1, true, ITB_TWO_PER_CU, false>(a);
}

template <int BITS, int TILES>
__global__ __launch_bounds__(THREADS) void attention_partial_kernel_n(PartialArgs a) {
    attention_partial_body<BITS, TILES, false, itb_rows<TILES>(), TILES == 1>(a);
}

template <int BITS>
__global__ __launch_bounds__(THREADS) void attention_partial_kernel_p(PartialArgs a) {
    attention_partial_body<BITS, 1, true, ITB_ONE_PER_CU, true>(a);
}

// What a wave of attention_partial_kernel_s does when a bounded wait on an LDS counter has run out (it never
// should): one lane stores a code in the device's sticky status word, which the host reads at its next call
// (a plain vector store to pinned host memory), and the workgroup's partials get l = NaN, so that the
// reduce stage gives NaN for these (row, head) pairs and never a plausible number.  (If the wave that stores
// the maxima and sums is still to come and has not given up itself, its store wins; the status word stands.)
__device__ __noinline__ void wait_gave_up(uint32_t *status, float *part_ml, uint32_t code, uint32_t rows, uint32_t nsplits,
                                          uint32_t split, uint32_t heads, uint32_t kv) {
    const uint32_t lane = threadIdx.x & 63;
    if (lane == 0) __hip_atomic_store(status, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (lane < 8 * rows) {
        const size_t slot = (size_t(lane >> 3) * nsplits + split) * heads + kv * 8 + (lane & 7);
        part_ml[2 * slot + 1] = __builtin_nanf("");
    }
}

// ---- one to four query rows over codes, keys first ------------------------------------------------
// attention_partial_kernel_s: the workgroup's share is taken in rounds of up to 17 blocks of 16
// tokens whose codes all lie in LDS at once (17: a context of 128 x 256 tokens and a few more still
// is one round).  The KEYS of a round are requested before its values, so they are there when half
// of the round's bytes are, and everything that does not need a value code runs while the values
// are still on their way: the scores of all the tokens, their softmax (every block relative to its
// own maximum, by the wave that computed its scores; the blocks are joined by one factor per block
// and head), and the probability operands P * value scale.  When the last values land, what is left
// is one k-step of O += P V per wave (8 LDS reads, 16 byte permutes, 4 MFMAs), the merge of two
// waves and the store.
// Eight computing waves and four loader waves that move codes from global memory straight into LDS
// (global_load_lds, no registers): two request the round's scales, biases and keys, and two, once
// those requests are out, the values.  A loader waits for its own loads in order and raises a
// counter in LDS when a part of the keys, or a 64-token slot of the values, has landed.  In phase A
// computing wave w takes the blocks w and w + 8 (wave 0 also block 16); in phase C waves 2g and
// 2g + 1 share quantization group g (dims 64g .. 64g + 63) and take alternate k-steps of 32 tokens,
// so that each of the round's value slots gives every wave one k-step.
// A wave that requests more than the memory pipeline takes stands still until it is accepted, so a
// wave that requests values cannot tell anybody that earlier data is there: that is why the keys and
// the values have different requesters, and why the waves meet through counters in LDS and not
// through s_barrier (which would wait for the loaders to finish requesting).  LDS executes a wave's
// instructions in order, so data written before a counter is raised is there when the counter is
// seen.  Every wait on a counter is bounded (SPIN_LIMIT polls), so every wave ends whatever happens.
// Longer shares take further rounds with an online softmax between the rounds.
// M query rows (a verify step, 2..4) take one round over codes that serve every row; two rows share a
// tile (see the rows' part of the kernel).
template <int BITS, int M>
struct KeysFirst {
    static constexpr int PAIRS = (M + 1) / 2;               // tiles of two query rows (one row: its own tile)
    static constexpr int LOADERS = 4, WAVES = 8;            // loader waves (keys: 0, 1; values: 2, 3), then the computing waves
    static constexpr int K_LOADERS = 2, V_LOADERS = 2;
    static constexpr int RB_ = BITS * 32;                   // bytes of a (token, kv head) row of codes
    static constexpr int ROUND_BLOCKS = 17, ROUND_TOKENS = ROUND_BLOCKS * BLOCK;
    // One row, a share of more than one round: rounds of ALT_BLOCKS blocks that ALTERNATE between two halves of the
    // keys' and the values' places (and of the scales and the block table), so that the loaders are a round ahead of
    // the computing waves and the stream from memory never waits for them.  The halves are the blocks 0-7 and 8-15 of
    // the single round's places.  (Rounds of 16 blocks for 4-bit codes, which are half the bytes, in places of 32
    // blocks: measured slower, 30.0 against 28.3 us at 150k tokens; the code below takes either.)
    static constexpr bool ALTERNATE = M == 1;
    static constexpr int ALT_BLOCKS = 8;
    static constexpr int AREA_BLOCKS = (ALTERNATE && 2 * ALT_BLOCKS > ROUND_BLOCKS) ? 2 * ALT_BLOCKS : ROUND_BLOCKS;  // blocks of codes LDS has room for, keys and values each
    static constexpr int SB_TOKENS = AREA_BLOCKS * BLOCK;
    static constexpr int KSTEPS = (ROUND_BLOCKS + 1) / 2;   // of 32 tokens; the last one is half there
    static constexpr int SLOTS = (KSTEPS + 1) / 2;          // value slots of 64 tokens: 5, the last one block 16 alone
    static constexpr int PIECES = RB_ / 16;
    static constexpr int PER_BLOCK = PIECES / 4;            // load instructions per block of keys, and of values: 4 | 2
    static constexpr int V_GROUP_TOKENS = 64 / PIECES;      // token rows one load instruction brings: 4 | 8
    static constexpr int K_BLOCK_BYTES = BLOCK * RB_;       // [64-byte piece][token]: what one load instruction brings
    // Values: whole token rows, each rotated by a quarter row per 8 tokens ((token / 8) % 4 quarters),
    // so that the four lane groups of a value read, which are 8 tokens apart, fall on different banks.
    static constexpr int V_ROT = RB_ / 4;
    static constexpr int K_LOADS = 8 * PER_BLOCK;           // per key-loader wave: blocks 0-15, half of them before the other
    static constexpr int V_LOADS = 8 * PER_BLOCK;           // per value-loader wave: slots 0-3
    static constexpr int SC_LOADS = 16;                     // scales and biases of a key loader's 128 tokens: 4 arrays x 2 planes x 2
    static constexpr int X_LOADS = 8 + PER_BLOCK;           // block 16: its scales and biases (4 arrays x 2 planes) and its keys
    static_assert(SC_LOADS + K_LOADS + X_LOADS < 64, "vmcnt is 6 bits");
    // LDS map, in bytes.  The scores of a block (its probabilities relative to the block's maximum,
    // [row][head][token] f32, 512 bytes a row) lie over the block's own keys, which only the wave that
    // writes them has read.
    static constexpr int Q_OFF = 0;                                // [k-step][lane] half8: one row's operands at a time
    static constexpr int QZ_OFF = Q_OFF + 8 * 64 * 16;             // [hi, lo][lane][k-step] f16
    // scales and biases: per array two planes of one dword per token, the f16 of groups (0, 1) and of (2, 3)
    static constexpr int SB_OFF = QZ_OFF + 2 * 64 * 16;            // [ks | kz | vs | vz][plane][token] u32
    static constexpr int SB_ARRAY = 2 * SB_TOKENS * 4;
    // the blocks' maxima and sums, [row][head][block]: one row has room for a stride of 20 (16-byte reads; blocks 17-19
    // never exist: maximum "none", sum 0), several rows have not
    static constexpr int BSTRIDE = M == 1 ? (AREA_BLOCKS + 3) / 4 * 4 : ROUND_BLOCKS;
    static constexpr int BSINGLE = (ROUND_BLOCKS + 3) / 4 * 4;      // entries of a row that a single round looks at (one row)
    static constexpr int BROW = 8 * BSTRIDE;                       // floats of a row's table
    static constexpr int BMAX_OFF = SB_OFF + 4 * SB_ARRAY;         // [row][head][block] f32: the block's maximum score
    static constexpr int BSUM_OFF = BMAX_OFF + M * BROW * 4;       // [row][head][block] f32: sum of 2^(score - maximum)
    static constexpr int ZS_OFF = BSUM_OFF + M * BROW * 4;         // [wave][pair][column] f32 (one row: [wave][head])
    static constexpr int SYNC_OFF = ZS_OFF + WAVES * PAIRS * 16 * 4;  // 32 counters, u32
    static constexpr int K_OFF = (SYNC_OFF + 32 * 4 + 255) / 256 * 256;
    static constexpr int V_OFF = K_OFF + AREA_BLOCKS * K_BLOCK_BYTES;
    // Several rows over a share of more than one round: rounds of SHORT_BLOCKS blocks, which leave room in
    // LDS for every pair's query operands to stay ([pair][hi, lo][k-step][lane] half8, then [pair][hi, lo][lane][k-step]
    // f16 of the key bias term), so that they need no registers between one round's scores and the next's.
    // 8-bit codes: over the keys' blocks that short rounds never fill; 4-bit: behind the values.
    static constexpr int SHORT_BLOCKS = 8;
    static constexpr int QP_PAIR_BYTES = 2 * 8 * 64 * 16, QPZ_PAIR_BYTES = 2 * 64 * 16;
    static constexpr int QP_BYTES = M > 1 ? PAIRS * (QP_PAIR_BYTES + QPZ_PAIR_BYTES) : 0;
    static constexpr int QP_OFF = BITS == 8 ? K_OFF + SHORT_BLOCKS * K_BLOCK_BYTES : V_OFF + AREA_BLOCKS * K_BLOCK_BYTES;
    static constexpr int QPZ_OFF = QP_OFF + PAIRS * QP_PAIR_BYTES;
    static_assert(BITS != 8 || QP_OFF + QP_BYTES <= V_OFF, "the query operands fit behind the short rounds' keys");
    static constexpr int LDS_BYTES = (BITS == 8 || M == 1) ? V_OFF + AREA_BLOCKS * K_BLOCK_BYTES : QP_OFF + QP_BYTES;
    // one row: the merge of two waves, [group][lane < 32][4 rows] of 16 bytes, lies over the query operands,
    // which nobody reads after the last scores
    static constexpr int X_OFF = Q_OFF;
    static_assert(LDS_BYTES <= 160 * 1024, "LDS of a CU");
    static_assert(M * 512 <= K_BLOCK_BYTES, "the scores fit over the keys");
    static_assert(4 * 32 * 64 <= QZ_OFF - Q_OFF, "the merge fits over the query operands");
    // the counters
    static constexpr int C_KEYS = 0;    // key loaders that have requested the first round's keys
    static constexpr int C_QUERY = 1;   // computing waves that have written a row's query operands (8 per row)
    static constexpr int C_SCORES = 2;  // ... written their scores (8 per round)
    static constexpr int C_BUILT = 3;   // ... built their probability operands (8 per round)
    static constexpr int C_DONE = 4;    // ... are through with the round's values (8 per round)
    static constexpr int C_LENGTH = 5;  // (not a counter: the context length or the position, for every wave)
    static constexpr int C_VREQ = 6;    // alternating rounds: value loaders that have requested a round's values (2 per round)
    static constexpr int C_QREAD = 7;   // computing waves that have a row's query operands in registers (several rows)
    static constexpr int C_KPART = 8;   // [3]: key loaders whose blocks 0-7 and scales | blocks 8-15 | block 16 have landed (2 per round)
    static constexpr int C_SLOT = 12;   // [5]: value loaders whose values of slot s have landed (2 per round)
    static constexpr int C_MERGE = 20;  // [4]: one row: wave 2g + 1 has written its sums for wave 2g | two pairs of rows: blocks
                                        // whose keys the two waves of scores w % 4 have in registers; then [4] as with one row
    static constexpr uint32_t SPIN_LIMIT = 1u << 20;
};

template <int BITS, int M>
__global__ __launch_bounds__((KeysFirst<BITS, M>::LOADERS + KeysFirst<BITS, M>::WAVES) * 64) void attention_partial_kernel_s(PartialArgs a) {
    using W = KeysFirst<BITS, M>;
    constexpr int RB = W::RB_, RT = W::SB_TOKENS, RBK = W::ROUND_BLOCKS;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int lane = threadIdx.x & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6);
    const int n = lane & 15, j = lane >> 4;
    const uint32_t split = blockIdx.x, kv = blockIdx.y, kvh = a.kv_heads;
    const bool loader = wave_all < W::LOADERS;
    const int wave = wave_all - W::LOADERS;          // computing waves: 0..7
    uint32_t *sync_lds = reinterpret_cast<uint32_t *>(lds_raw + W::SYNC_OFF);
    const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(lds_raw));

    // ---- query values: requested first (computing waves: thread = (k-step, lane) item of every row) ----
    auto load_query = [&](int r, float (&v)[8]) {
        const int step = wave, g = step >> 1, ab = step & 1;
        const float *src = a.q + (size_t(r) * a.heads + kv * 8 + (n & 7)) * DIM + 64 * g + 16 * j + 8 * ab;
        const float4 f0 = *reinterpret_cast<const float4 *>(src);
        const float4 f1 = *reinterpret_cast<const float4 *>(src + 4);
        v[0] = f0.x, v[1] = f0.y, v[2] = f0.z, v[3] = f0.w, v[4] = f1.x, v[5] = f1.y, v[6] = f1.z, v[7] = f1.w;
    };
    // (several rows: per pair of rows, the row that the lane's column of the pair's tile belongs to.  The
    // loader waves leave the registers as they are: a value set for them would have to be merged with the
    // loaded one, and that copy would wait for the load in front of the barrier, where the loader waves
    // stand until every wave has arrived.)
    float qv[W::PAIRS][8];
    if (!loader) {
#pragma unroll
        for (int p = 0; p < W::PAIRS; p++) load_query(M == 1 ? 0 : min(2 * p + (n >> 3), M - 1), qv[p]);
    }

    // ---- the context and this workgroup's share of it -----------------------------
    // One wave of the workgroup reads the token's parameters and hands them on through LDS.  The
    // counters start at zero behind the same barrier, the only s_barrier of the kernel, before
    // anybody requests anything of the cache.
    // (the context length of a decode step | the position of the first of a verify step's rows: one scalar load)
    static_assert(offsetof(saetta_token_params, position) == 4 && offsetof(saetta_token_params, kv_len) == 8, "dwords 1 and 2");
    if (threadIdx.x < 32) sync_lds[threadIdx.x] = threadIdx.x == W::C_LENGTH ? reinterpret_cast<const uint32_t *>(a.tp)[a.decode_len ? 2 : 1] : 0u;
    __syncthreads();
    const uint32_t tp_first = __builtin_amdgcn_readfirstlane(sync_lds[W::C_LENGTH]);
    // tokens row r sees; the last row's are the launch's
    auto len_of = [&](int r) -> uint32_t { return min<uint32_t>(a.decode_len ? tp_first : tp_first + uint32_t(r) + 1, a.capacity); };
    const uint32_t max_len = len_of(M - 1);
    const uint32_t nblocks = (max_len + BLOCK - 1) / BLOCK;
    uint32_t blk_begin, blk_end;
    if (nblocks <= a.nsplits) {
        blk_begin = split;
        blk_end = split + 1;
        if (split >= nblocks) return;
    } else {
        blk_begin = split * nblocks / a.nsplits;
        blk_end = (split + 1) * nblocks / a.nsplits;
    }
    const uint32_t limit = min(max_len, blk_end * BLOCK);  // tokens of this share end here
    const uint32_t last_tok = limit - 1;                   // rows past it are never read: loads are clamped to it
    const uint32_t range = blk_end - blk_begin;
    // rounds of equal size (to within a block), none longer than 17 blocks
    // (several rows: one round of up to 17 blocks, or rounds of up to 8)
    constexpr uint32_t LONG_ROUND = W::ALTERNATE ? W::ALT_BLOCKS : W::SHORT_BLOCKS;
    const uint32_t n_rounds = range > uint32_t(RBK) ? (range + LONG_ROUND - 1) / LONG_ROUND : 1;
    const bool alt = W::ALTERNATE && n_rounds > 1;  // rounds in alternate halves of LDS
    const uint32_t per_round = (range + n_rounds - 1) / n_rounds;
    auto blocks_of = [&](uint32_t round) { return min(range - round * per_round, per_round); };

    auto dma = [&](uint32_t lds_addr, uint32_t voff, const void *src) {
        asm volatile("s_mov_b32 m0, %0\n"
                     "s_nop 0\n"
                     "global_load_lds_dwordx4 %1, %2\n"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(src)
                     : "memory", "m0");
    };
    auto dma4 = [&](uint32_t lds_addr, uint32_t voff, const void *src) {
        asm volatile("s_mov_b32 m0, %0\n"
                     "s_nop 0\n"
                     "global_load_lds_dword %1, %2\n"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(src)
                     : "memory", "m0");
    };
    // counters: raised by one lane after the wave's LDS writes (LDS takes a wave's instructions in
    // order); a waiting wave polls, a bounded number of times
    auto raise = [&](int c) {
        asm volatile("" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(sync_lds + c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        asm volatile("" ::: "memory");
    };
    auto peek = [&](int c) {
        asm volatile("" ::: "memory");
        const uint32_t v = __hip_atomic_load(sync_lds + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        asm volatile("" ::: "memory");
        return uint32_t(__builtin_amdgcn_readfirstlane(v));
    };
    // A wait that runs out must not pass for a result: the wave notes which counter it was, goes on to its
    // end like any wave, and there (`leave`) leaves a code in the device's status word and l = NaN in the
    // workgroup's partials (wait_gave_up, out of line: it never runs); the wave that stores the maxima and
    // sums writes l = NaN itself if it has given up.  (The polling loop is kept rolled up: there are some
    // twenty waits in the kernel, and its code has to come through the instruction cache at every launch.)
    uint32_t lost = 0;
    auto await = [&](int c, uint32_t want) {
        asm volatile("" ::: "memory");
        uint32_t left = W::SPIN_LIMIT;
#pragma nounroll
        do {
            const uint32_t v = __hip_atomic_load(sync_lds + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (__builtin_amdgcn_readfirstlane(v) >= want) break;
            __builtin_amdgcn_s_sleep(1);
        } while (--left);
        if (__builtin_expect(left == 0, 0)) lost = 0x100u + uint32_t(c);
        asm volatile("" ::: "memory");
    };
    auto leave = [&]() {
        if (__builtin_expect(lost != 0, 0)) wait_gave_up(a.status, a.part_ml, lost, M, a.nsplits, split, a.heads, kv);
    };
    // l of a partial as the writer of the maxima and sums stores it
    auto marked = [&](float l) { return lost ? __builtin_nanf("") : l; };

    if (loader && wave_all < W::K_LOADERS) {
        // ---- a key-loader wave: scales and biases of tokens 128 L .. 128 L + 127, keys of blocks L, L + 2, ...;
        // loader 0 then block 16 with its scales and biases ----
        const uint32_t L = uint32_t(wave_all);
        const void *sb_src[4] = {a.kscales, a.kbiases, a.vscales, a.vbiases};
        if constexpr (W::ALTERNATE) if (alt) {
            // ---- rounds of up to 8 blocks in alternate halves of LDS: loader L takes the rounds L, L + 2, ... whole, so
            // that two rounds' keys can be on their way at once.  A round goes out when the values of the round before
            // have been requested (the stream keeps the order keys, values, keys, ...) and when the round before last,
            // which lay in the same half, has been used up: its scales are read until every wave has built its operands,
            // its keys until every wave has its scores. ----
            for (uint32_t round = L; round < n_rounds; round += 2) {
                const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
                const uint32_t half = L * W::ALT_BLOCKS;  // the blocks of LDS this round goes to start here
                if (round > 1) await(W::C_BUILT, W::WAVES * (round - 1));
                if (round > 0) await(W::C_VREQ, round);
#pragma unroll
                for (int h = 0; h < W::ALT_BLOCKS / 4; h++) {
                    const uint32_t voff = (min(base + 64 * h + lane, last_tok) * kvh + kv) * 8;
#pragma unroll
                    for (int arr = 0; arr < 4; arr++) {
#pragma unroll
                        for (int pl = 0; pl < 2; pl++) dma4(lds0 + W::SB_OFF + arr * W::SB_ARRAY + (pl * RT + BLOCK * half + 64 * h) * 4, voff + 4 * pl, sb_src[arr]);
                    }
                }
#pragma unroll
                for (int r = 0; r < W::ALT_BLOCKS; r++) {
                    if (uint32_t(r) < nb) {
                        const uint32_t tok = min(base + BLOCK * r + (lane >> 2), last_tok);
                        const uint32_t voff = (tok * kvh + kv) * RB + (lane & 3) * 16;
#pragma unroll
                        for (int i = 0; i < W::PER_BLOCK; i++) dma(lds0 + W::K_OFF + (half + r) * W::K_BLOCK_BYTES + i * 1024, voff + 64 * i, a.kdata);
                    }
                }
                raise(W::C_KEYS);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                raise(W::C_KPART + 0);
            }
            leave();
            return;
        }
        // (one row: more than one round is taken above)
        for (uint32_t round = 0; round < (M == 1 ? 1u : n_rounds); round++) {
            const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
            // the round before: its scales are read until every wave has built its operands, its keys until every wave has its scores
            if (round > 0) await(W::C_BUILT, W::WAVES * round);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                // a dword per lane and load: the token's four f16 of an array go to two planes
                const uint32_t voff = (min(base + 128 * L + 64 * h + lane, last_tok) * kvh + kv) * 8;
#pragma unroll
                for (int arr = 0; arr < 4; arr++) {
#pragma unroll
                    for (int pl = 0; pl < 2; pl++) dma4(lds0 + W::SB_OFF + arr * W::SB_ARRAY + (pl * RT + 128 * L + 64 * h) * 4, voff + 4 * pl, sb_src[arr]);
                }
            }
            auto request_block = [&](uint32_t blk) {
                // lane -> (token lane / 4, 16 bytes lane % 4 of the token's 64-byte piece i): four
                // neighbouring lanes read 64 contiguous bytes
                const uint32_t tok = min(base + BLOCK * blk + (lane >> 2), last_tok);
                const uint32_t voff = (tok * kvh + kv) * RB + (lane & 3) * 16;
#pragma unroll
                for (int i = 0; i < W::PER_BLOCK; i++) dma(lds0 + W::K_OFF + blk * W::K_BLOCK_BYTES + i * 1024, voff + 64 * i, a.kdata);
            };
#pragma unroll
            for (int r = 0; r < 8; r++) {
                if (L + 2 * r < nb) request_block(L + 2 * r);
            }
            const bool extra = nb == uint32_t(RBK) && L == 0;
            if (extra) {
                if (lane < BLOCK) {
                    const uint32_t voff = (min(base + 256 + lane, last_tok) * kvh + kv) * 8;
#pragma unroll
                    for (int arr = 0; arr < 4; arr++) {
#pragma unroll
                        for (int pl = 0; pl < 2; pl++) dma4(lds0 + W::SB_OFF + arr * W::SB_ARRAY + (pl * RT + 256) * 4, voff + 4 * pl, sb_src[arr]);
                    }
                }
                request_block(16);
            }
            if (round == 0) raise(W::C_KEYS);
            // loads return in order (a round of less than 16 blocks: all at once)
            if (extra) {
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::K_LOADS / 2 + W::X_LOADS));
                raise(W::C_KPART + 0);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::X_LOADS));
                raise(W::C_KPART + 1);
            } else if (nb >= 16) {
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::K_LOADS / 2));
                raise(W::C_KPART + 0);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                raise(W::C_KPART + 1);
            } else {
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                raise(W::C_KPART + 0);
                raise(W::C_KPART + 1);
            }
            __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
            raise(W::C_KPART + 2);
        }
        leave();
        return;
    }
    if (loader) {
        // ---- a value-loader wave: blocks L, L + 2, ... of every round, two of them in each 64-token slot;
        // loader 0 then block 16 (slot 4) ----
        const uint32_t L = uint32_t(wave_all) - W::K_LOADERS;
        if constexpr (W::ALTERNATE) if (alt) {
            // ---- alternate halves: loader L takes the values of the rounds L, L + 2, ... whole, each behind its round's
            // keys in the stream, into the half that the round before last has left (every wave through with its values) ----
            for (uint32_t round = L; round < n_rounds; round += 2) {
                const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
                const uint32_t half = L * W::ALT_BLOCKS;
                await(W::C_KEYS, round + 1);
                if (round > 1) await(W::C_DONE, W::WAVES * (round - 1));
#pragma unroll
                for (int r = 0; r < W::ALT_BLOCKS; r++) {
                    if (uint32_t(r) < nb) {
#pragma unroll
                        for (int i = 0; i < W::PER_BLOCK; i++) {
                            const uint32_t t = BLOCK * r + W::V_GROUP_TOKENS * i + lane / W::PIECES;  // token of the round
                            const uint32_t piece = (lane % W::PIECES + W::PIECES - ((t >> 3) & 3) * (W::PIECES / 4)) % W::PIECES;
                            dma(lds0 + W::V_OFF + (W::PER_BLOCK * (half + r) + i) * 1024, (min(base + t, last_tok) * kvh + kv) * RB + piece * 16, a.vdata);
                        }
                    }
                }
                raise(W::C_VREQ);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                raise(W::C_SLOT + 4);
            }
            leave();
            return;
        }
        for (uint32_t round = 0; round < (M == 1 ? 1u : n_rounds); round++) {
            const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
            // the keys of the first round have been requested | every wave is through with the values before
            if (round == 0) {
                await(W::C_KEYS, W::K_LOADERS);
            } else {
                await(W::C_DONE, W::WAVES * round);
            }
            auto request_block = [&](uint32_t blk) {
#pragma unroll
                for (int i = 0; i < W::PER_BLOCK; i++) {
                    // lane -> (token lane / PIECES of the instruction's group, the piece that goes to place lane % PIECES
                    // of the row, which is rotated by (token / 8) % 4 quarters: the same for the group's tokens)
                    const uint32_t t = BLOCK * blk + W::V_GROUP_TOKENS * i + lane / W::PIECES;  // token of the round
                    const uint32_t piece = (lane % W::PIECES + W::PIECES - ((t >> 3) & 3) * (W::PIECES / 4)) % W::PIECES;
                    dma(lds0 + W::V_OFF + (W::PER_BLOCK * blk + i) * 1024, (min(base + t, last_tok) * kvh + kv) * RB + piece * 16, a.vdata);
                }
            };
#pragma unroll
            for (int r = 0; r < 8; r++) {
                if (L + 2 * r < nb) request_block(L + 2 * r);
            }
            const bool extra = nb == uint32_t(RBK) && L == 0;
            if (extra) request_block(16);
            // loads return in order (a round of less than 16 blocks: all at once)
            if (extra) {
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::V_LOADS * 3 / 4 + W::PER_BLOCK));
                raise(W::C_SLOT + 0);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::V_LOADS * 2 / 4 + W::PER_BLOCK));
                raise(W::C_SLOT + 1);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::V_LOADS * 1 / 4 + W::PER_BLOCK));
                raise(W::C_SLOT + 2);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::PER_BLOCK));
                raise(W::C_SLOT + 3);
            } else if (nb >= 16) {
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::V_LOADS * 3 / 4));
                raise(W::C_SLOT + 0);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::V_LOADS * 2 / 4));
                raise(W::C_SLOT + 1);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(W::V_LOADS * 1 / 4));
                raise(W::C_SLOT + 2);
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                raise(W::C_SLOT + 3);
            } else {
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                raise(W::C_SLOT + 0);
                raise(W::C_SLOT + 1);
                raise(W::C_SLOT + 2);
                raise(W::C_SLOT + 3);
            }
            __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
            raise(W::C_SLOT + 4);
        }
        leave();
        return;
    }

    // ---- computing waves ------------------------------------------------------------------------
    half8 *q_lds = reinterpret_cast<half8 *>(lds_raw + W::Q_OFF);
    _Float16 *qz_lds = reinterpret_cast<_Float16 *>(lds_raw + W::QZ_OFF);
    const uint32_t *sb_lds = reinterpret_cast<const uint32_t *>(lds_raw + W::SB_OFF);
    float *bmax_lds = reinterpret_cast<float *>(lds_raw + W::BMAX_OFF);
    float *bsum_lds = reinterpret_cast<float *>(lds_raw + W::BSUM_OFF);
    float *zs_lds = reinterpret_cast<float *>(lds_raw + W::ZS_OFF);
    // the scores of block b, row r: [head][token] f32 over the block's keys
    auto s_block = [&](int b, int r) { return reinterpret_cast<float *>(lds_raw + W::K_OFF + b * W::K_BLOCK_BYTES + r * 512); };

    // the value codes of k-step ks for group g: the lane's dword of tokens 32 ks + 8j .. + 7
    auto read_values = [&](int ks, int g, ValRegs<BITS> &vreg) {
        const int jj = ks == 8 ? (j & 1) : j;
        // (tokens 8 jj .. 8 jj + 7 of a k-step: their rows are rotated by jj quarters)
        const unsigned char *vb = lds_raw + W::V_OFF + 8 * jj * RB + ((val_lane_offset<BITS>(g, n) + jj * W::V_ROT) & (RB - 1));
#pragma unroll
        for (int e = 0; e < 8; e++) vreg.w[e] = *reinterpret_cast<const uint32_t *>(vb + (32 * ks + e) * RB);
    };
    // a row's maximum per head over the round's blocks
    auto round_max = [&](int r, float start) {
        const float *bmx = bmax_lds + r * W::BROW + (n & 7) * W::BSTRIDE;
        float v = start;
        if constexpr (M == 1) {
#pragma unroll
            for (int i = 0; i < W::BSINGLE / 4; i++) {
                const floatx4 w = reinterpret_cast<const floatx4 *>(bmx)[i];
                v = fmaxf(v, fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3])));
            }
        } else {
#pragma unroll
            for (int i = 0; i < RBK; i++) v = fmaxf(v, bmx[i]);
        }
        return v;
    };
    // a row's sum of P of head n & 7 over the round's blocks, relative to the maximum nm: lane group j adds blocks j, j + 4, ...
    auto round_sum = [&](int r, float nm) {
        float sum = 0.0f;
        if constexpr (M == 1) {
            // lane group j adds blocks 5j .. 5j + 4
#pragma unroll
            for (int i = 0; i < W::BSINGLE / 4; i++) {
                const int b = (W::BSINGLE / 4) * j + i;
                sum += bsum_lds[r * W::BROW + (n & 7) * W::BSTRIDE + b] * __builtin_amdgcn_exp2f(bmax_lds[r * W::BROW + (n & 7) * W::BSTRIDE + b] - nm);
            }
            return across_rows<16, 64>(sum, SumOp());
        }
#pragma unroll
        for (int i = 0; i < (RBK + 3) / 4; i++) {
            const int b = j + 4 * i;
            if (b < RBK) sum += bsum_lds[r * W::BROW + (n & 7) * W::BSTRIDE + b] * __builtin_amdgcn_exp2f(bmax_lds[r * W::BROW + (n & 7) * W::BSTRIDE + b] - nm);  // (a block that is not there: sum 0)
        }
        return across_rows<16, 64>(sum, SumOp());
    };
    constexpr float unscale = code_up<BITS>() / P_UP;
    const int g = wave >> 1, b2 = wave & 1;  // O += P V: the wave's group and which k-steps of a slot

    if constexpr (M > 1) {
        // ---- several rows ------------------------------------------------------------------------
        // Two rows share a tile: its 16 columns are (row of the pair, head), and the hi and the lo parts of
        // an operand go through two MFMAs into one accumulator, so that every lane of a result holds a
        // whole score (or output) of its own column.  Three rows: the second pair's upper columns repeat
        // row 2 and are not written out.
        // Scores: with one pair every wave takes its blocks (wave, wave + 8; wave 0 also 16); with two
        // pairs waves 0-3 take the first and waves 4-7 the second, blocks w % 4 + 4 i.  The pair's query
        // operands stay in registers: they go through the one place in LDS, the hi parts and then the lo
        // parts of a pair, while the first keys are on their way.
        // O += P V: as with one row, waves 2g and 2g + 1 share group g and take alternate k-steps, for
        // every pair, the byte permutes of a value operand serving both pairs.
        constexpr int PAIRS = W::PAIRS, WT = W::WAVES / PAIRS;
        const int at = wave / WT, wt = wave % WT;
        const int col_row = n >> 3;  // the row of the pair that this lane's column belongs to
        auto row_of = [&](int pair, int half) { return min(2 * pair + half, M - 1); };
        if (range > uint32_t(RBK)) {
            // ---- a share of more than one round (a context of more than 17 blocks per split) ----------
            // Rounds of up to SHORT_BLOCKS blocks, in the blocks 0-7 of the keys' and the values' places.  What
            // a round leaves behind, per column: the maximum so far, the sums so far relative to it (O in
            // registers, l with wave 0), both brought to the new maximum before the next round's values are
            // added.  The query operands of every pair wait in LDS (the blocks that short rounds never fill) and
            // are read again for every round's scores, so that they hold no registers while the values are taken.
            constexpr int SB = W::SHORT_BLOCKS, A_SHORT = SB / WT, S_SLOTS = SB / 4;
            half8 *qp_lds = reinterpret_cast<half8 *>(lds_raw + W::QP_OFF);
            _Float16 *qpz_lds = reinterpret_cast<_Float16 *>(lds_raw + W::QPZ_OFF);
            {
                const float qmul = a.scale * 1.4426950408889634f * Q_UP;
#pragma unroll
                for (int pair = 0; pair < PAIRS; pair++) {
                    // this thread's item: k-step `wave`, lane `lane`: column n = (row n / 8 of the pair, head n % 8)
                    half8 hi, lo;
                    float sum = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        _Float16 h, lw;
                        split_hi_lo(qv[pair][key_slot_dim<BITS>(e)] * qmul, h, lw);
                        hi[e] = h, lo[e] = lw;
                        sum += (float)h + (float)lw;
                    }
                    qp_lds[((pair * 2 + 0) * 8 + wave) * 64 + lane] = hi;
                    qp_lds[((pair * 2 + 1) * 8 + wave) * 64 + lane] = lo;
                    _Float16 h, lw;
                    split_hi_lo(sum * (1.0f / Q_UP), h, lw);
                    qpz_lds[((pair * 2 + 0) * 64 + lane) * 8 + wave] = h;
                    qpz_lds[((pair * 2 + 1) * 64 + lane) * 8 + wave] = lw;
                }
                // blocks that a short round never has: maximum "none", sum 0 (the table of this wave's pair, by its first wave)
                if (wt == 0 && j == 0) {
                    const int my_row = row_of(at, col_row);
#pragma unroll
                    for (int b = SB; b < RBK; b++) bmax_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + b] = NO_SCORE, bsum_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + b] = 0.0f;
                }
            }
            raise(W::C_QUERY);

            float m_run[PAIRS], l_run[PAIRS], zacc[PAIRS];
            floatx4 acc[PAIRS][4];  // [pair][tile of 16 dims 4n' + e]: rows 4j .. 4j+3 (columns of the pair), column n'
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
                m_run[p] = NO_SCORE, l_run[p] = 0.0f, zacc[p] = 0.0f;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[p][e] = floatx4{0, 0, 0, 0};
            }
            uint32_t taken = 0;  // blocks whose scores this wave has written (two pairs: the handshake over a block's keys counts them)
            await(W::C_QUERY, W::WAVES);
#pragma unroll 1
            for (uint32_t round = 0; round < n_rounds; round++) {
                const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
                const uint32_t round_limit = min(limit, base + nb * BLOCK);  // tokens of this round end here
                const uint32_t live_blocks = (nb + 1) & ~1u;  // k-steps are two blocks: the blocks of the k-steps that have tokens

                // ---- phase A: the scores of this wave's blocks for its pair of rows ----
                {
                    const int my_row = row_of(at, col_row);
                    const uint32_t my_limit = min<uint32_t>(round_limit, len_of(my_row));
#pragma unroll 1
                    for (int i = 0; i < A_SHORT; i++) {
                        const int blk = wt + WT * i;
                        if (uint32_t(blk) >= live_blocks) {
                            // (no scores to take, and no operands will be made of this block; the table still holds the
                            // round before's entries until every wave has built its operands from them)
                            if (round > 0) await(W::C_BUILT, W::WAVES * round);
                            if (j == 0) bmax_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = NO_SCORE, bsum_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = 0.0f;
                            continue;
                        }
                        await(W::C_KPART + 0, W::K_LOADERS * (round + 1));  // the round's keys and scales are in LDS
                        const unsigned char *kb = lds_raw + W::K_OFF + blk * W::K_BLOCK_BYTES;
                        KeyRegs<BITS> kreg[4];
#pragma unroll
                        for (int gg = 0; gg < 4; gg++) {
                            if constexpr (BITS == 8) {
                                const u32x4 v = *reinterpret_cast<const u32x4 *>(kb + gg * 1024 + n * 64 + j * 16);
                                kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y, kreg[gg].w[2] = v.z, kreg[gg].w[3] = v.w;
                            } else {
                                const u32x2 v = *reinterpret_cast<const u32x2 *>(kb + (gg >> 1) * 1024 + n * 64 + (gg & 1) * 32 + j * 8);
                                kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y;
                            }
                        }
                        const int tok0 = BLOCK * blk + 4 * j;  // this lane's 4 tokens of the round in C layout
                        const uint32_t *sb_w = sb_lds + BLOCK * blk;
                        const u32x2 zr = {sb_w[W::SB_ARRAY / 4 + n], sb_w[W::SB_ARRAY / 4 + RT + n]};
                        const half8 zop = as_half8(perm(0, zr.x, 0x01000100u), perm(0, zr.x, 0x03020302u), perm(0, zr.y, 0x01000100u), perm(0, zr.y, 0x03020302u));
                        const u32x4 s01 = *reinterpret_cast<const u32x4 *>(sb_w + 4 * j);
                        const u32x4 s23 = *reinterpret_cast<const u32x4 *>(sb_w + RT + 4 * j);
                        const uint32_t sw[8] = {s01.x, s23.x, s01.y, s23.y, s01.z, s23.z, s01.w, s23.w};
                        floatx4 sc = {0, 0, 0, 0}, rr[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
                        sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, *reinterpret_cast<const half8 *>(qpz_lds + ((at * 2 + 0) * 64 + lane) * 8), sc, 0, 0, 0);
                        sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, *reinterpret_cast<const half8 *>(qpz_lds + ((at * 2 + 1) * 64 + lane) * 8), sc, 0, 0, 0);
                        // the hi parts of the pair's query operands, then the lo parts: one set in registers at a time
                        // (the accumulators of the rounds so far are held as well), the key operands made once for each
#pragma unroll
                        for (int part = 0; part < 2; part++) {
                            half8 q_part[8];
#pragma unroll
                            for (int k = 0; k < 8; k++) q_part[k] = qp_lds[((at * 2 + part) * 8 + k) * 64 + lane];
#pragma unroll
                            for (int gg = 0; gg < 4; gg++) {
#pragma unroll
                                for (int ab = 0; ab < 2; ab++) {
                                    rr[gg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(key_operand<BITS>(kreg[gg], ab), q_part[gg * 2 + ab], rr[gg], 0, 0, 0);
                                }
                            }
                            asm volatile("" ::: "memory");  // (the lo parts are not to be fetched while the hi parts are held)
                        }
                        constexpr float C1 = code_up<BITS>() / Q_UP;
#pragma unroll
                        for (int tk = 0; tk < 4; tk++) {
                            float d = 0.0f;
#pragma unroll
                            for (int gg = 0; gg < 4; gg++) d += half_bits_to_float(sw[2 * tk + (gg >> 1)] >> (16 * (gg & 1))) * rr[gg][tk];
                            const float v = sc[tk] + d * C1;
                            sc[tk] = base + tok0 + tk < my_limit ? v : NO_SCORE;  // (also whatever a block past the round left in LDS)
                        }
                        // the block's softmax relative to its own maximum, per column
                        float cm = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
                        cm = across_rows<16, 64>(cm, MaxOp());
                        float sum = 0.0f;
#pragma unroll
                        for (int tk = 0; tk < 4; tk++) {
                            sc[tk] = sc[tk] > 0.5f * NO_SCORE ? __builtin_amdgcn_exp2f(sc[tk] - cm) : 0.0f;
                            sum += sc[tk];
                        }
                        sum = across_rows<16, 64>(sum, SumOp());
                        if (j == 0) bmax_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = cm, bsum_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = sum;
                        // the scores go over the block's own keys: when this wave has them in registers, and with
                        // two pairs the other pair's wave of the same blocks, which takes them in the same order
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        taken++;
                        if constexpr (PAIRS > 1) {
                            raise(W::C_MERGE + wt);
                            await(W::C_MERGE + wt, PAIRS * taken);
                        }
                        *reinterpret_cast<floatx4 *>(s_block(blk, my_row) + (n & 7) * BLOCK + 4 * j) = sc;
                    }
                }
                raise(W::C_SCORES);
                await(W::C_SCORES, W::WAVES * (round + 1));

                // ---- the columns' maxima; what was summed so far brought to them; the probability operands ----
                float al[PAIRS];
#pragma unroll
                for (int p = 0; p < PAIRS; p++) {
                    const float nm = round_max(row_of(p, col_row), m_run[p]);
                    al[p] = __builtin_amdgcn_exp2f(m_run[p] - nm);  // (nothing summed so far: whatever it is, it scales zeros)
                    m_run[p] = nm;
                    zacc[p] *= al[p];
                    if (wave == 0) l_run[p] = l_run[p] * al[p] + round_sum(row_of(p, col_row), nm);
                }
                half8 p_hi[PAIRS][S_SLOTS], p_lo[PAIRS][S_SLOTS];
#pragma unroll
                for (int sl = 0; sl < S_SLOTS; sl++) {
                    if (uint32_t(2 * (2 * sl + b2)) >= nb) {  // the k-step has no tokens
#pragma unroll
                        for (int p = 0; p < PAIRS; p++) p_hi[p][sl] = p_lo[p][sl] = half8{0, 0, 0, 0, 0, 0, 0, 0};
                        continue;
                    }
                    const int ks = 2 * sl + b2;  // tokens 32 ks ..: blocks 2 ks and 2 ks + 1
                    const int blk = 2 * ks + (j >> 1);
                    const int sh = 16 * (g & 1);
                    const uint32_t *vsp = sb_lds + 2 * (W::SB_ARRAY / 4) + (g >> 1) * RT + 32 * ks + 8 * j;
                    const u32x4 sv0 = *reinterpret_cast<const u32x4 *>(vsp), sv1 = *reinterpret_cast<const u32x4 *>(vsp + 4);
                    const u32x4 zv0 = *reinterpret_cast<const u32x4 *>(vsp + W::SB_ARRAY / 4), zv1 = *reinterpret_cast<const u32x4 *>(vsp + W::SB_ARRAY / 4 + 4);
                    const uint32_t sw[8] = {sv0.x, sv0.y, sv0.z, sv0.w, sv1.x, sv1.y, sv1.z, sv1.w};
                    const uint32_t zw[8] = {zv0.x, zv0.y, zv0.z, zv0.w, zv1.x, zv1.y, zv1.z, zv1.w};
                    float vscale[8], vbias[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) vscale[e] = half_bits_to_float(sw[e] >> sh), vbias[e] = half_bits_to_float(zw[e] >> sh);
#pragma unroll
                    for (int p = 0; p < PAIRS; p++) {
                        const int r = row_of(p, col_row);
                        const float *sp = s_block(blk, r) + (n & 7) * BLOCK + 8 * (j & 1);
                        const floatx4 pt0 = *reinterpret_cast<const floatx4 *>(sp), pt1 = *reinterpret_cast<const floatx4 *>(sp + 4);
                        const float pt[8] = {pt0[0], pt0[1], pt0[2], pt0[3], pt1[0], pt1[1], pt1[2], pt1[3]};
                        // 2^(block maximum - maximum so far) * P_UP (2^8, so that the lo part stays a normal f16)
                        const float f = __builtin_amdgcn_exp2f(bmax_lds[r * W::BROW + (n & 7) * W::BSTRIDE + blk] - m_run[p] + 8.0f);
                        float x[8], lo[8], zb = 0.0f;
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            zb += pt[e] * vbias[e];
                            x[e] = pt[e] * f * vscale[e];
                            lo[e] = x[e] - __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x[e]) & 0xffffe000u);
                        }
                        zacc[p] += zb * f;
                        uint32_t o[8];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            // round toward zero: exact truncation to the hi part
                            o[e] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x[2 * e], x[2 * e + 1]));
                            o[4 + e] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo[2 * e], lo[2 * e + 1]));
                        }
                        asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]), "+v"(o[7]));
                        p_hi[p][sl] = as_half8(o[0], o[1], o[2], o[3]);
                        p_lo[p][sl] = as_half8(o[4], o[5], o[6], o[7]);
                    }
                }
                raise(W::C_BUILT);  // this wave is through with the round's scores, scales and biases

                // ---- phase C: O = O * 2^(old maximum - new) + P V ----
                if (round > 0) {
#pragma unroll
                    for (int p = 0; p < PAIRS; p++) {
                        // accumulator rows 4j + i are the pair's columns 4j + i: lane c (j = 0, n = c) holds column c's factor
                        floatx4 al4;
#pragma unroll
                        for (int i = 0; i < 4; i++) al4[i] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * (4 * j + i), __builtin_bit_cast(int, al[p])));
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[p][e] *= al4;
                    }
                }
#pragma unroll
                for (int sl = 0; sl < S_SLOTS; sl++) {
                    if (uint32_t(2 * (2 * sl + b2)) >= nb) continue;
                    await(W::C_SLOT + sl, W::V_LOADERS * (round + 1));  // value slot sl is in LDS
                    ValRegs<BITS> vreg;
                    read_values(2 * sl + b2, g, vreg);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const half8 vop = val_operand<BITS>(vreg, e, n);
#pragma unroll
                        for (int p = 0; p < PAIRS; p++) {
                            acc[p][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p_hi[p][sl], vop, acc[p][e], 0, 0, 0);
                            acc[p][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p_lo[p][sl], vop, acc[p][e], 0, 0, 0);
                        }
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the value codes are in registers
                raise(W::C_DONE);
            }

            // ---- epilogue: the two waves of a group add up, wave 2g writes the partials ----
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
                const float z = across_rows<16, 64>(zacc[p], SumOp());
                if (j == 0) zs_lds[(wave * PAIRS + p) * 16 + n] = z;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            floatx4 mine[PAIRS][4];  // column 4j + i of the pair, dims 64 g + 4n .. + 3
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float zb = zs_lds[(wave * PAIRS + p) * 16 + 4 * j + i] * (1.0f / P_UP);
#pragma unroll
                    for (int e = 0; e < 4; e++) mine[p][i][e] = acc[p][e][i] * unscale + zb;
                }
            }
            // (the merge lies over the keys, which hold the last round's scores until every wave has built its operands;
            // the key loaders request nothing after the last round)
            floatx4 *x_o = reinterpret_cast<floatx4 *>(lds_raw + W::K_OFF);  // [pair][group][lane][4 columns]
            static_assert(PAIRS * 4 * 64 * 4 * 16 <= W::SHORT_BLOCKS * W::K_BLOCK_BYTES || BITS == 4, "the merge stays clear of the query operands");
            await(W::C_BUILT, W::WAVES * n_rounds);
            if (b2 == 1) {
#pragma unroll
                for (int p = 0; p < PAIRS; p++) {
#pragma unroll
                    for (int i = 0; i < 4; i++) x_o[((p * 4 + g) * 64 + lane) * 4 + i] = mine[p][i];
                }
                raise(W::C_MERGE + 4 + g);
                leave();
                return;
            }
            if (wave == 0) {
#pragma unroll
                for (int p = 0; p < PAIRS; p++) {
                    const int r = 2 * p + col_row;
                    if (j == 0 && r < M) {
                        const size_t slot = (size_t(r) * a.nsplits + split) * a.heads + kv * 8 + (n & 7);
                        *reinterpret_cast<floatx2 *>(a.part_ml + 2 * slot) = floatx2{m_run[p], marked(l_run[p])};
                    }
                }
            }
            await(W::C_MERGE + 4 + g, 1);
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int c = 4 * j + i, r = 2 * p + (c >> 3);
                    if (r < M) {
                        const size_t slot = (size_t(r) * a.nsplits + split) * a.heads + kv * 8 + (c & 7);
                        __builtin_nontemporal_store(mine[p][i] + x_o[((p * 4 + g) * 64 + lane) * 4 + i], reinterpret_cast<floatx4 *>(a.part_o + slot * DIM + 64 * g + 4 * n));
                    }
                }
            }
            leave();
            return;
        }
        const uint32_t base = blk_begin * BLOCK;
        const bool extra = range >= uint32_t(RBK);  // the round has block 16
        const uint32_t live_blocks = (range + 1) & ~1u;  // k-steps are two blocks: the blocks of the k-steps that have tokens

        half8 q_hi[8], q_lo[8], qz_reg[2];
        {
            const float qmul = a.scale * 1.4426950408889634f * Q_UP;
#pragma unroll
            for (int pass = 0; pass < 2 * PAIRS; pass++) {
                const int pair = pass >> 1, lo_part = pass & 1;
                // this thread's item: k-step `wave`, lane `lane`: column n = (row n / 8 of the pair, head n % 8)
                half8 op;
                float sum = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    _Float16 h, lw;
                    split_hi_lo(qv[pair][key_slot_dim<BITS>(e)] * qmul, h, lw);
                    op[e] = lo_part ? lw : h;
                    sum += (float)h + (float)lw;
                }
                // the place is free when the readers of the pass before (the waves of its pair) have it in registers
                if (pass > 0) await(W::C_QREAD, WT * pass);
                q_lds[wave * 64 + lane] = op;
                if (!lo_part) {
                    // key bias term: slot `k-step` of this lane in the B operand of one more MFMA, as hi and lo halves
                    _Float16 h, lw;
                    split_hi_lo(sum * (1.0f / Q_UP), h, lw);
                    qz_lds[(0 * 64 + lane) * 8 + wave] = h;
                    qz_lds[(1 * 64 + lane) * 8 + wave] = lw;
                }
                raise(W::C_QUERY);
                if (pair == at) {
                    await(W::C_QUERY, W::WAVES * (pass + 1));
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const half8 v = q_lds[i * 64 + lane];
                        if (lo_part) q_lo[i] = v; else q_hi[i] = v;
                    }
                    if (!lo_part) {
                        qz_reg[0] = *reinterpret_cast<const half8 *>(qz_lds + lane * 8);
                        qz_reg[1] = *reinterpret_cast<const half8 *>(qz_lds + (64 + lane) * 8);
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    raise(W::C_QREAD);
                }
            }
        }

        // ---- phase A: the scores of this wave's blocks for its pair of rows ----
        {
            const int my_row = row_of(at, col_row);
            const uint32_t my_limit = min<uint32_t>(limit, len_of(my_row));
            constexpr int A_BLOCKS = (RBK + WT - 1) / WT;
#pragma unroll 1
            for (int i = 0; i < A_BLOCKS; i++) {
                const int blk = wt + WT * i;
                if (blk >= (extra ? RBK : RBK - 1)) break;
                if (uint32_t(blk) >= live_blocks) {
                    // (a short share: no scores to take, and no operands will be made of this block; the other
                    // pair's wave of the same blocks leaves it out as well)
                    if (j == 0) bmax_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = NO_SCORE, bsum_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = 0.0f;
                    continue;
                }
                await(W::C_KPART + (blk >> 3), W::K_LOADERS);  // this part of the keys is in LDS (first: and the scales)
                const unsigned char *kb = lds_raw + W::K_OFF + blk * W::K_BLOCK_BYTES;
                KeyRegs<BITS> kreg[4];
#pragma unroll
                for (int gg = 0; gg < 4; gg++) {
                    if constexpr (BITS == 8) {
                        const u32x4 v = *reinterpret_cast<const u32x4 *>(kb + gg * 1024 + n * 64 + j * 16);
                        kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y, kreg[gg].w[2] = v.z, kreg[gg].w[3] = v.w;
                    } else {
                        const u32x2 v = *reinterpret_cast<const u32x2 *>(kb + (gg >> 1) * 1024 + n * 64 + (gg & 1) * 32 + j * 8);
                        kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y;
                    }
                }
                const int tok0 = BLOCK * blk + 4 * j;  // this lane's 4 tokens of the round in C layout
                const uint32_t *sb_w = sb_lds + BLOCK * blk;
                const u32x2 zr = {sb_w[W::SB_ARRAY / 4 + n], sb_w[W::SB_ARRAY / 4 + RT + n]};
                const half8 zop = as_half8(perm(0, zr.x, 0x01000100u), perm(0, zr.x, 0x03020302u), perm(0, zr.y, 0x01000100u), perm(0, zr.y, 0x03020302u));
                const u32x4 s01 = *reinterpret_cast<const u32x4 *>(sb_w + 4 * j);
                const u32x4 s23 = *reinterpret_cast<const u32x4 *>(sb_w + RT + 4 * j);
                const uint32_t sw[8] = {s01.x, s23.x, s01.y, s23.y, s01.z, s23.z, s01.w, s23.w};
                floatx4 s = {0, 0, 0, 0}, rr[4];
                s = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz_reg[0], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz_reg[1], s, 0, 0, 0);
#pragma unroll
                for (int gg = 0; gg < 4; gg++) {
                    rr[gg] = floatx4{0, 0, 0, 0};
#pragma unroll
                    for (int ab = 0; ab < 2; ab++) {
                        const half8 kop = key_operand<BITS>(kreg[gg], ab);
                        rr[gg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop, q_hi[gg * 2 + ab], rr[gg], 0, 0, 0);
                        rr[gg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop, q_lo[gg * 2 + ab], rr[gg], 0, 0, 0);
                    }
                }
                constexpr float C1 = code_up<BITS>() / Q_UP;
#pragma unroll
                for (int tk = 0; tk < 4; tk++) {
                    float d = 0.0f;
#pragma unroll
                    for (int gg = 0; gg < 4; gg++) d += half_bits_to_float(sw[2 * tk + (gg >> 1)] >> (16 * (gg & 1))) * rr[gg][tk];
                    const float v = s[tk] + d * C1;
                    s[tk] = base + tok0 + tk < my_limit ? v : NO_SCORE;  // (also whatever a block past the round left in LDS)
                }
                // the block's softmax relative to its own maximum, per column
                float cm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
                cm = across_rows<16, 64>(cm, MaxOp());
                float sum = 0.0f;
#pragma unroll
                for (int tk = 0; tk < 4; tk++) {
                    s[tk] = s[tk] > 0.5f * NO_SCORE ? __builtin_amdgcn_exp2f(s[tk] - cm) : 0.0f;
                    sum += s[tk];
                }
                sum = across_rows<16, 64>(sum, SumOp());
                if (j == 0) bmax_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = cm, bsum_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + blk] = sum;
                // the scores go over the block's own keys: when this wave has them in registers, and with
                // two pairs the other pair's wave of the same blocks, which takes them in the same order
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if constexpr (PAIRS > 1) {
                    // (the blocks a wave leaves out are its last ones: i counts the ones it takes)
                    raise(W::C_MERGE + wt);
                    await(W::C_MERGE + wt, PAIRS * (i + 1));
                }
                *reinterpret_cast<floatx4 *>(s_block(blk, my_row) + (n & 7) * BLOCK + 4 * j) = s;
            }
            if (wt == 0 && !extra && j == 0) bmax_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + 16] = NO_SCORE, bsum_lds[my_row * W::BROW + (n & 7) * W::BSTRIDE + 16] = 0.0f;
        }
        raise(W::C_SCORES);
        await(W::C_SCORES, W::WAVES);

        // ---- the columns' maxima, the probability operands of this wave's k-steps ----
        // A operand: lane (n, j) holds tokens 8j .. 8j + 7 of the k-step for column n, as hi and as lo parts.
        float nm[PAIRS], zacc[PAIRS];
#pragma unroll
        for (int p = 0; p < PAIRS; p++) nm[p] = round_max(row_of(p, col_row), NO_SCORE), zacc[p] = 0.0f;
        const bool fifth = extra && b2 == 0;  // k-step 8: block 16 (lane groups 0 and 1; the others repeat them with factor 0)
        half8 p_hi[PAIRS][W::SLOTS], p_lo[PAIRS][W::SLOTS];
#pragma unroll
        for (int sl = 0; sl < W::SLOTS; sl++) {
            // (no block 16 | a short share: the k-step has no tokens)
            if ((sl == 4 && !fifth) || uint32_t(2 * (2 * sl + b2)) >= range) {
#pragma unroll
                for (int p = 0; p < PAIRS; p++) p_hi[p][sl] = p_lo[p][sl] = half8{0, 0, 0, 0, 0, 0, 0, 0};
                continue;
            }
            const int ks = 2 * sl + b2;  // tokens 32 ks ..: blocks 2 ks and 2 ks + 1
            const int jj = sl == 4 ? (j & 1) : j;
            const int blk = 2 * ks + (jj >> 1);
            const int sh = 16 * (g & 1);
            // value scales and biases of group g: half g % 2 of the tokens' dwords of groups (g, g ^ 1).
            // (Tokens past the share have probability 0 and the scales of the share's last token:
            // every load is clamped to it, so nothing but cache rows in use is ever read.)
            const uint32_t *vsp = sb_lds + 2 * (W::SB_ARRAY / 4) + (g >> 1) * RT + 32 * ks + 8 * jj;
            const u32x4 sv0 = *reinterpret_cast<const u32x4 *>(vsp), sv1 = *reinterpret_cast<const u32x4 *>(vsp + 4);
            const u32x4 zv0 = *reinterpret_cast<const u32x4 *>(vsp + W::SB_ARRAY / 4), zv1 = *reinterpret_cast<const u32x4 *>(vsp + W::SB_ARRAY / 4 + 4);
            const uint32_t sw[8] = {sv0.x, sv0.y, sv0.z, sv0.w, sv1.x, sv1.y, sv1.z, sv1.w};
            const uint32_t zw[8] = {zv0.x, zv0.y, zv0.z, zv0.w, zv1.x, zv1.y, zv1.z, zv1.w};
            float vscale[8], vbias[8];
#pragma unroll
            for (int e = 0; e < 8; e++) vscale[e] = half_bits_to_float(sw[e] >> sh), vbias[e] = half_bits_to_float(zw[e] >> sh);
            const int fb = 2 * ks + (j >> 1);  // block 17 does not exist: factor 0
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
                const int r = row_of(p, col_row);
                const float *sp = s_block(blk, r) + (n & 7) * BLOCK + 8 * (jj & 1);
                const floatx4 pt0 = *reinterpret_cast<const floatx4 *>(sp), pt1 = *reinterpret_cast<const floatx4 *>(sp + 4);
                const float pt[8] = {pt0[0], pt0[1], pt0[2], pt0[3], pt1[0], pt1[1], pt1[2], pt1[3]};
                // 2^(block maximum - round maximum) * P_UP (2^8, so that the lo part stays a normal f16)
                const float f = fb < RBK ? __builtin_amdgcn_exp2f(bmax_lds[r * W::BROW + (n & 7) * W::BSTRIDE + (fb < RBK ? fb : 0)] - nm[p] + 8.0f) : 0.0f;
                float x[8], lo[8], zb = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    zb += pt[e] * vbias[e];
                    x[e] = pt[e] * f * vscale[e];
                    lo[e] = x[e] - __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x[e]) & 0xffffe000u);
                }
                zacc[p] += zb * f;
                uint32_t o[8];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // round toward zero: exact truncation to the hi part
                    o[e] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x[2 * e], x[2 * e + 1]));
                    o[4 + e] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo[2 * e], lo[2 * e + 1]));
                }
                // (pinned: left alone, the compiler moves an operand's arithmetic down to its use, behind the wait for the values)
                asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]), "+v"(o[7]));
                p_hi[p][sl] = as_half8(o[0], o[1], o[2], o[3]);
                p_lo[p][sl] = as_half8(o[4], o[5], o[6], o[7]);
            }
        }
        raise(W::C_BUILT);  // this wave is through with the scores

        // ---- phase C: O += P V, one k-step per value slot as the slots land ----
        floatx4 acc[PAIRS][4];  // [pair][tile of 16 dims 4n' + e]: rows 4j .. 4j+3 (columns of the pair), column n'
#pragma unroll
        for (int p = 0; p < PAIRS; p++) {
#pragma unroll
            for (int e = 0; e < 4; e++) acc[p][e] = floatx4{0, 0, 0, 0};
        }
#pragma unroll
        for (int sl = 0; sl < W::SLOTS; sl++) {
            if ((sl == 4 && !fifth) || uint32_t(2 * (2 * sl + b2)) >= range) continue;
            await(W::C_SLOT + sl, W::V_LOADERS);  // value slot sl is in LDS
            ValRegs<BITS> vreg;
            read_values(sl == 4 ? 8 : 2 * sl + b2, g, vreg);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const half8 vop = val_operand<BITS>(vreg, e, n);
#pragma unroll
                for (int p = 0; p < PAIRS; p++) {
                    acc[p][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p_hi[p][sl], vop, acc[p][e], 0, 0, 0);
                    acc[p][e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p_lo[p][sl], vop, acc[p][e], 0, 0, 0);
                }
            }
        }

        // ---- epilogue: the two waves of a group add up, wave 2g writes the partials ----
#pragma unroll
        for (int p = 0; p < PAIRS; p++) {
            // a column's bias sum: over the four lane groups
            const float z = across_rows<16, 64>(zacc[p], SumOp());
            if (j == 0) zs_lds[(wave * PAIRS + p) * 16 + n] = z;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        floatx4 mine[PAIRS][4];  // column 4j + i of the pair, dims 64 g + 4n .. + 3
#pragma unroll
        for (int p = 0; p < PAIRS; p++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float zb = zs_lds[(wave * PAIRS + p) * 16 + 4 * j + i] * (1.0f / P_UP);
#pragma unroll
                for (int e = 0; e < 4; e++) mine[p][i][e] = acc[p][e][i] * unscale + zb;
            }
        }
        // (the merge lies over the keys, which hold the scores until every wave has built its operands)
        floatx4 *x_o = reinterpret_cast<floatx4 *>(lds_raw + W::K_OFF);  // [pair][group][lane][4 columns]
        await(W::C_BUILT, W::WAVES);
        if (b2 == 1) {
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
#pragma unroll
                for (int i = 0; i < 4; i++) x_o[((p * 4 + g) * 64 + lane) * 4 + i] = mine[p][i];
            }
            raise(W::C_MERGE + 4 + g);
            leave();
            return;
        }
        if (wave == 0) {
#pragma unroll
            for (int p = 0; p < PAIRS; p++) {
                const int r = 2 * p + col_row;
                const float l = round_sum(row_of(p, col_row), nm[p]);
                if (j == 0 && r < M) {
                    const size_t slot = (size_t(r) * a.nsplits + split) * a.heads + kv * 8 + (n & 7);
                    *reinterpret_cast<floatx2 *>(a.part_ml + 2 * slot) = floatx2{nm[p], marked(l)};
                }
            }
        }
        await(W::C_MERGE + 4 + g, 1);
#pragma unroll
        for (int p = 0; p < PAIRS; p++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = 4 * j + i, r = 2 * p + (c >> 3);
                if (r < M) {
                    const size_t slot = (size_t(r) * a.nsplits + split) * a.heads + kv * 8 + (c & 7);
                    // (nobody on this CU reads the partials again: past the caches)
                    __builtin_nontemporal_store(mine[p][i] + x_o[((p * 4 + g) * 64 + lane) * 4 + i], reinterpret_cast<floatx4 *>(a.part_o + slot * DIM + 64 * g + 4 * n));
                }
            }
        }
    } else {
        // ---- one row -----------------------------------------------------------------------------
        // Scores: wave w takes the blocks w and w + 8 (wave 0 also 16).  O += P V: waves 2g and 2g + 1 share
        // group g and take alternate k-steps, so that each value slot gives every wave one k-step.
        // ---- prologue: the query row to f16 hi/lo operands in LDS (operand row n: head n & 7, hi part in
        // rows 0-7 and lo part in rows 8-15 of the one tile) ---------------------------------------------
        {
            const float qmul = a.scale * 1.4426950408889634f * Q_UP;
            half8 op;
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                _Float16 h, lw;
                split_hi_lo(qv[0][key_slot_dim<BITS>(e)] * qmul, h, lw);
                const _Float16 x = n < 8 ? h : lw;
                op[e] = x;
                sum += (float)x;
            }
            q_lds[wave * 64 + lane] = op;
            // key bias term: slot `k-step` of this lane in the B operand of one more MFMA, as hi and lo halves
            _Float16 h, lw;
            split_hi_lo(sum * (1.0f / Q_UP), h, lw);
            qz_lds[(0 * 64 + lane) * 8 + wave] = h;
            qz_lds[(1 * 64 + lane) * 8 + wave] = lw;
            // blocks that never exist
            if (wave == 0 && lane < 8 * (W::BSINGLE - RBK)) {
                const int idx = (lane / (W::BSINGLE - RBK)) * W::BSTRIDE + RBK + lane % (W::BSINGLE - RBK);
                bmax_lds[idx] = NO_SCORE, bsum_lds[idx] = 0.0f;
            }
        }
        raise(W::C_QUERY);

        // ---- running state -------------------------------------------------------------
        float m_run = NO_SCORE;
        float l_run = 0.0f;    // sum of P of head n & 7 (wave 0 keeps it)
        float zacc = 0.0f;     // sum of P * P_UP * value bias of group g over this lane's tokens
        floatx4 acc[4];        // [tile of 16 dims 4n' + e]: rows 4j .. 4j+3 (operand rows), column n'
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] = floatx4{0, 0, 0, 0};
        await(W::C_QUERY, W::WAVES);

        if constexpr (W::ALTERNATE) if (alt) {
            // ---- a share of more than one round: rounds of up to ALT_BLOCKS blocks in alternate halves of LDS ----
            // Round r lies in the blocks ALT_BLOCKS (r % 2) .. of the keys' and the values' places, of the scales and of
            // the block table: every computing wave takes the scores of one block (4-bit codes: two) and two k-steps (four)
            // of O += P V per round, and the loaders fill the other half meanwhile.  A half is free for round r + 2 when
            // every wave has built its operands (keys, scales, scores) and is through with the values of round r.
            constexpr int AB = W::ALT_BLOCKS, WAVE_BLOCKS = AB / W::WAVES, WAVE_STEPS = AB / 4;
#pragma unroll 1
            for (uint32_t round = 0; round < n_rounds; round++) {
                const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
                const int half = int(round & 1) * AB;  // the round's first block in LDS
                const uint32_t round_limit = min(limit, base + nb * BLOCK);  // tokens of this round end here
                const uint32_t live_blocks = (nb + 1) & ~1u;  // k-steps are two blocks: the blocks of the k-steps that have tokens
                // ---- phase A: the scores of the blocks wave (, wave + 8) of the round ----
#pragma unroll 1
                for (int part = 0; part < WAVE_BLOCKS; part++) {
                    const int rblk = wave + W::WAVES * part;  // of the round
                    const int blk = half + rblk;              // in LDS
                    if (uint32_t(rblk) >= live_blocks) {
                        // (no scores to take, and no operands will be made of this block; the table still holds the entries of
                        // the round before last until every wave has built its operands from them)
                        if (round > 1) await(W::C_BUILT, W::WAVES * (round - 1));
                        if (j == 0 && n < 8) bmax_lds[n * W::BSTRIDE + blk] = NO_SCORE, bsum_lds[n * W::BSTRIDE + blk] = 0.0f;
                    } else {
                        half8 q_reg[8], qz_reg[2];
#pragma unroll
                        for (int i = 0; i < 8; i++) q_reg[i] = q_lds[i * 64 + lane];
                        qz_reg[0] = *reinterpret_cast<const half8 *>(qz_lds + lane * 8);
                        qz_reg[1] = *reinterpret_cast<const half8 *>(qz_lds + (64 + lane) * 8);
                        await(W::C_KPART + 0, round + 1);  // the round's keys and scales are in LDS (one loader per round)
                        const unsigned char *kb = lds_raw + W::K_OFF + blk * W::K_BLOCK_BYTES;
                        KeyRegs<BITS> kreg[4];
#pragma unroll
                        for (int gg = 0; gg < 4; gg++) {
                            if constexpr (BITS == 8) {
                                const u32x4 v = *reinterpret_cast<const u32x4 *>(kb + gg * 1024 + n * 64 + j * 16);
                                kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y, kreg[gg].w[2] = v.z, kreg[gg].w[3] = v.w;
                            } else {
                                const u32x2 v = *reinterpret_cast<const u32x2 *>(kb + (gg >> 1) * 1024 + n * 64 + (gg & 1) * 32 + j * 8);
                                kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y;
                            }
                        }
                        const int tok0 = BLOCK * rblk + 4 * j;  // this lane's 4 tokens of the round in C layout
                        const uint32_t *sb_w = sb_lds + BLOCK * blk;  // the block's dwords of groups (0, 1); + RT: groups (2, 3)
                        floatx4 sc;
                        {
                            const u32x2 zr = {sb_w[W::SB_ARRAY / 4 + n], sb_w[W::SB_ARRAY / 4 + RT + n]};
                            const half8 zop = as_half8(perm(0, zr.x, 0x01000100u), perm(0, zr.x, 0x03020302u), perm(0, zr.y, 0x01000100u),
                                                       perm(0, zr.y, 0x03020302u));
                            sc = floatx4{0, 0, 0, 0};
                            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz_reg[0], sc, 0, 0, 0);
                            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz_reg[1], sc, 0, 0, 0);
                        }
                        floatx4 r[4];
#pragma unroll
                        for (int gg = 0; gg < 4; gg++) {
                            r[gg] = floatx4{0, 0, 0, 0};
#pragma unroll
                            for (int ab = 0; ab < 2; ab++) {
                                r[gg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(key_operand<BITS>(kreg[gg], ab), q_reg[gg * 2 + ab], r[gg], 0, 0, 0);
                            }
                        }
                        const u32x4 s01 = *reinterpret_cast<const u32x4 *>(sb_w + 4 * j);
                        const u32x4 s23 = *reinterpret_cast<const u32x4 *>(sb_w + RT + 4 * j);
                        const uint32_t sw[8] = {s01.x, s23.x, s01.y, s23.y, s01.z, s23.z, s01.w, s23.w};
                        constexpr float C1 = code_up<BITS>() / Q_UP;
#pragma unroll
                        for (int tk = 0; tk < 4; tk++) {
                            float d = 0.0f;
#pragma unroll
                            for (int gg = 0; gg < 4; gg++) d += half_bits_to_float(sw[2 * tk + (gg >> 1)] >> (16 * (gg & 1))) * r[gg][tk];
                            float v = sc[tk] + d * C1;
                            v += dpp<0x128>(v);  // row_ror 8: the other part (hi | lo) of the same head
                            sc[tk] = base + tok0 + tk < round_limit ? v : NO_SCORE;  // (also whatever a block past the round left in LDS)
                        }
                        float cm = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
                        cm = across_rows<16, 64>(cm, MaxOp());
                        float sum = 0.0f;
#pragma unroll
                        for (int tk = 0; tk < 4; tk++) {
                            sc[tk] = sc[tk] > 0.5f * NO_SCORE ? __builtin_amdgcn_exp2f(sc[tk] - cm) : 0.0f;
                            sum += sc[tk];
                        }
                        sum = across_rows<16, 64>(sum, SumOp());
                        // over the block's own keys (every lane of the wave has its key registers by now)
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        if (n < 8) *reinterpret_cast<floatx4 *>(s_block(blk, 0) + n * BLOCK + 4 * j) = sc;
                        if (j == 0 && n < 8) bmax_lds[n * W::BSTRIDE + blk] = cm, bsum_lds[n * W::BSTRIDE + blk] = sum;
                    }
                }
                raise(W::C_SCORES);
                await(W::C_SCORES, W::WAVES * (round + 1));

                // ---- the round's maximum per head, and what was summed so far brought to it ----
                float nm = m_run;
                {
                    const floatx4 *bmx = reinterpret_cast<const floatx4 *>(bmax_lds + (n & 7) * W::BSTRIDE + half);
#pragma unroll
                    for (int i = 0; i < AB / 4; i++) {
                        const floatx4 w = bmx[i];
                        nm = fmaxf(nm, fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3])));
                    }
                }
                const float al = __builtin_amdgcn_exp2f(m_run - nm);  // (first round: 2^(-1e30 - nm) = 0, and nothing to scale)
                if (round > 0) {
                    zacc *= al;
                    floatx4 al4;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        al4[i] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * ((4 * j + i) & 7), __builtin_bit_cast(int, al)));
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[e] *= al4;
                }
                m_run = nm;
                if (wave == 0) {
                    // the round's sum of P of head n & 7: lane group j adds the blocks (AB / 4) j ..
                    float sum = 0.0f;
#pragma unroll
                    for (int i = 0; i < AB / 4; i++) {
                        const int b = half + (AB / 4) * j + i;
                        sum += bsum_lds[(n & 7) * W::BSTRIDE + b] * __builtin_amdgcn_exp2f(bmax_lds[(n & 7) * W::BSTRIDE + b] - nm);  // (a block that is not there: sum 0)
                    }
                    l_run = l_run * al + across_rows<16, 64>(sum, SumOp());
                }

                // ---- probability operands of this wave's k-steps (as in a single round) ----
                half8 p_alt[WAVE_STEPS];
                {
                    const int hh = n >> 3;  // this lane makes tokens 8j + 4 hh .. + 3 of a k-step
                    const int sh = 16 * (g & 1);
#pragma unroll
                    for (int i = 0; i < WAVE_STEPS; i++) {
                        if (uint32_t(2 * (2 * i + b2)) >= nb) {  // the k-step has no tokens
                            p_alt[i] = half8{0, 0, 0, 0, 0, 0, 0, 0};
                            continue;
                        }
                        const int ks = half / 2 + 2 * i + b2;  // in LDS: tokens 32 ks ..: blocks 2 ks and 2 ks + 1
                        const int blk = 2 * ks + (j >> 1);
                        const floatx4 pt = *reinterpret_cast<const floatx4 *>(s_block(blk, 0) + (n & 7) * BLOCK + 8 * (j & 1) + 4 * hh);
                        const uint32_t *vsp = sb_lds + 2 * (W::SB_ARRAY / 4) + (g >> 1) * RT + 32 * ks + 8 * j + 4 * hh;
                        const u32x4 sv = *reinterpret_cast<const u32x4 *>(vsp);
                        const u32x4 zv = *reinterpret_cast<const u32x4 *>(vsp + W::SB_ARRAY / 4);
                        // 2^(block maximum - maximum so far) * P_UP (2^8, so that the lo part stays a normal f16)
                        const float f = __builtin_amdgcn_exp2f(bmax_lds[(n & 7) * W::BSTRIDE + blk] - nm + 8.0f);
                        const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w}, zw[4] = {zv.x, zv.y, zv.z, zv.w};
                        float x[4], lo[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float p = pt[e] * f;
                            zacc += p * half_bits_to_float(zw[e] >> sh);
                            x[e] = p * half_bits_to_float(sw[e] >> sh);
                            lo[e] = x[e] - __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x[e]) & 0xffffe000u);
                        }
                        // round toward zero: exact truncation to the hi part
                        const uint32_t hi0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x[0], x[1]));
                        const uint32_t hi1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x[2], x[3]));
                        const uint32_t lo0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo[0], lo[1]));
                        const uint32_t lo1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo[2], lo[3]));
                        const uint32_t send0 = hh ? hi0 : lo0, send1 = hh ? hi1 : lo1;
                        const uint32_t recv0 = uint32_t(__builtin_amdgcn_update_dpp(0, int(send0), 0x128, 0xf, 0xf, false));  // row_ror 8
                        const uint32_t recv1 = uint32_t(__builtin_amdgcn_update_dpp(0, int(send1), 0x128, 0xf, 0xf, false));
                        uint32_t o[4] = {hh ? recv0 : hi0, hh ? recv1 : hi1, hh ? lo0 : recv0, hh ? lo1 : recv1};
                        asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]));
                        p_alt[i] = as_half8(o[0], o[1], o[2], o[3]);
                    }
                }
                raise(W::C_BUILT);  // this wave is through with the round's keys, scores, scales and biases

                // ---- phase C: O += P V of the wave's k-steps ----
                await(W::C_SLOT + 4, round + 1);  // the round's values are in LDS (one loader per round)
                {
                    ValRegs<BITS> vreg[WAVE_STEPS];
#pragma unroll
                    for (int i = 0; i < WAVE_STEPS; i++) {
                        if (uint32_t(2 * (2 * i + b2)) >= nb) continue;
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            const int tk = BLOCK * half + 32 * (2 * i + b2) + 8 * j + e;
                            vreg[i].w[e] = *reinterpret_cast<const uint32_t *>(lds_raw + W::V_OFF + tk * RB + ((val_lane_offset<BITS>(g, n) + j * (RB / 4)) & (RB - 1)));
                        }
                    }
#pragma unroll
                    for (int i = 0; i < WAVE_STEPS; i++) {
                        if (uint32_t(2 * (2 * i + b2)) >= nb) continue;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p_alt[i], val_operand<BITS>(vreg[i], e, n), acc[e], 0, 0, 0);
                        }
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the value codes are in registers
                raise(W::C_DONE);
            }
        }
        if (!alt) {
            // ---- a share of up to 17 blocks: one round ----
            constexpr uint32_t round = 0;  // (written as the first of several rounds)
            constexpr bool more = false;
            const uint32_t base = (blk_begin + round * per_round) * BLOCK, nb = blocks_of(round);
            const bool extra = nb == uint32_t(RBK);  // the round has block 16
            const uint32_t round_limit = min(limit, base + nb * BLOCK);  // tokens of this round end here
            const uint32_t live_blocks = (nb + 1) & ~1u;  // k-steps are two blocks: the blocks of the k-steps that have tokens

            // ---- phase A: scores of blocks wave, wave + 8 (and wave 0: 16) --------------------------
            // (the query operands are read again in every round: they are not needed between the scores
            // of one round and the next, and the registers are)
            {
                half8 q_reg[8], qz_reg[2];
#pragma unroll
                for (int i = 0; i < 8; i++) q_reg[i] = q_lds[i * 64 + lane];
                qz_reg[0] = *reinterpret_cast<const half8 *>(qz_lds + lane * 8);
                qz_reg[1] = *reinterpret_cast<const half8 *>(qz_lds + (64 + lane) * 8);
                const int parts = (wave == 0 && extra) ? 3 : 2;
#pragma unroll 1
                for (int part = 0; part < parts; part++) {
                    const int blk = wave + 8 * part;
                    if (uint32_t(blk) >= live_blocks) {
                        // (a short round: no scores to take, and no operands will be made of this block; the
                        // table still holds the round before's entries until every wave has built its operands
                        // from them, which is also what the key loader waits for before it overwrites the keys)
                        if (round > 0) await(W::C_BUILT, W::WAVES * round);
                        if (j == 0 && n < 8) bmax_lds[n * W::BSTRIDE + blk] = NO_SCORE, bsum_lds[n * W::BSTRIDE + blk] = 0.0f;
                        continue;
                    }
                    await(W::C_KPART + part, W::K_LOADERS * (round + 1));  // this part of the keys is in LDS (first: and the scales)
                    const unsigned char *kb = lds_raw + W::K_OFF + blk * W::K_BLOCK_BYTES;
                    KeyRegs<BITS> kreg[4];
#pragma unroll
                    for (int gg = 0; gg < 4; gg++) {
                        if constexpr (BITS == 8) {
                            // the group's 64 bytes of token n are piece gg: 16 bytes j of them
                            const u32x4 v = *reinterpret_cast<const u32x4 *>(kb + gg * 1024 + n * 64 + j * 16);
                            kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y, kreg[gg].w[2] = v.z, kreg[gg].w[3] = v.w;
                        } else {
                            // the group's 32 bytes of token n are half gg % 2 of piece gg / 2: 8 bytes j of them
                            const u32x2 v = *reinterpret_cast<const u32x2 *>(kb + (gg >> 1) * 1024 + n * 64 + (gg & 1) * 32 + j * 8);
                            kreg[gg].w[0] = v.x, kreg[gg].w[1] = v.y;
                        }
                    }
                    const int tok0 = BLOCK * blk + 4 * j;  // this lane's 4 tokens of the round in C layout
                    const uint32_t *sb_w = sb_lds + BLOCK * blk;  // the block's dwords of groups (0, 1); + RT: groups (2, 3)
                    floatx4 s;
                    {
                        // bias term: slot e of every lane group belongs to group e / 2 of token n
                        const u32x2 zr = {sb_w[W::SB_ARRAY / 4 + n], sb_w[W::SB_ARRAY / 4 + RT + n]};
                        const half8 zop = as_half8(perm(0, zr.x, 0x01000100u), perm(0, zr.x, 0x03020302u), perm(0, zr.y, 0x01000100u),
                                                   perm(0, zr.y, 0x03020302u));
                        s = floatx4{0, 0, 0, 0};
                        s = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz_reg[0], s, 0, 0, 0);
                        s = __builtin_amdgcn_mfma_f32_16x16x32_f16(zop, qz_reg[1], s, 0, 0, 0);
                    }
                    floatx4 r[4];
#pragma unroll
                    for (int gg = 0; gg < 4; gg++) {
                        r[gg] = floatx4{0, 0, 0, 0};
#pragma unroll
                        for (int ab = 0; ab < 2; ab++) {
                            r[gg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(key_operand<BITS>(kreg[gg], ab), q_reg[gg * 2 + ab], r[gg], 0, 0, 0);
                        }
                    }
                    // scales of the lane's tokens 4j .. 4j+3 of the block: groups (0, 1) and groups (2, 3)
                    const u32x4 s01 = *reinterpret_cast<const u32x4 *>(sb_w + 4 * j);
                    const u32x4 s23 = *reinterpret_cast<const u32x4 *>(sb_w + RT + 4 * j);
                    const uint32_t sw[8] = {s01.x, s23.x, s01.y, s23.y, s01.z, s23.z, s01.w, s23.w};
                    constexpr float C1 = code_up<BITS>() / Q_UP;
#pragma unroll
                    for (int tk = 0; tk < 4; tk++) {
                        float d = 0.0f;
#pragma unroll
                        for (int gg = 0; gg < 4; gg++) d += half_bits_to_float(sw[2 * tk + (gg >> 1)] >> (16 * (gg & 1))) * r[gg][tk];
                        float v = s[tk] + d * C1;
                        v += dpp<0x128>(v);  // row_ror 8: the other part (hi | lo) of the same head
                        s[tk] = base + tok0 + tk < round_limit ? v : NO_SCORE;  // (also whatever a block past the round left in LDS)
                    }
                    // the block's softmax relative to its own maximum, per head
                    float cm = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
                    cm = across_rows<16, 64>(cm, MaxOp());
                    float sum = 0.0f;
#pragma unroll
                    for (int tk = 0; tk < 4; tk++) {
                        s[tk] = s[tk] > 0.5f * NO_SCORE ? __builtin_amdgcn_exp2f(s[tk] - cm) : 0.0f;
                        sum += s[tk];
                    }
                    sum = across_rows<16, 64>(sum, SumOp());
                    // over the block's own keys (every lane of the wave has its key registers by now)
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    if (n < 8) *reinterpret_cast<floatx4 *>(s_block(blk, 0) + n * BLOCK + 4 * j) = s;
                    if (j == 0 && n < 8) bmax_lds[n * W::BSTRIDE + blk] = cm, bsum_lds[n * W::BSTRIDE + blk] = sum;
                }
                if (wave == 0 && !extra) {
                    // (block 16 of the round before, if it had one, is read until every wave has built its operands)
                    if (round > 0) await(W::C_BUILT, W::WAVES * round);
                    if (j == 0 && n < 8) bmax_lds[n * W::BSTRIDE + 16] = NO_SCORE, bsum_lds[n * W::BSTRIDE + 16] = 0.0f;
                }
            }
            raise(W::C_SCORES);
            await(W::C_SCORES, W::WAVES * (round + 1));

            // ---- the round's maximum per head, and what was summed so far brought to it -------------
            float nm = m_run;
            {
                const floatx4 *bmx = reinterpret_cast<const floatx4 *>(bmax_lds + (n & 7) * W::BSTRIDE);
#pragma unroll
                for (int i = 0; i < W::BSINGLE / 4; i++) {
                    const floatx4 w = bmx[i];
                    nm = fmaxf(nm, fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3])));
                }
            }
            const float al = __builtin_amdgcn_exp2f(m_run - nm);  // (first round: 2^(-1e30 - nm) = 0, and nothing to scale)
            if (round > 0) {
                zacc *= al;
                // accumulator rows 4j + i are heads (4j + i) & 7: lane h (j = 0, n = h) holds head h's factor
                floatx4 al4;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    al4[i] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * ((4 * j + i) & 7), __builtin_bit_cast(int, al)));
                }
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] *= al4;
            }
            m_run = nm;
            if (wave == 0) {
                // the round's sum of P of head n & 7: lane group j adds blocks 5j .. 5j + 4
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < W::BSINGLE / 4; i++) {
                    const int b = (W::BSINGLE / 4) * j + i;
                    sum += bsum_lds[(n & 7) * W::BSTRIDE + b] * __builtin_amdgcn_exp2f(bmax_lds[(n & 7) * W::BSTRIDE + b] - nm);  // (a block that is not there: sum 0)
                }
                l_run = l_run * al + across_rows<16, 64>(sum, SumOp());
            }

            // ---- probability operands of this wave's k-steps: P * value scale of group g, hi part in
            // operand rows 0-7 and lo part in rows 8-15.  The two lanes of a head (n and n + 8) make four of
            // the lane group's eight tokens each, both parts, and exchange what the other one feeds. ----
            half8 p_op[W::SLOTS];
            {
                const int hh = n >> 3;  // this lane makes tokens 8j + 4 hh .. + 3 of a k-step
                const int sh = 16 * (g & 1);
                const bool fifth = extra && b2 == 0;  // k-step 8: block 16 (lane groups 0 and 1; the others repeat them with factor 0)
#pragma unroll
                for (int sl = 0; sl < W::SLOTS; sl++) {
                    // (no block 16 | a short round: the k-step has no tokens)
                    if ((sl == 4 && !fifth) || uint32_t(2 * (2 * sl + b2)) >= nb) {
                        p_op[sl] = half8{0, 0, 0, 0, 0, 0, 0, 0};
                        continue;
                    }
                    const int ks = 2 * sl + b2;  // tokens 32 ks ..: blocks 2 ks and 2 ks + 1
                    const int jj = sl == 4 ? (j & 1) : j;
                    const int blk = 2 * ks + (jj >> 1);
                    const floatx4 pt = *reinterpret_cast<const floatx4 *>(s_block(blk, 0) + (n & 7) * BLOCK + 8 * (jj & 1) + 4 * hh);
                    // value scales and biases of group g: half g % 2 of the tokens' dwords of groups (g, g ^ 1).
                    // (Tokens past the share have probability 0 and the scales of the share's last token:
                    // every load is clamped to it, so nothing but cache rows in use is ever read.)
                    const uint32_t *vsp = sb_lds + 2 * (W::SB_ARRAY / 4) + (g >> 1) * RT + 32 * ks + 8 * jj + 4 * hh;
                    const u32x4 sv = *reinterpret_cast<const u32x4 *>(vsp);
                    const u32x4 zv = *reinterpret_cast<const u32x4 *>(vsp + W::SB_ARRAY / 4);
                    // 2^(block maximum - round maximum) * P_UP (2^8, so that the lo part stays a normal f16)
                    const float f = __builtin_amdgcn_exp2f(bmax_lds[(n & 7) * W::BSTRIDE + 2 * ks + (j >> 1)] - nm + 8.0f);
                    const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w}, zw[4] = {zv.x, zv.y, zv.z, zv.w};
                    float x[4], lo[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float p = pt[e] * f;
                        zacc += p * half_bits_to_float(zw[e] >> sh);
                        x[e] = p * half_bits_to_float(sw[e] >> sh);
                        lo[e] = x[e] - __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x[e]) & 0xffffe000u);
                    }
                    // round toward zero: exact truncation to the hi part
                    const uint32_t hi0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x[0], x[1]));
                    const uint32_t hi1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x[2], x[3]));
                    const uint32_t lo0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo[0], lo[1]));
                    const uint32_t lo1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo[2], lo[3]));
                    // the hi lane (n < 8) feeds hi parts and wants the other lane's hi parts of tokens 4-7; the lo
                    // lane feeds lo parts and wants the other lane's lo parts of tokens 0-3
                    const uint32_t send0 = hh ? hi0 : lo0, send1 = hh ? hi1 : lo1;
                    const uint32_t recv0 = uint32_t(__builtin_amdgcn_update_dpp(0, int(send0), 0x128, 0xf, 0xf, false));  // row_ror 8
                    const uint32_t recv1 = uint32_t(__builtin_amdgcn_update_dpp(0, int(send1), 0x128, 0xf, 0xf, false));
                    uint32_t o[4] = {hh ? recv0 : hi0, hh ? recv1 : hi1, hh ? lo0 : recv0, hh ? lo1 : recv1};
                    // (pinned: left alone, the compiler moves an operand's arithmetic down to its use, behind the wait for the values)
                    asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]));
                    p_op[sl] = as_half8(o[0], o[1], o[2], o[3]);
                }
            }
            if (more) raise(W::C_BUILT);  // this wave is through with the round's scores, scales and biases

            // ---- phase C: O += P V, one k-step per value slot as the slots land ---------------------
            const unsigned char *vb = lds_raw + W::V_OFF;
            auto read_values = [&](int sl, ValRegs<BITS> &vreg) {
                const int jj = sl == 4 ? (j & 1) : j;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int tk = 32 * (2 * sl + b2) + 8 * jj + e;
                    vreg.w[e] = *reinterpret_cast<const uint32_t *>(vb + tk * RB + ((val_lane_offset<BITS>(g, n) + jj * (RB / 4)) & (RB - 1)));
                }
            };
            auto add_values = [&](int sl, const ValRegs<BITS> &vreg) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(p_op[sl], val_operand<BITS>(vreg, e, n), acc[e], 0, 0, 0);
                }
            };
            const bool fifth = extra && b2 == 0;
            // (a short round: not every k-step of this wave has tokens)
            auto has_tokens = [&](int sl) { return uint32_t(2 * (2 * sl + b2)) < nb; };
            if (nb >= 16 && peek(W::C_SLOT + 3) >= W::V_LOADERS * (round + 1)) {
                // slots 0-3 are there already (the slots land in order): every read at once
                ValRegs<BITS> vreg[4];
#pragma unroll
                for (int sl = 0; sl < 4; sl++) read_values(sl, vreg[sl]);
#pragma unroll
                for (int sl = 0; sl < 4; sl++) add_values(sl, vreg[sl]);
            } else {
#pragma unroll
                for (int sl = 0; sl < 4; sl++) {
                    if (!has_tokens(sl)) continue;
                    await(W::C_SLOT + sl, W::V_LOADERS * (round + 1));  // value slot sl is in LDS
                    ValRegs<BITS> vreg;
                    read_values(sl, vreg);
                    add_values(sl, vreg);
                }
            }
            if (fifth) {
                await(W::C_SLOT + 4, W::V_LOADERS * (round + 1));
                ValRegs<BITS> vreg;
                read_values(4, vreg);
                add_values(4, vreg);
            }
            if (more) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the value codes are in registers
                raise(W::C_DONE);
            }
        }

        // ---- epilogue: the two waves of a group add up, wave 2g writes the partial ---------------------
        {
            // the head's bias sum: over the four lane groups and the two lanes of the head
            float z = across_rows<16, 64>(zacc, SumOp());
            z += dpp<0x128>(z);
            if (j == 0 && n < 8) zs_lds[wave * 8 + n] = z;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        floatx4 mine[4];  // head 4j + i (j < 2), dims 64 g + 4n .. + 3
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float zb = zs_lds[wave * 8 + ((4 * j + i) & 7)] * (1.0f / P_UP);
#pragma unroll
            for (int e = 0; e < 4; e++) mine[i][e] = across_rows<32, 64>(acc[e][i], SumOp()) * unscale + zb;
        }
        // (the key area is free: the key loaders request nothing after the last round, and every wave is
        // past the last round's scores, having built its operands from them)
        floatx4 *x_o = reinterpret_cast<floatx4 *>(lds_raw + W::X_OFF);  // [group][lane < 32][4 rows]
        if (b2 == 1) {
            if (j < 2) {
#pragma unroll
                for (int i = 0; i < 4; i++) x_o[(g * 32 + lane) * 4 + i] = mine[i];
            }
            raise(W::C_MERGE + g);
            leave();
            return;
        }
        await(W::C_MERGE + g, 1);
        if (wave == 0 && j == 0 && n < 8) {
            const size_t slot = size_t(split) * a.heads + kv * 8 + n;
            *reinterpret_cast<floatx2 *>(a.part_ml + 2 * slot) = floatx2{m_run, marked(l_run)};
        }
        if (j < 2) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const size_t slot = size_t(split) * a.heads + kv * 8 + 4 * j + i;
                *reinterpret_cast<floatx4 *>(a.part_o + slot * DIM + 64 * g + 4 * n) = mine[i] + x_o[(g * 32 + lane) * 4 + i];
            }
        }
    }
    leave();
}

// Merges the splits of one (q head, row): weights 2^(m_c - M), then the gate
// (reference: attention_reduce / attention_reduce_rows,
// kernels/attention.metal:367-409, kernels/attention_rows.metal:296-342).
struct ReduceArgs {
    const float *part_o;
    const float *part_ml;
    const float *q_and_gate;
    float *out;
    uint32_t heads, capacity, nsplits, rows;
    const saetta_token_params *tp;
    uint32_t decode_len;
};

constexpr uint32_t MAX_SPLITS = 256;  // workgroups per kv head: 2 kv heads fill 512 slots of 256 CUs

// Partials of saetta_attn_decode_quant_static, the entry point that allocates nothing: room for one
// query row, 16 q heads and the most splits a launch uses: part_o f32 [256][16][256] (4 MiB), then
// part_ml f32 [256][16][2] (32 KiB).  Every device the library runs on holds its own copy of the
// array at its own address, until the process ends.  In host code the array's name is only a
// stand-in for hipGetSymbolAddress, never a device address: setup_decode asks for the address once
// per device and everything else uses g_static_scratch[device].
constexpr uint32_t STATIC_MAX_HEADS = 16;
constexpr size_t STATIC_PART_O_FLOATS = size_t(MAX_SPLITS) * STATIC_MAX_HEADS * DIM;
constexpr size_t STATIC_PART_ML_FLOATS = size_t(MAX_SPLITS) * STATIC_MAX_HEADS * 2;
static __device__ __align__(256) float scratch[STATIC_PART_O_FLOATS + STATIC_PART_ML_FLOATS];
constexpr int STATIC_MAX_DEVICES = 64;
float *g_static_scratch[STATIC_MAX_DEVICES] = {};

// One workgroup per (q head, row, 16 dims of the head): wave w takes a quarter of the splits, lane
// (slot = lane / 4, quad = lane % 4) up to four of them and four dims.  Every load is requested before
// anything is waited for; a wave sums its splits relative to its own maximum, so that the four waves
// meet once, through LDS.
constexpr int REDUCE_DIMS = 16;
__global__ __launch_bounds__(256) void attention_reduce_kernel(ReduceArgs a) {
    __shared__ float wave_m[4], wave_l[4];
    __shared__ floatx4 wave_o[4][4];
    const uint32_t h = blockIdx.x, row = blockIdx.y, slice = blockIdx.z;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, slot = lane >> 2, quad = lane & 3;
    const float *ml = a.part_ml + size_t(2) * row * a.nsplits * a.heads;
    const float *po = a.part_o + size_t(row) * a.nsplits * a.heads * DIM;
    // splits of this wave: per_wave (a multiple of 16) from per_wave * wave on; of this lane: slot + 16 i
    const uint32_t per_wave = (a.nsplits + 63) / 64 * 16;
    constexpr int PER_LANE = MAX_SPLITS / 64;
    // Slots past the splits at work hold old values: they are dropped by select, never multiplied.
    floatx2 mlv[PER_LANE];
    floatx4 pv[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; i++) {
        const uint32_t c = per_wave * wave + slot + 16 * i;
        mlv[i] = floatx2{NO_SCORE, 0.0f};
        pv[i] = floatx4{0, 0, 0, 0};
        if (16 * uint32_t(i) < per_wave && c < a.nsplits) {
            mlv[i] = *reinterpret_cast<const floatx2 *>(ml + 2 * (size_t(c) * a.heads + h));
            pv[i] = *reinterpret_cast<const floatx4 *>(po + (size_t(c) * a.heads + h) * DIM + REDUCE_DIMS * slice + 4 * quad);
        }
    }
    const size_t qh = size_t(row) * a.heads + h;
    const float g = tid < REDUCE_DIMS ? a.q_and_gate[qh * 2 * DIM + DIM + REDUCE_DIMS * slice + tid] : 0.0f;
    const uint32_t max_len = min(a.decode_len ? a.tp->kv_len : a.tp->position + a.rows, a.capacity);
    const uint32_t nblocks = (max_len + BLOCK - 1) / BLOCK;
    const uint32_t parts = min(a.nsplits, nblocks);
    float m[PER_LANE], mx = NO_SCORE;
#pragma unroll
    for (int i = 0; i < PER_LANE; i++) {
        const bool live = 16 * uint32_t(i) < per_wave && per_wave * wave + slot + 16 * i < parts;
        m[i] = live ? mlv[i][0] : NO_SCORE;
        if (!live) mlv[i][1] = 0.0f, pv[i] = floatx4{0, 0, 0, 0};
        mx = fmaxf(mx, m[i]);
    }
    mx = group_reduce<64>(mx, MaxOp());  // the wave's maximum
    float l = 0.0f;
    floatx4 o = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < PER_LANE; i++) {
        const float w = m[i] > 0.5f * NO_SCORE ? __builtin_amdgcn_exp2f(m[i] - mx) : 0.0f;
        l += w * mlv[i][1];
        o += pv[i] * w;
    }
    // over the 16 slots (lanes 4 apart: two steps inside a row of 16 lanes, two across rows); l is the same in the four quads
    l += dpp<0x124>(l), l += dpp<0x128>(l);  // row_ror 4, row_ror 8
    l = across_rows<16, 64>(l, SumOp());
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float x = o[e];
        x += dpp<0x124>(x), x += dpp<0x128>(x);
        o[e] = across_rows<16, 64>(x, SumOp());
    }
    if (lane == 0) wave_m[wave] = mx, wave_l[wave] = l;
    if (lane < 4) wave_o[wave][lane] = o;  // (lane = quad)
    __syncthreads();
    if (tid < REDUCE_DIMS) {
        const float M = fmaxf(fmaxf(wave_m[0], wave_m[1]), fmaxf(wave_m[2], wave_m[3]));
        float total = 0.0f, sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float f = wave_m[w] > 0.5f * NO_SCORE ? __builtin_amdgcn_exp2f(wave_m[w] - M) : 0.0f;
            total += f * wave_l[w];
            sum += f * wave_o[w][tid >> 2][tid & 3];
        }
        a.out[qh * DIM + REDUCE_DIMS * slice + tid] = sum * __builtin_amdgcn_rcpf(total) * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
    }
}

uint32_t splits_for(uint32_t capacity, uint32_t wanted) {
    // Never more than the 128-token chunks of the capacity, so that scratch sized as
    // rows * ceil(capacity / 128) * heads partials is always enough.
    const uint32_t chunks = (capacity + SAETTA_CHUNK - 1) / SAETTA_CHUNK;
    uint32_t s = chunks < MAX_SPLITS ? chunks : MAX_SPLITS;
    if (wanted && wanted < s) s = wanted;
    return s ? s : 1;
}

// One to four rows over codes: from this capacity on the kernel whose loader waves keep a workgroup's share in
// LDS, the keys first, is the faster one at every length (one row, 8-bit, against the register kernels: 10.0
// against 11.0 us per layer at 4k tokens, 10.1 against 12.5 at 32k, 29.7 against 31.1 at 131k; shares of more
// than one round in alternate halves of LDS: 13.4 against 14.1 us at 40k for the ring of four 64-token slots
// that served there before, 28.3 against 29.7 at 150k, 4-bit, for the two-workgroups-per-CU kernel).
constexpr uint32_t KEYS_FIRST_FROM = 24 * 1024;

template <int BITS, int TILES, bool PACKED>
void launch_partial(hipStream_t stream, const PartialArgs &a, bool one_per_cu, bool keys_first) {
    void (*kernel)(PartialArgs);
    int lds_bytes;
    if constexpr (BITS != 16) {
        if (keys_first) {
            auto launch = [&](auto rows_c) {
                constexpr int MR = decltype(rows_c)::value;
                using W = KeysFirst<BITS, MR>;
                attention_partial_kernel_s<BITS, MR><<<dim3(a.nsplits, a.kv_heads), (W::LOADERS + W::WAVES) * 64, W::LDS_BYTES, stream>>>(a);
            };
            if (a.rows == 1) launch(std::integral_constant<int, 1>());
            else if (a.rows == 2) launch(std::integral_constant<int, 2>());
            else if (a.rows == 3) launch(std::integral_constant<int, 3>());
            else launch(std::integral_constant<int, 4>());
            return;
        }
    }
    if constexpr (TILES == 1 && BITS != 16 && PACKED) {
        if (one_per_cu) {
            kernel = attention_partial_kernel_p<BITS>;
            lds_bytes = Shape<BITS, TILES, PACKED, ITB_ONE_PER_CU>::LDS_BYTES;
        } else {
            kernel = attention_partial_kernel_1<BITS>;
            lds_bytes = Shape<BITS, TILES, PACKED, ITB_TWO_PER_CU>::LDS_BYTES;
        }
    } else if constexpr (PACKED) {
        kernel = attention_partial_kernel_p<BITS>;  // f16 cache: its registers do not fit two waves
        lds_bytes = Shape<BITS, TILES, PACKED, ITB_ONE_PER_CU>::LDS_BYTES;
    } else {
        kernel = attention_partial_kernel_n<BITS, TILES>;
        lds_bytes = Shape<BITS, TILES, PACKED, itb_rows<TILES>()>::LDS_BYTES;
    }
    // (the dynamic LDS limit of every variant was raised in setup_decode)
    kernel<<<dim3(a.nsplits, a.kv_heads), THREADS, lds_bytes, stream>>>(a);
}

template <int BITS>
void launch_partial_rows(hipStream_t stream, const PartialArgs &a, bool one_per_cu, bool keys_first) {
    if (a.rows == 1) {
        launch_partial<BITS, 1, true>(stream, a, one_per_cu, keys_first);
    } else if (a.rows == 2) {
        launch_partial<BITS, 1, false>(stream, a, one_per_cu, keys_first);
    } else if (a.rows <= 4) {
        launch_partial<BITS, 2, false>(stream, a, one_per_cu, keys_first);
    } else {
        launch_partial<BITS, 4, false>(stream, a, one_per_cu, keys_first);
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
    // Byte offsets into the cache are 32-bit: capacity * kv_heads * 512 B (the f16 row) must fit.
    SAETTA_REQUIRE(capacity > 0 && uint64_t(capacity) * kv_heads * 512 < (uint64_t(1) << 31), SAETTA_E_SHAPE,
                   "%s: capacity %u out of range", what, capacity);
    // Whole 16-token blocks are read: the last one must lie inside the cache (the reference's caches
    // are multiples of 128, src/gpu_layers.rs:199).
    SAETTA_REQUIRE(capacity % BLOCK == 0, SAETTA_E_SHAPE, "%s: capacity %u is not a multiple of 16", what, capacity);
    SAETTA_REQUIRE(q && kdata && vdata && part_o && part_ml && q_and_gate && out && d_tp, SAETTA_E_NULL,
                   "%s: null buffer", what);
    SAETTA_REQUIRE(bits == 16 || (ks && kz && vs && vz), SAETTA_E_NULL, "%s: null scales or biases", what);
    SAETTA_REQUIRE(aligned(q, 16) && aligned(kdata, 16) && aligned(vdata, 16) && aligned(part_o, 16) &&
                       aligned(part_ml, 8) && aligned(q_and_gate, 4) && aligned(out, 4),
                   SAETTA_E_ALIGN, "%s: q, cache and scratch must be 16-byte aligned", what);
    SAETTA_REQUIRE(bits == 16 || (aligned(ks, 8) && aligned(kz, 8) && aligned(vs, 8) && aligned(vz, 8)),
                   SAETTA_E_ALIGN, "%s: scales and biases must be 8-byte aligned", what);
    if (int rc = ensure_device()) return rc;
    uint32_t nsplits = splits_for(capacity, wanted_splits);
    // One to four rows over codes in a cache of 24k tokens and more go to the kernel with loader waves, a
    // one-workgroup-per-CU kernel at every length: a share of up to 17 blocks (the kernel sees the length
    // when it runs: a step at 32k tokens is one round in a cache of any size) is one round, a longer one
    // rounds of 8 blocks.  SAETTA_STAGE_NO_LOADERS keeps to the register kernels (the caller's choice of
    // kernel family, as DecodeAttention.kernel is in the reference, src/attention.rs:36-38).
    // The register kernels: one workgroup per CU (half as many splits, each twice as long) or two.  Two
    // rows and more and a half cache need the whole register file anyway; one row over codes fits two
    // workgroups per CU, which pays only for long contexts: up to 64k tokens the shorter merge of half as
    // many partials is worth more (measured: 19.4 against 20.6 us per layer at 32k, 28.3 against 29.7 at
    // 64k, but 44 against 35 at 146k, 4-bit).  Both stages derive the same number from the same arguments.
    const bool keys_first = rows <= 4 && bits != 16 && capacity >= KEYS_FIRST_FROM && !(stages & SAETTA_STAGE_NO_LOADERS);
    const bool one_per_cu = rows >= 2 || bits == 16 || capacity <= 80 * 1024 || keys_first;
    if (one_per_cu && nsplits > MAX_SPLITS / 2) nsplits = MAX_SPLITS / 2;
    if (stages & SAETTA_STAGE_PARTIAL) {
        PartialArgs a{q,     kdata,    vdata,    ks,    kz,   vs,      vz,   part_o, part_ml,
                      heads, kv_heads, capacity, scale, rows, nsplits, d_tp, decode_len ? 1u : 0u, device_status_word()};
        if (bits == 8) {
            launch_partial_rows<8>(stream, a, one_per_cu, keys_first);
        } else if (bits == 4) {
            launch_partial_rows<4>(stream, a, one_per_cu, keys_first);
        } else {
            launch_partial_rows<16>(stream, a, one_per_cu, keys_first);
        }
    }
    if (stages & SAETTA_STAGE_REDUCE) {
        ReduceArgs r{part_o, part_ml, q_and_gate, out, heads, capacity, nsplits, rows, d_tp, decode_len ? 1u : 0u};
        attention_reduce_kernel<<<dim3(heads, rows, DIM / REDUCE_DIMS), 256, 0, stream>>>(r);
    }
    return launch_status(what);
}

}  // namespace

namespace {
template <int BITS, int TILES, bool PACKED, int ITB>
int raise_lds(void (*kernel)(PartialArgs)) {
    static_assert(Shape<BITS, TILES, PACKED, ITB>::LDS_BYTES <= 160 * 1024, "LDS of a CU");
    if (Shape<BITS, TILES, PACKED, ITB>::LDS_BYTES <= 48 * 1024) return 0;
    return int(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   Shape<BITS, TILES, PACKED, ITB>::LDS_BYTES));
}
template <int BITS, int M>
int raise_lds_keys_first() {
    return int(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_partial_kernel_s<BITS, M>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, KeysFirst<BITS, M>::LDS_BYTES));
}
template <int BITS>
int raise_lds_of_bits() {
    if (int rc = raise_lds<BITS, 1, true, ITB_ONE_PER_CU>(attention_partial_kernel_p<BITS>)) return rc;
    if (int rc = raise_lds<BITS, 1, false, itb_rows<1>()>(attention_partial_kernel_n<BITS, 1>)) return rc;
    if (int rc = raise_lds<BITS, 2, false, itb_rows<2>()>(attention_partial_kernel_n<BITS, 2>)) return rc;
    return raise_lds<BITS, 4, false, itb_rows<4>()>(attention_partial_kernel_n<BITS, 4>);
}
}  // namespace

int setup_decode() {
    if (int rc = load_kernel(reinterpret_cast<const void *>(attention_reduce_kernel))) return rc;
    {
        // (runs once per device, with that device current)
        int dev = 0;
        if (hipError_t e = hipGetDevice(&dev)) return int(e);
        if (dev < 0 || dev >= STATIC_MAX_DEVICES) return int(hipErrorInvalidDevice);
        float *ptr = nullptr;
        if (hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch))) return int(e);
        g_static_scratch[dev] = ptr;
    }
    if (int rc = raise_lds_keys_first<8, 1>()) return rc;
    if (int rc = raise_lds_keys_first<8, 2>()) return rc;
    if (int rc = raise_lds_keys_first<8, 3>()) return rc;
    if (int rc = raise_lds_keys_first<8, 4>()) return rc;
    if (int rc = raise_lds_keys_first<4, 1>()) return rc;
    if (int rc = raise_lds_keys_first<4, 2>()) return rc;
    if (int rc = raise_lds_keys_first<4, 3>()) return rc;
    if (int rc = raise_lds_keys_first<4, 4>()) return rc;
    if (int rc = raise_lds_of_bits<8>()) return rc;
    if (int rc = raise_lds_of_bits<4>()) return rc;
    if (int rc = raise_lds_of_bits<16>()) return rc;
    if (int rc = raise_lds<8, 1, true, ITB_TWO_PER_CU>(attention_partial_kernel_1<8>)) return rc;
    return raise_lds<4, 1, true, ITB_TWO_PER_CU>(attention_partial_kernel_1<4>);
}
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

extern "C" size_t saetta_static_scratch_bytes(void) { return sizeof(float) * (STATIC_PART_O_FLOATS + STATIC_PART_ML_FLOATS); }

extern "C" int saetta_attn_decode_quant_static(saetta_stream_t stream, int bits, const float *q,
                                               saetta_quant_rows keys, saetta_quant_rows values,
                                               const float *q_and_gate, float *out, saetta_decode_params p,
                                               const saetta_token_params *d_tp, uint32_t stages) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "attn_decode_quant_static: bits %d (8 or 4)", bits);
    // What the partials of this launch need against what the static array holds (the number of
    // splits never exceeds 256, so only the heads can outgrow it).
    const size_t need = saetta_part_o_bytes(p.heads, p.capacity, 1) + saetta_part_ml_bytes(p.heads, p.capacity, 1);
    SAETTA_REQUIRE(p.heads <= STATIC_MAX_HEADS && need <= saetta_static_scratch_bytes(), SAETTA_E_SCRATCH,
                   "attn_decode_quant_static: %u heads need %zu bytes of partials, the static scratch holds %zu "
                   "(up to %u heads); use saetta_attn_decode_quant with scratch of the caller's",
                   p.heads, need, saetta_static_scratch_bytes(), STATIC_MAX_HEADS);
    if (int rc = ensure_device()) return rc;
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return fail(int(e), "attn_decode_quant_static: %s", hipGetErrorString(e));
    float *part_o = (dev >= 0 && dev < STATIC_MAX_DEVICES) ? g_static_scratch[dev] : nullptr;
    SAETTA_REQUIRE(part_o, SAETTA_E_DEVICE, "attn_decode_quant_static: no static scratch on device %d", dev);
    return run_attention(as_stream(stream), bits, q, keys.data, values.data, keys.scales, keys.biases,
                         values.scales, values.biases, part_o, part_o + STATIC_PART_O_FLOATS, q_and_gate, out,
                         p.heads, p.kv_heads, p.capacity, p.scale, 1, 0, d_tp, true, stages,
                         "attn_decode_quant_static");
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
