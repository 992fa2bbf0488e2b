// Flash-style causal prefill attention for gfx950 (MI355X).
//
// What it computes (reference: attention_prefill::encode,
// src/attention_prefill.rs:39-72, kernel attention_fa<TQ>,
// kernels/attention_prefill.metal:38-169; over a quantized cache
// src/prefill.rs:1735-1776, kernels/attention_rows_q.metal:55-344): for the
// chunk's token i and each of the 16 q heads
//     out[i, h] = softmax(q[i, h] K^T * scale) V * sigmoid(gate[i, h])
// over keys 0 ..= pos + i, 8 q heads sharing one kv head, head dim 256.
// q is f16; the cache is f16 or 8/4-bit codes read in place.  A quantized
// cache is seen "through half": every value is f16(f32(s)*code + f32(z)),
// exactly what round_trip_as_half (src/kv_quant.rs:119-125) gives the CPU path.
//
// Two kernels.
//
// prefill_prepare_kernel<16|8|4> turns the keys and values the chunk can see into
// f16 tile images in a workspace, one image per (kv head, block of 32 keys): the K tile
// [32 keys][256 dims] and the transposed V^T tile [256 dims][32 keys], laid out byte for
// byte as the attention kernel wants them in LDS (padded rows, V^T keys in the order the
// MFMA accumulator hands them out).  The dequantization happens here, once per key, with
// exactly the arithmetic of round_trip_as_half, instead of once per workgroup that walks
// the key; it costs one pass over the cache (a few microseconds).
//
// attention_prefill_kernel: workgroup (token tile of 16, kv head), 4 waves (one per SIMD);
// wave w owns 4 tokens x 8 heads = 32 query rows, one 32-row MFMA tile.  Keys are walked in
// blocks of 32 whose images are copied global -> LDS by global_load_lds_dwordx4 (no vector
// registers, no vector ALU) into three rotating buffers, two blocks ahead.  Every wave
// computes with v_mfma_f32_32x32x16_f16
//     S^T = K Q^T      (A = K rows from LDS, B = Q^T held in registers)
//     O^T += V^T P^T   (A = V^T rows from LDS, B = P^T from the S^T registers)
// Both products are transposed so that a lane always owns one query row: in the 32x32
// accumulator layout a lane holds column l % 32, so the row's running max and sum, the
// rescale of O and the final 1/l and gate are plain per-lane values and the softmax needs one
// cross-lane exchange per block.  The loop is software-pipelined inside each wave, because
// MFMA and vector instructions of one wave run side by side when they are independent:
//   stage A   MFMA: S^T of block kb+1      |  VALU: exp / sum / pack of block kb
//   stage B   MFMA: O^T += V^T P^T (kb)    |  VALU: scale and row max of block kb+1
// with one barrier per block.  The running max is only raised when a block exceeds it by
// more than 2^8 (lazy rescale), so O is rarely rescaled.  Tiles are issued heaviest first and
// there are two per CU, which evens out the causal imbalance.
#include "common.hpp"

#include <mutex>

namespace saetta {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_ __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int DIM = SAETTA_HEAD_DIM;
constexpr int PREP_THREADS = 256;       // the prepare kernel's workgroup
constexpr int WAVES = 8;                // two per SIMD: one's softmax runs under the other's MFMAs
constexpr int THREADS = 64 * WAVES;
constexpr int TQ = 4 * WAVES;           // tokens per workgroup: a wave owns 4 tokens x 8 heads = 32 rows
constexpr int BK = 32;                  // keys per block
constexpr int K_STRIDE = DIM * 2 + 16;  // bytes per key row of the K tile (padded against bank conflicts)
constexpr int V_STRIDE = BK * 2 + 16;   // bytes per dim row of the V^T tile
constexpr int K_BYTES = BK * K_STRIDE;
constexpr int V_BYTES = DIM * V_STRIDE;  // V^T tile: row = dim, 32 keys in vt_pos order (+ padding)
constexpr int IMG_BYTES = (K_BYTES + V_BYTES + 1023) / 1024 * 1024;  // one block's image, whole KB
constexpr float NO_SCORE = -1e30f;
constexpr float TAU = 8.0f;  // the reference max is raised only past this many powers of two

struct PrepareArgs {
    const void *kdata;
    const void *vdata;
    const uint16_t *kscales, *kbiases, *vscales, *vbiases;
    unsigned char *images;  // [kv head][block][IMG_BYTES]
    uint32_t kv_heads, nblocks;
    uint32_t key_limit;  // pos + tokens: rows the cache holds; keys from here on are zeros
};

struct PrefillArgs {
    const uint16_t *q;  // f16 [tokens][heads][256]
    const unsigned char *images;
    const float *q_and_gate;
    float *out;
    uint32_t heads, kv_heads, pos, tokens;
    float scale;
    uint32_t nblocks;  // images per kv head
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, int(bytes), 0x00020000);
}

template <int BITS>
constexpr int row_bytes() {
    return BITS == 16 ? 512 : BITS * 32;
}

__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
    half2_ h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}

// f16(f32(s) * code + f32(z)): s * code is exact in f32, so the fma rounds as the CPU's
// multiply-then-add does, and the conversion rounds to nearest even.
__device__ __forceinline__ float dequant(float s, float z, uint32_t code) { return fmaf(s, float(code), z); }

// Code i (0..) of a little-endian packed word.
template <int BITS>
__device__ __forceinline__ uint32_t code_of(uint32_t w, int i) {
    return BITS == 8 ? ((w >> (8 * i)) & 0xffu) : ((w >> (4 * i)) & 0xfu);
}

// ---- staging registers: what one thread fetches for one key block ----------------
// K: thread (key = t / 8, piece = t % 8) takes 32 dims of one key.
// V: thread (dq = t % 64, kq = t / 64) takes 4 dims of 8 keys.
template <int BITS>
struct Stage {
    uint32_t k[BITS == 16 ? 16 : BITS];     // 32 dims: 64 B (f16), 32 B (8-bit), 16 B (4-bit)
    uint32_t v[8][BITS == 16 ? 2 : 1];      // per key 4 dims: 8 B (f16), 4 B (8-bit), 2 B (4-bit)
    uint32_t ks, kz;                        // f16 scale and bias of (key, group of the piece)
    uint32_t vs[8], vz[8];                  // per key, group of dq
};

struct Rsrc {
    __amdgpu_buffer_rsrc_t k, v, ks, kz, vs, vz;
};

template <int BITS>
__device__ __forceinline__ void stage_load(Stage<BITS> &st, const Rsrc &r, uint32_t kvh, uint32_t key0, uint32_t kv,
                                           int tid) {
    constexpr int RB = row_bytes<BITS>();
    {
        const int key = tid >> 3, piece = tid & 7;
        const int row = int((key0 + key) * kvh + kv);
        const int off = row * RB + piece * (RB / 8);
        if constexpr (BITS == 8) {
            const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(r.k, off, 0, 0);
            const u32x4 y = __builtin_amdgcn_raw_buffer_load_b128(r.k, off + 16, 0, 0);
            st.k[0] = x.x, st.k[1] = x.y, st.k[2] = x.z, st.k[3] = x.w;
            st.k[4] = y.x, st.k[5] = y.y, st.k[6] = y.z, st.k[7] = y.w;
        } else if constexpr (BITS == 4) {
            const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(r.k, off, 0, 0);
            st.k[0] = x.x, st.k[1] = x.y, st.k[2] = x.z, st.k[3] = x.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(r.k, off + 16 * i, 0, 0);
                st.k[4 * i] = x.x, st.k[4 * i + 1] = x.y, st.k[4 * i + 2] = x.z, st.k[4 * i + 3] = x.w;
            }
        }
        if constexpr (BITS != 16) {
            const int soff = (row * 4 + (piece >> 1)) * 2;
            st.ks = __builtin_amdgcn_raw_buffer_load_b16(r.ks, soff, 0, 0);
            st.kz = __builtin_amdgcn_raw_buffer_load_b16(r.kz, soff, 0, 0);
        }
    }
    {
        const int dq = tid & 63, kq = tid >> 6;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int row = int((key0 + 8 * kq + i) * kvh + kv);
            const int off = row * RB + dq * (RB / 64);
            if constexpr (BITS == 8) {
                st.v[i][0] = __builtin_amdgcn_raw_buffer_load_b32(r.v, off, 0, 0);
            } else if constexpr (BITS == 4) {
                st.v[i][0] = uint16_t(__builtin_amdgcn_raw_buffer_load_b16(r.v, off, 0, 0));
            } else {
                const u32x2 x = __builtin_amdgcn_raw_buffer_load_b64(r.v, off, 0, 0);
                st.v[i][0] = x.x, st.v[i][1] = x.y;
            }
            if constexpr (BITS != 16) {
                const int soff = (row * 4 + (dq >> 4)) * 2;
                st.vs[i] = __builtin_amdgcn_raw_buffer_load_b16(r.vs, soff, 0, 0);
                st.vz[i] = __builtin_amdgcn_raw_buffer_load_b16(r.vz, soff, 0, 0);
            }
        }
    }
}

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, uint16_t(bits16));
}

// Where key `key` (0..31) of the block sits inside a V^T row: the order in which the
// S^T accumulator hands its keys to the P^T operand (see the kernel).
__device__ __forceinline__ constexpr int vt_pos(int key) {
    const int s = key >> 4, u = key & 15;
    return 16 * s + 8 * ((u & 7) >> 2) + 4 * (u >> 3) + (u & 3);
}

// Dequantizes the staged registers into the LDS tiles.  Keys at or past key_limit
// (the end of the chunk) are written as zeros: their probabilities are 0, and 0 * 0
// stays 0 whatever the cache rows hold.
template <int BITS>
__device__ __forceinline__ void stage_store(const Stage<BITS> &st, unsigned char *k_lds, unsigned char *v_lds,
                                            uint32_t key0, uint32_t key_limit, int tid) {
    {
        const int key = tid >> 3, piece = tid & 7;
        uint32_t o[16];
        if constexpr (BITS == 16) {
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] = st.k[i];
        } else {
            const float s = h2f(st.ks), z = h2f(st.kz);
            constexpr int PER = 32 / BITS;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t w = st.k[(2 * i) / PER];
                o[i] = pack_half2(dequant(s, z, code_of<BITS>(w, (2 * i) % PER)),
                                  dequant(s, z, code_of<BITS>(w, (2 * i + 1) % PER)));
            }
        }
        if (key0 + key >= key_limit) {
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] = 0;
        }
        u32x4 *dst = reinterpret_cast<u32x4 *>(k_lds + key * K_STRIDE + piece * 64);
#pragma unroll
        for (int i = 0; i < 4; i++) dst[i] = u32x4{o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]};
    }
    {
        const int dq = tid & 63, kq = tid >> 6;
        // keys 8kq..8kq+7: two runs of 4 neighbours in the row's key order
        const int p0 = vt_pos(8 * kq), p1 = vt_pos(8 * kq + 4);
        uint32_t w[4][4];  // [dim][pair of keys]
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            float x[2][4];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const bool live = key0 + 8 * kq + i + u < key_limit;
                if constexpr (BITS == 16) {
#pragma unroll
                    for (int d = 0; d < 4; d++) x[u][d] = live ? h2f(st.v[i + u][d >> 1] >> (16 * (d & 1))) : 0.0f;
                } else {
                    const float s = h2f(st.vs[i + u]), z = h2f(st.vz[i + u]);
#pragma unroll
                    for (int d = 0; d < 4; d++) x[u][d] = live ? dequant(s, z, code_of<BITS>(st.v[i + u][0], d)) : 0.0f;
                }
            }
#pragma unroll
            for (int d = 0; d < 4; d++) w[d][i / 2] = pack_half2(x[0][d], x[1][d]);
        }
#pragma unroll
        for (int d = 0; d < 4; d++) {
            unsigned char *row = v_lds + (4 * dq + d) * V_STRIDE;
            *reinterpret_cast<u32x2 *>(row + 2 * p0) = u32x2{w[d][0], w[d][1]};
            *reinterpret_cast<u32x2 *>(row + 2 * p1) = u32x2{w[d][2], w[d][3]};
        }
    }
}

template <int BITS>
__global__ __launch_bounds__(PREP_THREADS) void prefill_prepare_kernel(PrepareArgs a) {
    constexpr int RB = row_bytes<BITS>();
    const uint32_t block = blockIdx.x, kv = blockIdx.y, kvh = a.kv_heads;
    const uint32_t cap_rows = a.key_limit * kvh;
    Rsrc rs;
    rs.k = make_rsrc(a.kdata, cap_rows * RB);
    rs.v = make_rsrc(a.vdata, cap_rows * RB);
    rs.ks = make_rsrc(a.kscales, BITS == 16 ? 0 : cap_rows * 8);
    rs.kz = make_rsrc(a.kbiases, BITS == 16 ? 0 : cap_rows * 8);
    rs.vs = make_rsrc(a.vscales, BITS == 16 ? 0 : cap_rows * 8);
    rs.vz = make_rsrc(a.vbiases, BITS == 16 ? 0 : cap_rows * 8);
    Stage<BITS> st;
    stage_load<BITS>(st, rs, kvh, block * BK, kv, threadIdx.x);
    unsigned char *img = a.images + (size_t(kv) * a.nblocks + block) * IMG_BYTES;
    stage_store<BITS>(st, img, img + K_BYTES, block * BK, a.key_limit, threadIdx.x);
}

// S^T = K Q^T of one block as one instruction stream: 16 LDS reads of K rows kept four ahead of
// the 16 MFMAs that use them.  kaddr: LDS byte address of the lane's key row (col) plus 16 hf.
// Ends with the wait states an MFMA result needs before vector ALU instructions may read it.
__device__ __forceinline__ void scores_block(floatx16 &s, const half8 (&q)[16], uint32_t kaddr) {
    half8 a0, a1, a2, a3;
#define SAETTA_S_STEP(A, Q, OFF, CNT)                                  \
    "s_waitcnt lgkmcnt(" #CNT ")\n"                                    \
    "v_mfma_f32_32x32x16_f16 %[s], %[" #A "], %[" #Q "], %[s]\n"       \
    "ds_read_b128 %[" #A "], %[addr] offset:" #OFF "\n"
#define SAETTA_S_LAST(A, Q, CNT)                                       \
    "s_waitcnt lgkmcnt(" #CNT ")\n"                                    \
    "v_mfma_f32_32x32x16_f16 %[s], %[" #A "], %[" #Q "], %[s]\n"
    asm volatile(
        "s_waitcnt lgkmcnt(0)\n"
        "ds_read_b128 %[a0], %[addr]\n"
        "ds_read_b128 %[a1], %[addr] offset:32\n"
        "ds_read_b128 %[a2], %[addr] offset:64\n"
        "ds_read_b128 %[a3], %[addr] offset:96\n"
        "s_waitcnt lgkmcnt(3)\n"
        "v_mfma_f32_32x32x16_f16 %[s], %[a0], %[q0], 0\n"
        "ds_read_b128 %[a0], %[addr] offset:128\n"
        SAETTA_S_STEP(a1, q1, 160, 3) SAETTA_S_STEP(a2, q2, 192, 3) SAETTA_S_STEP(a3, q3, 224, 3)
        SAETTA_S_STEP(a0, q4, 256, 3) SAETTA_S_STEP(a1, q5, 288, 3) SAETTA_S_STEP(a2, q6, 320, 3)
        SAETTA_S_STEP(a3, q7, 352, 3) SAETTA_S_STEP(a0, q8, 384, 3) SAETTA_S_STEP(a1, q9, 416, 3)
        SAETTA_S_STEP(a2, q10, 448, 3) SAETTA_S_STEP(a3, q11, 480, 3)
        SAETTA_S_LAST(a0, q12, 3) SAETTA_S_LAST(a1, q13, 2) SAETTA_S_LAST(a2, q14, 1) SAETTA_S_LAST(a3, q15, 0)
        "s_nop 15\n"
        "s_nop 3\n"
        : [s] "=&v"(s), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3)
        : [addr] "v"(kaddr), [q0] "v"(q[0]), [q1] "v"(q[1]), [q2] "v"(q[2]), [q3] "v"(q[3]), [q4] "v"(q[4]),
          [q5] "v"(q[5]), [q6] "v"(q[6]), [q7] "v"(q[7]), [q8] "v"(q[8]), [q9] "v"(q[9]), [q10] "v"(q[10]),
          [q11] "v"(q[11]), [q12] "v"(q[12]), [q13] "v"(q[13]), [q14] "v"(q[14]), [q15] "v"(q[15])
        : "memory");
#undef SAETTA_S_STEP
#undef SAETTA_S_LAST
}

// O^T += V^T P^T of one block, the same way: 16 reads of V^T rows four ahead of 16 MFMAs.
// vaddr: LDS byte address of the lane's dim row (col) of the V^T tile plus 16 hf; the tile of
// dims 32 mt .. 32 mt + 31 is 32 rows further, k-step sp 32 bytes further.
__device__ __forceinline__ void accumulate_block(floatx16 (&o)[8], const half8 (&p)[2], uint32_t vaddr) {
    half8 a0, a1, a2, a3;
#define SAETTA_O_STEP(A, ACC, P, OFF, CNT)                                   \
    "s_waitcnt lgkmcnt(" #CNT ")\n"                                          \
    "v_mfma_f32_32x32x16_f16 %[" #ACC "], %[" #A "], %[" #P "], %[" #ACC "]\n" \
    "ds_read_b128 %[" #A "], %[addr] offset:" #OFF "\n"
#define SAETTA_O_LAST(A, ACC, P, CNT)                                        \
    "s_waitcnt lgkmcnt(" #CNT ")\n"                                          \
    "v_mfma_f32_32x32x16_f16 %[" #ACC "], %[" #A "], %[" #P "], %[" #ACC "]\n"
    // read i serves MFMA i: i < 8 is (sp 0, mt i) at offset 2560 i, i >= 8 is (sp 1, mt i - 8) at 2560 (i - 8) + 32
    asm volatile(
        "s_waitcnt lgkmcnt(0)\n"
        "ds_read_b128 %[a0], %[addr]\n"
        "ds_read_b128 %[a1], %[addr] offset:2560\n"
        "ds_read_b128 %[a2], %[addr] offset:5120\n"
        "ds_read_b128 %[a3], %[addr] offset:7680\n"
        SAETTA_O_STEP(a0, o0, p0, 10240, 3) SAETTA_O_STEP(a1, o1, p0, 12800, 3) SAETTA_O_STEP(a2, o2, p0, 15360, 3)
        SAETTA_O_STEP(a3, o3, p0, 17920, 3) SAETTA_O_STEP(a0, o4, p0, 32, 3) SAETTA_O_STEP(a1, o5, p0, 2592, 3)
        SAETTA_O_STEP(a2, o6, p0, 5152, 3) SAETTA_O_STEP(a3, o7, p0, 7712, 3) SAETTA_O_STEP(a0, o0, p1, 10272, 3)
        SAETTA_O_STEP(a1, o1, p1, 12832, 3) SAETTA_O_STEP(a2, o2, p1, 15392, 3) SAETTA_O_STEP(a3, o3, p1, 17952, 3)
        SAETTA_O_LAST(a0, o4, p1, 3) SAETTA_O_LAST(a1, o5, p1, 2) SAETTA_O_LAST(a2, o6, p1, 1)
        SAETTA_O_LAST(a3, o7, p1, 0)
        : [o0] "+v"(o[0]), [o1] "+v"(o[1]), [o2] "+v"(o[2]), [o3] "+v"(o[3]), [o4] "+v"(o[4]), [o5] "+v"(o[5]),
          [o6] "+v"(o[6]), [o7] "+v"(o[7]), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3)
        : [addr] "v"(vaddr), [p0] "v"(p[0]), [p1] "v"(p[1])
        : "memory");
#undef SAETTA_O_STEP
#undef SAETTA_O_LAST
}

// The wait states after which vector ALU instructions may read what the last MFMAs wrote.
__device__ __forceinline__ void settle(floatx16 (&o)[8]) {
    asm volatile("s_nop 15\ns_nop 3\n"
                 : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]), "+v"(o[7]));
}

constexpr int NBUF = 3;
constexpr int LDS_BYTES = NBUF * IMG_BYTES;

__global__ __launch_bounds__(THREADS) void attention_prefill_kernel(PrefillArgs a) {
    // the image of block b lives in buffer b % 3
    extern __shared__ __attribute__((aligned(1024))) unsigned char tiles[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hf = lane >> 5;
    const uint32_t kv = blockIdx.y;
    const uint32_t ntiles = (a.tokens + TQ - 1) / TQ;
    const uint32_t tile = ntiles - 1 - blockIdx.x;  // the tiles with the most keys start first
    const uint32_t tok0 = tile * TQ + 4 * wave;     // this wave's first token
    const float c = a.scale * 1.4426950408889634f;  // scores are kept in units of log2(e)

    // Row of this lane: token tok0 + col / 8, head col % 8.
    const uint32_t tok = tok0 + (col >> 3);
    const uint32_t head = kv * 8 + (col & 7);

    // Keys this workgroup walks: up to what its last token sees; what this wave needs.
    const uint32_t wg_keys = a.pos + min(tile * TQ + TQ, a.tokens);
    const uint32_t nblocks = (wg_keys + BK - 1) / BK;
    const uint32_t wave_first_len = a.pos + tok0 + 1;            // keys the wave's first token sees
    const uint32_t wave_keys = a.pos + min(tok0 + 4, a.tokens);  // keys its last token sees
    const uint32_t wave_blocks = tok0 < a.tokens ? min((wave_keys + BK - 1) / BK, nblocks) : 0;
    const uint32_t full_blocks = min(wave_first_len / BK, wave_blocks);  // blocks that need no mask

    // Copies the image of block b into its LDS buffer: every lane moves 16 bytes per
    // instruction, a wave 1 KB, straight from global memory to LDS.
    const unsigned char *images = a.images + size_t(kv) * a.nblocks * IMG_BYTES;
    auto copy_block = [&](uint32_t b) {
        const unsigned char *src = images + size_t(b) * IMG_BYTES + lane * 16;
        unsigned char *dst = tiles + (b % NBUF) * IMG_BYTES;
        for (int i = wave; i < IMG_BYTES / 1024; i += WAVES) {
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(src + i * 1024),
                                             (void __attribute__((address_space(3))) *)(dst + i * 1024), 16, 0, 0);
        }
    };
    copy_block(0);
    if (nblocks > 1) copy_block(1);

    // Q^T operands: lane (col, hf), k-step st: dims 16 st + 8 hf .. + 7 of its row.
    half8 qb[16];
    {
        const uint32_t tk = min(tok, a.tokens - 1);
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.q + (size_t(tk) * a.heads + head) * DIM + 8 * hf);
#pragma unroll
        for (int st = 0; st < 16; st++) qb[st] = __builtin_bit_cast(half8, src[2 * st]);
    }

    floatx16 acc[8];
#pragma unroll
    for (int mt = 0; mt < 8; mt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[mt][r] = 0.0f;
    }
    float m_ref = NO_SCORE, l_sum = 0.0f;

    // Row maximum of a block's scaled scores (first half of the softmax).  Register r of the
    // accumulator is key 4 hf + r % 4 + 8 (r / 4) of the block; masked scores become NO_SCORE / c.
    auto mask_max = [&](floatx16 &s, uint32_t key0, bool masked) {
        float bm = NO_SCORE;
        if (masked) {
            const uint32_t len = a.pos + tok + 1;              // keys this row sees
            const uint32_t vis = len > key0 ? len - key0 : 0;  // of which in this block
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t key = 4 * hf + (r & 3) + 8 * (r >> 2);
                s[r] = key < vis ? s[r] : NO_SCORE;
            }
        }
#pragma unroll
        for (int r = 0; r < 16; r++) bm = fmaxf(bm, s[r]);
        bm = fmaxf(bm, __shfl_xor(bm, 32));
        return fmaxf(bm * c, NO_SCORE);
    };
    // Raises the reference maximum when a block tops it by more than 2^TAU, rescaling O and l.
    auto raise_max = [&](float bm) {
        if (__any(bm > m_ref + TAU)) {
            const float m_new = bm > m_ref + TAU ? bm : m_ref;
            const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
            m_ref = m_new;
            l_sum *= alpha;
#pragma unroll
            for (int mt = 0; mt < 8; mt++) {
#pragma unroll
                for (int r = 0; r < 16; r++) acc[mt][r] *= alpha;
            }
        }
    };
    // Second half of the softmax: probabilities 2^(s c - m), their sum, and the P^T operands
    // (k-step sp takes registers 8 sp .. 8 sp + 7, the order vt_pos mirrors).
    auto exp_pack = [&](const floatx16 &s, half8 (&pb)[2]) {
        float p[16];
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            p[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c, -m_ref));
            sum += p[r];
        }
        l_sum += sum;
#pragma unroll
        for (int sp = 0; sp < 2; sp++) {
            u32x4 w = {pack_half2(p[8 * sp], p[8 * sp + 1]), pack_half2(p[8 * sp + 2], p[8 * sp + 3]),
                       pack_half2(p[8 * sp + 4], p[8 * sp + 5]), pack_half2(p[8 * sp + 6], p[8 * sp + 7])};
            pb[sp] = __builtin_bit_cast(half8, w);
        }
    };
    // LDS addresses (bytes) of the lane's rows in buffer 0
    const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(tiles));
    const uint32_t k_lane = lds0 + col * K_STRIDE + 16 * hf;
    const uint32_t v_lane = lds0 + K_BYTES + col * V_STRIDE + 16 * hf;

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // blocks 0 and 1 are in LDS

    for (uint32_t kb = 0; kb < nblocks; kb++) {
        // Block kb + 2 goes where block kb - 1 was (every wave left it at the last barrier).
        if (kb + 2 < nblocks) copy_block(kb + 2);
        if (kb < wave_blocks) {
            const uint32_t buf = (kb % NBUF) * IMG_BYTES;
            floatx16 s;
            scores_block(s, qb, k_lane + buf);
            raise_max(mask_max(s, kb * BK, kb >= full_blocks));
            half8 pb[2];
            exp_pack(s, pb);
            accumulate_block(acc, pb, v_lane + buf);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    settle(acc);

    // ---- out = O / l * sigmoid(gate) ---------------------------------------------------
    // The lane's row sum is split over the two lane halves (each saw half the keys).
    const float l = l_sum + __shfl_xor(l_sum, 32);
    if (tok < a.tokens) {
        const float inv = 1.0f / l;
        const size_t row = size_t(tok) * a.heads + head;
        const float *gate = a.q_and_gate + row * 2 * DIM + DIM;
        float *out = a.out + row * DIM;
#pragma unroll
        for (int mt = 0; mt < 8; mt++) {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int d0 = 32 * mt + 8 * q4 + 4 * hf;
                const float4 g = *reinterpret_cast<const float4 *>(gate + d0);
                float4 o;
                o.x = acc[mt][4 * q4 + 0] * inv / (1.0f + __expf(-g.x));
                o.y = acc[mt][4 * q4 + 1] * inv / (1.0f + __expf(-g.y));
                o.z = acc[mt][4 * q4 + 2] * inv / (1.0f + __expf(-g.z));
                o.w = acc[mt][4 * q4 + 3] * inv / (1.0f + __expf(-g.w));
                *reinterpret_cast<float4 *>(out + d0) = o;
            }
        }
    }
}

// Workspace the library owns when the caller passes none: grown on demand, one per device.
struct OwnedWorkspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};
OwnedWorkspace g_owned[16];
std::mutex g_owned_mutex;

size_t workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t kv_heads) {
    const size_t blocks = (size_t(pos) + tokens + BK - 1) / BK;
    return blocks * kv_heads * IMG_BYTES;
}

int run_prefill(hipStream_t stream, int bits, const uint16_t *q, const void *kdata, const void *vdata,
                const uint16_t *ks, const uint16_t *kz, const uint16_t *vs, const uint16_t *vz,
                const float *q_and_gate, float *out, saetta_flash_params p, void *workspace, size_t workspace_size,
                const char *what) {
    SAETTA_REQUIRE(bits == 16 || bits == 8 || bits == 4, SAETTA_E_BITS, "%s: bits %d", what, bits);
    SAETTA_REQUIRE(p.kv_heads > 0 && p.heads == p.kv_heads * SAETTA_GQA_GROUP, SAETTA_E_SHAPE,
                   "%s needs 8 q heads per kv head (heads %u, kv heads %u)", what, p.heads, p.kv_heads);
    SAETTA_REQUIRE(q && kdata && vdata && q_and_gate && out, SAETTA_E_NULL, "%s: null buffer", what);
    SAETTA_REQUIRE(bits == 16 || (ks && kz && vs && vz), SAETTA_E_NULL, "%s: null scales or biases", what);
    SAETTA_REQUIRE(aligned(q, 16) && aligned(kdata, 16) && aligned(vdata, 16) && aligned(q_and_gate, 16) &&
                       aligned(out, 16) && aligned(workspace, 16),
                   SAETTA_E_ALIGN, "%s: buffers must be 16-byte aligned", what);
    const uint64_t rows = uint64_t(p.pos) + p.tokens;  // the cache holds the chunk's rows too
    SAETTA_REQUIRE(rows * p.kv_heads * 512 < (uint64_t(1) << 31), SAETTA_E_SHAPE, "%s: pos + tokens %llu out of range",
                   what, (unsigned long long)rows);
    if (int rc = ensure_device()) return rc;
    if (p.tokens == 0) return SAETTA_OK;
    const size_t need = workspace_bytes(p.pos, p.tokens, p.kv_heads);
    if (workspace) {
        SAETTA_REQUIRE(workspace_size >= need, SAETTA_E_SCRATCH, "%s: workspace of %zu bytes, %zu needed", what,
                       workspace_size, need);
    } else {
        // No workspace given: use (and grow) the library's own.  This allocates, so it cannot be
        // used under stream capture; work queued on other streams must not share it.
        int dev = 0;
        (void)hipGetDevice(&dev);
        std::lock_guard<std::mutex> lock(g_owned_mutex);
        OwnedWorkspace &w = g_owned[dev & 15];
        if (w.bytes < need) {
            if (w.ptr) {
                (void)hipDeviceSynchronize();
                (void)hipFree(w.ptr);
            }
            w.ptr = nullptr;
            w.bytes = 0;
            hipError_t e = hipMalloc(&w.ptr, need);
            if (e != hipSuccess) return fail(int(e), "%s: workspace of %zu bytes: %s", what, need, hipGetErrorString(e));
            w.bytes = need;
        }
        workspace = w.ptr;
    }
    const uint32_t nblocks = uint32_t((rows + BK - 1) / BK);
    PrepareArgs pa{kdata, vdata, ks, kz, vs, vz, static_cast<unsigned char *>(workspace), p.kv_heads, nblocks,
                   uint32_t(rows)};
    const dim3 pgrid(nblocks, p.kv_heads);
    if (bits == 8) {
        prefill_prepare_kernel<8><<<pgrid, PREP_THREADS, 0, stream>>>(pa);
    } else if (bits == 4) {
        prefill_prepare_kernel<4><<<pgrid, PREP_THREADS, 0, stream>>>(pa);
    } else {
        prefill_prepare_kernel<16><<<pgrid, PREP_THREADS, 0, stream>>>(pa);
    }
    PrefillArgs a{q, static_cast<const unsigned char *>(workspace), q_and_gate, out, p.heads, p.kv_heads, p.pos,
                  p.tokens, p.scale, nblocks};
    static bool attr_set = false;
    if (!attr_set) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(attention_prefill_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        attr_set = true;
    }
    const dim3 grid((p.tokens + TQ - 1) / TQ, p.kv_heads);
    attention_prefill_kernel<<<grid, THREADS, LDS_BYTES, stream>>>(a);
    return launch_status(what);
}

}  // namespace
}  // namespace saetta

using namespace saetta;

extern "C" size_t saetta_prefill_workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t kv_heads) {
    return workspace_bytes(pos, tokens, kv_heads);
}

extern "C" int saetta_attn_prefill(saetta_stream_t stream, const uint16_t *q_f16, const uint16_t *keys,
                                   const uint16_t *values, const float *q_and_gate, float *out,
                                   saetta_flash_params p, void *workspace, size_t workspace_bytes) {
    return run_prefill(as_stream(stream), 16, q_f16, keys, values, nullptr, nullptr, nullptr, nullptr, q_and_gate,
                       out, p, workspace, workspace_bytes, "attn_prefill");
}

extern "C" int saetta_attn_prefill_quant(saetta_stream_t stream, int bits, const uint16_t *q_f16,
                                         saetta_quant_rows keys, saetta_quant_rows values,
                                         const float *q_and_gate, float *out, saetta_flash_params p,
                                         void *workspace, size_t workspace_bytes) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "attn_prefill_quant: bits %d (8 or 4)", bits);
    return run_prefill(as_stream(stream), bits, q_f16, keys.data, values.data, keys.scales, keys.biases,
                       values.scales, values.biases, q_and_gate, out, p, workspace, workspace_bytes,
                       "attn_prefill_quant");
}
