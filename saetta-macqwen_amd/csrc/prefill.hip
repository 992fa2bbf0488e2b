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
// Work split: workgroup (token tile of 32, kv head), 8 waves; wave w owns 4
// tokens x 8 heads = 32 query rows, one 32-row MFMA tile.  Keys are walked
// in blocks of 32.  Per block the workgroup stages K[32][256] and the
// transposed V^T[256][32] as f16 in LDS (dequantizing on the way), then every
// wave computes with v_mfma_f32_32x32x16_f16
//     S^T = K Q^T      (A = K rows from LDS, B = Q^T held in registers)
//     O^T += V^T P^T   (A = V^T rows from LDS, B = P^T from the S^T registers)
// Both products are transposed so that a lane always owns one query row: in
// the 32x32 accumulator layout a lane holds column l % 32, so the row's
// running max and sum, the rescale of O and the final 1/l and gate are plain
// per-lane values and the softmax needs one cross-lane exchange per block.
// The accumulators (128 floats per lane) live in AGPRs; two waves share a
// SIMD, so one's staging and softmax overlap the other's MFMAs; the tiles are
// double-buffered (one barrier per block) and issued heaviest first.
// The running max is only raised when a block exceeds it by more than 2^8
// (the usual lazy rescale), so O is rarely rescaled.
// The next block's codes are fetched into registers while the current block
// is computed.
#include "common.hpp"

namespace saetta {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_ __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int DIM = SAETTA_HEAD_DIM;
constexpr int THREADS = 512;
constexpr int NT = 1;                   // 32-row MFMA tiles per wave (4 tokens x 8 heads each)
constexpr int WAVES = THREADS / 64;
constexpr int TQ = 4 * NT * WAVES;      // tokens per workgroup
constexpr int BK = 32;                  // keys per block
constexpr int K_STRIDE = DIM * 2 + 16;  // bytes per key row of the K tile (padded against bank conflicts)
constexpr int V_STRIDE = BK * 2 + 16;   // bytes per dim row of the V^T tile
constexpr int K_BYTES = BK * K_STRIDE;
constexpr int V_BYTES = DIM * V_STRIDE;
constexpr float NO_SCORE = -1e30f;
constexpr float TAU = 8.0f;  // the reference max is raised only past this many powers of two

struct PrefillArgs {
    const uint16_t *q;  // f16 [tokens][heads][256]
    const void *kdata;
    const void *vdata;
    const uint16_t *kscales, *kbiases, *vscales, *vbiases;
    const float *q_and_gate;
    float *out;
    uint32_t heads, kv_heads, pos, tokens;
    float scale;
    uint32_t capacity;  // rows the cache arrays hold (bound of the buffer loads)
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
// K: thread (key = t / 16, piece = t % 16) takes 16 dims of one key.
// V: thread (dq = t % 64, kq = t / 64) takes 4 dims of 4 keys.
template <int BITS>
struct Stage {
    uint32_t k[BITS == 16 ? 8 : BITS / 2];  // 16 dims: 32 B (f16), 16 B (8-bit), 8 B (4-bit)
    uint32_t v[4][BITS == 16 ? 2 : 1];      // per key 4 dims: 8 B (f16), 4 B (8-bit), 2 B (4-bit)
    uint32_t ks, kz;                        // f16 scale and bias of (key, group of the piece)
    uint32_t vs[4], vz[4];                  // per key, group of dq
};

template <int BITS>
__device__ __forceinline__ void stage_load(Stage<BITS> &st, const PrefillArgs &a, __amdgpu_buffer_rsrc_t k_rsrc,
                                           __amdgpu_buffer_rsrc_t v_rsrc, __amdgpu_buffer_rsrc_t ks_rsrc,
                                           __amdgpu_buffer_rsrc_t kz_rsrc, __amdgpu_buffer_rsrc_t vs_rsrc,
                                           __amdgpu_buffer_rsrc_t vz_rsrc, uint32_t key0, uint32_t kv, int tid) {
    constexpr int RB = row_bytes<BITS>();
    const uint32_t kvh = a.kv_heads;
    {
        const int key = tid >> 4, piece = tid & 15;
        const int row = int((key0 + key) * kvh + kv);
        const int off = row * RB + piece * (RB / 16);
        if constexpr (BITS == 8) {
            const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, off, 0, 0);
            st.k[0] = x.x, st.k[1] = x.y, st.k[2] = x.z, st.k[3] = x.w;
        } else if constexpr (BITS == 4) {
            const u32x2 x = __builtin_amdgcn_raw_buffer_load_b64(k_rsrc, off, 0, 0);
            st.k[0] = x.x, st.k[1] = x.y;
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, off + 16 * i, 0, 0);
                st.k[4 * i] = x.x, st.k[4 * i + 1] = x.y, st.k[4 * i + 2] = x.z, st.k[4 * i + 3] = x.w;
            }
        }
        if constexpr (BITS != 16) {
            const int soff = (row * 4 + (piece >> 2)) * 2;
            st.ks = __builtin_amdgcn_raw_buffer_load_b16(ks_rsrc, soff, 0, 0);
            st.kz = __builtin_amdgcn_raw_buffer_load_b16(kz_rsrc, soff, 0, 0);
        }
    }
    {
        const int dq = tid & 63, kq = tid >> 6;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = int((key0 + 4 * kq + i) * kvh + kv);
            const int off = row * RB + dq * (RB / 64);
            if constexpr (BITS == 8) {
                st.v[i][0] = __builtin_amdgcn_raw_buffer_load_b32(v_rsrc, off, 0, 0);
            } else if constexpr (BITS == 4) {
                st.v[i][0] = uint16_t(__builtin_amdgcn_raw_buffer_load_b16(v_rsrc, off, 0, 0));
            } else {
                const u32x2 x = __builtin_amdgcn_raw_buffer_load_b64(v_rsrc, off, 0, 0);
                st.v[i][0] = x.x, st.v[i][1] = x.y;
            }
            if constexpr (BITS != 16) {
                const int soff = (row * 4 + (dq >> 4)) * 2;
                st.vs[i] = __builtin_amdgcn_raw_buffer_load_b16(vs_rsrc, soff, 0, 0);
                st.vz[i] = __builtin_amdgcn_raw_buffer_load_b16(vz_rsrc, soff, 0, 0);
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
        const int key = tid >> 4, piece = tid & 15;
        uint32_t o[8];
        if constexpr (BITS == 16) {
#pragma unroll
            for (int i = 0; i < 8; i++) o[i] = st.k[i];
        } else {
            const float s = h2f(st.ks), z = h2f(st.kz);
            constexpr int PER = 32 / BITS;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t w = st.k[(2 * i) / PER];
                o[i] = pack_half2(dequant(s, z, code_of<BITS>(w, (2 * i) % PER)),
                                  dequant(s, z, code_of<BITS>(w, (2 * i + 1) % PER)));
            }
        }
        if (key0 + key >= key_limit) {
#pragma unroll
            for (int i = 0; i < 8; i++) o[i] = 0;
        }
        u32x4 *dst = reinterpret_cast<u32x4 *>(k_lds + key * K_STRIDE + piece * 32);
        dst[0] = u32x4{o[0], o[1], o[2], o[3]};
        dst[1] = u32x4{o[4], o[5], o[6], o[7]};
    }
    {
        const int dq = tid & 63, kq = tid >> 6;
        float x[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const bool live = key0 + 4 * kq + i < key_limit;
            if constexpr (BITS == 16) {
#pragma unroll
                for (int d = 0; d < 4; d++) x[i][d] = live ? h2f(st.v[i][d >> 1] >> (16 * (d & 1))) : 0.0f;
            } else {
                const float s = h2f(st.vs[i]), z = h2f(st.vz[i]);
#pragma unroll
                for (int d = 0; d < 4; d++) x[i][d] = live ? dequant(s, z, code_of<BITS>(st.v[i][0], d)) : 0.0f;
            }
        }
        // keys 4kq..4kq+3 are neighbours in the row's key order
        const int p0 = vt_pos(4 * kq);
#pragma unroll
        for (int d = 0; d < 4; d++) {
            u32x2 w = {pack_half2(x[0][d], x[1][d]), pack_half2(x[2][d], x[3][d])};
            *reinterpret_cast<u32x2 *>(v_lds + (4 * dq + d) * V_STRIDE + 2 * p0) = w;
        }
    }
}

template <int BITS>
__global__ __launch_bounds__(THREADS) void attention_prefill_kernel(PrefillArgs a) {
    constexpr int RB = row_bytes<BITS>();
    // two buffers of (K tile, V^T tile): block kb lives in buffer kb & 1
    extern __shared__ __attribute__((aligned(16))) unsigned char tiles[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hf = lane >> 5;
    const uint32_t kv = blockIdx.y;
    const uint32_t ntiles = (a.tokens + TQ - 1) / TQ;
    const uint32_t tile = ntiles - 1 - blockIdx.x;  // the tiles with the most keys start first
    const uint32_t tok0 = tile * TQ + 4 * NT * wave;  // this wave's first token
    const float c = a.scale * 1.4426950408889634f;   // scores are kept in units of log2(e)

    // Row of this lane in row tile nt: token tok0 + 4nt + col / 8, head col % 8.
    uint32_t tok[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) tok[nt] = tok0 + 4 * nt + (col >> 3);
    const uint32_t head = kv * 8 + (col & 7);

    // Q^T operands: lane (col, hf), k-step st: dims 16 st + 8 hf .. + 7 of its row.
    half8 qb[NT][16];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const uint32_t tk = min(tok[nt], a.tokens - 1);
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.q + (size_t(tk) * a.heads + head) * DIM + 8 * hf);
#pragma unroll
        for (int st = 0; st < 16; st++) qb[nt][st] = __builtin_bit_cast(half8, src[2 * st]);
    }

    const uint32_t cap_rows = a.capacity * a.kv_heads;
    const __amdgpu_buffer_rsrc_t k_rsrc = make_rsrc(a.kdata, cap_rows * RB);
    const __amdgpu_buffer_rsrc_t v_rsrc = make_rsrc(a.vdata, cap_rows * RB);
    const __amdgpu_buffer_rsrc_t ks_rsrc = make_rsrc(a.kscales, BITS == 16 ? 0 : cap_rows * 8);
    const __amdgpu_buffer_rsrc_t kz_rsrc = make_rsrc(a.kbiases, BITS == 16 ? 0 : cap_rows * 8);
    const __amdgpu_buffer_rsrc_t vs_rsrc = make_rsrc(a.vscales, BITS == 16 ? 0 : cap_rows * 8);
    const __amdgpu_buffer_rsrc_t vz_rsrc = make_rsrc(a.vbiases, BITS == 16 ? 0 : cap_rows * 8);

    // Keys this workgroup walks: up to what its last token sees; what this wave needs.
    const uint32_t key_limit = a.pos + a.tokens;  // end of the chunk: nothing past it is ever visible
    const uint32_t wg_keys = min(a.pos + min(tile * TQ + TQ, a.tokens), key_limit);
    const uint32_t nblocks = (wg_keys + BK - 1) / BK;
    const uint32_t wave_first_len = a.pos + tok0 + 1;                          // keys the wave's first token sees
    const uint32_t wave_keys = a.pos + min(tok0 + 4 * NT, a.tokens);                 // keys its last token sees

    floatx16 acc[8][NT];
#pragma unroll
    for (int mt = 0; mt < 8; mt++) {
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mt][nt][r] = 0.0f;
        }
    }
    float m_ref[NT], l_sum[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) m_ref[nt] = NO_SCORE, l_sum[nt] = 0.0f;

    Stage<BITS> st;
    stage_load<BITS>(st, a, k_rsrc, v_rsrc, ks_rsrc, kz_rsrc, vs_rsrc, vz_rsrc, 0, kv, tid);
    stage_store<BITS>(st, tiles, tiles + K_BYTES, 0, key_limit, tid);
    if (nblocks > 1) stage_load<BITS>(st, a, k_rsrc, v_rsrc, ks_rsrc, kz_rsrc, vs_rsrc, vz_rsrc, BK, kv, tid);
    __syncthreads();

    for (uint32_t kb = 0; kb < nblocks; kb++) {
        const uint32_t key0 = kb * BK;
        const unsigned char *k_lds = tiles + (kb & 1) * (K_BYTES + V_BYTES);
        const unsigned char *v_lds = k_lds + K_BYTES;
        // Block kb + 1 goes into the other buffer (every wave left it at the barrier below),
        // block kb + 2 into the registers.
        if (kb + 1 < nblocks) {
            unsigned char *nk = tiles + ((kb + 1) & 1) * (K_BYTES + V_BYTES);
            stage_store<BITS>(st, nk, nk + K_BYTES, key0 + BK, key_limit, tid);
            if (kb + 2 < nblocks) {
                stage_load<BITS>(st, a, k_rsrc, v_rsrc, ks_rsrc, kz_rsrc, vs_rsrc, vz_rsrc, key0 + 2 * BK, kv, tid);
            }
        }
        if (key0 >= wave_keys) {  // nothing in this block is visible to this wave (uniform)
            __syncthreads();
            continue;
        }
  // nothing in this block is visible to this wave (uniform)

        // ---- S^T = K Q^T: rows = the block's 32 keys, columns = query rows ----------
        floatx16 s[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
            for (int r = 0; r < 16; r++) s[nt][r] = 0.0f;
        }
#pragma unroll
        for (int stp = 0; stp < 16; stp++) {
            const half8 ka = *reinterpret_cast<const half8 *>(k_lds + col * K_STRIDE + (16 * stp + 8 * hf) * 2);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) s[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qb[nt][stp], s[nt], 0, 0, 0);
        }

        // ---- online softmax, one row per lane ---------------------------------------
        // Register r of the accumulator is key 4 hf + r % 4 + 8 (r / 4) of the block.
        const bool diagonal = key0 + BK > wave_first_len;  // some key of the block is hidden from some row
        half8 pb[NT][2];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            float v[16];
            float bm = NO_SCORE;
            if (diagonal) {
                const uint32_t vis = a.pos + tok[nt] + 1 - min(key0, a.pos + tok[nt] + 1);  // visible keys of the block
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const uint32_t key = 4 * hf + (r & 3) + 8 * (r >> 2);
                    v[r] = key < vis ? s[nt][r] * c : NO_SCORE;
                    bm = fmaxf(bm, v[r]);
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    v[r] = s[nt][r] * c;
                    bm = fmaxf(bm, v[r]);
                }
            }
            bm = fmaxf(bm, __shfl_xor(bm, 32));
            if (__any(bm > m_ref[nt] + TAU)) {
                const float m_new = bm > m_ref[nt] + TAU ? bm : m_ref[nt];
                const float alpha = __builtin_amdgcn_exp2f(m_ref[nt] - m_new);
                m_ref[nt] = m_new;
                l_sum[nt] *= alpha;
#pragma unroll
                for (int mt = 0; mt < 8; mt++) {
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[mt][nt][r] *= alpha;
                }
            }
            float sum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                v[r] = __builtin_amdgcn_exp2f(v[r] - m_ref[nt]);
                sum += v[r];
            }
            l_sum[nt] += sum;
            // P^T operands: k-step sp takes registers 8 sp .. 8 sp + 7 (the order vt_pos mirrors)
#pragma unroll
            for (int sp = 0; sp < 2; sp++) {
                u32x4 w = {pack_half2(v[8 * sp], v[8 * sp + 1]), pack_half2(v[8 * sp + 2], v[8 * sp + 3]),
                           pack_half2(v[8 * sp + 4], v[8 * sp + 5]), pack_half2(v[8 * sp + 6], v[8 * sp + 7])};
                pb[nt][sp] = __builtin_bit_cast(half8, w);
            }
        }

        // ---- O^T += V^T P^T: rows = dims, columns = query rows ------------------------
#pragma unroll
        for (int mt = 0; mt < 8; mt++) {
#pragma unroll
            for (int sp = 0; sp < 2; sp++) {
                const half8 va =
                    *reinterpret_cast<const half8 *>(v_lds + (32 * mt + col) * V_STRIDE + (16 * sp + 8 * hf) * 2);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pb[nt][sp], acc[mt][nt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    // ---- out = O / l * sigmoid(gate) ---------------------------------------------------
    // The lane's row sum is split over the two lane halves (each saw half the keys).
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const float l = l_sum[nt] + __shfl_xor(l_sum[nt], 32);
        if (tok[nt] >= a.tokens) continue;
        const float inv = 1.0f / l;
        const size_t row = size_t(tok[nt]) * a.heads + head;
        const float *gate = a.q_and_gate + row * 2 * DIM + DIM;
        float *out = a.out + row * DIM;
#pragma unroll
        for (int mt = 0; mt < 8; mt++) {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const int d0 = 32 * mt + 8 * q4 + 4 * hf;
                const float4 g = *reinterpret_cast<const float4 *>(gate + d0);
                float4 o;
                o.x = acc[mt][nt][4 * q4 + 0] * inv / (1.0f + __expf(-g.x));
                o.y = acc[mt][nt][4 * q4 + 1] * inv / (1.0f + __expf(-g.y));
                o.z = acc[mt][nt][4 * q4 + 2] * inv / (1.0f + __expf(-g.z));
                o.w = acc[mt][nt][4 * q4 + 3] * inv / (1.0f + __expf(-g.w));
                *reinterpret_cast<float4 *>(out + d0) = o;
            }
        }
    }
}

int run_prefill(hipStream_t stream, int bits, const uint16_t *q, const void *kdata, const void *vdata,
                const uint16_t *ks, const uint16_t *kz, const uint16_t *vs, const uint16_t *vz,
                const float *q_and_gate, float *out, saetta_flash_params p, const char *what) {
    SAETTA_REQUIRE(bits == 16 || bits == 8 || bits == 4, SAETTA_E_BITS, "%s: bits %d", what, bits);
    SAETTA_REQUIRE(p.kv_heads > 0 && p.heads == p.kv_heads * SAETTA_GQA_GROUP, SAETTA_E_SHAPE,
                   "%s needs 8 q heads per kv head (heads %u, kv heads %u)", what, p.heads, p.kv_heads);
    SAETTA_REQUIRE(q && kdata && vdata && q_and_gate && out, SAETTA_E_NULL, "%s: null buffer", what);
    SAETTA_REQUIRE(bits == 16 || (ks && kz && vs && vz), SAETTA_E_NULL, "%s: null scales or biases", what);
    SAETTA_REQUIRE(aligned(q, 16) && aligned(kdata, 16) && aligned(vdata, 16) && aligned(q_and_gate, 16) &&
                       aligned(out, 16),
                   SAETTA_E_ALIGN, "%s: buffers must be 16-byte aligned", what);
    const uint64_t rows = uint64_t(p.pos) + p.tokens;  // the cache holds the chunk's rows too
    SAETTA_REQUIRE(rows * p.kv_heads * 512 < (uint64_t(1) << 31), SAETTA_E_SHAPE, "%s: pos + tokens %llu out of range",
                   what, (unsigned long long)rows);
    if (int rc = ensure_device()) return rc;
    if (p.tokens == 0) return SAETTA_OK;
    PrefillArgs a{q, kdata, vdata, ks, kz, vs, vz, q_and_gate, out, p.heads, p.kv_heads, p.pos, p.tokens, p.scale,
                  uint32_t(rows)};
    const dim3 grid((p.tokens + TQ - 1) / TQ, p.kv_heads);
    constexpr int LDS = 2 * (K_BYTES + V_BYTES);
    static bool attr_set = false;
    if (!attr_set) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(attention_prefill_kernel<8>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(attention_prefill_kernel<4>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(attention_prefill_kernel<16>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        attr_set = true;
    }
    if (bits == 8) {
        attention_prefill_kernel<8><<<grid, THREADS, LDS, stream>>>(a);
    } else if (bits == 4) {
        attention_prefill_kernel<4><<<grid, THREADS, LDS, stream>>>(a);
    } else {
        attention_prefill_kernel<16><<<grid, THREADS, LDS, stream>>>(a);
    }
    return launch_status(what);
}

}  // namespace
}  // namespace saetta

using namespace saetta;

extern "C" int saetta_attn_prefill(saetta_stream_t stream, const uint16_t *q_f16, const uint16_t *keys,
                                   const uint16_t *values, const float *q_and_gate, float *out,
                                   saetta_flash_params p) {
    return run_prefill(as_stream(stream), 16, q_f16, keys, values, nullptr, nullptr, nullptr, nullptr, q_and_gate,
                       out, p, "attn_prefill");
}

extern "C" int saetta_attn_prefill_quant(saetta_stream_t stream, int bits, const uint16_t *q_f16,
                                         saetta_quant_rows keys, saetta_quant_rows values,
                                         const float *q_and_gate, float *out, saetta_flash_params p) {
    SAETTA_REQUIRE(bits == 8 || bits == 4, SAETTA_E_BITS, "attn_prefill_quant: bits %d (8 or 4)", bits);
    return run_prefill(as_stream(stream), bits, q_f16, keys.data, values.data, keys.scales, keys.biases,
                       values.scales, values.biases, q_and_gate, out, p, "attn_prefill_quant");
}
