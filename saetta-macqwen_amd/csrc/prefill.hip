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
// Two kernels (and, further down, the reference's other route to the same output, AttGemm of
// src/attention_gemm.rs: two more kernels on the same images, block by block of 1024 keys).
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
#include "lanes.hpp"

#include <map>
#include <mutex>
#include <utility>

namespace saetta {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2_ __attribute__((ext_vector_type(2)));
typedef float float2_ __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int DIM = SAETTA_HEAD_DIM;
constexpr int PREP_THREADS = 256;       // the prepare kernel's workgroup
constexpr int WAVES = 8;                // 4 row groups x 2 waves that take alternate key blocks
constexpr int THREADS = 64 * WAVES;
constexpr int TQ = 16;                  // tokens per workgroup: a row group is 4 tokens x 8 heads = 32 rows
constexpr int BK = 32;                  // keys per block
// One key block's image: the K tile and the V^T tile in MFMA fragment order, 16 KB each.  A
// fragment is what one ds_read_b128 of a wave fetches: 64 lanes x 16 bytes, lane (col, hf) at
// byte 512 hf + 16 col, so every fragment read is one contiguous kilobyte.
//   K fragment stp (0..15):           lane holds dims 16 stp + 8 hf .. + 7 of key col
//   V^T fragment 2 mt + sp (0..15):   lane holds key positions 16 sp + 8 hf .. + 7 of dim 32 mt + col
constexpr int PART_BYTES = BK * DIM * 2;
constexpr int IMG_BYTES = 2 * PART_BYTES;
constexpr float NO_SCORE = -1e30f;
constexpr float TAU = 8.0f;  // the reference max is raised only past this many powers of two

struct PrepareArgs {
    const void *kdata;
    const void *vdata;
    const uint16_t *kscales, *kbiases, *vscales, *vbiases;
    unsigned char *images;  // [kv head][block][IMG_BYTES]
    uint32_t kv_heads, nblocks;
    uint32_t key_limit;  // pos + tokens: rows the cache holds; keys from here on are zeros
    uint32_t *tiles_taken;  // behind the images (or nullptr): the attention kernel's count of tiles handed out, set to 0 here
};

struct PrefillArgs {
    const uint16_t *q;  // f16 [tokens][heads][256]
    const unsigned char *images;
    const float *q_and_gate;
    float *out;
    uint32_t heads, kv_heads, pos, tokens;
    float scale;
    uint32_t nblocks;  // images per kv head
    uint32_t *tiles_taken;  // tiles handed out past every workgroup's first (zero at the start: the prepare kernel's doing)
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
};

// Scales and biases of a block's 32 keys, staged in LDS by the first 128 threads (8 bytes each: the four f16
// of a key's groups) and read from there: per array [key][groups (0, 1) | groups (2, 3)] as pairs of f16.
struct BlockScales {
    uint32_t w[4][BK][2];  // [k scales | k biases | v scales | v biases]
    __device__ __forceinline__ float get(int arr, int key, int group) const {
        return (float)__builtin_bit_cast(_Float16, uint16_t(w[arr][key][group >> 1] >> (16 * (group & 1))));
    }
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

// Dequantizes the staged registers into the two parts of the block's image.  Keys at or past key_limit
// (the end of the chunk) are written as zeros: their probabilities are 0, and 0 * 0
// stays 0 whatever the cache rows hold.
template <int BITS>
__device__ __forceinline__ void stage_store(const Stage<BITS> &st, const BlockScales &sb, unsigned char *k_img, unsigned char *v_img,
                                            uint32_t key0, uint32_t key_limit, int tid) {
    {
        const int key = tid >> 3, piece = tid & 7;
        uint32_t o[16];
        if constexpr (BITS == 16) {
#pragma unroll
            for (int i = 0; i < 16; i++) o[i] = st.k[i];
        } else {
            const float s = sb.get(0, key, piece >> 1), z = sb.get(1, key, piece >> 1);
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
        // dims 32 piece + 8 j .. + 7 are the (hf = j % 2) half of fragment 2 piece + j / 2
#pragma unroll
        for (int j = 0; j < 4; j++) {
            *reinterpret_cast<u32x4 *>(k_img + (4 * piece + j) * 512 + key * 16) =
                u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
        }
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
                    const float s = sb.get(2, 8 * kq + i + u, dq >> 4), z = sb.get(3, 8 * kq + i + u, dq >> 4);
#pragma unroll
                    for (int d = 0; d < 4; d++) x[u][d] = live ? dequant(s, z, code_of<BITS>(st.v[i + u][0], d)) : 0.0f;
                }
            }
#pragma unroll
            for (int d = 0; d < 4; d++) w[d][i / 2] = pack_half2(x[0][d], x[1][d]);
        }
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const int dim = 4 * dq + d;
            unsigned char *frag = v_img + (dim >> 5) * 2048 + (dim & 31) * 16;  // position 0 of the dim
            *reinterpret_cast<u32x2 *>(frag + (p0 >> 3) * 512 + (p0 & 7) * 2) = u32x2{w[d][0], w[d][1]};
            *reinterpret_cast<u32x2 *>(frag + (p1 >> 3) * 512 + (p1 & 7) * 2) = u32x2{w[d][2], w[d][3]};
        }
    }
}

// One workgroup per (block of 32 keys, kv head).  The K tile goes out as it is made (a wave's store is eight runs
// of 128 bytes); the V^T tile is a transposition (a thread holds 4 dims of 8 keys, the image wants 8 keys of a dim
// side by side), so it is put together in LDS and copied out as whole lines.
template <int BITS>
__global__ __launch_bounds__(PREP_THREADS) void prefill_prepare_kernel(PrepareArgs a) {
    constexpr int RB = row_bytes<BITS>();
    __shared__ __attribute__((aligned(16))) unsigned char vt_lds[PART_BYTES];
    __shared__ BlockScales sb;
    const uint32_t block = blockIdx.x, kv = blockIdx.y, kvh = a.kv_heads;
    const int tid = threadIdx.x;
    if (a.tiles_taken && block == 0 && kv == 0 && tid == 0) *a.tiles_taken = 0;
    const uint32_t cap_rows = a.key_limit * kvh;
    Rsrc rs;
    rs.k = make_rsrc(a.kdata, cap_rows * RB);
    rs.v = make_rsrc(a.vdata, cap_rows * RB);
    rs.ks = make_rsrc(a.kscales, BITS == 16 ? 0 : cap_rows * 8);
    rs.kz = make_rsrc(a.kbiases, BITS == 16 ? 0 : cap_rows * 8);
    rs.vs = make_rsrc(a.vscales, BITS == 16 ? 0 : cap_rows * 8);
    rs.vz = make_rsrc(a.vbiases, BITS == 16 ? 0 : cap_rows * 8);
    if constexpr (BITS != 16) {
        if (tid < 4 * BK) {
            // (a key past the cache's end reads as zeros: its values are written as zeros whatever the scales are)
            const int arr = tid / BK, key = tid % BK;
            const int off = int((block * BK + key) * kvh + kv) * 8;
            const __amdgpu_buffer_rsrc_t r = arr == 0 ? rs.ks : arr == 1 ? rs.kz : arr == 2 ? rs.vs : rs.vz;
            const u32x2 x = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
            sb.w[arr][key][0] = x.x, sb.w[arr][key][1] = x.y;
        }
    }
    Stage<BITS> st;
    stage_load<BITS>(st, rs, kvh, block * BK, kv, tid);
    __syncthreads();  // the scales are in LDS
    unsigned char *img = a.images + (size_t(kv) * a.nblocks + block) * IMG_BYTES;
    stage_store<BITS>(st, sb, img, vt_lds, block * BK, a.key_limit, tid);
    __syncthreads();  // the V^T tile is in LDS
#pragma unroll
    for (int i = 0; i < PART_BYTES / 16 / PREP_THREADS; i++) {
        const int at = (i * PREP_THREADS + tid) * 16;
        *reinterpret_cast<u32x4 *>(img + PART_BYTES + at) = *reinterpret_cast<const u32x4 *>(vt_lds + at);
    }
}

#include "prefill_stream.hpp"  // Copy, copy_plain, scores_block, stream_block, settle

// max over the two lanes l and l ^ 32, without a trip through LDS
__device__ __forceinline__ float max_across_halves(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x), v = u;
    // Swaps the upper half of u with the lower half of v: u = (lo, lo), v = (hi, hi).  The
    // instruction may not read a register a vector instruction wrote in the two cycles before.
    asm volatile("s_nop 1\nv_permlane32_swap_b32 %0, %1\n" : "+v"(u), "+v"(v));
    return fmaxf(__builtin_bit_cast(float, u), __builtin_bit_cast(float, v));
}

// A workgroup barrier for data that went through LDS only: waits for this wave's LDS accesses, not for its
// loads and stores to memory (__syncthreads waits for those too: behind the gate loads of a tile's end, or
// the output stores, that is microseconds with nothing else to run).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// LDS: four K slots, then four V^T slots; block b uses slot b % 4 of each.
constexpr int MERGE_WAVE_BYTES = (4 * 16 + 2) * 64 * 4;  // half of a wave's O, its m and l, on their way to its partner
constexpr int LDS_BYTES = 8 * MERGE_WAVE_BYTES > 8 * PART_BYTES ? 8 * MERGE_WAVE_BYTES : 8 * PART_BYTES;
__device__ __forceinline__ uint32_t k_slot(uint32_t b) { return (b & 3) * PART_BYTES; }
__device__ __forceinline__ uint32_t v_slot(uint32_t b) { return (4 + (b & 3)) * PART_BYTES; }

// One tile of TQ tokens x 8 heads of kv head `kv` against the keys it sees.
__device__ __forceinline__ void prefill_tile(const PrefillArgs &a, unsigned char *tiles, uint32_t tile, uint32_t kv, bool ask, uint32_t *next_tile) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, hf = lane >> 5;
    const int group = wave & 3, parity = wave >> 2;  // the wave's rows; which key blocks it takes
    const uint32_t tok0 = tile * TQ + 4 * group;    // this wave's first token
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

    const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(tiles));
    const uint32_t lane16 = lane * 16;
    const unsigned char *images = a.images + size_t(kv) * a.nblocks * IMG_BYTES;
    // Half `half` (8 KB) of part `v` (0 = K, 1 = V^T) of block b.  Blocks past the cache's end
    // are read from the last image instead; nobody looks at their slots.
    auto piece = [&](uint32_t b, int v, int half) {
        const uint32_t bb = min(b, a.nblocks - 1);
        Copy cp;
        cp.src = reinterpret_cast<uint64_t>(images) + uint64_t(bb) * IMG_BYTES + v * PART_BYTES + half * 8192;
        cp.dst = lds0 + (v ? v_slot(b) : k_slot(b)) + half * 8192;
        return cp;
    };

    // Step s works on blocks 2s (waves 0..3: parity 0) and 2s + 1 (waves 4..7: parity 1).  A
    // wave's step is a softmax (vector ALU) and an MFMA stream that adds the block to O and
    // computes the scores of the wave's next block; the two waves of a SIMD run them in opposite
    // order, so that one's softmax runs under the other's MFMAs:
    //   parity 0:  softmax(2s)               | O(2s) + S(2s+2)
    //   parity 1:  O(2s+1) + S(2s+3)         | softmax(2s+3)
    // During step s the workgroup copies what step s + 1 reads: K(2s+4), K(2s+5), V(2s+2),
    // V(2s+3); wave w takes half (w % 2) of part w / 2 of that list.  Before the loop: K(0..3),
    // V(0), V(1), twelve kilobytes per wave.
    for (int i = wave; i < 48; i += WAVES) {
        const int part = i >> 3, v = part >= 4;
        const uint32_t b = v ? part - 4 : part;
        Copy cp = piece(b, v, 0);
        cp.src += (i & 7) * 2048, cp.dst += (i & 7) * 2048;
        asm volatile(
            "s_mov_b32 m0, %[dst]\n"
            "s_nop 0\n"
            "global_load_lds_dwordx4 %[off], %[src]\n"
            "global_load_lds_dwordx4 %[off], %[src] offset:1024\n"
            :
            : [off] "v"(lane16), [src] "s"(cp.src), [dst] "s"(cp.dst)
            : "memory", "m0");
    }

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
    // The reference maximum starts above what a block of masked scores gives (NO_SCORE * c), so that a row that sees
    // none of a wave's first block never takes that for its maximum: with m_ref equal to the rounded NO_SCORE * c the
    // exponent s * c - m_ref of a masked score is the product's rounding error, 1e21 either way, not minus infinity.
    // (The second wave of a row group starts at block 1: rows that end inside block 0 have nothing in it.)
    float m_ref = 0.25f * NO_SCORE * c, l_sum = 0.0f;

    // Row maximum of a block's scaled scores (first half of the softmax).  Register r of the
    // accumulator is key 4 hf + r % 4 + 8 (r / 4) of the block; masked scores become NO_SCORE (NO_SCORE * c in the units of the maximum).
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
        bm = max_across_halves(bm);
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

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // K(0..3), V(0), V(1) are in LDS

    const uint32_t nsteps = (nblocks + 1) / 2;
    const int part = wave >> 1, half = wave & 1;  // what the wave copies in every step
    auto copy_of = [&](uint32_t step) {
        const uint32_t cb = part == 0 ? 2 * step + 4 : part == 1 ? 2 * step + 5 : part == 2 ? 2 * step + 2 : 2 * step + 3;
        return piece(cb, part >= 2, half);
    };
    if (parity == 0) {
        floatx16 s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.0f;
        if (0 < wave_blocks) scores_block(s, qb, lds0 + k_slot(0) + lane16);
        __syncthreads();  // the first step's copies overwrite K(0) and K(1)
        for (uint32_t step = 0; step < nsteps; step++) {
            const Copy cp = copy_of(step);
            const uint32_t kb = 2 * step;
            if (kb < wave_blocks) {
                raise_max(mask_max(s, kb * BK, kb >= full_blocks));
                half8 pb[2];
                exp_pack(s, pb);
                // (past the wave's last block the scores are of stale keys and never looked at)
                stream_block(s, acc, qb, pb, lds0 + k_slot(kb + 2) + lane16, lds0 + v_slot(kb) + lane16, cp, lane16);
            } else {
                copy_plain(cp, lane16);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    } else {
        half8 pb[2] = {};
        if (1 < wave_blocks) {
            floatx16 s;
            scores_block(s, qb, lds0 + k_slot(1) + lane16);
            raise_max(mask_max(s, BK, 1 >= full_blocks));
            exp_pack(s, pb);
        }
        __syncthreads();
        for (uint32_t step = 0; step < nsteps; step++) {
            const Copy cp = copy_of(step);
            const uint32_t kb = 2 * step + 1;
            if (kb < wave_blocks) {
                // This wave's stream comes before its softmax, the other wave's of the SIMD after: let
                // this one's MFMAs go first, so that its softmax still finds the other's to run under.
                floatx16 s;
                __builtin_amdgcn_s_setprio(2);
                stream_block(s, acc, qb, pb, lds0 + k_slot(kb + 2) + lane16, lds0 + v_slot(kb) + lane16, cp, lane16);
                __builtin_amdgcn_s_setprio(0);
                if (kb + 2 < wave_blocks) {
                    raise_max(mask_max(s, (kb + 2) * BK, kb + 2 >= full_blocks));
                    exp_pack(s, pb);
                }
            } else {
                copy_plain(cp, lane16);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }

    settle(acc);
    // Which tile this workgroup takes next: asked for here, where the workgroups are apart in time (their tiles differ in
    // length; at the kernel's start every one of them would ask at once, and the adds on one word come one after the
    // other), and looked at when the tile has ended.  (Before the gate loads: behind them the one more register that is
    // live with them costs 150 bytes of spills.)
    uint32_t got = ask ? 0u : 0xffffffffu;
    if (ask && tid == 0) got = gridDim.x + atomicAdd(a.tiles_taken, 1u);

    // The gate values of this wave's half of the dims, asked for before the merge below so that they travel while
    // it runs (scattered 16-byte pieces, one round trip for the lot; a token past the end: the last token's, unused).
    float4 g[16];
    {
        const size_t grow = size_t(min(tok, a.tokens - 1)) * a.heads + head;
        const float *gate = a.q_and_gate + grow * 2 * DIM + DIM + 128 * parity;
#pragma unroll
        for (int i = 0; i < 16; i++) g[i] = *reinterpret_cast<const float4 *>(gate + 32 * (i >> 2) + 8 * (i & 3) + 4 * hf);
    }
    // ---- the two waves of a row group merge their halves of the keys ----------------------
    // Each wave finishes half of the dims: parity 0 the accumulators 0..3 (dims 0..127), parity 1
    // the rest.  It hands the other half, m and l to its partner through LDS (the tiles are done
    // with: the loop ended on a barrier); element e of lane L sits at word e * 64 + L.
    float *mine_out = reinterpret_cast<float *>(tiles + wave * MERGE_WAVE_BYTES) + lane;
    const float *theirs_in = reinterpret_cast<const float *>(tiles + (wave ^ 4) * MERGE_WAVE_BYTES) + lane;
    floatx16 fin[4];
    if (parity == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            fin[i] = acc[i];
#pragma unroll
            for (int r = 0; r < 16; r++) mine_out[(16 * i + r) * 64] = acc[4 + i][r];
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            fin[i] = acc[4 + i];
#pragma unroll
            for (int r = 0; r < 16; r++) mine_out[(16 * i + r) * 64] = acc[i][r];
        }
    }
    mine_out[64 * 64] = m_ref;
    mine_out[65 * 64] = l_sum;
    lds_barrier();  // (the gate values stay on their way)
    const float m_other = theirs_in[64 * 64], l_other = theirs_in[65 * 64];
    const float m_new = fmaxf(m_ref, m_other);
    const float mine = __builtin_amdgcn_exp2f(m_ref - m_new), theirs = __builtin_amdgcn_exp2f(m_other - m_new);
    l_sum = l_sum * mine + l_other * theirs;

    // ---- out = O / l * sigmoid(gate) ---------------------------------------------------
    // The lane's row sum is split over the two lane halves (each saw half the keys).
    const float l = l_sum + __shfl_xor(l_sum, 32);
    if (tok < a.tokens) {
        const float inv = 1.0f / l;
        const size_t row = size_t(tok) * a.heads + head;
        float *out = a.out + row * DIM + 128 * parity;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int mt = i >> 2, q4 = i & 3;
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int r = 4 * q4 + e;
                o[e] = (fin[mt][r] * mine + theirs_in[(16 * mt + r) * 64] * theirs) * inv;
            }
            float4 w;
            w.x = o[0] * __builtin_amdgcn_rcpf(1.0f + __expf(-g[i].x));
            w.y = o[1] * __builtin_amdgcn_rcpf(1.0f + __expf(-g[i].y));
            w.z = o[2] * __builtin_amdgcn_rcpf(1.0f + __expf(-g[i].z));
            w.w = o[3] * __builtin_amdgcn_rcpf(1.0f + __expf(-g[i].w));
            *reinterpret_cast<float4 *>(out + 32 * mt + 8 * q4 + 4 * hf) = w;
        }
    }
    if (tid == 0) *next_tile = got;
}

// A workgroup takes tiles until there are none left: with more tiles than workgroups (one per CU: the LDS ring
// fills a CU), the next tile starts without a new workgroup having to be dispatched.  Tiles are numbered from the
// one with the most keys down, the kv heads side by side.  Workgroup w starts with tile w; the others are handed
// out in that order to whoever asks next (one atomic add per tile on a counter behind the images, asked for
// before the tile's epilogue so that the answer is there when it ends): a workgroup that took a long tile, or runs
// on a slower CU, asks later and gets a shorter one, so that all of them end together (tiles dealt beforehand, the
// longest with the shortest, ended 40 us apart: the workgroups' rates differ by a tenth).
__global__ __launch_bounds__(THREADS, 2) void attention_prefill_kernel(PrefillArgs a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char tiles[];
    __shared__ uint32_t next_tile;
    const uint32_t ntiles = (a.tokens + TQ - 1) / TQ, total = ntiles * a.kv_heads, G = gridDim.x;
    for (uint32_t idx = blockIdx.x; idx < total;) {
        // (the tiles from G on are handed out by one question each: the tiles before the last G ask one, when they end,
        // and the last G none: nothing is left by then, and the kernel's last epilogues do not wait for an answer)
        prefill_tile(a, tiles, ntiles - 1 - idx / a.kv_heads, idx % a.kv_heads, idx + G < total, &next_tile);
        lds_barrier();  // the next tile is known; this tile's merge has been read: the next tile's keys may land on it (its stores go on meanwhile)
        idx = next_tile;
    }
}

// Workspaces the library owns when the caller passes none: one per (device, stream), grown on demand,
// so that calls on different streams never share one (work on one stream runs in order).  They are
// kept until the process ends: a caller with many short-lived streams passes its own.
struct OwnedWorkspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};
constexpr int OWNED_DEVICES = 64;  // as many devices as the library's set-up admits
std::map<std::pair<int, hipStream_t>, OwnedWorkspace> g_owned;
std::mutex g_owned_mutex;

// The images, then a line for the attention kernel's count of tiles handed out.
size_t images_bytes(uint32_t pos, uint32_t tokens, uint32_t kv_heads) {
    const size_t blocks = (size_t(pos) + tokens + BK - 1) / BK;
    return blocks * kv_heads * IMG_BYTES;
}
size_t workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t kv_heads) { return images_bytes(pos, tokens, kv_heads) + 256; }

// The checks both prefill paths share.
int check_prefill(int bits, const uint16_t *q, const void *kdata, const void *vdata, const uint16_t *ks,
                  const uint16_t *kz, const uint16_t *vs, const uint16_t *vz, const float *q_and_gate, const float *out,
                  saetta_flash_params p, const void *workspace, const char *what) {
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
    return SAETTA_OK;
}

// The caller's workspace if it gave one of at least `need` bytes, else the library's own for this device
// and stream, grown to `need`.  The library's own is held under the lock until the launches that use it
// are queued (the caller keeps `owned_lock` until then): a second host thread on the same stream that has
// to grow it waits for them (hipStreamSynchronize) before it frees.
int acquire_workspace(hipStream_t stream, void *&workspace, size_t workspace_size, size_t need,
                      std::unique_lock<std::mutex> &owned_lock, const char *what, const char *sizer) {
    if (workspace) {
        SAETTA_REQUIRE(workspace_size >= need, SAETTA_E_SCRATCH, "%s: workspace of %zu bytes, %zu needed", what,
                       workspace_size, need);
        return SAETTA_OK;
    }
    // No workspace given: use (and grow) the library's own for this stream.  This may allocate, which a
    // stream under capture cannot do.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
    SAETTA_REQUIRE(capturing == hipStreamCaptureStatusNone, SAETTA_E_SCRATCH,
                   "%s: a stream under capture needs a workspace of the caller's (%zu bytes, %s)", what, need, sizer);
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return fail(int(e), "%s: %s", what, hipGetErrorString(e));
    SAETTA_REQUIRE(dev >= 0 && dev < OWNED_DEVICES, SAETTA_E_DEVICE, "%s: device index %d (up to %d)", what, dev, OWNED_DEVICES - 1);
    owned_lock.lock();
    OwnedWorkspace &w = g_owned[std::make_pair(dev, stream)];
    if (w.bytes < need) {
        if (w.ptr) {
            (void)hipStreamSynchronize(stream);
            (void)hipFree(w.ptr);
        }
        w.ptr = nullptr;
        w.bytes = 0;
        hipError_t e = hipMalloc(&w.ptr, need);
        if (e != hipSuccess) return fail(int(e), "%s: workspace of %zu bytes: %s", what, need, hipGetErrorString(e));
        w.bytes = need;
    }
    workspace = w.ptr;
    return SAETTA_OK;
}

// The images of rows 0 .. rows - 1 of the cache, at the start of the workspace.
uint32_t launch_prepare(hipStream_t stream, int bits, const void *kdata, const void *vdata, const uint16_t *ks,
                        const uint16_t *kz, const uint16_t *vs, const uint16_t *vz, void *workspace, uint32_t kv_heads,
                        uint64_t rows, uint32_t *tiles_taken = nullptr) {
    const uint32_t nblocks = uint32_t((rows + BK - 1) / BK);
    PrepareArgs pa{kdata, vdata, ks, kz, vs, vz, static_cast<unsigned char *>(workspace), kv_heads, nblocks,
                   uint32_t(rows), tiles_taken};
    const dim3 pgrid(nblocks, kv_heads);
    if (bits == 8) {
        prefill_prepare_kernel<8><<<pgrid, PREP_THREADS, 0, stream>>>(pa);
    } else if (bits == 4) {
        prefill_prepare_kernel<4><<<pgrid, PREP_THREADS, 0, stream>>>(pa);
    } else {
        prefill_prepare_kernel<16><<<pgrid, PREP_THREADS, 0, stream>>>(pa);
    }
    return nblocks;
}

int run_prefill(hipStream_t stream, int bits, const uint16_t *q, const void *kdata, const void *vdata,
                const uint16_t *ks, const uint16_t *kz, const uint16_t *vs, const uint16_t *vz,
                const float *q_and_gate, float *out, saetta_flash_params p, void *workspace, size_t workspace_size,
                const char *what) {
    if (int rc = check_prefill(bits, q, kdata, vdata, ks, kz, vs, vz, q_and_gate, out, p, workspace, what)) return rc;
    const uint64_t rows = uint64_t(p.pos) + p.tokens;
    if (int rc = ensure_device()) return rc;
    if (p.tokens == 0) return SAETTA_OK;
    const size_t need = workspace_bytes(p.pos, p.tokens, p.kv_heads);
    std::unique_lock<std::mutex> owned_lock(g_owned_mutex, std::defer_lock);
    if (int rc = acquire_workspace(stream, workspace, workspace_size, need, owned_lock, what, "saetta_prefill_workspace_bytes")) return rc;
    uint32_t *tiles_taken = reinterpret_cast<uint32_t *>(static_cast<unsigned char *>(workspace) + images_bytes(p.pos, p.tokens, p.kv_heads));
    const uint32_t nblocks = launch_prepare(stream, bits, kdata, vdata, ks, kz, vs, vz, workspace, p.kv_heads, rows, tiles_taken);
    PrefillArgs a{q, static_cast<const unsigned char *>(workspace), q_and_gate, out, p.heads, p.kv_heads, p.pos,
                  p.tokens, p.scale, nblocks, tiles_taken};
    // one workgroup per CU at most: a workgroup's LDS ring fills a CU, and further tiles are taken in the kernel
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
        (void)hipGetLastError();
        cus = 256;
    }
    const uint32_t total = (p.tokens + TQ - 1) / TQ * p.kv_heads;
    attention_prefill_kernel<<<dim3(total < uint32_t(cus) ? total : uint32_t(cus)), THREADS, LDS_BYTES, stream>>>(a);
    return launch_status(what);
}

// ---- the same chunk as matrix products over blocks of 1024 keys ---------------------------------
// (reference: AttGemm, src/attention_gemm.rs:95-364, its default variant: prefill_ag_scores_t,
// prefill_ag_pv_t and prefill_ag_final of kernels/attention_gemm.metal.)  The reference's other route to
// the same output: the keys are walked in blocks of 1024; for a block, one launch writes the
// probabilities of every query row against the block's keys to a scratch, relative to the maximum of
// each tile of keys, with the tile's maximum and sum beside them, and a second launch folds the block
// into the running (m, l, O) of every row: O = alpha O + sum over tiles of e^(t - m) (P_tile V_tile).
// The scratch is for one slice of the chunk's tokens; the slices run one after the other.
//
// Here the pair of launches takes a span of AG_SPAN blocks (the scratch holds that many blocks'
// probabilities: q and the output sums then go through memory once per span, and there are as many times
// fewer launches).  A tile is 32 keys (one key image), a row group is 4 tokens x 8 heads as above, and a
// workgroup is 4 waves: a row group each in pv (a 16-token tile), two each in scores.  Both kernels take the
// image parts through LDS (the parts of the tiles ahead are fetched into registers while the current one
// is used; one barrier a tile) and run
// the same transposed products as the flash kernel, so a lane owns a query row in both:
//   scores   S^T = K Q^T (Q^T in registers), mask, tile maximum and sum per row, P = 2^(s - t) as f16,
//            stored as the P^T operands of the second product (the accumulator's registers 8 sp .. 8 sp + 7
//            are the operand of k-step sp: 1 KB per wave and k-step, read back as it was written);
//   pv       m' = max(m, max_t t), O^T = alpha O^T + sum_t V^T_t (f_t P^T_t) with f_t = 2^(t - m') rounded
//            to f16 (the row sum takes the same rounded f_t); the span that holds a tile's last visible
//            key writes out = O / l * sigmoid(gate) instead of O.
constexpr int AG_KEYS = SAETTA_AG_KEYS;
constexpr int AG_TILES = AG_KEYS / BK;
constexpr int AG_SPAN = 8;                // blocks that one pair of launches takes
constexpr int AG_SPAN_TILES = AG_SPAN * AG_TILES;
constexpr int AG_WAVES = 4;
constexpr int AG_THREADS = 64 * AG_WAVES;
constexpr int AG_TOKENS = 4 * AG_WAVES;   // tokens of a workgroup
constexpr int AG_WGS = 512;               // scores: workgroups a launch should have at least (two to a CU)
constexpr int AG_RG = 2;                  // scores: row groups per wave, which share every fragment of keys it reads
constexpr int AG_P_TILE_BYTES = BK * 32 * 2;  // the P^T operands of one row group and tile of keys

struct GemmArgs {
    const uint16_t *q;
    const unsigned char *images;
    const float *q_and_gate;
    float *out;
    unsigned char *p;    // f16 [kv head][token tile][tile of keys][row group of the token tile][2 k-steps][64 lanes][8]
    float *tmax, *tsum;  // [kv head][token tile][tile of keys][row group of the token tile][32 rows], log2 domain
    float *o;            // [kv head][row group][8 dim tiles][4][64 lanes][4]: the accumulators as they are
    float *m, *l;        // [kv head][row group][32 rows]
    uint32_t heads, kv_heads, pos, tokens;  // of the slice
    float c;             // scale * log2(e)
    uint32_t nblocks;    // images per kv head
    uint32_t row_groups; // per kv head in the scratch
    uint32_t g0;         // the first key of the span of blocks the launch takes
    uint32_t split;      // scores: workgroups that share a span's tiles for one token tile (a power of two)
    uint32_t write_out;  // 0: the outputs are never written (timing the passes apart)
};

// Key of the last token of a token tile of `span` tokens at tok0, and how many of the tiles of the launch's span
// of blocks hold keys that some token of the tile can see.
__device__ __forceinline__ uint32_t ag_last_key(const GemmArgs &a, uint32_t tok0, uint32_t span = AG_TOKENS) {
    const uint32_t end = tok0 + span < a.tokens ? tok0 + span : a.tokens;
    return a.pos + end - 1;
}
__device__ __forceinline__ uint32_t ag_tiles(const GemmArgs &a, uint32_t tok0, uint32_t span = AG_TOKENS) {
    const uint32_t last_key = ag_last_key(a, tok0, span);
    if (last_key < a.g0) return 0;
    const uint32_t n = (last_key - a.g0) / BK + 1;
    return n < uint32_t(AG_SPAN_TILES) ? n : uint32_t(AG_SPAN_TILES);
}

__global__ __launch_bounds__(AG_THREADS, 2) void attention_gemm_scores_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(1024))) unsigned char k_lds[3][PART_BYTES];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 31, hf = lane >> 5;
    // a workgroup takes AG_RG token tiles of the pv kernel: a wave AG_RG row groups in a row (8 tokens)
    const uint32_t tok0 = blockIdx.y * (AG_TOKENS * AG_RG), kv = blockIdx.z;
    const uint32_t need = ag_tiles(a, tok0, AG_TOKENS * AG_RG);
    const uint32_t per = AG_SPAN_TILES / a.split;
    const uint32_t first = blockIdx.x * per;
    if (first >= need) return;  // (the whole workgroup)
    const uint32_t count = need - first < per ? need - first : per;
    const uint32_t rg0 = (blockIdx.y * AG_WAVES + wave) * AG_RG;                    // the wave's first row group
    const uint32_t wtok0 = tok0 + 4 * AG_RG * wave, head = kv * SAETTA_GQA_GROUP + (col & 7);  // and its first token

    // A tile's K part goes global -> registers (two register sets, four and three tiles ahead) -> LDS (three
    // buffers, two and one tile ahead) -> MFMA operands.  One barrier a tile.
    const unsigned char *img = a.images + (size_t(kv) * a.nblocks + a.g0 / BK + first) * IMG_BYTES;
    u32x4 pre[2][4];
    // (Fetches and LDS writes past the last tile are made all the same, of the last tile again and into a
    // buffer nobody reads any more: with no branch around a load or a store the compiler knows how many are in
    // flight at each wait, and waits for the oldest only.)
    auto fetch = [&](u32x4 *set, uint32_t t) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(img + size_t(t < count ? t : count - 1) * IMG_BYTES);
#pragma unroll
        for (int i = 0; i < 4; i++) set[i] = src[tid + AG_THREADS * i];
    };
    auto put = [&](const u32x4 *set, uint32_t t) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(k_lds[t % 3]);
#pragma unroll
        for (int i = 0; i < 4; i++) dst[tid + AG_THREADS * i] = set[i];
    };
    fetch(pre[0], 0);
    fetch(pre[1], 1);

    // Q^T operands: lane (col, hf) holds dims 16 f + 8 hf .. + 7 of query row col
    half8 qf[AG_RG][16];
#pragma unroll
    for (int r = 0; r < AG_RG; r++) {
        const uint32_t tok = wtok0 + 4 * r + (col >> 3);
        if (tok < a.tokens) {
            const half8 *qp = reinterpret_cast<const half8 *>(a.q + (size_t(tok) * a.heads + head) * DIM) + hf;
#pragma unroll
            for (int f = 0; f < 16; f++) qf[r][f] = qp[2 * f];
        } else {
#pragma unroll
            for (int f = 0; f < 16; f++) qf[r][f] = half8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    typedef __attribute__((address_space(3))) half8 lds_half8;
    const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(&k_lds[0][0]));
    auto products = [&](uint32_t t, floatx16 (&acc)[AG_RG]) {
        // One address per tile, the fragments by the instruction's offset field (the address is hidden from
        // the loop optimizer, which otherwise keeps sixteen running addresses and two additions a read).
        uint32_t frag = lds0 + (t % 3) * PART_BYTES + lane * 16;
        asm volatile("" : "+v"(frag));
#pragma unroll
        for (int r = 0; r < AG_RG; r++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[r][i] = 0.0f;
#pragma unroll
        for (int f = 0; f < 16; f++) {
            const half8 kf = *reinterpret_cast<const lds_half8 *>(uintptr_t(frag + f * 1024));
#pragma unroll
            for (int r = 0; r < AG_RG; r++) acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[r][f], acc[r], 0, 0, 0);
        }
    };

    auto softmax = [&](floatx16 acc, uint32_t t, int r) {
        const uint32_t rg = rg0 + r;
        const uint32_t limit = a.pos + wtok0 + 4 * r + (col >> 3);  // the last key the row sees
        // slot of (row group, tile) in the scratch: the four row groups of a token tile side by side, tile after
        // tile, so that what a workgroup writes at a step and over its tiles are long runs of memory
        const size_t slot0 = ((size_t(kv) * a.row_groups + rg) / AG_WAVES * AG_SPAN_TILES + first) * AG_WAVES + rg % AG_WAVES;
        // register i is key 8 (i / 4) + 4 hf + i % 4 of the tile.  Only a tile that reaches past the first
        // token of the row group has anything to mask (wave-uniform).
        const uint32_t key0 = a.g0 + (first + t) * BK;
        if (key0 + BK - 1 > a.pos + wtok0 + 4 * r) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t key = key0 + 4 * hf + 8 * (i >> 2) + (i & 3);
                acc[i] = key <= limit ? acc[i] : NO_SCORE;
            }
        }
        // (v_max3 by hand: fmaxf first quiets each operand with a v_max of its own)
        float tmax;
        asm("v_max3_f32 %0, %1, %2, %3" : "=v"(tmax) : "v"(acc[0]), "v"(acc[1]), "v"(acc[2]));
#pragma unroll
        for (int i = 3; i < 15; i += 2) asm("v_max3_f32 %0, %1, %2, %3" : "=v"(tmax) : "v"(tmax), "v"(acc[i]), "v"(acc[i + 1]));
        asm("v_max_f32 %0, %1, %2" : "=v"(tmax) : "v"(tmax), "v"(acc[15]));
        tmax = across_rows<32, 64>(tmax, MaxOp{});
        // scores in the log2 domain: s = acc * c, the tile's maximum t = tmax * c (c > 0).  A masked score is
        // NO_SCORE * c - t: far below any exponent, 0.  With the whole tile masked t would be NO_SCORE * c itself
        // and the difference the product's rounding error: 0 is subtracted then, and every probability is 0.
        const float t_log2 = tmax * a.c;
        const bool none = tmax <= 0.5f * NO_SCORE;
        const float t_sub = none ? 0.0f : t_log2;
        half2_ ph[8];
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float2_ e = {__builtin_amdgcn_exp2f(fmaf(acc[i], a.c, -t_sub)), __builtin_amdgcn_exp2f(fmaf(acc[i + 1], a.c, -t_sub))};
            ph[i / 2] = __builtin_convertvector(e, half2_);
            // the sum of what the second product multiplies: the rounded halves, added in f32
            sum = __builtin_amdgcn_fdot2(ph[i / 2], half2_{(_Float16)1.0f, (_Float16)1.0f}, sum, false);
        }
        sum = across_rows<32, 64>(sum, SumOp{});
        const half8 p0 = {ph[0][0], ph[0][1], ph[1][0], ph[1][1], ph[2][0], ph[2][1], ph[3][0], ph[3][1]};
        const half8 p1 = {ph[4][0], ph[4][1], ph[5][0], ph[5][1], ph[6][0], ph[6][1], ph[7][0], ph[7][1]};
        const float tmax_out = none ? NO_SCORE : t_log2;
        const size_t slot = slot0 + size_t(t) * AG_WAVES;
        unsigned char *pt = a.p + slot * AG_P_TILE_BYTES + lane * 16;
        *reinterpret_cast<half8 *>(pt) = p0;
        *reinterpret_cast<half8 *>(pt + 1024) = p1;
        // (both lanes of a row hold the same two values: one stores the maximum, the other the sum)
        float *stat = (hf ? a.tsum : a.tmax) + slot * 32 + col;
        *stat = hf ? sum : tmax_out;
    };

    put(pre[0], 0);
    fetch(pre[0], 2);
    put(pre[1], 1);
    fetch(pre[1], 3);
    __syncthreads();
    // iteration t: behind its barrier tile t is in LDS (written two iterations ago) and every wave is done with
    // tile t - 1, whose buffer takes tile t + 2 from the register set, which is then sent for tile t + 4.
    auto step = [&](u32x4 *set, uint32_t t) {
        if (t) __syncthreads();
        put(set, t + 2);
        fetch(set, t + 4);
        floatx16 acc[AG_RG];
        products(t, acc);
#pragma unroll
        for (int r = 0; r < AG_RG; r++) softmax(acc[r], t, r);
    };
    // (The first pair stands in front of the loop: the loads and stores in flight where the loop is entered
    // are then the ones in flight where it repeats, and the waits inside it are exact.)
    uint32_t t = 0;
    if (count >= 2) {
        step(pre[0], 0);
        step(pre[1], 1);
        for (t = 2; t + 1 < count; t += 2) {
            step(pre[0], t);
            step(pre[1], t + 1);
        }
    }
    if (t < count) step(pre[0], t);
}

__global__ __launch_bounds__(AG_THREADS, 2) void attention_gemm_pv_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(1024))) unsigned char v_lds[2][PART_BYTES];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 31, hf = lane >> 5;
    const uint32_t tok0 = blockIdx.y * AG_TOKENS, kv = blockIdx.z;
    const uint32_t need = ag_tiles(a, tok0);
    if (need == 0) return;  // nothing of this span (the outputs were written at an earlier one)
    const bool last_block = ag_last_key(a, tok0) < a.g0 + AG_SPAN * AG_KEYS;
    const uint32_t rg = blockIdx.y * AG_WAVES + wave;
    const uint32_t tok = tok0 + 4 * wave + (col >> 3), head = kv * SAETTA_GQA_GROUP + (col & 7);
    const size_t rows = size_t(kv) * a.row_groups + rg;
    const size_t state = rows * 32 + col;
    const bool first_block = a.g0 == 0;

    // slot of (row group, tile): as the scores kernel wrote them
    const size_t slot0 = rows / AG_WAVES * AG_SPAN_TILES * AG_WAVES + wave;
    const float *tm = a.tmax + slot0 * 32 + col, *ts = a.tsum + slot0 * 32 + col;
    // (all of the block's tile maxima requested at once: a loop over `need` waits for each load in turn)
    float mb = NO_SCORE;
    for (uint32_t c = 0; c < need; c += 64) {  // (64 at a time: so many registers are free here)
        float tmaxes[64];
#pragma unroll
        for (int t = 0; t < 64; t++) tmaxes[t] = tm[(c + t < need ? c + t : need - 1) * AG_WAVES * 32];
#pragma unroll
        for (int t = 0; t < 64; t++) mb = fmaxf(mb, tmaxes[t]);
    }
    // (every row sees key 0, so m is a score from the first block on)
    const float m_old = first_block ? NO_SCORE : a.m[state], l_old = first_block ? 0.0f : a.l[state];
    const float m_new = fmaxf(m_old, mb);
    const float alpha = first_block ? 0.0f : __builtin_amdgcn_exp2f(m_old - m_new);

    floatx16 acc[8];
    float *op = a.o + rows * 8 * 1024 + lane * 4;
    if (first_block) {
#pragma unroll
        for (int mt = 0; mt < 8; mt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mt][i] = 0.0f;
    } else {
#pragma unroll
        for (int mt = 0; mt < 8; mt++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                const floatx4 x = *reinterpret_cast<const floatx4 *>(op + (mt * 4 + q4) * 256);
#pragma unroll
                for (int e = 0; e < 4; e++) acc[mt][4 * q4 + e] = x[e] * alpha;
            }
    }

    // the V^T part of an image
    const unsigned char *img = a.images + (size_t(kv) * a.nblocks + a.g0 / BK) * IMG_BYTES + PART_BYTES;
    // a tile's operands are fetched into registers two tiles ahead (two register sets, the loop in pairs)
    struct Ahead {
        u32x4 v[4];
        half8 p0, p1;
        float tm, ts;
    } pre[2];
    const unsigned char *pp = a.p + slot0 * AG_P_TILE_BYTES + lane * 16;
    auto fetch = [&](Ahead &set, uint32_t t) {  // (past the last tile: the last tile again, never used)
        t = t < need ? t : need - 1;
        const u32x4 *src = reinterpret_cast<const u32x4 *>(img + size_t(t) * IMG_BYTES);
#pragma unroll
        for (int i = 0; i < 4; i++) set.v[i] = src[tid + AG_THREADS * i];
        set.p0 = *reinterpret_cast<const half8 *>(pp + size_t(t) * AG_WAVES * AG_P_TILE_BYTES);
        set.p1 = *reinterpret_cast<const half8 *>(pp + size_t(t) * AG_WAVES * AG_P_TILE_BYTES + 1024);
        set.tm = tm[t * AG_WAVES * 32], set.ts = ts[t * AG_WAVES * 32];
    };
    fetch(pre[0], 0);
    fetch(pre[1], 1);
    float lsum = 0.0f;
    auto tile = [&](Ahead &set, uint32_t t) {
        unsigned char *buf = v_lds[t & 1];
#pragma unroll
        for (int i = 0; i < 4; i++) reinterpret_cast<u32x4 *>(buf)[tid + AG_THREADS * i] = set.v[i];
        __syncthreads();
        half8 pc0 = set.p0, pc1 = set.p1;
        const float tmc = set.tm, tsc = set.ts;
        fetch(set, t + 2);
        // a tile the row sees nothing of has t = NO_SCORE: its factor is 0, like its probabilities
        const _Float16 fh = (_Float16)__builtin_amdgcn_exp2f(tmc - m_new);
        lsum += (float)fh * tsc;
        pc0 *= fh, pc1 *= fh;
#pragma unroll
        for (int mt = 0; mt < 8; mt++) {
            const half8 v0 = *reinterpret_cast<const half8 *>(buf + (2 * mt) * 1024 + lane * 16);
            const half8 v1 = *reinterpret_cast<const half8 *>(buf + (2 * mt + 1) * 1024 + lane * 16);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(v0, pc0, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(v1, pc1, acc[mt], 0, 0, 0);
        }
    };
    uint32_t t = 0;
    if (need >= 2) {  // (the first pair in front of the loop, as in the scores kernel)
        tile(pre[0], 0);
        tile(pre[1], 1);
        for (t = 2; t + 1 < need; t += 2) {
            tile(pre[0], t);
            tile(pre[1], t + 1);
        }
    }
    if (t < need) tile(pre[0], t);
    const float l_new = alpha * l_old + lsum;

    if (last_block && a.write_out) {
        if (tok < a.tokens) {
            const float inv = 1.0f / l_new;
            const size_t row = size_t(tok) * a.heads + head;
#pragma unroll
            for (int dh = 0; dh < 2; dh++) {  // (half of the dims at a time: 16 gate loads in flight)
                const float *gate = a.q_and_gate + row * 2 * DIM + DIM + 128 * dh + 4 * hf;
                float *out = a.out + row * DIM + 128 * dh + 4 * hf;
                floatx4 g[16];
#pragma unroll
                for (int i = 0; i < 16; i++) g[i] = *reinterpret_cast<const floatx4 *>(gate + 32 * (i >> 2) + 8 * (i & 3));
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int mt = 4 * dh + (i >> 2), q4 = i & 3;
                    floatx4 w;
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = acc[mt][4 * q4 + e] * inv * __builtin_amdgcn_rcpf(1.0f + __expf(-g[i][e]));
                    *reinterpret_cast<floatx4 *>(out + 32 * (i >> 2) + 8 * q4) = w;
                }
                asm volatile("" ::: "memory");
            }
        }
        return;
    }
    if (hf == 0) a.m[state] = m_new, a.l[state] = l_new;
#pragma unroll
    for (int mt = 0; mt < 8; mt++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            floatx4 x;
#pragma unroll
            for (int e = 0; e < 4; e++) x[e] = acc[mt][4 * q4 + e];
            *reinterpret_cast<floatx4 *>(op + (mt * 4 + q4) * 256) = x;
        }
}

size_t align_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

// Row groups of the scratch per kv head for slices of up to `slice` tokens: whole workgroups.
size_t gemm_row_groups(uint32_t slice) {
    constexpr uint32_t SPAN = AG_TOKENS * AG_RG;  // what a scores workgroup covers
    return size_t((slice + SPAN - 1) / SPAN) * AG_WAVES * AG_RG;
}

size_t gemm_scratch_bytes(uint32_t slice, uint32_t kv_heads) {
    const size_t groups = gemm_row_groups(slice) * kv_heads;
    return groups * (size_t(AG_SPAN_TILES) * AG_P_TILE_BYTES + 2 * size_t(AG_SPAN_TILES) * 32 * 4 + 32 * size_t(DIM) * 4 + 2 * 32 * 4);
}

uint32_t gemm_slice(uint32_t tokens, uint32_t slice_tokens) {
    return slice_tokens == 0 || slice_tokens > tokens ? tokens : slice_tokens;
}

size_t gemm_workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t slice_tokens, uint32_t kv_heads) {
    return align_up(workspace_bytes(pos, tokens, kv_heads), 256) + gemm_scratch_bytes(gemm_slice(tokens, slice_tokens), kv_heads);
}

int run_gemm(hipStream_t stream, int bits, const uint16_t *q, const void *kdata, const void *vdata, const uint16_t *ks,
             const uint16_t *kz, const uint16_t *vs, const uint16_t *vz, const float *q_and_gate, float *out,
             saetta_flash_params p, uint32_t slice_tokens, uint32_t stages, void *workspace, size_t workspace_size) {
    const char *what = "attn_gemm";
    if (int rc = check_prefill(bits, q, kdata, vdata, ks, kz, vs, vz, q_and_gate, out, p, workspace, what)) return rc;
    SAETTA_REQUIRE(stages <= 3, SAETTA_E_SHAPE, "%s: stages %u (0: all passes; 1, 2: scores only; 3: no outputs)", what, stages);
    const uint64_t rows = uint64_t(p.pos) + p.tokens;
    if (int rc = ensure_device()) return rc;
    if (p.tokens == 0) return SAETTA_OK;
    const uint32_t slice = gemm_slice(p.tokens, slice_tokens);
    const size_t need = gemm_workspace_bytes(p.pos, p.tokens, slice, p.kv_heads);
    std::unique_lock<std::mutex> owned_lock(g_owned_mutex, std::defer_lock);
    if (int rc = acquire_workspace(stream, workspace, workspace_size, need, owned_lock, what, "saetta_attn_gemm_workspace_bytes")) return rc;
    const uint32_t nblocks = launch_prepare(stream, bits, kdata, vdata, ks, kz, vs, vz, workspace, p.kv_heads, rows);

    const size_t groups = gemm_row_groups(slice) * p.kv_heads;
    unsigned char *at = static_cast<unsigned char *>(workspace) + align_up(workspace_bytes(p.pos, p.tokens, p.kv_heads), 256);
    GemmArgs a{};
    a.images = static_cast<const unsigned char *>(workspace);
    a.p = at, at += groups * AG_SPAN_TILES * AG_P_TILE_BYTES;
    a.tmax = reinterpret_cast<float *>(at), at += groups * AG_SPAN_TILES * 32 * 4;
    a.tsum = reinterpret_cast<float *>(at), at += groups * AG_SPAN_TILES * 32 * 4;
    a.o = reinterpret_cast<float *>(at), at += groups * 32 * DIM * 4;
    a.m = reinterpret_cast<float *>(at), at += groups * 32 * 4;
    a.l = reinterpret_cast<float *>(at);
    a.heads = p.heads, a.kv_heads = p.kv_heads;
    a.c = p.scale * 1.4426950408889634f;
    a.nblocks = nblocks;
    a.row_groups = uint32_t(gemm_row_groups(slice));
    a.write_out = stages == 0;
    const size_t width = size_t(p.heads) * DIM;
    // A slice of tokens is a chunk of its own at pos + t0: its rows of q, q_and_gate and out, the whole
    // cache (src/attention_gemm.rs:162-188).
    for (uint32_t t0 = 0; t0 < p.tokens; t0 += slice) {
        a.tokens = p.tokens - t0 < slice ? p.tokens - t0 : slice;
        a.pos = p.pos + t0;
        a.q = q + t0 * width, a.q_and_gate = q_and_gate + t0 * width * 2, a.out = out + t0 * width;
        const uint32_t tiles = (a.tokens + AG_TOKENS - 1) / AG_TOKENS;
        const uint64_t end = uint64_t(a.pos) + a.tokens;
        // scores: as many workgroups per token tile as make AG_WGS in all (2 for chunks of 4096 tokens, 4 for 2048)
        const uint32_t wide = (tiles + AG_RG - 1) / AG_RG;
        a.split = 2;
        while (a.split < 16 && a.split * wide * p.kv_heads < uint32_t(AG_WGS)) a.split *= 2;
        // a span of AG_SPAN blocks of AG_KEYS keys at a time: its scores, then its pv
        for (uint64_t g0 = 0; g0 < end; g0 += uint64_t(AG_SPAN) * AG_KEYS) {
            a.g0 = uint32_t(g0);
            attention_gemm_scores_kernel<<<dim3(a.split, wide, p.kv_heads), AG_THREADS, 0, stream>>>(a);
            if (stages == 1 || stages == 2) continue;
            attention_gemm_pv_kernel<<<dim3(1, tiles, p.kv_heads), AG_THREADS, 0, stream>>>(a);
        }
    }
    return launch_status(what);
}

}  // namespace

int setup_prefill() {
    if (int rc = load_kernel(reinterpret_cast<const void *>(attention_prefill_kernel))) return rc;
    if (int rc = load_kernel(reinterpret_cast<const void *>(attention_gemm_scores_kernel))) return rc;
    if (int rc = load_kernel(reinterpret_cast<const void *>(attention_gemm_pv_kernel))) return rc;
    return int(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_prefill_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
}
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

extern "C" size_t saetta_attn_gemm_workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t slice_tokens, uint32_t kv_heads) {
    return gemm_workspace_bytes(pos, tokens, slice_tokens, kv_heads);
}

extern "C" int saetta_attn_gemm(saetta_stream_t stream, int bits, const uint16_t *q_f16, saetta_quant_rows keys,
                                saetta_quant_rows values, const float *q_and_gate, float *out, saetta_flash_params p,
                                uint32_t slice_tokens, uint32_t stages, void *workspace, size_t workspace_bytes) {
    return run_gemm(as_stream(stream), bits, q_f16, keys.data, values.data, keys.scales, keys.biases, values.scales,
                    values.biases, q_and_gate, out, p, slice_tokens, stages, workspace, workspace_bytes);
}
