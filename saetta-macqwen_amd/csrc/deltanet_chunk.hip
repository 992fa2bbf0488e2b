// Gated DeltaNet over the tokens of a prefill chunk on the matrix cores: the delta rule in its
// chunked form, blocks of 64 tokens.
//
// What it computes is what deltanet_rows_kernel computes token by token (the reference's definition:
// src/cpu/deltanet.rs:69-155, delta_rule :148-155; the kernels it stands for: delta_prep + delta_rows3,
// kernels/prefill.metal:788-1116): per value head, with state S [v_dim][128],
//     S <- g_t S;  u_t = beta_t (v_t - S k_t);  S += u_t k_t^T;  o_t = S q_t.
// Inside a block of C = 64 tokens, with c_t = sum_{r <= t} log g_r and S0 the state before the block,
//     S_t = e^{c_t} S0 + sum_{s <= t} e^{c_t - c_s} u_s k_s^T,
// so the u_t solve a triangular system that does not involve the state's rows one by one:
//     (I + A) U = diag(beta) (V - diag(e^c) K S0^T),   A_ts = beta_t e^{c_t - c_s} (k_t . k_s)  (s < t)
//     O = diag(e^c) Q S0^T + M U,                       M_ts = e^{c_t - c_s} (q_t . k_s)         (s <= t)
//     S1^T = e^{c_last} S0^T + K^T diag(e^{c_last - c}) U
// (U, V, O: [C][v_dim]; K, Q: [C][128], normalised as the reference does).  Two kernels:
//   deltanet_chunk_prepare_kernel   one workgroup per (block, key head) with its two value heads (or per
//       value head, for another ratio), all blocks at once: the
//       normalised q and k, A and M (64 x 64 x 128 products), T = (I + A)^-1 diag(beta) by forward
//       substitution, and the decay factors, to a workspace;
//   deltanet_chunk_chain_kernel     one workgroup per (16 value dims, value head) walks the blocks in
//       order with its slice of the state in registers: five small products per block.
// All products run on v_mfma_f32_16x16x32_f16 with every operand split into an f16 hi and lo part
// (hi * hi + hi * lo + lo * hi: about 2^-21 relative, against 2^-24 of the f32 chain; f32 MFMA has an
// eighth of the rate per k and wants one LDS read per operand element).  The exponents e^{c_t - c_s}
// never exceed 1 and come from running sums of log g kept in f64 (in f32 the difference of two sums of
// some tens loses what the product of the g themselves keeps).  The output differs from the
// token-by-token kernels' by rounding only (tests hold it to 2e-5 of the largest value, also over a
// 4096-token chunk; measured 2e-6).
#include "common.hpp"
#include "deltanet_gates.hpp"
#include "lanes.hpp"

#include <type_traits>

namespace saetta {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int K_DIM = 128;
constexpr int C = 64;                 // tokens per block
constexpr int DV = 16;                // value dims per workgroup of the chain kernel (32: 317 against 253 us per 4096 tokens)
constexpr float Q_SCALE = 0.08838834764831845f;  // 1 / sqrt(128), the reference's factor on q
// LDS images of the prepare kernel: rows padded so that 16 rows' 16-byte reads fall on all banks
constexpr int KROW = K_DIM + 8;       // f16 per row of a q / k image: 272 bytes
constexpr int TROW = C + 8;           // f16 per row of a T / M image (and of the chain's [dv][token] images): 144 bytes
constexpr int K_IMG = C * KROW * 2;   // bytes: 17408
constexpr int T_IMG = C * TROW * 2;   // bytes: 9216

// Workspace, per block.  Everything the chain kernel reads lies in the order its waves take it as MFMA
// operands: an operand of a wave is 64 lanes x 16 bytes = 1 KB (lane (n, j): row or column n, 8 values of
// the k index from 8j), so a load instruction of a wave reads one contiguous kilobyte.
//   per key head:   K hi | K lo | Q hi | Q lo   [wave 4][k-step 4][lane]: row 16 wave + n, key dims 32 ks + 8j ..
//   per value head: T hi | T lo | M hi | M lo   [wave 4][k-step 2][lane]: row 16 wave + n, columns 32 ks + 8j ..
//                   128 floats: e^{c_t} and e^{c_last - c_t}
constexpr int OPERAND = 1024;
constexpr int K_GL = 4 * 4 * OPERAND, T_GL = 4 * 2 * OPERAND;
constexpr size_t KHEAD_BYTES = 4 * size_t(K_GL);
constexpr size_t VHEAD_BYTES = 4 * size_t(T_GL) + 2 * C * sizeof(float);
__host__ __device__ inline size_t block_bytes(uint32_t k_heads, uint32_t v_heads) { return k_heads * KHEAD_BYTES + v_heads * VHEAD_BYTES; }

struct ChunkArgs {
    const float *mixed, *a, *b, *a_log, *dt_bias;
    float *state;
    float *o;  // [tokens][v_heads][v_dim], before the gated norm
    unsigned char *ws;
    uint32_t k_heads, v_heads, v_dim, tokens, channels;
    float eps;
};

// x as an f16 hi part and an f16 lo part.  The lo part has to complete the hi part that is stored: where x is
// a product, the compiler may round the exact product to f16 for the one and the f32 product for the other, and
// next to a midpoint between two f16 numbers the two roundings differ by an ulp of the hi part (one value in
// some thousands: an error of 2^-11 of it instead of 2^-22).  So x is pinned as the f32 number it is, and the
// hi part as the number that the lo part is taken against.
__device__ __forceinline__ void split2(float x, _Float16 &hi, _Float16 &lo) {
    asm volatile("" : "+v"(x));
    float h = (float)(_Float16)x;
    asm volatile("" : "+v"(h));
    hi = (_Float16)h;  // (exact)
    lo = (_Float16)(x - h);
}

// acc += A B with both operands in hi and lo parts
__device__ __forceinline__ floatx4 mma3(half8 ah, half8 al, half8 bh, half8 bl, floatx4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bh, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bl, acc, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bh, acc, 0, 0, 0);
}

// ---- prepare: everything of a block that does not depend on the state ------------------------------
// One workgroup takes G value heads of one key head: the q / k images and the k . k and q . k products
// belong to the key head, the gates, A, M and T to a value head.  (G = 2, the model's two value heads
// per key head: the four waves take the heads' four diagonal blocks of the triangular solve; G = 1: any
// other ratio, one workgroup per value head, the first of a key head's writing the key head's images.)
// LDS: the four q / k images; once the products are taken, the heads' A (f32) go over kh | kl, their M
// images and later their T images over qh | ql (and 2 KB more), so that they leave as whole 16-byte stores.
template <int G>
struct PrepLds {
    // per head, over kh | kl once the products are taken: the two diagonal 32 x 32 blocks of A as f32, rows of
    // DROW ([t][q * 16 + m] holds A_t,s of s = 2m + q; the product of the off-diagonal block goes over them
    // later), then the block below the diagonal and the inverse of the second diagonal block as f16 images
    static constexpr int DROW = 32 + 4, D_BYTES = 32 * DROW * 4;
    static constexpr int HROW = 32 + 8, H_IMG = 32 * HROW * 2;  // f16 per row of a 32 x 32 image; bytes of one part
    static constexpr int W_OFF = 0, LBA_OFF = 2 * D_BYTES, XBB_OFF = LBA_OFF + 2 * H_IMG, HEAD_BYTES = XBB_OFF + 2 * H_IMG;
    static_assert(2 * H_IMG <= 2 * D_BYTES, "the product's images fit over the diagonal blocks");
    static constexpr int M_BYTES = 2 * T_IMG;  // mh | ml (then th | tl) of a head
    static constexpr int M_OFF = G * HEAD_BYTES > 2 * K_IMG ? G * HEAD_BYTES : 2 * K_IMG;
    static constexpr int GATES = M_OFF + G * M_BYTES > 4 * K_IMG ? M_OFF + G * M_BYTES : 4 * K_IMG;  // [head]: cum f64 [C] | beta f32 [C]
    static constexpr int GATE_BYTES = C * 8 + C * 4;
    static constexpr int BYTES = GATES + G * GATE_BYTES;
    static_assert(2 * BYTES <= 160 * 1024, "two workgroups per CU");
};

// The B operand of a 16-column tile out of a row-major f16 image in LDS (hi part at `at`, lo part `part_bytes`
// on; `at`: the byte address of row 8j + e, column 4a of the tile for lane a + 4e of its 16): lane (n, j)
// gets column n of rows 8j .. 8j + 7.  ds_read_b64_tr_b16 works on 16 lanes: lane a + 4e of them names 8
// bytes (4 values of a row), and lane 4a + c receives value c of the lanes a, a + 4, a + 8, a + 12.
__device__ __forceinline__ void read_by_column(uint32_t at, uint32_t part_bytes, uint32_t four_rows_bytes, half8 &hi, half8 &lo) {
    u32x2 r[2][2];
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r[0][0]) : "v"(at) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r[0][1]) : "v"(at + four_rows_bytes) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r[1][0]) : "v"(at + part_bytes) : "memory");
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r[1][1]) : "v"(at + part_bytes + four_rows_bytes) : "memory");
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[1][0]), "+v"(r[1][1])::"memory");
    hi = __builtin_bit_cast(half8, u32x4{r[0][0].x, r[0][0].y, r[0][1].x, r[0][1].y});
    lo = __builtin_bit_cast(half8, u32x4{r[1][0].x, r[1][0].y, r[1][1].x, r[1][1].y});
}

template <int G>
__global__ __launch_bounds__(256) void deltanet_chunk_prepare_kernel(ChunkArgs a) {
    using L = PrepLds<G>;
    constexpr int DROW = L::DROW, HROW = L::HROW;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    _Float16 *kh = reinterpret_cast<_Float16 *>(lds), *kl = kh + C * KROW, *qh = kl + C * KROW, *ql = qh + C * KROW;
    auto diag_lds = [&](int hh, int half) { return reinterpret_cast<float *>(lds + hh * L::HEAD_BYTES + half * L::D_BYTES); };
    auto half_img = [&](int hh, int off) { return reinterpret_cast<_Float16 *>(lds + hh * L::HEAD_BYTES + off); };  // hi part; lo: 32 * HROW on
    auto m_lds = [&](int hh) { return reinterpret_cast<_Float16 *>(lds + L::M_OFF + hh * L::M_BYTES); };
    // The running sums of log g are kept in f64: the decay between two tokens is e^(c_t - c_s), the sums reach
    // -100 and beyond inside a block, and an f32 difference of two of them carries the ulp of the sums (1e-5), which
    // is then the relative error of every entry of A and M: three orders above the rest of this path's arithmetic.
    auto cum_lds = [&](int hh) { return reinterpret_cast<double *>(lds + L::GATES + hh * L::GATE_BYTES); };
    auto beta_lds = [&](int hh) { return reinterpret_cast<float *>(lds + L::GATES + hh * L::GATE_BYTES + C * 8); };
    const uint32_t blk = blockIdx.x, group = a.v_heads / a.k_heads;
    const uint32_t h0 = blockIdx.y * G, khd = h0 / group;  // the workgroup's first value head, its key head
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), n = lane & 15, j = lane >> 4;
    const uint32_t key_size = a.k_heads * K_DIM;
    unsigned char *ws_blk = a.ws + size_t(blk) * block_bytes(a.k_heads, a.v_heads);
    unsigned char *ws_k = ws_blk + khd * KHEAD_BYTES;
    auto ws_v = [&](int hh) { return ws_blk + a.k_heads * KHEAD_BYTES + (h0 + hh) * VHEAD_BYTES; };
    const bool writer = h0 % group == 0;  // one workgroup of the key head's keeps the q / k images

    // ---- q and k of the block's tokens, normalised (src/cpu/deltanet.rs:133-146), as hi and lo parts ----
    {
        // thread (token t, part): the 8-value pieces part, part + 4, part + 8, part + 12 of the token's q and k, so
        // that the four threads of a token read 128 bytes in a row with every pair of loads
        const uint32_t t = tid >> 2, part = tid & 3, tok = blk * C + t;
        float4 qv[8], kv[8];
        float qs = 0.0f, ks = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            qv[i] = kv[i] = make_float4(0, 0, 0, 0);
            if (tok < a.tokens) {
                const float *row = a.mixed + size_t(tok) * a.channels + khd * K_DIM + 8 * (part + 4 * (i >> 1)) + 4 * (i & 1);
                qv[i] = *reinterpret_cast<const float4 *>(row);
                kv[i] = *reinterpret_cast<const float4 *>(row + key_size);
            }
            qs += qv[i].x * qv[i].x + qv[i].y * qv[i].y + qv[i].z * qv[i].z + qv[i].w * qv[i].w;
            ks += kv[i].x * kv[i].x + kv[i].y * kv[i].y + kv[i].z * kv[i].z + kv[i].w * kv[i].w;
        }
        qs = group_reduce<4>(qs, SumOp());
        ks = group_reduce<4>(ks, SumOp());
        const bool real = tok < a.tokens;
        // (q's factor 1 / sqrt(128) is applied to the output: at unit length the lo parts stay clear of the f16 underflow)
        const float qi = real ? __builtin_amdgcn_rsqf(qs + a.eps) : 0.0f;
        const float ki = real ? __builtin_amdgcn_rsqf(ks + a.eps) : 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            half8 a_qh, a_ql, a_kh, a_kl;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float4 qq = qv[i + e / 4], kk = kv[i + e / 4];
                const float qf = (e % 4 == 0 ? qq.x : e % 4 == 1 ? qq.y : e % 4 == 2 ? qq.z : qq.w) * qi;
                const float kf = (e % 4 == 0 ? kk.x : e % 4 == 1 ? kk.y : e % 4 == 2 ? kk.z : kk.w) * ki;
                _Float16 hi, lo;
                split2(qf, hi, lo);
                a_qh[e] = hi, a_ql[e] = lo;
                split2(kf, hi, lo);
                a_kh[e] = hi, a_kl[e] = lo;
            }
            const int at = t * KROW + 8 * (part + 2 * i);  // piece part + 4 (i / 2): key dims 32 (i / 2) + 8 part ..
            *reinterpret_cast<half8 *>(kh + at) = a_kh, *reinterpret_cast<half8 *>(kl + at) = a_kl;
            *reinterpret_cast<half8 *>(qh + at) = a_qh, *reinterpret_cast<half8 *>(ql + at) = a_ql;
            if (writer) {
                // operand (wave t / 16, k-step i / 2), lane (n = t % 16, j = part): a wave's store is one kilobyte in a row
                unsigned char *g = ws_k + ((((t >> 4) * 4 + (i >> 1)) * 64 + part * 16 + (t & 15)) * 16);
                *reinterpret_cast<half8 *>(g) = a_kh, *reinterpret_cast<half8 *>(g + K_GL) = a_kl;
                *reinterpret_cast<half8 *>(g + 2 * K_GL) = a_qh, *reinterpret_cast<half8 *>(g + 3 * K_GL) = a_ql;
            }
        }
    }
    // ---- the gates of head h0 + wave: c_t = sum of log g up to t, beta_t (tokens past the end: g = 1, beta = 0) ----
    if (wave < G) {
        const uint32_t tok = blk * C + lane, h = h0 + wave;
        float lg = 0.0f, beta = 0.0f;
        if (tok < a.tokens) {
            float g;
            fast_gates(a.a[size_t(tok) * a.v_heads + h] + a.dt_bias[h], __expf(a.a_log[h]), a.b[size_t(tok) * a.v_heads + h], g, beta, &lg);
        }
        // inclusive sum over the 64 lanes
        double c = lg;
#pragma unroll
        for (int d = 1; d < 64; d *= 2) {
            const double up = __shfl_up(c, d, 64);
            if (int(lane) >= d) c += up;
        }
        cum_lds(wave)[lane] = c, beta_lds(wave)[lane] = beta;
        const double last = __shfl(c, 63, 64);
        float *gam = reinterpret_cast<float *>(ws_v(wave) + 4 * T_GL);
        gam[lane] = __expf(float(c)), gam[C + lane] = __expf(float(last - c));
    }
    __syncthreads();

    // ---- k . k and q . k: rows 16 wave .. + 15, the column tiles at and below the diagonal ----
    floatx4 gk[4], gq[4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        gk[nt] = gq[nt] = floatx4{0, 0, 0, 0};
        if (nt <= int(wave)) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const int ao = (16 * wave + n) * KROW + 32 * ks + 8 * j, bo = (16 * nt + n) * KROW + 32 * ks + 8 * j;
                const half8 bh = *reinterpret_cast<const half8 *>(kh + bo), bl = *reinterpret_cast<const half8 *>(kl + bo);
                gk[nt] = mma3(*reinterpret_cast<const half8 *>(kh + ao), *reinterpret_cast<const half8 *>(kl + ao), bh, bl, gk[nt]);
                gq[nt] = mma3(*reinterpret_cast<const half8 *>(qh + ao), *reinterpret_cast<const half8 *>(ql + ao), bh, bl, gq[nt]);
            }
        }
    }
    __syncthreads();  // the images are read: A and M go over them

    // C layout: lane (n, j) holds column s = 16 nt + n of rows t = 16 wave + 4j + i
#pragma unroll
    for (int hh = 0; hh < G; hh++) {
#pragma unroll
        for (int nt = 0; nt < 4; nt++) {
            const uint32_t s = 16 * nt + n;
            const double cs = cum_lds(hh)[s];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t t = 16 * wave + 4 * j + i;
                const float decay = s <= t ? __expf(float(cum_lds(hh)[t] - cs)) : 0.0f;
                const float at_s = s < t ? beta_lds(hh)[t] * decay * gk[nt][i] : 0.0f;
                if ((nt >> 1) == int(wave >> 1)) {  // a diagonal 32 x 32 block, zeros above the diagonal included
                    diag_lds(hh, nt >> 1)[(t & 31) * DROW + (s & 1) * 16 + ((s & 31) >> 1)] = at_s;
                } else if (nt < 2) {  // the block below the diagonal, as an MFMA operand
                    _Float16 hi, lo;
                    split2(at_s, hi, lo);
                    half_img(hh, L::LBA_OFF)[(t - 32) * HROW + s] = hi, half_img(hh, L::LBA_OFF)[32 * HROW + (t - 32) * HROW + s] = lo;
                }
                _Float16 hi, lo;
                split2(decay * gq[nt][i], hi, lo);
                m_lds(hh)[t * TROW + s] = hi, m_lds(hh)[C * TROW + t * TROW + s] = lo;
            }
        }
    }
    __syncthreads();
    // A staged matrix leaves in operand order, 16 bytes per piece: piece (part hi | lo, wave w, k-step ks, lane (n, j))
    // is row 16 w + n, columns 32 ks + 8j .. of the part's image
    auto leave = [&](int hh, unsigned char *dst) {
        for (uint32_t i = tid; i < 2 * T_GL / 16; i += 256) {
            const uint32_t part = i >> 9, w = (i >> 7) & 3, ks = (i >> 6) & 1, nn = i & 15, jj = (i >> 4) & 3;
            reinterpret_cast<u32x4 *>(dst)[i] = *reinterpret_cast<const u32x4 *>(m_lds(hh) + part * C * TROW + (16 * w + nn) * TROW + 32 * ks + 8 * jj);
        }
    };
#pragma unroll
    for (int hh = 0; hh < G; hh++) leave(hh, ws_v(hh) + 2 * T_GL);

    // ---- T = (I + A)^-1 diag(beta), in 32 x 32 blocks: with L = I + A = [[L_AA, 0], [L_BA, L_BB]],
    //     T_AA = L_AA^-1 diag(beta_A),  T_BB = L_BB^-1 diag(beta_B),  T_BA = -L_BB^-1 (L_BA T_AA).
    // The diagonal blocks by forward substitution, one wave per (head, block): lane (column c, q) solves
    // x_t = [t = c] - sum_{s < t} A_ts x_s, lane group q keeps x_s of s = 2m + q in slot m and adds up those s.
    // The block below the diagonal: two products on the matrix cores. ----
    {
        const uint32_t hs = G == 2 ? wave >> 1 : 0, half = wave & 1;  // the wave's head and diagonal block
        const bool solver = G == 2 || wave < 2;
        const uint32_t c = lane & 31, q = lane >> 5;
        float x[16];
#pragma unroll
        for (int m = 0; m < 16; m++) x[m] = 0.0f;
        if (solver) {
            const float *ad = diag_lds(hs, half) + q * 16;
#pragma unroll
            for (int t = 0; t < 32; t++) {
                floatx4 part4 = {0, 0, 0, 0};  // (four chains of sums instead of one of up to 16)
#pragma unroll
                for (int m4 = 0; 8 * m4 < t; m4++) {  // s = 2m + q < t needs m <= (t - 1) / 2
                    const floatx4 av = *reinterpret_cast<const floatx4 *>(ad + t * DROW + 4 * m4);
#pragma unroll
                    for (int e = 0; e < 4; e++) part4[e] += av[e] * x[4 * m4 + e];
                }
                const float sum = across_rows<32, 64>((part4[0] + part4[1]) + (part4[2] + part4[3]), SumOp());
                const float xt = (uint32_t(t) == c ? 1.0f : 0.0f) - sum;
                if (q == uint32_t(t & 1)) x[t >> 1] = xt;
            }
        }
        __syncthreads();  // M has left: T goes over it
        if (solver) {
            const float bc = beta_lds(hs)[32 * half + c];
            _Float16 *th = m_lds(hs), *tl = th + C * TROW;
#pragma unroll
            for (int m = 0; m < 16; m++) {
                const uint32_t t = 2 * m + q;
                _Float16 hi, lo;
                split2(x[m] * bc, hi, lo);
                th[(32 * half + t) * TROW + 32 * half + c] = hi, tl[(32 * half + t) * TROW + 32 * half + c] = lo;
                if (half == 0) {
                    th[t * TROW + 32 + c] = (_Float16)0.0f, tl[t * TROW + 32 + c] = (_Float16)0.0f;  // nothing above the diagonal
                } else {
                    split2(x[m], hi, lo);
                    half_img(hs, L::XBB_OFF)[t * HROW + c] = hi, half_img(hs, L::XBB_OFF)[32 * HROW + t * HROW + c] = lo;
                }
            }
        }
        __syncthreads();
        // W = L_BA T_AA and then T_BA = -L_BB^-1 W: a wave takes 16 rows (two column tiles of its head; with one
        // head, one tile).  The right operands are read by column out of row-major images.
        const uint32_t r = wave & 1, la = lane & 3, le = (lane >> 2) & 3;
        const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(lds));
        floatx4 w[2];
#pragma unroll
        for (int ct = 0; ct < 2; ct++) {
            if (G == 1 && ct != int(wave >> 1)) continue;
            const int ao = (16 * r + n) * HROW + 8 * j;
            half8 bh, bl;
            read_by_column(lds0 + L::M_OFF + hs * L::M_BYTES + ((8 * j + le) * TROW + 16 * ct + 4 * la) * 2, C * TROW * 2, 4 * TROW * 2, bh, bl);
            w[ct] = mma3(*reinterpret_cast<const half8 *>(half_img(hs, L::LBA_OFF) + ao),
                         *reinterpret_cast<const half8 *>(half_img(hs, L::LBA_OFF) + 32 * HROW + ao), bh, bl, floatx4{0, 0, 0, 0});
        }
        // (the diagonal blocks were last read before the barrier above)
#pragma unroll
        for (int ct = 0; ct < 2; ct++) {
            if (G == 1 && ct != int(wave >> 1)) continue;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                _Float16 hi, lo;
                split2(w[ct][i], hi, lo);
                const int at = (16 * r + 4 * j + i) * HROW + 16 * ct + n;
                half_img(hs, L::W_OFF)[at] = hi, half_img(hs, L::W_OFF)[32 * HROW + at] = lo;
            }
        }
        __syncthreads();
#pragma unroll
        for (int ct = 0; ct < 2; ct++) {
            if (G == 1 && ct != int(wave >> 1)) continue;
            const int ao = (16 * r + n) * HROW + 8 * j;
            half8 bh, bl;
            read_by_column(lds0 + hs * L::HEAD_BYTES + L::W_OFF + ((8 * j + le) * HROW + 16 * ct + 4 * la) * 2, 32 * HROW * 2, 4 * HROW * 2, bh, bl);
            const floatx4 tba = mma3(*reinterpret_cast<const half8 *>(half_img(hs, L::XBB_OFF) + ao),
                                     *reinterpret_cast<const half8 *>(half_img(hs, L::XBB_OFF) + 32 * HROW + ao), bh, bl, floatx4{0, 0, 0, 0});
            _Float16 *th = m_lds(hs), *tl = th + C * TROW;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                _Float16 hi, lo;
                split2(-tba[i], hi, lo);
                const int at = (32 + 16 * r + 4 * j + i) * TROW + 16 * ct + n;
                th[at] = hi, tl[at] = lo;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int hh = 0; hh < G; hh++) leave(hh, ws_v(hh));
}

// ---- the chain over the blocks --------------------------------------------------------------------
// Per block, with S0 [dv][128] the state's slice: P = K S0^T and Q S0^T (rows: tokens); R = V - e^c P;
// U = T R; O = (e^c (Q S0^T) + M U) / sqrt(128); S1 = e^{c_last} S0 + (e^{c_last - c} U)^T K.
// A wave takes 16 tokens' rows of K, Q, T and M, and nobody else reads those: they come from the workspace
// straight into its registers, a whole block ahead, as the MFMA operands they are.  LDS holds what the
// waves hand to each other: the state's image, R, U and the scaled U, the block's values and decay
// factors, and the block's keys, which the state's update contracts over the tokens: every wave puts
// its rows there, and ds_read_b64_tr_b16 hands them out by key dim.
struct ChainLds {
    static constexpr int GAM = 0;                          // e^{c_t}, e^{c_last - c_t}: 128 f32
    static constexpr int V = GAM + 2 * C * 4;              // [token][DV] f32
    static constexpr int SROW = K_DIM + 8;                 // f16 per row of the state's operand image [dv][128]
    static constexpr int SH = V + C * DV * 4, SL = SH + DV * SROW * 2;
    static constexpr int RH = SL + DV * SROW * 2;          // [dv][64 tokens] images, rows of TROW f16: R, U, U scaled
    static constexpr int RL = RH + DV * TROW * 2, UH = RL + DV * TROW * 2, UL = UH + DV * TROW * 2;
    static constexpr int WH = UL + DV * TROW * 2, WL = WH + DV * TROW * 2;
    // the block's keys [token][128] as hi and lo images, two sets for alternate blocks: every wave puts its 16
    // rows there, and the state's update reads them by key dim (transposing reads)
    static constexpr int KIMG = (WL + DV * TROW * 2 + 15) / 16 * 16;
    static constexpr int BYTES = KIMG + 4 * K_IMG;
};

// Eight waves in two teams.  Waves 0-3 carry the state: K S0^T, R, U and the state's update, each for 16 of
// the block's tokens (the update: for 32 key dims).  Waves 4-7 make the outputs, which nothing in the chain
// waits for: Q S0^T beside the first team's K S0^T, M U beside its update of the state, and the stores.
// What a wave reads of a block: its 16 rows of K (or Q) and of T (or M), 12 operands at most, and, in the
// first team, its share of the block's values and factors.
struct ChainBlock {
    u32x4 kq[2][4];  // [hi | lo][k-step]: rows 16 w + n of K | Q
    u32x4 tm[2][2];  // [hi | lo][k-step]: rows 16 w + n of T | M
    static constexpr int V_LOADS = C * DV * 4 / 16 / 256;  // 16-byte pieces per thread of the block's [token][DV] values
    u32x4 v[V_LOADS], gam;   // ...; 16 bytes of the 128 factors (threads 0-31)
};

__global__ __launch_bounds__(512) void deltanet_chunk_chain_kernel(ChunkArgs a) {
    using L = ChainLds;
    constexpr int NT = DV / 16;  // 16-wide tiles of value dims
    constexpr int V_LOADS = ChainBlock::V_LOADS;
    static_assert(V_LOADS >= 1 && V_LOADS * 256 * 16 == C * DV * 4, "whole 16-byte pieces of the block's values per thread");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    // Workgroups go to the 8 XCDs in turn, and each XCD has its own L2: workgroup w of the launch runs on
    // XCD w % 8.  The slices of a value head, and the value heads of a key head, read the same operands, so
    // they are given to one XCD (v_heads / 8 value heads each, where that divides).
    const uint32_t slices = a.v_dim / DV;
    uint32_t slice = blockIdx.x % slices, h = blockIdx.x / slices;
    if (a.v_heads % 8 == 0) {
        const uint32_t xcd = blockIdx.x % 8, at = blockIdx.x / 8;  // at: the XCD's workgroups in order
        h = xcd * (a.v_heads / 8) + at / slices, slice = at % slices;
    }
    const uint32_t group = a.v_heads / a.k_heads, khd = h / group;
    const uint32_t lane = threadIdx.x & 63, wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n = lane & 15, j = lane >> 4;
    const bool state_team = wave_all < 4;
    const uint32_t wave = wave_all & 3, tid = threadIdx.x & 255;  // the wave and the thread inside the team
    const uint32_t nblocks = (a.tokens + C - 1) / C;
    const size_t per_block = block_bytes(a.k_heads, a.v_heads);
    auto img = [&](int off) { return reinterpret_cast<const _Float16 *>(lds + off); };
    auto img_w = [&](int off) { return reinterpret_cast<_Float16 *>(lds + off); };
    const float *gam = reinterpret_cast<const float *>(lds + L::GAM);
    float *v_lds = reinterpret_cast<float *>(lds + L::V);

    // A block's operands are asked for in three lots, each as soon as the registers it goes to have been read
    // for the block two before: the rows of K | Q, the rows of T | M, the block's values and factors.
    auto clamp_block = [&](uint32_t blk) { return blk < nblocks ? blk : nblocks - 1; };  // (past the last block: its operands again, unused)
    auto request_kq = [&](uint32_t at, ChainBlock &b) {
        const uint32_t blk = clamp_block(at);
        // (the second team's operands lie two parts on: Q behind K, M behind T)
        const u32x4 *wk = reinterpret_cast<const u32x4 *>(a.ws + size_t(blk) * per_block + khd * KHEAD_BYTES + (state_team ? 0 : 2 * K_GL));
#pragma unroll
        for (int part = 0; part < 2; part++) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++) b.kq[part][ks] = wk[(part * K_GL) / 16 + (wave * 4 + ks) * 64 + lane];
        }
    };
    auto request_tm = [&](uint32_t at, ChainBlock &b) {
        const uint32_t blk = clamp_block(at);
        const u32x4 *wv = reinterpret_cast<const u32x4 *>(a.ws + size_t(blk) * per_block + a.k_heads * KHEAD_BYTES + h * VHEAD_BYTES);
        const u32x4 *wt = wv + (state_team ? 0 : 2 * T_GL) / 16;
#pragma unroll
        for (int part = 0; part < 2; part++) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                // (T and M are lower triangular: rows 16 wave .. have nothing in columns 32 ks .. beyond their own)
                if (ks <= int(wave) / 2) b.tm[part][ks] = wt[(part * T_GL) / 16 + (wave * 2 + ks) * 64 + lane];
            }
        }
    };
    auto request_values = [&](uint32_t at, ChainBlock &b) {  // (the first team)
        const uint32_t blk = clamp_block(at);
        const u32x4 *wv = reinterpret_cast<const u32x4 *>(a.ws + size_t(blk) * per_block + a.k_heads * KHEAD_BYTES + h * VHEAD_BYTES);
#pragma unroll
        for (int i = 0; i < V_LOADS; i++) {
            // piece p of the block's [token][DV] values: token p / (DV / 4), four dims (a token past the end: unused, see `place`)
            const uint32_t p = tid + 256 * i, tok = min(blk * C + p / (DV / 4), a.tokens - 1);
            b.v[i] = *reinterpret_cast<const u32x4 *>(a.mixed + size_t(tok) * a.channels + 2 * a.k_heads * K_DIM + h * a.v_dim + DV * slice + 4 * (p % (DV / 4)));
        }
        b.gam = wv[(4 * T_GL) / 16 + (tid & 31)];
    };
    // the block's values (tokens past the end: zeros) and factors to LDS (the first team)
    auto place = [&](uint32_t blk, const ChainBlock &b) {
#pragma unroll
        for (int i = 0; i < V_LOADS; i++) {
            const uint32_t p = tid + 256 * i;
            const bool real = blk * C + p / (DV / 4) < a.tokens;
            reinterpret_cast<u32x4 *>(v_lds)[p] = real ? b.v[i] : u32x4{0, 0, 0, 0};
        }
        if (tid < 32) reinterpret_cast<u32x4 *>(lds + L::GAM)[tid] = b.gam;
    };

    // ---- the state's slice: S [dv][128]; wave w of the first team keeps columns 32 w .. + 31: lane (n, j) the four
    // rows dv = 16 mt + 4j + i of columns 32 w + 16 nt + n.  Its image for the products lies in LDS as hi and lo parts. ----
    float *state = a.state + (size_t(h) * a.v_dim + DV * slice) * K_DIM;
    floatx4 s_reg[NT][2];
    auto publish_state = [&]() {
#pragma unroll
        for (int mt = 0; mt < NT; mt++) {
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    _Float16 hi, lo;
                    split2(s_reg[mt][nt][i], hi, lo);
                    const int at = (16 * mt + 4 * j + i) * L::SROW + 32 * wave + 16 * nt + n;
                    img_w(L::SH)[at] = hi, img_w(L::SL)[at] = lo;
                }
            }
        }
    };
#pragma unroll
    for (int mt = 0; mt < NT; mt++) {
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
#pragma unroll
            for (int i = 0; i < 4; i++) s_reg[mt][nt][i] = state_team ? state[(16 * mt + 4 * j + i) * K_DIM + 32 * wave + 16 * nt + n] : 0.0f;
        }
    }

    // One block: `cur` holds its operands, `next` those of the block after it (asked for during the block before
    // this one).  Each lot of `cur`, once read, is asked for again for the block after next: a load has two
    // blocks' time to come back (one block's time is less than the 2.9 us a wave's batch takes under this load).
    // (the team is a type, so that a team's blocks are one piece of code: what one team asks for is not taken to be
    // in flight where the other team waits)
    auto step = [&](auto team, uint32_t blk, ChainBlock &cur, const ChainBlock &next) {
        constexpr bool STATE = decltype(team)::value;
        const uint32_t nxt = blk + 1 < nblocks ? blk + 1 : blk;
        if constexpr (STATE) {
            request_values(blk + 2, cur);  // (this block's values went to LDS during the block before)
            __builtin_amdgcn_sched_barrier(0);
            // this wave's rows of the block's keys, for the state's update (the set of two blocks ago is read no more:
            // every wave has been through the three barriers of the block between)
            _Float16 *kimg = img_w(L::KIMG + int(blk & 1) * 2 * K_IMG);
#pragma unroll
            for (int part = 0; part < 2; part++) {
#pragma unroll
                for (int ks = 0; ks < 4; ks++) {
                    *reinterpret_cast<u32x4 *>(kimg + part * C * KROW + (16 * wave + n) * KROW + 32 * ks + 8 * j) = cur.kq[part][ks];
                }
            }
        }
        __syncthreads();  // the block's values and factors, the state's image and the keys are in LDS

        // ---- K S0^T (first team) | Q S0^T (second team): rows t = 16 wave + n, columns dv = 16 vt + n' ----
        floatx4 pkq[NT];
#pragma unroll
        for (int vt = 0; vt < NT; vt++) pkq[vt] = floatx4{0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int vt = 0; vt < NT; vt++) {
                const int bo = (16 * vt + n) * L::SROW + 32 * ks + 8 * j;
                const half8 bh = *reinterpret_cast<const half8 *>(img(L::SH) + bo), bl = *reinterpret_cast<const half8 *>(img(L::SL) + bo);
                pkq[vt] = mma3(__builtin_bit_cast(half8, cur.kq[0][ks]), __builtin_bit_cast(half8, cur.kq[1][ks]), bh, bl, pkq[vt]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        request_kq(blk + 2, cur);
        __builtin_amdgcn_sched_barrier(0);
        // C layout: lane (n, j) holds dv = 16 vt + n of tokens t = 16 wave + 4j + i
        const floatx4 gam4 = *reinterpret_cast<const floatx4 *>(gam + 16 * wave + 4 * j);
        const floatx4 gk4 = *reinterpret_cast<const floatx4 *>(gam + C + 16 * wave + 4 * j);
        const float glast = gam[C - 1];
        if constexpr (STATE) {
#pragma unroll
            for (int vt = 0; vt < NT; vt++) {
                // R = V - e^c (K S0^T), as the [dv][token] image
                half4 rh, rl;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    _Float16 hi, lo;
                    split2(v_lds[(16 * wave + 4 * j + i) * DV + 16 * vt + n] - gam4[i] * pkq[vt][i], hi, lo);
                    rh[i] = hi, rl[i] = lo;
                }
                const int at = (16 * vt + n) * TROW + 16 * wave + 4 * j;
                *reinterpret_cast<half4 *>(img_w(L::RH) + at) = rh, *reinterpret_cast<half4 *>(img_w(L::RL) + at) = rl;
            }
        }
        __syncthreads();  // R is whole

        if constexpr (STATE) {
            // ---- U = T R (T is lower triangular: k-steps up to the row tile's own) ----
#pragma unroll
            for (int vt = 0; vt < NT; vt++) {
                floatx4 u = {0, 0, 0, 0};
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    if (ks > int(wave) / 2) continue;
                    const int bo = (16 * vt + n) * TROW + 32 * ks + 8 * j;
                    u = mma3(__builtin_bit_cast(half8, cur.tm[0][ks]), __builtin_bit_cast(half8, cur.tm[1][ks]),
                             *reinterpret_cast<const half8 *>(img(L::RH) + bo), *reinterpret_cast<const half8 *>(img(L::RL) + bo), u);
                }
                half4 uh, ul, wh, wl;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    _Float16 hi, lo;
                    split2(u[i], hi, lo);
                    uh[i] = hi, ul[i] = lo;
                    split2(u[i] * gk4[i], hi, lo);  // scaled by e^{c_last - c_t} for the state
                    wh[i] = hi, wl[i] = lo;
                }
                const int at = (16 * vt + n) * TROW + 16 * wave + 4 * j;
                *reinterpret_cast<half4 *>(img_w(L::UH) + at) = uh, *reinterpret_cast<half4 *>(img_w(L::UL) + at) = ul;
                *reinterpret_cast<half4 *>(img_w(L::WH) + at) = wh, *reinterpret_cast<half4 *>(img_w(L::WL) + at) = wl;
            }
            __builtin_amdgcn_sched_barrier(0);
            request_tm(blk + 2, cur);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();  // U is whole; every wave is through with the state's image, the values and the factors

        if constexpr (STATE) {
            // ---- S1 = e^{c_last} S0 + (U scaled)^T K: rows dv, columns 32 wave + 16 nt + n, over the 64 tokens ----
            // The B operands, K by key dim: lane (n, j) wants column 32 wave + 16 nt + n, tokens 32 ks + 8j .. + 7.
            // ds_read_b64_tr_b16 works on 16 lanes: lane a + 4e of them names 8 bytes (4 values of a row), and lane
            // 4a + c receives value c of the lanes a, a + 4, a + 8, a + 12.  So lane a + 4e names token .. + e, key
            // dims .. + 4a .. + 3, and lane n = 4a + c receives key dim .. + n of four tokens in a row; two reads an operand.
            u32x2 xr[2][2][2][2];  // [hi | lo][nt][k-step][tokens + 0 | + 4]
            {
                const uint32_t kbase = uint32_t(reinterpret_cast<uintptr_t>(lds)) + L::KIMG + (blk & 1) * 2 * K_IMG;
                const uint32_t la = lane & 3, le = (lane >> 2) & 3;
#pragma unroll
                for (int part = 0; part < 2; part++) {
#pragma unroll
                    for (int nt = 0; nt < 2; nt++) {
#pragma unroll
                        for (int ks = 0; ks < 2; ks++) {
#pragma unroll
                            for (int hf = 0; hf < 2; hf++) {
                                const uint32_t at = kbase + part * K_IMG + ((32 * ks + 8 * j + 4 * hf + le) * KROW + 32 * wave + 16 * nt + 4 * la) * 2;
                                asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(xr[part][nt][ks][hf]) : "v"(at) : "memory");
                            }
                        }
                    }
                }
                // (the registers are handed on only behind the wait, in the same straight piece of code)
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(xr[0][0][0][0]), "+v"(xr[0][0][0][1]), "+v"(xr[0][0][1][0]), "+v"(xr[0][0][1][1]), "+v"(xr[0][1][0][0]),
                               "+v"(xr[0][1][0][1]), "+v"(xr[0][1][1][0]), "+v"(xr[0][1][1][1]), "+v"(xr[1][0][0][0]), "+v"(xr[1][0][0][1]),
                               "+v"(xr[1][0][1][0]), "+v"(xr[1][0][1][1]), "+v"(xr[1][1][0][0]), "+v"(xr[1][1][0][1]), "+v"(xr[1][1][1][0]),
                               "+v"(xr[1][1][1][1])::"memory");
            }
            auto x_operand = [&](int part, int nt, int ks) {
                const u32x4 v = {xr[part][nt][ks][0].x, xr[part][nt][ks][0].y, xr[part][nt][ks][1].x, xr[part][nt][ks][1].y};
                return __builtin_bit_cast(half8, v);
            };
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                floatx4 acc[NT];
#pragma unroll
                for (int mt = 0; mt < NT; mt++) acc[mt] = floatx4{0, 0, 0, 0};
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
#pragma unroll
                    for (int mt = 0; mt < NT; mt++) {
                        const int ao = (16 * mt + n) * TROW + 32 * ks + 8 * j;
                        acc[mt] = mma3(*reinterpret_cast<const half8 *>(img(L::WH) + ao), *reinterpret_cast<const half8 *>(img(L::WL) + ao),
                                       x_operand(0, nt, ks), x_operand(1, nt, ks), acc[mt]);
                    }
                }
#pragma unroll
                for (int mt = 0; mt < NT; mt++) s_reg[mt][nt] = s_reg[mt][nt] * glast + acc[mt];
            }
            // the next block's state image, values and factors: their places were last read before the barrier above
            publish_state();
            place(nxt, next);
        } else {
            // ---- O = (e^c (Q S0^T) + M U) / sqrt(128) ----
            floatx4 mu[NT];
#pragma unroll
            for (int vt = 0; vt < NT; vt++) {
                mu[vt] = floatx4{0, 0, 0, 0};
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    if (ks > int(wave) / 2) continue;
                    const int bo = (16 * vt + n) * TROW + 32 * ks + 8 * j;
                    mu[vt] = mma3(__builtin_bit_cast(half8, cur.tm[0][ks]), __builtin_bit_cast(half8, cur.tm[1][ks]),
                                  *reinterpret_cast<const half8 *>(img(L::UH) + bo), *reinterpret_cast<const half8 *>(img(L::UL) + bo), mu[vt]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            request_tm(blk + 2, cur);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int vt = 0; vt < NT; vt++) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t tok = blk * C + 16 * wave + 4 * j + i;
                    if (tok < a.tokens) a.o[(size_t(tok) * a.v_heads + h) * a.v_dim + DV * slice + 16 * vt + n] = Q_SCALE * (gam4[i] * pkq[vt][i] + mu[vt][i]);
                }
            }
        }
    };
    // (two sets of operand registers that change roles, so that nothing is copied from one to the other)
    auto walk = [&](auto team) {
        constexpr bool STATE = decltype(team)::value;
        ChainBlock even, odd;
        // (in the order the blocks ask in, so that the first blocks' waits are those of every block)
        if constexpr (STATE) request_values(0, even);
        request_kq(0, even), request_tm(0, even);
        if constexpr (STATE) request_values(1, odd);
        request_kq(1, odd), request_tm(1, odd);
        if constexpr (STATE) {
            publish_state();
            place(0, even);
        }
        // (pairs of blocks without a branch between them, so that the loads asked for in one block are known to be
        // behind those of the block before wherever a wait is placed)
        uint32_t blk = 0;
        for (; blk + 1 < nblocks; blk += 2) {
            step(team, blk, even, odd);
            step(team, blk + 1, odd, even);
        }
        if (blk < nblocks) step(team, blk, even, odd);
    };
    if (state_team) {
        walk(std::true_type{});
    } else {
        walk(std::false_type{});
    }
    if (state_team) {
#pragma unroll
        for (int mt = 0; mt < NT; mt++) {
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
#pragma unroll
                for (int i = 0; i < 4; i++) state[(16 * mt + 4 * j + i) * K_DIM + 32 * wave + 16 * nt + n] = s_reg[mt][nt][i];
            }
        }
    }
}

}  // namespace

int setup_deltanet_chunk() {
    if (int rc = int(hipFuncSetAttribute(reinterpret_cast<const void *>(deltanet_chunk_prepare_kernel<1>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, PrepLds<1>::BYTES))) {
        return rc;
    }
    if (int rc = int(hipFuncSetAttribute(reinterpret_cast<const void *>(deltanet_chunk_prepare_kernel<2>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, PrepLds<2>::BYTES))) {
        return rc;
    }
    return int(hipFuncSetAttribute(reinterpret_cast<const void *>(deltanet_chunk_chain_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, ChainLds::BYTES));
}

size_t deltanet_chunk_workspace_bytes(const saetta_rows_step_params &p) {
    if (p.snapshots || p.tokens < DELTANET_CHUNK_FROM || p.v_dim % DV != 0 || p.k_heads == 0 || p.v_heads % p.k_heads != 0) return 0;
    return size_t((p.tokens + C - 1) / C) * block_bytes(p.k_heads, p.v_heads);
}

int run_deltanet_chunk(hipStream_t stream, const float *mixed, const float *a, const float *b, const float *a_log,
                       const float *dt_bias, float *state, float *o, const saetta_rows_step_params &p, uint32_t channels,
                       void *workspace) {
    const uint32_t nblocks = (p.tokens + C - 1) / C;
    ChunkArgs args{mixed, a, b, a_log, dt_bias, state, o, static_cast<unsigned char *>(workspace), p.k_heads, p.v_heads, p.v_dim, p.tokens, channels, p.eps};
    if (p.v_heads == 2 * p.k_heads) {
        deltanet_chunk_prepare_kernel<2><<<dim3(nblocks, p.k_heads), 256, PrepLds<2>::BYTES, stream>>>(args);
    } else {
        deltanet_chunk_prepare_kernel<1><<<dim3(nblocks, p.v_heads), 256, PrepLds<1>::BYTES, stream>>>(args);
    }
    deltanet_chunk_chain_kernel<<<dim3(p.v_dim / DV * p.v_heads), 512, ChainLds::BYTES, stream>>>(args);
    return SAETTA_OK;
}

}  // namespace saetta
