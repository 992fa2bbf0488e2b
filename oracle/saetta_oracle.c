/*
 * CPU oracle for the full-attention hot path and its next rows: TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the reference's CPU algorithms so that the
 * HIP kernels can be checked against them.  It is never linked into or called
 * from the product library; only tests, the smoke check and the CPU-baseline
 * leg of the benchmark load it.
 *
 * Every function names the reference lines it follows.  Build with
 * `-O2 -ffp-contract=off` (see the Makefile beside this file): the reference is
 * Rust, which never contracts a*b+c into an FMA and never reassociates float
 * sums, and the loops below rely on the compiler keeping both properties.
 *
 * Pinning status (what independent evidence each function is checked
 * against, in tests/test_oracle_*.py):
 *   orc_f32_to_f16 / orc_f16_to_f32     numpy.float16 (IEEE RNE), exhaustive over
 *                                       all 65536 halves and 2^20 sampled floats
 *   orc_quantize                        reference known answers
 *                                       (src/kv_quant.rs:319-332), half-a-step
 *                                       bound and exact constant group
 *                                       (src/kv_quant.rs:302-317), exact-rational
 *                                       re-derivation with Python fractions
 *   orc_dequantize                      definition + inverse on grid points
 *   orc_attend / orc_attention_layer    MLX golden vectors attention.json and
 *                                       ops.json (src/cpu/attention.rs:188-221,
 *                                       src/cpu/ops.rs:81-110), torch float64
 *                                       scaled_dot_product_attention, closed
 *                                       forms (len 1, equal keys, one huge key)
 *   orc_attention_f64                   same closed forms + torch float64 SDPA
 *   orc_rows / orc_prefill              definition as single-row calls, checked
 *                                       against torch float64 SDPA with a causal
 *                                       mask
 *   orc_rms_norm / orc_rope             MLX golden vectors ops.json
 *   orc_deltanet_conv / _step / _layer  MLX golden vectors deltanet.json (six
 *                                       tokens: outputs, conv state, recurrent
 *                                       state; src/cpu/deltanet.rs:162-204), an
 *                                       f64 restatement of the recurrence, its
 *                                       limits (beta -> 1: S k = v; g -> 0:
 *                                       S = beta v k^T), the conv as a causal
 *                                       filter over the input history
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_GROUP 64 /* src/kv_quant.rs:9 */

/* ---------------------------------------------------------------- f16 ---- */

/* IEEE binary16 <- binary32, round to nearest even, subnormals kept,
 * overflow to infinity, NaN kept quiet with its top payload bits.  This is
 * what `half::f16::from_f32` (crate half 2.7.1, Cargo.lock:131-134; call
 * sites src/kv_quant.rs:64-65) computes. */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) {
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x0200u | (man >> 13));
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        /* subnormal half or zero */
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t out = sign | ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (out & 1))) out++; /* may carry into exp: correct */
    return (uint16_t)out;
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3ffu;
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        x = sign | 0x7f800000u | (man << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void orc_f32_to_f16_array(const float *x, size_t n, uint16_t *out) {
    for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(x[i]);
}

void orc_f16_to_f32_array(const uint16_t *x, size_t n, float *out) {
    for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(x[i]);
}

/* -------------------------------------------------------- kv quantizer ---- */

/* f32::min / f32::max of Rust: a NaN operand is ignored. */
static float min_ignoring_nan(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    return a < b ? a : b;
}
static float max_ignoring_nan(float a, float b) {
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}

/* `f32::round_ties_even().clamp(0, levels) as u32` (src/kv_quant.rs:72-76):
 * clamp passes a NaN through and `as u32` turns it into 0. */
static uint32_t code_of(float scaled, float levels) {
    float r = nearbyintf(scaled); /* default rounding mode: ties to even */
    if (r != r) return 0;
    if (r < 0.0f) r = 0.0f;
    if (r > levels) r = levels;
    return (uint32_t)r;
}

/* quantize (src/kv_quant.rs:54-87).  x holds n values, n a multiple of 64;
 * data gets n/64 * 2*bits words, scales and biases n/64 halves (as bits).
 * Returns 0, or -1 on a bad argument (the reference asserts). */
int orc_quantize(const float *x, size_t n, int bits, uint32_t *data, uint16_t *scales,
                 uint16_t *biases) {
    if ((bits != 8 && bits != 4) || n % ORC_GROUP != 0) return -1;
    const float levels = (float)((1u << bits) - 1);
    const size_t per_word = 32 / (size_t)bits;
    size_t w = 0;
    for (size_t g = 0; g < n / ORC_GROUP; g++) {
        const float *group = x + g * ORC_GROUP;
        float lo = INFINITY, hi = -INFINITY;
        for (int i = 0; i < ORC_GROUP; i++) lo = min_ignoring_nan(lo, group[i]);
        for (int i = 0; i < ORC_GROUP; i++) hi = max_ignoring_nan(hi, group[i]);
        uint16_t s = orc_f32_to_f16((hi - lo) / levels);
        uint16_t z = orc_f32_to_f16(lo);
        float sf = orc_f16_to_f32(s), zf = orc_f16_to_f32(z);
        float inv = sf > 0.0f ? 1.0f / sf : 0.0f;
        for (size_t i = 0; i < ORC_GROUP; i += per_word) {
            uint32_t word = 0;
            for (size_t j = 0; j < per_word; j++) {
                float d = group[i + j] - zf;
                word |= code_of(d * inv, levels) << (j * (size_t)bits);
            }
            data[w++] = word;
        }
        scales[g] = s;
        biases[g] = z;
    }
    return 0;
}

/* dequantize (src/kv_quant.rs:90-105): f32(s) * q + f32(z), in that order. */
int orc_dequantize(const uint32_t *data, const uint16_t *scales, const uint16_t *biases,
                   size_t groups, int bits, float *out) {
    if (bits != 8 && bits != 4) return -1;
    const uint32_t mask = (1u << bits) - 1;
    const size_t per_word = 32 / (size_t)bits;
    const size_t words = 2 * (size_t)bits;
    size_t o = 0;
    for (size_t g = 0; g < groups; g++) {
        float s = orc_f16_to_f32(scales[g]), z = orc_f16_to_f32(biases[g]);
        for (size_t wi = 0; wi < words; wi++) {
            uint32_t w = data[g * words + wi];
            for (size_t i = 0; i < per_word; i++) {
                uint32_t q = (w >> (i * (size_t)bits)) & mask;
                float prod = s * (float)q;
                out[o++] = prod + z;
            }
        }
    }
    return 0;
}

/* round_trip (src/kv_quant.rs:127-135): bits 16 rounds through half, 8 and 4
 * through the codes. */
int orc_round_trip(const float *x, size_t n, int bits, float *out) {
    if (bits == 16) {
        for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(orc_f32_to_f16(x[i]));
        return 0;
    }
    if ((bits != 8 && bits != 4) || n % ORC_GROUP != 0) return -1;
    size_t groups = n / ORC_GROUP;
    uint32_t *data = malloc(groups * 2 * (size_t)bits * 4);
    uint16_t *s = malloc(groups * 2), *z = malloc(groups * 2);
    int rc = orc_quantize(x, n, bits, data, s, z);
    if (rc == 0) rc = orc_dequantize(data, s, z, groups, bits, out);
    free(data);
    free(s);
    free(z);
    return rc;
}

/* round_trip_as_half (src/kv_quant.rs:119-125). */
int orc_round_trip_as_half(const float *x, size_t n, int bits, float *out) {
    int rc = orc_round_trip(x, n, bits, out);
    if (rc) return rc;
    for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(orc_f32_to_f16(out[i]));
    return 0;
}

/* ------------------------------------------------------------ small ops ---- */

/* dot (src/cpu/ops.rs:13-15): products summed left to right in f32. */
static float dot_f32(const float *a, const float *b, size_t n) {
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float p = a[i] * b[i];
        sum += p;
    }
    return sum;
}

/* sigmoid (src/cpu/ops.rs:38-40). */
static float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

/* softmax (src/cpu/ops.rs:51-59): subtract the max, exp, divide by the sum. */
void orc_softmax(float *x, size_t n) {
    float max = -INFINITY;
    for (size_t i = 0; i < n; i++) max = max_ignoring_nan(max, x[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        x[i] = expf(x[i] - max);
        sum += x[i];
    }
    for (size_t i = 0; i < n; i++) x[i] /= sum;
}

/* rms_norm (src/cpu/ops.rs:19-36). */
void orc_rms_norm(float *x, const float *w, size_t n, float eps) {
    float ss = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float p = x[i] * x[i];
        ss += p;
    }
    float mean = ss / (float)n;
    float scale = 1.0f / sqrtf(mean + eps);
    for (size_t i = 0; i < n; i++) {
        float sg = scale * w[i];
        x[i] *= sg;
    }
}

/* rope (src/cpu/ops.rs:61-74): non-interleaved, first `dims` values. */
void orc_rope(float *head, size_t dims, size_t pos, float theta) {
    size_t half = dims / 2;
    for (size_t i = 0; i < half; i++) {
        double freq = pow((double)theta, -((double)i) / (double)half);
        double angle = (double)pos * freq;
        float s = (float)sin(angle), c = (float)cos(angle);
        float a = head[i], b = head[i + half];
        float ac = a * c, bs = b * s, as = a * s, bc = b * c;
        head[i] = ac - bs;
        head[i + half] = as + bc;
    }
}

/* ------------------------------------------------------------ attention ---- */

/* attend (src/cpu/attention.rs:158-181) for one query head over the first
 * `len` tokens of an f32 cache [len][kv_heads][dim]; writes out[dim].
 * scratch holds len floats. */
static void attend_head(const float *q, const float *keys, const float *values, size_t len,
                        size_t kv_heads, size_t dim, size_t kv, float *scratch, float *out) {
    size_t stride = kv_heads * dim, offset = kv * dim;
    float scale = 1.0f / sqrtf((float)dim);
    for (size_t t = 0; t < len; t++) {
        scratch[t] = dot_f32(q, keys + t * stride + offset, dim) * scale;
    }
    orc_softmax(scratch, len);
    for (size_t i = 0; i < dim; i++) out[i] = 0.0f;
    for (size_t t = 0; t < len; t++) {
        const float *v = values + t * stride + offset;
        float p = scratch[t];
        for (size_t i = 0; i < dim; i++) {
            float pv = p * v[i];
            out[i] += pv;
        }
    }
}

/* The attention of one token as attention_at runs it after the projections
 * (src/cpu/attention.rs:141-154): every q head attends over its kv head
 * (h / (heads / kv_heads)), then the output is multiplied by sigmoid(gate).
 * q is [heads][dim]; gate points at the gate of head 0 and the gate of head h
 * starts at gate + h * gate_stride (the GPU path's q_and_gate buffer has
 * gate = q_and_gate + dim, gate_stride = 2 * dim); gate may be NULL.
 * threads > 1 spreads the heads over OpenMP threads (the reference is
 * single-threaded; the results are the same bits either way). */
int orc_attend(const float *q, const float *keys, const float *values, size_t len,
               size_t heads, size_t kv_heads, size_t dim, const float *gate, size_t gate_stride,
               float *out, int threads) {
    if (len == 0 || kv_heads == 0 || heads % kv_heads != 0) return -1;
    size_t group = heads / kv_heads;
    int failed = 0;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (long h = 0; h < (long)heads; h++) {
        float *scratch = malloc(len * sizeof(float));
        if (!scratch) {
            failed = 1;
            continue;
        }
        attend_head(q + (size_t)h * dim, keys, values, len, kv_heads, dim, (size_t)h / group,
                    scratch, out + (size_t)h * dim);
        if (gate) {
            const float *g = gate + (size_t)h * gate_stride;
            float *o = out + (size_t)h * dim;
            for (size_t i = 0; i < dim; i++) o[i] *= sigmoid_f32(g[i]);
        }
        free(scratch);
    }
    return failed ? -2 : 0;
}

/* The f64 reference the decode kernels are held against
 * (tests/attention.rs:28-52): q [heads][dim], k and v [len][kv_heads][dim] in
 * f32, q_and_gate [heads][2*dim] with the gate in the second half; out is
 * f64 [heads][dim]. */
int orc_attention_f64(const float *q, const float *k, const float *v, const float *q_and_gate,
                      size_t len, size_t heads, size_t kv_heads, size_t dim, double *out,
                      int threads) {
    if (len == 0 || kv_heads == 0 || heads % kv_heads != 0) return -1;
    size_t per = heads / kv_heads;
    int failed = 0;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (long hh = 0; hh < (long)heads; hh++) {
        size_t h = (size_t)hh, kv = h / per;
        double *scores = malloc(len * sizeof(double));
        if (!scores) {
            failed = 1;
            continue;
        }
        double m = -1.7976931348623157e308; /* f64::MIN */
        for (size_t t = 0; t < len; t++) {
            double s = 0.0;
            for (size_t i = 0; i < dim; i++) {
                s += (double)q[h * dim + i] * (double)k[(t * kv_heads + kv) * dim + i];
            }
            scores[t] = s / sqrt((double)dim);
            if (scores[t] > m) m = scores[t];
        }
        double sum = 0.0;
        for (size_t t = 0; t < len; t++) {
            scores[t] = exp(scores[t] - m);
            sum += scores[t];
        }
        for (size_t i = 0; i < dim; i++) {
            double a = 0.0;
            for (size_t t = 0; t < len; t++) {
                a += scores[t] * (double)v[(t * kv_heads + kv) * dim + i];
            }
            double g = q_and_gate ? (double)q_and_gate[h * 2 * dim + dim + i] : INFINITY;
            out[h * dim + i] = a / sum / (1.0 + exp(-g));
        }
        free(scores);
    }
    return failed ? -2 : 0;
}

/* Verify rows: row r is one decode token at position pos + r, which sees
 * pos + r + 1 keys (kernels/attention_rows.metal:1-8; the reference tests it
 * as m single-row decodes, src/rows.rs:702-737).  q [m][heads][dim],
 * q_and_gate [m][heads][2*dim], out [m][heads][dim]. */
int orc_rows(const float *q, const float *keys, const float *values, size_t pos, size_t m,
             size_t heads, size_t kv_heads, size_t dim, const float *q_and_gate, float *out,
             int threads) {
    for (size_t r = 0; r < m; r++) {
        const float *gate = q_and_gate ? q_and_gate + r * heads * 2 * dim + dim : NULL;
        int rc = orc_attend(q + r * heads * dim, keys, values, pos + r + 1, heads, kv_heads, dim,
                            gate, 2 * dim, out + r * heads * dim, threads);
        if (rc) return rc;
    }
    return 0;
}

/* As orc_rows against the f64 formula. */
int orc_rows_f64(const float *q, const float *keys, const float *values, size_t pos, size_t m,
                 size_t heads, size_t kv_heads, size_t dim, const float *q_and_gate, double *out,
                 int threads) {
    for (size_t r = 0; r < m; r++) {
        int rc = orc_attention_f64(q + r * heads * dim, keys, values,
                                   q_and_gate ? q_and_gate + r * heads * 2 * dim : NULL,
                                   pos + r + 1, heads, kv_heads, dim, out + r * heads * dim,
                                   threads);
        if (rc) return rc;
    }
    return 0;
}

/* Prefill chunk: token i of the chunk is one decode token that sees keys
 * 0 ..= pos + i (src/attention_prefill.rs:9-12; src/prefill.rs:2489-2495 checks
 * the GPU chunk against the CPU run token by token).  The caller passes the
 * cache as the CPU reference would hold it (round_trip_as_half for a
 * quantized cache, src/cpu/attention.rs:131-139).  Tokens are spread over
 * OpenMP threads when threads > 1. */
int orc_prefill(const float *q, const float *keys, const float *values, size_t pos, size_t tokens,
                size_t heads, size_t kv_heads, size_t dim, const float *q_and_gate, float *out,
                int threads) {
    int failed = 0;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 4)
    for (long i = 0; i < (long)tokens; i++) {
        size_t r = (size_t)i;
        const float *gate = q_and_gate ? q_and_gate + r * heads * 2 * dim + dim : NULL;
        int rc = orc_attend(q + r * heads * dim, keys, values, pos + r + 1, heads, kv_heads, dim,
                            gate, 2 * dim, out + r * heads * dim, 1);
        if (rc) failed = rc;
    }
    return failed;
}

/* One token through the whole attention layer as attention_at does it
 * (src/cpu/attention.rs:103-156), with dense f32 projections: used only to
 * hold orc_attend, the head -> kv head map, the gate split and the cache
 * rounding against the MLX golden vectors of attention.json.
 * keys/values: caller-owned f32 cache [capacity][kv_heads*dim] holding `len`
 * tokens; the new token is appended at row len.  rounding: 0 none, 16/8/4 as
 * KvCache::round_to, negative (-8/-4) as round_to_as_half. */
static void matvec_f32(const float *w, const float *x, size_t rows, size_t cols, float *y) {
    for (size_t r = 0; r < rows; r++) y[r] = dot_f32(w + r * cols, x, cols);
}

int orc_attention_layer(const float *x, size_t hidden, size_t heads, size_t kv_heads, size_t dim,
                        size_t rope_dims, float rope_theta, float eps, const float *q_proj,
                        const float *k_proj, const float *v_proj, const float *o_proj,
                        const float *q_norm, const float *k_norm, float *keys, float *values,
                        size_t len, size_t pos, int rounding, float *out) {
    size_t kvw = kv_heads * dim;
    float *qg = malloc(heads * 2 * dim * sizeof(float));
    float *q = malloc(heads * dim * sizeof(float));
    float *k = malloc(kvw * sizeof(float)), *v = malloc(kvw * sizeof(float));
    float *att = malloc(heads * dim * sizeof(float));
    matvec_f32(q_proj, x, heads * 2 * dim, hidden, qg);
    for (size_t h = 0; h < heads; h++) memcpy(q + h * dim, qg + h * 2 * dim, dim * sizeof(float));
    matvec_f32(k_proj, x, kvw, hidden, k);
    matvec_f32(v_proj, x, kvw, hidden, v);
    for (size_t h = 0; h < heads; h++) {
        orc_rms_norm(q + h * dim, q_norm, dim, eps);
        orc_rope(q + h * dim, rope_dims, pos, rope_theta);
    }
    for (size_t h = 0; h < kv_heads; h++) {
        orc_rms_norm(k + h * dim, k_norm, dim, eps);
        orc_rope(k + h * dim, rope_dims, pos, rope_theta);
    }
    int rc = 0;
    if (rounding > 0) {
        rc |= orc_round_trip(k, kvw, rounding, keys + len * kvw);
        rc |= orc_round_trip(v, kvw, rounding, values + len * kvw);
    } else if (rounding < 0) {
        rc |= orc_round_trip_as_half(k, kvw, -rounding, keys + len * kvw);
        rc |= orc_round_trip_as_half(v, kvw, -rounding, values + len * kvw);
    } else {
        memcpy(keys + len * kvw, k, kvw * sizeof(float));
        memcpy(values + len * kvw, v, kvw * sizeof(float));
    }
    if (!rc) {
        rc = orc_attend(q, keys, values, len + 1, heads, kv_heads, dim, qg + dim, 2 * dim, att, 1);
    }
    if (!rc) matvec_f32(o_proj, att, hidden, heads * dim, out);
    free(qg);
    free(q);
    free(k);
    free(v);
    free(att);
    return rc;
}

/* ------------------------------------------------------ Gated DeltaNet ---- */
/* One token of the linear-attention layer, src/cpu/deltanet.rs:69-155.
 * Pinned by the MLX golden vectors of deltanet.json (six tokens: outputs, conv
 * state, recurrent state; src/cpu/deltanet.rs:162-204). */

static float silu_f32(float x) { return x * sigmoid_f32(x); }

/* log(1 + e^x) without overflow (src/cpu/ops.rs:46-49). */
static float softplus_f32(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }

/* conv_step (src/cpu/deltanet.rs:117-131): depthwise causal conv1d over the stored
 * inputs and `input`, then SiLU; `input` is shifted into the state.
 * weight [channels][kernel] (last column = newest token), state [kernel-1][channels]
 * oldest first. */
void orc_deltanet_conv(const float *weight, const float *input, float *state, size_t channels,
                       size_t kernel, float *out) {
    size_t past = kernel - 1; /* >= 1: the reference drains one input from a non-empty state */
    for (size_t c = 0; c < channels; c++) {
        const float *w = weight + c * kernel;
        float old = 0.0f;
        for (size_t t = 0; t < past; t++) old += w[t] * state[t * channels + c];
        out[c] = silu_f32(old + w[past] * input[c]);
    }
    memmove(state, state + channels, (past - 1) * channels * sizeof(float));
    memcpy(state + (past - 1) * channels, input, channels * sizeof(float));
}

/* normalize_qk + the per-head gates + delta_rule + the gated RMSNorm
 * (src/cpu/deltanet.rs:86-112,133-155): everything between the conv and out_proj.
 * q, k [k_heads][k_dim] (after the conv), v [v_heads][v_dim], a, b [v_heads],
 * state [v_heads][v_dim][k_dim] (updated), z [v_heads][v_dim], norm [v_dim],
 * y [v_heads][v_dim]. */
void orc_deltanet_step(const float *q_in, const float *k_in, const float *v, const float *a,
                       const float *b, const float *a_log, const float *dt_bias, float *state,
                       const float *z, const float *norm, size_t k_heads, size_t v_heads,
                       size_t k_dim, size_t v_dim, float eps, float *y) {
    float *q = malloc(k_heads * k_dim * sizeof(float)), *k = malloc(k_heads * k_dim * sizeof(float));
    float q_scale = 1.0f / sqrtf((float)k_dim);
    for (size_t h = 0; h < k_heads; h++) {
        const float *qh = q_in + h * k_dim, *kh = k_in + h * k_dim;
        float qi = q_scale / sqrtf(dot_f32(qh, qh, k_dim) + eps);
        float ki = 1.0f / sqrtf(dot_f32(kh, kh, k_dim) + eps);
        for (size_t i = 0; i < k_dim; i++) q[h * k_dim + i] = qh[i] * qi, k[h * k_dim + i] = kh[i] * ki;
    }
    size_t group = v_heads / k_heads;
    for (size_t h = 0; h < v_heads; h++) {
        float g = expf(-expf(a_log[h]) * softplus_f32(a[h] + dt_bias[h]));
        float beta = sigmoid_f32(b[h]);
        const float *qh = q + (h / group) * k_dim, *kh = k + (h / group) * k_dim;
        for (size_t i = 0; i < v_dim; i++) {
            float *row = state + (h * v_dim + i) * k_dim;
            for (size_t j = 0; j < k_dim; j++) row[j] *= g;
            float delta = (v[h * v_dim + i] - dot_f32(row, kh, k_dim)) * beta;
            for (size_t j = 0; j < k_dim; j++) row[j] += kh[j] * delta;
            y[h * v_dim + i] = dot_f32(row, qh, k_dim);
        }
        orc_rms_norm(y + h * v_dim, norm, v_dim, eps);
        for (size_t i = 0; i < v_dim; i++) y[h * v_dim + i] *= silu_f32(z[h * v_dim + i]);
    }
    free(q);
    free(k);
}

/* deltanet (src/cpu/deltanet.rs:69-114) with dense f32 projections [out][in]; used
 * to hold the two functions above against deltanet.json. */
void orc_deltanet_layer(const float *x, size_t hidden, size_t k_heads, size_t v_heads, size_t k_dim,
                        size_t v_dim, size_t kernel, float eps, const float *in_proj_qkv,
                        const float *in_proj_z, const float *in_proj_b, const float *in_proj_a,
                        const float *out_proj, const float *conv1d, const float *a_log,
                        const float *dt_bias, const float *norm, float *conv_state,
                        float *recurrent, float *out) {
    size_t key = k_heads * k_dim, val = v_heads * v_dim, conv = 2 * key + val;
    float *qkv = malloc(conv * sizeof(float)), *mixed = malloc(conv * sizeof(float));
    float *z = malloc(val * sizeof(float)), *y = malloc(val * sizeof(float));
    float *b = malloc(v_heads * sizeof(float)), *a = malloc(v_heads * sizeof(float));
    matvec_f32(in_proj_qkv, x, conv, hidden, qkv);
    matvec_f32(in_proj_z, x, val, hidden, z);
    matvec_f32(in_proj_b, x, v_heads, hidden, b);
    matvec_f32(in_proj_a, x, v_heads, hidden, a);
    orc_deltanet_conv(conv1d, qkv, conv_state, conv, kernel, mixed);
    orc_deltanet_step(mixed, mixed + key, mixed + 2 * key, a, b, a_log, dt_bias, recurrent, z, norm,
                      k_heads, v_heads, k_dim, v_dim, eps, y);
    matvec_f32(out_proj, y, hidden, val, out);
    free(qkv);
    free(mixed);
    free(z);
    free(y);
    free(b);
    free(a);
}

/* ------------------------------------------------- the reference's inputs ---- */

/* noise (tests/attention.rs:16-26, tests/kv_quant.rs:12-22): values in about
 * [-1, 1) from a 64-bit LCG. */
void orc_noise(float *out, size_t n, uint64_t seed) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; i++) {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        out[i] = (float)(s >> 40) / (float)(1ull << 23) - 1.0f;
    }
}

/* spread (src/attention_prefill.rs:103-108): halves in about -2 .. 2, as bits. */
void orc_spread(uint16_t *out, size_t n, size_t seed) {
    for (size_t i = 0; i < n; i++) {
        float v = (float)((i * 7919 + seed * 104729) % 1999) / 500.0f - 2.0f;
        out[i] = orc_f32_to_f16(v);
    }
}

/* rows (tests/kv_quant.rs:24-39): keys-like data, every third group x20 and
 * group 1 a constant -1.5. */
void orc_quant_rows(float *out, size_t tokens, size_t values) {
    size_t n = tokens * values;
    orc_noise(out, n, 7);
    for (size_t i = 0; i < n; i++) {
        if ((i / ORC_GROUP) % 3 == 0) out[i] *= 20.0f;
    }
    for (size_t i = ORC_GROUP; i < 2 * ORC_GROUP && i < n; i++) out[i] = -1.5f;
}
