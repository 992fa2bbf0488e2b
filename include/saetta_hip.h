/*
 * saetta_hip.h -- C ABI of the MI355X (gfx950) attention hot path.
 *
 * The library replaces, for this one path, what the reference's Rust modules
 * src/kv_quant.rs, src/attention.rs, src/rows.rs (verify attention),
 * src/attention_prefill.rs and src/attention_gemm.rs dispatch to Metal (and,
 * next to the path, the store step and the Gated DeltaNet kernels of
 * src/gpu_layers.rs and src/prefill.rs).  Every entry point is
 * extern "C", takes plain device pointers, POD parameter blocks that are
 * field-for-field the reference's #[repr(C)] structs, and an explicit HIP
 * stream; it enqueues work on that stream and returns without synchronising.
 *
 * Return value: 0 on success; a negative SAETTA_E_* code for a rejected
 * argument (the reference `assert!`s in these places, so a binding turns a
 * non-zero return into a panic); a positive value is the hipError_t of a
 * failed launch.  saetta_last_error() gives the text for the calling thread.
 * Nothing is thrown across the boundary and nothing aborts.
 *
 * Device pointers must be valid on the current HIP device.  "d_tp" arguments
 * point at a TokenParams record IN DEVICE MEMORY: launches read the position
 * and length from it when they run, so a recorded sequence of launches (a
 * plan, a HIP graph) serves every token position, as the reference's plans do
 * (src/plan.rs:1-11).
 */
#ifndef SAETTA_HIP_H
#define SAETTA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hipStream_t, spelled without the HIP headers. */
typedef void *saetta_stream_t;

/* Fixed shape of the path (src/attention.rs:14-17, src/kv_quant.rs:9). */
#define SAETTA_HEAD_DIM 256
#define SAETTA_GQA_GROUP 8   /* q heads per kv head */
#define SAETTA_QUANT_GROUP 64 /* values per scale/bias */
#define SAETTA_CHUNK 128      /* tokens per split-K chunk */
#define SAETTA_MAX_ROWS 8     /* src/rows.rs:9 */

enum {
    SAETTA_OK = 0,
    SAETTA_E_BITS = -1,     /* bits not one the call accepts */
    SAETTA_E_SHAPE = -2,    /* heads / kv_heads / head_dim / rows / capacity not supported */
    SAETTA_E_NULL = -3,     /* a required pointer is NULL */
    SAETTA_E_ALIGN = -4,    /* a pointer is not aligned as documented */
    SAETTA_E_DEVICE = -5,   /* no gfx950 device / code object not loadable */
    SAETTA_E_SCRATCH = -6,  /* scratch too small for the request */
    SAETTA_E_WAIT = -7      /* a kernel launched earlier on this device gave up a bounded wait: see
                               saetta_device_status */
};

/* TokenParams (src/plan.rs:16-35; kernels/params.metal:7-15). */
typedef struct saetta_token_params {
    uint32_t token;
    uint32_t position;
    uint32_t kv_len; /* position + 1 */
    uint32_t pad;
} saetta_token_params;

/* KvQuantParams (src/kv_quant.rs:147-153; kernels/kv_quant.metal:8-11). */
typedef struct saetta_kv_quant_params {
    uint32_t groups;    /* groups of 64 values to process, from x[0] */
    uint32_t per_token; /* groups per token: kv_heads * 256 / 64 */
} saetta_kv_quant_params;

/* DecodeParams (src/attention.rs:19-26; kernels/attention.metal:18-23). */
typedef struct saetta_decode_params {
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t capacity; /* tokens the cache has room for: a multiple of 16 (the reference's caches are
                          multiples of 128, src/gpu_layers.rs:199) */
    float scale;       /* 1/sqrt(256) */
} saetta_decode_params;

/* RowsAttentionParams (src/rows.rs:307-317; kernels/attention_rows.metal:58-65).
 * `splits` is the number of partial results per (row, q head) the scratch
 * has room for; the library uses min(splits, its own choice). */
typedef struct saetta_rows_params {
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t capacity;
    float scale;
    uint32_t rows;   /* m, 1..8 */
    uint32_t splits;
} saetta_rows_params;

/* FlashParams (src/attention_prefill.rs:4-14). */
typedef struct saetta_flash_params {
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t pos;    /* position of the chunk's first token; token i sees keys 0..=pos+i */
    uint32_t tokens;
    float scale;
} saetta_flash_params;

/* PrepParams (src/gpu_layers.rs:387-394; kernels/layers.metal:639-646). */
typedef struct saetta_prep_params {
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t dim;        /* head dim: 256 */
    uint32_t half_dims;  /* rotary dims / 2 */
    float log2_theta;
    float eps;
} saetta_prep_params;

/* ConvParams (kernels/layers.metal:198-201) and StepParams (kernels/layers.metal:290-295). */
typedef struct saetta_conv_params {
    uint32_t channels;
    uint32_t kernel_size;
} saetta_conv_params;
typedef struct saetta_step_params {
    uint32_t k_heads;
    uint32_t v_heads;
    uint32_t v_dim;
    float eps;
} saetta_step_params;
/* ConvRowsParams (kernels/prefill.metal:571-576). */
typedef struct saetta_conv_rows_params {
    uint32_t channels;
    uint32_t kernel_size;
    uint32_t tokens;
    uint32_t snapshots; /* write the state after each token to `snaps` */
} saetta_conv_rows_params;
/* DeltaRowsParams (kernels/prefill.metal:629-637) and RowsStepParams
 * (src/gpu_layers.rs:563-571); the floats per token of `mixed` follow from
 * the heads: 2 * k_heads * 128 + v_heads * v_dim. */
typedef struct saetta_rows_step_params {
    uint32_t k_heads;
    uint32_t v_heads;
    uint32_t v_dim;
    uint32_t tokens;
    float eps;
    uint32_t snapshots; /* write the state after each token to `snaps` */
} saetta_rows_step_params;
/* RowsStepParams (src/gpu_layers.rs:563-571), field for field. */
typedef struct saetta_rows_fused_params {
    uint32_t k_heads;
    uint32_t v_heads;
    uint32_t v_dim;
    uint32_t kernel_size;
    float eps;
    uint32_t rows;      /* 0..8 */
    uint32_t snapshots; /* write the states after each row to the snapshot buffers */
} saetta_rows_fused_params;

/* The three arrays of one quantized cache, keys or values: QuantRows
 * {data, scales, biases} (src/kv_quant.rs:156-180).  Token p's groups start
 * at group p * per_token; group G's codes are words 2*bits*G onward, lowest
 * bits first; scales and biases are IEEE halves. */
typedef struct saetta_quant_rows {
    uint32_t *data;
    uint16_t *scales;
    uint16_t *biases;
} saetta_quant_rows;

/* ---- set-up --------------------------------------------------------------- */

/* Checks that the current device is gfx950, loads the kernels and raises their
 * LDS limits; once per device.  Stands where Gpu::new() (src/gpu.rs:233-263)
 * stands for this path.  Every entry point does the same on its first use on a
 * device, but that first use must not be under stream capture: call this, with
 * the device current, before capturing a graph. */
int saetta_init(void);

/* Text of the last error on this thread ("" if none). */
const char *saetta_last_error(void);

/* The sticky status word of the current device; 0 as long as nothing went wrong.  The waves of the
 * decode / verify kernel that keeps a whole share of the cache in LDS meet through counters that
 * they poll a bounded number of times, so that every wave ends whatever happens.  A wave whose
 * wait runs out stores a code here (0x100 + the counter's index), marks the partial result of its
 * workgroup with l = NaN, so that the reduce stage gives NaN for the (row, head) and never a
 * plausible number, and goes on to its end.  The word lives in pinned host memory and is read
 * without synchronising: it shows what the kernels that have run so far have left.  Once it is
 * non-zero every entry point returns SAETTA_E_WAIT until a call with clear != 0 has reset it.
 * Returns the word as it was before clearing.  The reference has no counterpart: its kernels wait
 * at threadgroup barriers only. */
uint32_t saetta_device_status(int clear);

/* ---- kv_quant (src/kv_quant.rs) -------------------------------------------- */

/* QuantRows::record / record_at (src/kv_quant.rs:192-221) when d_tp != NULL:
 * quantizes p.groups groups of x into the slots from token d_tp->position.
 * QuantRows::encode (src/kv_quant.rs:256-282) when d_tp == NULL: the slots
 * from token `pos`.  Kernel: kv_quantize_{8,4} (kernels/kv_quant.metal:15-59).
 * Codes, scales and biases are bit-identical to the CPU quantize()
 * (src/kv_quant.rs:54-87).  x must be 16-byte aligned. */
int saetta_kv_quantize(saetta_stream_t stream, int bits, const float *x, saetta_quant_rows rows,
                       saetta_kv_quant_params p, const saetta_token_params *d_tp, uint32_t pos);

/* QuantRows::encode_dequantize (src/kv_quant.rs:225-252): groups 0..p.groups
 * as halves, out[i] = half(f32(s) * q + f32(z)). */
int saetta_kv_dequantize(saetta_stream_t stream, int bits, saetta_quant_rows rows, uint16_t *out_f16,
                         saetta_kv_quant_params p);

/* dequantize (src/kv_quant.rs:90-105), the CPU function: out f32
 * [groups][64] = f32(scale) * code + f32(bias), not rounded to half.  With
 * saetta_kv_quantize before it this is round_trip (src/kv_quant.rs:107-117). */
int saetta_kv_dequantize_f32(saetta_stream_t stream, int bits, saetta_quant_rows rows, float *out,
                             saetta_kv_quant_params p);

/* to_half (kernels/prefill.metal:1428-1432; src/prefill.rs:1658-1660,1690-1692):
 * n floats to halves, round to nearest even. */
int saetta_to_half(saetta_stream_t stream, const float *x, uint16_t *out_f16, size_t n);

/* ---- decode and verify attention (src/attention.rs, src/rows.rs) ----------- */

/* Bytes of part_o / part_ml scratch for a cache of `capacity` tokens and up
 * to `rows` rows: never more than the reference allocates
 * (rows * ceil(capacity/128) * heads * 256 * 4 and * 2 * 4,
 * src/attention.rs:58-64, src/rows.rs:358-359). */
size_t saetta_part_o_bytes(uint32_t heads, uint32_t capacity, uint32_t rows);
size_t saetta_part_ml_bytes(uint32_t heads, uint32_t capacity, uint32_t rows);

/* Stages of one attention call, for timing a kernel alone as the reference
 * does with Plan::build_where (src/plan.rs:187-226, src/attention.rs:206). */
#define SAETTA_STAGE_PARTIAL 1u
#define SAETTA_STAGE_REDUCE 2u
#define SAETTA_STAGE_ALL 3u
/* Or-ed into `stages`: keep to the kernels that load the cache into registers, also where the
 * library would pick the kernel whose extra waves stage the codes in LDS.  The counterpart of
 * DecodeAttention.kernel (src/attention.rs:36-38), which switches the reference between its two
 * kernel families.  The partial and the reduce stage of one step must be called with the same
 * flag: the number of splits follows from it. */
#define SAETTA_STAGE_NO_LOADERS 4u

/* DecodeAttention::record (src/attention.rs:73-92): one query token over a
 * half cache.  q f32 [heads][256]; keys, values f16 [capacity][kv_heads][256];
 * q_and_gate f32 [heads][512], the gate of head h at h*512+256; out f32
 * [heads][256].  out = softmax(q K^T scale) V * sigmoid(gate) over the first
 * min(d_tp->kv_len, capacity) tokens.  Kernels replaced: attention_partial,
 * attention_partial_mma, attention_reduce (kernels/attention.metal:25-226,
 * 367-409). */
int saetta_attn_decode(saetta_stream_t stream, const float *q, const uint16_t *keys,
                       const uint16_t *values, float *part_o, float *part_ml,
                       const float *q_and_gate, float *out, saetta_decode_params p,
                       const saetta_token_params *d_tp, uint32_t stages);

/* DecodeAttention::record_quant (src/attention.rs:95-135): as above over an
 * 8- or 4-bit cache.  Kernels replaced: attention_partial_mma_q{8,4}
 * (kernels/attention.metal:242-360), attention_partial_q{8,4}
 * (kernels/kv_quant.metal:101-204), attention_reduce. */
int saetta_attn_decode_quant(saetta_stream_t stream, int bits, const float *q,
                             saetta_quant_rows keys, saetta_quant_rows values, float *part_o,
                             float *part_ml, const float *q_and_gate, float *out,
                             saetta_decode_params p, const saetta_token_params *d_tp,
                             uint32_t stages);

/* saetta_attn_decode_quant without the part_o / part_ml arguments, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): the partials go to a buffer that is part of the library's code object, 4 MiB + 32 KiB
 * per device (saetta_static_scratch_bytes), and the call allocates nothing.  It has no counterpart
 * in the reference, whose DecodeAttention::new allocates its scratch (src/attention.rs:58-64).
 * Limit: p.heads <= 16 (any capacity: a launch never uses more than 256 splits); more is rejected
 * with SAETTA_E_SCRATCH.  Same kernels, same results, bit for bit, as saetta_attn_decode_quant.
 * All calls on one device share the one buffer: between the partial stage of a call and its reduce
 * stage no other call of this entry point may run on that device, so calls from different streams
 * or threads that overlap on a device race.  Nothing in the buffer needs clearing: every slot the
 * reduce stage reads was written by the partial stage of the same call.  saetta_init (or any
 * earlier call on the device) must have run outside stream capture. */
size_t saetta_static_scratch_bytes(void);
int saetta_attn_decode_quant_static(saetta_stream_t stream, int bits, const float *q,
                                    saetta_quant_rows keys, saetta_quant_rows values,
                                    const float *q_and_gate, float *out, saetta_decode_params p,
                                    const saetta_token_params *d_tp, uint32_t stages);

/* AttentionRows::record (src/rows.rs:369-412): p.rows query tokens over a
 * half cache; row r is at position d_tp->position + r and sees
 * min(d_tp->position + r + 1, capacity) tokens.  q f32 [rows][heads][256],
 * q_and_gate f32 [rows][heads][512], out f32 [rows][heads][256].  Kernels
 * replaced: attention_partial_rows_chunks, attention_reduce_rows_chunks
 * (kernels/attention_rows.metal:359-571). */
int saetta_attn_rows(saetta_stream_t stream, const float *q, const uint16_t *keys,
                     const uint16_t *values, float *part_o, float *part_ml,
                     const float *q_and_gate, float *out, saetta_rows_params p,
                     const saetta_token_params *d_tp, uint32_t stages);

/* AttentionRows::record_quant (src/rows.rs:416-493).  Kernels replaced:
 * attention_partial_rows<8|4>, attention_reduce_rows
 * (kernels/attention_rows.metal:108-342). */
int saetta_attn_rows_quant(saetta_stream_t stream, int bits, const float *q,
                           saetta_quant_rows keys, saetta_quant_rows values, float *part_o,
                           float *part_ml, const float *q_and_gate, float *out,
                           saetta_rows_params p, const saetta_token_params *d_tp,
                           uint32_t stages);

/* ---- the step before the scores (src/gpu_layers.rs) -------------------------- */

/* GpuAttention::record_store (src/gpu_layers.rs:370-411): q norm and RoPE into
 * q_out, k norm and RoPE, then the token's key and value into their cache
 * slot, in ONE launch.  Replaces attention_prep / attention_prep_float
 * (kernels/layers.metal:637-702) and, for a quantized cache, the two
 * kv_quantize dispatches that follow it (src/kv_quant.rs:192-221).
 * q_and_gate f32 [rows][heads][512], k, v f32 [rows][kv_heads][256], q_norm,
 * k_norm f32 [256], q_out f32 [rows][heads][256].  bits 16: keys_half,
 * values_half are the half cache [capacity][kv_heads][256] and the quantized
 * rows are ignored; bits 8 or 4: the other way round.  Row r is the token at
 * TokenParams.position + r; a row at or past `capacity` is not stored.
 * k_back (or NULL): f32 [rows][kv_heads][256] gets the normed, rotated key,
 * which is what attention_prep_float leaves in k. */
int saetta_attn_prep_store(saetta_stream_t stream, int bits, const float *q_and_gate, const float *k,
                           const float *v, const float *q_norm, const float *k_norm, float *q_out,
                           uint16_t *keys_half, uint16_t *values_half, saetta_quant_rows keys,
                           saetta_quant_rows values, float *k_back, saetta_prep_params p, uint32_t rows,
                           uint32_t capacity, const saetta_token_params *d_tp);

/* ---- Gated DeltaNet, one token (src/cpu/deltanet.rs, src/gpu_layers.rs) ------ */

/* conv_step (src/cpu/deltanet.rs:117-131); kernel deltanet_conv
 * (kernels/layers.metal:203-226): depthwise causal conv1d over the stored
 * inputs and x, then SiLU; x shifts into the state.  x, out f32 [channels];
 * w f32 [channels][kernel_size], last column = newest token; state f32
 * [kernel_size - 1][channels], oldest first, updated in place. */
int saetta_deltanet_conv(saetta_stream_t stream, const float *x, const float *w, float *state, float *out,
                         saetta_conv_params p);

/* Everything between the conv and out_proj (src/cpu/deltanet.rs:86-112,133-155);
 * kernel deltanet_step (kernels/layers.metal:297-357): L2 norm of q and k, the
 * gates, the delta rule on every value head's state and the gated RMSNorm.
 * q, k f32 [k_heads][128]; v, z, y f32 [v_heads][v_dim]; a, b, a_log, dt_bias
 * f32 [v_heads]; state f32 [v_heads][v_dim][128], updated in place; norm_w
 * f32 [v_dim].  Key dim 128, v_dim up to 256. */
int saetta_deltanet_step(saetta_stream_t stream, const float *q, const float *k, const float *v,
                         const float *a, const float *b, const float *a_log, const float *dt_bias,
                         float *state, const float *z, const float *norm_w, float *y,
                         saetta_step_params p);

/* saetta_deltanet_conv and saetta_deltanet_step of one token as one call of two
 * launches (GpuDeltaNet::record, src/gpu_layers.rs:633-684, records the two
 * kernels one after the other; nothing else reads the conv output): 32 state
 * rows per workgroup instead of a head, each workgroup computing the conv
 * outputs it needs, then the gated norm and the shift of x into the conv state.
 * Arguments as for the two calls; cp.channels = 2 * k_heads * 128 + v_heads * v_dim. */
int saetta_deltanet_token(saetta_stream_t stream, const float *x, const float *w, float *conv_state,
                          const float *a, const float *b, const float *a_log, const float *dt_bias,
                          float *state, const float *z, const float *norm_w, float *y,
                          saetta_conv_params cp, saetta_step_params sp);

/* ---- Gated DeltaNet, several tokens in order: verify rows and prefill chunks -- */

/* conv over `tokens` tokens: kernels conv_rows2 + conv_state
 * (kernels/prefill.metal:734-786, recorded by src/prefill.rs:1455-1485) and
 * deltanet_conv_rows (kernels/layers.metal:510-544).  x, out f32
 * [tokens][channels]; w and state as for saetta_deltanet_conv; the state ends as
 * the last kernel_size - 1 inputs.  With snapshots, snaps f32
 * [tokens][kernel_size - 1][channels] gets the state after each token (what
 * GpuDeltaNetSnaps.conv holds, src/gpu_layers.rs:819-836); else it may be NULL. */
int saetta_deltanet_conv_rows(saetta_stream_t stream, const float *x, const float *w, float *state, float *out,
                              float *snaps, saetta_conv_rows_params p);

/* What saetta_deltanet_step does, for `tokens` tokens one after the other:
 * kernels delta_prep + delta_rows3 and the gated norm (kernels/prefill.metal:788-1116,
 * src/prefill.rs:1487-1578), deltanet_step_rows (kernels/layers.metal:546-635,
 * GpuDeltaNet::record_rows, src/gpu_layers.rs:686-786).  mixed f32
 * [tokens][2 * k_heads * 128 + v_heads * v_dim] is the conv output: q of every
 * key head, then k, then v of every value head; unlike delta_prep the call
 * leaves it (and a, b) unchanged.  a, b f32 [tokens][v_heads]; z, y f32
 * [tokens][v_heads][v_dim]; state f32 [v_heads][v_dim][128] updated in place.
 * With snapshots, snaps f32 [tokens][v_heads][v_dim][128] gets the state after
 * each token (GpuDeltaNetSnaps.recurrent); else it may be NULL.  Key dim 128,
 * v_dim a multiple of 4 up to 256.  The call holds no buffer of the library's:
 * it runs token by token at every length and only enqueues kernels, so calls on
 * different streams share nothing.  A prefill chunk wants saetta_deltanet_rows_ws. */
int saetta_deltanet_rows(saetta_stream_t stream, const float *mixed, const float *a, const float *b,
                         const float *a_log, const float *dt_bias, float *state, const float *z,
                         const float *norm_w, float *y, float *snaps, saetta_rows_step_params p);

/* The same call with a workspace of the caller's (the reference's encode_deltanet
 * works in buffers of the prefill's own, src/prefill.rs:1433-1578): from 128 tokens
 * on, without snapshots and with v_dim a multiple of 16, the delta rule runs in
 * blocks of 64 tokens on the matrix cores (231 against 700 us for 4096 tokens of the
 * model's layer) and keeps per-block matrices in `workspace`
 * (saetta_deltanet_rows_workspace_bytes(p) bytes, 16-byte aligned; 0 bytes: the call
 * runs token by token and takes no workspace).  The workspace belongs to the call
 * until its kernels have run: calls that may overlap (different streams) bring
 * different workspaces.  With workspace NULL this is saetta_deltanet_rows.
 * Range of the blocked form: its operands (state, values and the products between
 * them) go to the matrix cores as pairs of halves, so magnitudes must stay below
 * 65504, and parts below 2^-25 of a value are dropped; the token-by-token form is
 * plain f32. */
size_t saetta_deltanet_rows_workspace_bytes(saetta_rows_step_params p);
int saetta_deltanet_rows_ws(saetta_stream_t stream, const float *mixed, const float *a, const float *b,
                            const float *a_log, const float *dt_bias, float *state, const float *z,
                            const float *norm_w, float *y, float *snaps, saetta_rows_step_params p,
                            void *workspace, size_t workspace_size);

/* Kernel deltanet_rows (recorded by GpuDeltaNet::record_rows with DN_SIMDS = 0,
 * src/gpu_layers.rs:737-757): conv and step of up to 8 rows as one op, what
 * saetta_deltanet_conv_rows + saetta_deltanet_rows give, in two launches
 * instead of four; the call for the verify step.  x f32 [rows][channels] is the
 * qkv projection (channels = 2 * k_heads * 128 + v_heads * v_dim); a, b f32
 * [rows][v_heads]; z, y f32 [rows][v_heads][v_dim]; conv_state, state as above.
 * With snapshots: conv_snaps f32 [rows][kernel_size - 1][channels], state_snaps
 * f32 [rows][v_heads][v_dim][128]; else both may be NULL. */
int saetta_deltanet_rows_fused(saetta_stream_t stream, const float *x, const float *w, float *conv_state,
                               const float *a, const float *b, const float *a_log, const float *dt_bias,
                               float *state, const float *z, const float *norm_w, float *y,
                               float *conv_snaps, float *state_snaps, saetta_rows_fused_params p);

/* ---- prefill attention (src/attention_prefill.rs, src/prefill.rs) ---------- */

/* Bytes of workspace a prefill chunk at (pos, tokens) needs: the f16 key and
 * value tile images of the pos + tokens rows the chunk can see.  The reference
 * has no counterpart (its kernels dequantize in place); the closest is the
 * half scratch of Prefill::new (src/prefill.rs:1674-1686). */
size_t saetta_prefill_workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t kv_heads);

/* attention_prefill::encode (src/attention_prefill.rs:39-72): a causal chunk
 * over a half cache that already holds the chunk's rows.  q f16
 * [tokens][heads][256]; keys, values f16 [capacity][kv_heads][256] from
 * position 0, capacity >= pos + tokens; q_and_gate f32 [tokens][heads][512];
 * out f32 [tokens][heads][256].  workspace: device memory of at least
 * saetta_prefill_workspace_bytes(pos, tokens, kv_heads) bytes, 16-byte
 * aligned, overwritten by the call; NULL makes the library use one of its own
 * per device and stream, which it grows with hipMalloc when needed (so not
 * under stream capture) and keeps until the process ends.  Kernel replaced:
 * attention_fa{4,8} (kernels/attention_prefill.metal:38-169). */
int saetta_attn_prefill(saetta_stream_t stream, const uint16_t *q_f16, const uint16_t *keys,
                        const uint16_t *values, const float *q_and_gate, float *out,
                        saetta_flash_params p, void *workspace, size_t workspace_bytes);

/* The same chunk over an 8- or 4-bit cache read in place
 * (src/prefill.rs:1674-1686,1735-1776); the cache is seen through half, as
 * round_trip_as_half (src/kv_quant.rs:119-125) defines.  Kernels replaced:
 * attention_rows_q{8,4}, attention_rows2_half_q{8,4}
 * (kernels/attention_rows_q.metal:55-344). */
int saetta_attn_prefill_quant(saetta_stream_t stream, int bits, const uint16_t *q_f16,
                              saetta_quant_rows keys, saetta_quant_rows values,
                              const float *q_and_gate, float *out, saetta_flash_params p,
                              void *workspace, size_t workspace_bytes);

/* ---- prefill attention as matrix products (src/attention_gemm.rs) ----------- */

/* attention_gemm::KEYS (src/attention_gemm.rs:28): keys per block. */
#define SAETTA_AG_KEYS 1024

/* Bytes of workspace AttGemm needs for a chunk at (pos, tokens) run in slices
 * of up to slice_tokens tokens (0: one slice): the key and value tile images
 * of saetta_prefill_workspace_bytes, then what AttGemm::new allocates for one
 * slice (src/attention_gemm.rs:118-142): the probabilities of eight blocks of
 * keys (a pair of launches takes eight blocks, so that q and the output sums
 * go through memory once per eight), the tile maxima and sums, the output sums
 * and the per-row softmax state; about 19 KB per query row of a slice. */
size_t saetta_attn_gemm_workspace_bytes(uint32_t pos, uint32_t tokens, uint32_t slice_tokens,
                                        uint32_t kv_heads);

/* AttGemm::encode (src/attention_gemm.rs:144-188, encode_slice :190-364), the
 * default (fused) variant: the same chunk and the same buffers as
 * saetta_attn_prefill / saetta_attn_prefill_quant, computed block by block of
 * SAETTA_AG_KEYS keys with the block's probabilities written out and read
 * back.  bits 16: keys.data and values.data are the half caches and the scales
 * and biases are not read (the reference's quant = None); bits 8 or 4: the
 * quantized rows, seen through half.  stages (AttGemm::stages,
 * src/attention_gemm.rs:112-114): 0 runs everything; 1 or 2 only the scores
 * pass of each block; 3 scores and pv and no outputs.  workspace as for
 * saetta_attn_prefill, of saetta_attn_gemm_workspace_bytes bytes.  Kernels
 * replaced: prefill_ag_scores_t{,_q8,_q4}, prefill_ag_pv_t{,_q8,_q4},
 * prefill_ag_final (kernels/attention_gemm.metal). */
int saetta_attn_gemm(saetta_stream_t stream, int bits, const uint16_t *q_f16, saetta_quant_rows keys,
                     saetta_quant_rows values, const float *q_and_gate, float *out,
                     saetta_flash_params p, uint32_t slice_tokens, uint32_t stages, void *workspace,
                     size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* SAETTA_HIP_H */
