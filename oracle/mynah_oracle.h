/* TEST INFRASTRUCTURE ONLY -- a CPU restatement of the reference's decode-step arithmetic.
 *
 * Nothing in the shipped library (mynah-tts_amd/csrc, include/) includes, links or calls
 * this file.  It exists so tests, the smoke check and the benchmark's CPU-baseline leg have
 * an independent statement of what the reference computes.  Each function cites the
 * reference file:line it restates (paths relative to the reference tree).
 *
 * Pinning status (which independent evidence checks each function; see tests/test_oracle_*.py):
 *   quantizers, int dots, matvec_q8/q4, act-quant   -- bit-compared with the compiled reference
 *                                                     (oracle/_ref, both flag sets) + brute force ties
 *   layernorm, gelu, softmax, argmax, residual      -- reference self-test KATs (src/kernels.c:439-517)
 *                                                     + float64 closed forms + compiled reference
 *   self/cross attention                            -- Metal resident-op KATs
 *                                                     (gpu/metal/backend_metal_ops.m:1049-1079) + float64
 *                                                     softmax(QK^T)V + compiled reference decode step
 *   decoder step                                    -- compiled reference decoder_step_batch (f32/int8/int4,
 *                                                     B=1 and ragged B=8) + batched==solo bit identity
 *   f16 rounding                                    -- numpy.float16 (IEEE RNE) over all 65536 halves and
 *                                                     random floats; ingot KATs 0x3c00<->1.0
 *   matvec_f16                                      -- no x86 reference build exists (src/qmat.c:25-28);
 *                                                     pinned by float64 dot of exactly-widened halves
 *   encoder prefill                                 -- the reference's form (causal mask, gain-only LayerNorm, plain and
 *                                                     kernel-3 conv FFN): compiled reference's transformer_stack
 *                                                     (src/graph.c:634-711) on f16-representable weights, 1 / 37 / 130 / 256
 *                                                     tokens, both flag sets, 1e-5; the same outputs committed as golden
 *                                                     vectors.  The bidirectional form with LayerNorm biases (the synthetic
 *                                                     prefill configuration, which the reference has no function for): a
 *                                                     float64 numpy restatement written from the definition, 1e-5.
 *   orc_gemm_nt                                     -- float64 matmul; a row equals orc_matvec_f32 of that row bit for bit
 *   orc_output_head                                 -- equals orc_linear + orc_softmax per head bit for bit (both pinned
 *                                                     above); float64 softmax and, for f32 weights, float64 logits
 *   local step (local_step_batch)                   -- compiled reference's own local_step_batch (f32/int8/int4, both
 *                                                     flag sets, three positions of a batch of three)
 *   local token choice and frame bookkeeping (sample_local_frame_batch)
 *                                                   -- the function needs a whole model object and is not reachable
 *                                                     in the compiled reference; pinned by what fixes it without it:
 *                                                     xorshift64 against numpy uint64, mask / first-max hand cases,
 *                                                     the sampled token against an independent numpy restatement
 *                                                     (stable sort, float32 sequential sums) on seeded rows with ties,
 *                                                     draw frequencies against softmax
 *   codec conv1d / transposed conv / snake          -- compiled reference's conv1d_causal, conv_transpose_causal and
 *                                                     mynah_backend_snake_dev on a synthetic safetensors file;
 *                                                     Metal self-test KAT (gpu/metal/backend_metal_ops.m:1026-1106);
 *                                                     float64 numpy convolution
 */
#ifndef MYNAH_ORACLE_H
#define MYNAH_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_F32 = 0, ORC_INT8 = 1, ORC_INT4 = 2, ORC_F16 = 3 };   /* src/qmat.c:36 */
enum { ORC_STRICT = 0, ORC_STOCK = 1 };   /* quantizer arithmetic: source as written / stock -ffast-math build */

/* ---- load-time weight conversion ---- */
void orc_quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales, int variant);
int orc_quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales, int variant);
uint16_t orc_f32_to_f16(float value);
float orc_f16_to_f32(uint16_t bits);
void orc_f32_to_f16_array(const float *in, uint16_t *out, size_t n);

/* ---- per-vector activation quantization ---- */
float orc_quantize_act_int8(int8_t *qx, const float *x, size_t k, int variant);

/* ---- matvec kernels ---- */
int32_t orc_dot_q8_i32(const int8_t *qx, const int8_t *w, size_t k);
void orc_matvec_q8(float *out, int32_t *acc_out, const int8_t *qx, float sx, const int8_t *weights,
                   const float *scales, const float *bias, size_t rows, size_t cols);
void orc_matvec_q4(float *out, int32_t *group_acc_out, const int8_t *qx, float sx, const uint8_t *weights,
                   const float *scales, const float *bias, size_t rows, size_t cols);
void orc_matvec_f16(float *out, const float *x, const uint16_t *weights, const float *bias,
                    size_t rows, size_t cols);
void orc_matvec_f32(float *out, const float *x, const float *weights, const float *bias,
                    size_t rows, size_t cols);

typedef struct {
    int qtype;           /* ORC_* */
    size_t n, k;         /* out rows, in columns */
    const void *data;    /* f32 [n,k] | int8 [n,k] | packed nibbles [n,k/2] | f16 bits [n,k] */
    const float *scales; /* int8: [n]; int4: [n,k/32]; else NULL */
} orc_weight;

/* out[n] = W x (+bias): act-quant for int8/int4, f32 activations for f16/f32. */
void orc_linear(const orc_weight *w, const float *x, float *out, const float *bias, int act_variant);

/* ---- f32 elementwise kernels ---- */
void orc_layernorm(const float *in, const float *gain, const float *bias, float *out,
                   size_t rows, size_t width, float eps);
void orc_gelu_scalar(float *data, size_t n);
void orc_gelu_pade(float *data, size_t n);
int orc_softmax(const float *logits, float *probs, size_t n);
void orc_softmax_row_inplace(float *values, size_t n);
void orc_softmax_masked(float *data, size_t rows, size_t cols, size_t valid);
void orc_residual_add(float *out, const float *in, size_t n);
int orc_argmax_constrained(const float *logits, size_t vocab, size_t codebook_size, size_t eos_id,
                           int allow_eos, unsigned *argmax);

/* ---- single-token attention ---- */
void orc_self_attention(const float *qkv, float *k_cache, float *v_cache, size_t position,
                        size_t cache_stride, size_t valid, size_t heads, size_t head_width,
                        float scale, float *out, float *scores_scratch);
void orc_cross_attention(const float *q, const float *k_cache, const float *v_cache, size_t valid,
                         size_t cache_stride, size_t heads, size_t head_width, float scale,
                         float *out, float *scores_scratch);

/* ---- whole decode step ---- */
typedef struct {
    size_t layers, width, heads, head_width, ffn;
    size_t cross_heads, cross_head_width;   /* xw = cross_heads * cross_head_width */
    size_t capacity;
    const orc_weight *qkv, *o_self, *q_cross, *o_cross, *ffn_up, *ffn_down;   /* [layers] each */
    const float *norm_self_g, *norm_self_b;     /* [layers,width]; *_b may be NULL (gain-only) */
    const float *norm_cross_g, *norm_cross_b;
    const float *norm_ff_g, *norm_ff_b;
    const float *norm_out_g, *norm_out_b;       /* [width] */
    const float *position;                      /* [capacity,width] or NULL (no position add) */
    int act_variant;
} orc_decoder;

/* B slots, one token each.  self_k/self_v[b]: [layers,capacity,width] appended at lengths[b];
 * cross_k/cross_v[b]: [layers,memory_lengths[b],xw].  outs[b]: [width] after the final norm.
 * hidden_out[b] (optional): the pre-final-norm residual stream.  lengths are NOT advanced. */
int orc_decoder_step(const orc_decoder *d, size_t batch, float *const *self_k, float *const *self_v,
                     const float *const *cross_k, const float *const *cross_v,
                     const size_t *lengths, const size_t *memory_lengths,
                     const float *const *inputs, float *const *outs);

/* Test hook: the same step, with stream 0's int8 activations at each projection optionally taken from the caller
 * (forced_qx [layers][6][ffn] bytes, forced_sx [layers][6]; projections in the order qkv, o_self, q_cross, o_cross,
 * ffn_up, ffn_down; both NULL: nothing forced) and the ones quantised here optionally written out (capture_*, same
 * layout).  counts[0]: elements in which the forced vectors differ from the ones quantised here; counts[1]: the largest
 * such difference in int8 steps. */
int orc_decoder_step_forced(const orc_decoder *d, size_t batch, float *const *self_k, float *const *self_v,
                            const float *const *cross_k, const float *const *cross_v,
                            const size_t *lengths, const size_t *memory_lengths,
                            const float *const *inputs, float *const *outs,
                            const int8_t *forced_qx, const float *forced_sx, size_t *counts, int8_t *capture_qx, float *capture_sx);

/* final-normed hidden [width] -> logits [heads_out*vocab] -> softmax per head. */
void orc_output_head(const orc_weight *w_out, const float *bias, const float *hidden, size_t heads_out,
                     size_t vocab, float *logits, float *probs, int act_variant);

/* ---- encoder prefill (pre-LN; causal or bidirectional; plain or causal conv FFN; f16-rounded weights) ---- */
typedef struct {
    size_t layers, width, heads, head_width, ffn, vocab, max_positions;
    const uint16_t *tok_table;   /* f16 bits [vocab,width] */
    const uint16_t *pos_table;   /* f16 bits [max_positions,width] */
    const uint16_t *qkv_w, *o_w, *up_w, *down_w;   /* f16 bits, per layer concatenated */
    const float *norm1_g, *norm1_b, *norm2_g, *norm2_b;   /* [layers,width]; *_b may be NULL */
    const float *norm_out_g, *norm_out_b;          /* [width] or NULL gain => no final norm */
    int causal;                  /* != 0: row t attends rows [0, t] (the reference's encoder); 0: the full row */
    size_t ffn_kernel;           /* 0 or 1: plain FFN, up_w [ffn,width], down_w [width,ffn]; k > 1: causal conv FFN,
                                    up_w [ffn,width,k], down_w [width,ffn,k] */
} orc_encoder;

/* embed_out: f16 bits [T,width] of the gathered token rows (bit-exact artefact);
 * out: f32 [T,width].  threads >= 1 splits GEMM rows over pthreads (results are thread-count independent). */
int orc_encoder_prefill(const orc_encoder *e, const int32_t *ids, size_t T, uint16_t *embed_out,
                        float *out, int threads);

/* f32 row-major C[m,n] = A[m,k] * B[n,k]^T, k-contiguous dots (used by the encoder and tests). */
void orc_gemm_nt(const float *a, const float *b, float *c, size_t m, size_t n, size_t k, int threads);

/* ---- local transformer frame: 16 sequential streams, each a local step + projection + token choice ---- */
typedef struct {
    float temperature;     /* sampling iff temperature > 0 && topk > 1 (src/graph.c:1487-1489) */
    size_t topk;
    uint64_t rng_state;    /* xorshift64 state, advanced once per sampled stream */
    int forbid_eos;        /* generated_raw_length < min_raw_length */
} orc_local_item;

/* One token from one row of logits, as sample_local_frame_batch chooses it (src/graph.c:1548-1616): constrained
 * first-max argmax (disallowed candidates are overwritten with -FLT_MAX in `logits`), then for sampling items the
 * top-k insertion sort, expf((l - max) / temperature), xorshift64 draw and cumulative pick.  Returns the value;
 * *greedy receives the argmax (EOS detection looks at both).  top_indices / top_values: scratch of topk entries. */
unsigned orc_local_choose(float *logits, size_t vocab, size_t codebook_size, size_t eos_id, orc_local_item *item,
                          unsigned *greedy, size_t *top_indices, float *top_values);

typedef struct {
    const orc_decoder *stack;              /* the local transformer: no cross attention, no final norm */
    size_t streams, vocab, codebook_size, eos_id, codebook_count;
    const orc_weight *projection;          /* [streams] packed [vocab, width] */
    const float *const *projection_bias;   /* [streams] [vocab] or NULL entries */
    const float *const *audio_table;       /* [streams] f32 [vocab, width] */
} orc_local;

/* sample_local_frame_batch (src/graph.c:1374-1656) for `batch` items that all stay live.  decoder_last[b]: [width].
 * k/v[b]: [layers, capacity, width] scratch caches (capacity >= streams).  values / stored: [batch, streams] the chosen
 * token and the code handed on (special tokens collapsed to 0); saw_eos / eos_frame: [batch] (eos_frame = SIZE_MAX when
 * none); logits_out (optional): [batch, streams, vocab] after the constraint mask. */
int orc_local_frame(const orc_local *L, size_t batch, const float *const *decoder_last, orc_local_item *items,
                    float *const *k, float *const *v, unsigned *values, unsigned *stored, int *saw_eos,
                    size_t *eos_frame, float *logits_out);

/* ---- codec operators (NanoCodec decoder), layout [channels, length] row-major ---- */

/* conv1d_causal (src/graph.c:2010-2160): out[o][t] = bias[o] + sum_i sum_k w[(o*in + i)*kernel + k] *
 * in[i][t - (kernel-1-k)*dilation], terms with a negative source index dropped.  Accumulates in the order of the
 * reference's scalar loop (:2141-2154: i outer, k inner); its usual path is im2col + sgemm, whose order is the BLAS's. */
void orc_conv1d_causal(const float *input, float *output, size_t in_channels, size_t out_channels, size_t length,
                       size_t kernel, size_t dilation, const float *weight, const float *bias);
/* conv_transpose_causal (src/graph.c:2179-2231): grouped transposed conv trimmed to output_length = length * stride
 * when kernel = 2 * stride (in general (length-1)*stride + kernel - (kernel - stride)); per output row the
 * contributions arrive in the reference's order (input channel, then input position, then tap). */
void orc_conv_transpose_causal(const float *input, float *output, size_t in_channels, size_t out_channels, size_t length,
                               size_t output_length, size_t kernel, size_t stride, size_t groups, const float *weight,
                               const float *bias);
/* snake_row (src/backend.c:643-658): channels below snake_channels get x + sin(a x)^2 * (1 / (a + 1e-9f)), the rest a
 * leaky ReLU with slope 0.01. */
void orc_snake(float *data, const float *alpha, size_t channels, size_t length, size_t snake_channels);

#ifdef __cplusplus
}
#endif
#endif
