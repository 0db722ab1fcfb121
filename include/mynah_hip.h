/* mynah_hip.h -- C ABI of the gfx950 (MI355X) HIP backend for Mynah TTS's decode-step kernels.
 *
 * Plain C: pointers, sizes, ints.  No C++ or framework types cross this boundary.
 * Conventions are the reference seam's (src/backend.c:137-139, :472):
 *   - every call returns 0 on success, -1 on failure, and writes a NUL-terminated message into
 *     `error` (capacity `error_capacity`; either may be NULL/0);
 *   - `state` is the opaque handle produced by mynah_backend_hip_open and destroyed by the close
 *     function it hands back;
 *   - "dev" pointers are device memory from mynah_hip_dev_alloc; weights, biases and LayerNorm
 *     gains are HOST pointers to immutable memory that outlives the backend, converted and cached
 *     on the device the first time they are seen, keyed by (address, byte size)
 *     (gpu/cuda/backend_cuda.cu:133-143,193-219);
 *   - resident ops enqueue on one internal stream and return without synchronising; only
 *     mynah_hip_sync, mynah_hip_d2h, mynah_hip_download, mynah_hip_argmax_dev and the host-pointer
 *     matmul/sgemm block;
 *   - a single-row LayerNorm or product (layer_norm_*, matmul_d2d / matmul_dev / matvec_dev with
 *     rows == 1) may be held back until the next call of this library: when that call continues
 *     on its buffers (LayerNorm -> product, product -> GELU, product -> residual add, as in
 *     src/graph.c:3391-3476) the calls run as one launch that writes every buffer the separate
 *     calls write; any other call first launches what is held back.  Nothing observable through
 *     this interface changes, except that a held-back launch that fails is reported by the call
 *     that launches it, or by the next mynah_hip_sync.  MYNAH_HIP_FUSE=0 in the environment at
 *     open makes every call a launch of its own;
 *   - threads: a state, and every decoder, encoder and local frame created from it, serves one
 *     thread at a time.  Its stream, upload buffer, staging memory and captured graphs are shared
 *     by all its calls without locks, as in the reference's GPU backends, whose state belongs to
 *     the one engine thread (gpu/cuda/backend_cuda.cu has no lock).  Separate states are
 *     independent and may be used from separate threads.  The pointer returned by
 *     mynah_hip_upload is the state's one upload buffer: the next upload, host-pointer
 *     matmul/sgemm, matmul_to_dev or embed_gather reuses it.
 *
 * Section 1 mirrors, symbol for symbol, what src/backend.c declares for a GPU backend
 * (src/backend.c:72-135) so `#if defined(MYNAH_ENABLE_HIP)` blocks can bind it unchanged.
 * Section 2 fills the gap the single-stream seam leaves: weight-stationary batched twins and a
 * whole-step entry for B concurrent streams (the reference only batches on the CPU,
 * src/graph.c:3127-3284, src/qmat.c:820-888).
 */
#ifndef MYNAH_HIP_H
#define MYNAH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Section 1 -- the reference seam (src/backend.h)
 * ------------------------------------------------------------------------------------------ */

/* src/backend.h:10-25 */
typedef int (*mynah_backend_matmul_fn)(void *, const float *, float *, size_t, size_t, size_t,
                                       const float *, const float *, char *, size_t);
typedef void (*mynah_backend_close_fn)(void *);
typedef int (*mynah_backend_self_test_fn)(void *, char *, size_t);
typedef int (*mynah_backend_sgemm_fn)(void *, int trans_a, int trans_b, size_t m, size_t n, size_t k,
                                      float alpha, const float *a, size_t lda, const float *b, size_t ldb,
                                      float beta, float *c, size_t ldc, char *, size_t);

/* Counterpart of mynah_backend_cuda_open (src/backend.c:106-109, gpu/cuda/backend_cuda.cu:540-565).
 * matmul: out[rows,ow] = in[rows,iw] W[ow,iw]^T + bias, all HOST pointers, synchronous
 *         (src/backend.h:32-35).  rows <= 16 takes the quantized matvec selected by MYNAH_QUANT,
 *         like mynah_qmat_linear_resolved (src/qmat.c:768-818); more rows use the f32 GEMM.
 * sgemm:  row-major C = alpha op(A) op(B) + beta C on HOST pointers (src/backend.h:15-25).
 * self_test: the matmul/sgemm KATs of gpu/cuda/backend_cuda.cu:514-529 and the resident-op KATs
 *         of gpu/metal/backend_metal_ops.m:1038-1107, codec operators included. */
int mynah_backend_hip_open(void **state, mynah_backend_matmul_fn *matmul, mynah_backend_sgemm_fn *sgemm,
                           mynah_backend_close_fn *close, mynah_backend_self_test_fn *self_test,
                           char *error, size_t error_capacity);

/* src/backend.h:181-186 */
int mynah_hip_dev_alloc(void *state, size_t n, float **dev_ptr, char *error, size_t error_capacity);
void mynah_hip_dev_free(void *state, float *dev_ptr);
/* src/backend.h:156-163.  h2d is asynchronous on the backend stream (the source is staged through
 * pinned memory before the call returns); d2h synchronises first. */
int mynah_hip_h2d(void *state, const float *host, float *dev_ptr, size_t n, char *error, size_t error_capacity);
int mynah_hip_d2h(void *state, const float *dev_ptr, float *host, size_t n, char *error, size_t error_capacity);
/* src/backend.h:78-85: upload returns a pointer into backend-owned scratch, valid until the next upload. */
int mynah_hip_upload(void *state, const float *host, size_t n, float **dev_ptr, char *error, size_t error_capacity);
int mynah_hip_download(void *state, const float *dev_ptr, float *host, size_t n, char *error, size_t error_capacity);
/* src/backend.h:86-93 */
int mynah_hip_sync(void *state, char *error, size_t error_capacity);
int mynah_hip_batch_begin(void *state, char *error, size_t error_capacity);

/* src/backend.h:53-58: in-place resident ops, no copy, no sync.
 * layer_norm_inplace: gain only, eps 1e-5 (src/graph.c:147-150). */
int mynah_hip_gelu_inplace(void *state, float *dev_data, size_t n, char *error, size_t error_capacity);
int mynah_hip_residual_inplace(void *state, float *dev_out, const float *dev_in, size_t n, char *error, size_t error_capacity);
int mynah_hip_layer_norm_inplace(void *state, const float *dev_in, float *dev_out, const float *gain,
                                 size_t rows, size_t width, char *error, size_t error_capacity);
/* out[rows,ow] = in[rows,iw] W[ow,iw]^T + bias; dev in/out, HOST W/bias.  rows <= 16 runs the
 * weight-stationary quantized matvec (activation quantisation fused), else the f32 GEMM. */
int mynah_hip_matmul_d2d(void *state, const float *dev_in, float *dev_out, size_t rows, size_t iw, size_t ow,
                         const float *weight, const float *bias, char *error, size_t error_capacity);
/* HOST input, dev output (src/backend.h:57). */
int mynah_hip_matmul_to_dev(void *state, const float *host_in, float *dev_out, size_t rows, size_t iw, size_t ow,
                            const float *weight, const float *bias, char *error, size_t error_capacity);
/* src/backend.h:66-71 */
int mynah_hip_matvec_dev(void *state, const float *dev_in, float *dev_out, size_t K, size_t N,
                         const float *weight, const float *bias, char *error, size_t error_capacity);
/* src/backend.h:95-128: device-buffer forms. layer_norm_dev honours `bias` (may be NULL). */
int mynah_hip_matmul_dev(void *state, const float *dev_in, float *dev_out, size_t rows, size_t iw, size_t ow,
                         const float *weight, const float *bias, char *error, size_t error_capacity);
int mynah_hip_sgemm_dev(void *state, int trans_a, int trans_b, size_t m, size_t n, size_t k, float alpha,
                        const float *dev_a, size_t lda, const float *dev_b, size_t ldb, float beta,
                        float *dev_c, size_t ldc, char *error, size_t error_capacity);
int mynah_hip_gelu_dev(void *state, float *dev_data, size_t n, char *error, size_t error_capacity);
int mynah_hip_layer_norm_dev(void *state, const float *dev_in, float *dev_out, const float *gain,
                             const float *bias, size_t rows, size_t width, char *error, size_t error_capacity);
int mynah_hip_softmax_dev(void *state, float *dev_data, size_t rows, size_t cols, size_t valid,
                          char *error, size_t error_capacity);
int mynah_hip_residual_add_dev(void *state, float *dev_out, const float *dev_in, size_t n,
                               char *error, size_t error_capacity);

/* src/backend.h:135-154.  Self: dev_qkv = [q | k | v] (3 * heads * head_width floats); the k and v
 * parts are first stored at row `position` of the per-layer caches (rows are `cache_stride` floats
 * apart), then rows [0, valid) are attended.  Cross: read-only caches.  heads * head_width may be
 * anything up to 4096, head_width <= 1024. */
int mynah_hip_self_attention_dev(void *state, const float *dev_qkv, float *dev_k_cache, float *dev_v_cache,
                                 size_t position, size_t cache_stride, size_t valid, size_t heads,
                                 size_t head_width, float scale, float *dev_out,
                                 char *error, size_t error_capacity);
int mynah_hip_cross_attention_dev(void *state, const float *dev_q, const float *dev_k_cache,
                                  const float *dev_v_cache, size_t valid, size_t cache_stride, size_t heads,
                                  size_t head_width, float scale, float *dev_out,
                                  char *error, size_t error_capacity);

/* No counterpart in the reference.  mynah_hip_self_attention_dev for callers that cannot allocate (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc): same arguments, same result bit for bit, but the split-L
 * partials live in a fixed array inside the library (about 1 MiB per GPU, held until the process ends) and the call makes
 * no hipMalloc, hipFree or memset node.  It fails with "exceeds the allocation-free workspace" when
 * heads * (ceil(valid / 64) + 1) * (head_width + 4) floats exceed 2^18 (12 heads of 64: valid up to 20,480 rows), or heads
 * exceed 4096.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two states, two streams) race. */
int mynah_hip_self_attention_dev_noalloc(void *state, const float *dev_qkv, float *dev_k_cache, float *dev_v_cache,
                                         size_t position, size_t cache_stride, size_t valid, size_t heads,
                                         size_t head_width, float scale, float *dev_out,
                                         char *error, size_t error_capacity);

/* src/backend.h:165-179.  clip: clamp to [-1, 1], NaN -> 0 (gpu/metal/backend_metal_ops.m:1090-1101).
 * argmax: candidates i < codebook_size plus eos_id iff allow_eos; strict > from -FLT_MAX, the first
 * index wins ties (src/backend.c:825-847).  Synchronises and returns one scalar. */
int mynah_hip_copy_dev(void *state, float *dev_dst, const float *dev_src, size_t n, char *error, size_t error_capacity);
int mynah_hip_scale_dev(void *state, float *dev_data, size_t n, float scale, char *error, size_t error_capacity);
int mynah_hip_clip_dev(void *state, float *dev_data, size_t n, char *error, size_t error_capacity);
int mynah_hip_argmax_dev(void *state, const float *dev_logits, size_t vocab, size_t codebook_size, size_t eos_id,
                         int allow_eos, unsigned *argmax, char *error, size_t error_capacity);

/* Codec operators of the resident NanoCodec decode (src/backend.h:60-61,129-133; called from src/graph.c:2463-2490,
 * 2553-2616), rows of layout [channels, length] in device memory, weight / bias / alpha HOST pointers.  A backend
 * that registers attention is also given the codec (src/graph.c:2514-2518), which fails hard without these
 * (:2552-2555): with them MYNAH_METAL_CPU_CODEC is not needed.
 * conv1d: causal, dilated; weight [out, in, kernel]; bias may be NULL (conv1d_causal, src/graph.c:2010-2160); runs
 *   on the f32 matrix cores; kernel <= 16, (kernel - 1) * dilation <= 128.
 * conv_transpose_dev: grouped, weight [in, out / groups, kernel], output trimmed to output_length; bit-identical to
 *   the reference's scalar loop (convt_channel, src/graph.c:2179-2198).
 * snake_dev: in place; rows below snake_channels get x + sin(a x)^2 / (a + 1e-9), the rest a leaky ReLU of slope 0.01
 *   (snake_row, src/backend.c:643-658). */
int mynah_hip_conv1d(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels, int length,
                     int kernel, int dilation, const float *weight, const float *bias, char *error, size_t error_capacity);
int mynah_hip_conv_transpose_dev(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels,
                                 int length, int output_length, int kernel, int stride, int groups, const float *weight,
                                 const float *bias, char *error, size_t error_capacity);
int mynah_hip_snake_dev(void *state, float *dev_data, const float *alpha, size_t channels, size_t length,
                        size_t snake_channels, char *error, size_t error_capacity);

/* The seam's remaining optional slots (src/backend.h:59,62-64; src/backend.c:60,63-65; CUDA: gpu/cuda/backend_cuda.cu:708-735,
 * :813-851, :874-950).  graph.c calls none of them today and the wrappers fall back when a slot is NULL (src/backend.c:900-952);
 * they exist so that the HIP block of backend.c can fill every field the CUDA block fills.
 * im2col: device rows [in_channels, length] -> columns [in_channels * kernel, length], columns[(i*kernel + k)*length + l] =
 *   input[i*length + l - (kernel-1-k)*dilation] or 0 in front of the row; no synchronisation.
 * gelu_host / gelu_host_f64: HOST data in place: upload, tanh-GELU (f32 as everywhere else / evaluated in double and rounded
 *   once), download, synchronise.
 * matmul_graph: the host-pointer matmul (same arguments and result as the `matmul` of mynah_backend_hip_open). */
int mynah_hip_im2col(void *state, const float *dev_input, float *dev_columns, int in_channels, int length, int kernel, int dilation,
                     char *error, size_t error_capacity);
int mynah_hip_gelu_host(void *state, float *data, size_t n, char *error, size_t error_capacity);
int mynah_hip_gelu_host_f64(void *state, float *data, size_t n, char *error, size_t error_capacity);
int mynah_hip_matmul_graph(void *state, const float *input, float *output, size_t rows, size_t input_width, size_t output_width,
                           const float *weight, const float *bias, char *error, size_t error_capacity);

/* The residual layer of the codec (res_layer_device, src/graph.c:2423-2498) spends a fifth of its time in the element-wise
 * operators between its convolutions: copy_dev, snake_dev, residual_inplace, scale_dev, each a pass over the rows in
 * device memory.  conv1d_fused is conv1d followed, value by value before the store, by the arithmetic of those operators
 * in this fixed order (every step optional), so that a sequence of fused calls gives the bits of the sequence it replaces:
 *   v  = conv + bias
 *   v  = dev_residual[i] + v          residual_inplace (src/backend.h:86-88); dev_residual may be dev_output
 *   v  = dev_residual2[i] + v         a second one
 *   v  = v * scale                    scale_dev, when scale != 1
 *   activate == 0:                    dev_output[i] = v
 *   activate != 0, dev_activated 0:   dev_output[i] = half-snake of v with the alpha of v's output channel (snake_dev on the result)
 *   activate != 0, dev_activated set: dev_output[i] = v and dev_activated[i] = half-snake of v (the copy_dev + snake_dev
 *                                     that prepare the next convolution's input while the plain value stays the residual)
 * snake_alpha is a host pointer like every weight.  snake_copy_dev is snake_dev from one row set into another (copy_dev +
 * snake_dev).  Neither has a counterpart in the reference's seam: they are for an engine whose residual layer calls them instead. */
typedef struct mynah_hip_conv1d_extra {
    const float *dev_residual;
    const float *dev_residual2;
    float scale;
    int activate;
    const float *snake_alpha;
    size_t snake_channels;
    float *dev_activated;
} mynah_hip_conv1d_extra;
int mynah_hip_conv1d_fused(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels, int length,
                           int kernel, int dilation, const float *weight, const float *bias, const mynah_hip_conv1d_extra *extra,
                           char *error, size_t error_capacity);
int mynah_hip_snake_copy_dev(void *state, const float *dev_input, float *dev_output, const float *alpha, size_t channels,
                             size_t length, size_t snake_channels, char *error, size_t error_capacity);
/* Up to four conv1d_fused calls of one shape (in_channels, out_channels, length) in ONE launch -- the three branches of a
 * residual layer (res_layer_device, src/graph.c:2423-2498, walks them one after the other) at the same block and position.
 * Each member has its own rows, weights, taps, dilation and epilogue and gets the values its own conv1d_fused call would
 * give, bit for bit; the members run at the same time, so no member may write rows that another reads or writes (refused).
 * With 3, 7 or 11 taps in every member the launch is shared; other tap counts run the members one after the other.
 * No counterpart in the reference's seam. */
typedef struct mynah_hip_conv1d_item {
    const float *dev_input;
    float *dev_output;
    int kernel, dilation;
    const float *weight, *bias;   /* host pointers, cached like every weight */
    mynah_hip_conv1d_extra extra;
} mynah_hip_conv1d_item;
int mynah_hip_conv1d_fused_batch(void *state, const mynah_hip_conv1d_item *items, size_t count, int in_channels, int out_channels,
                                 int length, char *error, size_t error_capacity);
/* One pass over up to four row sets [channels, length]: v = ((in0 + in1) + in2 ...) * scale, then every output j gets v, or
 * half-snake(v) with alphas[j] when that is non-null (host pointer, cached; alphas itself may be NULL) -- the arithmetic of
 * residual_inplace per addend, scale_dev and snake_dev / snake_copy_dev in that order, value by value.  An output may be one
 * of the inputs (a value is read before it is written); no output may be named twice.  It serves the residual layer with its
 * branches side by side: one input and three activated outputs at the layer's start, three branch results summed, scaled
 * by a third and activated at its end.  No counterpart in the reference's seam. */
int mynah_hip_rows_combine_dev(void *state, const float *const *dev_inputs, size_t inputs, float scale, float *const *dev_outputs,
                               const float *const *alphas, size_t outputs, size_t channels, size_t length, size_t snake_channels,
                               char *error, size_t error_capacity);

/* ------------------------------------------------------------------------------------------
 * Section 2 -- what the single-stream seam lacks
 * ------------------------------------------------------------------------------------------ */

#define MYNAH_HIP_MAX_BATCH 16   /* MYNAH_MAX_BATCH, src/graph.c:12 */

/* Weight storage, the strings of MYNAH_QUANT (src/qmat.c:571-576); numeric values are QMAT_* (src/qmat.c:36). */
enum { MYNAH_HIP_F32 = 0, MYNAH_HIP_INT8 = 1, MYNAH_HIP_INT4 = 2, MYNAH_HIP_F16 = 3 };
/* Quantiser arithmetic: 0 evaluates src/qmat.c:39-113 as written (IEEE, compiler independent);
 * 1 reproduces what the reference's stock build (gcc -O3 -ffast-math, Makefile:5) stores:
 * scale = amax * f32(1/127) and inv = 127/amax (int4: amax * f32(1/7), 6.9999995f/amax). */
enum { MYNAH_HIP_ARITH_STRICT = 0, MYNAH_HIP_ARITH_STOCK = 1 };

/* Selects the storage used for weights first seen AFTER the call (already cached weights keep
 * theirs).  The open call initialises it from MYNAH_QUANT ("int8" | "int4" | "f16", else f32) and
 * MYNAH_QUANT_ARITH ("stock", else strict).  int4 falls back to f32 when iw % 32 != 0
 * (src/qmat.c:630); quantised storage is used only for rows <= 16 and iw <= 8192 (src/qmat.c:32-33). */
int mynah_hip_set_quant(void *state, int qtype, int arith, char *error, size_t error_capacity);

/* Host-side load-time conversion used by the weight cache, exposed so callers (and tests) can
 * check or pre-pack bytes.  Restates quantize_weight_int8/int4 (src/qmat.c:39-91) and the
 * (__fp16) cast (src/qmat.c:655, IEEE round-to-nearest-even). */
void mynah_hip_quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales, int arith);
int mynah_hip_quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales, int arith);
void mynah_hip_convert_weight_f16(const float *w, size_t count, uint16_t *out);

/* Weight-stationary batched linear: `batch` single-row activations of different streams, one pass
 * over the weight.  Twin of mynah_qmat_linear_batched (src/qmat.h:53-58, src/qmat.c:820-888):
 * dev_in[b] / dev_out[b] are scattered device rows; every out[b] is bit-identical to the same row
 * run alone (src/qmat.c:1107-1179).  batch <= MYNAH_HIP_MAX_BATCH. */
int mynah_hip_matmul_d2d_batched(void *state, const float *const *dev_in, float *const *dev_out, size_t batch,
                                 size_t iw, size_t ow, const float *weight, const float *bias,
                                 char *error, size_t error_capacity);

/* Parity probe for the quantised matvec: like mynah_hip_matmul_d2d with rows == 1, and additionally
 * stores the int8 activation (iw bytes), its scale (1 float) and the int32 accumulators
 * (int8: ow values; int4: ow * iw/32 per-group values) to the given device buffers (any may be NULL). */
int mynah_hip_matmul_d2d_probe(void *state, const float *dev_in, float *dev_out, size_t iw, size_t ow,
                               const float *weight, const float *bias, int8_t *dev_qx, float *dev_sx,
                               int32_t *dev_acc, char *error, size_t error_capacity);

/* Batched single-token attention.  Arrays have `batch` entries and live on the HOST; the caches are
 * device pointers.  Same per-stream contract as the single-stream calls above; every stream's output
 * is bit-identical to that stream run alone. */
int mynah_hip_self_attention_dev_batched(void *state, const float *const *dev_qkv, float *const *dev_k_cache,
                                         float *const *dev_v_cache, const size_t *position, size_t cache_stride,
                                         const size_t *valid, size_t batch, size_t heads, size_t head_width,
                                         float scale, float *const *dev_out, char *error, size_t error_capacity);
int mynah_hip_cross_attention_dev_batched(void *state, const float *const *dev_q, const float *const *dev_k_cache,
                                          const float *const *dev_v_cache, const size_t *valid, size_t cache_stride,
                                          size_t batch, size_t heads, size_t head_width, float scale,
                                          float *const *dev_out, char *error, size_t error_capacity);

/* Cross-attention K/V of an utterance for every decoder layer, from encoder memory that is resident on the device
 * (decoder_cache_init, src/graph.c:3002-3028): per layer LayerNorm(memory; norm_xattn_memory) -> kv_net product -> K half
 * and V half, written to dev_cross_k / dev_cross_v as [layers, memory_length, xattn_width] (the layout the decoder slots
 * take).  norm_gain / norm_bias / kv_w are [layers] arrays of HOST pointers (kv_w[l]: [2 * xattn_width, width], K rows
 * first; norm_bias may be NULL).  Asynchronous on the backend stream. */
int mynah_hip_cross_kv_dev(void *state, const float *dev_memory, size_t memory_length, size_t width, size_t layers,
                           const float *const *norm_gain, const float *const *norm_bias, const float *const *kv_w,
                           size_t xattn_width, float *dev_cross_k, float *dev_cross_v, char *error, size_t error_capacity);

/* Embedding gather (src/graph.c:729-737 text rows, :764-804 audio frame): out[t,:] = sum over `tables`
 * of table_j[ids[t*tables + j], :] scaled by `scale` (1 for text, 1/16 for the stacked audio frame),
 * optionally + position[t0 + t, :] (src/graph.c:649-651, :3156-3157).  f32 tables are HOST pointers
 * cached on the device; ids are a HOST array.  With one table and scale 1 the row is copied bit for bit. */
int mynah_hip_embed_gather(void *state, const float *const *tables, const size_t *table_rows, size_t table_count,
                           const int32_t *ids, size_t tokens, size_t width, float scale, const float *position,
                           size_t position_offset, float *dev_out, char *error, size_t error_capacity);

/* ---- whole decode step ------------------------------------------------------------------- */

/* Pre-resolved decoder weights: HOST pointers, the fields of decoder_layer_resolved / decoder_cache
 * (src/graph.c:2795-2861) plus the generalisations the synthetic configurations need (LayerNorm
 * bias, several cross-attention heads).  Per-layer tensors are arrays of `layers` pointers. */
typedef struct {
    size_t layers, width, heads, head_width, ffn_width;
    size_t cross_heads, cross_head_width;   /* xattn_width = cross_heads * cross_head_width; 0 heads = no cross sublayer */
    size_t capacity;                        /* rows of each self K/V cache per layer */
    const float *const *norm_self;          /* [layers] -> [width] gain */
    const float *const *norm_self_bias;     /* NULL, or [layers] -> [width] (NULL entries allowed) */
    const float *const *norm_xattn_query;
    const float *const *norm_xattn_query_bias;
    const float *const *norm_pos_ff;
    const float *const *norm_pos_ff_bias;
    const float *const *qkv_w;              /* [3*width, width] */
    const float *const *o_self_w;           /* [width, width] */
    const float *const *q_cross_w;          /* [xattn_width, width] */
    const float *const *o_cross_w;          /* [width, xattn_width] */
    const float *const *ffn_up_w;           /* [ffn_width, width] */
    const float *const *ffn_down_w;         /* [width, ffn_width] */
    const float *norm_out;                  /* [width] gain, NULL = no final norm */
    const float *norm_out_bias;             /* NULL or [width] */
    const float *position;                  /* [capacity, width] position embeddings, or NULL */
} mynah_hip_decoder_desc;

typedef struct mynah_hip_decoder mynah_hip_decoder;

/* One live stream of a batched step: the device-side fields of decoder_cache (src/graph.c:2853-2857). */
typedef struct {
    float *dev_self_k;          /* [layers, capacity, width] */
    float *dev_self_v;
    const float *dev_cross_k;   /* [layers, memory_length, xattn_width] */
    const float *dev_cross_v;
    size_t length;              /* tokens already cached; this step appends row `length` */
    size_t memory_length;
    const float *dev_input;     /* [width] the embedded frame, before the position add */
    float *dev_output;          /* [width] after the final norm */
} mynah_hip_decoder_slot;

/* Converts and caches every weight under the current quant setting and builds the resident step. */
int mynah_hip_decoder_create(void *state, const mynah_hip_decoder_desc *desc, mynah_hip_decoder **out,
                             char *error, size_t error_capacity);
void mynah_hip_decoder_destroy(void *state, mynah_hip_decoder *decoder);

/* One decode step for `batch` streams: the fused order of decoder_step_batch (src/graph.c:3127-3284)
 * -- per layer LN -> QKV -> self-attention + KV append -> O -> +res -> LN -> Q -> cross-attention ->
 * O -> +res -> LN -> up -> GELU -> down -> +res, final LN -- with one pass over each weight for all
 * streams.  Enqueues and returns (no sync).  Fails with "decoder cache capacity exceeded" when a
 * slot's length >= capacity (src/graph.c:3152-3155) and with "decoder batch exceeds
 * MYNAH_MAX_BATCH" above 16 (:3133-3136).  Slot lengths are read, not advanced. */
int mynah_hip_decoder_step(void *state, mynah_hip_decoder *decoder, const mynah_hip_decoder_slot *slots,
                           size_t batch, char *error, size_t error_capacity);

/* The decoder head's token choice when no local transformer follows (slot_advance, src/graph.c:3873-3905; the rule of
 * mynah_matvec_argmax_f32, src/kernels.c:116-139, whose threaded form is src/qmat.c:500-536): for each of `batch` slots and each of
 * `streams` stacked streams the first maximum of final_proj's logits W[streams * vocab, width] hidden + bias among the codes
 * (candidate < codebook_size) and, unless forbid_eos[slot], eos_id; strict > from -FLT_MAX, 0 when nothing beats it.  HOST
 * outputs as mynah_hip_local_frame's: values / stored [batch * streams] (stored = the value if it is a code, else 0), saw_eos
 * [batch], eos_frame [batch] (stream / codebook_count of the earliest EOS, SIZE_MAX = none).  f32 arithmetic on the stored
 * weights (HOST pointers, cached on the device); the logits never leave the device.  One synchronisation for all slots. */
int mynah_hip_head_argmax(void *state, const float *const *dev_hidden, size_t batch, size_t width, const float *weight,
                          const float *bias, size_t streams, size_t vocab, size_t codebook_size, size_t eos_id,
                          size_t codebook_count, const int *forbid_eos, unsigned *values, unsigned *stored, int *saw_eos,
                          size_t *eos_frame, char *error, size_t error_capacity);

/* Output head for the step's final-normed rows: logits[b] = W[rows,width] hidden[b] + bias, then a
 * softmax over each consecutive group of `vocab` logits (mynah_softmax_f32, src/kernels.c:391-420).
 * dev_probs[b] may be NULL (logits only).  W/bias HOST pointers. */
int mynah_hip_output_head(void *state, const float *const *dev_hidden, size_t batch, size_t width,
                          const float *weight, const float *bias, size_t rows, size_t vocab,
                          float *const *dev_logits, float *const *dev_probs, char *error, size_t error_capacity);

/* mynah_hip_decoder_step followed by mynah_hip_output_head on the slots' outputs, as one call: what slot_advance does with every
 * step's rows (src/graph.c:3873-3905 takes final_proj of the step's output).  Same results in the same places -- every slot's
 * dev_output holds the final-normed row, dev_logits / dev_probs what the head gives -- within the head's own tolerance: where
 * the step runs as one group of stage kernels with a final LayerNorm (up to 8 streams, head shapes the fused matvec takes),
 * the LayerNorm is the head product's prologue instead of a kernel of its own, one dependent launch less per step; the
 * normalised rows are the bits of the separate form, and the head's launches are nodes of the step's captured graph (captured
 * again when weight, bias, dev_logits or dev_probs differ from the step before: keep them stable).  Elsewhere the two calls run
 * one after the other.  A step of this
 * entry whose bounded wait gives up is reported at the next synchronising call and not repeated (its rows have been consumed). */
int mynah_hip_decoder_step_head(void *state, mynah_hip_decoder *decoder, const mynah_hip_decoder_slot *slots, size_t batch,
                                const float *weight, const float *bias, size_t rows, size_t vocab, float *const *dev_logits,
                                float *const *dev_probs, char *error, size_t error_capacity);

/* Measurement helper (no counterpart in the reference): enqueue one stage of the step -- all layers, as its own
 * captured graph, with the slot table of the last mynah_hip_decoder_step of this batch size -- so that a caller can
 * time that kernel alone in the step's own setting between mynah_hip_timer_begin / _end.  Overwrites the decoder's
 * workspaces like a step does. */
enum {
    MYNAH_HIP_STAGE_SELF_ATTENTION = 0,   /* LN + Q/K/V rows + KV append + self-attention partials */
    MYNAH_HIP_STAGE_SELF_OUT = 1,         /* fold + O matvec + residual */
    MYNAH_HIP_STAGE_CROSS_ATTENTION = 2,  /* LN + Q rows + cross-attention partials */
    MYNAH_HIP_STAGE_CROSS_OUT = 3,        /* fold + O matvec + residual */
    MYNAH_HIP_STAGE_FFN_UP = 4,           /* LN + up matvec + GELU */
    MYNAH_HIP_STAGE_FFN_DOWN = 5,         /* down matvec + residual */
    MYNAH_HIP_STAGE_COUNT = 6
};
int mynah_hip_decoder_stage_enqueue(void *state, mynah_hip_decoder *decoder, size_t batch, int stage,
                                    char *error, size_t error_capacity);
/* Parity probe for the whole step (no counterpart in the reference): one step of ONE or TWO streams as plain launches,
 * like mynah_hip_decoder_step, which also stores, for stream 0, the int8 activation vector and the activation scale the
 * device formed at each of a layer's six projections (quantize_act_int8, src/qmat.c:94-113), in the order qkv, o_self,
 * q_cross, o_cross, ffn_up, ffn_down: dev_qx [layers][6][ffn_width] bytes (a projection's first k bytes are used),
 * dev_sx [layers][6] floats.  A CPU restatement fed these integers instead of its own reproduces the step to the f32
 * tolerance, which is how the tests separate arithmetic from the occasional int8 activation that a last-bit LayerNorm
 * difference moves across a rounding boundary.  int8 / int4 weights and 64-wide heads only. */
int mynah_hip_decoder_step_probe(void *state, mynah_hip_decoder *decoder, const mynah_hip_decoder_slot *slots, size_t batch,
                                 int8_t *dev_qx, float *dev_sx, char *error, size_t error_capacity);

/* ---- local-transformer frame ---------------------------------------------------------------- */

/* The per-frame token loop of sample_local_frame_batch (src/graph.c:1374-1656): for each of `streams` codebook
 * positions one step of the local stack (local_step_batch, :1234-1343 -- a decoder stack without cross attention
 * and without final norm, its KV cache restarting at 0 every frame), the width -> vocab projection of that position
 * (:1536-1547, quantised like every other matvec), the token choice (:1548-1616) and the embedding of the chosen
 * token as the next position's input (:1629-1652).  Everything stays on the device; the host sees the tokens once
 * per frame instead of once per position. */
typedef struct {
    size_t streams;                          /* positions per frame (dep_q * stack_factor; 16) */
    size_t vocab;                            /* projection rows (<= 8192) */
    size_t codebook_size;                    /* candidates [0, codebook_size) are codes */
    size_t eos_id;                           /* the one special token that may be allowed besides the codes */
    size_t codebook_count;                   /* eos_frame = position / codebook_count (src/graph.c:1620) */
    const float *const *projection_w;        /* [streams] -> HOST f32 [vocab, width] */
    const float *const *projection_bias;     /* NULL, or [streams] -> HOST f32 [vocab] (NULL entries allowed) */
    const float *const *audio_table;         /* [streams] -> HOST f32 [vocab, width]: input row of the next position */
} mynah_hip_local_desc;

/* One live utterance: the fields of local_batch_item (src/graph.c:1345-1372) the frame reads.  rng_state is the
 * xorshift64 state itself (the reference holds a pointer; NULL there means "greedy", which is topk <= 1 here) and is
 * advanced in place when the item samples.  forbid_eos is generated_raw_length < min_raw_length (:1504). */
typedef struct {
    const float *dev_decoder_last;   /* device [width]: the decoder's output row for this frame */
    float temperature;
    size_t topk;                     /* sampling needs temperature > 0 and topk > 1; min(topk, vocab) <= 256 then */
    uint64_t rng_state;
    int forbid_eos;
} mynah_hip_local_item;

typedef struct mynah_hip_local mynah_hip_local;

/* `stack` describes the local transformer's layers (cross_heads = 0, norm_out = NULL, capacity >= streams,
 * position = NULL or the local position table).  Converts and caches all weights; owns KV caches for
 * MYNAH_HIP_MAX_BATCH items. */
int mynah_hip_local_create(void *state, const mynah_hip_decoder_desc *stack, const mynah_hip_local_desc *desc,
                           mynah_hip_local **out, char *error, size_t error_capacity);
void mynah_hip_local_destroy(void *state, mynah_hip_local *local);

/* One frame for `batch` items.  HOST outputs: values[b*streams + s] = chosen token, stored[...] = the token if it
 * is a code else 0 (src/graph.c:1627), saw_eos[b], eos_frame[b] (SIZE_MAX = none).  dev_logits_copy (optional,
 * device f32 [batch, streams, vocab]) receives the masked logits every choice was made from.  Synchronous.
 * Fails with "local frame batch exceeds MYNAH_MAX_BATCH" (:1379-1382) and "local sampler scratch too small"
 * (:1416-1419; here: a sampling item's min(topk, vocab) above 256). */
int mynah_hip_local_frame(void *state, mynah_hip_local *local, mynah_hip_local_item *items, size_t batch,
                          unsigned *values, unsigned *stored, int *saw_eos, size_t *eos_frame,
                          float *dev_logits_copy, char *error, size_t error_capacity);

/* ---- text-encoder prefill (dense, MFMA) --------------------------------------------------- */

typedef struct {
    size_t layers, width, heads, head_width, ffn_width, vocab, max_positions;
    const float *tok_table;       /* HOST f32 [vocab, width]; stored as f16 on the device */
    const float *pos_table;       /* HOST f32 [max_positions, width]; stored as f16 */
    const float *const *qkv_w, *const *o_w, *const *up_w, *const *down_w;   /* [layers] HOST f32, stored f16 */
    const float *const *norm1, *const *norm1_bias, *const *norm2, *const *norm2_bias;
    const float *norm_out, *norm_out_bias;
    int causal;                   /* nonzero: query t attends to keys 0 .. t (src/graph.c:446-449); 0: every key */
    size_t ffn_kernel;            /* 0 or 1: plain FFN, up_w [ffn, width], down_w [width, ffn].  3: causal_conv_ffn
                                   * (src/graph.c:302-352), up_w [ffn, width, 3], down_w [width, ffn, 3] */
    int operands_f32;             /* nonzero: tables, weights and every product operand stay f32 -- transformer_stack's own
                                   * arithmetic (src/graph.c:634-711: f32 sgemm per head, f32 linears), to 1e-5 of the CPU.  The
                                   * accuracy form: the library's f32 operators one after the other, no graph, several times the
                                   * time of the f16 form.  0: f16 operands, f32 accumulation (2e-3) */
} mynah_hip_encoder_desc;
typedef struct mynah_hip_encoder mynah_hip_encoder;

int mynah_hip_encoder_create(void *state, const mynah_hip_encoder_desc *desc, mynah_hip_encoder **out,
                             char *error, size_t error_capacity);
void mynah_hip_encoder_destroy(void *state, mynah_hip_encoder *encoder);
/* ids: HOST int32 [tokens]; dev_embed_f16 (optional): [tokens,width] f16 bits of the gathered token rows;
 * dev_out: f32 [tokens,width].  Attention bidirectional or causal, FFN plain or the kernel-3 causal conv, as the
 * description says; pre-LayerNorm; f16 operands with f32 accumulation, or f32 operands (then dev_embed_f16 must be NULL). */
int mynah_hip_encoder_prefill(void *state, mynah_hip_encoder *encoder, const int32_t *ids, size_t tokens,
                              uint16_t *dev_embed_f16, float *dev_out, char *error, size_t error_capacity);

/* ---- measurement helpers ------------------------------------------------------------------ */

/* HIP events on the backend's own stream (a torch/other-runtime event would not see it).
 * timer_begin records, timer_end records + synchronises and returns elapsed milliseconds. */
int mynah_hip_timer_begin(void *state, char *error, size_t error_capacity);
int mynah_hip_timer_end(void *state, float *milliseconds, char *error, size_t error_capacity);
/* Streams `bytes` of backend-owned scratch through the chip (read+write) so that the last-level
 * cache holds none of the caller's data: used between timed iterations. */
int mynah_hip_flush_cache(void *state, size_t bytes, char *error, size_t error_capacity);
/* What one dependent stage costs on this device with the bytes taken out (no counterpart in the reference: a measurement
 * helper like the timers above).  Runs `nodes` kernel nodes as one captured graph on the backend's stream, `repeats` times:
 * every one of a node's `workgroups` workgroups reads the whole `floats`-long vector the node before it wrote (as a matvec
 * stage of the decode step reads its activation row, written by workgroups on every XCD), reduces it and writes its share
 * of the next vector.  *node_us = elapsed time (HIP events on the backend's stream) / (repeats * nodes).  chains > 1 (up
 * to 3) runs that many independent chains side by side, each on a stream of its own, forked from and joined to the
 * backend's stream once per repeat; *node_us is still elapsed / (repeats * nodes), so a value equal to the one-chain
 * figure means the chains overlap fully and `chains` times it that they do not overlap at all.  Synchronises. */
int mynah_hip_dependent_launch_probe(void *state, int nodes, int workgroups, int floats, int chains, int repeats, float *node_us,
                                     char *error, size_t error_capacity);
/* How mynah_hip_decoder_step runs: 0 = every stage kernel a launch of its own, 1 (default) = the step replayed as a
 * captured HIP graph, 2 = one persistent launch for the whole step where it applies (one or two streams, int8 / int4
 * weights, width 768 / FFN 3072 / 64-wide heads, attention units and row stages fitting the chip side by side), else as
 * 1.  All three give the same bits.  Form 2 waits inside the kernel for other workgroups' results; every such wait is
 * bounded (MYNAH_HIP_PERSIST_SPIN polls, default 2^20; a value that is not a number fails the open), and a step that gave
 * one up is repeated in form 0 by the next call that synchronises (mynah_hip_wait_fallbacks).  MYNAH_HIP_GRAPH in the environment at open sets the initial value. */
int mynah_hip_set_graph_mode(void *state, int enabled, char *error, size_t error_capacity);
/* Lanes of mynah_hip_decoder_step above two streams: the batch is cut into `lanes` groups (1..3) that step side by side,
 * each on a HIP stream of its own with rows and work tables of its own, forked from and joined to the backend's stream
 * by events (every lane replays a captured graph of its own: a chain of kernel nodes).  The reference serves up to MYNAH_MAX_BATCH streams in one pass over
 * each weight (src/qmat.c:820-888); here a lane is such a pass, and the lanes overlap each other's launch gaps.  A
 * stream's arithmetic does not depend on which streams share its lane, so every lane count gives the same bits.
 * 0 (default): chosen from the batch size.  MYNAH_HIP_LANES in the environment at open sets the initial value. */
int mynah_hip_set_step_lanes(void *state, int lanes, char *error, size_t error_capacity);
/* Free and total bytes of the backend's device (hipMemGetInfo); either pointer may be NULL.  Lets a caller, or a test,
 * check that a call it relies on not to allocate left the device's free memory where it was. */
int mynah_hip_device_memory(void *state, size_t *free_bytes, size_t *total_bytes, char *error, size_t error_capacity);
/* How often a resident step was run a second time because one of its workgroups had given up a bounded wait for another
 * one's result.  Two forms of mynah_hip_decoder_step wait inside a kernel: the persistent launch (graph mode 2) and, in
 * every mode, the attention launches of more than two streams, whose fold workgroups wait for the attending workgroups
 * of the same launch (they are numbered behind them and the device starts workgroups in index order, so the ones waited
 * for are running or done; the bound -- MYNAH_HIP_PERSIST_SPIN polls, default 2^20 -- is there for a device that does
 * otherwise, or is shared with other work).  A workgroup that gives up sets a host-visible word and leaves, so the launch
 * always drains.  The next call that synchronises finds the word and, when that step is the only one since the stream
 * was last idle and no other call has put work behind it, repeats it as plain launches in the form without such waits
 * (fold kernel, MYNAH_HIP_FOLD_IN_LAUNCH=0's form; the cache rows it appends are the ones the first run wrote to) and
 * returns its results -- the same bits, later.  So a step followed by mynah_hip_sync, mynah_hip_d2h or mynah_hip_download
 * never fails for this reason.  With several steps since the last synchronisation, or with work enqueued behind the step
 * (an output head, a local frame: it has read rows that meant nothing), the synchronising call fails with "gave up a
 * bounded wait" as before; a caller that wants the repeat there synchronises right after the step.  No counterpart in the
 * reference, whose CPU step cannot give up. */
size_t mynah_hip_wait_fallbacks(void *state);
/* Packed-weight file (the optional "pre-packed sidecar"; no counterpart in the reference, which converts every tensor at
 * its first use in every process, src/qmat.c:779-782).  export writes every converted weight the backend holds -- int8 /
 * int4 values and scales, f16 values -- to `path`; import reads such a file, and from then on a tensor whose shape,
 * storage type, quantiser arithmetic and content fingerprint (FNV-1a over its shape and 1,536 sampled f32 values) match an
 * entry is uploaded from the file instead of being converted.  Tensors the file does not hold are converted as always, so
 * a stale or partial file costs nothing but its reading.  *entries (may be NULL): entries written / read.
 * mynah_hip_weights_from_pack counts the weights taken from files.  MYNAH_HIP_PACK_VERIFY=1 at open: convert all the same
 * and fail the call that meets a difference. */
int mynah_hip_weights_export(void *state, const char *path, size_t *entries, char *error, size_t error_capacity);
int mynah_hip_weights_import(void *state, const char *path, size_t *entries, char *error, size_t error_capacity);
size_t mynah_hip_weights_from_pack(void *state);
/* Bytes of device memory held by the weight cache (packed weights + scales + vectors). */
size_t mynah_hip_cached_weight_bytes(void *state);

#ifdef __cplusplus
}
#endif
#endif
