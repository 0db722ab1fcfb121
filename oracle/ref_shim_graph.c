/* TEST INFRASTRUCTURE ONLY -- never linked into, loaded by, or timed as the product.
 *
 * Drives the reference's own batched decode step on synthetic weights, without a
 * model pack.  The reference engine source is NOT copied: the include below
 * resolves through -I<reference>/src (oracle/Makefile) and the object lives only
 * in oracle/_ref/.
 *
 * Reference functions reached through this shim (file:line in the reference tree):
 *   decoder_step_batch        src/graph.c:3127-3284  (B slots, weight-stationary projections)
 *   local_step_batch          src/graph.c:1234-1343  (the local transformer's batched step)
 *   layer_norm                src/graph.c:147-150    (gain only, eps 1e-5)
 *   transformer_stack         src/graph.c:634-711    (the text encoder's layer stack)
 *   softmax_row_inplace       src/graph.c:245-257
 *   batch_scratch_init        src/graph.c:121-144
 *   mynah_backend_open(CPU)   src/backend.c:367-475
 *   mynah_qmat_cache_new      src/qmat.c:567-591
 *
 * The shim fills a decoder_cache (src/graph.c:2813-2861) per slot by hand:
 * only plain-pointer fields are touched by decoder_step_batch.
 */
#include "graph.c"

typedef struct {
    size_t layers, width, heads, head_width, ffn, xw, capacity;
    /* per-layer tensors, concatenated over layers */
    const float *norm_self;   /* [layers, width] */
    const float *norm_xq;     /* [layers, width] */
    const float *norm_ff;     /* [layers, width] */
    const float *qkv_w;       /* [layers, 3*width, width] */
    const float *o_w;         /* [layers, width, width] */
    const float *qx_w;        /* [layers, xw, width] */
    const float *ox_w;        /* [layers, width, xw] */
    const float *up_w;        /* [layers, ffn, width] */
    const float *down_w;      /* [layers, width, ffn] */
    const float *norm_out;    /* [width] */
    const float *position;    /* [capacity, width] */
} ref_decoder_desc;

typedef struct {
    mynah_tts_model model;
    ref_decoder_desc desc;
    decoder_layer_resolved *resolved;
    decoder_cache caches[MYNAH_MAX_BATCH];
    batch_scratch scratch;
    size_t batch;
    /* the batched device step of the integration text (set up at its first use) */
    void *hip_batch;
    float *hip_in[MYNAH_MAX_BATCH], *hip_out[MYNAH_MAX_BATCH];
} ref_decoder;

void ref_decoder_free(ref_decoder *d) {
    if (d == NULL) return;
    for (size_t b = 0; b < MYNAH_MAX_BATCH; ++b) {
        decoder_cache *c = &d->caches[b];
        free(c->scratch_x); free(c->scratch_nrm); free(c->scratch_qkv); free(c->scratch_attn);
        free(c->scratch_proj); free(c->scratch_q_x); free(c->scratch_xctx);
        free(c->scratch_hidden); free(c->scratch_scores);
    }
    batch_scratch_free(&d->scratch);
    free(d->resolved);
    if (d->model.qcache != NULL) mynah_qmat_cache_free(d->model.qcache);
    if (d->model.backend != NULL) mynah_backend_close(d->model.backend);
    free(d);
}

/* qtype: 0 f32, 1 int8, 2 int4 (the reference's QMAT_* values, src/qmat.c:36). */
ref_decoder *ref_decoder_new(const ref_decoder_desc *desc, int qtype, size_t batch,
                             size_t max_memory_length) {
    if (batch == 0 || batch > MYNAH_MAX_BATCH) return NULL;
    ref_decoder *d = (ref_decoder *)calloc(1, sizeof(*d));
    if (d == NULL) return NULL;
    char error[256];
    d->desc = *desc;
    d->batch = batch;
    if (mynah_backend_open(MYNAH_TTS_DEVICE_CPU, &d->model.backend, error, sizeof error) != 0) goto fail;
    d->model.qcache = mynah_qmat_cache_new(qtype);
    if (d->model.qcache == NULL) goto fail;
    d->resolved = (decoder_layer_resolved *)calloc(desc->layers, sizeof(*d->resolved));
    if (d->resolved == NULL) goto fail;
    const size_t w = desc->width, f = desc->ffn, xw = desc->xw;
    for (size_t l = 0; l < desc->layers; ++l) {
        decoder_layer_resolved *r = &d->resolved[l];
        r->norm_self = desc->norm_self + l * w;
        r->norm_xattn_query = desc->norm_xq + l * w;
        r->norm_pos_ff = desc->norm_ff + l * w;
        r->qkv_w = desc->qkv_w + l * 3u * w * w;
        r->o_self_w = desc->o_w + l * w * w;
        r->q_cross_w = desc->qx_w + l * xw * w;
        r->o_cross_w = desc->ox_w + l * w * xw;
        r->ffn_up_w = desc->up_w + l * f * w;
        r->ffn_down_w = desc->down_w + l * w * f;
        snprintf(r->qkv, sizeof r->qkv, "synthetic.layer%zu.qkv", l);
        snprintf(r->o_self, sizeof r->o_self, "synthetic.layer%zu.o_self", l);
        snprintf(r->q_cross, sizeof r->q_cross, "synthetic.layer%zu.q_cross", l);
        snprintf(r->o_cross, sizeof r->o_cross, "synthetic.layer%zu.o_cross", l);
        snprintf(r->ffn_up, sizeof r->ffn_up, "synthetic.layer%zu.ffn_up", l);
        snprintf(r->ffn_down, sizeof r->ffn_down, "synthetic.layer%zu.ffn_down", l);
    }
    size_t score_len = desc->capacity > max_memory_length ? desc->capacity : max_memory_length;
    for (size_t b = 0; b < batch; ++b) {
        decoder_cache *c = &d->caches[b];
        c->layers = desc->layers; c->width = w; c->heads = desc->heads;
        c->head_width = desc->head_width; c->ffn_width = f; c->xattn_width = xw;
        c->capacity = desc->capacity;
        c->position = desc->position;
        c->resolved = d->resolved;
        c->norm_out = desc->norm_out;
        c->scratch_rows = 1;
        c->scratch_x = (float *)calloc(w, sizeof(float));
        c->scratch_nrm = (float *)calloc(w, sizeof(float));
        c->scratch_qkv = (float *)calloc(3u * w, sizeof(float));
        c->scratch_attn = (float *)calloc(w, sizeof(float));
        c->scratch_proj = (float *)calloc(w, sizeof(float));
        c->scratch_q_x = (float *)calloc(xw, sizeof(float));
        c->scratch_xctx = (float *)calloc(xw, sizeof(float));
        c->scratch_hidden = (float *)calloc(f, sizeof(float));
        c->scratch_scores = (float *)calloc(score_len + 1u, sizeof(float));
        if (!c->scratch_x || !c->scratch_nrm || !c->scratch_qkv || !c->scratch_attn || !c->scratch_proj ||
            !c->scratch_q_x || !c->scratch_xctx || !c->scratch_hidden || !c->scratch_scores) goto fail;
    }
    const size_t k_max = f > w ? f : w;
    if (batch_scratch_init(&d->scratch, batch, k_max > xw ? k_max : xw, error, sizeof error) != 0) goto fail;
    return d;
fail:
    ref_decoder_free(d);
    return NULL;
}

/* One batched step.  self_k/self_v[b]: [layers, capacity, width] (caller-owned, appended in
 * place at row lengths[b]); cross_k/cross_v[b]: [layers, memory_lengths[b], xw].
 * lengths[b] is advanced by one on success, exactly as the reference does (src/graph.c:3281). */
int ref_decoder_step(ref_decoder *d, float *const *self_k, float *const *self_v,
                     float *const *cross_k, float *const *cross_v,
                     size_t *lengths, const size_t *memory_lengths,
                     const float *const *inputs, float *const *outs,
                     char *error, size_t error_capacity) {
    decoder_cache *ptrs[MYNAH_MAX_BATCH];
    for (size_t b = 0; b < d->batch; ++b) {
        decoder_cache *c = &d->caches[b];
        c->self_k = self_k[b]; c->self_v = self_v[b];
        c->cross_k = cross_k[b]; c->cross_v = cross_v[b];
        c->length = lengths[b];
        c->memory_length = memory_lengths[b];
        ptrs[b] = c;
    }
    const int rc = decoder_step_batch(&d->model, ptrs, inputs, outs, d->batch,
                                      d->batch > 1u ? &d->scratch : NULL, error, error_capacity);
    for (size_t b = 0; b < d->batch; ++b) {
        decoder_cache *c = &d->caches[b];
        lengths[b] = c->length;
        c->self_k = c->self_v = c->cross_k = c->cross_v = NULL;
    }
    return rc;
}

void ref_layer_norm_gain(const float *input, float *output, size_t rows, size_t width, const float *gain) {
    layer_norm(input, output, rows, width, gain);
}

void ref_softmax_row_inplace(float *values, size_t length) { softmax_row_inplace(values, length); }

float ref_gelu_tanh(float x) { return gelu_tanh(x); }

/* ---- the local transformer's batched step (local_step_batch, src/graph.c:1234-1343) --------------------------
 * Same pattern: a local_cache (src/graph.c:810-851) and a local_workspace (:928-937) per slot filled by hand;
 * local_step_batch touches nothing else of the model but qcache and backend. */
typedef struct {
    size_t layers, width, heads, head_width, ffn, capacity;   /* layers <= 4 */
    const float *norm_self;   /* [layers, width] */
    const float *norm_ff;     /* [layers, width] */
    const float *qkv_w;       /* [layers, 3*width, width] */
    const float *o_w;         /* [layers, width, width] */
    const float *up_w;        /* [layers, ffn, width] */
    const float *down_w;      /* [layers, width, ffn] */
    const float *position;    /* [capacity, width] */
} ref_local_desc;

typedef struct {
    mynah_tts_model model;
    local_cache caches[MYNAH_MAX_BATCH];
    local_workspace workspaces[MYNAH_MAX_BATCH];
    batch_scratch scratch;
    size_t batch;
    void *hip_batch;                       /* the device frame of the integration text */
    float *hip_last[MYNAH_MAX_BATCH];
} ref_local;

void ref_local_free(ref_local *d) {
    if (d == NULL) return;
    for (size_t b = 0; b < MYNAH_MAX_BATCH; ++b) {
        local_workspace *w = &d->workspaces[b];
        free(w->x); free(w->nrm); free(w->qkv); free(w->attn); free(w->proj); free(w->hidden); free(w->scores);
        free(w->gelu_scratch);
    }
    batch_scratch_free(&d->scratch);
    if (d->model.qcache != NULL) mynah_qmat_cache_free(d->model.qcache);
    if (d->model.backend != NULL) mynah_backend_close(d->model.backend);
    free(d);
}

ref_local *ref_local_new(const ref_local_desc *desc, int qtype, size_t batch) {
    if (batch == 0 || batch > MYNAH_MAX_BATCH || desc->layers == 0 || desc->layers > 4) return NULL;
    ref_local *d = (ref_local *)calloc(1, sizeof(*d));
    if (d == NULL) return NULL;
    char error[256];
    d->batch = batch;
    if (mynah_backend_open(MYNAH_TTS_DEVICE_CPU, &d->model.backend, error, sizeof error) != 0) goto fail;
    d->model.qcache = mynah_qmat_cache_new(qtype);
    if (d->model.qcache == NULL) goto fail;
    const size_t w = desc->width, f = desc->ffn;
    for (size_t b = 0; b < batch; ++b) {
        local_cache *c = &d->caches[b];
        c->layers = desc->layers; c->width = w; c->heads = desc->heads; c->head_width = desc->head_width;
        c->ffn_width = f; c->capacity = desc->capacity; c->position = desc->position;
        for (size_t l = 0; l < desc->layers; ++l) {
            c->norm_self[l] = desc->norm_self + l * w;
            c->norm_ff[l] = desc->norm_ff + l * w;
            c->qkv_w[l] = desc->qkv_w + l * 3u * w * w;
            c->o_w[l] = desc->o_w + l * w * w;
            c->ffn_up_w[l] = desc->up_w + l * f * w;
            c->ffn_down_w[l] = desc->down_w + l * w * f;
            snprintf(c->qkv_name[l], sizeof c->qkv_name[l], "synthetic.local%zu.qkv", l);
            snprintf(c->o_name[l], sizeof c->o_name[l], "synthetic.local%zu.o", l);
            snprintf(c->ffn_up_name[l], sizeof c->ffn_up_name[l], "synthetic.local%zu.up", l);
            snprintf(c->ffn_down_name[l], sizeof c->ffn_down_name[l], "synthetic.local%zu.down", l);
        }
        local_workspace *ws = &d->workspaces[b];
        ws->x = (float *)calloc(w, sizeof(float));
        ws->nrm = (float *)calloc(w, sizeof(float));
        ws->qkv = (float *)calloc(3u * w, sizeof(float));
        ws->attn = (float *)calloc(w, sizeof(float));
        ws->proj = (float *)calloc(w, sizeof(float));
        ws->hidden = (float *)calloc(f, sizeof(float));
        ws->scores = (float *)calloc(desc->capacity + 1u, sizeof(float));
        ws->gelu_scratch = (float *)calloc(f, sizeof(float));
        if (!ws->x || !ws->nrm || !ws->qkv || !ws->attn || !ws->proj || !ws->hidden || !ws->scores || !ws->gelu_scratch) goto fail;
    }
    if (batch_scratch_init(&d->scratch, batch, f > w ? f : w, error, sizeof error) != 0) goto fail;
    return d;
fail:
    ref_local_free(d);
    return NULL;
}

/* One batched local step.  k/v[b]: [layers, capacity, width], appended in place at row lengths[b];
 * lengths[b] comes back advanced by one (src/graph.c:1340). */
int ref_local_step(ref_local *d, float *const *k, float *const *v, size_t *lengths, const float *const *inputs,
                   float *const *outs, char *error, size_t error_capacity) {
    local_cache *caches[MYNAH_MAX_BATCH];
    local_workspace *workspaces[MYNAH_MAX_BATCH];
    for (size_t b = 0; b < d->batch; ++b) {
        d->caches[b].k = k[b];
        d->caches[b].v = v[b];
        d->caches[b].length = lengths[b];
        caches[b] = &d->caches[b];
        workspaces[b] = &d->workspaces[b];
    }
    const int rc = local_step_batch(&d->model, caches, workspaces, inputs, outs, d->batch,
                                    d->batch > 1u ? &d->scratch : NULL, error, error_capacity);
    for (size_t b = 0; b < d->batch; ++b) {
        lengths[b] = d->caches[b].length;
        d->caches[b].k = d->caches[b].v = NULL;
    }
    return rc;
}

/* ---- codec operators (NanoCodec decoder) -------------------------------------------------------------------
 * Reference functions reached (file:line in the reference tree):
 *   conv1d_causal             src/graph.c:2010-2160  (causal dilated conv: im2col + sgemm on the CPU backend)
 *   conv_transpose_causal     src/graph.c:2200-2231  (grouped causal transposed conv, convt_channel :2179-2198)
 *   mynah_backend_snake_dev   src/backend.c:660-680  (CPU fallback snake_row :643-658)
 * The two convolutions look their weights up by name in a mynah_weights file; the caller passes the path of a
 * safetensors file it wrote itself (synthetic tensors). */
int ref_conv1d(const char *weights_path, const char *weight_name, const char *bias_name, const float *input, float *output,
               size_t in_channels, size_t out_channels, size_t length, size_t kernel, size_t dilation, char *error,
               size_t error_capacity) {
    mynah_weights *file = NULL;
    mynah_backend *backend = NULL;
    int rc = -1;
    if (mynah_weights_open(weights_path, &file, error, error_capacity) != 0) return -1;
    if (mynah_backend_open(MYNAH_TTS_DEVICE_CPU, &backend, error, error_capacity) == 0)
        rc = conv1d_causal(file, backend, NULL, weight_name, bias_name, input, output, in_channels, out_channels, length, kernel,
                           dilation, NULL, 0, NULL, error, error_capacity);
    if (backend != NULL) mynah_backend_close(backend);
    mynah_weights_close(file);
    return rc;
}

int ref_conv_transpose(const char *weights_path, const char *weight_name, const char *bias_name, const float *input, float *output,
                       size_t in_channels, size_t out_channels, size_t length, size_t kernel, size_t stride, size_t groups,
                       char *error, size_t error_capacity) {
    mynah_weights *file = NULL;
    if (mynah_weights_open(weights_path, &file, error, error_capacity) != 0) return -1;
    const int rc = conv_transpose_causal(file, weight_name, bias_name, input, output, in_channels, out_channels, length, kernel,
                                         stride, groups, NULL, error, error_capacity);
    mynah_weights_close(file);
    return rc;
}

int ref_snake(float *data, const float *alpha, size_t channels, size_t length, size_t snake_channels) {
    char error[256];
    mynah_backend *backend = NULL;
    if (mynah_backend_open(MYNAH_TTS_DEVICE_CPU, &backend, error, sizeof error) != 0) return -1;
    const int rc = mynah_backend_snake_dev(backend, data, alpha, channels, length, snake_channels, error, sizeof error);
    mynah_backend_close(backend);
    return rc;
}

/* ---- encoder stack --------------------------------------------------------------------------------------------
 * Reference function reached (file:line in the reference tree):
 *   transformer_stack         src/graph.c:634-711  (position add, per layer gain-only LayerNorm -> causal self_attention
 *                                                  :387-513 -> +res -> LayerNorm -> causal_conv_ffn :288-385 -> +res,
 *                                                  final norm) exactly as encode_text calls it (:738-740), on the CPU
 *                                                  backend, with `kernel` 1 (plain FFN) or 3 (the model's conv FFN).
 * Weights are looked up by name ("encoder....") in a safetensors file the caller wrote itself (synthetic tensors).
 * `states` are the gathered token rows [length, width]; `output` receives [length, width]. */
mynah_backend *ref_backend_open_hip(const char *library_path, char *error, size_t error_capacity);

/* hip_library NULL: the CPU backend; else the reference's backend struct filled with that library's entry points
 * (ref_shim_backend.c): every product of the stack is then a host-pointer `matmul` (the `linear` calls) or `sgemm`
 * (QK^T and PV per head, the unfolded conv FFN) of `length` rows through the seam. */
int ref_transformer_stack_on(const char *weights_path, const char *hip_library, size_t layers, size_t length, size_t width,
                             size_t ffn_width, size_t heads, size_t kernel, int apply_norm_out, const float *states, float *output,
                             char *error, size_t error_capacity) {
    mynah_weights *file = NULL;
    mynah_backend *backend = NULL;
    int rc = -1;
    if (error != NULL && error_capacity > 0) error[0] = '\0';
    if (mynah_weights_open(weights_path, &file, error, error_capacity) != 0) return -1;
    if (hip_library != NULL) backend = ref_backend_open_hip(hip_library, error, error_capacity);
    else if (mynah_backend_open(MYNAH_TTS_DEVICE_CPU, &backend, error, error_capacity) != 0) backend = NULL;
    if (backend != NULL) {
        float *copy = (float *)malloc(length * width * sizeof(float));   /* the function takes a non-const pointer */
        if (copy != NULL) {
            memcpy(copy, states, length * width * sizeof(float));
            rc = transformer_stack(file, backend, "encoder", layers, length, width, ffn_width, heads, kernel, 0, apply_norm_out,
                                   NULL, 0, copy, output, error, error_capacity);
            free(copy);
        }
    }
    if (backend != NULL) mynah_backend_close(backend);
    mynah_weights_close(file);
    return rc;
}

int ref_transformer_stack(const char *weights_path, size_t layers, size_t length, size_t width, size_t ffn_width,
                          size_t heads, size_t kernel, int apply_norm_out, const float *states, float *output, char *error,
                          size_t error_capacity) {
    return ref_transformer_stack_on(weights_path, NULL, layers, length, width, ffn_width, heads, kernel, apply_norm_out, states, output,
                                    error, error_capacity);
}

/* ---- the reference engine as a consumer of a device backend ---------------------------------------------------
 * Reference functions reached (file:line in the reference tree):
 *   decoder_run                 src/graph.c:3292-3654  count == 1 and a backend with device operators and attention:
 *                                                      the resident step, 18 seam calls per layer (:3368-3491)
 *   decoder_gpu_attention_init  src/graph.c:2901-2962  device K/V caches, uploaded from the host caches once
 *   local_step_device           src/graph.c:1106-1158  one resident local-transformer position
 * ref_backend_open_hip (ref_shim_backend.c) fills the reference's backend struct with the library's entry points. */
mynah_backend *ref_backend_open_hip(const char *library_path, char *error, size_t error_capacity);

static void ref_decoder_release_device(ref_decoder *d) {
    for (size_t b = 0; b < MYNAH_MAX_BATCH; ++b) {
        decoder_cache *c = &d->caches[b];
        if (c->dev_backend == NULL) continue;
        /* the device half of decoder_cache_free (src/graph.c:2881-2897); the host caches are the caller's */
        mynah_backend_dev_free(c->dev_backend, c->dev_nrm);
        mynah_backend_dev_free(c->dev_backend, c->dev_qkv);
        mynah_backend_dev_free(c->dev_backend, c->dev_attn);
        mynah_backend_dev_free(c->dev_backend, c->dev_proj);
        mynah_backend_dev_free(c->dev_backend, c->dev_qx);
        mynah_backend_dev_free(c->dev_backend, c->dev_xctx);
        mynah_backend_dev_free(c->dev_backend, c->dev_hidden);
        mynah_backend_dev_free(c->dev_backend, c->dev_x);
        if (c->dev_attention_allocated) {
            mynah_backend_dev_free(c->dev_backend, c->dev_self_k);
            mynah_backend_dev_free(c->dev_backend, c->dev_self_v);
            mynah_backend_dev_free(c->dev_backend, c->dev_cross_k);
            mynah_backend_dev_free(c->dev_backend, c->dev_cross_v);
        }
        c->dev_nrm = c->dev_qkv = c->dev_attn = c->dev_proj = c->dev_qx = c->dev_xctx = c->dev_hidden = c->dev_x = NULL;
        c->dev_self_k = c->dev_self_v = c->dev_cross_k = c->dev_cross_v = NULL;
        c->dev_allocated = 0;
        c->dev_attention_allocated = 0;
        c->dev_backend = NULL;
    }
}

/* Replaces the decoder's CPU backend by the library at library_path.  Device buffers of the previous backend are
 * released first. */
int ref_decoder_use_hip(ref_decoder *d, const char *library_path, char *error, size_t error_capacity) {
    mynah_backend *hip = ref_backend_open_hip(library_path, error, error_capacity);
    if (hip == NULL) return -1;
    ref_decoder_release_device(d);
    if (d->model.backend != NULL) mynah_backend_close(d->model.backend);
    d->model.backend = hip;
    return 0;
}

/* Call before ref_decoder_free when a device backend is attached (ref_decoder_free closes the backend). */
void ref_decoder_release(ref_decoder *d) { if (d != NULL) ref_decoder_release_device(d); }

/* The attached backend's own self-test through the struct's function pointer. */
int ref_backend_self_test(const mynah_backend *backend, char *error, size_t error_capacity);
int ref_decoder_self_test(ref_decoder *d, char *error, size_t error_capacity) {
    return ref_backend_self_test(d->model.backend, error, error_capacity);
}

/* One single-row decoder_run of slot `slot`.  On the first call of a slot the host caches (rows [0, *length) of
 * self_k/self_v, all of cross_k/cross_v) are what the engine uploads; afterwards the device caches are the live ones
 * and the pointers are only kept for the engine's bookkeeping.  *resident comes back 1 when the slot's device
 * buffers and device caches exist after the call, i.e. the resident path was taken. */
int ref_decoder_run_one(ref_decoder *d, size_t slot, float *self_k, float *self_v, float *cross_k, float *cross_v,
                        size_t *length, size_t memory_length, const float *input, float *out, int *resident,
                        char *error, size_t error_capacity) {
    if (slot >= d->batch) return -1;
    decoder_cache *c = &d->caches[slot];
    c->self_k = self_k; c->self_v = self_v; c->cross_k = cross_k; c->cross_v = cross_v;
    c->length = *length;
    c->memory_length = memory_length;
    const int rc = decoder_run(&d->model, c, input, 1u, out, NULL, error, error_capacity);
    *length = c->length;
    if (resident != NULL) *resident = c->dev_allocated && c->dev_attention_allocated;
    return rc;
}

/* A decoder_run of `count` > 1 rows of slot `slot` (the context prefill, src/graph.c:3506-3654): the projections go to the
 * backend as host-pointer products of `count` rows (or to the quantised CPU path when the cache is on and count <= 16,
 * src/qmat.c:768-818), self-attention as two sgemm calls per head (:3532-3545); the host caches are appended in place.  The
 * slot's one-row scratch is replaced by buffers of `count` rows for the call (decoder_cache_init sizes them so, :3086-3105). */
int ref_decoder_run_rows(ref_decoder *d, size_t slot, float *self_k, float *self_v, float *cross_k, float *cross_v,
                         size_t *length, size_t memory_length, const float *input_rows, size_t count, float *out_last,
                         char *error, size_t error_capacity) {
    if (slot >= d->batch || count < 2) return -1;
    decoder_cache *c = &d->caches[slot];
    const decoder_cache saved = *c;
    const size_t w = c->width, f = c->ffn_width, xw = c->xattn_width;
    const size_t score_len = c->capacity > memory_length ? c->capacity : memory_length;
    float *bufs[11] = {0};
    const size_t sizes[11] = {count * w, count * w, count * 3u * w, count * w, count * w, count * xw, count * xw, count * f,
                              score_len + 1u, count * c->capacity, count * c->head_width};
    int rc = -1;
    for (int i = 0; i < 11; ++i) {
        bufs[i] = (float *)calloc(sizes[i], sizeof(float));
        if (bufs[i] == NULL) { graph_error(error, error_capacity, "out of memory"); goto done; }
    }
    c->scratch_rows = count;
    c->scratch_x = bufs[0]; c->scratch_nrm = bufs[1]; c->scratch_qkv = bufs[2]; c->scratch_attn = bufs[3];
    c->scratch_proj = bufs[4]; c->scratch_q_x = bufs[5]; c->scratch_xctx = bufs[6]; c->scratch_hidden = bufs[7];
    c->scratch_scores = bufs[8]; c->scratch_score_matrix = bufs[9]; c->scratch_head_ctx = bufs[10];
    c->self_k = self_k; c->self_v = self_v; c->cross_k = cross_k; c->cross_v = cross_v;
    c->length = *length;
    c->memory_length = memory_length;
    rc = decoder_run(&d->model, c, input_rows, count, out_last, NULL, error, error_capacity);
    *length = c->length;
done:
    {
        const size_t new_length = c->length;
        *c = saved;               /* the one-row scratch again; the call leaves no device state behind */
        c->length = new_length;
    }
    for (int i = 0; i < 11; ++i) free(bufs[i]);
    return rc;
}

/* Row `row` of layer `layer` of the slot's device K and V caches, through the backend's own d2h. */
int ref_decoder_read_device_kv(ref_decoder *d, size_t slot, size_t layer, size_t row, float *k_row, float *v_row,
                               char *error, size_t error_capacity) {
    decoder_cache *c = &d->caches[slot];
    if (!c->dev_attention_allocated) return -1;
    const size_t offset = (layer * c->capacity + row) * c->width;
    if (mynah_backend_d2h(c->dev_backend, c->dev_self_k + offset, k_row, c->width, error, error_capacity) != 0) return -1;
    return mynah_backend_d2h(c->dev_backend, c->dev_self_v + offset, v_row, c->width, error, error_capacity);
}

/* -- local transformer, resident position ----------------------------------------------------------------------- */
static void ref_local_release_device(ref_local *d) {
    for (size_t b = 0; b < MYNAH_MAX_BATCH; ++b) {
        local_cache *c = &d->caches[b];
        if (c->dev_backend == NULL) continue;
        mynah_backend_dev_free(c->dev_backend, c->dev_k);      mynah_backend_dev_free(c->dev_backend, c->dev_v);
        mynah_backend_dev_free(c->dev_backend, c->dev_x);      mynah_backend_dev_free(c->dev_backend, c->dev_nrm);
        mynah_backend_dev_free(c->dev_backend, c->dev_qkv);    mynah_backend_dev_free(c->dev_backend, c->dev_attn);
        mynah_backend_dev_free(c->dev_backend, c->dev_proj);   mynah_backend_dev_free(c->dev_backend, c->dev_hidden);
        mynah_backend_dev_free(c->dev_backend, c->dev_input);
        c->dev_k = c->dev_v = c->dev_x = c->dev_nrm = c->dev_qkv = c->dev_attn = c->dev_proj = c->dev_hidden = NULL;
        c->dev_input = NULL;
        c->dev_backend = NULL;
        c->gpu_ready = 0;
    }
}

int ref_local_use_hip(ref_local *d, const char *library_path, char *error, size_t error_capacity) {
    mynah_backend *hip = ref_backend_open_hip(library_path, error, error_capacity);
    if (hip == NULL) return -1;
    ref_local_release_device(d);
    if (d->model.backend != NULL) mynah_backend_close(d->model.backend);
    d->model.backend = hip;
    return 0;
}

void ref_local_release(ref_local *d) { if (d != NULL) ref_local_release_device(d); }

/* One resident position of slot `slot`: the buffers local_cache_init allocates for a device backend
 * (src/graph.c:1058-1090; the logits buffer is not touched by the step and is left out), the input row uploaded,
 * local_step_device, and the output row read back.  *length is the slot's position before / after. */
int ref_local_device_step(ref_local *d, size_t slot, size_t *length, const float *input, float *out,
                          char *error, size_t error_capacity) {
    if (slot >= d->batch) return -1;
    local_cache *c = &d->caches[slot];
    const mynah_backend *bk = d->model.backend;
    if (!mynah_backend_has_dev_ops(bk) || !mynah_backend_has_attention_dev(bk)) {
        graph_error(error, error_capacity, "backend has no resident operators");
        return -1;
    }
    if (!c->gpu_ready) {
        const size_t kv_count = c->layers * c->capacity * c->width;
        c->dev_backend = bk;
        const int ok =
            mynah_backend_dev_alloc(bk, kv_count, &c->dev_k, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, kv_count, &c->dev_v, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->width, &c->dev_x, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->width, &c->dev_nrm, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->width * 3u, &c->dev_qkv, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->width, &c->dev_attn, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->width, &c->dev_proj, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->ffn_width, &c->dev_hidden, error, error_capacity) == 0 &&
            mynah_backend_dev_alloc(bk, c->width, &c->dev_input, error, error_capacity) == 0;
        if (!ok) { ref_local_release_device(d); return -1; }
        c->gpu_ready = 1;
    }
    c->length = *length;
    float *dev_out = NULL;
    if (mynah_backend_h2d(bk, input, c->dev_input, c->width, error, error_capacity) != 0) return -1;
    if (local_step_device(&d->model, c, c->dev_input, &dev_out, error, error_capacity) != 0) return -1;
    if (mynah_backend_sync(bk, error, error_capacity) != 0) return -1;
    if (mynah_backend_d2h(bk, dev_out, out, c->width, error, error_capacity) != 0) return -1;
    *length = c->length;
    return 0;
}

/* -- the codec decode, CPU orchestration against resident orchestration ------------------------------------------
 * Reference functions reached (file:line in the reference tree):
 *   decode_codec            src/graph.c:2640-2790  tries decode_codec_resident first, else the CPU sequence
 *   decode_codec_resident   src/graph.c:2508-2638  taken when the backend has device operators and attention
 *   res_layer_device        src/graph.c:2423-2505
 * The model is zero-filled except for its codec weight file (a safetensors file the caller wrote) and its backend. */
typedef struct {
    mynah_tts_model model;
} ref_codec_engine;

void ref_codec_engine_free(ref_codec_engine *e) {
    if (e == NULL) return;
    if (e->model.backend != NULL) mynah_backend_close(e->model.backend);
    if (e->model.codec != NULL) mynah_weights_close(e->model.codec);
    free(e);
}

/* hip_library == NULL: the reference's CPU backend. */
ref_codec_engine *ref_codec_engine_new(const char *weights_path, const char *hip_library, char *error, size_t error_capacity) {
    ref_codec_engine *e = (ref_codec_engine *)calloc(1, sizeof(*e));
    if (e == NULL) return NULL;
    if (mynah_weights_open(weights_path, &e->model.codec, error, error_capacity) != 0) { free(e); return NULL; }
    if (hip_library != NULL) {
        e->model.backend = ref_backend_open_hip(hip_library, error, error_capacity);
        if (e->model.backend == NULL) { ref_codec_engine_free(e); return NULL; }
    } else if (mynah_backend_open(MYNAH_TTS_DEVICE_CPU, &e->model.backend, error, error_capacity) != 0) {
        ref_codec_engine_free(e);
        return NULL;
    }
    return e;
}

/* codes: [8 groups, raw_length].  Returns the sample count through *count (raw_length * 1024) and copies at most
 * `capacity` samples into `samples`.  *resident says which of the two sequences the engine chose. */
int ref_codec_engine_decode(ref_codec_engine *e, const unsigned *codes, size_t raw_length, float *samples, size_t capacity,
                            size_t *count, int *resident, char *error, size_t error_capacity) {
    float *audio = NULL;
    size_t n = 0;
    const mynah_backend *bk = e->model.backend;
    if (resident != NULL) *resident = mynah_backend_has_dev_ops(bk) && mynah_backend_has_attention_dev(bk);
    if (decode_codec(&e->model, codes, raw_length, &audio, &n, error, error_capacity) != 0) return -1;
    memcpy(samples, audio, (n < capacity ? n : capacity) * sizeof(float));
    free(audio);
    *count = n;
    return 0;
}


/* ---- the integration text, compiled ------------------------------------------------------------------------------
 * oracle/integration_batched.inc is the engine-side code that the repository's integration notes quote.  In the engine its five
 * library calls are linked symbols; here the library is found with dlopen (so that this file still loads where no GPU
 * runtime is installed) and the calls go through pointers of the header's own prototype types.
 * Reference types it is compiled against: decoder_cache / decoder_layer_resolved (src/graph.c:2795-2861), local_cache
 * (:810-851), local_batch_item (:1346-1364); reference functions the drivers below use: decoder_gpu_attention_init
 * (:2901-2962). */
#include <dlfcn.h>

#include "mynah_hip.h"

static struct {
    __typeof__(&mynah_hip_decoder_create) decoder_create;
    __typeof__(&mynah_hip_decoder_destroy) decoder_destroy;
    __typeof__(&mynah_hip_decoder_step) decoder_step;
    __typeof__(&mynah_hip_local_create) local_create;
    __typeof__(&mynah_hip_local_destroy) local_destroy;
    __typeof__(&mynah_hip_local_frame) local_frame;
} hip_calls;
#define mynah_hip_decoder_create (*hip_calls.decoder_create)
#define mynah_hip_decoder_destroy (*hip_calls.decoder_destroy)
#define mynah_hip_decoder_step (*hip_calls.decoder_step)
#define mynah_hip_local_create (*hip_calls.local_create)
#define mynah_hip_local_destroy (*hip_calls.local_destroy)
#define mynah_hip_local_frame (*hip_calls.local_frame)
#include "integration_batched.inc"
#undef mynah_hip_decoder_create
#undef mynah_hip_decoder_destroy
#undef mynah_hip_decoder_step
#undef mynah_hip_local_create
#undef mynah_hip_local_destroy
#undef mynah_hip_local_frame

void *ref_backend_state(const mynah_backend *backend);   /* ref_shim_backend.c: the accessor the integration text asks for */

static int integration_bind(const char *library_path, char *error, size_t error_capacity) {
    if (hip_calls.decoder_create != NULL) return 0;
    void *handle = dlopen(library_path, RTLD_NOW | RTLD_GLOBAL);
    if (handle == NULL) {
        snprintf(error, error_capacity, "dlopen: %s", dlerror());
        return -1;
    }
    hip_calls.decoder_create = (__typeof__(hip_calls.decoder_create))dlsym(handle, "mynah_hip_decoder_create");
    hip_calls.decoder_destroy = (__typeof__(hip_calls.decoder_destroy))dlsym(handle, "mynah_hip_decoder_destroy");
    hip_calls.decoder_step = (__typeof__(hip_calls.decoder_step))dlsym(handle, "mynah_hip_decoder_step");
    hip_calls.local_create = (__typeof__(hip_calls.local_create))dlsym(handle, "mynah_hip_local_create");
    hip_calls.local_destroy = (__typeof__(hip_calls.local_destroy))dlsym(handle, "mynah_hip_local_destroy");
    hip_calls.local_frame = (__typeof__(hip_calls.local_frame))dlsym(handle, "mynah_hip_local_frame");
    if (!hip_calls.decoder_create || !hip_calls.decoder_destroy || !hip_calls.decoder_step || !hip_calls.local_create ||
        !hip_calls.local_destroy || !hip_calls.local_frame) {
        snprintf(error, error_capacity, "the library lacks a batched entry point");
        hip_calls.decoder_create = NULL;
        return -1;
    }
    return 0;
}

/* One batched device step of the decoder's first `d->batch` slots through hip_decoder_step_batch.  The decoder must have
 * the library attached (ref_decoder_use_hip).  At a slot's first call its host caches (rows [0, lengths[b]) of
 * self_k / self_v, all of cross_k / cross_v) are uploaded by the reference's own decoder_gpu_attention_init; afterwards the
 * device caches are the live ones.  lengths[b] comes back advanced by one. */
int ref_decoder_hip_step_batch(ref_decoder *d, const char *library_path, float *const *self_k, float *const *self_v,
                               float *const *cross_k, float *const *cross_v, size_t *lengths, const size_t *memory_lengths,
                               const float *const *inputs, float *const *outs, char *error, size_t error_capacity) {
    const mynah_backend *backend = d->model.backend;
    void *state = ref_backend_state(backend);
    if (integration_bind(library_path, error, error_capacity) != 0) return -1;
    decoder_cache *ptrs[MYNAH_MAX_BATCH];
    for (size_t b = 0; b < d->batch; ++b) {
        decoder_cache *c = &d->caches[b];
        c->self_k = self_k[b]; c->self_v = self_v[b]; c->cross_k = cross_k[b]; c->cross_v = cross_v[b];
        c->length = lengths[b];
        c->memory_length = memory_lengths[b];
        if (decoder_gpu_attention_init(c, backend, error, error_capacity) != 0) return -1;
        if (d->hip_in[b] == NULL &&
            (mynah_backend_dev_alloc(backend, c->width, &d->hip_in[b], error, error_capacity) != 0 ||
             mynah_backend_dev_alloc(backend, c->width, &d->hip_out[b], error, error_capacity) != 0))
            return -1;
        if (mynah_backend_h2d(backend, inputs[b], d->hip_in[b], c->width, error, error_capacity) != 0) return -1;
        ptrs[b] = c;
    }
    if (d->hip_batch == NULL) {
        hip_decoder_batch *h = (hip_decoder_batch *)calloc(1, sizeof(*h));
        if (h == NULL || hip_decoder_batch_init(state, &d->caches[0], h, error, error_capacity) != 0) {
            free(h);
            return -1;
        }
        d->hip_batch = h;
    }
    if (hip_decoder_step_batch(state, (hip_decoder_batch *)d->hip_batch, ptrs, (const float *const *)d->hip_in, d->hip_out, d->batch,
                               error, error_capacity) != 0)
        return -1;
    for (size_t b = 0; b < d->batch; ++b) {
        if (mynah_backend_d2h(backend, d->hip_out[b], outs[b], d->caches[b].width, error, error_capacity) != 0) return -1;
        lengths[b] = d->caches[b].length;
    }
    return 0;
}

/* Releases what ref_decoder_hip_step_batch set up; call before ref_decoder_release. */
void ref_decoder_hip_batch_release(ref_decoder *d) {
    if (d == NULL) return;
    if (d->hip_batch != NULL) {
        hip_decoder_batch_free(ref_backend_state(d->model.backend), (hip_decoder_batch *)d->hip_batch);
        free(d->hip_batch);
        d->hip_batch = NULL;
    }
    for (size_t b = 0; b < MYNAH_MAX_BATCH; ++b) {
        if (d->hip_in[b] != NULL) mynah_backend_dev_free(d->model.backend, d->hip_in[b]);
        if (d->hip_out[b] != NULL) mynah_backend_dev_free(d->model.backend, d->hip_out[b]);
        d->hip_in[b] = d->hip_out[b] = NULL;
    }
}

/* One device frame for `count` items through hip_sample_local_frame_batch, on the local stack of `d` (library attached
 * with ref_local_use_hip).  The items are the reference's own local_batch_item: decoder_last[i] is uploaded to a device
 * row; rng_states[i] is used when has_rng[i] (else the item is greedy, rng_state == NULL); codes is
 * [count][codebook_count][code_stride] and receives the stored codes at column raw_offset + frame. */
int ref_local_hip_frame(ref_local *d, const char *library_path, size_t streams, size_t vocab, size_t codebook_size, size_t eos_id,
                        size_t codebook_count, const float *const *projection_w, const float *const *projection_bias,
                        const float *const *audio_table, size_t count, const float *const *decoder_last, const float *temperature,
                        const unsigned *topk, uint64_t *rng_states, const int *has_rng, const size_t *generated_raw_length,
                        const size_t *min_raw_length, unsigned *codes, size_t code_stride, size_t raw_offset, int *saw_eos,
                        size_t *eos_frame, char *error, size_t error_capacity) {
    const mynah_backend *backend = d->model.backend;
    void *state = ref_backend_state(backend);
    if (integration_bind(library_path, error, error_capacity) != 0) return -1;
    if (count > MYNAH_MAX_BATCH) return -1;
    if (d->hip_batch == NULL) {
        hip_local_batch *h = (hip_local_batch *)calloc(1, sizeof(*h));
        if (h == NULL || hip_local_batch_init(state, &d->caches[0], streams, vocab, codebook_size, eos_id, codebook_count, projection_w,
                                              projection_bias, audio_table, h, error, error_capacity) != 0) {
            free(h);
            return -1;
        }
        d->hip_batch = h;
    }
    local_batch_item items[MYNAH_MAX_BATCH];
    memset(items, 0, sizeof items);
    const size_t width = d->caches[0].width;
    for (size_t i = 0; i < count; ++i) {
        if (d->hip_last[i] == NULL && mynah_backend_dev_alloc(backend, width, &d->hip_last[i], error, error_capacity) != 0) return -1;
        if (mynah_backend_h2d(backend, decoder_last[i], d->hip_last[i], width, error, error_capacity) != 0) return -1;
        items[i].decoder_last = decoder_last[i];
        items[i].decoder_dev_last = d->hip_last[i];
        items[i].codes = codes + i * codebook_count * code_stride;
        items[i].raw_offset = raw_offset;
        items[i].code_stride = code_stride;
        items[i].generated_raw_length = generated_raw_length[i];
        items[i].min_raw_length = min_raw_length[i];
        items[i].temperature = temperature[i];
        items[i].topk = topk[i];
        items[i].rng_state = has_rng[i] ? &rng_states[i] : NULL;
    }
    if (hip_sample_local_frame_batch(state, (hip_local_batch *)d->hip_batch, items, count, error, error_capacity) != 0) return -1;
    for (size_t i = 0; i < count; ++i) {
        saw_eos[i] = items[i].saw_eos;
        eos_frame[i] = items[i].eos_frame;
    }
    return 0;
}

void ref_local_hip_batch_release(ref_local *d) {
    if (d == NULL) return;
    if (d->hip_batch != NULL) {
        hip_local_batch *h = (hip_local_batch *)d->hip_batch;
        if (h->local != NULL) (*hip_calls.local_destroy)(ref_backend_state(d->model.backend), h->local);
        free(h);
        d->hip_batch = NULL;
    }
    for (size_t b = 0; b < MYNAH_MAX_BATCH; ++b) {
        if (d->hip_last[b] != NULL) mynah_backend_dev_free(d->model.backend, d->hip_last[b]);
        d->hip_last[b] = NULL;
    }
}
