// The resident batched decode step: decoder_step_batch (src/graph.c:3127-3284) as six fused
// kernels per layer, replayed as one HIP graph.
//
//   per layer   1  LN(norm_self) + act-quant + per-head Q/K/V rows + KV append + split-L self-attention -> partials
//               2  fold partials + act-quant + O matvec + residual                                       -> x
//               3  LN(norm_xattn_query) + act-quant + per-head Q rows + split-L cross-attention          -> partials
//               4  fold partials + act-quant + O matvec + residual                                       -> x
//               5  LN(norm_pos_ff) + act-quant + up matvec + tanh-GELU                                   -> hidden
//               6  act-quant + down matvec + residual                                                    -> x
//   begin / end    x = input + position[length]   /   out = LN(norm_out)(x)
//
// Head shapes the fused attention kernel does not take (head width other than 64) run the same step as
// eight kernels per layer: projection, stand-alone attention, projection.
//
// Everything that changes from step to step (cache pointers, lengths, input/output rows) lives in a
// small device-side slot table written by the begin kernel, so the captured graph is replayed
// unchanged for the life of a (decoder, batch size) pair.
#include <stdlib.h>
#include <string.h>

#include <new>

#include "device_common.h"

namespace mynah {

struct LayerWeights {
    const CachedWeight *qkv, *o_self, *q_cross, *o_cross, *up, *down;
    const float *norm_self, *norm_self_b, *norm_cross, *norm_cross_b, *norm_ff, *norm_ff_b;
};

}  // namespace mynah

struct mynah_hip_decoder {
    size_t layers, width, heads, head_width, ffn, cross_heads, cross_head_width, xw, capacity;
    std::vector<mynah::LayerWeights> lw;
    const float *norm_out = nullptr, *norm_out_b = nullptr, *position = nullptr;
    // workspaces, kMaxBatch rows each
    float *x = nullptr, *qkv = nullptr, *attn = nullptr, *qx = nullptr, *ctx = nullptr, *hidden = nullptr;
    mynah::StepSlots *dev_slots = nullptr;
    float *partial = nullptr;   // split-L attention partials of the fused path
    float *partial_ml = nullptr;
    // Split-L partials of the stand-alone attention kernels (head widths the fused kernel does not take).  Owned by the
    // decoder, not the backend's shared workspace: that one is freed and reallocated when a later call needs more room,
    // and the captured graphs of this decoder hold the address they were recorded with.
    float *seam_partial = nullptr;
    mynah::StepItem *self_items = nullptr, *cross_items = nullptr;   // work tables of the many-stream attention launches
    // many streams: the attention launches fold their own partials, which travel as tagged records
    // [kMaxBatch, heads, max_units, kStepRecord] (one area per attention kind); null: a fold kernel follows each launch
    unsigned long long *self_records = nullptr, *cross_records = nullptr;
    size_t records_bytes = 0;
    int self_slots = 0, cross_slots = 0;   // workgroups of the many-stream attention kernels that the device holds at once
    unsigned item_epoch = 0;                    // next step counter for the tables (24 bits, never 0)
    mynah::StepSlots last_slots;                // of the last step of this lane
    mynah::StepSlots last_batch_slots;          // of the last step, every stream of it (the single-stage measurement graphs rebuild the tables from it)
    int last_lanes = 1;                         // lanes the last step ran in
    int last_batch = 0;                         // streams of the last step
    // parity probe (mynah_hip_decoder_step_probe only, null otherwise): [layers][6][ffn] int8 activations and [layers][6]
    // activation scales of stream 0, one slot per projection in the order qkv, o_self, q_cross, o_cross, up, down
    int8_t *probe_qx = nullptr;
    float *probe_sx = nullptr;
    int max_units = 0;
    bool fused_attention = false;
    // [with the end kernel or without it][stream count]: this lane's layer kernels as one chain of kernel nodes (without the
    // end kernel: the step whose final LayerNorm the output head's product does, mynah_hip_decoder_step_head)
    // forms: 0 the layers and the end kernel, 1 the layers alone, 2 the layers and the output head of HeadCall (its pointers are
    // part of the captured nodes: head_signature says whose they are, and the graph is captured again when they change)
    hipGraphExec_t graphs[3][mynah::kMaxBatch + 1] = {};
    int eager_steps[3][mynah::kMaxBatch + 1] = {};   // a stream count runs eagerly once before it is captured
    unsigned long long head_signature[mynah::kMaxBatch + 1] = {};
    int head_recaptures = 0;
    hipGraphExec_t stage_graphs[MYNAH_HIP_STAGE_COUNT][mynah::kMaxBatch + 1] = {};   // single-stage graphs (measurement only)
    int arith = 0;
    // Lanes: a batch above two streams is cut into groups that step side by side, each on a stream of its own with
    // workspaces, slot table and work tables of its own (a sibling decoder that shares this one's weights).  A stream's
    // arithmetic does not depend on who else is in its group, so the cut changes no bit of any output; what it buys is
    // that one group's launch gaps and staging phases are filled by the others' work.  lanes[0] is this decoder.
    std::vector<mynah_hip_decoder *> lanes;
    bool is_lane = false;
    // the step as one persistent launch (one or two streams): per-layer pointer table, exchange area and its tag counter
    mynah::PersistLayer *persist_layers = nullptr;
    unsigned long long *persist_exchange = nullptr;
    size_t persist_exchange_words = 0;
    unsigned persist_epoch = 8;
    int qtype = 0;
};

namespace mynah {

// fold: 0 = plain input rows, 1 = fold of the self-attention partials, 2 = fold of the cross-attention partials
static int enqueue_linear(State *st, const mynah_hip_decoder *d, const CachedWeight *w, const float *in, size_t in_stride,
                          float *out, size_t out_stride, int batch, const float *ln_gain, const float *ln_bias, int epilogue,
                          char *error, size_t capacity, int fold = 0, int probe_slot = -1) {
    for (int b0 = 0; b0 < batch; b0 += kBatchTile) {
        LinearArgs a{};
        if (d->probe_qx != nullptr && probe_slot >= 0 && b0 == 0) {
            a.probe_qx = d->probe_qx + (size_t)probe_slot * d->ffn;
            a.probe_sx = d->probe_sx + probe_slot;
        }
        if (fold != 0) {
            a.fold_partial = d->partial;
            a.fold_partial_ml = d->partial_ml;
            a.fold_slots = d->dev_slots;
            a.fold_heads = (int)(fold == 1 ? d->heads : d->cross_heads);
            a.fold_head_width = (int)(fold == 1 ? d->head_width : d->cross_head_width);
            a.fold_max_units = d->max_units;
            a.fold_is_self = fold == 1 ? 1 : 0;
            a.fold_stream0 = b0;
        }
        a.w = w->data;
        a.scales = w->scales;
        a.bias = nullptr;   // no decoder linear has a bias (src/graph.c:3169-3272 pass NULL)
        a.qtype = w->qtype;
        a.n = (int)w->n;
        a.k = (int)w->k;
        a.batch = batch - b0 < kBatchTile ? batch - b0 : kBatchTile;
        for (int b = 0; b < a.batch; ++b) {
            a.in[b] = in + (size_t)(b0 + b) * in_stride;
            a.out[b] = out + (size_t)(b0 + b) * out_stride;
        }
        a.ln_gain = ln_gain;
        a.ln_bias = ln_bias;
        a.epilogue = epilogue;
        a.arith = d->arith;
        if (launch_linear(st, a, error, capacity) != 0) return -1;
    }
    return 0;
}

static int enqueue_attention(State *st, const mynah_hip_decoder *d, int is_self, size_t layer, int batch, char *error,
                             size_t capacity) {
    AttnArgs a{};
    a.slots = d->dev_slots;
    a.layer = layer;
    a.capacity = d->capacity;
    a.batch = batch;
    a.is_self = is_self;
    a.partial = d->seam_partial;
    a.counters = st->attn_counters;   // allocated once per backend and never moved
    if (is_self) {
        a.q[0] = d->qkv;
        a.out[0] = d->attn;
        a.heads = (int)d->heads;
        a.head_width = (int)d->head_width;
        a.stride = (int)d->width;
        a.q_stride = (int)(3 * d->width);
        a.scale = 1.0f / sqrtf((float)d->head_width);
        a.max_chunks = (int)((d->capacity + kAttnChunk - 1) / kAttnChunk);
    } else {
        a.q[0] = d->qx;
        a.out[0] = d->ctx;
        a.heads = (int)d->cross_heads;
        a.head_width = (int)d->cross_head_width;
        a.stride = (int)d->xw;
        a.q_stride = (int)d->xw;
        a.scale = 1.0f / sqrtf((float)d->cross_head_width);
        a.max_chunks = (int)((d->capacity + kAttnChunk - 1) / kAttnChunk);   // memory_length <= capacity is checked per step
    }
    return launch_attention(st, a, error, capacity);
}


static int enqueue_step_attention(State *st, const mynah_hip_decoder *d, int is_self, size_t layer, int batch, const CachedWeight *w,
                                  const float *ln_gain, const float *ln_bias, char *error, size_t capacity) {
    StepAttnArgs a{};
    if (d->probe_qx != nullptr) {
        const size_t slot = layer * 6 + (is_self ? 0 : 2);
        a.probe_qx = d->probe_qx + slot * d->ffn;
        a.probe_sx = d->probe_sx + slot;
    }
    a.slots = d->dev_slots;
    a.items = is_self ? d->self_items : d->cross_items;
    a.x = d->x;
    a.batch = batch;
    a.width = (int)d->width;
    a.ln_gain = ln_gain;
    a.ln_bias = ln_bias;
    a.w = w->data;
    a.scales = w->scales;
    a.qtype = w->qtype;
    a.arith = d->arith;
    a.is_self = is_self;
    a.heads = (int)(is_self ? d->heads : d->cross_heads);
    a.head_width = (int)(is_self ? d->head_width : d->cross_head_width);
    a.layer = layer;
    a.capacity = d->capacity;
    a.max_units = d->max_units;
    a.scale = 1.0f / sqrtf((float)a.head_width);
    a.partial = d->partial;
    a.partial_ml = d->partial_ml;
    a.records = batch > kConsumerFoldMaxBatch ? (is_self ? d->self_records : d->cross_records) : nullptr;
    a.fold_out = is_self ? d->attn : d->ctx;
    a.spin_limit = st->persist_spin_limit;
    a.abort_word = st->persist_abort_dev;
    if (launch_step_attention(st, a, error, capacity) != 0) return -1;
    if (batch > kConsumerFoldMaxBatch && a.records == nullptr) return launch_step_fold(st, a, a.fold_out, error, capacity);
    return 0;
}

// The layer loop; everything here is replayable (no per-step scalars in kernel arguments).
// `stages` selects which of the six per-layer stages are enqueued (bit MYNAH_HIP_STAGE_*); the step itself
// passes kAllStages, the per-stage timing entry one bit at a time.
constexpr unsigned kAllStages = 0x3fu;

static int enqueue_layers(State *st, const mynah_hip_decoder *d, int batch, char *error, size_t capacity, unsigned stages = kAllStages,
                          bool with_end = true) {
    const size_t w = d->width;
    const auto on = [stages](int stage) { return (stages >> stage) & 1u; };
    if (d->fused_attention) {
        for (size_t l = 0; l < d->layers; ++l) {
            const LayerWeights &lw = d->lw[l];
            if (on(MYNAH_HIP_STAGE_SELF_ATTENTION) &&
                enqueue_step_attention(st, d, 1, l, batch, lw.qkv, lw.norm_self, lw.norm_self_b, error, capacity) != 0) return -1;
            const bool consumer_fold = batch <= kConsumerFoldMaxBatch;
            const int slot0 = (int)l * 6;
            if (on(MYNAH_HIP_STAGE_SELF_OUT) &&
                enqueue_linear(st, d, lw.o_self, d->attn, w, d->x, w, batch, nullptr, nullptr, EPI_RESIDUAL, error, capacity, consumer_fold ? 1 : 0, slot0 + 1) != 0) return -1;
            if (d->xw != 0) {
                if (on(MYNAH_HIP_STAGE_CROSS_ATTENTION) &&
                    enqueue_step_attention(st, d, 0, l, batch, lw.q_cross, lw.norm_cross, lw.norm_cross_b, error, capacity) != 0) return -1;
                if (on(MYNAH_HIP_STAGE_CROSS_OUT) &&
                    enqueue_linear(st, d, lw.o_cross, d->ctx, d->xw, d->x, w, batch, nullptr, nullptr, EPI_RESIDUAL, error, capacity, consumer_fold ? 2 : 0, slot0 + 3) != 0) return -1;
            }
            if (on(MYNAH_HIP_STAGE_FFN_UP) &&
                enqueue_linear(st, d, lw.up, d->x, w, d->hidden, d->ffn, batch, lw.norm_ff, lw.norm_ff_b, EPI_GELU, error, capacity, 0, slot0 + 4) != 0) return -1;
            if (on(MYNAH_HIP_STAGE_FFN_DOWN) &&
                enqueue_linear(st, d, lw.down, d->hidden, d->ffn, d->x, w, batch, nullptr, nullptr, EPI_RESIDUAL, error, capacity, 0, slot0 + 5) != 0) return -1;
        }
        if (stages != kAllStages || !with_end) return 0;
        return launch_step_end(st, d->dev_slots, batch, w, d->x, w, d->norm_out, d->norm_out_b, error, capacity);
    }
    for (size_t l = 0; l < d->layers; ++l) {
        const LayerWeights &lw = d->lw[l];
        if (enqueue_linear(st, d, lw.qkv, d->x, w, d->qkv, 3 * w, batch, lw.norm_self, lw.norm_self_b, EPI_NONE, error, capacity) != 0) return -1;
        if (enqueue_attention(st, d, 1, l, batch, error, capacity) != 0) return -1;
        if (enqueue_linear(st, d, lw.o_self, d->attn, w, d->x, w, batch, nullptr, nullptr, EPI_RESIDUAL, error, capacity) != 0) return -1;
        if (d->xw != 0) {
            if (enqueue_linear(st, d, lw.q_cross, d->x, w, d->qx, d->xw, batch, lw.norm_cross, lw.norm_cross_b, EPI_NONE, error, capacity) != 0) return -1;
            if (enqueue_attention(st, d, 0, l, batch, error, capacity) != 0) return -1;
            if (enqueue_linear(st, d, lw.o_cross, d->ctx, d->xw, d->x, w, batch, nullptr, nullptr, EPI_RESIDUAL, error, capacity) != 0) return -1;
        }
        if (enqueue_linear(st, d, lw.up, d->x, w, d->hidden, d->ffn, batch, lw.norm_ff, lw.norm_ff_b, EPI_GELU, error, capacity) != 0) return -1;
        if (enqueue_linear(st, d, lw.down, d->hidden, d->ffn, d->x, w, batch, nullptr, nullptr, EPI_RESIDUAL, error, capacity) != 0) return -1;
    }
    if (!with_end) return 0;
    return launch_step_end(st, d->dev_slots, batch, w, d->x, w, d->norm_out, d->norm_out_b, error, capacity);
}

DecoderRows decoder_rows(mynah_hip_decoder *d) { return DecoderRows{d->x, d->dev_slots, d->position}; }

StepItemTables decoder_item_tables(mynah_hip_decoder *d, int batch) {
    if (!d->fused_attention || batch <= kConsumerFoldMaxBatch) return StepItemTables{};
    return step_item_tables(batch, (int)d->heads, (int)d->cross_heads, d->max_units, d->self_items, d->cross_items, d->self_records != nullptr,
                            d->self_slots, d->cross_slots);
}

int decoder_enqueue_layers(State *st, mynah_hip_decoder *d, int batch, char *error, size_t capacity) {
    return enqueue_layers(st, d, batch, error, capacity, kAllStages, false);
}

// The rows, slot table, partial areas and work tables one group of streams steps on: the owner's, and each lane's.
static int allocate_workspaces(State *st, mynah_hip_decoder *d, char *error, size_t capacity) {
    int rc = 0;
    const size_t w = d->width, xw = d->xw;
    const size_t B = kMaxBatch;
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->x), B * w * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->qkv), B * 3 * w * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->attn), B * w * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->qx), B * (xw ? xw : 4) * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->ctx), B * (xw ? xw : 4) * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->hidden), B * d->ffn * sizeof(float)), "malloc", error, capacity);
    if (rc == 0) rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->dev_slots), sizeof(StepSlots)), "malloc", error, capacity);
    const size_t hw_max = d->head_width > d->cross_head_width ? d->head_width : d->cross_head_width;
    const size_t heads_max = d->heads > d->cross_heads ? d->heads : d->cross_heads;
    if (rc == 0) rc |= ensure_attention_workspace(st, B, heads_max, hw_max, d->capacity, error, capacity);
    if (rc == 0) {
        const char *env = getenv("MYNAH_HIP_FUSED_ATTENTION");
        const LayerWeights &l0 = d->lw[0];
        d->fused_attention = !(env != nullptr && strcmp(env, "0") == 0) &&
                             step_attention_supported(l0.qkv->qtype, w, d->heads, d->head_width) &&
                             (xw == 0 || (l0.q_cross->qtype == l0.qkv->qtype &&
                                          step_attention_supported(l0.q_cross->qtype, w, d->cross_heads, d->cross_head_width)));
        d->max_units = (int)((d->capacity + kStepUnitRows - 1) / kStepUnitRows) + 1;
        if (!d->fused_attention) {
            const size_t chunks = (d->capacity + kAttnChunk - 1) / kAttnChunk + 1;
            rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->seam_partial), B * heads_max * chunks * (hw_max + 4) * sizeof(float)),
                            "malloc", error, capacity);
        }
        if (d->fused_attention) {
            const size_t floats = B * heads_max * (size_t)d->max_units * hw_max;
            rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->partial), floats * sizeof(float)), "malloc", error, capacity);
            if (rc == 0)
                rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->partial_ml), B * heads_max * 2 * (size_t)d->max_units * sizeof(float)),
                                "malloc", error, capacity);
            // one entry per workgroup of the largest attention grid (kMaxBatch streams), self and cross
            if (rc == 0)
                rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->self_items),
                                          (size_t)step_attention_grid((int)d->heads, kMaxBatch, d->max_units, 1, true) * sizeof(StepItem)), "malloc", error, capacity);
            // The launches fold their own partials unless switched off, the wait has no abort word to report through, or
            // a (stream, head)'s records do not fit the LDS every launch may use without asking (long caches: the fold kernel then)
            const char *fold_env = getenv("MYNAH_HIP_FOLD_IN_LAUNCH");
            const bool fold_in_launch = !(fold_env != nullptr && strcmp(fold_env, "0") == 0) && st->persist_abort_dev != nullptr &&
                                        d->layers < 255 && step_fold_lds_bytes(d->max_units) <= 40 * 1024;
            if (rc == 0 && fold_in_launch) {
                d->records_bytes = B * heads_max * (size_t)d->max_units * kStepRecord * sizeof(unsigned long long);
                rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->self_records), d->records_bytes), "malloc", error, capacity);
                if (rc == 0) rc |= hip_check(hipMemset(d->self_records, 0, d->records_bytes), "memset", error, capacity);   // tag 0 is never waited for
                if (rc == 0 && xw != 0) {
                    rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->cross_records), d->records_bytes), "malloc", error, capacity);
                    if (rc == 0) rc |= hip_check(hipMemset(d->cross_records, 0, d->records_bytes), "memset", error, capacity);
                }
            }
            if (rc == 0) {
                // Chunks per workgroup: one, unless MYNAH_HIP_ATTN_SLOTS names a number of workgroup slots to fit the launch into
                // ("device": what the device holds of this kernel at once).  Measured with eight ragged streams, same box, twice
                // each: grouped to fit the device (pairs of chunks, one round of workgroups instead of two) 654 us per step,
                // one chunk per workgroup 649 us -- the second chunk of a pair waits for its rows a full round trip after the first.
                d->self_slots = d->cross_slots = 1 << 30;
                const char *slots_env = getenv("MYNAH_HIP_ATTN_SLOTS");
                if (slots_env != nullptr && strcmp(slots_env, "device") == 0) {
                    d->self_slots = step_attention_slots(l0.qkv->qtype, (int)w, d->max_units, 1, d->self_records != nullptr);
                    d->cross_slots = xw != 0 ? step_attention_slots(l0.q_cross->qtype, (int)w, d->max_units, 0, d->cross_records != nullptr) : 0;
                } else if (slots_env != nullptr && atoi(slots_env) > 0) {
                    d->self_slots = d->cross_slots = atoi(slots_env);
                }
            }
            if (rc == 0 && xw != 0)
                rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->cross_items),
                                          (size_t)step_attention_grid((int)d->cross_heads, kMaxBatch, d->max_units, 0, true) * sizeof(StepItem)), "malloc", error, capacity);
        }
    }
    return rc;
}

static int per_layer_vector(State *st, const float *const *arr, size_t layer, size_t n, const float **dev, char *error,
                            size_t capacity) {
    *dev = nullptr;
    if (arr == nullptr || arr[layer] == nullptr) return 0;
    return cached_vector(st, arr[layer], n, dev, error, capacity);
}

}  // namespace mynah

using namespace mynah;

extern "C" void mynah_hip_decoder_destroy(void *opaque, mynah_hip_decoder *d) {
    State *st = enter_state(opaque);
    if (d == nullptr) return;
    if (st != nullptr) (void)hipStreamSynchronize(st->stream);
    if (st != nullptr && st->last_step_decoder == d) st->last_step_decoder = nullptr;
    for (size_t i = 1; i < d->lanes.size(); ++i) {   // the lanes' streams have joined the backend's stream after every step
        d->lanes[i]->lanes.clear();
        mynah_hip_decoder_destroy(opaque, d->lanes[i]);
    }
    d->lanes.clear();
    for (auto &form : d->graphs)
        for (auto &g : form)
            if (g != nullptr) (void)hipGraphExecDestroy(g);
    for (auto &row : d->stage_graphs)
        for (auto &g : row)
            if (g != nullptr) (void)hipGraphExecDestroy(g);
    float *bufs[] = {d->x, d->qkv, d->attn, d->qx, d->ctx, d->hidden, d->partial, d->partial_ml, d->seam_partial};
    for (float *p : bufs)
        if (p != nullptr) (void)hipFree(p);
    if (d->dev_slots != nullptr) (void)hipFree(d->dev_slots);
    if (d->self_items != nullptr) (void)hipFree(d->self_items);
    if (d->self_records != nullptr) (void)hipFree(d->self_records);
    if (d->cross_records != nullptr) (void)hipFree(d->cross_records);
    if (d->cross_items != nullptr) (void)hipFree(d->cross_items);
    if (d->persist_layers != nullptr) (void)hipFree(d->persist_layers);
    if (d->persist_exchange != nullptr) (void)hipFree(d->persist_exchange);
    delete d;
}

extern "C" int mynah_hip_decoder_create(void *opaque, const mynah_hip_decoder_desc *desc, mynah_hip_decoder **out, char *error,
                                        size_t capacity) {
    State *st = enter_state(opaque);
    if (out != nullptr) *out = nullptr;
    if (st == nullptr || desc == nullptr || out == nullptr || desc->layers == 0 || desc->layers > 4096 || desc->width == 0 || desc->heads == 0 ||
        desc->heads * desc->head_width != desc->width || desc->ffn_width == 0 || desc->capacity == 0 ||
        desc->capacity > 0x7ffffff0u || desc->norm_self == nullptr || desc->norm_pos_ff == nullptr || desc->qkv_w == nullptr ||
        desc->o_self_w == nullptr || desc->ffn_up_w == nullptr || desc->ffn_down_w == nullptr) {
        set_error(error, capacity, "invalid decoder description");
        return -1;
    }
    const size_t xw = desc->cross_heads * desc->cross_head_width;
    if (xw != 0 && (desc->q_cross_w == nullptr || desc->o_cross_w == nullptr || desc->norm_xattn_query == nullptr)) {
        set_error(error, capacity, "decoder description lacks cross-attention weights");
        return -1;
    }
    if (desc->head_width > 1024 || desc->cross_head_width > 1024 || desc->width > 4096 || xw > 4096) {
        set_error(error, capacity, "decoder head shape not supported");
        return -1;
    }
    if (!linear_fast_supported(MYNAH_HIP_F32, desc->width, desc->width) ||
        !linear_fast_supported(MYNAH_HIP_F32, desc->width, desc->ffn_width) ||
        (xw != 0 && !linear_fast_supported(MYNAH_HIP_F32, desc->width, xw))) {
        set_error(error, capacity, "decoder widths must be multiples of 256 and at most 3072 for the resident step");
        return -1;
    }
    mynah_hip_decoder *d = new (std::nothrow) mynah_hip_decoder();
    if (d == nullptr) {
        set_error(error, capacity, "out of memory creating decoder");
        return -1;
    }
    d->layers = desc->layers; d->width = desc->width; d->heads = desc->heads; d->head_width = desc->head_width;
    d->ffn = desc->ffn_width; d->cross_heads = desc->cross_heads; d->cross_head_width = desc->cross_head_width;
    d->xw = xw; d->capacity = desc->capacity; d->arith = st->arith;
    d->lw.resize(desc->layers);
    const size_t w = d->width;
    int rc = 0;
    for (size_t l = 0; l < d->layers && rc == 0; ++l) {
        LayerWeights &lw = d->lw[l];
        rc |= cached_matrix(st, desc->qkv_w[l], 3 * w, w, st->qtype, &lw.qkv, error, capacity);
        rc |= cached_matrix(st, desc->o_self_w[l], w, w, st->qtype, &lw.o_self, error, capacity);
        if (xw != 0) {
            rc |= cached_matrix(st, desc->q_cross_w[l], xw, w, st->qtype, &lw.q_cross, error, capacity);
            rc |= cached_matrix(st, desc->o_cross_w[l], w, xw, st->qtype, &lw.o_cross, error, capacity);
            rc |= per_layer_vector(st, desc->norm_xattn_query, l, w, &lw.norm_cross, error, capacity);
            rc |= per_layer_vector(st, desc->norm_xattn_query_bias, l, w, &lw.norm_cross_b, error, capacity);
        }
        rc |= cached_matrix(st, desc->ffn_up_w[l], d->ffn, w, st->qtype, &lw.up, error, capacity);
        rc |= cached_matrix(st, desc->ffn_down_w[l], w, d->ffn, st->qtype, &lw.down, error, capacity);
        rc |= per_layer_vector(st, desc->norm_self, l, w, &lw.norm_self, error, capacity);
        rc |= per_layer_vector(st, desc->norm_self_bias, l, w, &lw.norm_self_b, error, capacity);
        rc |= per_layer_vector(st, desc->norm_pos_ff, l, w, &lw.norm_ff, error, capacity);
        rc |= per_layer_vector(st, desc->norm_pos_ff_bias, l, w, &lw.norm_ff_b, error, capacity);
        if (rc == 0 && (lw.norm_self == nullptr || lw.norm_ff == nullptr || (xw != 0 && lw.norm_cross == nullptr))) {
            set_error(error, capacity, "decoder description lacks a LayerNorm gain");
            rc = -1;
        }
    }
    if (rc == 0) rc |= cached_vector(st, desc->norm_out, w, &d->norm_out, error, capacity);
    if (rc == 0) rc |= cached_vector(st, desc->norm_out_bias, w, &d->norm_out_b, error, capacity);
    if (rc == 0 && desc->position != nullptr) rc |= cached_vector(st, desc->position, d->capacity * w, &d->position, error, capacity);
    if (rc == 0) rc |= allocate_workspaces(st, d, error, capacity);
    if (rc == 0) {
        const LayerWeights &l0 = d->lw[0];
        d->qtype = l0.qkv->qtype;
        bool one_type = true;
        for (const LayerWeights &lw : d->lw)
            one_type = one_type && lw.qkv->qtype == d->qtype && lw.o_self->qtype == d->qtype && lw.up->qtype == d->qtype && lw.down->qtype == d->qtype &&
                       (xw == 0 || (lw.q_cross->qtype == d->qtype && lw.o_cross->qtype == d->qtype));
        if (d->fused_attention && one_type &&
            step_persistent_supported(d->qtype, w, d->heads, d->head_width, d->ffn, d->cross_heads, d->cross_head_width)) {
            std::vector<PersistLayer> table(d->layers);
            for (size_t l = 0; l < d->layers; ++l) {
                const LayerWeights &lw = d->lw[l];
                PersistLayer &t = table[l];
                memset(&t, 0, sizeof t);
                t.qkv_w = lw.qkv->data; t.qkv_s = lw.qkv->scales;
                t.o_w = lw.o_self->data; t.o_s = lw.o_self->scales;
                if (xw != 0) {
                    t.qx_w = lw.q_cross->data; t.qx_s = lw.q_cross->scales;
                    t.ox_w = lw.o_cross->data; t.ox_s = lw.o_cross->scales;
                }
                t.up_w = lw.up->data; t.up_s = lw.up->scales;
                t.down_w = lw.down->data; t.down_s = lw.down->scales;
                t.norm_self = lw.norm_self; t.norm_self_b = lw.norm_self_b;
                t.norm_cross = lw.norm_cross; t.norm_cross_b = lw.norm_cross_b;
                t.norm_ff = lw.norm_ff; t.norm_ff_b = lw.norm_ff_b;
            }
            PersistArgs shape{};
            shape.heads = (int)d->heads;
            shape.cross_heads = (int)d->cross_heads;
            shape.max_units = d->max_units;
            d->persist_exchange_words = step_persistent_exchange_words(shape);
            rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->persist_layers), table.size() * sizeof(PersistLayer)), "malloc", error, capacity);
            if (rc == 0)
                rc |= hip_check(hipMemcpy(d->persist_layers, table.data(), table.size() * sizeof(PersistLayer), hipMemcpyHostToDevice), "layer table upload",
                                error, capacity);
            if (rc == 0)
                rc |= hip_check(hipMalloc(reinterpret_cast<void **>(&d->persist_exchange), d->persist_exchange_words * sizeof(unsigned long long)), "malloc",
                                error, capacity);
            if (rc == 0)   // tag 0 is never expected: a fresh area holds nothing that could be taken for a result
                rc |= hip_check(hipMemset(d->persist_exchange, 0, d->persist_exchange_words * sizeof(unsigned long long)), "exchange clear", error, capacity);
        }
    }
    if (rc != 0) {
        mynah_hip_decoder_destroy(opaque, d);
        return -1;
    }
    *out = d;
    return 0;
}

namespace mynah {

// The step as one persistent launch, when this batch fits it: one or two streams, int8 / int4 weights, the stack's own
// shape, and few enough attention units for one workgroup each.  Returns 1 when launched, 0 when the step has to take
// the launched-kernels path, -1 on error.
static int try_persistent_step(State *st, mynah_hip_decoder *d, const mynah_hip_decoder_slot *slots, size_t batch, char *error, size_t capacity) {
    if (st->graph_mode != 2 || d->persist_layers == nullptr || batch > 2 || st->persist_abort_dev == nullptr) return 0;
    PersistArgs a{};
    a.layers = d->persist_layers;
    a.n_layers = (int)d->layers;
    a.batch = (int)batch;
    a.heads = (int)d->heads;
    a.cross_heads = (int)d->cross_heads;
    a.arith = d->arith;
    a.capacity = d->capacity;
    a.max_units = d->max_units;
    a.scale = 1.0f / sqrtf((float)d->head_width);
    for (size_t b = 0; b < batch; ++b) {
        a.self_k[b] = slots[b].dev_self_k;
        a.self_v[b] = slots[b].dev_self_v;
        a.cross_k[b] = slots[b].dev_cross_k;
        a.cross_v[b] = slots[b].dev_cross_v;
        a.input[b] = slots[b].dev_input;
        a.output[b] = slots[b].dev_output;
        a.length[b] = (int)slots[b].length;
        a.memory_length[b] = (int)slots[b].memory_length;
    }
    a.position = d->position;
    a.norm_out = d->norm_out;
    a.norm_out_b = d->norm_out_b;
    a.exchange = d->persist_exchange;
    a.spin_limit = st->persist_spin_limit;
    a.abort_word = st->persist_abort_dev;
    const int grid = st->cu_count;
    const int attn = step_persistent_attention_workgroups(a);
    a.attention_wgs = attn;
    // Row stages count their workgroups from the end of the grid, attention roles from its start: with room for both a
    // workgroup has one kind of role and requests its next stage's operands a whole stage ahead.  Rows per workgroup are what
    // the kernel requests ahead (32 rows of an output projection and of FFN up, 8 of FFN down); MYNAH_HIP_PERSIST_ROW_WGS
    // spreads the FFN rows over more workgroups.
    a.rows_out = 32;
    a.wgs_out = (768 + a.rows_out - 1) / a.rows_out;
    a.rows_up = 32;
    a.rows_down = 8;
    if (st->persist_row_wgs > 0) {
        const int wide = st->persist_row_wgs < grid ? st->persist_row_wgs : grid;
        a.rows_up = (3072 + wide - 1) / wide;
        a.rows_down = (768 + wide - 1) / wide;
    }
    a.wgs_up = (3072 + a.rows_up - 1) / a.rows_up;
    a.wgs_down = (768 + a.rows_down - 1) / a.rows_down;
    // When the attention units of these lengths and the row stages do not fit the grid side by side, or a stream's partial
    // records do not fit a workgroup's LDS, the step takes the launched-kernels path -- decided before a tag range is used up.
    if (!step_persistent_fits(a, grid)) return 0;
    const unsigned span = 8u * (unsigned)(d->layers + 2);
    if (d->persist_epoch > 0xffffffffu - 2u * span) {   // the tag counter is about to wrap: start over on a cleared area
        if (hip_check(hipMemsetAsync(d->persist_exchange, 0, d->persist_exchange_words * sizeof(unsigned long long), st->stream), "exchange clear", error,
                      capacity) != 0)
            return -1;
        d->persist_epoch = 8;
    }
    a.epoch = d->persist_epoch;
    d->persist_epoch += span;
    if (launch_step_persistent(st, a, d->qtype, grid, error, capacity) != 0) return -1;
    return 1;
}

}  // namespace mynah

namespace mynah {

// ---- lanes: groups of a batch's streams that step side by side --------------------------------------------------
// A sibling decoder for one lane: the owner's shape and (cached, shared) weights, rows and tables of its own.
static mynah_hip_decoder *new_lane(State *st, const mynah_hip_decoder *owner, char *error, size_t capacity) {
    mynah_hip_decoder *l = new (std::nothrow) mynah_hip_decoder();
    if (l == nullptr) {
        set_error(error, capacity, "out of memory creating a decoder lane");
        return nullptr;
    }
    l->layers = owner->layers; l->width = owner->width; l->heads = owner->heads; l->head_width = owner->head_width;
    l->ffn = owner->ffn; l->cross_heads = owner->cross_heads; l->cross_head_width = owner->cross_head_width;
    l->xw = owner->xw; l->capacity = owner->capacity; l->arith = owner->arith; l->qtype = owner->qtype;
    l->lw = owner->lw;
    l->norm_out = owner->norm_out; l->norm_out_b = owner->norm_out_b; l->position = owner->position;
    l->is_lane = true;
    if (allocate_workspaces(st, l, error, capacity) != 0) {
        mynah_hip_decoder_destroy(st, l);
        return nullptr;
    }
    return l;
}

static int ensure_lanes(State *st, mynah_hip_decoder *d, int n, char *error, size_t capacity) {
    if (d->lanes.empty()) d->lanes.push_back(d);
    for (int i = 1; i < n; ++i) {
        hipStream_t unused;
        if (lane_stream(st, i, &unused, error, capacity) != 0) return -1;
    }
    while ((int)d->lanes.size() < n) {
        mynah_hip_decoder *l = new_lane(st, d, error, capacity);
        if (l == nullptr) return -1;
        d->lanes.push_back(l);
    }
    return 0;
}

// How many lanes a batch of this size steps in.  One or two streams run the latency layout in one lane; the head shapes
// the fused attention kernel does not take share one backend-wide counter area and stay in one lane too.
static int lanes_for(const State *st, const mynah_hip_decoder *d, int batch) {
    if (d->is_lane || !d->fused_attention || batch <= kConsumerFoldMaxBatch) return 1;
    int n = st->step_lanes > 0 ? st->step_lanes : (batch + kLaneStreams - 1) / kLaneStreams;
    if (n > kMaxLanes) n = kMaxLanes;
    if (n > batch) n = batch;
    return n < 1 ? 1 : n;
}

// Which stream steps in which lane.  Lane sizes are fixed by (batch, lanes) -- the captured graph holds them as kernel
// arguments -- and the streams are dealt longest first to the lane with the least cache rows so far that still has room,
// so that ragged batches give the lanes equal work.  Any assignment yields the same bits for every stream.
struct LanePlan {
    int lanes;
    int count[kMaxLanes];
    int member[kMaxLanes][kMaxBatch];
};
static LanePlan plan_lanes(const StepSlots &s, int batch, int lanes) {
    LanePlan p{};
    p.lanes = lanes;
    for (int i = 0; i < lanes; ++i) p.count[i] = batch / lanes + (i < batch % lanes ? 1 : 0);
    int order[kMaxBatch];
    for (int b = 0; b < batch; ++b) order[b] = b;
    const auto cost = [&s](int b) { return (long)s.length[b] + (long)s.memory_length[b]; };
    for (int i = 1; i < batch; ++i) {   // insertion sort, descending cost, stable
        const int v = order[i];
        int j = i;
        while (j > 0 && cost(order[j - 1]) < cost(v)) { order[j] = order[j - 1]; --j; }
        order[j] = v;
    }
    int filled[kMaxLanes] = {};
    long load[kMaxLanes] = {};
    for (int i = 0; i < batch; ++i) {
        int best = -1;
        for (int l = 0; l < lanes; ++l)
            if (filled[l] < p.count[l] && (best < 0 || load[l] < load[best])) best = l;
        p.member[best][filled[best]++] = order[i];
        load[best] += cost(order[i]);
    }
    return p;
}

static StepSlots lane_slots(const StepSlots &s, const LanePlan &p, int lane) {
    StepSlots out;
    memset(&out, 0, sizeof out);
    for (int i = 0; i < p.count[lane]; ++i) {
        const int b = p.member[lane][i];
        out.self_k[i] = s.self_k[b]; out.self_v[i] = s.self_v[b];
        out.cross_k[i] = s.cross_k[b]; out.cross_v[i] = s.cross_v[b];
        out.input[i] = s.input[b]; out.output[i] = s.output[b];
        out.length[i] = s.length[b]; out.memory_length[i] = s.memory_length[b];
    }
    return out;
}

// One lane's layer kernels for `count` streams on `stream`: as plain launches the first time a lane meets a count (one-time
// kernel attribute set-up does not belong in a capture) and in graph mode 0, else as the lane's captured graph of that count.
// A graph is a single chain of kernel nodes -- the form the runtime replays without touching each node on the host; one
// graph with a branch per lane was measured at 4.2 us of host time per node, 670 us for the two chains of a batch of eight.
// The output head that follows a step in the same call (mynah_hip_decoder_step_head): with one lane it is enqueued behind the
// layers inside the lane's graph, two dependent graph nodes instead of two launches behind the graph.
struct HeadCall {
    const float *weight, *bias;
    size_t rows, vocab;
    float *const *dlogits;
    float *const *dprobs;
};
static unsigned long long head_signature_of(const State *st, const HeadCall &h, int count) {
    unsigned long long x = 0xcbf29ce484222325ull;
    const auto mix = [&](unsigned long long v) { x = (x ^ v) * 0x100000001b3ull; };
    mix((unsigned long long)st->qtype);   // the storage the head's weight is looked up under
    mix(reinterpret_cast<unsigned long long>(h.weight)); mix(reinterpret_cast<unsigned long long>(h.bias)); mix(h.rows); mix(h.vocab);
    for (int b = 0; b < count; ++b) {
        mix(reinterpret_cast<unsigned long long>(h.dlogits[b]));
        mix(h.dprobs != nullptr ? reinterpret_cast<unsigned long long>(h.dprobs[b]) : 0ull);
    }
    return x | 1ull;   // never 0
}
static int enqueue_head(State *st, mynah_hip_decoder *d, int count, const HeadCall &h, char *error, size_t capacity) {
    const float *hidden[kMaxBatch] = {};   // (not read: the product takes the residual rows and normalises them itself)
    return output_head_rows(st, hidden, (size_t)count, d->width, h.weight, h.bias, h.rows, h.vocab, h.dlogits, h.dprobs, d->x, d->norm_out, d->norm_out_b,
                            error, capacity, d->dev_slots);
}

static int run_lane(State *st, mynah_hip_decoder *lane, int count, hipStream_t stream, char *error, size_t capacity, bool with_end = true,
                    const HeadCall *head = nullptr) {
    hipStream_t main_stream = st->stream;
    st->stream = stream;   // the launch wrappers enqueue on the state's stream
    int rc = 0;
    const int form = head != nullptr ? 2 : with_end ? 0 : 1;
    const auto enqueue = [&]() {
        int r = enqueue_layers(st, lane, count, error, capacity, kAllStages, with_end);
        if (r == 0 && head != nullptr) r = enqueue_head(st, lane, count, *head, error, capacity);
        return r;
    };
    if (head != nullptr) {
        // another head, or other rows for its results, than this stream count's last step had: captured again, behind one
        // eager step (a weight seen for the first time is converted and uploaded there: no part of a capture)
        const unsigned long long signature = head_signature_of(st, *head, count);
        if (lane->head_signature[count] != signature) {
            if (lane->graphs[2][count] != nullptr) {
                (void)hipGraphExecDestroy(lane->graphs[2][count]);
                lane->graphs[2][count] = nullptr;
            }
            if (lane->head_signature[count] != 0) ++lane->head_recaptures;
            lane->eager_steps[2][count] = 0;
            lane->head_signature[count] = signature;
        }
    }
    if (st->graph_mode == 0 || lane->eager_steps[form][count] == 0) {
        lane->eager_steps[form][count] = 1;
        rc = enqueue();
    } else {
        hipGraphExec_t &exec = lane->graphs[form][count];
        if (exec == nullptr) {
            hipGraph_t graph = nullptr;
            rc = hip_check(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal), "begin capture", error, capacity);
            if (rc == 0) {
                rc = enqueue();
                const hipError_t end = hipStreamEndCapture(stream, &graph);
                if (rc == 0) rc = hip_check(end, "end capture", error, capacity);
                if (rc == 0) rc = hip_check(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "graph instantiate", error, capacity);
                if (graph != nullptr) (void)hipGraphDestroy(graph);
                if (rc != 0) exec = nullptr;
            }
        }
        if (rc == 0) rc = hip_check(hipGraphLaunch(exec, stream), "graph launch", error, capacity);
    }
    st->stream = main_stream;
    return rc;
}

// Every lane of a step: lane 0 on the backend's stream, the others on theirs, forked from and joined to it by events.
static int run_lanes(State *st, mynah_hip_decoder *d, const LanePlan &p, char *error, size_t capacity, bool with_end = true,
                     const HeadCall *head = nullptr) {
    hipStream_t main_stream = st->stream;
    if (p.lanes > 1) {
        MYNAH_TRY(hipEventRecord(st->lane_fork, main_stream));
        for (int i = 1; i < p.lanes; ++i) MYNAH_TRY(hipStreamWaitEvent(st->lane_streams[i], st->lane_fork, 0));
    }
    int rc = 0;
    for (int i = p.lanes - 1; i >= 0 && rc == 0; --i) {   // the owner's lane last: its stream is the one the caller's next work queues behind
        rc = run_lane(st, d->lanes[i], p.count[i], i == 0 ? main_stream : st->lane_streams[i], error, capacity, with_end, p.lanes == 1 ? head : nullptr);
        if (i > 0 && rc == 0) rc = hip_check(hipEventRecord(st->lane_done[i], st->lane_streams[i]), "lane event", error, capacity);
    }
    for (int i = 1; i < p.lanes && rc == 0; ++i) rc = hip_check(hipStreamWaitEvent(main_stream, st->lane_done[i], 0), "lane join", error, capacity);
    return rc;
}

}  // namespace mynah

namespace mynah {
// `count` consecutive step counters (24 bits, never 0).  When the counter wraps, the tags of 2^24 steps ago are forgotten
// first (outside any capture; the stream orders it).
int decoder_next_epochs(State *st, mynah_hip_decoder *d, unsigned count, unsigned *first, char *error, size_t capacity) {
    if (d->item_epoch + count >= 0xffffffu || d->item_epoch == 0) {
        if (d->self_records != nullptr) MYNAH_TRY(hipMemsetAsync(d->self_records, 0, d->records_bytes, st->stream));
        if (d->cross_records != nullptr) MYNAH_TRY(hipMemsetAsync(d->cross_records, 0, d->records_bytes, st->stream));
        d->item_epoch = 1;
    }
    *first = d->item_epoch;
    d->item_epoch += count;
    return 0;
}
}  // namespace mynah

// The step, with its end kernel (the final LayerNorm into every slot's output) or -- one lane, no persistent form -- without:
// *ended says which it was.
// head (optional): the output head to run behind the step; *head_done says whether the step took it along (one lane of stage
// kernels without the end kernel: the head is then part of the lane's graph), else the caller runs it.
static int decoder_step(State *st, mynah_hip_decoder *d, const mynah_hip_decoder_slot *slots, size_t batch, bool want_end, bool *ended, char *error,
                        size_t capacity, const HeadCall *head = nullptr, bool *head_done = nullptr) {
    *ended = true;
    if (head_done != nullptr) *head_done = false;
    if (batch == 0) return 0;   // src/graph.c:3132
    if (batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "decoder batch exceeds MYNAH_MAX_BATCH");   // src/graph.c:3133-3136
        return -1;
    }
    if (st == nullptr || d == nullptr || slots == nullptr) {
        set_error(error, capacity, "invalid decoder step arguments");
        return -1;
    }
    StepSlots s;
    memset(&s, 0, sizeof s);
    for (size_t b = 0; b < batch; ++b) {
        const mynah_hip_decoder_slot &in = slots[b];
        if (in.length >= d->capacity) {
            set_error(error, capacity, "decoder cache capacity exceeded");   // src/graph.c:3152-3155
            return -1;
        }
        if (in.dev_self_k == nullptr || in.dev_self_v == nullptr || in.dev_input == nullptr || in.dev_output == nullptr ||
            (d->xw != 0 && in.memory_length != 0 && (in.dev_cross_k == nullptr || in.dev_cross_v == nullptr))) {
            set_error(error, capacity, "decoder slot has a null buffer");
            return -1;
        }
        if (in.memory_length > d->capacity) {
            set_error(error, capacity, "decoder memory length exceeds the attention workspace (capacity)");
            return -1;
        }
        s.self_k[b] = in.dev_self_k;
        s.self_v[b] = in.dev_self_v;
        s.cross_k[b] = in.dev_cross_k;
        s.cross_v[b] = in.dev_cross_v;
        s.input[b] = in.dev_input;
        s.output[b] = in.dev_output;
        s.length[b] = (int)in.length;
        s.memory_length[b] = (int)in.memory_length;
    }
    const int B = (int)batch;
    st->last_step_decoder = d;   // kept so that the step can be repeated should one of its bounded waits give up (synchronise)
    st->last_step_slots = s;
    st->last_step_batch = B;
    ++st->steps_since_sync;
    st->calls_since_step = 0;
    {
        const int taken = try_persistent_step(st, d, slots, batch, error, capacity);
        if (taken != 0) return taken < 0 ? -1 : 0;
    }
    const int lanes = lanes_for(st, d, B);
    if (ensure_lanes(st, d, lanes, error, capacity) != 0) return -1;
    const bool with_end = want_end || lanes != 1 || !d->fused_attention;
    *ended = with_end;
    // (a caller that hands over other rows for the results at every step would have the graph captured at every step)
    static const bool head_in_graph = !(getenv("MYNAH_HIP_HEAD_IN_GRAPH") != nullptr && strcmp(getenv("MYNAH_HIP_HEAD_IN_GRAPH"), "0") == 0);
    const bool head_along = head_in_graph && head != nullptr && !with_end && head_done != nullptr && d->head_recaptures < 8;
    if (head_along) *head_done = true;
    const LanePlan plan = plan_lanes(s, B, lanes);
    d->last_batch_slots = s;
    d->last_lanes = lanes;
    d->last_batch = B;
    for (int i = 0; i < lanes; ++i) {
        mynah_hip_decoder *lane = d->lanes[i];
        StepSlots ls = lanes == 1 ? s : lane_slots(s, plan, i);
        if (decoder_next_epochs(st, lane, 1, &ls.epoch, error, capacity) != 0) return -1;
        lane->last_slots = ls;
        if (launch_step_begin(st, ls, lane->dev_slots, plan.count[i], d->width, d->position, lane->x, d->width, decoder_item_tables(lane, plan.count[i]), error,
                              capacity) != 0)
            return -1;
    }
    return run_lanes(st, d, plan, error, capacity, with_end, head_along ? head : nullptr);
}

extern "C" int mynah_hip_decoder_step(void *opaque, mynah_hip_decoder *d, const mynah_hip_decoder_slot *slots, size_t batch,
                                      char *error, size_t capacity) {
    State *st = enter_state(opaque);
    bool ended = true;
    return decoder_step(st, d, slots, batch, true, &ended, error, capacity);
}

// The step and the output head in one call.  Where the step runs as one lane of stage kernels, its end kernel is left out and
// the head's product does the final LayerNorm in its prologue -- it reads the residual rows, and its first workgroup writes
// every stream's normalised row to the slot's output, so the caller finds there what mynah_hip_decoder_step leaves -- which
// takes one dependent launch off the step.  Elsewhere (lanes, the persistent form, head shapes the matvec does not take) the
// two calls run one after the other.  A step whose bounded wait gives up is reported, not repeated: the head has consumed it.
extern "C" int mynah_hip_decoder_step_head(void *opaque, mynah_hip_decoder *d, const mynah_hip_decoder_slot *slots, size_t batch, const float *weight,
                                           const float *bias, size_t rows, size_t vocab, float *const *dlogits, float *const *dprobs, char *error,
                                           size_t capacity) {
    State *st = enter_state(opaque);
    if (batch == 0) return 0;
    if (st == nullptr || d == nullptr || slots == nullptr || weight == nullptr || dlogits == nullptr || vocab == 0 || rows % vocab != 0 || rows == 0 ||
        batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "invalid decoder step + head arguments");
        return -1;
    }
    const float *hidden[kMaxBatch];
    for (size_t b = 0; b < batch; ++b) hidden[b] = slots[b].dev_output;
    // (the fused form's product takes one weight pass and the matvec's shapes; the decision must precede the step)
    const bool fusable = batch <= (size_t)kBatchTile && d->norm_out != nullptr && linear_fast_supported(st->qtype, rows, d->width) && rows <= 0x7fffffffu;
    bool ended = true, head_done = false;
    const HeadCall head{weight, bias, rows, vocab, dlogits, dprobs};
    if (decoder_step(st, d, slots, batch, !fusable, &ended, error, capacity, fusable ? &head : nullptr, &head_done) != 0) return -1;
    if (head_done) {
        st->last_step_decoder = nullptr;   // (not repeatable behind the head)
        return 0;
    }
    if (ended) return output_head_rows(st, hidden, batch, d->width, weight, bias, rows, vocab, dlogits, dprobs, nullptr, nullptr, nullptr, error, capacity);
    st->last_step_decoder = nullptr;   // (not repeatable behind the head)
    return output_head_rows(st, hidden, batch, d->width, weight, bias, rows, vocab, dlogits, dprobs, d->x, d->norm_out, d->norm_out_b, error, capacity,
                            d->dev_slots);
}

int mynah::rerun_last_step_without_waits(State *st, char *error, size_t capacity) {
    mynah_hip_decoder *d = st->last_step_decoder;
    const int B = st->last_step_batch;
    if (d == nullptr || B < 1 || B > kMaxBatch) {
        set_error(error, capacity, "no resident step to repeat");
        return -1;
    }
    StepSlots s = st->last_step_slots;
    s.epoch = 1;
    // One lane, every kernel a launch of its own, and no record areas: the attention launches then take the build that
    // finds its work from the workgroup index and a fold kernel follows each of them -- nothing in this form waits for
    // another workgroup.  The arithmetic is the one of every other form, so these are the bits the step would have given.
    unsigned long long *const self_records = d->self_records, *const cross_records = d->cross_records;
    d->self_records = d->cross_records = nullptr;
    int rc = launch_step_begin(st, s, d->dev_slots, B, d->width, d->position, d->x, d->width, StepItemTables{}, error, capacity);
    if (rc == 0) rc = enqueue_layers(st, d, B, error, capacity);
    d->self_records = self_records;
    d->cross_records = cross_records;
    d->last_batch_slots = s;
    d->last_lanes = 1;
    d->last_batch = B;
    return rc;
}

// Parity probe: one step of one or two streams as plain launches in one lane, with the int8 activations and activation scale
// of stream 0 at every projection written to the caller's device buffers -- what lets a CPU restatement be run on the very
// integers the device used.  Same kernels and arithmetic as mynah_hip_decoder_step (the matvec launches take the build that
// carries the probe stores); not part of the decode path.
extern "C" int mynah_hip_decoder_step_probe(void *opaque, mynah_hip_decoder *d, const mynah_hip_decoder_slot *slots, size_t batch, int8_t *dev_qx,
                                            float *dev_sx, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (st == nullptr || d == nullptr || slots == nullptr || dev_qx == nullptr || dev_sx == nullptr || batch < 1 || batch > (size_t)kConsumerFoldMaxBatch) {
        set_error(error, capacity, "step probe: one or two streams and both probe buffers");
        return -1;
    }
    if (!d->fused_attention || (d->qtype != MYNAH_HIP_INT8 && d->qtype != MYNAH_HIP_INT4)) {
        set_error(error, capacity, "step probe: int8 / int4 weights and 64-wide heads only");
        return -1;
    }
    StepSlots s;
    memset(&s, 0, sizeof s);
    for (size_t b = 0; b < batch; ++b) {
        const mynah_hip_decoder_slot &in = slots[b];
        if (in.length >= d->capacity || in.memory_length > d->capacity || in.dev_self_k == nullptr || in.dev_self_v == nullptr || in.dev_input == nullptr ||
            in.dev_output == nullptr || (d->xw != 0 && in.memory_length != 0 && (in.dev_cross_k == nullptr || in.dev_cross_v == nullptr))) {
            set_error(error, capacity, "step probe: invalid slot");
            return -1;
        }
        s.self_k[b] = in.dev_self_k; s.self_v[b] = in.dev_self_v; s.cross_k[b] = in.dev_cross_k; s.cross_v[b] = in.dev_cross_v;
        s.input[b] = in.dev_input; s.output[b] = in.dev_output; s.length[b] = (int)in.length; s.memory_length[b] = (int)in.memory_length;
    }
    s.epoch = 1;
    d->last_batch_slots = s;
    d->last_lanes = 1;
    d->last_batch = (int)batch;
    if (launch_step_begin(st, s, d->dev_slots, (int)batch, d->width, d->position, d->x, d->width, StepItemTables{}, error, capacity) != 0) return -1;
    d->probe_qx = dev_qx;
    d->probe_sx = dev_sx;
    const int rc = enqueue_layers(st, d, (int)batch, error, capacity);
    d->probe_qx = nullptr;
    d->probe_sx = nullptr;
    return rc;
}

// Measurement helper: enqueue ONE stage of the step (all layers, back to back, as its own captured graph) on the
// backend's stream, reusing the slot table of the last mynah_hip_decoder_step with this batch size.  The kernels,
// their arguments and their order among themselves are those of the real step; only the other stages are left out,
// so a caller can bracket a loop of these with mynah_hip_timer_begin / _end and get that kernel's launch time in the
// step's own setting (dependent graph nodes, weights and caches coming from HBM).  It perturbs the decoder's
// workspaces (x, hidden) like a step does and is not part of the decode path.
extern "C" int mynah_hip_decoder_stage_enqueue(void *opaque, mynah_hip_decoder *d, size_t batch, int stage, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (st == nullptr || d == nullptr || batch == 0 || batch > (size_t)kMaxBatch || stage < 0 || stage >= MYNAH_HIP_STAGE_COUNT) {
        set_error(error, capacity, "invalid stage arguments");
        return -1;
    }
    if (!d->fused_attention || d->last_batch != (int)batch) {
        set_error(error, capacity, "stage timing needs the fused step and follows a step with this batch size");
        return -1;
    }
    if ((stage == MYNAH_HIP_STAGE_CROSS_ATTENTION || stage == MYNAH_HIP_STAGE_CROSS_OUT) && d->xw == 0) {
        set_error(error, capacity, "decoder has no cross-attention sublayer");
        return -1;
    }
    hipGraphExec_t &exec = d->stage_graphs[stage][batch];
    // The stage runs in one lane whatever the step does: when the last step ran in several, the owner's slot table holds one
    // lane's streams only and is rewritten for the whole batch first.  A fresh step counter, as every real step has one, for the
    // attention launches that fold their own partials: the workgroups that wait for tagged values then really wait.
    const bool attention_stage = stage == MYNAH_HIP_STAGE_SELF_ATTENTION || stage == MYNAH_HIP_STAGE_CROSS_ATTENTION;
    if (d->last_lanes > 1 || exec == nullptr || (batch > (size_t)kConsumerFoldMaxBatch && attention_stage)) {
        if (decoder_next_epochs(st, d, 1, &d->last_batch_slots.epoch, error, capacity) != 0) return -1;
        if (launch_step_begin(st, d->last_batch_slots, d->dev_slots, (int)batch, d->width, d->position, d->x, d->width, decoder_item_tables(d, (int)batch),
                              error, capacity) != 0)
            return -1;
    }
    if (exec == nullptr) {
        // once as plain launches (one-time kernel attributes of this batch size's builds do not belong in a capture)
        if (enqueue_layers(st, d, (int)batch, error, capacity, 1u << stage) != 0) return -1;
        hipGraph_t graph = nullptr;
        MYNAH_TRY(hipStreamBeginCapture(st->stream, hipStreamCaptureModeThreadLocal));
        const int rc = enqueue_layers(st, d, (int)batch, error, capacity, 1u << stage);
        const hipError_t end = hipStreamEndCapture(st->stream, &graph);
        if (rc != 0) {
            if (graph != nullptr) (void)hipGraphDestroy(graph);
            return -1;
        }
        MYNAH_TRY(end);
        const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (hip_check(inst, "stage graph instantiate", error, capacity) != 0) {
            exec = nullptr;
            return -1;
        }
    }
    return hip_check(hipGraphLaunch(exec, st->stream), "stage graph launch", error, capacity);
}
