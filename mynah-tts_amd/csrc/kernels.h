// Launch wrappers of the device kernels (kernels_linear.hip, kernels_attention.hip, kernels_misc.hip).
#pragma once

#include "common.h"

namespace mynah {

enum { EPI_NONE = 0, EPI_GELU = 1, EPI_RESIDUAL = 2 };

// One weight-stationary pass: out[b][n] = epilogue(W * prologue(in[b])) for up to kBatchTile streams.
struct LinearArgs {
    const void *w;          // packed weight, storage `qtype`
    const float *scales;    // int8 [n] | int4 [n, k/32]
    const float *bias;      // [n] or null
    int qtype;
    int n, k;
    int batch;              // streams in this pass (<= kBatchTile)
    const float *in[kBatchTile];
    float *out[kBatchTile];
    const float *ln_gain;   // non-null: LayerNorm prologue (eps 1e-5)
    const float *ln_bias;   // may be null
    int epilogue;           // EPI_*
    int arith;              // MYNAH_HIP_ARITH_*: how the activation scale is formed
    // Resident step only: take in[b] from the fold of split-L attention partials instead of a device row
    // (stream fold_stream0 + b of the slot table; see kernels_step_attention.hip).
    const float *fold_partial;
    const float *fold_partial_ml;
    const StepSlots *fold_slots;
    int fold_heads, fold_head_width, fold_max_units, fold_is_self, fold_stream0;
    int8_t *probe_qx;       // parity probes (null in production)
    float *probe_sx;
    int32_t *probe_acc;
    // Seam calls folded into one launch (single row only): ln_out receives the LayerNorm prologue's row, aux_out the
    // value of the product before the residual epilogue adds it -- the buffers the separate calls would have written.
    float *ln_out;
    // The same for every stream of a launch: stream b's LayerNorm row goes to ln_out_slots->output[b] (the resident step's
    // final LayerNorm done by the output head's product, which then stands in for the step's end kernel).
    const StepSlots *ln_out_slots;
    float *aux_out;
    float *act_out;         // the input row as the prologue formed it (the fold of attention partials), before any LayerNorm
};

// True when the fused matvec kernel supports this shape/storage; otherwise use linear_generic.
bool linear_fast_supported(int qtype, size_t n, size_t k);
int launch_linear(State *st, const LinearArgs &args, char *error, size_t capacity);
// Any shape, f32 weights: out[r,n] = in[r,k] W[n,k]^T + bias (rows may be large).
int launch_gemm_f32(State *st, const float *in, float *out, size_t rows, size_t k, size_t n, const float *w,
                    const float *bias, char *error, size_t capacity);
int launch_sgemm(State *st, int ta, int tb, size_t m, size_t n, size_t k, float alpha, const float *a, size_t lda,
                 const float *b, size_t ldb, float beta, float *c, size_t ldc, char *error, size_t capacity);

// Single-token attention for up to kMaxBatch streams.  Pointers come either from the by-value table
// (seam calls) or from `slots` in device memory (resident step, replayable as a graph).
struct AttnArgs {
    const StepSlots *slots;        // non-null: resident-step mode
    size_t layer;                  // slots mode: cache offsets are layer * capacity * stride etc.
    size_t capacity;
    const float *q[kMaxBatch];     // table mode: q rows (self: the qkv row)
    float *k_cache[kMaxBatch];
    float *v_cache[kMaxBatch];
    float *out[kMaxBatch];
    int position[kMaxBatch];       // self only: row to append
    int valid[kMaxBatch];
    int batch;
    int heads, head_width;
    int stride;                    // floats between cache rows
    int q_stride;                  // slots mode: floats between streams in the q/qkv and out workspaces
    float scale;
    int is_self;
    int max_chunks;                // grid.x
    // Consumer-side fold (single-stream seam calls): instead of folding, every chunk leaves its partial in the layout
    // the fused matvec's fold prologue reads -- unit_partial [stream][head][max_chunks][head_width], unit_ml [stream][head][2][max_chunks]
    // -- per stream, and the stream's chunk count, as "rows" of kStepUnitRows per chunk, in unit_slots->memory_length[stream].
    float *unit_partial;
    float *unit_ml;
    StepSlots *unit_slots;
    int two_pass;                  // set by launch_attention: the fold is a launch of its own (no arrival counters)
    int chunk_rows;                // cache rows per workgroup: 0 / kAttnChunk, or kWideRows (from attention_chunk_rows)
    float *partial;                // [batch, heads, max_chunks, head_width + 2]
    unsigned *counters;            // [batch, heads], zero between launches
};
int launch_attention(State *st, const AttnArgs &args, char *error, size_t capacity);
// Folds partials left in the unit layout into out[heads * head_width] (what the consumer's prologue would have formed).
int launch_unit_fold(State *st, const float *partial, const float *ml, const StepSlots *slots, int heads, int head_width,
                     int max_units, float *out, char *error, size_t capacity);
int launch_unit_fold_streams(State *st, const AttnArgs &args, char *error, size_t capacity);
int attention_chunk_rows(int is_self, size_t head_width, bool vector_rows, size_t max_valid);

// Resident step: LayerNorm + activation quantisation + this head's slice of the Q (self: Q, K, V) projection +
// attention over one cache chunk, per workgroup; writes split-L partials that the next matvec folds.
// What one workgroup of a many-stream attention grid does: written once per pass through the layers, read by that workgroup.
struct StepItem {
    float *k, *v;      // the stream's K and V cache (self or cross), all layers
    int length;        // rows in it before this step
    int code;          // head | stream << 8 | unit << 16, or -1: nothing to do
    int epoch;         // step counter (24 bits): with the layer, the tag of what workgroups of one launch hand each other
    int group;         // consecutive cache chunks a chunk workgroup takes (unit u: chunks group * (u - first) ..)
};
struct StepAttnArgs {
    const StepSlots *slots;
    const StepItem *items;    // batch > kConsumerFoldMaxBatch: one entry per workgroup of this launch's grid
    const float *x;           // [batch, width] residual stream
    int batch, width;
    const float *ln_gain, *ln_bias;
    const void *w;            // self: [3*width, width] qkv weight; cross: [heads*head_width, width] q weight
    const float *scales;
    int qtype, arith;
    int is_self;
    int heads, head_width;
    size_t layer, capacity;   // cache addressing (self: rows `capacity` apart per layer; cross: memory_length)
    int max_units;            // per stream, incl. the new-row unit for self-attention
    float scale;
    float *partial;           // partial outputs [batch, heads, max_units, head_width]
    float *partial_ml;        // chunk maxima and sums [batch, heads, 2, max_units]
    // many streams, fold inside the launch: the partials as tagged records [batch, heads, max_units, kStepRecord] (non-null
    // selects this form), the folded rows [batch, heads * head_width], and the bound of the fold workgroups' wait
    unsigned long long *records;
    float *fold_out;
    unsigned spin_limit;
    unsigned *abort_word;
    // parity probes (null in production): the int8 activations and the activation scale of stream 0, as this launch quantised them
    int8_t *probe_qx;
    float *probe_sx;
};
int launch_step_attention(State *st, const StepAttnArgs &args, char *error, size_t capacity);
// Workgroups of the attention launch for this shape (the table below has as many entries).
int step_attention_grid(int heads, int batch, int max_units, int is_self, bool packed);
// Both work tables of one pass through the layers, as the kernel that starts the pass needs them to fill them (extra
// workgroups of its grid run write_step_item of step_items.h, one entry per thread).  No entries: the batch size takes no
// tables.  self_slots / cross_slots: workgroups of the attention kernel that the device holds at once.
struct StepItemTables {
    StepItem *self_items, *cross_items;
    int self_entries, cross_entries;
    int batch, heads, cross_heads;
    int with_fold, self_budget, cross_budget;
};
StepItemTables step_item_tables(int batch, int heads, int cross_heads, int max_units, StepItem *self_items, StepItem *cross_items, bool with_fold,
                                int self_slots, int cross_slots);
inline unsigned step_item_workgroups(const StepItemTables &t) { return (unsigned)((t.self_entries + t.cross_entries + 255) / 256); }
// Workgroups of the many-stream attention kernel for this weight storage and shape that the device holds at once.
int step_attention_slots(int qtype, int width, int max_units, int is_self, bool with_fold);
// LDS a fold workgroup needs: the launch's dynamic LDS is at least this when it folds its own partials.
size_t step_fold_lds_bytes(int max_units);
// Folds the partials of the same arguments into out[batch][heads * head_width] (large batches only).
int launch_step_fold(State *st, const StepAttnArgs &args, float *out, char *error, size_t capacity);
bool step_attention_supported(int qtype, size_t width, size_t heads, size_t head_width);

// The whole resident step as one persistent launch (kernels_step_persistent.hip): one or two streams, int8 / int4 weights,
// the decoder stack's own shape (width 768, FFN 3072, 64-wide heads).
struct PersistLayer {   // one per layer, in device memory
    const void *qkv_w, *o_w, *qx_w, *ox_w, *up_w, *down_w;
    const float *qkv_s, *o_s, *qx_s, *ox_s, *up_s, *down_s;
    const float *norm_self, *norm_self_b, *norm_cross, *norm_cross_b, *norm_ff, *norm_ff_b;
};
struct PersistArgs {
    const PersistLayer *layers;
    int n_layers, batch, heads, cross_heads, arith;
    size_t capacity;
    int max_units;                  // partial records per (stream, head) the exchange area holds
    float scale;
    float *self_k[2], *self_v[2];
    const float *cross_k[2], *cross_v[2];
    const float *input[2];
    float *output[2];
    int length[2], memory_length[2];
    const float *position, *norm_out, *norm_out_b;
    unsigned long long *exchange;   // tagged vectors and partial records (step_persistent_exchange_words of them)
    unsigned epoch;                 // tags of this step start here; a step uses 8 * (layers + 1) of them
    unsigned spin_limit;            // polls a wait may make before the step is given up
    unsigned *abort_word;           // set when a wait gave up (host-visible)
    int attention_wgs;              // workgroups [0, attention_wgs) run the attention stages, the row stages count from the grid's end
    int wgs_out, rows_out;          // workgroups and rows per workgroup of the [768, 768] output projections
    int wgs_up, rows_up;            // ... of FFN up [3072, 768]
    int wgs_down, rows_down;        // ... of FFN down [768, 3072]
};
bool step_persistent_supported(int qtype, size_t width, size_t heads, size_t head_width, size_t ffn, size_t cross_heads, size_t cross_head_width);
size_t step_persistent_exchange_words(const PersistArgs &args);
int step_persistent_attention_workgroups(const PersistArgs &args);
bool step_persistent_fits(const PersistArgs &args, int grid);
int launch_step_persistent(State *st, const PersistArgs &args, int qtype, int grid, char *error, size_t capacity);

int launch_layernorm(State *st, const float *in, float *out, const float *gain, const float *bias, size_t rows,
                     size_t width, char *error, size_t capacity);
int launch_gelu(State *st, float *data, size_t n, char *error, size_t capacity);
int launch_residual(State *st, float *out, const float *in, size_t n, char *error, size_t capacity);
int launch_copy(State *st, float *dst, const float *src, size_t n, char *error, size_t capacity);
int launch_scale(State *st, float *data, size_t n, float scale, char *error, size_t capacity);
int launch_clip(State *st, float *data, size_t n, char *error, size_t capacity);
int launch_softmax(State *st, float *data, size_t rows, size_t cols, size_t valid, char *error, size_t capacity);
int launch_softmax_heads(State *st, const float *const *logits, float *const *probs, size_t streams, size_t rows, size_t cols, char *error,
                         size_t capacity);
int launch_argmax(State *st, const float *logits, size_t vocab, size_t codebook, size_t eos, int allow_eos,
                  unsigned *dev_result, char *error, size_t capacity);
int launch_gather(State *st, const float *const *dev_tables, size_t table_count, const int32_t *dev_ids,
                  size_t tokens, size_t width, float scale, const float *dev_position, float *out, char *error,
                  size_t capacity);
int launch_stream_copy(State *st, const void *src, void *dst, size_t bytes, char *error, size_t capacity);

// Token choice of the decoder head for `batch` slots (kernels_misc.hip).
struct HeadArgmaxArgs {
    const float *logits[kMaxBatch];   // [streams, vocab] per slot
    int forbid_eos[kMaxBatch];
    int streams, vocab, codebook_size, eos_id, codebook_count;
    unsigned *values, *stored;        // device [batch, streams]
    int *saw_eos;                     // device [batch]
    unsigned long long *eos_frame;    // device [batch], ~0 = none
};
int launch_head_argmax(State *st, const HeadArgmaxArgs &args, int batch, char *error, size_t capacity);
// Resident step: writes the slot table to device memory, forms x[b] = input[b] + position[length[b]] and fills the work
// tables of the step's many-stream attention launches (step counter: the slot table's).
int launch_step_begin(State *st, const StepSlots &slots, StepSlots *dev_slots, int batch, size_t width,
                      const float *dev_position, float *x, size_t x_stride, const StepItemTables &tables, char *error, size_t capacity);
// Final norm of the step: out = slots->output[b]; gain may be null (plain copy).
int launch_step_end(State *st, const StepSlots *dev_slots, int batch, size_t width, const float *x, size_t x_stride,
                    const float *gain, const float *bias, char *error, size_t capacity);

// Resident decoder internals for a caller that drives the layers itself (the local frame): the residual rows
// x[kMaxBatch][width] the layer kernels read and update, the device slot table they take caches and lengths from,
// and the device position table.  decoder_enqueue_layers puts one step's layer kernels on the stream -- no begin
// kernel, no output kernel, no graph launch -- and may be captured once every kernel shape has run eagerly.  The caller's
// own kernels fill the work tables decoder_item_tables names before each pass (no entries: none needed at this batch size).
struct DecoderRows {
    float *x;
    StepSlots *slots;
    const float *position;
};
DecoderRows decoder_rows(mynah_hip_decoder *decoder);
// A caller that runs the layers several times per slot table gives each pass's tables a step counter of its own:
// decoder_next_epochs reserves `count` consecutive counters and returns the first.
StepItemTables decoder_item_tables(mynah_hip_decoder *decoder, int batch);
int decoder_enqueue_layers(State *st, mynah_hip_decoder *decoder, int batch, char *error, size_t capacity);
int decoder_next_epochs(State *st, mynah_hip_decoder *decoder, unsigned count, unsigned *first, char *error, size_t capacity);

}  // namespace mynah
