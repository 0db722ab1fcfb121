// Shared host/device definitions for the gfx950 backend.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <cstdio>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/mynah_hip.h"

namespace mynah {

constexpr int kWave = 64;            // CDNA wavefront
constexpr int kMaxBatch = MYNAH_HIP_MAX_BATCH;
constexpr int kBatchTile = 8;        // streams served by one pass over a weight tile
constexpr size_t kQuantMaxRows = 16; // QMAT_SMALL_COUNT, src/qmat.c:32
constexpr size_t kQuantMaxK = 8192;  // QMAT_K_MAX, src/qmat.c:33
constexpr int kWideRows = 16;        // the same for their wide-head form (one wavefront per row)
constexpr int kAttnChunk = 64;       // cache positions handled by one workgroup of the stand-alone attention kernels
constexpr int kStepUnitRows = 128;   // cache rows per attention unit (workgroup) of the fused resident step
// Up to this many streams the resident step is laid out for latency: the output projection folds the attention
// partials itself and attention workgroups request their weights before looking at the slot table.  Above it a
// separate fold kernel runs once (every workgroup folding every stream would outweigh one extra launch) and
// workgroups of units a stream does not have leave before requesting anything.
constexpr int kConsumerFoldMaxBatch = 2;
constexpr int kMaxLanes = 3;         // groups of a batch's streams that step side by side, each on a stream of its own (a process has four
                                     // hardware queues here: with a fourth stream in use two of them share one, and chains that share a queue run one after the other)
constexpr int kLaneStreams = 8;      // streams per lane when the caller names no lane count: one weight pass serves eight, so nine to sixteen streams step
                                     // as two lanes (measured, sixteen uniform streams: 1048 us in one lane, 856 us in two, 942 us in three; eight ragged
                                     // streams: 602 / 596 / 633 us -- a lane of four takes 480 us alone, and two chains side by side 1.24 times one)
constexpr int kStepRecord = 68;      // 64-bit slots of one attention partial of the persistent step: out[64] | max | sum | two unused

// ---- error plumbing (0 / -1 + message, src/backend.c:137-139) ----
inline void set_error(char *error, size_t capacity, const char *message) {
    if (error != nullptr && capacity > 0) snprintf(error, capacity, "%s", message);
}
inline int hip_check(hipError_t r, const char *what, char *error, size_t capacity) {
    if (r == hipSuccess) return 0;
    if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP %s: %s", what, hipGetErrorString(r));
    return -1;
}
#define MYNAH_TRY(expr) do { if (hip_check((expr), #expr, error, capacity) != 0) return -1; } while (0)
struct State;
// Stream synchronisation that also reports a failure an earlier call could not return (backend_hip.hip).
int synchronise(State *st, char *error, size_t capacity);
#define MYNAH_NEED_STATE(st) do { if ((st) == nullptr) { set_error(error, capacity, "backend state is null"); return -1; } } while (0)

// ---- device-resident copy of one host tensor, converted at first sight ----
struct CachedWeight {
    int qtype = MYNAH_HIP_F32;   // storage actually used
    size_t n = 0, k = 0;
    void *data = nullptr;        // f32 [n,k] | int8 [n,k] | nibbles [n,k/2] | f16 [n,k]
    float *scales = nullptr;     // int8 [n] | int4 [n,k/32]
    size_t bytes = 0;
    int arith = 0;               // quantiser arithmetic the values were formed with (int8 / int4)
    uint64_t fingerprint = 0;    // of the f32 tensor it was converted from (converted storages only; weight_pack.cpp)
};

// One entry of a packed-weight file, waiting in host memory for the tensor it belongs to (weight_pack.cpp).
struct PackKey {
    uint64_t fingerprint, n, k;
    int qtype, arith;
    bool operator==(const PackKey &o) const { return fingerprint == o.fingerprint && n == o.n && k == o.k && qtype == o.qtype && arith == o.arith; }
};
struct PackKeyHash {
    size_t operator()(const PackKey &p) const { return (size_t)(p.fingerprint ^ (p.n * 0x9e3779b97f4a7c15ull) ^ (p.k << 20) ^ ((uint64_t)p.qtype << 60) ^ ((uint64_t)p.arith << 59)); }
};
struct PackedWeight {
    std::vector<unsigned char> values;
    std::vector<float> scales;
};

struct WeightKey {
    const void *host;
    size_t bytes;
    int kind;   // 0 plain f32 vector/matrix, 1 + qtype*2 + arith for converted matrices, 64 + kernel + 32 * in_ch for conv1d chunks
    bool operator==(const WeightKey &o) const { return host == o.host && bytes == o.bytes && kind == o.kind; }
};
struct WeightKeyHash {
    size_t operator()(const WeightKey &k) const {
        return std::hash<const void *>()(k.host) ^ (k.bytes * 0x9e3779b97f4a7c15ull) ^ ((size_t)k.kind << 56);
    }
};

// Per-step dynamic data of the resident decode step; lives in device memory so a captured graph can
// be replayed with new lengths and pointers.
struct StepSlots {
    float *self_k[kMaxBatch];
    float *self_v[kMaxBatch];
    const float *cross_k[kMaxBatch];
    const float *cross_v[kMaxBatch];
    const float *input[kMaxBatch];
    float *output[kMaxBatch];
    int length[kMaxBatch];
    int memory_length[kMaxBatch];
    unsigned epoch;   // step counter (24 bits, never 0): goes into the tags of what workgroups of one launch hand each other
};

// A seam call held back for one call so that the next one can join its launch (backend_hip.hip, "seam fusion").
struct PendingOp {
    enum { kNone = 0, kLayerNorm = 1, kLinear = 2, kAttentionFold = 3 };
    int kind = kNone;
    // LayerNorm of one row (alone, or as the prologue of the product)
    const float *ln_in = nullptr;
    float *ln_out = nullptr;
    const float *ln_gain = nullptr, *ln_bias = nullptr;   // device copies
    // product of one row
    bool has_ln = false;
    const float *in = nullptr;
    float *out = nullptr;
    size_t iw = 0, ow = 0;
    const CachedWeight *weight = nullptr;
    const float *bias = nullptr;                           // device copy
    // attention whose chunks are still to be folded (alone, or as the prologue of the product that reads its output row)
    bool has_fold = false;
    float *fold_out = nullptr;
    const float *fold_partial = nullptr, *fold_ml = nullptr;
    int fold_heads = 0, fold_head_width = 0, fold_max_units = 0;
};

// Device copy of the leading rows of a host position table (mynah_hip_embed_gather).
struct PositionTable {
    float *data = nullptr;
    size_t capacity_rows = 0, filled_rows = 0;
};

struct State {
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    int cu_count = 256;
    int qtype = MYNAH_HIP_F32;
    int arith = MYNAH_HIP_ARITH_STRICT;
    // The last resident step since the stream was last waited for, kept so that it can be run again in the form without waits
    // between workgroups should one of its bounded waits give up: its decoder, every stream's slot, how many steps were
    // enqueued since the last synchronisation (only a single one can be repeated: the inputs of earlier ones may be gone),
    // whether anything was enqueued behind it (that work has read the step's rows and cannot be repeated from here), and how
    // often a step was repeated.
    mynah_hip_decoder *last_step_decoder = nullptr;
    StepSlots last_step_slots;
    int last_step_batch = 0;
    unsigned steps_since_sync = 0;
    unsigned calls_since_step = 0;   // entry points since that step that may have put work behind it (work that has read its rows)
    bool rerunning = false;
    unsigned long long wait_fallbacks = 0;
    int step_lanes = 0;   // lanes of a resident step above two streams (0: chosen from the batch size)
    // the streams lanes 1.. step on, and the events that fork them from and join them to `stream` (created at first use, shared
    // by every decoder of the backend: more streams would not mean more hardware queues)
    hipStream_t lane_streams[kMaxLanes] = {};
    hipEvent_t lane_fork = nullptr, lane_done[kMaxLanes] = {};
    int graph_mode = 1;   // resident step: 0 = every stage kernel a launch, 1 = captured graph, 2 = one persistent launch where it applies (else graph)
    // persistent step: word a workgroup sets when a bounded wait gave up (pinned host memory, mapped), polls a wait may make,
    // and an override of the row stages' workgroup count (0 = chosen from the batch)
    unsigned *persist_abort_host = nullptr;
    unsigned *persist_abort_dev = nullptr;
    unsigned persist_spin_limit = 1u << 20;
    int persist_row_wgs = 0;
    std::mutex mu;
    std::unordered_map<WeightKey, CachedWeight, WeightKeyHash> weights;
    size_t weight_bytes = 0;
    std::unordered_map<PackKey, PackedWeight, PackKeyHash> packs;   // entries of imported packed-weight files not yet taken
    size_t pack_hits = 0;                                           // weights that came out of such a file instead of a conversion
    int pack_verify = 0;                                            // MYNAH_HIP_PACK_VERIFY: convert anyway and compare
    std::map<std::pair<const float *, size_t>, PositionTable> position_tables;   // by (host table, width)
    float *head_logits = nullptr;        // logits of mynah_hip_head_argmax, [kMaxBatch, rows] (grown on demand)
    size_t head_logits_floats = 0;
    void *head_result = nullptr;         // its results on the device: values | stored | saw_eos | eos_frame
    size_t head_result_bytes = 0;
    std::vector<void *> pending_free;   // from mynah_hip_dev_free, freed at the next synchronisation
    // upload scratch (src/backend.h:78-81) and pinned staging for h2d/d2h
    float *scratch = nullptr;
    size_t scratch_bytes = 0;
    void *pinned = nullptr;
    size_t pinned_bytes = 0;
    // normalised encoder memory of mynah_hip_cross_kv_dev (grown on demand; an outgrown one waits in pending_free)
    float *cross_norm = nullptr;
    size_t cross_norm_floats = 0;
    // cache-flush buffer
    void *flush = nullptr;
    size_t flush_bytes = 0;
    // attention split-L partials + arrival counters
    float *attn_partial = nullptr;
    size_t attn_partial_floats = 0;
    unsigned *attn_counters = nullptr;
    // this device's address of the library's fixed scratch array (the allocation-free entry point's workspace)
    void *noalloc = nullptr;
    // small device block for batched pointer tables of the section-2 calls
    void *ptr_table = nullptr;
    void *ptr_table_host = nullptr;   // pinned
    // result word of the argmax operator: its own allocation, so that it can never alias a caller's upload buffer
    unsigned *argmax_result = nullptr;
    // seam fusion: the held-back call, whether holding back is on (MYNAH_HIP_FUSE=0 turns it off), and the message of a
    // held-back launch that failed where no caller could be told (reported by the next sync)
    PendingOp pending;
    StepSlots *seam_slots = nullptr;   // device word the chunk count of a held-back fold travels in
    int fuse = 1;
    char deferred_error[160] = {0};
};

// The stream of lane `lane` (0: the backend's own), created at first use (backend_hip.hip).
int lane_stream(State *st, int lane, hipStream_t *stream, char *error, size_t capacity);

// Runs the step recorded in the state again, as plain launches in the form whose workgroups never wait for each other (fold
// kernel behind the attention launches, no persistent launch); the cache rows it appends are the ones the first run wrote to
// (decoder_step.hip).
// The output head on normalised rows, or on residual rows with the final LayerNorm as the product's prologue (backend_hip.hip).
int output_head_rows(State *st, const float *const *dhidden, size_t batch, size_t width, const float *weight, const float *bias, size_t rows,
                     size_t vocab, float *const *dlogits, float *const *dprobs, const float *x_rows, const float *ln_gain, const float *ln_bias,
                     char *error, size_t capacity, const StepSlots *ln_out_slots = nullptr);
int rerun_last_step_without_waits(State *st, char *error, size_t capacity);

// First statement of every entry point that is not itself part of the seam fusion: launches what is held back, so that
// the stream holds every earlier call's work before this one adds its own.
// `enqueues`: the entry point may put work on the stream (false for those that only wait or copy to the host).
State *enter_state(void *opaque, bool enqueues = true);

// weight cache (backend_hip.hip)
int cached_matrix(State *st, const float *host, size_t n, size_t k, int want_qtype, const CachedWeight **out,
                  char *error, size_t capacity);
int cached_vector(State *st, const float *host, size_t n, const float **dev, char *error, size_t capacity);
// A conv1d weight [out_ch, in_ch, kernel] in the form the convolution kernels stage it (codec_ops.hip): cut into chunks of
// 32 output channels x 8 input channels, each chunk 32 rows of 8 * kernel + 4 floats (a row holds the taps of its eight
// channels one after the other, then four floats of padding: the row stride the kernels keep in LDS), zeros where the
// tensor has no row or channel.  Chunk (block b of input channels, tile t of output channels) starts at float
// (b * tiles + t) * conv_chunk_floats(kernel); `tiles` is even and `blocks` a multiple of four (whole chunks of zeros
// past the tensor), and four kilobytes of zeros follow the last chunk, so a kernel copies whole chunks without a bounds check.
struct ConvBlocks {
    const float *data = nullptr;
    int tiles = 0, blocks = 0;
};
constexpr int kConvChannels = 8;      // input channels per chunk: the convolution kernels' step along the inner dimension
inline size_t conv_chunk_floats(size_t kernel) { return 32u * (kConvChannels * kernel + 4u); }
int cached_conv_blocks(State *st, const float *host, size_t out_ch, size_t in_ch, size_t kernel, ConvBlocks *out, char *error, size_t capacity);
int ensure_attention_workspace(State *st, size_t batch, size_t heads, size_t head_width, size_t max_valid,
                               char *error, size_t capacity, size_t chunk_rows = kAttnChunk);
int ensure_pinned(State *st, size_t bytes, char *error, size_t capacity);

// packed-weight files (weight_pack.cpp)
uint64_t weight_fingerprint(const float *host, size_t n, size_t k);
int pack_lookup(State *st, const float *host, size_t n, size_t k, int qtype, int arith, uint64_t fingerprint, const PackedWeight **found);

// host quantisers (quantize_host.cpp)
void quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales, int arith);
int quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales, int arith);
uint16_t f32_to_f16_rne(float value);

}  // namespace mynah
