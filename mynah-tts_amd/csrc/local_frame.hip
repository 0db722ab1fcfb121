// The local transformer's frame on the device: sample_local_frame_batch (src/graph.c:1374-1656).
//
// Per stacked frame the reference runs, for each of the (16) codebook streams in turn: one step of a small decoder
// stack without cross attention or final norm (local_step_batch, :1234-1343), a width -> vocab projection with that
// stream's weight and bias (:1536-1547), the token choice (:1548-1616: constraint mask, first-max argmax, and for
// sampling items top-k insertion, temperature softmax, one xorshift64 draw, cumulative pick), EOS bookkeeping
// (:1617-1628) and the lookup of the token's embedding as the next position's input (:1629-1652).  Its resident GPU path
// crosses to the host once per stream (argmax_dev or a d2h of the logits, then an h2d of the embedding row).
//
// Here the whole frame stays on the device: the stack's step is the resident decode step of this library
// (mynah_hip_decoder_step on a decoder without cross attention), the projection is the batched matvec, and one small
// kernel per stream chooses the token for every item, keeps the generator state and the EOS flags in device memory and
// gathers the next input row.  The host uploads the per-item parameters once and downloads the tokens once.
//
// The token choice follows the reference decision for decision: disallowed candidates count as -FLT_MAX, the first
// maximum wins, the top-k list is ordered by (logit descending, index ascending) -- which is what the reference's
// insertion loop produces -- the numerators are expf((l - max) / temperature), and total and cumulative sums are formed
// sequentially in list order by one thread, so that the comparison `draw <= cumulative` sees the same float32 sums.
#include <float.h>

#include <new>

#include "kernels.h"

using namespace mynah;

namespace {

constexpr int kMaxTopK = 256;     // sampling list kept in LDS
constexpr int kMaxVocab = 8192;   // logits of one item staged in LDS

struct LocalItemDev {
    const float *decoder_last;   // device [width]
    float temperature;
    unsigned topk;
    unsigned long long rng_state;
    int forbid_eos;
    int saw_eos;
    unsigned long long eos_frame;   // ~0 = none
};

struct SampleArgs {
    LocalItemDev *items;          // [batch], generator state and EOS flags updated in place
    const float *logits;          // [batch, logits_stride]
    size_t logits_stride;
    float *logits_copy;           // optional [batch, streams, vocab]: the masked logits, for parity tests
    const float *audio_table;     // [vocab, width] of this stream
    float *row_in;                // [batch, width]: next input of the stack
    unsigned *values, *stored;    // [batch, streams]
    int stream, streams, vocab, codebook_size, eos_id, codebook_count, width;
};

// Monotone map float -> unsigned: a > b  <=>  key(a) > key(b)  (no NaNs among logits that matter).
__device__ __forceinline__ unsigned order_key(float v) {
    const unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Exclusive prefix sum of one int per thread over the 256-thread workgroup; *total receives the sum.
__device__ __forceinline__ int block_exclusive_scan(int v, int *s_scan, int *total) {
    const int tid = threadIdx.x;
    s_scan[tid] = v;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        const int add = tid >= off ? s_scan[tid - off] : 0;
        __syncthreads();
        s_scan[tid] += add;
        __syncthreads();
    }
    const int inclusive = s_scan[tid];
    *total = s_scan[255];
    __syncthreads();
    return inclusive - v;
}

__global__ void __launch_bounds__(256) k_local_begin(LocalItemDev *items, float *row_in, int width) {
    const int b = blockIdx.x;
    const float *src = items[b].decoder_last;
    for (int d = threadIdx.x; d < width; d += 256) row_in[(size_t)b * width + d] = src[d];   // src/graph.c:1420-1422
    if (threadIdx.x == 0) {
        items[b].saw_eos = 0;
        items[b].eos_frame = ~0ull;
    }
}

__global__ void __launch_bounds__(256) k_local_sample(const SampleArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    float *s_lg = reinterpret_cast<float *>(smem);                 // [vocab] masked logits
    __shared__ int s_scan[256];
    __shared__ unsigned s_hist[256];
    __shared__ float s_best[4];
    __shared__ int s_best_idx[4];
    __shared__ unsigned s_sel_key[kMaxTopK];
    __shared__ int s_sel_idx[kMaxTopK];
    __shared__ float s_top_val[kMaxTopK];
    __shared__ int s_top_idx[kMaxTopK];
    __shared__ unsigned s_prefix;
    __shared__ int s_remaining;
    __shared__ unsigned s_value;

    const int tid = threadIdx.x, b = blockIdx.x;
    LocalItemDev &item = a.items[b];
    const int V = a.vocab;
    const float *lg = a.logits + (size_t)b * a.logits_stride;
    const int forbid_eos = item.forbid_eos;

    // ---- constraint mask (src/graph.c:1556-1563) and first-max argmax (:1564-1569)
    float best = -FLT_MAX;
    int best_idx = 0x7fffffff;
    for (int c = tid; c < V; c += 256) {
        const bool allowed = c < a.codebook_size || (c == a.eos_id && !forbid_eos);
        const float v = allowed ? lg[c] : -FLT_MAX;
        s_lg[c] = v;
        if (a.logits_copy != nullptr) a.logits_copy[((size_t)b * a.streams + a.stream) * V + c] = v;
        if (allowed && v > best) { best = v; best_idx = c; }   // strided ascending: the first of equal maxima stays
    }
    // lanes, then wavefronts: larger value wins, equal values keep the smaller index
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(best_idx, off);
        if (ov > best || (ov == best && oi < best_idx)) { best = ov; best_idx = oi; }
    }
    if ((tid & 63) == 0) { s_best[tid >> 6] = best; s_best_idx[tid >> 6] = best_idx; }
    __syncthreads();
    best = s_best[0]; best_idx = s_best_idx[0];
    for (int w = 1; w < 4; ++w)
        if (s_best[w] > best || (s_best[w] == best && s_best_idx[w] < best_idx)) { best = s_best[w]; best_idx = s_best_idx[w]; }
    const unsigned argmax = best_idx == 0x7fffffff ? 0u : (unsigned)best_idx;   // nothing above -FLT_MAX: the reference keeps 0

    const float temperature = item.temperature;
    const int top_count = min((int)min(item.topk, (unsigned)V), kMaxTopK);
    const bool sampling = temperature > 0.0f && item.topk > 1u;
    if (tid == 0) s_value = argmax;
    if (sampling) {
        // ---- the top_count-th largest key by radix selection (four 8-bit digits, most significant first)
        if (tid == 0) { s_prefix = 0u; s_remaining = top_count; }
        for (int shift = 24; shift >= 0; shift -= 8) {
            s_hist[tid] = 0u;
            __syncthreads();
            const unsigned prefix = s_prefix;
            const unsigned high_mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
            for (int c = tid; c < V; c += 256) {
                const unsigned key = order_key(s_lg[c]);
                if ((key & high_mask) == (prefix & high_mask)) atomicAdd(&s_hist[(key >> shift) & 0xffu], 1u);
            }
            __syncthreads();
            if (tid == 0) {
                int remaining = s_remaining;
                int digit = 255;
                for (; digit > 0; --digit) {
                    const int n = (int)s_hist[digit];
                    if (n >= remaining) break;
                    remaining -= n;
                }
                s_prefix = prefix | ((unsigned)digit << shift);
                s_remaining = remaining;
            }
            __syncthreads();
        }
        const unsigned threshold = s_prefix;    // key of the top_count-th largest logit
        const int take_equal = s_remaining;     // how many candidates with exactly that key belong to the list (earliest first)

        // ---- compaction in index order: [keys above the threshold ..., the first take_equal keys equal to it ...]
        const int per = (V + 255) / 256;
        const int c0 = tid * per, c1 = min(V, c0 + per);
        int n_gt = 0, n_eq = 0;
        for (int c = c0; c < c1; ++c) {
            const unsigned key = order_key(s_lg[c]);
            n_gt += key > threshold;
            n_eq += key == threshold;
        }
        int total_gt = 0, total_eq = 0;
        int pos_gt = block_exclusive_scan(n_gt, s_scan, &total_gt);
        int pos_eq = block_exclusive_scan(n_eq, s_scan, &total_eq);
        for (int c = c0; c < c1; ++c) {
            const unsigned key = order_key(s_lg[c]);
            if (key > threshold) {
                s_sel_key[pos_gt] = key; s_sel_idx[pos_gt] = c; ++pos_gt;
            } else if (key == threshold) {
                if (pos_eq < take_equal) { s_sel_key[total_gt + pos_eq] = key; s_sel_idx[total_gt + pos_eq] = c; }
                ++pos_eq;
            }
        }
        __syncthreads();
        // ---- order the list by (logit descending, index ascending): the order the reference's insertion loop builds
        for (int q = tid; q < top_count; q += 256) {
            const unsigned key = s_sel_key[q];
            const int idx = s_sel_idx[q];
            int rank = 0;
            for (int j = 0; j < top_count; ++j) rank += s_sel_key[j] > key || (s_sel_key[j] == key && s_sel_idx[j] < idx);
            s_top_idx[rank] = idx;
            s_top_val[rank] = s_lg[idx];
        }
        __syncthreads();
        // ---- numerators in parallel, sums in list order by one thread (src/graph.c:1599-1616)
        const float maximum = s_top_val[0];
        __syncthreads();
        for (int q = tid; q < top_count; q += 256) s_top_val[q] = expf((s_top_val[q] - maximum) / temperature);
        __syncthreads();
        if (tid == 0) {
            float total = 0.0f;
            for (int q = 0; q < top_count; ++q) total += s_top_val[q];
            unsigned long long bits = item.rng_state;
            bits ^= bits << 13;
            bits ^= bits >> 7;
            bits ^= bits << 17;
            bits = bits == 0ull ? 0x9e3779b97f4a7c15ull : bits;
            item.rng_state = bits;
            const float draw = ((float)((bits >> 40) & 0xffffffull) / 16777216.0f) * total;
            float cumulative = 0.0f;
            unsigned value = argmax;
            for (int q = 0; q < top_count; ++q) {
                cumulative += s_top_val[q];
                if (draw <= cumulative || q + 1 == top_count) {
                    value = (unsigned)s_top_idx[q];
                    break;
                }
            }
            s_value = value;
        }
    }
    __syncthreads();
    const unsigned value = s_value;
    // ---- EOS in either the greedy or the chosen token (src/graph.c:1572-1574,1617-1622), codes, next input row
    if (tid == 0) {
        if (argmax == (unsigned)a.eos_id || value == (unsigned)a.eos_id) {
            item.saw_eos = 1;
            const unsigned long long frame = (unsigned long long)(a.stream / a.codebook_count);
            if (frame < item.eos_frame) item.eos_frame = frame;
        }
        a.values[(size_t)b * a.streams + a.stream] = value;
        a.stored[(size_t)b * a.streams + a.stream] = value < (unsigned)a.codebook_size ? value : 0u;   // :1627
    }
    const unsigned emit = value < (unsigned)V ? value : 0u;                                              // :1626
    const float *row = a.audio_table + (size_t)emit * a.width;
    for (int d = tid; d < a.width; d += 256) a.row_in[(size_t)b * a.width + d] = row[d];              // :1651
}

}  // namespace

struct mynah_hip_local {
    mynah_hip_decoder *stack = nullptr;
    size_t layers = 0, width = 0, capacity = 0;
    size_t streams = 0, vocab = 0, codebook_size = 0, eos_id = 0, codebook_count = 0;
    std::vector<const float *> projection_w, projection_bias;   // host pointers (the weight cache keys on them)
    std::vector<const float *> audio_table;                      // device f32 [vocab, width]
    float *k = nullptr, *v = nullptr;                            // [kMaxBatch, layers, capacity, width]
    float *row_in = nullptr, *row_out = nullptr, *logits = nullptr;
    LocalItemDev *items = nullptr, *items_host = nullptr;        // device / pinned
    unsigned *values = nullptr, *values_host = nullptr;          // [2, kMaxBatch, streams]: values | stored
};

extern "C" void mynah_hip_local_destroy(void *state, mynah_hip_local *l) {
    State *st = static_cast<State *>(state);
    if (l == nullptr) return;
    if (st != nullptr) (void)hipStreamSynchronize(st->stream);
    if (l->stack != nullptr) mynah_hip_decoder_destroy(state, l->stack);
    for (void *p : {(void *)l->k, (void *)l->v, (void *)l->row_in, (void *)l->row_out, (void *)l->logits, (void *)l->items, (void *)l->values})
        if (p != nullptr) (void)hipFree(p);
    if (l->items_host != nullptr) (void)hipHostFree(l->items_host);
    if (l->values_host != nullptr) (void)hipHostFree(l->values_host);
    delete l;
}

extern "C" int mynah_hip_local_create(void *state, const mynah_hip_decoder_desc *stack, const mynah_hip_local_desc *desc,
                                      mynah_hip_local **out, char *error, size_t capacity) {
    State *st = static_cast<State *>(state);
    if (out != nullptr) *out = nullptr;
    if (st == nullptr || stack == nullptr || desc == nullptr || out == nullptr) {
        set_error(error, capacity, "local_create: null argument");
        return -1;
    }
    if (stack->cross_heads * stack->cross_head_width != 0 || stack->norm_out != nullptr || desc->streams == 0 ||
        stack->capacity < desc->streams || desc->vocab == 0 || desc->vocab > (size_t)kMaxVocab || desc->codebook_count == 0 ||
        desc->projection_w == nullptr || desc->audio_table == nullptr) {
        set_error(error, capacity, "local_create: the stack must have no cross attention and no final norm, capacity >= streams, vocab <= 8192");
        return -1;
    }
    mynah_hip_local *l = new (std::nothrow) mynah_hip_local();
    if (l == nullptr) {
        set_error(error, capacity, "out of memory creating the local frame");
        return -1;
    }
    auto fail = [&]() { mynah_hip_local_destroy(state, l); return -1; };
    if (mynah_hip_decoder_create(state, stack, &l->stack, error, capacity) != 0) return fail();
    l->layers = stack->layers; l->width = stack->width; l->capacity = stack->capacity;
    l->streams = desc->streams; l->vocab = desc->vocab; l->codebook_size = desc->codebook_size; l->eos_id = desc->eos_id;
    l->codebook_count = desc->codebook_count;
    for (size_t s = 0; s < desc->streams; ++s) {
        if (desc->projection_w[s] == nullptr || desc->audio_table[s] == nullptr) {
            set_error(error, capacity, "local_create: missing projection weight or audio table");
            return fail();
        }
        const CachedWeight *cw = nullptr;
        // converted and cached now, so that the first frame does not pay for it
        if (cached_matrix(st, desc->projection_w[s], desc->vocab, stack->width, st->qtype, &cw, error, capacity) != 0) return fail();
        l->projection_w.push_back(desc->projection_w[s]);
        const float *bias = desc->projection_bias != nullptr ? desc->projection_bias[s] : nullptr;
        const float *dev_bias = nullptr;
        if (cached_vector(st, bias, desc->vocab, &dev_bias, error, capacity) != 0) return fail();
        l->projection_bias.push_back(bias);
        if (cached_matrix(st, desc->audio_table[s], desc->vocab, stack->width, MYNAH_HIP_F32, &cw, error, capacity) != 0) return fail();
        if (cw->qtype != MYNAH_HIP_F32) {
            set_error(error, capacity, "local_create: audio table could not be kept as f32");
            return fail();
        }
        l->audio_table.push_back(static_cast<const float *>(cw->data));
    }
    const size_t B = kMaxBatch, cache_floats = B * l->layers * l->capacity * l->width;
    auto alloc = [&](void **p, size_t bytes) {
        if (hip_check(hipMalloc(p, bytes), "local frame workspace", error, capacity) != 0) return -1;
        return hip_check(hipMemset(*p, 0, bytes), "local frame workspace clear", error, capacity);
    };
    if (alloc(reinterpret_cast<void **>(&l->k), cache_floats * sizeof(float)) != 0 || alloc(reinterpret_cast<void **>(&l->v), cache_floats * sizeof(float)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->row_in), B * l->width * sizeof(float)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->row_out), B * l->width * sizeof(float)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->logits), B * l->vocab * sizeof(float)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->items), B * sizeof(LocalItemDev)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->values), 2 * B * l->streams * sizeof(unsigned)) != 0)
        return fail();
    if (hip_check(hipHostMalloc(reinterpret_cast<void **>(&l->items_host), B * sizeof(LocalItemDev), hipHostMallocDefault), "local frame staging", error, capacity) != 0 ||
        hip_check(hipHostMalloc(reinterpret_cast<void **>(&l->values_host), 2 * B * l->streams * sizeof(unsigned), hipHostMallocDefault), "local frame staging", error, capacity) != 0)
        return fail();
    *out = l;
    return 0;
}

extern "C" int mynah_hip_local_frame(void *state, mynah_hip_local *l, mynah_hip_local_item *items, size_t batch, unsigned *values,
                                     unsigned *stored, int *saw_eos, size_t *eos_frame, float *dev_logits_copy, char *error,
                                     size_t capacity) {
    State *st = static_cast<State *>(state);
    if (batch == 0) return 0;   // src/graph.c:1378
    if (batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "local frame batch exceeds MYNAH_MAX_BATCH");   // src/graph.c:1379-1382
        return -1;
    }
    if (st == nullptr || l == nullptr || items == nullptr || values == nullptr || stored == nullptr || saw_eos == nullptr || eos_frame == nullptr) {
        set_error(error, capacity, "local_frame: null argument");
        return -1;
    }
    for (size_t b = 0; b < batch; ++b) {
        if (items[b].dev_decoder_last == nullptr) {
            set_error(error, capacity, "local_frame: item has no input row");
            return -1;
        }
        const bool sampling = items[b].temperature > 0.0f && items[b].topk > 1u;
        const size_t top_count = items[b].topk < l->vocab ? items[b].topk : l->vocab;
        if (sampling && top_count > (size_t)kMaxTopK) {
            set_error(error, capacity, "local sampler scratch too small");   // src/graph.c:1416-1419 (here: top-k list of at most 256)
            return -1;
        }
    }
    MYNAH_TRY(hipStreamSynchronize(st->stream));   // the staging buffers of the previous frame may still be in flight
    for (size_t b = 0; b < batch; ++b) {
        LocalItemDev &d = l->items_host[b];
        d.decoder_last = items[b].dev_decoder_last;
        d.temperature = items[b].temperature;
        d.topk = items[b].topk > 0xffffffffu ? 0xffffffffu : (unsigned)items[b].topk;
        d.rng_state = items[b].rng_state;
        d.forbid_eos = items[b].forbid_eos;
        d.saw_eos = 0;
        d.eos_frame = ~0ull;
    }
    MYNAH_TRY(hipMemcpyAsync(l->items, l->items_host, batch * sizeof(LocalItemDev), hipMemcpyHostToDevice, st->stream));
    const int B = (int)batch, width = (int)l->width;
    hipLaunchKernelGGL(k_local_begin, dim3(B), dim3(256), 0, st->stream, l->items, l->row_in, width);
    MYNAH_TRY(hipGetLastError());

    mynah_hip_decoder_slot slots[kMaxBatch];
    const float *proj_in[kMaxBatch];
    float *proj_out[kMaxBatch];
    const size_t per_slot = l->layers * l->capacity * l->width;
    for (int b = 0; b < B; ++b) {
        slots[b] = mynah_hip_decoder_slot{};
        slots[b].dev_self_k = l->k + (size_t)b * per_slot;
        slots[b].dev_self_v = l->v + (size_t)b * per_slot;
        slots[b].memory_length = 0;
        slots[b].dev_input = l->row_in + (size_t)b * width;
        slots[b].dev_output = l->row_out + (size_t)b * width;
        proj_in[b] = slots[b].dev_output;
        proj_out[b] = l->logits + (size_t)b * l->vocab;
    }
    unsigned *dev_values = l->values, *dev_stored = l->values + (size_t)kMaxBatch * l->streams;
    for (size_t stream = 0; stream < l->streams; ++stream) {
        for (int b = 0; b < B; ++b) slots[b].length = stream;   // the local cache restarts at 0 every frame (src/graph.c:1412)
        if (mynah_hip_decoder_step(state, l->stack, slots, batch, error, capacity) != 0) return -1;
        if (mynah_hip_matmul_d2d_batched(state, proj_in, proj_out, batch, l->width, l->vocab, l->projection_w[stream],
                                         l->projection_bias[stream], error, capacity) != 0)
            return -1;
        SampleArgs a{};
        a.items = l->items; a.logits = l->logits; a.logits_stride = l->vocab; a.logits_copy = dev_logits_copy;
        a.audio_table = l->audio_table[stream]; a.row_in = l->row_in; a.values = dev_values; a.stored = dev_stored;
        a.stream = (int)stream; a.streams = (int)l->streams; a.vocab = (int)l->vocab; a.codebook_size = (int)l->codebook_size;
        a.eos_id = (int)l->eos_id; a.codebook_count = (int)l->codebook_count; a.width = width;
        hipLaunchKernelGGL(k_local_sample, dim3(B), dim3(256), l->vocab * sizeof(float), st->stream, a);
        MYNAH_TRY(hipGetLastError());
    }
    MYNAH_TRY(hipMemcpyAsync(l->values_host, l->values, 2 * (size_t)kMaxBatch * l->streams * sizeof(unsigned), hipMemcpyDeviceToHost, st->stream));
    MYNAH_TRY(hipMemcpyAsync(l->items_host, l->items, batch * sizeof(LocalItemDev), hipMemcpyDeviceToHost, st->stream));
    MYNAH_TRY(hipStreamSynchronize(st->stream));
    for (size_t b = 0; b < batch; ++b) {
        for (size_t s = 0; s < l->streams; ++s) {
            values[b * l->streams + s] = l->values_host[b * l->streams + s];
            stored[b * l->streams + s] = l->values_host[(size_t)kMaxBatch * l->streams + b * l->streams + s];
        }
        items[b].rng_state = l->items_host[b].rng_state;
        saw_eos[b] = l->items_host[b].saw_eos;
        eos_frame[b] = l->items_host[b].eos_frame == ~0ull ? SIZE_MAX : (size_t)l->items_host[b].eos_frame;
    }
    return 0;
}
