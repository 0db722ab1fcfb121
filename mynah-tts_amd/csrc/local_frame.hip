// The local transformer's frame on the device: sample_local_frame_batch (src/graph.c:1374-1656).
//
// Per stacked frame the reference runs, for each of the (16) codebook streams in turn: one step of a small decoder
// stack without cross attention or final norm (local_step_batch, :1234-1343), a width -> vocab projection with that
// stream's weight and bias (:1536-1547), the token choice (:1548-1616: constraint mask, first-max argmax, and for
// sampling items top-k insertion, temperature softmax, one xorshift64 draw, cumulative pick), EOS bookkeeping
// (:1617-1628) and the lookup of the token's embedding as the next position's input (:1629-1652).  Its resident GPU path
// crosses to the host once per stream (argmax_dev or a d2h of the logits, then an h2d of the embedding row).
//
// Here the whole frame stays on the device and is replayed as ONE captured graph per batch size: per position the layer
// kernels of the resident decode step (a decoder without cross attention), the batched matvec for the projection, and
// one small kernel that chooses the token for every item, keeps the generator state and the EOS flags in device memory,
// forms the next position's input row (embedding + position) directly in the stack's residual rows and advances the
// cache length in the device slot table.  The caches belong to this object, so nothing in the graph changes from frame
// to frame; what does change (the items) is uploaded once before the graph and the tokens are downloaded once after it.
//
// The token choice follows the reference decision for decision: disallowed candidates count as -FLT_MAX, the first
// maximum wins, the top-k list is ordered by (logit descending, index ascending) -- which is what the reference's
// insertion loop produces -- the numerators are expf((l - max) / temperature), and total and cumulative sums are formed
// sequentially in list order by one thread, so that the comparison `draw <= cumulative` sees the same float32 sums.
#include <float.h>
#include <string.h>

#include <new>

#include "device_common.h"
#include "kernels.h"
#include "step_items.h"

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

// Everything a frame brings from the host, uploaded in one copy.
struct LocalFrameDev {
    float *logits_copy;             // optional [batch, streams, vocab]: the masked logits, for parity tests
    unsigned epoch_base;            // step counter of this frame's first pass through the stack (pass s uses base + s)
    unsigned reserved;
    LocalItemDev items[kMaxBatch];  // generator state and EOS flags updated in place
};

struct SampleArgs {
    LocalFrameDev *frame;
    const float *logits;          // [batch, vocab]
    const float *audio_table;     // [vocab, width] of this position
    const float *next_position;   // position row of the next step, or null
    float *x;                     // [batch, width]: residual rows of the stack = its next input
    StepSlots *slots;             // cache lengths advance here
    unsigned *values, *stored;    // [batch, streams]
    int stream, streams, vocab, codebook_size, eos_id, codebook_count, width;
    int batch;                    // workgroups behind the items' fill `tables` for the next pass through the stack
    StepItemTables tables;
};

// Monotone map float -> unsigned: a > b  <=>  key(a) > key(b)  (no NaNs among logits that matter), and back.
__device__ __forceinline__ unsigned order_key(float v) {
    const unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(unsigned key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}
// (key, index) in one integer whose order is the order of the reference's candidate list: larger logit first, among
// equal logits the smaller index first.  No two candidates share one, and every one is above zero.
__device__ __forceinline__ unsigned long long candidate(unsigned key, int index) {
    return ((unsigned long long)key << 32) | (unsigned long long)(0xffffffffu - (unsigned)index);
}
__device__ __forceinline__ int candidate_index(unsigned long long c) { return (int)(0xffffffffu - (unsigned)(c & 0xffffffffull)); }
__device__ __forceinline__ unsigned candidate_key(unsigned long long c) { return (unsigned)(c >> 32); }

// Largest value over the wavefront, in every lane: four steps inside the rows of sixteen lanes on the DPP path, then the
// four rows through scalar registers.  All 64 lanes must be active.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
    v = max(v, (unsigned)dpp_i<kDppXor1>((int)v));
    v = max(v, (unsigned)dpp_i<kDppXor2>((int)v));
    v = max(v, (unsigned)dpp_i<kDppHalfMirror>((int)v));
    v = max(v, (unsigned)dpp_i<kDppMirror>((int)v));
    const unsigned r0 = (unsigned)__builtin_amdgcn_readlane((int)v, 0), r1 = (unsigned)__builtin_amdgcn_readlane((int)v, 16);
    const unsigned r2 = (unsigned)__builtin_amdgcn_readlane((int)v, 32), r3 = (unsigned)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(r0, r1), max(r2, r3));
}

// How many of list[0, n) are above `mine` (pairs of entries per LDS read; the list is 16-byte aligned), counted by four
// adjacent threads: thread `part` of the four looks at pairs part, part + 4, ... and the four sums meet by shuffles.  Every
// lane of the wavefront must call it.
__device__ __forceinline__ int count_above_by_four(const unsigned long long *list, int n, unsigned long long mine, int part) {
    const ulonglong2 *pairs = reinterpret_cast<const ulonglong2 *>(list);
    int above = 0;
#pragma unroll 4
    for (int j = part; j < n / 2; j += 4) {
        const ulonglong2 p = pairs[j];
        above += (p.x > mine ? 1 : 0) + (p.y > mine ? 1 : 0);
    }
    if ((n & 1) && part == 0) above += list[n - 1] > mine ? 1 : 0;
    above += dpp_i<kDppXor1>(above);
    above += dpp_i<kDppXor2>(above);
    return above;
}

// The same for a list of at most 64 entries followed by zeros up to 64 (no candidate is zero): every thread's eight reads
// are requested at once.
__device__ __forceinline__ int count_above_in_64(const unsigned long long *list, unsigned long long mine, int part) {
    const ulonglong2 *pairs = reinterpret_cast<const ulonglong2 *>(list);
    ulonglong2 p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) p[j] = pairs[part + 4 * j];
    int above = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) above += (p[j].x > mine ? 1 : 0) + (p[j].y > mine ? 1 : 0);
    above += dpp_i<kDppXor1>(above);
    above += dpp_i<kDppXor2>(above);
    return above;
}

// Frame start: the slot table (caches of this object, every length 0), x[b] = decoder_last[b] + position[0]
// (src/graph.c:1420-1422 and :1262-1264), EOS flags cleared (:1409-1410).
// Workgroups behind the items' fill the work tables of the first pass's many-stream attention launch (every cache empty).
__global__ void __launch_bounds__(256) k_local_begin(LocalFrameDev *frame, const StepSlots slots, StepSlots *dev_slots, float *x,
                                                     const float *position, int width, int batch, const StepItemTables tables) {
    const int b = blockIdx.x;
    if (b >= batch) {
        write_step_item(tables, slots, 0, (int)(frame->epoch_base & 0xffffffu), (b - batch) * 256 + (int)threadIdx.x);
        return;
    }
    if (b == 0 && threadIdx.x == 0) {
        *dev_slots = slots;
        dev_slots->epoch = frame->epoch_base;
    }
    const float *src = frame->items[b].decoder_last;
    for (int d = threadIdx.x; d < width; d += 256) x[(size_t)b * width + d] = position != nullptr ? src[d] + position[d] : src[d];
    if (threadIdx.x == 0) {
        frame->items[b].saw_eos = 0;
        frame->items[b].eos_frame = ~0ull;
    }
}

// Token choice for one item per workgroup.
//
// Sampling needs the top_count largest candidates in list order.  Common case: every thread keeps the best of its own
// (strided) candidates; each wavefront finds the ceil(top_count / 4)-th best among its 64 (bit by bit, with ballots),
// and the smallest of the four is a lower bound of the wanted threshold with at least top_count candidates at or above
// it, and usually not many more (some 60 for top-50 of 2048 logits).  Those are collected and ranked against each other,
// all pairs.  When more than kFastCandidates qualify (large top-k, many equal logits) the
// threshold is found exactly by radix selection instead and exactly top_count candidates are collected.  Both ways end in
// the same list, ranked the same way.
constexpr int kFastCandidates = 512;

__global__ void __launch_bounds__(256) k_local_sample(const SampleArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned *s_key = reinterpret_cast<unsigned *>(smem);          // [vocab] order keys of the masked logits
    __shared__ unsigned long long s_head[4];                       // every wavefront's best candidate
    __shared__ unsigned s_bound[4];
    __shared__ __align__(16) unsigned long long s_cand[kFastCandidates];
    __shared__ unsigned s_hist[4][256];
    __shared__ __align__(16) float s_top_val[kMaxTopK + 32];
    __shared__ int s_top_idx[kMaxTopK];
    __shared__ unsigned s_wave_total[4];
    __shared__ unsigned s_prefix, s_count;
    __shared__ int s_remaining, s_pick;
    __shared__ float s_draw;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, b = blockIdx.x;
    if (b >= a.batch) {
        // the next pass's caches hold stream + 1 rows each whatever is chosen here; the slot table's pointers are the frame's
        if (a.stream + 1 < a.streams)
            write_step_item(a.tables, *a.slots, a.stream + 1, (int)((a.frame->epoch_base + (unsigned)a.stream + 1u) & 0xffffffu), (b - a.batch) * 256 + tid);
        return;
    }
    LocalItemDev &item = a.frame->items[b];
    const int V = a.vocab;
    const float *lg = a.logits + (size_t)b * V;
    // Everything the kernel takes from memory before the choice is requested here, side by side and under no condition
    // (ids past the vocabulary repeat its last one): one round trip.  Requested where they are used, the item's fields, the
    // frame's pointer and the logits were three round trips one after the other, and the generator state a fourth.
    float first_logits[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) first_logits[i] = lg[min(tid + 256 * i, V - 1)];
    const int forbid_eos = item.forbid_eos;
    const float temperature = item.temperature;
    const unsigned topk = item.topk;
    const unsigned long long rng_before = item.rng_state;
    float *logits_copy = a.frame->logits_copy;

    // ---- constraint mask (src/graph.c:1556-1563); eight candidates per thread at a time, the first eight already requested
    unsigned long long mine = 0ull;
    constexpr int kKeysInRegisters = 8;              // a vocabulary of up to 8 * 256 ids: a thread's keys stay in registers for the collection below
    const bool keys_in_registers = V <= kKeysInRegisters * 256;
    unsigned own_key[kKeysInRegisters];
    const auto mask_eight = [&](const int c0, const float (&v)[8], const bool keep) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = c0 + 256 * i;
            const bool allowed = c < a.codebook_size || (c == a.eos_id && !forbid_eos);
            const float masked = allowed ? v[i] : -FLT_MAX;
            const unsigned key = order_key(masked);
            if (keep) own_key[i] = c < V ? key : 0u;
            if (c < V) {
                s_key[c] = key;
                if (logits_copy != nullptr) logits_copy[((size_t)b * a.streams + a.stream) * V + c] = masked;
                const unsigned long long cand = candidate(key, c);
                mine = cand > mine ? cand : mine;
            }
        }
    };
    mask_eight(tid, first_logits, true);
    for (int c0 = tid + 8 * 256; c0 < V; c0 += 8 * 256) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = c0 + 256 * i < V ? lg[c0 + 256 * i] : 0.0f;
        mask_eight(c0, v, false);
    }
    const int top_count = min((int)min(topk, (unsigned)V), kMaxTopK);
    const bool sampling = temperature > 0.0f && topk > 1u;
    for (int p = 0; p < 4; ++p) s_hist[p][tid] = 0u;
    if (tid < 64) s_cand[tid] = 0ull;   // a list of up to 64 candidates is followed by zeros (see count_above_in_64)
    if (tid == 0) { s_prefix = 0u; s_remaining = top_count; s_count = 0u; s_pick = top_count - 1; }
    // ---- the head of the list: the largest candidate of the wavefront (the largest key, and among the lanes that hold it the
    // largest low word = the smallest id), then of the four
    const unsigned head_key = wave_max_u32(candidate_key(mine));
    const unsigned head_low = wave_max_u32(candidate_key(mine) == head_key ? (unsigned)(mine & 0xffffffffull) : 0u);
    unsigned long long head = ((unsigned long long)head_key << 32) | (unsigned long long)head_low;
    // (sampling) the largest key with its low half clear that at least `want` of the wavefront's 64 bests reach: sixteen
    // ballots; the keys between this bound and the exact one (1/128 of the logit's magnitude) add a candidate or two
    unsigned bound = 0u;
    if (sampling) {
        const int want = (top_count + 3) / 4;
        const unsigned own = candidate_key(mine);
        for (int bit = 31; bit >= 16; --bit) {
            const unsigned trial = bound | (1u << bit);
            if ((int)__popcll(__ballot(own >= trial)) >= want) bound = trial;
        }
    }
    if (lane == 0) { s_head[wave] = head; s_bound[wave] = bound; }
    __syncthreads();
    for (int w = 0; w < 4; ++w) {
        head = s_head[w] > head ? s_head[w] : head;
        bound = s_bound[w] < bound ? s_bound[w] : bound;
    }
    // first-max argmax (src/graph.c:1564-1569): a candidate counts only above -FLT_MAX, otherwise the reference keeps 0
    const unsigned argmax = candidate_key(head) > order_key(-FLT_MAX) ? (unsigned)candidate_index(head) : 0u;
    const float maximum = key_value(candidate_key(head));   // the list's first logit (src/graph.c:1599)
    unsigned value = argmax;

    if (sampling) {
        // ---- collect the candidates at or above the bound: one LDS counter update per wavefront, places by ballot
        if (keys_in_registers) {
            // from the keys the thread kept (ids tid + 256 i): eight ballots, no LDS read
            unsigned long long masks[kKeysInRegisters];
            unsigned in_wave = 0u;
#pragma unroll
            for (int i = 0; i < kKeysInRegisters; ++i) {
                masks[i] = __ballot(tid + 256 * i < V && own_key[i] >= bound);
                in_wave += (unsigned)__popcll(masks[i]);
            }
            unsigned next_slot = 0u;
            if (lane == 0) next_slot = atomicAdd(&s_count, in_wave);
            next_slot = (unsigned)__builtin_amdgcn_readfirstlane((int)next_slot);
#pragma unroll
            for (int i = 0; i < kKeysInRegisters; ++i) {
                const bool take = (masks[i] >> lane) & 1ull;
                const unsigned slot = next_slot + (unsigned)__popcll(masks[i] & ((1ull << lane) - 1ull));
                if (take && slot < (unsigned)kFastCandidates) s_cand[slot] = candidate(own_key[i], tid + 256 * i);
                next_slot += (unsigned)__popcll(masks[i]);
            }
        } else {
            unsigned in_wave = 0u;
            for (int base = wave * 64; base < V; base += 256) {
                const int c = base + lane;
                in_wave += (unsigned)__popcll(__ballot(c < V && s_key[c] >= bound));
            }
            unsigned next_slot = 0u;
            if (lane == 0) next_slot = atomicAdd(&s_count, in_wave);
            next_slot = __shfl(next_slot, 0);
            for (int base = wave * 64; base < V; base += 256) {
                const int c = base + lane;
                const unsigned key = c < V ? s_key[c] : 0u;
                const bool take = c < V && key >= bound;
                const unsigned long long mask = __ballot(take);
                const unsigned slot = next_slot + (unsigned)__popcll(mask & ((1ull << lane) - 1ull));
                if (take && slot < (unsigned)kFastCandidates) s_cand[slot] = candidate(key, c);
                next_slot += (unsigned)__popcll(mask);
            }
        }
        __syncthreads();
        int listed = (int)s_count;
        if (listed > kFastCandidates) {
            // ---- the top_count-th largest key by radix selection: four 8-bit digits, most significant first.  Per digit
            // one LDS histogram of the candidates that share the digits chosen so far; the first wavefront then finds the
            // bin in which the wanted rank falls (four bins per lane, suffix sums across lanes by shuffles).
            for (int p = 0; p < 4; ++p) {
                const int shift = 24 - 8 * p;
                const unsigned prefix = s_prefix;
                const int remaining = s_remaining;
                const unsigned high_mask = p == 0 ? 0u : (0xffffffffu << (shift + 8));
                for (int c = tid; c < V; c += 256) {
                    const unsigned key = s_key[c];
                    if ((key & high_mask) == prefix) atomicAdd(&s_hist[p][(key >> shift) & 0xffu], 1u);
                }
                __syncthreads();
                if (wave == 0) {
                    int h[4];
                    for (int j = 0; j < 4; ++j) h[j] = (int)s_hist[p][4 * lane + j];
                    const int own = h[0] + h[1] + h[2] + h[3];
                    int suffix = own;   // candidates in the bins of this lane and of all higher lanes
                    for (int off = 1; off < 64; off <<= 1) {
                        const int other = __shfl_down(suffix, off);
                        if (lane + off < 64) suffix += other;
                    }
                    int above = suffix - own;   // candidates in bins above the one looked at
                    for (int j = 3; j >= 0; --j) {
                        if (above < remaining && remaining <= above + h[j]) {   // true for exactly one bin of one lane
                            s_prefix = prefix | ((unsigned)(4 * lane + j) << shift);
                            s_remaining = remaining - above;
                        }
                        above += h[j];
                    }
                }
                __syncthreads();
            }
            const unsigned threshold = s_prefix;    // key of the top_count-th largest logit
            const int take_equal = s_remaining;     // how many candidates with exactly that key belong to the list (earliest first)
            // compaction in index order: [keys above the threshold ..., the first take_equal keys equal to it ...]
            const int per = (V + 255) / 256;
            const int c0 = min(V, tid * per), c1 = min(V, c0 + per);
            unsigned counts = 0u;   // low half: keys above the threshold in [c0, c1); high half: keys equal to it
            for (int c = c0; c < c1; ++c) {
                const unsigned key = s_key[c];
                counts += (key > threshold ? 1u : 0u) + (key == threshold ? 0x10000u : 0u);
            }
            unsigned inclusive = counts;
            for (int off = 1; off < 64; off <<= 1) {
                const unsigned other = __shfl_up(inclusive, off);
                if (lane >= off) inclusive += other;
            }
            if (lane == 63) s_wave_total[wave] = inclusive;
            __syncthreads();
            unsigned before = 0u, total = 0u;
            for (int w = 0; w < 4; ++w) {
                if (w < wave) before += s_wave_total[w];
                total += s_wave_total[w];
            }
            const unsigned exclusive = before + inclusive - counts;
            int pos_gt = (int)(exclusive & 0xffffu), pos_eq = (int)(exclusive >> 16);
            const int total_gt = (int)(total & 0xffffu);
            for (int c = c0; c < c1; ++c) {
                const unsigned key = s_key[c];
                if (key > threshold) {
                    s_cand[pos_gt++] = candidate(key, c);
                } else if (key == threshold) {
                    if (pos_eq < take_equal) s_cand[total_gt + pos_eq] = candidate(key, c);
                    ++pos_eq;
                }
            }
            listed = top_count;
            if (tid >= top_count && tid < 64) s_cand[tid] = 0ull;   // behind a short list: zeros again (count_above_in_64)
            __syncthreads();
        }
        // ---- list position = how many collected candidates come before; numerators expf((l - max) / T) (src/graph.c:1599-1604)
        for (int q0 = 0; q0 < listed; q0 += 64) {   // four adjacent threads per candidate; every lane takes part in the exchanges
            const int q = q0 + (tid >> 2);
            const unsigned long long own = s_cand[q < listed ? q : listed - 1];
            const int place = listed <= 64 ? count_above_in_64(s_cand, own, tid & 3) : count_above_by_four(s_cand, listed, own, tid & 3);
            if (q < listed && (tid & 3) == 0 && place < top_count) {
                s_top_idx[place] = candidate_index(own);
                s_top_val[place] = expf((key_value(candidate_key(own)) - maximum) / temperature);
            }
        }
        if (tid < 32) s_top_val[top_count + tid] = 0.0f;   // lets the running sum below go in whole groups of 32
        __syncthreads();
        // ---- running sums in list order by one thread, kept in place (src/graph.c:1605-1616): float32 sums depend on
        // the order, and the last running sum is the reference's total
        if (tid == 0) {
            float running = 0.0f;
            for (int q0 = 0; q0 < top_count; q0 += 32) {   // a group's reads are requested together, its sums stay in registers
                float4 part[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) part[i] = *reinterpret_cast<const float4 *>(&s_top_val[q0 + 4 * i]);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    running += part[i].x; part[i].x = running;
                    running += part[i].y; part[i].y = running;
                    running += part[i].z; part[i].z = running;
                    running += part[i].w; part[i].w = running;
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) *reinterpret_cast<float4 *>(&s_top_val[q0 + 4 * i]) = part[i];
            }
            unsigned long long bits = rng_before;
            bits ^= bits << 13;
            bits ^= bits >> 7;
            bits ^= bits << 17;
            bits = bits == 0ull ? 0x9e3779b97f4a7c15ull : bits;
            item.rng_state = bits;
            s_draw = ((float)((bits >> 40) & 0xffffffull) / 16777216.0f) * running;
        }
        __syncthreads();
        // the first list position whose running sum reaches the draw; the last one if rounding leaves none
        const float draw = s_draw;
        for (int q = tid; q < top_count; q += 256)
            if (draw <= s_top_val[q] && !(q > 0 && draw <= s_top_val[q - 1])) s_pick = q;
        __syncthreads();
        value = (unsigned)s_top_idx[s_pick];
    }
    // ---- EOS in either the greedy or the chosen token (src/graph.c:1572-1574,1617-1622), codes, next input row
    if (tid == 0) {
        if (argmax == (unsigned)a.eos_id || value == (unsigned)a.eos_id) {
            item.saw_eos = 1;
            const unsigned long long frame = (unsigned long long)(a.stream / a.codebook_count);
            if (frame < item.eos_frame) item.eos_frame = frame;
        }
        a.values[(size_t)b * a.streams + a.stream] = value;
        a.stored[(size_t)b * a.streams + a.stream] = value < (unsigned)a.codebook_size ? value : 0u;   // :1627
        a.slots->length[b] = a.stream + 1;
    }
    if (a.stream + 1 < a.streams) {
        const unsigned emit = value < (unsigned)V ? value : 0u;                                          // :1626
        const float *row = a.audio_table + (size_t)emit * a.width;                                      // :1651
        const float *pe = a.next_position;                                                             // :1262-1264
        if (a.width <= 1024) {   // one round trip: every request before the first sum
            float rv[4], pv[4];
            const float *second = pe != nullptr ? pe : row;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int d = tid + 256 * u, at = d < a.width ? d : a.width - 1;
                rv[u] = row[at];
                pv[u] = second[at];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int d = tid + 256 * u;
                if (d < a.width) a.x[(size_t)b * a.width + d] = pe != nullptr ? rv[u] + pv[u] : rv[u];
            }
        } else {
            for (int d = tid; d < a.width; d += 256) a.x[(size_t)b * a.width + d] = pe != nullptr ? row[d] + pe[d] : row[d];
        }
    }
}

}  // namespace

struct mynah_hip_local {
    mynah_hip_decoder *stack = nullptr;
    size_t layers = 0, width = 0, capacity = 0;
    size_t streams = 0, vocab = 0, codebook_size = 0, eos_id = 0, codebook_count = 0;
    std::vector<const CachedWeight *> projection;   // [streams], storage of the current quant setting
    std::vector<const float *> projection_bias;     // [streams] device, or null
    std::vector<const float *> audio_table;         // [streams] device f32 [vocab, width]
    int arith = 0;
    float *k = nullptr, *v = nullptr;               // [kMaxBatch, layers, capacity, width]
    float *logits = nullptr;                        // [kMaxBatch, vocab]
    LocalFrameDev *frame = nullptr, *frame_host = nullptr;   // device / pinned
    unsigned *values = nullptr, *values_host = nullptr;      // [2, kMaxBatch, streams]: values | stored
    hipGraphExec_t graphs[kMaxBatch + 1] = {};
    int eager_frames[kMaxBatch + 1] = {};   // a batch size runs eagerly once (one-time kernel set-up) before it is captured
};

// One frame's kernels on the stream; replayable: nothing here depends on the items.
static int enqueue_frame(State *st, mynah_hip_local *l, int B, char *error, size_t capacity) {
    const DecoderRows rows = decoder_rows(l->stack);
    const int width = (int)l->width;
    StepSlots slots;
    memset(&slots, 0, sizeof slots);
    const size_t per_slot = l->layers * l->capacity * l->width;
    for (int b = 0; b < B; ++b) {
        slots.self_k[b] = l->k + (size_t)b * per_slot;
        slots.self_v[b] = l->v + (size_t)b * per_slot;
        slots.input[b] = rows.x + (size_t)b * width;
        slots.output[b] = rows.x + (size_t)b * width;
    }
    const StepItemTables tables = decoder_item_tables(l->stack, B);
    const unsigned table_workgroups = step_item_workgroups(tables);
    hipLaunchKernelGGL(k_local_begin, dim3(B + table_workgroups), dim3(256), 0, st->stream, l->frame, slots, rows.slots, rows.x, rows.position, width, B,
                       tables);
    MYNAH_TRY(hipGetLastError());
    for (size_t stream = 0; stream < l->streams; ++stream) {
        if (decoder_enqueue_layers(st, l->stack, B, error, capacity) != 0) return -1;
        const CachedWeight *cw = l->projection[stream];
        for (int b0 = 0; b0 < B; b0 += kBatchTile) {
            LinearArgs p{};
            p.w = cw->data;
            p.scales = cw->scales;
            p.bias = l->projection_bias[stream];
            p.qtype = cw->qtype;
            p.n = (int)l->vocab;
            p.k = width;
            p.batch = B - b0 < kBatchTile ? B - b0 : kBatchTile;
            for (int b = 0; b < p.batch; ++b) {
                p.in[b] = rows.x + (size_t)(b0 + b) * width;
                p.out[b] = l->logits + (size_t)(b0 + b) * l->vocab;
            }
            p.arith = l->arith;
            p.epilogue = EPI_NONE;
            if (launch_linear(st, p, error, capacity) != 0) return -1;
        }
        SampleArgs a{};
        a.frame = l->frame; a.logits = l->logits; a.audio_table = l->audio_table[stream];
        a.next_position = rows.position != nullptr ? rows.position + (stream + 1) * l->width : nullptr;
        a.x = rows.x; a.slots = rows.slots; a.values = l->values; a.stored = l->values + (size_t)kMaxBatch * l->streams;
        a.stream = (int)stream; a.streams = (int)l->streams; a.vocab = (int)l->vocab; a.codebook_size = (int)l->codebook_size;
        a.eos_id = (int)l->eos_id; a.codebook_count = (int)l->codebook_count; a.width = width;
        a.batch = B; a.tables = tables;
        hipLaunchKernelGGL(k_local_sample, dim3(B + (stream + 1 < l->streams ? table_workgroups : 0u)), dim3(256), l->vocab * sizeof(float), st->stream, a);
        MYNAH_TRY(hipGetLastError());
    }
    return 0;
}

extern "C" void mynah_hip_local_destroy(void *state, mynah_hip_local *l) {
    State *st = enter_state(state);
    if (l == nullptr) return;
    if (st != nullptr) (void)hipStreamSynchronize(st->stream);
    for (auto &g : l->graphs)
        if (g != nullptr) (void)hipGraphExecDestroy(g);
    if (l->stack != nullptr) mynah_hip_decoder_destroy(state, l->stack);
    for (void *p : {(void *)l->k, (void *)l->v, (void *)l->logits, (void *)l->frame, (void *)l->values})
        if (p != nullptr) (void)hipFree(p);
    if (l->frame_host != nullptr) (void)hipHostFree(l->frame_host);
    if (l->values_host != nullptr) (void)hipHostFree(l->values_host);
    delete l;
}

extern "C" int mynah_hip_local_create(void *state, const mynah_hip_decoder_desc *stack, const mynah_hip_local_desc *desc,
                                      mynah_hip_local **out, char *error, size_t capacity) {
    State *st = enter_state(state);
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
    // with a position table, position streams (one past the last step) is never read: the last choice forms no next row
    mynah_hip_local *l = new (std::nothrow) mynah_hip_local();
    if (l == nullptr) {
        set_error(error, capacity, "out of memory creating the local frame");
        return -1;
    }
    auto fail = [&]() { mynah_hip_local_destroy(state, l); return -1; };
    if (mynah_hip_decoder_create(state, stack, &l->stack, error, capacity) != 0) return fail();
    l->layers = stack->layers; l->width = stack->width; l->capacity = stack->capacity; l->arith = st->arith;
    l->streams = desc->streams; l->vocab = desc->vocab;
    // The kernels hold these as int.  Ids at or above the vocabulary do not exist, so a codebook larger than it allows the
    // same ids as one of its size, and an end-of-sequence id outside it can match no id: keep that meaning after narrowing.
    l->codebook_size = desc->codebook_size < desc->vocab ? desc->codebook_size : desc->vocab;
    l->eos_id = desc->eos_id < desc->vocab ? desc->eos_id : (size_t)0x7fffffff;
    l->codebook_count = desc->codebook_count < (size_t)0x7fffffff ? desc->codebook_count : (size_t)0x7fffffff;
    for (size_t s = 0; s < desc->streams; ++s) {
        if (desc->projection_w[s] == nullptr || desc->audio_table[s] == nullptr) {
            set_error(error, capacity, "local_create: missing projection weight or audio table");
            return fail();
        }
        const CachedWeight *cw = nullptr;
        if (cached_matrix(st, desc->projection_w[s], desc->vocab, stack->width, st->qtype, &cw, error, capacity) != 0) return fail();
        if (!linear_fast_supported(cw->qtype, desc->vocab, stack->width)) {
            set_error(error, capacity, "local_create: projection shape not supported by the fused matvec");
            return fail();
        }
        l->projection.push_back(cw);
        const float *dev_bias = nullptr;
        if (cached_vector(st, desc->projection_bias != nullptr ? desc->projection_bias[s] : nullptr, desc->vocab, &dev_bias, error, capacity) != 0)
            return fail();
        l->projection_bias.push_back(dev_bias);
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
        alloc(reinterpret_cast<void **>(&l->logits), B * l->vocab * sizeof(float)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->frame), sizeof(LocalFrameDev)) != 0 ||
        alloc(reinterpret_cast<void **>(&l->values), 2 * B * l->streams * sizeof(unsigned)) != 0)
        return fail();
    if (hip_check(hipHostMalloc(reinterpret_cast<void **>(&l->frame_host), sizeof(LocalFrameDev), hipHostMallocDefault), "local frame staging", error, capacity) != 0 ||
        hip_check(hipHostMalloc(reinterpret_cast<void **>(&l->values_host), 2 * B * l->streams * sizeof(unsigned), hipHostMallocDefault), "local frame staging", error, capacity) != 0)
        return fail();
    *out = l;
    return 0;
}

extern "C" int mynah_hip_local_frame(void *state, mynah_hip_local *l, mynah_hip_local_item *items, size_t batch, unsigned *values,
                                     unsigned *stored, int *saw_eos, size_t *eos_frame, float *dev_logits_copy, char *error,
                                     size_t capacity) {
    State *st = enter_state(state);
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
    const int B = (int)batch;
    MYNAH_TRY(hipStreamSynchronize(st->stream));   // the staging buffers of the previous frame may still be in flight
    l->frame_host->logits_copy = dev_logits_copy;
    // a frame's many-stream attention launches wait like a decode step's, but a frame cannot be repeated from here (its
    // generator states have moved on): a wait given up inside it is reported as the error it is, never taken for a decode step's
    st->last_step_decoder = nullptr;
    st->steps_since_sync += 2;
    if (decoder_next_epochs(st, l->stack, (unsigned)l->streams, &l->frame_host->epoch_base, error, capacity) != 0) return -1;
    l->frame_host->reserved = 0;
    for (size_t b = 0; b < batch; ++b) {
        LocalItemDev &d = l->frame_host->items[b];
        d.decoder_last = items[b].dev_decoder_last;
        d.temperature = items[b].temperature;
        d.topk = items[b].topk > 0xffffffffu ? 0xffffffffu : (unsigned)items[b].topk;
        d.rng_state = items[b].rng_state;
        d.forbid_eos = items[b].forbid_eos;
        d.saw_eos = 0;
        d.eos_frame = ~0ull;
    }
    MYNAH_TRY(hipMemcpyAsync(l->frame, l->frame_host, sizeof(LocalFrameDev), hipMemcpyHostToDevice, st->stream));
    if (!st->graph_mode || l->eager_frames[B] == 0) {
        l->eager_frames[B] = 1;
        if (enqueue_frame(st, l, B, error, capacity) != 0) return -1;
    } else {
        if (l->graphs[B] == nullptr) {
            hipGraph_t graph = nullptr;
            MYNAH_TRY(hipStreamBeginCapture(st->stream, hipStreamCaptureModeThreadLocal));
            const int rc = enqueue_frame(st, l, B, error, capacity);
            const hipError_t end = hipStreamEndCapture(st->stream, &graph);
            if (rc != 0) {
                if (graph != nullptr) (void)hipGraphDestroy(graph);
                return -1;
            }
            MYNAH_TRY(end);
            const hipError_t inst = hipGraphInstantiate(&l->graphs[B], graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            if (hip_check(inst, "local frame graph instantiate", error, capacity) != 0) {
                l->graphs[B] = nullptr;
                return -1;
            }
        }
        MYNAH_TRY(hipGraphLaunch(l->graphs[B], st->stream));
    }
    MYNAH_TRY(hipMemcpyAsync(l->values_host, l->values, 2 * (size_t)kMaxBatch * l->streams * sizeof(unsigned), hipMemcpyDeviceToHost, st->stream));
    MYNAH_TRY(hipMemcpyAsync(l->frame_host, l->frame, sizeof(LocalFrameDev), hipMemcpyDeviceToHost, st->stream));
    if (synchronise(st, error, capacity) != 0) return -1;
    for (size_t b = 0; b < batch; ++b) {
        for (size_t s = 0; s < l->streams; ++s) {
            values[b * l->streams + s] = l->values_host[b * l->streams + s];
            stored[b * l->streams + s] = l->values_host[(size_t)kMaxBatch * l->streams + b * l->streams + s];
        }
        items[b].rng_state = l->frame_host->items[b].rng_state;
        saw_eos[b] = l->frame_host->items[b].saw_eos;
        eos_frame[b] = l->frame_host->items[b].eos_frame == ~0ull ? SIZE_MAX : (size_t)l->frame_host->items[b].eos_frame;
    }
    return 0;
}
