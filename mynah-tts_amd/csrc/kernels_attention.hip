// Single-token attention over an HBM-resident KV cache, spread over the whole chip.
//
// The reference walks one head at a time over the whole cache (src/graph.c:3182-3202 self,
// :3221-3247 cross; Metal: one threadgroup per head, gpu/metal/backend_metal_ops.m:605-621), which
// yields 12 units of work per stream -- far too few to pull HBM bandwidth on 256 CUs.  Here one
// workgroup owns (stream, head, chunk of 64 cache rows): 16 lanes read one 64-float K row as four
// coalesced float4 each, scores are reduced inside the 16-lane group, the chunk's (max, sum, partial
// output) goes to a small workspace, and the LAST workgroup of a (stream, head) to arrive folds the
// chunks in a fixed order with the usual log-sum-exp rescaling.  Which workgroup arrives last does not
// change the arithmetic, and the chunking depends only on the stream's own length, so a stream in a
// batch is bit-identical to the same stream alone.
//
// A decode step is a chain of ~100 dependent kernels, each a few microseconds long, so what matters
// inside a kernel is the number of dependent memory round trips.  The head_width == 64 path therefore
// issues every global load it will need (q, its four K rows and its four V rows) before it waits for
// anything, and the fold reads the partials with ordinary pipelined loads after the acquire fence.
//
// The self variant first appends this step's k/v at row `position` (src/graph.c:3180-3181): the
// workgroup whose chunk contains that row writes its head's slice of the cache row and takes the
// values from the qkv vector instead of reading them back.
#include "device_common.h"

namespace mynah {
namespace {

constexpr int kPosLanes = 16;                     // lanes cooperating on one cache row
constexpr int kPosPerPass = kThreads / kPosLanes; // 16 rows in flight per pass
constexpr int kRowsPerThread = kAttnChunk / kPosPerPass;   // 4

struct Resolved {
    const float *q;
    float *kc, *vc, *out;
    int valid, position;
};

__device__ __forceinline__ Resolved resolve(const AttnArgs &a, int b) {
    Resolved r;
    if (a.slots != nullptr) {
        const StepSlots *s = a.slots;
        if (a.is_self) {
            r.position = s->length[b];
            r.valid = r.position + 1;
            r.kc = s->self_k[b] + a.layer * a.capacity * (size_t)a.stride;
            r.vc = s->self_v[b] + a.layer * a.capacity * (size_t)a.stride;
        } else {
            r.position = -1;
            r.valid = s->memory_length[b];
            r.kc = const_cast<float *>(s->cross_k[b]) + a.layer * (size_t)r.valid * a.stride;
            r.vc = const_cast<float *>(s->cross_v[b]) + a.layer * (size_t)r.valid * a.stride;
        }
        r.q = a.q[0] + (size_t)b * a.q_stride;
        r.out = a.out[0] + (size_t)b * (a.heads * a.head_width);
    } else {
        r.position = a.is_self ? a.position[b] : -1;
        r.valid = a.valid[b];
        r.q = a.q[b];
        r.kc = a.k_cache[b];
        r.vc = a.v_cache[b];
        r.out = a.out[b];
    }
    return r;
}

// Unit layout for a stream without memory: one unit of zeros with sum 1, which folds to the zero row.
__device__ __forceinline__ void empty_unit(const AttnArgs &a, int b, int head, int hw) {
    for (int d = threadIdx.x; d < hw; d += kThreads) a.unit_partial[((size_t)b * a.heads + head) * a.max_chunks * hw + d] = 0.0f;
    if (threadIdx.x == 0) {
        a.unit_ml[((size_t)b * a.heads + head) * 2 * a.max_chunks] = 0.0f;
        a.unit_ml[((size_t)b * a.heads + head) * 2 * a.max_chunks + a.max_chunks] = 1.0f;
        if (head == 0) a.unit_slots->memory_length[b] = kStepUnitRows;
    }
}

// Softmax statistics of one chunk: s_score[0..63] holds scaled scores (-3e38 beyond `count`);
// afterwards it holds exp(score - max), and (max, sum) are in s_ml.
__device__ __forceinline__ void chunk_stats(float *s_score, float *s_ml, int count) {
    if (threadIdx.x < 64) {
        const float sc = s_score[threadIdx.x];
        const float m = wave_max(sc);
        const float e = (int)threadIdx.x < count ? expf(sc - m) : 0.0f;
        const float l = wave_sum(e);
        s_score[threadIdx.x] = e;
        if (threadIdx.x == 0) { s_ml[0] = m; s_ml[1] = l; }
    }
}

__device__ __forceinline__ void fold_chunks(const AttnArgs &a, const float *part, int nchunks, int hw, float *outh, float *s_w,
                                            float *s_fold);

// Publishes this chunk's (max, sum, partial output) and lets the last arrival of the (stream, head)
// fold all chunks: out = sum_c o_c e^(m_c - M) / sum_c l_c e^(m_c - M), chunks taken in four interleaved
// sequences (c = g, g+4, ...) that are then added in order g = 0..3 -- fixed, whoever folds.
__device__ __forceinline__ void publish_and_fold(const AttnArgs &a, int b, int head, int chunk, int nchunks, int hw,
                                                 const float *s_red, float m_c, float l_c, float *outh, float *s_w,
                                                 float *s_fold, int *s_last) {
    const int tid = threadIdx.x;
    const size_t pstride = (size_t)hw + 2;
    float *part = a.partial + (((size_t)b * a.heads + head) * a.max_chunks) * pstride;
    float *mine = part + (size_t)chunk * pstride;
    for (int d = tid; d < hw; d += kThreads) {
        float o = 0.0f;
#pragma unroll
        for (int gg = 0; gg < kPosPerPass; ++gg) o += s_red[(size_t)gg * hw + d];
        mine[2 + d] = o;
    }
    if (tid == 0) { mine[0] = m_c; mine[1] = l_c; }
    if (a.two_pass) return;   // a launch of k_attention_fold follows: the kernel boundary publishes the partials
    __syncthreads();   // every store of this workgroup has reached the L2 (workgroup-scope release) ...
    if (tid == 0) {
        __threadfence();   // ... and one device-scope release publishes them: a fence per wave would serialise hundreds of L2 write-backs
        unsigned *counter = a.counters + (size_t)b * a.heads + head;
        const unsigned before = atomicAdd(counter, 1u);
        const int last = (before == (unsigned)(nchunks - 1)) ? 1 : 0;
        if (last) *counter = 0u;   // every other chunk has already arrived: ready for the next launch
        *s_last = last;
    }
    __syncthreads();
    if (!*s_last) return;
    __threadfence();   // acquire: the partials below are read with ordinary loads
    fold_chunks(a, part, nchunks, hw, outh, s_w, s_fold);
}

// out = sum_c o_c e^(m_c - M) / sum_c l_c e^(m_c - M) over the chunks of one (stream, head), in a fixed order.
__device__ __forceinline__ void fold_chunks(const AttnArgs &a, const float *part, int nchunks, int hw, float *outh, float *s_w,
                                            float *s_fold) {
    const int tid = threadIdx.x;
    const size_t pstride = (size_t)hw + 2;
    // s_w[c] = m_c, s_w[max_chunks + c] = l_c
    for (int c = tid; c < nchunks; c += kThreads) {
        s_w[c] = part[(size_t)c * pstride];
        s_w[a.max_chunks + c] = part[(size_t)c * pstride + 1];
    }
    __syncthreads();
    float M = -3.0e38f;
    for (int c = 0; c < nchunks; ++c) M = fmaxf(M, s_w[c]);
    __syncthreads();
    for (int c = tid; c < nchunks; c += kThreads) s_w[c] = expf(s_w[c] - M);
    __syncthreads();
    float L = 0.0f;
    for (int c = 0; c < nchunks; ++c) L = __builtin_fmaf(s_w[a.max_chunks + c], s_w[c], L);

    const int gsize = hw <= 64 ? 64 : (hw <= 128 ? 128 : 256);
    const int ngroups = kThreads / gsize;
    const int g = tid / gsize;
    for (int d0 = 0; d0 < hw; d0 += gsize) {
        const int d = d0 + (tid % gsize);
        float o = 0.0f;
        if (d < hw)
            for (int c = g; c < nchunks; c += ngroups) o = __builtin_fmaf(part[(size_t)c * pstride + 2 + d], s_w[c], o);
        s_fold[tid] = o;
        __syncthreads();
        if (g == 0 && d < hw) {
            float total = s_fold[tid];
            for (int gg = 1; gg < ngroups; ++gg) total += s_fold[gg * gsize + tid];
            outh[d] = total / L;
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------
// head_width == 64, aligned rows: everything prefetched, no LDS staging of q.
__global__ void __launch_bounds__(kThreads) k_attention_hw64(const AttnArgs a) {
    extern __shared__ __align__(16) float lds[];
    float *s_score = lds;                     // [64]
    float *s_red = s_score + kAttnChunk;      // [16][64]
    float *s_w = s_red + kPosPerPass * 64;    // [2 * max_chunks]
    float *s_fold = s_w + 2 * a.max_chunks;   // [256]
    __shared__ float s_ml[2];
    __shared__ int s_last;
    constexpr int hw = 64;

    const int chunk = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const Resolved r = resolve(a, b);
    const int nchunks = r.valid > 0 ? (r.valid + kAttnChunk - 1) / kAttnChunk : 1;
    if (chunk >= nchunks) return;
    const int width = a.heads * hw;
    float *outh = r.out + (size_t)head * hw;
    if (r.valid <= 0) {   // empty memory: the reference leaves the context at zero (src/graph.c:3242)
        if (tid < hw) outh[tid] = 0.0f;
        if (a.unit_partial != nullptr) empty_unit(a, b, head, hw);
        return;
    }
    const int p0 = chunk * kAttnChunk;
    const int count = min(kAttnChunk, r.valid - p0);
    const int j = tid & (kPosLanes - 1);
    const int g = tid / kPosLanes;
    const size_t col = (size_t)head * hw + 4 * j;

    // ---- every load this workgroup needs, issued before anything is consumed: unconditional global loads from a row
    // index clamped into the chunk (a request under a condition would make every later wait a wait for all of them);
    // rows past the chunk's end get the score -3e38 and the weight 0 below
    const float4 qv = load_global4(r.q + col);
    float4 kv[kRowsPerThread], vv[kRowsPerThread];
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int p = p0 + min(g + kPosPerPass * i, count - 1);
        const bool fresh = p == r.position;
        kv[i] = load_global4(fresh ? r.q + width + col : r.kc + (size_t)p * a.stride + col);
    }
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int p = p0 + min(g + kPosPerPass * i, count - 1);
        const bool fresh = p == r.position;
        vv[i] = load_global4(fresh ? r.q + 2 * (size_t)width + col : r.vc + (size_t)p * a.stride + col);
    }
    requests_issued();
    // ---- scores (+ append of the new row)
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int pi = g + kPosPerPass * i;
        const int p = p0 + pi;
        const bool in_range = pi < count;
        float dot = 0.0f;
        dot = __builtin_fmaf(qv.x, kv[i].x, dot);
        dot = __builtin_fmaf(qv.y, kv[i].y, dot);
        dot = __builtin_fmaf(qv.z, kv[i].z, dot);
        dot = __builtin_fmaf(qv.w, kv[i].w, dot);
        dot = row16_sum(dot);
        if (j == 0) s_score[pi] = in_range ? dot * a.scale : -3.0e38f;
        if (in_range && p == r.position) {
            *reinterpret_cast<float4 *>(r.kc + (size_t)p * a.stride + col) = kv[i];
            *reinterpret_cast<float4 *>(r.vc + (size_t)p * a.stride + col) = vv[i];
        }
    }
    __syncthreads();
    chunk_stats(s_score, s_ml, count);
    __syncthreads();
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const float e = s_score[g + kPosPerPass * i];   // 0 beyond `count`
        acc.x = __builtin_fmaf(e, vv[i].x, acc.x);
        acc.y = __builtin_fmaf(e, vv[i].y, acc.y);
        acc.z = __builtin_fmaf(e, vv[i].z, acc.z);
        acc.w = __builtin_fmaf(e, vv[i].w, acc.w);
    }
    *reinterpret_cast<float4 *>(s_red + (size_t)g * hw + 4 * j) = acc;
    __syncthreads();
    const float m_c = s_ml[0], l_c = s_ml[1];
    if (a.unit_partial != nullptr) {   // the consumer folds: leave this chunk's partial in its layout
        if (tid < hw) {
            float o = 0.0f;
#pragma unroll
            for (int gg = 0; gg < kPosPerPass; ++gg) o += s_red[(size_t)gg * hw + tid];
            a.unit_partial[(((size_t)b * a.heads + head) * a.max_chunks + chunk) * hw + tid] = o;
        }
        if (tid == 0) {
            a.unit_ml[((size_t)b * a.heads + head) * 2 * a.max_chunks + chunk] = m_c;
            a.unit_ml[((size_t)b * a.heads + head) * 2 * a.max_chunks + a.max_chunks + chunk] = l_c;
            if (chunk == 0 && head == 0) a.unit_slots->memory_length[b] = nchunks * kStepUnitRows;
        }
        return;
    }
    if (nchunks == 1) {
        if (tid < hw) {
            float o = 0.0f;
#pragma unroll
            for (int gg = 0; gg < kPosPerPass; ++gg) o += s_red[(size_t)gg * hw + tid];
            outh[tid] = o / l_c;
        }
        return;
    }
    publish_and_fold(a, b, head, chunk, nchunks, hw, s_red, m_c, l_c, outh, s_w, s_fold, &s_last);
}

// ------------------------------------------------------------------------------------------------
// Any head width (the engine passes one 768-wide head for cross attention, src/graph.c:3443-3448;
// self-test shapes are 2 wide).  VEC: head_width % 4 == 0 and all rows 16-byte aligned.
template <bool VEC>
__global__ void __launch_bounds__(kThreads) k_attention_any(const AttnArgs a) {
    extern __shared__ __align__(16) float lds[];
    const int hw = a.head_width;
    float *s_q = lds;                           // [hw]
    float *s_score = s_q + hw;                  // [64]
    float *s_red = s_score + kAttnChunk;        // [16][hw]
    float *s_w = s_red + (size_t)kPosPerPass * hw;   // [2 * max_chunks]
    float *s_fold = s_w + 2 * a.max_chunks;     // [256]
    __shared__ float s_ml[2];
    __shared__ int s_last;

    const int chunk = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const Resolved r = resolve(a, b);
    const int nchunks = r.valid > 0 ? (r.valid + kAttnChunk - 1) / kAttnChunk : 1;
    if (chunk >= nchunks) return;
    const int width = a.heads * hw;
    const float *qh = r.q + (size_t)head * hw;
    const float *knew = r.q + width + (size_t)head * hw;
    const float *vnew = r.q + 2 * (size_t)width + (size_t)head * hw;
    float *outh = r.out + (size_t)head * hw;
    if (r.valid <= 0) {
        for (int d = tid; d < hw; d += kThreads) outh[d] = 0.0f;
        return;
    }
    for (int d = tid; d < hw; d += kThreads) s_q[d] = qh[d];
    __syncthreads();

    const int p0 = chunk * kAttnChunk;
    const int count = min(kAttnChunk, r.valid - p0);
    const int j = tid & (kPosLanes - 1);
    const int g = tid / kPosLanes;

    for (int pi = g; pi < kAttnChunk; pi += kPosPerPass) {
        const int p = p0 + pi;
        const bool in_range = pi < count;
        const bool fresh = in_range && p == r.position;
        const float *krow = fresh ? knew : r.kc + (size_t)p * a.stride + (size_t)head * hw;
        float dot = 0.0f;
        if (in_range) {
            if constexpr (VEC) {
                for (int d = 4 * j; d < hw; d += 4 * kPosLanes) {
                    const float4 kv = *reinterpret_cast<const float4 *>(krow + d);
                    const float4 qv = *reinterpret_cast<const float4 *>(s_q + d);
                    dot = __builtin_fmaf(qv.x, kv.x, dot);
                    dot = __builtin_fmaf(qv.y, kv.y, dot);
                    dot = __builtin_fmaf(qv.z, kv.z, dot);
                    dot = __builtin_fmaf(qv.w, kv.w, dot);
                    if (fresh) *reinterpret_cast<float4 *>(r.kc + (size_t)p * a.stride + (size_t)head * hw + d) = kv;
                }
            } else {
                for (int d = j; d < hw; d += kPosLanes) {
                    const float kv = krow[d];
                    dot = __builtin_fmaf(s_q[d], kv, dot);
                    if (fresh) r.kc[(size_t)p * a.stride + (size_t)head * hw + d] = kv;
                }
            }
        }
        dot = row16_sum(dot);
        if (j == 0) s_score[pi] = in_range ? dot * a.scale : -3.0e38f;
    }
    __syncthreads();
    chunk_stats(s_score, s_ml, count);
    __syncthreads();

    if constexpr (VEC) {
        for (int d = 4 * j; d < hw; d += 4 * kPosLanes) {
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int pi = g; pi < count; pi += kPosPerPass) {
                const int p = p0 + pi;
                const bool fresh = p == r.position;
                const float *vrow = fresh ? vnew : r.vc + (size_t)p * a.stride + (size_t)head * hw;
                const float4 vv = *reinterpret_cast<const float4 *>(vrow + d);
                const float e = s_score[pi];
                acc.x = __builtin_fmaf(e, vv.x, acc.x);
                acc.y = __builtin_fmaf(e, vv.y, acc.y);
                acc.z = __builtin_fmaf(e, vv.z, acc.z);
                acc.w = __builtin_fmaf(e, vv.w, acc.w);
                if (fresh) *reinterpret_cast<float4 *>(r.vc + (size_t)p * a.stride + (size_t)head * hw + d) = vv;
            }
            *reinterpret_cast<float4 *>(s_red + (size_t)g * hw + d) = acc;
        }
    } else {
        for (int d = j; d < hw; d += kPosLanes) {
            float acc = 0.0f;
            for (int pi = g; pi < count; pi += kPosPerPass) {
                const int p = p0 + pi;
                const bool fresh = p == r.position;
                const float vv = fresh ? vnew[d] : r.vc[(size_t)p * a.stride + (size_t)head * hw + d];
                acc = __builtin_fmaf(s_score[pi], vv, acc);
                if (fresh) r.vc[(size_t)p * a.stride + (size_t)head * hw + d] = vv;
            }
            s_red[(size_t)g * hw + d] = acc;
        }
    }
    __syncthreads();

    const float m_c = s_ml[0], l_c = s_ml[1];
    if (nchunks == 1) {
        for (int d = tid; d < hw; d += kThreads) {
            float o = 0.0f;
#pragma unroll
            for (int gg = 0; gg < kPosPerPass; ++gg) o += s_red[(size_t)gg * hw + d];
            outh[d] = o / l_c;
        }
        return;
    }
    publish_and_fold(a, b, head, chunk, nchunks, hw, s_red, m_c, l_c, outh, s_w, s_fold, &s_last);
}


// ------------------------------------------------------------------------------------------------
// Second pass of the two-pass form: one workgroup per (stream, head) folds the chunks the first launch left in the
// workspace.  A device-scope release per workgroup costs about 60 ns of serialised L2 write-back, so with hundreds of
// chunk workgroups (twelve 64-wide heads over a long cache) two launches are shorter than one with a last-arrival fold.
__global__ void __launch_bounds__(kThreads) k_attention_fold(const AttnArgs a) {
    extern __shared__ __align__(16) float lds[];
    float *s_w = lds;                          // [2 * max_chunks]
    float *s_fold = s_w + 2 * a.max_chunks;    // [256]
    const int head = blockIdx.x, b = blockIdx.y;
    const Resolved r = resolve(a, b);
    const int nchunks = r.valid > 0 ? (r.valid + kAttnChunk - 1) / kAttnChunk : 1;
    if (nchunks <= 1) return;   // written by the first pass
    const int hw = a.head_width;
    const float *part = a.partial + (((size_t)b * a.heads + head) * a.max_chunks) * ((size_t)hw + 2);
    fold_chunks(a, part, nchunks, hw, r.out + (size_t)head * hw, s_w, s_fold);
}

// Fold of partials in the unit layout by a launch of its own: what the fused matvec's prologue forms when it is the
// consumer (the same device function), for the case that some other call comes next.
__global__ void __launch_bounds__(kThreads) k_unit_fold(const float *partial, const float *ml, const StepSlots *slots, int heads, int hw,
                                                        int max_units, const AttnArgs a, float *single_out) {
    const int f4 = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (f4 >= heads * hw / 4) return;
    ActSource src;
    src.partial = partial; src.partial_ml = ml; src.slots = slots; src.heads = heads; src.head_width = hw;
    src.max_units = max_units; src.is_self = 0; src.stream0 = 0;
    float *out = single_out != nullptr ? single_out : a.out[b];
    reinterpret_cast<float4 *>(out)[f4] = fold_partials(src, b, f4);
}

// ------------------------------------------------------------------------------------------------
// Wide heads (head_width = 256 * NV; the engine's cross attention is ONE head as wide as the model,
// src/graph.c:3443-3448), read-only caches.  With one head there are only valid / 64 workgroups of
// the kernel above, each walking 64 rows of 3 KB through a dozen dependent round trips.  Here a
// workgroup takes kWideRows rows, a wavefront takes a whole row per pass (lane l holds the float4 at
// columns 4 l + 256 i), and every row the workgroup will touch is requested before anything is used.
// Partial layout per chunk: out[hw], max, sum, 2 floats of padding (rows stay 16-byte aligned).
template <int NV>
__global__ void __launch_bounds__(kThreads) k_attention_wide(const AttnArgs a) {
    extern __shared__ __align__(16) float lds[];
    constexpr int hw = 256 * NV;
    constexpr int kPasses = kWideRows / 4;
    float *s_score = lds;                    // [64]
    float *s_red = s_score + kAttnChunk;     // [4][hw]
    float *s_w = s_red + 4 * hw;             // [2 * max_chunks]
    __shared__ float s_ml[2];
    __shared__ int s_last;

    const int chunk = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const Resolved r = resolve(a, b);
    const int nchunks = r.valid > 0 ? (r.valid + kWideRows - 1) / kWideRows : 1;
    if (chunk >= nchunks) return;
    float *outh = r.out + (size_t)head * hw;
    if (r.valid <= 0) {   // empty memory: the context stays zero (src/graph.c:3242)
        for (int d = tid; d < hw; d += kThreads) outh[d] = 0.0f;
        if (a.unit_partial != nullptr) empty_unit(a, b, head, hw);
        return;
    }
    const int p0 = chunk * kWideRows;
    const int count = min(kWideRows, r.valid - p0);
    const size_t col = (size_t)head * hw + 4 * lane;

    // ---- every request first, from a row index clamped into the chunk (rows past its end get the weight 0)
    float4 qv[NV], kv[kPasses][NV], vv[kPasses][NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) qv[i] = load_global4(r.q + col + 256 * i);
#pragma unroll
    for (int rr = 0; rr < kPasses; ++rr) {
        const int p = p0 + min(wave + 4 * rr, count - 1);
        const float *krow = r.kc + (size_t)p * a.stride + col;
#pragma unroll
        for (int i = 0; i < NV; ++i) kv[rr][i] = load_global4(krow + 256 * i);
    }
#pragma unroll
    for (int rr = 0; rr < kPasses; ++rr) {
        const int p = p0 + min(wave + 4 * rr, count - 1);
        const float *vrow = r.vc + (size_t)p * a.stride + col;
#pragma unroll
        for (int i = 0; i < NV; ++i) vv[rr][i] = load_global4(vrow + 256 * i);
    }
    requests_issued();
    if (tid >= kWideRows && tid < kAttnChunk) s_score[tid] = -3.0e38f;
#pragma unroll
    for (int rr = 0; rr < kPasses; ++rr) {
        const int pi = wave + 4 * rr;
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            dot = __builtin_fmaf(qv[i].x, kv[rr][i].x, dot);
            dot = __builtin_fmaf(qv[i].y, kv[rr][i].y, dot);
            dot = __builtin_fmaf(qv[i].z, kv[rr][i].z, dot);
            dot = __builtin_fmaf(qv[i].w, kv[rr][i].w, dot);
        }
        dot = wave_sum(dot);
        if (lane == 0) s_score[pi] = pi < count ? dot * a.scale : -3.0e38f;
    }
    __syncthreads();
    chunk_stats(s_score, s_ml, count);
    __syncthreads();
    float4 acc[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int rr = 0; rr < kPasses; ++rr) {
        const float e = s_score[wave + 4 * rr];   // 0 beyond `count`
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            acc[i].x = __builtin_fmaf(e, vv[rr][i].x, acc[i].x);
            acc[i].y = __builtin_fmaf(e, vv[rr][i].y, acc[i].y);
            acc[i].z = __builtin_fmaf(e, vv[rr][i].z, acc[i].z);
            acc[i].w = __builtin_fmaf(e, vv[rr][i].w, acc[i].w);
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) *reinterpret_cast<float4 *>(s_red + (size_t)wave * hw + 4 * lane + 256 * i) = acc[i];
    __syncthreads();
    const float m_c = s_ml[0], l_c = s_ml[1];
    // the four wavefronts' sums, in order; thread t owns the float4 column t
    const bool owner = tid < hw / 4;
    float4 mine = make_float4(0.f, 0.f, 0.f, 0.f);
    if (owner) {
        mine = *reinterpret_cast<const float4 *>(s_red + 4 * tid);
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const float4 o = *reinterpret_cast<const float4 *>(s_red + (size_t)w * hw + 4 * tid);
            mine.x += o.x; mine.y += o.y; mine.z += o.z; mine.w += o.w;
        }
    }
    if (a.unit_partial != nullptr) {   // the consumer folds: leave this chunk's partial in its layout
        if (owner) *reinterpret_cast<float4 *>(a.unit_partial + (((size_t)b * a.heads + head) * a.max_chunks + chunk) * hw + 4 * tid) = mine;
        if (tid == 0) {
            a.unit_ml[((size_t)b * a.heads + head) * 2 * a.max_chunks + chunk] = m_c;
            a.unit_ml[((size_t)b * a.heads + head) * 2 * a.max_chunks + a.max_chunks + chunk] = l_c;
            if (chunk == 0 && head == 0) a.unit_slots->memory_length[b] = nchunks * kStepUnitRows;
        }
        return;
    }
    if (nchunks == 1) {
        if (owner) *reinterpret_cast<float4 *>(outh + 4 * tid) = make_float4(mine.x / l_c, mine.y / l_c, mine.z / l_c, mine.w / l_c);
        return;
    }
    constexpr size_t pstride = hw + 4;
    float *part = a.partial + (((size_t)b * a.heads + head) * a.max_chunks) * pstride;
    float *slot = part + (size_t)chunk * pstride;
    if (owner) *reinterpret_cast<float4 *>(slot + 4 * tid) = mine;
    if (tid == 0) { slot[hw] = m_c; slot[hw + 1] = l_c; }
    __syncthreads();   // the workgroup's stores are in the L2 ...
    if (tid == 0) {
        __threadfence();   // ... and one device-scope release publishes them
        unsigned *counter = a.counters + (size_t)b * a.heads + head;
        const unsigned before = atomicAdd(counter, 1u);
        const int last = (before == (unsigned)(nchunks - 1)) ? 1 : 0;
        if (last) *counter = 0u;   // every other chunk has arrived: ready for the next launch
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();   // acquire

    // fold, chunks in index order: out = sum_c o_c e^(m_c - M) / sum_c l_c e^(m_c - M)
    for (int c = tid; c < nchunks; c += kThreads) {
        s_w[c] = part[(size_t)c * pstride + hw];
        s_w[a.max_chunks + c] = part[(size_t)c * pstride + hw + 1];
    }
    __syncthreads();
    float M = -3.0e38f;
    for (int c = 0; c < nchunks; ++c) M = fmaxf(M, s_w[c]);
    __syncthreads();
    for (int c = tid; c < nchunks; c += kThreads) s_w[c] = expf(s_w[c] - M);
    __syncthreads();
    float L = 0.0f;
    for (int c = 0; c < nchunks; ++c) L = __builtin_fmaf(s_w[a.max_chunks + c], s_w[c], L);
    if (!owner) return;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int c0 = 0; c0 < nchunks; c0 += 8) {
        float4 pv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) pv[u] = *reinterpret_cast<const float4 *>(part + (size_t)min(c0 + u, nchunks - 1) * pstride + 4 * tid);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float w = c0 + u < nchunks ? s_w[min(c0 + u, nchunks - 1)] : 0.0f;
            o.x = __builtin_fmaf(pv[u].x, w, o.x);
            o.y = __builtin_fmaf(pv[u].y, w, o.y);
            o.z = __builtin_fmaf(pv[u].z, w, o.z);
            o.w = __builtin_fmaf(pv[u].w, w, o.w);
        }
    }
    *reinterpret_cast<float4 *>(outh + 4 * tid) = make_float4(o.x / L, o.y / L, o.z / L, o.w / L);
}

}  // namespace

int launch_unit_fold(State *st, const float *partial, const float *ml, const StepSlots *slots, int heads, int head_width,
                     int max_units, float *out, char *error, size_t capacity) {
    const int f4 = heads * head_width / 4;
    hipLaunchKernelGGL(k_unit_fold, dim3((unsigned)((f4 + kThreads - 1) / kThreads), 1u), dim3(kThreads), 0, st->stream, partial, ml, slots, heads,
                       head_width, max_units, AttnArgs{}, out);
    return hip_check(hipGetLastError(), "unit fold launch", error, capacity);
}

// The same for every stream of a table-mode call, into the call's own output rows.
int launch_unit_fold_streams(State *st, const AttnArgs &a, char *error, size_t capacity) {
    const int f4 = a.heads * a.head_width / 4;
    hipLaunchKernelGGL(k_unit_fold, dim3((unsigned)((f4 + kThreads - 1) / kThreads), (unsigned)a.batch), dim3(kThreads), 0, st->stream,
                       a.unit_partial, a.unit_ml, a.unit_slots, a.heads, a.head_width, a.max_chunks, a, static_cast<float *>(nullptr));
    return hip_check(hipGetLastError(), "unit fold launch", error, capacity);
}

// Rows of the cache one workgroup takes for this call: kWideRows when the wide-head kernel applies, else kAttnChunk.
int attention_chunk_rows(int is_self, size_t head_width, bool vector_rows, size_t max_valid) {
    const bool wide = !is_self && vector_rows && head_width >= 256 && head_width <= 1024 && head_width % 256 == 0 &&
                      (max_valid + kWideRows - 1) / kWideRows <= 4096;
    return wide ? kWideRows : kAttnChunk;
}

int launch_attention(State *st, const AttnArgs &a, char *error, size_t capacity) {
    if (a.batch < 1 || a.batch > kMaxBatch || a.heads < 1 || a.head_width < 1 || a.head_width > 1024 ||
        a.max_chunks < 1 || a.max_chunks > 4096 || a.partial == nullptr || a.counters == nullptr) {
        set_error(error, capacity, "attention: invalid shape");
        return -1;
    }
    const bool vec = (a.head_width % 4) == 0 && (a.stride % 4) == 0 && (a.q_stride % 4) == 0;
    const bool fast = vec && a.head_width == 64;
    if (a.chunk_rows == kWideRows) {
        if (a.chunk_rows != attention_chunk_rows(a.is_self, (size_t)a.head_width, vec, 1)) {
            set_error(error, capacity, "attention: the wide-head kernel does not take this shape");
            return -1;
        }
        const size_t wide_lds = (kAttnChunk + 4 * (size_t)a.head_width + 2 * (size_t)a.max_chunks) * sizeof(float);
        const dim3 wide_grid((unsigned)a.max_chunks, (unsigned)a.heads, (unsigned)a.batch);
        switch (a.head_width / 256) {
            case 1: hipLaunchKernelGGL(k_attention_wide<1>, wide_grid, dim3(kThreads), wide_lds, st->stream, a); break;
            case 2: hipLaunchKernelGGL(k_attention_wide<2>, wide_grid, dim3(kThreads), wide_lds, st->stream, a); break;
            case 3: hipLaunchKernelGGL(k_attention_wide<3>, wide_grid, dim3(kThreads), wide_lds, st->stream, a); break;
            default: hipLaunchKernelGGL(k_attention_wide<4>, wide_grid, dim3(kThreads), wide_lds, st->stream, a); break;
        }
        return hip_check(hipGetLastError(), "attention launch", error, capacity);
    }
    const size_t hw = (size_t)a.head_width;
    const size_t lds = ((fast ? 0 : hw) + kAttnChunk + (size_t)kPosPerPass * hw + 2 * (size_t)a.max_chunks + kThreads) * sizeof(float);
    const dim3 grid((unsigned)a.max_chunks, (unsigned)a.heads, (unsigned)a.batch);
    static bool raised[2] = {false, false};
    if (lds > 48 * 1024 && !fast && !raised[vec ? 1 : 0]) {
        const void *fn = vec ? reinterpret_cast<const void *>(&k_attention_any<true>) : reinterpret_cast<const void *>(&k_attention_any<false>);
        MYNAH_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        raised[vec ? 1 : 0] = true;
    }
    if (lds > 128 * 1024) {
        set_error(error, capacity, "attention: head width and cache length exceed the workgroup's LDS");
        return -1;
    }
    // many chunk workgroups: fold in a second launch instead of a device-scope release per workgroup
    AttnArgs args = a;
    args.two_pass = a.unit_partial == nullptr && a.max_chunks > 1 && (size_t)a.max_chunks * a.heads * a.batch >= 64 ? 1 : 0;
    if (a.unit_partial != nullptr && !fast) {
        set_error(error, capacity, "attention: the unit layout is written by the 64-wide and the wide-head kernels only");
        return -1;
    }
    if (fast) hipLaunchKernelGGL(k_attention_hw64, grid, dim3(kThreads), lds, st->stream, args);
    else if (vec) hipLaunchKernelGGL(k_attention_any<true>, grid, dim3(kThreads), lds, st->stream, args);
    else hipLaunchKernelGGL(k_attention_any<false>, grid, dim3(kThreads), lds, st->stream, args);
    if (args.two_pass) {
        if (hip_check(hipGetLastError(), "attention launch", error, capacity) != 0) return -1;
        const size_t fold_lds = (2 * (size_t)a.max_chunks + kThreads) * sizeof(float);
        hipLaunchKernelGGL(k_attention_fold, dim3((unsigned)a.heads, (unsigned)a.batch), dim3(kThreads), fold_lds, st->stream, args);
    }
    return hip_check(hipGetLastError(), "attention launch", error, capacity);
}

}  // namespace mynah
