// Single-token attention over an HBM-resident KV cache, spread over the whole chip.
//
// The reference walks one head at a time over the whole cache (src/graph.c:3182-3202 self,
// :3221-3247 cross; Metal: one threadgroup per head, gpu/metal/backend_metal_ops.m:605-621), which
// yields 12 units of work per stream -- far too few to pull HBM bandwidth on 256 CUs.  Here one
// workgroup owns (stream, head, chunk of 64 cache rows): 16 lanes read one 64-float K row as four
// coalesced float4 each, scores are reduced inside the 16-lane group, the chunk's (max, sum, partial
// output) goes to a small workspace, and the LAST workgroup of a (stream, head) to arrive folds the
// chunks in chunk order with the usual log-sum-exp rescaling.  Which workgroup arrives last does not
// change the arithmetic, and the chunking depends only on the stream's own length, so a stream in a
// batch is bit-identical to the same stream alone.
//
// The self variant first appends this step's k/v at row `position` (src/graph.c:3180-3181): the
// workgroup whose chunk contains that row writes its head's slice of the cache row and takes the
// values from the qkv vector instead of reading them back.
#include "kernels.h"

namespace mynah {
namespace {

constexpr int kThreads = 256;
constexpr int kPosLanes = 16;                    // lanes cooperating on one cache row
constexpr int kPosPerPass = kThreads / kPosLanes; // 16 rows in flight per pass

__device__ __forceinline__ float group16_sum(float v) {
    v += __shfl_xor(v, 8);
    v += __shfl_xor(v, 4);
    v += __shfl_xor(v, 2);
    v += __shfl_xor(v, 1);
    return v;
}

// VEC: head_width % 4 == 0 and all rows 16-byte aligned -> float4 path
template <bool VEC>
__global__ void __launch_bounds__(kThreads) k_attention(const AttnArgs a) {
    extern __shared__ __align__(16) float lds[];
    const int hw = a.head_width;
    float *s_q = lds;                      // [hw]
    float *s_score = s_q + hw;             // [kAttnChunk]
    float *s_red = s_score + kAttnChunk;   // [kPosPerPass][hw]
    __shared__ float s_m, s_l;
    __shared__ int s_last;

    const int chunk = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    int valid, position;
    const float *q;
    float *kc, *vc, *out;
    if (a.slots != nullptr) {
        const StepSlots *s = a.slots;
        if (a.is_self) {
            position = s->length[b];
            valid = position + 1;
            kc = s->self_k[b] + a.layer * a.capacity * (size_t)a.stride;
            vc = s->self_v[b] + a.layer * a.capacity * (size_t)a.stride;
        } else {
            position = -1;
            valid = s->memory_length[b];
            kc = const_cast<float *>(s->cross_k[b]) + a.layer * (size_t)valid * a.stride;
            vc = const_cast<float *>(s->cross_v[b]) + a.layer * (size_t)valid * a.stride;
        }
        q = a.q[0] + (size_t)b * a.q_stride;
        out = a.out[0] + (size_t)b * (a.heads * hw);
    } else {
        position = a.is_self ? a.position[b] : -1;
        valid = a.valid[b];
        q = a.q[b];
        kc = a.k_cache[b];
        vc = a.v_cache[b];
        out = a.out[b];
    }
    const int nchunks = valid > 0 ? (valid + kAttnChunk - 1) / kAttnChunk : 1;
    if (chunk >= nchunks) return;

    const int width = a.heads * hw;
    const float *qh = q + (size_t)head * hw;
    const float *knew = q + width + (size_t)head * hw;       // self only
    const float *vnew = q + 2 * (size_t)width + (size_t)head * hw;
    float *outh = out + (size_t)head * hw;

    if (valid <= 0) {   // empty memory: the reference leaves the context at zero (src/graph.c:3242)
        for (int d = tid; d < hw; d += kThreads) outh[d] = 0.0f;
        return;
    }

    for (int d = tid; d < hw; d += kThreads) s_q[d] = qh[d];
    __syncthreads();

    const int p0 = chunk * kAttnChunk;
    const int count = min(kAttnChunk, valid - p0);
    const int j = tid & (kPosLanes - 1);     // lane inside the row group
    const int g = tid / kPosLanes;           // row group 0..15

    // ---- scores
    for (int pi = g; pi < kAttnChunk; pi += kPosPerPass) {
        const int p = p0 + pi;
        const bool in_range = pi < count;
        const bool fresh = in_range && p == position;
        const float *krow = fresh ? knew : kc + (size_t)p * a.stride + (size_t)head * hw;
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
                    if (fresh) *reinterpret_cast<float4 *>(kc + (size_t)p * a.stride + (size_t)head * hw + d) = kv;
                }
            } else {
                for (int d = j; d < hw; d += kPosLanes) {
                    const float kv = krow[d];
                    dot = __builtin_fmaf(s_q[d], kv, dot);
                    if (fresh) kc[(size_t)p * a.stride + (size_t)head * hw + d] = kv;
                }
            }
        }
        dot = group16_sum(dot);
        if (j == 0) s_score[pi] = in_range ? dot * a.scale : -3.0e38f;
    }
    __syncthreads();

    // ---- chunk softmax statistics (one wave, 64 scores)
    if (tid < 64) {
        const float sc = s_score[tid];
        float m = sc;
#pragma unroll
        for (int x = 32; x > 0; x >>= 1) m = fmaxf(m, __shfl_xor(m, x));
        const float e = tid < count ? expf(sc - m) : 0.0f;
        float l = e;
#pragma unroll
        for (int x = 32; x > 0; x >>= 1) l += __shfl_xor(l, x);
        s_score[tid] = e;
        if (tid == 0) { s_m = m; s_l = l; }
    }
    __syncthreads();

    // ---- weighted sum of V rows: each row group accumulates its rows, then groups are folded in order
    if constexpr (VEC) {
        for (int d = 4 * j; d < hw; d += 4 * kPosLanes) {
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int pi = g; pi < count; pi += kPosPerPass) {
                const int p = p0 + pi;
                const bool fresh = p == position;
                const float *vrow = fresh ? vnew : vc + (size_t)p * a.stride + (size_t)head * hw;
                const float4 vv = *reinterpret_cast<const float4 *>(vrow + d);
                const float e = s_score[pi];
                acc.x = __builtin_fmaf(e, vv.x, acc.x);
                acc.y = __builtin_fmaf(e, vv.y, acc.y);
                acc.z = __builtin_fmaf(e, vv.z, acc.z);
                acc.w = __builtin_fmaf(e, vv.w, acc.w);
                if (fresh) *reinterpret_cast<float4 *>(vc + (size_t)p * a.stride + (size_t)head * hw + d) = vv;
            }
            *reinterpret_cast<float4 *>(s_red + (size_t)g * hw + d) = acc;
        }
    } else {
        for (int d = j; d < hw; d += kPosLanes) {
            float acc = 0.0f;
            for (int pi = g; pi < count; pi += kPosPerPass) {
                const int p = p0 + pi;
                const bool fresh = p == position;
                const float vv = fresh ? vnew[d] : vc[(size_t)p * a.stride + (size_t)head * hw + d];
                acc = __builtin_fmaf(s_score[pi], vv, acc);
                if (fresh) vc[(size_t)p * a.stride + (size_t)head * hw + d] = vv;
            }
            s_red[(size_t)g * hw + d] = acc;
        }
    }
    __syncthreads();

    const float m_c = s_m, l_c = s_l;
    if (nchunks == 1) {
        for (int d = tid; d < hw; d += kThreads) {
            float o = 0.0f;
#pragma unroll
            for (int gg = 0; gg < kPosPerPass; ++gg) o += s_red[(size_t)gg * hw + d];
            outh[d] = o / l_c;
        }
        return;
    }

    // ---- several chunks: publish the partial, the last arrival folds them
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
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        unsigned *counter = a.counters + (size_t)b * a.heads + head;
        const unsigned before = atomicAdd(counter, 1u);
        s_last = (before == (unsigned)(nchunks - 1)) ? 1 : 0;
        if (s_last) *counter = 0u;   // every other chunk has already arrived: ready for the next launch
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();

    float M = -3.0e38f;
    for (int c = 0; c < nchunks; ++c) M = fmaxf(M, __hip_atomic_load(part + (size_t)c * pstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    float L = 0.0f;
    for (int c = 0; c < nchunks; ++c) {
        const float mc = __hip_atomic_load(part + (size_t)c * pstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float lc = __hip_atomic_load(part + (size_t)c * pstride + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        L = __builtin_fmaf(lc, expf(mc - M), L);
    }
    for (int d = tid; d < hw; d += kThreads) {
        float o = 0.0f;
        for (int c = 0; c < nchunks; ++c) {
            const float mc = __hip_atomic_load(part + (size_t)c * pstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float oc = __hip_atomic_load(part + (size_t)c * pstride + 2 + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            o = __builtin_fmaf(oc, expf(mc - M), o);
        }
        outh[d] = o / L;
    }
}

}  // namespace

int launch_attention(State *st, const AttnArgs &a, char *error, size_t capacity) {
    if (a.batch < 1 || a.batch > kMaxBatch || a.heads < 1 || a.head_width < 1 || a.head_width > 1024 ||
        a.max_chunks < 1 || a.partial == nullptr || a.counters == nullptr) {
        set_error(error, capacity, "attention: invalid shape");
        return -1;
    }
    const size_t lds = ((size_t)a.head_width * (1 + kPosPerPass) + kAttnChunk) * sizeof(float);
    const bool vec = (a.head_width % 4) == 0 && (a.stride % 4) == 0 && (a.q_stride % 4) == 0;
    const dim3 grid((unsigned)a.max_chunks, (unsigned)a.heads, (unsigned)a.batch);
    static bool raised[2] = {false, false};
    if (lds > 48 * 1024 && !raised[vec ? 1 : 0]) {
        const void *fn = vec ? reinterpret_cast<const void *>(&k_attention<true>) : reinterpret_cast<const void *>(&k_attention<false>);
        MYNAH_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        raised[vec ? 1 : 0] = true;
    }
    if (vec) hipLaunchKernelGGL(k_attention<true>, grid, dim3(kThreads), lds, st->stream, a);
    else hipLaunchKernelGGL(k_attention<false>, grid, dim3(kThreads), lds, st->stream, a);
    return hip_check(hipGetLastError(), "attention launch", error, capacity);
}

}  // namespace mynah
