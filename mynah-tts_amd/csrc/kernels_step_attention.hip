// Attention stage of the resident decode step, fused with the projection that feeds it.
//
// decoder_step_batch (src/graph.c:3161-3205, :3213-3247) runs LayerNorm -> Q(KV) projection -> per-head
// attention as separate passes.  On this GPU every pass boundary is a grid-wide dependency that costs
// several microseconds, more than the work between two of them, so here one workgroup does all of it
// for one (head, stream, unit):
//     LayerNorm(x) -> int8 activation quantisation -> this head's 64 rows of the Q projection
//     -> scores against one 128-row unit of the K cache -> unit softmax statistics -> weighted V rows
//     -> partial (max, sum, output[64]) to a workspace.
// Units of a stream: its cache chunks, plus -- for self-attention -- one "new row" unit that also
// computes this head's K and V rows of the step, appends them to the cache (src/graph.c:3180-3181) and
// contributes the new row's own score.  The next kernel (the output projection) folds the partials in
// its prologue, so no fence, atomic or second pass is needed here.  How a stream is cut into units
// depends on its own length only, and a unit's arithmetic on nothing but its own inputs, so a stream in
// a batch is bit-identical to the same stream alone.
//
// The LayerNorm/quantisation is recomputed per workgroup (3 KB of input), and the 64 x 768 weight slice
// of a head is read by every unit of that head.  Work items are ordered head-major and cut into eight
// contiguous ranges, one per XCD (workgroup i runs on XCD i % 8): a head's slice is fetched from HBM by
// at most two XCDs and served to the other units from their L2, and since every head carries the same
// work the XCDs stay balanced whatever the streams' lengths are.
//
// The mapping from workgroup to (head, stream, unit) is static, so the weight slice and x are requested
// before the slot table (lengths, cache pointers) has arrived; K and V rows follow as soon as it has.
#include "device_common.h"

namespace mynah {
namespace {

constexpr int kHw = 64;                          // head width handled by the fused kernel
constexpr int kPosLanes = 16;                    // lanes cooperating on one cache row
constexpr int kPosPerPass = kThreads / kPosLanes;
constexpr int kRowsPerThread = kStepUnitRows / kPosPerPass;   // 8
constexpr int kPrefetchPasses = 4;

struct PassRegs {
    uint4 wv[4];
    float sc[4];
};

// Weight row of projection output r for this head: r = part * 64 + i, part 0/1/2 = q/k/v.
__device__ __forceinline__ int weight_row(int r, int head, int width) { return (r >> 6) * width + head * kHw + (r & 63); }

template <int QT>
__device__ __forceinline__ void load_pass(PassRegs &p, const StepAttnArgs &a, int pass, int row0, int nrows, int head, int lg, int chunks) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int G = 1 << lg, gl = lane & (G - 1), gidx = lane >> lg;
    const int rpp = 64 >> lg;
    int r = row0 + pass * 4 * rpp + wave * rpp + gidx;
    if (r >= row0 + nrows) r = row0 + nrows - 1;
    const int wrow_id = weight_row(r, head, a.width);
    const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(a.w) + (size_t)wrow_id * chunks * 16);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int c = gl + u * G;
        p.wv[u] = c < chunks ? wrow[c] : make_uint4(0, 0, 0, 0);
        p.sc[u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? a.scales[(size_t)wrow_id * chunks + c] : 0.0f;
    }
}

// Projection rows [row0, row0 + nrows) of this head (row numbering of weight_row) -> s_proj.
// `pre` holds the first kPrefetchPasses passes when `preloaded`.
template <int QT>
__device__ __forceinline__ void project_rows(const StepAttnArgs &a, PassRegs (&pre)[kPrefetchPasses], bool preloaded, int row0, int nrows,
                                             int head, int lg, int chunks, const unsigned char *smem, const float sx, float *s_proj) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int G = 1 << lg, gl = lane & (G - 1), gidx = lane >> lg;
    const int rpp = 64 >> lg;
    const int passes = (nrows + 4 * rpp - 1) / (4 * rpp);
    for (int pb = 0; pb < passes; pb += kPrefetchPasses) {
        if (pb > 0 || !preloaded) {
#pragma unroll
            for (int p = 0; p < kPrefetchPasses; ++p)
                if (pb + p < passes) load_pass<QT>(pre[p], a, pb + p, row0, nrows, head, lg, chunks);
        }
#pragma unroll
        for (int p = 0; p < kPrefetchPasses; ++p) {
            const int pass = pb + p;
            if (pass < passes) {
                const int r = row0 + pass * 4 * rpp + wave * rpp + gidx;
                int iacc[1] = {0};
                float facc[1] = {0.0f};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int c = gl + u * G;
                    if (c < chunks) dot_chunk<QT, 1>(pre[p].wv[u], pre[p].sc[u], c, smem, a.width, iacc, facc, nullptr);
                }
                group_reduce<QT, 1>(iacc, facc, lg);
                if (gl == 0 && r < row0 + nrows) {
                    float wscale = 1.0f;
                    if constexpr (QT == MYNAH_HIP_INT8) wscale = a.scales[weight_row(r, head, a.width)];
                    s_proj[r] = finish_value<QT>(iacc[0], facc[0], wscale, sx);
                }
            }
        }
    }
}

template <int QT, int NVT>
__global__ void __launch_bounds__(kThreads) k_step_attention(const StepAttnArgs a, const int lg, const int per_xcd) {
    extern __shared__ __align__(16) unsigned char smem[];   // staged activations: width bytes (int8/int4) or floats
    __shared__ __align__(16) float s_proj[3 * kHw];         // q | k | v of this head
    __shared__ __align__(16) float s_score[kStepUnitRows];
    __shared__ __align__(16) float s_red[kPosPerPass * kHw];
    __shared__ float s_sx[1];
    __shared__ float s_scratch[4];
    __shared__ float s_ml[2];

    const int tid = threadIdx.x;
    const StepSlots *slots = a.slots;

    // ---- static work decode: item = (head * batch + stream) * max_units + unit, XCD x owns items [x*per_xcd, (x+1)*per_xcd)
    const int items = a.heads * a.batch * a.max_units;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int item = xcd * per_xcd + slot;
    if (slot >= per_xcd || item >= items) return;
    const int unit = item % a.max_units;
    const int hb = item / a.max_units;
    const int b = hb % a.batch;
    const int head = hb / a.batch;

    constexpr int kEpc = Chunk<QT>::n;
    const int chunks = a.width / kEpc;

    // ---- requests that need neither activations nor the slot table: the head's Q weight rows
    PassRegs pre[kPrefetchPasses];
    const int rpp = 64 >> lg;
    const int q_passes = (kHw + 4 * rpp - 1) / (4 * rpp);
#pragma unroll
    for (int p = 0; p < kPrefetchPasses; ++p)
        if (p < q_passes) load_pass<QT>(pre[p], a, p, 0, kHw, head, lg, chunks);

    // ---- slot table: is this unit live, and where are its cache rows?
    const int units_b = attention_units(slots, b, a.is_self);
    if (unit >= units_b) return;
    const int length = a.is_self ? slots->length[b] : slots->memory_length[b];   // cache rows that exist before this step
    const bool new_row = a.is_self && unit == units_b - 1;
    const int stride = a.heads * kHw;   // floats between cache rows
    float *kc, *vc;
    if (a.is_self) {
        kc = slots->self_k[b] + a.layer * a.capacity * (size_t)stride;
        vc = slots->self_v[b] + a.layer * a.capacity * (size_t)stride;
    } else {
        kc = const_cast<float *>(slots->cross_k[b]) + a.layer * (size_t)length * stride;
        vc = const_cast<float *>(slots->cross_v[b]) + a.layer * (size_t)length * stride;
    }
    const int j = tid & (kPosLanes - 1);
    const int g = tid / kPosLanes;
    const size_t col = (size_t)head * kHw + 4 * j;
    const int p0 = unit * kStepUnitRows;
    const int count = new_row ? 0 : max(0, min(kStepUnitRows, length - p0));
    float4 kv[kRowsPerThread], vv[kRowsPerThread];
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int pi = g + kPosPerPass * i;
        const bool in_range = pi < count;
        kv[i] = in_range ? *reinterpret_cast<const float4 *>(kc + (size_t)(p0 + pi) * stride + col) : make_float4(0.f, 0.f, 0.f, 0.f);
        vv[i] = in_range ? *reinterpret_cast<const float4 *>(vc + (size_t)(p0 + pi) * stride + col) : make_float4(0.f, 0.f, 0.f, 0.f);
    }

    // ---- LayerNorm + activation quantisation of x[b], staged in LDS
    {
        PrologueParams p;
        p.k = a.width; p.batch = 1; p.ln_gain = a.ln_gain; p.ln_bias = a.ln_bias; p.arith = a.arith;
        p.probe_qx = nullptr; p.probe_sx = nullptr;
        ActSource src;
        src.rows[0] = a.x + (size_t)b * a.width;
        src.partial = nullptr;
        stage_activations<QT, 1, NVT>(p, src, smem, s_sx, s_scratch);
    }

    // ---- this head's projection rows -> s_proj (q always; k and v for the new-row unit)
    project_rows<QT>(a, pre, true, 0, kHw, head, lg, chunks, smem, s_sx[0], s_proj);
    if (new_row) project_rows<QT>(a, pre, false, kHw, 2 * kHw, head, lg, chunks, smem, s_sx[0], s_proj);
    __syncthreads();

    const size_t sh = (size_t)b * a.heads + head;
    float *out_m = a.partial_ml + sh * 2 * a.max_units;
    float *out_l = out_m + a.max_units;
    float *out_o = a.partial + (sh * a.max_units + unit) * kHw;

    if (new_row) {
        // append this step's k / v (this head's slice) and contribute the new row's own score
        if (tid < kHw) kc[(size_t)length * stride + (size_t)head * kHw + tid] = s_proj[kHw + tid];
        else if (tid < 2 * kHw) vc[(size_t)length * stride + (size_t)head * kHw + (tid - kHw)] = s_proj[2 * kHw + (tid - kHw)];
        if (tid < 64) {
            float d = s_proj[tid] * s_proj[kHw + tid];
            d = wave_sum(d);
            out_o[tid] = s_proj[2 * kHw + tid];   // exp(score - max) = 1
            if (tid == 0) { out_m[unit] = d * a.scale; out_l[unit] = 1.0f; }
        }
        return;
    }
    if (count <= 0) {   // empty memory (cross only): the context stays zero (src/graph.c:3242)
        if (tid < kHw) out_o[tid] = 0.0f;
        if (tid == 0) { out_m[unit] = 0.0f; out_l[unit] = 1.0f; }
        return;
    }

    // ---- scores of this unit
    const float4 qv = *reinterpret_cast<const float4 *>(s_proj + 4 * j);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int pi = g + kPosPerPass * i;
        float dot = 0.0f;
        dot = __builtin_fmaf(qv.x, kv[i].x, dot);
        dot = __builtin_fmaf(qv.y, kv[i].y, dot);
        dot = __builtin_fmaf(qv.z, kv[i].z, dot);
        dot = __builtin_fmaf(qv.w, kv[i].w, dot);
        dot = row16_sum(dot);
        if (j == 0) s_score[pi] = pi < count ? dot * a.scale : -3.0e38f;
    }
    __syncthreads();
    if (tid < 64) {   // kStepUnitRows scores, kStepUnitRows / 64 per lane
        constexpr int kPerLane = kStepUnitRows / 64;
        float sc[kPerLane], m = -3.0e38f;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            sc[i] = s_score[tid + 64 * i];
            m = fmaxf(m, sc[i]);
        }
        m = wave_max(m);
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const float e = tid + 64 * i < count ? expf(sc[i] - m) : 0.0f;
            s_score[tid + 64 * i] = e;
            l += e;
        }
        l = wave_sum(l);
        if (tid == 0) { s_ml[0] = m; s_ml[1] = l; }
    }
    __syncthreads();
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const float e = s_score[g + kPosPerPass * i];
        acc.x = __builtin_fmaf(e, vv[i].x, acc.x);
        acc.y = __builtin_fmaf(e, vv[i].y, acc.y);
        acc.z = __builtin_fmaf(e, vv[i].z, acc.z);
        acc.w = __builtin_fmaf(e, vv[i].w, acc.w);
    }
    *reinterpret_cast<float4 *>(s_red + (size_t)g * kHw + 4 * j) = acc;
    __syncthreads();
    if (tid < kHw) {
        float o = 0.0f;
#pragma unroll
        for (int gg = 0; gg < kPosPerPass; ++gg) o += s_red[(size_t)gg * kHw + tid];
        out_o[tid] = o;
        if (tid == 0) { out_m[unit] = s_ml[0]; out_l[unit] = s_ml[1]; }
    }
}

// Stand-alone fold of the partials into out[stream][heads * 64]: used instead of the consumer-side fold when
// the batch is large enough that every workgroup of the output projection folding every stream would cost more
// than one extra launch.  Same arithmetic (fold_partials), so the result does not depend on which path ran.
__global__ void __launch_bounds__(kThreads) k_step_fold(const float *partial, const float *partial_ml, const StepSlots *slots, int heads,
                                                        int max_units, int is_self, float *out) {
    const int stream = blockIdx.y;
    const int f4 = blockIdx.x * kThreads + threadIdx.x;
    if (f4 >= heads * (kHw / 4)) return;
    ActSource src;
    src.partial = partial; src.partial_ml = partial_ml; src.slots = slots; src.heads = heads; src.head_width = kHw;
    src.max_units = max_units; src.is_self = is_self; src.stream0 = 0;
    reinterpret_cast<float4 *>(out + (size_t)stream * heads * kHw)[f4] = fold_partials(src, stream, f4);
}

template <int QT>
int launch_t(State *st, const StepAttnArgs &a, char *error, size_t capacity) {
    const int chunks = a.width / Chunk<QT>::n;
    const int lg = lane_group_log2(chunks);
    const int items = a.heads * a.batch * a.max_units;
    const int per_xcd = (items + 7) / 8;
    const int grid = 8 * per_xcd;
    const size_t lds = (size_t)a.width * (kQuantised<QT> ? 1 : 4);
    if (a.width <= 1024) hipLaunchKernelGGL((k_step_attention<QT, 1>), dim3(grid), dim3(kThreads), lds, st->stream, a, lg, per_xcd);
    else hipLaunchKernelGGL((k_step_attention<QT, 3>), dim3(grid), dim3(kThreads), lds, st->stream, a, lg, per_xcd);
    return hip_check(hipGetLastError(), "step attention launch", error, capacity);
}

}  // namespace

bool step_attention_supported(int qtype, size_t width, size_t heads, size_t head_width) {
    if (head_width != (size_t)kHw || heads == 0 || heads * head_width > 4096) return false;
    if (!linear_fast_supported(qtype, head_width, width)) return false;
    const int epc = qtype == MYNAH_HIP_F32 ? 4 : qtype == MYNAH_HIP_F16 ? 8 : qtype == MYNAH_HIP_INT8 ? 16 : 32;
    const int chunks = (int)width / epc;
    const int group = 1 << lane_group_log2(chunks);
    return (chunks + group - 1) / group <= 4;   // one register group of four chunks per lane and pass
}

int launch_step_fold(State *st, const StepAttnArgs &a, float *out, char *error, size_t capacity) {
    const int f4 = a.heads * (kHw / 4);
    const dim3 grid((unsigned)((f4 + kThreads - 1) / kThreads), (unsigned)a.batch);
    hipLaunchKernelGGL(k_step_fold, grid, dim3(kThreads), 0, st->stream, a.partial, a.partial_ml, a.slots, a.heads, a.max_units, a.is_self, out);
    return hip_check(hipGetLastError(), "step fold launch", error, capacity);
}

int launch_step_attention(State *st, const StepAttnArgs &a, char *error, size_t capacity) {
    if (a.batch < 1 || a.batch > kMaxBatch || a.max_units < 1 || a.partial == nullptr || a.partial_ml == nullptr || a.slots == nullptr ||
        !step_attention_supported(a.qtype, (size_t)a.width, (size_t)a.heads, (size_t)a.head_width)) {
        set_error(error, capacity, "step attention: invalid or unsupported shape");
        return -1;
    }
    switch (a.qtype) {
        case MYNAH_HIP_F32: return launch_t<MYNAH_HIP_F32>(st, a, error, capacity);
        case MYNAH_HIP_F16: return launch_t<MYNAH_HIP_F16>(st, a, error, capacity);
        case MYNAH_HIP_INT8: return launch_t<MYNAH_HIP_INT8>(st, a, error, capacity);
        default: return launch_t<MYNAH_HIP_INT4>(st, a, error, capacity);
    }
}

}  // namespace mynah
