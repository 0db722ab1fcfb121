// Attention stage of the resident decode step, fused with the projection that feeds it.
//
// decoder_step_batch (src/graph.c:3161-3205, :3213-3247) runs LayerNorm -> Q(KV) projection -> per-head
// attention as separate passes.  On this GPU every pass boundary is a grid-wide dependency that costs
// several microseconds, more than the work between two of them, so here one workgroup does all of it
// for one (head, stream, unit):
//     LayerNorm(x) -> int8 activation quantisation -> this head's 64 rows of the Q projection
//     -> scores against one 128-row unit of the K cache -> unit softmax statistics -> weighted V rows
//     -> partial (max, sum, output[64]) to a workspace.
// Units of a stream: its cache chunks, plus -- for self-attention -- the step's new row, whose work is
// split over two workgroups with fixed indices so that each can request all of its weight rows before
// anything else has arrived: workgroup 0 computes this head's Q and K rows, appends K
// (src/graph.c:3180-3181) and contributes the new row's own score; workgroup 1 computes the V row,
// appends it and contributes it as that partial's output.  The next kernel (the output projection) folds
// the partials in its prologue, so no fence, atomic or second pass is needed here.  How a stream is cut
// into units depends on its own length only, and a unit's arithmetic on nothing but its own inputs, so a
// stream in a batch is bit-identical to the same stream alone.
//
// The LayerNorm/quantisation is recomputed per workgroup (3 KB of input), and the 64 x 768 weight slice
// of a head is read by every unit of that head.  Work items are ordered head-major and cut into eight
// contiguous ranges, one per XCD (workgroup i runs on XCD i % 8): a head's slice is fetched from HBM by
// at most two XCDs and served to the other units from their L2, and since every head carries the same
// work the XCDs stay balanced whatever the streams' lengths are.
//
// The mapping from workgroup to (head, stream, unit) is static, so the weight slice and x are requested
// before the slot table (lengths, cache pointers) has arrived; K and V rows follow as soon as it has.
#include "step_attention_core.h"

namespace mynah {
namespace {

// WFIX: model width known at compile time (0 = taken from the arguments): lane-group width, chunks per lane and passes
// per bank become constants and the per-chunk range checks fold away.  The decoder stack's width (768) gets such a build.
// SELF: 1 / 0 = self / cross attention known at compile time (the cross build has no new-row roles at all), -1 = from the arguments.
// PACKED: how a workgroup finds its work.  0: from its index alone (one or two streams: nearly every unit of the grid
// exists, and the weight rows can be requested before the slot table has arrived).  1: from its index and the slot
// table (more streams, ragged lengths: most of a grid sized for the longest possible stream would belong to units that
// short streams do not have; here the workgroups are numbered over the units that exist, so those with nothing to do
// are the last ones of the grid and leave after one read instead of holding places among the working ones).
template <int QT, int NVT, int PF, int WFIX, int SELF, int PACKED>
__global__ void __launch_bounds__(kThreads) k_step_attention(const StepAttnArgs a_arg, const int lg_arg, const int per_xcd_arg) {
    extern __shared__ __align__(16) unsigned char smem[];   // staged activations: width bytes (int8/int4) or floats
    __shared__ __align__(16) float s_proj[3 * kHw];         // q | k | v of this head
    // CP: consecutive cache chunks of a stream per chunk workgroup; the code below is written for any CP.  With CP chunks one
    // LayerNorm and one Q projection serve them all, their rows are requested at once, and each chunk still becomes a
    // partial of its own, computed as a workgroup with that chunk alone would compute it, so results do not depend on CP.
    // Measured with eight ragged streams, CP = 2 against 1: 42 % fewer workgroups and one round instead of two, yet the
    // self-attention stage stays where it was (22.2 -> 21.8 us) and the cross-attention stage, whose memories are one or
    // two chunks long, loses (9.4 -> 10.3 us): a workgroup's requests double as their number halves.
    constexpr int CP = 1;
    __shared__ __align__(16) float s_red[CP][4 * kHw];      // per-wavefront weighted V sums, per chunk
    __shared__ float s_wave_ml[CP][8];                      // per-wavefront max | sum, per chunk
    __shared__ float s_sx[1];
    __shared__ float s_scratch[kPrologueScratch];

    constexpr int kEpc = Chunk<QT>::n;
    const int lg = WFIX != 0 ? lane_group_log2(WFIX / kEpc) : lg_arg;
    StepAttnArgs a = a_arg;
    if constexpr (WFIX != 0) a.width = WFIX;
    const bool is_self = SELF >= 0 ? SELF == 1 : a.is_self != 0;
    const int tid = threadIdx.x;
    const StepSlots *slots = a.slots;

    // ---- static work decode: item = (head * batch + stream) * wg_units + unit, XCD x owns items [x*per_xcd, (x+1)*per_xcd).
    // Self-attention: unit 0 = Q+K of the new row, unit 1 = V of the new row, unit 2 + c = cache chunk c.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    int unit, b, head;
    if constexpr (PACKED == 0) {
        const int wg_units = a.max_units + (is_self ? 1 : 0);
        const int items = a.heads * a.batch * wg_units;
        const int item = xcd * per_xcd_arg + slot;
        if (slot >= per_xcd_arg || item >= items) return;
        unit = item % wg_units;
        const int hb = item / wg_units;
        b = hb % a.batch;
        head = hb / a.batch;
    } else {
        // per head: [Q+K and V of every stream's new row (self only)] [groups of CP cache chunks that exist, stream by stream]
        int chunk_items = 0;
        for (int s = 0; s < a.batch; ++s) {
            const int len = is_self ? slots->length[s] : slots->memory_length[s];
            const int live = (len + kStepUnitRows - 1) / kStepUnitRows;
            chunk_items += ((is_self ? live : max(live, 1)) + CP - 1) / CP;
        }
        const int row_items = is_self ? 2 * a.batch : 0;
        const int per_head = row_items + chunk_items;
        const int items = a.heads * per_head;
        const int per_xcd = (items + 7) / 8;
        const int item = xcd * per_xcd + slot;
        if (slot >= per_xcd || item >= items) return;
        head = item / per_head;
        int r = item - head * per_head;
        if (r < row_items) {
            b = r >> 1;
            unit = r & 1;
        } else {
            r -= row_items;
            b = 0;
            unit = 0;
            int before = 0;
            for (int s = 0; s < a.batch; ++s) {
                const int len = is_self ? slots->length[s] : slots->memory_length[s];
                const int live = (len + kStepUnitRows - 1) / kStepUnitRows;
                const int n = ((is_self ? live : max(live, 1)) + CP - 1) / CP;
                if (r >= before && r < before + n) { b = s; unit = r - before + (is_self ? 2 : 0); }
                before += n;
            }
        }
    }
    const bool role_qk = is_self && unit == 0;
    const bool role_v = is_self && unit == 1;
    const int chunk = CP * (is_self ? unit - 2 : unit);   // first cache chunk of this workgroup (chunk roles only)
    const int pidx = is_self ? chunk + 1 : chunk;         // partial slot of that chunk (slot 0 of self-attention = the new row)

    const int chunks = a.width / kEpc;

    // ---- slot table: read before any vector request.  The stream is the same for the whole workgroup and nothing has
    // been stored yet, so these are scalar loads, whose answers do not queue behind the vector loads below (vector loads
    // return in order: a table word requested after the weight rows could only be looked at once all of them had come).
    const int length = is_self ? slots->length[b] : slots->memory_length[b];   // cache rows that exist before this step
    float *const k_base = is_self ? slots->self_k[b] : const_cast<float *>(slots->cross_k[b]);
    float *const v_base = is_self ? slots->self_v[b] : const_cast<float *>(slots->cross_v[b]);

    // With many streams most of the grid belongs to units that short streams do not have: there the slot table is
    // looked at first, so that such a workgroup leaves without having requested anything.  With one or two streams
    // nearly every unit is live and the weight rows are requested before the table has arrived (latency matters more).
    if (PACKED == 0 && a.batch > kConsumerFoldMaxBatch && !(is_self && unit < 2)) {
        const int len = is_self ? slots->length[b] : slots->memory_length[b];
        const int live = (len + kStepUnitRows - 1) / kStepUnitRows;
        if (chunk >= (is_self ? live : max(live, 1))) return;
    }

    // ---- requests that need neither the slot table nor each other.  Latency layout: the activation row and its
    // LayerNorm vectors go first -- the prologue's arithmetic waits for these only and runs while the weight rows,
    // requested right after, are still on their way.  Throughput layout: after the cache rows (fewer live registers).
    PrologueParams pro;
    pro.k = a.width; pro.batch = 1; pro.ln_gain = a.ln_gain; pro.ln_bias = a.ln_bias; pro.arith = a.arith;
    pro.probe_qx = nullptr; pro.probe_sx = nullptr;
    float4 xr[1][NVT], gv[NVT], bv[NVT];
    ActSource act;
    act.rows[0] = a.x + (size_t)b * a.width;
    act.partial = nullptr;
    if constexpr (PF == kPrefetchLatency) load_activations<1, NVT>(pro, act, whole_workgroup(), xr, gv, bv);
    PassRegs pre[PF];
    if (role_qk) load_bank<QT, PF>(pre, a, 0, 0, 2 * kHw, head, lg, chunks);
    else if (role_v) load_bank<QT, PF>(pre, a, 0, 2 * kHw, kHw, head, lg, chunks);
    else load_bank<QT, PF>(pre, a, 0, 0, kHw, head, lg, chunks);
    if constexpr (PF == kPrefetchLatency) requests_issued();

    // ---- is this unit live, and where are its cache rows?
    const int nchunks = (length + kStepUnitRows - 1) / kStepUnitRows;
    const bool new_row = role_qk || role_v;
    if (!new_row && chunk >= (is_self ? nchunks : max(nchunks, 1))) return;
    const int stride = a.heads * kHw;   // floats between cache rows
    float *kc, *vc;
    if (is_self) {
        kc = k_base + a.layer * a.capacity * (size_t)stride;
        vc = v_base + a.layer * a.capacity * (size_t)stride;
    } else {
        kc = k_base + a.layer * (size_t)length * stride;
        vc = v_base + a.layer * (size_t)length * stride;
    }
    const int j = tid & (kPosLanes - 1);
    const int g = tid / kPosLanes;
    const size_t col = (size_t)head * kHw + 4 * j;
    const int p0 = chunk * kStepUnitRows;
    int count[CP];
#pragma unroll
    for (int cc = 0; cc < CP; ++cc) count[cc] = new_row ? 0 : max(0, min(kStepUnitRows, length - p0 - cc * kStepUnitRows));
    // A chunk role keeps its cache rows here.  The Q+K role has no cache rows and parks its second bank of weight
    // passes in the same registers (as raw bits), so that no role needs more registers than the largest one.
    static_assert(2 * kRowsPerThread >= 4 * PF, "the second weight bank must fit the cache-row registers");
    float4 kv[CP][kRowsPerThread], vv[CP][kRowsPerThread];
    float sc2[4 * PF];   // int4 only: group scales of the second bank
    float ws2[PF];       // int8 only: row scales of the second bank
    if (role_qk) {
        PassRegs bank2[PF];
#pragma unroll
        for (int p = 0; p < PF; ++p) {
#pragma unroll
            for (int u = 0; u < 4; ++u) { bank2[p].wv[u] = make_uint4(0, 0, 0, 0); bank2[p].sc[u] = 0.0f; }
            bank2[p].ws = 1.0f;
        }
        load_bank<QT, PF>(bank2, a, PF, 0, 2 * kHw, head, lg, chunks);
#pragma unroll
        for (int p = 0; p < PF; ++p) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = 4 * p + u;
                if (idx < kRowsPerThread) kv[0][idx] = __builtin_bit_cast(float4, bank2[p].wv[u]);
                else vv[0][idx - kRowsPerThread] = __builtin_bit_cast(float4, bank2[p].wv[u]);
                sc2[idx] = bank2[p].sc[u];
            }
            ws2[p] = bank2[p].ws;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4 * PF; ++i) sc2[i] = 0.0f;
#pragma unroll
        for (int i = 0; i < PF; ++i) ws2[i] = 1.0f;
        // Every request is issued, whatever the lane's row: a row past the chunk's end repeats the chunk's last row, and a
        // workgroup without cache rows (the new row's V role; an empty memory, whose pointers may be null) reads the
        // activation buffer, which always holds heads x 64 floats.  Under a per-lane condition each request would sit in
        // a branch of its own with a wait behind it, and the next one would leave only after it had come back.
        const bool have_rows = count[0] > 0;
        const float *const k_from = have_rows ? kc : a.x;
        const float *const v_from = have_rows ? vc : a.x;
#pragma unroll
        for (int cc = 0; cc < CP; ++cc) {
            const int rows = count[cc];
#pragma unroll
            for (int i = 0; i < kRowsPerThread; ++i) {
                const int pi = g + kPosPerPass * i;
                const int row = !have_rows ? 0 : rows > 0 ? p0 + cc * kStepUnitRows + min(pi, rows - 1) : p0;
                const size_t at = (size_t)row * stride + col;
                kv[cc][i] = load_global4(k_from + at);
                vv[cc][i] = load_global4(v_from + at);
            }
        }
        // The repeated rows need no clearing: further down a row past the chunk's end gets the score -3e38 and the weight
        // exactly 0, and fma(0, v, acc) is acc for the finite v of a real cache row -- the bits a zero row would give.
    }

    // ---- LayerNorm + activation quantisation of x[b], staged in LDS (the cache rows requested above stay in flight)
    if constexpr (PF != kPrefetchLatency) load_activations<1, NVT>(pro, act, whole_workgroup(), xr, gv, bv);
    finish_activations<QT, 1, NVT>(pro, whole_workgroup(), xr, gv, bv, smem, s_sx, s_scratch);

    const size_t sh = (size_t)b * a.heads + head;
    float *out_m = a.partial_ml + sh * 2 * a.max_units;
    float *out_l = out_m + a.max_units;

    if (role_qk) {
        // this head's q and k of the new row; append k; the new row's own score opens partial 0
        {
            PassRegs bank2[PF];
#pragma unroll
            for (int p = 0; p < PF; ++p) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int idx = 4 * p + u;
                    bank2[p].wv[u] = __builtin_bit_cast(uint4, idx < kRowsPerThread ? kv[0][idx] : vv[0][idx - kRowsPerThread]);
                    bank2[p].sc[u] = sc2[idx];
                }
                bank2[p].ws = ws2[p];
            }
            project_bank<QT, PF>(a, pre, 0, 0, 2 * kHw, head, lg, chunks, smem, s_sx[0], s_proj);
            project_bank<QT, PF>(a, bank2, PF, 0, 2 * kHw, head, lg, chunks, smem, s_sx[0], s_proj);
            const int rpp = 64 >> lg;
            const int passes = (2 * kHw + 4 * rpp - 1) / (4 * rpp);
            for (int pb = 2 * PF; pb < passes; pb += PF) {   // passes beyond the two banks (wide f32 / f16 rows, or the two-pass banks)
                load_bank<QT, PF>(pre, a, pb, 0, 2 * kHw, head, lg, chunks);
                project_bank<QT, PF>(a, pre, pb, 0, 2 * kHw, head, lg, chunks, smem, s_sx[0], s_proj);
            }
        }
        __syncthreads();
        if (tid < 64) {
            const float kval = s_proj[kHw + tid];
            store_global(kc + (size_t)length * stride + (size_t)head * kHw + tid, kval);
            float d = s_proj[tid] * kval;
            d = wave_sum(d);
            if (tid == 0) { out_m[0] = d * a.scale; out_l[0] = 1.0f; }   // exp(score - max) = 1
        }
        return;
    }
    if (role_v) {
        // this head's v of the new row: appended, and the output of partial 0
        project_rows<QT, PF>(a, pre, PF, 2 * kHw, kHw, head, lg, chunks, smem, s_sx[0], s_proj);
        __syncthreads();
        if (tid < kHw) {
            const float vval = s_proj[2 * kHw + tid];
            store_global(vc + (size_t)length * stride + (size_t)head * kHw + tid, vval);
            a.partial[sh * a.max_units * kHw + tid] = vval;
        }
        return;
    }

    // ---- cache chunk: this head's q, then the chunk's scores
    project_rows<QT, PF>(a, pre, PF, 0, kHw, head, lg, chunks, smem, s_sx[0], s_proj);
    __syncthreads();
    float *out_o = a.partial + (sh * a.max_units + pidx) * kHw;   // the first chunk's partial; the second follows it
    if (count[0] <= 0) {   // empty memory (cross only): the context stays zero (src/graph.c:3242)
        if (tid < kHw) out_o[tid] = 0.0f;
        if (tid == 0) { out_m[pidx] = 0.0f; out_l[pidx] = 1.0f; }
        return;
    }

    // ---- scores, softmax statistics and weighted V rows, one wavefront at a time: a wavefront owns 32 rows of a chunk
    // (its four 16-lane row groups x 8 passes) and nothing leaves it until its own (max, sum, out[64]) is complete;
    // the four results of a chunk meet once in LDS.
    const float4 qv = *reinterpret_cast<const float4 *>(s_proj + 4 * j);
#pragma unroll
    for (int cc = 0; cc < CP; ++cc) {
        if (count[cc] <= 0) continue;   // the stream's last group may hold one chunk only (same for the whole workgroup)
        attend_chunk(qv, kv[cc], vv[cc], count[cc], a.scale, s_red[cc], s_wave_ml[cc]);
    }
    __syncthreads();
    if (tid < CP * kPosLanes) {   // merge a chunk's four wavefronts in order 0..3: lanes 0-15 the first chunk, 16-31 the second
        const int cc = tid / kPosLanes, t = tid - cc * kPosLanes;
        if (count[cc] > 0) {
            float4 o;
            float M, L;
            merge_chunk(t, s_red[cc], s_wave_ml[cc], o, M, L);
            *reinterpret_cast<float4 *>(out_o + (size_t)cc * kHw + 4 * t) = o;
            if (t == 0) { out_m[pidx + cc] = M; out_l[pidx + cc] = L; }
        }
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
    const int items = a.heads * a.batch * (a.max_units + (a.is_self ? 1 : 0));   // self: the new row takes two workgroups
    const int per_xcd = (items + 7) / 8;
    const int grid = 8 * per_xcd;
    const size_t lds = (size_t)a.width * (kQuantised<QT> ? 1 : 4);
    const bool latency = a.batch <= kConsumerFoldMaxBatch;
    const dim3 g(grid), t(kThreads);
    if (a.width == 768) {
        // the fixed-shape build needs few enough registers (154 for int8) to hold three workgroups per CU with four-pass banks
        if (a.is_self && latency) hipLaunchKernelGGL((k_step_attention<QT, 1, kPrefetchLatency, 768, 1, 0>), g, t, lds, st->stream, a, lg, per_xcd);
        else if (a.is_self) hipLaunchKernelGGL((k_step_attention<QT, 1, kPrefetchLatency, 768, 1, 1>), g, t, lds, st->stream, a, lg, per_xcd);
        else if (latency) hipLaunchKernelGGL((k_step_attention<QT, 1, kPrefetchLatency, 768, 0, 0>), g, t, lds, st->stream, a, lg, per_xcd);
        else hipLaunchKernelGGL((k_step_attention<QT, 1, kPrefetchLatency, 768, 0, 1>), g, t, lds, st->stream, a, lg, per_xcd);
    } else if (a.width <= 1024) {
        if (latency) hipLaunchKernelGGL((k_step_attention<QT, 1, kPrefetchLatency, 0, -1, 0>), g, t, lds, st->stream, a, lg, per_xcd);
        else hipLaunchKernelGGL((k_step_attention<QT, 1, kPrefetchThroughput, 0, -1, 1>), g, t, lds, st->stream, a, lg, per_xcd);
    } else {
        if (latency) hipLaunchKernelGGL((k_step_attention<QT, 3, kPrefetchLatency, 0, -1, 0>), g, t, lds, st->stream, a, lg, per_xcd);
        else hipLaunchKernelGGL((k_step_attention<QT, 3, kPrefetchThroughput, 0, -1, 1>), g, t, lds, st->stream, a, lg, per_xcd);
    }
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
