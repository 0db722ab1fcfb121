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
#include "step_items.h"
#include "tagged_exchange.h"

namespace mynah {
namespace {

// max | sum of a record, and its two unused words: a reader takes a record as 68 tagged words
__device__ __forceinline__ void put_ml(u64 *rec, unsigned tag, float m, float l) {
    put(rec + kHw, tag, m);
    put(rec + kHw + 1, tag, l);
    put(rec + kHw + 2, tag, 0.0f);
    put(rec + kHw + 3, tag, 0.0f);
}

// The fold of one (stream, head)'s partial records (fold_partials' arithmetic, units in order) from LDS, by 16 threads.
// weight[u] = expf(max[u] - M), M the largest max: computed beforehand, one unit per thread, instead of one after the
// other by each of the sixteen.
__device__ __forceinline__ float fold_max(const float *rec, const int units) {
    float M = -3.0e38f;
    for (int u = 0; u < units; ++u) M = fmaxf(M, rec[u * kStepRecord + kHw]);
    return M;
}
__device__ __forceinline__ float4 fold_records(const float *rec, const float *weight, const int units, const int t) {
    float L = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int u = 0; u < units; ++u) {
        const float *p = rec + u * kStepRecord;
        const float wgt = weight[u];
        const float4 ou = *reinterpret_cast<const float4 *>(p + 4 * t);
        L = __builtin_fmaf(p[kHw + 1], wgt, L);
        acc.x = __builtin_fmaf(ou.x, wgt, acc.x);
        acc.y = __builtin_fmaf(ou.y, wgt, acc.y);
        acc.z = __builtin_fmaf(ou.z, wgt, acc.z);
        acc.w = __builtin_fmaf(ou.w, wgt, acc.w);
    }
    acc.x /= L; acc.y /= L; acc.z /= L; acc.w /= L;
    return acc;
}


// WFIX: model width known at compile time (0 = taken from the arguments): lane-group width, chunks per lane and passes
// per bank become constants and the per-chunk range checks fold away.  The decoder stack's width (768) gets such a build.
// SELF: 1 / 0 = self / cross attention known at compile time (the cross build has no new-row roles at all), -1 = from the arguments.
// PACKED: how a workgroup finds its work.  0: from its index alone (one or two streams: nearly every unit of the grid
// exists, and the weight rows can be requested before the slot table has arrived).  1: from its index and the slot
// table (more streams, ragged lengths: most of a grid sized for the longest possible stream would belong to units that
// short streams do not have; here the workgroups are numbered over the units that exist, so those with nothing to do
// are the last ones of the grid and leave after one read instead of holding places among the working ones).
template <int QT, int NVT, int PF, int WFIX, int SELF, int PACKED>
__global__ void __launch_bounds__(kThreads)
k_step_attention(const StepSlots *const slots_arg, const float *const x_arg, const void *const w_arg, const float *const scales_arg,
                 const float *const ln_gain_arg, const float *const ln_bias_arg, const StepItem *const items_arg, const int per_xcd_arg,
                 const int lg_arg, const StepAttnArgs a_arg) {
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
    // The seven pointers and two counts in front repeat fields of a_arg: the first sixteen dwords of the kernel arguments are
    // in registers when a wavefront starts (the build asks for that); the structure behind them is fetched from memory.
    StepAttnArgs a = a_arg;
    a.slots = slots_arg; a.x = x_arg; a.w = w_arg; a.scales = scales_arg; a.ln_gain = ln_gain_arg; a.ln_bias = ln_bias_arg; a.items = items_arg;
    if constexpr (WFIX != 0) a.width = WFIX;
    // Only fourteen dwords of arguments are in registers at wavefront start (the seven pointers): per_xcd_arg, lg_arg and every
    // field of a_arg come out of memory, and the first request for the activation row cannot be formed before the stream
    // index is known.  The builds that find their work from the workgroup index have no use for the work table's pointer, so
    // there the launch passes in its place the few small numbers that decide a workgroup's role (pack_grid_shape): the
    // activation row, its LayerNorm vectors and the head's weight rows are then requested without waiting for anything.
    // (the argument structure ends 0xf8 bytes into the kernel arguments: three lines behind the first)
    static_assert(64 + sizeof(StepAttnArgs) > 0xc0 + 4, "the warmed lines lie inside the kernel arguments");
    // (one or two streams only: with more, 1,800 workgroups asking for three more lines each made both attention stages 0.2 us slower)
    WarmArguments warm{0u, 0u, 0u, 0u};
    if constexpr (PACKED == 0) warm = warm_kernel_arguments<3>();
    int per_xcd = per_xcd_arg;
    if constexpr (PACKED == 0) {
        const unsigned long long shape = reinterpret_cast<unsigned long long>(items_arg);
        per_xcd = (int)(shape & 0xffffu);
        a.max_units = (int)((shape >> 16) & 0xffffu);
        a.batch = (int)((shape >> 32) & 0xffu);
        a.heads = (int)((shape >> 40) & 0xffu);
        a.items = nullptr;
    }
    const bool is_self = SELF >= 0 ? SELF == 1 : a.is_self != 0;
    const int tid = threadIdx.x;
    const StepSlots *slots = a.slots;

    // ---- static work decode: item = (head * batch + stream) * wg_units + unit, XCD x owns items [x*per_xcd, (x+1)*per_xcd).
    // Self-attention: unit 0 = Q+K of the new row, unit 1 = V of the new row, unit 2 + c = cache chunk c.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    int unit, b, head;
    int item_length = 0;
    unsigned item_epoch = 0;
    int item_group = 1;   // consecutive cache chunks this workgroup takes, one after the other
    float *item_k = nullptr, *item_v = nullptr;
    if constexpr (PACKED == 0) {
        const int wg_units = a.max_units + (is_self ? 1 : 0);
        const int items = a.heads * a.batch * wg_units;
        const int item = xcd * per_xcd + slot;
        if (slot >= per_xcd || item >= items) return;
        unit = item % wg_units;
        const int hb = item / wg_units;
        b = hb % a.batch;
        head = hb / a.batch;
    } else {
        // one table entry, written at the step's start for this very workgroup index (write_step_item): one read instead of
        // the lengths, two loops over the streams and then the stream's cache pointers, each a round trip of its own
        typedef int int8v __attribute__((ext_vector_type(8)));
        static_assert(sizeof(StepItem) == sizeof(int8v), "an entry is read as one 32-byte scalar load");
        const int8v raw = *reinterpret_cast<const int8v *>(a.items + blockIdx.x);   // all of it before the first branch
        const int code = raw[5];
        if (code < 0) return;
        head = code & 0xff;
        b = (code >> 8) & 0xff;
        unit = code >> 16;
        item_length = raw[4];
        item_epoch = (unsigned)raw[6];
        item_group = raw[7];
        item_k = reinterpret_cast<float *>(((unsigned long long)(unsigned)raw[1] << 32) | (unsigned)raw[0]);
        item_v = reinterpret_cast<float *>(((unsigned long long)(unsigned)raw[3] << 32) | (unsigned)raw[2]);
    }
    // ---- many streams: the fold of one (stream, head), by a workgroup numbered behind every workgroup that writes one of
    // its records -- those are running or done when this one starts.  The records arrive as tagged words (tagged_exchange.h),
    // tag = step counter | layer; the wait is bounded.  The next kernel reads the folded rows as plain memory.
    if constexpr (PACKED == 1) {
        if (unit == kFoldUnit) {
            const int live = (item_length + kStepUnitRows - 1) / kStepUnitRows;
            const int units = is_self ? live + 1 : max(live, 1);
            const size_t sh = (size_t)b * a.heads + head;
            float *s_fold = reinterpret_cast<float *>(smem);
            Waiter wt{a.spin_limit, a.abort_word, false};
            float *s_weight = s_fold + (size_t)a.max_units * kStepRecord;
            // (Measured and not kept: continuous requests for every word -- the polling took bandwidth from the workgroups
            // that read the caches, batch-8 step 650 -> 666 us; one slow poll per record and then the fetch -- a second round
            // trip behind the last record, 655 -> 672 us.)
            const u64 *records = a.records + sh * a.max_units * kStepRecord;
            const unsigned fold_tag = (item_epoch << 8) | (unsigned)(a.layer + 1);
            fetch_tagged<8, true>(records, s_fold, units * kStepRecord, fold_tag, wt);
            if (__syncthreads_or(wt.dead ? 1 : 0)) {   // gave up: say so and leave; the host reports it at its next synchronisation
                if (tid == 0) __hip_atomic_store(a.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                return;
            }
            const float M = fold_max(s_fold, units);
            for (int u = tid; u < units; u += kThreads) s_weight[u] = expf(s_fold[u * kStepRecord + kHw] - M);
            __syncthreads();
            if (tid < kPosLanes) *reinterpret_cast<float4 *>(a.fold_out + sh * kHw + 4 * tid) = fold_records(s_fold, s_weight, units, tid);
            return;
        }
    }
    const bool role_qk = is_self && unit == 0;
    const bool role_v = is_self && unit == 1;
    const int chunk = (PACKED == 1 ? item_group : CP) * (is_self ? unit - 2 : unit);   // first cache chunk of this workgroup (chunk roles only)
    const int pidx = is_self ? chunk + 1 : chunk;         // partial slot of that chunk (slot 0 of self-attention = the new row)

    const int chunks = a.width / kEpc;

    // ---- slot table: read before any vector request.  The stream is the same for the whole workgroup and nothing has
    // been stored yet, so these are scalar loads, whose answers do not queue behind the vector loads below (vector loads
    // return in order: a table word requested after the weight rows could only be looked at once all of them had come).
    // (asked for as scalar loads outright -- scalar_load_int, device_common.h -- and first looked at behind the row requests)
    int length = item_length;   // cache rows that exist before this step
    unsigned long long k_bits = reinterpret_cast<unsigned long long>(item_k), v_bits = reinterpret_cast<unsigned long long>(item_v);
    if constexpr (PACKED == 0) {
        const int bu = __builtin_amdgcn_readfirstlane(b);
        length = scalar_load_int(is_self ? &slots->length[bu] : &slots->memory_length[bu]);
        k_bits = scalar_load_u64(is_self ? static_cast<const void *>(&slots->self_k[bu]) : static_cast<const void *>(&slots->cross_k[bu]));
        v_bits = scalar_load_u64(is_self ? static_cast<const void *>(&slots->self_v[bu]) : static_cast<const void *>(&slots->cross_v[bu]));
    }

    // With many streams most of the grid belongs to units that short streams do not have: there the slot table is
    // looked at first, so that such a workgroup leaves without having requested anything.  With one or two streams
    // nearly every unit is live and the weight rows are requested before the table has arrived (latency matters more).
    if (PACKED == 0 && a.batch > kConsumerFoldMaxBatch && !(is_self && unit < 2)) {
        scalar_words_arrived(length, k_bits, v_bits);   // (only on this path: with one or two streams the table is first looked at behind the requests)
        const int live = (length + kStepUnitRows - 1) / kStepUnitRows;
        if (chunk >= (is_self ? live : max(live, 1))) return;
    }

    // ---- requests that need neither the slot table nor each other.  Latency layout: the activation row and its
    // LayerNorm vectors go first -- the prologue's arithmetic waits for these only and runs while the weight rows,
    // requested right after, are still on their way.  Throughput layout: after the cache rows (fewer live registers).
    PrologueParams pro;
    pro.k = a.width; pro.batch = 1; pro.ln_gain = a.ln_gain; pro.ln_bias = a.ln_bias; pro.arith = a.arith;
    // (the probes name stream 0: finish_activations writes them from workgroup 0, which always belongs to it)
    pro.probe_qx = PACKED == 0 ? a.probe_qx : nullptr; pro.probe_sx = PACKED == 0 ? a.probe_sx : nullptr;
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
    if constexpr (PACKED == 0) scalar_words_arrived(length, k_bits, v_bits);
    float *const k_base = reinterpret_cast<float *>(k_bits), *const v_base = reinterpret_cast<float *>(v_bits);
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
    // ---- many streams, cache chunks: the whole of this role here, ahead of the new row's roles.  Kept apart from the code
    // below so that nothing of those roles (their second weight bank, parked in registers) is alive while this one runs:
    // the chunk loop then fits the registers that one chunk needs.
    if constexpr (PACKED == 1) {
        if (!new_row) {
            static_assert(CP == 1, "the chunk loop keeps one chunk's rows in registers");
            const bool have_rows = count[0] > 0;   // an empty memory has none (its pointers may be null): read the activation buffer
            const float *const k_from = have_rows ? kc : a.x;
            const float *const v_from = have_rows ? vc : a.x;
            float4 kv[kRowsPerThread], vv[kRowsPerThread];
#pragma unroll
            for (int i = 0; i < kRowsPerThread; ++i) {
                // every request is issued, whatever the lane's row: a row past the chunk's end repeats the chunk's last row
                const int row = have_rows ? p0 + min(g + kPosPerPass * i, count[0] - 1) : 0;
                const size_t at = (size_t)row * stride + col;
                kv[i] = load_global4(k_from + at);
                vv[i] = load_global4(v_from + at);
            }
            if constexpr (PF != kPrefetchLatency) load_activations<1, NVT>(pro, act, whole_workgroup(), xr, gv, bv);
            finish_activations<QT, 1, NVT>(pro, whole_workgroup(), xr, gv, bv, smem, s_sx, s_scratch);
            const size_t sh = (size_t)b * a.heads + head;
            u64 *const rec0 = a.records + sh * a.max_units * kStepRecord;   // the partials leave as tagged records (see the fold role)
            const unsigned tag = (item_epoch << 8) | (unsigned)(a.layer + 1);
            project_rows<QT, PF>(a, pre, PF, 0, kHw, head, lg, chunks, smem, s_sx[0], s_proj);
            __syncthreads();
            if (!have_rows) {   // empty memory (cross only): the context stays zero (src/graph.c:3242)
                if (tid < kHw) put(rec0 + (size_t)pidx * kStepRecord + tid, tag, 0.0f);
                if (tid == 0) put_ml(rec0 + (size_t)pidx * kStepRecord, tag, 0.0f, 1.0f);
                return;
            }
            const float4 qv = *reinterpret_cast<const float4 *>(s_proj + 4 * j);
            const auto finish_chunk = [&](const int cc) {   // behind a barrier after attend_chunk: merge the four wavefronts in order 0..3
                if (tid < kPosLanes) {
                    float4 o;
                    float M, L;
                    merge_chunk(tid, s_red[0], s_wave_ml[0], o, M, L);
                    u64 *rec = rec0 + (size_t)(pidx + cc) * kStepRecord;
                    put(rec + 4 * tid, tag, o.x); put(rec + 4 * tid + 1, tag, o.y); put(rec + 4 * tid + 2, tag, o.z); put(rec + 4 * tid + 3, tag, o.w);
                    if (tid == 0) put_ml(rec, tag, M, L);
                }
            };
            attend_chunk(qv, kv, vv, count[0], a.scale, s_red[0], s_wave_ml[0]);
            __syncthreads();
            finish_chunk(0);
            // The workgroup goes on to the next chunks of its group, one at a time in the same registers.  A chunk's partial
            // is what a workgroup with that chunk alone computes, so the bits do not depend on how chunks are grouped; the
            // group size only sets how many workgroups the launch has (few enough to be resident at once, see make_item).
            // The stream's last group may be short; the count is the same for the whole workgroup.
            const int trips = __builtin_amdgcn_readfirstlane(min(item_group, nchunks - chunk));
            const int first_row = __builtin_amdgcn_readfirstlane(p0);
            const int total_rows = __builtin_amdgcn_readfirstlane(length);
#pragma nounroll
            for (int cc = 1; cc < trips; ++cc) {
                const int row0 = first_row + cc * kStepUnitRows;
                const int rows = min(kStepUnitRows, total_rows - row0);
#pragma unroll
                for (int i = 0; i < kRowsPerThread; ++i) {
                    const size_t at = (size_t)(row0 + min(g + kPosPerPass * i, rows - 1)) * stride + col;
                    kv[i] = load_global4(kc + at);
                    vv[i] = load_global4(vc + at);
                }
                __syncthreads();            // the merge of the chunk before has read what this one writes
                attend_chunk(qv, kv, vv, rows, a.scale, s_red[0], s_wave_ml[0]);
                __syncthreads();
                finish_chunk(cc);
            }
            return;
        }
    }

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
    if constexpr (PACKED == 0) release_warm(warm);

    const size_t sh = (size_t)b * a.heads + head;
    float *out_m = a.partial_ml + sh * 2 * a.max_units;
    float *out_l = out_m + a.max_units;
    // many streams: the partials leave as tagged records that the fold workgroups of this same launch wait for
    constexpr bool tagged = PACKED == 1;
    u64 *const rec0 = a.records + sh * a.max_units * kStepRecord;
    const unsigned tag = (item_epoch << 8) | (unsigned)(a.layer + 1);

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
            if (tid == 0) {   // exp(score - max) = 1
                if (tagged) put_ml(rec0, tag, d * a.scale, 1.0f);
                else { out_m[0] = d * a.scale; out_l[0] = 1.0f; }
            }
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
            if (tagged) put(rec0 + tid, tag, vval);
            else a.partial[sh * a.max_units * kHw + tid] = vval;
        }
        return;
    }

    if constexpr (PACKED == 1) return;   // the chunk role of the many-stream build is complete further up

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

using StepAttnKernel = void (*)(const StepSlots *, const float *, const void *, const float *, const float *, const float *, const StepItem *, const int,
                                const int, const StepAttnArgs);

// The build that runs a shape: fixed-width builds for the decoder stack's width; `latency`: the build for one or two
// streams (work found from the workgroup index; it also serves more streams when the launch cannot fold its own partials),
// else the many-stream build (work table, partials as tagged records, fold inside the launch).
template <int QT>
StepAttnKernel kernel_for(int width, bool is_self, bool latency) {
    if (width == 768) {
        // the fixed-shape build needs few enough registers (154 for int8) to hold three workgroups per CU with four-pass banks
        if (is_self && latency) return k_step_attention<QT, 1, kPrefetchLatency, 768, 1, 0>;
        if (is_self) return k_step_attention<QT, 1, kPrefetchLatency, 768, 1, 1>;
        if (latency) return k_step_attention<QT, 1, kPrefetchLatency, 768, 0, 0>;
        return k_step_attention<QT, 1, kPrefetchLatency, 768, 0, 1>;
    }
    if (width <= 1024) {
        if (latency) return k_step_attention<QT, 1, kPrefetchLatency, 0, -1, 0>;
        return k_step_attention<QT, 1, kPrefetchThroughput, 0, -1, 1>;
    }
    if (latency) return k_step_attention<QT, 3, kPrefetchLatency, 0, -1, 0>;
    return k_step_attention<QT, 3, kPrefetchThroughput, 0, -1, 1>;
}

template <int QT>
size_t lds_for(int width, int max_units, bool with_fold) {
    size_t lds = (size_t)width * (kQuantised<QT> ? 1 : 4);
    if (with_fold) {   // the fold workgroups stage a (stream, head)'s records there
        const size_t fold_bytes = step_fold_lds_bytes(max_units);
        lds = lds > fold_bytes ? lds : fold_bytes;
    }
    return lds;
}

template <int QT>
int launch_t(State *st, const StepAttnArgs &a, char *error, size_t capacity) {
    const int chunks = a.width / Chunk<QT>::n;
    const int lg = lane_group_log2(chunks);
    const bool packed_grid = a.records != nullptr;
    const int grid = step_attention_grid(a.heads, a.batch, a.max_units, a.is_self, packed_grid);
    const int per_xcd = grid / 8;
    const bool packed = a.records != nullptr;
    const size_t lds = lds_for<QT>(a.width, a.max_units, packed);
    // the builds without a work table take the grid's shape in the table pointer's place (see the kernel): 16 bits each for the
    // workgroups per XCD and the units per stream, 8 each for streams and heads
    const StepItem *items_or_shape = a.items;
    if (!packed) {
        if (per_xcd > 0xffff || a.max_units > 0xffff || a.batch > 0xff || a.heads > 0xff) {
            set_error(error, capacity, "step attention: grid too large for the launch's packed shape");
            return -1;
        }
        const unsigned long long shape = (unsigned long long)per_xcd | ((unsigned long long)a.max_units << 16) | ((unsigned long long)a.batch << 32) |
                                         ((unsigned long long)a.heads << 40);
        items_or_shape = reinterpret_cast<const StepItem *>(shape);
    }
    hipLaunchKernelGGL(kernel_for<QT>(a.width, a.is_self != 0, !packed), dim3(grid), dim3(kThreads), lds, st->stream, a.slots, a.x, a.w, a.scales, a.ln_gain,
                       a.ln_bias, items_or_shape, per_xcd, lg, a);
    return hip_check(hipGetLastError(), "step attention launch", error, capacity);
}

template <int QT>
int slots_t(int width, int max_units, bool is_self, bool with_fold) {
    int per_cu = 0, device = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(kernel_for<QT>(width, is_self, false)), kThreads,
                                                     lds_for<QT>(width, max_units, with_fold)) != hipSuccess ||
        hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
        return 0;
    return per_cu * cus;
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

int step_attention_slots(int qtype, int width, int max_units, int is_self, bool with_fold) {
    switch (qtype) {
        case MYNAH_HIP_F32: return slots_t<MYNAH_HIP_F32>(width, max_units, is_self != 0, with_fold);
        case MYNAH_HIP_F16: return slots_t<MYNAH_HIP_F16>(width, max_units, is_self != 0, with_fold);
        case MYNAH_HIP_INT8: return slots_t<MYNAH_HIP_INT8>(width, max_units, is_self != 0, with_fold);
        default: return slots_t<MYNAH_HIP_INT4>(width, max_units, is_self != 0, with_fold);
    }
}

int launch_step_fold(State *st, const StepAttnArgs &a, float *out, char *error, size_t capacity) {
    const int f4 = a.heads * (kHw / 4);
    const dim3 grid((unsigned)((f4 + kThreads - 1) / kThreads), (unsigned)a.batch);
    hipLaunchKernelGGL(k_step_fold, grid, dim3(kThreads), 0, st->stream, a.partial, a.partial_ml, a.slots, a.heads, a.max_units, a.is_self, out);
    return hip_check(hipGetLastError(), "step fold launch", error, capacity);
}

size_t step_fold_lds_bytes(int max_units) { return (size_t)max_units * (kStepRecord + 1) * sizeof(float); }   // records + one weight per unit

int step_attention_grid(int heads, int batch, int max_units, int is_self, bool packed) {
    if (packed) {
        // table order: the new rows' two roles (self; max_units counts the new row), the cache chunks, the folds
        const int producers = is_self ? 8 * ((2 * batch * heads + 7) / 8) : 0;
        const int chunks = heads * batch * (max_units - (is_self ? 1 : 0));
        return producers + 8 * ((chunks + 7) / 8) + 8 * ((heads * batch + 7) / 8);
    }
    const int items = heads * batch * (max_units + (is_self ? 1 : 0));   // self: the new row takes two workgroups
    return 8 * ((items + 7) / 8);
}

StepItemTables step_item_tables(int batch, int heads, int cross_heads, int max_units, StepItem *self_items, StepItem *cross_items, bool with_fold,
                                int self_slots, int cross_slots) {
    StepItemTables t{};
    if (batch < 1 || batch > kMaxBatch || heads < 1 || heads > 255 || cross_heads < 0 || cross_heads > 255 || max_units < 1 || max_units > 32000 ||
        self_items == nullptr || (cross_heads > 0 && cross_items == nullptr))
        return t;
    t.self_items = self_items;
    t.cross_items = cross_items;
    t.self_entries = step_attention_grid(heads, batch, max_units, 1, true);
    t.cross_entries = cross_heads > 0 ? step_attention_grid(cross_heads, batch, max_units, 0, true) : 0;
    t.batch = batch;
    t.heads = heads;
    t.cross_heads = cross_heads;
    t.with_fold = with_fold ? 1 : 0;
    t.self_budget = self_slots - 8 * ((2 * batch * heads + 7) / 8) - (with_fold ? heads * batch : 0);
    t.cross_budget = cross_slots - (with_fold ? cross_heads * batch : 0);
    return t;
}

int launch_step_attention(State *st, const StepAttnArgs &a, char *error, size_t capacity) {
    if (a.batch < 1 || a.batch > kMaxBatch || a.max_units < 1 || a.partial == nullptr || a.partial_ml == nullptr || a.slots == nullptr ||
        (a.records != nullptr && (a.batch <= kConsumerFoldMaxBatch || a.items == nullptr || a.layer >= 255 || a.abort_word == nullptr ||
                                  a.fold_out == nullptr)) ||
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
