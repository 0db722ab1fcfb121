// The resident decode step as ONE launch: every layer, every stage, in a kernel whose workgroups stay on the chip and hand
// vectors to each other through memory instead of through kernel boundaries.
//
// OPT-IN (graph mode 2), and slower than the default: measured at one stream, int8, 12 layers, 400 us per step against 331 us
// for the captured graph of stage kernels.  It is kept as the measured answer to "are the kernel boundaries what holds the
// step": they are not -- a hand-over through memory costs what a graph node's boundary costs.
//
// decoder_step_batch (src/graph.c:3127-3284) is a chain of dependent stages, per layer
//     1  LN + Q/K/V rows + KV append + split-L self-attention  -> partials      (k_step_attention as a launch)
//     2  fold + O matvec + residual                            -> x             (k_linear)
//     3  LN + Q rows + split-L cross-attention                 -> partials
//     4  fold + O matvec + residual                            -> x
//     5  LN + up matvec + GELU                                 -> hidden
//     6  down matvec + residual                                -> x
// and at one or two streams each stage moves a few megabytes at most: as launches, the 4 us a dependent kernel needs to
// start and to see its predecessor's output outweigh the work.  Here a stage's output is written as (tag, value) pairs
// -- one 64-bit store per value, tag = a number that names the step, the layer and the stage -- and a consumer polls the
// pairs it needs until they carry the tag it expects: the data is its own flag, one memory round trip per hand-over, no
// counters, no fences.  Weight rows, cache rows and LayerNorm vectors of a workgroup's NEXT stage are requested before
// it starts to wait for the current one's input, so they travel while it waits.
//
// The arithmetic of every stage is that of the launched kernels, through the same device functions (device_common.h,
// step_attention_core.h): lane groups, reduction trees, attention units and fold order are identical, so a step gives
// the same bits whichever form ran it.
//
// Every wait is bounded: a poll that exceeds its spin limit (or sees the abort word set) makes its workgroup set the
// abort word and leave; every other workgroup then runs into the same bound or sees the word, so the grid always drains.
// The host finds the word at its next synchronisation and repeats the step as launched kernels.  The grid never exceeds
// what the chip holds at once.
#include "step_attention_core.h"
#include "tagged_exchange.h"

namespace mynah {
namespace {

constexpr int kW = 768;        // model width of this build
constexpr int kF = 3072;       // FFN width of this build
constexpr int kPF = kPrefetchLatency;

// ---- workgroup roles ---------------------------------------------------------------------------------------------------

struct AttnRole {
    bool active, qk, v;
    int head, b;
    int chunk;   // cache chunk of a chunk role
    int count;   // its rows
    int pidx;    // the partial it writes
};

// Workgroup wg of the attention stage: items are numbered head-major over the units that exist -- per head, for self
// attention the Q+K and V roles of every stream's new row, then every stream's cache chunks -- and cut into eight
// contiguous ranges, one per XCD (workgroup i runs on XCD i % 8), so that a head's weight slice is fetched by one or two
// XCDs.  Units depend on each stream's own length only.
__device__ __forceinline__ AttnRole attention_role(const PersistArgs &a, const int wg, const bool is_self) {
    AttnRole r;
    r.active = false; r.qk = false; r.v = false; r.head = 0; r.b = 0; r.chunk = 0; r.count = 0; r.pidx = 0;
    int chunk_items = 0;
    for (int s = 0; s < a.batch; ++s) {
        const int len = is_self ? a.length[s] : a.memory_length[s];
        const int live = (len + kStepUnitRows - 1) / kStepUnitRows;
        chunk_items += is_self ? live : max(live, 1);
    }
    const int heads = is_self ? a.heads : a.cross_heads;
    const int row_items = is_self ? 2 * a.batch : 0;
    const int per_head = row_items + chunk_items;
    const int items = heads * per_head;
    const int per_xcd = (items + 7) / 8;
    const int xcd = wg & 7, slot = wg >> 3;
    const int item = xcd * per_xcd + slot;
    if (slot >= per_xcd || item >= items) return r;
    r.active = true;
    r.head = item / per_head;
    int q = item - r.head * per_head;
    if (q < row_items) {
        r.b = q >> 1;
        r.qk = (q & 1) == 0;
        r.v = !r.qk;
        return r;
    }
    q -= row_items;
    int before = 0;
    for (int s = 0; s < a.batch; ++s) {
        const int len = is_self ? a.length[s] : a.memory_length[s];
        const int live = (len + kStepUnitRows - 1) / kStepUnitRows;
        const int n = is_self ? live : max(live, 1);
        if (q >= before && q < before + n) {
            r.b = s;
            r.chunk = q - before;
            r.count = max(0, min(kStepUnitRows, len - r.chunk * kStepUnitRows));
            r.pidx = is_self ? r.chunk + 1 : r.chunk;
        }
        before += n;
    }
    return r;
}

struct RowRole {
    bool active;
    int row_begin, row_end;
};
// Rows of an [n, k] product for workgroup wg, counted from the END of the grid (the attention roles fill it from the start,
// so the two kinds of stage share as few workgroups as the sizes allow): `wgs` workgroups take rows_per_wg rows each.
__device__ __forceinline__ RowRole row_role(const int wg, const int grid, const int n, const int wgs, const int rows_per_wg) {
    const int i = grid - 1 - wg;
    RowRole r;
    r.active = i < wgs && i * rows_per_wg < n;
    r.row_begin = i * rows_per_wg;
    r.row_end = min(n, r.row_begin + rows_per_wg);
    return r;
}

// ---- attention stage -----------------------------------------------------------------------------------------------------

struct AttnRegs {
    PassRegs pre[kPF];
    // a chunk role's cache rows (K rows in raw[0..8), V rows in raw[8..16), as bits) or the Q+K role's second weight bank
    // (pass p, chunk u in raw[4 p + u]): no role needs both
    uint4 raw[2 * kRowsPerThread];
    float sc2[4 * kPF];
    float ws2[kPF];
    float4 gv[1], bv[1];
};
static_assert(2 * kRowsPerThread == 4 * kPF, "the second weight bank and the cache rows share registers");

// Everything of an attention role that does not depend on the residual stream: weight passes, cache rows, LayerNorm vectors.
template <int QT, bool SELF>
__device__ __forceinline__ void attention_request(AttnRegs &g, const AttnRole &r, const StepAttnArgs &w, const float *kc, const float *vc,
                                                  const float *spare_row, const float *gain, const float *bias) {
    constexpr int kEpc = Chunk<QT>::n;
    constexpr int lg = lane_group_log2(kW / kEpc);
    constexpr int chunks = kW / kEpc;
    const int tid = threadIdx.x;
    g.gv[0] = tid < kW / 4 ? load_global4(gain + 4 * tid) : make_float4(0.f, 0.f, 0.f, 0.f);
    g.bv[0] = (tid < kW / 4 && bias != nullptr) ? load_global4(bias + 4 * tid) : make_float4(0.f, 0.f, 0.f, 0.f);
    if (r.qk) load_bank<QT, kPF>(g.pre, w, 0, 0, 2 * kHw, r.head, lg, chunks);
    else if (r.v) load_bank<QT, kPF>(g.pre, w, 0, 2 * kHw, kHw, r.head, lg, chunks);
    else load_bank<QT, kPF>(g.pre, w, 0, 0, kHw, r.head, lg, chunks);
    // Row scales of the Q+K role's second weight bank (int8): requested by every role of the SELF stage -- the K rows of
    // the q | k | v matrix exist whatever the role -- so that no store into these registers depends on the role.  The
    // cross stage's matrix has Q rows only and no such role.
    constexpr int rpp = 64 >> lg;
    constexpr int qk_passes = (2 * kHw + 4 * rpp - 1) / (4 * rpp);
#pragma unroll
    for (int p = 0; p < kPF; ++p) {
        const int row = min((kPF + p) * 4 * rpp + (tid >> 6) * rpp + ((tid & 63) >> lg), 2 * kHw - 1);
        g.ws2[p] = (SELF && QT == MYNAH_HIP_INT8 && kPF + p < qk_passes) ? load_global(w.scales + weight_row(row, r.head, kW)) : 1.0f;
    }
    if (r.qk) {
#pragma unroll
        for (int p = 0; p < kPF; ++p) {
            PassRegs t;
#pragma unroll
            for (int u = 0; u < 4; ++u) { t.wv[u] = make_uint4(0, 0, 0, 0); t.sc[u] = 0.0f; }
            t.ws = 1.0f;
            if (kPF + p < qk_passes) load_pass<QT, kPF>(t, w, kPF + p, 0, 2 * kHw, r.head, lg, chunks);
#pragma unroll
            for (int u = 0; u < 4; ++u) { g.raw[4 * p + u] = t.wv[u]; g.sc2[4 * p + u] = t.sc[u]; }
        }
        // (emits nothing; it keeps the two branches' last stores apart: merged into one store through a selected address
        // they would pin these registers to scratch memory)
        requests_issued();
    } else {
#pragma unroll
        for (int i = 0; i < 4 * kPF; ++i) g.sc2[i] = 0.0f;
        // every request is issued: a row past the chunk's end repeats the chunk's last row, a role without cache rows
        // (the new row's V role, an empty memory) reads a row that always exists
        const int j = tid & (kPosLanes - 1), grp = tid / kPosLanes;
        const int stride = w.heads * kHw;
        const size_t col = (size_t)r.head * kHw + 4 * j;
        const bool have_rows = r.count > 0;
        const float *const k_from = have_rows ? kc : spare_row;
        const float *const v_from = have_rows ? vc : spare_row;
        const int p0 = r.chunk * kStepUnitRows;
#pragma unroll
        for (int i = 0; i < kRowsPerThread; ++i) {
            const int pi = grp + kPosPerPass * i;
            const int row = !have_rows ? 0 : p0 + min(pi, r.count - 1);
            const size_t at = (size_t)row * stride + col;
            g.raw[i] = __builtin_bit_cast(uint4, load_global4(k_from + at));
            g.raw[kRowsPerThread + i] = __builtin_bit_cast(uint4, load_global4(v_from + at));
        }
    }
}

// The role's arithmetic, from the stream's residual row in x_lds (floats) to its tagged partial.
// part: the stream's partial records [unit][head][kStepRecord]; is_self roles append to the caches.
template <int QT>
__device__ __forceinline__ void attention_compute(AttnRegs &g, const AttnRole &r, const StepAttnArgs &w, const float *x_lds, float *kc, float *vc,
                                                  const int length, const bool has_bias, u64 *part, const int rec_heads, const unsigned tag,
                                                  unsigned char *smem, float *s_sx, float *s_scratch, float *s_proj, float *s_red,
                                                  float *s_wave_ml) {
    constexpr int kEpc = Chunk<QT>::n;
    constexpr int lg = lane_group_log2(kW / kEpc);
    constexpr int chunks = kW / kEpc;
    const int tid = threadIdx.x;
    PrologueParams pro;
    pro.k = kW; pro.batch = 1; pro.ln_gain = x_lds;   // any non-null address: LayerNorm on (the vectors themselves are in g.gv / g.bv)
    pro.ln_bias = has_bias ? pro.ln_gain : nullptr; pro.arith = w.arith;
    pro.probe_qx = nullptr; pro.probe_sx = nullptr;
    float4 xr[1][1];
    xr[0][0] = tid < kW / 4 ? reinterpret_cast<const float4 *>(x_lds)[tid] : make_float4(0.f, 0.f, 0.f, 0.f);
    finish_activations<QT, 1, 1>(pro, whole_workgroup(), xr, g.gv, g.bv, smem, s_sx, s_scratch);
    const int stride = w.heads * kHw;
    u64 *rec0 = part + (size_t)r.head * kStepRecord;                                   // unit 0 (self: the new row)
    u64 *rec = part + ((size_t)r.pidx * rec_heads + r.head) * kStepRecord;
    if (r.qk) {
        PassRegs bank2[kPF];
#pragma unroll
        for (int p = 0; p < kPF; ++p) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                bank2[p].wv[u] = g.raw[4 * p + u];
                bank2[p].sc[u] = g.sc2[4 * p + u];
            }
            bank2[p].ws = g.ws2[p];
        }
        project_bank<QT, kPF>(w, g.pre, 0, 0, 2 * kHw, r.head, lg, chunks, smem, s_sx[0], s_proj);
        project_bank<QT, kPF>(w, bank2, kPF, 0, 2 * kHw, r.head, lg, chunks, smem, s_sx[0], s_proj);
        __syncthreads();
        if (tid < 64) {
            const float kval = s_proj[kHw + tid];
            store_global(kc + (size_t)length * stride + (size_t)r.head * kHw + tid, kval);
            float d = s_proj[tid] * kval;
            d = wave_sum(d);
            if (tid < 4) put(rec0 + kHw + tid, tag, tid == 0 ? d * w.scale : tid == 1 ? 1.0f : 0.0f);   // max | sum (exp(score - max) = 1) | two unused slots
        }
        return;
    }
    if (r.v) {
        project_rows<QT, kPF>(w, g.pre, kPF, 2 * kHw, kHw, r.head, lg, chunks, smem, s_sx[0], s_proj);
        __syncthreads();
        if (tid < kHw) {
            const float vval = s_proj[2 * kHw + tid];
            store_global(vc + (size_t)length * stride + (size_t)r.head * kHw + tid, vval);
            put(rec0 + tid, tag, vval);
        }
        return;
    }
    project_rows<QT, kPF>(w, g.pre, kPF, 0, kHw, r.head, lg, chunks, smem, s_sx[0], s_proj);
    __syncthreads();
    if (r.count <= 0) {   // empty memory (cross only): the context stays zero (src/graph.c:3242)
        if (tid < kHw) put(rec + tid, tag, 0.0f);
        if (tid < 4) put(rec + kHw + tid, tag, tid == 1 ? 1.0f : 0.0f);
        return;
    }
    const int j = tid & (kPosLanes - 1);
    const float4 qv = *reinterpret_cast<const float4 *>(s_proj + 4 * j);
    float4 kv[kRowsPerThread], vv[kRowsPerThread];
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        kv[i] = __builtin_bit_cast(float4, g.raw[i]);
        vv[i] = __builtin_bit_cast(float4, g.raw[kRowsPerThread + i]);
    }
    attend_chunk(qv, kv, vv, r.count, w.scale, s_red, s_wave_ml);
    __syncthreads();
    if (tid < kPosLanes) {
        float4 o;
        float M, L;
        merge_chunk(tid, s_red, s_wave_ml, o, M, L);
        put(rec + 4 * tid, tag, o.x);
        put(rec + 4 * tid + 1, tag, o.y);
        put(rec + 4 * tid + 2, tag, o.z);
        put(rec + 4 * tid + 3, tag, o.w);
        if (tid < 4) put(rec + kHw + tid, tag, tid == 0 ? M : tid == 1 ? L : 0.0f);
    }
}

// ---- matvec stages -------------------------------------------------------------------------------------------------------

// Operands of a row role requested ahead: the first P passes of its rows (a pass = the 4 x (64 / lane group) rows the
// workgroup's four wavefronts take at a time); passes beyond P are requested when their turn comes.
template <int BT, int NVT, int P>
struct RowRegs {
    uint4 wv[P][4];
    float sc[P][4];
    float ws[P];
    u64 res[P];         // the residual value of this lane's (row, stream), tagged
    float4 gv[NVT], bv[NVT];
};

// Where the residual of a row comes from: a tagged vector of an earlier stage, or -- first layer -- input + position.
struct Residual {
    const u64 *tagged;          // [BT][kW], or null
    unsigned tag;
    const float *input[2];
    const float *position[2];   // null entries: no position table
};
__device__ __forceinline__ u64 residual_request(const Residual &src, const int stream, const int row) {
    if (src.tagged != nullptr) return get(src.tagged + (size_t)stream * kW + row);
    const float *in = stream == 0 ? src.input[0] : src.input[1];
    const float *pe = stream == 0 ? src.position[0] : src.position[1];
    const float v = pe != nullptr ? load_global(in + row) + load_global(pe + row) : load_global(in + row);
    return ((u64)src.tag << 32) | (u64)__float_as_uint(v);
}

template <int QT, int BT, int NVT, int K, int P>
__device__ __forceinline__ void rows_request(RowRegs<BT, NVT, P> &g, const RowRole &r, const void *w, const float *scales, const bool with_res,
                                             const Residual &res, const int batch, const float *gain, const float *bias) {
    constexpr int kEpc = Chunk<QT>::n;
    constexpr int chunks = K / kEpc;
    constexpr int lg = lane_group_log2(chunks);
    constexpr int G = 1 << lg;
    constexpr int rpp = 64 >> lg;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gl = lane & (G - 1), gidx = lane >> lg;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int row = r.row_begin + p * 4 * rpp + wave * rpp + gidx;
        const int rowc = row < r.row_end ? row : r.row_end - 1;
        const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(w) + (size_t)rowc * chunks * 16);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = gl + u * G;
            g.wv[p][u] = c < chunks ? load_global_u4(wrow + c) : make_uint4(0, 0, 0, 0);
            g.sc[p][u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? load_global(scales + (size_t)rowc * chunks + c) : 0.0f;
        }
        g.ws[p] = 1.0f;
        g.res[p] = 0;
        if (gl < BT) {
            if constexpr (QT == MYNAH_HIP_INT8) g.ws[p] = load_global(scales + rowc);
            if (with_res && gl < batch) g.res[p] = residual_request(res, gl, rowc);
        }
    }
#pragma unroll
    for (int i = 0; i < NVT; ++i) {
        const int f = tid + kThreads * i;
        g.gv[i] = (gain != nullptr && f < K / 4) ? load_global4(gain + 4 * f) : make_float4(0.f, 0.f, 0.f, 0.f);
        g.bv[i] = (gain != nullptr && bias != nullptr && f < K / 4) ? load_global4(bias + 4 * f) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

// The residual values of a role's requested passes alone (for a role whose weights were requested while the residual
// stream was still being written).
template <int QT, int BT, int NVT, int K, int P>
__device__ __forceinline__ void rows_request_residual(RowRegs<BT, NVT, P> &g, const RowRole &r, const Residual &res, const int batch) {
    constexpr int lg = lane_group_log2(K / Chunk<QT>::n);
    constexpr int G = 1 << lg;
    constexpr int rpp = 64 >> lg;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int gl = lane & (G - 1), gidx = lane >> lg;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int row = r.row_begin + p * 4 * rpp + wave * rpp + gidx;
        const int rowc = row < r.row_end ? row : r.row_end - 1;
        if (gl < BT && gl < batch) g.res[p] = residual_request(res, gl, rowc);
    }
}

// One pass of rows: products against the activations staged in smem, lane-group reduction, epilogue, tagged stores.
// Lane b of a row's lane group finishes stream b.  EPI: EPI_GELU or EPI_RESIDUAL.
template <int QT, int BT, int K, int EPI>
__device__ __forceinline__ void rows_pass(const uint4 (&wv)[4], const float (&sc)[4], const float ws, const u64 resv, const int row, const bool valid,
                                          const Residual &res, const int batch, const unsigned char *smem, const float *s_sx, u64 *dst,
                                          const int dst_stride, const unsigned tag, Waiter &wt) {
    constexpr int kEpc = Chunk<QT>::n;
    constexpr int chunks = K / kEpc;
    constexpr int lg = lane_group_log2(chunks);
    constexpr int G = 1 << lg;
    static_assert(G >= BT, "a lane group must have a lane per stream");
    static_assert((chunks + G - 1) / G <= 4, "one register group of four chunks per lane");
    const int gl = (threadIdx.x & 63) & (G - 1);
    int iacc[BT];
    float facc[BT];
#pragma unroll
    for (int b = 0; b < BT; ++b) { iacc[b] = 0; facc[b] = 0.0f; }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int c = gl + u * G;
        if (c < chunks) dot_chunk<QT, BT>(wv[u], sc[u], c, smem, K, iacc, facc, nullptr);
    }
    group_reduce<QT, BT>(iacc, facc, lg);
    if (gl < batch && valid) {
        int mi = iacc[0];
        float mf = facc[0];
#pragma unroll
        for (int b = 1; b < BT; ++b)
            if (gl == b) { mi = iacc[b]; mf = facc[b]; }
        float val = finish_value<QT>(mi, mf, ws, s_sx[gl]);
        if (EPI == EPI_GELU) val = gelu_tanh(val);
        if (EPI == EPI_RESIDUAL) {
            const float before = res.tagged != nullptr ? settle(resv, res.tagged + (size_t)gl * kW + row, res.tag, wt) : value_of(resv);
            val = before + val;
        }
        put(dst + (size_t)gl * dst_stride + row, tag, val);
    }
}

template <int QT, int BT, int NVT, int K, int P, int EPI>
__device__ __forceinline__ void rows_compute(RowRegs<BT, NVT, P> &g, const RowRole &r, const void *w, const float *scales, const Residual &res,
                                             const int batch, const unsigned char *smem, const float *s_sx, u64 *dst, const int dst_stride,
                                             const unsigned tag, Waiter &wt) {
    constexpr int kEpc = Chunk<QT>::n;
    constexpr int chunks = K / kEpc;
    constexpr int lg = lane_group_log2(chunks);
    constexpr int G = 1 << lg;
    constexpr int rpp = 64 >> lg;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gl = lane & (G - 1), gidx = lane >> lg;
#pragma unroll
    for (int p = 0; p < P; ++p) {   // the passes requested ahead
        const int row = r.row_begin + p * 4 * rpp + wave * rpp + gidx;
        if (r.row_begin + p * 4 * rpp + wave * rpp < r.row_end)   // the same for the whole wavefront
            rows_pass<QT, BT, K, EPI>(g.wv[p], g.sc[p], g.ws[p], g.res[p], row, row < r.row_end, res, batch, smem, s_sx, dst, dst_stride, tag, wt);
    }
    for (int base = r.row_begin + P * 4 * rpp + wave * rpp; base < r.row_end; base += 4 * rpp) {   // any further pass
        const int row = base + gidx;
        const bool valid = row < r.row_end;
        const int rowc = valid ? row : r.row_end - 1;
        const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(w) + (size_t)rowc * chunks * 16);
        uint4 wv[4];
        float sc[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = gl + u * G;
            wv[u] = c < chunks ? load_global_u4(wrow + c) : make_uint4(0, 0, 0, 0);
            sc[u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? load_global(scales + (size_t)rowc * chunks + c) : 0.0f;
        }
        float ws = 1.0f;
        u64 resv = 0;
        if (gl < batch && valid) {
            if constexpr (QT == MYNAH_HIP_INT8) ws = load_global(scales + row);
            if (EPI == EPI_RESIDUAL) resv = residual_request(res, gl, row);
        }
        rows_pass<QT, BT, K, EPI>(wv, sc, ws, resv, row, valid, res, batch, smem, s_sx, dst, dst_stride, tag, wt);
    }
}

// The fold of a stream's attention partials (fold_partials' arithmetic, units in order) for this thread's float4 of the row.
__device__ __forceinline__ float4 fold_from_lds(const float *rec, const int rec_heads, const int units, const int f4) {
    const int d = 4 * f4;
    const int head = d / kHw, dh = d - head * kHw;
    const float *base = rec + (size_t)head * kStepRecord;
    const size_t ustride = (size_t)rec_heads * kStepRecord;
    float M = -3.0e38f;
    for (int u = 0; u < units; ++u) M = fmaxf(M, base[u * ustride + kHw]);
    float L = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int u = 0; u < units; ++u) {
        const float *p = base + u * ustride;
        const float wgt = expf(p[kHw] - M);
        const float4 ou = *reinterpret_cast<const float4 *>(p + dh);
        L = __builtin_fmaf(p[kHw + 1], wgt, L);
        acc.x = __builtin_fmaf(ou.x, wgt, acc.x);
        acc.y = __builtin_fmaf(ou.y, wgt, acc.y);
        acc.z = __builtin_fmaf(ou.z, wgt, acc.z);
        acc.w = __builtin_fmaf(ou.w, wgt, acc.w);
    }
    acc.x /= L; acc.y /= L; acc.z /= L; acc.w /= L;
    return acc;
}

// ---- the kernel ------------------------------------------------------------------------------------------------------------

// What both kinds of workgroup need to find the exchange area's parts and the step's tags.
struct Exchange {
    u64 *X6, *X2, *X4, *H, *PS, *PC;
    size_t ps_stream, pc_stream;
};
__device__ __forceinline__ Exchange exchange_of(const PersistArgs &a) {
    Exchange e;
    e.X6 = a.exchange;
    e.X2 = e.X6 + 2 * kW;
    e.X4 = e.X2 + 2 * kW;
    e.H = e.X4 + 2 * kW;
    e.PS = e.H + 2 * kF;
    e.ps_stream = (size_t)a.max_units * a.heads * kStepRecord;
    e.PC = e.PS + 2 * e.ps_stream;
    e.pc_stream = (size_t)a.max_units * (a.cross_heads > 0 ? a.cross_heads : 1) * kStepRecord;
    return e;
}

// One stream's kernel arguments as values (an argument array indexed by a run-time stream number would be read with
// vector loads at every use).
struct StreamArgs {
    float *self_k, *self_v;
    const float *cross_k, *cross_v, *input, *pos_row;
    float *output;
    int length, memory_length;
};
__device__ __forceinline__ StreamArgs stream_of(const PersistArgs &a, const int b) {
    StreamArgs s;
    s.self_k = b == 0 ? a.self_k[0] : a.self_k[1];
    s.self_v = b == 0 ? a.self_v[0] : a.self_v[1];
    s.cross_k = b == 0 ? a.cross_k[0] : a.cross_k[1];
    s.cross_v = b == 0 ? a.cross_v[0] : a.cross_v[1];
    s.input = b == 0 ? a.input[0] : a.input[1];
    s.output = b == 0 ? a.output[0] : a.output[1];
    s.length = b == 0 ? a.length[0] : a.length[1];
    s.memory_length = b == 0 ? a.memory_length[0] : a.memory_length[1];
    s.pos_row = a.position != nullptr ? a.position + (size_t)s.length * kW : nullptr;
    return s;
}

// a workgroup that cannot go on: say so, and leave (every barrier of this kernel is passed by whole workgroups)
#define MYNAH_LEAVE_IF_DEAD()                                                                                           \
    if (__syncthreads_or(wt.dead ? 1 : 0)) {                                                                            \
        if (threadIdx.x == 0) __hip_atomic_store(a.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);         \
        return;                                                                                                         \
    }
// development builds only: clock readings (100 MHz) of one layer, per workgroup: slot 3 (stage - 1) + {0 before the wait,
// 1 input there, 2 stage done}
struct SharedBlocks {
    float *s_in;
    unsigned char *smem;
    float *s_proj, *s_red, *s_wave_ml, *s_sx, *s_scratch, *s4;
};

// A workgroup of the attention stages: per layer, stage 1 (self) and stage 3 (cross).  Everything of a stage that does not
// depend on the residual stream is requested as soon as the stage before it is done.
template <int QT>
__device__ __forceinline__ void attention_path(const PersistArgs &a, const SharedBlocks &sh, const AttnRole r1, const AttnRole r3) {
    const int tid = threadIdx.x;
    const Exchange ex = exchange_of(a);
    Waiter wt{a.spin_limit, a.abort_word, false};
    const StreamArgs s1 = stream_of(a, r1.b), s3 = stream_of(a, r3.b);
    const int stride_self = a.heads * kHw, stride_cross = a.cross_heads * kHw;
    StepAttnArgs aw{};
    aw.width = kW;
    aw.arith = a.arith;
    aw.scale = a.scale;
    AttnRegs g;
    if (r1.active) {
        const PersistLayer &lw = a.layers[0];
        aw.w = lw.qkv_w; aw.scales = lw.qkv_s; aw.heads = a.heads;
        attention_request<QT, true>(g, r1, aw, s1.self_k, s1.self_v, s1.input, lw.norm_self, lw.norm_self_b);
        requests_issued();
    }
    for (int layer = 0; layer < a.n_layers; ++layer) {
        const PersistLayer &lw = a.layers[layer];
        const unsigned t0 = a.epoch + 8u * (unsigned)layer;
        if (r1.active) {
            if (layer == 0) {
                for (int i = tid; i < kW; i += kThreads)
                    sh.s_in[i] = s1.pos_row != nullptr ? load_global(s1.input + i) + load_global(s1.pos_row + i) : load_global(s1.input + i);
            } else {
                fetch_tagged<3, false>(ex.X6 + (size_t)r1.b * kW, sh.s_in, kW, t0, wt);
            }
            MYNAH_LEAVE_IF_DEAD();
            aw.w = lw.qkv_w; aw.scales = lw.qkv_s; aw.heads = a.heads;
            float *kc = s1.self_k + (size_t)layer * a.capacity * stride_self;
            float *vc = s1.self_v + (size_t)layer * a.capacity * stride_self;
            attention_compute<QT>(g, r1, aw, sh.s_in, kc, vc, s1.length, lw.norm_self_b != nullptr, ex.PS + (size_t)r1.b * ex.ps_stream, a.heads,
                                  t0 + 1u, sh.smem, sh.s_sx, sh.s_scratch, sh.s_proj, sh.s_red, sh.s_wave_ml);
        }
        if (r3.active) {
            aw.w = lw.qx_w; aw.scales = lw.qx_s; aw.heads = a.cross_heads;
            const size_t at = (size_t)layer * s3.memory_length * stride_cross;
            attention_request<QT, false>(g, r3, aw, s3.cross_k != nullptr ? s3.cross_k + at : nullptr, s3.cross_v != nullptr ? s3.cross_v + at : nullptr,
                                         s3.input, lw.norm_cross, lw.norm_cross_b);
            requests_issued();
            fetch_tagged<3, false>(ex.X2 + (size_t)r3.b * kW, sh.s_in, kW, t0 + 2u, wt);
            MYNAH_LEAVE_IF_DEAD();
            attention_compute<QT>(g, r3, aw, sh.s_in, nullptr, nullptr, 0, lw.norm_cross_b != nullptr, ex.PC + (size_t)r3.b * ex.pc_stream, a.cross_heads,
                                  t0 + 3u, sh.smem, sh.s_sx, sh.s_scratch, sh.s_proj, sh.s_red, sh.s_wave_ml);
        }
        if (r1.active && layer + 1 < a.n_layers) {
            const PersistLayer &nx = a.layers[layer + 1];
            aw.w = nx.qkv_w; aw.scales = nx.qkv_s; aw.heads = a.heads;
            const size_t at = (size_t)(layer + 1) * a.capacity * stride_self;
            attention_request<QT, true>(g, r1, aw, s1.self_k + at, s1.self_v + at, s1.input, nx.norm_self, nx.norm_self_b);
            requests_issued();
        }
    }
}

// A workgroup of the row stages: per layer, stages 2, 4, 5, 6 for its rows, and at the end the final norm of one stream.
// A stage's weight rows are requested when the stage before it has its input, i.e. they travel during that stage's
// arithmetic and the wait that follows.
template <int QT, int BT>
__device__ __forceinline__ void rows_path(const PersistArgs &a, const SharedBlocks &sh, const RowRole r2, const RowRole r5, const RowRole r6,
                                          const int final_stream) {
    // passes of rows requested ahead per role: 32 rows of FFN up, 8 of FFN down, one pass of the output projections
    constexpr int rpp768 = 64 >> lane_group_log2(kW / Chunk<QT>::n), rpp3072 = 64 >> lane_group_log2(kF / Chunk<QT>::n);
    constexpr int kUpPasses = 32 / (4 * rpp768) > 0 ? 32 / (4 * rpp768) : 1, kDownPasses = 8 / (4 * rpp3072) > 0 ? 8 / (4 * rpp3072) : 1;
    constexpr int kOutPasses = kUpPasses;   // 32 rows of an output projection: every partial record is read by 24 workgroups
    const int tid = threadIdx.x;
    const Exchange ex = exchange_of(a);
    Waiter wt{a.spin_limit, a.abort_word, false};
    const StreamArgs sa = stream_of(a, 0), sb = stream_of(a, 1);
    const bool cross = a.cross_heads > 0;
    PrologueParams pro;
    pro.batch = a.batch; pro.arith = a.arith; pro.probe_qx = nullptr; pro.probe_sx = nullptr;

    RowRegs<BT, 1, kOutPasses> g2;
    if (r2.active) {
        Residual res0;
        res0.tagged = nullptr; res0.tag = a.epoch;
        res0.input[0] = sa.input; res0.input[1] = sb.input; res0.position[0] = sa.pos_row; res0.position[1] = sb.pos_row;
        rows_request<QT, BT, 1, kW, kOutPasses>(g2, r2, a.layers[0].o_w, a.layers[0].o_s, true, res0, a.batch, nullptr, nullptr);
        requests_issued();
    }
    for (int layer = 0; layer < a.n_layers; ++layer) {
        const PersistLayer &lw = a.layers[layer];
        const unsigned t0 = a.epoch + 8u * (unsigned)layer;
        Residual res_prev;   // x before this layer
        res_prev.tagged = layer == 0 ? nullptr : ex.X6;
        res_prev.tag = t0;
        res_prev.input[0] = sa.input; res_prev.input[1] = sb.input; res_prev.position[0] = sa.pos_row; res_prev.position[1] = sb.pos_row;
        Residual res2;
        res2.tagged = ex.X2; res2.tag = t0 + 2u;
        res2.input[0] = res2.input[1] = nullptr; res2.position[0] = res2.position[1] = nullptr;
        Residual res_mid = res2;   // x before the FFN: after the cross sublayer when there is one
        if (cross) { res_mid.tagged = ex.X4; res_mid.tag = t0 + 4u; }

        // ---------------------------------------------------------------- 2: fold + O + residual
        RowRegs<BT, 1, kOutPasses> g4;
        if (r2.active) {
            int off = 0;
            for (int b = 0; b < a.batch; ++b) {
                const int units = ((b == 0 ? sa.length : sb.length) + kStepUnitRows - 1) / kStepUnitRows + 1;
                const int n = units * a.heads * kStepRecord;
                fetch_tagged<32, true>(ex.PS + (size_t)b * ex.ps_stream, sh.s_in + off, n, t0 + 1u, wt);
                off += n;
            }
            MYNAH_LEAVE_IF_DEAD();
            if (layer > 0) rows_request_residual<QT, BT, 1, kW, kOutPasses>(g2, r2, res_prev, a.batch);   // the partials are there, so the stream they were made from is
            if (cross) {
                rows_request<QT, BT, 1, kW, kOutPasses>(g4, r2, lw.ox_w, lw.ox_s, true, res2, a.batch, nullptr, nullptr);
                requests_issued();
            }
            float4 xr[BT][1];
            off = 0;
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                xr[b][0] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (b < a.batch) {
                    const int units = ((b == 0 ? sa.length : sb.length) + kStepUnitRows - 1) / kStepUnitRows + 1;
                    if (tid < kW / 4) xr[b][0] = fold_from_lds(sh.s_in + off, a.heads, units, tid);
                    off += units * a.heads * kStepRecord;
                }
            }
            pro.k = kW; pro.ln_gain = nullptr; pro.ln_bias = nullptr;
            finish_activations<QT, BT, 1>(pro, whole_workgroup(), xr, g2.gv, g2.bv, sh.smem, sh.s_sx, sh.s_scratch);
            rows_compute<QT, BT, 1, kW, kOutPasses, EPI_RESIDUAL>(g2, r2, lw.o_w, lw.o_s, res_prev, a.batch, sh.smem, sh.s_sx, ex.X2, kW, t0 + 2u, wt);
        }
        // ---------------------------------------------------------------- 4: fold + O + residual (cross)
        RowRegs<BT, 1, kUpPasses> g5;
        if (r2.active && cross) {
            int off = 0;
            for (int b = 0; b < a.batch; ++b) {
                const int units = max(((b == 0 ? sa.memory_length : sb.memory_length) + kStepUnitRows - 1) / kStepUnitRows, 1);
                const int n = units * a.cross_heads * kStepRecord;
                fetch_tagged<32, true>(ex.PC + (size_t)b * ex.pc_stream, sh.s_in + off, n, t0 + 3u, wt);
                off += n;
            }
            MYNAH_LEAVE_IF_DEAD();
        }
        if (r5.active) {
            rows_request<QT, BT, 1, kW, kUpPasses>(g5, r5, lw.up_w, lw.up_s, false, res_mid, a.batch, lw.norm_ff, lw.norm_ff_b);
            requests_issued();
        }
        if (r2.active && cross) {
            float4 xr[BT][1];
            int off = 0;
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                xr[b][0] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (b < a.batch) {
                    const int units = max(((b == 0 ? sa.memory_length : sb.memory_length) + kStepUnitRows - 1) / kStepUnitRows, 1);
                    if (tid < kW / 4) xr[b][0] = fold_from_lds(sh.s_in + off, a.cross_heads, units, tid);
                    off += units * a.cross_heads * kStepRecord;
                }
            }
            pro.k = kW; pro.ln_gain = nullptr; pro.ln_bias = nullptr;
            finish_activations<QT, BT, 1>(pro, whole_workgroup(), xr, g4.gv, g4.bv, sh.smem, sh.s_sx, sh.s_scratch);
            rows_compute<QT, BT, 1, kW, kOutPasses, EPI_RESIDUAL>(g4, r2, lw.ox_w, lw.ox_s, res2, a.batch, sh.smem, sh.s_sx, ex.X4, kW, t0 + 4u, wt);
        }
        // ---------------------------------------------------------------- 5: LN + up + GELU
        RowRegs<BT, 3, kDownPasses> g6;
        if (r5.active) {
            fetch_tagged<3 * BT, false>(res_mid.tagged, sh.s_in, a.batch * kW, res_mid.tag, wt);
            MYNAH_LEAVE_IF_DEAD();
        }
        if (r6.active) {
            rows_request<QT, BT, 3, kF, kDownPasses>(g6, r6, lw.down_w, lw.down_s, true, res_mid, a.batch, nullptr, nullptr);
            requests_issued();
        }
        if (r5.active) {
            float4 xr[BT][1];
#pragma unroll
            for (int b = 0; b < BT; ++b)
                xr[b][0] = (b < a.batch && tid < kW / 4) ? reinterpret_cast<const float4 *>(sh.s_in)[b * (kW / 4) + tid] : make_float4(0.f, 0.f, 0.f, 0.f);
            pro.k = kW; pro.ln_gain = lw.norm_ff; pro.ln_bias = lw.norm_ff_b;
            finish_activations<QT, BT, 1>(pro, whole_workgroup(), xr, g5.gv, g5.bv, sh.smem, sh.s_sx, sh.s_scratch);
            rows_compute<QT, BT, 1, kW, kUpPasses, EPI_GELU>(g5, r5, lw.up_w, lw.up_s, res_mid, a.batch, sh.smem, sh.s_sx, ex.H, kF, t0 + 5u, wt);
        }
        // ---------------------------------------------------------------- 6: down + residual
        if (r6.active) {
            fetch_tagged<12 * BT, true>(ex.H, sh.s_in, a.batch * kF, t0 + 5u, wt);
            MYNAH_LEAVE_IF_DEAD();
        }
        if (r2.active && layer + 1 < a.n_layers) {
            Residual res_next;
            res_next.tagged = ex.X6; res_next.tag = t0 + 8u;
            res_next.input[0] = res_next.input[1] = nullptr; res_next.position[0] = res_next.position[1] = nullptr;
            // the weights only: this layer's residual stream is still being written (the row's value is polled for at its use)
            rows_request<QT, BT, 1, kW, kOutPasses>(g2, r2, a.layers[layer + 1].o_w, a.layers[layer + 1].o_s, false, res_next, a.batch, nullptr, nullptr);
            requests_issued();
        }
        if (r6.active) {
            float4 xr[BT][3];
#pragma unroll
            for (int b = 0; b < BT; ++b)
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    xr[b][i] = b < a.batch ? reinterpret_cast<const float4 *>(sh.s_in)[b * (kF / 4) + tid + kThreads * i] : make_float4(0.f, 0.f, 0.f, 0.f);
            pro.k = kF; pro.ln_gain = nullptr; pro.ln_bias = nullptr;
            finish_activations<QT, BT, 3>(pro, whole_workgroup(), xr, g6.gv, g6.bv, sh.smem, sh.s_sx, sh.s_scratch);
            rows_compute<QT, BT, 3, kF, kDownPasses, EPI_RESIDUAL>(g6, r6, lw.down_w, lw.down_s, res_mid, a.batch, sh.smem, sh.s_sx, ex.X6, kW, t0 + 8u, wt);
        }
    }
    // ---------------------------------------------------------------- final norm of one stream's row
    if (final_stream >= 0) {
        const StreamArgs sf = stream_of(a, final_stream);
        __syncthreads();
        fetch_tagged<3, false>(ex.X6 + (size_t)final_stream * kW, sh.s_in, kW, a.epoch + 8u * (unsigned)a.n_layers, wt);
        MYNAH_LEAVE_IF_DEAD();
        if (a.norm_out == nullptr) {
            for (int d = tid; d < kW; d += kThreads) store_global(sf.output + d, sh.s_in[d]);
        } else {
            layernorm_row(sh.s_in, sf.output, a.norm_out, a.norm_out_b, kW, sh.s4);
        }
    }
}

// The grid: attention workgroups [0, a.attention_wgs), row workgroups counted from the end.  The two ranges never overlap
// (the host takes another path when they would), so a workgroup runs one of the two loops.
template <int QT, int BT>
__global__ void __launch_bounds__(kThreads) k_step_persistent(const PersistArgs a) {
    extern __shared__ __align__(16) float s_in[];               // what a stage waits for: residual rows, hidden rows or partial records
    __shared__ __align__(16) unsigned char smem[BT * kF];        // staged (quantised) activations
    __shared__ __align__(16) float s_proj[3 * kHw];
    __shared__ __align__(16) float s_red[4 * kHw];
    __shared__ float s_wave_ml[8];
    __shared__ float s_sx[BT];
    __shared__ float s_scratch[kPrologueScratch * BT];
    __shared__ float s4[4];
    const SharedBlocks sh{s_in, smem, s_proj, s_red, s_wave_ml, s_sx, s_scratch, s4};
    const int wg = blockIdx.x, grid = gridDim.x;
    if (wg < a.attention_wgs) {
        const AttnRole r1 = attention_role(a, wg, true);
        AttnRole r3 = attention_role(a, wg, false);
        if (a.cross_heads == 0) r3.active = false;
        if (r1.active || r3.active) attention_path<QT>(a, sh, r1, r3);
        return;
    }
    const RowRole r2 = row_role(wg, grid, kW, a.wgs_out, a.rows_out);
    const RowRole r5 = row_role(wg, grid, kF, a.wgs_up, a.rows_up);
    const RowRole r6 = row_role(wg, grid, kW, a.wgs_down, a.rows_down);
    const int final_stream = grid - 1 - wg < a.batch ? grid - 1 - wg : -1;
    if (r2.active || r5.active || r6.active || final_stream >= 0) rows_path<QT, BT>(a, sh, r2, r5, r6, final_stream);
}
#undef MYNAH_LEAVE_IF_DEAD

}  // namespace

bool step_persistent_supported(int qtype, size_t width, size_t heads, size_t head_width, size_t ffn, size_t cross_heads, size_t cross_head_width) {
    if (qtype != MYNAH_HIP_INT8 && qtype != MYNAH_HIP_INT4) return false;
    if (width != (size_t)kW || ffn != (size_t)kF || head_width != (size_t)kHw || heads * head_width != width) return false;
    if (cross_heads != 0 && (cross_head_width != (size_t)kHw || cross_heads * cross_head_width != width)) return false;
    return true;
}

size_t step_persistent_exchange_words(const PersistArgs &a) {
    const size_t cross_heads = a.cross_heads > 0 ? a.cross_heads : 1;
    return 3 * 2 * (size_t)kW + 2 * (size_t)kF + 2 * (size_t)a.max_units * a.heads * kStepRecord + 2 * (size_t)a.max_units * cross_heads * kStepRecord;
}

// Workgroups the attention stages need for these lengths (the launch is refused when the grid has fewer).
int step_persistent_attention_workgroups(const PersistArgs &a) {
    int self_items = 0, cross_items = 0;
    for (int s = 0; s < a.batch; ++s) {
        self_items += 2 + (a.length[s] + kStepUnitRows - 1) / kStepUnitRows;
        const int live = (a.memory_length[s] + kStepUnitRows - 1) / kStepUnitRows;
        cross_items += live > 1 ? live : 1;
    }
    const int self_wgs = 8 * ((a.heads * self_items + 7) / 8);
    const int cross_wgs = 8 * ((a.cross_heads * cross_items + 7) / 8);
    return self_wgs > cross_wgs ? self_wgs : cross_wgs;
}

// LDS for the largest thing a stage waits for: all partial records of the streams, or their hidden rows
static size_t persistent_lds_bytes(const PersistArgs &a) {
    size_t floats = (size_t)a.batch * kF;
    size_t rec = 0;
    for (int s = 0; s < a.batch; ++s) {
        const size_t self_units = (size_t)(a.length[s] + kStepUnitRows - 1) / kStepUnitRows + 1;
        size_t cross_units = (size_t)(a.memory_length[s] + kStepUnitRows - 1) / kStepUnitRows;
        if (cross_units < 1) cross_units = 1;
        const size_t self_rec = self_units * a.heads, cross_rec = cross_units * a.cross_heads;
        rec += (self_rec > cross_rec ? self_rec : cross_rec) * kStepRecord;
    }
    if (rec > floats) floats = rec;
    return floats * sizeof(float);
}
constexpr size_t kPersistentLdsLimit = 120 * 1024;

template <int QT, int BT>
static int launch_pt(State *st, const PersistArgs &a, int grid, char *error, size_t capacity) {
    const size_t lds = persistent_lds_bytes(a);
    if (lds > kPersistentLdsLimit) {
        set_error(error, capacity, "persistent step: the attention partials of these lengths exceed the workgroup's LDS");
        return -1;
    }
    static bool raised = false;   // per instantiation
    if (!raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_step_persistent<QT, BT>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      120 * 1024));
        int per_cu = 0;
        MYNAH_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(&k_step_persistent<QT, BT>), kThreads,
                                                               120 * 1024));
        if (per_cu < 1) {
            set_error(error, capacity, "persistent step: the kernel does not fit a compute unit");
            return -1;
        }
        raised = true;
    }
    hipLaunchKernelGGL((k_step_persistent<QT, BT>), dim3(grid), dim3(kThreads), lds, st->stream, a);
    return hip_check(hipGetLastError(), "persistent step launch", error, capacity);
}

// Whether these lengths and workgroup counts fit the launch (what launch_step_persistent would refuse for its shape): asked
// before a step commits to this form, so that a step that does not fit runs as launched kernels instead of failing.
bool step_persistent_fits(const PersistArgs &a, int grid) {
    const int row_wgs = a.wgs_up > a.wgs_down ? (a.wgs_up > a.wgs_out ? a.wgs_up : a.wgs_out) : (a.wgs_down > a.wgs_out ? a.wgs_down : a.wgs_out);
    return a.batch >= 1 && a.batch <= 2 && a.rows_out > 0 && a.rows_up > 0 && a.rows_down > 0 && a.wgs_out > 0 && a.wgs_up > 0 && a.wgs_down > 0 &&
           a.attention_wgs == step_persistent_attention_workgroups(a) && a.attention_wgs + row_wgs <= grid && a.batch <= row_wgs &&
           persistent_lds_bytes(a) <= kPersistentLdsLimit;
}

int launch_step_persistent(State *st, const PersistArgs &a, int qtype, int grid, char *error, size_t capacity) {
    const int row_wgs = a.wgs_up > a.wgs_down ? (a.wgs_up > a.wgs_out ? a.wgs_up : a.wgs_out) : (a.wgs_down > a.wgs_out ? a.wgs_down : a.wgs_out);
    if (a.batch < 1 || a.batch > 2 || a.exchange == nullptr || a.abort_word == nullptr || a.layers == nullptr || a.n_layers < 1 ||
        a.attention_wgs != step_persistent_attention_workgroups(a) || a.attention_wgs + row_wgs > grid || a.batch > row_wgs) {
        set_error(error, capacity, "persistent step: invalid arguments or too few workgroups for these lengths");
        return -1;
    }
    if (qtype == MYNAH_HIP_INT8) return a.batch == 1 ? launch_pt<MYNAH_HIP_INT8, 1>(st, a, grid, error, capacity) : launch_pt<MYNAH_HIP_INT8, 2>(st, a, grid, error, capacity);
    if (qtype == MYNAH_HIP_INT4) return a.batch == 1 ? launch_pt<MYNAH_HIP_INT4, 1>(st, a, grid, error, capacity) : launch_pt<MYNAH_HIP_INT4, 2>(st, a, grid, error, capacity);
    set_error(error, capacity, "persistent step: int8 and int4 weights only");
    return -1;
}

}  // namespace mynah
