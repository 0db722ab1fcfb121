// Weight-stationary decode matvec for gfx950, fused with its neighbours.
//
// One launch computes, for up to 8 concurrent streams b,
//     out[b] = epilogue( W . prologue(in[b]) )
// prologue : the activation row (a device vector, or the fold of the split-L attention partials written
//            by the preceding attention kernel), optional LayerNorm (two-pass mean / variance, eps 1e-5,
//            gain and optional bias), then for int8/int4 weights the per-vector absmax int8 activation
//            quantisation (quantize_act_int8, src/qmat.c:94-113) -- each workgroup recomputes it from the
//            3-12 KB input vector instead of paying a grid-wide dependency for it;
// body     : every 16-byte weight chunk is fetched from HBM exactly once per launch (128-bit loads,
//            a row's chunks spread over a lane group of G lanes so a group reads 16*G contiguous
//            bytes) and dotted against all streams' activations held in LDS: v_dot4_i32_i8 for
//            int8/int4 (dot_q8/dot_q4, src/qmat.c:136-185), f32 FMA of exactly widened halves for f16
//            (matvec_f16, src/qmat.c:306-378), f32 FMA for f32; lane-group butterfly reduction;
// epilogue : ((float)acc * scale[row]) * sx (+ bias), optional tanh-GELU (src/kernels.c:382-389),
//            optional residual accumulate into out (src/graph.c:3212,3254,3275).
//
// A decode step is a chain of dependent launches of a few microseconds each, so the kernel is organised
// around memory round trips rather than bytes: the weight chunks of the first row pass, the row scale,
// the bias and the residual value do not depend on the activations, so their loads are issued at the top
// of the kernel and are in flight while the prologue waits for the vector written by the previous kernel.
//
// Every (row, stream) result is a function of (k, storage type) only: the lane-group width, the
// per-lane chunk order and the reduction trees never depend on the batch size or on which streams
// are live, so a stream inside a batch is bit-identical to the same stream run alone
// (the contract of src/qmat.c:1107-1179).
#include <stdlib.h>

#include <stdlib.h>
#include <string.h>

#include "device_common.h"

namespace mynah {
namespace {

// Output row pointer of stream b (b < BT, not known at compile time): a select chain over the kernel arguments.
template <int BT>
__device__ __forceinline__ float *stream_out(const LinearArgs &a, int b) {
    float *o = a.out[0];
#pragma unroll
    for (int i = 1; i < BT; ++i)
        if (b == i) o = a.out[i];
    return o;
}

// KFIX: row length known at compile time (0 = taken from the arguments).  With it the lane-group width and the number of
// chunks per lane are constants, so the per-chunk range checks fold away and the weight requests are straight-line code;
// the two row lengths of the decoder stack (768 and 3072) get such a build.
// SPEC: what the launch is known not to use, so that the corresponding code is not there at all (0 = everything
// decided at run time).  SPEC_RESIDUAL: no LayerNorm, no bias, no probes, residual epilogue (the step's output and
// FFN-down projections; the fold source stays a run-time choice).  SPEC_UP: LayerNorm, no fold, no bias, no probes,
// GELU epilogue (the step's FFN-up projection).
enum { SPEC_ANY = 0, SPEC_RESIDUAL = 1, SPEC_UP = 2 };

// More than two streams with int8 / int4 weights: one wavefront stages one stream (load_stream_row / finish_stream_row,
// device_common.h) -- staging every stream's activations is what such a launch spends most of its time on, every workgroup
// has to do all of it, and a wavefront that owns a whole row needs no barrier and no exchange to normalise and quantise it.
// The workgroup has as many wavefronts as the batch tile has streams (at least four); the products then go to sets of four
// wavefronts, each set doing the matvec as the four wavefronts of a small-batch workgroup would for four of the streams.
// For f16 / f32 weights staging is a LayerNorm or a copy by the 256 threads together.
template <int BT, int QT>
constexpr bool kWaveStaging = BT > kConsumerFoldMaxBatch && kQuantised<QT>;
template <int BT, int QT>
constexpr int kLinearThreads = kWaveStaging<BT, QT> ? 64 * (BT > 4 ? BT : 4) : kThreads;

// The builds whose leading arguments are repacked (see the kernel): specialised ones, one or two streams.
template <int BT, int SPEC>
constexpr bool kPackedLead = BT <= 2 && SPEC != SPEC_ANY;
// The same for more streams, when the rows of a launch lie at a fixed stride (the step's workspaces do): the specialised
// builds that stage a stream per wavefront take two row pointers and two strides instead of sixteen row pointers.
template <int BT, int QT, int SPEC>
constexpr bool kStridedLead = kWaveStaging<BT, QT> && SPEC != SPEC_ANY;

// n:20 | rows per workgroup:12 | streams:4 | input stride / 4:14 | output stride / 4:14 (strides in floats)
struct StridedShape {
    int n, rows_per_wg, batch;
    size_t in_stride, out_stride;
};
__host__ __device__ inline bool strided_fits(const StridedShape &s) {
    return s.n >= 0 && s.n < (1 << 20) && s.rows_per_wg >= 0 && s.rows_per_wg < (1 << 12) && s.batch >= 0 && s.batch < 16 && s.in_stride % 4 == 0 &&
           s.in_stride / 4 < (1u << 14) && s.out_stride % 4 == 0 && s.out_stride / 4 < (1u << 14);
}
__host__ __device__ inline unsigned long long pack_strided(const StridedShape &s) {
    return (unsigned long long)s.n | ((unsigned long long)s.rows_per_wg << 20) | ((unsigned long long)s.batch << 32) |
           ((unsigned long long)(s.in_stride / 4) << 36) | ((unsigned long long)(s.out_stride / 4) << 50);
}
__device__ __forceinline__ StridedShape unpack_strided(const unsigned long long v) {
    StridedShape s;
    s.n = (int)(v & 0xfffffu); s.rows_per_wg = (int)((v >> 20) & 0xfffu); s.batch = (int)((v >> 32) & 0xfu);
    s.in_stride = (size_t)((v >> 36) & 0x3fffu) * 4; s.out_stride = (size_t)((v >> 50) & 0x3fffu) * 4;
    return s;
}
// rows of a launch at one stride (floats) from the first, or no stride at all
inline bool rows_strided(const LinearArgs &a, size_t *in_stride, size_t *out_stride) {
    *in_stride = *out_stride = 0;
    if (a.batch < 2) return true;
    if (a.in[1] < a.in[0] || a.out[1] < a.out[0]) return false;
    const size_t si = (size_t)(a.in[1] - a.in[0]), so = (size_t)(a.out[1] - a.out[0]);
    for (int b = 2; b < a.batch; ++b)
        if (a.in[b] != a.in[0] + (size_t)b * si || a.out[b] != a.out[0] + (size_t)b * so) return false;
    *in_stride = si; *out_stride = so;
    return true;
}

// The small numbers such a launch needs before its first request, in the 64 bits of one pointer argument.
struct LeadShape {
    int n, rows_per_wg, batch, folding, is_self, stream0, heads, max_units, head_width;
};
__host__ __device__ inline bool lead_fits(const LeadShape &s) {
    return s.n >= 0 && s.n < (1 << 20) && s.rows_per_wg >= 0 && s.rows_per_wg < (1 << 12) && s.batch >= 0 && s.batch < 16 && s.stream0 >= 0 && s.stream0 < 32 &&
           s.heads >= 0 && s.heads < 64 && s.max_units >= 0 && s.max_units < (1 << 11) && s.head_width >= 0 && s.head_width % 64 == 0 && s.head_width / 64 < 16;
}
__host__ __device__ inline unsigned long long pack_lead(const LeadShape &s) {
    return (unsigned long long)s.n | ((unsigned long long)s.rows_per_wg << 20) | ((unsigned long long)s.batch << 32) | ((unsigned long long)(s.folding & 1) << 36) |
           ((unsigned long long)(s.is_self & 1) << 37) | ((unsigned long long)s.stream0 << 38) | ((unsigned long long)s.heads << 43) |
           ((unsigned long long)s.max_units << 49) | ((unsigned long long)(s.head_width / 64) << 60);
}
__device__ __forceinline__ LeadShape unpack_lead(const unsigned long long v) {
    LeadShape s;
    s.n = (int)(v & 0xfffffu); s.rows_per_wg = (int)((v >> 20) & 0xfffu); s.batch = (int)((v >> 32) & 0xfu); s.folding = (int)((v >> 36) & 1u);
    s.is_self = (int)((v >> 37) & 1u); s.stream0 = (int)((v >> 38) & 0x1fu); s.heads = (int)((v >> 43) & 0x3fu); s.max_units = (int)((v >> 49) & 0x7ffu);
    s.head_width = (int)((v >> 60) & 0xfu) * 64;
    return s;
}

template <int QT, int BT, int NVT, int KFIX, int SPEC>
__global__ void __launch_bounds__((kLinearThreads<BT, QT>))
k_linear(const float *const in0, const float *const fold_partial, const float *const fold_partial_ml, const StepSlots *const fold_slots,
         const void *const w, const float *const scales, float *const out0, const int n, const int batch, const LinearArgs a_arg,
         const int rows_per_wg_arg, const int lg_arg) {
    // The seven pointers and two counts in front repeat fields of a_arg: the first sixteen dwords of the kernel arguments are
    // in registers when a wavefront starts (the build asks for that), the structure behind them is fetched from memory, and
    // these are what the first requests are formed from.
    // (Only for one or two streams: with more, the rows of a.in and a.out are picked by a run-time index, and a structure that
    // has been written to is then kept in scratch memory -- the eight-stream matvecs took 20 us instead of 4.5.)
    static_assert(64 + sizeof(LinearArgs) > 0x100 + 4, "the warmed lines lie inside the kernel arguments");
    constexpr bool kStrided = kStridedLead<BT, QT, SPEC>;
    WarmArguments warm{0u, 0u, 0u, 0u};
    if constexpr (BT <= 2 || kStrided) warm = warm_kernel_arguments<4>();
    LinearArgs a = a_arg;
    int rows_per_wg = rows_per_wg_arg;
    size_t in_stride = 0, out_stride = 0;   // (strided builds: rows b of the launch are in0 + b * in_stride, out0 + b * out_stride)
    // Strided builds: the grid's second dimension names a group of BT streams (launch_linear_t): five to eight streams run as
    // two groups of four side by side, each workgroup staging four rows instead of eight.
    const float *in_base = in0;
    float *out_base = out0;
    if constexpr (kStrided) {
        // As for one or two streams below: what the first requests are formed from arrives in the fourteen dwords that are in
        // registers at wavefront start -- first rows, weights, scales, the LayerNorm vectors in the two places that carry fold
        // arguments for fewer streams, every small number in the slot table pointer's place (pack_strided).
        const StridedShape shape = unpack_strided(reinterpret_cast<unsigned long long>(fold_slots));
        a.w = w; a.scales = scales; a.n = shape.n;
        rows_per_wg = shape.rows_per_wg;
        in_stride = shape.in_stride; out_stride = shape.out_stride;
        const int first_stream = (int)blockIdx.y * BT;
        a.batch = min(BT, shape.batch - first_stream);
        in_base = in0 + (size_t)first_stream * in_stride;
        out_base = out0 + (size_t)first_stream * out_stride;
        a.fold_partial = nullptr; a.fold_partial_ml = nullptr; a.fold_slots = nullptr;
        a.fold_heads = 0; a.fold_head_width = 0; a.fold_max_units = 0; a.fold_is_self = 0; a.fold_stream0 = 0;
        if constexpr (SPEC == SPEC_UP) {
            a.ln_gain = fold_partial; a.ln_bias = fold_partial_ml;
        }
    }
    if constexpr (kPackedLead<BT, SPEC>) {
        // Fourteen dwords of arguments -- the seven pointers -- are in registers at wavefront start; n, batch, the structure and
        // rows_per_wg_arg come out of memory, a round trip that stood in front of the first request.  The specialised builds for
        // one or two streams never use all seven pointers at once, so the launch (pack_lead) passes in the free places what
        // the first requests are formed from: LayerNorm vectors where nothing is folded, the slot table's address in the place
        // of the unused input row where something is, and every small number in the place of the slot table's pointer.
        const LeadShape shape = unpack_lead(reinterpret_cast<unsigned long long>(fold_slots));
        a.w = w; a.scales = scales; a.out[0] = out0; a.n = shape.n; a.batch = shape.batch;
        rows_per_wg = shape.rows_per_wg;
        a.fold_partial = nullptr; a.fold_partial_ml = nullptr; a.fold_slots = nullptr;
        a.in[0] = in0;   // (never read as a row when something is folded)
        // assigned whatever the case, so that no field of the structure in memory is asked for on their account
        a.fold_heads = shape.heads; a.fold_head_width = shape.head_width; a.fold_max_units = shape.max_units;
        a.fold_is_self = shape.is_self; a.fold_stream0 = shape.stream0;
        if constexpr (SPEC == SPEC_UP) {
            a.ln_gain = fold_partial; a.ln_bias = fold_partial_ml;
        } else {
            if (shape.folding) {
                a.fold_partial = fold_partial; a.fold_partial_ml = fold_partial_ml; a.fold_slots = reinterpret_cast<const StepSlots *>(in0);
            }
        }
    } else if constexpr (BT <= 2) {
        a.in[0] = in0; a.fold_partial = fold_partial; a.fold_partial_ml = fold_partial_ml; a.fold_slots = fold_slots;
        a.w = w; a.scales = scales; a.out[0] = out0; a.n = n; a.batch = batch;
    }
    // a one-stream build is launched for exactly one stream (launch_linear_b): its first request then depends on no argument
    // that comes out of memory (n and batch are the fifteenth and sixteenth dword, one past what is in registers at start)
    if constexpr (BT == 1) a.batch = 1;
    constexpr bool kWaves = kWaveStaging<BT, QT>;   // a wavefront per stream (see above); otherwise the 256 threads stage every stream together
    // The kernel arguments that the first requests are formed from, fetched here in one go: left to the compiler each is
    // fetched where it is first used, with a wait of its own, and three such round trips stood in a row in front of the
    // first request for an activation row.
    // (One or two streams: only what the first requests are formed from -- fetching every argument first delays them.
    // More streams: the eight row pointers of a.in and a.out as one operand each, or they are fetched in rounds of their own.)
    if constexpr (BT > 2 && !kStrided) {
        typedef unsigned row_pointers __attribute__((ext_vector_type(2 * BT)));
        const row_pointers ins = *reinterpret_cast<const row_pointers *>(&a.in[0]), outs = *reinterpret_cast<const row_pointers *>(&a.out[0]);
        __asm__ volatile("" ::"s"(a.w), "s"(a.scales), "s"(ins), "s"(outs), "s"(a.fold_partial), "s"(a.fold_partial_ml), "s"(a.fold_slots),
                         "s"(a.ln_gain), "s"(a.ln_bias), "s"(a.n), "s"(a.k), "s"(a.batch), "s"(a.fold_heads), "s"(a.fold_head_width),
                         "s"(a.fold_max_units), "s"(a.fold_is_self), "s"(a.fold_stream0), "s"(rows_per_wg), "s"(a.arith), "s"(a.epilogue));
    }
    const Team team = whole_workgroup();
    // Products.  A workgroup's rows go to four wavefronts (wave_row); where the stream-per-wavefront builds have eight, the
    // second four take the same rows for the upper half of the streams: PB streams per wavefront, from stream_base on.  Every
    // wavefront works, so no request stands under a condition.
    constexpr int PB = (kWaves && BT > 4) ? BT / 2 : BT;
    static_assert(!kWaves || kLinearThreads<BT, QT> == kThreads * (BT / PB), "one set of four wavefronts per PB streams");
    // the arguments a specialised build does not look at
    const float *const arg_bias = SPEC != SPEC_ANY ? nullptr : a.bias;
    int8_t *const arg_probe_qx = SPEC != SPEC_ANY ? nullptr : a.probe_qx;
    float *const arg_probe_sx = SPEC != SPEC_ANY ? nullptr : a.probe_sx;
    int32_t *const arg_probe_acc = SPEC != SPEC_ANY ? nullptr : a.probe_acc;
    float *const arg_aux_out = SPEC != SPEC_ANY ? nullptr : a.aux_out;
    const int arg_epilogue = SPEC == SPEC_UP ? EPI_GELU : SPEC == SPEC_RESIDUAL ? EPI_RESIDUAL : a.epilogue;
    const float *const arg_ln_gain = SPEC == SPEC_RESIDUAL ? nullptr : a.ln_gain;
    const float *const arg_ln_bias = SPEC == SPEC_RESIDUAL ? nullptr : a.ln_bias;
    const float *const arg_fold_partial = (SPEC == SPEC_UP || BT > kConsumerFoldMaxBatch) ? nullptr : a.fold_partial;   // larger batches fold in a kernel of their own
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float s_sx[BT];
    __shared__ float s_scratch[kPrologueScratch * BT];
    constexpr int kEpc = Chunk<QT>::n;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    // (constants where the workgroup has four wavefronts, so that the small-batch builds are the code they were)
    const int wave_row = PB != BT ? (wave & 3) : wave;
    const int stream_base = PB != BT ? __builtin_amdgcn_readfirstlane(wave >> 2) * PB : 0;
    const int k = KFIX != 0 ? KFIX : a.k;
    const int lg = KFIX != 0 ? lane_group_log2(KFIX / kEpc) : lg_arg;

    const int G = 1 << lg;
    const int gl = lane & (G - 1);
    const int gidx = lane >> lg;
    const int rows_per_pass = 64 >> lg;
    const int chunks = k / kEpc;
    const int row_begin = blockIdx.x * rows_per_wg;
    const int row_end = min(a.n, row_begin + rows_per_wg);
    const size_t row_bytes = (size_t)chunks * 16;
    const int pass_stride = 4 * rows_per_pass;

    // ------------------------------------------------------------------ activation rows first: the prologue's arithmetic
    // waits for these only, so it runs while the weight rows requested after them are still on their way
    PrologueParams pro;
    pro.k = k; pro.batch = a.batch; pro.ln_gain = arg_ln_gain; pro.ln_bias = arg_ln_bias; pro.arith = a.arith;
    pro.probe_qx = arg_probe_qx; pro.probe_sx = arg_probe_sx;
    pro.ln_out = SPEC != SPEC_ANY ? nullptr : a.ln_out;
    pro.ln_out_slots = SPEC != SPEC_ANY ? nullptr : a.ln_out_slots;
    pro.act_out = SPEC != SPEC_ANY ? nullptr : a.act_out;
    constexpr int XB = kWaves ? 1 : BT, XN = kWaves ? 4 * NVT : NVT;
    float4 xr[XB][XN], gv[XN], bv[XN];
    const int stream = __builtin_amdgcn_readfirstlane(wave);   // a wavefront's stream is its index (the same for all of its lanes)
    const bool live = !kWaves || stream < a.batch;
    // output row of stream b
    const auto out_of = [&](const int b) -> float * {
        if constexpr (kStrided) return out_base + (size_t)b * out_stride;
        else return stream_out<BT>(a, b);
    };
    if constexpr (kWaves) {
        const float *row = kStrided ? in_base : a.in[0];   // a place of the tile without a stream reads stream 0's row and stages zeros
        if constexpr (kStrided) {
            if (live) row = in_base + (size_t)stream * in_stride;
        } else {
#pragma unroll
            for (int q = 1; q < BT; ++q)
                if (stream == q && q < a.batch) row = a.in[q];   // (select chain over the kernel arguments)
        }
        load_stream_row<NVT>(pro, row, live, lane, xr[0], gv, bv);
    } else {
        ActSource src;
#pragma unroll
        for (int b = 0; b < kBatchTile; ++b) src.rows[b] = a.in[b < BT ? b : 0];
        src.partial = arg_fold_partial; src.partial_ml = a.fold_partial_ml; src.slots = a.fold_slots; src.heads = a.fold_heads; src.head_width = a.fold_head_width;
        src.max_units = a.fold_max_units; src.is_self = a.fold_is_self; src.stream0 = a.fold_stream0;
        load_activations<BT, NVT>(pro, src, team, xr, gv, bv);
    }
    requests_issued();

    // ------------------------------------------------------------------ loads that need no activation
    uint4 wv[4];
    float sc[4];
    float pre_scale = 1.0f, pre_bias = 0.0f, pre_res[PB];
#pragma unroll
    for (int b = 0; b < PB; ++b) pre_res[b] = 0.0f;
    const bool lanes_finish = BT > 1 && G >= PB;
    {
        const int row = row_begin + wave_row * rows_per_pass + gidx;
        const int rowc = row < row_end ? row : row_end - 1;
        const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(a.w) + (size_t)rowc * row_bytes);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = gl + u * G;
            wv[u] = c < chunks ? wrow[c] : make_uint4(0, 0, 0, 0);
            sc[u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? a.scales[(size_t)rowc * chunks + c] : 0.0f;
        }
        // Epilogue operands.  One stream: lane 0 of a group finishes the row.  Several streams: lane b of a group
        // finishes stream b (when the group has that many lanes), so the epilogues of a row run side by side.
        // Requested by every lane, whichever of them finishes the row: a request under a per-lane condition cannot be
        // counted by the waits that follow, and the prologue's wait for the activation rows then also waited for the
        // first weight pieces.  (Lanes of a group ask for the same address; the conditions left are the same for the
        // whole launch.)
        if (lanes_finish) {
            if constexpr (QT == MYNAH_HIP_INT8) pre_scale = a.scales[rowc];
            if (arg_bias != nullptr) pre_bias = arg_bias[rowc];
            if (arg_epilogue == EPI_RESIDUAL) pre_res[0] = out_of(stream_base + gl < a.batch ? stream_base + gl : 0)[rowc];
        } else {
            if constexpr (QT == MYNAH_HIP_INT8) pre_scale = a.scales[rowc];
            if (arg_bias != nullptr) pre_bias = arg_bias[rowc];
#pragma unroll
            for (int b = 0; b < PB; ++b) pre_res[b] = (arg_epilogue == EPI_RESIDUAL && stream_base + b < a.batch) ? out_of(stream_base + b)[rowc] : 0.0f;
        }
    }

    // The stream-group builds (strided rows, residual epilogue) may be launched with two row passes per workgroup: the second
    // pass's first weight group and its epilogue operands are requested here as well -- asked for inside the row loop they
    // are two dependent round trips behind the first pass's products.  Requested whatever the launch (rows past the
    // workgroup's range repeat its last row): a request under a condition could not be counted by the waits below.
    // (not in the build for rows of 768: the stack's output projections, whose 48 row blocks never need a second pass)
    constexpr bool kSecondAhead = kStrided && SPEC == SPEC_RESIDUAL && KFIX != 768;
    uint4 wv_second[kSecondAhead ? 4 : 1];
    float sc_second[kSecondAhead ? 4 : 1];
    float scale_second = 1.0f, res_second[kSecondAhead ? PB : 1];
    if constexpr (kSecondAhead) {
        const int row = row_begin + pass_stride + wave_row * rows_per_pass + gidx;
        const int rowc = row < row_end ? row : row_end - 1;
        const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(a.w) + (size_t)rowc * row_bytes);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = gl + u * G;
            wv_second[u] = c < chunks ? wrow[c] : make_uint4(0, 0, 0, 0);
            sc_second[u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? a.scales[(size_t)rowc * chunks + c] : 0.0f;
        }
        if constexpr (QT == MYNAH_HIP_INT8) scale_second = a.scales[rowc];
        if (lanes_finish) {
            res_second[0] = out_of(stream_base + gl < a.batch ? stream_base + gl : 0)[rowc];
        } else {
#pragma unroll
            for (int b = 0; b < PB; ++b) res_second[b] = stream_base + b < a.batch ? out_of(stream_base + b)[rowc] : 0.0f;
        }
    }

    requests_issued();

    // ------------------------------------------------------------------ prologue arithmetic (the weight requests above stay in flight)
    if constexpr (kWaves) {
        finish_stream_row<QT, NVT>(pro, stream, live, lane, xr[0], gv, bv, smem, s_sx);
        __syncthreads();
    } else {
        finish_activations<QT, BT, NVT>(pro, team, xr, gv, bv, smem, s_sx, s_scratch);
    }
    release_warm(warm);

    // ------------------------------------------------------------------ body
    bool first = true;
    bool second = false;   // (stream-group builds) the pass whose operands were requested ahead as well
    const unsigned char *const staged = smem + (size_t)stream_base * k * (kQuantised<QT> ? 1 : 4);   // this wavefront's streams
    for (int base = row_begin + wave_row * rows_per_pass; base < row_end; base += pass_stride) {
        const int row = base + gidx;
        const bool valid = row < row_end;
        const int rowc = valid ? row : row_end - 1;
        const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(a.w) + (size_t)rowc * row_bytes);
        int iacc[PB];
        float facc[PB];
#pragma unroll
        for (int b = 0; b < PB; ++b) { iacc[b] = 0; facc[b] = 0.0f; }
        for (int c0 = gl; c0 < chunks; c0 += 4 * G) {
            if (kSecondAhead && second && c0 == gl) {
#pragma unroll
                for (int u = 0; u < 4; ++u) { wv[u] = wv_second[kSecondAhead ? u : 0]; sc[u] = sc_second[kSecondAhead ? u : 0]; }
            } else if (!(first && c0 == gl)) {   // the first group of the first pass was loaded before the prologue
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int c = c0 + u * G;
                    wv[u] = c < chunks ? wrow[c] : make_uint4(0, 0, 0, 0);
                    sc[u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? a.scales[(size_t)rowc * chunks + c] : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u * G;
                if (c < chunks) {
                    int group_int = 0;
                    dot_chunk<QT, PB>(wv[u], sc[u], c, staged, k, iacc, facc, &group_int);
                    if (QT == MYNAH_HIP_INT4 && arg_probe_acc != nullptr && valid && stream_base == 0) arg_probe_acc[(size_t)row * chunks + c] = group_int;
                }
            }
        }
        group_reduce<QT, PB>(iacc, facc, lg);
        if (lanes_finish) {
            const int sb = stream_base + gl;   // the stream this lane finishes
            if (gl < PB && sb < a.batch && valid) {
                int mi = iacc[0];
                float mf = facc[0];
#pragma unroll
                for (int b = 1; b < PB; ++b)
                    if (gl == b) { mi = iacc[b]; mf = facc[b]; }
                float wscale = 1.0f, bias = 0.0f;
                if (first) {
                    wscale = pre_scale;
                    bias = pre_bias;
                } else if (kSecondAhead && second) {
                    wscale = scale_second;
                } else {
                    if constexpr (QT == MYNAH_HIP_INT8) wscale = a.scales[row];
                    if (arg_bias != nullptr) bias = arg_bias[row];
                }
                float val = finish_value<QT>(mi, mf, wscale, s_sx[sb]);
                if (QT == MYNAH_HIP_INT8 && arg_probe_acc != nullptr && sb == 0) arg_probe_acc[row] = mi;
                if (arg_bias != nullptr) val += bias;
                if (arg_epilogue == EPI_GELU) val = gelu_tanh(val);
                float *o = out_of(sb) + row;
                if (arg_aux_out != nullptr && sb == 0) arg_aux_out[row] = val;
                if (arg_epilogue == EPI_RESIDUAL) val = (first ? pre_res[0] : (kSecondAhead && second) ? res_second[0] : *o) + val;
                *o = val;
            }
        } else if (gl == 0 && valid) {
            float wscale = 1.0f, bias = 0.0f;
            if (first) {
                wscale = pre_scale;
                bias = pre_bias;
            } else if (kSecondAhead && second) {
                wscale = scale_second;
            } else {
                if constexpr (QT == MYNAH_HIP_INT8) wscale = a.scales[row];
                if (arg_bias != nullptr) bias = arg_bias[row];
            }
#pragma unroll
            for (int b = 0; b < PB; ++b) {
                const int sb = stream_base + b;
                if (sb < a.batch) {
                    float val = finish_value<QT>(iacc[b], facc[b], wscale, s_sx[sb]);
                    if (QT == MYNAH_HIP_INT8 && arg_probe_acc != nullptr && sb == 0) arg_probe_acc[row] = iacc[b];
                    if (arg_bias != nullptr) val += bias;
                    if (arg_epilogue == EPI_GELU) val = gelu_tanh(val);
                    float *o = out_of(sb) + row;
                    if (arg_aux_out != nullptr && sb == 0) arg_aux_out[row] = val;
                    if (arg_epilogue == EPI_RESIDUAL) val = (first ? pre_res[b] : (kSecondAhead && second) ? res_second[kSecondAhead ? b : 0] : *o) + val;
                    *o = val;
                }
            }
        }
        second = first;   // the pass behind the first
        first = false;
    }
}

// ---------------------------------------------------------------------------------------------
// Generic f32 kernels for shapes the fused matvec does not take (tiny KAT shapes, rows > 16).
// out[r, col] = sum_p in[r,p] * w[col,p] + bias[col]; 16x16 output tile, K tiled through LDS.
__global__ void __launch_bounds__(256) k_gemm_nt_f32(const float *__restrict__ in, const float *__restrict__ w,
                                                     const float *__restrict__ bias, float *__restrict__ out,
                                                     int rows, int k, int n) {
    __shared__ float sa[16][17];
    __shared__ float sb[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int r = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
    float acc = 0.0f;
    for (int p0 = 0; p0 < k; p0 += 16) {
        const int pa = p0 + tx;
        sa[ty][tx] = (r < rows && pa < k) ? in[(size_t)r * k + pa] : 0.0f;
        const int wr = blockIdx.x * 16 + ty;
        sb[ty][tx] = (wr < n && pa < k) ? w[(size_t)wr * k + pa] : 0.0f;
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 16; ++p) acc = __builtin_fmaf(sa[ty][p], sb[tx][p], acc);
        __syncthreads();
    }
    if (r < rows && col < n) out[(size_t)r * n + col] = acc + (bias != nullptr ? bias[col] : 0.0f);
}

// Row-major C = alpha * op(A) op(B) + beta * C  (src/backend.h:15-25), one thread per output.
__global__ void __launch_bounds__(256) k_sgemm(int ta, int tb, int m, int n, int k, float alpha, const float *__restrict__ a,
                                               int lda, const float *__restrict__ b, int ldb, float beta,
                                               float *__restrict__ c, int ldc) {
    const int j = blockIdx.x * 16 + (threadIdx.x & 15);
    const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
    if (i >= m || j >= n) return;
    float sum = 0.0f;
    for (int p = 0; p < k; ++p) {
        const float av = ta ? a[(size_t)p * lda + i] : a[(size_t)i * lda + p];
        const float bv = tb ? b[(size_t)j * ldb + p] : b[(size_t)p * ldb + j];
        sum = __builtin_fmaf(av, bv, sum);
    }
    float *dst = c + (size_t)i * ldc + j;
    *dst = beta == 0.0f ? alpha * sum : alpha * sum + beta * *dst;
}

// The same products for many rows, on the matrix cores: C[m][n] = alpha * sum_k A[m][k] * B(n, k) + beta * C[m][n] + bias[n],
// A row-major with row stride lda; TB = 1: B[n][k] (both operands K-contiguous, "NT" -- the seam's matmul and its scores
// Q K^T), TB = 0: B[k][n] ("NN" -- P V).  f32 in, f32 multiply-add (v_mfma_f32_32x32x2_f32: lane l supplies row l % 32 and
// k l / 32 of each operand), so the result differs from a serial sum only in the order of the additions.
// Workgroup tile 64 x 64, a wavefront 32 x 32; K in steps of 32 through LDS (rows padded to 33 floats: the 32 rows a
// wavefront reads fall into 32 banks).  The next step's operands are requested before the current step's products and
// stored after them.  VEC: rows are whole aligned float4s (strides and K multiples of 4, 16-byte bases); otherwise the
// staging is scalar with the same bounds.  Rows and columns past the matrix are staged as zeros and not written.
constexpr int kGemmTile = 64, kGemmStep = 32, kGemmPad = 33;

template <int TB, int VEC>
__global__ void __launch_bounds__(256) k_gemm_f32_mfma(const float *__restrict__ A, int lda, const float *__restrict__ B, int ldb, float *__restrict__ C,
                                                       int ldc, int M, int N, int K, float alpha, float beta, const float *__restrict__ bias) {
    typedef float floatx16 __attribute__((ext_vector_type(16)));
    __shared__ float s_a[kGemmTile * kGemmPad];
    __shared__ float s_b[kGemmTile * kGemmPad];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    const int m0 = blockIdx.y * kGemmTile, n0 = blockIdx.x * kGemmTile;

    // staging slots.  K-contiguous operand (A, and B when TB): rows r and r + 32, four k from 4 * (tid % 8).
    // N-contiguous operand (B when !TB): k rows kr and kr + 16, four n from 4 * (tid % 16).
    const int kr = tid >> 3, kc = (tid & 7) * 4;
    const int nr = tid >> 4, nc = (tid & 15) * 4;
    float4 ra[2], rb[2];
    const auto fetch_k_major = [&](const float *base, int ld, int row, int rows, int k0) -> float4 {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row < rows) {
            const float *p = base + (size_t)row * ld + k0;
            if (VEC && k0 + 3 < K) v = *reinterpret_cast<const float4 *>(p);
            else {
                if (k0 < K) v.x = p[0];
                if (k0 + 1 < K) v.y = p[1];
                if (k0 + 2 < K) v.z = p[2];
                if (k0 + 3 < K) v.w = p[3];
            }
        }
        return v;
    };
    const auto fetch_n_major = [&](int k, int n) -> float4 {   // B[k][n .. n + 3]
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < K) {
            const float *p = B + (size_t)k * ldb + n;
            if (VEC && n + 3 < N) v = *reinterpret_cast<const float4 *>(p);
            else {
                if (n < N) v.x = p[0];
                if (n + 1 < N) v.y = p[1];
                if (n + 2 < N) v.z = p[2];
                if (n + 3 < N) v.w = p[3];
            }
        }
        return v;
    };
    const auto request = [&](int k0) {
        ra[0] = fetch_k_major(A, lda, m0 + kr, M, k0 + kc);
        ra[1] = fetch_k_major(A, lda, m0 + kr + 32, M, k0 + kc);
        if constexpr (TB) {
            rb[0] = fetch_k_major(B, ldb, n0 + kr, N, k0 + kc);
            rb[1] = fetch_k_major(B, ldb, n0 + kr + 32, N, k0 + kc);
        } else {
            rb[0] = fetch_n_major(k0 + nr, n0 + nc);
            rb[1] = fetch_n_major(k0 + nr + 16, n0 + nc);
        }
    };
    const auto stage = [&]() {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float *pa = s_a + (kr + 32 * h) * kGemmPad + kc;
            pa[0] = ra[h].x; pa[1] = ra[h].y; pa[2] = ra[h].z; pa[3] = ra[h].w;
            if constexpr (TB) {
                float *pb = s_b + (kr + 32 * h) * kGemmPad + kc;
                pb[0] = rb[h].x; pb[1] = rb[h].y; pb[2] = rb[h].z; pb[3] = rb[h].w;
            } else {
                float *pb = s_b + nc * kGemmPad + nr + 16 * h;   // transposed: s_b[n][k]
                pb[0] = rb[h].x; pb[kGemmPad] = rb[h].y; pb[2 * kGemmPad] = rb[h].z; pb[3 * kGemmPad] = rb[h].w;
            }
        }
    };

    floatx16 acc = {0};
    const float *fa = s_a + (wm * 32 + (lane & 31)) * kGemmPad + (lane >> 5);
    const float *fb = s_b + (wn * 32 + (lane & 31)) * kGemmPad + (lane >> 5);
    request(0);
    for (int k0 = 0; k0 < K; k0 += kGemmStep) {
        __syncthreads();   // the products of the step before have read the tiles
        stage();
        __syncthreads();
        if (k0 + kGemmStep < K) request(k0 + kGemmStep);
#pragma unroll
        for (int s2 = 0; s2 < kGemmStep / 2; ++s2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[2 * s2], fb[2 * s2], acc, 0, 0, 0);
    }
    const int n = n0 + wn * 32 + (lane & 31);
    if (n >= N) return;
    const float add = bias != nullptr ? bias[n] : 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);   // row of accumulator register r
        if (m < M) {
            float *dst = C + (size_t)m * ldc + n;
            const float v = alpha * acc[r] + add;
            *dst = beta == 0.0f ? v : v + beta * *dst;
        }
    }
}

static bool gemm_vec_ok(const float *a, size_t lda, const float *b, size_t ldb, size_t k, size_t inner_b) {
    return (reinterpret_cast<uintptr_t>(a) % 16 == 0) && (reinterpret_cast<uintptr_t>(b) % 16 == 0) && lda % 4 == 0 && ldb % 4 == 0 && k % 4 == 0 &&
           inner_b % 4 == 0;
}

// MYNAH_HIP_STREAM_GROUPS=0: five to eight streams as one tile of eight again
static bool stream_groups_enabled() {
    static const bool on = !(getenv("MYNAH_HIP_STREAM_GROUPS") != nullptr && strcmp(getenv("MYNAH_HIP_STREAM_GROUPS"), "0") == 0);
    return on;
}

template <int QT, int BT, int NVT, int KFIX, int SPEC>
int launch_linear_t(State *st, const LinearArgs &a, char *error, size_t capacity) {
    constexpr int epc = Chunk<QT>::n;
    const int chunks = a.k / epc;
    const int lg = lane_group_log2(chunks);
    const int rows_per_wg_pass = 4 * (64 >> lg);
    const int target_wgs = st->cu_count * 3;
    int passes = (a.n + rows_per_wg_pass * target_wgs - 1) / (rows_per_wg_pass * target_wgs);
    if (passes < 1) passes = 1;
    // strided builds take more streams than their tile holds as groups of BT side by side (the grid's second dimension);
    // with twice the rows per workgroup when the groups together would otherwise be more workgroups than the chip has CUs
    const int groups = kStridedLead<BT, QT, SPEC> ? (a.batch + BT - 1) / BT : 1;
    if (groups > 1 && (long)((a.n + rows_per_wg_pass * passes - 1) / (rows_per_wg_pass * passes)) * groups > st->cu_count) passes *= 2;
    const int rows_per_wg = rows_per_wg_pass * passes;
    const int grid = (a.n + rows_per_wg - 1) / rows_per_wg;
    const size_t lds = (size_t)BT * a.k * (kQuantised<QT> ? 1 : 4);
    static bool raised = false;   // per instantiation
    if (lds > 48 * 1024 && !raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_linear<QT, BT, NVT, KFIX, SPEC>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        raised = true;
    }
    if constexpr (kStridedLead<BT, QT, SPEC>) {
        StridedShape shape{};
        shape.n = a.n; shape.rows_per_wg = rows_per_wg; shape.batch = a.batch;
        if (!rows_strided(a, &shape.in_stride, &shape.out_stride) || !strided_fits(shape)) {   // launch_linear_q sends such launches to the general build; this is the backstop
            set_error(error, capacity, "linear: rows do not fit the strided launch arguments");
            return -1;
        }
        const StepSlots *const packed = reinterpret_cast<const StepSlots *>(pack_strided(shape));
        hipLaunchKernelGGL((k_linear<QT, BT, NVT, KFIX, SPEC>), dim3(grid, groups), dim3(kLinearThreads<BT, QT>), lds, st->stream, a.in[0],
                           SPEC == SPEC_UP ? a.ln_gain : nullptr, SPEC == SPEC_UP ? a.ln_bias : nullptr, packed, a.w, a.scales, a.out[0], a.n, a.batch, a,
                           rows_per_wg, lg);
    } else if constexpr (kPackedLead<BT, SPEC>) {
        // the launch's small numbers in the slot table pointer's place, and what the free pointer places carry (see the kernel)
        LeadShape shape{};
        shape.n = a.n; shape.rows_per_wg = rows_per_wg; shape.batch = a.batch;
        const bool folding = SPEC == SPEC_RESIDUAL && a.fold_partial != nullptr;
        if (folding) {
            shape.folding = 1; shape.is_self = a.fold_is_self; shape.stream0 = a.fold_stream0; shape.heads = a.fold_heads;
            shape.max_units = a.fold_max_units; shape.head_width = a.fold_head_width;
        }
        if (!lead_fits(shape)) {   // launch_linear_q sends what does not fit to the general build; this is the backstop
            set_error(error, capacity, "linear: shape does not fit the packed launch arguments");
            return -1;
        }
        const StepSlots *const packed = reinterpret_cast<const StepSlots *>(pack_lead(shape));
        const float *lead0 = a.in[0], *lead1 = nullptr, *lead2 = nullptr;
        if (SPEC == SPEC_UP) { lead1 = a.ln_gain; lead2 = a.ln_bias; }
        else if (folding) { lead0 = reinterpret_cast<const float *>(a.fold_slots); lead1 = a.fold_partial; lead2 = a.fold_partial_ml; }
        hipLaunchKernelGGL((k_linear<QT, BT, NVT, KFIX, SPEC>), dim3(grid), dim3(kLinearThreads<BT, QT>), lds, st->stream, lead0, lead1, lead2, packed,
                           a.w, a.scales, a.out[0], a.n, a.batch, a, rows_per_wg, lg);
    } else {
        hipLaunchKernelGGL((k_linear<QT, BT, NVT, KFIX, SPEC>), dim3(grid), dim3(kLinearThreads<BT, QT>), lds, st->stream, a.in[0], a.fold_partial,
                           a.fold_partial_ml, a.fold_slots, a.w, a.scales, a.out[0], a.n, a.batch, a, rows_per_wg, lg);
    }
    return hip_check(hipGetLastError(), "linear launch", error, capacity);
}

template <int QT, int NVT, int KFIX, int SPEC>
int launch_linear_b(State *st, const LinearArgs &a, char *error, size_t capacity) {
    if (a.batch <= 1) return launch_linear_t<QT, 1, NVT, KFIX, SPEC>(st, a, error, capacity);
    if (a.batch == 2) return launch_linear_t<QT, 2, NVT, KFIX, SPEC>(st, a, error, capacity);
    if (a.batch <= 4) return launch_linear_t<QT, 4, NVT, KFIX, SPEC>(st, a, error, capacity);
    // five to eight streams, rows at a fixed stride, int8 / int4 weights, residual epilogue (the output projections and the
    // FFN-down product): two groups of four in one launch -- what a workgroup stages, every stream of its tile, halves, and a
    // stream's bits do not depend on the tile it runs in.  (Measured with eight ragged streams: step 497 -> 483 us; the FFN-up
    // product the same way, whose LayerNorm prologue each group then runs for its four rows, 497 us with twice the rows per
    // workgroup and 486 us with twice the workgroups; with the second pass's operands requested ahead as below, 476 against 477 us:
    // it keeps the tile of eight.)
    if (kStridedLead<4, QT, SPEC> && SPEC == SPEC_RESIDUAL && stream_groups_enabled()) return launch_linear_t<QT, 4, NVT, KFIX, SPEC>(st, a, error, capacity);
    return launch_linear_t<QT, 8, NVT, KFIX, SPEC>(st, a, error, capacity);
}

template <int QT>
int launch_linear_q(State *st, const LinearArgs &a, char *error, size_t capacity) {
    // what the arguments rule out decides the build (see SPEC above)
    const bool plain = a.bias == nullptr && a.probe_qx == nullptr && a.probe_sx == nullptr && a.probe_acc == nullptr &&
                       a.ln_out == nullptr && a.ln_out_slots == nullptr && a.aux_out == nullptr && a.act_out == nullptr;
    // (the specialised builds for one or two streams take their small numbers packed into one argument: when one of them
    // does not fit its bit field the launch takes the general build, with the same arithmetic)
    LeadShape fit{};
    fit.n = a.n; fit.batch = a.batch; fit.rows_per_wg = 2048;   // above what launch_linear_t chooses for any n that fits (256 rows per 196,608 of n)
    if (a.fold_partial != nullptr) {
        fit.is_self = a.fold_is_self; fit.stream0 = a.fold_stream0; fit.heads = a.fold_heads; fit.max_units = a.fold_max_units; fit.head_width = a.fold_head_width;
    }
    bool packs = lead_fits(fit);
    if (a.batch > 2) {   // more streams: the specialised builds of quantised weights take rows at a fixed stride
        StridedShape strided{};
        strided.n = a.n; strided.batch = a.batch; strided.rows_per_wg = 2048;
        packs = !kQuantised<QT> || (rows_strided(a, &strided.in_stride, &strided.out_stride) && strided_fits(strided));
    }
    const bool residual = plain && packs && a.epilogue == EPI_RESIDUAL && a.ln_gain == nullptr;
    const bool up = plain && packs && a.epilogue == EPI_GELU && a.ln_gain != nullptr && a.fold_partial == nullptr;
    if (a.k == 768) {
        if (residual) return launch_linear_b<QT, 1, 768, SPEC_RESIDUAL>(st, a, error, capacity);
        if (up) return launch_linear_b<QT, 1, 768, SPEC_UP>(st, a, error, capacity);
        return launch_linear_b<QT, 1, 768, SPEC_ANY>(st, a, error, capacity);
    }
    if (a.k == 3072) {
        if (residual) return launch_linear_b<QT, 3, 3072, SPEC_RESIDUAL>(st, a, error, capacity);
        return launch_linear_b<QT, 3, 3072, SPEC_ANY>(st, a, error, capacity);
    }
    if (a.k <= 1024) return launch_linear_b<QT, 1, 0, SPEC_ANY>(st, a, error, capacity);
    return launch_linear_b<QT, 3, 0, SPEC_ANY>(st, a, error, capacity);
}

}  // namespace

bool linear_fast_supported(int qtype, size_t n, size_t k) {
    if (n == 0 || k == 0 || n > 0x7fffffffu) return false;
    if ((k % 32u) != 0 || k > 3072u) return false;   // whole 16-byte chunks for every storage; staged row <= 3 float4 per thread
    return qtype == MYNAH_HIP_F32 || qtype == MYNAH_HIP_F16 || qtype == MYNAH_HIP_INT8 || qtype == MYNAH_HIP_INT4;
}

int launch_linear(State *st, const LinearArgs &a, char *error, size_t capacity) {
    if (a.batch < 1 || a.batch > kBatchTile) {
        set_error(error, capacity, "linear: batch tile out of range");
        return -1;
    }
    if (a.fold_partial != nullptr && (a.batch > kConsumerFoldMaxBatch || a.k != a.fold_heads * a.fold_head_width || a.fold_slots == nullptr ||
                                      a.fold_partial_ml == nullptr)) {
        set_error(error, capacity, "linear: the fold source takes at most two streams and rows of heads x head width");
        return -1;
    }
    if (!linear_fast_supported(a.qtype, (size_t)a.n, (size_t)a.k)) {
        set_error(error, capacity, "linear: shape not supported by the fused matvec");
        return -1;
    }
    switch (a.qtype) {
        case MYNAH_HIP_F32: return launch_linear_q<MYNAH_HIP_F32>(st, a, error, capacity);
        case MYNAH_HIP_F16: return launch_linear_q<MYNAH_HIP_F16>(st, a, error, capacity);
        case MYNAH_HIP_INT8: return launch_linear_q<MYNAH_HIP_INT8>(st, a, error, capacity);
        default: return launch_linear_q<MYNAH_HIP_INT4>(st, a, error, capacity);
    }
}

// Products of fewer rows than this stay on the scalar tile kernels (a 64-row tile would be mostly padding).
constexpr size_t kGemmMfmaMinRows = 24;

int launch_gemm_f32(State *st, const float *in, float *out, size_t rows, size_t k, size_t n, const float *w,
                    const float *bias, char *error, size_t capacity) {
    if (rows == 0 || n == 0) return 0;
    if (rows >= kGemmMfmaMinRows && k > 0) {
        const dim3 grid((unsigned)((n + kGemmTile - 1) / kGemmTile), (unsigned)((rows + kGemmTile - 1) / kGemmTile));
        if (gemm_vec_ok(in, k, w, k, k, k))
            hipLaunchKernelGGL((k_gemm_f32_mfma<1, 1>), grid, dim3(256), 0, st->stream, in, (int)k, w, (int)k, out, (int)n, (int)rows, (int)n, (int)k, 1.0f,
                               0.0f, bias);
        else
            hipLaunchKernelGGL((k_gemm_f32_mfma<1, 0>), grid, dim3(256), 0, st->stream, in, (int)k, w, (int)k, out, (int)n, (int)rows, (int)n, (int)k, 1.0f,
                               0.0f, bias);
        return hip_check(hipGetLastError(), "gemm launch", error, capacity);
    }
    const dim3 grid((unsigned)((n + 15) / 16), (unsigned)((rows + 15) / 16));
    hipLaunchKernelGGL(k_gemm_nt_f32, grid, dim3(256), 0, st->stream, in, w, bias, out, (int)rows, (int)k, (int)n);
    return hip_check(hipGetLastError(), "gemm launch", error, capacity);
}

int launch_sgemm(State *st, int ta, int tb, size_t m, size_t n, size_t k, float alpha, const float *a, size_t lda,
                 const float *b, size_t ldb, float beta, float *c, size_t ldc, char *error, size_t capacity) {
    if (m == 0 || n == 0) return 0;
    if (!ta && m >= kGemmMfmaMinRows && k > 0) {   // op(A) = A: the forms the engine's attention makes (Q K^T, P V) and its row products
        const dim3 grid((unsigned)((n + kGemmTile - 1) / kGemmTile), (unsigned)((m + kGemmTile - 1) / kGemmTile));
        const bool vec = gemm_vec_ok(a, lda, b, ldb, tb ? k : 0, tb ? k : n);
        if (tb && vec)
            hipLaunchKernelGGL((k_gemm_f32_mfma<1, 1>), grid, dim3(256), 0, st->stream, a, (int)lda, b, (int)ldb, c, (int)ldc, (int)m, (int)n, (int)k, alpha, beta, nullptr);
        else if (tb)
            hipLaunchKernelGGL((k_gemm_f32_mfma<1, 0>), grid, dim3(256), 0, st->stream, a, (int)lda, b, (int)ldb, c, (int)ldc, (int)m, (int)n, (int)k, alpha, beta, nullptr);
        else if (vec && k % 4 == 0)
            hipLaunchKernelGGL((k_gemm_f32_mfma<0, 1>), grid, dim3(256), 0, st->stream, a, (int)lda, b, (int)ldb, c, (int)ldc, (int)m, (int)n, (int)k, alpha, beta, nullptr);
        else
            hipLaunchKernelGGL((k_gemm_f32_mfma<0, 0>), grid, dim3(256), 0, st->stream, a, (int)lda, b, (int)ldb, c, (int)ldc, (int)m, (int)n, (int)k, alpha, beta, nullptr);
        return hip_check(hipGetLastError(), "sgemm launch", error, capacity);
    }
    const dim3 grid((unsigned)((n + 15) / 16), (unsigned)((m + 15) / 16));
    hipLaunchKernelGGL(k_sgemm, grid, dim3(256), 0, st->stream, ta, tb, (int)m, (int)n, (int)k, alpha, a, (int)lda, b,
                       (int)ldb, beta, c, (int)ldc);
    return hip_check(hipGetLastError(), "sgemm launch", error, capacity);
}

}  // namespace mynah
