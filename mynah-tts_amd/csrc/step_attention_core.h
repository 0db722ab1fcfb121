// Building blocks of the resident step's attention stage, shared by the kernel that runs it as a launch of its own
// (kernels_step_attention.hip) and the persistent whole-step kernel (kernels_step_persistent.hip): the per-head projection
// passes and the arithmetic of one cache chunk.  Both kernels go through the same functions, so a stream's bits do not
// depend on which of them ran.
#pragma once

#include "device_common.h"

namespace mynah {

constexpr int kHw = 64;                          // head width handled by the fused kernel
constexpr int kPosLanes = 16;                    // lanes cooperating on one cache row
constexpr int kPosPerPass = kThreads / kPosLanes;
constexpr int kRowsPerThread = kStepUnitRows / kPosPerPass;   // 8
// PF = passes of weight rows per register bank: one bank is in flight for a cache-chunk or V workgroup, two for the
// Q+K workgroup of the new row (twice the rows).  4 when one or two streams are stepped (every weight row of a head is
// requested at once: shortest path), 2 for larger batches (fewer registers: three workgroups per CU instead of two,
// which is what matters once there are more workgroups than the chip holds at a time).  The arithmetic is the same.
constexpr int kPrefetchLatency = 4, kPrefetchThroughput = 2;

struct PassRegs {
    uint4 wv[4];
    float sc[4];   // int4: group scales of the four chunks
    float ws;      // int8: scale of the row
};

// Weight row of projection output r for this head: r = part * 64 + i, part 0/1/2 = q/k/v.
__device__ __forceinline__ int weight_row(int r, int head, int width) { return (r >> 6) * width + head * kHw + (r & 63); }

template <int QT, int PF>
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
        p.wv[u] = c < chunks ? load_global_u4(wrow + c) : make_uint4(0, 0, 0, 0);
        p.sc[u] = (QT == MYNAH_HIP_INT4 && c < chunks) ? load_global(a.scales + (size_t)wrow_id * chunks + c) : 0.0f;
    }
    // the row scale travels with the weights in the latency layout; the throughput layout fetches it at use (registers)
    p.ws = (QT == MYNAH_HIP_INT8 && PF == kPrefetchLatency) ? load_global(a.scales + wrow_id) : 1.0f;
}

// Requests passes [pass0, pass0 + PF) of rows [row0, row0 + nrows) into `bank`.
template <int QT, int PF>
__device__ __forceinline__ void load_bank(PassRegs (&bank)[PF], const StepAttnArgs &a, int pass0, int row0, int nrows, int head,
                                          int lg, int chunks) {
    const int rpp = 64 >> lg;
    const int passes = (nrows + 4 * rpp - 1) / (4 * rpp);
#pragma unroll
    for (int p = 0; p < PF; ++p)
        if (pass0 + p < passes) load_pass<QT, PF>(bank[p], a, pass0 + p, row0, nrows, head, lg, chunks);
}

// Passes [pass0, pass0 + PF) of the projection rows [row0, row0 + nrows) of this head (row numbering
// of weight_row), whose weights are in `bank` -> s_proj.
template <int QT, int PF>
__device__ __forceinline__ void project_bank(const StepAttnArgs &a, const PassRegs (&bank)[PF], int pass0, int row0, int nrows,
                                             int head, int lg, int chunks, const unsigned char *smem, const float sx, float *s_proj) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int G = 1 << lg, gl = lane & (G - 1), gidx = lane >> lg;
    const int rpp = 64 >> lg;
    const int passes = (nrows + 4 * rpp - 1) / (4 * rpp);
    // int4: a lane's chunk columns are the same in every pass, so their staged activations (and eight times their sums, what
    // the offset-binary nibbles need taken off) are read once here instead of once per row
    uint4 held_a[QT == MYNAH_HIP_INT4 ? 4 : 1], held_b[QT == MYNAH_HIP_INT4 ? 4 : 1];
    int held_sum8[QT == MYNAH_HIP_INT4 ? 4 : 1];
    if constexpr (QT == MYNAH_HIP_INT4) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = gl + u * G;
            const uint4 *xp = reinterpret_cast<const uint4 *>(smem + (size_t)(c < chunks ? c : 0) * 32);
            held_a[u] = xp[0];
            held_b[u] = xp[1];
            held_sum8[u] = group_sum8(held_a[u], held_b[u]);
        }
    }
#pragma unroll
    for (int p = 0; p < PF; ++p) {
        const int pass = pass0 + p;
        if (pass < passes) {
            const int r = row0 + pass * 4 * rpp + wave * rpp + gidx;
            int iacc[1] = {0};
            float facc[1] = {0.0f};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = gl + u * G;
                if constexpr (QT == MYNAH_HIP_INT4) {
                    if (c < chunks) dot_chunk_q4_held(bank[p].wv[u], bank[p].sc[u], held_a[u], held_b[u], held_sum8[u], facc[0]);
                } else {
                    if (c < chunks) dot_chunk<QT, 1>(bank[p].wv[u], bank[p].sc[u], c, smem, a.width, iacc, facc, nullptr);
                }
            }
            group_reduce<QT, 1>(iacc, facc, lg);
            if (gl == 0 && r < row0 + nrows) {
                float wscale = bank[p].ws;
                if constexpr (QT == MYNAH_HIP_INT8 && PF != kPrefetchLatency) wscale = load_global(a.scales + weight_row(r, head, a.width));
                s_proj[r] = finish_value<QT>(iacc[0], facc[0], wscale, sx);
            }
        }
    }
}

// Projection rows [row0, row0 + nrows): passes [0, PF) are in `bank` on entry, those from `next_pass`
// on are fetched here, a bank at a time.
template <int QT, int PF>
__device__ __forceinline__ void project_rows(const StepAttnArgs &a, PassRegs (&bank)[PF], int next_pass, int row0, int nrows,
                                             int head, int lg, int chunks, const unsigned char *smem, const float sx, float *s_proj) {
    const int rpp = 64 >> lg;
    const int passes = (nrows + 4 * rpp - 1) / (4 * rpp);
    project_bank<QT, PF>(a, bank, 0, row0, nrows, head, lg, chunks, smem, sx, s_proj);
    for (int pb = next_pass; pb < passes; pb += PF) {
        load_bank<QT, PF>(bank, a, pb, row0, nrows, head, lg, chunks);
        project_bank<QT, PF>(a, bank, pb, row0, nrows, head, lg, chunks, smem, sx, s_proj);
    }
}

// Scores, softmax statistics and weighted V rows of one cache chunk, one wavefront at a time: a wavefront owns 32 rows of
// the chunk (its four 16-lane row groups x 8 passes) and nothing leaves it until its own (max, sum, out[64]) is complete;
// the four results of a chunk meet once in LDS (s_red: 4 x 64 floats, s_wave_ml: max[4] | sum[4]).  kv / vv: this thread's
// float4 of the chunk's K and V rows g + 16 i, i < 8 (rows at or beyond `count` hold anything finite).
__device__ __forceinline__ void attend_chunk(const float4 qv, const float4 (&kv)[kRowsPerThread], const float4 (&vv)[kRowsPerThread],
                                             const int count, const float scale, float *s_red, float *s_wave_ml) {
    const int tid = threadIdx.x;
    const int g = tid / kPosLanes;
    const int lane = tid & 63, wave = tid >> 6;
    float sc[kRowsPerThread];
    float m = -3.0e38f;
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int pi = g + kPosPerPass * i;
        float dot = 0.0f;
        dot = __builtin_fmaf(qv.x, kv[i].x, dot);
        dot = __builtin_fmaf(qv.y, kv[i].y, dot);
        dot = __builtin_fmaf(qv.z, kv[i].z, dot);
        dot = __builtin_fmaf(qv.w, kv[i].w, dot);
        dot = row16_sum(dot);   // every lane of the row group holds the row's score
        sc[i] = pi < count ? dot * scale : -3.0e38f;
        m = fmaxf(m, sc[i]);
    }
    m = fmaxf(fmaxf(lane_f(m, 0), lane_f(m, 16)), fmaxf(lane_f(m, 32), lane_f(m, 48)));
    float l = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        // hardware exponential (2^(x log2 e), relative error about 1e-6 for the arguments met here) for the chunk's 128 weights;
        // the few exponentials that combine partial results stay exact
        const float e = g + kPosPerPass * i < count ? __expf(sc[i] - m) : 0.0f;
        l += e;
        acc.x = __builtin_fmaf(e, vv[i].x, acc.x);
        acc.y = __builtin_fmaf(e, vv[i].y, acc.y);
        acc.z = __builtin_fmaf(e, vv[i].z, acc.z);
        acc.w = __builtin_fmaf(e, vv[i].w, acc.w);
    }
    l = ((lane_f(l, 0) + lane_f(l, 16)) + lane_f(l, 32)) + lane_f(l, 48);
    acc.x += __shfl_xor(acc.x, 16); acc.y += __shfl_xor(acc.y, 16); acc.z += __shfl_xor(acc.z, 16); acc.w += __shfl_xor(acc.w, 16);
    acc.x += __shfl_xor(acc.x, 32); acc.y += __shfl_xor(acc.y, 32); acc.z += __shfl_xor(acc.z, 32); acc.w += __shfl_xor(acc.w, 32);
    if (lane < kPosLanes) *reinterpret_cast<float4 *>(s_red + wave * kHw + 4 * lane) = acc;
    if (lane == 0) { s_wave_ml[wave] = m; s_wave_ml[4 + wave] = l; }
}

// The merge of a chunk's four wavefront results in order 0..3, by the 16 threads t = 0..15 (each a float4 of the output),
// after a barrier behind attend_chunk.
__device__ __forceinline__ void merge_chunk(const int t, const float *s_red, const float *s_wave_ml, float4 &o, float &M, float &L) {
    const float *ml = s_wave_ml;
    const float *red = s_red;
    const float m0 = ml[0], m1 = ml[1], m2 = ml[2], m3 = ml[3];
    M = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
    const float w0 = expf(m0 - M), w1 = expf(m1 - M), w2 = expf(m2 - M), w3 = expf(m3 - M);   // a wavefront without rows: exp(-3e38 - M) = 0
    L = ml[4] * w0;
    L = __builtin_fmaf(ml[5], w1, L);
    L = __builtin_fmaf(ml[6], w2, L);
    L = __builtin_fmaf(ml[7], w3, L);
    const float4 o0 = *reinterpret_cast<const float4 *>(red + 4 * t), o1 = *reinterpret_cast<const float4 *>(red + kHw + 4 * t);
    const float4 o2 = *reinterpret_cast<const float4 *>(red + 2 * kHw + 4 * t), o3 = *reinterpret_cast<const float4 *>(red + 3 * kHw + 4 * t);
    o.x = __builtin_fmaf(o3.x, w3, __builtin_fmaf(o2.x, w2, __builtin_fmaf(o1.x, w1, o0.x * w0)));
    o.y = __builtin_fmaf(o3.y, w3, __builtin_fmaf(o2.y, w2, __builtin_fmaf(o1.y, w1, o0.y * w0)));
    o.z = __builtin_fmaf(o3.z, w3, __builtin_fmaf(o2.z, w2, __builtin_fmaf(o1.z, w1, o0.z * w0)));
    o.w = __builtin_fmaf(o3.w, w3, __builtin_fmaf(o2.w, w2, __builtin_fmaf(o1.w, w1, o0.w * w0)));
}

}  // namespace mynah
