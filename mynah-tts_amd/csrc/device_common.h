// Device-side building blocks shared by the matvec and attention kernels (gfx950, wave64).
#pragma once

#include "kernels.h"

namespace mynah {

constexpr int kThreads = 256;             // every fused kernel runs 4 waves per workgroup

// ---- wavefront reductions on the DPP data path (no LDS round trips) -------------------------------------
// Lane permutations inside a row of 16 lanes: xor 1, xor 2, mirror within 8, mirror within 16.  After the
// four steps every lane of a row holds the row's total (float addition is commutative, so all lanes of a
// row compute bit-identical values).  Rows are then combined through v_readlane in the fixed order
// ((r0 + r1) + r2) + r3.  All 64 lanes must be active.
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // row_half_mirror
constexpr int kDppMirror = 0x140;     // row_mirror

template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_f(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<kDppMirror>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    v = fmaxf(v, dpp_f<kDppXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f<kDppMirror>(v));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return ((lane_f(v, 0) + lane_f(v, 16)) + lane_f(v, 32)) + lane_f(v, 48);
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(lane_f(v, 0), lane_f(v, 16)), fmaxf(lane_f(v, 32), lane_f(v, 48)));
}

// Sum over aligned groups of 1 << lg lanes (lg uniform, 0..6); every lane of a group gets the group's total.
__device__ __forceinline__ float group_sum_f(float v, int lg) {
    if (lg >= 1) v += dpp_f<kDppXor1>(v);
    if (lg >= 2) v += dpp_f<kDppXor2>(v);
    if (lg >= 3) v += dpp_f<kDppHalfMirror>(v);
    if (lg >= 4) v += dpp_f<kDppMirror>(v);
    if (lg >= 5) {
        const float r0 = lane_f(v, 0), r1 = lane_f(v, 16), r2 = lane_f(v, 32), r3 = lane_f(v, 48);
        if (lg == 5) v = (threadIdx.x & 32) ? r2 + r3 : r0 + r1;
        else v = ((r0 + r1) + r2) + r3;
    }
    return v;
}
__device__ __forceinline__ int group_sum_i(int v, int lg) {
    if (lg >= 1) v += dpp_i<kDppXor1>(v);
    if (lg >= 2) v += dpp_i<kDppXor2>(v);
    if (lg >= 3) v += dpp_i<kDppHalfMirror>(v);
    if (lg >= 4) v += dpp_i<kDppMirror>(v);
    if (lg >= 5) {
        const int r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
        const int r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
        if (lg == 5) v = (threadIdx.x & 32) ? r2 + r3 : r0 + r1;
        else v = r0 + r1 + r2 + r3;
    }
    return v;
}

// Reduces BT independent values over the 256-thread workgroup in a fixed order: lanes by butterfly,
// then waves 0..3.  The order never depends on how many of the BT slots are live.  `s_scratch` is 4 * BT floats
// that no earlier reduction of this workgroup used (each reduction of a kernel gets its own region, so a single
// barrier per reduction is enough).
// `wave` is the caller's wavefront index among the four that reduce together (see Team below).
template <int BT, bool IS_MAX>
__device__ __forceinline__ void block_reduce(float (&v)[BT], float *s_scratch, const int wave) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int b = 0; b < BT; ++b) v[b] = IS_MAX ? wave_max(v[b]) : wave_sum(v[b]);
    if (lane == 0) {
#pragma unroll
        for (int b = 0; b < BT; ++b) s_scratch[wave * BT + b] = v[b];
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < BT; ++b) {
        const float a0 = s_scratch[b], a1 = s_scratch[BT + b], a2 = s_scratch[2 * BT + b], a3 = s_scratch[3 * BT + b];
        v[b] = IS_MAX ? fmaxf(fmaxf(a0, a1), fmaxf(a2, a3)) : ((a0 + a1) + a2) + a3;
    }
}

// Sum over a 256-thread workgroup in a fixed order: lanes by butterfly, then waves 0..3.
__device__ __forceinline__ float block_sum(float v, float *s4) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s4[threadIdx.x >> 6] = v;
    __syncthreads();
    return ((s4[0] + s4[1]) + s4[2]) + s4[3];
}
__device__ __forceinline__ float block_max(float v, float *s4) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s4[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(s4[0], s4[1]), fmaxf(s4[2], s4[3]));
}

// mynah_layernorm_f32 (src/kernels.c:186-244): mean, then the variance of (x - mean), eps inside the
// square root, y = (x - mean) * scale * gain (+ bias).  One workgroup per row.
// Rows of up to 256 * NV values stay in registers: one round trip for the row, its gain and its bias (requested side by
// side, none under a condition) instead of three passes over memory with a round trip per 256 values each.  A thread
// adds its values in the order of the loop below, so the results are the same bits.
template <int NV>
__device__ __forceinline__ void layernorm_row_in_registers(const float *x, float *y, const float *gain, const float *bias, int width,
                                                           float *s4) {
    float xv[NV], gv[NV], bv[NV];
    const float *bias_or_gain = bias != nullptr ? bias : gain;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = threadIdx.x + 256 * u, at = i < width ? i : width - 1;
        xv[u] = x[at];
        gv[u] = gain[at];
        bv[u] = bias_or_gain[at];
    }
    float s = 0.0f;
#pragma unroll
    for (int u = 0; u < NV; ++u)
        if ((int)threadIdx.x + 256 * u < width) s += xv[u];
    const float mean = block_sum(s, s4) / (float)width;
    float v = 0.0f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        if ((int)threadIdx.x + 256 * u < width) {
            const float d = xv[u] - mean;
            v = __builtin_fmaf(d, d, v);
        }
    }
    const float variance = block_sum(v, s4);
    const float scale = 1.0f / sqrtf(variance / (float)width + 1.0e-5f);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = threadIdx.x + 256 * u;
        if (i < width) {
            float z = ((xv[u] - mean) * scale) * gv[u];
            if (bias != nullptr) z += bv[u];
            y[i] = z;
        }
    }
}

// The same for rows of whole float4s (width a multiple of 4, at most 1024 * NV4 values, 16-byte aligned rows), with every sum
// formed exactly as the fused matvec's LayerNorm prologue forms it (finish_activations below: a thread's float4s f = tid + 256 i,
// each added as (x + y) + (z + w), lanes by butterfly, wavefronts 0..3) -- so a row normalised here and a row normalised by a
// product's prologue are the same bits, whichever of the two a caller's sequence of calls ends up in.
template <int NV4>
__device__ __forceinline__ void layernorm_row_as_prologue(const float *x, float *y, const float *gain, const float *bias, int width, float *s4) {
    const int nf4 = width >> 2;
    const int tid = threadIdx.x & 255;
    float4 xv[NV4], gv[NV4], bv[NV4];
    const float *bias_or_gain = bias != nullptr ? bias : gain;
#pragma unroll
    for (int i = 0; i < NV4; ++i) {
        const int f = tid + 256 * i, at = f < nf4 ? f : nf4 - 1;
        xv[i] = reinterpret_cast<const float4 *>(x)[at];
        gv[i] = reinterpret_cast<const float4 *>(gain)[at];
        bv[i] = reinterpret_cast<const float4 *>(bias_or_gain)[at];
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < NV4; ++i) {
        const float4 v = tid + 256 * i < nf4 ? xv[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        s += (v.x + v.y) + (v.z + v.w);
    }
    const float mean = block_sum(s, s4) / (float)width;
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < NV4; ++i)
        if (tid + 256 * i < nf4) {
            const float d0 = xv[i].x - mean, d1 = xv[i].y - mean, d2 = xv[i].z - mean, d3 = xv[i].w - mean;
            q = __builtin_fmaf(d0, d0, q);
            q = __builtin_fmaf(d1, d1, q);
            q = __builtin_fmaf(d2, d2, q);
            q = __builtin_fmaf(d3, d3, q);
        }
    const float variance = block_sum(q, s4);
    const float scale = 1.0f / sqrtf(variance / (float)width + 1.0e-5f);
#pragma unroll
    for (int i = 0; i < NV4; ++i) {
        const int f = tid + 256 * i;
        if (f < nf4) {
            float4 z;
            z.x = ((xv[i].x - mean) * scale) * gv[i].x;
            z.y = ((xv[i].y - mean) * scale) * gv[i].y;
            z.z = ((xv[i].z - mean) * scale) * gv[i].z;
            z.w = ((xv[i].w - mean) * scale) * gv[i].w;
            if (bias != nullptr) { z.x += bv[i].x; z.y += bv[i].y; z.z += bv[i].z; z.w += bv[i].w; }
            reinterpret_cast<float4 *>(y)[f] = z;
        }
    }
}

__device__ __forceinline__ void layernorm_row(const float *x, float *y, const float *gain, const float *bias, int width,
                                              float *s4) {
    const bool whole4 = (width & 3) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(gain) |
                                              reinterpret_cast<uintptr_t>(bias)) & 15) == 0;
    if (whole4 && width <= 1024) return layernorm_row_as_prologue<1>(x, y, gain, bias, width, s4);
    if (whole4 && width <= 3072) return layernorm_row_as_prologue<3>(x, y, gain, bias, width, s4);
    if (width <= 1024) return layernorm_row_in_registers<4>(x, y, gain, bias, width, s4);
    if (width <= 4096) return layernorm_row_in_registers<16>(x, y, gain, bias, width, s4);
    float s = 0.0f;
    for (int i = threadIdx.x; i < width; i += 256) s += x[i];
    const float mean = block_sum(s, s4) / (float)width;
    float v = 0.0f;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float d = x[i] - mean;
        v = __builtin_fmaf(d, d, v);
    }
    const float variance = block_sum(v, s4);
    const float scale = 1.0f / sqrtf(variance / (float)width + 1.0e-5f);
    for (int i = threadIdx.x; i < width; i += 256) {
        float z = ((x[i] - mean) * scale) * gain[i];
        if (bias != nullptr) z += bias[i];
        y[i] = z;
    }
}

// round half away from zero by truncation (src/qmat.c:106-110); the half with v's sign is one bit-field instruction where
// the comparison and selection of the reference's form are two, with the same sum for every v.  The reference then clamps
// to +-127, which changes nothing when inv is 127 / amax and amax the largest |x| of the row this x belongs to -- the only
// way this is called: |x * inv| <= 127 (1 + 2^-23), plus a half stays below 128, and truncation gives at most 127.
__device__ __forceinline__ int quant_act(float x, float inv) {
    const float v = x * inv;
    return (int)(v + __builtin_copysignf(0.5f, v));
}
// the low bytes of four such integers in one dword, q0 lowest (three byte-permute instructions)
__device__ __forceinline__ unsigned pack_bytes(int q0, int q1, int q2, int q3) {
    const unsigned lo = __builtin_amdgcn_perm((unsigned)q1, (unsigned)q0, 0x0c0c0400u);   // [q0.b0, q1.b0, 0, 0]
    const unsigned hi = __builtin_amdgcn_perm((unsigned)q3, (unsigned)q2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);                                    // [lo.b0, lo.b1, hi.b0, hi.b1]
}

// src/kernels.c:382-389
__device__ __forceinline__ float gelu_tanh(float x) {
    const float cubic = x * x * x;
    const float c = 0.7978845608f * (x + 0.044715f * cubic);
    return 0.5f * x * (1.0f + tanhf(c));
}

__device__ __forceinline__ int dot4(unsigned a, unsigned b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// offset-binary nibbles (q + 8) of one dword -> four signed bytes each for the even and odd elements
__device__ __forceinline__ void unpack_q4(unsigned w, unsigned &even, unsigned &odd) {
    const unsigned lo = w & 0x0f0f0f0fu;
    const unsigned hi = (w >> 4) & 0x0f0f0f0fu;
    even = ((lo | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
    odd = ((hi | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

// exact widening of an IEEE half (v_cvt_f32_f16)
__device__ __forceinline__ float half_bits_to_float(unsigned short h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, sizeof v);
    return (float)v;
}

template <int QT> struct Chunk;   // elements per 16-byte weight chunk
template <> struct Chunk<MYNAH_HIP_F32> { static constexpr int n = 4; };
template <> struct Chunk<MYNAH_HIP_F16> { static constexpr int n = 8; };
template <> struct Chunk<MYNAH_HIP_INT8> { static constexpr int n = 16; };
template <> struct Chunk<MYNAH_HIP_INT4> { static constexpr int n = 32; };

template <int QT>
constexpr bool kQuantised = (QT == MYNAH_HIP_INT8 || QT == MYNAH_HIP_INT4);

// Lane-group width for a row of `chunks` 16-byte chunks: the widest power of two that still leaves
// about three chunks per lane (k = 768 int8 -> 16 lanes, k = 3072 int8 -> 64 lanes).
__host__ __device__ constexpr int lane_group_log2(int chunks) {
    int lg = 6;
    while (lg > 0 && (chunks >> lg) < 3) --lg;
    return lg;
}

// int4, one stream, the group's activations already in registers (xa | xb: its 32 staged bytes; sum8: eight times their sum):
// facc += (float)(sum n x - 8 sum x) * scale with n the offset-binary nibbles -- the integer of dot_q4 (src/qmat.c:156-185),
// since n = q + 8.  A caller whose lanes keep their chunk columns over many rows reads and sums the activations once.
__device__ __forceinline__ void dot_chunk_q4_held(const uint4 wv, const float sc, const uint4 xa, const uint4 xb, const int sum8, float &facc) {
    const unsigned m = 0x0f0f0f0fu;
    int gi = 0;
    gi = dot4(wv.x & m, xa.x, gi); gi = dot4((wv.x >> 4) & m, xa.y, gi);
    gi = dot4(wv.y & m, xa.z, gi); gi = dot4((wv.y >> 4) & m, xa.w, gi);
    gi = dot4(wv.z & m, xb.x, gi); gi = dot4((wv.z >> 4) & m, xb.y, gi);
    gi = dot4(wv.w & m, xb.z, gi); gi = dot4((wv.w >> 4) & m, xb.w, gi);
    gi -= sum8;
    const float term = (float)gi * sc;
    facc = facc + term;
}
// eight times the sum of a group's 32 staged int8 activations
__device__ __forceinline__ int group_sum8(const uint4 xa, const uint4 xb) {
    const unsigned ones = 0x01010101u;
    int s = 0;
    s = dot4(ones, xa.x, s); s = dot4(ones, xa.y, s); s = dot4(ones, xa.z, s); s = dot4(ones, xa.w, s);
    s = dot4(ones, xb.x, s); s = dot4(ones, xb.y, s); s = dot4(ones, xb.z, s); s = dot4(ones, xb.w, s);
    return 8 * s;
}

// One 16-byte weight chunk against the staged activations of BT streams.
//   int8 : iacc += sum w*qx                         (dot_q8, src/qmat.c:136-152)
//   int4 : facc += (float)(group int32) * scale[g]  (dot_q4, src/qmat.c:156-185; one chunk = one group of 32)
//   f16  : facc = fma(widen(w), x, facc)            (matvec_f16, src/qmat.c:306-378)
//   f32  : facc = fma(w, x, facc)
// group_out (int4 probe): per-group integer of stream 0.
template <int QT, int BT>
__device__ __forceinline__ void dot_chunk(const uint4 wv, const float sc, const int c, const unsigned char *smem, const int k,
                                          int (&iacc)[BT], float (&facc)[BT], int *group_out) {
    if constexpr (QT == MYNAH_HIP_INT8) {
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const uint4 xv = *reinterpret_cast<const uint4 *>(smem + (size_t)b * k + (size_t)c * 16);
            int s = iacc[b];
            s = dot4(wv.x, xv.x, s);
            s = dot4(wv.y, xv.y, s);
            s = dot4(wv.z, xv.z, s);
            s = dot4(wv.w, xv.w, s);
            iacc[b] = s;
        }
    } else if constexpr (QT == MYNAH_HIP_INT4 && BT == 1) {
        // One stream: the nibbles stay offset-binary (q + 8, 0 .. 15 -- a signed byte as well) and the offset comes off the
        // group's integer at the end: sum (n - 8) x = sum n x - 8 sum x, exact in int32 (|sum n x| <= 32 * 15 * 127).  Twelve
        // mask / shift operations and eight more dot products instead of the thirty-six that make signed bytes of the nibbles.
        const uint4 *xp = reinterpret_cast<const uint4 *>(smem + (size_t)c * 32);
        const uint4 xa = xp[0], xb = xp[1];
        const unsigned m = 0x0f0f0f0fu;
        int gi = 0;
        gi = dot4(wv.x & m, xa.x, gi); gi = dot4((wv.x >> 4) & m, xa.y, gi);
        gi = dot4(wv.y & m, xa.z, gi); gi = dot4((wv.y >> 4) & m, xa.w, gi);
        gi = dot4(wv.z & m, xb.x, gi); gi = dot4((wv.z >> 4) & m, xb.y, gi);
        gi = dot4(wv.w & m, xb.z, gi); gi = dot4((wv.w >> 4) & m, xb.w, gi);
        gi -= group_sum8(xa, xb);
        const float term = (float)gi * sc;   // acc += (float)gi * scales[g]  (src/qmat.c:181)
        facc[0] = facc[0] + term;
        if (group_out != nullptr) *group_out = gi;
    } else if constexpr (QT == MYNAH_HIP_INT4) {
        unsigned e0, o0, e1, o1, e2, o2, e3, o3;
        unpack_q4(wv.x, e0, o0);
        unpack_q4(wv.y, e1, o1);
        unpack_q4(wv.z, e2, o2);
        unpack_q4(wv.w, e3, o3);
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const uint4 *xp = reinterpret_cast<const uint4 *>(smem + (size_t)b * k + (size_t)c * 32);
            const uint4 xa = xp[0], xb = xp[1];
            int gi = 0;
            gi = dot4(e0, xa.x, gi); gi = dot4(o0, xa.y, gi);
            gi = dot4(e1, xa.z, gi); gi = dot4(o1, xa.w, gi);
            gi = dot4(e2, xb.x, gi); gi = dot4(o2, xb.y, gi);
            gi = dot4(e3, xb.z, gi); gi = dot4(o3, xb.w, gi);
            const float term = (float)gi * sc;   // acc += (float)gi * scales[g]  (src/qmat.c:181)
            facc[b] = facc[b] + term;
            if (b == 0 && group_out != nullptr) *group_out = gi;
        }
    } else if constexpr (QT == MYNAH_HIP_F16) {
        const unsigned wd[4] = {wv.x, wv.y, wv.z, wv.w};
        float wf[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wf[2 * i] = half_bits_to_float((unsigned short)(wd[i] & 0xffffu));
            wf[2 * i + 1] = half_bits_to_float((unsigned short)(wd[i] >> 16));
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float4 *xp = reinterpret_cast<const float4 *>(smem) + (size_t)b * (k >> 2) + (size_t)c * 2;
            const float4 xa = xp[0], xb = xp[1];
            float s = facc[b];
            s = __builtin_fmaf(wf[0], xa.x, s); s = __builtin_fmaf(wf[1], xa.y, s);
            s = __builtin_fmaf(wf[2], xa.z, s); s = __builtin_fmaf(wf[3], xa.w, s);
            s = __builtin_fmaf(wf[4], xb.x, s); s = __builtin_fmaf(wf[5], xb.y, s);
            s = __builtin_fmaf(wf[6], xb.z, s); s = __builtin_fmaf(wf[7], xb.w, s);
            facc[b] = s;
        }
    } else {
        const float w0 = __uint_as_float(wv.x), w1 = __uint_as_float(wv.y);
        const float w2 = __uint_as_float(wv.z), w3 = __uint_as_float(wv.w);
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float4 xa = reinterpret_cast<const float4 *>(smem)[(size_t)b * (k >> 2) + c];
            float s = facc[b];
            s = __builtin_fmaf(w0, xa.x, s); s = __builtin_fmaf(w1, xa.y, s);
            s = __builtin_fmaf(w2, xa.z, s); s = __builtin_fmaf(w3, xa.w, s);
            facc[b] = s;
        }
    }
}

// Reduction over a lane group of G = 1 << lg lanes: the same tree for every batch size.
template <int QT, int BT>
__device__ __forceinline__ void group_reduce(int (&iacc)[BT], float (&facc)[BT], const int lg) {
#pragma unroll
    for (int b = 0; b < BT; ++b) {
        if constexpr (QT == MYNAH_HIP_INT8) iacc[b] = group_sum_i(iacc[b], lg);
        else facc[b] = group_sum_f(facc[b], lg);
    }
}

// ((float)acc * scale[row]) * sx (src/qmat.c:224) / acc * sx (src/qmat.c:292) / acc
template <int QT>
__device__ __forceinline__ float finish_value(const int iacc, const float facc, const float wscale, const float sx) {
    if constexpr (QT == MYNAH_HIP_INT8) return ((float)iacc * wscale) * sx;
    else if constexpr (QT == MYNAH_HIP_INT4) return facc * sx;
    else return facc;
}

// Where the prologue takes a stream's activation row from.
struct ActSource {
    const float *rows[kBatchTile];   // plain device rows, one per stream of the team (rows[0] = the team's first stream) ...
    // ... or the fold of split-L attention partials (resident step): row[b] = sum_u o_u e^(m_u-M) / sum_u l_u e^(m_u-M)
    const float *partial;            // non-null selects the fold: partial outputs [stream][head][max_units][head_width]
    const float *partial_ml;         // chunk maxima and sums [stream][head][2][max_units]
    const StepSlots *slots;
    int heads, head_width, max_units, is_self, stream0;
};

// Units a stream's attention was split into: cache chunks of kStepUnitRows rows, plus the step's new row for
// self-attention.  Depends on that stream's own length only.
__device__ __forceinline__ int units_of_length(int rows, int is_self) {
    const int chunks = (rows + kStepUnitRows - 1) / kStepUnitRows;
    return is_self ? chunks + 1 : (chunks > 0 ? chunks : 1);
}
__device__ __forceinline__ int attention_units(const StepSlots *s, int stream, int is_self) {
    return units_of_length(is_self ? s->length[stream] : s->memory_length[stream], is_self);
}

// A pointer that comes out of memory (the slot table's cache, input and output rows) carries no address space, and a load
// or store through it is a flat instruction, which counts against the LDS counter as well as the vector-memory one: every
// wait in front of a barrier then also waits for it.  These go through the pointer as what it is, a global address.
typedef float float_x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load_global4(const float *p) {
    const float_x4 v = *(const __attribute__((address_space(1))) float_x4 *)p;
    return make_float4(v.x, v.y, v.z, v.w);
}
typedef unsigned uint_x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_global_u4(const uint4 *p) {
    const uint_x4 v = *(const __attribute__((address_space(1))) uint_x4 *)p;
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float load_global(const float *p) { return *(const __attribute__((address_space(1))) float *)p; }
__device__ __forceinline__ void store_global(float *p, float v) { *(__attribute__((address_space(1))) float *)p = v; }
__device__ __forceinline__ void store_global4(float *p, float4 v) {
    const float_x4 w = {v.x, v.y, v.z, v.w};
    *(__attribute__((address_space(1))) float_x4 *)p = w;
}

// Kernel arguments beyond the fourteen dwords that are in registers at wavefront start are read from memory where the
// compiler first needs them, and the first read of every 64-byte line of them is a round trip of a few hundred nanoseconds --
// wherever it stands: in front of the cache-row requests, between two barriers of the activation quantisation.  This asks
// for one dword of each of the first LINES lines at the top of a kernel, without waiting: when the fields are needed they
// come out of the scalar cache.  The four destination registers must stay reserved until the answers are in: release_warm
// (below) ends the reservation with a wait of its own.  A wavefront that ends before that waits for what it has
// outstanding as part of ending.
struct WarmArguments { unsigned r0, r1, r2, r3; };
template <int LINES>
__device__ __forceinline__ WarmArguments warm_kernel_arguments() {
    static_assert(LINES >= 1 && LINES <= 4, "one dword from each of up to four lines behind the first");
    WarmArguments w{0u, 0u, 0u, 0u};
    const auto args = __builtin_amdgcn_kernarg_segment_ptr();   // a constant-address-space pointer: two scalar registers
    if constexpr (LINES >= 1) __asm__ volatile("s_load_dword %0, %1, 0x40" : "=&s"(w.r0) : "s"(args));
    if constexpr (LINES >= 2) __asm__ volatile("s_load_dword %0, %1, 0x80" : "=&s"(w.r1) : "s"(args));
    if constexpr (LINES >= 3) __asm__ volatile("s_load_dword %0, %1, 0xc0" : "=&s"(w.r2) : "s"(args));
    if constexpr (LINES >= 4) __asm__ volatile("s_load_dword %0, %1, 0x100" : "=&s"(w.r3) : "s"(args));
    return w;
}
// Lets go of the registers the lines were asked into.  The compiler does not know that the statements above are loads, so it
// would hand these registers to other values while the answers are still on their way: they stay reserved up to here, and
// the wait makes sure the answers are in (placed where the kernel has long waited for later requests, it costs nothing).
__device__ __forceinline__ void release_warm(const WarmArguments &w) {
    __asm__ volatile("s_waitcnt lgkmcnt(0)" ::"s"(w.r0), "s"(w.r1), "s"(w.r2), "s"(w.r3));
}
// Table words through the scalar cache, whatever the compiler can prove.  A wavefront-uniform word from memory is a scalar
// load only when the compiler can show that nothing before it may have written memory; behind any of the statements above
// (which it must take for writes) it becomes a vector load, and vector loads return in order -- a table word then arrives
// behind every row requested before it, or, requested first, makes the kernel wait a whole round trip before its first
// row request.  These ask for the word as a scalar load outright; scalar_words_arrived() is the wait, to be placed in front
// of the first use (the answers of scalar loads do not queue behind vector requests).
__device__ __forceinline__ int scalar_load_int(const int *p) {
    int v;
    __asm__ volatile("s_load_dword %0, %1, 0x0" : "=&s"(v) : "s"(p));
    return v;
}
__device__ __forceinline__ unsigned long long scalar_load_u64(const void *p) {
    unsigned long long v;
    __asm__ volatile("s_load_dwordx2 %0, %1, 0x0" : "=&s"(v) : "s"(p));
    return v;
}
__device__ __forceinline__ void scalar_words_arrived(int &a, unsigned long long &b, unsigned long long &c) {
    __asm__ volatile("s_waitcnt lgkmcnt(0)" : "+s"(a), "+s"(b), "+s"(c));
}

// Keeps the memory requests written above this point above it: without it the compiler is free to sink a load to its
// first use, i.e. behind whatever that use waits for.  Emits no instruction and waits for nothing.
__device__ __forceinline__ void requests_issued() { __asm__ volatile("" ::: "memory"); }

// One float4 of a stream's folded attention output.  Units are taken in order 0..units-1.  How many units the stream
// has is in the slot table, a read that takes as long as the partials themselves: so the first kFoldAhead partial slots
// (they exist whatever the stream's length: the workspace is sized for max_units) are requested before the count is
// looked at, and masked by it afterwards.  Streams with more units continue from memory.
constexpr int kFoldAhead = 10;
__device__ __forceinline__ float4 fold_partials(const ActSource &src, int stream, int f4) {
    const int hw = src.head_width;
    const int d = 4 * f4;
    const int head = d / hw, dh = d - head * hw;
    const size_t sh = (size_t)stream * src.heads + head;
    const float *m = src.partial_ml + sh * 2 * src.max_units;
    const float *l = m + src.max_units;
    const float *o = src.partial + sh * src.max_units * hw + dh;
    // The unit count is read first: the stream is the same for the whole workgroup and nothing has been stored yet, so it is
    // a scalar load, whose answer neither queues behind the vector requests below nor makes them wait; it is looked at
    // after they have all been issued.  (Read after them it was a vector load -- nothing after requests_issued() can be
    // proven unwritten -- that could only be looked at once every partial had come back: a round trip on top of theirs.)
    // (every caller's stream is the same for a whole wavefront -- it depends on the team and the loop index only -- which
    // the compiler cannot see through the thread index: readfirstlane says so)
    const int stream_u = __builtin_amdgcn_readfirstlane(stream);
    int rows = src.is_self ? src.slots->length[stream_u] : src.slots->memory_length[stream_u];
    float pm[kFoldAhead], pl[kFoldAhead];
    float4 po[kFoldAhead];
#pragma unroll
    for (int u = 0; u < kFoldAhead; ++u) {
        // no request under a condition (the compiler would have to wait for all of them at the first use): a slot the
        // workspace does not have repeats its last one, and is never used since units <= max_units
        const int uu = u < src.max_units ? u : src.max_units - 1;
        pm[u] = m[uu];
        pl[u] = l[uu];
        po[u] = *reinterpret_cast<const float4 *>(o + (size_t)uu * hw);
    }
    requests_issued();
    rows = __builtin_amdgcn_readfirstlane(rows);   // the same for the whole wavefront
    __asm__ volatile("" : "+s"(rows));               // the table word is first looked at here, behind the requests (emits nothing)
    const int units = units_of_length(rows, src.is_self);
    float M = -3.0e38f;
#pragma unroll
    for (int u = 0; u < kFoldAhead; ++u)
        if (u < units) M = fmaxf(M, pm[u]);
    for (int u = kFoldAhead; u < units; ++u) M = fmaxf(M, m[u]);
    float L = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < kFoldAhead; ++u) {
        if (u < units) {
            const float w = expf(pm[u] - M);
            L = __builtin_fmaf(pl[u], w, L);
            acc.x = __builtin_fmaf(po[u].x, w, acc.x);
            acc.y = __builtin_fmaf(po[u].y, w, acc.y);
            acc.z = __builtin_fmaf(po[u].z, w, acc.z);
            acc.w = __builtin_fmaf(po[u].w, w, acc.w);
        }
    }
#pragma unroll 4
    for (int u = kFoldAhead; u < units; ++u) {
        const float w = expf(m[u] - M);
        const float4 ou = *reinterpret_cast<const float4 *>(o + (size_t)u * hw);
        L = __builtin_fmaf(l[u], w, L);
        acc.x = __builtin_fmaf(ou.x, w, acc.x);
        acc.y = __builtin_fmaf(ou.y, w, acc.y);
        acc.z = __builtin_fmaf(ou.z, w, acc.z);
        acc.w = __builtin_fmaf(ou.w, w, acc.w);
    }
    acc.x /= L; acc.y /= L; acc.z /= L; acc.w /= L;
    return acc;
}

constexpr int kPrologueScratch = 12;   // floats of reduction scratch per stream slot

struct PrologueParams {
    int k;                  // row length (multiple of 4; k/4 <= 256 * NVT)
    int batch;              // live streams (<= BT)
    const float *ln_gain;   // non-null: LayerNorm, eps 1e-5 (mynah_layernorm_f32, src/kernels.c:186-244)
    const float *ln_bias;
    int arith;
    int8_t *probe_qx;       // parity probes for stream 0 (written by workgroup 0 only)
    float *probe_sx;
    float *ln_out = nullptr;   // non-null: workgroup 0 also stores stream 0's LayerNorm row here
    const StepSlots *ln_out_slots = nullptr;   // non-null: workgroup 0 stores every stream's LayerNorm row at this table's output[stream]
    float *act_out = nullptr;  // non-null: workgroup 0 also stores stream 0's row as loaded (after a fold, before LayerNorm)
};

// Who stages which streams: the 256 threads tid = 0..255 of a workgroup stage the streams [stream0, stream0 + count) together
// with the scheme below.  (Matvec builds for more than two streams with quantised weights stage a stream per wavefront
// instead: load_stream_row / finish_stream_row further down, same bytes.)
struct Team {
    int tid;       // 0..255 within the team
    int stream0;   // first stream of the team
};
// (every kernel that stages this way has 256 threads; the mask says so to the compiler, which then drops the range checks of a
// row that fills the workgroup's places exactly -- k = 3072 -- and requests it unconditionally)
__device__ __forceinline__ Team whole_workgroup() { return Team{(int)(threadIdx.x & (kThreads - 1)), 0}; }

// Stages the activations of up to BT streams in LDS, all 256 threads of a team cooperating on every stream:
// load (or fold) -> optional LayerNorm -> for int8/int4 weights the per-vector absmax int8 quantisation
// (quantize_act_int8, src/qmat.c:94-113; int4 additionally de-interleaves even/odd elements per run of 8
// so they line up with the low/high nibbles of a weight dword).  NVT = float4 per thread per stream.
// s_scratch: kPrologueScratch * BT floats (one region per reduction: mean, variance, absmax).
//
// First half of the prologue: request (or fold) the activation rows and the LayerNorm vectors.  Split from the
// arithmetic so that a kernel can put other requests between the two (they are served while these are in flight).
template <int BT, int NVT>
__device__ __forceinline__ void load_activations(const PrologueParams &p, const ActSource &src, const Team team, float4 (&xr)[BT][NVT],
                                                 float4 (&gv)[NVT], float4 (&bv)[NVT]) {
    const int tid = team.tid;
    const int nf4 = p.k >> 2;
#pragma unroll
    for (int b = 0; b < BT; ++b)
#pragma unroll
        for (int i = 0; i < NVT; ++i) {
            const int f = tid + kThreads * i;
            const int stream = team.stream0 + b;
            const bool on = stream < p.batch && f < nf4;
            if (!on) xr[b][i] = make_float4(0.f, 0.f, 0.f, 0.f);
            else if (src.partial != nullptr) xr[b][i] = fold_partials(src, src.stream0 + stream, f);
            else xr[b][i] = reinterpret_cast<const float4 *>(src.rows[b])[f];
        }
#pragma unroll
    for (int i = 0; i < NVT; ++i) {
        const int f = tid + kThreads * i;
        gv[i] = (p.ln_gain != nullptr && f < nf4) ? reinterpret_cast<const float4 *>(p.ln_gain)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
        bv[i] = (p.ln_gain != nullptr && f < nf4 && p.ln_bias != nullptr) ? reinterpret_cast<const float4 *>(p.ln_bias)[f] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

// Second half: optional LayerNorm -> quantisation (or plain copy) -> LDS.
// s_scratch: kPrologueScratch floats per stream of the workgroup (all teams).
template <int QT, int BT, int NVT>
__device__ __forceinline__ void finish_activations(const PrologueParams &p, const Team team, float4 (&xr)[BT][NVT], const float4 (&gv)[NVT],
                                                   const float4 (&bv)[NVT], unsigned char *smem, float *s_sx, float *s_scratch_all) {
    const int tid = team.tid;
    const int wave = tid >> 6;
    float *s_scratch = s_scratch_all + team.stream0 * kPrologueScratch;   // the team's own region
    const int nf4 = p.k >> 2;
    if (p.act_out != nullptr && blockIdx.x == 0 && team.stream0 == 0) {
#pragma unroll
        for (int i = 0; i < NVT; ++i)
            if (tid + kThreads * i < nf4) reinterpret_cast<float4 *>(p.act_out)[tid + kThreads * i] = xr[0][i];
    }
    if (p.ln_gain != nullptr) {
        float s[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            s[b] = 0.0f;
#pragma unroll
            for (int i = 0; i < NVT; ++i) s[b] += (xr[b][i].x + xr[b][i].y) + (xr[b][i].z + xr[b][i].w);
        }
        block_reduce<BT, false>(s, s_scratch, wave);
        float mean[BT], v[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            mean[b] = s[b] / (float)p.k;
            v[b] = 0.0f;
#pragma unroll
            for (int i = 0; i < NVT; ++i)
                if (tid + kThreads * i < nf4) {
                    const float d0 = xr[b][i].x - mean[b], d1 = xr[b][i].y - mean[b], d2 = xr[b][i].z - mean[b], d3 = xr[b][i].w - mean[b];
                    v[b] = __builtin_fmaf(d0, d0, v[b]);
                    v[b] = __builtin_fmaf(d1, d1, v[b]);
                    v[b] = __builtin_fmaf(d2, d2, v[b]);
                    v[b] = __builtin_fmaf(d3, d3, v[b]);
                }
        }
        block_reduce<BT, false>(v, s_scratch + 4 * BT, wave);
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float rstd = 1.0f / sqrtf(v[b] / (float)p.k + 1.0e-5f);
#pragma unroll
            for (int i = 0; i < NVT; ++i) {
                float4 y;
                y.x = ((xr[b][i].x - mean[b]) * rstd) * gv[i].x;
                y.y = ((xr[b][i].y - mean[b]) * rstd) * gv[i].y;
                y.z = ((xr[b][i].z - mean[b]) * rstd) * gv[i].z;
                y.w = ((xr[b][i].w - mean[b]) * rstd) * gv[i].w;
                if (p.ln_bias != nullptr) {
                    y.x += bv[i].x; y.y += bv[i].y; y.z += bv[i].z; y.w += bv[i].w;
                }
                xr[b][i] = y;   // lanes beyond the row hold gain 0 -> 0
                if (p.ln_out != nullptr && blockIdx.x == 0 && team.stream0 + b == 0 && tid + kThreads * i < nf4)
                    reinterpret_cast<float4 *>(p.ln_out)[tid + kThreads * i] = y;
                if (p.ln_out_slots != nullptr && blockIdx.x == 0 && team.stream0 + b < p.batch && tid + kThreads * i < nf4)
                    reinterpret_cast<float4 *>(p.ln_out_slots->output[team.stream0 + b])[tid + kThreads * i] = y;
            }
        }
    }
    if constexpr (kQuantised<QT>) {
        float amax[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            amax[b] = 0.0f;
#pragma unroll
            for (int i = 0; i < NVT; ++i)
                if (tid + kThreads * i < nf4)
                    amax[b] = fmaxf(fmaxf(amax[b], fmaxf(fabsf(xr[b][i].x), fabsf(xr[b][i].y))), fmaxf(fabsf(xr[b][i].z), fabsf(xr[b][i].w)));
        }
        block_reduce<BT, true>(amax, s_scratch + 8 * BT, wave);
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float inv = amax[b] > 0.0f ? 127.0f / amax[b] : 0.0f;
            const int stream = team.stream0 + b;
            unsigned char *dst = smem + (size_t)stream * p.k;
#pragma unroll
            for (int i = 0; i < NVT; ++i) {
                const int f = tid + kThreads * i;
                if (f < nf4) {
                    const int q0 = quant_act(xr[b][i].x, inv), q1 = quant_act(xr[b][i].y, inv);
                    const int q2 = quant_act(xr[b][i].z, inv), q3 = quant_act(xr[b][i].w, inv);
                    const int idx = 4 * f;
                    if constexpr (QT == MYNAH_HIP_INT8) {
                        *reinterpret_cast<unsigned *>(dst + idx) = pack_bytes(q0, q1, q2, q3);
                    } else {
                        const int block = idx & ~7, half = (idx & 4) >> 1;
                        *reinterpret_cast<unsigned short *>(dst + block + half) = (unsigned short)((q0 & 0xff) | ((q2 & 0xff) << 8));
                        *reinterpret_cast<unsigned short *>(dst + block + 4 + half) = (unsigned short)((q1 & 0xff) | ((q3 & 0xff) << 8));
                    }
                    if (p.probe_qx != nullptr && blockIdx.x == 0 && stream == 0) {
                        p.probe_qx[idx] = (int8_t)q0; p.probe_qx[idx + 1] = (int8_t)q1;
                        p.probe_qx[idx + 2] = (int8_t)q2; p.probe_qx[idx + 3] = (int8_t)q3;
                    }
                }
            }
            if (tid == 0) {
                // returned activation scale (src/qmat.c:112): amax/127, or amax * f32(1/127) as the stock build folds it
                const float sx = amax[b] > 0.0f ? (p.arith == MYNAH_HIP_ARITH_STOCK ? amax[b] * (1.0f / 127.0f) : amax[b] / 127.0f) : 0.0f;
                s_sx[stream] = sx;
                if (p.probe_sx != nullptr && blockIdx.x == 0 && stream == 0) p.probe_sx[0] = sx;
            }
        }
    } else {
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            float4 *dst = reinterpret_cast<float4 *>(smem) + (size_t)(team.stream0 + b) * nf4;
#pragma unroll
            for (int i = 0; i < NVT; ++i) {
                const int f = tid + kThreads * i;
                if (f < nf4) dst[f] = xr[b][i];
            }
            if (tid == 0) s_sx[team.stream0 + b] = 1.0f;
        }
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------------------------------------------
// One wavefront stages one stream (matvec builds for more than two streams with int8 / int4 weights).  Lane l holds, for
// each of the four "virtual wavefronts" v of the 256-thread scheme above and each i < NVT, the float4 f = 64 v + l + 256 i:
// what thread 64 v + l of that scheme holds, at xr[v * NVT + i].  Every sum is formed per virtual wavefront in that
// thread's order, reduced over the lanes by the same butterfly and combined ((a0 + a1) + a2) + a3 as block_reduce does, so
// the staged bytes of a stream are those of the 256-thread scheme bit for bit -- with no barrier and no exchange through
// LDS: the wavefronts of a workgroup stage their streams independently of each other, where sixteen wavefronts used to
// meet at three workgroup barriers.  (The maximum is exact in any order.)
template <int NVT>
__device__ __forceinline__ void load_stream_row(const PrologueParams &p, const float *row, const bool live, const int lane, float4 (&xr)[4 * NVT],
                                                float4 (&gv)[4 * NVT], float4 (&bv)[4 * NVT]) {
    const int nf4 = p.k >> 2;
    // no request under a condition: a place beyond the row asks for the row's last float4 and is zeroed afterwards
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int i = 0; i < NVT; ++i) {
            const int f = 64 * v + lane + kThreads * i;
            xr[v * NVT + i] = reinterpret_cast<const float4 *>(row)[f < nf4 ? f : nf4 - 1];
        }
    if (p.ln_gain != nullptr) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int i = 0; i < NVT; ++i) {
                const int f = 64 * v + lane + kThreads * i;
                gv[v * NVT + i] = reinterpret_cast<const float4 *>(p.ln_gain)[f < nf4 ? f : nf4 - 1];
                bv[v * NVT + i] = reinterpret_cast<const float4 *>(p.ln_bias != nullptr ? p.ln_bias : p.ln_gain)[f < nf4 ? f : nf4 - 1];
            }
    }
    (void)live;
}

// Second half for one wavefront and its stream: LayerNorm (optional) -> quantisation -> the stream's bytes in LDS.  The caller
// puts one workgroup barrier behind it.  live == false (a place of the batch tile without a stream): zeros are staged.
template <int QT, int NVT>
__device__ __forceinline__ void finish_stream_row(const PrologueParams &p, const int stream, const bool live, const int lane, float4 (&xr)[4 * NVT],
                                                  const float4 (&gv)[4 * NVT], const float4 (&bv)[4 * NVT], unsigned char *smem, float *s_sx) {
    static_assert(kQuantised<QT>, "only the quantising builds stage a stream per wavefront");
    const int nf4 = p.k >> 2;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int i = 0; i < NVT; ++i)
            if (!live || 64 * v + lane + kThreads * i >= nf4) xr[v * NVT + i] = zero;
    const bool first = blockIdx.x == 0 && stream == 0 && live;
    if (p.act_out != nullptr && first) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int i = 0; i < NVT; ++i)
                if (64 * v + lane + kThreads * i < nf4) reinterpret_cast<float4 *>(p.act_out)[64 * v + lane + kThreads * i] = xr[v * NVT + i];
    }
    if (p.ln_gain != nullptr) {
        float part[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < NVT; ++i) s += (xr[v * NVT + i].x + xr[v * NVT + i].y) + (xr[v * NVT + i].z + xr[v * NVT + i].w);
            part[v] = wave_sum(s);
        }
        const float mean = (((part[0] + part[1]) + part[2]) + part[3]) / (float)p.k;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float q = 0.0f;
#pragma unroll
            for (int i = 0; i < NVT; ++i)
                if (64 * v + lane + kThreads * i < nf4) {
                    const float4 x = xr[v * NVT + i];
                    const float d0 = x.x - mean, d1 = x.y - mean, d2 = x.z - mean, d3 = x.w - mean;
                    q = __builtin_fmaf(d0, d0, q);
                    q = __builtin_fmaf(d1, d1, q);
                    q = __builtin_fmaf(d2, d2, q);
                    q = __builtin_fmaf(d3, d3, q);
                }
            part[v] = wave_sum(q);
        }
        const float rstd = 1.0f / sqrtf((((part[0] + part[1]) + part[2]) + part[3]) / (float)p.k + 1.0e-5f);
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int i = 0; i < NVT; ++i) {
                const int f = 64 * v + lane + kThreads * i;
                const float4 x = xr[v * NVT + i], g = f < nf4 ? gv[v * NVT + i] : zero;   // places beyond the row: gain 0 -> 0
                float4 y;
                y.x = ((x.x - mean) * rstd) * g.x;
                y.y = ((x.y - mean) * rstd) * g.y;
                y.z = ((x.z - mean) * rstd) * g.z;
                y.w = ((x.w - mean) * rstd) * g.w;
                if (p.ln_bias != nullptr && f < nf4) {
                    const float4 b = bv[v * NVT + i];
                    y.x += b.x; y.y += b.y; y.z += b.z; y.w += b.w;
                }
                xr[v * NVT + i] = y;
                if (p.ln_out != nullptr && first && f < nf4) reinterpret_cast<float4 *>(p.ln_out)[f] = y;
                if (p.ln_out_slots != nullptr && blockIdx.x == 0 && live && f < nf4) reinterpret_cast<float4 *>(p.ln_out_slots->output[stream])[f] = y;
            }
    }
    float amax = 0.0f;
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int i = 0; i < NVT; ++i)
            if (64 * v + lane + kThreads * i < nf4) {
                const float4 x = xr[v * NVT + i];
                amax = fmaxf(fmaxf(amax, fmaxf(fabsf(x.x), fabsf(x.y))), fmaxf(fabsf(x.z), fabsf(x.w)));
            }
    amax = wave_max(amax);
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    unsigned char *dst = smem + (size_t)stream * p.k;
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int i = 0; i < NVT; ++i) {
            const int f = 64 * v + lane + kThreads * i;
            if (f < nf4) {
                const float4 x = xr[v * NVT + i];
                const int q0 = quant_act(x.x, inv), q1 = quant_act(x.y, inv), q2 = quant_act(x.z, inv), q3 = quant_act(x.w, inv);
                const int idx = 4 * f;
                if constexpr (QT == MYNAH_HIP_INT8) {
                    *reinterpret_cast<unsigned *>(dst + idx) = pack_bytes(q0, q1, q2, q3);
                } else {
                    const int block = idx & ~7, half = (idx & 4) >> 1;
                    *reinterpret_cast<unsigned short *>(dst + block + half) = (unsigned short)((q0 & 0xff) | ((q2 & 0xff) << 8));
                    *reinterpret_cast<unsigned short *>(dst + block + 4 + half) = (unsigned short)((q1 & 0xff) | ((q3 & 0xff) << 8));
                }
                if (p.probe_qx != nullptr && first) {
                    p.probe_qx[idx] = (int8_t)q0; p.probe_qx[idx + 1] = (int8_t)q1;
                    p.probe_qx[idx + 2] = (int8_t)q2; p.probe_qx[idx + 3] = (int8_t)q3;
                }
            }
        }
    if (lane == 0) {
        const float sx = amax > 0.0f ? (p.arith == MYNAH_HIP_ARITH_STOCK ? amax * (1.0f / 127.0f) : amax / 127.0f) : 0.0f;
        s_sx[stream] = sx;
        if (p.probe_sx != nullptr && first) p.probe_sx[0] = sx;
    }
}

template <int QT, int BT, int NVT>
__device__ __forceinline__ void stage_activations(const PrologueParams &p, const ActSource &src, unsigned char *smem, float *s_sx,
                                                  float *s_scratch) {
    float4 xr[BT][NVT], gv[NVT], bv[NVT];
    load_activations<BT, NVT>(p, src, whole_workgroup(), xr, gv, bv);
    finish_activations<QT, BT, NVT>(p, whole_workgroup(), xr, gv, bv, smem, s_sx, s_scratch);
}

}  // namespace mynah
