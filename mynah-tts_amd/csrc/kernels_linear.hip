// Weight-stationary decode matvec for gfx950, fused with its neighbours.
//
// One launch computes, for up to 8 concurrent streams b,
//     out[b] = epilogue( W . prologue(in[b]) )
// prologue : optional LayerNorm (two-pass mean / variance, eps 1e-5, gain and optional bias), then for
//            int8/int4 weights the per-vector absmax int8 activation quantisation
//            (quantize_act_int8, src/qmat.c:94-113) -- each workgroup recomputes it from the 3-12 KB
//            input vector instead of paying a grid-wide dependency for it;
// body     : every 16-byte weight chunk is fetched from HBM exactly once per launch (128-bit loads,
//            a row's chunks spread over a lane group of G lanes so a group reads 16*G contiguous
//            bytes) and dotted against all streams' activations held in LDS: v_dot4_i32_i8 for
//            int8/int4 (dot_q8/dot_q4, src/qmat.c:136-185), f32 FMA of exactly widened halves for f16
//            (matvec_f16, src/qmat.c:306-378), f32 FMA for f32; lane-group butterfly reduction;
// epilogue : ((float)acc * scale[row]) * sx (+ bias), optional tanh-GELU (src/kernels.c:382-389),
//            optional residual accumulate into out (src/graph.c:3212,3254,3275).
//
// Every (row, stream) result is a function of (k, storage type) only: the lane-group width, the
// per-lane chunk order and the reduction tree never depend on the batch size or on which streams
// are live, so a stream inside a batch is bit-identical to the same stream run alone
// (the contract of src/qmat.c:1107-1179).
#include "kernels.h"

namespace mynah {
namespace {

constexpr int kMaxVec = 12;   // prologue keeps k/256 <= 12 float4 per lane (k <= 3072)

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
}

// round half away from zero by truncation, clamp to +-127 (src/qmat.c:106-110)
__device__ __forceinline__ int quant_act(float x, float inv) {
    const float v = x * inv;
    int q = (int)(v >= 0.0f ? v + 0.5f : v - 0.5f);
    q = q > 127 ? 127 : q;
    q = q < -127 ? -127 : q;
    return q;
}

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

template <int QT, int BT>
__global__ void __launch_bounds__(256) k_linear(const LinearArgs a, const int rows_per_wg, const int lg) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float s_sx[BT];
    constexpr bool kQuant = (QT == MYNAH_HIP_INT8 || QT == MYNAH_HIP_INT4);
    constexpr int kEpc = Chunk<QT>::n;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int k = a.k;
    const int nvec = k >> 8;

    // ------------------------------------------------------------------ prologue: one wave per stream
    for (int b = wave; b < BT; b += nwaves) {
        float4 xr[kMaxVec];
        const bool live = b < a.batch;
        const float4 *xin = reinterpret_cast<const float4 *>(live ? a.in[b] : a.in[0]);
#pragma unroll
        for (int i = 0; i < kMaxVec; ++i)
            xr[i] = (live && i < nvec) ? xin[lane + 64 * i] : make_float4(0.f, 0.f, 0.f, 0.f);
        if (a.ln_gain != nullptr && live) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i)
                if (i < nvec) s += (xr[i].x + xr[i].y) + (xr[i].z + xr[i].w);
            const float mean = wave_sum(s) / (float)k;
            float v = 0.0f;
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i)
                if (i < nvec) {
                    const float d0 = xr[i].x - mean, d1 = xr[i].y - mean, d2 = xr[i].z - mean, d3 = xr[i].w - mean;
                    v = __builtin_fmaf(d0, d0, v);
                    v = __builtin_fmaf(d1, d1, v);
                    v = __builtin_fmaf(d2, d2, v);
                    v = __builtin_fmaf(d3, d3, v);
                }
            const float variance = wave_sum(v);
            const float rstd = 1.0f / sqrtf(variance / (float)k + 1.0e-5f);
            const float4 *g4 = reinterpret_cast<const float4 *>(a.ln_gain);
            const float4 *b4 = reinterpret_cast<const float4 *>(a.ln_bias);
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i)
                if (i < nvec) {
                    const float4 g = g4[lane + 64 * i];
                    float4 y;
                    y.x = ((xr[i].x - mean) * rstd) * g.x;
                    y.y = ((xr[i].y - mean) * rstd) * g.y;
                    y.z = ((xr[i].z - mean) * rstd) * g.z;
                    y.w = ((xr[i].w - mean) * rstd) * g.w;
                    if (b4 != nullptr) {
                        const float4 bb = b4[lane + 64 * i];
                        y.x += bb.x; y.y += bb.y; y.z += bb.z; y.w += bb.w;
                    }
                    xr[i] = y;
                }
        }
        if constexpr (kQuant) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i)
                if (i < nvec)
                    amax = fmaxf(fmaxf(amax, fmaxf(fabsf(xr[i].x), fabsf(xr[i].y))), fmaxf(fabsf(xr[i].z), fabsf(xr[i].w)));
            amax = wave_max(amax);
            const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
            unsigned char *dst = smem + (size_t)b * k;
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i)
                if (i < nvec) {
                    const int q0 = quant_act(xr[i].x, inv), q1 = quant_act(xr[i].y, inv);
                    const int q2 = quant_act(xr[i].z, inv), q3 = quant_act(xr[i].w, inv);
                    const int idx = 4 * (lane + 64 * i);
                    if constexpr (QT == MYNAH_HIP_INT8) {
                        const unsigned packed = (unsigned)(q0 & 0xff) | ((unsigned)(q1 & 0xff) << 8) |
                                                ((unsigned)(q2 & 0xff) << 16) | ((unsigned)(q3 & 0xff) << 24);
                        *reinterpret_cast<unsigned *>(dst + idx) = packed;
                    } else {
                        // int4 path: inside each run of 8 activations store [4 even | 4 odd] so they line
                        // up with the low / high nibbles of one weight dword.
                        const int block = idx & ~7, half = (idx & 4) >> 1;
                        *reinterpret_cast<unsigned short *>(dst + block + half) =
                            (unsigned short)((q0 & 0xff) | ((q2 & 0xff) << 8));
                        *reinterpret_cast<unsigned short *>(dst + block + 4 + half) =
                            (unsigned short)((q1 & 0xff) | ((q3 & 0xff) << 8));
                    }
                    if (a.probe_qx != nullptr && blockIdx.x == 0 && b == 0) {
                        a.probe_qx[idx] = (int8_t)q0; a.probe_qx[idx + 1] = (int8_t)q1;
                        a.probe_qx[idx + 2] = (int8_t)q2; a.probe_qx[idx + 3] = (int8_t)q3;
                    }
                }
            if (lane == 0) {
                // returned activation scale (src/qmat.c:112): amax/127, or amax*f32(1/127) as the stock build folds it
                const float sx = amax > 0.0f ? (a.arith == MYNAH_HIP_ARITH_STOCK ? amax * (1.0f / 127.0f) : amax / 127.0f) : 0.0f;
                s_sx[b] = sx;
                if (a.probe_sx != nullptr && blockIdx.x == 0 && b == 0) a.probe_sx[0] = sx;
            }
        } else {
            float4 *dst = reinterpret_cast<float4 *>(smem) + (size_t)b * (k >> 2);
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i)
                if (i < nvec) dst[lane + 64 * i] = xr[i];
            if (lane == 0) s_sx[b] = 1.0f;
        }
    }
    __syncthreads();

    // ------------------------------------------------------------------ body
    const int G = 1 << lg;
    const int gl = lane & (G - 1);
    const int gidx = lane >> lg;
    const int rows_per_pass = 64 >> lg;
    const int chunks = k / kEpc;
    const int row_begin = blockIdx.x * rows_per_wg;
    const int row_end = min(a.n, row_begin + rows_per_wg);
    const size_t row_bytes = (size_t)chunks * 16;

    for (int base = row_begin + wave * rows_per_pass; base < row_end; base += nwaves * rows_per_pass) {
        const int row = base + gidx;
        const bool valid = row < row_end;
        const int rowc = valid ? row : row_end - 1;
        const uint4 *wrow = reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(a.w) + (size_t)rowc * row_bytes);
        const float *srow = (QT == MYNAH_HIP_INT4) ? a.scales + (size_t)rowc * chunks : nullptr;
        int iacc[BT];
        float facc[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) { iacc[b] = 0; facc[b] = 0.0f; }

        for (int c0 = gl; c0 < chunks; c0 += 4 * G) {
            uint4 wv[4];
            float sc[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u * G;
                wv[u] = c < chunks ? wrow[c] : make_uint4(0, 0, 0, 0);
                if constexpr (QT == MYNAH_HIP_INT4) sc[u] = c < chunks ? srow[c] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u * G;
                if (c < chunks) {
                    if constexpr (QT == MYNAH_HIP_INT8) {
#pragma unroll
                        for (int b = 0; b < BT; ++b) {
                            const uint4 xv = *reinterpret_cast<const uint4 *>(smem + (size_t)b * k + (size_t)c * 16);
                            int s = iacc[b];
                            s = dot4(wv[u].x, xv.x, s);
                            s = dot4(wv[u].y, xv.y, s);
                            s = dot4(wv[u].z, xv.z, s);
                            s = dot4(wv[u].w, xv.w, s);
                            iacc[b] = s;
                        }
                    } else if constexpr (QT == MYNAH_HIP_INT4) {
                        unsigned e0, o0, e1, o1, e2, o2, e3, o3;
                        unpack_q4(wv[u].x, e0, o0);
                        unpack_q4(wv[u].y, e1, o1);
                        unpack_q4(wv[u].z, e2, o2);
                        unpack_q4(wv[u].w, e3, o3);
#pragma unroll
                        for (int b = 0; b < BT; ++b) {
                            const uint4 *xp = reinterpret_cast<const uint4 *>(smem + (size_t)b * k + (size_t)c * 32);
                            const uint4 xa = xp[0], xb = xp[1];
                            int gi = 0;
                            gi = dot4(e0, xa.x, gi); gi = dot4(o0, xa.y, gi);
                            gi = dot4(e1, xa.z, gi); gi = dot4(o1, xa.w, gi);
                            gi = dot4(e2, xb.x, gi); gi = dot4(o2, xb.y, gi);
                            gi = dot4(e3, xb.z, gi); gi = dot4(o3, xb.w, gi);
                            // acc += (float)gi * scales[g]  (src/qmat.c:181)
                            const float term = (float)gi * sc[u];
                            facc[b] = facc[b] + term;
                            if (a.probe_acc != nullptr && b == 0 && valid) a.probe_acc[(size_t)row * chunks + c] = gi;
                        }
                    } else if constexpr (QT == MYNAH_HIP_F16) {
                        const unsigned wd[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
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
                        const float w0 = __uint_as_float(wv[u].x), w1 = __uint_as_float(wv[u].y);
                        const float w2 = __uint_as_float(wv[u].z), w3 = __uint_as_float(wv[u].w);
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
            }
        }
        // lane-group butterfly: the same tree for every batch size
        for (int m = G >> 1; m > 0; m >>= 1) {
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                if constexpr (QT == MYNAH_HIP_INT8) iacc[b] += __shfl_xor(iacc[b], m);
                else facc[b] += __shfl_xor(facc[b], m);
            }
        }
        if (gl == 0 && valid) {
            const float wscale = (QT == MYNAH_HIP_INT8) ? a.scales[row] : 1.0f;
            const float bias = a.bias != nullptr ? a.bias[row] : 0.0f;
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                if (b < a.batch) {
                    float val;
                    if constexpr (QT == MYNAH_HIP_INT8) {
                        val = ((float)iacc[b] * wscale) * s_sx[b];
                        if (a.probe_acc != nullptr && b == 0) a.probe_acc[row] = iacc[b];
                    } else if constexpr (QT == MYNAH_HIP_INT4) {
                        val = facc[b] * s_sx[b];
                    } else {
                        val = facc[b];
                    }
                    if (a.bias != nullptr) val += bias;
                    if (a.epilogue == EPI_GELU) val = gelu_tanh(val);
                    float *o = a.out[b] + row;
                    if (a.epilogue == EPI_RESIDUAL) val = *o + val;
                    *o = val;
                }
            }
        }
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

template <int QT, int BT>
int launch_linear_t(State *st, const LinearArgs &a, char *error, size_t capacity) {
    constexpr int epc = Chunk<QT>::n;
    const int chunks = a.k / epc;
    int lg = 6;
    while (lg > 0 && (chunks >> lg) < 3) --lg;
    const int rows_per_pass = 64 >> lg;
    const int threads = a.batch <= 1 ? 64 : (a.batch == 2 ? 128 : 256);
    const int nwaves = threads / 64;
    const int rows_per_wg_pass = rows_per_pass * nwaves;
    const int target_wgs = st->cu_count * 3;
    int passes = (a.n + rows_per_wg_pass * target_wgs - 1) / (rows_per_wg_pass * target_wgs);
    if (passes < 1) passes = 1;
    const int rows_per_wg = rows_per_wg_pass * passes;
    const int grid = (a.n + rows_per_wg - 1) / rows_per_wg;
    const bool quant = (QT == MYNAH_HIP_INT8 || QT == MYNAH_HIP_INT4);
    const size_t lds = (size_t)BT * a.k * (quant ? 1 : 4);
    static bool raised = false;   // per instantiation
    if (lds > 48 * 1024 && !raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_linear<QT, BT>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        raised = true;
    }
    hipLaunchKernelGGL((k_linear<QT, BT>), dim3(grid), dim3(threads), lds, st->stream, a, rows_per_wg, lg);
    return hip_check(hipGetLastError(), "linear launch", error, capacity);
}

template <int QT>
int launch_linear_q(State *st, const LinearArgs &a, char *error, size_t capacity) {
    if (a.batch <= 1) return launch_linear_t<QT, 1>(st, a, error, capacity);
    if (a.batch == 2) return launch_linear_t<QT, 2>(st, a, error, capacity);
    if (a.batch <= 4) return launch_linear_t<QT, 4>(st, a, error, capacity);
    return launch_linear_t<QT, 8>(st, a, error, capacity);
}

}  // namespace

bool linear_fast_supported(int qtype, size_t n, size_t k) {
    if (n == 0 || k == 0 || n > 0x7fffffffu) return false;
    if ((k % 256u) != 0 || k > 256u * kMaxVec) return false;   // prologue: float4 per lane, registers
    return qtype == MYNAH_HIP_F32 || qtype == MYNAH_HIP_F16 || qtype == MYNAH_HIP_INT8 || qtype == MYNAH_HIP_INT4;
}

int launch_linear(State *st, const LinearArgs &a, char *error, size_t capacity) {
    if (a.batch < 1 || a.batch > kBatchTile) {
        set_error(error, capacity, "linear: batch tile out of range");
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

int launch_gemm_f32(State *st, const float *in, float *out, size_t rows, size_t k, size_t n, const float *w,
                    const float *bias, char *error, size_t capacity) {
    if (rows == 0 || n == 0) return 0;
    const dim3 grid((unsigned)((n + 15) / 16), (unsigned)((rows + 15) / 16));
    hipLaunchKernelGGL(k_gemm_nt_f32, grid, dim3(256), 0, st->stream, in, w, bias, out, (int)rows, (int)k, (int)n);
    return hip_check(hipGetLastError(), "gemm launch", error, capacity);
}

int launch_sgemm(State *st, int ta, int tb, size_t m, size_t n, size_t k, float alpha, const float *a, size_t lda,
                 const float *b, size_t ldb, float beta, float *c, size_t ldc, char *error, size_t capacity) {
    if (m == 0 || n == 0) return 0;
    const dim3 grid((unsigned)((n + 15) / 16), (unsigned)((m + 15) / 16));
    hipLaunchKernelGGL(k_sgemm, grid, dim3(256), 0, st->stream, ta, tb, (int)m, (int)n, (int)k, alpha, a, (int)lda, b,
                       (int)ldb, beta, c, (int)ldc);
    return hip_check(hipGetLastError(), "sgemm launch", error, capacity);
}

}  // namespace mynah
