// Text-encoder prefill on the matrix cores: the dense, many-rows twin of the decode step.
//
// encode_text / transformer_stack (src/graph.c:713-748, :634-711) run, per layer, LayerNorm -> QKV
// linear -> per-head scaled QK^T -> row softmax -> PV -> O -> residual -> LayerNorm -> FFN -> residual
// through an f32 BLAS.  Here the weights are f16 (converted once at load, IEEE round to nearest even,
// third_party/ingot/src/dtype.c:246-268), the activations entering a product are rounded to f16, and
// every product accumulates in f32 on v_mfma_f32_32x32x16_f16.  The residual stream, the LayerNorm
// statistics, the softmax and the GELU stay f32.  Attention is bidirectional or causal (the mask of
// src/graph.c:446-449: query t sees keys 0 .. t).  The FFN is causal_conv_ffn (src/graph.c:302-352) with kernel 1
// (two plain products) or kernel 3: out[t][o] = sum_{i,j} W[o][i][j] * in[t - 2 + j][i], rows before the first
// being zero.  The conv is an NT product too: its weights are stored tap-major, W'[o][j * in + i], so that the
// A operand of token t is rows t-2, t-1, t of the activation side by side, and a K step of the product reads one
// of those rows -- addressing only, no unfolded copy.  The two rows before row 0 of nrm and hid exist and stay zero.
//
// Layout in device memory (T tokens padded to a multiple of 64 rows; pad rows are kept finite and are
// masked out as attention keys, so they never reach a real row):
//   x    f32 [Tpad, w]       residual stream
//   nrm  f16 [2 + Tpad, w]   LayerNorm output = A operand of the QKV / FFN-up products (after two zero rows)
//   qk   f16 [2, heads, Tpad/32][2048]   q, then k, operand-major: per (head, 32-token tile) the 32 x 64 block in the order in
//                            which a wavefront's four matrix instructions take it -- element (token r of the tile, d) at
//                            ((d / 16) * 64 + ((d % 16) / 8) * 32 + r) * 8 + d % 8 -- so that one operand request of
//                            the attention kernel is 1 KiB of consecutive bytes (read row-major, lane l: 16 bytes of row
//                            l % 32, a request touches 32 cache lines for 32 bytes each)
//   vt   f16 [heads*2, Tpad/16][512]     v, operand-major for PV (rows = 32 output columns, inner index = 16 keys): element
//                            (d, t) at block (d / 32, t / 16), ((t % 16) / 8 * 32 + d % 32) * 8 + t % 8
//   ctx  f16 [Tpad, w]       attention output = A operand of the O product
//   hid  f16 [2 + Tpad, ffn] GELU(up) = A operand of the FFN-down product (after two zero rows)
//   part f32 [4, Tpad, w]    K-split partial sums of the O and FFN-down products; the row pass that follows
//                            adds them to x in a fixed order (no atomics: results do not depend on scheduling)
//
// All products are "NT": C[m][n] = sum_k A[m][k] * W[n][k], both operands K-contiguous, which is how
// the 32x32x16 MFMA wants them: lane l supplies row (l % 32) of A (or of W) and the eight consecutive
// k values 8*(l / 32) .. +7 of the 16-deep step.
#include <new>

#include "device_common.h"

using namespace mynah;

// Per-call values read by the kernels from device memory, so that one captured graph per padded length
// serves every call: the token count and the caller's output pointers.
struct EncParams {
    int tokens;
    int reserved;
    uint16_t *embed_out;
    float *out;
};

struct mynah_hip_encoder {
    size_t layers = 0, width = 0, heads = 0, head_width = 0, ffn = 0, vocab = 0, max_positions = 0, tpad_max = 0;
    size_t taps = 1;           // FFN conv kernel size, 1 or 3
    int causal = 0;
    const CachedWeight *tok = nullptr, *pos = nullptr;
    std::vector<const CachedWeight *> qkv, o, up, down;
    std::vector<_Float16 *> conv_up, conv_down;   // taps == 3: tap-major f16 copies owned by the encoder
    std::vector<const float *> n1g, n1b, n2g, n2b;
    const float *nog = nullptr, *nob = nullptr;
    float *x = nullptr, *part = nullptr;   // part: [splits, Tpad, w] partial products of the O and FFN-down products
    _Float16 *nrm = nullptr, *qk = nullptr, *vt = nullptr, *ctx = nullptr, *hid = nullptr;
    _Float16 *nrm_alloc = nullptr, *hid_alloc = nullptr;   // nrm and hid begin kLeadRows rows into these
    int *ids = nullptr;        // [tpad_max] token ids, followed by one EncParams
    int *ids_host = nullptr;   // pinned twin of ids
    EncParams *params = nullptr;
    std::unordered_map<int, hipGraphExec_t> graphs;   // by padded length
    std::unordered_map<int, int> eager_runs;          // a padded length runs eagerly once before it is captured
    size_t max_lds = 0;
    // f32 operands (the reference's own arithmetic, src/graph.c:634-711: every product an f32 GEMM): f32 copies of the tables
    // and weights (conv weights tap-major, owned here), and f32 workspaces for exactly max_positions rows
    bool f32 = false;
    const CachedWeight *tok32 = nullptr, *pos32 = nullptr;
    std::vector<const float *> qkv32, o32, up32, down32;
    std::vector<float *> conv32;   // owned tap-major copies behind up32 / down32 when taps == 3
    float *f_nrm = nullptr, *f_qkv = nullptr, *f_scores = nullptr, *f_ctx = nullptr, *f_hid = nullptr, *f_col = nullptr, *f_tmp = nullptr;
    int *f_ids = nullptr;
};

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kTile = 64;            // workgroup tile of the products: 64 x 64, K step 64
constexpr int kLdsStride = 72;       // halfs per staged row: 64 + 8 keeps 16-byte reads of 32 rows off each other's banks
constexpr int kQTile = 32;           // queries per attention workgroup
constexpr int kScorePad = 8;         // floats appended to a score row (bank spread for the row-wise softmax)
constexpr int kGemmDepth = 4;        // K steps of operand tiles in flight in the products (see k_enc_gemm)
constexpr int kLeadRows = 2;         // zero rows in front of the conv FFN's activations (kernel size 3 looks two rows back)

enum { ENC_QKV = 0, ENC_PARTIAL = 1, ENC_GELU = 2 };

struct GemmArgs {
    const _Float16 *a;     // [M, K] row-major, lda = K
    const _Float16 *w;     // [N, K]
    int M, N, K;
    float *part;           // ENC_PARTIAL: part[z][m][n] = this K split's share of the product (summed by the next LayerNorm pass)
    _Float16 *out;         // ENC_QKV: qk [M, 2*width];  ENC_GELU: hid [M, N]
    _Float16 *vt;          // ENC_QKV: v, operand-major (see the layout note)
    int width;
    int taps, cin;         // conv form: K = taps * cin, A is [M, cin] with (taps - 1) zero rows before row 0
};

// tanh-GELU (src/kernels.c:382-389) for a value that is rounded to f16 at once: 0.5 x (1 + tanh c) = x / (1 + e^(-2c)),
// with the hardware exponential and reciprocal (relative error about 1e-6, a five-hundredth of the f16 rounding that
// follows).  c -> -inf gives x * 0, c -> +inf gives x.  The decode step's GELU is gelu_tanh of device_common.h, with tanhf.
__device__ __forceinline__ float gelu_tanh_for_f16(float x) {
    const float cubic = x * x * x;
    const float c = 0.7978845608f * (x + 0.044715f * cubic);
    return x * __builtin_amdgcn_rcpf(1.0f + __expf(-2.0f * c));
}

// Row of C held in accumulator register r of lane l for a 32x32 MFMA tile; the column is l % 32.
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// One K step of both operand tiles on its way from global memory to LDS (four 16-byte pieces per thread).
struct StagedTiles {
    u32x4 a0 = {0, 0, 0, 0}, a1 = {0, 0, 0, 0}, w0 = {0, 0, 0, 0}, w1 = {0, 0, 0, 0};
    __device__ __forceinline__ void load(const u32x4 *ga0, const u32x4 *ga1, const u32x4 *gw0, const u32x4 *gw1, int a_chunk, int w_chunk) {
        a0 = ga0[a_chunk]; a1 = ga1[a_chunk]; w0 = gw0[w_chunk]; w1 = gw1[w_chunk];
    }
    __device__ __forceinline__ void store(_Float16 *sa, _Float16 *sw, int off0, int off1) const {
        *reinterpret_cast<u32x4 *>(sa + off0) = a0;
        *reinterpret_cast<u32x4 *>(sa + off1) = a1;
        *reinterpret_cast<u32x4 *>(sw + off0) = w0;
        *reinterpret_cast<u32x4 *>(sw + off1) = w1;
    }
};

// The fragments of one 64-deep K step of a wavefront's 32 x 32 tile (four 32x32x16 MFMAs), read from LDS into registers
// a step ahead of their use, so that the reads' round trip runs beside the previous step's matrix instructions.
struct StepFragments {
    half8 a[kTile / 16], w[kTile / 16];
    __device__ __forceinline__ void read(const _Float16 *pa, const _Float16 *pw) {
#pragma unroll
        for (int j = 0; j < kTile / 16; ++j) {
            a[j] = *reinterpret_cast<const half8 *>(pa + 16 * j);
            w[j] = *reinterpret_cast<const half8 *>(pw + 16 * j);
        }
    }
    __device__ __forceinline__ void multiply(floatx16 &acc) const {
#pragma unroll
        for (int j = 0; j < kTile / 16; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j], w[j], acc, 0, 0, 0);
    }
};

// D: K steps whose operand tiles are on their way from global memory at any time (even, so that a step's LDS buffer
// is the parity of its register stage; 16 registers per step).
// EXACT: the number of K steps is a multiple of D, and the loop body has no branch at all: every iteration stores,
// requests, reads and multiplies, the requests past the last step repeating the last step's (never used).  This is what
// makes the depth real.  Loads return in order and a wait names how many may still be out, so when a request is issued
// under a condition the compiler must assume it was not, and the wait before storing the oldest block then drains every
// younger one as well: with `if (kt + D < nk)` around the requests the pipeline was one step deep whatever D said.
// Without EXACT (an odd number of steps) the guarded form is used, with that cost.
// CONV: the A operand of K step s is the 64 channels (s % (cin / 64)) * 64 .. of row m - (taps - 1) + s / (cin / 64).
// The fields of GemmArgs as scalar arguments, in the order in which the kernel needs them: the first sixteen dwords of
// scalar kernel arguments are in registers when a wavefront starts (the build asks for that), a structure passed by value
// is fetched from memory.
template <int EPI, int D, bool EXACT, bool CONV>
__global__ void __launch_bounds__(kThreads)
k_enc_gemm(const _Float16 *const a_arg, const _Float16 *const w_arg, const int M, const int N, const int K, const int taps, const int cin,
           const int splits, float *const part, _Float16 *const out, _Float16 *const vt, const int width) {
    GemmArgs g;
    g.a = a_arg; g.w = w_arg; g.M = M; g.N = N; g.K = K; g.part = part; g.out = out; g.vt = vt; g.width = width;
    g.taps = taps; g.cin = cin;
    static_assert(D >= 2 && D % 2 == 0, "stage parity must equal step parity");
    __shared__ __align__(16) _Float16 s_a[2][kTile * kLdsStride];
    __shared__ __align__(16) _Float16 s_w[2][kTile * kLdsStride];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
    // staging: thread -> (row tid / 8 and + 32, 16-byte chunk tid % 8) of both tiles
    const int srow = tid >> 3, schunk = tid & 7;
    const int lda = CONV ? g.cin : g.K;
    const u32x4 *ga0 = reinterpret_cast<const u32x4 *>(g.a + (ptrdiff_t)(m0 + srow) * lda) + schunk;
    const u32x4 *ga1 = reinterpret_cast<const u32x4 *>(g.a + (ptrdiff_t)(m0 + srow + 32) * lda) + schunk;
    const u32x4 *gw0 = reinterpret_cast<const u32x4 *>(g.w + (size_t)(n0 + srow) * g.K) + schunk;
    const u32x4 *gw1 = reinterpret_cast<const u32x4 *>(g.w + (size_t)(n0 + srow + 32) * g.K) + schunk;
    const int soff0 = srow * kLdsStride + schunk * 8, soff1 = (srow + 32) * kLdsStride + schunk * 8;

    // K range of this workgroup (blockIdx.z splits K; only ENC_PARTIAL launches more than one split)
    // (the K split is an argument among the first fourteen dwords, which are in registers at wavefront start; the grid's own
    // dimensions would come out of memory, a round trip in front of the first request)
    const int nk = g.K / kTile / splits;
    const int kbase = (int)blockIdx.z * nk * (kTile / 8);   // in 16-byte chunks
    gw0 += kbase; gw1 += kbase;
    if constexpr (!CONV) { ga0 += kbase; ga1 += kbase; }
    const int first_step = (int)blockIdx.z * nk;
    const int steps_per_tap = CONV ? g.cin / kTile : 1;
    const int row_chunks = lda / 8;   // 16-byte chunks per row of A

    // Global -> register -> LDS -> register pipeline.  Step kt waits in register stage kt % D, is stored to LDS buffer
    // kt % 2 one iteration before its products, and after that iteration's barrier its fragments are read into registers
    // while the matrix instructions of step kt - 1 run from the other fragment set; the same stage then requests step
    // kt + D.  A buffer is overwritten two steps after it was read: every wavefront has passed a barrier in between, which
    // it reaches only with its LDS reads complete.  The products are issued in ascending K order.
    StagedTiles st[D];
    const int last = nk - 1;
    const auto chunk_of = [&](int step) { return (step < last ? step : last) * (kTile / 8); };   // past the end: the last step again
    // chunk offset of a step's A operand from ga0 / ga1: along the row, or (conv form) to an earlier row as well
    const auto a_chunk_of = [&](int step) {
        if constexpr (!CONV) return chunk_of(step);
        else {
            const int s = first_step + (step < last ? step : last);
            const int tap = (s >= steps_per_tap ? 1 : 0) + (s >= 2 * steps_per_tap ? 1 : 0);   // taps <= 3
            return (tap - (g.taps - 1)) * row_chunks + (s - tap * steps_per_tap) * (kTile / 8);
        }
    };
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (EXACT || d < nk) st[d].load(ga0, ga1, gw0, gw1, a_chunk_of(d), chunk_of(d));

    floatx16 acc = {0};
    const int frag = (lane & 31) * kLdsStride + 8 * (lane >> 5);
    const int fa_off = wm * 32 * kLdsStride + frag, fw_off = wn * 32 * kLdsStride + frag;
    StepFragments fr[2];   // fragments of step kt in fr[kt % 2]
    st[0].store(&s_a[0][0], &s_w[0][0], soff0, soff1);
    if (EXACT || D < nk) st[0].load(ga0, ga1, gw0, gw1, a_chunk_of(D), chunk_of(D));
    __syncthreads();
    fr[0].read(&s_a[0][fa_off], &s_w[0][fw_off]);
    // iteration kt: stage step kt + 1, barrier, read its fragments, multiply step kt
    for (int base = 0; base < nk; base += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int kt = base + d;
            const int dn = (d + 1) % D;   // register stage of step kt + 1 (a constant after unrolling)
            if constexpr (EXACT) {
                st[dn].store(&s_a[(d + 1) & 1][0], &s_w[(d + 1) & 1][0], soff0, soff1);
                st[dn].load(ga0, ga1, gw0, gw1, a_chunk_of(kt + 1 + D), chunk_of(kt + 1 + D));
                __syncthreads();
                fr[(d + 1) & 1].read(&s_a[(d + 1) & 1][fa_off], &s_w[(d + 1) & 1][fw_off]);
                fr[d & 1].multiply(acc);
            } else if (kt < nk) {   // the same for every thread of the grid
                if (kt + 1 < nk) {
                    st[dn].store(&s_a[(d + 1) & 1][0], &s_w[(d + 1) & 1][0], soff0, soff1);
                    if (kt + 1 + D < nk) st[dn].load(ga0, ga1, gw0, gw1, a_chunk_of(kt + 1 + D), chunk_of(kt + 1 + D));
                }
                __syncthreads();
                if (kt + 1 < nk) fr[(d + 1) & 1].read(&s_a[(d + 1) & 1][fa_off], &s_w[(d + 1) & 1][fw_off]);
                fr[d & 1].multiply(acc);
            }
        }
    }

    const int n = n0 + wn * 32 + (lane & 31);
    const int mbase = m0 + wm * 32;
    if constexpr (EPI == ENC_PARTIAL) {
        float *part = g.part + (size_t)blockIdx.z * g.M * g.N;
#pragma unroll
        for (int r = 0; r < 16; ++r) part[(size_t)(mbase + acc_row(r, lane)) * g.N + n] = acc[r];
    } else if constexpr (EPI == ENC_GELU) {
#pragma unroll
        for (int r = 0; r < 16; ++r) g.out[(size_t)(mbase + acc_row(r, lane)) * g.N + n] = (_Float16)gelu_tanh_for_f16(acc[r]);
    } else {
        // q, k and v leave in the order in which the attention kernel's matrix instructions take them (see the layout
        // note at the top): a wavefront's 32 x 32 piece lies inside one (part, head, 32-token tile) block.
        const int heads = g.width / 64;
        if (n < 2 * g.width) {   // uniform per workgroup: width is a multiple of the tile
            const int part = n >= g.width ? 1 : 0, d = n & 63, head = (n - part * g.width) >> 6;
            _Float16 *block = g.out + ((size_t)(part * heads + head) * (g.M / 32) + mbase / 32) * 2048 + ((d >> 4) * 64 + ((d >> 3) & 1) * 32) * 8 + (d & 7);
#pragma unroll
            for (int r = 0; r < 16; ++r) block[acc_row(r, lane) * 8] = (_Float16)acc[r];
        } else {
            const int d = n - 2 * g.width;   // d / 32: the (head, 32-column half) block row; d % 32 = lane % 32
            _Float16 *block = g.vt + ((size_t)(d >> 5) * (g.M / 16) + mbase / 16) * 512 + (d & 31) * 8 + 4 * (lane >> 5);
#pragma unroll
            for (int q = 0; q < 4; ++q) {   // registers 4q .. 4q+3 are the four consecutive tokens mbase + 8q + 4 (lane / 32) ..
                half4 v = {(_Float16)acc[4 * q], (_Float16)acc[4 * q + 1], (_Float16)acc[4 * q + 2], (_Float16)acc[4 * q + 3]};
                *reinterpret_cast<half4 *>(block + (q >> 1) * 512 + (q & 1) * 256) = v;
            }
        }
    }
}

// Token gather + position add (src/graph.c:729-737, :649-651).  Rows [tokens, tpad) are zeroed.
__global__ void __launch_bounds__(kThreads) k_enc_embed(const int *ids, const EncParams *params, const _Float16 *tok, const _Float16 *pos,
                                                        float *x, int width) {
    const int t = blockIdx.x;
    const int tokens = params->tokens;
    uint16_t *embed_out = params->embed_out;
    for (int c = threadIdx.x * 8; c < width; c += kThreads * 8) {
        float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
        if (t < tokens) {
            const uint4 traw = *reinterpret_cast<const uint4 *>(tok + (size_t)ids[t] * width + c);
            const half8 tv = *reinterpret_cast<const half8 *>(&traw);
            const half8 pv = *reinterpret_cast<const half8 *>(pos + (size_t)t * width + c);
            if (embed_out != nullptr) *reinterpret_cast<uint4 *>(embed_out + (size_t)t * width + c) = traw;
            lo = make_float4((float)tv[0] + (float)pv[0], (float)tv[1] + (float)pv[1], (float)tv[2] + (float)pv[2], (float)tv[3] + (float)pv[3]);
            hi = make_float4((float)tv[4] + (float)pv[4], (float)tv[5] + (float)pv[5], (float)tv[6] + (float)pv[6], (float)tv[7] + (float)pv[7]);
        }
        *reinterpret_cast<float4 *>(x + (size_t)t * width + c) = lo;
        *reinterpret_cast<float4 *>(x + (size_t)t * width + c + 4) = hi;
    }
}

// Row pass between two products, one wavefront per row: first the residual update
// x += sum over K splits of the previous product's partials (src/graph.c:470, :316), then LayerNorm with
// two-pass statistics (src/kernels.c:186-244, eps 1e-5) written as f16 (operand of the next product) or
// f32 (the encoder's output, to params->out, rows below params->tokens only).  gain == nullptr: no
// LayerNorm, the updated row is copied out as f32.  A lane keeps its NV float4 pieces of the row in
// registers (width <= 256 * NV; the widest supported row, 4096, takes NV = 16).
// (Argument order: what the row's first requests are formed from stands among the first fourteen dwords, which are in registers
// at wavefront start; bias and the f16 destination, needed last, come out of memory.)
// RPW: rows (wavefronts) per workgroup.  One: a row's 3 KB and the up to four partial planes that go with it are 15 KB of
// requests, and four rows to a workgroup put 60 KB through one CU's L1 while three quarters of the CUs have nothing to do
// (256 rows: 64 workgroups) -- a row per workgroup spreads them over the chip.
// No request stands under a condition (a place beyond the row, or a partial plane the product did not write, asks for a
// place that exists and is set to zero afterwards): the waits then name exactly the requests they need.
template <bool F16_OUT, int NV, int RPW>
__global__ void __launch_bounds__(64 * RPW) k_enc_rows(float *x, const float *part, const EncParams *params, int rows, int width, int splits,
                                                        size_t split_stride, const float *gain, const float *bias, _Float16 *out_f16) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * RPW + (threadIdx.x >> 6);
    if (row >= rows) return;
    if constexpr (!F16_OUT) {
        if (row >= params->tokens) return;
    }
    float4 *xr = reinterpret_cast<float4 *>(x + (size_t)row * width);
    const int n4 = width / 4;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 v[NV], gg[NV], bb[NV];
    const float4 *const gain4 = reinterpret_cast<const float4 *>(gain != nullptr ? gain : x);   // (x: a place that exists)
    const float4 *const bias4 = reinterpret_cast<const float4 *>(bias != nullptr ? bias : x);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = lane + 64 * u, at = i < n4 ? i : n4 - 1;
        v[u] = xr[at];
        gg[u] = gain4[at];
        bb[u] = bias4[at];
    }
    if (part != nullptr) {
        // all splits are requested at once and added in split order: the sum does not depend on how the splits were scheduled
        constexpr int kSplits = 4;   // kMaxSplits of the products
        float4 p[kSplits][NV];
#pragma unroll
        for (int z = 0; z < kSplits; ++z) {
            const float4 *const plane = reinterpret_cast<const float4 *>(part + (z < splits ? z : splits - 1) * split_stride + (size_t)row * width);
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                const int i = lane + 64 * u;
                p[z][u] = plane[i < n4 ? i : n4 - 1];
            }
        }
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            if (lane + 64 * u >= n4) v[u] = zero4;
#pragma unroll
            for (int z = 0; z < kSplits; ++z)
                if (z >= splits || lane + 64 * u >= n4) p[z][u] = zero4;
        }
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int i = lane + 64 * u;
            float4 t = p[0][u];
#pragma unroll
            for (int z = 1; z < kSplits; ++z) { t.x += p[z][u].x; t.y += p[z][u].y; t.z += p[z][u].z; t.w += p[z][u].w; }
            v[u].x += t.x; v[u].y += t.y; v[u].z += t.z; v[u].w += t.w;
            if (i < n4) xr[i] = v[u];
        }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const bool in = lane + 64 * u < n4;
        if (!in) v[u] = zero4;
        if (!in || gain == nullptr) gg[u] = zero4;
        if (!in || bias == nullptr) bb[u] = zero4;
    }
    if (gain == nullptr) {
        if constexpr (!F16_OUT) {
#pragma unroll
            for (int u = 0; u < NV; ++u)
                if (lane + 64 * u < n4) reinterpret_cast<float4 *>(params->out + (size_t)row * width)[lane + 64 * u] = v[u];
        }
        return;
    }
    float s = 0.0f;
#pragma unroll
    for (int u = 0; u < NV; ++u) s += (v[u].x + v[u].y) + (v[u].z + v[u].w);   // pieces past the row are zero
    const float mean = wave_sum(s) / (float)width;
    float q = 0.0f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        if (lane + 64 * u < n4) {
            const float a = v[u].x - mean, b = v[u].y - mean, c = v[u].z - mean, d = v[u].w - mean;
            q += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)width + 1.0e-5f);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = lane + 64 * u;
        if (i < n4) {
            const float y0 = (v[u].x - mean) * rstd * gg[u].x + bb[u].x, y1 = (v[u].y - mean) * rstd * gg[u].y + bb[u].y;
            const float y2 = (v[u].z - mean) * rstd * gg[u].z + bb[u].z, y3 = (v[u].w - mean) * rstd * gg[u].w + bb[u].w;
            if constexpr (F16_OUT) {
                half4 h = {(_Float16)y0, (_Float16)y1, (_Float16)y2, (_Float16)y3};
                reinterpret_cast<half4 *>(out_f16 + (size_t)row * width)[i] = h;
            } else {
                reinterpret_cast<float4 *>(params->out + (size_t)row * width)[i] = make_float4(y0, y1, y2, y3);
            }
        }
    }
}

template <bool F16_OUT>
void launch_rows(State *st, int width, dim3 grid, float *x, const float *part, int splits, size_t split_stride, const float *gain,
                 const float *bias, _Float16 *out_f16, const EncParams *params, int rows) {
    (void)grid;
    constexpr int kRowsPerWg = 1;
    const dim3 rows_grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
    if (width <= 1024)
        hipLaunchKernelGGL((k_enc_rows<F16_OUT, 4, kRowsPerWg>), rows_grid, dim3(64 * kRowsPerWg), 0, st->stream, x, part, params, rows, width, splits, split_stride,
                           gain, bias, out_f16);
    else
        hipLaunchKernelGGL((k_enc_rows<F16_OUT, 16, kRowsPerWg>), rows_grid, dim3(64 * kRowsPerWg), 0, st->stream, x, part, params, rows, width, splits, split_stride,
                           gain, bias, out_f16);
}

// One (32-query tile, head): S = scale * Q K^T over all keys (f32, in LDS) -> row softmax numerators
// (f16, written over the row's own storage) and denominators -> O = P V / denom.
// Wavefront w takes key tiles w, w+4, ... for the scores and, for PV, output columns 32*(w & 1) .. +31
// over the key half (w >> 1); the two halves meet in LDS.
// kKeyTiles, kValueSteps: score tiles and PV steps of a wavefront whose fragments are requested up front; the launch
// picks the smallest pair that covers the padded length (up to 4 and 16: 512 tokens), so that none is requested in vain.
template <int kKeyTiles, int kValueSteps>
__global__ void __launch_bounds__(kThreads) k_enc_attention(const _Float16 *qk, const _Float16 *vt, _Float16 *ctx, const EncParams *params,
                                                            int tpad, int width, float scale, int causal) {
    const int tokens = params->tokens;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float s_inv[kQTile];
    __shared__ __align__(16) float s_half[2][16][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q0 = blockIdx.x * kQTile, head = blockIdx.y;
    const int sstride = tpad + kScorePad;                    // floats per score row
    float *S = reinterpret_cast<float *>(smem);

    // ---- every global request of this workgroup is independent of the others and is issued here: the query
    // fragments, the key fragments of this wavefront's first kKeyTiles score tiles and the V fragments of its first
    // kValueSteps PV steps (all of them up to 512 tokens); they are consumed in that order while the rest arrives.
    // None of the requests is under a condition -- a tile or step this call does not have repeats the last one it has and
    // is never used -- so that the number of requests behind each one is a constant: loads return in order, a wait names
    // how many may still be out, and behind a conditional request the compiler has to wait for everything.
    const int heads = width / 64;
    const int ntiles = tpad / 32;
    const int wn = wave & 1, kh = wave >> 1;
    const int kspan = tpad / 2;                              // keys per PV half, multiple of 32
    // Every request is one operand of one matrix instruction for the whole wavefront, 1 KiB of consecutive bytes (see the
    // layout note at the top).
    const half8 *qblock = reinterpret_cast<const half8 *>(qk + ((size_t)head * ntiles + q0 / 32) * 2048) + lane;
    const half8 *kblocks = reinterpret_cast<const half8 *>(qk + (size_t)(heads + head) * ntiles * 2048) + lane;
    const half8 *vblocks = reinterpret_cast<const half8 *>(vt + ((size_t)(head * 2 + wn) * (tpad / 16) + kh * (kspan / 16)) * 512) + lane;
    half8 fq[4], fk[kKeyTiles][4], fv[kValueSteps];
#pragma unroll
    for (int j = 0; j < 4; ++j) fq[j] = qblock[j * 64];
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t) {
        const int tile = min(wave + 4 * t, ntiles - 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) fk[t][j] = kblocks[(size_t)tile * 256 + j * 64];
    }
#pragma unroll
    for (int st = 0; st < kValueSteps; ++st) fv[st] = vblocks[min(st, kspan / 16 - 1) * 64];

    // ---- scores
    {
        auto score_tile = [&](int tile, const half8 (&k4)[4]) {
            floatx16 acc = {0};
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fq[j], k4[j], acc, 0, 0, 0);
            const int key = tile * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                // causal: query q0 + row sees keys up to itself (src/graph.c:446-449); its own key is always in range
                const bool seen = key < tokens && (!causal || key <= q0 + acc_row(r, lane));
                S[acc_row(r, lane) * sstride + key] = seen ? acc[r] * scale : -3.0e38f;
            }
        };
#pragma unroll
        for (int t = 0; t < kKeyTiles; ++t)
            if (wave + 4 * t < ntiles) score_tile(wave + 4 * t, fk[t]);
        for (int tile = wave + 4 * kKeyTiles; tile < ntiles; tile += 4) {   // beyond the tiles requested up front (more than 512 tokens)
            half8 k4[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) k4[j] = kblocks[(size_t)tile * 256 + j * 64];
            score_tile(tile, k4);
        }
    }
    __syncthreads();

    // ---- softmax of row tid / 8 by eight adjacent lanes (softmax_row_inplace, src/graph.c:245-257).  A lane takes
    // float4 pieces part, part + 8, ... of the row (up to kPieces of them in registers, i.e. 1024 keys), so the row is
    // read from LDS once.  The numerators go back as f16 over the first half of the row's own bytes: the eight lanes
    // of a row belong to one wavefront and all of their reads are done before the first of these writes is issued.
    {
        constexpr int kPieces = 32;
        const int row = tid >> 3, part = tid & 7;
        const float4 *srow = reinterpret_cast<const float4 *>(S + row * sstride);
        half4 *prow = reinterpret_cast<half4 *>(S + row * sstride);
        const int npieces = tpad / 4;
        float4 v[kPieces];
        float m = -3.0e38f;
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int c = part + 8 * i;
            if (c < npieces) {
                v[i] = srow[c];
                m = fmaxf(fmaxf(m, fmaxf(v[i].x, v[i].y)), fmaxf(v[i].z, v[i].w));
            }
        }
        m = fmaxf(m, __shfl_xor(m, 1));
        m = fmaxf(m, __shfl_xor(m, 2));
        m = fmaxf(m, __shfl_xor(m, 4));
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int c = part + 8 * i;
            if (c < npieces) {
                // hardware exponential: the numerators are rounded to f16 anyway; masked keys hold -3e38 and give 0
                const float e0 = __expf(v[i].x - m), e1 = __expf(v[i].y - m), e2 = __expf(v[i].z - m), e3 = __expf(v[i].w - m);
                l += (e0 + e1) + (e2 + e3);
                const half4 h = {(_Float16)e0, (_Float16)e1, (_Float16)e2, (_Float16)e3};
                prow[c] = h;
            }
        }
        l += __shfl_xor(l, 1);
        l += __shfl_xor(l, 2);
        l += __shfl_xor(l, 4);
        if (part == 0) s_inv[row] = 1.0f / l;
    }
    __syncthreads();

    // ---- P V
    {
        const _Float16 *prow = reinterpret_cast<const _Float16 *>(S + (lane & 31) * sstride) + kh * kspan + 8 * (lane >> 5);
        floatx16 acc = {0};
#pragma unroll
        for (int st = 0; st < kValueSteps; ++st) {
            if (16 * st < kspan) {
                const half8 fp = *reinterpret_cast<const half8 *>(prow + 16 * st);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fp, fv[st], acc, 0, 0, 0);
            }
        }
        for (int k = 16 * kValueSteps; k < kspan; k += 16) {   // beyond the steps requested up front (more than 512 tokens)
            const half8 fp = *reinterpret_cast<const half8 *>(prow + k);
            const half8 fvk = vblocks[(k / 16) * 64];
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fp, fvk, acc, 0, 0, 0);
        }
        if (kh == 1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s_half[wn][r][lane] = acc[r];
        }
        __syncthreads();
        if (kh == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = acc_row(r, lane);
                const float o = (acc[r] + s_half[wn][r][lane]) * s_inv[row];
                ctx[(size_t)(q0 + row) * width + head * 64 + wn * 32 + (lane & 31)] = (_Float16)o;
            }
        }
    }
}

template <int EPI, bool CONV = false>
int launch_gemm(State *st, const GemmArgs &g, int splits, char *error, size_t capacity) {
    if (g.M % kTile != 0 || g.N % kTile != 0 || g.M <= 0 || g.N <= 0 || g.K <= 0 || splits < 1 || g.K % (kTile * splits) != 0 ||
        (splits > 1 && EPI != ENC_PARTIAL) ||
        (CONV && (g.taps < 1 || g.taps > kLeadRows + 1 || g.cin <= 0 || g.cin % kTile != 0 || g.taps * g.cin != g.K))) {
        set_error(error, capacity, "encoder product: shape is not a multiple of the 64 x 64 x 64 tile");
        return -1;
    }
    const int steps = g.K / kTile / splits;
    const dim3 grid(g.N / kTile, g.M / kTile, splits), block(kThreads);
    if (steps % kGemmDepth == 0)
        hipLaunchKernelGGL((k_enc_gemm<EPI, kGemmDepth, true, CONV>), grid, block, 0, st->stream, g.a, g.w, g.M, g.N, g.K, g.taps, g.cin, splits, g.part, g.out,
                           g.vt, g.width);
    else if (steps % 2 == 0)
        hipLaunchKernelGGL((k_enc_gemm<EPI, 2, true, CONV>), grid, block, 0, st->stream, g.a, g.w, g.M, g.N, g.K, g.taps, g.cin, splits, g.part, g.out, g.vt, g.width);
    else
        hipLaunchKernelGGL((k_enc_gemm<EPI, 2, false, CONV>), grid, block, 0, st->stream, g.a, g.w, g.M, g.N, g.K, g.taps, g.cin, splits, g.part, g.out, g.vt, g.width);
    return hip_check(hipGetLastError(), "encoder product launch", error, capacity);
}

int f16_matrix(State *st, const float *host, size_t n, size_t k, const CachedWeight **out, char *error, size_t capacity) {
    if (cached_matrix(st, host, n, k, MYNAH_HIP_F16, out, error, capacity) != 0) return -1;
    if ((*out)->qtype != MYNAH_HIP_F16) {
        set_error(error, capacity, "encoder: weight shape cannot be stored as f16");
        return -1;
    }
    return 0;
}

// Conv weight [n][cin][taps] (the reference's conv1d layout, src/graph.c:318-352) as f16 [n][taps][cin] in device memory:
// the K order in which k_enc_gemm's conv form walks the activation rows.  The caller owns the allocation.
int tap_major_f16(State *st, const float *host, size_t n, size_t cin, size_t taps, _Float16 **out, char *error, size_t capacity) {
    *out = nullptr;
    std::vector<uint16_t> packed;
    try {
        packed.resize(n * cin * taps);
    } catch (...) {
        set_error(error, capacity, "out of memory converting an encoder conv weight");
        return -1;
    }
    for (size_t o = 0; o < n; ++o)
        for (size_t i = 0; i < cin; ++i)
            for (size_t j = 0; j < taps; ++j) packed[(o * taps + j) * cin + i] = f32_to_f16_rne(host[(o * cin + i) * taps + j]);
    void *dev = nullptr;
    if (hip_check(hipMalloc(&dev, packed.size() * sizeof(uint16_t)), "encoder conv weight", error, capacity) != 0) return -1;
    if (hip_check(hipMemcpy(dev, packed.data(), packed.size() * sizeof(uint16_t), hipMemcpyHostToDevice), "encoder conv weight upload", error, capacity) != 0) {
        (void)hipFree(dev);
        return -1;
    }
    *out = static_cast<_Float16 *>(dev);
    return 0;
}

size_t attention_lds_bytes(size_t tpad) { return (size_t)kQTile * (tpad + kScorePad) * sizeof(float); }

constexpr int kMaxSplits = 4;   // k_enc_rows reads exactly this many partial planes at most
// Most splits that leave each workgroup at least three K steps, preferring a step count the products' pipeline takes
// without guards: a multiple of its depth, else an even one.
int pick_splits(int k) {
    for (const int multiple : {kGemmDepth, 2, 1})
        for (int s = kMaxSplits; s > 1; --s)
            if (k % (kTile * s) == 0 && k / (kTile * s) >= 3 && (k / (kTile * s)) % multiple == 0) return s;
    return 1;
}

// Every kernel of one prefill over `tpad` padded rows, in stream order.  Everything that changes from call to
// call (token count, output pointers) is read from e->params on the device, so the sequence can be captured once.
int enqueue_prefill(State *st, mynah_hip_encoder *e, int tpad, char *error, size_t capacity) {
    const int w = (int)e->width, f = (int)e->ffn;
    hipLaunchKernelGGL(k_enc_embed, dim3(tpad), dim3(kThreads), 0, st->stream, e->ids, e->params, static_cast<const _Float16 *>(e->tok->data),
                       static_cast<const _Float16 *>(e->pos->data), e->x, w);
    const dim3 row_grid((tpad + 3) / 4);
    const float scale = 1.0f / sqrtf((float)e->head_width);
    const size_t lds = attention_lds_bytes((size_t)tpad);
    const size_t split_stride = (size_t)tpad * w;
    // K splits of the two width-wide products (few output tiles, long K): enough workgroups to occupy the chip
    const int taps = (int)e->taps;
    const int o_splits = pick_splits(w), down_splits = pick_splits(f * taps);
    const float *pending = nullptr;   // partials of the last product, not yet added to x
    int pending_splits = 0;
    for (size_t l = 0; l < e->layers; ++l) {
        launch_rows<true>(st, w, row_grid, e->x, pending, pending_splits, split_stride, e->n1g[l], e->n1b[l], e->nrm, e->params, tpad);
        GemmArgs g{};
        g.a = e->nrm; g.w = static_cast<const _Float16 *>(e->qkv[l]->data); g.M = tpad; g.N = 3 * w; g.K = w;
        g.out = e->qk; g.vt = e->vt; g.width = w;
        if (launch_gemm<ENC_QKV>(st, g, 1, error, capacity) != 0) return -1;
        {
            // a wavefront scores every fourth 32-key tile and multiplies half of the keys in steps of 16
            const dim3 agrid(tpad / kQTile, (unsigned)e->heads), ablock(kThreads);
            if (tpad <= 128) hipLaunchKernelGGL((k_enc_attention<1, 4>), agrid, ablock, lds, st->stream, e->qk, e->vt, e->ctx, e->params, tpad, w, scale, e->causal);
            else if (tpad <= 256) hipLaunchKernelGGL((k_enc_attention<2, 8>), agrid, ablock, lds, st->stream, e->qk, e->vt, e->ctx, e->params, tpad, w, scale, e->causal);
            else hipLaunchKernelGGL((k_enc_attention<4, 16>), agrid, ablock, lds, st->stream, e->qk, e->vt, e->ctx, e->params, tpad, w, scale, e->causal);
        }
        g = GemmArgs{};
        g.a = e->ctx; g.w = static_cast<const _Float16 *>(e->o[l]->data); g.M = tpad; g.N = w; g.K = w; g.part = e->part;
        if (launch_gemm<ENC_PARTIAL>(st, g, o_splits, error, capacity) != 0) return -1;
        launch_rows<true>(st, w, row_grid, e->x, e->part, o_splits, split_stride, e->n2g[l], e->n2b[l], e->nrm, e->params, tpad);
        g = GemmArgs{};
        g.a = e->nrm; g.M = tpad; g.N = f; g.K = w * taps; g.out = e->hid; g.taps = taps; g.cin = w;
        g.w = taps > 1 ? e->conv_up[l] : static_cast<const _Float16 *>(e->up[l]->data);
        if ((taps > 1 ? launch_gemm<ENC_GELU, true>(st, g, 1, error, capacity) : launch_gemm<ENC_GELU>(st, g, 1, error, capacity)) != 0) return -1;
        g = GemmArgs{};
        g.a = e->hid; g.M = tpad; g.N = w; g.K = f * taps; g.part = e->part; g.taps = taps; g.cin = f;
        g.w = taps > 1 ? e->conv_down[l] : static_cast<const _Float16 *>(e->down[l]->data);
        if ((taps > 1 ? launch_gemm<ENC_PARTIAL, true>(st, g, down_splits, error, capacity)
                      : launch_gemm<ENC_PARTIAL>(st, g, down_splits, error, capacity)) != 0)
            return -1;
        pending = e->part;
        pending_splits = down_splits;
    }
    // last residual update, then the final norm (src/graph.c:696-701) or a plain copy when the stack has none
    launch_rows<false>(st, w, row_grid, e->x, pending, pending_splits, split_stride, e->nog, e->nob, nullptr, e->params, tpad);
    return hip_check(hipGetLastError(), "encoder prefill launch", error, capacity);
}

// ---- f32 operands: the stack as the reference computes it ---------------------------------------------------------------
// transformer_stack (src/graph.c:634-711) is LayerNorm -> QKV linear -> per head sgemm(Q K^T, alpha = scale) -> masked row
// softmax -> sgemm(P V) -> O linear -> residual -> LayerNorm -> causal_conv_ffn -> residual, all f32.  This form runs exactly
// that sequence on the library's f32 operators (LayerNorm rows, the f32 matrix-core product, GELU with tanhf, residual add),
// so that only the order of additions inside a product differs from the CPU: 1e-5 instead of the 2e-3 of f16 operands.
// It is the accuracy form, not the fast one: some forty launches per layer, no graph.

// Row r = h * T + t of the scores [heads, T, T]: softmax over the keys the query may see (src/graph.c:446-449 masks key > query;
// softmax_row_inplace, src/graph.c:245-257: max, exp, sum, divide), zeros behind them.
__global__ void __launch_bounds__(256) k_enc_softmax_rows(float *scores, int T, int causal) {
    __shared__ float s4[4];
    const int t = (int)(blockIdx.x % (unsigned)T);
    float *row = scores + (size_t)blockIdx.x * T;
    const int valid = causal ? t + 1 : T;
    float m = -3.0e38f;
    for (int i = threadIdx.x; i < valid; i += 256) m = fmaxf(m, row[i]);
    m = block_max(m, s4);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < valid; i += 256) {
        const float e = expf(row[i] - m);
        row[i] = e;
        sum += e;
    }
    sum = block_sum(sum, s4);
    for (int i = threadIdx.x; i < T; i += 256) row[i] = i < valid ? row[i] / sum : 0.0f;
}

// unfold_causal (src/graph.c:271-286) in the tap-major order of the conv weights here: col[t][j * C + i] = in[t - (taps - 1) + j][i],
// zero for rows before the first.
__global__ void __launch_bounds__(256) k_enc_unfold(const float *in, float *col, int T, int C, int taps) {
    const size_t n = (size_t)T * taps * C;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (size_t)gridDim.x * 256) {
        const int i = (int)(idx % (size_t)C);
        const size_t tj = idx / (size_t)C;
        const int j = (int)(tj % (size_t)taps);
        const int t = (int)(tj / (size_t)taps);
        const int src = t - (taps - 1) + j;
        col[idx] = src >= 0 ? in[(size_t)src * C + i] : 0.0f;
    }
}

// Conv weight [n][cin][taps] as f32 [n][taps][cin] in device memory (the caller owns it).
int tap_major_f32(const float *host, size_t n, size_t cin, size_t taps, float **out, char *error, size_t capacity) {
    *out = nullptr;
    std::vector<float> packed;
    try {
        packed.resize(n * cin * taps);
    } catch (...) {
        set_error(error, capacity, "out of memory converting an encoder conv weight");
        return -1;
    }
    for (size_t o = 0; o < n; ++o)
        for (size_t i = 0; i < cin; ++i)
            for (size_t j = 0; j < taps; ++j) packed[(o * taps + j) * cin + i] = host[(o * cin + i) * taps + j];
    void *dev = nullptr;
    if (hip_check(hipMalloc(&dev, packed.size() * sizeof(float)), "encoder conv weight", error, capacity) != 0) return -1;
    if (hip_check(hipMemcpy(dev, packed.data(), packed.size() * sizeof(float), hipMemcpyHostToDevice), "encoder conv weight upload", error, capacity) != 0) {
        (void)hipFree(dev);
        return -1;
    }
    *out = static_cast<float *>(dev);
    return 0;
}

int f32_matrix(State *st, const float *host, size_t n, size_t k, const CachedWeight **out, char *error, size_t capacity) {
    return cached_matrix(st, host, n, k, MYNAH_HIP_F32, out, error, capacity);
}

int prefill_f32(State *st, mynah_hip_encoder *e, int T, float *dev_out, char *error, size_t capacity) {
    const size_t w = e->width, f = e->ffn, taps = e->taps, heads = e->heads, hw = e->head_width;
    const float scale = 1.0f / sqrtf((float)hw);
    const float *tables[1] = {static_cast<const float *>(e->tok32->data)};
    if (launch_gather(st, tables, 1, e->f_ids, (size_t)T, w, 1.0f, static_cast<const float *>(e->pos32->data), e->x, error, capacity) != 0) return -1;
    for (size_t l = 0; l < e->layers; ++l) {
        if (launch_layernorm(st, e->x, e->f_nrm, e->n1g[l], e->n1b[l], (size_t)T, w, error, capacity) != 0) return -1;
        if (launch_gemm_f32(st, e->f_nrm, e->f_qkv, (size_t)T, w, 3 * w, e->qkv32[l], nullptr, error, capacity) != 0) return -1;
        for (size_t h = 0; h < heads; ++h)   // scores_h = scale * Q_h K_h^T (src/graph.c:428-445)
            if (launch_sgemm(st, 0, 1, (size_t)T, (size_t)T, hw, scale, e->f_qkv + h * hw, 3 * w, e->f_qkv + w + h * hw, 3 * w, 0.0f,
                             e->f_scores + h * (size_t)T * T, (size_t)T, error, capacity) != 0)
                return -1;
        hipLaunchKernelGGL(k_enc_softmax_rows, dim3((unsigned)(heads * (size_t)T)), dim3(256), 0, st->stream, e->f_scores, T, e->causal);
        MYNAH_TRY(hipGetLastError());
        for (size_t h = 0; h < heads; ++h)   // ctx_h = P_h V_h (src/graph.c:451-462)
            if (launch_sgemm(st, 0, 0, (size_t)T, hw, (size_t)T, 1.0f, e->f_scores + h * (size_t)T * T, (size_t)T, e->f_qkv + 2 * w + h * hw, 3 * w, 0.0f,
                             e->f_ctx + h * hw, w, error, capacity) != 0)
                return -1;
        if (launch_gemm_f32(st, e->f_ctx, e->f_tmp, (size_t)T, w, w, e->o32[l], nullptr, error, capacity) != 0) return -1;
        if (launch_residual(st, e->x, e->f_tmp, (size_t)T * w, error, capacity) != 0) return -1;
        if (launch_layernorm(st, e->x, e->f_nrm, e->n2g[l], e->n2b[l], (size_t)T, w, error, capacity) != 0) return -1;
        const float *up_in = e->f_nrm;
        if (taps > 1) {
            hipLaunchKernelGGL(k_enc_unfold, dim3(1024), dim3(256), 0, st->stream, e->f_nrm, e->f_col, T, (int)w, (int)taps);
            MYNAH_TRY(hipGetLastError());
            up_in = e->f_col;
        }
        if (launch_gemm_f32(st, up_in, e->f_hid, (size_t)T, w * taps, f, e->up32[l], nullptr, error, capacity) != 0) return -1;
        if (launch_gelu(st, e->f_hid, (size_t)T * f, error, capacity) != 0) return -1;
        const float *down_in = e->f_hid;
        if (taps > 1) {
            hipLaunchKernelGGL(k_enc_unfold, dim3(1024), dim3(256), 0, st->stream, e->f_hid, e->f_col, T, (int)f, (int)taps);
            MYNAH_TRY(hipGetLastError());
            down_in = e->f_col;
        }
        if (launch_gemm_f32(st, down_in, e->f_tmp, (size_t)T, f * taps, w, e->down32[l], nullptr, error, capacity) != 0) return -1;
        if (launch_residual(st, e->x, e->f_tmp, (size_t)T * w, error, capacity) != 0) return -1;
    }
    if (e->nog != nullptr) return launch_layernorm(st, e->x, dev_out, e->nog, e->nob, (size_t)T, w, error, capacity);
    return launch_copy(st, dev_out, e->x, (size_t)T * w, error, capacity);
}

}  // namespace

extern "C" int mynah_hip_encoder_create(void *state, const mynah_hip_encoder_desc *d, mynah_hip_encoder **out, char *error, size_t capacity) {
    State *st = enter_state(state);
    if (out != nullptr) *out = nullptr;
    if (st == nullptr || d == nullptr || out == nullptr) {
        set_error(error, capacity, "encoder_create: null argument");
        return -1;
    }
    if (d->layers == 0 || d->width == 0 || d->heads == 0 || d->heads * d->head_width != d->width || d->head_width != 64 ||
        d->width % kTile != 0 || d->ffn_width % kTile != 0 || d->ffn_width == 0 || d->vocab == 0 || d->max_positions == 0 ||
        d->width > 4096 || d->ffn_width > 32768 || d->max_positions > 4096 || d->tok_table == nullptr || d->pos_table == nullptr ||
        d->qkv_w == nullptr || d->o_w == nullptr || d->up_w == nullptr || d->down_w == nullptr || d->norm1 == nullptr || d->norm2 == nullptr) {
        set_error(error, capacity, "encoder_create: unsupported shape (needs 64-wide heads, widths that are multiples of 64) or missing weights");
        return -1;
    }
    if (d->ffn_kernel != 0 && d->ffn_kernel != 1 && d->ffn_kernel != 3) {
        set_error(error, capacity, "encoder_create: ffn_kernel must be 1 or 3");
        return -1;
    }
    auto *e = new (std::nothrow) mynah_hip_encoder();
    if (e == nullptr) {
        set_error(error, capacity, "out of memory creating the encoder");
        return -1;
    }
    e->layers = d->layers; e->width = d->width; e->heads = d->heads; e->head_width = d->head_width; e->ffn = d->ffn_width;
    e->vocab = d->vocab; e->max_positions = d->max_positions;
    e->taps = d->ffn_kernel == 3 ? 3 : 1;
    e->causal = d->causal != 0;
    e->tpad_max = (d->max_positions + kTile - 1) / kTile * kTile;
    int lds = 0;
    if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, 0) != hipSuccess || lds <= 0) lds = 65536;
    e->max_lds = (size_t)lds;
    auto fail = [&](void) { mynah_hip_encoder_destroy(state, e); return -1; };
    if (e->tpad_max > 1024 || attention_lds_bytes(e->tpad_max) + 10 * 1024 > e->max_lds) {   // 1024: a softmax lane keeps 32 float4 pieces of its row
        set_error(error, capacity, "encoder_create: max_positions beyond 1024, or more LDS per workgroup than this device has");
        return fail();
    }
    e->f32 = d->operands_f32 != 0;
    if (e->f32) {
        if (f32_matrix(st, d->tok_table, d->vocab, d->width, &e->tok32, error, capacity) != 0) return fail();
        if (f32_matrix(st, d->pos_table, d->max_positions, d->width, &e->pos32, error, capacity) != 0) return fail();
    } else {
        if (f16_matrix(st, d->tok_table, d->vocab, d->width, &e->tok, error, capacity) != 0) return fail();
        if (f16_matrix(st, d->pos_table, d->max_positions, d->width, &e->pos, error, capacity) != 0) return fail();
    }
    for (size_t l = 0; l < d->layers; ++l) {
        const CachedWeight *cw = nullptr;
        const float *v = nullptr;
        if (d->qkv_w[l] == nullptr || d->o_w[l] == nullptr || d->up_w[l] == nullptr || d->down_w[l] == nullptr || d->norm1[l] == nullptr ||
            d->norm2[l] == nullptr) {
            set_error(error, capacity, "encoder_create: missing layer weight");
            return fail();
        }
        if (e->f32) {
            if (f32_matrix(st, d->qkv_w[l], 3 * d->width, d->width, &cw, error, capacity) != 0) return fail();
            e->qkv32.push_back(static_cast<const float *>(cw->data));
            if (f32_matrix(st, d->o_w[l], d->width, d->width, &cw, error, capacity) != 0) return fail();
            e->o32.push_back(static_cast<const float *>(cw->data));
            if (e->taps == 1) {
                if (f32_matrix(st, d->up_w[l], d->ffn_width, d->width, &cw, error, capacity) != 0) return fail();
                e->up32.push_back(static_cast<const float *>(cw->data));
                if (f32_matrix(st, d->down_w[l], d->width, d->ffn_width, &cw, error, capacity) != 0) return fail();
                e->down32.push_back(static_cast<const float *>(cw->data));
            } else {
                float *dev = nullptr;
                if (tap_major_f32(d->up_w[l], d->ffn_width, d->width, e->taps, &dev, error, capacity) != 0) return fail();
                e->conv32.push_back(dev);
                e->up32.push_back(dev);
                if (tap_major_f32(d->down_w[l], d->width, d->ffn_width, e->taps, &dev, error, capacity) != 0) return fail();
                e->conv32.push_back(dev);
                e->down32.push_back(dev);
            }
        } else {
        if (f16_matrix(st, d->qkv_w[l], 3 * d->width, d->width, &cw, error, capacity) != 0) return fail();
        e->qkv.push_back(cw);
        if (f16_matrix(st, d->o_w[l], d->width, d->width, &cw, error, capacity) != 0) return fail();
        e->o.push_back(cw);
        if (e->taps == 1) {
            if (f16_matrix(st, d->up_w[l], d->ffn_width, d->width, &cw, error, capacity) != 0) return fail();
            e->up.push_back(cw);
            if (f16_matrix(st, d->down_w[l], d->width, d->ffn_width, &cw, error, capacity) != 0) return fail();
            e->down.push_back(cw);
        } else {
            _Float16 *dev = nullptr;
            if (tap_major_f16(st, d->up_w[l], d->ffn_width, d->width, e->taps, &dev, error, capacity) != 0) return fail();
            e->conv_up.push_back(dev);
            if (tap_major_f16(st, d->down_w[l], d->width, d->ffn_width, e->taps, &dev, error, capacity) != 0) return fail();
            e->conv_down.push_back(dev);
        }
        }
        if (cached_vector(st, d->norm1[l], d->width, &v, error, capacity) != 0) return fail();
        e->n1g.push_back(v);
        v = nullptr;
        if (d->norm1_bias != nullptr && d->norm1_bias[l] != nullptr && cached_vector(st, d->norm1_bias[l], d->width, &v, error, capacity) != 0) return fail();
        e->n1b.push_back(v);
        if (cached_vector(st, d->norm2[l], d->width, &v, error, capacity) != 0) return fail();
        e->n2g.push_back(v);
        v = nullptr;
        if (d->norm2_bias != nullptr && d->norm2_bias[l] != nullptr && cached_vector(st, d->norm2_bias[l], d->width, &v, error, capacity) != 0) return fail();
        e->n2b.push_back(v);
    }
    if (d->norm_out != nullptr && cached_vector(st, d->norm_out, d->width, &e->nog, error, capacity) != 0) return fail();
    if (d->norm_out != nullptr && d->norm_out_bias != nullptr && cached_vector(st, d->norm_out_bias, d->width, &e->nob, error, capacity) != 0) return fail();
    const size_t tp = e->tpad_max, w = e->width, f = e->ffn;
    auto alloc = [&](void **p, size_t bytes) {
        if (hip_check(hipMalloc(p, bytes), "encoder workspace", error, capacity) != 0) return -1;
        return hip_check(hipMemsetAsync(*p, 0, bytes, st->stream), "encoder workspace clear", error, capacity);
    };
    if (e->f32) {
        const size_t T = d->max_positions, wide = (w > f ? w : f) * e->taps;
        if (alloc(reinterpret_cast<void **>(&e->x), T * w * sizeof(float)) != 0 || alloc(reinterpret_cast<void **>(&e->f_nrm), T * w * sizeof(float)) != 0 ||
            alloc(reinterpret_cast<void **>(&e->f_qkv), T * 3 * w * sizeof(float)) != 0 ||
            alloc(reinterpret_cast<void **>(&e->f_scores), e->heads * T * T * sizeof(float)) != 0 ||
            alloc(reinterpret_cast<void **>(&e->f_ctx), T * w * sizeof(float)) != 0 || alloc(reinterpret_cast<void **>(&e->f_hid), T * f * sizeof(float)) != 0 ||
            alloc(reinterpret_cast<void **>(&e->f_col), T * wide * sizeof(float)) != 0 || alloc(reinterpret_cast<void **>(&e->f_tmp), T * w * sizeof(float)) != 0 ||
            alloc(reinterpret_cast<void **>(&e->f_ids), T * sizeof(int)) != 0)
            return fail();
        if (hip_check(hipHostMalloc(reinterpret_cast<void **>(&e->ids_host), T * sizeof(int), hipHostMallocDefault), "encoder ids staging", error, capacity) != 0)
            return fail();
        if (hip_check(hipStreamSynchronize(st->stream), "encoder create", error, capacity) != 0) return fail();
        *out = e;
        return 0;
    }
    if (alloc(reinterpret_cast<void **>(&e->x), tp * w * sizeof(float)) != 0 || alloc(reinterpret_cast<void **>(&e->nrm_alloc), (kLeadRows + tp) * w * 2) != 0 ||
        alloc(reinterpret_cast<void **>(&e->qk), tp * 2 * w * 2) != 0 || alloc(reinterpret_cast<void **>(&e->vt), w * tp * 2) != 0 ||
        alloc(reinterpret_cast<void **>(&e->ctx), tp * w * 2) != 0 || alloc(reinterpret_cast<void **>(&e->hid_alloc), (kLeadRows + tp) * f * 2) != 0 ||
        alloc(reinterpret_cast<void **>(&e->ids), tp * sizeof(int) + sizeof(EncParams)) != 0 ||
        alloc(reinterpret_cast<void **>(&e->part), kMaxSplits * tp * w * sizeof(float)) != 0)
        return fail();
    if (hip_check(hipHostMalloc(reinterpret_cast<void **>(&e->ids_host), tp * sizeof(int) + sizeof(EncParams), hipHostMallocDefault),
                  "encoder ids staging", error, capacity) != 0)
        return fail();
    e->params = reinterpret_cast<EncParams *>(e->ids + tp);   // tp is a multiple of 64: 8-byte aligned
    e->nrm = e->nrm_alloc + kLeadRows * w;   // rows -2 and -1 stay zero; widths are multiples of 64, so both stay 16-byte aligned
    e->hid = e->hid_alloc + kLeadRows * f;
    if (attention_lds_bytes(e->tpad_max) > 48 * 1024) {
        const int bytes = (int)attention_lds_bytes(e->tpad_max);
        if (hip_check(hipFuncSetAttribute(reinterpret_cast<const void *>(k_enc_attention<1, 4>), hipFuncAttributeMaxDynamicSharedMemorySize, bytes), "encoder attention LDS size", error, capacity) != 0 ||
            hip_check(hipFuncSetAttribute(reinterpret_cast<const void *>(k_enc_attention<2, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, bytes), "encoder attention LDS size", error, capacity) != 0 ||
            hip_check(hipFuncSetAttribute(reinterpret_cast<const void *>(k_enc_attention<4, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, bytes), "encoder attention LDS size", error, capacity) != 0)
            return fail();
    }
    if (hip_check(hipStreamSynchronize(st->stream), "encoder create", error, capacity) != 0) return fail();
    *out = e;
    return 0;
}

extern "C" void mynah_hip_encoder_destroy(void *state, mynah_hip_encoder *e) {
    State *st = enter_state(state);
    if (e == nullptr) return;
    if (st != nullptr) (void)hipStreamSynchronize(st->stream);
    for (auto &g : e->graphs)
        if (g.second != nullptr) (void)hipGraphExecDestroy(g.second);
    for (void *p : {(void *)e->x, (void *)e->nrm_alloc, (void *)e->qk, (void *)e->vt, (void *)e->ctx, (void *)e->hid_alloc, (void *)e->ids, (void *)e->part})
        if (p != nullptr) (void)hipFree(p);
    for (_Float16 *p : e->conv_up) (void)hipFree(p);
    for (_Float16 *p : e->conv_down) (void)hipFree(p);
    for (float *p : e->conv32) (void)hipFree(p);
    for (void *p : {(void *)e->f_nrm, (void *)e->f_qkv, (void *)e->f_scores, (void *)e->f_ctx, (void *)e->f_hid, (void *)e->f_col, (void *)e->f_tmp, (void *)e->f_ids})
        if (p != nullptr) (void)hipFree(p);
    if (e->ids_host != nullptr) (void)hipHostFree(e->ids_host);
    delete e;
}

extern "C" int mynah_hip_encoder_prefill(void *state, mynah_hip_encoder *e, const int32_t *ids, size_t tokens, uint16_t *dev_embed_f16,
                                         float *dev_out, char *error, size_t capacity) {
    State *st = enter_state(state);
    if (st == nullptr || e == nullptr || ids == nullptr || dev_out == nullptr) {
        set_error(error, capacity, "encoder_prefill: null argument");
        return -1;
    }
    if (tokens == 0 || tokens > e->max_positions) {
        set_error(error, capacity, "encoder_prefill: token count outside [1, max_positions]");
        return -1;
    }
    for (size_t t = 0; t < tokens; ++t) {
        if (ids[t] < 0 || (size_t)ids[t] >= e->vocab) {   // src/graph.c:730-735
            set_error(error, capacity, "encoder_prefill: token id out of range");
            return -1;
        }
    }
    // the staging buffer of the previous call may still be in flight
    MYNAH_TRY(hipStreamSynchronize(st->stream));
    if (e->f32) {
        if (dev_embed_f16 != nullptr) {
            set_error(error, capacity, "encoder_prefill: with f32 operands there are no f16 token rows to return");
            return -1;
        }
        for (size_t t = 0; t < tokens; ++t) e->ids_host[t] = ids[t];
        MYNAH_TRY(hipMemcpyAsync(e->f_ids, e->ids_host, tokens * sizeof(int), hipMemcpyHostToDevice, st->stream));
        return prefill_f32(st, e, (int)tokens, dev_out, error, capacity);
    }
    const size_t tp = e->tpad_max;
    for (size_t t = 0; t < tokens; ++t) e->ids_host[t] = ids[t];
    EncParams *hp = reinterpret_cast<EncParams *>(e->ids_host + tp);
    hp->tokens = (int)tokens;
    hp->reserved = 0;
    hp->embed_out = dev_embed_f16;
    hp->out = dev_out;
    MYNAH_TRY(hipMemcpyAsync(e->ids, e->ids_host, tokens * sizeof(int), hipMemcpyHostToDevice, st->stream));
    MYNAH_TRY(hipMemcpyAsync(e->params, hp, sizeof(EncParams), hipMemcpyHostToDevice, st->stream));

    const int tpad = ((int)tokens + kTile - 1) / kTile * kTile;
    if (!st->graph_mode || e->eager_runs[tpad] == 0) {
        e->eager_runs[tpad] = 1;
        return enqueue_prefill(st, e, tpad, error, capacity);
    }
    hipGraphExec_t &exec = e->graphs[tpad];
    if (exec == nullptr) {
        hipGraph_t graph = nullptr;
        MYNAH_TRY(hipStreamBeginCapture(st->stream, hipStreamCaptureModeThreadLocal));
        const int rc = enqueue_prefill(st, e, tpad, error, capacity);
        const hipError_t end = hipStreamEndCapture(st->stream, &graph);
        if (rc != 0 || end != hipSuccess) {
            if (graph != nullptr) (void)hipGraphDestroy(graph);
            if (rc == 0) (void)hip_check(end, "encoder graph capture", error, capacity);
            return -1;
        }
        const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (hip_check(inst, "encoder graph instantiate", error, capacity) != 0) {
            exec = nullptr;
            return -1;
        }
    }
    return hip_check(hipGraphLaunch(exec, st->stream), "encoder graph launch", error, capacity);
}
