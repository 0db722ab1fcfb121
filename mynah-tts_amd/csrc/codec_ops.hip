// Codec operators of the resident NanoCodec decode (decode_codec_resident, src/graph.c:2504-2638; res_layer_device
// :2423-2498): causal dilated conv1d, grouped causal transposed conv and the half-snake activation, on device rows of
// layout [channels, length].  Weights, biases and snake alphas arrive as HOST pointers and are cached on the device at
// first sight like every other weight (the seam's contract).  None of the three synchronises.
//
//   conv1d          out[o][t] = bias[o] + sum_i sum_k w[(o*in + i)*K + k] * in[i][t - (K-1-k)*dilation]   (conv1d_causal,
//                   src/graph.c:2010-2160).  The reference builds an im2col matrix and calls sgemm; here the same GEMM
//                   (M = out channels, N = length, inner = in channels x taps) runs on the f32 matrix cores with the
//                   im2col done by addressing: a workgroup stages the input rows of eight channels once, with a halo of
//                   (K-1)*dilation positions, and every tap reads the same rows at its own offset.  f32 operands,
//                   f32 accumulation (v_mfma_f32_32x32x2_f32); only the order of the additions differs from the CPU's.
//   conv_transpose  grouped, trimmed to output_length (conv_transpose_causal / convt_channel, src/graph.c:2179-2231):
//                   one thread per output element, contributions added in the reference's order (input channel, then
//                   input position), so the result is bit-identical to the scalar CPU loop.
//   snake           x + sin(a x)^2 * (1 / (a + 1e-9)) on the first snake_channels rows, leaky ReLU (0.01) on the rest
//                   (snake_row, src/backend.c:643-658).
#include <limits.h>

#include <type_traits>

#include "kernels.h"

using namespace mynah;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kConvMaxKernel = 16;
constexpr int kConvMaxHalo = 128;     // (kernel - 1) * dilation
constexpr int kTileStride = 65;       // floats per row of a wavefront's 32 x 64 tile in LDS (fused epilogue)

struct ConvArgs {
    const float *in;     // [in_ch, length]
    float *out;          // [out_ch, length]
    const float *bias;   // [out_ch] or null
    int in_ch, out_ch, length, kernel, dilation;
    // what mynah_hip_conv1d_fused adds after conv + bias, in this order (each step is the arithmetic of the seam operator it replaces)
    const float *residual = nullptr;    // [out_ch, length] added (residual_inplace); may be `out` itself
    const float *residual2 = nullptr;   // then this one
    float scale = 1.0f;                 // then multiplied (scale_dev) when `scaled`
    int scaled = 0;
    int activate = 0;                   // then the half-snake of the value's output channel (snake_dev)
    const float *alpha = nullptr;       // [snake_channels]
    int snake_channels = 0;
    float *act_out = nullptr;           // null: `out` gets the activated value; else `out` keeps the value before it and this gets the activated one
};

// sin(x) in some twenty instructions for |x| < kShortSineLimit (the library routine, which also serves arguments of any
// size, is about 150, and inside a convolution's epilogue nothing hides them): x = k * pi/2 + r with pi/2 in three pieces
// and fused multiply-adds, then the sine or cosine polynomial of r on [-pi/4, pi/4] (Cephes' single-precision
// coefficients).  Largest difference from the double-precision sine over every 7th float of (-8192, 8192): 9.3e-8, against
// 6e-8 for a correctly rounded result near 1.
constexpr float kShortSineLimit = 8192.0f;
__device__ __forceinline__ float short_sine(float x) {
    const float k = __builtin_rintf(x * 0.636619772367581343f);
    float r = __builtin_fmaf(k, -1.57079637050628662109375f, x);
    r = __builtin_fmaf(k, 4.37113882867379289e-8f, r);
    r = __builtin_fmaf(k, 1.71512460692744033e-15f, r);
    const float z = r * r;
    const float s = __builtin_fmaf(r * z, __builtin_fmaf(z, __builtin_fmaf(z, -1.9515295891e-4f, 8.3321608736e-3f), -1.6666654611e-1f), r);
    const float c = __builtin_fmaf(z * z, __builtin_fmaf(z, __builtin_fmaf(z, 2.443315711809948e-5f, -1.388731625493765e-3f), 4.166664568298827e-2f),
                                   __builtin_fmaf(z, -0.5f, 1.0f));
    const int q = (int)k;
    const float v = (q & 1) ? c : s;
    return (q & 2) ? -v : v;
}
// The codec's sine: the short routine where it holds, the library's beyond.
__device__ __forceinline__ float snake_sine(float x) { return fabsf(x) < kShortSineLimit ? short_sine(x) : sinf(x); }

// snake_row, src/backend.c:643-658.  inv_a = 1 / (alpha + 1e-9) for a snake row; a row past snake_channels is a leaky ReLU.
__device__ __forceinline__ float half_snake(float v, bool snake_row, float al, float inv_a) {
    if (snake_row) {
        const float sn = snake_sine(al * v);
        return v + sn * sn * inv_a;
    }
    return v < 0.0f ? v * 0.01f : v;
}

// One finished output value (conv + bias) on its way to memory, in two steps so that a kernel can run the first (two
// requests and three operations) for all of a thread's values at once, requests side by side, and the second (some
// hundred instructions when there is an activation) in a rolled loop.
__device__ __forceinline__ float conv_combine(const ConvArgs &a, size_t index, float v) {
    if (a.residual != nullptr) v = a.residual[index] + v;
    if (a.residual2 != nullptr) v = a.residual2[index] + v;
    return v * a.scale;   // 1.0f when there is no scaling: the value's own bits
}
// al, inv_a: the output channel's alpha and 1 / (alpha + 1e-9), which the kernels keep in LDS: read from global memory value
// by value inside the rolled loops, that request was most of what an activation cost.
__device__ __forceinline__ void conv_emit(const ConvArgs &a, int m, size_t index, float v, float al, float inv_a) {
    if (a.activate) {
        const float act = half_snake(v, m < a.snake_channels, al, inv_a);
        if (a.act_out != nullptr) {
            a.out[index] = v;
            a.act_out[index] = act;
        } else {
            a.out[index] = act;
        }
    } else {
        a.out[index] = v;
    }
}

// The products of one staged block of eight input channels for a wavefront's 32 x 64 tile.  The two inner indices one
// matrix instruction consumes are the same tap of two neighbouring channels (lanes 0-31: the even channel, lanes 32-63:
// the odd one), so a lane walks its channel's taps with plain increments.  wrow: this lane's output row at its first
// channel; irow: its first channel's staged row at its output position.
// With the tap count known at compile time the operands are requested TWO products ahead and the scheduler is fenced
// around every product: left to itself the compiler reads a product's input operand into one and the same register right
// before it, and with one wavefront on a SIMD every product then waits out an LDS read (some 120 cycles against the 64
// of the instruction itself).  Past the last product the requests stay inside the staging area and are not used.
// pairs: channel pairs of the block that exist (the tensor's last block may hold fewer than four; the rest is zeros in
// both operands and is left out -- the same for every lane of the wavefront).
template <int KF, int NT = 2>
__device__ __forceinline__ void conv_products(const float *wrow, const float *irow, const int kernel_arg, const int dilation, const int win,
                                              floatx16 &acc0, floatx16 &acc1, const int pairs = kConvChannels / 2) {
    if constexpr (KF != 0) {
        constexpr int kSteps = (kConvChannels / 2) * KF;
        float wv[3], x0[3], x1[3];
        int tap = 0;
        const auto request = [&](int slot) {
            wv[slot] = wrow[0];
            x0[slot] = irow[0];
            x1[slot] = NT > 1 ? irow[32] : 0.0f;
            const bool wrap = tap + 1 == KF;   // then: the first tap of the next channel pair
            wrow += wrap ? KF + 1 : 1;
            irow += wrap ? 2 * win - (KF - 1) * dilation : dilation;
            tap = wrap ? 0 : tap + 1;
        };
        request(0);
        request(1);
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            if (s % KF == 0 && s != 0 && s / KF >= pairs) break;   // (looked at where a pair begins)
            request((s + 2) % 3);
            __builtin_amdgcn_sched_barrier(0x77);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[s % 3], x0[s % 3], acc0, 0, 0, 0);
            if constexpr (NT > 1) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[s % 3], x1[s % 3], acc1, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0x77);
        }
        return;
    }
    const int kernel = kernel_arg;
    float wv = wrow[0], x0 = irow[0], x1 = NT > 1 ? irow[32] : 0.0f;
#pragma unroll
    for (int pair = 0; pair < kConvChannels / 2; ++pair) {
        for (int k = 0; k < kernel; ++k) {
            // the product after this one: the next tap, or the first tap of the next channel pair
            const bool wrap = k + 1 == kernel;
            wrow += wrap ? kernel + 1 : 1;
            irow += wrap ? 2 * win - (kernel - 1) * dilation : dilation;
            const float nw = wrow[0], n0 = irow[0], n1 = NT > 1 ? irow[32] : 0.0f;
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(wv, x0, acc0, 0, 0, 0);
            if constexpr (NT > 1) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wv, x1, acc1, 0, 0, 0);
            wv = nw; x0 = n0; x1 = n1;
        }
    }
}

// Workgroup tile: (32 * WM) output channels x (64 * WN) positions; a wavefront owns 32 x 64 (two 32 x 32 accumulators).
// KF: number of taps known at compile time (0 = from the arguments): the staging loops then have exactly as many slots as
// the block has 16-byte pieces and the product loop is straight-line code.  The codec's 3, 7 and 11 taps get such builds.
// The weights arrive cut into chunks (ConvBlocks): the tile's block of a step is WM whole chunks in a row, already in the
// layout LDS keeps, so staging it is a plain copy -- no index arithmetic, no bounds.
// FUSED: the build that mynah_hip_conv1d_fused launches (residuals, scale, activation after the products); the seam's
// conv1d keeps a build without any of it.
// (the tile's work as a function: the kernel of one convolution and the kernel of several side by side both run it)
// LEAN: the residual values are requested in the epilogue instead of before the last block's products (64 registers less:
// the build that runs several convolutions side by side wants three workgroups on a CU).
template <int WM, int WN, int KF, bool FUSED, bool LEAN = false>
__device__ __forceinline__ void conv_tile(const ConvArgs &a_arg, const float *const chunks_arg, const int tiles_arg, float *const lds) {
    constexpr int TM = 32 * WM, TN = 64 * WN;
    ConvArgs a = a_arg;
    if constexpr (KF != 0) a.kernel = KF;
    const int kb = kConvChannels * a.kernel;   // inner elements per step
    const int a_stride = kb + 4;               // the chunks' row stride: rows stay 16-byte aligned, and a stride of 4 mod 8 words
                                               // spreads the 32 rows a wavefront reads for a product over eight banks
    const int halo = (a.kernel - 1) * a.dilation;
    const int win = TN + halo;                 // staged positions per input channel
    // 16-byte pieces of the tile's weight block, and the slots (one piece per thread) that cover them; the last slot may
    // reach past the block, into the next chunk or the zeros after the last one, and lands in LDS the products never read
    constexpr int kSlots = (WM * 8 * (kConvChannels * (KF != 0 ? KF : kConvMaxKernel) + 4) + 255) / 256;
    const int pieces = WM * 8 * a_stride;
    const int slots = KF != 0 ? kSlots : (pieces + 255) / 256;
    // (the input rows first: their LDS addresses are then the staged positions themselves, with nothing to add per request)
    float *s_in = lds;                         // [kConvChannels][win]
    float *s_w = lds + kConvChannels * win;    // [TM][a_stride], then the last slot's excess; 16-byte aligned
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int m0 = blockIdx.y * TM, t0 = blockIdx.x * TN;

    // Staging slots of a thread: weights -- piece tid + 256 * c of the block; input rows -- channel ch, position
    // tid + 256 * x of the window (its place in the row is the same for every block: kept, -1 outside the row).
    constexpr int kWinParts = (TN + kConvMaxHalo + 255) / 256;
    floatx4 stage_w[kSlots];
    float stage_in[kConvChannels][kWinParts];
    int in_pos[kWinParts];
#pragma unroll
    for (int x = 0; x < kWinParts; ++x) {
        const int xx = tid + 256 * x, t = t0 - halo + xx;
        in_pos[x] = (xx < win && t >= 0 && t < a.length) ? t : -1;
    }
    const floatx4 *w_next = reinterpret_cast<const floatx4 *>(chunks_arg) + (size_t)(WM * blockIdx.y) * (8 * a_stride) + tid;   // this thread's first piece
    const size_t w_step = (size_t)tiles_arg * (8 * a_stride);   // pieces from a block to the next
    const auto fetch = [&](int i0) {   // global -> registers: the weight block and input rows of channels [i0, i0 + 8); nothing waits here
#pragma unroll
        for (int c = 0; c < kSlots; ++c)
            if (KF != 0 || c < slots) stage_w[c] = w_next[256 * c];
        w_next += w_step;
#pragma unroll
        for (int ch = 0; ch < kConvChannels; ++ch) {
            const bool row_exists = i0 + ch < a.in_ch;
            const float *row = a.in + (row_exists ? (size_t)(i0 + ch) * a.length : 0);
#pragma unroll
            for (int x = 0; x < kWinParts; ++x) stage_in[ch][x] = row[in_pos[x] >= 0 ? in_pos[x] : 0];   // always a legal address
        }
    };
    const auto publish = [&](int i0) {   // registers -> LDS (zeros where the input has no such channel or position)
#pragma unroll
        for (int c = 0; c < kSlots; ++c)
            if (KF != 0 || c < slots) reinterpret_cast<floatx4 *>(s_w)[tid + 256 * c] = stage_w[c];
#pragma unroll
        for (int ch = 0; ch < kConvChannels; ++ch) {
            const bool row_exists = i0 + ch < a.in_ch;
#pragma unroll
            for (int x = 0; x < kWinParts; ++x) {
                const int xx = tid + 256 * x;
                if (xx < win) s_in[ch * win + xx] = (row_exists && in_pos[x] >= 0) ? stage_in[ch][x] : 0.0f;
            }
        }
    };

    // The accumulators start from the rows' biases (requested here, beside the first block: at the end each would be a
    // round trip of its own in front of the stores), so a value is bias + products in the products' order.
    const int half = lane >> 5, col = lane & 31;
    floatx16 acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        acc0[r] = (a.bias != nullptr && m < a.out_ch) ? a.bias[m] : 0.0f;
    }
    acc1 = acc0;
    // The fused build's residual values are requested before the last block's products instead of behind them (a round
    // trip in front of the stores otherwise); a residual may be the output itself -- every workgroup reads and writes its
    // own tile only.
    float res_first[FUSED ? 32 : 1], res_second[FUSED ? 32 : 1];
    const auto request_residuals = [&]() {
        if constexpr (FUSED) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                const int t = t0 + wn * 64 + col;
                const bool in0 = m < a.out_ch && t < a.length, in1 = m < a.out_ch && t + 32 < a.length;
                const size_t i0 = in0 ? (size_t)m * a.length + t : 0, i1 = in1 ? (size_t)m * a.length + t + 32 : 0;
                if (a.residual != nullptr) { res_first[r] = a.residual[i0]; res_first[16 + r] = a.residual[i1]; }
                if (a.residual2 != nullptr) { res_second[r] = a.residual2[i0]; res_second[16 + r] = a.residual2[i1]; }
            }
        }
    };
    fetch(0);
    for (int i0 = 0; i0 < a.in_ch; i0 += kConvChannels) {
        publish(i0);
        __syncthreads();
        if (i0 + kConvChannels < a.in_ch) fetch(i0 + kConvChannels);   // in flight during the products below
        else if constexpr (!LEAN) request_residuals();
        conv_products<KF>(s_w + (wm * 32 + col) * a_stride + half * a.kernel, s_in + half * win + wn * 64 + col, a.kernel, a.dilation,
                          win, acc0, acc1, min(kConvChannels / 2, (a.in_ch - i0 + 1) / 2));
        __syncthreads();
    }
    // accumulator element r of a lane: row 8 * (r / 4) + 4 * (lane / 32) + r % 4, column lane % 32
    // conv + bias, then the residuals (requested before the last products, to a legal address whatever the value's place)
    // and the scale, in conv_combine's order, without a branch per value: an addition that is not wanted at all is left out
    // by the build of this loop that runs.
    // A finished tile on its way to memory: from the accumulators' layout (a store instruction there covers 32 positions of
    // two rows, and a row's validity differs between the halves of a wavefront: a mask and a branch per store) through the
    // wavefront's own piece of LDS (free after the last products' barrier) to whole rows of 64 consecutive positions, whose
    // validity is the same for every lane -- a loop over the rows that exist, the positions' own check once around it.
    const auto store_tile = [&](float *dst, const floatx16 &first, const floatx16 &second) {
        float *s_tile = lds + wave * (32 * kTileStride);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 8 * (r >> 2) + 4 * half + (r & 3);
            s_tile[row * kTileStride + col] = first[r];
            s_tile[row * kTileStride + col + 32] = second[r];
        }
        const int t = t0 + wn * 64 + lane;
        const int rows = min(32, a.out_ch - (m0 + wm * 32));   // the same for the whole wavefront
        if (t < a.length) {
            float *p = dst + (size_t)(m0 + wm * 32) * a.length + t;
#pragma unroll 8
            for (int row = 0; row < rows; ++row, p += a.length) *p = s_tile[row * kTileStride + lane];
        }
    };
    if constexpr (LEAN) request_residuals();
    const auto combine = [&](auto has_first, auto has_second) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float v0 = acc0[r], v1 = acc1[r];
            if constexpr (decltype(has_first)::value) { v0 = res_first[r] + v0; v1 = res_first[16 + r] + v1; }
            if constexpr (decltype(has_second)::value) { v0 = res_second[r] + v0; v1 = res_second[16 + r] + v1; }
            if constexpr (FUSED) {
                v0 = v0 * a.scale;   // 1.0f when there is no scaling: the value's own bits
                v1 = v1 * a.scale;
            }
            acc0[r] = v0;
            acc1[r] = v1;
        }
        if (!FUSED || !a.activate) store_tile(a.out, acc0, acc1);
    };
    if constexpr (!FUSED) {   // the seam's conv1d
        combine(std::false_type{}, std::false_type{});
        return;
    }
    if (a.residual2 != nullptr) combine(std::true_type{}, std::true_type{});    // the launch refuses a second residual without a first
    else if (a.residual != nullptr) combine(std::true_type{}, std::false_type{});
    else combine(std::false_type{}, std::false_type{});
    if (!a.activate) return;
    // The rows' alphas and 1 / (alpha + 1e-9) through the wavefront's own piece of LDS (free after the last products' barrier)
    float *s_alpha = lds + 4 * (32 * kTileStride) + wave * 64;
    if (lane < 32) {
        const int m = m0 + wm * 32 + lane;
        const float al = m < a.snake_channels ? a.alpha[m] : 0.0f;
        s_alpha[lane] = al;
        s_alpha[32 + lane] = 1.0f / (al + 1e-9f);
    }
    // Common case, every sine argument below the short routine's limit: the activation on the values where they are, in
    // registers, the short sine inlined 32 times and no branch among them.
    bool large = false;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float al = s_alpha[8 * (r >> 2) + 4 * half + (r & 3)];
        large = large || !(fabsf(al * acc0[r]) < kShortSineLimit) || !(fabsf(al * acc1[r]) < kShortSineLimit);
    }
    if (!__any(large)) {
        floatx16 act0, act1;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 8 * (r >> 2) + 4 * half + (r & 3), m = m0 + wm * 32 + row;
            const float al = s_alpha[row], inv_a = s_alpha[32 + row];
            const float v0 = acc0[r], v1 = acc1[r];
            const float s0 = short_sine(al * v0), s1 = short_sine(al * v1);
            const bool snake_row = m < a.snake_channels;
            act0[r] = snake_row ? v0 + s0 * s0 * inv_a : (v0 < 0.0f ? v0 * 0.01f : v0);
            act1[r] = snake_row ? v1 + s1 * s1 * inv_a : (v1 < 0.0f ? v1 * 0.01f : v1);
        }
        if (a.act_out != nullptr) {
            store_tile(a.out, acc0, acc1);
            store_tile(a.act_out, act0, act1);
        } else {
            store_tile(a.out, act0, act1);
        }
        return;
    }
    // Some argument needs the library's sine: the wavefront's 32 x 64 tile goes through LDS and a rolled loop finishes it
    // a row at a time, with one copy of that long routine.
    float *s_tile = lds + wave * (32 * kTileStride);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * half + (r & 3);
        s_tile[row * kTileStride + col] = acc0[r];
        s_tile[row * kTileStride + col + 32] = acc1[r];
    }
    const int t = t0 + wn * 64 + lane;
    if (t >= a.length) return;
    const int rows = min(32, a.out_ch - (m0 + wm * 32));   // the same for the whole wavefront
    size_t index = (size_t)(m0 + wm * 32) * a.length + t;
#pragma unroll 1
    for (int row = 0; row < rows; ++row, index += a.length)
        conv_emit(a, m0 + wm * 32 + row, index, s_tile[row * kTileStride + lane], s_alpha[row], s_alpha[32 + row]);
}

template <int WM, int WN, int KF, bool FUSED>
__global__ void __launch_bounds__(256) k_conv1d(const float *const in_arg, float *const out_arg, const float *const chunks_arg, const float *const bias_arg, const int in_ch_arg,
                                                const int out_ch_arg, const int length_arg, const int kernel_arg, const int dilation_arg, const int tiles_arg,
                                                const ConvArgs a_arg) {
    extern __shared__ __align__(16) float lds[];
    // (the rows, the weights and the shape lead the arguments and repeat fields of a_arg: leading scalar arguments are in
    // registers when a wavefront starts, a structure passed by value is fetched from memory where its fields are first used)
    ConvArgs a = a_arg;
    a.in = in_arg; a.out = out_arg; a.bias = bias_arg; a.in_ch = in_ch_arg; a.out_ch = out_ch_arg; a.length = length_arg;
    a.kernel = kernel_arg; a.dilation = dilation_arg;
    conv_tile<WM, WN, KF, FUSED>(a, chunks_arg, tiles_arg, lds);
}

// The same product for short rows (few positions, many channels: the codec's first stages), where 64 x 128 tiles would
// leave most of the chip idle: a workgroup owns a 32 x 64 tile and its four wavefronts split the input channels between
// them (wavefront w takes channel blocks w, w + 4, ...: one weight chunk each), each staging its own blocks in its own
// part of LDS; the four partial tiles are added in wavefront order at the end, so the result does not depend on timing.
// NT: 32-position halves per tile (2, or 1 for the very shortest rows: twice the workgroups).
template <int KF, int NT>
__device__ __forceinline__ void conv_split_tile(const ConvArgs &a_arg, const float *const chunks_arg, const int tiles_arg, float *const lds) {
    constexpr int TM = 32, TN = 32 * NT;
    ConvArgs a = a_arg;
    if constexpr (KF != 0) a.kernel = KF;
    const int kb = kConvChannels * a.kernel;
    const int a_stride = kb + 4;   // the chunks' row stride (see k_conv1d)
    const int halo = (a.kernel - 1) * a.dilation;
    const int win = TN + halo;
    // a chunk is 8 * a_stride 16-byte pieces; a lane's slots (one piece each) cover it, the last one possibly reaching past
    // it (into the next chunk or the zeros after the last one: LDS the products never read)
    constexpr int kSlots = (8 * (kConvChannels * (KF != 0 ? KF : kConvMaxKernel) + 4) + 63) / 64;
    const int slots = KF != 0 ? kSlots : (8 * a_stride + 63) / 64;
    const int per_wave = slots * 256 + kConvChannels * win;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float *s_in = lds + wave * per_wave;       // [kConvChannels][win] of this wavefront
    float *s_w = s_in + kConvChannels * win;   // [TM][a_stride], then the last slot's excess; 16-byte aligned
    const int m0 = blockIdx.y * TM, t0 = blockIdx.x * TN;
    constexpr int kWinParts = (TN + kConvMaxHalo + 63) / 64;

    floatx16 acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
    const int half = lane >> 5, col = lane & 31;
    const int blocks = (a.in_ch + kConvChannels - 1) / kConvChannels;
    const int rounds = (blocks + 3) / 4;   // the same count for every wavefront (a block past the end is a chunk of zeros)
    floatx4 stage_w[kSlots];
    float stage_in[kConvChannels][kWinParts];
    int in_pos[kWinParts];    // input: position in the row, the same in every round (-1: outside the row or the window)
#pragma unroll
    for (int x = 0; x < kWinParts; ++x) {
        const int xx = lane + 64 * x, t = t0 - halo + xx;
        in_pos[x] = (xx < win && t >= 0 && t < a.length) ? t : -1;
    }
    // this lane's first piece of the wavefront's first chunk; four blocks on from round to round
    const floatx4 *w_next = reinterpret_cast<const floatx4 *>(chunks_arg) + ((size_t)wave * tiles_arg + blockIdx.y) * (8 * a_stride) + lane;
    const size_t w_step = (size_t)4 * tiles_arg * (8 * a_stride);
    const auto fetch = [&](int round) {   // global -> registers: this wavefront's channel block of the round; nothing waits here
        const int i0 = (4 * round + wave) * kConvChannels;
#pragma unroll
        for (int c = 0; c < kSlots; ++c)
            if (KF != 0 || c < slots) stage_w[c] = w_next[64 * c];
        w_next += w_step;
#pragma unroll
        for (int ch = 0; ch < kConvChannels; ++ch) {
            const bool row_exists = i0 + ch < a.in_ch;
            const float *row = a.in + (row_exists ? (size_t)(i0 + ch) * a.length : 0);
#pragma unroll
            for (int x = 0; x < kWinParts; ++x) stage_in[ch][x] = row[in_pos[x] >= 0 ? in_pos[x] : 0];   // always a legal address
        }
    };
    fetch(0);
    for (int round = 0; round < rounds; ++round) {
        const int i0 = (4 * round + wave) * kConvChannels;
#pragma unroll
        for (int c = 0; c < kSlots; ++c)
            if (KF != 0 || c < slots) reinterpret_cast<floatx4 *>(s_w)[lane + 64 * c] = stage_w[c];
#pragma unroll
        for (int ch = 0; ch < kConvChannels; ++ch) {
            const bool row_exists = i0 + ch < a.in_ch;
#pragma unroll
            for (int x = 0; x < kWinParts; ++x) {
                const int xx = lane + 64 * x;
                if (xx < win) s_in[ch * win + xx] = (row_exists && in_pos[x] >= 0) ? stage_in[ch][x] : 0.0f;
            }
        }
        // (no workgroup barrier in the loop: a wavefront stages into its own part of LDS and reads nothing else, and its own
        // LDS accesses complete in the order it issued them -- the four wavefronts walk their channel blocks independently)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        if (round + 1 < rounds) fetch(round + 1);   // in flight during the products below
        conv_products<KF, NT>(s_w + col * a_stride + half * a.kernel, s_in + half * win + col, a.kernel, a.dilation, win, acc0, acc1);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    __syncthreads();   // the partial tiles below overwrite every wavefront's staging area
    // partial tiles through LDS: [wavefront][element r][lane], then ((p0 + p1) + p2) + p3 + bias
    float *s_part = lds;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s_part[(wave * 32 + r) * 64 + lane] = acc0[r];
        s_part[(wave * 32 + 16 + r) * 64 + lane] = acc1[r];
    }
    __syncthreads();
    // A thread finishes the tile's values at (row (tid / 64) + 4 j, position tid % 64): a store instruction then covers one
    // row's 64 consecutive positions and whether the row exists is the same for all its lanes (in the accumulators' order an
    // instruction covers halves of two rows, four apart).  e: where that value sits in a partial tile (element r of lane l).
    const int pos = tid & 63;
    const int t = t0 + pos;
    const bool t_ok = (NT > 1 || pos < 32) && t < a.length;
    float value[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int row = (tid >> 6) + 4 * j, m = m0 + row;
        const int e = ((((row >> 3) << 2) | (row & 3)) + 16 * (pos >> 5)) * 64 + ((row >> 2) & 1) * 32 + (pos & 31);
        const float sum = ((s_part[e] + s_part[2048 + e]) + s_part[4096 + e]) + s_part[6144 + e];
        value[j] = 0.0f;
        if (t_ok && m < a.out_ch) value[j] = conv_combine(a, (size_t)m * a.length + t, sum + (a.bias != nullptr ? a.bias[m] : 0.0f));
    }
    if (!a.activate) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = m0 + (tid >> 6) + 4 * j;
            if (t_ok && m < a.out_ch) a.out[(size_t)m * a.length + t] = value[j];
        }
        return;
    }
    // with an activation: the values go back through LDS (a thread reads what it wrote) so that one copy of the
    // activation's code serves the eight of them
    float *s_alpha = lds + 4 * 32 * 64;   // [32] alpha, [32] 1 / (alpha + 1e-9) of the tile's rows
    if (tid < 32) {
        const float al = m0 + tid < a.snake_channels ? a.alpha[m0 + tid] : 0.0f;
        s_alpha[tid] = al;
        s_alpha[32 + tid] = 1.0f / (al + 1e-9f);
    }
    __syncthreads();   // every sum has been read
#pragma unroll
    for (int j = 0; j < 8; ++j) s_part[tid + 256 * j] = value[j];
#pragma unroll 2
    for (int j = 0; j < 8; ++j) {
        const int row = (tid >> 6) + 4 * j, m = m0 + row;
        if (t_ok && m < a.out_ch) conv_emit(a, m, (size_t)m * a.length + t, s_part[tid + 256 * j], s_alpha[row], s_alpha[32 + row]);
    }
}

template <int KF, int NT>
__global__ void __launch_bounds__(256) k_conv1d_split(const float *const in_arg, float *const out_arg, const float *const chunks_arg, const float *const bias_arg, const int in_ch_arg,
                                                      const int out_ch_arg, const int length_arg, const int kernel_arg, const int dilation_arg, const int tiles_arg,
                                                      const ConvArgs a_arg) {
    extern __shared__ __align__(16) float lds[];
    // (leading scalar arguments: see k_conv1d)
    ConvArgs a = a_arg;
    a.in = in_arg; a.out = out_arg; a.bias = bias_arg; a.in_ch = in_ch_arg; a.out_ch = out_ch_arg; a.length = length_arg;
    a.kernel = kernel_arg; a.dilation = dilation_arg;
    conv_split_tile<KF, NT>(a, chunks_arg, tiles_arg, lds);
}

// Several convolutions of one shape side by side in one launch (the three branches of a residual layer: same rows in and
// out, own weights, taps, dilation and epilogue): blockIdx.z names the convolution, every workgroup runs the tile's work of
// its own, so the values are those of the single launches.  A launch's fixed cost (dispatch, kernel start, the first
// block's round trip, the stores behind the last product) is paid once for all of them, and a CU holds workgroups of
// different convolutions whose staging and products overlap.  Tap counts 3, 7 and 11 only (the builds with straight-line
// products); always the build with the fused epilogue (with nothing to add it leaves the product's own bits).
constexpr int kConvBatchMax = 4;
struct ConvBatchArgs {
    ConvArgs item[kConvBatchMax];
    const float *chunks[kConvBatchMax];
    int tiles;
};

// (three wavefronts per SIMD asked of the compiler: alone, a 256-thread workgroup is given every register of the CU)
template <int WM, int WN>
__global__ void __launch_bounds__(256, 3) k_conv1d_batch(const ConvBatchArgs b) {
    extern __shared__ __align__(16) float lds[];
    const int z = blockIdx.z;
    switch (b.item[z].kernel) {
        case 3: conv_tile<WM, WN, 3, true, true>(b.item[z], b.chunks[z], b.tiles, lds); break;
        case 7: conv_tile<WM, WN, 7, true, true>(b.item[z], b.chunks[z], b.tiles, lds); break;
        default: conv_tile<WM, WN, 11, true, true>(b.item[z], b.chunks[z], b.tiles, lds); break;
    }
}

template <int NT>
__global__ void __launch_bounds__(256, 2) k_conv1d_split_batch(const ConvBatchArgs b) {
    extern __shared__ __align__(16) float lds[];
    const int z = blockIdx.z;
    switch (b.item[z].kernel) {
        case 3: conv_split_tile<3, NT>(b.item[z], b.chunks[z], b.tiles, lds); break;
        case 7: conv_split_tile<7, NT>(b.item[z], b.chunks[z], b.tiles, lds); break;
        default: conv_split_tile<11, NT>(b.item[z], b.chunks[z], b.tiles, lds); break;
    }
}

struct ConvTransposeArgs {
    const float *in;     // [in_ch, length]
    float *out;          // [out_ch, output_length]
    const float *w;      // [in_ch, out_ch / groups, kernel]
    const float *bias;   // [out_ch] or null
    int in_ch, out_ch, length, output_length, kernel, stride, groups;
};

__global__ void __launch_bounds__(256) k_conv_transpose(const ConvTransposeArgs a) {
    const size_t index = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (index >= (size_t)a.out_ch * a.output_length) return;
    const int p = (int)(index % a.output_length), o = (int)(index / a.output_length);
    const int ipg = a.in_ch / a.groups, opg = a.out_ch / a.groups;
    const int group = o / opg, o_local = o - group * opg;
    float value = a.bias != nullptr ? a.bias[o] : 0.0f;
    // input positions t with 0 <= p - t * stride < kernel
    const int t_hi = min(a.length - 1, p / a.stride);
    const int t_lo = p < a.kernel ? 0 : (p - a.kernel) / a.stride + 1;
    for (int i = group * ipg; i < (group + 1) * ipg; ++i) {
        const float *in_row = a.in + (size_t)i * a.length;
        const float *w = a.w + ((size_t)i * opg + o_local) * a.kernel;
        for (int t = t_lo; t <= t_hi; ++t) value += in_row[t] * w[p - t * a.stride];
    }
    a.out[index] = value;
}

__global__ void __launch_bounds__(256) k_snake(const float *in, float *out, const float *alpha, size_t count, int length, int snake_channels) {
    const size_t index = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (index >= count) return;
    const int channel = (int)(index / (size_t)length);
    const bool snake_row = channel < snake_channels;
    const float al = snake_row ? alpha[channel] : 0.0f;
    const float v = in[index];
    if (in == out && !snake_row && !(v < 0.0f)) return;   // in place, a leaky row's value that stays as it is: no store
    out[index] = half_snake(v, snake_row, al, 1.0f / (al + 1e-9f));
}

// Row sets added in order, scaled, and written to one or more outputs, each plain or through its own half-snake:
// v = ((in0 + in1) + in2 ...) * scale; out_j = alpha_j ? half_snake(v) : v.  One pass instead of residual_inplace per
// addend, scale_dev and snake_dev (or snake_copy_dev per output), with the same arithmetic in the same order.
constexpr int kRowsMax = 4;
struct RowsCombineArgs {
    const float *in[kRowsMax];
    float *out[kRowsMax];
    const float *alpha[kRowsMax];   // null: the value as it is
    int inputs, outputs;
    float scale;
    size_t count;
    int length, snake_channels;
};

__global__ void __launch_bounds__(256) k_rows_combine(const RowsCombineArgs a) {
    const size_t index = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (index >= a.count) return;
    float v = a.in[0][index];
    if (a.inputs > 1) v = v + a.in[1][index];
    if (a.inputs > 2) v = v + a.in[2][index];
    if (a.inputs > 3) v = v + a.in[3][index];
    v = v * a.scale;   // 1.0f keeps the bits
    const int channel = (int)(index / (size_t)a.length);
    const bool snake_row = channel < a.snake_channels;
#pragma unroll
    for (int j = 0; j < kRowsMax; ++j) {
        if (j >= a.outputs) break;
        float y = v;
        if (a.alpha[j] != nullptr) {
            const float al = snake_row ? a.alpha[j][channel] : 0.0f;
            y = half_snake(v, snake_row, al, 1.0f / (al + 1e-9f));
        }
        a.out[j][index] = y;
    }
}

template <int WM, int WN, int KF, bool FUSED>
int launch_conv_f(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    constexpr int TM = 32 * WM, TN = 64 * WN;
    const int slots = (WM * 8 * (kConvChannels * a.kernel + 4) + 255) / 256;
    // two more staged rows than are filled: the product loop requests the operands of two products past its last one
    size_t lds = ((size_t)slots * 1024 + (size_t)(kConvChannels + 2) * (TN + (a.kernel - 1) * a.dilation) + 64) * sizeof(float);
    if (lds < (4 * 32 * kTileStride + 4 * 64) * sizeof(float)) lds = (4 * 32 * kTileStride + 4 * 64) * sizeof(float);   // the fused epilogue's tiles and alphas
    static bool raised = false;   // per instantiation
    if (lds > 48 * 1024 && !raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_conv1d<WM, WN, KF, FUSED>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
        raised = true;
    }
    const dim3 grid((unsigned)((a.length + TN - 1) / TN), (unsigned)((a.out_ch + TM - 1) / TM));
    hipLaunchKernelGGL((k_conv1d<WM, WN, KF, FUSED>), grid, dim3(256), lds, st->stream, a.in, a.out, chunks.data, a.bias, a.in_ch, a.out_ch, a.length, a.kernel, a.dilation,
                       chunks.tiles, a);
    return hip_check(hipGetLastError(), "conv1d launch", error, capacity);
}

template <int WM, int WN, int KF>
int launch_conv_k(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    if (a.residual != nullptr || a.residual2 != nullptr || a.scaled || a.activate) return launch_conv_f<WM, WN, KF, true>(st, a, chunks, error, capacity);
    return launch_conv_f<WM, WN, KF, false>(st, a, chunks, error, capacity);
}

template <int WM, int WN>
int launch_conv(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    switch (a.kernel) {
        case 3: return launch_conv_k<WM, WN, 3>(st, a, chunks, error, capacity);
        case 7: return launch_conv_k<WM, WN, 7>(st, a, chunks, error, capacity);
        case 11: return launch_conv_k<WM, WN, 11>(st, a, chunks, error, capacity);
        default: return launch_conv_k<WM, WN, 0>(st, a, chunks, error, capacity);
    }
}

template <int KF, int NT>
int launch_conv_split_k(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    const int slots = (8 * (kConvChannels * a.kernel + 4) + 63) / 64;
    const size_t per_wave = (size_t)slots * 256 + (size_t)kConvChannels * (32 * NT + (a.kernel - 1) * a.dilation);
    size_t lds = (4 * per_wave + 2 * (32 * NT + (a.kernel - 1) * a.dilation) + 64) * sizeof(float);   // see launch_conv_f about the two extra rows
    if (lds < (4 * 32 * 64 + 64) * sizeof(float)) lds = (4 * 32 * 64 + 64) * sizeof(float);   // the partial tiles, and the rows' alphas behind them
    static bool raised = false;
    if (!raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_conv1d_split<KF, NT>), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        raised = true;
    }
    const dim3 grid((unsigned)((a.length + 32 * NT - 1) / (32 * NT)), (unsigned)((a.out_ch + 31) / 32));
    hipLaunchKernelGGL((k_conv1d_split<KF, NT>), grid, dim3(256), lds, st->stream, a.in, a.out, chunks.data, a.bias, a.in_ch, a.out_ch, a.length, a.kernel, a.dilation,
                       chunks.tiles, a);
    return hip_check(hipGetLastError(), "conv1d launch", error, capacity);
}

template <int NT>
int launch_conv_split_n(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    switch (a.kernel) {
        case 3: return launch_conv_split_k<3, NT>(st, a, chunks, error, capacity);
        case 7: return launch_conv_split_k<7, NT>(st, a, chunks, error, capacity);
        case 11: return launch_conv_split_k<11, NT>(st, a, chunks, error, capacity);
        default: return launch_conv_split_k<0, NT>(st, a, chunks, error, capacity);
    }
}

int launch_conv_split(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    const long tiles = (long)((a.out_ch + 31) / 32) * ((a.length + 63) / 64);
    if (tiles < st->cu_count) return launch_conv_split_n<1>(st, a, chunks, error, capacity);
    return launch_conv_split_n<2>(st, a, chunks, error, capacity);
}

// LDS of the largest member, as the single launches size it
template <int WM, int WN>
int launch_conv_batch(State *st, const ConvBatchArgs &b, int count, char *error, size_t capacity) {
    constexpr int TM = 32 * WM, TN = 64 * WN;
    size_t lds = (4 * 32 * kTileStride + 4 * 64) * sizeof(float);
    for (int i = 0; i < count; ++i) {
        const ConvArgs &a = b.item[i];
        const int slots = (WM * 8 * (kConvChannels * a.kernel + 4) + 255) / 256;
        const size_t need = ((size_t)slots * 1024 + (size_t)(kConvChannels + 2) * (TN + (a.kernel - 1) * a.dilation) + 64) * sizeof(float);
        lds = need > lds ? need : lds;
    }
    static bool raised = false;   // per instantiation
    if (!raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_conv1d_batch<WM, WN>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
        raised = true;
    }
    const ConvArgs &a = b.item[0];
    const dim3 grid((unsigned)((a.length + TN - 1) / TN), (unsigned)((a.out_ch + TM - 1) / TM), (unsigned)count);
    hipLaunchKernelGGL((k_conv1d_batch<WM, WN>), grid, dim3(256), lds, st->stream, b);
    return hip_check(hipGetLastError(), "conv1d batch launch", error, capacity);
}

template <int NT>
int launch_conv_split_batch(State *st, const ConvBatchArgs &b, int count, char *error, size_t capacity) {
    size_t lds = (4 * 32 * 64 + 64) * sizeof(float);
    for (int i = 0; i < count; ++i) {
        const ConvArgs &a = b.item[i];
        const int slots = (8 * (kConvChannels * a.kernel + 4) + 63) / 64;
        const size_t per_wave = (size_t)slots * 256 + (size_t)kConvChannels * (32 * NT + (a.kernel - 1) * a.dilation);
        const size_t need = (4 * per_wave + 2 * (32 * NT + (a.kernel - 1) * a.dilation) + 64) * sizeof(float);
        lds = need > lds ? need : lds;
    }
    static bool raised = false;
    if (!raised) {
        MYNAH_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&k_conv1d_split_batch<NT>), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        raised = true;
    }
    const ConvArgs &a = b.item[0];
    const dim3 grid((unsigned)((a.length + 32 * NT - 1) / (32 * NT)), (unsigned)((a.out_ch + 31) / 32), (unsigned)count);
    hipLaunchKernelGGL((k_conv1d_split_batch<NT>), grid, dim3(256), lds, st->stream, b);
    return hip_check(hipGetLastError(), "conv1d batch launch", error, capacity);
}

}  // namespace

// Checks one convolution's arguments, caches its weights and fills the kernels' argument block.
static int conv1d_prepare(State *st, const float *dev_input, float *dev_output, int in_channels, int out_channels, int length,
                          int kernel, int dilation, const float *weight, const float *bias, const mynah_hip_conv1d_extra *extra,
                          ConvArgs *out_args, ConvBlocks *out_chunks, char *error, size_t capacity) {
    if (st == nullptr || dev_input == nullptr || dev_output == nullptr || weight == nullptr || in_channels <= 0 || out_channels <= 0 ||
        length <= 0 || kernel <= 0 || dilation <= 0) {
        set_error(error, capacity, "invalid conv1d arguments");   // the checks of metal_ops_conv1d, gpu/metal/backend_metal_ops.m:371-372
        return -1;
    }
    if (kernel > kConvMaxKernel || (kernel - 1) * (long)dilation > kConvMaxHalo || (size_t)in_channels * kernel > (size_t)INT_MAX ||
        (size_t)in_channels * (size_t)length > (size_t)INT_MAX * 4u || (size_t)out_channels * (size_t)length > (size_t)INT_MAX * 4u) {
        set_error(error, capacity, "conv1d: kernel above 16 taps, reach above 128 positions or tensor too large");
        return -1;
    }
    ConvBlocks chunks;
    if (cached_conv_blocks(st, weight, (size_t)out_channels, (size_t)in_channels, (size_t)kernel, &chunks, error, capacity) != 0) return -1;
    const float *dev_bias = nullptr;
    if (cached_vector(st, bias, (size_t)out_channels, &dev_bias, error, capacity) != 0) return -1;
    ConvArgs a{dev_input, dev_output, dev_bias, in_channels, out_channels, length, kernel, dilation};
    if (extra != nullptr) {
        if (extra->snake_channels > (size_t)out_channels || (extra->snake_channels != 0 && extra->snake_alpha == nullptr) ||
            (extra->dev_activated != nullptr && !extra->activate) || extra->dev_activated == dev_output || dev_input == dev_output ||
            (extra->dev_residual2 != nullptr && extra->dev_residual == nullptr) || !(extra->scale == extra->scale) ||
            extra->dev_activated == dev_input) {
            set_error(error, capacity, "conv1d_fused: invalid activation or residual arguments, or the input is also an output");
            return -1;
        }
        a.residual = extra->dev_residual;
        a.residual2 = extra->dev_residual2;
        a.scaled = extra->scale != 1.0f;
        a.scale = extra->scale;
        a.activate = extra->activate != 0;
        a.snake_channels = (int)extra->snake_channels;
        a.act_out = extra->dev_activated;
        if (a.activate && a.snake_channels != 0 && cached_vector(st, extra->snake_alpha, extra->snake_channels, &a.alpha, error, capacity) != 0) return -1;
    }
    *out_args = a;
    *out_chunks = chunks;
    return 0;
}

// few output channels: one row of wavefronts, wider in time; too few large tiles to fill the chip (and enough input
// channels to share out): small tiles with the channels split over the wavefronts
static bool conv_takes_split(const State *st, int in_channels, int out_channels, int length) {
    const long tiles = out_channels <= 32 ? (long)((length + 255) / 256) : (long)((out_channels + 63) / 64) * ((length + 127) / 128);
    return tiles < st->cu_count && in_channels >= 4 * kConvChannels;
}

static int conv1d_launch(State *st, const ConvArgs &a, const ConvBlocks &chunks, char *error, size_t capacity) {
    if (conv_takes_split(st, a.in_ch, a.out_ch, a.length)) return launch_conv_split(st, a, chunks, error, capacity);
    if (a.out_ch <= 32) return launch_conv<1, 4>(st, a, chunks, error, capacity);
    return launch_conv<2, 2>(st, a, chunks, error, capacity);
}

static int conv1d_entry(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels, int length,
                        int kernel, int dilation, const float *weight, const float *bias, const mynah_hip_conv1d_extra *extra,
                        char *error, size_t capacity) {
    State *st = enter_state(state);
    ConvArgs a;
    ConvBlocks chunks;
    if (conv1d_prepare(st, dev_input, dev_output, in_channels, out_channels, length, kernel, dilation, weight, bias, extra, &a, &chunks, error, capacity) != 0)
        return -1;
    return conv1d_launch(st, a, chunks, error, capacity);
}

extern "C" int mynah_hip_conv1d(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels, int length,
                                int kernel, int dilation, const float *weight, const float *bias, char *error, size_t capacity) {
    return conv1d_entry(state, dev_input, dev_output, in_channels, out_channels, length, kernel, dilation, weight, bias, nullptr, error, capacity);
}

extern "C" int mynah_hip_conv1d_fused(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels, int length,
                                      int kernel, int dilation, const float *weight, const float *bias, const mynah_hip_conv1d_extra *extra,
                                      char *error, size_t capacity) {
    if (extra == nullptr) {
        set_error(error, capacity, "conv1d_fused: null extra");
        return -1;
    }
    return conv1d_entry(state, dev_input, dev_output, in_channels, out_channels, length, kernel, dilation, weight, bias, extra, error, capacity);
}

extern "C" int mynah_hip_conv1d_fused_batch(void *state, const mynah_hip_conv1d_item *items, size_t count, int in_channels, int out_channels,
                                            int length, char *error, size_t capacity) {
    State *st = enter_state(state);
    if (st == nullptr || items == nullptr || count == 0 || count > (size_t)kConvBatchMax) {
        set_error(error, capacity, "conv1d_fused_batch: one to four convolutions");
        return -1;
    }
    ConvBatchArgs b{};
    ConvBlocks chunks[kConvBatchMax];
    bool side_by_side = true;
    for (size_t i = 0; i < count; ++i) {
        const mynah_hip_conv1d_item &it = items[i];
        if (conv1d_prepare(st, it.dev_input, it.dev_output, in_channels, out_channels, length, it.kernel, it.dilation, it.weight, it.bias, &it.extra,
                           &b.item[i], &chunks[i], error, capacity) != 0)
            return -1;
        b.chunks[i] = chunks[i].data;
        side_by_side = side_by_side && (it.kernel == 3 || it.kernel == 7 || it.kernel == 11) && chunks[i].tiles == chunks[0].tiles;
        // the members run at the same time: what one writes, no other may read or write
        for (size_t j = 0; j < count; ++j) {
            if (j == i) continue;
            const mynah_hip_conv1d_item &o = items[j];
            const float *const written[2] = {it.dev_output, it.extra.dev_activated};
            for (const float *w : written) {
                if (w == nullptr) continue;
                if (w == o.dev_input || w == o.dev_output || w == o.extra.dev_residual || w == o.extra.dev_residual2 || w == o.extra.dev_activated) {
                    set_error(error, capacity, "conv1d_fused_batch: a member writes rows that another member reads or writes");
                    return -1;
                }
            }
        }
    }
    b.tiles = chunks[0].tiles;
    if (!side_by_side || count == 1) {   // other tap counts: one after the other (the same values)
        for (size_t i = 0; i < count; ++i)
            if (conv1d_launch(st, b.item[i], chunks[i], error, capacity) != 0) return -1;
        return 0;
    }
    if (conv_takes_split(st, in_channels, out_channels, length)) {
        // (the tile's width does not enter a value's arithmetic -- same channel blocks per wavefront, same order -- so the
        // members may take the wider tile, half the weight traffic per product, as soon as all of them together fill the chip)
        const long tiles = (long)((out_channels + 31) / 32) * ((length + 63) / 64);
        if (tiles * (long)count < st->cu_count) return launch_conv_split_batch<1>(st, b, (int)count, error, capacity);
        return launch_conv_split_batch<2>(st, b, (int)count, error, capacity);
    }
    if (out_channels <= 32) return launch_conv_batch<1, 4>(st, b, (int)count, error, capacity);
    return launch_conv_batch<2, 2>(st, b, (int)count, error, capacity);
}

extern "C" int mynah_hip_conv_transpose_dev(void *state, const float *dev_input, float *dev_output, int in_channels, int out_channels,
                                            int length, int output_length, int kernel, int stride, int groups, const float *weight,
                                            const float *bias, char *error, size_t capacity) {
    State *st = enter_state(state);
    if (st == nullptr || dev_input == nullptr || dev_output == nullptr || weight == nullptr || in_channels <= 0 || out_channels <= 0 ||
        length <= 0 || output_length <= 0 || kernel <= 0 || stride <= 0 || groups <= 0 || in_channels % groups != 0 ||
        out_channels % groups != 0) {
        set_error(error, capacity, "invalid conv_transpose arguments");
        return -1;
    }
    const size_t per_in = (size_t)(out_channels / groups) * kernel;
    const CachedWeight *cw = nullptr;
    if (cached_matrix(st, weight, (size_t)in_channels, per_in, MYNAH_HIP_F32, &cw, error, capacity) != 0) return -1;
    if (cw->qtype != MYNAH_HIP_F32) {
        set_error(error, capacity, "conv_transpose: weight could not be kept as f32");
        return -1;
    }
    const float *dev_bias = nullptr;
    if (cached_vector(st, bias, (size_t)out_channels, &dev_bias, error, capacity) != 0) return -1;
    ConvTransposeArgs a{dev_input, dev_output, static_cast<const float *>(cw->data), dev_bias, in_channels, out_channels, length,
                        output_length, kernel, stride, groups};
    const size_t count = (size_t)out_channels * output_length;
    if (count > (size_t)INT_MAX * 256u) {   // one thread per output value, 256 to a workgroup
        set_error(error, capacity, "conv_transpose: output too large");
        return -1;
    }
    hipLaunchKernelGGL(k_conv_transpose, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st->stream, a);
    return hip_check(hipGetLastError(), "conv_transpose launch", error, capacity);
}

static int snake_entry(void *state, const float *dev_input, float *dev_output, const float *alpha, size_t channels, size_t length,
                       size_t snake_channels, char *error, size_t capacity) {
    State *st = enter_state(state);
    if (st == nullptr || dev_input == nullptr || dev_output == nullptr || channels > (size_t)INT_MAX || length > (size_t)INT_MAX ||
        snake_channels > channels || (snake_channels != 0 && alpha == nullptr)) {
        set_error(error, capacity, "invalid snake arguments");   // metal_ops_snake, gpu/metal/backend_metal_ops.m:343-346
        return -1;
    }
    const size_t count = channels * length;
    if (count == 0) return 0;
    if (count > (size_t)INT_MAX * 256u) {   // one thread per value, 256 to a workgroup
        set_error(error, capacity, "snake: tensor too large");
        return -1;
    }
    const float *dev_alpha = nullptr;
    if (snake_channels != 0 && cached_vector(st, alpha, snake_channels, &dev_alpha, error, capacity) != 0) return -1;
    hipLaunchKernelGGL(k_snake, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st->stream, dev_input, dev_output, dev_alpha, count,
                       (int)length, (int)snake_channels);
    return hip_check(hipGetLastError(), "snake launch", error, capacity);
}

extern "C" int mynah_hip_rows_combine_dev(void *state, const float *const *dev_inputs, size_t inputs, float scale, float *const *dev_outputs,
                                          const float *const *alphas, size_t outputs, size_t channels, size_t length, size_t snake_channels,
                                          char *error, size_t capacity) {
    State *st = enter_state(state);
    if (st == nullptr || dev_inputs == nullptr || dev_outputs == nullptr || inputs == 0 || inputs > (size_t)kRowsMax || outputs == 0 ||
        outputs > (size_t)kRowsMax || channels > (size_t)INT_MAX || length > (size_t)INT_MAX || snake_channels > channels || !(scale == scale)) {
        set_error(error, capacity, "invalid rows_combine arguments (one to four inputs and outputs)");
        return -1;
    }
    RowsCombineArgs a{};
    a.inputs = (int)inputs;
    a.outputs = (int)outputs;
    a.scale = scale;
    a.count = channels * length;
    a.length = (int)length;
    a.snake_channels = (int)snake_channels;
    if (a.count == 0) return 0;
    if (a.count > (size_t)INT_MAX * 256u) {
        set_error(error, capacity, "rows_combine: tensor too large");
        return -1;
    }
    for (size_t i = 0; i < inputs; ++i) {
        if (dev_inputs[i] == nullptr) { set_error(error, capacity, "rows_combine: null input"); return -1; }
        a.in[i] = dev_inputs[i];
    }
    for (size_t j = 0; j < outputs; ++j) {
        if (dev_outputs[j] == nullptr) { set_error(error, capacity, "rows_combine: null output"); return -1; }
        for (size_t k = 0; k < j; ++k)
            if (dev_outputs[k] == dev_outputs[j]) { set_error(error, capacity, "rows_combine: an output named twice"); return -1; }
        a.out[j] = dev_outputs[j];
        if (alphas != nullptr && alphas[j] != nullptr) {
            if (snake_channels == 0) { a.alpha[j] = reinterpret_cast<const float *>(a.in[0]); continue; }   // only leaky rows: any non-null pointer, never read
            if (cached_vector(st, alphas[j], snake_channels, &a.alpha[j], error, capacity) != 0) return -1;
        }
    }
    hipLaunchKernelGGL(k_rows_combine, dim3((unsigned)((a.count + 255) / 256)), dim3(256), 0, st->stream, a);
    return hip_check(hipGetLastError(), "rows_combine launch", error, capacity);
}

extern "C" int mynah_hip_snake_dev(void *state, float *dev_data, const float *alpha, size_t channels, size_t length, size_t snake_channels,
                                   char *error, size_t capacity) {
    return snake_entry(state, dev_data, dev_data, alpha, channels, length, snake_channels, error, capacity);
}

extern "C" int mynah_hip_snake_copy_dev(void *state, const float *dev_input, float *dev_output, const float *alpha, size_t channels,
                                        size_t length, size_t snake_channels, char *error, size_t capacity) {
    return snake_entry(state, dev_input, dev_output, alpha, channels, length, snake_channels, error, capacity);
}
