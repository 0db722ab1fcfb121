// Small resident ops of the seam: LayerNorm, GELU, residual, copy/scale/clip, softmax, constrained
// argmax, embedding gather, and the begin/end kernels of the resident decode step.
#include <float.h>

#include "device_common.h"
#include "step_items.h"

namespace mynah {
namespace {

__global__ void __launch_bounds__(256) k_layernorm(const float *in, float *out, const float *gain, const float *bias, int width) {
    __shared__ float s4[4];
    layernorm_row(in + (size_t)blockIdx.x * width, out + (size_t)blockIdx.x * width, gain, bias, width, s4);
}

__global__ void __launch_bounds__(256) k_gelu(float *data, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const float x = data[i];
        const float cubic = x * x * x;
        const float c = 0.7978845608f * (x + 0.044715f * cubic);
        data[i] = 0.5f * x * (1.0f + tanhf(c));
    }
}
__global__ void __launch_bounds__(256) k_residual(float *out, const float *in, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] += in[i];
}
__global__ void __launch_bounds__(256) k_copy(float *dst, const float *src, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}
__global__ void __launch_bounds__(256) k_scale(float *data, size_t n, float scale) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) data[i] *= scale;
}
// clamp to [-1, 1]; NaN becomes 0 (gpu/metal/backend_metal_ops.m:1090-1101)
__global__ void __launch_bounds__(256) k_clip(float *data, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const float v = data[i];
        data[i] = (v != v) ? 0.0f : (v > 1.0f ? 1.0f : (v < -1.0f ? -1.0f : v));
    }
}

// mynah_backend_softmax_dev (src/backend.c:602-619): in place, first `valid` columns, zero tail.
__global__ void __launch_bounds__(256) k_softmax_masked(float *data, int cols, int valid) {
    __shared__ float s4[4];
    float *row = data + (size_t)blockIdx.x * cols;
    const int v = valid < cols ? valid : cols;
    float mx = -1e30f;
    for (int i = threadIdx.x; i < v; i += 256) mx = fmaxf(mx, row[i]);
    mx = block_max(mx, s4);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < v; i += 256) {
        const float e = expf(row[i] - mx);
        row[i] = e;
        sum += e;
    }
    sum = block_sum(sum, s4);
    const float inv = 1.0f / sum;
    for (int i = threadIdx.x; i < v; i += 256) row[i] *= inv;
    for (int i = v + threadIdx.x; i < cols; i += 256) row[i] = 0.0f;
}

// mynah_softmax_f32 (src/kernels.c:391-420) per head: p = expf(x - max) * (1 / total).
// Rows of up to 256 * NV values stay in registers (one round trip instead of three passes over memory; a thread's
// values are taken in the same order, so the bits are the same).
template <int NV>
__device__ __forceinline__ void softmax_row_in_registers(const float *row, float *prow, int cols, float *s4) {
    float v[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = threadIdx.x + 256 * u;
        v[u] = row[i < cols ? i : cols - 1];
    }
    float mx = -FLT_MAX;
#pragma unroll
    for (int u = 0; u < NV; ++u)
        if ((int)threadIdx.x + 256 * u < cols) mx = fmaxf(mx, v[u]);
    mx = block_max(mx, s4);
    float sum = 0.0f;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        v[u] = expf(v[u] - mx);
        if ((int)threadIdx.x + 256 * u < cols) sum += v[u];
    }
    sum = block_sum(sum, s4);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = threadIdx.x + 256 * u;
        if (i < cols) prow[i] = v[u] * inv;
    }
}

// The rows of up to kMaxBatch streams in one launch: blockIdx.y names the stream (a select over the kernel arguments).
struct SoftmaxStreams {
    const float *logits[kMaxBatch];
    float *probs[kMaxBatch];
};
// (the first stream's rows and the row length lead the arguments: those are in registers when a wavefront starts, the
// structure behind them is fetched from memory by the streams that need it)
__global__ void __launch_bounds__(256) k_softmax_heads(const float *logits0, float *probs0, int cols, const SoftmaxStreams streams) {
    __shared__ float s4[4];
    const float *logits = logits0;
    float *probs = probs0;
    if (blockIdx.y != 0) {   // (a branch, so that the first stream's workgroups do not wait for the structure)
#pragma unroll
        for (int b = 1; b < kMaxBatch; ++b)
            if ((int)blockIdx.y == b) { logits = streams.logits[b]; probs = streams.probs[b]; }
    }
    const float *row = logits + (size_t)blockIdx.x * cols;
    float *prow = probs + (size_t)blockIdx.x * cols;
    if (cols <= 1024) return softmax_row_in_registers<4>(row, prow, cols, s4);
    if (cols <= 4096) return softmax_row_in_registers<16>(row, prow, cols, s4);
    float mx = -FLT_MAX;
    for (int i = threadIdx.x; i < cols; i += 256) mx = fmaxf(mx, row[i]);
    mx = block_max(mx, s4);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < cols; i += 256) sum += expf(row[i] - mx);
    sum = block_sum(sum, s4);
    const float inv = 1.0f / sum;
    for (int i = threadIdx.x; i < cols; i += 256) prow[i] = expf(row[i] - mx) * inv;
}

// mynah_backend_argmax_dev (src/backend.c:825-847): strict > from -FLT_MAX, first index on ties,
// result 0 when no candidate beats -FLT_MAX.  One workgroup.
__global__ void __launch_bounds__(256) k_argmax(const float *logits, int vocab, int codebook, int eos, int allow_eos,
                                                unsigned *result) {
    __shared__ float s_val[256];
    __shared__ int s_idx[256];
    float best = -FLT_MAX;
    int at = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += 256) {
        if (!(i < codebook || (allow_eos && i == eos))) continue;
        const float v = logits[i];
        if (v > best) { best = v; at = i; }   // ascending i inside a thread: first max kept
    }
    s_val[threadIdx.x] = best;
    s_idx[threadIdx.x] = at;
    __syncthreads();
    for (int half = 128; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) {
            const float ov = s_val[threadIdx.x + half];
            const int oi = s_idx[threadIdx.x + half];
            const float mv = s_val[threadIdx.x];
            const int mi = s_idx[threadIdx.x];
            if (ov > mv || (ov == mv && oi < mi)) { s_val[threadIdx.x] = ov; s_idx[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) result[0] = s_idx[0] == 0x7fffffff ? 0u : (unsigned)s_idx[0];
}

// The decoder head's token choice for every stream of every slot at once (slot_advance, src/graph.c:3873-3905; the rule of
// mynah_matvec_argmax_f32, src/kernels.c:116-139): per (slot, stream) the first maximum among the codes and, unless forbidden
// for that slot, the end-of-sequence id, strict > from -FLT_MAX, 0 when nothing beats it; then the slot's bookkeeping -- EOS seen,
// the earliest frame it was seen in, the stored code.  One workgroup per slot; logits[slot] is [streams, vocab].
__global__ void __launch_bounds__(256) k_head_argmax(HeadArgmaxArgs a) {
    __shared__ float s_val[4];
    __shared__ int s_idx[4];
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *logits = a.logits[b];
    const bool allow_eos = a.forbid_eos[b] == 0;
    int saw_eos = 0;
    unsigned long long eos_frame = ~0ull;
    for (int s = 0; s < a.streams; ++s) {
        const float *row = logits + (size_t)s * a.vocab;
        float best = -FLT_MAX;
        int at = 0x7fffffff;
        for (int i = tid; i < a.vocab; i += 256) {
            if (!(i < a.codebook_size || (allow_eos && i == a.eos_id))) continue;
            const float v = row[i];
            if (v > best) { best = v; at = i; }   // ascending i inside a thread: the first maximum is kept
        }
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(best, off);
            const int oi = __shfl_xor(at, off);
            if (ov > best || (ov == best && oi < at)) { best = ov; at = oi; }
        }
        __syncthreads();   // the slots below are free again
        if (lane == 0) { s_val[wave] = best; s_idx[wave] = at; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < 4; ++w)
                if (s_val[w] > best || (s_val[w] == best && s_idx[w] < at)) { best = s_val[w]; at = s_idx[w]; }
            const unsigned value = at == 0x7fffffff ? 0u : (unsigned)at;
            if ((int)value == a.eos_id) {
                saw_eos = 1;
                const unsigned long long frame = (unsigned long long)(s / a.codebook_count);
                if (frame < eos_frame) eos_frame = frame;
            }
            a.values[(size_t)b * a.streams + s] = value;
            a.stored[(size_t)b * a.streams + s] = (int)value < a.codebook_size ? value : 0u;
        }
    }
    if (tid == 0) {
        a.saw_eos[b] = saw_eos;
        a.eos_frame[b] = eos_frame;
    }
}

// Embedding gather: sum of table rows (bit-exact copy for one table and scale 1) + optional position.
struct GatherTables { const float *t[32]; };
__global__ void __launch_bounds__(256) k_gather(GatherTables tables, int table_count, const int32_t *ids, int width, float scale,
                                                const float *position, float *out) {
    const int t = blockIdx.x;
    for (int d = threadIdx.x; d < width; d += 256) {
        float v = tables.t[0][(size_t)ids[(size_t)t * table_count] * width + d];
        for (int j = 1; j < table_count; ++j) v += tables.t[j][(size_t)ids[(size_t)t * table_count + j] * width + d];
        if (scale != 1.0f) v *= scale;
        if (position != nullptr) v += position[(size_t)t * width + d];
        out[(size_t)t * width + d] = v;
    }
}

// Decode-step begin: record the slot table, x[b] = input[b] + position[length[b]] (src/graph.c:3156-3157).
// (The scalar arguments stand in front of the table: leading scalars are in registers when a wavefront starts.)
// Workgroups behind the streams' fill the work tables of the step's many-stream attention launches, from the table in the
// kernel's arguments.
__global__ void __launch_bounds__(256) k_step_begin(StepSlots *dev_slots, int width, const float *position, float *x, size_t x_stride, int batch,
                                                    const StepSlots slots, const StepItemTables tables) {
    const int b = blockIdx.x;
    if (b >= batch) {
        write_step_item(tables, slots, -1, (int)(slots.epoch & 0xffffffu), (b - batch) * 256 + (int)threadIdx.x);
        return;
    }
    if (b == 0 && threadIdx.x == 0) *dev_slots = slots;
    const float *in = slots.input[b];
    const float *pe = position != nullptr ? position + (size_t)slots.length[b] * width : nullptr;
    if (width <= 1024) {   // one round trip: every request issued before the first sum
        float iv[4], pv[4];
        const float *second = pe != nullptr ? pe : in;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int d = threadIdx.x + 256 * u, at = d < width ? d : width - 1;
            iv[u] = in[at];
            pv[u] = second[at];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int d = threadIdx.x + 256 * u;
            if (d < width) x[(size_t)b * x_stride + d] = pe != nullptr ? iv[u] + pv[u] : iv[u];
        }
        return;
    }
    for (int d = threadIdx.x; d < width; d += 256) x[(size_t)b * x_stride + d] = pe != nullptr ? in[d] + pe[d] : in[d];
}

__global__ void __launch_bounds__(256) k_step_end(const StepSlots *slots, int width, const float *x, size_t x_stride,
                                                  const float *gain, const float *bias) {
    __shared__ float s4[4];
    const int b = blockIdx.x;
    float *out = slots->output[b];
    const float *row = x + (size_t)b * x_stride;
    if (gain == nullptr) {
        for (int d = threadIdx.x; d < width; d += 256) out[d] = row[d];
        return;
    }
    layernorm_row(row, out, gain, bias, width, s4);
}

inline unsigned blocks_for(size_t n) { return (unsigned)((n + 255) / 256); }

// one workgroup per row: the row count has to fit a grid dimension
inline int check_grid_rows(size_t rows, const char *what, char *error, size_t capacity) {
    if (rows <= 0x7fffffffu) return 0;
    if (error != nullptr && capacity > 0) snprintf(error, capacity, "%s: too many rows", what);
    return -1;
}

}  // namespace

int launch_layernorm(State *st, const float *in, float *out, const float *gain, const float *bias, size_t rows,
                     size_t width, char *error, size_t capacity) {
    if (rows == 0 || width == 0) return 0;
    if (check_grid_rows(rows, "layernorm", error, capacity) != 0) return -1;
    hipLaunchKernelGGL(k_layernorm, dim3((unsigned)rows), dim3(256), 0, st->stream, in, out, gain, bias, (int)width);
    return hip_check(hipGetLastError(), "layernorm launch", error, capacity);
}
int launch_gelu(State *st, float *data, size_t n, char *error, size_t capacity) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_gelu, dim3(blocks_for(n)), dim3(256), 0, st->stream, data, n);
    return hip_check(hipGetLastError(), "gelu launch", error, capacity);
}
int launch_residual(State *st, float *out, const float *in, size_t n, char *error, size_t capacity) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_residual, dim3(blocks_for(n)), dim3(256), 0, st->stream, out, in, n);
    return hip_check(hipGetLastError(), "residual launch", error, capacity);
}
int launch_copy(State *st, float *dst, const float *src, size_t n, char *error, size_t capacity) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_copy, dim3(blocks_for(n)), dim3(256), 0, st->stream, dst, src, n);
    return hip_check(hipGetLastError(), "copy launch", error, capacity);
}
int launch_scale(State *st, float *data, size_t n, float scale, char *error, size_t capacity) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_scale, dim3(blocks_for(n)), dim3(256), 0, st->stream, data, n, scale);
    return hip_check(hipGetLastError(), "scale launch", error, capacity);
}
int launch_clip(State *st, float *data, size_t n, char *error, size_t capacity) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(k_clip, dim3(blocks_for(n)), dim3(256), 0, st->stream, data, n);
    return hip_check(hipGetLastError(), "clip launch", error, capacity);
}
int launch_softmax(State *st, float *data, size_t rows, size_t cols, size_t valid, char *error, size_t capacity) {
    if (rows == 0 || cols == 0) return 0;
    if (check_grid_rows(rows, "softmax", error, capacity) != 0) return -1;
    if (valid > cols) valid = cols;   // src/backend.c:609; also keeps the narrowing below exact
    hipLaunchKernelGGL(k_softmax_masked, dim3((unsigned)rows), dim3(256), 0, st->stream, data, (int)cols, (int)valid);
    return hip_check(hipGetLastError(), "softmax launch", error, capacity);
}
int launch_softmax_heads(State *st, const float *const *logits, float *const *probs, size_t streams, size_t rows, size_t cols, char *error,
                         size_t capacity) {
    if (rows == 0 || cols == 0 || streams == 0) return 0;
    if (streams > (size_t)kMaxBatch) {
        set_error(error, capacity, "softmax: more streams than one launch takes");
        return -1;
    }
    if (check_grid_rows(rows, "softmax", error, capacity) != 0) return -1;
    SoftmaxStreams s{};
    for (size_t b = 0; b < streams; ++b) { s.logits[b] = logits[b]; s.probs[b] = probs[b]; }
    hipLaunchKernelGGL(k_softmax_heads, dim3((unsigned)rows, (unsigned)streams), dim3(256), 0, st->stream, s.logits[0], s.probs[0], (int)cols, s);
    return hip_check(hipGetLastError(), "softmax launch", error, capacity);
}
int launch_argmax(State *st, const float *logits, size_t vocab, size_t codebook, size_t eos, int allow_eos,
                  unsigned *dev_result, char *error, size_t capacity) {
    hipLaunchKernelGGL(k_argmax, dim3(1), dim3(256), 0, st->stream, logits, (int)vocab, (int)codebook, (int)eos, allow_eos,
                       dev_result);
    return hip_check(hipGetLastError(), "argmax launch", error, capacity);
}
int launch_head_argmax(State *st, const HeadArgmaxArgs &a, int batch, char *error, size_t capacity) {
    hipLaunchKernelGGL(k_head_argmax, dim3((unsigned)batch), dim3(256), 0, st->stream, a);
    return hip_check(hipGetLastError(), "head argmax launch", error, capacity);
}
int launch_gather(State *st, const float *const *dev_tables, size_t table_count, const int32_t *dev_ids, size_t tokens,
                  size_t width, float scale, const float *dev_position, float *out, char *error, size_t capacity) {
    if (tokens == 0) return 0;
    if (table_count < 1 || table_count > 32) {
        set_error(error, capacity, "gather: between 1 and 32 tables");
        return -1;
    }
    if (check_grid_rows(tokens, "gather", error, capacity) != 0) return -1;
    GatherTables t;
    for (size_t j = 0; j < 32; ++j) t.t[j] = j < table_count ? dev_tables[j] : nullptr;
    hipLaunchKernelGGL(k_gather, dim3((unsigned)tokens), dim3(256), 0, st->stream, t, (int)table_count, dev_ids, (int)width, scale,
                       dev_position, out);
    return hip_check(hipGetLastError(), "gather launch", error, capacity);
}
int launch_step_begin(State *st, const StepSlots &slots, StepSlots *dev_slots, int batch, size_t width,
                      const float *dev_position, float *x, size_t x_stride, const StepItemTables &tables, char *error, size_t capacity) {
    hipLaunchKernelGGL(k_step_begin, dim3((unsigned)batch + step_item_workgroups(tables)), dim3(256), 0, st->stream, dev_slots, (int)width, dev_position, x,
                       x_stride, batch, slots, tables);
    return hip_check(hipGetLastError(), "step begin launch", error, capacity);
}
int launch_step_end(State *st, const StepSlots *dev_slots, int batch, size_t width, const float *x, size_t x_stride,
                    const float *gain, const float *bias, char *error, size_t capacity) {
    hipLaunchKernelGGL(k_step_end, dim3((unsigned)batch), dim3(256), 0, st->stream, dev_slots, (int)width, x, x_stride, gain, bias);
    return hip_check(hipGetLastError(), "step end launch", error, capacity);
}

}  // namespace mynah
