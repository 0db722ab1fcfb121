// C ABI of the gfx950 backend: state, pointer-keyed weight cache, and the seam's resident ops.
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <new>

#include "kernels.h"

namespace mynah {

// ------------------------------------------------------------------------------------------ allocation-free workspace
// Scratch of mynah_hip_self_attention_dev_noalloc: split-L partials, the device word the chunk count travels in, and
// arrival counters, in one file-scope device array so that the call never allocates.  Each GPU holds its own copy at its
// own address; host code reaches it only through the pointer hipGetSymbolAddress returned with that device current
// (State::noalloc) -- the array's name here is a host-side stand-in, never a device address.
constexpr size_t kNoAllocPartialFloats = (size_t)1 << 18;   // 1 MiB of partials
constexpr size_t kNoAllocCounters = 4096;                    // heads of one stream
struct NoAllocScratch {
    float partial[kNoAllocPartialFloats];
    StepSlots slots;
    unsigned counters[kNoAllocCounters];
};
static __device__ __align__(256) unsigned char scratch[sizeof(NoAllocScratch)];

// Where an attention call keeps its partials: the backend's growable workspace, or a fixed one that must suffice.
struct AttnWorkspace {
    float *partial;
    size_t partial_floats;
    unsigned *counters;
    size_t counter_count;
    StepSlots *slots;
};

__global__ void __launch_bounds__(256) k_zero_words(unsigned *p, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ------------------------------------------------------------------------------------------ helpers
int ensure_pinned(State *st, size_t bytes, char *error, size_t capacity) {
    if (st->pinned_bytes >= bytes) return 0;
    if (bytes > (SIZE_MAX >> 1)) {   // the doubling below would never reach it
        set_error(error, capacity, "staging request too large");
        return -1;
    }
    if (st->pinned != nullptr) {
        MYNAH_TRY(hipStreamSynchronize(st->stream));
        (void)hipHostFree(st->pinned);
        st->pinned = nullptr;
        st->pinned_bytes = 0;
    }
    size_t cap = 1u << 20;
    while (cap < bytes) cap <<= 1;
    MYNAH_TRY(hipHostMalloc(&st->pinned, cap, hipHostMallocDefault));
    st->pinned_bytes = cap;
    return 0;
}

static int ensure_scratch(State *st, size_t bytes, char *error, size_t capacity) {
    if (st->scratch_bytes >= bytes) return 0;
    if (bytes > (SIZE_MAX >> 1)) {   // the doubling below would never reach it
        set_error(error, capacity, "staging request too large");
        return -1;
    }
    if (st->scratch != nullptr) {
        MYNAH_TRY(hipStreamSynchronize(st->stream));
        (void)hipFree(st->scratch);
        st->scratch = nullptr;
        st->scratch_bytes = 0;
    }
    size_t cap = 1u << 20;
    while (cap < bytes) cap <<= 1;
    MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->scratch), cap));
    st->scratch_bytes = cap;
    return 0;
}

// Host memory -> device, ordered on the backend's stream.  The source is pageable memory of the caller: the runtime has
// taken its contents when the call returns, so the caller may reuse it at once.
static int copy_to_device(State *st, void *dst, const void *src, size_t bytes, char *error, size_t capacity) {
    if (bytes == 0) return 0;
    MYNAH_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, st->stream));
    return 0;
}

// n floats as a byte count, or false when that does not fit a size_t
static bool float_bytes(size_t n, size_t *bytes) {
    if (n > SIZE_MAX / sizeof(float)) return false;
    *bytes = n * sizeof(float);
    return true;
}

// One device block holding a copy of `bytes` host bytes; nothing stays allocated when it fails.
static int device_copy_of(const void *host, size_t bytes, void **dev, char *error, size_t capacity) {
    *dev = nullptr;
    MYNAH_TRY(hipMalloc(dev, bytes));
    if (hip_check(hipMemcpy(*dev, host, bytes, hipMemcpyHostToDevice), "weight upload", error, capacity) != 0) {
        (void)hipFree(*dev);
        *dev = nullptr;
        return -1;
    }
    return 0;
}

int ensure_attention_workspace(State *st, size_t batch, size_t heads, size_t head_width, size_t max_valid,
                               char *error, size_t capacity, size_t chunk_rows) {
    const size_t chunks = (max_valid + chunk_rows - 1) / chunk_rows + 1;
    const size_t need = batch * heads * chunks * (head_width + 4);
    if (st->attn_partial_floats < need) {
        if (st->attn_partial != nullptr) {
            MYNAH_TRY(hipStreamSynchronize(st->stream));
            (void)hipFree(st->attn_partial);
            st->attn_partial = nullptr;
            st->attn_partial_floats = 0;
        }
        MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->attn_partial), need * sizeof(float)));
        st->attn_partial_floats = need;
    }
    if (st->attn_counters == nullptr) {
        const size_t count = (size_t)kMaxBatch * 4096;   // heads * batch upper bound
        MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->attn_counters), count * sizeof(unsigned)));
        MYNAH_TRY(hipMemsetAsync(st->attn_counters, 0, count * sizeof(unsigned), st->stream));
    }
    return 0;
}

// ------------------------------------------------------------------------------------------ weight cache
// Keyed by (host address, byte size, conversion), on the contract that the host memory is an
// immutable model tensor that outlives the backend (gpu/cuda/backend_cuda.cu:193-219).
int cached_matrix(State *st, const float *host, size_t n, size_t k, int want_qtype, const CachedWeight **out,
                  char *error, size_t capacity) {
    if (host == nullptr || n == 0 || k == 0 || n > SIZE_MAX / k / sizeof(float)) {
        set_error(error, capacity, "invalid weight tensor");
        return -1;
    }
    int qtype = want_qtype;
    if (qtype == MYNAH_HIP_INT4 && (k % 32u) != 0) qtype = MYNAH_HIP_F32;   // src/qmat.c:630
    if (qtype != MYNAH_HIP_F32 && k > kQuantMaxK) qtype = MYNAH_HIP_F32;    // src/qmat.c:33,774
    if (qtype != MYNAH_HIP_F32 && !linear_fast_supported(qtype, n, k)) qtype = MYNAH_HIP_F32;
    const WeightKey key{host, n * k * sizeof(float), 1 + qtype * 2 + (qtype == MYNAH_HIP_INT8 || qtype == MYNAH_HIP_INT4 ? st->arith : 0)};
    std::lock_guard<std::mutex> lock(st->mu);
    auto it = st->weights.find(key);
    if (it != st->weights.end()) {
        *out = &it->second;
        return 0;
    }
    CachedWeight cw;
    cw.qtype = qtype;
    cw.n = n;
    cw.k = k;
    cw.arith = (qtype == MYNAH_HIP_INT8 || qtype == MYNAH_HIP_INT4) ? st->arith : 0;
    const size_t count = n * k;
    int rc = 0;
    const PackedWeight *pack = nullptr;
    if (qtype != MYNAH_HIP_F32) {
        cw.fingerprint = weight_fingerprint(host, n, k);
        (void)pack_lookup(st, host, n, k, qtype, cw.arith, cw.fingerprint, &pack);
    }
    if (pack != nullptr && !st->pack_verify) {
        // converted in an earlier process and read from a packed-weight file: upload, nothing to convert
        cw.bytes = pack->values.size() + pack->scales.size() * sizeof(float);
        rc = device_copy_of(pack->values.data(), pack->values.size(), &cw.data, error, capacity);
        if (rc == 0 && !pack->scales.empty())
            rc = device_copy_of(pack->scales.data(), pack->scales.size() * sizeof(float), reinterpret_cast<void **>(&cw.scales), error, capacity);
        if (rc == 0) {
            ++st->pack_hits;
            st->packs.erase(PackKey{cw.fingerprint, (uint64_t)n, (uint64_t)k, qtype, cw.arith});
        }
    } else if (qtype == MYNAH_HIP_F32) {
        cw.bytes = count * sizeof(float);
        rc = device_copy_of(host, cw.bytes, &cw.data, error, capacity);
    } else if (qtype == MYNAH_HIP_F16) {
        std::vector<uint16_t> packed(count);
        for (size_t i = 0; i < count; ++i) packed[i] = f32_to_f16_rne(host[i]);
        cw.bytes = count * sizeof(uint16_t);
        rc = device_copy_of(packed.data(), cw.bytes, &cw.data, error, capacity);
    } else if (qtype == MYNAH_HIP_INT8) {
        std::vector<int8_t> packed(count);
        std::vector<float> scales(n);
        quantize_weight_int8(host, n, k, packed.data(), scales.data(), st->arith);
        cw.bytes = count + n * sizeof(float);
        rc = device_copy_of(packed.data(), count, &cw.data, error, capacity);
        if (rc == 0) rc = device_copy_of(scales.data(), n * sizeof(float), reinterpret_cast<void **>(&cw.scales), error, capacity);
    } else {
        const size_t groups = k / 32u;
        std::vector<uint8_t> packed(count / 2u);
        std::vector<float> scales(n * groups);
        if (quantize_weight_int4(host, n, k, packed.data(), scales.data(), st->arith) != 0) {
            set_error(error, capacity, "int4 weight needs a width that is a multiple of 32");
            return -1;
        }
        cw.bytes = count / 2u + n * groups * sizeof(float);
        rc = device_copy_of(packed.data(), count / 2u, &cw.data, error, capacity);
        if (rc == 0)
            rc = device_copy_of(scales.data(), n * groups * sizeof(float), reinterpret_cast<void **>(&cw.scales), error, capacity);
    }
    if (rc == 0 && pack != nullptr && st->pack_verify) {
        // the file's bytes against the conversion just made (read back from the device: one comparison for every storage)
        std::vector<unsigned char> values(pack->values.size());
        std::vector<float> scales(pack->scales.size());
        const size_t made = cw.bytes - scales.size() * sizeof(float);
        if (made != values.size() || hipMemcpy(values.data(), cw.data, values.size(), hipMemcpyDeviceToHost) != hipSuccess ||
            (!scales.empty() && hipMemcpy(scales.data(), cw.scales, scales.size() * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) ||
            memcmp(values.data(), pack->values.data(), values.size()) != 0 ||
            (!scales.empty() && memcmp(scales.data(), pack->scales.data(), scales.size() * sizeof(float)) != 0)) {
            set_error(error, capacity, "packed-weight file does not hold what this tensor converts to");
            rc = -1;
        } else {
            ++st->pack_hits;
            st->packs.erase(PackKey{cw.fingerprint, (uint64_t)n, (uint64_t)k, qtype, cw.arith});
        }
    }
    if (rc != 0) {
        if (cw.data != nullptr) (void)hipFree(cw.data);   // the scales failed after the values had gone up
        if (cw.scales != nullptr) (void)hipFree(cw.scales);
        return -1;
    }
    st->weight_bytes += cw.bytes;
    auto ins = st->weights.emplace(key, cw);
    *out = &ins.first->second;   // unordered_map never moves its nodes: the pointer stays valid
    return 0;
}

int cached_conv_blocks(State *st, const float *host, size_t out_ch, size_t in_ch, size_t kernel, ConvBlocks *out, char *error, size_t capacity) {
    if (host == nullptr || out_ch == 0 || in_ch == 0 || kernel == 0 || kernel > 64 || in_ch > (size_t)(INT_MAX / 64) ||
        out_ch > SIZE_MAX / in_ch / kernel / sizeof(float)) {
        set_error(error, capacity, "invalid convolution weight");
        return -1;
    }
    const size_t tiles = ((out_ch + 31) / 32 + 1) & ~(size_t)1, blocks = ((in_ch + kConvChannels - 1) / kConvChannels + 3) & ~(size_t)3;
    const size_t row = kConvChannels * kernel + 4, chunk = conv_chunk_floats(kernel);
    out->tiles = (int)tiles;
    out->blocks = (int)blocks;
    const WeightKey key{host, out_ch * in_ch * kernel * sizeof(float), (int)(64 + kernel + 32 * in_ch)};
    std::lock_guard<std::mutex> lock(st->mu);
    auto it = st->weights.find(key);
    if (it != st->weights.end()) {
        out->data = static_cast<const float *>(it->second.data);
        return 0;
    }
    if (tiles > (size_t)INT_MAX || tiles * blocks > SIZE_MAX / sizeof(float) / chunk / 2) {
        set_error(error, capacity, "convolution weight too large");
        return -1;
    }
    std::vector<float> packed(tiles * blocks * chunk + 1024, 0.0f);
    for (size_t o = 0; o < out_ch; ++o)
        for (size_t i = 0; i < in_ch; ++i) {
            float *dst = packed.data() + ((i / kConvChannels) * tiles + o / 32) * chunk + (o % 32) * row + (i % kConvChannels) * kernel;
            const float *src = host + (o * in_ch + i) * kernel;
            for (size_t k = 0; k < kernel; ++k) dst[k] = src[k];
        }
    CachedWeight cw;
    cw.n = out_ch;
    cw.k = in_ch * kernel;
    cw.bytes = packed.size() * sizeof(float);
    if (device_copy_of(packed.data(), cw.bytes, &cw.data, error, capacity) != 0) return -1;
    st->weight_bytes += cw.bytes;
    st->weights.emplace(key, cw);
    out->data = static_cast<const float *>(cw.data);
    return 0;
}

int cached_vector(State *st, const float *host, size_t n, const float **dev, char *error, size_t capacity) {
    if (host == nullptr || n == 0) {
        *dev = nullptr;
        return 0;
    }
    size_t bytes = 0;
    if (!float_bytes(n, &bytes)) {
        set_error(error, capacity, "invalid vector size");
        return -1;
    }
    const WeightKey key{host, bytes, 0};
    std::lock_guard<std::mutex> lock(st->mu);
    auto it = st->weights.find(key);
    if (it != st->weights.end()) {
        *dev = static_cast<const float *>(it->second.data);
        return 0;
    }
    CachedWeight cw;
    cw.n = 1;
    cw.k = n;
    cw.bytes = bytes;
    if (device_copy_of(host, cw.bytes, &cw.data, error, capacity) != 0) return -1;
    st->weight_bytes += cw.bytes;
    st->weights.emplace(key, cw);
    *dev = static_cast<const float *>(cw.data);
    return 0;
}

// out[b] = W in[b] (+bias) for `batch` device rows: fused matvec tiles, or the generic f32 GEMM.
// ln_gain (device vector) non-null: the rows are normalised first (LayerNorm prologue of the product; one weight pass only), and
// with ln_out_slots every stream's normalised row is also stored at that device table's output[stream].
static int linear_rows(State *st, const float *const *in, float *const *out, size_t batch, size_t iw, size_t ow,
                       const float *weight, const float *bias, int8_t *probe_qx, float *probe_sx, int32_t *probe_acc,
                       char *error, size_t capacity, const float *ln_gain = nullptr, const float *ln_bias = nullptr,
                       const StepSlots *ln_out_slots = nullptr) {
    const float *dbias = nullptr;
    if (cached_vector(st, bias, ow, &dbias, error, capacity) != 0) return -1;
    const CachedWeight *cw = nullptr;
    const int want = batch <= kQuantMaxRows ? st->qtype : MYNAH_HIP_F32;
    if (cached_matrix(st, weight, ow, iw, want, &cw, error, capacity) != 0) return -1;
    if (ln_gain != nullptr && (!linear_fast_supported(cw->qtype, ow, iw) || batch > (size_t)kBatchTile)) {
        set_error(error, capacity, "linear: a LayerNorm prologue takes one weight pass of the fused matvec");
        return -1;
    }
    if (!linear_fast_supported(cw->qtype, ow, iw)) {
        for (size_t b = 0; b < batch; ++b)
            if (launch_gemm_f32(st, in[b], out[b], 1, iw, ow, static_cast<const float *>(cw->data), dbias, error, capacity) != 0)
                return -1;
        return 0;
    }
    for (size_t b0 = 0; b0 < batch; b0 += kBatchTile) {
        LinearArgs a{};
        a.w = cw->data;
        a.scales = cw->scales;
        a.bias = dbias;
        a.qtype = cw->qtype;
        a.n = (int)ow;
        a.k = (int)iw;
        a.batch = (int)(batch - b0 < (size_t)kBatchTile ? batch - b0 : (size_t)kBatchTile);
        for (int b = 0; b < a.batch; ++b) {
            a.in[b] = in[b0 + b];
            a.out[b] = out[b0 + b];
        }
        a.arith = st->arith;
        a.epilogue = EPI_NONE;
        a.ln_gain = ln_gain;
        a.ln_bias = ln_bias;
        a.ln_out_slots = ln_out_slots;
        a.probe_qx = probe_qx;
        a.probe_sx = probe_sx;
        a.probe_acc = probe_acc;
        if (launch_linear(st, a, error, capacity) != 0) return -1;
    }
    return 0;
}

static int check_rows(const void *in, const void *out, size_t rows, size_t iw, size_t ow, const float *weight,
                      char *error, size_t capacity) {
    if (in == nullptr || out == nullptr || weight == nullptr || rows == 0 || iw == 0 || ow == 0 ||
        iw > 0x7fffffffu || ow > 0x7fffffffu || rows > 0x7fffffffu) {
        set_error(error, capacity, "invalid matmul arguments");
        return -1;
    }
    return 0;
}

static int matmul_device(State *st, const float *din, float *dout, size_t rows, size_t iw, size_t ow,
                         const float *weight, const float *bias, char *error, size_t capacity) {
    if (check_rows(din, dout, rows, iw, ow, weight, error, capacity) != 0) return -1;
    if (rows <= kQuantMaxRows) {
        const float *in[kMaxBatch];
        float *out[kMaxBatch];
        for (size_t r = 0; r < rows; ++r) {
            in[r] = din + r * iw;
            out[r] = dout + r * ow;
        }
        return linear_rows(st, in, out, rows, iw, ow, weight, bias, nullptr, nullptr, nullptr, error, capacity);
    }
    const float *dbias = nullptr;
    if (cached_vector(st, bias, ow, &dbias, error, capacity) != 0) return -1;
    const CachedWeight *cw = nullptr;
    if (cached_matrix(st, weight, ow, iw, MYNAH_HIP_F32, &cw, error, capacity) != 0) return -1;
    return launch_gemm_f32(st, din, dout, rows, iw, ow, static_cast<const float *>(cw->data), dbias, error, capacity);
}

// host in / host out, synchronous (mynah_backend_matmul, src/backend.h:32-35)
static int hip_matmul(void *opaque, const float *input, float *output, size_t rows, size_t iw, size_t ow,
                      const float *weight, const float *bias, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (check_rows(input, output, rows, iw, ow, weight, error, capacity) != 0) return -1;
    MYNAH_NEED_STATE(st);
    const size_t in_n = rows * iw, out_n = rows * ow;   // each factor is below 2^31
    if (ensure_scratch(st, (in_n + out_n) * sizeof(float), error, capacity) != 0) return -1;
    float *din = st->scratch, *dout = st->scratch + in_n;
    MYNAH_TRY(hipMemcpyAsync(din, input, in_n * sizeof(float), hipMemcpyHostToDevice, st->stream));
    if (matmul_device(st, din, dout, rows, iw, ow, weight, bias, error, capacity) != 0) return -1;
    MYNAH_TRY(hipMemcpyAsync(output, dout, out_n * sizeof(float), hipMemcpyDeviceToHost, st->stream));
    return synchronise(st, error, capacity);
}

static int hip_sgemm(void *opaque, int ta, int tb, size_t m, size_t n, size_t k, float alpha, const float *a, size_t lda,
                     const float *b, size_t ldb, float beta, float *c, size_t ldc, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (a == nullptr || b == nullptr || c == nullptr || m == 0 || n == 0) {
        set_error(error, capacity, "invalid sgemm arguments");
        return -1;
    }
    MYNAH_NEED_STATE(st);
    const size_t limit = (size_t)1 << 31;   // keeps every product below exact in a size_t
    if (m >= limit || n >= limit || k >= limit || lda >= limit || ldb >= limit || ldc >= limit) {
        set_error(error, capacity, "sgemm dimensions too large");
        return -1;
    }
    const size_t a_n = (ta ? k : m) * lda, b_n = (tb ? n : k) * ldb, c_n = m * ldc;
    if (ensure_scratch(st, (a_n + b_n + c_n) * sizeof(float), error, capacity) != 0) return -1;
    float *da = st->scratch, *db = da + a_n, *dc = db + b_n;
    MYNAH_TRY(hipMemcpyAsync(da, a, a_n * sizeof(float), hipMemcpyHostToDevice, st->stream));
    MYNAH_TRY(hipMemcpyAsync(db, b, b_n * sizeof(float), hipMemcpyHostToDevice, st->stream));
    if (beta != 0.0f) MYNAH_TRY(hipMemcpyAsync(dc, c, c_n * sizeof(float), hipMemcpyHostToDevice, st->stream));
    if (launch_sgemm(st, ta, tb, m, n, k, alpha, da, lda, db, ldb, beta, dc, ldc, error, capacity) != 0) return -1;
    // only the m x n result goes back: what lies between a row's end and the next row (ldc > n) is the caller's
    MYNAH_TRY(hipMemcpy2DAsync(c, ldc * sizeof(float), dc, ldc * sizeof(float), n * sizeof(float), m, hipMemcpyDeviceToHost, st->stream));
    return synchronise(st, error, capacity);
}

// Buffers handed to mynah_hip_dev_free wait here until the stream is next idle: work enqueued before the call may still
// read them, nothing enqueued after it does, so any later synchronisation makes them safe to free -- and a caller that
// frees per-utterance buffers in a loop does not stall the stream once per buffer.
static void free_pending(State *st) {   // the stream is idle
    for (void *p : st->pending_free) (void)hipFree(p);
    st->pending_free.clear();
}
constexpr size_t kMaxPendingFrees = 64;

static void hip_close(void *opaque) {
    State *st = enter_state(opaque);
    if (st == nullptr) return;
    (void)hipStreamSynchronize(st->stream);
    free_pending(st);
    for (auto &kv : st->position_tables)
        if (kv.second.data != nullptr) (void)hipFree(kv.second.data);
    for (auto &kv : st->weights) {
        if (kv.second.data != nullptr) (void)hipFree(kv.second.data);
        if (kv.second.scales != nullptr) (void)hipFree(kv.second.scales);
    }
    if (st->scratch != nullptr) (void)hipFree(st->scratch);
    if (st->pinned != nullptr) (void)hipHostFree(st->pinned);
    if (st->flush != nullptr) (void)hipFree(st->flush);
    if (st->cross_norm != nullptr) (void)hipFree(st->cross_norm);
    if (st->attn_partial != nullptr) (void)hipFree(st->attn_partial);
    if (st->attn_counters != nullptr) (void)hipFree(st->attn_counters);
    if (st->seam_slots != nullptr) (void)hipFree(st->seam_slots);
    if (st->argmax_result != nullptr) (void)hipFree(st->argmax_result);
    if (st->head_logits != nullptr) (void)hipFree(st->head_logits);
    if (st->head_result != nullptr) (void)hipFree(st->head_result);
    if (st->ptr_table != nullptr) (void)hipFree(st->ptr_table);
    if (st->ptr_table_host != nullptr) (void)hipHostFree(st->ptr_table_host);
    if (st->persist_abort_host != nullptr) (void)hipHostFree(st->persist_abort_host);
    if (st->ev0 != nullptr) (void)hipEventDestroy(st->ev0);
    if (st->ev1 != nullptr) (void)hipEventDestroy(st->ev1);
    for (int i = 1; i < kMaxLanes; ++i) {
        if (st->lane_streams[i] != nullptr) {
            (void)hipStreamSynchronize(st->lane_streams[i]);
            (void)hipStreamDestroy(st->lane_streams[i]);
        }
        if (st->lane_done[i] != nullptr) (void)hipEventDestroy(st->lane_done[i]);
    }
    if (st->lane_fork != nullptr) (void)hipEventDestroy(st->lane_fork);
    if (st->stream != nullptr) (void)hipStreamDestroy(st->stream);
    delete st;
}

int lane_stream(State *st, int lane, hipStream_t *stream, char *error, size_t capacity) {
    if (lane < 0 || lane >= kMaxLanes) {
        set_error(error, capacity, "no such lane");
        return -1;
    }
    if (lane == 0) {
        *stream = st->stream;
        return 0;
    }
    if (st->lane_fork == nullptr) MYNAH_TRY(hipEventCreateWithFlags(&st->lane_fork, hipEventDisableTiming));
    if (st->lane_streams[lane] == nullptr) MYNAH_TRY(hipStreamCreateWithFlags(&st->lane_streams[lane], hipStreamNonBlocking));   // default priority
    if (st->lane_done[lane] == nullptr) MYNAH_TRY(hipEventCreateWithFlags(&st->lane_done[lane], hipEventDisableTiming));
    *stream = st->lane_streams[lane];
    return 0;
}

static int attention_table(State *st, int is_self, const float *const *q, float *const *kc, float *const *vc,
                           const size_t *position, const size_t *valid, size_t stride, size_t batch, size_t heads,
                           size_t hw, float scale, float *const *out, char *error, size_t capacity, bool hold = false,
                           const AttnWorkspace *fixed = nullptr) {
    if (batch == 0) return 0;
    if (batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "attention batch exceeds MYNAH_MAX_BATCH");
        return -1;
    }
    if (heads == 0 || hw == 0 || hw > 1024 || heads * hw > 4096 || stride > 0x7fffffffu) {
        set_error(error, capacity, "attention: unsupported head shape");
        return -1;
    }
    size_t max_valid = 1;
    AttnArgs a{};
    for (size_t b = 0; b < batch; ++b) {
        if (q[b] == nullptr || kc[b] == nullptr || vc[b] == nullptr || out[b] == nullptr || valid[b] > 0x7ffffff0u) {
            set_error(error, capacity, "attention: null buffer");
            return -1;
        }
        if (is_self && (position[b] >= valid[b])) {
            set_error(error, capacity, "attention: position must lie inside the valid range");
            return -1;
        }
        a.q[b] = q[b];
        a.k_cache[b] = kc[b];
        a.v_cache[b] = vc[b];
        a.out[b] = out[b];
        a.position[b] = is_self ? (int)position[b] : -1;
        a.valid[b] = (int)valid[b];
        if (valid[b] > max_valid) max_valid = valid[b];
    }
    // the vector paths need 16-byte aligned rows everywhere
    bool aligned = true;
    for (size_t b = 0; b < batch; ++b)
        aligned = aligned && ((reinterpret_cast<uintptr_t>(q[b]) | reinterpret_cast<uintptr_t>(kc[b]) |
                               reinterpret_cast<uintptr_t>(vc[b]) | reinterpret_cast<uintptr_t>(out[b])) & 15u) == 0;
    const size_t chunk_rows = (size_t)attention_chunk_rows(is_self, hw, aligned && hw % 4 == 0 && stride % 4 == 0, max_valid);
    float *ws_partial = nullptr;
    unsigned *ws_counters = nullptr;
    if (fixed != nullptr) {
        // same sizing as ensure_attention_workspace, but the memory is what it is: refuse what does not fit
        const size_t chunks = (max_valid + chunk_rows - 1) / chunk_rows + 1;
        if (batch * heads * chunks * (hw + 4) > fixed->partial_floats || batch * heads > fixed->counter_count) {
            set_error(error, capacity, "attention: the call exceeds the allocation-free workspace (heads x chunks x (head width + 4) floats above 2^18)");
            return -1;
        }
        ws_partial = fixed->partial;
        ws_counters = fixed->counters;
        // the counters must read zero when the kernel starts; whatever an earlier call left there is cleared by a kernel
        // (a memset node would not survive a caller's graph capture)
        hipLaunchKernelGGL(k_zero_words, dim3((unsigned)((batch * heads + 255) / 256)), dim3(256), 0, st->stream, ws_counters, batch * heads);
        MYNAH_TRY(hipGetLastError());
    } else {
        if (ensure_attention_workspace(st, batch, heads, hw, max_valid, error, capacity, chunk_rows) != 0) return -1;
        ws_partial = st->attn_partial;
        ws_counters = st->attn_counters;
    }
    a.slots = nullptr;
    a.batch = (int)batch;
    a.heads = (int)heads;
    a.head_width = (int)hw;
    a.stride = (int)stride;
    a.q_stride = 0;
    a.scale = scale;
    a.is_self = is_self;
    a.chunk_rows = (int)chunk_rows;
    a.max_chunks = (int)((max_valid + chunk_rows - 1) / chunk_rows);
    a.partial = ws_partial;
    a.counters = ws_counters;
    if (!aligned) a.q_stride = 1;   // any value that is not a multiple of 4 selects the scalar path
    // A single-stream seam call over more than one chunk leaves its partials for the product that will read its output
    // row (seam fusion): the fold becomes that product's prologue instead of a device-scope hand-over or a launch.
    const bool unit_kernel = aligned && stride % 4 == 0 && (hw == 64 || chunk_rows == (size_t)kWideRows);
    if (a.max_chunks > 1 && unit_kernel) {
        // Whatever the batch, the chunks are folded by the one device function (fold_partials), so a stream's bits do not
        // depend on who called: the batched twin folds in a launch of its own, a single-stream call is held back.
        if (fixed == nullptr && st->seam_slots == nullptr) {
            MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->seam_slots), sizeof(StepSlots)));
            MYNAH_TRY(hipMemsetAsync(st->seam_slots, 0, sizeof(StepSlots), st->stream));
        }
        a.unit_partial = ws_partial;
        a.unit_ml = ws_partial + batch * heads * (size_t)a.max_chunks * hw;
        a.unit_slots = fixed != nullptr ? fixed->slots : st->seam_slots;   // the kernel writes the one word the fold reads
        if (launch_attention(st, a, error, capacity) != 0) return -1;
        if (fixed != nullptr || !(hold && st->fuse && batch == 1)) return launch_unit_fold_streams(st, a, error, capacity);
        PendingOp p;
        p.kind = PendingOp::kAttentionFold;
        p.has_fold = true;
        p.fold_out = out[0];
        p.fold_partial = a.unit_partial;
        p.fold_ml = a.unit_ml;
        p.fold_heads = (int)heads;
        p.fold_head_width = (int)hw;
        p.fold_max_units = a.max_chunks;
        p.iw = heads * hw;
        st->pending = p;
        return 0;
    }
    return launch_attention(st, a, error, capacity);
}

static int backend_self_test(void *opaque, char *error, size_t capacity);

}  // namespace mynah

using namespace mynah;

// =========================================================================================== open
extern "C" int mynah_backend_hip_open(void **state_out, mynah_backend_matmul_fn *matmul, mynah_backend_sgemm_fn *sgemm,
                                      mynah_backend_close_fn *close, mynah_backend_self_test_fn *self_test, char *error,
                                      size_t capacity) {
    if (state_out == nullptr) {
        set_error(error, capacity, "invalid backend state pointer");
        return -1;
    }
    *state_out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0) {
        set_error(error, capacity, "no HIP device");
        return -1;
    }
    MYNAH_TRY(hipSetDevice(0));
    hipDeviceProp_t prop;
    MYNAH_TRY(hipGetDeviceProperties(&prop, 0));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        if (error != nullptr && capacity > 0)
            snprintf(error, capacity, "HIP backend is built for gfx950 (MI355X); found %s", prop.gcnArchName);
        return -1;
    }
    State *st = new (std::nothrow) State();
    if (st == nullptr) {
        set_error(error, capacity, "out of memory creating HIP backend");
        return -1;
    }
    st->cu_count = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    if (hip_check(hipStreamCreate(&st->stream), "stream create", error, capacity) != 0 ||
        hip_check(hipEventCreate(&st->ev0), "event create", error, capacity) != 0 ||
        hip_check(hipEventCreate(&st->ev1), "event create", error, capacity) != 0) {
        hip_close(st);
        return -1;
    }
    // the allocation-free entry point's workspace: this device's copy of the file-scope array
    if (hip_check(hipGetSymbolAddress(reinterpret_cast<void **>(&st->noalloc), HIP_SYMBOL(scratch)), "scratch symbol address", error, capacity) != 0 ||
        st->noalloc == nullptr) {
        if (error != nullptr && capacity > 0 && error[0] == '\0') set_error(error, capacity, "scratch symbol has no device address");
        hip_close(st);
        return -1;
    }
    const char *quant = getenv("MYNAH_QUANT");   // same strings as src/qmat.c:571-576
    if (quant != nullptr && strcmp(quant, "int8") == 0) st->qtype = MYNAH_HIP_INT8;
    else if (quant != nullptr && strcmp(quant, "int4") == 0) st->qtype = MYNAH_HIP_INT4;
    else if (quant != nullptr && strcmp(quant, "f16") == 0) st->qtype = MYNAH_HIP_F16;
    const char *arith = getenv("MYNAH_QUANT_ARITH");
    if (arith != nullptr && strcmp(arith, "stock") == 0) st->arith = MYNAH_HIP_ARITH_STOCK;
    const char *fuse = getenv("MYNAH_HIP_FUSE");   // 0: every seam call is a launch of its own
    if (fuse != nullptr && strcmp(fuse, "0") == 0) st->fuse = 0;
    const char *graph = getenv("MYNAH_HIP_GRAPH");   // 0: every stage a launch, 1 (default): captured graph, 2: persistent launch where it applies
    if (graph != nullptr && (strcmp(graph, "0") == 0 || strcmp(graph, "1") == 0 || strcmp(graph, "2") == 0)) st->graph_mode = graph[0] - '0';
    const char *verify = getenv("MYNAH_HIP_PACK_VERIFY");   // 1: weights found in a packed-weight file are converted anyway and compared
    if (verify != nullptr && strcmp(verify, "1") == 0) st->pack_verify = 1;
    const char *lanes = getenv("MYNAH_HIP_LANES");   // lanes of a resident step above two streams; unset or 0: chosen from the batch size
    if (lanes != nullptr && lanes[0] >= '0' && lanes[0] <= '0' + kMaxLanes && lanes[1] == '\0') st->step_lanes = lanes[0] - '0';
    const char *spin = getenv("MYNAH_HIP_PERSIST_SPIN");
    if (spin != nullptr && spin[0] != '\0') {   // a value that is not a number would read as 0: every wait giving up at once
        char *end = nullptr;
        const unsigned long polls = strtoul(spin, &end, 10);
        if (end == spin || *end != '\0' || polls > 0xffffffffUL) {
            set_error(error, capacity, "MYNAH_HIP_PERSIST_SPIN is not a number of polls");
            hip_close(st);
            return -1;
        }
        st->persist_spin_limit = (unsigned)polls;
    }
    const char *row_wgs = getenv("MYNAH_HIP_PERSIST_ROW_WGS");
    if (row_wgs != nullptr && row_wgs[0] != '\0') st->persist_row_wgs = atoi(row_wgs);
    // the word a persistent step sets when one of its bounded waits gave up: host memory the device writes directly
    if (hip_check(hipHostMalloc(reinterpret_cast<void **>(&st->persist_abort_host), 64, hipHostMallocMapped), "abort word", error, capacity) != 0 ||
        hip_check(hipHostGetDevicePointer(reinterpret_cast<void **>(&st->persist_abort_dev), st->persist_abort_host, 0), "abort word", error, capacity) != 0) {
        hip_close(st);
        return -1;
    }
    st->persist_abort_host[0] = 0u;
    *state_out = st;
    if (matmul != nullptr) *matmul = hip_matmul;
    if (sgemm != nullptr) *sgemm = hip_sgemm;
    if (close != nullptr) *close = hip_close;
    if (self_test != nullptr) *self_test = backend_self_test;
    if (error != nullptr && capacity > 0) error[0] = '\0';
    return 0;
}

// =========================================================================================== memory
extern "C" int mynah_hip_dev_alloc(void *opaque, size_t n, float **dev_ptr, char *error, size_t capacity) {
    State *st = opaque != nullptr ? enter_state(opaque) : nullptr;
    if (dev_ptr == nullptr || n == 0 || n > SIZE_MAX / sizeof(float)) {
        set_error(error, capacity, "invalid device allocation size");
        return -1;
    }
    hipError_t r = hipMalloc(reinterpret_cast<void **>(dev_ptr), n * sizeof(float));
    if (r == hipErrorOutOfMemory && st != nullptr && !st->pending_free.empty()) {   // memory that is only waiting to be freed
        (void)hipGetLastError();
        if (hipStreamSynchronize(st->stream) == hipSuccess) free_pending(st);
        r = hipMalloc(reinterpret_cast<void **>(dev_ptr), n * sizeof(float));
    }
    return hip_check(r, "malloc", error, capacity);
}

extern "C" void mynah_hip_dev_free(void *opaque, float *dev_ptr) {
    State *st = enter_state(opaque);
    if (dev_ptr == nullptr) return;
    if (st == nullptr) {
        (void)hipDeviceSynchronize();
        (void)hipFree(dev_ptr);
        return;
    }
    st->pending_free.push_back(dev_ptr);
    if (st->pending_free.size() >= kMaxPendingFrees && hipStreamSynchronize(st->stream) == hipSuccess) free_pending(st);
}

extern "C" int mynah_hip_h2d(void *opaque, const float *host, float *dev_ptr, size_t n, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    size_t bytes = 0;
    if (st == nullptr || host == nullptr || dev_ptr == nullptr || !float_bytes(n, &bytes)) {
        set_error(error, capacity, "invalid h2d arguments");
        return -1;
    }
    return copy_to_device(st, dev_ptr, host, bytes, error, capacity);
}

// Waits for the stream, and reports what an earlier call could not: a held-back launch that failed inside a call with
// no way to say so, and a step whose workgroups gave up one of their bounded waits (its results mean nothing).  Every
// entry point that hands data or a completion to the host ends here, so the first of them after the failure returns it.
int mynah::synchronise(State *st, char *error, size_t capacity) {
    if (st->deferred_error[0] != '\0') {
        set_error(error, capacity, st->deferred_error);
        st->deferred_error[0] = '\0';
        (void)hipStreamSynchronize(st->stream);
        st->steps_since_sync = 0;
        return -1;
    }
    MYNAH_TRY(hipStreamSynchronize(st->stream));
    free_pending(st);
    const unsigned steps = st->steps_since_sync;
    st->steps_since_sync = 0;
    if (st->persist_abort_host != nullptr && st->persist_abort_host[0] != 0u) {
        st->persist_abort_host[0] = 0u;
        // A workgroup of a resident step gave up waiting for another one's result (it never hangs: every such wait is bounded).
        // When that step is the only one since the stream was last idle and nothing was enqueued behind it, its inputs are
        // still where they were and nobody has read its rows: it runs again here in the form without such waits and the caller
        // never sees the difference, apart from the time.  With several steps in between, which of them it was cannot be told
        // and the earlier ones' inputs may be gone; work enqueued behind the step has used rows that meant nothing: an error.
        if (steps == 1 && st->calls_since_step == 0 && !st->rerunning && st->last_step_decoder != nullptr) {
            st->rerunning = true;
            int rc = rerun_last_step_without_waits(st, error, capacity);
            if (rc == 0) rc = hip_check(hipStreamSynchronize(st->stream), "synchronise", error, capacity);
            st->rerunning = false;
            st->steps_since_sync = 0;
            if (rc == 0 && st->persist_abort_host[0] == 0u) {
                ++st->wait_fallbacks;
                return 0;
            }
            st->persist_abort_host[0] = 0u;
            if (rc != 0) return -1;
        }
        set_error(error, capacity, "resident decode step gave up a bounded wait between its workgroups; its outputs are invalid");
        return -1;
    }
    return 0;
}

extern "C" int mynah_hip_d2h(void *opaque, const float *dev_ptr, float *host, size_t n, char *error, size_t capacity) {
    State *st = enter_state(opaque, false);
    size_t bytes = 0;
    if (st == nullptr || host == nullptr || dev_ptr == nullptr || !float_bytes(n, &bytes)) {
        set_error(error, capacity, "invalid d2h arguments");
        return -1;
    }
    // a resident step still on the stream is waited for first: should it have given up a wait it is repeated before its rows are copied
    if (st->steps_since_sync != 0 && synchronise(st, error, capacity) != 0) return -1;
    if (bytes != 0) MYNAH_TRY(hipMemcpyAsync(host, dev_ptr, bytes, hipMemcpyDeviceToHost, st->stream));
    return synchronise(st, error, capacity);
}

extern "C" int mynah_hip_upload(void *opaque, const float *host, size_t n, float **dev_ptr, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    size_t bytes = 0;
    if (st == nullptr || host == nullptr || dev_ptr == nullptr || n == 0 || !float_bytes(n, &bytes)) {
        set_error(error, capacity, "invalid upload arguments");
        return -1;
    }
    if (ensure_scratch(st, bytes, error, capacity) != 0) return -1;
    *dev_ptr = st->scratch;
    return copy_to_device(st, st->scratch, host, bytes, error, capacity);
}

extern "C" int mynah_hip_download(void *opaque, const float *dev_ptr, float *host, size_t n, char *error, size_t capacity) {
    return mynah_hip_d2h(opaque, dev_ptr, host, n, error, capacity);
}

extern "C" int mynah_hip_sync(void *opaque, char *error, size_t capacity) {
    State *st = enter_state(opaque, false);
    MYNAH_NEED_STATE(st);
    return synchronise(st, error, capacity);
}

extern "C" int mynah_hip_batch_begin(void *opaque, char *error, size_t capacity) {
    (void)opaque;   // a command-buffer hint on Metal; nothing to do on a HIP stream (src/backend.c:571-577)
    if (error != nullptr && capacity > 0) error[0] = '\0';
    return 0;
}

// ---- seam fusion -------------------------------------------------------------------------------------------------
// The engine's resident step makes 18 seam calls per layer (src/graph.c:3391-3476), most of them tiny dependent
// launches: LayerNorm -> product, product -> GELU, product -> residual add.  A single-row LayerNorm or product is
// therefore held back for one call.  When the next call continues the chain on the same buffers, the two (or three)
// become one launch of the fused matvec kernel, which writes every buffer the separate calls would have written (the
// LayerNorm row, the product before the residual add); any other call launches what is held back first
// (enter_state).  Chains: LayerNorm + product, LayerNorm + product + GELU, product + GELU, product + residual.
static bool ranges_overlap(const float *a, size_t na, const float *b, size_t nb) {
    if (a == nullptr || b == nullptr) return false;
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + nb * sizeof(float) && b0 < a0 + na * sizeof(float);
}

static int launch_pending_linear(State *st, const PendingOp &p, int epilogue, float *residual_row, char *error, size_t capacity) {
    LinearArgs a{};
    a.w = p.weight->data;
    a.scales = p.weight->scales;
    a.bias = p.bias;
    a.qtype = p.weight->qtype;
    a.n = (int)p.ow;
    a.k = (int)p.iw;
    a.batch = 1;
    a.in[0] = p.has_ln ? p.ln_in : p.in;
    if (p.has_fold) {   // the row is the fold of the attention partials; workgroup 0 also leaves it where the attention call's output goes
        a.fold_partial = p.fold_partial;
        a.fold_partial_ml = p.fold_ml;
        a.fold_slots = st->seam_slots;
        a.fold_heads = p.fold_heads;
        a.fold_head_width = p.fold_head_width;
        a.fold_max_units = p.fold_max_units;
        a.fold_is_self = 0;
        a.fold_stream0 = 0;
        a.act_out = p.fold_out;
    }
    a.arith = st->arith;
    a.epilogue = epilogue;
    if (p.has_ln) {
        a.ln_gain = p.ln_gain;
        a.ln_bias = p.ln_bias;
        a.ln_out = p.ln_out;
    }
    if (epilogue == EPI_RESIDUAL) {
        a.out[0] = residual_row;   // row += product
        a.aux_out = p.out;         // the product itself, where the separate call would have left it
    } else {
        a.out[0] = p.out;
    }
    return launch_linear(st, a, error, capacity);
}

static int seam_flush(State *st, char *error, size_t capacity) {
    const PendingOp p = st->pending;
    st->pending = PendingOp{};
    if (p.kind == PendingOp::kLayerNorm) return launch_layernorm(st, p.ln_in, p.ln_out, p.ln_gain, p.ln_bias, 1, p.iw, error, capacity);
    if (p.kind == PendingOp::kLinear) return launch_pending_linear(st, p, EPI_NONE, nullptr, error, capacity);
    if (p.kind == PendingOp::kAttentionFold)
        return launch_unit_fold(st, p.fold_partial, p.fold_ml, st->seam_slots, p.fold_heads, p.fold_head_width, p.fold_max_units, p.fold_out,
                                error, capacity);
    return 0;
}

State *mynah::enter_state(void *opaque, bool enqueues) {
    State *st = static_cast<State *>(opaque);
    if (st != nullptr && enqueues) ++st->calls_since_step;
    if (st != nullptr && st->pending.kind != PendingOp::kNone) {
        char message[sizeof st->deferred_error] = {0};
        if (seam_flush(st, message, sizeof message) != 0 && st->deferred_error[0] == '\0')
            snprintf(st->deferred_error, sizeof st->deferred_error, "%s", message[0] != '\0' ? message : "a held-back launch failed");
    }
    return st;
}

// =========================================================================================== resident ops
extern "C" int mynah_hip_gelu_inplace(void *opaque, float *d, size_t n, char *error, size_t capacity) {
    State *st = static_cast<State *>(opaque);
    MYNAH_NEED_STATE(st);
    if (d == nullptr) { set_error(error, capacity, "invalid gelu arguments"); return -1; }
    if (st->pending.kind == PendingOp::kLinear && st->pending.out == d && st->pending.ow == n) {
        const PendingOp p = st->pending;
        st->pending = PendingOp{};
        return launch_pending_linear(st, p, EPI_GELU, nullptr, error, capacity);
    }
    if (seam_flush(st, error, capacity) != 0) return -1;
    return launch_gelu(st, d, n, error, capacity);
}
extern "C" int mynah_hip_gelu_dev(void *opaque, float *d, size_t n, char *error, size_t capacity) {
    return mynah_hip_gelu_inplace(opaque, d, n, error, capacity);
}
// ---- the seam's remaining optional slots (src/backend.h:59,62-64; CUDA forms gpu/cuda/backend_cuda.cu:708-735,813-851,874-950).
// graph.c calls none of them and a backend may leave them null; they are here so that a HIP block in backend.c can fill
// every field the CUDA block fills.
namespace mynah {
namespace {
// columns[(i * kernel + k) * length + l] = input[i * length + l - (kernel - 1 - k) * dilation], 0 in front of the row
__global__ void __launch_bounds__(256) k_im2col_causal(const float *__restrict__ input, float *__restrict__ columns, size_t total, int length,
                                                       int kernel, int dilation) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int l = (int)(idx % (size_t)length);
    const size_t ik = idx / (size_t)length;
    const int k = (int)(ik % (size_t)kernel);
    const size_t i = ik / (size_t)kernel;
    const long src = (long)l - (long)(kernel - 1 - k) * dilation;
    columns[idx] = src >= 0 ? input[i * (size_t)length + (size_t)src] : 0.0f;
}
// tanh-GELU evaluated in double, rounded once (gpu/cuda/backend_cuda.cu:827-837)
__global__ void __launch_bounds__(256) k_gelu_f64(float *data, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const double x = (double)data[i];
    const double inner = 0.7978845608028654 * (x + 0.044715 * (x * x * x));
    data[i] = (float)(0.5 * x * (1.0 + tanh(inner)));
}
int gelu_on_host_rows(State *st, float *data, size_t n, bool in_double, char *error, size_t capacity) {
    size_t bytes = 0;
    if (st == nullptr || data == nullptr || !float_bytes(n, &bytes)) {
        set_error(error, capacity, "invalid gelu arguments");
        return -1;
    }
    if (n == 0) return 0;
    if (ensure_scratch(st, bytes, error, capacity) != 0) return -1;
    if (copy_to_device(st, st->scratch, data, bytes, error, capacity) != 0) return -1;
    if (in_double) {
        hipLaunchKernelGGL(k_gelu_f64, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st->stream, st->scratch, n);
        MYNAH_TRY(hipGetLastError());
    } else if (launch_gelu(st, st->scratch, n, error, capacity) != 0) {
        return -1;
    }
    MYNAH_TRY(hipMemcpyAsync(data, st->scratch, bytes, hipMemcpyDeviceToHost, st->stream));
    return synchronise(st, error, capacity);
}
}  // namespace
}  // namespace mynah

extern "C" int mynah_hip_im2col(void *opaque, const float *dev_input, float *dev_columns, int in_channels, int length, int kernel, int dilation,
                                char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (dev_input == nullptr || dev_columns == nullptr || in_channels < 0 || length < 0 || kernel < 1 || dilation < 1) {
        set_error(error, capacity, "invalid im2col arguments");
        return -1;
    }
    const size_t total = (size_t)in_channels * (size_t)kernel * (size_t)length;
    if (total == 0) return 0;
    if ((total + 255) / 256 > 0x7fffffffu) {
        set_error(error, capacity, "im2col: too many elements");
        return -1;
    }
    hipLaunchKernelGGL(k_im2col_causal, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st->stream, dev_input, dev_columns, total, length, kernel,
                       dilation);
    return hip_check(hipGetLastError(), "im2col launch", error, capacity);
}
extern "C" int mynah_hip_gelu_host(void *opaque, float *data, size_t n, char *error, size_t capacity) {
    return gelu_on_host_rows(enter_state(opaque), data, n, false, error, capacity);
}
extern "C" int mynah_hip_gelu_host_f64(void *opaque, float *data, size_t n, char *error, size_t capacity) {
    return gelu_on_host_rows(enter_state(opaque), data, n, true, error, capacity);
}
// The CUDA backend replays a captured graph of its upload, product and download to save launch overhead and falls back to
// its plain matmul; here the plain host-pointer matmul is already one launch between two copies, so this is that call.
extern "C" int mynah_hip_matmul_graph(void *opaque, const float *input, float *output, size_t rows, size_t iw, size_t ow, const float *weight,
                                      const float *bias, char *error, size_t capacity) {
    return hip_matmul(opaque, input, output, rows, iw, ow, weight, bias, error, capacity);
}

extern "C" int mynah_hip_residual_inplace(void *opaque, float *dout, const float *din, size_t n, char *error, size_t capacity) {
    State *st = static_cast<State *>(opaque);
    MYNAH_NEED_STATE(st);
    if (dout == nullptr || din == nullptr) { set_error(error, capacity, "invalid residual arguments"); return -1; }
    {
        // product -> `dout += product`: one launch, unless the row being updated is one the product reads or writes
        const PendingOp &p = st->pending;
        if (p.kind == PendingOp::kLinear && p.out == din && p.ow == n && !ranges_overlap(dout, n, p.out, p.ow) &&
            !ranges_overlap(dout, n, p.in, p.iw) && !(p.has_ln && (ranges_overlap(dout, n, p.ln_in, p.iw) || ranges_overlap(dout, n, p.ln_out, p.iw)))) {
            const PendingOp q = p;
            st->pending = PendingOp{};
            return launch_pending_linear(st, q, EPI_RESIDUAL, dout, error, capacity);
        }
    }
    if (seam_flush(st, error, capacity) != 0) return -1;
    // The engine passes a HOST row of the mmapped position table in the device slot (src/graph.c:1118-1120):
    // resolve it through the pointer-keyed cache when the address is not device memory.
    hipPointerAttribute_t attr;
    const hipError_t r = hipPointerGetAttributes(&attr, din);
    if (r != hipSuccess || (attr.type != hipMemoryTypeDevice && attr.type != hipMemoryTypeManaged)) {
        (void)hipGetLastError();
        const float *cached = nullptr;
        if (cached_vector(st, din, n, &cached, error, capacity) != 0) return -1;
        din = cached;
    }
    return launch_residual(st, dout, din, n, error, capacity);
}
extern "C" int mynah_hip_residual_add_dev(void *opaque, float *dout, const float *din, size_t n, char *error, size_t capacity) {
    return mynah_hip_residual_inplace(opaque, dout, din, n, error, capacity);
}
extern "C" int mynah_hip_layer_norm_dev(void *opaque, const float *din, float *dout, const float *gain, const float *bias,
                                        size_t rows, size_t width, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (din == nullptr || dout == nullptr || gain == nullptr || width == 0 || width > 0x7fffffffu) {
        set_error(error, capacity, "invalid layer norm arguments");
        return -1;
    }
    const float *dgain = nullptr, *dbias = nullptr;
    if (cached_vector(st, gain, width, &dgain, error, capacity) != 0) return -1;
    if (cached_vector(st, bias, width, &dbias, error, capacity) != 0) return -1;
    if (st->fuse && rows == 1 && !ranges_overlap(din, width, dout, width)) {   // held back: a product may follow
        PendingOp &p = st->pending;
        p.kind = PendingOp::kLayerNorm;
        p.ln_in = din;
        p.ln_out = dout;
        p.ln_gain = dgain;
        p.ln_bias = dbias;
        p.iw = width;
        return 0;
    }
    return launch_layernorm(st, din, dout, dgain, dbias, rows, width, error, capacity);
}
extern "C" int mynah_hip_layer_norm_inplace(void *opaque, const float *din, float *dout, const float *gain, size_t rows,
                                            size_t width, char *error, size_t capacity) {
    return mynah_hip_layer_norm_dev(opaque, din, dout, gain, nullptr, rows, width, error, capacity);
}

// Single-row products of the seam: joins a held-back LayerNorm of its input row, and is itself held back for a GELU or
// residual add of its output row.
static int seam_matmul(void *opaque, const float *din, float *dout, size_t rows, size_t iw, size_t ow, const float *weight,
                       const float *bias, char *error, size_t capacity) {
    State *st = static_cast<State *>(opaque);
    MYNAH_NEED_STATE(st);
    if (check_rows(din, dout, rows, iw, ow, weight, error, capacity) != 0) return -1;
    if (st->fuse && rows == 1) {
        const float *dbias = nullptr;
        const CachedWeight *cw = nullptr;
        if (cached_vector(st, bias, ow, &dbias, error, capacity) != 0) return -1;
        if (cached_matrix(st, weight, ow, iw, st->qtype, &cw, error, capacity) != 0) return -1;
        if (linear_fast_supported(cw->qtype, ow, iw) && !ranges_overlap(din, iw, dout, ow)) {
            PendingOp p = st->pending;
            const bool joins = p.kind == PendingOp::kLayerNorm && p.ln_out == din && p.iw == iw &&
                               !ranges_overlap(dout, ow, p.ln_in, iw) && !ranges_overlap(dout, ow, p.ln_out, iw);
            const bool folds = p.kind == PendingOp::kAttentionFold && p.fold_out == din && p.iw == iw;
            if (!joins && !folds) {
                if (seam_flush(st, error, capacity) != 0) return -1;
                p = PendingOp{};
            }
            p.kind = PendingOp::kLinear;
            p.has_ln = joins;
            p.in = din;
            p.out = dout;
            p.iw = iw;
            p.ow = ow;
            p.weight = cw;
            p.bias = dbias;
            st->pending = p;
            return 0;
        }
    }
    if (seam_flush(st, error, capacity) != 0) return -1;
    return matmul_device(st, din, dout, rows, iw, ow, weight, bias, error, capacity);
}
extern "C" int mynah_hip_matmul_d2d(void *opaque, const float *din, float *dout, size_t rows, size_t iw, size_t ow,
                                    const float *weight, const float *bias, char *error, size_t capacity) {
    return seam_matmul(opaque, din, dout, rows, iw, ow, weight, bias, error, capacity);
}
extern "C" int mynah_hip_matmul_dev(void *opaque, const float *din, float *dout, size_t rows, size_t iw, size_t ow,
                                    const float *weight, const float *bias, char *error, size_t capacity) {
    return seam_matmul(opaque, din, dout, rows, iw, ow, weight, bias, error, capacity);
}
extern "C" int mynah_hip_matvec_dev(void *opaque, const float *din, float *dout, size_t K, size_t N, const float *weight,
                                    const float *bias, char *error, size_t capacity) {
    return seam_matmul(opaque, din, dout, 1, K, N, weight, bias, error, capacity);
}
extern "C" int mynah_hip_matmul_to_dev(void *opaque, const float *host_in, float *dout, size_t rows, size_t iw, size_t ow,
                                       const float *weight, const float *bias, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (check_rows(host_in, dout, rows, iw, ow, weight, error, capacity) != 0) return -1;
    if (ensure_scratch(st, rows * iw * sizeof(float), error, capacity) != 0) return -1;
    if (copy_to_device(st, st->scratch, host_in, rows * iw * sizeof(float), error, capacity) != 0) return -1;
    return matmul_device(st, st->scratch, dout, rows, iw, ow, weight, bias, error, capacity);
}
extern "C" int mynah_hip_sgemm_dev(void *opaque, int ta, int tb, size_t m, size_t n, size_t k, float alpha, const float *da,
                                   size_t lda, const float *db, size_t ldb, float beta, float *dc, size_t ldc, char *error,
                                   size_t capacity) {
    if (da == nullptr || db == nullptr || dc == nullptr) { set_error(error, capacity, "invalid sgemm arguments"); return -1; }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return launch_sgemm(st, ta, tb, m, n, k, alpha, da, lda, db, ldb, beta, dc, ldc, error, capacity);
}
extern "C" int mynah_hip_softmax_dev(void *opaque, float *d, size_t rows, size_t cols, size_t valid, char *error, size_t capacity) {
    if (d == nullptr || cols > 0x7fffffffu) { set_error(error, capacity, "invalid softmax arguments"); return -1; }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return launch_softmax(st, d, rows, cols, valid, error, capacity);
}
extern "C" int mynah_hip_copy_dev(void *opaque, float *dst, const float *src, size_t n, char *error, size_t capacity) {
    if (dst == nullptr || src == nullptr) { set_error(error, capacity, "invalid copy arguments"); return -1; }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return launch_copy(st, dst, src, n, error, capacity);
}
extern "C" int mynah_hip_scale_dev(void *opaque, float *d, size_t n, float scale, char *error, size_t capacity) {
    if (d == nullptr) { set_error(error, capacity, "invalid scale arguments"); return -1; }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return launch_scale(st, d, n, scale, error, capacity);
}
extern "C" int mynah_hip_clip_dev(void *opaque, float *d, size_t n, char *error, size_t capacity) {
    if (d == nullptr) { set_error(error, capacity, "invalid clip arguments"); return -1; }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return launch_clip(st, d, n, error, capacity);
}
extern "C" int mynah_hip_argmax_dev(void *opaque, const float *dlogits, size_t vocab, size_t codebook_size, size_t eos_id,
                                    int allow_eos, unsigned *argmax, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (st == nullptr || dlogits == nullptr || argmax == nullptr || vocab == 0 || codebook_size > vocab || eos_id > 0xffffffffu ||
        vocab > 0x7fffffffu) {   // src/backend.c:829-830
        set_error(error, capacity, "invalid argmax arguments");
        return -1;
    }
    if (st->argmax_result == nullptr) MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->argmax_result), 256));
    if (ensure_pinned(st, 256, error, capacity) != 0) return -1;
    unsigned *dres = st->argmax_result;
    if (launch_argmax(st, dlogits, vocab, codebook_size, eos_id >= 0x7fffffffu ? 0x7ffffffeu : eos_id, allow_eos, dres, error, capacity) != 0)
        return -1;
    MYNAH_TRY(hipMemcpyAsync(st->pinned, dres, sizeof(unsigned), hipMemcpyDeviceToHost, st->stream));
    if (synchronise(st, error, capacity) != 0) return -1;
    *argmax = *static_cast<unsigned *>(st->pinned);
    return 0;
}

extern "C" int mynah_hip_self_attention_dev(void *opaque, const float *dqkv, float *dk, float *dv, size_t position,
                                            size_t cache_stride, size_t valid, size_t heads, size_t head_width, float scale,
                                            float *dout, char *error, size_t capacity) {
    const float *q[1] = {dqkv};
    float *k[1] = {dk}, *v[1] = {dv}, *o[1] = {dout};
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return attention_table(st, 1, q, k, v, &position, &valid, cache_stride, 1, heads, head_width,
                           scale, o, error, capacity, true);
}
extern "C" int mynah_hip_cross_attention_dev(void *opaque, const float *dq, const float *dk, const float *dv, size_t valid,
                                             size_t cache_stride, size_t heads, size_t head_width, float scale, float *dout,
                                             char *error, size_t capacity) {
    const float *q[1] = {dq};
    float *k[1] = {const_cast<float *>(dk)}, *v[1] = {const_cast<float *>(dv)}, *o[1] = {dout};
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return attention_table(st, 0, q, k, v, nullptr, &valid, cache_stride, 1, heads, head_width,
                           scale, o, error, capacity, true);
}

// The same call on the library's fixed workspace: no hipMalloc, no hipFree, no memset node.  It is never held back for
// fusion, and refuses a shape whose partials do not fit instead of growing anything.
extern "C" int mynah_hip_self_attention_dev_noalloc(void *opaque, const float *dqkv, float *dk, float *dv, size_t position,
                                                    size_t cache_stride, size_t valid, size_t heads, size_t head_width, float scale,
                                                    float *dout, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    NoAllocScratch *ws = static_cast<NoAllocScratch *>(st->noalloc);
    const AttnWorkspace fixed{ws->partial, kNoAllocPartialFloats, ws->counters, kNoAllocCounters, &ws->slots};
    const float *q[1] = {dqkv};
    float *k[1] = {dk}, *v[1] = {dv}, *o[1] = {dout};
    return attention_table(st, 1, q, k, v, &position, &valid, cache_stride, 1, heads, head_width, scale, o, error, capacity, false, &fixed);
}

// The cross-attention keys and values of an utterance, all layers, from the encoder memory that is already on the device
// (decoder_cache_init, src/graph.c:3002-3028): per layer LayerNorm(memory) -> kv product [T, 2 * xw] -> K and V halves.
// Here the two halves are two products, each writing its half straight into the cache (the rows of kv_net are independent,
// so each half's weights -- and, for quantised storage, their scales -- are what they are in the whole matrix).  Products of
// up to 16 rows take the current quantisation like every seam product, more rows are f32 (src/qmat.c row limit).
// Everything is enqueued on the backend's stream; nothing is copied to the host.
extern "C" int mynah_hip_cross_kv_dev(void *opaque, const float *dev_memory, size_t memory_length, size_t width, size_t layers,
                                      const float *const *norm_gain, const float *const *norm_bias, const float *const *kv_w, size_t xattn_width,
                                      float *dev_cross_k, float *dev_cross_v, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (dev_memory == nullptr || norm_gain == nullptr || kv_w == nullptr || dev_cross_k == nullptr || dev_cross_v == nullptr || width == 0 ||
        width > 0x7fffffffu || xattn_width == 0 || xattn_width > 0x7fffffffu || memory_length > 0x7fffffffu || layers > 4096) {
        set_error(error, capacity, "invalid cross K/V arguments");
        return -1;
    }
    if (memory_length == 0 || layers == 0) return 0;
    // The normalised rows live in a buffer the backend keeps and grows: one allocation per call would add up between
    // synchronisations when a caller prepares many utterances in a row.  An outgrown buffer may still be read by earlier
    // launches: it waits in the list that the next idle stream frees (bounded like mynah_hip_dev_free's).
    if (st->cross_norm_floats < memory_length * width) {
        if (st->cross_norm != nullptr) {
            st->pending_free.push_back(st->cross_norm);
            st->cross_norm = nullptr;
            st->cross_norm_floats = 0;
            if (st->pending_free.size() >= kMaxPendingFrees && hipStreamSynchronize(st->stream) == hipSuccess) free_pending(st);
        }
        MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->cross_norm), memory_length * width * sizeof(float)));
        st->cross_norm_floats = memory_length * width;
    }
    float *const normed = st->cross_norm;
    const size_t per_layer = memory_length * xattn_width;
    for (size_t l = 0; l < layers; ++l) {
        if (norm_gain[l] == nullptr || kv_w[l] == nullptr) {
            set_error(error, capacity, "cross K/V: missing layer weight");
            return -1;
        }
        const float *dgain = nullptr, *dbias = nullptr;
        if (cached_vector(st, norm_gain[l], width, &dgain, error, capacity) != 0) return -1;
        if (norm_bias != nullptr && cached_vector(st, norm_bias[l], width, &dbias, error, capacity) != 0) return -1;
        if (launch_layernorm(st, dev_memory, normed, dgain, dbias, memory_length, width, error, capacity) != 0) return -1;
        if (matmul_device(st, normed, dev_cross_k + l * per_layer, memory_length, width, xattn_width, kv_w[l], nullptr, error, capacity) != 0) return -1;
        if (matmul_device(st, normed, dev_cross_v + l * per_layer, memory_length, width, xattn_width, kv_w[l] + xattn_width * width, nullptr, error,
                          capacity) != 0)
            return -1;
    }
    return 0;
}

// =========================================================================================== section 2
extern "C" int mynah_hip_set_quant(void *opaque, int qtype, int arith, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (qtype < MYNAH_HIP_F32 || qtype > MYNAH_HIP_F16 || arith < 0 || arith > 1) {
        set_error(error, capacity, "unknown quantisation mode");
        return -1;
    }
    st->qtype = qtype;
    st->arith = arith;
    return 0;
}

extern "C" int mynah_hip_matmul_d2d_batched(void *opaque, const float *const *din, float *const *dout, size_t batch, size_t iw,
                                            size_t ow, const float *weight, const float *bias, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (batch == 0) return 0;   // src/qmat.c:826
    if (batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "batch exceeds MYNAH_MAX_BATCH");
        return -1;
    }
    if (check_rows(din, dout, batch, iw, ow, weight, error, capacity) != 0) return -1;
    for (size_t b = 0; b < batch; ++b)
        if (din[b] == nullptr || dout[b] == nullptr) {
            set_error(error, capacity, "invalid matmul arguments");
            return -1;
        }
    return linear_rows(st, din, dout, batch, iw, ow, weight, bias, nullptr, nullptr, nullptr, error, capacity);
}

extern "C" int mynah_hip_matmul_d2d_probe(void *opaque, const float *din, float *dout, size_t iw, size_t ow,
                                          const float *weight, const float *bias, int8_t *dqx, float *dsx, int32_t *dacc,
                                          char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (check_rows(din, dout, 1, iw, ow, weight, error, capacity) != 0) return -1;
    const float *in[1] = {din};
    float *out[1] = {dout};
    return linear_rows(st, in, out, 1, iw, ow, weight, bias, dqx, dsx, dacc, error, capacity);
}

extern "C" int mynah_hip_self_attention_dev_batched(void *opaque, const float *const *dqkv, float *const *dk, float *const *dv,
                                                    const size_t *position, size_t cache_stride, const size_t *valid,
                                                    size_t batch, size_t heads, size_t head_width, float scale,
                                                    float *const *dout, char *error, size_t capacity) {
    if (dqkv == nullptr || dk == nullptr || dv == nullptr || position == nullptr || valid == nullptr || dout == nullptr) {
        set_error(error, capacity, "attention: null buffer");
        return -1;
    }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return attention_table(st, 1, dqkv, dk, dv, position, valid, cache_stride, batch, heads,
                           head_width, scale, dout, error, capacity);
}
extern "C" int mynah_hip_cross_attention_dev_batched(void *opaque, const float *const *dq, const float *const *dk,
                                                     const float *const *dv, const size_t *valid, size_t cache_stride,
                                                     size_t batch, size_t heads, size_t head_width, float scale,
                                                     float *const *dout, char *error, size_t capacity) {
    if (dq == nullptr || dk == nullptr || dv == nullptr || valid == nullptr || dout == nullptr || batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "attention: null buffer or batch exceeds MYNAH_MAX_BATCH");
        return -1;
    }
    float *k[kMaxBatch], *v[kMaxBatch];
    for (size_t b = 0; b < batch; ++b) {
        k[b] = const_cast<float *>(dk[b]);
        v[b] = const_cast<float *>(dv[b]);
    }
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return attention_table(st, 0, dq, k, v, nullptr, valid, cache_stride, batch, heads, head_width,
                           scale, dout, error, capacity);
}

// Device copy of rows [0, rows) of the host position table at `table`: one growing buffer per table, filled up to the
// highest row any call has needed.  The table's own row count is not known here, so rows are uploaded as calls reach
// them (a decode loop asks for one more row per step) and the buffer doubles when it runs out.
static int position_rows(State *st, const float *table, size_t rows, size_t width, const float **dev, char *error, size_t capacity) {
    if (rows > SIZE_MAX / sizeof(float) / width) {
        set_error(error, capacity, "position table too large");
        return -1;
    }
    PositionTable &t = st->position_tables[std::make_pair(table, width)];
    if (rows > t.capacity_rows) {
        const size_t grown = rows > 2 * t.capacity_rows ? rows : 2 * t.capacity_rows;
        float *bigger = nullptr;
        MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&bigger), grown * width * sizeof(float)));
        if (t.filled_rows != 0) MYNAH_TRY(hipMemcpyAsync(bigger, t.data, t.filled_rows * width * sizeof(float), hipMemcpyDeviceToDevice, st->stream));
        if (t.data != nullptr) st->pending_free.push_back(t.data);   // earlier launches may still read it
        t.data = bigger;
        t.capacity_rows = grown;
    }
    if (rows > t.filled_rows) {
        if (copy_to_device(st, t.data + t.filled_rows * width, table + t.filled_rows * width, (rows - t.filled_rows) * width * sizeof(float), error,
                           capacity) != 0)
            return -1;
        t.filled_rows = rows;
    }
    *dev = t.data;
    return 0;
}

extern "C" int mynah_hip_embed_gather(void *opaque, const float *const *tables, const size_t *table_rows, size_t table_count,
                                      const int32_t *ids, size_t tokens, size_t width, float scale, const float *position,
                                      size_t position_offset, float *dout, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (tables == nullptr || table_rows == nullptr || ids == nullptr || dout == nullptr || table_count == 0 || table_count > 32 ||
        width == 0 || width > 0x7fffffffu) {
        set_error(error, capacity, "invalid gather arguments");
        return -1;
    }
    if (tokens == 0) return 0;
    for (size_t t = 0; t < tokens; ++t)
        for (size_t j = 0; j < table_count; ++j) {
            const int32_t id = ids[t * table_count + j];
            if (id < 0 || (size_t)id >= table_rows[j]) {   // src/graph.c:730-735
                set_error(error, capacity, "text token id is outside vocabulary");
                return -1;
            }
        }
    const float *dtables[32];
    for (size_t j = 0; j < table_count; ++j) {
        const CachedWeight *cw = nullptr;
        if (cached_matrix(st, tables[j], table_rows[j], width, MYNAH_HIP_F32, &cw, error, capacity) != 0) return -1;
        dtables[j] = static_cast<const float *>(cw->data);
    }
    const float *dpos = nullptr;
    if (position != nullptr && position_rows(st, position, position_offset + tokens, width, &dpos, error, capacity) != 0) return -1;
    if (dpos != nullptr) dpos += position_offset * width;
    const size_t id_bytes = tokens * table_count * sizeof(int32_t);
    if (ensure_scratch(st, id_bytes, error, capacity) != 0) return -1;
    if (copy_to_device(st, st->scratch, ids, id_bytes, error, capacity) != 0) return -1;
    return launch_gather(st, dtables, table_count, reinterpret_cast<const int32_t *>(st->scratch), tokens, width, scale, dpos,
                         dout, error, capacity);
}

// The output head on rows that are already normalised (x_rows null), or on the residual rows x_rows[b * width] with the final
// LayerNorm as the product's prologue, the normalised rows written through ln_out_slots (mynah_hip_decoder_step_head).
int mynah::output_head_rows(State *st, const float *const *dhidden, size_t batch, size_t width, const float *weight, const float *bias, size_t rows,
                            size_t vocab, float *const *dlogits, float *const *dprobs, const float *x_rows, const float *ln_gain, const float *ln_bias,
                            char *error, size_t capacity, const StepSlots *ln_out_slots) {
    if (batch == 0) return 0;
    if (batch > (size_t)kMaxBatch || dhidden == nullptr || dlogits == nullptr || vocab == 0 || rows % vocab != 0) {
        set_error(error, capacity, "invalid output head arguments");
        return -1;
    }
    const float *residual[kMaxBatch];
    if (x_rows != nullptr)
        for (size_t b = 0; b < batch; ++b) residual[b] = x_rows + b * width;
    if (linear_rows(st, x_rows != nullptr ? residual : dhidden, dlogits, batch, width, rows, weight, bias, nullptr, nullptr, nullptr, error, capacity,
                    x_rows != nullptr ? ln_gain : nullptr, x_rows != nullptr ? ln_bias : nullptr, x_rows != nullptr ? ln_out_slots : nullptr) != 0)
        return -1;
    if (dprobs != nullptr) {   // every stream that wants probabilities, in one launch
        const float *from[kMaxBatch];
        float *to[kMaxBatch];
        size_t wanted = 0;
        for (size_t b = 0; b < batch; ++b)
            if (dprobs[b] != nullptr) { from[wanted] = dlogits[b]; to[wanted] = dprobs[b]; ++wanted; }
        if (launch_softmax_heads(st, from, to, wanted, rows / vocab, vocab, error, capacity) != 0) return -1;
    }
    return 0;
}

extern "C" int mynah_hip_output_head(void *opaque, const float *const *dhidden, size_t batch, size_t width, const float *weight,
                                     const float *bias, size_t rows, size_t vocab, float *const *dlogits,
                                     float *const *dprobs, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    return output_head_rows(st, dhidden, batch, width, weight, bias, rows, vocab, dlogits, dprobs, nullptr, nullptr, nullptr, error, capacity);
}

// The decoder head when no local transformer follows (slot_advance, src/graph.c:3873-3905): for every slot and every stacked
// stream the constrained first maximum of final_proj's logits (mynah_matvec_argmax_f32's rule, src/kernels.c:116-139), the
// stored code and the EOS bookkeeping.  The reference computes one stream of one slot at a time on the host; here all
// slots and streams are two launches -- the f32 projection of every slot's row (weights read once for the batch; the
// logits stay in a device buffer of the library and never travel) and one workgroup per slot that chooses -- and one
// synchronisation.  f32 weights whatever the quantisation setting, like the reference's own loop.
extern "C" int mynah_hip_head_argmax(void *opaque, const float *const *dev_hidden, size_t batch, size_t width, const float *weight,
                                     const float *bias, size_t streams, size_t vocab, size_t codebook_size, size_t eos_id,
                                     size_t codebook_count, const int *forbid_eos, unsigned *values, unsigned *stored, int *saw_eos,
                                     size_t *eos_frame, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (batch == 0) return 0;
    if (batch > (size_t)kMaxBatch) {
        set_error(error, capacity, "head argmax batch exceeds MYNAH_MAX_BATCH");
        return -1;
    }
    if (dev_hidden == nullptr || weight == nullptr || forbid_eos == nullptr || values == nullptr || stored == nullptr || saw_eos == nullptr ||
        eos_frame == nullptr || streams == 0 || vocab == 0 || vocab > 0x7fffffffu || streams > 0xffffu || codebook_count == 0 ||
        codebook_size > vocab || streams * vocab > 0x7fffffffu || width == 0 || width > 0x7fffffffu) {
        set_error(error, capacity, "invalid head argmax arguments");
        return -1;
    }
    const size_t rows = streams * vocab;
    if (st->head_logits_floats < (size_t)kMaxBatch * rows) {
        if (st->head_logits != nullptr) st->pending_free.push_back(st->head_logits);
        st->head_logits = nullptr;
        st->head_logits_floats = 0;
        MYNAH_TRY(hipMalloc(reinterpret_cast<void **>(&st->head_logits), (size_t)kMaxBatch * rows * sizeof(float)));
        st->head_logits_floats = (size_t)kMaxBatch * rows;
    }
    const size_t n = batch * streams;
    const size_t result_bytes = 2 * n * sizeof(unsigned) + batch * sizeof(int) + 8 + batch * sizeof(unsigned long long);
    if (st->head_result_bytes < result_bytes) {
        if (st->head_result != nullptr) st->pending_free.push_back(st->head_result);
        st->head_result = nullptr;
        st->head_result_bytes = 0;
        const size_t cap = (size_t)kMaxBatch * (2 * streams * sizeof(unsigned) + sizeof(int) + sizeof(unsigned long long)) + 64;
        MYNAH_TRY(hipMalloc(&st->head_result, cap));
        st->head_result_bytes = cap;
    }
    if (ensure_pinned(st, st->head_result_bytes, error, capacity) != 0) return -1;
    float *dlogits[kMaxBatch];
    HeadArgmaxArgs a{};
    for (size_t b = 0; b < batch; ++b) {
        if (dev_hidden[b] == nullptr) {
            set_error(error, capacity, "invalid head argmax arguments");
            return -1;
        }
        dlogits[b] = st->head_logits + b * rows;
        a.logits[b] = dlogits[b];
        a.forbid_eos[b] = forbid_eos[b] != 0;
    }
    const int saved_qtype = st->qtype;   // the reference's head loop is f32 arithmetic on the stored weights
    st->qtype = MYNAH_HIP_F32;
    const int rc = linear_rows(st, dev_hidden, dlogits, batch, width, rows, weight, bias, nullptr, nullptr, nullptr, error, capacity);
    st->qtype = saved_qtype;
    if (rc != 0) return -1;
    unsigned char *res = static_cast<unsigned char *>(st->head_result);
    a.values = reinterpret_cast<unsigned *>(res);
    a.stored = a.values + n;
    size_t off = 2 * n * sizeof(unsigned);
    a.saw_eos = reinterpret_cast<int *>(res + off);
    off = (off + batch * sizeof(int) + 7) & ~(size_t)7;
    a.eos_frame = reinterpret_cast<unsigned long long *>(res + off);
    a.streams = (int)streams; a.vocab = (int)vocab; a.codebook_size = (int)codebook_size;
    a.eos_id = eos_id >= 0x7fffffffu ? 0x7ffffffe : (int)eos_id;   // an id beyond the vocabulary matches no candidate
    a.codebook_count = (int)codebook_count;
    if (launch_head_argmax(st, a, (int)batch, error, capacity) != 0) return -1;
    const size_t used = off + batch * sizeof(unsigned long long);
    MYNAH_TRY(hipMemcpyAsync(st->pinned, st->head_result, used, hipMemcpyDeviceToHost, st->stream));
    if (synchronise(st, error, capacity) != 0) return -1;
    const unsigned char *host = static_cast<const unsigned char *>(st->pinned);
    memcpy(values, host, n * sizeof(unsigned));
    memcpy(stored, host + n * sizeof(unsigned), n * sizeof(unsigned));
    const int *hs = reinterpret_cast<const int *>(host + 2 * n * sizeof(unsigned));
    const unsigned long long *hf = reinterpret_cast<const unsigned long long *>(host + off);
    for (size_t b = 0; b < batch; ++b) {
        saw_eos[b] = hs[b];
        eos_frame[b] = hf[b] == ~0ull ? SIZE_MAX : (size_t)hf[b];
    }
    return 0;
}

// =========================================================================================== measurement
__global__ void __launch_bounds__(256) k_flush(uint4 *p, size_t n16) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < n16; i += stride) {
        uint4 v = p[i];
        v.x += 1u;
        p[i] = v;
    }
}

extern "C" int mynah_hip_timer_begin(void *opaque, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    return hip_check(hipEventRecord(st->ev0, st->stream), "event record", error, capacity);
}
extern "C" int mynah_hip_timer_end(void *opaque, float *ms, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    if (st == nullptr || ms == nullptr) {
        set_error(error, capacity, "invalid timer arguments");
        return -1;
    }
    MYNAH_TRY(hipEventRecord(st->ev1, st->stream));
    MYNAH_TRY(hipEventSynchronize(st->ev1));
    MYNAH_TRY(hipEventElapsedTime(ms, st->ev0, st->ev1));
    return 0;
}
extern "C" int mynah_hip_flush_cache(void *opaque, size_t bytes, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (bytes < (1u << 20)) bytes = 1u << 20;
    if (st->flush_bytes < bytes) {
        if (st->flush != nullptr) {
            MYNAH_TRY(hipStreamSynchronize(st->stream));
            (void)hipFree(st->flush);
            st->flush = nullptr;
            st->flush_bytes = 0;
        }
        MYNAH_TRY(hipMalloc(&st->flush, bytes));
        MYNAH_TRY(hipMemsetAsync(st->flush, 0, bytes, st->stream));
        st->flush_bytes = bytes;
    }
    hipLaunchKernelGGL(k_flush, dim3(2048), dim3(256), 0, st->stream, static_cast<uint4 *>(st->flush), bytes / 16);
    return hip_check(hipGetLastError(), "flush launch", error, capacity);
}
extern "C" int mynah_hip_set_graph_mode(void *opaque, int enabled, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (enabled < 0 || enabled > 2) {
        set_error(error, capacity, "graph mode is 0 (launches), 1 (captured graph) or 2 (persistent launch where it applies)");
        return -1;
    }
    st->graph_mode = enabled;
    return 0;
}
extern "C" int mynah_hip_set_step_lanes(void *opaque, int lanes, char *error, size_t capacity) {
    State *st = enter_state(opaque);
    MYNAH_NEED_STATE(st);
    if (lanes < 0 || lanes > kMaxLanes) {
        set_error(error, capacity, "step lanes: 0 (chosen from the batch size) to 3");
        return -1;
    }
    st->step_lanes = lanes;
    return 0;
}
extern "C" int mynah_hip_device_memory(void *opaque, size_t *free_bytes, size_t *total_bytes, char *error, size_t capacity) {
    State *st = enter_state(opaque, false);
    MYNAH_NEED_STATE(st);
    size_t f = 0, t = 0;
    MYNAH_TRY(hipMemGetInfo(&f, &t));
    if (free_bytes != nullptr) *free_bytes = f;
    if (total_bytes != nullptr) *total_bytes = t;
    return 0;
}
extern "C" size_t mynah_hip_wait_fallbacks(void *opaque) {
    return opaque != nullptr ? (size_t)static_cast<State *>(opaque)->wait_fallbacks : 0;
}
extern "C" size_t mynah_hip_cached_weight_bytes(void *opaque) {
    return opaque != nullptr ? static_cast<State *>(opaque)->weight_bytes : 0;
}

// =========================================================================================== self test
namespace mynah {

static bool near(float a, float b, float tol) { return fabsf(a - b) <= tol; }

// The matmul/sgemm KATs of gpu/cuda/backend_cuda.cu:514-529 (same numbers as src/backend.c:290-310) and
// the resident-op KATs of gpu/metal/backend_metal_ops.m:1038-1107, codec operators included.
// Arrays are static: the weight cache keys on the host address and never refreshes it.
static int backend_self_test(void *opaque, char *error, size_t capacity) {
    static const float in[6] = {1, 2, 3, -1, 0.5f, 2};
    static const float w[12] = {1, 0, 0, 0, 1, 0, 0, 0, 1, 1, 1, 1};
    static const float bi[4] = {0.5f, -0.5f, 1, 2};
    const float want[8] = {1.5f, 1.5f, 4, 8, -0.5f, 0, 3, 3.5f};
    float got[8] = {0};
    if (hip_matmul(opaque, in, got, 2, 3, 4, w, bi, error, capacity) != 0) return -1;
    for (int i = 0; i < 8; ++i)
        if (!near(got[i], want[i], 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP matmul mismatch %d: %f != %f", i, got[i], want[i]);
            return -1;
        }
    float so[8] = {0};
    if (hip_sgemm(opaque, 0, 1, 2, 4, 3, 1.0f, in, 3, w, 3, 0.0f, so, 4, error, capacity) != 0) return -1;
    const float sw[8] = {1, 2, 3, 6, -1, 0.5f, 2, 1.5f};
    for (int i = 0; i < 8; ++i)
        if (!near(so[i], sw[i], 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP sgemm mismatch %d: %f != %f", i, so[i], sw[i]);
            return -1;
        }

    static const float vin[2] = {1.0f, 2.0f};
    static const float eye[4] = {1.0f, 0.0f, 0.0f, 1.0f};
    static const float b2[2] = {0.5f, -0.5f};
    static const float qkv1[6] = {1.0f, 0.0f, 1.0f, 0.0f, 2.0f, 3.0f};
    static const float qkv2[6] = {1.0f, 0.0f, 0.0f, 1.0f, 4.0f, 5.0f};
    static const float gain[2] = {1.0f, 1.0f};
    float *din = nullptr, *dout = nullptr, *dtmp = nullptr, *dqkv = nullptr, *dsk = nullptr, *dsv = nullptr;
    float o[2];
    int rc = -1;
    const float e1 = expf(1.0f);
    do {
        if (mynah_hip_dev_alloc(opaque, 2, &din, error, capacity) != 0 || mynah_hip_dev_alloc(opaque, 2, &dout, error, capacity) != 0 ||
            mynah_hip_dev_alloc(opaque, 2, &dtmp, error, capacity) != 0 || mynah_hip_dev_alloc(opaque, 6, &dqkv, error, capacity) != 0 ||
            mynah_hip_dev_alloc(opaque, 4, &dsk, error, capacity) != 0 || mynah_hip_dev_alloc(opaque, 4, &dsv, error, capacity) != 0)
            break;
        if (mynah_hip_h2d(opaque, vin, din, 2, error, capacity) != 0 ||
            mynah_hip_matmul_d2d(opaque, din, dout, 1, 2, 2, eye, b2, error, capacity) != 0 ||
            mynah_hip_d2h(opaque, dout, o, 2, error, capacity) != 0)
            break;
        if (!near(o[0], 1.5f, 1e-5f) || !near(o[1], 1.5f, 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP matmul_d2d mismatch: %.8g %.8g (want 1.5 1.5)", o[0], o[1]);
            break;
        }
        if (mynah_hip_h2d(opaque, qkv1, dqkv, 6, error, capacity) != 0 ||
            mynah_hip_self_attention_dev(opaque, dqkv, dsk, dsv, 0, 2, 1, 1, 2, 1.0f, dout, error, capacity) != 0 ||
            mynah_hip_d2h(opaque, dout, o, 2, error, capacity) != 0)
            break;
        if (!near(o[0], 2.0f, 1e-5f) || !near(o[1], 3.0f, 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP 1-token attention mismatch: %.8g %.8g (want 2 3)", o[0], o[1]);
            break;
        }
        if (mynah_hip_h2d(opaque, qkv2, dqkv, 6, error, capacity) != 0 ||
            mynah_hip_self_attention_dev(opaque, dqkv, dsk, dsv, 1, 2, 2, 1, 2, 1.0f, dout, error, capacity) != 0 ||
            mynah_hip_d2h(opaque, dout, o, 2, error, capacity) != 0)
            break;
        if (!near(o[0], (2.0f * e1 + 4.0f) / (e1 + 1.0f), 1e-5f) || !near(o[1], (3.0f * e1 + 5.0f) / (e1 + 1.0f), 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP 2-token attention mismatch: %.8g %.8g", o[0], o[1]);
            break;
        }
        if (mynah_hip_cross_attention_dev(opaque, din, dsk, dsv, 1, 2, 1, 2, 1.0f, dout, error, capacity) != 0 ||
            mynah_hip_d2h(opaque, dout, o, 2, error, capacity) != 0)
            break;
        if (!near(o[0], 2.0f, 1e-5f) || !near(o[1], 3.0f, 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP cross attention mismatch: %.8g %.8g", o[0], o[1]);
            break;
        }
        const float zeros[2] = {0.0f, 0.0f};
        if (mynah_hip_h2d(opaque, zeros, dtmp, 2, error, capacity) != 0 || mynah_hip_sync(opaque, error, capacity) != 0 ||
            mynah_hip_gelu_inplace(opaque, dout, 2, error, capacity) != 0 ||
            mynah_hip_residual_inplace(opaque, dtmp, dout, 2, error, capacity) != 0 ||
            mynah_hip_layer_norm_inplace(opaque, dout, dtmp, gain, 1, 2, error, capacity) != 0 ||
            mynah_hip_d2h(opaque, dtmp, o, 2, error, capacity) != 0)
            break;
        // gelu(2), gelu(3) normalised over two elements: -1/+1 up to eps
        if (!near(o[0], -1.0f, 1e-3f) || !near(o[1], 1.0f, 1e-3f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP gelu/residual/layer norm chain mismatch: %.8g %.8g", o[0], o[1]);
            break;
        }
        const float clip_values[2] = {-2.0f, NAN};
        if (mynah_hip_h2d(opaque, clip_values, dtmp, 2, error, capacity) != 0 || mynah_hip_sync(opaque, error, capacity) != 0 ||
            mynah_hip_clip_dev(opaque, dtmp, 2, error, capacity) != 0 || mynah_hip_d2h(opaque, dtmp, o, 2, error, capacity) != 0)
            break;
        if (o[0] != -1.0f || o[1] != 0.0f) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP clip mismatch: %.8g %.8g (want -1 0)", o[0], o[1]);
            break;
        }
        // codec operators (gpu/metal/backend_metal_ops.m:1026-1030,1085,1099-1106): snake with alpha 1 on the row the clip
        // left (-1, 0), then the three-position causal conv with taps 1 2: 2 5 8
        static const float alpha[2] = {1.0f, 1.0f};
        static const float conv_input[3] = {1.0f, 2.0f, 3.0f};
        static const float conv_weight[2] = {1.0f, 2.0f};
        float c3[3];
        if (mynah_hip_snake_dev(opaque, dtmp, alpha, 2, 1, 2, error, capacity) != 0 || mynah_hip_d2h(opaque, dtmp, o, 2, error, capacity) != 0)
            break;
        const float s1 = sinf(-1.0f);
        if (!near(o[0], -1.0f + s1 * s1, 1e-5f) || !near(o[1], 0.0f, 1e-6f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP snake mismatch: %.8g %.8g", o[0], o[1]);
            break;
        }
        if (mynah_hip_h2d(opaque, conv_input, dqkv, 3, error, capacity) != 0 ||
            mynah_hip_conv1d(opaque, dqkv, dsk, 1, 1, 3, 2, 1, conv_weight, nullptr, error, capacity) != 0 ||
            mynah_hip_d2h(opaque, dsk, c3, 3, error, capacity) != 0)
            break;
        if (!near(c3[0], 2.0f, 1e-5f) || !near(c3[1], 5.0f, 1e-5f) || !near(c3[2], 8.0f, 1e-5f)) {
            if (error != nullptr && capacity > 0) snprintf(error, capacity, "HIP conv1d mismatch: %.8g %.8g %.8g (want 2 5 8)", c3[0], c3[1], c3[2]);
            break;
        }
        rc = 0;
    } while (0);
    mynah_hip_dev_free(opaque, din);
    mynah_hip_dev_free(opaque, dout);
    mynah_hip_dev_free(opaque, dtmp);
    mynah_hip_dev_free(opaque, dqkv);
    mynah_hip_dev_free(opaque, dsk);
    mynah_hip_dev_free(opaque, dsv);
    if (rc != 0 && error != nullptr && capacity > 0 && error[0] == '\0') snprintf(error, capacity, "HIP resident ops self-test mismatch");
    return rc;
}

}  // namespace mynah
