// Packed-weight file: the converted weights of a backend (int8 / int4 values and scales, f16 values) written once and taken
// at the next start instead of converting the f32 tensors again.
//
// The reference converts lazily, at the first use of each tensor (src/qmat.c:779-782), and keeps no such file; this is the
// optional "pre-packed sidecar" of a deployment that wants the load-time conversion gone.  The library's cache is keyed by
// the host address of a tensor, which means nothing across processes, so an entry of the file is found by what the tensor
// is: its shape, the storage type and quantiser arithmetic it was converted with, and a fingerprint of its f32 contents
// (FNV-1a over the shape and 1,536 sampled values: the first and last 256 and 1,024 at an even stride).  A tensor whose
// fingerprint is not in the file is converted as always.  MYNAH_HIP_PACK_VERIFY=1 converts every tensor all the same and
// fails the call when the file's bytes differ -- for tests, and for a deployment that does not trust a file.
//
// File (little-endian): "MYNAHQW1", u32 version = 1, u32 entries, then per entry
//   u32 qtype, u32 arith, u64 n, u64 k, u64 fingerprint, u64 value_bytes, u64 scale_floats, values, scales.
#include <string.h>

#include <cstdio>
#include <memory>
#include <string>

#include "common.h"

namespace mynah {

namespace {

constexpr char kMagic[8] = {'M', 'Y', 'N', 'A', 'H', 'Q', 'W', '1'};

uint64_t fnv1a(uint64_t h, const void *data, size_t bytes) {
    const unsigned char *p = static_cast<const unsigned char *>(data);
    for (size_t i = 0; i < bytes; ++i) {
        h ^= p[i];
        h *= 0x100000001b3ull;
    }
    return h;
}

struct EntryHeader {
    uint32_t qtype, arith;
    uint64_t n, k, fingerprint, value_bytes, scale_floats;
};

size_t expected_value_bytes(int qtype, size_t n, size_t k) {
    return qtype == MYNAH_HIP_INT8 ? n * k : qtype == MYNAH_HIP_INT4 ? n * k / 2u : n * k * 2u;
}
size_t expected_scale_floats(int qtype, size_t n, size_t k) { return qtype == MYNAH_HIP_INT8 ? n : qtype == MYNAH_HIP_INT4 ? n * (k / 32u) : 0; }

}  // namespace

uint64_t weight_fingerprint(const float *host, size_t n, size_t k) {
    const size_t count = n * k;
    uint64_t h = 0xcbf29ce484222325ull;
    const uint64_t shape[2] = {(uint64_t)n, (uint64_t)k};
    h = fnv1a(h, shape, sizeof shape);
    const size_t edge = count < 256 ? count : 256;
    h = fnv1a(h, host, edge * sizeof(float));
    h = fnv1a(h, host + (count - edge), edge * sizeof(float));
    const size_t stride = count / 1024u;
    if (stride > 0)
        for (size_t i = 0; i < 1024; ++i) h = fnv1a(h, host + i * stride, sizeof(float));
    return h;
}

int pack_lookup(State *st, const float *host, size_t n, size_t k, int qtype, int arith, uint64_t fingerprint, const PackedWeight **found) {
    *found = nullptr;
    (void)host;
    if (st->packs.empty()) return 0;
    const PackKey key{fingerprint, (uint64_t)n, (uint64_t)k, qtype, qtype == MYNAH_HIP_F16 ? 0 : arith};
    auto it = st->packs.find(key);
    if (it != st->packs.end()) *found = &it->second;
    return 0;
}

}  // namespace mynah

using namespace mynah;

extern "C" int mynah_hip_weights_export(void *opaque, const char *path, size_t *entries, char *error, size_t capacity) {
    State *st = enter_state(opaque, false);
    MYNAH_NEED_STATE(st);
    if (entries != nullptr) *entries = 0;
    if (path == nullptr) {
        set_error(error, capacity, "weights export: no path");
        return -1;
    }
    MYNAH_TRY(hipStreamSynchronize(st->stream));
    std::lock_guard<std::mutex> lock(st->mu);
    std::unique_ptr<FILE, int (*)(FILE *)> f(fopen(path, "wb"), fclose);
    if (!f) {
        set_error(error, capacity, "weights export: cannot open the file for writing");
        return -1;
    }
    uint32_t count = 0;
    for (const auto &kv : st->weights)
        if (kv.second.qtype != MYNAH_HIP_F32 && kv.second.fingerprint != 0) ++count;
    const uint32_t version = 1;
    bool ok = fwrite(kMagic, 1, 8, f.get()) == 8 && fwrite(&version, 4, 1, f.get()) == 1 && fwrite(&count, 4, 1, f.get()) == 1;
    std::vector<unsigned char> values;
    std::vector<float> scales;
    for (const auto &kv : st->weights) {
        const CachedWeight &cw = kv.second;
        if (!ok || cw.qtype == MYNAH_HIP_F32 || cw.fingerprint == 0) continue;
        EntryHeader h{};
        h.qtype = (uint32_t)cw.qtype;
        h.arith = (uint32_t)cw.arith;
        h.n = cw.n; h.k = cw.k; h.fingerprint = cw.fingerprint;
        h.value_bytes = expected_value_bytes(cw.qtype, cw.n, cw.k);
        h.scale_floats = expected_scale_floats(cw.qtype, cw.n, cw.k);
        values.resize(h.value_bytes);
        scales.resize(h.scale_floats);
        if (hipMemcpy(values.data(), cw.data, h.value_bytes, hipMemcpyDeviceToHost) != hipSuccess ||
            (h.scale_floats != 0 && hipMemcpy(scales.data(), cw.scales, h.scale_floats * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)) {
            set_error(error, capacity, "weights export: reading a weight back from the device failed");
            return -1;
        }
        ok = fwrite(&h, sizeof h, 1, f.get()) == 1 && fwrite(values.data(), 1, values.size(), f.get()) == values.size() &&
             (scales.empty() || fwrite(scales.data(), sizeof(float), scales.size(), f.get()) == scales.size());
    }
    if (!ok || fflush(f.get()) != 0) {
        set_error(error, capacity, "weights export: writing the file failed");
        return -1;
    }
    if (entries != nullptr) *entries = count;
    return 0;
}

extern "C" int mynah_hip_weights_import(void *opaque, const char *path, size_t *entries, char *error, size_t capacity) {
    State *st = enter_state(opaque, false);
    MYNAH_NEED_STATE(st);
    if (entries != nullptr) *entries = 0;
    if (path == nullptr) {
        set_error(error, capacity, "weights import: no path");
        return -1;
    }
    std::unique_ptr<FILE, int (*)(FILE *)> f(fopen(path, "rb"), fclose);
    if (!f) {
        set_error(error, capacity, "weights import: cannot open the file");
        return -1;
    }
    char magic[8];
    uint32_t version = 0, count = 0;
    if (fread(magic, 1, 8, f.get()) != 8 || memcmp(magic, kMagic, 8) != 0 || fread(&version, 4, 1, f.get()) != 1 || version != 1 ||
        fread(&count, 4, 1, f.get()) != 1) {
        set_error(error, capacity, "weights import: not a packed-weight file of version 1");
        return -1;
    }
    std::unordered_map<PackKey, PackedWeight, PackKeyHash> loaded;
    for (uint32_t i = 0; i < count; ++i) {
        EntryHeader h{};
        if (fread(&h, sizeof h, 1, f.get()) != 1 || (h.qtype != MYNAH_HIP_INT8 && h.qtype != MYNAH_HIP_INT4 && h.qtype != MYNAH_HIP_F16) || h.arith > 1 ||
            h.n == 0 || h.k == 0 || h.n > (1ull << 32) || h.k > (1ull << 32) || h.value_bytes != expected_value_bytes((int)h.qtype, h.n, h.k) ||
            h.scale_floats != expected_scale_floats((int)h.qtype, h.n, h.k)) {
            set_error(error, capacity, "weights import: damaged entry");
            return -1;
        }
        PackedWeight p;
        try {
            p.values.resize(h.value_bytes);
            p.scales.resize(h.scale_floats);
        } catch (...) {
            set_error(error, capacity, "weights import: out of memory");
            return -1;
        }
        if (fread(p.values.data(), 1, p.values.size(), f.get()) != p.values.size() ||
            (!p.scales.empty() && fread(p.scales.data(), sizeof(float), p.scales.size(), f.get()) != p.scales.size())) {
            set_error(error, capacity, "weights import: the file ends inside an entry");
            return -1;
        }
        loaded.emplace(PackKey{h.fingerprint, h.n, h.k, (int)h.qtype, (int)h.arith}, std::move(p));
    }
    std::lock_guard<std::mutex> lock(st->mu);
    for (auto &kv : loaded) st->packs[kv.first] = std::move(kv.second);
    if (entries != nullptr) *entries = count;
    return 0;
}

extern "C" size_t mynah_hip_weights_from_pack(void *opaque) { return opaque != nullptr ? static_cast<State *>(opaque)->pack_hits : 0; }
