// Load-time weight conversion, run on the host when the weight cache first sees a tensor.
//
// The packed bytes are an integer artefact that must match the reference's bit for bit, and the
// reference's bits depend on how it was compiled, so both arithmetics are provided:
//   strict : src/qmat.c:39-91 evaluated as written in IEEE binary32
//   stock  : what gcc -O3 -ffast-math (reference Makefile:5) makes of the same lines -- the division
//            by a constant becomes a multiplication by its rounded reciprocal and 1/scale is refolded.
// This translation unit must be compiled without fast-math and with -ffp-contract=off.
#include <math.h>
#include <string.h>

#include "common.h"

namespace mynah {

namespace {
// Round half away from zero through truncation, no clamp (src/qmat.c:54).
inline int round_away(float v) { return (int)(v >= 0.0f ? v + 0.5f : v - 0.5f); }

inline float row_absmax(const float *p, size_t count) {
    float amax = 0.0f;
    for (size_t j = 0; j < count; ++j) {
        const float a = fabsf(p[j]);
        if (a > amax) amax = a;
    }
    return amax;
}
}  // namespace

void quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales, int arith) {
    const float recip127 = 1.0f / 127.0f;
    for (size_t i = 0; i < n; ++i) {
        const float *row = w + i * k;
        const float amax = row_absmax(row, k);
        float scale = 1.0f, inv = 1.0f;
        if (amax > 0.0f) {
            if (arith == MYNAH_HIP_ARITH_STOCK) {
                scale = amax * recip127;
                inv = 127.0f / amax;
            } else {
                scale = amax / 127.0f;
                inv = 1.0f / scale;
            }
        }
        scales[i] = scale;
        int8_t *dst = q + i * k;
        for (size_t j = 0; j < k; ++j) dst[j] = (int8_t)round_away(row[j] * inv);
    }
}

int quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales, int arith) {
    if (k == 0 || (k % 32u) != 0) return -1;   // src/qmat.c:630: unrepresentable, caller stays f32
    const float recip7 = 1.0f / 7.0f;
    const float seven_refolded = 1.0f / recip7;   // 6.9999995f
    const size_t groups = k / 32u;
    for (size_t i = 0; i < n; ++i) {
        for (size_t g = 0; g < groups; ++g) {
            const float *grp = w + i * k + g * 32u;
            const float amax = row_absmax(grp, 32u);
            float scale = 1.0f, inv = 1.0f;
            if (amax > 0.0f) {
                if (arith == MYNAH_HIP_ARITH_STOCK) {
                    scale = amax * recip7;
                    inv = seven_refolded / amax;
                } else {
                    scale = amax / 7.0f;
                    inv = 1.0f / scale;
                }
            }
            scales[i * groups + g] = scale;
            uint8_t *dst = q + i * (k / 2u) + g * 16u;
            for (size_t j = 0; j < 16u; ++j) {
                int lo = round_away(grp[2 * j] * inv);
                int hi = round_away(grp[2 * j + 1] * inv);
                lo = lo < -8 ? -8 : (lo > 7 ? 7 : lo);
                hi = hi < -8 ? -8 : (hi > 7 ? 7 : hi);
                dst[j] = (uint8_t)((lo + 8) | ((hi + 8) << 4));   // low nibble = even index
            }
        }
    }
    return 0;
}

// IEEE binary32 -> binary16, round to nearest even (the (__fp16) cast of src/qmat.c:655).
uint16_t f32_to_f16_rne(float value) {
    uint32_t u;
    memcpy(&u, &value, sizeof u);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    u &= 0x7fffffffu;
    if (u > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((u >> 13) & 0x03ffu));   // NaN, quieted
    if (u == 0x7f800000u || u >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);      // inf / overflow
    if (u <= 0x33000000u) return sign;                                                // rounds to zero
    const int e = (int)(u >> 23) - 127;
    const uint32_t m = (u & 0x007fffffu) | 0x00800000u;
    const int drop = e < -14 ? 13 + (-14 - e) : 13;      // mantissa bits that do not fit
    uint32_t r = m >> drop;
    const uint32_t rest = m & ((1u << drop) - 1u);
    const uint32_t half = 1u << (drop - 1);
    if (e >= -14) r += (uint32_t)(e + 14) << 10;         // the implicit one carries the last exponent step
    if (rest > half || (rest == half && (r & 1u))) ++r;
    return (uint16_t)(sign | r);
}

}  // namespace mynah

extern "C" void mynah_hip_quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales, int arith) {
    mynah::quantize_weight_int8(w, n, k, q, scales, arith);
}

extern "C" int mynah_hip_quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales, int arith) {
    return mynah::quantize_weight_int4(w, n, k, q, scales, arith);
}

extern "C" void mynah_hip_convert_weight_f16(const float *w, size_t count, uint16_t *out) {
    for (size_t i = 0; i < count; ++i) out[i] = mynah::f32_to_f16_rne(w[i]);
}
