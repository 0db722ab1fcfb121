/* TEST INFRASTRUCTURE ONLY -- see mynah_oracle.h.  Never part of the shipped library.
 *
 * Built with -O2 -fno-fast-math -ffp-contract=off: every float operation below is the single
 * IEEE-754 binary32 operation the source names; fused multiply-adds appear only where fmaf()
 * is written.  Citations are file:line in the reference tree.
 */
#include "mynah_oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define ORC_Q4_GROUP 32u   /* src/qmat.c:34 */

/* ===================================================================== quantizers */

/* The rounding used everywhere: round half away from zero by truncation (src/qmat.c:54). */
static inline int round_half_away(float v) { return (int)(v >= 0.0f ? v + 0.5f : v - 0.5f); }

/* src/qmat.c:39-57.  ORC_STRICT evaluates the source as written.  ORC_STOCK is the closed form of
 * what gcc 11.4 -O3 -ffast-math emits for it: the division by the constant becomes a multiplication
 * by f32(1/127) and 1/scale is refolded to 127/amax. */
void orc_quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales, int variant) {
    for (size_t i = 0; i < n; ++i) {
        const float *row = w + i * k;
        float amax = 0.0f;
        for (size_t j = 0; j < k; ++j) {
            const float a = fabsf(row[j]);
            if (a > amax) amax = a;
        }
        float scale, inv;
        if (variant == ORC_STOCK) {
            const float r127 = 1.0f / 127.0f;   /* 0x1.020408p-7f */
            scale = amax > 0.0f ? amax * r127 : 1.0f;
            inv = amax > 0.0f ? 127.0f / amax : 1.0f;
        } else {
            scale = amax > 0.0f ? amax / 127.0f : 1.0f;
            inv = 1.0f / scale;
        }
        scales[i] = scale;
        int8_t *qrow = q + i * k;
        for (size_t j = 0; j < k; ++j) qrow[j] = (int8_t)round_half_away(row[j] * inv);
    }
}

/* src/qmat.c:61-91.  Low nibble = even index, nibbles offset by +8, clamp [-8,7].
 * ORC_STOCK: scale = amax * f32(1/7), inv = 6.9999995f / amax (0x40dfffff = f32(1/f32(1/7))). */
int orc_quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales, int variant) {
    if (k == 0 || (k % ORC_Q4_GROUP) != 0) return -1;   /* src/qmat.c:630 refuses such shapes */
    const size_t groups = k / ORC_Q4_GROUP;
    for (size_t i = 0; i < n; ++i) {
        const float *row = w + i * k;
        uint8_t *qrow = q + i * (k / 2u);
        float *srow = scales + i * groups;
        for (size_t g = 0; g < groups; ++g) {
            const float *grp = row + g * ORC_Q4_GROUP;
            float amax = 0.0f;
            for (size_t j = 0; j < ORC_Q4_GROUP; ++j) {
                const float a = fabsf(grp[j]);
                if (a > amax) amax = a;
            }
            float scale, inv;
            if (variant == ORC_STOCK) {
                const float r7 = 1.0f / 7.0f;             /* 0.14285715f */
                const float inv7 = 1.0f / r7;             /* 6.9999995f  */
                scale = amax > 0.0f ? amax * r7 : 1.0f;
                inv = amax > 0.0f ? inv7 / amax : 1.0f;
            } else {
                scale = amax > 0.0f ? amax / 7.0f : 1.0f;
                inv = 1.0f / scale;
            }
            srow[g] = scale;
            for (size_t j = 0; j < ORC_Q4_GROUP; j += 2) {
                int q0 = round_half_away(grp[j] * inv);
                int q1 = round_half_away(grp[j + 1] * inv);
                if (q0 < -8) q0 = -8;
                if (q0 > 7) q0 = 7;
                if (q1 < -8) q1 = -8;
                if (q1 > 7) q1 = 7;
                qrow[(g * ORC_Q4_GROUP + j) / 2] = (uint8_t)((q0 + 8) | ((q1 + 8) << 4));
            }
        }
    }
    return 0;
}

/* IEEE-754 round-to-nearest-even binary32 -> binary16, the semantics of the (__fp16) cast at
 * src/qmat.c:655.  (third_party/ingot/src/dtype.c:246-268 agrees except for exact ties in the
 * f16 subnormal range, where it rounds half up.) */
uint16_t orc_f32_to_f16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const uint32_t absb = bits & 0x7fffffffu;
    if (absb >= 0x7f800000u) {   /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((absb > 0x7f800000u) ? (0x0200u | ((absb >> 13) & 0x03ffu)) : 0u));
    }
    if (absb >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);   /* rounds to >= 65520 -> inf */
    if (absb < 0x33000001u) return (uint16_t)sign;                /* <= 2^-25 -> 0 (tie to even = 0) */
    const int exponent = (int)(absb >> 23) - 127;
    uint32_t frac = (absb & 0x007fffffu) | 0x00800000u;
    uint32_t half;
    uint32_t shift;
    if (exponent < -14) {   /* subnormal half */
        shift = (uint32_t)(13 + (-14 - exponent));
        half = 0;
    } else {
        shift = 13;
        half = (uint32_t)(exponent + 15 - 1) << 10;   /* implicit one of frac adds the last exponent step */
    }
    const uint32_t kept = frac >> shift;
    const uint32_t rem = frac & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1u);
    uint32_t result = half + kept;
    if (rem > halfway || (rem == halfway && (result & 1u))) result++;
    return (uint16_t)(sign | result);
}

/* third_party/ingot/src/dtype.c:218-244 (exact widening; NaN quieted). */
float orc_f16_to_f32(uint16_t value) {
    const uint32_t sign = (uint32_t)(value & 0x8000u) << 16;
    int exponent = (value >> 10) & 0x1f;
    uint32_t frac = value & 0x03ffu;
    uint32_t bits;
    if (exponent == 0) {
        if (frac == 0) {
            bits = sign;
        } else {
            exponent = 1;
            while ((frac & 0x0400u) == 0) { frac <<= 1; exponent--; }
            bits = sign | ((uint32_t)(exponent + 112) << 23) | ((frac & 0x03ffu) << 13);
        }
    } else if (exponent == 31) {
        bits = sign | 0x7f800000u | (frac << 13) | (frac != 0 ? 0x00400000u : 0u);
    } else {
        bits = sign | ((uint32_t)(exponent + 112) << 23) | (frac << 13);
    }
    float out;
    memcpy(&out, &bits, sizeof out);
    return out;
}

void orc_f32_to_f16_array(const float *in, uint16_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16(in[i]);
}

/* src/qmat.c:94-113.  ORC_STOCK differs only in the returned scale (amax * f32(1/127)). */
float orc_quantize_act_int8(int8_t *qx, const float *x, size_t k, int variant) {
    float amax = 0.0f;
    for (size_t i = 0; i < k; ++i) {
        const float a = fabsf(x[i]);
        if (a > amax) amax = a;
    }
    if (amax == 0.0f) {
        memset(qx, 0, k);
        return 0.0f;
    }
    const float inv = 127.0f / amax;
    for (size_t i = 0; i < k; ++i) {
        int q = round_half_away(x[i] * inv);
        if (q > 127) q = 127;
        if (q < -127) q = -127;
        qx[i] = (int8_t)q;
    }
    if (variant == ORC_STOCK) {
        const float r127 = 1.0f / 127.0f;
        return amax * r127;
    }
    return amax / 127.0f;
}

/* ===================================================================== integer matvecs */

/* src/qmat.c:117-152: exact int32 sum, so evaluation order is irrelevant. */
int32_t orc_dot_q8_i32(const int8_t *qx, const int8_t *w, size_t k) {
    int32_t s = 0;
    for (size_t j = 0; j < k; ++j) s += (int32_t)w[j] * (int32_t)qx[j];
    return s;
}

/* src/qmat.c:191-252: out = (float)s * scale[row] * sx (+ bias), evaluated left to right. */
void orc_matvec_q8(float *out, int32_t *acc_out, const int8_t *qx, float sx, const int8_t *weights,
                   const float *scales, const float *bias, size_t rows, size_t cols) {
    for (size_t row = 0; row < rows; ++row) {
        const int32_t s = orc_dot_q8_i32(qx, weights + row * cols, cols);
        if (acc_out != NULL) acc_out[row] = s;
        float value = (float)s * scales[row];
        value = value * sx;
        if (bias != NULL) value += bias[row];
        out[row] = value;
    }
}

/* src/qmat.c:156-185,254-304: int32 per group of 32, then a sequential f32 sum over groups. */
void orc_matvec_q4(float *out, int32_t *group_acc_out, const int8_t *qx, float sx, const uint8_t *weights,
                   const float *scales, const float *bias, size_t rows, size_t cols) {
    const size_t groups = cols / ORC_Q4_GROUP;
    for (size_t row = 0; row < rows; ++row) {
        const uint8_t *q = weights + row * (cols / 2u);
        const float *srow = scales + row * groups;
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            int32_t gi = 0;
            for (size_t j = 0; j < ORC_Q4_GROUP; j += 2) {
                const uint8_t b = q[g * 16u + j / 2u];
                const int lo = (int)(b & 0x0F) - 8;
                const int hi = (int)(b >> 4) - 8;
                gi += lo * (int32_t)qx[g * 32u + j] + hi * (int32_t)qx[g * 32u + j + 1u];
            }
            if (group_acc_out != NULL) group_acc_out[row * groups + g] = gi;
            const float term = (float)gi * srow[g];
            acc = acc + term;
        }
        float value = acc * sx;
        if (bias != NULL) value += bias[row];
        out[row] = value;
    }
}

/* src/qmat.c:319-377 semantics: halves widened exactly, f32 FMA into two 4-lane accumulators per
 * row (a: elements 0-3, b: 4-7 of each group of 8), s = hsum(a+b), scalar tail. */
void orc_matvec_f16(float *out, const float *x, const uint16_t *weights, const float *bias,
                    size_t rows, size_t cols) {
    for (size_t row = 0; row < rows; ++row) {
        const uint16_t *w = weights + row * cols;
        float a[4] = {0, 0, 0, 0}, b[4] = {0, 0, 0, 0};
        size_t j = 0;
        for (; j + 8u <= cols; j += 8u) {
            for (int l = 0; l < 4; ++l) a[l] = fmaf(orc_f16_to_f32(w[j + l]), x[j + l], a[l]);
            for (int l = 0; l < 4; ++l) b[l] = fmaf(orc_f16_to_f32(w[j + 4 + l]), x[j + 4 + l], b[l]);
        }
        float c[4];
        for (int l = 0; l < 4; ++l) c[l] = a[l] + b[l];
        float s = (c[0] + c[1]) + (c[2] + c[3]);   /* vaddvq_f32 pairwise */
        for (; j < cols; ++j) s += orc_f16_to_f32(w[j]) * x[j];
        out[row] = s + (bias == NULL ? 0.0f : bias[row]);
    }
}

/* src/kernels.c:17-114 (AVX2 form): one 8-lane FMA accumulator per row, lanes summed 0..7,
 * scalar tail, then the bias add of mynah_matvec_bias_f32. */
void orc_matvec_f32(float *out, const float *x, const float *weights, const float *bias,
                    size_t rows, size_t cols) {
    for (size_t row = 0; row < rows; ++row) {
        const float *w = weights + row * cols;
        float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        size_t i = 0;
        for (; i + 8u <= cols; i += 8u)
            for (int l = 0; l < 8; ++l) lanes[l] = fmaf(w[i + l], x[i + l], lanes[l]);
        float s = 0.0f;
        for (int l = 0; l < 8; ++l) s += lanes[l];
        for (; i < cols; ++i) s += w[i] * x[i];
        if (bias != NULL) s += bias[row];
        out[row] = s;
    }
}

/* src/qmat.c:768-818 for one activation row (count == 1).
 * forced_qx / forced_sx (test hook, both or neither): use this int8 activation vector and scale instead of quantising x --
 * what another implementation formed at this very projection.  *flips, when given, is increased by the number of
 * elements in which the forced vector differs from the one quantised here, *max_step raised to the largest such
 * difference: a forced vector from a correct implementation differs only where x sits on a rounding boundary, by 1. */
static void linear_forced(const orc_weight *w, const float *x, float *out, const float *bias, int act_variant,
                          const int8_t *forced_qx, const float *forced_sx, size_t *flips, int *max_step, int8_t *capture_qx, float *capture_sx) {
    if (w->qtype == ORC_F32) {
        orc_matvec_f32(out, x, (const float *)w->data, bias, w->n, w->k);
    } else if (w->qtype == ORC_F16) {
        orc_matvec_f16(out, x, (const uint16_t *)w->data, bias, w->n, w->k);
    } else {
        int8_t *qx = (int8_t *)malloc(w->k);
        float sx = orc_quantize_act_int8(qx, x, w->k, act_variant);
        if (capture_qx != NULL && capture_sx != NULL) {   /* what was quantised here, before any forcing */
            memcpy(capture_qx, qx, w->k);
            *capture_sx = sx;
        }
        if (forced_qx != NULL && forced_sx != NULL) {
            for (size_t i = 0; i < w->k; ++i) {
                const int step = abs((int)qx[i] - (int)forced_qx[i]);
                if (step != 0 && flips != NULL) ++*flips;
                if (max_step != NULL && step > *max_step) *max_step = step;
            }
            memcpy(qx, forced_qx, w->k);
            sx = *forced_sx;
        }
        if (w->qtype == ORC_INT8)
            orc_matvec_q8(out, NULL, qx, sx, (const int8_t *)w->data, w->scales, bias, w->n, w->k);
        else
            orc_matvec_q4(out, NULL, qx, sx, (const uint8_t *)w->data, w->scales, bias, w->n, w->k);
        free(qx);
    }
}

void orc_linear(const orc_weight *w, const float *x, float *out, const float *bias, int act_variant) {
    linear_forced(w, x, out, bias, act_variant, NULL, NULL, NULL, NULL, NULL, NULL);
}

/* ===================================================================== f32 kernels */

/* src/kernels.c:186-244 (AVX2 form): scalar sequential mean; variance through an 8-lane FMA
 * accumulator whose lanes are summed 0..7, scalar tail; y = (x-mean)*scale*gain (+bias). */
void orc_layernorm(const float *in, const float *gain, const float *bias, float *out,
                   size_t rows, size_t width, float eps) {
    for (size_t row = 0; row < rows; ++row) {
        const float *x = in + row * width;
        float *y = out + row * width;
        float mean = 0.0f;
        for (size_t i = 0; i < width; ++i) mean += x[i];
        mean /= (float)width;
        float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        size_t i = 0;
        for (; i + 8u <= width; i += 8u)
            for (int l = 0; l < 8; ++l) {
                const float d = x[i + l] - mean;
                lanes[l] = fmaf(d, d, lanes[l]);
            }
        float variance = 0.0f;
        for (int l = 0; l < 8; ++l) variance += lanes[l];
        for (; i < width; ++i) {
            const float d = x[i] - mean;
            variance += d * d;
        }
        const float scale = 1.0f / sqrtf(variance / (float)width + eps);
        for (i = 0; i < width; ++i) {
            float z = ((x[i] - mean) * scale) * gain[i];
            if (bias != NULL) z += bias[i];
            y[i] = z;
        }
    }
}

/* src/kernels.c:382-389: libm tanhf form, the one the decode step uses (src/graph.c:3265). */
void orc_gelu_scalar(float *data, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        const float x = data[i];
        const float cubic = x * x * x;
        const float c = 0.7978845608f * (x + 0.044715f * cubic);
        data[i] = 0.5f * x * (1.0f + tanhf(c));
    }
}

/* src/kernels.c:259-314: Pade [5/5] tanh clamped to +-6 (prefill, count > 1). */
void orc_gelu_pade(float *data, size_t n) {
    const float p1 = 1.0f / 7.0f, p2 = 4.0f / 855.0f, p3 = 1.0f / 20349.0f, p4 = 1.0f / 6409935.0f,
                p5 = 1.0f / 13749310575.0f;
    const float q1 = 10.0f / 21.0f, q2 = 4.0f / 133.0f, q3 = 8.0f / 14535.0f, q4 = 1.0f / 305235.0f,
                q5 = 2.0f / 416645775.0f;
    for (size_t i = 0; i < n; ++i) {
        const float x = data[i];
        const float x3 = (x * x) * x;
        const float inner = 0.7978845608f * (x + 0.044715f * x3);
        const float u = fminf(fmaxf(inner, -6.0f), 6.0f);
        const float u2 = u * u;
        float num = p5;
        num = fmaf(num, u2, p4);
        num = fmaf(num, u2, p3);
        num = fmaf(num, u2, p2);
        num = fmaf(num, u2, p1);
        num = fmaf(num, u2, 1.0f);
        float den = q5;
        den = fmaf(den, u2, q4);
        den = fmaf(den, u2, q3);
        den = fmaf(den, u2, q2);
        den = fmaf(den, u2, q1);
        den = den * u2 + 1.0f;
        const float t = u * (num / den);
        data[i] = (0.5f * x) * (1.0f + t);
    }
}

/* src/kernels.c:391-420. */
int orc_softmax(const float *logits, float *probs, size_t n) {
    if (n == 0) return -1;
    float maximum = logits[0];
    if (!isfinite(maximum)) return -1;
    for (size_t i = 1; i < n; ++i) {
        if (!isfinite(logits[i])) return -1;
        if (logits[i] > maximum) maximum = logits[i];
    }
    float total = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        probs[i] = expf(logits[i] - maximum);
        total += probs[i];
    }
    if (!(total > 0.0f) || !isfinite(total)) return -1;
    const float inverse_total = 1.0f / total;
    for (size_t i = 0; i < n; ++i) probs[i] *= inverse_total;
    return 0;
}

/* src/graph.c:245-257. */
void orc_softmax_row_inplace(float *values, size_t n) {
    float maximum = -FLT_MAX;
    for (size_t i = 0; i < n; ++i)
        if (values[i] > maximum) maximum = values[i];
    float total = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        values[i] = expf(values[i] - maximum);
        total += values[i];
    }
    const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
    for (size_t i = 0; i < n; ++i) values[i] *= inverse;
}

/* src/backend.c:602-619. */
void orc_softmax_masked(float *data, size_t rows, size_t cols, size_t valid) {
    for (size_t r = 0; r < rows; ++r) {
        float *row = data + r * cols;
        const size_t v = valid < cols ? valid : cols;
        float mx = -1e30f;
        for (size_t i = 0; i < v; ++i) mx = fmaxf(mx, row[i]);
        float sum = 0.0f;
        for (size_t i = 0; i < v; ++i) { row[i] = expf(row[i] - mx); sum += row[i]; }
        const float inv = 1.0f / sum;
        for (size_t i = 0; i < v; ++i) row[i] *= inv;
        for (size_t i = v; i < cols; ++i) row[i] = 0.0f;
    }
}

/* src/kernels.c:246-257. */
void orc_residual_add(float *out, const float *in, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] += in[i];
}

/* src/backend.c:825-847: strict > from -FLT_MAX keeps the first index on ties. */
int orc_argmax_constrained(const float *logits, size_t vocab, size_t codebook_size, size_t eos_id,
                           int allow_eos, unsigned *argmax) {
    if (logits == NULL || argmax == NULL || vocab == 0u || codebook_size > vocab) return -1;
    float best = -FLT_MAX;
    unsigned result = 0u;
    for (size_t i = 0; i < vocab; ++i) {
        if (!(i < codebook_size || (allow_eos && i == eos_id))) continue;
        if (logits[i] > best) {
            best = logits[i];
            result = (unsigned)i;
        }
    }
    *argmax = result;
    return 0;
}

/* ===================================================================== attention */

/* src/graph.c:3182-3202 / 3221-3247 core: per head, sequential dot over d, running max,
 * p = expf(sc - max), denom = sum p, out = sum_s (p_s/denom) * v_s via axpy in s order
 * (axpy_f32, src/graph.c:195-208, scalar form: out[i] += weight * src[i]). */
static void attend_heads(const float *q, const float *k_cache, const float *v_cache, size_t valid,
                         size_t stride, size_t heads, size_t hw, float scale, float *out, float *scores) {
    for (size_t h = 0; h < heads; ++h) {
        const float *qh = q + h * hw;
        float maxv = -FLT_MAX;
        for (size_t s = 0; s < valid; ++s) {
            const float *k = k_cache + s * stride + h * hw;
            float sc = 0.0f;
            for (size_t d = 0; d < hw; ++d) sc += qh[d] * k[d];
            sc *= scale;
            scores[s] = sc;
            if (sc > maxv) maxv = sc;
        }
        float denom = 0.0f;
        for (size_t s = 0; s < valid; ++s) {
            scores[s] = expf(scores[s] - maxv);
            denom += scores[s];
        }
        float *outh = out + h * hw;
        memset(outh, 0, hw * sizeof(float));
        for (size_t s = 0; s < valid; ++s) {
            const float weight = scores[s] / denom;
            const float *v = v_cache + s * stride + h * hw;
            for (size_t d = 0; d < hw; ++d) outh[d] += weight * v[d];
        }
    }
}

/* src/backend.h:139-146 contract; body src/graph.c:3172-3202: append k,v at `position`, then attend
 * over rows [0, valid). */
void orc_self_attention(const float *qkv, float *k_cache, float *v_cache, size_t position,
                        size_t cache_stride, size_t valid, size_t heads, size_t head_width,
                        float scale, float *out, float *scores_scratch) {
    const size_t width = heads * head_width;
    memcpy(k_cache + position * cache_stride, qkv + width, width * sizeof(float));
    memcpy(v_cache + position * cache_stride, qkv + 2u * width, width * sizeof(float));
    attend_heads(qkv, k_cache, v_cache, valid, cache_stride, heads, head_width, scale, out, scores_scratch);
}

/* src/backend.h:147-154 contract; body src/graph.c:3221-3247 generalised to `heads` heads. */
void orc_cross_attention(const float *q, const float *k_cache, const float *v_cache, size_t valid,
                         size_t cache_stride, size_t heads, size_t head_width, float scale,
                         float *out, float *scores_scratch) {
    attend_heads(q, k_cache, v_cache, valid, cache_stride, heads, head_width, scale, out, scores_scratch);
}

/* ===================================================================== decode step */

/* src/graph.c:3127-3284, one slot at a time (the reference's batched form is bit-identical to this
 * per-slot form by its own contract, src/qmat.c:1107-1179).  Generalisations for the synthetic
 * configurations: optional LayerNorm bias, cross_heads x cross_head_width cross attention. */
static int decoder_step_body(const orc_decoder *d, size_t batch, float *const *self_k, float *const *self_v,
                             const float *const *cross_k, const float *const *cross_v,
                             const size_t *lengths, const size_t *memory_lengths,
                             const float *const *inputs, float *const *outs,
                             const int8_t *forced_qx, const float *forced_sx, size_t *flips, int *max_step, int8_t *capture_qx,
                             float *capture_sx) {
    /* forced_qx [layers][6][ffn], forced_sx [layers][6]: stream 0's int8 activations per projection (qkv, o_self, q_cross,
     * o_cross, ffn_up, ffn_down), or NULL */
#define FORCED(slot) (forced_qx != NULL && b == 0 ? forced_qx + (layer * 6u + (slot)) * ffn : NULL), \
                     (forced_sx != NULL && b == 0 ? forced_sx + layer * 6u + (slot) : NULL), flips, max_step, \
                     (capture_qx != NULL && b == 0 ? capture_qx + (layer * 6u + (slot)) * ffn : NULL), \
                     (capture_sx != NULL && b == 0 ? capture_sx + layer * 6u + (slot) : NULL)
    const size_t width = d->width, ffn = d->ffn;
    const size_t xw = d->cross_heads * d->cross_head_width;
    const float self_scale = 1.0f / sqrtf((float)d->head_width);
    const float cross_scale = 1.0f / sqrtf((float)d->cross_head_width);
    size_t max_scores = d->capacity;
    for (size_t b = 0; b < batch; ++b)
        if (memory_lengths[b] > max_scores) max_scores = memory_lengths[b];
    float *x = (float *)malloc(width * sizeof(float));
    float *nrm = (float *)malloc(width * sizeof(float));
    float *qkv = (float *)malloc(3u * width * sizeof(float));
    float *attn = (float *)malloc(width * sizeof(float));
    float *proj = (float *)malloc(width * sizeof(float));
    float *qx = (float *)malloc(xw * sizeof(float));
    float *xctx = (float *)malloc(xw * sizeof(float));
    float *hidden = (float *)malloc(ffn * sizeof(float));
    float *scores = (float *)malloc((max_scores + 1u) * sizeof(float));
    int rc = 0;
    for (size_t b = 0; b < batch && rc == 0; ++b) {
        const size_t start = lengths[b];
        if (start >= d->capacity) { rc = -1; break; }   /* src/graph.c:3152-3155 */
        if (d->position != NULL) {
            const float *pe = d->position + start * width;
            for (size_t i = 0; i < width; ++i) x[i] = inputs[b][i] + pe[i];
        } else {
            memcpy(x, inputs[b], width * sizeof(float));
        }
        for (size_t layer = 0; layer < d->layers; ++layer) {
            const float *bs = d->norm_self_b ? d->norm_self_b + layer * width : NULL;
            const float *bc = d->norm_cross_b ? d->norm_cross_b + layer * width : NULL;
            const float *bf = d->norm_ff_b ? d->norm_ff_b + layer * width : NULL;
            orc_layernorm(x, d->norm_self_g + layer * width, bs, nrm, 1, width, 1.0e-5f);
            linear_forced(&d->qkv[layer], nrm, qkv, NULL, d->act_variant, FORCED(0));
            orc_self_attention(qkv, self_k[b] + layer * d->capacity * width,
                               self_v[b] + layer * d->capacity * width, start, width, start + 1u,
                               d->heads, d->head_width, self_scale, attn, scores);
            linear_forced(&d->o_self[layer], attn, proj, NULL, d->act_variant, FORCED(1));
            for (size_t i = 0; i < width; ++i) x[i] += proj[i];
            if (xw != 0) {
                orc_layernorm(x, d->norm_cross_g + layer * width, bc, nrm, 1, width, 1.0e-5f);
                linear_forced(&d->q_cross[layer], nrm, qx, NULL, d->act_variant, FORCED(2));
                orc_cross_attention(qx, cross_k[b] + layer * memory_lengths[b] * xw,
                                    cross_v[b] + layer * memory_lengths[b] * xw, memory_lengths[b], xw,
                                    d->cross_heads, d->cross_head_width, cross_scale, xctx, scores);
                linear_forced(&d->o_cross[layer], xctx, proj, NULL, d->act_variant, FORCED(3));
                for (size_t i = 0; i < width; ++i) x[i] += proj[i];
            }
            orc_layernorm(x, d->norm_ff_g + layer * width, bf, nrm, 1, width, 1.0e-5f);
            linear_forced(&d->ffn_up[layer], nrm, hidden, NULL, d->act_variant, FORCED(4));
            orc_gelu_scalar(hidden, ffn);
            linear_forced(&d->ffn_down[layer], hidden, proj, NULL, d->act_variant, FORCED(5));
            for (size_t i = 0; i < width; ++i) x[i] += proj[i];
        }
        if (d->norm_out_g != NULL) orc_layernorm(x, d->norm_out_g, d->norm_out_b, outs[b], 1, width, 1.0e-5f);
        else memcpy(outs[b], x, width * sizeof(float));
    }
    free(x); free(nrm); free(qkv); free(attn); free(proj); free(qx); free(xctx); free(hidden); free(scores);
    return rc;
#undef FORCED
}

int orc_decoder_step(const orc_decoder *d, size_t batch, float *const *self_k, float *const *self_v,
                     const float *const *cross_k, const float *const *cross_v,
                     const size_t *lengths, const size_t *memory_lengths,
                     const float *const *inputs, float *const *outs) {
    return decoder_step_body(d, batch, self_k, self_v, cross_k, cross_v, lengths, memory_lengths, inputs, outs, NULL, NULL, NULL, NULL, NULL, NULL);
}

/* Test hook: the same step with stream 0's int8 activations at every projection taken from the caller (see linear_forced;
 * forced_qx / forced_sx may be NULL: nothing forced); counts[0] receives the number of activation elements in which they
 * differ from the ones quantised here, counts[1] the largest difference in int8 steps.  capture_qx / capture_sx (same
 * layout, may be NULL) receive the activations this implementation quantised itself at each projection. */
int orc_decoder_step_forced(const orc_decoder *d, size_t batch, float *const *self_k, float *const *self_v,
                            const float *const *cross_k, const float *const *cross_v,
                            const size_t *lengths, const size_t *memory_lengths,
                            const float *const *inputs, float *const *outs,
                            const int8_t *forced_qx, const float *forced_sx, size_t *counts, int8_t *capture_qx, float *capture_sx) {
    size_t flips = 0;
    int max_step = 0;
    const int rc = decoder_step_body(d, batch, self_k, self_v, cross_k, cross_v, lengths, memory_lengths, inputs, outs, forced_qx, forced_sx,
                                     &flips, &max_step, capture_qx, capture_sx);
    if (counts != NULL) { counts[0] = flips; counts[1] = (size_t)max_step; }
    return rc;
}

/* Output projection + per-head softmax (src/kernels.c:391-420 applied to each codebook head). */
void orc_output_head(const orc_weight *w_out, const float *bias, const float *hidden, size_t heads_out,
                     size_t vocab, float *logits, float *probs, int act_variant) {
    orc_linear(w_out, hidden, logits, bias, act_variant);
    for (size_t h = 0; h < heads_out; ++h) orc_softmax(logits + h * vocab, probs + h * vocab, vocab);
}

/* ===================================================================== encoder prefill */

typedef struct {
    const float *a, *b;
    float *c;
    size_t m, n, k;
    size_t row0, row1;
} gemm_job;

static void gemm_rows(const gemm_job *j) {
    const size_t n = j->n, k = j->k;
    for (size_t i = j->row0; i < j->row1; ++i) {
        const float *ar = j->a + i * k;
        for (size_t col = 0; col < n; ++col) {
            const float *br = j->b + col * k;
            float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            size_t p = 0;
            for (; p + 8u <= k; p += 8u)
                for (int l = 0; l < 8; ++l) lanes[l] = fmaf(ar[p + l], br[p + l], lanes[l]);
            float s = 0.0f;
            for (int l = 0; l < 8; ++l) s += lanes[l];
            for (; p < k; ++p) s += ar[p] * br[p];
            j->c[i * n + col] = s;
        }
    }
}

static void *gemm_thread(void *arg) {
    gemm_rows((const gemm_job *)arg);
    return NULL;
}

/* C[m,n] = A[m,k] B[n,k]^T with the row-times-row dot of orc_matvec_f32, so a prefill row equals
 * the decode matvec of the same row bit for bit. */
void orc_gemm_nt(const float *a, const float *b, float *c, size_t m, size_t n, size_t k, int threads) {
    if (threads < 1) threads = 1;
    if ((size_t)threads > m) threads = (int)m;
    if (threads <= 1) {
        const gemm_job j = {a, b, c, m, n, k, 0, m};
        gemm_rows(&j);
        return;
    }
    pthread_t tid[64];
    gemm_job jobs[64];
    if (threads > 64) threads = 64;
    const size_t per = (m + (size_t)threads - 1u) / (size_t)threads;
    int started = 0;
    for (int t = 0; t < threads; ++t) {
        const size_t r0 = (size_t)t * per;
        if (r0 >= m) break;
        const size_t r1 = r0 + per > m ? m : r0 + per;
        jobs[t] = (gemm_job){a, b, c, m, n, k, r0, r1};
        pthread_create(&tid[t], NULL, gemm_thread, &jobs[t]);
        started++;
    }
    for (int t = 0; t < started; ++t) pthread_join(tid[t], NULL);
}

/* Causal unfold of [T, channels] rows over `kernel` taps (unfold_causal, src/graph.c:271-286):
 * col[t][i * kernel + j] = input[t - (kernel - 1) + j][i], zero before the start. */
static void unfold_rows(const float *input, float *col, size_t T, size_t channels, size_t kernel) {
    for (size_t t = 0; t < T; ++t)
        for (size_t j = 0; j < kernel; ++j) {
            const long src = (long)t - (long)(kernel - 1u) + (long)j;
            for (size_t i = 0; i < channels; ++i)
                col[(t * channels + i) * kernel + j] = src < 0 ? 0.0f : input[(size_t)src * channels + i];
        }
}

/* Text-encoder prefill (transformer_stack, src/graph.c:634-711, as encode_text calls it, :738-740): gather
 * (:729-737) + position add (:649-651), then per layer pre-LN -> QKV -> per-head scaled QK^T -> row softmax
 * (softmax_row_inplace, :245-257) -> PV -> O -> +res (:387-470) -> LN -> FFN -> +res; optional final norm (:696-701).
 *   causal != 0: row t attends rows [0, t] only and the rest of its weights are zero (:446-449), the reference's form;
 *                causal == 0: the full row (the synthetic bidirectional configuration).
 *   ffn_kernel == 1: plain FFN with the scalar GELU (:302-316); ffn_kernel > 1: the causal conv FFN as one product
 *                over the unfolded rows, weights [out][in][kernel] (:317-352); 0 means 1.
 * Weights are f16 values widened exactly; all arithmetic f32. */
int orc_encoder_prefill(const orc_encoder *e, const int32_t *ids, size_t T, uint16_t *embed_out,
                        float *out, int threads) {
    const size_t w = e->width, f = e->ffn, H = e->heads, hw = e->head_width;
    if (T == 0 || T > e->max_positions || H * hw != w) return -1;
    for (size_t t = 0; t < T; ++t)
        if (ids[t] < 0 || (size_t)ids[t] >= e->vocab) return -1;   /* src/graph.c:730-735 */
    float *x = (float *)malloc(T * w * sizeof(float));
    float *nrm = (float *)malloc(T * w * sizeof(float));
    float *qkv = (float *)malloc(T * 3u * w * sizeof(float));
    float *ctx = (float *)malloc(T * w * sizeof(float));
    float *proj = (float *)malloc(T * w * sizeof(float));
    float *hidden = (float *)malloc(T * f * sizeof(float));
    float *scores = (float *)malloc(T * T * sizeof(float));
    float *qh = (float *)malloc(T * hw * sizeof(float));
    float *kh = (float *)malloc(T * hw * sizeof(float));
    float *vt = (float *)malloc(T * hw * sizeof(float));
    float *hc = (float *)malloc(T * hw * sizeof(float));
    const size_t kn = e->ffn_kernel == 0 ? 1u : e->ffn_kernel;
    const size_t wmax = 3u * w * w > f * w * kn ? 3u * w * w : f * w * kn;
    float *wf = (float *)malloc(wmax * sizeof(float));
    float *col = kn > 1u ? (float *)malloc(T * (f > w ? f : w) * kn * sizeof(float)) : NULL;
    for (size_t t = 0; t < T; ++t) {
        const uint16_t *row = e->tok_table + (size_t)ids[t] * w;
        const uint16_t *pos = e->pos_table + t * w;
        if (embed_out != NULL) memcpy(embed_out + t * w, row, w * sizeof(uint16_t));
        for (size_t i = 0; i < w; ++i) x[t * w + i] = orc_f16_to_f32(row[i]) + orc_f16_to_f32(pos[i]);
    }
    const float scale = 1.0f / sqrtf((float)hw);
    for (size_t layer = 0; layer < e->layers; ++layer) {
        orc_layernorm(x, e->norm1_g + layer * w, e->norm1_b ? e->norm1_b + layer * w : NULL, nrm, T, w, 1.0e-5f);
        for (size_t i = 0; i < 3u * w * w; ++i) wf[i] = orc_f16_to_f32(e->qkv_w[layer * 3u * w * w + i]);
        orc_gemm_nt(nrm, wf, qkv, T, 3u * w, w, threads);
        for (size_t h = 0; h < H; ++h) {
            for (size_t t = 0; t < T; ++t) {
                const float *row = qkv + t * 3u * w;
                memcpy(qh + t * hw, row + h * hw, hw * sizeof(float));
                memcpy(kh + t * hw, row + w + h * hw, hw * sizeof(float));
                for (size_t dd = 0; dd < hw; ++dd) vt[dd * T + t] = row[2u * w + h * hw + dd];
            }
            orc_gemm_nt(qh, kh, scores, T, T, hw, threads);
            for (size_t t = 0; t < T; ++t) {
                for (size_t s = 0; s < T; ++s) scores[t * T + s] *= scale;
                if (e->causal) {
                    orc_softmax_row_inplace(scores + t * T, t + 1u);
                    for (size_t s = t + 1u; s < T; ++s) scores[t * T + s] = 0.0f;
                } else {
                    orc_softmax_row_inplace(scores + t * T, T);
                }
            }
            orc_gemm_nt(scores, vt, hc, T, hw, T, threads);
            for (size_t t = 0; t < T; ++t) memcpy(ctx + t * w + h * hw, hc + t * hw, hw * sizeof(float));
        }
        for (size_t i = 0; i < w * w; ++i) wf[i] = orc_f16_to_f32(e->o_w[layer * w * w + i]);
        orc_gemm_nt(ctx, wf, proj, T, w, w, threads);
        for (size_t i = 0; i < T * w; ++i) x[i] += proj[i];
        orc_layernorm(x, e->norm2_g + layer * w, e->norm2_b ? e->norm2_b + layer * w : NULL, nrm, T, w, 1.0e-5f);
        for (size_t i = 0; i < f * w * kn; ++i) wf[i] = orc_f16_to_f32(e->up_w[layer * f * w * kn + i]);
        if (kn == 1u) {
            orc_gemm_nt(nrm, wf, hidden, T, f, w, threads);
        } else {
            unfold_rows(nrm, col, T, w, kn);
            orc_gemm_nt(col, wf, hidden, T, f, w * kn, threads);
        }
        orc_gelu_scalar(hidden, T * f);
        for (size_t i = 0; i < w * f * kn; ++i) wf[i] = orc_f16_to_f32(e->down_w[layer * w * f * kn + i]);
        if (kn == 1u) {
            orc_gemm_nt(hidden, wf, proj, T, w, f, threads);
        } else {
            unfold_rows(hidden, col, T, f, kn);
            orc_gemm_nt(col, wf, proj, T, w, f * kn, threads);
        }
        for (size_t i = 0; i < T * w; ++i) x[i] += proj[i];
    }
    if (e->norm_out_g != NULL) orc_layernorm(x, e->norm_out_g, e->norm_out_b, out, T, w, 1.0e-5f);
    else memcpy(out, x, T * w * sizeof(float));
    free(x); free(nrm); free(qkv); free(ctx); free(proj); free(hidden); free(scores);
    free(qh); free(kh); free(vt); free(hc); free(wf); free(col);
    return 0;
}

/* ---- local transformer frame ------------------------------------------------------------------------------------ */

unsigned orc_local_choose(float *logits, size_t vocab, size_t codebook_size, size_t eos_id, orc_local_item *item,
                          unsigned *greedy, size_t *top_indices, float *top_values) {
    const int sampling = item->temperature > 0.0f && item->topk > 1u;   /* src/graph.c:1549-1550 (rng_state always present here) */
    const size_t top_count = item->topk < vocab ? item->topk : vocab;
    /* src/graph.c:1556-1570: mask and first-max argmax */
    float best = -FLT_MAX;
    unsigned argmax = 0;
    for (size_t c = 0; c < vocab; ++c) {
        const int is_code = c < codebook_size;
        const int is_eos = c == eos_id;
        if (!is_code && !(is_eos && !item->forbid_eos)) {
            logits[c] = -FLT_MAX;
            continue;
        }
        if (logits[c] > best) {
            best = logits[c];
            argmax = (unsigned)c;
        }
    }
    if (greedy != NULL) *greedy = argmax;
    unsigned value = argmax;
    if (sampling) {
        /* src/graph.c:1577-1598: stable insertion of every candidate into a descending list of top_count */
        size_t used = 0;
        for (size_t c = 0; c < vocab; ++c) {
            size_t insert = used;
            while (insert > 0 && logits[c] > top_values[insert - 1u]) --insert;
            if (used < top_count) {
                for (size_t q = used; q > insert; --q) {
                    top_indices[q] = top_indices[q - 1u];
                    top_values[q] = top_values[q - 1u];
                }
                top_indices[insert] = c;
                top_values[insert] = logits[c];
                ++used;
            } else if (insert < top_count) {
                for (size_t q = top_count - 1u; q > insert; --q) {
                    top_indices[q] = top_indices[q - 1u];
                    top_values[q] = top_values[q - 1u];
                }
                top_indices[insert] = c;
                top_values[insert] = logits[c];
            }
        }
        /* src/graph.c:1599-1616 */
        const float maximum = top_values[0];
        float total = 0.0f;
        for (size_t q = 0; q < used; ++q) {
            top_values[q] = expf((top_values[q] - maximum) / item->temperature);
            total += top_values[q];
        }
        uint64_t bits = item->rng_state;
        bits ^= bits << 13;
        bits ^= bits >> 7;
        bits ^= bits << 17;
        item->rng_state = bits == 0 ? UINT64_C(0x9e3779b97f4a7c15) : bits;
        const float draw = ((float)((item->rng_state >> 40) & UINT64_C(0xffffff)) / (float)UINT64_C(0x1000000)) * total;
        float cumulative = 0.0f;
        for (size_t q = 0; q < used; ++q) {
            cumulative += top_values[q];
            if (draw <= cumulative || q + 1u == used) {
                value = (unsigned)top_indices[q];
                break;
            }
        }
    }
    return value;
}

int orc_local_frame(const orc_local *L, size_t batch, const float *const *decoder_last, orc_local_item *items,
                    float *const *k, float *const *v, unsigned *values, unsigned *stored, int *saw_eos,
                    size_t *eos_frame, float *logits_out) {
    const orc_decoder *d = L->stack;
    const size_t width = d->width, vocab = L->vocab;
    if (batch == 0 || batch > 16 || d->cross_heads * d->cross_head_width != 0 || d->capacity < L->streams) return -1;
    float *row_in = (float *)malloc(batch * width * sizeof(float));
    float *row_out = (float *)malloc(batch * width * sizeof(float));
    float *logits = (float *)malloc(vocab * sizeof(float));
    size_t max_top = 1;
    for (size_t b = 0; b < batch; ++b)
        if (items[b].topk > max_top) max_top = items[b].topk;
    if (max_top > vocab) max_top = vocab;
    size_t *top_indices = (size_t *)malloc(max_top * sizeof(size_t));
    float *top_values = (float *)malloc(max_top * sizeof(float));
    const float *in_ptrs[16];
    float *out_ptrs[16];
    size_t lengths[16], no_memory[16];
    for (size_t b = 0; b < batch; ++b) {
        memcpy(row_in + b * width, decoder_last[b], width * sizeof(float));   /* src/graph.c:1421 */
        in_ptrs[b] = row_in + b * width;
        out_ptrs[b] = row_out + b * width;
        saw_eos[b] = 0;
        eos_frame[b] = SIZE_MAX;
        no_memory[b] = 0;
    }
    int rc = 0;
    for (size_t stream = 0; stream < L->streams && rc == 0; ++stream) {
        for (size_t b = 0; b < batch; ++b) lengths[b] = stream;   /* cache.length restarts at 0 every frame (:1412) */
        rc = orc_decoder_step(d, batch, k, v, NULL, NULL, lengths, no_memory, in_ptrs, out_ptrs);
        if (rc != 0) break;
        for (size_t b = 0; b < batch; ++b) {
            /* the same projection weight for every item of this stream (:1536-1547) */
            orc_linear(&L->projection[stream], out_ptrs[b], logits, L->projection_bias != NULL ? L->projection_bias[stream] : NULL,
                       d->act_variant);
            unsigned greedy = 0;
            const unsigned value = orc_local_choose(logits, vocab, L->codebook_size, L->eos_id, &items[b], &greedy, top_indices,
                                                    top_values);
            if (logits_out != NULL) memcpy(logits_out + (b * L->streams + stream) * vocab, logits, vocab * sizeof(float));
            if (greedy == L->eos_id || value == L->eos_id) {   /* :1572-1574, :1617-1622 */
                saw_eos[b] = 1;
                const size_t frame = stream / L->codebook_count;
                if (frame < eos_frame[b]) eos_frame[b] = frame;
            }
            const unsigned emit = value < vocab ? value : 0u;                    /* :1626 */
            values[b * L->streams + stream] = value;
            stored[b * L->streams + stream] = value < L->codebook_size ? value : 0u;   /* :1627 */
            memcpy(row_in + b * width, L->audio_table[stream] + (size_t)emit * width, width * sizeof(float));   /* :1651 */
        }
    }
    free(row_in); free(row_out); free(logits); free(top_indices); free(top_values);
    return rc;
}


/* ---- codec operators ------------------------------------------------------------------------------------ */

void orc_conv1d_causal(const float *input, float *output, size_t in_channels, size_t out_channels, size_t length,
                       size_t kernel, size_t dilation, const float *weight, const float *bias) {
    /* src/graph.c:2141-2154 */
    for (size_t o = 0; o < out_channels; ++o) {
        for (size_t t = 0; t < length; ++t) {
            float value = bias != NULL ? bias[o] : 0.0f;
            for (size_t i = 0; i < in_channels; ++i) {
                for (size_t k = 0; k < kernel; ++k) {
                    const long source = (long)t - (long)((kernel - 1u) * dilation) + (long)(k * dilation);
                    if (source >= 0) value += weight[(o * in_channels + i) * kernel + k] * input[i * length + (size_t)source];
                }
            }
            output[o * length + t] = value;
        }
    }
}

void orc_conv_transpose_causal(const float *input, float *output, size_t in_channels, size_t out_channels, size_t length,
                               size_t output_length, size_t kernel, size_t stride, size_t groups, const float *weight,
                               const float *bias) {
    /* src/graph.c:2179-2198 */
    const size_t in_per_group = in_channels / groups, out_per_group = out_channels / groups;
    for (size_t o = 0; o < out_channels; ++o) {
        const size_t group = o / out_per_group, o_local = o % out_per_group;
        float *row = output + o * output_length;
        for (size_t t = 0; t < output_length; ++t) row[t] = bias != NULL ? bias[o] : 0.0f;
        for (size_t i = group * in_per_group; i < (group + 1) * in_per_group; ++i) {
            const float *in_row = input + i * length;
            const float *w = weight + (i * out_per_group + o_local) * kernel;
            for (size_t t = 0; t < length; ++t) {
                const float in_v = in_row[t];
                for (size_t k = 0; k < kernel; ++k) {
                    const size_t position = t * stride + k;
                    if (position < output_length) row[position] += in_v * w[k];
                }
            }
        }
    }
}

void orc_snake(float *data, const float *alpha, size_t channels, size_t length, size_t snake_channels) {
    /* src/backend.c:643-658 */
    for (size_t c = 0; c < channels; ++c) {
        float *row = data + c * length;
        if (c < snake_channels) {
            const float a = alpha[c];
            const float inv_a = 1.0f / (a + 1e-9f);
            for (size_t t = 0; t < length; ++t) {
                const float v = row[t];
                const float sn = sinf(a * v);
                row[t] = v + sn * sn * inv_a;
            }
        } else {
            for (size_t t = 0; t < length; ++t)
                if (row[t] < 0.0f) row[t] *= 0.01f;
        }
    }
}
