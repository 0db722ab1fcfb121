/* TEST INFRASTRUCTURE ONLY -- never linked into, loaded by, or timed as the product.
 *
 * Exposes the file-local functions of the reference's quantized-linear
 * translation unit through plain C wrappers.  The reference source itself is
 * NOT copied: the compiler reads it from where it lies under the reference
 * tree (the include below resolves through -I<reference>/src given by
 * oracle/Makefile), and the resulting object lives only in oracle/_ref/.
 *
 * Wrapped reference functions (file:line in the reference tree):
 *   quantize_weight_int8   src/qmat.c:39-57
 *   quantize_weight_int4   src/qmat.c:61-91
 *   quantize_act_int8      src/qmat.c:94-113
 *   dot_q8 / dot_q4        src/qmat.c:136-152 / 156-185
 *   matvec_q8 / matvec_q4  src/qmat.c:191-252 / 254-304
 *   qmat_rows_block        src/qmat.c:423-430  (32-row block partition)
 * The public API of that file (mynah_qmat_linear_resolved, _batched, _self_test,
 * cache_new/free) is exported by the same object unchanged.
 */
#include "qmat.c"

void ref_quantize_weight_int8(const float *w, size_t n, size_t k, int8_t *q, float *scales) {
    quantize_weight_int8(w, n, k, q, scales);
}

void ref_quantize_weight_int4(const float *w, size_t n, size_t k, uint8_t *q, float *scales) {
    quantize_weight_int4(w, n, k, q, scales);
}

float ref_quantize_act_int8(int8_t *qx, const float *x, size_t k) {
    return quantize_act_int8(qx, x, k);
}

float ref_dot_q8(const int8_t *qx, float sx, const int8_t *w, float ws, size_t k) {
    return dot_q8(qx, sx, w, ws, k);
}

float ref_dot_q4(const int8_t *qx, float sx, const uint8_t *q, const float *scales, size_t k) {
    return dot_q4(qx, sx, q, scales, k);
}

void ref_matvec_q8(float *out, const int8_t *qx, float sx, const int8_t *weights,
                   const float *scales, const float *bias, size_t rows, size_t cols) {
    matvec_q8(out, qx, sx, weights, scales, bias, rows, cols);
}

void ref_matvec_q4(float *out, const int8_t *qx, float sx, const uint8_t *weights,
                   const float *scales, const float *bias, size_t rows, size_t cols) {
    matvec_q4(out, qx, sx, weights, scales, bias, rows, cols);
}

/* Row-blocked dispatch exactly as the reference's pool would partition it, walked serially. */
void ref_matvec_rows_blocked(float *out, const int8_t *qx, float sx, const void *weights,
                             const float *scales, const float *bias, size_t rows, size_t cols,
                             int qtype) {
    const qmat_rows_job job = {out, qx, NULL, sx, weights, scales, bias, rows, cols, qtype};
    const int blocks = (int)((rows + QMAT_ROW_BLOCK - 1u) / QMAT_ROW_BLOCK);
    for (int b = 0; b < blocks; ++b) qmat_rows_block((void *)&job, b);
}

/* Threaded matvec through the reference's own pool (the CPU baseline's inner call). */
void ref_matvec_q_rows(float *out, const int8_t *qx, float sx, const void *weights,
                       const float *scales, const float *bias, size_t rows, size_t cols,
                       int qtype) {
    matvec_q_rows(out, qx, NULL, sx, weights, scales, bias, rows, cols, qtype);
}

int ref_num_threads(void) { return mynah_num_threads(); }
