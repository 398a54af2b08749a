/*
 * Plain-C restatement of the reference's naive attention.  TEST INFRASTRUCTURE ONLY: linked by
 * the tests (through ctypes) to pin the torch oracle with an independent implementation; never
 * linked or called by the product library.
 *
 * Follows reference tests/naive_implementation.py:4-18 literally, one scalar at a time:
 *   head h of a [B, L, R*H] tensor is columns [h*H, (h+1)*H)           (:8-10, and the kernel's
 *                                                 own indexing, reference include/fused_attn.cuh:683-690)
 *   score(i, j) = sum_d q[i][d] * k[j][d] / sqrt(H)                     (:12)
 *   p(i, j)     = exp(score(i, j) - max_j score) / sum_j exp(...)       (:13)
 *   out[i][d]   = sum_j p(i, j) * v[j][d]                               (:14)
 * Inputs are float32 arrays holding the exactly upcast fp16 values; all arithmetic is double.
 * mask may be NULL; otherwise additive [B, L, L] float32 shared by all heads (reference
 * README.md:88-89).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

int attention_ref_f64(const float* q, const float* k, const float* v, const float* mask, double* out,
                      int64_t B, int64_t L, int64_t R, int64_t H) {
    const int64_t F = R * H;
    const double inv_sqrt_h = 1.0 / sqrt((double)H);
    double* p = (double*)malloc((size_t)L * sizeof(double));
    if (p == NULL) return -1;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t h = 0; h < R; ++h) {
            const float* qb = q + b * L * F + h * H;
            const float* kb = k + b * L * F + h * H;
            const float* vb = v + b * L * F + h * H;
            double* ob = out + b * L * F + h * H;
            for (int64_t i = 0; i < L; ++i) {
                double mx = -INFINITY;
                for (int64_t j = 0; j < L; ++j) {
                    double acc = 0.0;
                    for (int64_t d = 0; d < H; ++d) acc += (double)qb[i * F + d] * (double)kb[j * F + d];
                    acc *= inv_sqrt_h;
                    if (mask != NULL) acc += (double)mask[(b * L + i) * L + j];
                    p[j] = acc;
                    if (acc > mx) mx = acc;
                }
                double den = 0.0;
                for (int64_t j = 0; j < L; ++j) {
                    p[j] = exp(p[j] - mx);
                    den += p[j];
                }
                for (int64_t d = 0; d < H; ++d) {
                    double acc = 0.0;
                    for (int64_t j = 0; j < L; ++j) acc += p[j] * (double)vb[j * F + d];
                    ob[i * F + d] = acc / den;
                }
            }
        }
    }
    free(p);
    return 0;
}
