/* Plain-C float64 restatement of the attention column-mean oracle.
 * TEST INFRASTRUCTURE ONLY: linked by nothing in the shipped library.
 *
 * Follows reference flash_colsum/baselines.py:35-78:
 *   score(i,j) = scale * sum_d q[i][d] * k[j][d]                 (baselines.py:42)
 *   causal: j visible to i  <=>  j <= max(0, Sk - Sq) + i       (baselines.py:49-62,
 *                                                    kernel_causal.py:39,57,113)
 *   p(i,j)  = exp(score - rowmax) / sum_j exp(score - rowmax)   (baselines.py:66)
 *   rows    = min(cls_len, Sq) when cls_len > 0 and not causal  (baselines.py:68-73)
 *   out[b][j] = (1 / (H * rows)) * sum_h sum_{i < rows} p(i,j)  (baselines.py:73,76)
 * Inputs are dense row-major (B,H,Sq,D) and (B,H,Sk,D) float32; everything else is
 * double.  No BLAS, no vector intrinsics: one scalar triple loop.
 */
#include <math.h>
#include <stdlib.h>

int colsum_ref(const float *q, const float *k, double *out, int B, int H, int Sq,
               int Sk, int D, double scale, int causal, int cls_len)
{
    if (!q || !k || !out || B < 1 || H < 1 || Sq < 1 || Sk < 1 || D < 1)
        return -1;
    int rows = Sq;
    if (!causal && cls_len > 0 && cls_len < Sq)
        rows = cls_len;
    const long k_past = (Sk > Sq) ? (long)(Sk - Sq) : 0;
    double *s = (double *)malloc(sizeof(double) * (size_t)Sk);
    if (!s)
        return -2;
    for (long n = 0; n < (long)B * Sk; ++n)
        out[n] = 0.0;
    for (int b = 0; b < B; ++b) {
        for (int h = 0; h < H; ++h) {
            const float *qh = q + ((size_t)b * H + h) * (size_t)Sq * D;
            const float *kh = k + ((size_t)b * H + h) * (size_t)Sk * D;
            for (int i = 0; i < rows; ++i) {
                long last = Sk - 1;
                if (causal && k_past + i < last)
                    last = k_past + i;
                double top = -INFINITY;
                for (long j = 0; j <= last; ++j) {
                    double acc = 0.0;
                    for (int d = 0; d < D; ++d)
                        acc += (double)qh[(size_t)i * D + d] * (double)kh[(size_t)j * D + d];
                    s[j] = acc * scale;
                    if (s[j] > top)
                        top = s[j];
                }
                double denom = 0.0;
                for (long j = 0; j <= last; ++j) {
                    s[j] = exp(s[j] - top);
                    denom += s[j];
                }
                for (long j = 0; j <= last; ++j)
                    out[(size_t)b * Sk + j] += s[j] / denom;
            }
        }
    }
    const double inv = 1.0 / ((double)H * rows);
    for (long n = 0; n < (long)B * Sk; ++n)
        out[n] *= inv;
    free(s);
    return 0;
}

/* The same triple loop for the shapes beyond the reference operator's domain: Hq query heads
 * over Hk key heads (query head h reads key head h / (Hq / Hk)), any batch size with the causal
 * mask, an explicit k_past (negative: max(0, Sk - Sq)), and cls_len (> 0) honoured with the
 * causal mask too.  With Hq == Hk, k_past < 0 and no cls_len under the mask it equals colsum_ref. */
int colsum_ref_ext(const float *q, const float *k, double *out, int B, int Hq, int Hk, int Sq,
                   int Sk, int D, double scale, int causal, int cls_len, long k_past)
{
    if (!q || !k || !out || B < 1 || Hq < 1 || Hk < 1 || Hq % Hk || Sq < 1 || Sk < 1 || D < 1)
        return -1;
    const int grp = Hq / Hk;
    int rows = Sq;
    if (cls_len > 0 && cls_len < Sq)
        rows = cls_len;
    if (k_past < 0)
        k_past = (Sk > Sq) ? (long)(Sk - Sq) : 0;
    double *s = (double *)malloc(sizeof(double) * (size_t)Sk);
    if (!s)
        return -2;
    for (long n = 0; n < (long)B * Sk; ++n)
        out[n] = 0.0;
    for (int b = 0; b < B; ++b) {
        for (int h = 0; h < Hq; ++h) {
            const float *qh = q + ((size_t)b * Hq + h) * (size_t)Sq * D;
            const float *kh = k + ((size_t)b * Hk + h / grp) * (size_t)Sk * D;
            for (int i = 0; i < rows; ++i) {
                long last = Sk - 1;
                if (causal && k_past + i < last)
                    last = k_past + i;
                double top = -INFINITY;
                for (long j = 0; j <= last; ++j) {
                    double acc = 0.0;
                    for (int d = 0; d < D; ++d)
                        acc += (double)qh[(size_t)i * D + d] * (double)kh[(size_t)j * D + d];
                    s[j] = acc * scale;
                    if (s[j] > top)
                        top = s[j];
                }
                double denom = 0.0;
                for (long j = 0; j <= last; ++j) {
                    s[j] = exp(s[j] - top);
                    denom += s[j];
                }
                for (long j = 0; j <= last; ++j)
                    out[(size_t)b * Sk + j] += s[j] / denom;
            }
        }
    }
    const double inv = 1.0 / ((double)Hq * rows);
    for (long n = 0; n < (long)B * Sk; ++n)
        out[n] *= inv;
    free(s);
    return 0;
}
