/* CPU oracle in plain C for the sparse-mask-attention hot path.  TEST INFRASTRUCTURE ONLY:
 * it is built into oracle/libsma_oracle.so and loaded by the tests, the smoke check and the
 * benchmark's CPU-baseline leg, never by the shipped library.
 *
 * It is a second, independent statement (different language, scalar double arithmetic) of
 * what oracle/sma_oracle.py states with numpy/torch, so that the two can check each other.
 *
 * oracle_pack_mask   bit format of the reference packer, csrc/sparse_attention.cu:549-568:
 *                    word w of row i holds columns 32w..32w+31, column 32w+j in bit j,
 *                    bits for columns >= N are zero.
 * oracle_attn_fwd    the masked softmax attention of python/sparse_attention.py:29-42
 *                    (scores*scale, -inf where mask is false, softmax, NaN rows -> 0, times V),
 *                    one query row at a time in double precision; lse as in
 *                    python/sparse_attention.py:72-74 (-inf for a row that keeps no key).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

int oracle_pack_mask(const uint8_t *mask, uint32_t *packed, int B, int H, int N)
{
    if (!mask || !packed || B < 0 || H < 0 || N < 0) return -1;
    const int nw = (N + 31) / 32;
    const long rows = (long)B * H * N;
    for (long r = 0; r < rows; ++r) {
        const uint8_t *src = mask + r * (long)N;
        uint32_t *dst = packed + r * (long)nw;
        for (int w = 0; w < nw; ++w) {
            uint32_t acc = 0;
            for (int j = 0; j < 32; ++j) {
                const int col = 32 * w + j;
                if (col < N && src[col]) acc |= (uint32_t)1 << j;
            }
            dst[w] = acc;
        }
    }
    return 0;
}

int oracle_attn_fwd(const float *q, const float *k, const float *v, const uint8_t *mask,
                    float *out, float *lse, int B, int H, int N, int D, float scale)
{
    if (!q || !k || !v || !mask || !out || B < 0 || H < 0 || N < 0 || D <= 0) return -1;
    double *s = (double *)malloc(sizeof(double) * (size_t)(N > 0 ? N : 1));
    double *o = (double *)malloc(sizeof(double) * (size_t)D);
    if (!s || !o) { free(s); free(o); return -2; }
    for (long bh = 0; bh < (long)B * H; ++bh) {
        const float *qb = q + bh * (long)N * D, *kb = k + bh * (long)N * D, *vb = v + bh * (long)N * D;
        const uint8_t *mb = mask + bh * (long)N * N;
        for (int i = 0; i < N; ++i) {
            double mx = -INFINITY;
            for (int j = 0; j < N; ++j) {
                if (!mb[(long)i * N + j]) { s[j] = -INFINITY; continue; }
                double acc = 0.0;
                for (int d = 0; d < D; ++d) acc += (double)qb[(long)i * D + d] * (double)kb[(long)j * D + d];
                s[j] = acc * (double)scale;
                if (s[j] > mx) mx = s[j];
            }
            for (int d = 0; d < D; ++d) o[d] = 0.0;
            double den = 0.0;
            if (mx > -INFINITY) {
                for (int j = 0; j < N; ++j) {
                    if (s[j] == -INFINITY) continue;
                    const double p = exp(s[j] - mx);
                    den += p;
                    for (int d = 0; d < D; ++d) o[d] += p * (double)vb[(long)j * D + d];
                }
            }
            for (int d = 0; d < D; ++d)
                out[(bh * N + i) * (long)D + d] = (float)(den > 0.0 ? o[d] / den : 0.0);
            if (lse) lse[bh * N + i] = (float)(den > 0.0 ? mx + log(den) : -INFINITY);
        }
    }
    free(s); free(o);
    return 0;
}
