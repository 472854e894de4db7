/*
 * Plain-C restatement of the attention-JVP path (fp64).  TEST INFRASTRUCTURE ONLY: linked by nothing
 * in the product; loaded by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
 *
 * Reference (olsdavis/semicat) being restated:
 *   forward   O, TO, M (= lse), MU, LI      semicat/jvp_utils/ryu_triton.py:188-291
 *   backward  sum_4, sum_7                  semicat/jvp_utils/flash_jvp_backward.py:2266-2287
 *             dS_dot = P*(dTO V^T - sum_4)  flash_jvp_backward.py:251-257
 *             P_dot  = P*(S_dot - mu)       flash_jvp_backward.py:947-954
 *             dS (tangent cotangent part)   flash_jvp_backward.py:1364-1407
 *             dS (primal cotangent part)    semicat/jvp_utils/flash_attn_triton.py:600-610
 *             delta = rowsum(O*dO)          flash_attn_triton.py:317-363
 *   math path it must agree with            ryu_triton.py:426-454
 *
 * Layout: every tensor is [BH][L][D] contiguous doubles; statistics are [BH][Lr] with
 * Lr = ceil(Lq/128)*128 and rows >= Lq holding log(Lk), 0, Lk (functional.py:57-59,228-229).
 * The loops are written row by row, two passes per row, with no blocking: a third implementation
 * independent of the numpy closed forms and of torch autograd.  Pinned in tests/test_oracle.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double dot(const double *a, const double *b, int n) {
    double s = 0.0;
    for (int i = 0; i < n; ++i) s += a[i] * b[i];
    return s;
}

int attn_jvp_ref_forward(const double *q, const double *k, const double *v, const double *tq,
                         const double *tk, const double *tv, double *o, double *to, double *lse,
                         double *mu, double *li, int64_t BH, int64_t Lq, int64_t Lk, int64_t D,
                         double scale) {
    int64_t Lr = ((Lq + 127) / 128) * 128;
    double *s = (double *)malloc(sizeof(double) * (size_t)Lk * 2);
    if (!s) return -1;
    double *ts = s + Lk;
    for (int64_t g = 0; g < BH; ++g) {
        const double *kg = k + g * Lk * D, *vg = v + g * Lk * D;
        const double *tkg = tk + g * Lk * D, *tvg = tv + g * Lk * D;
        for (int64_t i = 0; i < Lr; ++i) {
            if (i >= Lq) {
                lse[g * Lr + i] = log((double)Lk);
                mu[g * Lr + i] = 0.0;
                li[g * Lr + i] = (double)Lk;
                continue;
            }
            const double *qi = q + (g * Lq + i) * D, *tqi = tq + (g * Lq + i) * D;
            double m = -INFINITY;
            for (int64_t j = 0; j < Lk; ++j) {
                s[j] = scale * dot(qi, kg + j * D, (int)D);
                ts[j] = scale * (dot(tqi, kg + j * D, (int)D) + dot(qi, tkg + j * D, (int)D));
                if (s[j] > m) m = s[j];
            }
            double l = 0.0, mu_un = 0.0;
            for (int64_t j = 0; j < Lk; ++j) {
                s[j] = exp(s[j] - m);
                l += s[j];
                mu_un += s[j] * ts[j];
            }
            double mui = mu_un / l;
            double *oi = o + (g * Lq + i) * D, *toi = to + (g * Lq + i) * D;
            for (int64_t d = 0; d < D; ++d) {
                double a = 0.0, b = 0.0;
                for (int64_t j = 0; j < Lk; ++j) {
                    double p = s[j] / l;
                    a += p * vg[j * D + d];
                    b += p * (ts[j] - mui) * vg[j * D + d] + p * tvg[j * D + d];
                }
                oi[d] = a;
                toi[d] = b;
            }
            lse[g * Lr + i] = m + log(l);
            mu[g * Lr + i] = mui;
            li[g * Lr + i] = l;
        }
    }
    free(s);
    return 0;
}

/* dO or dTO may be NULL (treated as zero).  o, to, lse, mu come from the forward. */
int attn_jvp_ref_backward(const double *q, const double *k, const double *v, const double *tq,
                          const double *tk, const double *tv, const double *o, const double *to,
                          const double *dO, const double *dTO, const double *lse, const double *mu,
                          double *dq, double *dk, double *dv, double *dtq, double *dtk, double *dtv,
                          int64_t BH, int64_t Lq, int64_t Lk, int64_t D, double scale) {
    int64_t Lr = ((Lq + 127) / 128) * 128;
    double *zero = (double *)calloc((size_t)D, sizeof(double));
    if (!zero) return -1;
    memset(dq, 0, sizeof(double) * (size_t)(BH * Lq * D));
    memset(dtq, 0, sizeof(double) * (size_t)(BH * Lq * D));
    memset(dk, 0, sizeof(double) * (size_t)(BH * Lk * D));
    memset(dtk, 0, sizeof(double) * (size_t)(BH * Lk * D));
    memset(dv, 0, sizeof(double) * (size_t)(BH * Lk * D));
    memset(dtv, 0, sizeof(double) * (size_t)(BH * Lk * D));
    for (int64_t g = 0; g < BH; ++g) {
        for (int64_t i = 0; i < Lq; ++i) {
            int64_t r = (g * Lq + i) * D;
            const double *qi = q + r, *tqi = tq + r, *oi = o + r, *toi = to + r;
            const double *gi = dTO ? dTO + r : zero;
            const double *doi = dO ? dO + r : zero;
            double sum_4 = dot(gi, oi, (int)D), sum_7 = dot(gi, toi, (int)D);
            double delta = dot(doi, oi, (int)D);
            double lsei = lse[g * Lr + i], mui = mu[g * Lr + i];
            for (int64_t j = 0; j < Lk; ++j) {
                int64_t c = (g * Lk + j) * D;
                double p = exp(scale * dot(qi, k + c, (int)D) - lsei);
                double n = scale * (dot(tqi, k + c, (int)D) + dot(qi, tk + c, (int)D)) - mui;
                double w = dot(gi, v + c, (int)D);
                double x = dot(gi, tv + c, (int)D);
                double y = dot(doi, v + c, (int)D);
                double dts = p * (w - sum_4);
                double ds = dts * n + p * (x + y - sum_7 - delta);
                double pd = p * n;
                for (int64_t d = 0; d < D; ++d) {
                    dtq[r + d] += scale * dts * k[c + d];
                    dq[r + d] += scale * (ds * k[c + d] + dts * tk[c + d]);
                    dtk[c + d] += scale * dts * qi[d];
                    dk[c + d] += scale * (ds * qi[d] + dts * tqi[d]);
                    dtv[c + d] += p * gi[d];
                    dv[c + d] += pd * gi[d] + p * doi[d];
                }
            }
        }
    }
    free(zero);
    return 0;
}
