/*
 * Plain-C fp64 restatement of sliding-window 2-simplicial attention, forward and
 * backward.  TEST INFRASTRUCTURE ONLY: it is linked by nothing in the product and
 * may be called only from tests/, the smoke check and the CPU-baseline leg of the
 * benchmark.
 *
 * It is written as explicit loops over (i, j, k), independent of the tensor
 * library used by oracle/reference_attend.py, so that the two pin each other.
 *
 * Reference algorithm followed (paths relative to the reference checkout):
 *   logits, scale once       simplicial_attention/simplicial_attention.py:102-109
 *   windows 0<=i-j<w1, 0<=i-k<w2
 *                            simplicial_attention/triton_two_simplicial_attention.py:191-193
 *   joint softmax over (j,k) simplicial_attention/simplicial_attention.py:119-123
 *   value contraction        simplicial_attention/simplicial_attention.py:125
 *   M = m + log(l)           triton_two_simplicial_attention.py:225-228
 *   delta = rowsum(o*do)     triton_two_simplicial_attention.py:282
 *   dp, ds                   triton_two_simplicial_attention.py:481-482, 686-687
 *   dv1, dk1                 triton_two_simplicial_attention.py:478-479, 487-489
 *   dv2, dk2, dq             triton_two_simplicial_attention.py:680-683, 695, 697-699, 709
 *
 * Layout: every tensor is contiguous (b, n, h, d) in double precision; lse and
 * delta are (b, h, n).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX(b, i, h) ((((size_t)(b) * n + (size_t)(i)) * nh + (size_t)(h)) * d)

static double trilinear(const double *x, const double *y, const double *z, int d) {
    double s = 0.0;
    for (int c = 0; c < d; ++c) s += x[c] * y[c] * z[c];
    return s;
}

/* forward: out (b,n,h,d), lse (b,h,n) */
int sa2_oracle_fwd(const double *q, const double *k1, const double *k2,
                   const double *v1, const double *v2, double *out, double *lse,
                   int nb, int n, int nh, int d, int w1, int w2, double scale) {
    for (int b = 0; b < nb; ++b)
        for (int h = 0; h < nh; ++h)
            for (int i = 0; i < n; ++i) {
                const double *qi = q + IDX(b, i, h);
                int jlo = i - w1 + 1 < 0 ? 0 : i - w1 + 1;
                int klo = i - w2 + 1 < 0 ? 0 : i - w2 + 1;
                double m = -INFINITY;
                for (int j = jlo; j <= i; ++j)
                    for (int k = klo; k <= i; ++k) {
                        double s = scale * trilinear(qi, k1 + IDX(b, j, h), k2 + IDX(b, k, h), d);
                        if (s > m) m = s;
                    }
                double l = 0.0;
                double *o = out + IDX(b, i, h);
                memset(o, 0, sizeof(double) * (size_t)d);
                for (int j = jlo; j <= i; ++j)
                    for (int k = klo; k <= i; ++k) {
                        double s = scale * trilinear(qi, k1 + IDX(b, j, h), k2 + IDX(b, k, h), d);
                        double p = exp(s - m);
                        l += p;
                        const double *a = v1 + IDX(b, j, h), *c2 = v2 + IDX(b, k, h);
                        for (int c = 0; c < d; ++c) o[c] += p * a[c] * c2[c];
                    }
                for (int c = 0; c < d; ++c) o[c] /= l;
                lse[((size_t)b * nh + h) * n + i] = m + log(l);
            }
    return 0;
}

/* backward: needs out and lse from the forward; all gradients are overwritten */
int sa2_oracle_bwd(const double *q, const double *k1, const double *k2,
                   const double *v1, const double *v2, const double *out,
                   const double *dout, const double *lse,
                   double *dq, double *dk1, double *dk2, double *dv1, double *dv2,
                   int nb, int n, int nh, int d, int w1, int w2, double scale) {
    size_t total = (size_t)nb * n * nh * d;
    memset(dq, 0, total * sizeof(double));
    memset(dk1, 0, total * sizeof(double));
    memset(dk2, 0, total * sizeof(double));
    memset(dv1, 0, total * sizeof(double));
    memset(dv2, 0, total * sizeof(double));
    for (int b = 0; b < nb; ++b)
        for (int h = 0; h < nh; ++h)
            for (int i = 0; i < n; ++i) {
                size_t xi = IDX(b, i, h);
                double delta = 0.0;
                for (int c = 0; c < d; ++c) delta += out[xi + c] * dout[xi + c];
                double L = lse[((size_t)b * nh + h) * n + i];
                int jlo = i - w1 + 1 < 0 ? 0 : i - w1 + 1;
                int klo = i - w2 + 1 < 0 ? 0 : i - w2 + 1;
                for (int j = jlo; j <= i; ++j)
                    for (int k = klo; k <= i; ++k) {
                        size_t xj = IDX(b, j, h), xk = IDX(b, k, h);
                        double s = scale * trilinear(q + xi, k1 + xj, k2 + xk, d);
                        double p = exp(s - L);
                        double dp = trilinear(dout + xi, v1 + xj, v2 + xk, d);
                        double ds = p * (dp - delta);
                        for (int c = 0; c < d; ++c) {
                            dv1[xj + c] += p * dout[xi + c] * v2[xk + c];
                            dv2[xk + c] += p * dout[xi + c] * v1[xj + c];
                            dk1[xj + c] += scale * ds * q[xi + c] * k2[xk + c];
                            dk2[xk + c] += scale * ds * q[xi + c] * k1[xj + c];
                            dq[xi + c] += scale * ds * k1[xj + c] * k2[xk + c];
                        }
                    }
            }
    return 0;
}
