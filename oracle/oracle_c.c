/* TEST INFRASTRUCTURE ONLY: plain C restatement of the path, double precision, scalar loops.
 *
 *   lm2exp_c   baselines/lm2exp.py:11-14   m = clamp(max_j b, +-1e38); c = m + log(sum_j a exp(b - m))
 *   lt2exp_c   baselines/lt2exp.py:15-25   two shifts; c = ma + mb + log(sum_ij w exp(a - ma) exp(b - mb))
 *   vmax_c     triturus/max.py:62-122      max and first-occurrence argmax; a NaN wins (torch.max)
 *   matmax_c   triturus/max.py:125-226     max along axis 0 or 1 of a row-major matrix (torch.amax)
 *
 * Inputs are the fp32 arrays the kernels receive (contiguous, row-major); all arithmetic is
 * double.  No library but libm; nothing here is shared with the torch / NumPy oracle, which the
 * tests compare it with.  Built by oracle/build_c.py (gcc); never linked into the product.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

static double clamp38(double m) {
    if (m < -1e38) return -1e38;
    if (m > 1e38) return 1e38;
    return m; /* NaN passes through, as torch.clamp does */
}

/* max that lets a NaN through from either side (torch.amax) */
static double max_nan(double x, double y) { return (x > y || x != x) ? x : y; }

void lm2exp_c(const float *a, const float *b, double *c, int64_t R, int64_t I, int64_t J, int64_t K) {
    for (int64_t r = 0; r < R; ++r)
        for (int64_t k = 0; k < K; ++k) {
            double m = -INFINITY;
            for (int64_t j = 0; j < J; ++j) m = max_nan(m, (double)b[(r * J + j) * K + k]);
            m = clamp38(m);
            for (int64_t i = 0; i < I; ++i) {
                double s = 0.0;
                for (int64_t j = 0; j < J; ++j)
                    s += (double)a[(r * I + i) * J + j] * exp((double)b[(r * J + j) * K + k] - m);
                c[(r * I + i) * K + k] = m + log(s);
            }
        }
}

void lt2exp_c(const float *w, const float *a, const float *b, double *c, int64_t R, int64_t S, int64_t I,
              int64_t J, int64_t K) {
    for (int64_t r = 0; r < R; ++r)
        for (int64_t k = 0; k < K; ++k) {
            double ma = -INFINITY, mb = -INFINITY;
            for (int64_t i = 0; i < I; ++i) ma = max_nan(ma, (double)a[(r * I + i) * K + k]);
            for (int64_t j = 0; j < J; ++j) mb = max_nan(mb, (double)b[(r * J + j) * K + k]);
            ma = clamp38(ma);
            mb = clamp38(mb);
            for (int64_t s = 0; s < S; ++s) {
                double t = 0.0;
                for (int64_t i = 0; i < I; ++i) {
                    const double ea = exp((double)a[(r * I + i) * K + k] - ma);
                    for (int64_t j = 0; j < J; ++j)
                        t += (double)w[((r * S + s) * I + i) * J + j] * (ea * exp((double)b[(r * J + j) * K + k] - mb));
                }
                c[(r * S + s) * K + k] = ma + mb + log(t);
            }
        }
}

void vmax_c(const float *x, int64_t n, float *val, int64_t *idx) {
    float best = x[0];
    int64_t at = 0;
    for (int64_t i = 1; i < n; ++i) {
        if (best != best) break; /* the first NaN wins */
        if (x[i] > best || x[i] != x[i]) {
            best = x[i];
            at = i;
        }
    }
    *val = best;
    *idx = at;
}

void matmax_c(const float *x, float *y, int64_t m, int64_t n, int axis) {
    if (axis == 0) {
        for (int64_t j = 0; j < n; ++j) {
            double v = -INFINITY;
            for (int64_t i = 0; i < m; ++i) v = max_nan(v, (double)x[i * n + j]);
            y[j] = (float)v;
        }
    } else {
        for (int64_t i = 0; i < m; ++i) {
            double v = -INFINITY;
            for (int64_t j = 0; j < n; ++j) v = max_nan(v, (double)x[i * n + j]);
            y[i] = (float)v;
        }
    }
}
