/* Closed-form Gaussian kernel products in plain C -- test infrastructure only.
 *
 * K_ij = exp(-1/2 * sum_k ((x_ik - c_jk) / sigma_k)^2), the definition the
 * reference documents (falkon/kernels/distance_kernel.py:366-370) and that its
 * tests use as the naive oracle (falkon/tests/naive_kernels.py:23-25), evaluated
 * in difference form with long-double accumulation.  Nothing here follows the
 * expanded-norm route of the shipped kernels, so it is an independent witness.
 *
 *   out[i,t] = sum_j K_ij v[j,t]                      (brute_mmv)
 *   out[j,t] = sum_i K_ij (sum_j' K_ij' v[j',t] + w[i,t])   (brute_dmmv)
 *
 * All matrices are dense row-major doubles; sigma has ns = 1 or d entries.
 */
#include <math.h>
#include <stdlib.h>

static long double kij(const double *x, const double *c, const double *sigma, long ns, long d) {
    long double s = 0.0L;
    for (long k = 0; k < d; k++) {
        long double z = ((long double)x[k] - (long double)c[k]) / (long double)sigma[ns == 1 ? 0 : k];
        s += z * z;
    }
    return expl(-0.5L * s);
}

int brute_mmv(const double *X, long n, const double *C, long m, long d, const double *sigma, long ns,
              const double *v, long t, double *out) {
    if (ns != 1 && ns != d) return -1;
    #pragma omp parallel for schedule(static)
    for (long i = 0; i < n; i++) {
        long double acc[64];
        for (long q = 0; q < t; q++) acc[q] = 0.0L;
        for (long j = 0; j < m; j++) {
            long double k = kij(X + i * d, C + j * d, sigma, ns, d);
            for (long q = 0; q < t; q++) acc[q] += k * (long double)v[j * t + q];
        }
        for (long q = 0; q < t; q++) out[i * t + q] = (double)acc[q];
    }
    return 0;
}

/* v may be NULL (treated as zero) and w may be NULL (treated as zero). */
int brute_dmmv(const double *X, long n, const double *C, long m, long d, const double *sigma, long ns,
               const double *v, const double *w, long t, double *out) {
    if (ns != 1 && ns != d) return -1;
    if (t > 64) return -2;
    long double *u = (long double *)malloc(sizeof(long double) * (size_t)n * (size_t)t);
    if (!u) return -3;
    #pragma omp parallel for schedule(static)
    for (long i = 0; i < n; i++) {
        for (long q = 0; q < t; q++) u[i * t + q] = w ? (long double)w[i * t + q] : 0.0L;
        if (v) for (long j = 0; j < m; j++) {
            long double k = kij(X + i * d, C + j * d, sigma, ns, d);
            for (long q = 0; q < t; q++) u[i * t + q] += k * (long double)v[j * t + q];
        }
    }
    #pragma omp parallel for schedule(static)
    for (long j = 0; j < m; j++) {
        long double acc[64];
        for (long q = 0; q < t; q++) acc[q] = 0.0L;
        for (long i = 0; i < n; i++) {
            long double k = kij(X + i * d, C + j * d, sigma, ns, d);
            for (long q = 0; q < t; q++) acc[q] += k * u[i * t + q];
        }
        for (long q = 0; q < t; q++) out[j * t + q] = (double)acc[q];
    }
    free(u);
    return 0;
}
