/* CPU oracle, float64 arithmetic, for the fused selective scan.  TEST INFRASTRUCTURE ONLY:
 * loaded by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the
 * shipped package.
 *
 * Restates the sequential form of the reference's selective scan
 * (mambapy/mamba.py:297-327):
 *     a[t,d,n] = exp(delta[t,d] * A[d,n])                 (mamba.py:309)
 *     h[t,d,n] = a[t,d,n] * h[t-1,d,n] + delta[t,d] * B[t,n] * x[t,d]   (:310-318)
 *     y[t,d]   = sum_n C[t,n] * h[t,d,n] + D[d] * x[t,d]  (:323-325)
 * and the gradients that autograd derives from it; the reverse recurrence is the one the
 * reference writes by hand in mambapy/pscan.py:216-222:
 *     g[t] = dy[t] * C[t] + a[t+1] * g[t+1]          (gradient w.r.t. the scan input BX)
 *     da[t] = g[t] * h[t-1]                            (gradient w.r.t. deltaA, 0 at t = 0)
 * chained through exp and the products of mamba.py:284-287.
 *
 * The analytic gradients here are pinned in tests/test_oracle.py against plain fp64
 * autograd through the Python sequential oracle, which derives them independently.
 *
 * Inputs are float32 arrays (values already rounded to the I/O precision under test),
 * contiguous: x, delta, dy (B,L,ED); A (ED,N); Bm, C (B,L,N); D (ED).  Outputs float64.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* y (B,L,ED) float64; h_last (B,ED,N) float64 or NULL; h0 (B,ED,N) float64 or NULL (= 0) */
int oracle_sscan_fwd(const float* x, const float* delta, const float* A, const float* Bm,
                     const float* C, const float* D, const double* h0, double* y,
                     double* h_last, long Bs, long L, long ED, long N) {
    if (N > 1024) return 1;
#pragma omp parallel for collapse(2) schedule(static)
    for (long b = 0; b < Bs; ++b) {
        for (long d = 0; d < ED; ++d) {
            double h[1024];
            for (long n = 0; n < N; ++n) h[n] = h0 ? h0[(b * ED + d) * N + n] : 0.0;
            for (long t = 0; t < L; ++t) {
                const long i = (b * L + t) * ED + d;
                const double dl = delta[i], xv = x[i];
                const float* Bt = Bm + (b * L + t) * N;
                const float* Ct = C + (b * L + t) * N;
                double acc = 0.0;
                for (long n = 0; n < N; ++n) {
                    const double a = exp(dl * (double)A[d * N + n]);
                    h[n] = a * h[n] + dl * (double)Bt[n] * xv;
                    acc += (double)Ct[n] * h[n];
                }
                y[i] = acc + (double)D[d] * xv;
            }
            if (h_last)
                for (long n = 0; n < N; ++n) h_last[(b * ED + d) * N + n] = h[n];
        }
    }
    return 0;
}

/* Gradients of sum(y * dy).  dx, ddelta (B,L,ED); dA (ED,N); dB, dC (B,L,N); dD (ED). */
int oracle_sscan_bwd(const float* x, const float* delta, const float* A, const float* Bm,
                     const float* C, const float* D, const float* dy, double* dx,
                     double* ddelta, double* dA, double* dB, double* dC, double* dD,
                     long Bs, long L, long ED, long N) {
    int nthreads = oracle_num_threads();
    const long bln = Bs * L * N;
    double* partB = (double*)calloc((size_t)nthreads * bln, sizeof(double));
    double* partC = (double*)calloc((size_t)nthreads * bln, sizeof(double));
    if (!partB || !partC) { free(partB); free(partC); return 2; }
    int fail = 0;
#pragma omp parallel
    {
#ifdef _OPENMP
        const int tid = omp_get_thread_num();
#else
        const int tid = 0;
#endif
        double* hs = (double*)malloc((size_t)(L + 1) * N * sizeof(double)); /* hs[t+1] = h[t] */
        double* as = (double*)malloc((size_t)L * N * sizeof(double));
        double* g = (double*)malloc((size_t)N * sizeof(double));
        double* pB = partB + (size_t)tid * bln;
        double* pC = partC + (size_t)tid * bln;
        if (!hs || !as || !g) {
#pragma omp atomic write
            fail = 1;
        } else {
#pragma omp for schedule(static)
            for (long d = 0; d < ED; ++d) {
                double dDacc = 0.0;
                for (long n = 0; n < N; ++n) dA[d * N + n] = 0.0;
                for (long b = 0; b < Bs; ++b) {
                    for (long n = 0; n < N; ++n) hs[n] = 0.0;
                    for (long t = 0; t < L; ++t) {
                        const long i = (b * L + t) * ED + d;
                        const double dl = delta[i], xv = x[i];
                        const float* Bt = Bm + (b * L + t) * N;
                        for (long n = 0; n < N; ++n) {
                            const double a = exp(dl * (double)A[d * N + n]);
                            as[t * N + n] = a;
                            hs[(t + 1) * N + n] = a * hs[t * N + n] + dl * (double)Bt[n] * xv;
                        }
                    }
                    for (long n = 0; n < N; ++n) g[n] = 0.0;
                    for (long t = L - 1; t >= 0; --t) {
                        const long i = (b * L + t) * ED + d;
                        const double dl = delta[i], xv = x[i], dyv = dy[i];
                        const float* Bt = Bm + (b * L + t) * N;
                        const float* Ct = C + (b * L + t) * N;
                        double gB = 0.0, dd = 0.0;
                        for (long n = 0; n < N; ++n) {
                            const double anext = (t + 1 < L) ? as[(t + 1) * N + n] : 0.0;
                            const double gn = dyv * (double)Ct[n] + anext * g[n];
                            g[n] = gn;
                            const double da = gn * hs[t * N + n];          /* h[t-1] */
                            const double dexp = da * as[t * N + n];        /* d/d(delta*A) */
                            dd += dexp * (double)A[d * N + n];
                            dA[d * N + n] += dexp * dl;
                            gB += gn * (double)Bt[n];
                            pB[(b * L + t) * N + n] += gn * dl * xv;
                            pC[(b * L + t) * N + n] += dyv * hs[(t + 1) * N + n];
                        }
                        dx[i] = dl * gB + (double)D[d] * dyv;
                        ddelta[i] = dd + xv * gB;
                        dDacc += dyv * xv;
                    }
                }
                dD[d] = dDacc;
            }
        }
        free(hs); free(as); free(g);
    }
    if (!fail) {
#pragma omp parallel for schedule(static)
        for (long i = 0; i < bln; ++i) {
            double sb = 0.0, sc = 0.0;
            for (int t = 0; t < nthreads; ++t) {
                sb += partB[(size_t)t * bln + i];
                sc += partC[(size_t)t * bln + i];
            }
            dB[i] = sb;
            dC[i] = sc;
        }
    }
    free(partB); free(partC);
    return fail ? 2 : 0;
}
