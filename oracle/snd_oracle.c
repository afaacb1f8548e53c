/* CPU restatement of the 2D-CrossScan selective scan in plain C (forward + hand adjoint).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py.  Nothing in the shipped package links or loads it.
 *
 * Follows the reference cell by cell (same citations as snd_oracle.py):
 *   forward  kernels/selective_nd_scan/include/cusoflex/selective_scan_fwd_kernel_oflex.cuh:189-346
 *   backward kernels/selective_nd_scan/include/cusoflex/selective_scan_bwd_kernel_oflex.cuh:207-214,
 *            383-612, 621-775, 785-819
 *   scan op  kernels/selective_nd_scan/include/selective_scan_common.h:100-107, constants :13-21
 * It is pinned by tests/test_oracle_c.py against snd_oracle.py (which carries the closed-form,
 * symmetry and autograd pins).  Arithmetic type is SND_REAL (float by default = the reference's
 * fp32 state; build with -DSND_REAL=double for a float64 checker).  Dense row-major fp32 I/O.
 * Parallel over (batch, group) pairs with OpenMP: each pair owns its dB/dC slice.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#ifndef SND_REAL
#define SND_REAL float
#endif
typedef SND_REAL real;

static real softplus20(real x) { return x <= (real)20 ? (real)log1p(exp((double)x)) : x; } /* fwd.cuh:223 */

/* a, bu, h, s of one (b, c, n) plane; dl = delta' (after bias/softplus) of the channel. */
static void plane_forward(int H, int W, real An, real adec, const real *dl, const float *u, const float *Bn,
                          real *a, real *bu, real *h, real *s) {
    for (int i = 0; i < H; ++i)
        for (int j = 0; j < W; ++j) {
            const int k = i * W + j;
            a[k] = (real)exp((double)(dl[k] * An)) * adec;                       /* fwd.cuh:194-195,245 */
            bu[k] = (real)Bn[k] * dl[k] * (real)u[k];                            /* fwd.cuh:225,265 */
            const real left = j > 0 ? h[k - 1] : 0, up = i > 0 ? h[k - W] : 0;
            real corr = 0;
            if (i > 0 && j > 0) corr = (real)0.5 * (a[k - W] + a[k - 1]) * h[k - W - 1]; /* fwd.cuh:265,270 */
            h[k] = a[k] * (left + up - corr) + bu[k];                            /* fwd.cuh:263-272,290 */
            s[k] = a[k] * (j > 0 ? s[k - 1] : 0) + bu[k];                        /* fwd.cuh:309-327 */
        }
}

static void channel_delta(int HW, const float *delta, real bias, int softplus, real *raw, real *dl) {
    for (int k = 0; k < HW; ++k) {
        raw[k] = (real)delta[k] + bias;                                          /* fwd.cuh:221 */
        dl[k] = softplus ? softplus20(raw[k]) : raw[k];
    }
}

int snd_oracle_real_bytes(void) { return (int)sizeof(real); }

int snd_oracle_fwd(int Bt, int Dm, int H, int W, int N, int G, int Dd, const float *u, const float *delta,
                   const float *A, const float *B, const float *C, const float *D, const float *bias,
                   int softplus, const float *A_decay, float *out, int nthreads) {
    const int HW = H * W, rg = Dm / G, rd = Dm / Dd;
    const real adec = A_decay ? (real)A_decay[0] : (real)1;                      /* fwd.cuh:131-134 */
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel
    {
        real *buf = (real *)malloc(sizeof(real) * HW * 6);
        real *raw = buf, *dl = buf + HW, *a = buf + 2 * HW, *bu = buf + 3 * HW, *h = buf + 4 * HW, *s = buf + 5 * HW;
#pragma omp for schedule(dynamic, 1)
        for (int bc = 0; bc < Bt * Dm; ++bc) {
            const int b = bc / Dm, c = bc % Dm, g = c / rg, dg = c / rd;
            const float *uc = u + (size_t)bc * HW;
            channel_delta(HW, delta + ((size_t)b * Dd + dg) * HW, bias ? (real)bias[dg] : 0, softplus, raw, dl);
            float *oc = out + (size_t)bc * HW;
            const real Dv = D ? (real)D[c] : 0;                                  /* fwd.cuh:121-124 */
            for (int k = 0; k < HW; ++k) oc[k] = (float)(Dv * (real)uc[k]);      /* fwd.cuh:227 */
            for (int n = 0; n < N; ++n) {
                const float *Bn = B + (((size_t)b * G + g) * N + n) * HW, *Cn = C + (((size_t)b * G + g) * N + n) * HW;
                plane_forward(H, W, (real)A[c * N + n], adec, dl, uc, Bn, a, bu, h, s);
                for (int k = 0; k < HW; ++k)
                    oc[k] += (float)((real)Cn[k] * (h[k] - s[k] + (real)0.25 * bu[k])); /* fwd.cuh:301,334 */
            }
        }
        free(buf);
    }
    return 0;
}

/* du, ddelta [Bt,Dm,H,W]; dA [Dm,N]; dB, dC [Bt,G,N,H,W]; dD, dbias [Dm]; dA_decay [1].
 * Optional outputs may be NULL.  All outputs are overwritten. */
int snd_oracle_bwd(int Bt, int Dm, int H, int W, int N, int G, int Dd, const float *u, const float *delta,
                   const float *A, const float *B, const float *C, const float *D, const float *bias,
                   int softplus, const float *A_decay, const float *dout, float *du, float *ddelta, float *dA,
                   float *dB, float *dC, float *dD, float *dbias, float *dA_decay, int nthreads) {
    const int HW = H * W, rg = Dm / G, rd = Dm / Dd;
    const real adec = A_decay ? (real)A_decay[0] : (real)1;
    double *accA = (double *)calloc((size_t)Dm * N, sizeof(double));
    double *accD = (double *)calloc((size_t)Dm, sizeof(double));
    double *accB = (double *)calloc((size_t)Dm, sizeof(double));
    double accDec = 0;
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel
    {
        real *buf = (real *)malloc(sizeof(real) * HW * 10);
        real *raw = buf, *dl = buf + HW, *a = buf + 2 * HW, *bu = buf + 3 * HW, *h = buf + 4 * HW, *s = buf + 5 * HW;
        real *g_ = buf + 6 * HW, *gs = buf + 7 * HW, *q = buf + 8 * HW, *p = buf + 9 * HW;
#pragma omp for schedule(dynamic, 1)
        for (int bg = 0; bg < Bt * G; ++bg) {
            const int b = bg / G, g = bg % G;
            float *dBg = dB + (size_t)bg * N * HW, *dCg = dC + (size_t)bg * N * HW;
            memset(dBg, 0, sizeof(float) * (size_t)N * HW);
            memset(dCg, 0, sizeof(float) * (size_t)N * HW);
            for (int c = g * rg; c < (g + 1) * rg; ++c) {
                const int dg = c / rd;
                const size_t bc = (size_t)b * Dm + c;
                const float *uc = u + bc * HW, *doc = dout + bc * HW;
                channel_delta(HW, delta + ((size_t)b * Dd + dg) * HW, bias ? (real)bias[dg] : 0, softplus, raw, dl);
                for (int k = 0; k < HW; ++k) { q[k] = 0; p[k] = 0; }
                double sD = 0;
                for (int n = 0; n < N; ++n) {
                    const real An = (real)A[c * N + n];
                    const float *Bn = B + ((size_t)bg * N + n) * HW, *Cn = C + ((size_t)bg * N + n) * HW;
                    plane_forward(H, W, An, adec, dl, uc, Bn, a, bu, h, s);
                    double sA = 0, sDec = 0;
                    for (int i = H - 1; i >= 0; --i)
                        for (int j = W - 1; j >= 0; --j) {
                            const int k = i * W + j;
                            const real dyC = (real)doc[k] * (real)Cn[k];                      /* bwd.cuh:469 */
                            const real Gr = j + 1 < W ? a[k + 1] * g_[k + 1] : 0;
                            const real Gd = i + 1 < H ? a[k + W] * g_[k + W] : 0;
                            real acc = dyC + Gr + Gd;
                            if (i + 1 < H && j + 1 < W)                                        /* bwd.cuh:463-467 */
                                acc -= (real)0.5 * a[k + W + 1] * (a[k + 1] + a[k + W]) * g_[k + W + 1];
                            g_[k] = acc;                                                       /* bwd.cuh:486-488 */
                            gs[k] = -dyC + (j + 1 < W ? a[k + 1] * gs[k + 1] : 0);             /* bwd.cuh:710,722 */
                            const real hl = j > 0 ? h[k - 1] : 0, hu = i > 0 ? h[k - W] : 0;
                            const real hd = (i > 0 && j > 0) ? h[k - W - 1] : 0;
                            const real al = j > 0 ? a[k - 1] : 0, au = i > 0 ? a[k - W] : 0;
                            const real Y = hl + hu - (real)0.5 * (au + al) * hd;               /* (h-bu)/a, bwd.cuh:515 */
                            const real sl = j > 0 ? s[k - 1] : 0;
                            /* total derivative w.r.t. a[i,j]: own multiplier and the two neighbours it feeds */
                            const real da = g_[k] * Y + gs[k] * sl - (real)0.5 * (Gd * hl + Gr * hu); /* bwd.cuh:516-587,751-753 */
                            const real da_a = da * a[k];
                            const real dbu = g_[k] + gs[k] + (real)0.25 * dyC;                 /* bwd.cuh:750-754 */
                            p[k] += An * da_a;                                                 /* bwd.cuh:516 */
                            q[k] += dbu * (real)Bn[k];                                         /* bwd.cuh:513 */
                            sA += (double)(dl[k] * da_a);                                      /* bwd.cuh:518,753 */
                            sDec += (double)da_a;
                            dBg[(size_t)n * HW + k] += (float)(dbu * dl[k] * (real)uc[k]);     /* bwd.cuh:589,754 */
                            dCg[(size_t)n * HW + k] += (float)((real)doc[k] * (h[k] - s[k] + (real)0.25 * bu[k])); /* :590,755 */
                        }
#pragma omp atomic
                    accA[c * N + n] += sA;
#pragma omp atomic
                    accDec += sDec;
                }
                double sB = 0;
                const real Dv = D ? (real)D[c] : 0;
                for (int k = 0; k < HW; ++k) {
                    real ddl = p[k] + q[k] * (real)uc[k];                                      /* bwd.cuh:516,752 */
                    if (softplus && raw[k] <= (real)20) ddl = ddl / ((real)1 + (real)exp(-(double)raw[k])); /* :785-806 */
                    du[bc * HW + k] = (float)(Dv * (real)doc[k] + q[k] * dl[k]);               /* bwd.cuh:211,514 */
                    ddelta[bc * HW + k] = (float)ddl;
                    sB += (double)ddl;
                    sD += (double)doc[k] * (double)uc[k];                                      /* bwd.cuh:212 */
                }
#pragma omp atomic
                accD[c] += sD;
#pragma omp atomic
                accB[c] += sB;
            }
        }
        free(buf);
    }
    for (int k = 0; k < Dm * N; ++k) dA[k] = (float)accA[k];
    if (dD) for (int k = 0; k < Dm; ++k) dD[k] = (float)accD[k];
    if (dbias) for (int k = 0; k < Dm; ++k) dbias[k] = (float)accB[k];
    if (dA_decay) dA_decay[0] = (float)(accDec / (double)adec);
    free(accA); free(accD); free(accB);
    return 0;
}
