/* Plain-C restatement of the Vision-RWKV WKV recurrences (double accumulators).
 * TEST INFRASTRUCTURE ONLY: linked by the tests, the smoke check and the
 * benchmark's CPU-baseline leg, never by the shipped operators.
 *
 * Bi-WKV  : state update  classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:103-108
 *           output combine                                                     ...:95-100
 *           (the future state is built by a descending pass, not by the
 *           subtractive update at :109-113; EPS of :16 is left out)
 * wkv6    : classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:23-96, with
 *           d = exp(-exp(w_raw)) as in vrwkv6.py:48 + wkv6_cuda.cu:26.
 *
 * Inputs are fp32 arrays in the operator's (B,T,C) layout (C fastest); outputs
 * are double so that the checker itself adds no rounding.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define MIN_VALUE (-1e38)

/* returns 0 on success */
int oracle_biwkv_fwd(const float *w, const float *u, const float *k, const float *v,
                     double *y, int B, int T, int C)
{
    if (B <= 0 || T <= 0 || C <= 0) return 1;
    int rc = 0;
#pragma omp parallel
    {
        double *A = (double *)malloc(sizeof(double) * 3 * (size_t)T);
        if (!A) {
#pragma omp atomic write
            rc = 2;
        } else {
            double *Bd = A + T, *P = A + 2 * (size_t)T;
#pragma omp for collapse(2) schedule(static)
            for (int b = 0; b < B; ++b)
                for (int c = 0; c < C; ++c) {
                    const size_t off = (size_t)b * T * C + c;
                    const double wc = w[c], uc = u[c];
                    double a = 0, bb = 0, p = MIN_VALUE;
                    for (int t = 0; t < T; ++t) {
                        A[t] = a; Bd[t] = bb; P[t] = p;
                        const double kt = k[off + (size_t)t * C], vt = v[off + (size_t)t * C];
                        const double q = fmax(p - wc, kt);
                        const double e1 = exp(p - wc - q), e2 = exp(kt - q);
                        a = e1 * a + e2 * vt;
                        bb = e1 * bb + e2;
                        p = q;
                    }
                    double cc = 0, d = 0, o = MIN_VALUE;
                    for (int t = T - 1; t >= 0; --t) {
                        const double kt = k[off + (size_t)t * C], vt = v[off + (size_t)t * C];
                        const double m = fmax(fmax(P[t], o), uc + kt);
                        const double ea = exp(P[t] - m), ec = exp(o - m), eu = exp(uc + kt - m);
                        y[off + (size_t)t * C] = (ea * A[t] + ec * cc + eu * vt) / (ea * Bd[t] + ec * d + eu);
                        const double q = fmax(o - wc, kt);
                        const double e1 = exp(o - wc - q), e2 = exp(kt - q);
                        cc = e1 * cc + e2 * vt;
                        d = e1 * d + e2;
                        o = q;
                    }
                }
            free(A);
        }
    }
    return rc;
}

/* r,k,v,w_raw: (B,T,C) fp32; u: (H,N) fp32; y: (B,T,C) double.  N = C/H (any N). */
int oracle_wkv6_fwd(const float *r, const float *k, const float *v, const float *w_raw,
                    const float *u, double *y, int B, int T, int C, int H)
{
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0 || C % H) return 1;
    const int N = C / H;
    int rc = 0;
#pragma omp parallel
    {
        double *S = (double *)malloc(sizeof(double) * (size_t)N * N);
        if (!S) {
#pragma omp atomic write
            rc = 2;
        } else {
#pragma omp for collapse(2) schedule(static)
            for (int b = 0; b < B; ++b)
                for (int h = 0; h < H; ++h) {
                    const size_t base = (size_t)b * T * C + (size_t)h * N;
                    const float *uh = u + (size_t)h * N;
                    /* descending pass: y_t = r_t . S' ; S' = d_t S' + k_t v_t^T */
                    memset(S, 0, sizeof(double) * (size_t)N * N);
                    for (int t = T - 1; t >= 0; --t) {
                        const size_t o = base + (size_t)t * C;
                        for (int i = 0; i < N; ++i) {
                            double acc = 0;
                            for (int j = 0; j < N; ++j) acc += (double)r[o + j] * S[(size_t)j * N + i];
                            y[o + i] = acc;
                        }
                        for (int j = 0; j < N; ++j) {
                            const double d = exp(-exp((double)w_raw[o + j])), kj = k[o + j];
                            for (int i = 0; i < N; ++i)
                                S[(size_t)j * N + i] = d * S[(size_t)j * N + i] + kj * (double)v[o + i];
                        }
                    }
                    /* ascending pass with the bonus */
                    memset(S, 0, sizeof(double) * (size_t)N * N);
                    for (int t = 0; t < T; ++t) {
                        const size_t o = base + (size_t)t * C;
                        for (int i = 0; i < N; ++i) {
                            double acc = 0;
                            for (int j = 0; j < N; ++j)
                                acc += (double)r[o + j] *
                                       ((double)uh[j] * (double)k[o + j] * (double)v[o + i] + S[(size_t)j * N + i]);
                            y[o + i] += acc;
                        }
                        for (int j = 0; j < N; ++j) {
                            const double d = exp(-exp((double)w_raw[o + j])), kj = k[o + j];
                            for (int i = 0; i < N; ++i)
                                S[(size_t)j * N + i] = d * S[(size_t)j * N + i] + kj * (double)v[o + i];
                        }
                    }
                }
            free(S);
        }
    }
    return rc;
}
