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

/* ---- gradients ---------------------------------------------------------------------------------------------
 * Bi-WKV backward, the contract of bi_wkv_backward (classification/mmcls_custom/models/backbones/cuda_new/
 * bi_wkv.cpp:35-47, launcher bi_wkv_kernel.cu:401-443): gk, gv (B,T,C); gw, gu (C,) summed over batch and tokens.
 * Evaluated by brute force from the definition, O(T^2) per sequence, not by a recurrence: output t is a softmax
 * over i of the logits  l_ti = k_i - w (|t-i| - 1)  (i != t),  l_tt = u + k_t,  weighted mean of v.  With
 * p_ti = softmax_i(l_ti) and y_t = sum_i p_ti v_i:
 *   gv_i = sum_t gy_t p_ti                      gk_i = sum_t gy_t p_ti (v_i - y_t)
 *   gu   = sum_t gy_t p_tt (v_t - y_t)          gw   = - sum_t sum_{i != t} (|t-i| - 1) gy_t p_ti (v_i - y_t)
 * (d l_ti / d k_i = 1, d l_tt / d u = 1, d l_ti / d w = -(|t-i| - 1)). */
int oracle_biwkv_bwd(const float *w, const float *u, const float *k, const float *v, const float *gy,
                     double *gw, double *gu, double *gk, double *gv, int B, int T, int C)
{
    if (B <= 0 || T <= 0 || C <= 0) return 1;
    int rc = 0;
    for (int c = 0; c < C; ++c) { gw[c] = 0; gu[c] = 0; }
#pragma omp parallel
    {
        double *buf = (double *)malloc(sizeof(double) * 5 * (size_t)T);
        if (!buf) {
#pragma omp atomic write
            rc = 2;
        } else {
            double *kk = buf, *vv = buf + T, *p = buf + 2 * (size_t)T, *gki = buf + 3 * (size_t)T, *gvi = buf + 4 * (size_t)T;
            /* one channel per iteration so that the per-channel sums need no atomics */
#pragma omp for schedule(dynamic, 1)
            for (int c = 0; c < C; ++c) {
                const double wc = w[c], uc = u[c];
                double sw = 0, su = 0;
                for (int b = 0; b < B; ++b) {
                    const size_t off = (size_t)b * T * C + c;
                    for (int t = 0; t < T; ++t) {
                        kk[t] = k[off + (size_t)t * C]; vv[t] = v[off + (size_t)t * C];
                        gki[t] = 0; gvi[t] = 0;
                    }
                    for (int t = 0; t < T; ++t) {
                        double m = uc + kk[t];
                        for (int i = 0; i < T; ++i) {
                            const int dist = (i > t ? i - t : t - i) - 1;
                            p[i] = (i == t) ? uc + kk[t] : kk[i] - wc * (double)dist;
                            if (p[i] > m) m = p[i];
                        }
                        double den = 0, num = 0;
                        for (int i = 0; i < T; ++i) { p[i] = exp(p[i] - m); den += p[i]; num += p[i] * vv[i]; }
                        const double y = num / den;
                        const double g = (double)gy[off + (size_t)t * C] / den;
                        for (int i = 0; i < T; ++i) {
                            const double pg = p[i] * g, dv = vv[i] - y;
                            gvi[i] += pg;
                            gki[i] += pg * dv;
                            if (i == t) su += pg * dv;
                            else sw -= (double)((i > t ? i - t : t - i) - 1) * pg * dv;
                        }
                    }
                    for (int t = 0; t < T; ++t) { gk[off + (size_t)t * C] = gki[t]; gv[off + (size_t)t * C] = gvi[t]; }
                }
                gw[c] = sw; gu[c] = su;
            }
            free(buf);
        }
    }
    return rc;
}

/* wkv6 backward, the contract of backward(B,T,C,H,r,k,v,w,u,gy,gr,gk,gv,gw,gu) (classification/mmcls_custom/models/
 * backbones/cuda_v6/wkv6_op.cpp:10-12, kernels wkv6_cuda.cu:99-346) with gu already summed over the batch
 * (vrwkv6.py:69) and gw taken with respect to the raw decay logit (d = exp(-exp(w_raw))).
 * Each of the two passes (ascending with the bonus u, descending without) is the causal recurrence in its own token
 * order n:   y_n = r_n (diag(u) k_n v_n^T + S_n),   S_{n+1} = diag(d_n) S_n + k_n v_n^T,  S_0 = 0.
 * Its adjoint state  G_n = sum_{m>n} (prod_{n<l<m} d_l) r_m gy_m^T  obeys  G_n = r_{n+1} gy_{n+1}^T + diag(d_{n+1}) G_{n+1}:
 *   gr_n[j] = sum_i gy_n[i] (u_j k_n[j] v_n[i] + S_n[j][i])
 *   gk_n[j] = sum_i v_n[i]  (u_j r_n[j] gy_n[i] + G_n[j][i])
 *   gv_n[i] = sum_j k_n[j]  (u_j r_n[j] gy_n[i] + G_n[j][i])
 *   gd_n[j] = sum_i S_n[j][i] G_n[j][i]          (S_{n+1} depends on d_n through d_n S_n; its gradient is G_n)
 *   gw_n[j] = gd_n[j] d_n[j] (-exp(w_raw_n[j]))
 *   gu[j]   = sum_n r_n[j] k_n[j] (v_n . gy_n)   (ascending pass only)
 * The states S_n of a pass are kept for all n (T N^2 doubles per thread). */
int oracle_wkv6_bwd(const float *r, const float *k, const float *v, const float *w_raw, const float *u,
                    const float *gy, double *gr, double *gk, double *gv, double *gw, double *gu,
                    int B, int T, int C, int H)
{
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0 || C % H) return 1;
    const int N = C / H;
    const size_t NN = (size_t)N * N;
    int rc = 0;
    for (int c = 0; c < C; ++c) gu[c] = 0;
#pragma omp parallel
    {
        double *S = (double *)malloc(sizeof(double) * ((size_t)T + 1) * NN);
        double *G = (double *)malloc(sizeof(double) * NN);
        double *gul = (double *)calloc((size_t)C, sizeof(double));
        if (!S || !G || !gul) {
#pragma omp atomic write
            rc = 2;
        } else {
#pragma omp for collapse(2) schedule(dynamic, 1)
            for (int b = 0; b < B; ++b)
                for (int h = 0; h < H; ++h) {
                    const size_t base = (size_t)b * T * C + (size_t)h * N;
                    const float *uh = u + (size_t)h * N;
                    for (int pass = 0; pass < 2; ++pass) {               /* 0: descending (writes), 1: ascending (adds) */
                        const int asc = pass;
                        /* states S_n before token n of the pass, n = 0..T-1 */
                        memset(S, 0, sizeof(double) * NN);
                        for (int n = 0; n < T; ++n) {
                            const size_t o = base + (size_t)(asc ? n : T - 1 - n) * C;
                            double *Sn = S + (size_t)n * NN, *Sx = Sn + NN;
                            for (int j = 0; j < N; ++j) {
                                const double d = exp(-exp((double)w_raw[o + j])), kj = k[o + j];
                                for (int i = 0; i < N; ++i) Sx[(size_t)j * N + i] = d * Sn[(size_t)j * N + i] + kj * (double)v[o + i];
                            }
                        }
                        memset(G, 0, sizeof(double) * NN);
                        for (int n = T - 1; n >= 0; --n) {
                            const size_t o = base + (size_t)(asc ? n : T - 1 - n) * C;
                            const double *Sn = S + (size_t)n * NN;
                            double vg = 0;
                            for (int i = 0; i < N; ++i) vg += (double)v[o + i] * (double)gy[o + i];
                            for (int j = 0; j < N; ++j) {
                                const double uj = asc ? (double)uh[j] : 0.0;
                                double sgr = 0, sgk = 0, sgd = 0;
                                for (int i = 0; i < N; ++i) {
                                    sgr += (double)gy[o + i] * Sn[(size_t)j * N + i];
                                    sgk += (double)v[o + i] * G[(size_t)j * N + i];
                                    sgd += Sn[(size_t)j * N + i] * G[(size_t)j * N + i];
                                }
                                const double ew = exp((double)w_raw[o + j]);
                                const double vgr = sgr + uj * (double)k[o + j] * vg;
                                const double vgk = sgk + uj * (double)r[o + j] * vg;
                                const double vgw = sgd * exp(-ew) * (-ew);
                                if (asc) { gr[o + j] += vgr; gk[o + j] += vgk; gw[o + j] += vgw; }
                                else     { gr[o + j] = vgr;  gk[o + j] = vgk;  gw[o + j] = vgw; }
                                if (asc) gul[(size_t)h * N + j] += (double)r[o + j] * (double)k[o + j] * vg;
                            }
                            for (int i = 0; i < N; ++i) {
                                double s = 0;
                                for (int j = 0; j < N; ++j)
                                    s += (double)k[o + j] * ((asc ? (double)uh[j] : 0.0) * (double)r[o + j] * (double)gy[o + i] + G[(size_t)j * N + i]);
                                if (asc) gv[o + i] += s; else gv[o + i] = s;
                            }
                            /* G_{n-1} = r_n gy_n^T + diag(d_n) G_n */
                            for (int j = 0; j < N; ++j) {
                                const double d = exp(-exp((double)w_raw[o + j])), rj = r[o + j];
                                for (int i = 0; i < N; ++i) G[(size_t)j * N + i] = rj * (double)gy[o + i] + d * G[(size_t)j * N + i];
                            }
                        }
                    }
                }
#pragma omp critical
            for (int c = 0; c < C; ++c) gu[c] += gul[c];
        }
        free(S); free(G); free(gul);
    }
    return rc;
}
