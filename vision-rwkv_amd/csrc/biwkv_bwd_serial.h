// Bi-WKV backward, sequential form: one lane owns one (batch, channel) sequence and walks it three
// times, lanes of a wave being 64 adjacent channels (every access is a contiguous 64-channel row segment):
//   pass A (ascending)   past state (a, b, p) before each token            -> workspace
//   pass B (descending)  future state, y_t, z_t; future scans; partial gk, gv; gu, gw partials
//   pass C (ascending)   past scans; final gk, gv; gw partial
// Every running sum is a (mantissa, exponent) pair renormalised at each token, i.e. the reference's own
// stabilised recurrence (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:103-108),
// so any w, u, k and any T is handled.  Workspace: 5 floats per element.
#pragma once
#include "vrwkv_common.h"

namespace vrwkv {
namespace biwkv_bwd_detail {

// (mantissas..., exponent) <- decay by one token, then add a term with exponent e
struct Scan {
    float s0 = 0.f, s1 = 0.f, l0 = 0.f, l1 = 0.f, p = NEG_BIG;   // sums of z, z*y; distance-weighted sums
    __device__ __forceinline__ void push(float om, float z, float zy, float e) {
        const float pw = fmaxf(p - om, NEG_BIG);
        const float q = fmaxf(pw, e);
        const float c1 = fast_exp2(pw - q), c2 = fast_exp2(e - q);
        l0 = c1 * (l0 + s0);                 // distances grow by one; the new term enters at distance 0
        l1 = c1 * (l1 + s1);
        s0 = c1 * s0 + c2 * z;
        s1 = c1 * s1 + c2 * zy;
        p = q;
    }
};

// One lane: the whole sequence of batch element b, channel c (c < C).
template <typename IO>
__device__ __forceinline__
void biwkv_bwd_serial_seq(const float* __restrict__ w_, const float* __restrict__ u_,
                          const IO* __restrict__ k_, const IO* __restrict__ v_, const IO* __restrict__ gy_,
                          IO* __restrict__ gk_, IO* __restrict__ gv_, float* __restrict__ ws,
                          float* __restrict__ gw_part, float* __restrict__ gu_part, int B, int T, int C, int b, int c,
                          int rows_per_batch = 1)
{
    const float om = w_[c] * LOG2E, mu = u_[c] * LOG2E;
    const size_t base = (size_t)b * T * C + c;
    const size_t plane = (size_t)B * T * C;
    float* W0 = ws;                 // a      -> later z mantissa
    float* W1 = ws + plane;         // b      -> later y
    float* W2 = ws + 2 * plane;     // p      -> later m (exponent of z)
    float* W3 = ws + 3 * plane;     // partial gv
    float* W4 = ws + 4 * plane;     // partial gk

    // ---- pass A: past state before each token ----
    {
        float a = 0.f, bb = 0.f, p = NEG_BIG;
        for (int t = 0; t < T; ++t) {
            const size_t o = base + (size_t)t * C;
            W0[o] = a; W1[o] = bb; W2[o] = p;
            const float kap = to_f32(k_[o]) * LOG2E, v = to_f32(v_[o]);
            const float pw = fmaxf(p - om, NEG_BIG), q = fmaxf(pw, kap);
            const float e1 = fast_exp2(pw - q), e2 = fast_exp2(kap - q);
            a = e1 * a + e2 * v; bb = e1 * bb + e2; p = q;
        }
    }
    float gu_acc = 0.f, gw_acc = 0.f;
    // ---- pass B: future state, y, z; future scans ----
    {
        float cc = 0.f, d = 0.f, o_ = NEG_BIG;
        Scan f;
        for (int t = T - 1; t >= 0; --t) {
            const size_t o = base + (size_t)t * C;
            const float kap = to_f32(k_[o]) * LOG2E, v = to_f32(v_[o]), gy = to_f32(gy_[o]);
            const float a = W0[o], bb = W1[o], p = W2[o];
            const float uk = mu + kap;
            const float m = fmaxf(fmaxf(p, o_), uk);
            const float ea = fast_exp2(p - m), ec = fast_exp2(o_ - m), eu = fast_exp2(uk - m);
            const float den = ea * bb + ec * d + eu;
            const float y = (ea * a + ec * cc + eu * v) / den;
            const float z = gy / den;                       // z_t = z * 2^-m in absolute scale
            const float zy = z * y;
            // contributions of later tokens (t' > t) and of the token itself
            const float sf = fast_exp2(kap + f.p);          // 2^(kappa_i + exponent of the scan)
            const float self = z * eu;
            const float gv = sf * f.s0 + self;
            const float gk = v * gv - (sf * f.s1 + self * y);
            gu_acc += self * (v - y);
            gw_acc -= sf * (v * f.l0 - f.l1);
            W3[o] = gv; W4[o] = gk;
            W0[o] = z; W1[o] = y; W2[o] = m;
            // this token joins the future of the earlier ones
            f.push(om, z, zy, -m);
            const float pw = fmaxf(o_ - om, NEG_BIG), q = fmaxf(pw, kap);
            const float e1 = fast_exp2(pw - q), e2 = fast_exp2(kap - q);
            cc = e1 * cc + e2 * v; d = e1 * d + e2; o_ = q;
        }
    }
    // ---- pass C: past scans, final gk, gv ----
    {
        Scan g;
        for (int t = 0; t < T; ++t) {
            const size_t o = base + (size_t)t * C;
            const float kap = to_f32(k_[o]) * LOG2E, v = to_f32(v_[o]);
            const float z = W0[o], y = W1[o], m = W2[o];
            const float sp = fast_exp2(kap + g.p);
            const float gvp = sp * g.s0;
            gv_[o] = from_f32<IO>(W3[o] + gvp);
            gk_[o] = from_f32<IO>(W4[o] + v * gvp - sp * g.s1);
            gw_acc -= sp * (v * g.l0 - g.l1);
            g.push(om, z, z * y, -m);
        }
    }
    // the partial-sum table has rows_per_batch rows per batch element (the tiled kernel writes one per
    // super-chunk); the whole-sequence sums go to the first, zeros to the others
    gw_part[(size_t)b * rows_per_batch * C + c] = gw_acc;
    gu_part[(size_t)b * rows_per_batch * C + c] = gu_acc;
    for (int r = 1; r < rows_per_batch; ++r) {
        gw_part[((size_t)b * rows_per_batch + r) * C + c] = 0.f;
        gu_part[((size_t)b * rows_per_batch + r) * C + c] = 0.f;
    }
}

}  // namespace biwkv_bwd_detail
}  // namespace vrwkv
