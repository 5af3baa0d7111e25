// Bi-WKV backward for gfx950: gw, gu (C,), gk, gv (B,T,C) from gy.
// Replaces bi_wkv_backward (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:35-47,
// kernel .../cuda_new/bi_wkv_kernel.cu:119-367).
//
// With W[t,i] = e^{k_i - w(|t-i|-1)} (i != t), W[t,t] = e^{u+k_t}, y_t = N_t/D_t and z_t = gy_t/D_t:
//   gv_i = sum_t z_t W[t,i]                     gk_i = sum_t z_t W[t,i] (v_i - y_t)
//   gu   = sum_t z_t W[t,t] (v_t - y_t)         gw   = - sum_t sum_{i!=t} (|t-i|-1) z_t W[t,i] (v_i - y_t)
// so besides the forward states only decayed scans of z_t and z_t*y_t over past and future are
// needed (and, for gw, the same scans weighted by the distance: B' = g (B + A)).
//
// One lane owns one (batch, channel) sequence and walks it three times, lanes of a wave being 64
// adjacent channels (every access is a contiguous 64-channel row segment):
//   pass A (ascending)   past state (a, b, p) before each token            -> workspace
//   pass B (descending)  future state, y_t, z_t; future scans; partial gk, gv; gu, gw partials
//   pass C (ascending)   past scans; final gk, gv; gw partial
// Every running sum is a (mantissa, exponent) pair renormalised at each token, i.e. the
// reference's own stabilised recurrence (bi_wkv_kernel.cu:103-108), so any w, u, k is handled.
// gw and gu are reduced over the batch by a second small kernel (deterministic, no atomics).
// The reference needs 3 scratch tensors and atomicAdd (bi_wkv_kernel.cu:303-304, 415-417);
// here the workspace is 5 floats per element + 2*B*C.
#include "vrwkv_common.h"

namespace vrwkv {
namespace {

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

template <typename IO>
__global__ __launch_bounds__(64)
void biwkv_bwd_kernel(const float* __restrict__ w_, const float* __restrict__ u_,
                      const IO* __restrict__ k_, const IO* __restrict__ v_, const IO* __restrict__ gy_,
                      IO* __restrict__ gk_, IO* __restrict__ gv_, float* __restrict__ ws,
                      float* __restrict__ gw_part, float* __restrict__ gu_part, int B, int T, int C)
{
    const int c = blockIdx.x * 64 + threadIdx.x;
    const int b = blockIdx.y;
    if (c >= C) return;
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
    gw_part[(size_t)b * C + c] = gw_acc;
    gu_part[(size_t)b * C + c] = gu_acc;
}

__global__ void biwkv_bwd_reduce_kernel(const float* __restrict__ gw_part, const float* __restrict__ gu_part,
                                        float* __restrict__ gw, float* __restrict__ gu, int B, int C)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    float sw = 0.f, su = 0.f;
    for (int b = 0; b < B; ++b) { sw += gw_part[(size_t)b * C + c]; su += gu_part[(size_t)b * C + c]; }
    gw[c] = sw; gu[c] = su;
}

int validate(int B, int T, int C, int io_dtype) {
    if (B <= 0 || T <= 0 || C <= 0) {
        set_error("biwkv_bwd: B, T, C must be positive (got %d, %d, %d)", B, T, C);
        return VRWKV_INVALID_ARG;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("biwkv_bwd: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (B > 65535 || (long long)B * T * C >= (1LL << 40)) {
        set_error("biwkv_bwd: B must be <= 65535 and B*T*C < 2^40");
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    return VRWKV_OK;
}

template <typename IO>
int launch(const float* w, const float* u, const void* k, const void* v, const void* gy, float* gw, float* gu,
           void* gk, void* gv, float* ws, int B, int T, int C, hipStream_t st) {
    const size_t plane = (size_t)B * T * C;
    float* gw_part = ws + 5 * plane;
    float* gu_part = gw_part + (size_t)B * C;
    hipLaunchKernelGGL((biwkv_bwd_kernel<IO>), dim3((C + 63) / 64, B), dim3(64), 0, st, w, u,
                       static_cast<const IO*>(k), static_cast<const IO*>(v), static_cast<const IO*>(gy),
                       static_cast<IO*>(gk), static_cast<IO*>(gv), ws, gw_part, gu_part, B, T, C);
    hipLaunchKernelGGL(biwkv_bwd_reduce_kernel, dim3((C + 255) / 256), dim3(256), 0, st, gw_part, gu_part, gw, gu, B, C);
    return check_launch("biwkv_bwd");
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" size_t vrwkv_biwkv_bwd_workspace_bytes(int B, int T, int C, int io_dtype) {
    if (validate(B, T, C, io_dtype) != VRWKV_OK) return 0;
    return ((size_t)5 * B * T * C + (size_t)2 * B * C) * sizeof(float);
}

extern "C" int vrwkv_biwkv_bwd(const float* w, const float* u, const void* k, const void* v, const void* gy,
                               float* gw, float* gu, void* gk, void* gv, int B, int T, int C, int io_dtype,
                               void* workspace, size_t workspace_bytes, void* hip_stream) {
    int rc = validate(B, T, C, io_dtype);
    if (rc != VRWKV_OK) return rc;
    if (!w || !u || !k || !v || !gy || !gw || !gu || !gk || !gv) {
        set_error("biwkv_bwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    const size_t need = ((size_t)5 * B * T * C + (size_t)2 * B * C) * sizeof(float);
    if (!workspace || workspace_bytes < need) {
        set_error("biwkv_bwd: workspace of %zu bytes required (got %zu)", need, workspace ? workspace_bytes : (size_t)0);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    const size_t esz = io_dtype == VRWKV_F32 ? 4 : 2;
    if ((((uintptr_t)k | (uintptr_t)v | (uintptr_t)gy | (uintptr_t)gk | (uintptr_t)gv) & (esz - 1)) ||
        (((uintptr_t)w | (uintptr_t)u | (uintptr_t)gw | (uintptr_t)gu | (uintptr_t)workspace) & 3)) {
        set_error("biwkv_bwd: pointers must be aligned to their element size");
        return VRWKV_INVALID_ARG;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* ws = static_cast<float*>(workspace);
    switch (io_dtype) {
        case VRWKV_F32:  return launch<float>(w, u, k, v, gy, gw, gu, gk, gv, ws, B, T, C, st);
        case VRWKV_BF16: return launch<__hip_bfloat16>(w, u, k, v, gy, gw, gu, gk, gv, ws, B, T, C, st);
        case VRWKV_F16:  return launch<__half>(w, u, k, v, gy, gw, gu, gk, gv, ws, B, T, C, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
