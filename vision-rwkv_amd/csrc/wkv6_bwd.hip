// wkv6 backward for gfx950: gr, gk, gv, gw (B,T,C) fp32 and gu (H,64) from gy.
// Replaces backward(B,T,C,H,r,k,v,ew,u,gy,gr,gk,gv,gw,gu)
// (classification/mmcls_custom/models/backbones/cuda_v6/wkv6_op.cpp:10-12, kernels
//  .../cuda_v6/wkv6_cuda.cu:99-346), without its T <= 256 limit (per-thread arrays of length _T_).
//
// The forward is the sum of two causal passes (DIR 0: tokens ascending, with the bonus u; DIR 1:
// descending, no bonus).  In a pass's own token order n, with S_n the state before token n,
//   y_n = r_n (diag(u) k_n v_n^T + S_n),   S_{n+1} = diag(d_n) S_n + k_n v_n^T,  d = exp(ew), ew = -exp(w)
// the gradients are, with the adjoint state G_n = r_n gy_n^T + diag(d_n) G_{n+1}:
//   gr_n[j] = u_j k_n[j] (v_n.gy_n) + (S_n gy_n)[j]
//   gk_n[j] = u_j r_n[j] (v_n.gy_n) + (G_{n+1} v_n)[j]
//   gv_n[i] = sum_j k_n[j] ( u_j r_n[j] gy_n[i] + G_{n+1}[j,i] )
//   gu[j]   = sum_n r_n[j] k_n[j] (v_n.gy_n)
//   gw_n[j] = ew_n[j] * ( sum_{m>n} (a_m[j] - b_m[j]) - b_n[j] ),
//             a_n = r_n[j] (S_n gy_n)[j],  b_n = k_n[j] (G_{n+1} v_n)[j]
// (the last line follows from X_n = sum_i S_n[j,i] G_n[j,i]:  d_n * dL/dd_n = X_n - a_n = X_{n+1} - b_n;
//  gw is the gradient w.r.t. the raw decay logit, as in wkv6_cuda.cu:248,277.)
//
// Three sweeps per pass, each a sequential 64x64-state scan like the forward's exact kernel: one
// 256-thread workgroup per (b,h); a lane owns one "own" index and a 16-wide slice of the other
// index, quads finish the contractions with two quad-permute adds; each wave stages the rows of a
// token in its own LDS slot, so the token loop has no workgroup barrier.
//   sweep S (ascending)   own = key j:    S  -> gr, a (workspace), gu partial
//   sweep G (descending)  own = key j:    G  -> gk, gw
//   sweep V (descending)  own = value i:  G^T -> gv
#include "wkv6_bwd_chunk.h"
#include <cstdlib>
#include <type_traits>

namespace vrwkv {
namespace {

constexpr int N = 64;

template <typename T> __device__ __forceinline__ float ldf(const T* p, size_t o) { return to_f32(p[o]); }
__device__ __forceinline__ float quad_sum(float x) {
    x += __shfl_xor(x, 1);
    x += __shfl_xor(x, 2);
    return x;
}
__device__ __forceinline__ void lds_order() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
template <typename WT, bool W_IS_EW>
__device__ __forceinline__ float log_decay(const WT* w_, size_t o) {
    const float w = to_f32(w_[o]);
    return W_IS_EW ? w : -__expf(w);
}

// ---- sweep S: state S, own = j ----------------------------------------------------------------
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__device__ __forceinline__
void wkv6_bwd_sweep_s_body(int bh, const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                      const WT* __restrict__ w_, const float* __restrict__ u_, const float* __restrict__ gy_,
                      float* __restrict__ gr_, float* __restrict__ a_, float* __restrict__ gu_part,
                      int T, int C, int H)
{
    __shared__ __attribute__((aligned(16))) float s_row[4][2][N];       // [wave][v, gy][i]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = bh / H, h = bh % H;
    const int sq = lane & 3, j = wave * 16 + (lane >> 2);
    const size_t base = (size_t)b * T * C + (size_t)h * N;
    const float uj = DIR == 0 ? u_[h * N + j] : 0.f;
    float S[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) S[e] = 0.f;
    float gu = 0.f;
    for (int n = 0; n < T; ++n) {
        const int t = DIR == 0 ? n : T - 1 - n;
        const size_t o = base + (size_t)t * C;
        s_row[wave][0][lane] = ldf(v_, o + lane);
        s_row[wave][1][lane] = gy_[o + lane];
        const float rj = ldf(r_, o + j), kj = ldf(k_, o + j), dj = __expf(log_decay<WT, W_IS_EW>(w_, o + j));
        lds_order();
        float dot = 0.f, sg = 0.f;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const float4 v4 = *reinterpret_cast<const float4*>(&s_row[wave][0][sq * 16 + q4 * 4]);
            const float4 g4 = *reinterpret_cast<const float4*>(&s_row[wave][1][sq * 16 + q4 * 4]);
            const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float& s = S[q4 * 4 + e];
                dot = fmaf(vv[e], gg[e], dot);
                sg = fmaf(s, gg[e], sg);
                s = fmaf(s, dj, kj * vv[e]);
            }
        }
        dot = quad_sum(dot);
        sg = quad_sum(sg);
        if (sq == 0) {
            const float gr = uj * kj * dot + sg;
            if (DIR == 0) gr_[o + j] += gr; else gr_[o + j] = gr;
            a_[o + j] = rj * sg;
        }
        gu = fmaf(rj * kj, dot, gu);
        lds_order();
    }
    if (DIR == 0 && sq == 0) gu_part[(size_t)b * C + h * N + j] = gu;
}

// ---- sweep G: adjoint G, own = j, descending in pass order ---------------------------------------
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__device__ __forceinline__
void wkv6_bwd_sweep_g_body(int bh, const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                      const WT* __restrict__ w_, const float* __restrict__ u_, const float* __restrict__ gy_,
                      const float* __restrict__ a_, float* __restrict__ gk_, float* __restrict__ gw_,
                      int T, int C, int H)
{
    __shared__ __attribute__((aligned(16))) float s_row[4][2][N];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = bh / H, h = bh % H;
    const int sq = lane & 3, j = wave * 16 + (lane >> 2);
    const size_t base = (size_t)b * T * C + (size_t)h * N;
    const float uj = DIR == 0 ? u_[h * N + j] : 0.f;
    float G[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) G[e] = 0.f;
    float X = 0.f;                                        // sum over later tokens of (a - b)
    for (int n = T - 1; n >= 0; --n) {
        const int t = DIR == 0 ? n : T - 1 - n;
        const size_t o = base + (size_t)t * C;
        s_row[wave][0][lane] = ldf(v_, o + lane);
        s_row[wave][1][lane] = gy_[o + lane];
        const float rj = ldf(r_, o + j), kj = ldf(k_, o + j), ew = log_decay<WT, W_IS_EW>(w_, o + j);
        const float dj = __expf(ew), an = a_[o + j];
        lds_order();
        float dot = 0.f, gvv = 0.f;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const float4 v4 = *reinterpret_cast<const float4*>(&s_row[wave][0][sq * 16 + q4 * 4]);
            const float4 g4 = *reinterpret_cast<const float4*>(&s_row[wave][1][sq * 16 + q4 * 4]);
            const float vv[4] = {v4.x, v4.y, v4.z, v4.w}, gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float& gq = G[q4 * 4 + e];
                dot = fmaf(vv[e], gg[e], dot);
                gvv = fmaf(gq, vv[e], gvv);
                gq = fmaf(gq, dj, rj * gg[e]);
            }
        }
        dot = quad_sum(dot);
        gvv = quad_sum(gvv);
        const float bn = kj * gvv;
        if (sq == 0) {
            const float gk = uj * rj * dot + gvv;
            const float gw = ew * (X - bn);
            if (DIR == 0) { gk_[o + j] += gk; gw_[o + j] += gw; } else { gk_[o + j] = gk; gw_[o + j] = gw; }
        }
        X += an - bn;
        lds_order();
    }
}

// ---- sweep V: adjoint G^T, own = i, descending in pass order --------------------------------------
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__device__ __forceinline__
void wkv6_bwd_sweep_v_body(int bh, const IO* __restrict__ r_, const IO* __restrict__ k_,
                      const WT* __restrict__ w_, const float* __restrict__ u_, const float* __restrict__ gy_,
                      float* __restrict__ gv_, int T, int C, int H)
{
    __shared__ __attribute__((aligned(16))) float s_row[4][3][N];       // [wave][r, k, d][j]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = bh / H, h = bh % H;
    const int sq = lane & 3, i = wave * 16 + (lane >> 2);
    const size_t base = (size_t)b * T * C + (size_t)h * N;
    float uu[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) uu[e] = DIR == 0 ? u_[h * N + sq * 16 + e] : 0.f;
    float G[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) G[e] = 0.f;
    for (int n = T - 1; n >= 0; --n) {
        const int t = DIR == 0 ? n : T - 1 - n;
        const size_t o = base + (size_t)t * C;
        s_row[wave][0][lane] = ldf(r_, o + lane);
        s_row[wave][1][lane] = ldf(k_, o + lane);
        s_row[wave][2][lane] = __expf(log_decay<WT, W_IS_EW>(w_, o + lane));
        const float gyi = gy_[o + i];
        lds_order();
        float gv = 0.f;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const float4 r4 = *reinterpret_cast<const float4*>(&s_row[wave][0][sq * 16 + q4 * 4]);
            const float4 k4 = *reinterpret_cast<const float4*>(&s_row[wave][1][sq * 16 + q4 * 4]);
            const float4 d4 = *reinterpret_cast<const float4*>(&s_row[wave][2][sq * 16 + q4 * 4]);
            const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, dd[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float& gq = G[q4 * 4 + e];
                const float rg = rr[e] * gyi;
                gv = fmaf(kk[e], fmaf(uu[q4 * 4 + e], rg, gq), gv);
                gq = fmaf(gq, dd[e], rg);
            }
        }
        gv = quad_sum(gv);
        if (sq == 0) {
            if (DIR == 0) gv_[o + i] += gv; else gv_[o + i] = gv;
        }
        lds_order();
    }
}

// ---- kernels: one sweep each (sequential path), or all six for the sequences the chunked scans left ----
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__global__ __launch_bounds__(256)
void wkv6_bwd_sweep_s(const IO* r_, const IO* k_, const IO* v_, const WT* w_, const float* u_, const float* gy_,
                      float* gr_, float* a_, float* gu_part, int T, int C, int H) {
    wkv6_bwd_sweep_s_body<IO, WT, DIR, W_IS_EW>(blockIdx.x, r_, k_, v_, w_, u_, gy_, gr_, a_, gu_part, T, C, H);
}
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__global__ __launch_bounds__(256)
void wkv6_bwd_sweep_g(const IO* r_, const IO* k_, const IO* v_, const WT* w_, const float* u_, const float* gy_,
                      const float* a_, float* gk_, float* gw_, int T, int C, int H) {
    wkv6_bwd_sweep_g_body<IO, WT, DIR, W_IS_EW>(blockIdx.x, r_, k_, v_, w_, u_, gy_, a_, gk_, gw_, T, C, H);
}
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__global__ __launch_bounds__(256)
void wkv6_bwd_sweep_v(const IO* r_, const IO* k_, const WT* w_, const float* u_, const float* gy_,
                      float* gv_, int T, int C, int H) {
    wkv6_bwd_sweep_v_body<IO, WT, DIR, W_IS_EW>(blockIdx.x, r_, k_, w_, u_, gy_, gv_, T, C, H);
}
// Sequences flagged by the chunked scans (a chunk decaying below e^-60): all six sweeps, descending pass
// first.  Every sweep maps (token, channel) to the same thread as the sweep it depends on, so program
// order is enough between them.
template <typename IO, typename WT, bool W_IS_EW>
__global__ __launch_bounds__(256)
void wkv6_bwd_fallback(const IO* r_, const IO* k_, const IO* v_, const WT* w_, const float* u_, const float* gy_,
                       float* gr_, float* gk_, float* gv_, float* gw_, float* a_, float* gu_part,
                       const unsigned char* todo, int T, int C, int H) {
    const int bh = blockIdx.x;
    if (!todo[bh]) return;
    wkv6_bwd_sweep_s_body<IO, WT, 1, W_IS_EW>(bh, r_, k_, v_, w_, u_, gy_, gr_, a_, gu_part, T, C, H);
    wkv6_bwd_sweep_g_body<IO, WT, 1, W_IS_EW>(bh, r_, k_, v_, w_, u_, gy_, a_, gk_, gw_, T, C, H);
    wkv6_bwd_sweep_v_body<IO, WT, 1, W_IS_EW>(bh, r_, k_, w_, u_, gy_, gv_, T, C, H);
    wkv6_bwd_sweep_s_body<IO, WT, 0, W_IS_EW>(bh, r_, k_, v_, w_, u_, gy_, gr_, a_, gu_part, T, C, H);
    wkv6_bwd_sweep_g_body<IO, WT, 0, W_IS_EW>(bh, r_, k_, v_, w_, u_, gy_, a_, gk_, gw_, T, C, H);
    wkv6_bwd_sweep_v_body<IO, WT, 0, W_IS_EW>(bh, r_, k_, w_, u_, gy_, gv_, T, C, H);
}

template <typename IO, typename WT, bool EW>
int launch_all(const void* r, const void* k, const void* v, const void* w, const float* u, const float* gy,
               float* gr, float* gk, float* gv, float* gw, float* gu, float* ws, int B, int T, int C, int H, hipStream_t st) {
    const IO* rr = static_cast<const IO*>(r);
    const IO* kk = static_cast<const IO*>(k);
    const IO* vv = static_cast<const IO*>(v);
    const WT* ww = static_cast<const WT*>(w);
    float* a = ws;                                       // (B,T,C)
    float* gu_part = ws + (size_t)B * T * C;             // (B,C)
    const dim3 grid(B * H), block(256);
    {
        if (!option(OPT_WKV6_BWD_SCALAR) && (long long)T * C < (1LL << 29)) {   // the option forces the sequential sweeps (testing)
            using namespace wkv6_detail;
            unsigned char* todo = reinterpret_cast<unsigned char*>(gu_part + (size_t)B * C);
            const dim3 blk(128);
#define VRWKV_SCAN(KIND, DIR, OUT) hipLaunchKernelGGL((wkv6_bwd_scan_kernel<IO, WT, KIND, DIR, EW>), grid, blk, 0, st, \
                                                      rr, kk, vv, ww, u, gy, OUT, a, gw, gu_part, todo, T, C, H)
            // gr descending first: it clears the fallback flags
            VRWKV_SCAN(SCAN_GR, 1, gr); VRWKV_SCAN(SCAN_GK, 1, gk); VRWKV_SCAN(SCAN_GV, 1, gv);
            VRWKV_SCAN(SCAN_GR, 0, gr); VRWKV_SCAN(SCAN_GK, 0, gk); VRWKV_SCAN(SCAN_GV, 0, gv);
#undef VRWKV_SCAN
            hipLaunchKernelGGL((wkv6_bwd_fallback<IO, WT, EW>), grid, block, 0, st, rr, kk, vv, ww, u, gy, gr, gk, gv, gw,
                               a, gu_part, todo, T, C, H);
            hipLaunchKernelGGL(batch_sum_kernel, dim3((C + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, gu_part, gu, (const float*)nullptr,
                               (float*)nullptr, B, C);
            return check_launch("wkv6_bwd (chunked)");
        }
    }
    // descending pass first (writes), ascending pass second (accumulates), as in the forward
    hipLaunchKernelGGL((wkv6_bwd_sweep_s<IO, WT, 1, EW>), grid, block, 0, st, rr, kk, vv, ww, u, gy, gr, a, gu_part, T, C, H);
    hipLaunchKernelGGL((wkv6_bwd_sweep_g<IO, WT, 1, EW>), grid, block, 0, st, rr, kk, vv, ww, u, gy, a, gk, gw, T, C, H);
    hipLaunchKernelGGL((wkv6_bwd_sweep_v<IO, WT, 1, EW>), grid, block, 0, st, rr, kk, ww, u, gy, gv, T, C, H);
    hipLaunchKernelGGL((wkv6_bwd_sweep_s<IO, WT, 0, EW>), grid, block, 0, st, rr, kk, vv, ww, u, gy, gr, a, gu_part, T, C, H);
    hipLaunchKernelGGL((wkv6_bwd_sweep_g<IO, WT, 0, EW>), grid, block, 0, st, rr, kk, vv, ww, u, gy, a, gk, gw, T, C, H);
    hipLaunchKernelGGL((wkv6_bwd_sweep_v<IO, WT, 0, EW>), grid, block, 0, st, rr, kk, ww, u, gy, gv, T, C, H);
    hipLaunchKernelGGL(batch_sum_kernel, dim3((C + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, gu_part, gu, (const float*)nullptr, (float*)nullptr, B, C);   // torch.sum(gu, 0), vrwkv6.py:69
    return check_launch("wkv6_bwd");
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" size_t vrwkv_wkv6_bwd_workspace_bytes(int B, int T, int C, int H) {
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0) return 0;
    return ((size_t)B * T * C + (size_t)B * C) * sizeof(float) + (((size_t)B * H + 255) & ~(size_t)255);
}

extern "C" int vrwkv_wkv6_bwd(const void* r, const void* k, const void* v, const void* w, const float* u,
                              const float* gy, float* gr, float* gk, float* gv, float* gw, float* gu,
                              int B, int T, int C, int H, int rkv_dtype, int w_dtype, int w_is_ew,
                              void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0) {
        set_error("wkv6_bwd: B, T, C, H must be positive (got %d, %d, %d, %d)", B, T, C, H);
        return VRWKV_INVALID_ARG;
    }
    if (C != H * N) {
        set_error("wkv6_bwd: C must equal H*64 (got C=%d, H=%d)", C, H);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    for (int dt : {rkv_dtype, w_dtype})
        if (dt != VRWKV_F32 && dt != VRWKV_BF16 && dt != VRWKV_F16) {
            set_error("wkv6_bwd: unsupported dtype code %d", dt);
            return VRWKV_UNSUPPORTED_DTYPE;
        }
    if (w_dtype != VRWKV_F32 && w_dtype != rkv_dtype) {
        set_error("wkv6_bwd: w must be fp32 or have the dtype of r, k, v");
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (!r || !k || !v || !w || !u || !gy || !gr || !gk || !gv || !gw || !gu) {
        set_error("wkv6_bwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    const size_t need = ((size_t)B * T * C + (size_t)B * C) * sizeof(float) + (((size_t)B * H + 255) & ~(size_t)255);
    if (!workspace || workspace_bytes < need) {
        set_error("wkv6_bwd: workspace of %zu bytes required (got %zu)", need, workspace ? workspace_bytes : (size_t)0);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* ws = static_cast<float*>(workspace);
    const bool ew = w_is_ew != 0;
#define VRWKV_GO(IO, WT) (ew ? launch_all<IO, WT, true>(r, k, v, w, u, gy, gr, gk, gv, gw, gu, ws, B, T, C, H, st) \
                             : launch_all<IO, WT, false>(r, k, v, w, u, gy, gr, gk, gv, gw, gu, ws, B, T, C, H, st))
    switch (rkv_dtype) {
        case VRWKV_F32:  return VRWKV_GO(float, float);
        case VRWKV_BF16: return w_dtype == VRWKV_F32 ? VRWKV_GO(__hip_bfloat16, float) : VRWKV_GO(__hip_bfloat16, __hip_bfloat16);
        case VRWKV_F16:  return w_dtype == VRWKV_F32 ? VRWKV_GO(__half, float) : VRWKV_GO(__half, __half);
    }
#undef VRWKV_GO
    return VRWKV_UNSUPPORTED_DTYPE;
}
