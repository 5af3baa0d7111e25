// wkv6 forward, sequential-state kernel (exact for any decay; also the fallback of the chunked
// matrix-core kernel).  Bidirectional RWKV-6 scan of
// classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:6-97:
//   y_t[i] = sum_j r_t[j] ( u[j] k_t[j] v_t[i] + S_t[j,i] + S'_t[j,i] ),  S <- diag(d_t) S + k_t v_t^T
// with d_t = exp(-exp(w_t)) (vrwkv6.py:48 + wkv6_cuda.cu:26).
//
// Mapping (the reference uses one 64-thread block per (b,h) with a 64-float state column per
// thread): one 256-thread workgroup per (b,h); a wave owns 16 value channels i, and inside it
// the four lanes of a quad split the 64 key channels j, so a lane keeps a 16-float slice of the
// state column and the read-out r_t . S[:,i] is finished by two quad-permute adds.  Each wave
// stages the r, k, d rows of a token in its own LDS slot (no workgroup barrier in the loop) and
// fetches the next token's rows while it works on the current one.
#pragma once
#include "vrwkv_common.h"

namespace vrwkv {
namespace wkv6_detail {

constexpr int N = 64;            // head size (vrwkv6.py:23)

// One pass over one (b,h) sequence by a 256-thread workgroup.  DIR 0: ascending pass with the bonus,
// accumulates into y.  DIR 1: descending pass, writes y.  s_row: 4*2*3*64 floats of LDS.
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__device__ __forceinline__
void wkv6_scalar_pass(const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                      const WT* __restrict__ w_, const float* __restrict__ u_, float* __restrict__ y_,
                      float* __restrict__ s_row_raw, int bh, int T, int C, int H)
{
    float (*s_row)[2][3][N] = reinterpret_cast<float (*)[2][3][N]>(s_row_raw);   // [wave][buffer][r,k,d][j]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int b = bh / H, h = bh % H;
    const int jg = lane & 3;                             // which 16 key channels
    const int i = wave * 16 + (lane >> 2);               // value channel
    const size_t base = (size_t)b * T * C + (size_t)h * N;

    float S[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) S[j] = 0.f;
    float uu[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) uu[j] = DIR == 0 ? u_[h * N + jg * 16 + j] : 0.f;

    auto fetch = [&](int t, float& fr, float& fk, float& fd, float& fv) {
        const size_t o = base + (size_t)t * C;
        fr = to_f32(r_[o + lane]);
        fk = to_f32(k_[o + lane]);
        const float w = to_f32(w_[o + lane]);
        fd = W_IS_EW ? __expf(w) : __expf(-__expf(w));
        fv = to_f32(v_[o + i]);
    };
    const int t_first = DIR == 0 ? 0 : T - 1;
    const int step = DIR == 0 ? 1 : -1;
    float fr, fk, fd, fv;
    fetch(t_first, fr, fk, fd, fv);
    int buf = 0;
    for (int n = 0, t = t_first; n < T; ++n, t += step) {
        float(*row)[N] = s_row[wave][buf];
        row[0][lane] = fr; row[1][lane] = fk; row[2][lane] = fd;
        const float v = fv;
        if (n + 1 < T) fetch(t + step, fr, fk, fd, fv);  // next token, behind the arithmetic
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        float y = 0.f;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const float4 r4 = *reinterpret_cast<const float4*>(&row[0][jg * 16 + q4 * 4]);
            const float4 k4 = *reinterpret_cast<const float4*>(&row[1][jg * 16 + q4 * 4]);
            const float4 d4 = *reinterpret_cast<const float4*>(&row[2][jg * 16 + q4 * 4]);
            const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, dd[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = q4 * 4 + e;
                const float kv = kk[e] * v;
                y = fmaf(rr[e], DIR == 0 ? fmaf(uu[j], kv, S[j]) : S[j], y);
                S[j] = fmaf(S[j], dd[e], kv);
            }
        }
        // sum over the four lanes of the quad (the four key-channel slices)
        y += __shfl_xor(y, 1);
        y += __shfl_xor(y, 2);
        if (jg == 0) {
            const size_t o = base + (size_t)t * C + i;
            if (DIR == 0) y_[o] += y; else y_[o] = y;
        }
        buf ^= 1;
    }
}

template <typename IO, typename WT, int DIR, bool W_IS_EW>
__global__ __launch_bounds__(256)
void wkv6_fwd_scalar_kernel(const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                            const WT* __restrict__ w_, const float* __restrict__ u_, float* __restrict__ y_,
                            int T, int C, int H)
{
    __shared__ __attribute__((aligned(16))) float s_row[4 * 2 * 3 * N];
    wkv6_scalar_pass<IO, WT, DIR, W_IS_EW>(r_, k_, v_, w_, u_, y_, s_row, blockIdx.x, T, C, H);
}

}  // namespace wkv6_detail
}  // namespace vrwkv
