// wkv6 forward, chunked matrix-core kernel for gfx950 (bf16 MFMA, fp32 accumulate).
//
// Bidirectional RWKV-6 scan of
// classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:6-97, evaluated as two
// passes (DIR 1: tokens descending, writes y; DIR 0: ascending with the bonus u, adds to y),
// each pass being the same causal algorithm on its own token order n = 0..T-1:
//
//   y_n = sum_j r_n[j] ( u[j] k_n[j] v_n  +  sum_{m<n} (prod_{m<l<n} d_l[j]) k_m[j] v_m )
//
// Chunks of 32 tokens.  With the in-chunk cumulative log-decay P_n = sum_{l<=n} log d_l
// (Pex_n = P_n - log d_n) and the mid-chunk reference Pref = P_15:
//   rt_n = r_n * exp(Pex_n - Pref),   kt_m = k_m * exp(Pref - P_m)      (rt_n . kt_m = decay for m<n)
//   A[n][m] = rt_n . kt_m  (m < n),  0 otherwise                          -> MFMA 1
//   Y       = A V  +  rt (diag(e^Pref) S)                                 -> MFMA 2, 3
//   S'      = diag(e^P31) S + diag(e^(P31-Pref)) (kt^T V)                 -> MFMA 4
// S (64x64 fp32) never leaves the accumulator registers: each wave owns the 32 value columns of
// one half and feeds its S tiles straight back as the B operand of MFMA 3 (the contraction index
// is taken in the order the accumulator layout provides, and the A operand is read from LDS in
// that same order); likewise A goes from the accumulators of MFMA 1 into the A operand of MFMA 2.
//
// Precision: every operand that is computed rather than loaded (rt, kt, A, S) is split into a
// bf16 head and a bf16 tail and the products head*head + head*tail + tail*head are accumulated,
// which keeps the result within ~3e-5 of the fp32 recurrence (one bf16 rounding of any of them
// alone costs ~1e-2).  v is exact in bf16 for bf16 input and split in two for fp16 / fp32 input.
//
// Range: the factorisation needs |P31| <= 60 in every chunk (decay over 32 tokens no stronger
// than e^-60).  A (b,h) sequence with a chunk outside that range is left to the sequential-state
// kernel: the pass records it in `todo` and stops.
#pragma once
#include "vrwkv_common.h"
#include <type_traits>

namespace vrwkv {
namespace wkv6_detail {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int LC = 32;           // chunk length
constexpr int HN = 64;           // head size
constexpr int PJ = 72;           // row pitch (bf16) of the [token][channel] operand arrays
constexpr int PS = 40;           // row pitch (bf16) of the [channel][token] operand arrays
constexpr float SAFE_DECAY = 60.f;

__device__ __forceinline__ bf16x8 cat8(bf16x4 a, bf16x4 b) {
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}
// Sum over the 64 lanes, result wave-uniform: four DPP steps inside each 16-lane row (VALU rate),
// then the four row sums through scalar registers.
__device__ __forceinline__ float wave_sum(float x) {
    auto dpp = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xf, 0xf, true));
    };
    x += dpp(x, std::integral_constant<int, 0xB1>{});    // quad_perm [1,0,3,2]
    x += dpp(x, std::integral_constant<int, 0x4E>{});    // quad_perm [2,3,0,1]
    x += dpp(x, std::integral_constant<int, 0x141>{});   // row_half_mirror
    x += dpp(x, std::integral_constant<int, 0x140>{});   // row_mirror
    const int xi = __builtin_bit_cast(int, x);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 48));
}
// head/tail split of eight fp32 accumulator values into two packed bf16 operands
__device__ __forceinline__ void split8(const float (&x)[8], bf16x8& hi, bf16x8& lo) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const __bf16 h = (__bf16)x[e];
        hi[e] = h;
        lo[e] = (__bf16)(x[e] - (float)h);
    }
}

// VSPLIT: v is given in a type that is not exact in bf16 (fp16, fp32) and is split in two.
template <typename IO, typename WT, int DIR, bool W_IS_EW>
__global__ __launch_bounds__(128)
void wkv6_fwd_chunk_kernel(const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                           const WT* __restrict__ w_, const float* __restrict__ u_, float* __restrict__ y_,
                           unsigned char* __restrict__ todo, int T, int C, int H)
{
    constexpr bool VSPLIT = !(sizeof(IO) == 2 && __is_same(IO, __hip_bfloat16));
    __shared__ __attribute__((aligned(16))) __bf16 sRh[LC][PJ], sRl[LC][PJ], sKh[LC][PJ], sKl[LC][PJ];
    __shared__ __attribute__((aligned(16))) __bf16 sKth[HN][PS], sKtl[HN][PS], sVt[HN][PS], sVtl[VSPLIT ? HN : 1][PS];
    __shared__ __attribute__((aligned(16))) float sC1[HN], sC2[HN], sC3[HN], sTot[HN], sBonus[LC];
    __shared__ int sFlag;

    const int lane = threadIdx.x & 63;
    const int q = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);    // wave: token half in stage E, value half in stage M
    const int g = lane >> 5, x = lane & 31;
    const int bh = blockIdx.x;
    const int b = bh / H, h = bh % H;
    const size_t base = (size_t)b * T * C + (size_t)h * HN;
    const int nchunk = (T + LC - 1) / LC;
    const float uj = DIR == 0 ? u_[h * HN + lane] : 0.f;
    if (threadIdx.x == 0) sFlag = 0;

    f32x16 S0 = {0}, S1 = {0};          // state tiles: rows j = 32*jh + 8(r/4)+4g+(r%4), column i = 32q + x

    for (int ch = 0; ch < nchunk; ++ch) {
        // =============================== stage E: elementwise =================================
        // wave q prepares tokens n = 16q .. 16q+15 of the chunk; lane = channel j (and i for v)
        float rr[16], kk[16], vv[16], ld[16];
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            const int ng = ch * LC + 16 * q + m;
            const bool ok = ng < T;
            const int t = DIR == 0 ? ng : T - 1 - ng;
            const size_t o = base + (size_t)(ok ? t : 0) * C + lane;
            const float fr = to_f32(r_[o]), fk = to_f32(k_[o]), fv = to_f32(v_[o]), fw = to_f32(w_[o]);
            rr[m] = ok ? fr : 0.f;
            kk[m] = ok ? fk : 0.f;
            vv[m] = ok ? fv : 0.f;
            ld[m] = ok ? (W_IS_EW ? fw : -__expf(fw)) : 0.f;
        }
        float p[16];
        p[0] = ld[0];
#pragma unroll
        for (int m = 1; m < 16; ++m) p[m] = p[m - 1] + ld[m];
        if (q == 0) sTot[lane] = p[15];
        lds_barrier();                                                   // (1)
        const float pref = sTot[lane];                                   // P_15
        const float off = q == 1 ? pref : 0.f;
        if (q == 1) {
            const float p31 = p[15] + off;
            sC2[lane] = __expf(p31);
            sC3[lane] = __expf(p31 - pref);
            if (__builtin_amdgcn_ballot_w64(!(p31 >= -SAFE_DECAY)) != 0ull && lane == 0) sFlag = 1;
        } else {
            sC1[lane] = __expf(pref);
        }
        {
            bf16x8 kth[2], ktl[2], vth[2], vtl[2];
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                const int n = 16 * q + m;
                const float P = p[m] + off;
                const float f1 = __expf(P - ld[m] - pref);               // exp(Pex - Pref)
                const float f2 = __expf(pref - P);                        // exp(Pref - P)
                const float rt = rr[m] * f1, kt = kk[m] * f2;
                const __bf16 rh = (__bf16)rt, kh = (__bf16)kt;
                const __bf16 rl = (__bf16)(rt - (float)rh), kl = (__bf16)(kt - (float)kh);
                sRh[n][lane] = rh; sRl[n][lane] = rl;
                sKh[n][lane] = kh; sKl[n][lane] = kl;
                kth[m >> 3][m & 7] = kh; ktl[m >> 3][m & 7] = kl;
                const __bf16 vh = (__bf16)vv[m];
                vth[m >> 3][m & 7] = vh;
                if (VSPLIT) vtl[m >> 3][m & 7] = (__bf16)(vv[m] - (float)vh);
                if (DIR == 0) {
                    const float c = wave_sum(rr[m] * uj * kk[m]);
                    if (lane == 0) sBonus[n] = c;
                }
            }
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<bf16x8*>(&sKth[lane][16 * q + 8 * e]) = kth[e];
                *reinterpret_cast<bf16x8*>(&sKtl[lane][16 * q + 8 * e]) = ktl[e];
                *reinterpret_cast<bf16x8*>(&sVt[lane][16 * q + 8 * e]) = vth[e];
                if (VSPLIT) *reinterpret_cast<bf16x8*>(&sVtl[lane][16 * q + 8 * e]) = vtl[e];
            }
        }
        lds_barrier();                                                   // (2)
        if (sFlag) {                                                      // out of range: leave to the exact kernel
            if (threadIdx.x == 0) todo[(size_t)DIR * gridDim.x + bh] = 1;
            return;
        }

        // ================================= stage M: matrix cores ===============================
        const int icol = 32 * q + x;                                      // value column of this lane
        // ---- MFMA 1: A^T: acc[m = s][n = t]; lane holds t = x, rows s = 8(r/4)+4g+(r%4) ----
        f32x16 accA = {0};
#pragma unroll
        for (int kq = 0; kq < 4; ++kq) {
            const bf16x8 ah = *reinterpret_cast<const bf16x8*>(&sKh[x][16 * kq + 8 * g]);
            const bf16x8 al = *reinterpret_cast<const bf16x8*>(&sKl[x][16 * kq + 8 * g]);
            const bf16x8 bh_ = *reinterpret_cast<const bf16x8*>(&sRh[x][16 * kq + 8 * g]);
            const bf16x8 bl = *reinterpret_cast<const bf16x8*>(&sRl[x][16 * kq + 8 * g]);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh_, accA, 0, 0, 0);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, accA, 0, 0, 0);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh_, accA, 0, 0, 0);
        }
        bf16x8 Ah[2], Al[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            float a8[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int r = 8 * ks + e;
                const int s = 8 * (r / 4) + 4 * g + (r % 4);
                a8[e] = s < x ? accA[r] : 0.f;                            // strictly earlier tokens only
            }
            split8(a8, Ah[ks], Al[ks]);
        }
        // ---- MFMA 2: Y[t][i] = sum_s A[t][s] V[s][i]; contraction order = accumulator order ----
        f32x16 accY = {0};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bf16x8 bv = cat8(*reinterpret_cast<const bf16x4*>(&sVt[icol][16 * ks + 4 * g]),
                                   *reinterpret_cast<const bf16x4*>(&sVt[icol][16 * ks + 8 + 4 * g]));
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ah[ks], bv, accY, 0, 0, 0);
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Al[ks], bv, accY, 0, 0, 0);
            if (VSPLIT) {
                const bf16x8 bvl = cat8(*reinterpret_cast<const bf16x4*>(&sVtl[icol][16 * ks + 4 * g]),
                                        *reinterpret_cast<const bf16x4*>(&sVtl[icol][16 * ks + 8 + 4 * g]));
                accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ah[ks], bvl, accY, 0, 0, 0);
            }
        }
        // ---- MFMA 3: Y += rt (diag(e^Pref) S), S straight from the accumulators ----
#pragma unroll
        for (int jh = 0; jh < 2; ++jh) {
            const f32x16& S = jh == 0 ? S0 : S1;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float s8[8];
#pragma unroll
                for (int e4 = 0; e4 < 2; ++e4) {
                    const f32x4 c1 = *reinterpret_cast<const f32x4*>(&sC1[32 * jh + 16 * ks + 8 * e4 + 4 * g]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) s8[4 * e4 + e] = S[8 * ks + 4 * e4 + e] * c1[e];
                }
                bf16x8 sh, sl;
                split8(s8, sh, sl);
                const int j0 = 32 * jh + 16 * ks + 4 * g;
                const bf16x8 ah = cat8(*reinterpret_cast<const bf16x4*>(&sRh[x][j0]),
                                       *reinterpret_cast<const bf16x4*>(&sRh[x][j0 + 8]));
                const bf16x8 al = cat8(*reinterpret_cast<const bf16x4*>(&sRl[x][j0]),
                                       *reinterpret_cast<const bf16x4*>(&sRl[x][j0 + 8]));
                accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, sh, accY, 0, 0, 0);
                accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, sl, accY, 0, 0, 0);
                accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, sh, accY, 0, 0, 0);
            }
        }
        // ---- MFMA 4: M[j][i] = sum_s kt[s][j] V[s][i];  S' = e^P31 S + e^(P31-Pref) M ----
#pragma unroll
        for (int jh = 0; jh < 2; ++jh) {
            f32x16 accM = {0};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const bf16x8 ah = *reinterpret_cast<const bf16x8*>(&sKth[32 * jh + x][16 * ks + 8 * g]);
                const bf16x8 al = *reinterpret_cast<const bf16x8*>(&sKtl[32 * jh + x][16 * ks + 8 * g]);
                const bf16x8 bv = *reinterpret_cast<const bf16x8*>(&sVt[icol][16 * ks + 8 * g]);
                accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bv, accM, 0, 0, 0);
                accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bv, accM, 0, 0, 0);
                if (VSPLIT) {
                    const bf16x8 bvl = *reinterpret_cast<const bf16x8*>(&sVtl[icol][16 * ks + 8 * g]);
                    accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bvl, accM, 0, 0, 0);
                }
            }
            f32x16& S = jh == 0 ? S0 : S1;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const f32x4 c2 = *reinterpret_cast<const f32x4*>(&sC2[32 * jh + 8 * r4 + 4 * g]);
                const f32x4 c3 = *reinterpret_cast<const f32x4*>(&sC3[32 * jh + 8 * r4 + 4 * g]);
#pragma unroll
                for (int e = 0; e < 4; ++e) S[4 * r4 + e] = c2[e] * S[4 * r4 + e] + c3[e] * accM[4 * r4 + e];
            }
        }
        // ---- bonus (ascending pass) and store: lane = column i, register r = token 8(r/4)+4g+(r%4) ----
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int n0 = 8 * r4 + 4 * g;
            f32x4 bon = {0.f, 0.f, 0.f, 0.f};
            if (DIR == 0) {
                const f32x4 c = *reinterpret_cast<const f32x4*>(&sBonus[n0]);
                const bf16x4 vh = *reinterpret_cast<const bf16x4*>(&sVt[icol][n0]);
#pragma unroll
                for (int e = 0; e < 4; ++e) bon[e] = c[e] * (float)vh[e];
                if (VSPLIT) {
                    const bf16x4 vl = *reinterpret_cast<const bf16x4*>(&sVtl[icol][n0]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) bon[e] += c[e] * (float)vl[e];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int ng = ch * LC + n0 + e;
                if (ng < T) {
                    const int t = DIR == 0 ? ng : T - 1 - ng;
                    float* yp = y_ + base + (size_t)t * C + icol;
                    const float val = accY[4 * r4 + e] + bon[e];
                    if (DIR == 0) *yp += val; else *yp = val;
                }
            }
        }
        lds_barrier();                                                   // (3) LDS is rewritten by the next chunk
    }
    if (threadIdx.x == 0) todo[(size_t)DIR * gridDim.x + bh] = 0;
}

}  // namespace wkv6_detail
}  // namespace vrwkv
