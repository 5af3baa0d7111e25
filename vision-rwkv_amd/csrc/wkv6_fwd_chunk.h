// wkv6 forward, chunked matrix-core kernel for gfx950 (bf16 MFMA, fp32 accumulate).
//
// Bidirectional RWKV-6 scan of
// classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:6-97, evaluated as two
// passes (descending; ascending with the bonus u), each the same causal algorithm on its own
// token order n = 0..T-1:
//
//   y_n = sum_j r_n[j] ( u[j] k_n[j] v_n  +  sum_{m<n} (prod_{m<l<n} d_l[j]) k_m[j] v_m )
//
// One 256-thread workgroup per (b,h): waves 0,1 run the descending pass, waves 2,3 the ascending
// one, side by side and in lockstep (chunk step s of both passes between the same barriers).
// Chunks of 32 tokens.  With the in-chunk cumulative log-decay P_n = sum_{l<=n} log d_l
// (Pex_n = P_n - log d_n) and the mid-chunk reference Pref = P_15:
//   rt_n = r_n * exp(Pex_n - Pref),   kt_m = k_m * exp(Pref - P_m)      (rt_n . kt_m = decay for m<n)
//   A[n][m] = rt_n . kt_m  (m < n),  bonus_n = (r_n u) . k_n  (m = n, ascending pass), 0 otherwise -> MFMA 1
//   Y       = A V  +  rt (diag(e^Pref) S)                                 -> MFMA 2, 3
//   S'      = diag(e^P31) S + diag(e^(P31-Pref)) (kt^T V)                 -> MFMA 4
// S (64x64 fp32) never leaves the accumulator registers: each wave owns the 32 value columns of
// one half and feeds its S tiles straight back as the B operand of MFMA 3 (the contraction index
// is taken in the order the accumulator layout provides, and the A operand is read from LDS in
// that same order); likewise A goes from the accumulators of MFMA 1 into the A operand of MFMA 2.
//
// y: both passes walk the same chunk grid from opposite ends.  The pass that reaches a chunk at the
// earlier step stores, the other one adds at its (later) step, after the barrier that ends every step (at
// the middle chunk of an odd count the descending pass stores before that barrier and the ascending pass
// adds after it) -- y is never zero-filled, and there is no second launch.
//
// Precision: every operand that is computed rather than loaded (rt, kt, A, S) is split into a
// bf16 head and a bf16 tail and the products head*head + head*tail + tail*head are accumulated,
// which keeps the result within ~3e-5 of the fp32 recurrence (one bf16 rounding of any of them
// alone costs ~1e-2).  v is exact in bf16 for bf16 input and split in two for fp16 / fp32 input.
//
// Range: the factorisation needs |P31| <= 60 in every chunk (decay over 32 tokens no stronger
// than e^-60).  A (b,h) sequence with a chunk outside that range is redone from scratch by the same
// workgroup with the sequential-state recurrence.
#pragma once
#include "vrwkv_common.h"
#include "wkv6_fwd_scalar.h"
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
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
constexpr float LOG2_LOG2E = 0.5287663729448977f;     // log2(log2(e))
// two fp32 values rounded to bf16 in one register (a low, b high), and the halves widened back
__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
__device__ __forceinline__ float bf16_lo(unsigned w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(unsigned w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
__device__ __forceinline__ void st_bf16_pair(__bf16* lo, __bf16* hi, unsigned w) {
    *reinterpret_cast<unsigned short*>(lo) = (unsigned short)w;
    *reinterpret_cast<unsigned short*>(hi) = (unsigned short)(w >> 16);
}

// head/tail split of eight fp32 accumulator values into two packed bf16 operands (two values per conversion)
__device__ __forceinline__ void split8(const float (&x)[8], bf16x8& hi, bf16x8& lo) {
    u32x4 h, l;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const unsigned w = pack_bf16(x[2 * p], x[2 * p + 1]);
        h[p] = w;
        l[p] = pack_bf16(x[2 * p] - bf16_lo(w), x[2 * p + 1] - bf16_hi(w));
    }
    hi = __builtin_bit_cast(bf16x8, h);
    lo = __builtin_bit_cast(bf16x8, l);
}

// DPP move: lane reads `v` of the lane selected by CTRL (0 where there is none).
template <int CTRL>
__device__ __forceinline__ float dpp_get(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// 16 values per lane -> per 16-lane row, the row sums of all 16: lane l ends up with the sum over
// its row of value index 8*(l&1) + 4*((l>>1)&1) + 2*((l>>3)&1) + ((l>>2)&1).  Transposing butterfly:
// at each step a lane keeps one half of its values and hands the other half to its partner.
__device__ __forceinline__ float row_sums16(const float (&p)[16], int lane, int& index) {
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4, b3 = lane & 8;
    float a8[8], a4[4], a2[2];
#pragma unroll
    for (int i = 0; i < 8; ++i) a8[i] = (b0 ? p[8 + i] : p[i]) + dpp_get<0xB1>(b0 ? p[i] : p[8 + i]);     // quad_perm [1,0,3,2]
#pragma unroll
    for (int i = 0; i < 4; ++i) a4[i] = (b1 ? a8[4 + i] : a8[i]) + dpp_get<0x4E>(b1 ? a8[i] : a8[4 + i]); // quad_perm [2,3,0,1]
#pragma unroll
    for (int i = 0; i < 2; ++i) a2[i] = (b3 ? a4[2 + i] : a4[i]) + dpp_get<0x128>(b3 ? a4[i] : a4[2 + i]); // row_ror:8
    const float give = b2 ? a2[0] : a2[1];
    const float from_lo = dpp_get<0x114>(give), from_hi = dpp_get<0x104>(give);   // row_shr:4 (from l-4), row_shl:4 (from l+4)
    const float recv = b2 ? from_lo : from_hi;                            // both moves run with every lane active
    index = (b0 ? 8 : 0) + (b1 ? 4 : 0) + (b3 ? 2 : 0) + (b2 ? 1 : 0);
    return (b2 ? a2[1] : a2[0]) + recv;
}

// Per-pass LDS operands.  VSPLIT: v is given in a type that is not exact in bf16 (fp16, fp32) and is split in two.
template <bool VSPLIT>
struct __attribute__((aligned(16))) PassLds {
    __bf16 Rh[LC][PJ], Rl[LC][PJ], Kh[LC][PJ], Kl[LC][PJ];
    __bf16 Kth[HN][PS], Ktl[HN][PS], Vt[HN][PS], Vtl[VSPLIT ? HN : 1][PS];
    float C1[HN], C2[HN], C3[HN], Tot[HN], Bon[4][LC];
};

template <typename IO, typename WT, bool W_IS_EW>
__global__ __launch_bounds__(256, 2)
void wkv6_fwd_chunk_kernel(const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                           const WT* __restrict__ w_, const float* __restrict__ u_, float* __restrict__ y_,
                           int T, int C, int H)
{
    constexpr bool VSPLIT = !(sizeof(IO) == 2 && __is_same(IO, __hip_bfloat16));
    __shared__ PassLds<VSPLIT> lds[2];
    __shared__ int sFlag;
    static_assert(sizeof(PassLds<VSPLIT>) * 2 >= 4 * 2 * 3 * N * sizeof(float), "fallback staging must fit");

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = wave & 1;                      // token half in stage E, value half in stage M
    const bool asc = wave >= 2;                  // waves 2,3: ascending pass (with the bonus)
    PassLds<VSPLIT>& L = lds[asc ? 1 : 0];
    const int g = lane >> 5, x = lane & 31;
    const int bh = blockIdx.x;
    const int b = bh / H, h = bh % H;
    const size_t base = (size_t)b * T * C + (size_t)h * HN;
    const int nchunk = (T + LC - 1) / LC;
    const float uj = asc ? u_[h * HN + lane] : 0.f;
    if (threadIdx.x == 0) sFlag = 0;
    __syncthreads();

    f32x16 S0 = {0}, S1 = {0};          // state tiles: rows j = 32*jh + 8(r/4)+4g+(r%4), column i = 32q + x
    bool bail = false;

    // The decay rows of a chunk are fetched one step ahead (when the previous step enters its matrix stage),
    // so the cumulative decay can start at once; r, k, v follow at the top of the step and are needed only
    // after the first barrier.
    using RawIO = typename BufRaw<sizeof(IO)>::type;
    using RawW = typename BufRaw<sizeof(WT)>::type;
    // descriptors over this (b,h)'s 64-channel column block of the batch slab; token rows are C elements apart
    const unsigned span_io = (unsigned)(((size_t)(T - 1) * C + HN) * sizeof(IO));
    const unsigned span_w = (unsigned)(((size_t)(T - 1) * C + HN) * sizeof(WT));
    const __amdgpu_buffer_rsrc_t rsr = make_rsrc(r_ + base, span_io), rsk = make_rsrc(k_ + base, span_io),
                                 rsv = make_rsrc(v_ + base, span_io), rsw = make_rsrc(w_ + base, span_w),
                                 rsy = make_rsrc(y_ + base, (unsigned)(((size_t)(T - 1) * C + HN) * sizeof(float)));
    RawIO rraw[16], kraw[16], vraw[16];
    RawW wraw[16];
    // Both passes walk the same 32-token chunks of the token axis (the ascending pass chunk 0, 1, ..., the
    // descending pass chunk nchunk-1, ..., 0), so everything that depends on the position is wave-uniform.
    // Pass index n = 0..31 inside a chunk is token 32c + n (ascending) or 32c + 31 - n (descending); tokens
    // past T (only in the last chunk; for the descending pass they come first) read the last row and count as
    // k = 0, d = 1 (their own y rows are dropped by the store's range check).
    auto chunk_of = [&](int ch) { return asc ? ch : nchunk - 1 - ch; };
    const int sgn = asc ? 1 : -1, n0 = asc ? 0 : LC - 1;
    auto token_of = [&](int c, int n) { return c * LC + n0 + sgn * n; };
    // Row offsets walk the 16 tokens of this wave's block with one scalar add each; rows past T (last chunk
    // only) are clamped to the last row and switched off where they are used.
    auto fetch_w = [&](int ch, int C) {
        const unsigned step = (unsigned)(sgn * C * (int)sizeof(WT)), last = (unsigned)(T - 1) * C * (unsigned)sizeof(WT);
        unsigned so = (unsigned)token_of(chunk_of(ch), 16 * q) * C * (unsigned)sizeof(WT);
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            wraw[m] = BufRaw<sizeof(WT)>::ld(rsw, lane * (unsigned)sizeof(WT), so < last ? so : last);
            so += step;
        }
    };
    auto fetch_rkv = [&](int ch, int C) {
        const unsigned step = (unsigned)(sgn * C * (int)sizeof(IO)), last = (unsigned)(T - 1) * C * (unsigned)sizeof(IO);
        unsigned so = (unsigned)token_of(chunk_of(ch), 16 * q) * C * (unsigned)sizeof(IO);
        const unsigned vo = lane * (unsigned)sizeof(IO);
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            const unsigned sc = so < last ? so : last;
            rraw[m] = BufRaw<sizeof(IO)>::ld(rsr, vo, sc);
            kraw[m] = BufRaw<sizeof(IO)>::ld(rsk, vo, sc);
            vraw[m] = BufRaw<sizeof(IO)>::ld(rsv, vo, sc);
            so += step;
        }
    };
    auto cvt = [](RawIO raw) { IO t; __builtin_memcpy(&t, &raw, sizeof(t)); return to_f32(t); };
    auto cvtw = [](RawW raw) { WT t; __builtin_memcpy(&t, &raw, sizeof(t)); return to_f32(t); };
    // y[t][icol] of accumulator register r (pass index n = 8(r/4) + 4g + (r%4)): a per-lane byte offset plus a
    // wave-uniform one; rows past T fall outside the descriptor and are dropped by the hardware.
    const unsigned y_lane = (unsigned)(((asc ? 4 * g : 4 * (1 - g)) * C + 32 * q + x) * sizeof(float));
    const int y_n0 = asc ? 0 : 27;                                        // 8(3 - r/4) + (3 - r%4) = 27 - (8(r/4) + r%4)
    auto y_off = [&](int c, int r, int C) -> unsigned {
        return y_lane + (unsigned)((c * LC + y_n0) * C * 4) + (unsigned)((8 * (r / 4) + (r % 4)) * (sgn * C * 4));
    };
    fetch_w(0, C);
    // causal masks of the in-chunk matrix, one word per pair of accumulator registers (r = 2p low half, 2p + 1 high)
    unsigned keepw[8], diagw[8];
#pragma unroll
    for (int pr = 0; pr < 8; ++pr) {
        const int s0 = 8 * ((2 * pr) / 4) + 4 * g + ((2 * pr) % 4);     // row s of register 2p; register 2p + 1 holds s0 + 1
        keepw[pr] = (s0 < x ? 0xffffu : 0u) | (s0 + 1 < x ? 0xffff0000u : 0u);
        diagw[pr] = (s0 == x ? 0xffffu : 0u) | (s0 + 1 == x ? 0xffff0000u : 0u);
    }

    for (int ch = 0; ch < nchunk; ++ch) {
        // =============================== stage E: elementwise =================================
        // wave q of the pass prepares tokens n = 16q .. 16q+15 of the chunk; lane = channel j (and i for v)
        // Row offsets are recomputed per step from an opaque copy of C: hoisted out of the loop they would
        // occupy ~100 scalar registers and spill.
        int Cs = C;
        asm volatile("" : "+s"(Cs));
        fetch_rkv(ch, Cs);                                                   // used after the first barrier
        // log decays in log2 units: ld2 = -log2(e) exp(w) = -exp2(w log2(e) + log2(log2(e)))
        const bool full = (chunk_of(ch) + 1) * LC <= T;                  // wave-uniform: no token of the chunk is past T
        float p[16];
        {
            float e[16];
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                const float fw = cvtw(wraw[m]);
                e[m] = W_IS_EW ? -fw * LOG2E : fast_exp2(fmaf(fw, LOG2E, LOG2_LOG2E));
            }
            if (!full) {
#pragma unroll
                for (int m = 0; m < 16; ++m)
                    if (token_of(chunk_of(ch), 16 * q + m) >= T) e[m] = 0.f;
            }
            p[0] = -e[0];
#pragma unroll
            for (int m = 1; m < 16; ++m) p[m] = p[m - 1] - e[m];
        }
        if (q == 0) L.Tot[lane] = p[15];
        lds_barrier();                                                   // (1)
        const float pref = L.Tot[lane];                                  // P_15 (log2 units)
        const float dq = q == 1 ? 0.f : -pref;                           // z_m = P_m - Pref = p[m] + dq
        if (q == 1) {
            const float p31 = p[15] + pref;
            L.C2[lane] = fast_exp2(p31);
            L.C3[lane] = fast_exp2(p[15]);
            if (__builtin_amdgcn_ballot_w64(!(p31 >= -SAFE_DECAY * LOG2E)) != 0ull && lane == 0) sFlag = 1;
        } else {
            L.C1[lane] = fast_exp2(pref);
        }
        {
            if (!full) {                                                  // k = 0 switches a token past T off everywhere
#pragma unroll
                for (int m = 0; m < 16; ++m)
                    if (token_of(chunk_of(ch), 16 * q + m) >= T) kraw[m] = RawIO{};
            }
            unsigned kthw[8], ktlw[8], vthw[8], vtlw[8];
            float pu[16];
            float zp = dq;                                                // Pex_m - Pref = z_(m-1)
#pragma unroll
            for (int m = 0; m < 16; m += 2) {
                const int n = 16 * q + m;
                const float z0 = p[m] + dq, z1 = p[m + 1] + dq;
                const float f1a = fast_exp2(zp), f2a = fast_exp2(-z0);    // exp(Pex - Pref), exp(Pref - P)
                const float f1b = fast_exp2(z0), f2b = fast_exp2(-z1);
                zp = z1;
                const float r0 = cvt(rraw[m]), r1 = cvt(rraw[m + 1]), k0 = cvt(kraw[m]), k1 = cvt(kraw[m + 1]);
                const float rt0 = r0 * f1a, rt1 = r1 * f1b, kt0 = k0 * f2a, kt1 = k1 * f2b;
                const unsigned rh = pack_bf16(rt0, rt1), kh = pack_bf16(kt0, kt1);    // token m low, m + 1 high
                const unsigned rl = pack_bf16(rt0 - bf16_lo(rh), rt1 - bf16_hi(rh));
                const unsigned kl = pack_bf16(kt0 - bf16_lo(kh), kt1 - bf16_hi(kh));
                st_bf16_pair(&L.Rh[n][lane], &L.Rh[n + 1][lane], rh);
                st_bf16_pair(&L.Rl[n][lane], &L.Rl[n + 1][lane], rl);
                st_bf16_pair(&L.Kh[n][lane], &L.Kh[n + 1][lane], kh);
                st_bf16_pair(&L.Kl[n][lane], &L.Kl[n + 1][lane], kl);
                kthw[m >> 1] = kh;
                ktlw[m >> 1] = kl;
                if constexpr (!VSPLIT) {
                    vthw[m >> 1] = (unsigned)vraw[m] | ((unsigned)vraw[m + 1] << 16);   // bf16 bits as loaded
                } else {
                    const float v0 = cvt(vraw[m]), v1 = cvt(vraw[m + 1]);
                    const unsigned vh = pack_bf16(v0, v1);
                    vthw[m >> 1] = vh;
                    vtlw[m >> 1] = pack_bf16(v0 - bf16_lo(vh), v1 - bf16_hi(vh));
                }
                pu[m] = r0 * uj * k0;
                pu[m + 1] = r1 * uj * k1;
            }
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<u32x4*>(&L.Kth[lane][16 * q + 8 * e]) = u32x4{kthw[4 * e], kthw[4 * e + 1], kthw[4 * e + 2], kthw[4 * e + 3]};
                *reinterpret_cast<u32x4*>(&L.Ktl[lane][16 * q + 8 * e]) = u32x4{ktlw[4 * e], ktlw[4 * e + 1], ktlw[4 * e + 2], ktlw[4 * e + 3]};
                *reinterpret_cast<u32x4*>(&L.Vt[lane][16 * q + 8 * e]) = u32x4{vthw[4 * e], vthw[4 * e + 1], vthw[4 * e + 2], vthw[4 * e + 3]};
                if constexpr (VSPLIT)
                    *reinterpret_cast<u32x4*>(&L.Vtl[lane][16 * q + 8 * e]) = u32x4{vtlw[4 * e], vtlw[4 * e + 1], vtlw[4 * e + 2], vtlw[4 * e + 3]};
            }
            if (asc) {                                                    // bonus_n = sum_j r_n[j] u[j] k_n[j]
                int idx;
                const float rs = row_sums16(pu, lane, idx);
                L.Bon[lane >> 4][16 * q + idx] = rs;                      // the four 16-channel rows are added by the reader
            }
        }
        lds_barrier();                                                   // (2)
        if (sFlag) { bail = true; break; }                               // out of range: redo with the exact recurrence

        if (ch + 1 < nchunk) fetch_w(ch + 1, Cs);                             // next chunk's decays, behind the matrix stage

        // ================================= stage M: matrix cores ===============================
        const int icol = 32 * q + x;                                      // value column of this lane
        // y: the other pass reaches this chunk at step nchunk-1-ch.  If that was earlier, its values are in
        // memory already (made visible by that step's closing barrier): fetch them now, behind the MFMAs.
        const int cy = chunk_of(ch);
        const bool y_second = ch > nchunk - 1 - ch, y_tie = asc && ch == nchunk - 1 - ch;     // wave-uniform
        float prev[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) prev[r] = 0.f;
        if (y_second) {
#pragma unroll
            for (int r = 0; r < 16; ++r) prev[r] = __builtin_bit_cast(float, BufRaw<4>::ld(rsy, y_off(cy, r, Cs), 0));
        }
        // ---- MFMA 1: A^T: acc[m = s][n = t]; lane holds t = x, rows s = 8(r/4)+4g+(r%4) ----
        f32x16 accA = {0};
#pragma unroll
        for (int kq = 0; kq < 4; ++kq) {
            const bf16x8 ah = *reinterpret_cast<const bf16x8*>(&L.Kh[x][16 * kq + 8 * g]);
            const bf16x8 al = *reinterpret_cast<const bf16x8*>(&L.Kl[x][16 * kq + 8 * g]);
            const bf16x8 bh_ = *reinterpret_cast<const bf16x8*>(&L.Rh[x][16 * kq + 8 * g]);
            const bf16x8 bl = *reinterpret_cast<const bf16x8*>(&L.Rl[x][16 * kq + 8 * g]);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh_, accA, 0, 0, 0);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, accA, 0, 0, 0);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh_, accA, 0, 0, 0);
        }
        // A[t][s] keeps s < t and takes the bonus at s = t: applied to the packed bf16 words with the lane's
        // constant bit masks (the lane holds t = x, rows s = 8(r/4) + 4g + (r%4))
        const float diag = asc ? (L.Bon[0][x] + L.Bon[1][x]) + (L.Bon[2][x] + L.Bon[3][x]) : 0.f;
        const unsigned dgh = pack_bf16(diag, diag), dgl = pack_bf16(diag - bf16_lo(dgh), diag - bf16_lo(dgh));
        bf16x8 Ah[2], Al[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            float a8[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) a8[e] = accA[8 * ks + e];
            bf16x8 h8, l8;
            split8(a8, h8, l8);
            u32x4 hw = __builtin_bit_cast(u32x4, h8), lw = __builtin_bit_cast(u32x4, l8);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                hw[p] = (hw[p] & keepw[4 * ks + p]) | (dgh & diagw[4 * ks + p]);
                lw[p] = (lw[p] & keepw[4 * ks + p]) | (dgl & diagw[4 * ks + p]);
            }
            Ah[ks] = __builtin_bit_cast(bf16x8, hw);
            Al[ks] = __builtin_bit_cast(bf16x8, lw);
        }
        // ---- MFMA 2: Y[t][i] = sum_s A[t][s] V[s][i]; contraction order = accumulator order ----
        f32x16 accY = {0};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bf16x8 bv = cat8(*reinterpret_cast<const bf16x4*>(&L.Vt[icol][16 * ks + 4 * g]),
                                   *reinterpret_cast<const bf16x4*>(&L.Vt[icol][16 * ks + 8 + 4 * g]));
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ah[ks], bv, accY, 0, 0, 0);
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Al[ks], bv, accY, 0, 0, 0);
            if (VSPLIT) {
                const bf16x8 bvl = cat8(*reinterpret_cast<const bf16x4*>(&L.Vtl[icol][16 * ks + 4 * g]),
                                        *reinterpret_cast<const bf16x4*>(&L.Vtl[icol][16 * ks + 8 + 4 * g]));
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
                    const f32x4 c1 = *reinterpret_cast<const f32x4*>(&L.C1[32 * jh + 16 * ks + 8 * e4 + 4 * g]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) s8[4 * e4 + e] = S[8 * ks + 4 * e4 + e] * c1[e];
                }
                bf16x8 sh, sl;
                split8(s8, sh, sl);
                const int j0 = 32 * jh + 16 * ks + 4 * g;
                const bf16x8 ah = cat8(*reinterpret_cast<const bf16x4*>(&L.Rh[x][j0]),
                                       *reinterpret_cast<const bf16x4*>(&L.Rh[x][j0 + 8]));
                const bf16x8 al = cat8(*reinterpret_cast<const bf16x4*>(&L.Rl[x][j0]),
                                       *reinterpret_cast<const bf16x4*>(&L.Rl[x][j0 + 8]));
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
                const bf16x8 ah = *reinterpret_cast<const bf16x8*>(&L.Kth[32 * jh + x][16 * ks + 8 * g]);
                const bf16x8 al = *reinterpret_cast<const bf16x8*>(&L.Ktl[32 * jh + x][16 * ks + 8 * g]);
                const bf16x8 bv = *reinterpret_cast<const bf16x8*>(&L.Vt[icol][16 * ks + 8 * g]);
                accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bv, accM, 0, 0, 0);
                accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bv, accM, 0, 0, 0);
                if (VSPLIT) {
                    const bf16x8 bvl = *reinterpret_cast<const bf16x8*>(&L.Vtl[icol][16 * ks + 8 * g]);
                    accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bvl, accM, 0, 0, 0);
                }
            }
            f32x16& S = jh == 0 ? S0 : S1;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const f32x4 c2 = *reinterpret_cast<const f32x4*>(&L.C2[32 * jh + 8 * r4 + 4 * g]);
                const f32x4 c3 = *reinterpret_cast<const f32x4*>(&L.C3[32 * jh + 8 * r4 + 4 * g]);
#pragma unroll
                for (int e = 0; e < 4; ++e) S[4 * r4 + e] = c2[e] * S[4 * r4 + e] + c3[e] * accM[4 * r4 + e];
            }
        }
        // ---- y: store (sum with the other pass's value where it came first); on a tie the descending pass
        //      stores here and the ascending pass adds after the barrier ----
        if (!y_tie) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                BufRaw<4>::st(__builtin_bit_cast(unsigned, prev[r] + accY[r]), rsy, y_off(cy, r, Cs), 0);
        }
        // end of the step: every LDS read of this chunk is done, and the stores above become visible
        // to the other pass of this workgroup
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();                                    // (3)
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (y_tie) {
#pragma unroll
            for (int r = 0; r < 16; ++r) prev[r] = __builtin_bit_cast(float, BufRaw<4>::ld(rsy, y_off(cy, r, Cs), 0));
#pragma unroll
            for (int r = 0; r < 16; ++r)
                BufRaw<4>::st(__builtin_bit_cast(unsigned, prev[r] + accY[r]), rsy, y_off(cy, r, Cs), 0);
        }
    }

    if (bail) {
        // Some chunk decays faster than the factorisation can represent: recompute the whole sequence
        // with the sequential recurrence (it rewrites every y of this (b,h)).
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        float* stage = reinterpret_cast<float*>(&lds[0]);
        wkv6_scalar_pass<IO, WT, 1, W_IS_EW>(r_, k_, v_, w_, u_, y_, stage, bh, T, C, H);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        wkv6_scalar_pass<IO, WT, 0, W_IS_EW>(r_, k_, v_, w_, u_, y_, stage, bh, T, C, H);
    }
}

}  // namespace wkv6_detail
}  // namespace vrwkv
