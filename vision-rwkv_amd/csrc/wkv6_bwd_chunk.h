// wkv6 backward, chunked matrix-core scans for gfx950 (bf16 MFMA, fp32 accumulate; r, k, v in bf16, fp16 or fp32).
//
// One causal pass of the forward (tokens in pass order n, state S_n before token n, d_n = exp(ld_n)):
//   y_n = r_n (diag(u) k_n v_n^T + S_n),   S_{n+1} = diag(d_n) S_n + k_n v_n^T
// and its adjoint state G_n = r_n gy_n^T + diag(d_n) G_{n+1} give
//   gr_n[j] = u_j k_n[j] (v_n.gy_n) + (S_n gy_n)[j]            scan GR  (pass order,     state S^T[i][j])
//   gk_n[j] = u_j r_n[j] (v_n.gy_n) + (G_{n+1} v_n)[j]         scan GK  (reverse order,  state G^T[i][j])
//   gv_n[i] = sum_j k_n[j] (u_j r_n[j] gy_n[i] + G_{n+1}[j,i]) scan GV  (reverse order,  state G[j][i])
//   gw_n[j] = ld_n[j] ( sum_{m>n} (a_m - b_m) - b_n ),  a = r (S gy),  b = k (G v)   (GR stores a, GK finishes gw)
// (formulas of classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:99-346).
//
// Every scan is the same chunked algorithm as the forward kernel, on 32-token chunks, with other operands.
// In scan order rho (the pass order or its reverse) and with c the contracted channel, o the output channel:
//   A[t][s]   = sum_c Q[t][c] Kc[s][c]   (s before t in scan order; the bonus on the diagonal for GV)
//   Out[t][o] = sum_s A[t][s] Val[s][o]  +  sum_c Q[t][c] (state, rescaled)[c][o]
//   state'    = decay * state + scale * sum_s Kc[s][c] Val[s][o]
// With P the in-chunk cumulative log decay in PASS order, Pex = P - ld, Pref = P_15, f1 = e^(Pex-Pref),
// f2 = e^(Pref-P), rt = r f1, kt = k f2, c1 = e^Pref, c2 = e^P31, c3 = e^(P31-Pref):
//   GR: Q = gy, Kc = v,  Val = kt, state read * c1[j], update c2[j], c3[j];  gr = f1 Out + u k A[t][t], a = r f1 Out
//   GK: Q = v,  Kc = gy, Val = rt, state read * c3[j], update c2[j], c1[j];  gk = f2 Out + u r A[t][t], b = k f2 Out
//   GV: Q = kt, Kc = rt, Val = gy, state read * c3[j] (rows), update c2[j], c1[j] (rows);  gv = Out
// GR and GK contract over the value channel i and own output columns j (the state is kept transposed, so its
// decay is a per-lane factor); GV contracts over j like the forward.  The state never leaves the accumulator
// registers; computed operands (and fp16 / fp32 inputs) are split into bf16 head + tail (hh + ht + th), loaded
// bf16 ones are exact.
//
// One 128-thread workgroup per (b,h) and pass; the descending pass is launched first and writes, the
// ascending pass adds (put_f32).  A sequence with a chunk that decays by
// more than e^-60 is flagged in `todo` and left to the sequential kernels: the first scan launched (gr, descending)
// clears its sequence's flag on entry and a scan only ever sets one, so a sequence that any of the six scans gave
// up on is redone.
#pragma once
#include "wkv6_chunk_common.h"

namespace vrwkv {
namespace wkv6_detail {

enum { SCAN_GR = 0, SCAN_GK = 1, SCAN_GV = 2 };


// One fp32 result of a scan: the descending pass (launched first) stores it, the ascending pass adds its own.  The
// gr and gv scans fetch the old values behind their matrix stage and store the sums; the gk / gw scan has no registers
// left for that: it fetches the old gk rows just before its epilogue and adds gw with a no-return atomic at the L2
// (every address is touched once per pass, so the sum does not depend on any order).  Measured at 64 x 196 x 768: an
// atomic costs about 1.2 us per million, a read-modify-write whose loads are hidden about a quarter of that.  Rows past
// T fall to the descriptor's range check either way.
template <bool ADD>
__device__ __forceinline__ void put_f32(float val, __amdgpu_buffer_rsrc_t r, unsigned voff) {
    if (ADD) (void)__builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(val, r, voff, 0, 0);
    else {
        unsigned bits;
        __builtin_memcpy(&bits, &val, 4);
        BufRaw<4>::st(bits, r, voff, 0);
    }
}

template <bool QS, bool KS, bool GW>
struct __attribute__((aligned(16))) ScanLds {
    __bf16 Qh[LC][PJ], Ql[QS ? LC : 1][PJ];               // Q rows   [rho][c]
    __bf16 Kh[LC][PJ], Kl[KS ? LC : 1][PJ];               // Kc rows  [rho][c]
    __bf16 KTh[HN][PS], KTl[KS ? HN : 1][PS];             // Kc^T     [c][rho]
    __bf16 VTh[HN][PS], VTl[HN][PS];                      // Val^T    [o][rho]
    float Post[LC][HN];                                   // f1 / f2 in [rho][j]  (GR, GK)
    float Ld[GW ? LC : 1][HN];                            // -log2 of the decay in [rho][j]  (GK: the factor of gw)
    float C1[HN], C2[HN], C3[HN], Tot[HN], Bon[4][LC], Diag[LC];
};

// DIR 0: ascending pass (bonus u, adds to the outputs).  DIR 1: descending pass (writes them).
template <typename IO, typename WT, int KIND, int DIR, bool W_IS_EW>
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(2, 2)))
void wkv6_bwd_scan_kernel(const IO* __restrict__ r_, const IO* __restrict__ k_,
                          const IO* __restrict__ v_, const WT* __restrict__ w_,
                          const float* __restrict__ u_, const float* __restrict__ gy_,
                          float* __restrict__ out_,        // gr / gk / gv
                          float* __restrict__ a_,          // GR: written; GK: read
                          float* __restrict__ gw_,         // GK
                          float* __restrict__ gu_part,     // GR, DIR 0
                          unsigned char* __restrict__ todo, int T, int C, int H)
{
    constexpr bool EXACT = __is_same(IO, __hip_bfloat16);  // r, k, v are bf16 values as loaded (fp16 / fp32 inputs are split in two)
    constexpr unsigned ES = (unsigned)sizeof(IO);
    constexpr bool REV = KIND != SCAN_GR;                  // scan order = reverse pass order
    constexpr bool TT = KIND != SCAN_GV;                   // transposed state: contraction over i, output columns j
    constexpr bool QS = KIND != SCAN_GK || !EXACT;         // Q is computed (gy, kt) -> split; bf16 v is exact
    constexpr bool KS = KIND != SCAN_GR || !EXACT;         // Kc is computed (gy, rt) -> split; bf16 v is exact
    constexpr bool ASC = DIR == 0;
    constexpr bool LL = KIND != SCAN_GV;                   // tail x tail products too: gw is a difference of these sums
    __shared__ ScanLds<QS, KS, KIND == SCAN_GK> L;
    __shared__ int sFlag;

    const int lane = threadIdx.x & 63;
    const int q = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = q;                                    // name used by the timing hook
    (void)wave;
    const int g = lane >> 5, x = lane & 31;
    const int bh = blockIdx.x;
    const int b = bh / H, h = bh % H;
    const size_t base = (size_t)b * T * C + (size_t)h * HN;
    const int nchunk = (T + LC - 1) / LC;
    const int ocol = 32 * q + x;                           // output column of this lane in the matrix stage
    const float u_e = ASC ? u_[h * HN + lane] : 0.f;       // bonus weight of the elementwise stage's channel
    const float u_o = ASC ? u_[h * HN + ocol] : 0.f;       // ... and of the output column (GR, GK)
    if (threadIdx.x == 0) {
        sFlag = 0;
        // the scan that is launched first clears the sequence's fallback flag; a scan only ever sets it afterwards
        if (KIND == SCAN_GR && DIR == 1) todo[bh] = 0;
    }
    __syncthreads();

    using RawIO = typename BufRaw<sizeof(IO)>::type;
    using RawW = typename BufRaw<sizeof(WT)>::type;
    const unsigned span_io = (unsigned)(((size_t)(T - 1) * C + HN) * ES);
    const unsigned span_w = (unsigned)(((size_t)(T - 1) * C + HN) * sizeof(WT));
    const unsigned span_f = (unsigned)(((size_t)(T - 1) * C + HN) * 4);
    const __amdgpu_buffer_rsrc_t rsr = make_rsrc(r_ + base, span_io), rsk = make_rsrc(k_ + base, span_io),
                                 rsv = make_rsrc(v_ + base, span_io), rsw = make_rsrc(w_ + base, span_w),
                                 rsg = make_rsrc(gy_ + base, span_f), rso = make_rsrc(out_ + base, span_f);
    const __amdgpu_buffer_rsrc_t rsa = make_rsrc((KIND != SCAN_GV ? a_ : out_) + base, span_f);
    const __amdgpu_buffer_rsrc_t rsgw = make_rsrc((KIND == SCAN_GK ? gw_ : out_) + base, span_f);
    auto cvt = [](RawIO raw) { IO t; __builtin_memcpy(&t, &raw, sizeof(t)); return to_f32(t); };
    auto cvtw = [](RawW raw) { WT t; __builtin_memcpy(&t, &raw, sizeof(t)); return to_f32(t); };

    // Chunks are 32-token blocks of the token axis.  The scan walks them upwards when (ascending pass) !=
    // (reversed scan), downwards otherwise; pass index n inside a chunk is token 32c + n (ascending pass) or
    // 32c + 31 - n (descending); scan row rho = n, or 31 - n for a reversed scan.
    constexpr bool UP = ASC != REV;
    auto chunk_of = [&](int ch) { return UP ? ch : nchunk - 1 - ch; };
    auto token_of_n = [&](int c, int n) { return c * LC + (ASC ? n : LC - 1 - n); };
    // matrix-stage register r of a lane <-> scan row rho = 8(r/4) + 4g + (r%4) <-> token 32c + (UP ? rho : 31-rho)
    const unsigned o_lane = (unsigned)(((UP ? 4 * g : 4 * (1 - g)) * C + ocol) * 4);
    auto row_off = [&](int c, int r, int C, int esz) -> unsigned {   // byte offset of (token of register r, column ocol)
        const int rl = 8 * (r / 4) + (r % 4);
        return (o_lane / 4) * esz + (unsigned)((c * LC + (UP ? rl : 27 - rl)) * C * esz);
    };

    f32x16 S0 = {0}, S1 = {0};      // state tiles: rows c = 32*ch2 + 8(r/4)+4g+(r%4), column o = ocol
    float xcarry = 0.f, gu_acc = 0.f;   // GK: sum of (a - b) over the tokens scanned so far; GR: gu
    RawW wraw[16];
    // Row offsets walk the 16 tokens of this wave's block with one scalar add each; rows past T (last chunk only)
    // are clamped to the last row and switched off where they are used.
    const int sgn = ASC ? 1 : -1;
    auto fetch_w = [&](int ch, int C) {
        const unsigned step = (unsigned)(sgn * C * (int)sizeof(WT)), last = (unsigned)(T - 1) * C * (unsigned)sizeof(WT);
        unsigned so = (unsigned)token_of_n(chunk_of(ch), 16 * q) * C * (unsigned)sizeof(WT);
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            wraw[m] = BufRaw<sizeof(WT)>::ld(rsw, lane * (unsigned)sizeof(WT), so < last ? so : last);
            so += step;
        }
    };
    fetch_w(0, C);
    // causal masks of the in-chunk matrix, one word per pair of accumulator registers (r = 2p low half, 2p + 1 high):
    // the lane holds column t = x and rows s = 8(r/4) + 4g + (r%4).  The GK scans have no registers to spare for
    // them and mask with compares instead.
    constexpr bool MASK_REGS = KIND != SCAN_GK;
    unsigned keepw[8], diagw[8];
    if (MASK_REGS) {
#pragma unroll
        for (int pr = 0; pr < 8; ++pr) {
            const int s0 = 8 * ((2 * pr) / 4) + 4 * g + ((2 * pr) % 4);
            keepw[pr] = (s0 < x ? 0xffffu : 0u) | (s0 + 1 < x ? 0xffff0000u : 0u);
            diagw[pr] = (s0 == x ? 0xffffu : 0u) | (s0 + 1 == x ? 0xffff0000u : 0u);
        }
    }

    for (int ch = 0; ch < nchunk; ++ch) {
        int Cs = C;
        asm volatile("" : "+s"(Cs));                       // keep row offsets out of the loop-invariant scalars
        const int cc = chunk_of(ch);
        // =============================== stage E: elementwise =================================
        // wave q prepares pass indices n = 16q .. 16q+15 of the chunk; lane = channel
        RawIO xraw[16], yraw[16];                          // the two bf16 tensors this scan needs here
        unsigned graw[16];                                 // gy (fp32 bits)
        {
            const unsigned last = (unsigned)(T - 1) * Cs;
            unsigned so = (unsigned)token_of_n(cc, 16 * q) * Cs;          // element offset of the row
            const unsigned step = (unsigned)(sgn * Cs);
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                const unsigned sc = so < last ? so : last;
                const unsigned vo = lane * ES;
                if (KIND == SCAN_GR) { xraw[m] = BufRaw<ES>::ld(rsv, vo, sc * ES); yraw[m] = BufRaw<ES>::ld(rsk, vo, sc * ES); }
                if (KIND == SCAN_GK) { xraw[m] = BufRaw<ES>::ld(rsv, vo, sc * ES); yraw[m] = BufRaw<ES>::ld(rsr, vo, sc * ES); }
                if (KIND == SCAN_GV) { xraw[m] = BufRaw<ES>::ld(rsk, vo, sc * ES); yraw[m] = BufRaw<ES>::ld(rsr, vo, sc * ES); }
                graw[m] = BufRaw<4>::ld(rsg, lane * 4u, sc * 4u);
                so += step;
            }
        }
        // log decays in log2 units: ld2 = -log2(e) exp(w) = -exp2(w log2(e) + log2(log2(e)))
        const bool full = (cc + 1) * LC <= T;                             // wave-uniform: no token of the chunk is past T
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
                    if (token_of_n(cc, 16 * q + m) >= T) e[m] = 0.f;
            }
            if (KIND == SCAN_GK) {                                        // scan row of pass index 16q + m: 16(1-q) + 15 - m
#pragma unroll
                for (int m = 0; m < 16; ++m) L.Ld[16 * (1 - q) + 15 - m][lane] = e[m];
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
            if (!full) {
                // a token past T is switched off through the one operand every product of this scan contains
                // (k for GR, r for GK and GV); its own output rows are dropped by the stores
#pragma unroll
                for (int m = 0; m < 16; ++m)
                    if (token_of_n(cc, 16 * q + m) >= T) yraw[m] = RawIO{};
            }
            unsigned kthw[8], ktlw[8], vthw[8], vtlw[8];
            float pu[16];
            const int r0 = REV ? 16 * (1 - q) : 16 * q;                   // first scan row of this wave's block
            float zp = dq;                                                // Pex_m - Pref = z_(m-1)
#pragma unroll
            for (int m = 0; m < 16; m += 2) {
                const float z0 = p[m] + dq, z1 = p[m + 1] + dq;
                const float f1a = fast_exp2(zp), f2a = fast_exp2(-z0);    // exp(Pex - Pref), exp(Pref - P)
                const float f1b = fast_exp2(z0), f2b = fast_exp2(-z1);
                zp = z1;
                // tokens (lo, hi) of a packed word: scan rows rho_lo (even position e) and rho_lo + 1
                const int e_lo = REV ? 14 - m : m;                        // position inside this wave's 16 scan rows
                const int rho_lo = r0 + e_lo, rho_hi = rho_lo + 1;
                const int m_lo = REV ? m + 1 : m, m_hi = REV ? m : m + 1;
                const float f1_lo = REV ? f1b : f1a, f1_hi = REV ? f1a : f1b;
                const float f2_lo = REV ? f2b : f2a, f2_hi = REV ? f2a : f2b;
                const float xa_lo = cvt(xraw[m_lo]), xa_hi = cvt(xraw[m_hi]);
                const float ya_lo = cvt(yraw[m_lo]), ya_hi = cvt(yraw[m_hi]);
                const float gy_lo = __builtin_bit_cast(float, graw[m_lo]), gy_hi = __builtin_bit_cast(float, graw[m_hi]);
                unsigned xbits = 0u;                                      // bf16 pair as loaded
                if constexpr (EXACT) xbits = (unsigned)xraw[m_lo] | ((unsigned)xraw[m_hi] << 16);
                // per scan: Q, Kc, Val of this (token, channel); exact bf16 inputs keep their bits
                float q_lo, q_hi, k_lo, k_hi, v_lo, v_hi;
                if (KIND == SCAN_GR) { q_lo = gy_lo; q_hi = gy_hi; k_lo = xa_lo; k_hi = xa_hi; v_lo = ya_lo * f2_lo; v_hi = ya_hi * f2_hi;
                                       L.Post[rho_lo][lane] = f1_lo; L.Post[rho_hi][lane] = f1_hi; }
                if (KIND == SCAN_GK) { q_lo = xa_lo; q_hi = xa_hi; k_lo = gy_lo; k_hi = gy_hi; v_lo = ya_lo * f1_lo; v_hi = ya_hi * f1_hi;
                                       L.Post[rho_lo][lane] = f2_lo; L.Post[rho_hi][lane] = f2_hi; }
                if (KIND == SCAN_GV) { q_lo = xa_lo * f2_lo; q_hi = xa_hi * f2_hi; k_lo = ya_lo * f1_lo; k_hi = ya_hi * f1_hi;
                                       v_lo = gy_lo; v_hi = gy_hi;
                                       pu[m_lo] = ya_lo * u_e * xa_lo; pu[m_hi] = ya_hi * u_e * xa_hi; }
                if (QS) {
                    const unsigned qh = pack_bf16(q_lo, q_hi);
                    st_bf16_pair(&L.Qh[rho_lo][lane], &L.Qh[rho_hi][lane], qh);
                    st_bf16_pair(&L.Ql[rho_lo][lane], &L.Ql[rho_hi][lane], pack_bf16(q_lo - bf16_lo(qh), q_hi - bf16_hi(qh)));
                } else {
                    st_bf16_pair(&L.Qh[rho_lo][lane], &L.Qh[rho_hi][lane], xbits);
                }
                if (KS) {
                    const unsigned kh = pack_bf16(k_lo, k_hi);
                    const unsigned kl = pack_bf16(k_lo - bf16_lo(kh), k_hi - bf16_hi(kh));
                    st_bf16_pair(&L.Kh[rho_lo][lane], &L.Kh[rho_hi][lane], kh);
                    st_bf16_pair(&L.Kl[rho_lo][lane], &L.Kl[rho_hi][lane], kl);
                    kthw[e_lo >> 1] = kh;
                    ktlw[e_lo >> 1] = kl;
                } else {
                    st_bf16_pair(&L.Kh[rho_lo][lane], &L.Kh[rho_hi][lane], xbits);
                    kthw[e_lo >> 1] = xbits;
                }
                const unsigned vh = pack_bf16(v_lo, v_hi);
                vthw[e_lo >> 1] = vh;
                vtlw[e_lo >> 1] = pack_bf16(v_lo - bf16_lo(vh), v_hi - bf16_hi(vh));
            }
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                *reinterpret_cast<u32x4*>(&L.KTh[lane][r0 + 8 * e]) = u32x4{kthw[4 * e], kthw[4 * e + 1], kthw[4 * e + 2], kthw[4 * e + 3]};
                if (KS) *reinterpret_cast<u32x4*>(&L.KTl[lane][r0 + 8 * e]) = u32x4{ktlw[4 * e], ktlw[4 * e + 1], ktlw[4 * e + 2], ktlw[4 * e + 3]};
                *reinterpret_cast<u32x4*>(&L.VTh[lane][r0 + 8 * e]) = u32x4{vthw[4 * e], vthw[4 * e + 1], vthw[4 * e + 2], vthw[4 * e + 3]};
                *reinterpret_cast<u32x4*>(&L.VTl[lane][r0 + 8 * e]) = u32x4{vtlw[4 * e], vtlw[4 * e + 1], vtlw[4 * e + 2], vtlw[4 * e + 3]};
            }
            if (KIND == SCAN_GV && ASC) {                                 // bonus_n = sum_j r_n[j] u[j] k_n[j]
                int idx;
                const float rs = row_sums16(pu, lane, idx);
                L.Bon[lane >> 4][r0 + (REV ? 15 - idx : idx)] = rs;
            }
        }
        lds_barrier();                                                   // (2)
        if (sFlag) {                                                      // out of range: left to the sequential kernels
            if (threadIdx.x == 0) todo[bh] = 1;
            return;
        }
        if (ch + 1 < nchunk) fetch_w(ch + 1, Cs);                         // next chunk's decays, behind the matrix stage

        // ================================= stage M: matrix cores ===============================
        // values the epilogue needs in the output layout (lane = column ocol, register r = scan row)
        constexpr bool RMW = ASC && KIND != SCAN_GK;      // ascending gr / gv: old values fetched here, sums stored
        constexpr bool GK_RMW = ASC && KIND == SCAN_GK;   // ascending gk: old values fetched just before the epilogue
        float prev[16];
        RawIO rraw[16], kraw[16];
        unsigned araw[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            prev[r] = RMW ? __builtin_bit_cast(float, BufRaw<4>::ld(rso, row_off(cc, r, Cs, 4), 0)) : 0.f;
            // the bonus terms (u k for gr, u r for gk) exist in the ascending pass only
            if (KIND == SCAN_GR || (KIND == SCAN_GK && ASC)) rraw[r] = BufRaw<ES>::ld(rsr, row_off(cc, r, Cs, ES), 0);
            else rraw[r] = RawIO{};
            if (KIND == SCAN_GK || (KIND == SCAN_GR && ASC)) kraw[r] = BufRaw<ES>::ld(rsk, row_off(cc, r, Cs, ES), 0);
            else kraw[r] = RawIO{};
        }
        // ---- MFMA 1: A^T: acc[s][t] = sum_c Kc[s][c] Q[t][c]; lane holds t = x, rows s = 8(r/4)+4g+(r%4) ----
        f32x16 accA = {0};
#pragma unroll
        for (int kq = 0; kq < 4; ++kq) {
            const bf16x8 ah = *reinterpret_cast<const bf16x8*>(&L.Kh[x][16 * kq + 8 * g]);
            const bf16x8 bh_ = *reinterpret_cast<const bf16x8*>(&L.Qh[x][16 * kq + 8 * g]);
            accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh_, accA, 0, 0, 0);
            if (QS) {
                const bf16x8 bl = *reinterpret_cast<const bf16x8*>(&L.Ql[x][16 * kq + 8 * g]);
                accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, accA, 0, 0, 0);
            }
            if (KS) {
                const bf16x8 al = *reinterpret_cast<const bf16x8*>(&L.Kl[x][16 * kq + 8 * g]);
                accA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh_, accA, 0, 0, 0);
            }
        }
        // A[t][s] keeps s before t and takes the bonus at s = t (GV); GR and GK pick A[t][t] = v_t . gy_t up on the
        // way.  All on the packed bf16 words with the lane's constant bit masks.
        const float bon = (KIND == SCAN_GV && ASC) ? (L.Bon[0][x] + L.Bon[1][x]) + (L.Bon[2][x] + L.Bon[3][x]) : 0.f;
        const unsigned dgh = pack_bf16(bon, bon), dgl = pack_bf16(bon - bf16_lo(dgh), bon - bf16_lo(dgh));
        bf16x8 Ah[2], Al[2];
        if (MASK_REGS) {
            unsigned dh = 0u, dl = 0u;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float a8[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) a8[e] = accA[8 * ks + e];
                bf16x8 h8, l8;
                split8(a8, h8, l8);
                u32x4 hw = __builtin_bit_cast(u32x4, h8), lw = __builtin_bit_cast(u32x4, l8);
#pragma unroll
                for (int pr = 0; pr < 4; ++pr) {
                    const unsigned kw = keepw[4 * ks + pr], dw = diagw[4 * ks + pr];
                    if (KIND != SCAN_GV) {
                        dh |= hw[pr] & dw;
                        dl |= lw[pr] & dw;
                        hw[pr] &= kw;
                        lw[pr] &= kw;
                    } else if (ASC) {
                        hw[pr] = (hw[pr] & kw) | (dgh & dw);
                        lw[pr] = (lw[pr] & kw) | (dgl & dw);
                    } else {
                        hw[pr] &= kw;
                        lw[pr] &= kw;
                    }
                }
                Ah[ks] = __builtin_bit_cast(bf16x8, hw);
                Al[ks] = __builtin_bit_cast(bf16x8, lw);
            }
            if (KIND != SCAN_GV) {
                // exactly one lane of each column x holds the diagonal element (head + tail of the split, one half
                // of each word); both waves computed the same A
                const float dsel = (bf16_lo(dh) + bf16_hi(dh)) + (bf16_lo(dl) + bf16_hi(dl));
                if (((x >> 2) & 1) == g) L.Diag[x] = dsel;
            }
        } else {
            int dx = 4 * g - x;
            asm volatile("" : "+v"(dx));
            float dsel = 0.f;                                             // A[t][t] (v_t . gy_t)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float a8[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int r = 8 * ks + e;
                    const int sx = 8 * (r / 4) + (r % 4) + dx;            // s - x
                    a8[e] = sx < 0 ? accA[r] : 0.f;
                    dsel = sx == 0 ? accA[r] : dsel;
                }
                split8(a8, Ah[ks], Al[ks]);
            }
            if (((x >> 2) & 1) == g) L.Diag[x] = dsel;
        }
        // ---- MFMA 2: Out[t][o] = sum_s A[t][s] Val[s][o] ----
        f32x16 accY = {0};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bf16x8 bv = cat8(*reinterpret_cast<const bf16x4*>(&L.VTh[ocol][16 * ks + 4 * g]),
                                   *reinterpret_cast<const bf16x4*>(&L.VTh[ocol][16 * ks + 8 + 4 * g]));
            const bf16x8 bvl = cat8(*reinterpret_cast<const bf16x4*>(&L.VTl[ocol][16 * ks + 4 * g]),
                                    *reinterpret_cast<const bf16x4*>(&L.VTl[ocol][16 * ks + 8 + 4 * g]));
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ah[ks], bv, accY, 0, 0, 0);
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Al[ks], bv, accY, 0, 0, 0);
            accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ah[ks], bvl, accY, 0, 0, 0);
            if (LL) accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Al[ks], bvl, accY, 0, 0, 0);
        }
        // ---- MFMA 3: Out += Q (rescaled state), the state straight from the accumulators ----
        const float cr_lane = TT ? (KIND == SCAN_GR ? L.C1[ocol] : L.C3[ocol]) : 0.f;
#pragma unroll
        for (int ch2 = 0; ch2 < 2; ++ch2) {
            const f32x16& S = ch2 == 0 ? S0 : S1;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float s8[8];
#pragma unroll
                for (int e4 = 0; e4 < 2; ++e4) {
                    f32x4 cr = {cr_lane, cr_lane, cr_lane, cr_lane};
                    if (!TT) cr = *reinterpret_cast<const f32x4*>(&L.C3[32 * ch2 + 16 * ks + 8 * e4 + 4 * g]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) s8[4 * e4 + e] = S[8 * ks + 4 * e4 + e] * cr[e];
                }
                bf16x8 sh, sl;
                split8(s8, sh, sl);
                const int c0 = 32 * ch2 + 16 * ks + 4 * g;
                const bf16x8 ah = cat8(*reinterpret_cast<const bf16x4*>(&L.Qh[x][c0]),
                                       *reinterpret_cast<const bf16x4*>(&L.Qh[x][c0 + 8]));
                accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, sh, accY, 0, 0, 0);
                accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, sl, accY, 0, 0, 0);
                if (QS) {
                    const bf16x8 al = cat8(*reinterpret_cast<const bf16x4*>(&L.Ql[x][c0]),
                                           *reinterpret_cast<const bf16x4*>(&L.Ql[x][c0 + 8]));
                    accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, sh, accY, 0, 0, 0);
                    if (LL) accY = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, sl, accY, 0, 0, 0);
                }
            }
        }
        if (KIND == SCAN_GK) {                                            // late: these would not fit beside MFMA 1-3
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                araw[r] = BufRaw<4>::ld(rsa, row_off(cc, r, Cs, 4), 0);
            }
        }
        // ---- MFMA 4: M[c][o] = sum_s Kc[s][c] Val[s][o];  state' = decay * state + scale * M ----
        const float c2_lane = TT ? L.C2[ocol] : 0.f;
        const float cu_lane = TT ? (KIND == SCAN_GR ? L.C3[ocol] : L.C1[ocol]) : 0.f;
#pragma unroll
        for (int ch2 = 0; ch2 < 2; ++ch2) {
            f32x16 accM = {0};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const bf16x8 ah = *reinterpret_cast<const bf16x8*>(&L.KTh[32 * ch2 + x][16 * ks + 8 * g]);
                const bf16x8 bv = *reinterpret_cast<const bf16x8*>(&L.VTh[ocol][16 * ks + 8 * g]);
                const bf16x8 bvl = *reinterpret_cast<const bf16x8*>(&L.VTl[ocol][16 * ks + 8 * g]);
                accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bv, accM, 0, 0, 0);
                accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bvl, accM, 0, 0, 0);
                if (KS) {
                    const bf16x8 al = *reinterpret_cast<const bf16x8*>(&L.KTl[32 * ch2 + x][16 * ks + 8 * g]);
                    accM = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bv, accM, 0, 0, 0);
                }
            }
            f32x16& S = ch2 == 0 ? S0 : S1;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                f32x4 c2 = {c2_lane, c2_lane, c2_lane, c2_lane}, cu = {cu_lane, cu_lane, cu_lane, cu_lane};
                if (!TT) {
                    c2 = *reinterpret_cast<const f32x4*>(&L.C2[32 * ch2 + 8 * r4 + 4 * g]);
                    cu = *reinterpret_cast<const f32x4*>(&L.C1[32 * ch2 + 8 * r4 + 4 * g]);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) S[4 * r4 + e] = c2[e] * S[4 * r4 + e] + cu[e] * accM[4 * r4 + e];
            }
        }
        // ================================== epilogue ==================================
        if (GK_RMW) {
#pragma unroll
            for (int r = 0; r < 16; ++r) prev[r] = __builtin_bit_cast(float, BufRaw<4>::ld(rso, row_off(cc, r, Cs, 4), 0));
        }
        if (KIND == SCAN_GV) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                put_f32<false>(prev[r] + accY[r], rso, row_off(cc, r, Cs, 4));
        } else {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");       // Diag: written and read inside a wave
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
            float dd[16];                                                         // GK: a - b per row
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const f32x4 dg = *reinterpret_cast<const f32x4*>(&L.Diag[8 * r4 + 4 * g]);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = 4 * r4 + e;
                    const int rho = 8 * r4 + 4 * g + e;
                    const float post = L.Post[rho][ocol];
                    const float rr = cvt(rraw[r]), kk = cvt(kraw[r]);
                    const float px = post * accY[r];
                    if (KIND == SCAN_GR) {
                        const float gr = ASC ? fmaf(u_o * kk, dg[e], px) : px;
                        put_f32<false>(prev[r] + gr, rso, row_off(cc, r, Cs, 4));
                        BufRaw<4>::st(__builtin_bit_cast(unsigned, rr * px), rsa, row_off(cc, r, Cs, 4), 0);
                        if (ASC) gu_acc = fmaf(rr * kk, dg[e], gu_acc);
                    } else {
                        const float gk = ASC ? fmaf(u_o * rr, dg[e], px) : px;
                        put_f32<false>(prev[r] + gk, rso, row_off(cc, r, Cs, 4));
                        dd[r] = __builtin_bit_cast(float, araw[r]) - kk * px;     // rows past T: a = 0, k = 0
                    }
                }
            }
            if (KIND == SCAN_GK) {
                // gw_n = ld_n (sum over the tokens scanned before n of (a - b)  -  b_n): a running sum over the
                // scan rows.  A lane holds rows 8 r4 + 4g + e; its partner (lane ^ 32) the other half of each 8.
                float bs[4], pbs[4];
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    bs[r4] = (dd[4 * r4] + dd[4 * r4 + 1]) + (dd[4 * r4 + 2] + dd[4 * r4 + 3]);
                    pbs[r4] = __shfl_xor(bs[r4], 32);
                }
                float before = xcarry;
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float run = before + (g == 1 ? pbs[r4] : 0.f);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = 4 * r4 + e;
                        const float kk = cvt(kraw[r]);
                        const float bn = kk * L.Post[8 * r4 + 4 * g + e][ocol] * accY[r];
                        const float ldn = -L.Ld[8 * r4 + 4 * g + e][ocol] * (1.0f / LOG2E);   // log decay of the row's token
                        const float gw = ldn * (run - bn);
                        put_f32<ASC>(gw, rsgw, row_off(cc, r, Cs, 4));
                        run += dd[r];
                    }
                    before += bs[r4] + pbs[r4];
                }
                xcarry = before;
            }
        }
        lds_barrier();                                                   // (3) LDS is rewritten by the next chunk
    }
    if (KIND == SCAN_GR && ASC) {
        gu_acc += __shfl_xor(gu_acc, 32);
        if (g == 0) gu_part[(size_t)b * C + h * HN + ocol] = gu_acc;
    }
}

}  // namespace wkv6_detail
}  // namespace vrwkv
