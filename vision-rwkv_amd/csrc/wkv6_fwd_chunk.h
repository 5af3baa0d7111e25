// wkv6 forward, chunked matrix-core kernel for gfx950 (bf16 MFMA, fp32 accumulate).
//
// Bidirectional RWKV-6 scan of
// classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:6-97, evaluated as two
// passes (descending; ascending with the bonus u), each the same causal algorithm on its own
// token order n = 0..T-1:
//
//   y_n = sum_j r_n[j] ( u[j] k_n[j] v_n  +  sum_{m<n} (prod_{m<l<n} d_l[j]) k_m[j] v_m )
//
// One 512-thread workgroup per (b,h): waves 0-3 run the descending pass, waves 4-7 the ascending one, half a
// step apart (see "schedule" in the kernel); two workgroups per CU put four waves on every SIMD.  Chunks of 32
// tokens.  With the in-chunk cumulative log-decay P_n = sum_{l<=n} log d_l (Pex_n = P_n - log d_n) and the
// chunk's end as the reference, P31:
//   rt_n = r_n * exp(Pex_n - P31),   kt_m = k_m * exp(P31 - P_m)       (rt_n . kt_m = decay for m<n)
//   A[n][m] = rt_n . kt_m  (m < n),  bonus_n = (r_n u) . k_n  (m = n, ascending pass), 0 otherwise -> MFMA 1
//   Z       = diag(e^P31) S                                  the state as the chunk's end sees it
//   Y       = A V  +  rt Z                                                     -> MFMA 2, 3
//   S'      = Z + kt^T V                                                       -> MFMA 4, accumulated onto Z
// so one scaled copy of the state serves the read-out and the update.  In the matrix stage a wave owns 16
// value columns: S (64 x 16, four 16x16 accumulator tiles) never leaves its registers and goes straight
// back in as an operand of MFMA 3 -- the contraction index is taken in the order the accumulator layout
// provides, the [token][channel] arrays in LDS keep their channels in that same order (an operand is one
// 16-byte read), and MFMA 1 contracts in it too, so one set of rt registers feeds both.  Likewise A goes from
// the accumulators of MFMA 1 into an operand of MFMA 2 (every wave forms the whole 32 x 32 A: three 16x16
// blocks, the fourth is masked out as a whole).  The y tiles are accumulated transposed, so that a lane holds
// four neighbouring columns of a token and a tile is stored with 16-byte accesses.
//
// y: both passes walk the same chunk grid from opposite ends.  The pass that reaches a chunk first stores,
// the other one fetches those values ahead of its matrix stage and accumulates on top of them -- y is never
// zero-filled, and there is no second launch.
//
// Precision: every operand that is computed rather than loaded (rt, kt, A, Z) is split into a
// bf16 head and a bf16 tail and the products head*head + head*tail + tail*head are accumulated,
// which keeps the result within ~3e-5 of the fp32 recurrence (one bf16 rounding of any of them
// alone costs ~1e-2).  v is exact in bf16 for bf16 input and split in two for fp16 / fp32 input.
//
// Range: the factorisation needs |P31| <= 60 in every chunk (decay over 32 tokens no stronger
// than e^-60).  A (b,h) sequence with a chunk outside that range is redone from scratch by the same
// workgroup with the sequential-state recurrence.
#pragma once
#include "wkv6_chunk_common.h"

namespace vrwkv {
namespace wkv6_detail {

constexpr int FW_WAVES = 8;      // waves per workgroup: four per pass
constexpr int FW_PJ = 72;        // row pitch (bf16) of the [token][channel] operand arrays: 16-byte reads of eight
                                 // consecutive rows fall into distinct banks (36 dwords = 4 mod 32)
constexpr int FW_PS = 40;        // row pitch (bf16) of the [channel][token] operand arrays

typedef float f32x4v __attribute__((ext_vector_type(4)));

// 8 values per lane -> per 16-lane row, the row sums of all 8: lane l ends up with the sum over its row of value
// index 4*(l&1) + 2*((l>>1)&1) + ((l>>2)&1).  Transposing butterfly over lane bits 0..2, plain add over bit 3.
__device__ __forceinline__ float row_sums8(const float (&p)[8], int lane, int& index) {
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4;
    float a4[4], a2[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) a4[i] = (b0 ? p[4 + i] : p[i]) + dpp_get<0xB1>(b0 ? p[i] : p[4 + i]);       // quad_perm [1,0,3,2]
#pragma unroll
    for (int i = 0; i < 2; ++i) a2[i] = (b1 ? a4[2 + i] : a4[i]) + dpp_get<0x4E>(b1 ? a4[i] : a4[2 + i]);   // quad_perm [2,3,0,1]
    const float give = b2 ? a2[0] : a2[1];
    const float from_lo = dpp_get<0x114>(give), from_hi = dpp_get<0x104>(give);   // row_shr:4 (from l-4), row_shl:4 (from l+4)
    float s = (b2 ? a2[1] : a2[0]) + (b2 ? from_lo : from_hi);
    s += dpp_get<0x128>(s);                                                       // row_ror:8
    index = (b0 ? 4 : 0) + (b1 ? 2 : 0) + (b2 ? 1 : 0);
    return s;
}

// head/tail split of four fp32 accumulator values into two packed bf16 word pairs
__device__ __forceinline__ void split4(const float (&x)[4], unsigned (&h)[2], unsigned (&l)[2]) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        h[p] = pack_bf16(x[2 * p], x[2 * p + 1]);
        l[p] = pack_bf16(x[2 * p] - bf16_lo(h[p]), x[2 * p + 1] - bf16_hi(h[p]));
    }
}
__device__ __forceinline__ bf16x8 words8(unsigned a, unsigned b, unsigned c, unsigned d) {
    return __builtin_bit_cast(bf16x8, u32x4{a, b, c, d});
}

// Per-pass LDS operands.  VSPLIT: v is given in a type that is not exact in bf16 (fp16, fp32) and is split in two.
template <bool VSPLIT>
struct __attribute__((aligned(16))) FwdLds {
    __bf16 Rh[LC][FW_PJ], Rl[LC][FW_PJ], Kh[LC][FW_PJ], Kl[LC][FW_PJ];
    __bf16 Kth[HN][FW_PS], Ktl[HN][FW_PS], Vt[HN][FW_PS], Vtl[VSPLIT ? HN : 1][FW_PS];
    float C2[4][HN], Tot[4][HN], Bon[4][LC];     // C2: e^P31 per channel, one copy per wave (written and read by that wave only)
};

// Phase stamps (STAMPS = true, the profiling entry point only): lane 0 of every wave stores the shader clock at
// FW_STAMP_POINTS points of every chunk step into stamps[((b*H + h) * FW_WAVES + wave) * nchunk + step][point]:
//   0 stage E entered   1 operands written, before the barrier   2 after that barrier
//   4 stage M entered   5 y stored and next decays summed, before the barrier   6 after that barrier   3, 7 unused
constexpr int FW_STAMP_POINTS = 8;

template <typename IO, typename WT, bool W_IS_EW, bool STAMPS = false>
__global__ __launch_bounds__(64 * FW_WAVES, 4)   // four waves per SIMD: at most 128 registers
void wkv6_fwd_chunk_kernel(const IO* __restrict__ r_, const IO* __restrict__ k_, const IO* __restrict__ v_,
                           const WT* __restrict__ w_, const float* __restrict__ u_, float* __restrict__ y_,
                           int T, int C, int H, unsigned long long* __restrict__ stamps = nullptr)
{
    constexpr bool VSPLIT = !(sizeof(IO) == 2 && __is_same(IO, __hip_bfloat16));
    __shared__ FwdLds<VSPLIT> lds[2];
    __shared__ int sFlag[2];                   // out-of-range flags, one per half-period parity
    static_assert(sizeof(FwdLds<VSPLIT>) * 2 >= 4 * 2 * 3 * N * sizeof(float), "fallback staging must fit");

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w4 = wave & 3;                     // token quarter in stage E, value-column quarter in stage M
    const bool asc = wave >= 4;                  // waves 4-7: ascending pass (with the bonus)
    FwdLds<VSPLIT>& L = lds[asc ? 1 : 0];
    const int bh = blockIdx.x;
    const int b = bh / H, h = bh % H;
    const size_t base = (size_t)b * T * C + (size_t)h * HN;
    const int nchunk = (T + LC - 1) / LC;
    const float uj = asc ? u_[h * HN + lane] : 0.f;
    if (threadIdx.x < 2) sFlag[threadIdx.x] = 0;
    __syncthreads();
    unsigned long long* stamp_row = nullptr;
    if constexpr (STAMPS) stamp_row = stamps + ((size_t)bh * FW_WAVES + wave) * nchunk * FW_STAMP_POINTS;
    auto stamp = [&](int ch, int point) {
        if constexpr (STAMPS) {
            const unsigned long long now = __builtin_readcyclecounter();
            if (lane == 0) stamp_row[ch * FW_STAMP_POINTS + point] = now;
        }
    };

    // state tiles: S[jt] holds rows j = 16 jt + 4 g4 + r (r = 0..3), column i = 16 w4 + c16
    f32x4v S[4];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) S[jt] = f32x4v{0.f, 0.f, 0.f, 0.f};
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
    RawIO rraw[8], kraw[8], vraw[8];
    RawW wraw[8];
    // Both passes walk the same 32-token chunks of the token axis (the ascending pass chunk 0, 1, ..., the
    // descending pass chunk nchunk-1, ..., 0), so everything that depends on the position is wave-uniform.
    // Pass index n = 0..31 inside a chunk is token 32c + n (ascending) or 32c + 31 - n (descending); tokens
    // past T (only in the last chunk; for the descending pass they come first) read zeros and count as
    // k = 0, d = 1 (their own y rows are dropped by the store's range check).
    auto chunk_of = [&](int ch) { return asc ? ch : nchunk - 1 - ch; };
    const int sgn = asc ? 1 : -1, n0 = asc ? 0 : LC - 1;
    auto token_of = [&](int c, int n) { return c * LC + n0 + sgn * n; };
    // Row offsets walk the 8 tokens of this wave's block with one scalar add each (the scalar offset of the access;
    // the hardware's range check covers it).  Rows past T (last chunk only) lie outside the descriptors and read 0:
    // k = 0 switches such a token off everywhere, and its decay is set to 1 where the decays are summed.
    auto fetch_w = [&](int ch, int C) {
        const unsigned step = (unsigned)(sgn * C * (int)sizeof(WT));
        unsigned so = (unsigned)token_of(chunk_of(ch), 8 * w4) * C * (unsigned)sizeof(WT);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            wraw[m] = BufRaw<sizeof(WT)>::ld(rsw, lane * (unsigned)sizeof(WT), so);
            so += step;
        }
    };
    auto fetch_rkv = [&](int ch, int C) {
        const unsigned step = (unsigned)(sgn * C * (int)sizeof(IO));
        unsigned so = (unsigned)token_of(chunk_of(ch), 8 * w4) * C * (unsigned)sizeof(IO);
        const unsigned vo = lane * (unsigned)sizeof(IO);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            rraw[m] = BufRaw<sizeof(IO)>::ld(rsr, vo, so);
            kraw[m] = BufRaw<sizeof(IO)>::ld(rsk, vo, so);
            vraw[m] = BufRaw<sizeof(IO)>::ld(rsv, vo, so);
            so += step;
        }
    };
    auto cvt = [](RawIO raw) { IO t; __builtin_memcpy(&t, &raw, sizeof(t)); return to_f32(t); };
    auto cvtw = [](RawW raw) { WT t; __builtin_memcpy(&t, &raw, sizeof(t)); return to_f32(t); };
    // The y tiles are accumulated transposed (rows = value columns): register r of tile tb holds y[t][i] for pass index
    // n = 16 tb + c16 and column i = 16 w4 + 4 g4 + r, i.e. a lane owns four neighbouring columns of one token and a
    // tile is one 16-byte access per lane.  Its address is a per-lane byte offset plus a wave-uniform one that goes into
    // the scalar offset of the access; rows past T fall outside the descriptor and are dropped by the hardware.
    auto y_row = [&](int c, int tb, int C) -> unsigned {
        return (unsigned)((c * LC + (asc ? 16 * tb : 16 - 16 * tb)) * C * 4);
    };
    // ---- schedule -------------------------------------------------------------------------------------------
    // A chunk step of a pass is an element-wise stage E (factors, split operands into LDS) and a matrix stage M.
    // The two passes run them in opposite halves of a period, one workgroup barrier per half:
    //     half h:       0      1      2      3      4    ...
    //     ascending   E(0)   M(0)   E(1)   M(1)   E(2)
    //     descending   -     E(0)   M(0)   E(1)   M(1)
    // so that on every SIMD (it holds one wave of each pass) vector-ALU work and matrix / LDS work overlap, and a
    // step costs two barriers.  The barrier between E and M publishes the operands; the one between M and the next E
    // frees them, publishes the y rows stored in M to the other pass, and carries the next chunk's decay sums: M ends
    // by summing the log decays of chunk ch + 1 (rows fetched at its start) and writing the four waves' totals.
    //
    // y: chunk c is reached by the ascending pass in half 2c + 1 (its M) and by the descending pass in half
    // 2(nchunk - c) (its M).  The earlier one stores; the later one fetches those values at the end of its E, ahead of
    // the barrier, and accumulates on top of them -- unless the other pass's M runs in that very half (one step per
    // pass at most): then it fetches them at the start of its own M, behind the barrier.
    auto decay_sums = [&](int ch, int C, float (&p)[8]) {
        // log decays in log2 units: ld2 = -log2(e) exp(w) = -exp2(w log2(e) + log2(log2(e)))
        float e[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const float fw = cvtw(wraw[m]);
            e[m] = W_IS_EW ? -fw * LOG2E : fast_exp2(fmaf(fw, LOG2E, LOG2_LOG2E));
        }
        if ((chunk_of(ch) + 1) * LC > T) {                                // wave-uniform: some token of the chunk is past T
#pragma unroll
            for (int m = 0; m < 8; ++m)
                if (token_of(chunk_of(ch), 8 * w4 + m) >= T) e[m] = 0.f;
        }
        p[0] = -e[0];
#pragma unroll
        for (int m = 1; m < 8; ++m) p[m] = p[m - 1] - e[m];
        L.Tot[w4][lane] = p[7];
    };
    auto sync_step = [&]() {
        // every LDS access of the half is done, and the y stores of a matrix stage become visible to the other pass
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    };
    float p[8];                                                          // in-wave cumulative log2 decays of the next E
    fetch_w(0, C);
    fetch_rkv(0, C);
    decay_sums(0, C, p);
    f32x4v accY[2];                                                      // y tiles of the step: filled in E (earlier values), finished in M
    bf16x8 zh[2], zl[2];                                                 // the scaled state of the step as MFMA operands (formed in E)
    unsigned y_lane = 0;
    sync_step();

    // The descending pass starts one half later (first line of the table): from here on both passes run the same loop,
    // E, barrier, M, barrier, and the ascending pass adds the barrier the other one's last M still needs.
    int hp = asc ? 0 : 1;                                                // common-clock index of the half that E(0) runs in
    if (!asc) sync_step();
    for (int ch = 0; ch < nchunk; ++ch, hp += 2) {
        // Row offsets are recomputed per step from an opaque copy of C: hoisted out of the loop they would
        // occupy scalar registers by the dozen and spill.
        int Cs = C;
        asm volatile("" : "+s"(Cs));
        // Per-lane addresses are formed again in every step from an opaque copy of the lane number: kept across the
        // loop they would hold a dozen registers (128 per wave is the budget for four waves per SIMD).
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        int w4s = w4, hps = hp;                                           // the same for what depends on the wave number
        asm volatile("" : "+s"(w4s), "+s"(hps));
        const int cy = chunk_of(ch);
        // the other pass's M of chunk cy on the common clock: the descending one runs in half 2 (nchunk - cy), the
        // ascending one in half 2 cy + 1; this step's E runs in half hp, its M in half hp + 1
        const int other_m = asc ? 2 * (nchunk - cy) : 2 * cy + 1;
        const bool y_second = other_m < hp + 1, y_late = other_m == hp;   // wave-uniform
        // ... and if the other pass runs its E of chunk cy in the half of this step's M, it fetches this step's y rows
        // right behind the barrier that ends that half: then the stores are waited for before that barrier (the barrier
        // orders the instructions' issue, not the arrival of the data)
        const bool y_drain = (asc ? 2 * (nchunk - 1 - cy) + 1 : 2 * cy) == hp + 1;
        {
            // =============================== stage E: elementwise =================================
            // wave w4s of the pass prepares tokens n = 8 w4s .. 8 w4s + 7 of the chunk; lane = channel j (and i for v)
            // Column of channel j = lane_e in the [token][channel] arrays: the matrix stage contracts over the channels
            // in the order the state's accumulator tiles give (slot (g4, e) of contraction half kb <-> j = 32 kb + 4 g4 + e
            // for e < 4, 32 kb + 16 + 4 g4 + e - 4 for e >= 4), so the arrays keep the channels in that order and an
            // operand is one 16-byte read: j = 32 kb + 16 hf + 4 g + e  ->  column 32 kb + 8 g + 4 hf + e.
            const int jcol = (lane_e & 32) | ((lane_e & 12) << 1) | ((lane_e & 16) >> 2) | (lane_e & 3);
            stamp(ch, 0);
            // The next chunk's decay rows: summed at the end of this step's matrix stage, a whole step of latency away (the
            // last step re-reads its own rows: no branch, so the compiler's wait counts stay exact).
            fetch_w(ch + 1 < nchunk ? ch + 1 : ch, Cs);
            // rest = log2 decay from the start of this wave's tokens to the chunk's end (P_m - P31 = p[m] - rest >= 0),
            // p31 = that of the whole chunk; the waves' totals were written at the end of the previous matrix stage
            const float t0 = L.Tot[0][lane_e], t1 = L.Tot[1][lane_e], t2 = L.Tot[2][lane_e], t3 = L.Tot[3][lane_e];
            const float m0 = w4s == 0 ? 1.f : 0.f, m1 = w4s <= 1 ? 1.f : 0.f, m2 = w4s <= 2 ? 1.f : 0.f;     // wave-uniform
            const float rest = fmaf(m0, t0, fmaf(m1, t1, fmaf(m2, t2, t3)));
            const float p31 = (t0 + t1) + (t2 + t3);
            if (w4s == 0 && __builtin_amdgcn_ballot_w64(!(p31 >= -SAFE_DECAY * LOG2E)) != 0ull && lane == 0) sFlag[hps & 1] = 1;
            // Z = diag(e^P31) S, in place, split into head and tail for MFMA 3 (done here, while the r, k, v rows are still
            // on their way): a lane needs e^P31 of the channels its state rows belong to, taken from the wave's own copy
            L.C2[w4s][lane_e] = fast_exp2(p31);
            {
                const int g4 = lane_e >> 4;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    float z8[8];
#pragma unroll
                    for (int hf = 0; hf < 2; ++hf) {
                        const f32x4 c2 = *reinterpret_cast<const f32x4*>(&L.C2[w4s][16 * (2 * kb + hf) + 4 * g4]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) { S[2 * kb + hf][e] *= c2[e]; z8[4 * hf + e] = S[2 * kb + hf][e]; }
                    }
                    split8(z8, zh[kb], zl[kb]);
                }
            }
            {
                unsigned kthw[4], ktlw[4], vthw[4], vtlw[4];
                float pu[8];
                float zp = -rest;                                         // Pex_m - P31 = z_(m-1)
#pragma unroll
                for (int m = 0; m < 8; m += 2) {
                    const int n = 8 * w4s + m;
                    const float z0 = p[m] - rest, z1 = p[m + 1] - rest;
                    const float f1a = fast_exp2(zp), f2a = fast_exp2(-z0);    // exp(Pex - P31), exp(P31 - P)
                    const float f1b = fast_exp2(z0), f2b = fast_exp2(-z1);
                    zp = z1;
                    const float r0 = cvt(rraw[m]), r1 = cvt(rraw[m + 1]), k0 = cvt(kraw[m]), k1 = cvt(kraw[m + 1]);
                    const float rt0 = r0 * f1a, rt1 = r1 * f1b, kt0 = k0 * f2a, kt1 = k1 * f2b;
                    const unsigned rh = pack_bf16(rt0, rt1), kh = pack_bf16(kt0, kt1);    // token m low, m + 1 high
                    const unsigned rl = pack_bf16(rt0 - bf16_lo(rh), rt1 - bf16_hi(rh));
                    const unsigned kl = pack_bf16(kt0 - bf16_lo(kh), kt1 - bf16_hi(kh));
                    st_bf16_pair(&L.Rh[n][jcol], &L.Rh[n + 1][jcol], rh);
                    st_bf16_pair(&L.Rl[n][jcol], &L.Rl[n + 1][jcol], rl);
                    st_bf16_pair(&L.Kh[n][jcol], &L.Kh[n + 1][jcol], kh);
                    st_bf16_pair(&L.Kl[n][jcol], &L.Kl[n + 1][jcol], kl);
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
                *reinterpret_cast<u32x4*>(&L.Kth[lane_e][8 * w4s]) = u32x4{kthw[0], kthw[1], kthw[2], kthw[3]};
                *reinterpret_cast<u32x4*>(&L.Ktl[lane_e][8 * w4s]) = u32x4{ktlw[0], ktlw[1], ktlw[2], ktlw[3]};
                *reinterpret_cast<u32x4*>(&L.Vt[lane_e][8 * w4s]) = u32x4{vthw[0], vthw[1], vthw[2], vthw[3]};
                if constexpr (VSPLIT)
                    *reinterpret_cast<u32x4*>(&L.Vtl[lane_e][8 * w4s]) = u32x4{vtlw[0], vtlw[1], vtlw[2], vtlw[3]};
                if (asc) {                                                // bonus_n = sum_j r_n[j] u[j] k_n[j]
                    int idx;
                    const float rs = row_sums8(pu, lane_e, idx);
                    L.Bon[lane_e >> 4][8 * w4s + idx] = rs;                // the four 16-channel rows are added by the reader
                }
            }
            // earlier y values of this chunk (none: an out-of-range offset reads 0 without a memory access)
            {
                const int g4 = lane_e >> 4, c16 = lane_e & 15;
                y_lane = (unsigned)(((asc ? c16 : 15 - c16) * Cs + 16 * w4s + 4 * g4) * sizeof(float));
                const unsigned vo = y_second && !y_late ? y_lane : OOB_OFFSET;
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) accY[tb] = __builtin_bit_cast(f32x4v, BufRaw<16>::ld(rsy, vo, y_row(cy, tb, Cs)));
            }
            stamp(ch, 1);
        }
        sync_step();
        stamp(ch, 2);
        if (sFlag[hps & 1]) { bail = true; break; }                       // out of range: redo with the exact recurrence
        {
            // ================================= stage M: matrix cores ===============================
            const int g4 = lane_e >> 4, c16 = lane_e & 15;                // lane = (column c16, slot group g4)
            stamp(ch, 4);
            __builtin_amdgcn_s_setprio(2);        // the matrix stage goes first on its SIMD: its MFMA chains and LDS round trips are the long pole
            if (y_late) {
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) accY[tb] = __builtin_bit_cast(f32x4v, BufRaw<16>::ld(rsy, y_lane, y_row(cy, tb, Cs)));
            }
            // The stage is written in phases, each starting with the LDS reads of all its operands (so one latency is
            // paid per phase, not one per MFMA) and pinned in that order by scheduling barriers; the registers of a
            // phase's operands are dead when the next one loads (128 registers per wave hold one phase at a time).
            // rt rows t = 16 tb + c16 and kt rows s = 16 sb + c16 as MFMA operands, contraction slot (g4, e) <-> column
            // 32 kb + 8 g4 + e of the arrays, i.e. channel j = 32 kb + 4 g4 + e (e < 4), 32 kb + 16 + 4 g4 + e - 4 (e >= 4):
            // the order the state tiles give for MFMA 3, used by MFMA 1 as well, so one set of rt registers feeds both.
            auto rows_op = [&](const __bf16 (*arr)[FW_PJ], int blk, int kb) -> bf16x8 {
                return *reinterpret_cast<const bf16x8*>(&arr[16 * blk + c16][32 * kb + 8 * g4]);
            };
            f32x4v accA[3] = {f32x4v{0.f, 0.f, 0.f, 0.f}, f32x4v{0.f, 0.f, 0.f, 0.f}, f32x4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                // ---- phase kb: operands of contraction half kb ----
                bf16x8 RH[2], RL[2], KH[2], KL[2];
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    RH[blk] = rows_op(L.Rh, blk, kb);
                    RL[blk] = rows_op(L.Rl, blk, kb);
                    KH[blk] = rows_op(L.Kh, blk, kb);
                    KL[blk] = rows_op(L.Kl, blk, kb);
                }
                __builtin_amdgcn_sched_barrier(0);
                // MFMA 3: Y^T += Z^T rt^T with Z straight from the accumulators (the state tile is the A operand: rows = value
            // columns, so the y tiles come out transposed);
                // MFMA 1: A^T blocks (s block, t block) = (0,0), (0,1), (1,1): acc[m = s][n = t]; the lane holds t = c16 of the
                // block, rows s = 4 g4 + r.  Block (1,0) has s > t throughout.
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    accY[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(zh[kb], RH[tb], accY[tb], 0, 0, 0);
                    accA[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KH[0], RH[tb], accA[tb], 0, 0, 0);
                }
                accA[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KH[1], RH[1], accA[2], 0, 0, 0);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    accY[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(zl[kb], RH[tb], accY[tb], 0, 0, 0);
                    accA[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KH[0], RL[tb], accA[tb], 0, 0, 0);
                }
                accA[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KH[1], RL[1], accA[2], 0, 0, 0);
#pragma unroll
                for (int tb = 0; tb < 2; ++tb) {
                    accY[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(zh[kb], RL[tb], accY[tb], 0, 0, 0);
                    accA[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KL[0], RH[tb], accA[tb], 0, 0, 0);
                }
                accA[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(KL[1], RH[1], accA[2], 0, 0, 0);
                // While the matrix pipe works these off, the vector ALUs form the next chunk's decay sums (its rows were
                // fetched at the top of stage E; p and the totals of this step are no longer read).
                if (kb == 1) decay_sums(ch + 1 < nchunk ? ch + 1 : ch, Cs, p);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- phase 2: operands of the products over the chunk's tokens ----
            // The next step's r, k, v rows go out first (the operand registers of the phases above are free): their latency
            // runs behind the rest of this stage, the barrier and the first part of stage E (the last step re-reads its own
            // rows: no branch, the compiler's wait counts stay exact).
            fetch_rkv(ch + 1 < nchunk ? ch + 1 : ch, Cs);
            const int icol = 16 * w4s + c16;
            const bf16x8 bv = cat8(*reinterpret_cast<const bf16x4*>(&L.Vt[icol][4 * g4]),
                                   *reinterpret_cast<const bf16x4*>(&L.Vt[icol][16 + 4 * g4]));
            const bf16x8 bs = *reinterpret_cast<const bf16x8*>(&L.Vt[icol][8 * g4]);
            bf16x8 bvl, bsl;
            if constexpr (VSPLIT) {
                bvl = cat8(*reinterpret_cast<const bf16x4*>(&L.Vtl[icol][4 * g4]), *reinterpret_cast<const bf16x4*>(&L.Vtl[icol][16 + 4 * g4]));
                bsl = *reinterpret_cast<const bf16x8*>(&L.Vtl[icol][8 * g4]);
            }
            bf16x8 kth[4];
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) kth[jt] = *reinterpret_cast<const bf16x8*>(&L.Kth[16 * jt + c16][8 * g4]);
            float bon[2];
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) {
                const int t = 16 * tb + c16;
                bon[tb] = (L.Bon[0][t] + L.Bon[1][t]) + (L.Bon[2][t] + L.Bon[3][t]);
            }
            __builtin_amdgcn_sched_barrier(0);
            // A[t][s] keeps s < t and takes the bonus at s = t: applied to the packed bf16 words of the two diagonal
            // blocks with the lane's constant bit masks (the descending pass has no bonus; its Bon rows are never written)
            // causal masks of the two diagonal 16x16 blocks, one word per pair of accumulator registers (r = 2p low half,
            // 2p + 1 high): the lane holds t = c16, rows s = 4 g4 + r (formed here: kept across the step they cost registers)
            unsigned keepw[2], diagw[2];
            {
                const int d = c16 - 4 * g4;                                   // t - s of register 0
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    keepw[pr] = (2 * pr < d ? 0xffffu : 0u) | (2 * pr + 1 < d ? 0xffff0000u : 0u);
                    diagw[pr] = (2 * pr == d ? 0xffffu : 0u) | (2 * pr + 1 == d ? 0xffff0000u : 0u);
                }
            }
            unsigned ahw[3][2], alw[3][2];
#pragma unroll
            for (int blk = 0; blk < 3; ++blk) {
                const float a4[4] = {accA[blk][0], accA[blk][1], accA[blk][2], accA[blk][3]};
                split4(a4, ahw[blk], alw[blk]);
            }
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) {
                const int blk = 2 * tb;
                const float diag = asc ? bon[tb] : 0.f;
                const unsigned dgh = pack_bf16(diag, diag), dgl = pack_bf16(diag - bf16_lo(dgh), diag - bf16_lo(dgh));
#pragma unroll
                for (int pr = 0; pr < 2; ++pr) {
                    ahw[blk][pr] = (ahw[blk][pr] & keepw[pr]) | (dgh & diagw[pr]);
                    alw[blk][pr] = (alw[blk][pr] & keepw[pr]) | (dgl & diagw[pr]);
                }
            }
            // ---- MFMA 2: Y^T[i][t] += sum_s V[s][i] A[t][s]; contraction slot (g4, e) <-> s = 4 g4 + e (e < 4),
            //      16 + 4 g4 + e - 4 (e >= 4): accumulator order of the blocks (0, tb) and (1, tb);
            //      MFMA 4: S' = Z + kt^T V, accumulated onto the scaled state, contraction over s in its natural order ----
            {
                const bf16x8 Ah0 = words8(ahw[0][0], ahw[0][1], 0u, 0u), Al0 = words8(alw[0][0], alw[0][1], 0u, 0u);
                const bf16x8 Ah1 = words8(ahw[1][0], ahw[1][1], ahw[2][0], ahw[2][1]), Al1 = words8(alw[1][0], alw[1][1], alw[2][0], alw[2][1]);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) S[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kth[jt], bs, S[jt], 0, 0, 0);
                accY[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bv, Ah0, accY[0], 0, 0, 0);
                accY[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bv, Ah1, accY[1], 0, 0, 0);
                if constexpr (VSPLIT) {
#pragma unroll
                    for (int jt = 0; jt < 4; ++jt) S[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kth[jt], bsl, S[jt], 0, 0, 0);
                    accY[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bvl, Ah0, accY[0], 0, 0, 0);
                    accY[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bvl, Ah1, accY[1], 0, 0, 0);
                }
                // the tails of kt^T take the heads' registers: read while the MFMAs above run
                __builtin_amdgcn_sched_barrier(0);
                bf16x8 ktl[4];
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) ktl[jt] = *reinterpret_cast<const bf16x8*>(&L.Ktl[16 * jt + c16][8 * g4]);
#pragma unroll
                for (int jt = 0; jt < 4; ++jt) S[jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ktl[jt], bs, S[jt], 0, 0, 0);
                accY[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bv, Al0, accY[0], 0, 0, 0);
                accY[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bv, Al1, accY[1], 0, 0, 0);
            }
            // ---- y: store (the sum with the other pass's values where it came first) ----
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
                BufRaw<16>::st(__builtin_bit_cast(typename BufRaw<16>::type, accY[tb]), rsy, y_lane, y_row(cy, tb, Cs));
            __builtin_amdgcn_s_setprio(0);
            if (y_drain) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            stamp(ch, 5);
        }
        sync_step();
        stamp(ch, 6);
        if (sFlag[(hps + 1) & 1]) { bail = true; break; }
    }
    if (asc && !bail) sync_step();

    if (bail) {
        // Some chunk decays faster than the factorisation can represent: recompute the whole sequence
        // with the sequential recurrence (it rewrites every y of this (b,h)); its mapping is four waves wide.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        float* stage = reinterpret_cast<float*>(&lds[0]);
        if (wave < 4) wkv6_scalar_pass<IO, WT, 1, W_IS_EW>(r_, k_, v_, w_, u_, y_, stage, bh, T, C, H);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (wave < 4) wkv6_scalar_pass<IO, WT, 0, W_IS_EW>(r_, k_, v_, w_, u_, y_, stage, bh, T, C, H);
    }
}

}  // namespace wkv6_detail
}  // namespace vrwkv
