// Bi-WKV backward, tiled kernel.
//
// Same decomposition as the forward kernel: lane = channel, wave = L consecutive tokens in registers,
// workgroup = S <= 8 waves = one (batch, super-chunk of S*L tokens, 64 channels) tile, persistent
// workgroups walking the tiles.  When the sequence fits one super-chunk (T <= 224) k, v, gy are read
// from HBM once and gk, gv written once (MODE 0).  Longer sequences take three launches, because both
// scans need every other super-chunk's sums before they can finish:
//   MODE 1  forward aggregates of every super-chunk                      (reads k, v)
//   MODE 2  forward with carries -> z, z*y -> per-wave sums of the adjoint scans   (reads k, v, gy)
//   MODE 3  the same again, then the adjoint scans with carries -> gk, gv          (reads k, v, gy)
// i.e. 10 tensor passes instead of 5, through a small auxiliary table.
//
// With E_i = e^{k_i}, g = e^{-w}, cu = e^{u}:
//   phase 1 (the forward):  D_t = sum_{i<t} g^{t-i-1} E_i + sum_{i>t} g^{i-t-1} E_i + cu E_t, N_t likewise
//                           with E_i v_i;  y_t = N_t / D_t,  z_t = gy_t / D_t
//   phase 2 (its adjoint):  Z_i = sum_{t<i} g^{i-t-1} z_t + sum_{t>i} g^{t-i-1} z_t + cu z_i, ZY_i likewise
//                           with z_t y_t;  gv_i = E_i Z_i,  gk_i = v_i gv_i - E_i ZY_i
//   gu = sum_i cu E_i (v_i z_i - z_i y_i)
//   gw = - sum_i E_i (v_i Lz_i - Lzy_i),  Lz_i = sum_{t!=i} (|t-i|-1) g^{|t-i|-1} z_t  (running sums
//        l <- g (l + s) next to s <- g s + z, so no per-token storage)
// Each phase is: per-wave chunk aggregates -> one LDS exchange -> carry-in from the other waves ->
// ascending sweep (past side) -> descending sweep (future side).
//
// Scaling: as in the forward's plain-sum path every wave works in units of 2^Rw, Rw = ceil(max kappa)
// over its tokens, and z carries 2^-Re with Re = max(Rw, R - plain_sum_up_cap) the scale its denominators were
// actually formed at.  Another wave's z-aggregates are brought over with the exact factor
// 2^(Rw_mine - Re_theirs): that is the same power of two by which my E entered their denominators, so
// the product stays below |gy| 2^41 and nothing overflows.  Tiles outside the plain-sum regime
// (outside_plain_sum) are left to the sequential kernel, which renormalises at every token.
#pragma once
#include "biwkv_fwd_impl.h"
#include "biwkv_bwd_serial.h"

namespace vrwkv {
namespace biwkv_bwd_detail {

using namespace biwkv_fwd_detail;

constexpr int BWD_SMAX = 8;

template <typename IO>
__device__ __forceinline__ float unpack1(typename BufRaw<sizeof(IO)>::type raw) {
    IO tmp;
    __builtin_memcpy(&tmp, &raw, sizeof(raw));
    return to_f32(tmp);
}
template <typename IO>
__device__ __forceinline__ void store1(__amdgpu_buffer_rsrc_t r, unsigned voff, float x) {
    const IO tmp = from_f32<IO>(x);
    typename BufRaw<sizeof(IO)>::type raw;
    __builtin_memcpy(&raw, &tmp, sizeof(raw));
    BufRaw<sizeof(IO)>::template st<CPOL_NT>(raw, r, voff, 0);
}

// True when this wave's 64 channels may use the plain-sum path (wave-uniform).
__device__ __forceinline__ bool bwd_tile_is_fast(float om, float mu, int T) {
    const bool bad = outside_plain_sum(om, mu, T);
    return __builtin_amdgcn_ballot_w64(bad) == 0ull;
}

struct ZScan {
    float s0 = 0.f, s1 = 0.f, l0 = 0.f, l1 = 0.f;
    __device__ __forceinline__ void push(float g, float z, float zy) {
        l0 = g * (l0 + s0);
        l1 = g * (l1 + s1);
        s0 = fmaf(g, s0, z);
        s1 = fmaf(g, s1, zy);
    }
    // n tokens of another wave pass in between: decay, then add that wave's own sums
    __device__ __forceinline__ void hop(float G, float n, float a0, float a1, float b0, float b1) {
        l0 = fmaf(G, fmaf(n, s0, l0), b0);
        l1 = fmaf(G, fmaf(n, s1, l1), b1);
        s0 = fmaf(G, s0, a0);
        s1 = fmaf(G, s1, a1);
    }
};

// Auxiliary table of the long-sequence path (floats):
//   agg1 [B][nSC][5][C]      forward aggregates of a super-chunk at its own scale R: A, B, R, Cg, D
//   agg2 [B][nSC][8][C]      z-sums of a super-chunk at the common scale 2^-R: past side (s0, s1, l0, l1), future side
struct BwdGeom {
    int n_ctile, nSC, n_tiles;      // tile id = (b * nSC + sc) * n_ctile + ctile
};

// STAGED (MODE 0, fp32 I/O, C % 4 == 0, 16-byte aligned k, v): the next tile's k, v rows are fetched straight into
// LDS in 16-byte pieces (buffer_load ... lds) while this tile is computed; gy stays a register load.
template <typename IO, int L, int MODE, bool STAGED = false>
__global__ __launch_bounds__(BWD_SMAX * WAVE)
void biwkv_bwd_tile_kernel(const float* __restrict__ w_, const float* __restrict__ u_,
                           const IO* __restrict__ k_, const IO* __restrict__ v_, const IO* __restrict__ gy_,
                           IO* __restrict__ gk_, IO* __restrict__ gv_,
                           float* __restrict__ ws, float* __restrict__ agg1, float* __restrict__ agg2,
                           float* __restrict__ gw_part, float* __restrict__ gu_part,
                           int B, int T, int C, BwdGeom geo)
{
    using Raw = typename BufRaw<sizeof(IO)>::type;
    __shared__ float s1[BWD_SMAX][5][WAVE];
    __shared__ float s2[BWD_SMAX][9][WAVE];
    __shared__ float s3[BWD_SMAX][2][WAVE];
    __shared__ float s_in[MODE >= 2 ? BWD_SMAX : 1][13][WAVE];   // what other super-chunks contribute, parked per wave
    constexpr int NI = (L + 3) / 4, LR = 4 * NI;              // staging instructions (four fp32 rows each) and LDS rows per tensor
    __shared__ __attribute__((aligned(16))) float s_stage[STAGED ? BWD_SMAX : 1][2][STAGED ? LR : 1][WAVE];

    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int S = blockDim.x >> 6;
    const int nSC = geo.nSC, n_ctile = geo.n_ctile, n_tiles = geo.n_tiles;
    const float NEG_INF = -__builtin_inff();
    const unsigned row = (unsigned)(C * sizeof(IO));
    const unsigned bytes = (unsigned)((size_t)T * C * sizeof(IO));
    auto shift_of = [](float d) -> int { return (int)fminf(fmaxf(d, -300.f), 300.f); };

    // workgroup barrier that orders LDS traffic only; the staged variant must not use the fence form, which
    // would also wait for the next tile's staging loads
    auto wg_barrier = [&]() {
        if (STAGED) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else lds_barrier();
    };
    float* const stage = &s_stage[STAGED ? wave : 0][0][0][0];
    auto issue_stage = [&](int tile) {                       // this wave's L rows of k and v, 4 rows per instruction
        const int ctile = tile % n_ctile;
        const int sc = (tile / n_ctile) % nSC, b = tile / n_ctile / nSC;
        const int tw = (sc * S + wave) * L;
        const size_t slab = (size_t)b * T * C;
        const __amdgpu_buffer_rsrc_t rk = make_rsrc(k_ + slab, bytes);
        const __amdgpu_buffer_rsrc_t rv = make_rsrc(v_ + slab, bytes);
        const int cq = ctile * WAVE + (lane & 15) * 4;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int rl = 4 * i + (lane >> 4);                           // row inside this wave's chunk
            const int rowt = tw + rl;
            const unsigned vo = (rl < L && rowt < T && cq < C) ? (unsigned)(((size_t)rowt * C + cq) * 4) : OOB_OFFSET;
            typedef __attribute__((address_space(3))) void* lds_ptr;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)(stage + i * 256), 16, vo, 0, 0, CPOL_NT);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (lds_ptr)(stage + LR * WAVE + i * 256), 16, vo, 0, 0, CPOL_NT);
        }
    };
    // workgroups are dealt round-robin to the 8 XCDs: per round, XCD x takes a contiguous eighth of the tiles
    const int wg = (gridDim.x & 7) == 0 ? (int)((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3)) : (int)blockIdx.x;
    if (STAGED && wg < n_tiles) issue_stage(wg);

    for (int tile = wg; tile < n_tiles; tile += gridDim.x) {
        const int ctile = tile % n_ctile;
        const int sc = (tile / n_ctile) % nSC, b = tile / n_ctile / nSC;
        const int c0 = ctile * WAVE + lane;
        const bool cok = c0 < C;
        const int tw = (sc * S + wave) * L;
        const unsigned voff0 = cok ? (unsigned)(((size_t)tw * C + c0) * sizeof(IO)) : OOB_OFFSET;
        const size_t slab = (size_t)b * T * C;
        const float om = (cok ? w_[c0] : 0.f) * LOG2E;
        const float mu = (cok ? u_[c0] : 0.f) * LOG2E;
        const int next_tile = tile + gridDim.x;
        if (!bwd_tile_is_fast(om, mu, T)) {                   // workgroup-uniform: same channels in every wave
            if (STAGED && next_tile < n_tiles) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // the skipped tile's rows must have landed
                issue_stage(next_tile);
            }
            wg_barrier();                                     // keeps the LDS reuse order of the computed tiles around it
            continue;
        }
        const int cc = cok ? c0 : 0;                         // in-range column for the auxiliary table
        auto a1 = [&](int s, int slot) -> float& { return agg1[(((size_t)b * nSC + s) * 5 + slot) * C + cc]; };
        auto a2 = [&](int s, int slot) -> float& { return agg2[(((size_t)b * nSC + s) * 8 + slot) * C + cc]; };

        // Long-sequence modes: what the other super-chunks contribute depends on the auxiliary tables alone, so it is
        // folded here, before this tile's rows are requested (the temporaries are dead by then).  Entries are fetched
        // eight (four where the z-sums come along) per direction at a time -- one memory round trip per batch instead of one per super-chunk; the forward
        // aggregates are summed at the running maximum of the scales met so far (integers: re-scaling is an exact
        // ldexp) and brought to the sequence's common scale R at the end; the z-sums already are at 2^-R.
        if (MODE >= 2) {
            float r_seq = NEG_BIG, a_in = 0.f, b_in = 0.f, c_in = 0.f, d_in = 0.f;
            ZScan p_in, f_in;
            constexpr int NB = MODE == 3 ? 4 : 8;
            const float GS = fast_exp2(-om * (float)(S * L)), nSL = (float)(S * L);
            // uniform entry offsets go into the scalar offset of a buffer load: one address register for all of them
            const __amdgpu_buffer_rsrc_t r1d = make_rsrc(agg1 + (size_t)b * nSC * 5 * C, (unsigned)((size_t)nSC * 5 * C * 4));
            const __amdgpu_buffer_rsrc_t r2d = make_rsrc(agg2 + (size_t)b * nSC * 8 * C, (unsigned)((size_t)nSC * 8 * C * 4));
            const unsigned vcol = (unsigned)cc * 4u;
            auto g1 = [&](int s, int slot) -> float {
                return __builtin_bit_cast(float, BufRaw<4>::ld(r1d, vcol, (unsigned)((s * 5 + slot) * C) * 4u));
            };
            auto g2 = [&](int s, int slot) -> float {
                return __builtin_bit_cast(float, BufRaw<4>::ld(r2d, vcol, (unsigned)((s * 8 + slot) * C) * 4u));
            };
            const float r_own = g1(sc, 2);
            float r1 = NEG_BIG, r2 = NEG_BIG;
            const int n_before = sc, n_after = nSC - 1 - sc;
            for (int j0 = 0; j0 < n_before || j0 < n_after; j0 += NB) {
                float pr[NB], p0[NB], p1[NB], fr[NB], f0[NB], f1[NB], pz[NB][4], fz[NB][4];
#pragma unroll
                for (int i = 0; i < NB; ++i) {                           // all conditions are workgroup-uniform
                    const int sp = j0 + i, sf = nSC - 1 - j0 - i;
                    if (j0 + i < n_before) {
                        pr[i] = g1(sp, 2); p0[i] = g1(sp, 0); p1[i] = g1(sp, 1);
                        if (MODE == 3) {
#pragma unroll
                            for (int x = 0; x < 4; ++x) pz[i][x] = g2(sp, x);
                        }
                    }
                    if (j0 + i < n_after) {
                        fr[i] = g1(sf, 2); f0[i] = g1(sf, 3); f1[i] = g1(sf, 4);
                        if (MODE == 3) {
#pragma unroll
                            for (int x = 0; x < 4; ++x) fz[i][x] = g2(sf, 4 + x);
                        }
                    }
                }
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    if (j0 + i < n_before) {
                        const float m = fmaxf(r1, pr[i]);
                        const int so = shift_of(r1 - m), sn = shift_of(pr[i] - m);
                        a_in = fmaf(GS, ldexpf(a_in, so), ldexpf(p0[i], sn));
                        b_in = fmaf(GS, ldexpf(b_in, so), ldexpf(p1[i], sn));
                        r1 = m;
                        if (MODE == 3) p_in.hop(GS, nSL, pz[i][0], pz[i][1], pz[i][2], pz[i][3]);
                    }
                    if (j0 + i < n_after) {
                        const float m = fmaxf(r2, fr[i]);
                        const int so = shift_of(r2 - m), sn = shift_of(fr[i] - m);
                        c_in = fmaf(GS, ldexpf(c_in, so), ldexpf(f0[i], sn));
                        d_in = fmaf(GS, ldexpf(d_in, so), ldexpf(f1[i], sn));
                        r2 = m;
                        if (MODE == 3) f_in.hop(GS, nSL, fz[i][0], fz[i][1], fz[i][2], fz[i][3]);
                    }
                }
            }
            r_seq = fmaxf(r_own, fmaxf(r1, r2));                         // common scale of the whole sequence
            const int s1 = shift_of(r1 - r_seq), s2 = shift_of(r2 - r_seq);
            // parked in this wave's own LDS slots until they are needed after the exchange: thirteen registers less
            // across the forward pass, where the kernel has none to spare
            float (*in)[WAVE] = s_in[wave];
            in[0][lane] = ldexpf(a_in, s1); in[1][lane] = ldexpf(b_in, s1);
            in[2][lane] = ldexpf(c_in, s2); in[3][lane] = ldexpf(d_in, s2);
            in[4][lane] = r_seq;
            if (MODE == 3) {
                in[5][lane] = p_in.s0; in[6][lane] = p_in.s1; in[7][lane] = p_in.l0; in[8][lane] = p_in.l1;
                in[9][lane] = f_in.s0; in[10][lane] = f_in.s1; in[11][lane] = f_in.l0; in[12][lane] = f_in.l1;
            }
            asm volatile("" ::: "memory");                               // the row loads below stay below
        }

        const __amdgpu_buffer_rsrc_t rk = make_rsrc(k_ + slab, bytes);
        const __amdgpu_buffer_rsrc_t rv = make_rsrc(v_ + slab, bytes);
        const __amdgpu_buffer_rsrc_t rg = make_rsrc(gy_ + slab, bytes);
        Raw Kr[L], Vr[L], Gr[L];
        float Ks[L], Vs[L];
        if (STAGED) {
            // this tile's rows have landed (loads and the previous tile's stores share one counter)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < L; ++j)                      // gy first: it must not queue behind the next tile's rows
                Gr[j] = BufRaw<sizeof(IO)>::template ld<CPOL_NT>(rg, voff0 + (unsigned)j * row, 0);
#pragma unroll
            for (int j = 0; j < L; ++j) { Ks[j] = stage[j * WAVE + lane]; Vs[j] = stage[(LR + j) * WAVE + lane]; }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // rows are in registers: the region is free
            if (next_tile < n_tiles) issue_stage(next_tile);
        } else {
#pragma unroll
            for (int j = 0; j < L; ++j) {
                const unsigned vo = voff0 + (unsigned)j * row;
                Kr[j] = BufRaw<sizeof(IO)>::template ld<CPOL_NT>(rk, vo, 0);
                Vr[j] = BufRaw<sizeof(IO)>::template ld<CPOL_NT>(rv, vo, 0);
            }
            if (MODE != 1) {
#pragma unroll
                for (int j = 0; j < L; ++j)
                    Gr[j] = BufRaw<sizeof(IO)>::template ld<CPOL_NT>(rg, voff0 + (unsigned)j * row, 0);
            }
        }

        const float gd = fast_exp2(-om), cu = fast_exp2(mu);
        const float G = fast_exp2(-om * (float)L);
        const float up_cap = floorf(plain_sum_up_cap(om, T));

        // ------------------------------ phase 1: the forward ------------------------------
        float E[L], V[L];
        float m = NEG_INF;
#pragma unroll
        for (int j = 0; j < L; ++j) {
            const float kk = STAGED ? Ks[j] : unpack1<IO>(Kr[j]);
            E[j] = (tw + j < T) ? kk : NEG_INF;               // tokens past T: k = -inf
            V[j] = STAGED ? ((tw + j < T) ? Vs[j] : 0.f) : unpack1<IO>(Vr[j]);   // staged rows past T are stale LDS
            m = fmaxf(m, E[j]);
        }
        const bool any = m > NEG_INF;
        const float Rw = any ? ceilf(m * LOG2E) : 0.f;
        float A = 0.f, Bd = 0.f, Cg = 0.f, Dg = 0.f;
#pragma unroll
        for (int j = 0; j < L; ++j) {
            E[j] = fast_exp2(fmaf(E[j], LOG2E, -Rw));
            A = fmaf(gd, A, E[j] * V[j]);
            Bd = fmaf(gd, Bd, E[j]);
        }
#pragma unroll
        for (int j = L - 1; j >= 0; --j) {
            Cg = fmaf(gd, Cg, E[j] * V[j]);
            Dg = fmaf(gd, Dg, E[j]);
        }
        s1[wave][0][lane] = A;
        s1[wave][1][lane] = Bd;
        s1[wave][2][lane] = any ? Rw : NEG_BIG;
        s1[wave][3][lane] = Cg;
        s1[wave][4][lane] = Dg;
        wg_barrier();

        float a = 0.f, bb = 0.f, c = 0.f, d = 0.f, Re, Rw_to_R;
        {
            float la[BWD_SMAX], lb[BWD_SMAX], lc[BWD_SMAX], ld[BWD_SMAX], lr[BWD_SMAX];
#pragma unroll
            for (int s = 0; s < BWD_SMAX; ++s) {
                // slots of waves the workgroup does not have hold stale data: read (constant LDS offsets), never used
                la[s] = s1[s][0][lane]; lb[s] = s1[s][1][lane]; lr[s] = s < S ? s1[s][2][lane] : NEG_BIG;
                lc[s] = s1[s][3][lane]; ld[s] = s1[s][4][lane];
            }
            float r = NEG_BIG;
            if (MODE >= 2) {
                r = s_in[wave][4][lane];
            } else {
#pragma unroll
                for (int s = 0; s < BWD_SMAX; ++s) r = fmaxf(r, lr[s]);
            }
            r = (r > NEG_BIG) ? r : 0.f;
            if (MODE == 1) {
                // fold the waves into the super-chunk's aggregates (both referenced to its ends) and publish
#pragma unroll
                for (int s = 0; s < BWD_SMAX; ++s)
                    if (s < S) {
                        const int sh = shift_of(lr[s] - r);
                        a = fmaf(G, a, ldexpf(la[s], sh));
                        bb = fmaf(G, bb, ldexpf(lb[s], sh));
                    }
#pragma unroll
                for (int s = BWD_SMAX - 1; s >= 0; --s)
                    if (s < S) {
                        const int sh = shift_of(lr[s] - r);
                        c = fmaf(G, c, ldexpf(lc[s], sh));
                        d = fmaf(G, d, ldexpf(ld[s], sh));
                    }
                if (wave == 0 && cok) {
                    a1(sc, 0) = a; a1(sc, 1) = bb; a1(sc, 2) = r; a1(sc, 3) = c; a1(sc, 4) = d;
                }
                wg_barrier();                                // s1 is rewritten by the next tile
                continue;
            }
            if (MODE >= 2) { a = s_in[wave][0][lane]; bb = s_in[wave][1][lane]; c = s_in[wave][2][lane]; d = s_in[wave][3][lane]; }
#pragma unroll
            for (int s = 0; s < BWD_SMAX; ++s)
                if (s < wave) {
                    const int sh = shift_of(lr[s] - r);
                    a = fmaf(G, a, ldexpf(la[s], sh));
                    bb = fmaf(G, bb, ldexpf(lb[s], sh));
                }
#pragma unroll
            for (int s = BWD_SMAX - 1; s >= 0; --s)
                if (s > wave && s < S) {
                    const int sh = shift_of(lr[s] - r);
                    c = fmaf(G, c, ldexpf(lc[s], sh));
                    d = fmaf(G, d, ldexpf(ld[s], sh));
                }
            Rw_to_R = r - Rw;
            const float upf = fminf(r - Rw, up_cap);
            const int up = (int)upf;
            a = ldexpf(a, up); bb = ldexpf(bb, up); c = ldexpf(c, up); d = ldexpf(d, up);
            Re = r - upf;                                     // the scale the carried terms really have
        }

        float Z[L], ZY[L];                                    // first N, D partials, then z and z*y
#pragma unroll
        for (int j = 0; j < L; ++j) {
            const float ev = E[j] * V[j];
            Z[j] = fmaf(cu, ev, a);
            ZY[j] = fmaf(cu, E[j], bb);
            a = fmaf(gd, a, ev);
            bb = fmaf(gd, bb, E[j]);
        }
        float gu_acc = 0.f, gw_acc = 0.f;
        ZScan fl;                                             // local future-side sums, zero carry
#pragma unroll
        for (int j = L - 1; j >= 0; --j) {
            const float ev = E[j] * V[j];
            const float rD = (tw + j < T) ? fast_rcp(ZY[j] + d) : 0.f;   // tokens past T contribute nothing
            const float y = (Z[j] + c) * rD;
            const float z = unpack1<IO>(Gr[j]) * rD;
            const float zy = z * y;
            c = fmaf(gd, c, ev);
            d = fmaf(gd, d, E[j]);
            Z[j] = z;
            ZY[j] = zy;
            gu_acc = fmaf(cu * E[j], fmaf(V[j], z, -zy), gu_acc);
            fl.push(gd, z, zy);
        }
        ZScan pl;                                             // local past-side sums
#pragma unroll
        for (int j = 0; j < L; ++j) pl.push(gd, Z[j], ZY[j]);

        if (MODE == 2) {
            // fold the waves' z-sums into one entry per super-chunk at the sequence's common scale 2^-R
            // (z 2^R = gy / (D 2^-R) stays within |gy| 2^+-50 under the plain-sum bound, so this is safe)
            s2[wave][0][lane] = pl.s0; s2[wave][1][lane] = pl.s1; s2[wave][2][lane] = pl.l0; s2[wave][3][lane] = pl.l1;
            s2[wave][4][lane] = fl.s0; s2[wave][5][lane] = fl.s1; s2[wave][6][lane] = fl.l0; s2[wave][7][lane] = fl.l1;
            s2[wave][8][lane] = Re;
            wg_barrier();
            if (wave == 0 && cok) {
                const float Rg = Re + fminf(Rw_to_R, up_cap);                 // = R (Re = R - min(R - Rw, up_cap))
                ZScan ps, fs;
                const float nL = (float)L;
                for (int sw = 0; sw < S; ++sw) {
                    const int sh = shift_of(Rg - s2[sw][8][lane]);
                    ps.hop(G, nL, ldexpf(s2[sw][0][lane], sh), ldexpf(s2[sw][1][lane], sh),
                           ldexpf(s2[sw][2][lane], sh), ldexpf(s2[sw][3][lane], sh));
                }
                for (int sw = S - 1; sw >= 0; --sw) {
                    const int sh = shift_of(Rg - s2[sw][8][lane]);
                    fs.hop(G, nL, ldexpf(s2[sw][4][lane], sh), ldexpf(s2[sw][5][lane], sh),
                           ldexpf(s2[sw][6][lane], sh), ldexpf(s2[sw][7][lane], sh));
                }
                a2(sc, 0) = ps.s0; a2(sc, 1) = ps.s1; a2(sc, 2) = ps.l0; a2(sc, 3) = ps.l1;
                a2(sc, 4) = fs.s0; a2(sc, 5) = fs.s1; a2(sc, 6) = fs.l0; a2(sc, 7) = fs.l1;
            }
            wg_barrier();                                    // s1, s2 are rewritten by the next tile
            continue;
        }

        // ------------------------------ phase 2: the adjoint ------------------------------
        s2[wave][0][lane] = pl.s0; s2[wave][1][lane] = pl.s1; s2[wave][2][lane] = pl.l0; s2[wave][3][lane] = pl.l1;
        s2[wave][4][lane] = fl.s0; s2[wave][5][lane] = fl.s1; s2[wave][6][lane] = fl.l0; s2[wave][7][lane] = fl.l1;
        s2[wave][8][lane] = Re;
        wg_barrier();

        ZScan p, f;
        {
            const float nL = (float)L;
            if (MODE == 3) {
                // the other super-chunks (their sums are at the common scale 2^-R), nearest last; then to my scale
                const float (*in)[WAVE] = s_in[wave];
                p.s0 = in[5][lane]; p.s1 = in[6][lane]; p.l0 = in[7][lane]; p.l1 = in[8][lane];
                f.s0 = in[9][lane]; f.s1 = in[10][lane]; f.l0 = in[11][lane]; f.l1 = in[12][lane];
                const int sh = shift_of(-Rw_to_R);                        // 2^(Rw - R) <= 1
                p.s0 = ldexpf(p.s0, sh); p.s1 = ldexpf(p.s1, sh); p.l0 = ldexpf(p.l0, sh); p.l1 = ldexpf(p.l1, sh);
                f.s0 = ldexpf(f.s0, sh); f.s1 = ldexpf(f.s1, sh); f.l0 = ldexpf(f.l0, sh); f.l1 = ldexpf(f.l1, sh);
            }
#pragma unroll
            for (int s = 0; s < BWD_SMAX; ++s)
                if (s < wave) {
                    const int sh = shift_of(Rw - s2[s][8][lane]);
                    p.hop(G, nL, ldexpf(s2[s][0][lane], sh), ldexpf(s2[s][1][lane], sh),
                          ldexpf(s2[s][2][lane], sh), ldexpf(s2[s][3][lane], sh));
                }
#pragma unroll
            for (int s = BWD_SMAX - 1; s >= 0; --s)
                if (s > wave && s < S) {
                    const int sh = shift_of(Rw - s2[s][8][lane]);
                    f.hop(G, nL, ldexpf(s2[s][4][lane], sh), ldexpf(s2[s][5][lane], sh),
                          ldexpf(s2[s][6][lane], sh), ldexpf(s2[s][7][lane], sh));
                }
        }
        float GV[L], GK[L];
#pragma unroll
        for (int j = 0; j < L; ++j) {
            GV[j] = fmaf(cu, Z[j], p.s0);
            GK[j] = fmaf(cu, ZY[j], p.s1);
            gw_acc = fmaf(-E[j], fmaf(V[j], p.l0, -p.l1), gw_acc);
            p.push(gd, Z[j], ZY[j]);
        }
        const __amdgpu_buffer_rsrc_t rgk = make_rsrc(gk_ + slab, bytes);
        const __amdgpu_buffer_rsrc_t rgv = make_rsrc(gv_ + slab, bytes);
        // the per-token offsets are formed again here (one add each) instead of staying in 28 registers since the loads
        unsigned vst = voff0;
        asm volatile("" : "+v"(vst));
#pragma unroll
        for (int j = L - 1; j >= 0; --j) {
            const float gv = E[j] * (GV[j] + f.s0);
            const float gk = fmaf(V[j], gv, -E[j] * (GK[j] + f.s1));
            gw_acc = fmaf(-E[j], fmaf(V[j], f.l0, -f.l1), gw_acc);
            f.push(gd, Z[j], ZY[j]);
            const unsigned vo = vst + (unsigned)j * row;      // tokens >= T fall outside the descriptor
            store1<IO>(rgv, vo, gv);
            store1<IO>(rgk, vo, gk);
        }

        // partial sums of gw, gu per (b, super-chunk, c): over this wave's tokens, then over the waves
        s3[wave][0][lane] = gw_acc;
        s3[wave][1][lane] = gu_acc;
        wg_barrier();
        if (wave == 0 && cok) {
            float sw = 0.f, su = 0.f;
            for (int s = 0; s < S; ++s) { sw += s3[s][0][lane]; su += s3[s][1][lane]; }
            gw_part[((size_t)b * nSC + sc) * C + c0] = sw;
            gu_part[((size_t)b * nSC + sc) * C + c0] = su;
        }
    }

    if (MODE == 1 || MODE == 2) return;
    // second walk: (batch, channel tile) pairs outside the plain-sum regime, one wave each, sequential form
    const int n_pairs = n_tiles / nSC;
    for (int pair = blockIdx.x * S + wave; pair < n_pairs; pair += gridDim.x * S) {
        const int ctile = pair % n_ctile, b = pair / n_ctile;
        const int c0 = ctile * WAVE + lane;
        const bool cok = c0 < C;
        const float om = (cok ? w_[c0] : 0.f) * LOG2E;
        const float mu = (cok ? u_[c0] : 0.f) * LOG2E;
        if (bwd_tile_is_fast(om, mu, T)) continue;
        if (cok) biwkv_bwd_serial_seq<IO>(w_, u_, k_, v_, gy_, gk_, gv_, ws, gw_part, gu_part, B, T, C, b, c0, nSC);
    }
}

}  // namespace biwkv_bwd_detail
}  // namespace vrwkv
