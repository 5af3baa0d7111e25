// Bi-WKV forward for gfx950: kernels and launch plan (included by one .hip file per I/O type).
//
// Computes, per batch b and channel c (w, u already divided by T by the caller),
//   y[t] = ( sum_{i!=t} e^{k_i - w(|t-i|-1)} v_i + e^{u+k_t} v_t ) / ( same with v -> 1 )
// i.e. the formula evaluated by the in-chunk recurrence of
// classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:93-108.
//
// Work decomposition (nothing like the reference's 32 token-chunks x 32 channels block):
//   lane      = one channel -> every load/store instruction of a wave touches one contiguous
//               64-channel row segment of k, v or y;
//   wave      = L consecutive tokens of those channels, held in registers;
//   workgroup = S <= 8 waves = S*L consecutive tokens (a "super-chunk") of 64 channels;
//   tile      = (batch, super-chunk, channel tile); workgroups are persistent and walk the
//               tiles with stride gridDim.x, loading tile n+1 into a second register set
//               while tile n is being computed, so HBM traffic overlaps the arithmetic.
// k and v are read from HBM once: a wave keeps its L tokens in VGPRs between the
// aggregate phase and the emit phase.  Only when T exceeds what one workgroup can hold
// does a first kernel publish per-super-chunk aggregates to a small workspace and the
// main kernel read the tokens a second time.
// All tensor accesses are raw buffer loads/stores on a per-batch-element descriptor, so
// tokens past T and channels past C are dropped by the hardware range check instead of
// by exec-mask branches; the streamed tensors use the non-temporal cache policy.
//
// Arithmetic is in the log2 domain (kappa = k*log2e, omega = w*log2e, mu = u*log2e) so
// that every exponential is one v_exp_f32.
//
// Two code paths, chosen per tile from (w, u, T) alone and therefore identically by
// every wave that touches a channel tile:
//   fast   |omega|*(T+1) + |mu| <= 40, and for negative omega (weights that grow with distance) |omega|*(T+1) <= 16.
//          Each wave uses its own integer reference exponent
//          Rw = ceil(max kappa) over its tokens; E_t = 2^(kappa_t-Rw) <= 1 is computed once per
//          token and reused by both directions and both phases; states are plain decayed sums
//          a <- g*a + E_t v_t (g = 2^-omega), no per-token max.  Waves exchange their chunk
//          aggregates once per tile and rescale each other's by exact powers of two.  A carried sum is at
//          most T * 2^growth (growth = max(0, -omega) (T+1) <= 16) in units of the largest wave scale, and the
//          shift that brings it to a wave's own scale is capped (plain_sum_up_cap) so that it stays below
//          2^96 |v|: nothing overflows, and a term that the cap or an underflow drops is below 2^-27 of its
//          denominator.
//   robust anything else: every state is a (num, den, exponent) triple renormalised at
//          every token, exactly the reference's recurrence, for both directions; those tiles
//          are done in a second walk after the fast ones.
#pragma once
#include "vrwkv_common.h"

namespace vrwkv {
namespace biwkv_fwd_detail {

constexpr float FAST_LIMIT = 40.0f;
constexpr float GROW_LIMIT = 16.0f;

// True when a channel is outside the plain-sum regime (log2 units: om = w log2e, mu = u log2e).
__device__ __forceinline__ bool outside_plain_sum(float om, float mu, int T) {
    const float span = fabsf(om) * (float)(T + 1);
    return !(span + fabsf(mu) <= FAST_LIMIT) || (om < 0.f && span > GROW_LIMIT);
}
// Upper limit of the exponent by which a carried sum is raised from the common scale 2^R to a wave's own scale
// 2^Rw: the sum is at most T 2^growth |v| in units of 2^R, so below 2^96 |v| afterwards.  Past the limit the wave's
// own terms are negligible against the carry (the carry has decayed by at most 2^-40), so the limit only keeps
// fp32 finite.
__device__ __forceinline__ float plain_sum_up_cap(float om, int T) {
    return 96.f - fmaxf(-om, 0.f) * (float)(T + 1) - __builtin_amdgcn_logf((float)T);
}
constexpr int NSLOT = 6;   // workspace floats per (b, super-chunk, channel): A, B, pA|R, Cg, D, pC

// Waves per workgroup: at most 8, i.e. two per SIMD, which leaves every wave 256 VGPRs -- enough
// for the longest chunk (28 tokens: k, v, two partial arrays and the prefetched k, v of the next
// tile, about 7 floats per token) without spilling.
constexpr int smax_for(int L, int VEC) {
    return (7 * L * VEC + 40 <= 256) ? 8 : 4;
}

// state <- decay-by-one-token(state) (+) token, all exponents in log2 units.
__device__ __forceinline__ void tri_push(float& a, float& b, float& p, float om, float kap, float v) {
    const float pw = fmaxf(p - om, NEG_BIG);
    const float q = fmaxf(pw, kap);
    const float e1 = fast_exp2(pw - q);
    const float e2 = fast_exp2(kap - q);
    a = e1 * a + e2 * v;
    b = e1 * b + e2;
    p = q;
}
// state <- decay-by-n-tokens(state) (+) other triple
__device__ __forceinline__ void tri_merge(float& a, float& b, float& p, float om_n,
                                          float a2, float b2, float p2) {
    const float pw = fmaxf(p - om_n, NEG_BIG);
    const float q = fmaxf(pw, p2);
    const float e1 = fast_exp2(pw - q);
    const float e2 = fast_exp2(p2 - q);
    a = e1 * a + e2 * a2;
    b = e1 * b + e2 * b2;
    p = q;
}

// Raw (still packed) registers of one token: converted to fp32 only when consumed, so a
// prefetched 16-bit tile costs half the registers.
template <typename IO, int VEC> struct Packed { typename BufRaw<sizeof(IO) * VEC>::type raw; };

template <typename IO, int VEC>
__device__ __forceinline__ void unpack(const Packed<IO, VEC>& p, float (&out)[VEC]) {
    IO tmp[VEC];
    __builtin_memcpy(tmp, &p.raw, sizeof(p.raw));
#pragma unroll
    for (int e = 0; e < VEC; ++e) out[e] = to_f32(tmp[e]);
}
template <typename IO, int VEC>
__device__ __forceinline__ void buf_store(__amdgpu_buffer_rsrc_t r, unsigned voff, const float (&in)[VEC]) {
    IO tmp[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) tmp[e] = from_f32<IO>(in[e]);
    typename BufRaw<sizeof(IO) * VEC>::type raw;
    __builtin_memcpy(&raw, tmp, sizeof(raw));
    BufRaw<sizeof(IO) * VEC>::template st<CPOL_NT>(raw, r, voff, 0);
}

struct TileGeom {
    int n_ctile, nSC, n_tiles;      // tile id = (b * nSC + sc) * n_ctile + ctile
};

// MODE 0: whole sequence in one workgroup.  MODE 1: aggregate-only pass of the long-
// sequence path (writes the workspace).  MODE 2: emit pass of the long-sequence path.
// STAGED (C a multiple of the 4 or 8 elements in 16 bytes, 16-byte aligned k, v, y): a tile's k, v rows are fetched as 16-byte pieces straight
// into LDS (buffer_load ... lds, no registers, 1 KB contiguous per wave instruction instead of 256 B) while the
// previous tile is computed, and each wave then reads its own rows back lane-per-channel.
// GATE: the emitted rows leave as sigmoid(r) * y (the receptance gate of vrwkv.py:186 applied before the store); r is
// fetched lane-per-channel at the top of the tile, ahead of the next tile's rows, and waits packed in registers.
template <typename IO, int VEC, int L, int MODE, bool STAGED = false, bool GATE = false>
struct BiwkvTile {
    static_assert(!GATE || (VEC == 1 && MODE != 1), "the gate is applied where y is emitted, one channel per lane");
    static constexpr int SMAX = smax_for(L, VEC);
    static constexpr int CH = WAVE * VEC;
    using P = Packed<IO, VEC>;
    typedef float (*AggPtr)[NSLOT][CH];
    // staging geometry: a lane moves 16 bytes = EPL elements; LPR lanes cover a 64-channel row; an instruction RPI rows
    static constexpr int EPL = 16 / (int)sizeof(IO), LPR = WAVE / EPL, RPI = WAVE / LPR;
    static constexpr int NI = (L + RPI - 1) / RPI, LR = NI * RPI;         // instructions and LDS rows per tensor
    // The wait for the next tile's rows stands before this tile's first store (loads and stores share one counter:
    // a wait at the top of the next tile would also wait for the stores issued a moment before it).
    static constexpr bool EARLY_WAIT = true;
    // s_waitcnt vmcnt(0) as an instruction the compiler's own wait-count bookkeeping sees (it does not look into
    // inline assembly and would add a wait of its own in front of the next read of a staged row)
    static __device__ __forceinline__ void wait_vm0() {
        __builtin_amdgcn_s_waitcnt(0x0F70);                               // vmcnt = 0, expcnt and lgkmcnt untouched
        asm volatile("" ::: "memory");
    }
    // 16-bit y goes out in 16-byte pieces as well (through an LDS array of its own: an LDS read waits for every
    // LDS-direct load that may write the array it reads).  fp32 y keeps its lane-per-channel 256-byte row stores:
    // parked in LDS and flushed eight rows at a time it measured 2 % slower (24.6 vs 24.1 us at 64 x 196 x 768), the
    // extra LDS round trip costing more than the wider stores save.
    static constexpr bool OUT_STAGED = STAGED && sizeof(IO) == 2;
    static constexpr int STAGE_ELEMS = 2 * LR * WAVE;                     // per wave: k rows, v rows
    static constexpr int YSTAGE_ELEMS = OUT_STAGED ? LR * WAVE : 8;       // per wave: y rows

    const float* __restrict__ w_;
    const float* __restrict__ u_;
    const IO* __restrict__ k_;
    const IO* __restrict__ v_;
    const IO* __restrict__ r_;  // GATE: receptance (B,T,C)
    IO* __restrict__ y_;
    float* __restrict__ ws;
    int T, C;
    TileGeom g;
    int lane, wave, S;
    AggPtr s_agg0, s_agg1;      // two LDS exchange buffers, alternated tile by tile
    float (*s_fold)[WAVE];      // MODE 2: [2][6][64] what the other super-chunks contribute, alternated like s_agg
    IO* s_stage;                // STAGED: this wave's LDS rows [LR][64] of k, then v
    IO* s_y;                    // STAGED: this wave's LDS rows [YR][64] of y

    struct Where {
        int b, sc, ctile, c0, tw;
        bool cok;
        unsigned voff0;          // byte offset of this lane's first token inside the batch slab
        size_t slab;             // element offset of the batch slab
    };

    __device__ __forceinline__ Where locate(int tile) const {
        Where q;
        q.ctile = tile % g.n_ctile;
        const int r = tile / g.n_ctile;
        q.sc = r % g.nSC;
        q.b = r / g.nSC;
        q.c0 = (q.ctile * WAVE + lane) * VEC;
        q.cok = q.c0 < C;
        q.tw = (q.sc * S + wave) * L;
        q.voff0 = q.cok ? (unsigned)(((size_t)q.tw * C + q.c0) * sizeof(IO)) : OOB_OFFSET;
        q.slab = (size_t)q.b * T * C;
        return q;
    }

    // Per-lane parameters of a tile, fetched together with its tokens so that consuming them
    // never has to wait for the previous tile's stores.
    // MODE 2 also fetches, together with a tile's parameters, the workspace entries of the other super-chunks of its
    // sequence: wave 0 those of the earlier super-chunks (farthest first), wave 1 those of the later ones (farthest
    // first), up to NBF each -- a whole tile ahead, so that folding them (fold_others) waits for no memory round trip.
    static constexpr int NBF = MODE == 2 ? 16 : 1;
    struct WU { float w[VEC], u[VEC]; float fr[NBF], f0[NBF], f1[NBF]; };

    // super-chunk whose entry is the i-th one folded by `wave` (0: earlier ones ascending, 1: later ones descending)
    __device__ __forceinline__ int fold_source(int i) const { return wave == 0 ? i : g.nSC - 1 - i; }
    __device__ __forceinline__ float table_entry(const Where& q, int se, int slot) const {
        // one descriptor over the batch element's table, the entry's offset in the scalar operand
        const __amdgpu_buffer_rsrc_t rtab = make_rsrc(ws + (size_t)q.b * g.nSC * NSLOT * C, (unsigned)((size_t)g.nSC * NSLOT * C * 4));
        const unsigned vcol = q.cok ? (unsigned)q.c0 * 4u : OOB_OFFSET;
        return __builtin_bit_cast(float, BufRaw<4>::ld(rtab, vcol, (unsigned)((se * NSLOT + slot) * C) * 4u));
    }

    __device__ __forceinline__ void issue_wu(int tile, WU& wu) const {
        const Where q = locate(tile);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            wu.w[e] = q.cok ? w_[q.c0 + e] : 0.f;
            wu.u[e] = q.cok ? u_[q.c0 + e] : 0.f;
        }
        if (MODE == 2 && wave < 2) {                     // wave-uniform
#pragma unroll
            for (int i = 0; i < NBF; ++i) {
                int se = fold_source(i);                 // past the ends: clamped to an entry that exists, not used
                se = se < 0 ? 0 : (se >= g.nSC ? g.nSC - 1 : se);
                wu.fr[i] = table_entry(q, se, 2);
                wu.f0[i] = table_entry(q, se, wave == 0 ? 0 : 3);
                wu.f1[i] = table_entry(q, se, wave == 0 ? 1 : 4);
            }
        }
    }

    // MODE 2, waves 0 and 1: what the other super-chunks contribute to this tile -- wave 0: (A, B) of the earlier ones
    // decayed to this super-chunk's first token; wave 1: (C, D) of the later ones decayed to its last -- left in LDS
    // (s_fold[par]) for every wave to pick up after the tile's barrier.  The sum is kept at the running maximum of
    // the scales met so far (all scales are integers, so re-scaling is an exact ldexp).
    __device__ __forceinline__ void fold_others(const Where& q, const WU& wu, float om, int par) const {
        auto shift_of = [](float r_from, float r_to) -> int { return (int)fmaxf(r_from - r_to, -300.f); };
        const int n = wave == 0 ? q.sc : g.nSC - 1 - q.sc;               // entries to fold
        const float GS = fast_exp2(-om * (float)(S * L));
        float r1 = NEG_BIG, aa = 0.f, ab = 0.f;
        auto push = [&](float tr, float t0, float t1) {
            const float m = fmaxf(r1, tr);
            const int so = shift_of(r1, m), sn = shift_of(tr, m);
            aa = fmaf(GS, ldexpf(aa, so), ldexpf(t0, sn));
            ab = fmaf(GS, ldexpf(ab, so), ldexpf(t1, sn));
            r1 = m;
        };
#pragma unroll
        for (int i = 0; i < NBF; ++i)
            if (i < n) push(wu.fr[i], wu.f0[i], wu.f1[i]);               // wave-uniform
        for (int i0 = NBF; i0 < n; i0 += 8) {                            // longer sequences: the rest, eight at a time
            float tr[8], t0[8], t1[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int se = fold_source(i0 + i);
                se = se < 0 ? 0 : (se >= g.nSC ? g.nSC - 1 : se);
                tr[i] = table_entry(q, se, 2);
                t0[i] = table_entry(q, se, wave == 0 ? 0 : 3);
                t1[i] = table_entry(q, se, wave == 0 ? 1 : 4);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i0 + i < n) push(tr[i], t0[i], t1[i]);
        }
        float (*f)[WAVE] = s_fold + (par * 6 + wave * 3);
        f[0][lane] = r1; f[1][lane] = aa; f[2][lane] = ab;
    }
    static __device__ __forceinline__ typename BufRaw<sizeof(IO) * VEC>::type load_raw(__amdgpu_buffer_rsrc_t r, unsigned vo) {
        return BufRaw<sizeof(IO) * VEC>::template ld<CPOL_NT>(r, vo, 0);
    }
    // GATE: this lane's r values of the tile (tokens past T read as zero and are never stored)
    __device__ __forceinline__ void issue_gate(const Where& q, unsigned row, typename BufRaw<sizeof(IO)>::type (&Rr)[GATE ? L : 1]) const {
        if constexpr (GATE) {
            const __amdgpu_buffer_rsrc_t rr = make_rsrc(r_ + q.slab, (unsigned)((size_t)T * C * sizeof(IO)));
#pragma unroll
            for (int j = 0; j < L; ++j) Rr[j] = BufRaw<sizeof(IO)>::template ld<CPOL_NT>(rr, q.voff0 + (unsigned)j * row, 0);
        }
    }
    static __device__ __forceinline__ float gate_of(typename BufRaw<sizeof(IO)>::type raw) {
        IO t;
        __builtin_memcpy(&t, &raw, sizeof(t));
        return fast_rcp(1.f + fast_exp2(-to_f32(t) * LOG2E));
    }
    __device__ __forceinline__ void issue_loads(int tile, P (&K)[L], P (&V)[L], WU& wu) const {
        issue_wu(tile, wu);
        const Where q = locate(tile);
        const unsigned bytes = (unsigned)((size_t)T * C * sizeof(IO));
        const __amdgpu_buffer_rsrc_t rk = make_rsrc(k_ + q.slab, bytes);
        const __amdgpu_buffer_rsrc_t rv = make_rsrc(v_ + q.slab, bytes);
        const unsigned row = (unsigned)(C * sizeof(IO));
#pragma unroll
        for (int j = 0; j < L; ++j) {
            const unsigned vo = q.voff0 + (unsigned)j * row;
            K[j].raw = load_raw(rk, vo);
            V[j].raw = load_raw(rv, vo);
        }
    }

    // STAGED: this wave's L rows of k and v of `tile`, RPI rows per instruction (lane = row l/LPR, EPL channels),
    // land in s_stage as [row][64 channels]; rows past T and channels past C are dropped by the range check.
    __device__ __forceinline__ void issue_stage(int tile, WU& wu) const {
        issue_wu(tile, wu);
        issue_stage_rows(tile, 0, NI);
    }
    // instructions [i0, i1) of the NI that stage a tile's rows
    __device__ __forceinline__ void issue_stage_rows(int tile, int i0, int i1) const {
        const Where q = locate(tile);
        const unsigned bytes = (unsigned)((size_t)T * C * sizeof(IO));
        const __amdgpu_buffer_rsrc_t rk = make_rsrc(k_ + q.slab, bytes);
        const __amdgpu_buffer_rsrc_t rv = make_rsrc(v_ + q.slab, bytes);
        const int cq = q.ctile * WAVE + (lane % LPR) * EPL;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            if (i < i0 || i >= i1) continue;
            const int rl = RPI * i + lane / LPR;                          // row inside this wave's chunk
            const int row = q.tw + rl;
            const unsigned vo = (rl < L && row < T && cq < C) ? (unsigned)(((size_t)row * C + cq) * sizeof(IO)) : OOB_OFFSET;
            typedef __attribute__((address_space(3))) void* lds_ptr;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)(s_stage + i * RPI * WAVE), 16, vo, 0, 0, CPOL_NT);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (lds_ptr)(s_stage + (LR + i * RPI) * WAVE), 16, vo, 0, 0, CPOL_NT);
        }
    }
    // One-launch kernel, 16-bit rows: the next tile's rows are requested in two halves, the second behind the exchange
    // barrier (16.2 -> 15.9 us at 64 x 196 x 768; fp32 rows: no difference with two portions, slower with four).
    static constexpr int STAGE_PARTS = (STAGED && MODE == 0 && sizeof(IO) == 2) ? 2 : 1;
    __device__ __forceinline__ void issue_stage_part(int next, int part, WU& wun) const {
        constexpr int NP = STAGE_PARTS;
        if (next >= g.n_tiles || part >= NP) return;
        if (part == 0) issue_wu(next, wun);
        issue_stage_rows(next, NI * part / NP, NI * (part + 1) / NP);
    }

    // Computes one tile from the packed registers K, V; in the middle (once K, V have been
    // consumed) issues the loads of `next` into Kn, Vn when next < n_tiles.
    // True when any channel of the tile is outside the plain-sum regime (wave-uniform, and the
    // same for every wave and every super-chunk of a channel tile).
    __device__ __forceinline__ bool tile_is_robust(const WU& wu, float (&om)[VEC], float (&mu)[VEC]) const {
        bool bad = false;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            om[e] = wu.w[e] * LOG2E;
            mu[e] = wu.u[e] * LOG2E;
            bad = bad || outside_plain_sum(om[e], mu[e], T);
        }
        return __builtin_amdgcn_ballot_w64(bad) != 0ull;
    }

    // Fast path of one tile from the packed registers K, V; in the middle (once K, V have been
    // consumed) issues the loads of `next` into Kn, Vn when next < n_tiles.  Tiles that need
    // the robust path are skipped here and handled by run_robust() afterwards.
    // Consecutive tiles alternate between the two LDS buffers (`par`), so one barrier per
    // exchange is enough: a wave can only write buffer `par` again after passing the barrier of
    // the tile in between (a skipped tile has one too), which every wave reaches after its last
    // read of this tile.
    __device__ __forceinline__ void run(int tile, int next, int par, P (&K)[L], P (&V)[L], const WU& wu,
                                        P (&Kn)[L], P (&Vn)[L], WU& wun) const {
        const Where q = locate(tile);
        const AggPtr s_agg = par ? s_agg1 : s_agg0;
        const float NEG_INF = -__builtin_inff();
        const int nSC = g.nSC;
        const int li = lane * VEC;
        const int round = tile / (int)gridDim.x + (MODE == 1 ? 2 : 0);   // which of this workgroup's tiles (cycle stamps;
                                                                         // the aggregate-only pass uses slots 2, 3)
        (void)round;
        VRWKV_STAMP(wave, round, 0);                      // tile entered

        float om[VEC], mu[VEC];
        if (tile_is_robust(wu, om, mu)) {
            // workgroup-uniform branch; the barrier stands in for the exchange barrier of a computed tile
            if (STAGED) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); else lds_barrier();
            if (next < g.n_tiles) {
                if (STAGED) {
                    if (!EARLY_WAIT) wait_vm0();                          // the skipped tile's rows must have landed
                    issue_stage(next, wun);
                    if (EARLY_WAIT) wait_vm0();                           // ... and the next tile's, before its turn
                } else {
                    issue_loads(next, Kn, Vn, wun);
                }
            }
            return;
        }

        const unsigned row = (unsigned)(C * sizeof(IO));
        const __amdgpu_buffer_rsrc_t ry = make_rsrc(y_ + q.slab, (unsigned)((size_t)T * C * sizeof(IO)));
        const size_t ws_b = (size_t)q.b * nSC * NSLOT * C;
        auto ws_at = [&](int s, int slot, int e) -> float& {
            return ws[ws_b + ((size_t)s * NSLOT + slot) * C + q.c0 + e];
        };
        // The next tile is fetched a token at a time behind the arithmetic (k during the
        // aggregate pass, v during the ascending sweep): few vector-memory instructions are
        // outstanding per CU at any moment, so issuing them never stalls the wave for long.
        const bool have_next = next < g.n_tiles && !STAGED;          // register prefetch of the next tile
        const Where qn = locate(have_next ? next : tile);
        const __amdgpu_buffer_rsrc_t rkn = make_rsrc(k_ + qn.slab, (unsigned)((size_t)T * C * sizeof(IO)));
        const __amdgpu_buffer_rsrc_t rvn = make_rsrc(v_ + qn.slab, (unsigned)((size_t)T * C * sizeof(IO)));
        if (have_next) issue_wu(next, wun);

        auto shift_of = [](float r_from, float r_to) -> int { return (int)fmaxf(r_from - r_to, -300.f); };
        // MODE 2: what the other super-chunks contribute is folded by waves 0 and 1 from entries fetched a tile ago
        float ra[VEC], rc[VEC], ca[VEC], cb[VEC], cc[VEC], cd[VEC];
        if (MODE == 2 && wave < 2) fold_others(q, wu, om[0], par);
        VRWKV_STAMP(wave, round, 1);                      // other super-chunks folded (MODE 2)
        // unpack; tokens past T read as zero from the buffer and get k = -inf here
        float X0[L][VEC], X1[L][VEC];                    // k / v, later E / E*v
        typename BufRaw<sizeof(IO)>::type Rr[GATE ? L : 1];              // GATE: this lane's r, packed
        if (STAGED) {
            // This tile's rows have landed: the wait for them stands before the previous tile's first store (and
            // before the loop for the first tile).  Loads and stores share one counter and may retire in either
            // order, so a wait here would also wait for the stores that were issued a moment ago.
            if (!EARLY_WAIT) wait_vm0();
            if (q.tw + L <= T) {                         // wave-uniform: every token of the chunk exists
#pragma unroll
                for (int j = 0; j < L; ++j) {
                    X0[j][0] = to_f32(s_stage[j * WAVE + lane]);
                    X1[j][0] = to_f32(s_stage[(LR + j) * WAVE + lane]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < L; ++j) {
                    const bool tok = q.tw + j < T;
                    const float kk = to_f32(s_stage[j * WAVE + lane]), vv = to_f32(s_stage[(LR + j) * WAVE + lane]);
                    X0[j][0] = tok ? kk : NEG_INF;
                    X1[j][0] = tok ? vv : 0.f;           // rows past T were not written: LDS holds stale bits
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // rows are in registers: the region is free
            VRWKV_STAMP(wave, round, 2);                                  // rows copied from LDS
            issue_gate(q, row, Rr);                                       // first: it must not queue behind the next tile's rows
            if (STAGE_PARTS > 1) issue_stage_part(next, 0, wun);
            else if (next < g.n_tiles) issue_stage(next, wun);
            VRWKV_STAMP(wave, round, 3);                                  // next tile's loads issued
        } else {
#pragma unroll
            for (int j = 0; j < L; ++j) {
                unpack<IO, VEC>(K[j], X0[j]);
                unpack<IO, VEC>(V[j], X1[j]);
                const bool tok = q.tw + j < T;               // wave-uniform
#pragma unroll
                for (int e = 0; e < VEC; ++e) X0[j][e] = tok ? X0[j][e] : NEG_INF;
            }
            issue_gate(q, row, Rr);
        }

        // ================================== fast path ==================================
        // ONE workgroup barrier per tile:
        //  1. the wave takes its own reference exponent Rw = ceil(max kappa over its L tokens),
        //     forms E = 2^(kappa-Rw) <= 1 and E*v, and its two chunk aggregates in units of 2^Rw;
        //  2. it publishes (A, B, Cg, D, Rw); barrier; every wave reads all S entries at once;
        //  3. R = max Rw.  All Rw are integers, so bringing another wave's aggregate to the common
        //     scale is an exact ldexp (no exponential); the carry-in is accumulated at scale 2^R
        //     and then shifted to the wave's own scale 2^Rw, in which the sweeps run unchanged
        //     (y is a ratio, the scale cancels).  The shift is capped (plain_sum_up_cap).
        float gd[VEC], Rw[VEC], Rpub[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            gd[e] = fast_exp2(-om[e]);
            float m = NEG_INF;
#pragma unroll
            for (int j = 0; j < L; ++j) m = fmaxf(m, X0[j][e]);
            const bool any = m > NEG_INF;
            Rw[e] = any ? ceilf(m * LOG2E) : 0.f;
            Rpub[e] = any ? Rw[e] : NEG_BIG;              // a wave with no token must not set the scale
        }
        float A[VEC], Bd[VEC], Cg[VEC], D[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) { A[e] = 0.f; Bd[e] = 0.f; Cg[e] = 0.f; D[e] = 0.f; }
#pragma unroll
        for (int j = 0; j < L; ++j) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                // one rounding for k*log2e - Rw: the heaviest tokens have the smallest argument
                const float E = fast_exp2(fmaf(X0[j][e], LOG2E, -Rw[e]));
                X0[j][e] = E;
                X1[j][e] = E * X1[j][e];
                A[e] = fmaf(gd[e], A[e], X1[j][e]);       // referenced to the chunk end
                Bd[e] = fmaf(gd[e], Bd[e], E);
            }
            if (have_next) Kn[j].raw = load_raw(rkn, qn.voff0 + (unsigned)j * row);
        }
#pragma unroll
        for (int j = L - 1; j >= 0; --j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                Cg[e] = fmaf(gd[e], Cg[e], X1[j][e]);      // referenced to the chunk start
                D[e] = fmaf(gd[e], D[e], X0[j][e]);
            }
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            s_agg[wave][0][li + e] = A[e];
            s_agg[wave][1][li + e] = Bd[e];
            s_agg[wave][2][li + e] = Rpub[e];
            s_agg[wave][3][li + e] = Cg[e];
            s_agg[wave][4][li + e] = D[e];
        }
        VRWKV_STAMP(wave, round, 4);                      // aggregate pass done, aggregates written
        if (STAGED) {
            // LDS-only barrier by hand: the fence form would also wait for the next tile's staging loads
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        } else {
            lds_barrier();
        }
        VRWKV_STAMP(wave, round, 5);                      // barrier passed
        if (STAGE_PARTS > 1) issue_stage_part(next, 1, wun);

        if (MODE == 2) {
            static_assert(MODE != 2 || VEC == 1, "the long-sequence emit pass handles one channel per lane");
            const float (*f)[WAVE] = s_fold + par * 6;
            ra[0] = f[0][lane]; ca[0] = f[1][lane]; cb[0] = f[2][lane];
            rc[0] = f[3][lane]; cc[0] = f[4][lane]; cd[0] = f[5][lane];
        }
        float G[VEC];                                     // decay over one wave's chunk
#pragma unroll
        for (int e = 0; e < VEC; ++e) G[e] = fast_exp2(-om[e] * (float)L);
        float a[VEC], bb[VEC], c[VEC], d[VEC], R[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            // all reads are issued before the dependent steps (one LDS latency, not S of them)
            float la[SMAX], lb[SMAX], lc[SMAX], ld[SMAX], lr[SMAX];
#pragma unroll
            for (int s = 0; s < SMAX; ++s) {
                const int ss = s < S ? s : S - 1;
                la[s] = s_agg[ss][0][li + e];
                lb[s] = s_agg[ss][1][li + e];
                lr[s] = s_agg[ss][2][li + e];
                lc[s] = s_agg[ss][3][li + e];
                ld[s] = s_agg[ss][4][li + e];
            }
            float r = NEG_BIG;
#pragma unroll
            for (int s = 0; s < SMAX; ++s) r = fmaxf(r, lr[s]);
            if (MODE == 2) r = fmaxf(r, fmaxf(ra[e], rc[e]));
            r = (r > NEG_BIG) ? r : 0.f;
            R[e] = r;
            float aa = 0.f, ab = 0.f, ac = 0.f, ad = 0.f;
            if (MODE == 1) {
                // fold all S wave aggregates into the super-chunk aggregate (published by wave 0)
#pragma unroll
                for (int s = 0; s < SMAX; ++s)
                    if (s < S) {
                        const int sh = shift_of(lr[s], r);
                        aa = fmaf(G[e], aa, ldexpf(la[s], sh));
                        ab = fmaf(G[e], ab, ldexpf(lb[s], sh));
                    }
#pragma unroll
                for (int s = SMAX - 1; s >= 0; --s)
                    if (s < S) {
                        const int sh = shift_of(lr[s], r);
                        ac = fmaf(G[e], ac, ldexpf(lc[s], sh));
                        ad = fmaf(G[e], ad, ldexpf(ld[s], sh));
                    }
            } else {
                if (MODE == 2) {
                    const int s1 = shift_of(ra[e], r), s2 = shift_of(rc[e], r);
                    aa = ldexpf(ca[e], s1); ab = ldexpf(cb[e], s1); ac = ldexpf(cc[e], s2); ad = ldexpf(cd[e], s2);
                }
#pragma unroll
                for (int s = 0; s < SMAX; ++s)
                    if (s < wave) {                      // wave-uniform
                        const int sh = shift_of(lr[s], r);
                        aa = fmaf(G[e], aa, ldexpf(la[s], sh));
                        ab = fmaf(G[e], ab, ldexpf(lb[s], sh));
                    }
#pragma unroll
                for (int s = SMAX - 1; s >= 0; --s)
                    if (s > wave && s < S) {
                        const int sh = shift_of(lr[s], r);
                        ac = fmaf(G[e], ac, ldexpf(lc[s], sh));
                        ad = fmaf(G[e], ad, ldexpf(ld[s], sh));
                    }
                // to the wave's own scale
                const int up = (int)fminf(r - Rw[e], plain_sum_up_cap(om[e], T));
                aa = ldexpf(aa, up); ab = ldexpf(ab, up); ac = ldexpf(ac, up); ad = ldexpf(ad, up);
            }
            a[e] = aa; bb[e] = ab; c[e] = ac; d[e] = ad;
        }

        if (MODE == 1) {
            if (wave == 0 && q.cok) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    ws_at(q.sc, 0, e) = a[e];
                    ws_at(q.sc, 1, e) = bb[e];
                    ws_at(q.sc, 2, e) = R[e];
                    ws_at(q.sc, 3, e) = c[e];
                    ws_at(q.sc, 4, e) = d[e];
                    ws_at(q.sc, 5, e) = R[e];
                }
            }
            if (have_next) {
#pragma unroll
                for (int j = 0; j < L; ++j) Vn[j].raw = load_raw(rvn, qn.voff0 + (unsigned)j * row);
            }
            VRWKV_STAMP(wave, round, 8);
            if (STAGED && EARLY_WAIT) wait_vm0();                         // the next tile's rows
            VRWKV_STAMP(wave, round, 9);
            return;
        }

        VRWKV_STAMP(wave, round, 6);                      // carries formed
        // emit: ascending sweep leaves past + bonus partials, descending sweep adds the future
        float cu[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) cu[e] = fast_exp2(mu[e]);
        float PN[L][VEC], PD[L][VEC];
#pragma unroll
        for (int j = 0; j < L; ++j) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                PN[j][e] = fmaf(cu[e], X1[j][e], a[e]);
                PD[j][e] = fmaf(cu[e], X0[j][e], bb[e]);
                a[e] = fmaf(gd[e], a[e], X1[j][e]);
                bb[e] = fmaf(gd[e], bb[e], X0[j][e]);
            }
            if (have_next) Vn[j].raw = load_raw(rvn, qn.voff0 + (unsigned)j * row);
        }
        VRWKV_STAMP(wave, round, 7);                      // ascending sweep done
#pragma unroll
        for (int j = L - 1; j >= 0; --j) {
            float out[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                out[e] = (PN[j][e] + c[e]) * fast_rcp(PD[j][e] + d[e]);
                c[e] = fmaf(gd[e], c[e], X1[j][e]);
                d[e] = fmaf(gd[e], d[e], X0[j][e]);
            }
            if (GATE) out[0] *= gate_of(Rr[j]);
            // the next tile's rows must have landed before this tile's first store joins them in the queue
            if (STAGED && EARLY_WAIT && j == (OUT_STAGED ? 0 : L - 1)) {
                VRWKV_STAMP(wave, round, 8);              // (16-bit: descending sweep done) waiting for the next tile's rows
                wait_vm0();
                VRWKV_STAMP(wave, round, 9);              // next tile's rows have landed
            }
            if (OUT_STAGED) {
                s_y[j * WAVE + lane] = from_f32<IO>(out[0]);
                if (j == 0) flush_y(q, ry);
            } else {
                buf_store<IO, VEC>(ry, q.voff0 + (unsigned)j * row, out);   // tokens >= T fall outside the descriptor
            }
        }
        VRWKV_STAMP(wave, round, 10);                     // descending sweep done, stores issued
    }

    // The y rows of this wave's chunk, parked lane-per-channel in the y region, leave as 16-byte pieces (RPI rows per
    // store instruction); the region may be rewritten afterwards.
    __device__ __forceinline__ void flush_y(const Where& q, __amdgpu_buffer_rsrc_t ry) const {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const int cq = q.ctile * WAVE + (lane % LPR) * EPL;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            {
                const int rl = RPI * i + lane / LPR;
                const int rowt = q.tw + rl;
                const unsigned vo = (rl < L && rowt < T && cq < C) ? (unsigned)(((size_t)rowt * C + cq) * sizeof(IO)) : OOB_OFFSET;
                const BufRaw<16>::type val = *reinterpret_cast<const BufRaw<16>::type*>(s_y + rl * WAVE + (lane % LPR) * EPL);
                BufRaw<16>::template st<CPOL_NT>(val, ry, vo, 0);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                // the rows are read before they are rewritten
    }

    // Robust path of one tile, self-contained (own loads, no prefetch); a no-op for tiles the
    // fast path has already done.  Ends with a barrier so that the LDS buffer can be reused.
    __device__ __forceinline__ void run_robust(int tile) const {
        const Where q = locate(tile);
        const AggPtr s_agg = s_agg0;
        const float NEG_INF = -__builtin_inff();
        const int nSC = g.nSC;
        const int li = lane * VEC;
        float om[VEC], mu[VEC];
        WU wu;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            wu.w[e] = q.cok ? w_[q.c0 + e] : 0.f;
            wu.u[e] = q.cok ? u_[q.c0 + e] : 0.f;
        }
        if (!tile_is_robust(wu, om, mu)) return;

        const unsigned row = (unsigned)(C * sizeof(IO));
        const __amdgpu_buffer_rsrc_t ry = make_rsrc(y_ + q.slab, (unsigned)((size_t)T * C * sizeof(IO)));
        const size_t ws_b = (size_t)q.b * nSC * NSLOT * C;
        auto ws_at = [&](int s, int slot, int e) -> float& {
            return ws[ws_b + ((size_t)s * NSLOT + slot) * C + q.c0 + e];
        };
        float X0[L][VEC], X1[L][VEC];
        {
            P K[L], V[L];
            WU unused;
            issue_loads(tile, K, V, unused);
#pragma unroll
            for (int j = 0; j < L; ++j) {
                unpack<IO, VEC>(K[j], X0[j]);
                unpack<IO, VEC>(V[j], X1[j]);
                const bool tok = q.tw + j < T;
#pragma unroll
                for (int e = 0; e < VEC; ++e) X0[j][e] = tok ? X0[j][e] * LOG2E : NEG_INF;
            }
        }
        // ================================== robust path ==================================
        float A[VEC], Bd[VEC], pA[VEC], Cg[VEC], D[VEC], pC[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            A[e] = 0.f; Bd[e] = 0.f; pA[e] = NEG_BIG; Cg[e] = 0.f; D[e] = 0.f; pC[e] = NEG_BIG;
        }
#pragma unroll
        for (int j = 0; j < L; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) tri_push(A[e], Bd[e], pA[e], om[e], X0[j][e], X1[j][e]);
#pragma unroll
        for (int j = L - 1; j >= 0; --j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) tri_push(Cg[e], D[e], pC[e], om[e], X0[j][e], X1[j][e]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            s_agg[wave][0][li + e] = A[e];
            s_agg[wave][1][li + e] = Bd[e];
            s_agg[wave][2][li + e] = pA[e];
            s_agg[wave][3][li + e] = Cg[e];
            s_agg[wave][4][li + e] = D[e];
            s_agg[wave][5][li + e] = pC[e];
        }
        lds_barrier();

        if (MODE == 1) {
            if (wave == 0 && q.cok) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float omL = om[e] * (float)L;
                    float a = 0.f, bb = 0.f, p = NEG_BIG, c = 0.f, d = 0.f, o = NEG_BIG;
                    for (int s = 0; s < S; ++s)
                        tri_merge(a, bb, p, omL, s_agg[s][0][li + e], s_agg[s][1][li + e], s_agg[s][2][li + e]);
                    for (int s = S - 1; s >= 0; --s)
                        tri_merge(c, d, o, omL, s_agg[s][3][li + e], s_agg[s][4][li + e], s_agg[s][5][li + e]);
                    ws_at(q.sc, 0, e) = a; ws_at(q.sc, 1, e) = bb; ws_at(q.sc, 2, e) = p;
                    ws_at(q.sc, 3, e) = c; ws_at(q.sc, 4, e) = d;  ws_at(q.sc, 5, e) = o;
                }
            }
            lds_barrier();
            return;
        }

        float a[VEC], bb[VEC], p[VEC], c[VEC], d[VEC], o[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            a[e] = 0.f; bb[e] = 0.f; p[e] = NEG_BIG; c[e] = 0.f; d[e] = 0.f; o[e] = NEG_BIG;
        }
        if (MODE == 2 && q.cok) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float omSL = om[e] * (float)(S * L);
                for (int s = 0; s < q.sc; ++s)
                    tri_merge(a[e], bb[e], p[e], omSL, ws_at(s, 0, e), ws_at(s, 1, e), ws_at(s, 2, e));
                for (int s = nSC - 1; s > q.sc; --s)
                    tri_merge(c[e], d[e], o[e], omSL, ws_at(s, 3, e), ws_at(s, 4, e), ws_at(s, 5, e));
            }
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float omL = om[e] * (float)L;
            for (int s = 0; s < wave; ++s)
                tri_merge(a[e], bb[e], p[e], omL, s_agg[s][0][li + e], s_agg[s][1][li + e], s_agg[s][2][li + e]);
            for (int s = S - 1; s > wave; --s)
                tri_merge(c[e], d[e], o[e], omL, s_agg[s][3][li + e], s_agg[s][4][li + e], s_agg[s][5][li + e]);
        }

        float PN[L][VEC], PD[L][VEC], PM[L][VEC];
#pragma unroll
        for (int j = 0; j < L; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float uk = mu[e] + X0[j][e];
                const float pm = fmaxf(p[e], uk);
                const float ea = fast_exp2(p[e] - pm);
                const float eu = fast_exp2(uk - pm);
                PN[j][e] = ea * a[e] + eu * X1[j][e];
                PD[j][e] = ea * bb[e] + eu;
                PM[j][e] = pm;
                tri_push(a[e], bb[e], p[e], om[e], X0[j][e], X1[j][e]);
            }
#pragma unroll
        for (int j = L - 1; j >= 0; --j) {
            float out[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float m = fmaxf(PM[j][e], o[e]);
                const float e1 = fast_exp2(PM[j][e] - m);
                const float e2 = fast_exp2(o[e] - m);
                out[e] = (e1 * PN[j][e] + e2 * c[e]) / (e1 * PD[j][e] + e2 * d[e]);
                tri_push(c[e], d[e], o[e], om[e], X0[j][e], X1[j][e]);
            }
            if constexpr (GATE) {
                const __amdgpu_buffer_rsrc_t rr = make_rsrc(r_ + q.slab, (unsigned)((size_t)T * C * sizeof(IO)));
                out[0] *= gate_of(BufRaw<sizeof(IO)>::ld(rr, q.voff0 + (unsigned)j * row, 0));
            }
            buf_store<IO, VEC>(ry, q.voff0 + (unsigned)j * row, out);
        }
        lds_barrier();
    }
};


template <typename IO, int VEC, int L, int MODE, bool STAGED = false, bool GATE = false>
__global__ __launch_bounds__(smax_for(L, VEC) * WAVE)
void biwkv_fwd_kernel(const float* __restrict__ w_, const float* __restrict__ u_,
                      const IO* __restrict__ k_, const IO* __restrict__ v_, IO* __restrict__ y_,
                      float* __restrict__ ws, int T, int C, TileGeom g, const IO* __restrict__ r_ = nullptr)
{
    using Tile = BiwkvTile<IO, VEC, L, MODE, STAGED, GATE>;
    __shared__ float s_agg[2][Tile::SMAX][NSLOT][Tile::CH];   // fast path: slot 2 carries the wave maxima
    __shared__ __attribute__((aligned(16))) IO s_stage[STAGED ? Tile::SMAX : 1][STAGED ? Tile::STAGE_ELEMS : 1];
    __shared__ __attribute__((aligned(16))) IO s_y[Tile::OUT_STAGED ? Tile::SMAX : 1][Tile::YSTAGE_ELEMS];
    __shared__ float s_fold[MODE == 2 ? 12 : 1][WAVE];

    Tile t;
    t.w_ = w_; t.u_ = u_; t.k_ = k_; t.v_ = v_; t.r_ = r_; t.y_ = y_; t.ws = ws;
    t.T = T; t.C = C; t.g = g;
    t.lane = threadIdx.x & (WAVE - 1);
    t.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    t.S = blockDim.x >> 6;
    t.s_agg0 = s_agg[0];
    t.s_agg1 = s_agg[1];
    t.s_fold = s_fold;
    t.s_stage = &s_stage[STAGED ? t.wave : 0][0];
    t.s_y = &s_y[Tile::OUT_STAGED ? t.wave : 0][0];

    typename Tile::P K0[L], V0[L], K1[L], V1[L];
    typename Tile::WU wu0, wu1;
    // Workgroups are dealt round-robin to the 8 XCDs: in every round XCD x takes a contiguous eighth of the round's
    // tiles, so neighbouring 64-channel segments of the same token rows go through one L2 and one translation cache
    // (measured 1 % faster than tile = workgroup index; giving an XCD one contiguous run over all rounds is 3 % slower).
    int tile = blockIdx.x;
    if ((gridDim.x & 7) == 0) tile = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (tile < g.n_tiles) {
        if (STAGED) t.issue_stage(tile, wu0); else t.issue_loads(tile, K0, V0, wu0);
        if (STAGED && Tile::EARLY_WAIT) Tile::wait_vm0();                 // every tile starts with its rows landed
        for (;;) {
            int next = tile + gridDim.x;
            t.run(tile, next, 0, K0, V0, wu0, K1, V1, wu1);
            if (next >= g.n_tiles) break;
            tile = next;
            next = tile + gridDim.x;
            t.run(tile, next, 1, K1, V1, wu1, K0, V0, wu0);
            if (next >= g.n_tiles) break;
            tile = next;
        }
    }
    // second walk: tiles whose parameters need the renormalising recurrence
    lds_barrier();
    for (tile = blockIdx.x; tile < g.n_tiles; tile += gridDim.x) t.run_robust(tile);
}

}  // namespace biwkv_fwd_detail
}  // namespace vrwkv
#include "biwkv_fwd_resident.h"
namespace vrwkv {
namespace biwkv_fwd_detail {

// ------------------------------- host-side dispatch ---------------------------------
struct Plan {
    int L = 0, S = 0, nSC = 0, VEC = 0, grid = 0;
    TileGeom geom{};
    bool multi() const { return nSC > 1; }
};

constexpr int kLs[] = {4, 8, 16, 25, 28};
constexpr int kNumL = sizeof(kLs) / sizeof(kLs[0]);

inline int num_cus() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            n = prop.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

inline Plan make_plan(int B, int T, int C, int io_dtype) {
    Plan p;
    const int el = option(OPT_BIWKV_L);              // tuning overrides
    const int es = option(OPT_BIWKV_S);
    p.VEC = 1;
    int best = -1, best_waste = 1 << 30;
    for (int i = 0; i < kNumL; ++i) {
        const int L = kLs[i];
        if (el && L != el) continue;
        const int S = (T + L - 1) / L;
        if (S > smax_for(L, p.VEC)) continue;
        // 25-token chunks exist for 16-bit rows of 176..200 tokens (196: eight waves, two per SIMD, where 7 x 28 leaves
        // one SIMD a single wave; the 16-bit kernel is bound by instruction issue: 17.3 -> 16.7 us at 64 x 196 x 768)
        if (L == 25 && !el && (S != 8 || io_dtype == VRWKV_F32)) continue;
        if (L == 25 && !el) { best = i; break; }
        const int waste = S * L - T;
        if (waste < best_waste) { best = i; best_waste = waste; }
    }
    if (best >= 0) {
        p.L = kLs[best];
        p.S = (T + p.L - 1) / p.L;
        p.nSC = 1;
    } else {
        p.L = 28;
        for (int i = 0; i < kNumL; ++i) if (el == kLs[i]) p.L = el;
        p.S = smax_for(p.L, p.VEC);
        if (es >= 2 && es <= smax_for(p.L, p.VEC)) p.S = es;      // at least two waves: the emit pass gives two of them a job of their own
        p.nSC = (T + p.S * p.L - 1) / (p.S * p.L);
    }
    const int cap = smax_for(p.L, p.VEC);
    p.geom.n_ctile = (C + WAVE * p.VEC - 1) / (WAVE * p.VEC);
    p.geom.nSC = p.nSC;
    p.geom.n_tiles = B * p.nSC * p.geom.n_ctile;
    // persistent grid: as many workgroups as can be resident at once
    const int wg_per_cu = (cap / p.S) > 0 ? (cap / p.S) : 1;
    int grid = num_cus() * wg_per_cu;
    const int eg = option(OPT_BIWKV_GRID);
    if (eg > 0) grid = eg;
    p.grid = grid < p.geom.n_tiles ? grid : p.geom.n_tiles;
    return p;
}

// Returned (never to the caller of the C ABI) when a gate was asked for and the kernels this call would run have no
// gated variant: rows that cannot be staged, or the one-launch kernel for two or three super-chunks.
constexpr int GATE_NOT_FUSED = -100;

// r: null, or the receptance whose sigmoid gates y inside the emitting kernel.
template <typename IO, int VEC, int L>
int launch_L(const Plan& p, const float* w, const float* u, const void* k, const void* v, const void* r, void* y,
             float* ws, int B, int T, int C, hipStream_t st) {
    const dim3 block(p.S * WAVE);
    const dim3 grid(p.grid);
    const IO* kk = static_cast<const IO*>(k);
    const IO* vv = static_cast<const IO*>(v);
    const IO* rr = static_cast<const IO*>(r);
    IO* yy = static_cast<IO*>(y);
    // fp32 rows are staged through LDS in 16-byte pieces when the layout allows it
    if constexpr (VEC == 1) {
        const bool aligned = C % (16 / (int)sizeof(IO)) == 0 && (((uintptr_t)k | (uintptr_t)v | (uintptr_t)y) & 15) == 0;
        if (aligned && !option(OPT_BIWKV_NO_STAGE)) {
            if (!p.multi()) {
                if (rr) hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 0, true, true>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
                else hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 0, true>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
            } else if (sizeof(IO) == 2 && L == 28 && p.nSC <= 3 && !option(OPT_BIWKV_NO_RESIDENT)) {
                if (rr) return GATE_NOT_FUSED;
                // two or three super-chunks of 16-bit rows fit a workgroup's registers: one launch, k and v read once
                if constexpr (sizeof(IO) == 2 && L == 28) {
                    const int n_seq = B * p.geom.n_ctile;
                    const int eg = option(OPT_BIWKV_GRID);
                    const int g1 = eg > 0 ? eg : num_cus();
                    const dim3 rgrid(g1 < n_seq ? g1 : n_seq);
                    const bool short_chunks = T <= p.nSC * 8 * 24;        // 24-token chunks need no spills with three super-chunks
                    const int RL = short_chunks ? 24 : 28;
                    const dim3 rblock(((T + p.nSC * RL - 1) / (p.nSC * RL)) * WAVE);
#define VRWKV_RESIDENT(NSC_, L_) hipLaunchKernelGGL((biwkv_fwd_resident_kernel<IO, NSC_, L_>), rgrid, rblock, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom.n_ctile, n_seq)
                    if (p.nSC == 2) { if (short_chunks) VRWKV_RESIDENT(2, 24); else VRWKV_RESIDENT(2, 28); }
                    else            { if (short_chunks) VRWKV_RESIDENT(3, 24); else VRWKV_RESIDENT(3, 28); }
#undef VRWKV_RESIDENT
                }
            } else {
                // fp32 rows: the emitting kernel of long sequences has no registers left for r (measured at 2 x 4150 x 768:
                // 61 us with the gate inside against 50 us with the gate as a pass of its own); 16-bit rows: 32 against 37 us
                if (rr && sizeof(IO) == 4) return GATE_NOT_FUSED;
                hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 1, true>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
                if constexpr (sizeof(IO) == 2) {
                    if (rr) {
                        hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 2, true, true>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
                        return check_launch("biwkv_fwd");
                    }
                }
                hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 2, true>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
            }
            return check_launch("biwkv_fwd");
        }
    }
    if (rr) return GATE_NOT_FUSED;
    if (!p.multi()) {
        hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 0>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
    } else {
        hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 1>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
        hipLaunchKernelGGL((biwkv_fwd_kernel<IO, VEC, L, 2>), grid, block, 0, st, w, u, kk, vv, yy, ws, T, C, p.geom, rr);
    }
    return check_launch("biwkv_fwd");
}

template <typename IO, int VEC>
int launch_VEC(const Plan& p, const float* w, const float* u, const void* k, const void* v, const void* r, void* y,
               float* ws, int B, int T, int C, hipStream_t st) {
    switch (p.L) {
#define VRWKV_CASE(LL) case LL: return launch_L<IO, VEC, LL>(p, w, u, k, v, r, y, ws, B, T, C, st); break;
        VRWKV_CASE(4) VRWKV_CASE(8) VRWKV_CASE(16) VRWKV_CASE(25) VRWKV_CASE(28)
#undef VRWKV_CASE
    }
    set_error("biwkv_fwd: internal error, no kernel for L=%d VEC=%d", p.L, VEC);
    return VRWKV_INVALID_ARG;
}

template <typename IO>
int biwkv_fwd_launch_io(const Plan& p, const float* w, const float* u, const void* k, const void* v, const void* r, void* y,
                        float* ws, int B, int T, int C, hipStream_t st) {
    return launch_VEC<IO, 1>(p, w, u, k, v, r, y, ws, B, T, C, st);
}

}  // namespace biwkv_fwd_detail
}  // namespace vrwkv
