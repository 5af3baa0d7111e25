// Bi-WKV forward, one launch for sequences of two or three super-chunks with 16-bit I/O (included by
// biwkv_fwd_impl.h).
//
// A workgroup owns a whole (batch, 64 channels) sequence of NSC super-chunks of S waves x L tokens (L = 24 where the
// sequence allows it, L = 28 for longer ones at the price of more spills with three super-chunks).  k and v are read
// from HBM once: every wave keeps the rows of its NSC chunks packed in registers (k in the low, v in the high half
// of a register) between
//   phase A  per super-chunk: the wave's aggregates, one LDS exchange, and from it the carries inside the
//            super-chunk and the super-chunk totals (every wave forms all totals, so the carries across
//            super-chunks need no further exchange), and
//   phase B  per super-chunk: the two emit sweeps (E = 2^(k - Rw) recomputed from the packed rows in each) and
//            the stores.
// Rows travel as 16-byte pieces through NREG LDS regions per wave (HBM -> LDS directly), super-chunk n of the
// workgroup's stream in region n % NREG: the rows of the next NREG-1 super-chunks are on their way while one is
// computed (three regions for three super-chunks of 24-token chunks, two otherwise), and y leaves through the
// region read last.
// Same arithmetic as BiwkvTile::run (log2 domain, integer reference exponents, exact ldexp rescaling); channel tiles
// outside the plain-sum regime are redone inside the same launch by the renormalising recurrence
// (BiwkvTile::run_robust, aggregates through the workspace).
#pragma once

namespace vrwkv {
namespace biwkv_fwd_detail {

// k and v of eight (four) tokens from a wave's row region: the LDS reads are issued back to back and waited for inside
// the same statement (the compiler does not know that the registers are still being written); k goes to the low,
// v to the high half of one register per token.  Written with plain loads the compiler, short of registers, reads
// token after token and waits for each.  (Loads that write one half of a register and keep the other do not exist
// on this target: with SRAM ECC a 16-bit load clears the other half.)  Rows are 128 bytes apart.
__device__ __forceinline__ void lds_row_octet(unsigned k_addr, unsigned v_addr, unsigned* bits) {
    unsigned k0, k1, k2, k3, k4, k5, k6, k7, v0, v1, v2, v3, v4, v5, v6, v7;
    asm volatile("ds_read_u16 %0, %16\n\t"
                 "ds_read_u16 %1, %16 offset:128\n\t"
                 "ds_read_u16 %2, %16 offset:256\n\t"
                 "ds_read_u16 %3, %16 offset:384\n\t"
                 "ds_read_u16 %4, %16 offset:512\n\t"
                 "ds_read_u16 %5, %16 offset:640\n\t"
                 "ds_read_u16 %6, %16 offset:768\n\t"
                 "ds_read_u16 %7, %16 offset:896\n\t"
                 "ds_read_u16 %8, %17\n\t"
                 "ds_read_u16 %9, %17 offset:128\n\t"
                 "ds_read_u16 %10, %17 offset:256\n\t"
                 "ds_read_u16 %11, %17 offset:384\n\t"
                 "ds_read_u16 %12, %17 offset:512\n\t"
                 "ds_read_u16 %13, %17 offset:640\n\t"
                 "ds_read_u16 %14, %17 offset:768\n\t"
                 "ds_read_u16 %15, %17 offset:896\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(k0), "=&v"(k1), "=&v"(k2), "=&v"(k3), "=&v"(k4), "=&v"(k5), "=&v"(k6), "=&v"(k7),
                   "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5), "=&v"(v6), "=&v"(v7)
                 : "v"(k_addr), "v"(v_addr)
                 : "memory");
    bits[0] = k0 | (v0 << 16); bits[1] = k1 | (v1 << 16); bits[2] = k2 | (v2 << 16); bits[3] = k3 | (v3 << 16);
    bits[4] = k4 | (v4 << 16); bits[5] = k5 | (v5 << 16); bits[6] = k6 | (v6 << 16); bits[7] = k7 | (v7 << 16);
}
__device__ __forceinline__ void lds_row_quad(unsigned k_addr, unsigned v_addr, unsigned* bits) {
    unsigned k0, k1, k2, k3, v0, v1, v2, v3;
    asm volatile("ds_read_u16 %0, %8\n\t"
                 "ds_read_u16 %1, %8 offset:128\n\t"
                 "ds_read_u16 %2, %8 offset:256\n\t"
                 "ds_read_u16 %3, %8 offset:384\n\t"
                 "ds_read_u16 %4, %9\n\t"
                 "ds_read_u16 %5, %9 offset:128\n\t"
                 "ds_read_u16 %6, %9 offset:256\n\t"
                 "ds_read_u16 %7, %9 offset:384\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(k0), "=&v"(k1), "=&v"(k2), "=&v"(k3), "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
                 : "v"(k_addr), "v"(v_addr)
                 : "memory");
    bits[0] = k0 | (v0 << 16); bits[1] = k1 | (v1 << 16); bits[2] = k2 | (v2 << 16); bits[3] = k3 | (v3 << 16);
}
// all L tokens of a wave's chunk: k rows at lds_addr, v rows LR rows further on
template <int L, int LR>
__device__ __forceinline__ void lds_read_rows(unsigned lds_addr, unsigned (&bits)[L]) {
    static_assert(L % 4 == 0, "rows are read eight or four tokens at a time");
#pragma unroll
    for (int j = 0; j + 8 <= L; j += 8) lds_row_octet(lds_addr + j * 128, lds_addr + (LR + j) * 128, &bits[j]);
    if constexpr (L % 8 != 0) lds_row_quad(lds_addr + (L - 4) * 128, lds_addr + (LR + L - 4) * 128, &bits[L - 4]);
}
// y staging and the exchange buffer (plain LDS accesses)
template <typename IO>
__device__ __forceinline__ void lds_put(IO* __restrict__ rows, int idx, IO val) { rows[idx] = val; }
template <typename IO>
__device__ __forceinline__ BufRaw<16>::type lds_get16(const IO* __restrict__ rows, int idx) {
    return *reinterpret_cast<const BufRaw<16>::type*>(rows + idx);
}
__device__ __forceinline__ void agg_put(float (*__restrict__ agg)[NSLOT][WAVE], int wave, int lane,
                                        float a, float b, float r, float c, float d) {
    agg[wave][0][lane] = a;
    agg[wave][1][lane] = b;
    agg[wave][2][lane] = r;
    agg[wave][3][lane] = c;
    agg[wave][4][lane] = d;
}
template <int SMAX>
__device__ __forceinline__ void agg_get(const float (*__restrict__ agg)[NSLOT][WAVE], int S, int lane, float (&la)[SMAX],
                                        float (&lb)[SMAX], float (&lr)[SMAX], float (&lc)[SMAX], float (&ld)[SMAX]) {
    (void)S;                                     // entries of waves past S hold neutral values (set once per kernel)
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        la[s] = agg[s][0][lane];
        lb[s] = agg[s][1][lane];
        lr[s] = agg[s][2][lane];
        lc[s] = agg[s][3][lane];
        ld[s] = agg[s][4][lane];
    }
}

// One sequence outside the plain-sum regime: the renormalising recurrence of BiwkvTile::run_robust, first the
// aggregates of every super-chunk (into the workspace), then the outputs.
template <typename IO, int NSC, int L>
__device__ __forceinline__ void resident_robust(const float* w_, const float* u_, const IO* k_, const IO* v_, IO* y_,
                                                          float* ws, int T, int C, int n_ctile, int n_seq, int b, int ctile,
                                                          float (*agg0)[NSLOT][WAVE], float (*agg1)[NSLOT][WAVE]) {
    TileGeom g;
    g.n_ctile = n_ctile; g.nSC = NSC; g.n_tiles = n_seq * NSC;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int S = blockDim.x >> 6;
    BiwkvTile<IO, 1, L, 1, false> t1;
    t1.w_ = w_; t1.u_ = u_; t1.k_ = k_; t1.v_ = v_; t1.y_ = y_; t1.ws = ws; t1.T = T; t1.C = C; t1.g = g;
    t1.lane = lane; t1.wave = wave; t1.S = S; t1.s_agg0 = agg0; t1.s_agg1 = agg1; t1.s_stage = nullptr; t1.s_y = nullptr; t1.s_fold = nullptr;
    for (int sc = 0; sc < NSC; ++sc) t1.run_robust((b * NSC + sc) * n_ctile + ctile);
    __threadfence();
    __syncthreads();
    BiwkvTile<IO, 1, L, 2, false> t2;
    t2.w_ = w_; t2.u_ = u_; t2.k_ = k_; t2.v_ = v_; t2.y_ = y_; t2.ws = ws; t2.T = T; t2.C = C; t2.g = g;
    t2.lane = lane; t2.wave = wave; t2.S = S; t2.s_agg0 = agg0; t2.s_agg1 = agg1; t2.s_stage = nullptr; t2.s_y = nullptr; t2.s_fold = nullptr;
    for (int sc = 0; sc < NSC; ++sc) t2.run_robust((b * NSC + sc) * n_ctile + ctile);
}

template <typename IO, int NSC, int L>
__global__ __launch_bounds__(8 * WAVE)
void biwkv_fwd_resident_kernel(const float* __restrict__ w_, const float* __restrict__ u_,
                               const IO* __restrict__ k_, const IO* __restrict__ v_, IO* __restrict__ y_,
                               float* __restrict__ ws, int T, int C, int n_ctile, int n_seq)
{
    static_assert(sizeof(IO) == 2 && WAVE * sizeof(IO) == 128, "packed register rows need 16-bit elements (128-byte LDS rows)");
    constexpr int SMAX = 8;
    constexpr int EPL = 8, LPR = 8, RPI = 8, NI = (L + RPI - 1) / RPI, LR = NI * RPI;   // 16-byte pieces: 8 lanes per row, 8 rows per instruction
    // Row regions per wave (160 KB of LDS hold three of 24 rows or two of 32).  They are separate arrays: the compiler
    // makes an LDS read wait for every LDS-direct load that may write the array it reads, so only with one array per
    // region -- and the region of a super-chunk known at compile time, i.e. NREG == NSC -- can the rows of the
    // following super-chunks stay in flight across the reads of the current one.
    constexpr int NREG = (NSC == 3 && LR <= 24) ? 3 : 2;
    constexpr bool STATIC_REG = NREG == NSC;
    __shared__ float s_agg[SMAX][NSLOT][WAVE];
    __shared__ __attribute__((aligned(16))) IO s_rows0[SMAX][2 * LR * WAVE];
    __shared__ __attribute__((aligned(16))) IO s_rows1[SMAX][2 * LR * WAVE];
    __shared__ __attribute__((aligned(16))) IO s_rows2[NREG == 3 ? SMAX : 1][NREG == 3 ? 2 * LR * WAVE : 8];
    auto region = [&](int reg) -> IO* { return reg == 0 ? &s_rows0[0][0] : reg == 1 ? &s_rows1[0][0] : &s_rows2[0][0]; };

    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int S = blockDim.x >> 6;
    const float NEG_INF = -__builtin_inff();
    const unsigned short ninf_bits = __builtin_bit_cast(unsigned short, from_f32<IO>(NEG_INF));
    const unsigned bytes = (unsigned)((size_t)T * C * sizeof(IO));
    typedef __attribute__((address_space(3))) void* lds_ptr;
    auto shift_of = [](float r_from, float r_to) -> int { return (int)fmaxf(r_from - r_to, -300.f); };

    // workgroups are dealt round-robin to the 8 XCDs: per round, XCD x takes a contiguous eighth of the sequences
    const int wg = (gridDim.x & 7) == 0 ? (int)((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3)) : (int)blockIdx.x;
    // Super-chunk number m of this workgroup's stream (sequence wg + (m / NSC) gridDim.x, super-chunk m % NSC):
    // its rows for this wave -> region m % NREG.  Nothing is issued past the last sequence.
    auto stream_exists = [&](int m) { return wg + (m / NSC) * (int)gridDim.x < n_seq; };
    auto issue_rows = [&](int m, int reg) {
        if (!stream_exists(m)) return;
        const int seq = wg + (m / NSC) * (int)gridDim.x, sc = m % NSC;
        const int ctile = seq % n_ctile, b = seq / n_ctile;
        const size_t slab = (size_t)b * T * C;
        const __amdgpu_buffer_rsrc_t rk = make_rsrc(k_ + slab, bytes), rv = make_rsrc(v_ + slab, bytes);
        const int cq = ctile * WAVE + (lane % LPR) * EPL;
        int tw = (sc * S + wave) * L;
        asm volatile("" : "+s"(tw));                 // rows and offsets are recomputed here: hoisted out of the sequence loop they spill
        IO* dst = region(reg) + wave * (2 * LR * WAVE);
        const int Cs = C;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int rl = RPI * i + lane / LPR;
            const int row = tw + rl;
            const unsigned vo = (rl < L && row < T && cq < Cs) ? (unsigned)((row * Cs + cq) * (int)sizeof(IO)) : OOB_OFFSET;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (lds_ptr)(dst + i * RPI * WAVE), 16, vo, 0, 0, CPOL_NT);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (lds_ptr)(dst + (LR + i * RPI) * WAVE), 16, vo, 0, 0, CPOL_NT);
        }
    };

    // exchange entries of the waves this workgroup does not have: no tokens (read with fixed addresses below)
    for (int s2 = S + wave; s2 < SMAX; s2 += S) agg_put(s_agg, s2, lane, 0.f, 0.f, NEG_BIG, 0.f, 0.f);
    __syncthreads();

    int n = 0;                                   // stream position
    int seq = wg;
    if (seq >= n_seq) return;
#pragma unroll
    for (int m = 0; m < NREG - 1; ++m) issue_rows(m, m % NREG);
    for (; seq < n_seq; seq += gridDim.x) {
        const int ctile = seq % n_ctile, b = seq / n_ctile;
        const int c0 = ctile * WAVE + lane;
        const bool cok = c0 < C;
        const float wv = cok ? w_[c0] : 0.f, uv = cok ? u_[c0] : 0.f;
        const float om = wv * LOG2E, mu = uv * LOG2E;
        const bool bad = outside_plain_sum(om, mu, T);
        if (__builtin_amdgcn_ballot_w64(bad) != 0ull) {
            // outside the plain-sum regime: the renormalising recurrence, super-chunk aggregates through the workspace
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");              // the rows already on their way must land first
            __syncthreads();
            resident_robust<IO, NSC, L>(w_, u_, k_, v_, y_, ws, T, C, n_ctile, n_seq, b, ctile, s_agg, s_agg);
#pragma unroll
            for (int sc = 0; sc < NSC; ++sc, ++n)                         // what its super-chunks would have asked for
                issue_rows(n + NREG - 1, STATIC_REG ? (sc + NREG - 1) % NREG : (n + NREG - 1) % NREG);
            continue;
        }

        const float gd = fast_exp2(-om);                                  // decay per token
        const float G = fast_exp2(-om * (float)L);                        // ... per wave chunk
        const float GS = fast_exp2(-om * (float)(S * L));                 // ... per super-chunk
        const float cu = fast_exp2(mu);
        const float Gpre = fast_exp2(-om * (float)(L * wave));            // decay over the waves before this one
        const float Gpost = fast_exp2(-om * (float)(L * (S - 1 - wave))); // ... and after it
        const __amdgpu_buffer_rsrc_t ry = make_rsrc(y_ + (size_t)b * T * C, bytes);
        const int cq = ctile * WAVE + (lane % LPR) * EPL;
        unsigned raw[NSC][L];                                             // k | v << 16 of every super-chunk, as loaded
        float Rw[NSC], Rs[NSC], ia[NSC], ib[NSC], ic[NSC], id[NSC], ta[NSC], tb[NSC], tc[NSC], td[NSC];

        // ---- phase A per super-chunk ----
#pragma unroll
        for (int sc = 0; sc < NSC; ++sc, ++n) {
            // with as many regions as super-chunks the region of a super-chunk is fixed at compile time
            const int reg = STATIC_REG ? sc : n % NREG;
            // one opaque per-lane element offset, so that the 2 L row reads are one address register plus immediates
            // (folded into the array's address they exceed the 16-bit offset field and become 2 L registers)
            unsigned row_base = (unsigned)(wave * (2 * LR * WAVE) + lane);
            asm volatile("" : "+v"(row_base));
            typedef __attribute__((address_space(3))) const IO* lds_cptr;
            const unsigned rows_addr = (unsigned)(size_t)(lds_cptr)(region(reg) + row_base);     // LDS byte address of the lane's first row
            const int tw = (sc * S + wave) * L;
            // This super-chunk's rows have landed.  Loads complete in order, so the younger super-chunk on its way
            // (three regions) may stay in flight -- unless stores are pending too (first super-chunk of a sequence:
            // the previous sequence's y), which complete in no fixed order relative to loads.
            if (STATIC_REG && NREG == 3 && sc > 0 && stream_exists(n + 1)) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * NI) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            float X0[L], X1[L];
            unsigned rw_bits[L];                                          // k | v << 16, as loaded
            if (tw + L <= T) {                                            // wave-uniform: every token of the chunk exists
                lds_read_rows<L, LR>(rows_addr, rw_bits);
            } else {
                int nvalid = T - tw;                                      // rows past T were not written: LDS holds stale bits
                asm volatile("" : "+v"(nvalid));                          // compared per lane: 28 scalar masks would spill
                lds_read_rows<L, LR>(rows_addr, rw_bits);
#pragma unroll
                for (int j = 0; j < L; ++j) rw_bits[j] = j < nvalid ? rw_bits[j] : (unsigned)ninf_bits;
            }
#pragma unroll
            for (int j = 0; j < L; ++j) {
                raw[sc][j] = rw_bits[j];
                X0[j] = to_f32(__builtin_bit_cast(IO, (unsigned short)(rw_bits[j] & 0xffffu)));
                X1[j] = to_f32(__builtin_bit_cast(IO, (unsigned short)(rw_bits[j] >> 16)));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // rows are in registers
            // the region read one super-chunk ago takes the rows NREG-1 positions ahead
            issue_rows(n + NREG - 1, STATIC_REG ? (sc + NREG - 1) % NREG : (n + NREG - 1) % NREG);

            float m = NEG_INF;
#pragma unroll
            for (int j = 0; j < L; ++j) m = fmaxf(m, X0[j]);
            const bool any = m > NEG_INF;
            const float rw = any ? ceilf(m * LOG2E) : 0.f;
            float A = 0.f, Bd = 0.f, Cg = 0.f, D = 0.f;
#pragma unroll
            for (int j = 0; j < L; ++j) {
                const float E = fast_exp2(fmaf(X0[j], LOG2E, -rw));
                X0[j] = E;
                X1[j] = E * X1[j];
                A = fmaf(gd, A, X1[j]);
                Bd = fmaf(gd, Bd, E);
            }
#pragma unroll
            for (int j = L - 1; j >= 0; --j) {
                Cg = fmaf(gd, Cg, X1[j]);
                D = fmaf(gd, D, X0[j]);
            }
            float (*agg)[NSLOT][WAVE] = s_agg;
            int lo = lane;
            asm volatile("" : "+v"(lo));             // exchange addresses formed here: kept across the loop they are spilled, and
                                                     // a reload from scratch has to wait for every row load issued before it
            agg_put(agg, wave, lo, A, Bd, any ? rw : NEG_BIG, Cg, D);     // a wave with no token must not set the scale
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // LDS only: the row loads stay in flight

            float la[SMAX], lb[SMAX], lc[SMAX], ld[SMAX], lr[SMAX];
            agg_get<SMAX>(agg, S, lo, la, lb, lr, lc, ld);
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // everyone has read: the buffer may be rewritten
            float r = NEG_BIG;
#pragma unroll
            for (int s = 0; s < SMAX; ++s) r = fmaxf(r, lr[s]);
            r = (r > NEG_BIG) ? r : 0.f;
            // carries inside the super-chunk (waves before / after this one) and its totals, all at scale 2^r
            float aa = 0.f, ab = 0.f, ac = 0.f, ad = 0.f;
            float pa = 0.f, pb = 0.f, pc = 0.f, pd = 0.f;
#pragma unroll
            for (int s = 0; s < SMAX; ++s) {
                if (s == wave) { pa = aa; pb = ab; }
                if (s < S) {
                    const int sh = shift_of(lr[s], r);
                    aa = fmaf(G, aa, ldexpf(la[s], sh));
                    ab = fmaf(G, ab, ldexpf(lb[s], sh));
                }
            }
#pragma unroll
            for (int s = SMAX - 1; s >= 0; --s) {
                if (s == wave) { pc = ac; pd = ad; }
                if (s < S) {
                    const int sh = shift_of(lr[s], r);
                    ac = fmaf(G, ac, ldexpf(lc[s], sh));
                    ad = fmaf(G, ad, ldexpf(ld[s], sh));
                }
            }
            Rw[sc] = rw; Rs[sc] = r;
            ia[sc] = pa; ib[sc] = pb; ic[sc] = pc; id[sc] = pd;
            ta[sc] = aa; tb[sc] = ab; tc[sc] = ac; td[sc] = ad;
        }

        // ---- phase B: the carries of every super-chunk first (twelve values instead of thirty stay live), then the
        //      emit sweeps straight from the packed rows: E and E v are recomputed in both sweeps rather than kept,
        //      which is what lets three super-chunks fit the registers ----
        float fa[NSC], fb[NSC], fc[NSC], fd[NSC];
#pragma unroll
        for (int sc = 0; sc < NSC; ++sc) {
            // what the other super-chunks contribute: totals of the earlier ones decayed to this super-chunk's first
            // token, of the later ones to its last, each at the running maximum of the (integer) scales met so far
            float r1 = NEG_BIG, r2 = NEG_BIG, ca = 0.f, cb = 0.f, cc = 0.f, cd = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < NSC; ++s2)
                if (s2 < sc) {
                    const float mm = fmaxf(r1, Rs[s2]);
                    const int so = shift_of(r1, mm), sn = shift_of(Rs[s2], mm);
                    ca = fmaf(GS, ldexpf(ca, so), ldexpf(ta[s2], sn));
                    cb = fmaf(GS, ldexpf(cb, so), ldexpf(tb[s2], sn));
                    r1 = mm;
                }
#pragma unroll
            for (int s2 = NSC - 1; s2 >= 0; --s2)
                if (s2 > sc) {
                    const float mm = fmaxf(r2, Rs[s2]);
                    const int so = shift_of(r2, mm), sn = shift_of(Rs[s2], mm);
                    cc = fmaf(GS, ldexpf(cc, so), ldexpf(tc[s2], sn));
                    cd = fmaf(GS, ldexpf(cd, so), ldexpf(td[s2], sn));
                    r2 = mm;
                }
            const float r = fmaxf(Rs[sc], fmaxf(r1, r2));
            const int s0 = shift_of(Rs[sc], r), s1 = shift_of(r1, r), s2_ = shift_of(r2, r);
            const int up = (int)fminf(r - Rw[sc], plain_sum_up_cap(om, T));   // to the wave's own scale
            fa[sc] = ldexpf(fmaf(Gpre, ldexpf(ca, s1), ldexpf(ia[sc], s0)), up);
            fb[sc] = ldexpf(fmaf(Gpre, ldexpf(cb, s1), ldexpf(ib[sc], s0)), up);
            fc[sc] = ldexpf(fmaf(Gpost, ldexpf(cc, s2_), ldexpf(ic[sc], s0)), up);
            fd[sc] = ldexpf(fmaf(Gpost, ldexpf(cd, s2_), ldexpf(id[sc], s0)), up);
        }
        // y leaves through the region read last (the others are being filled)
        unsigned y_base = (unsigned)(wave * (2 * LR * WAVE));
        asm volatile("" : "+v"(y_base));                                  // as for the row reads
        IO* yrows = region(STATIC_REG ? NSC - 1 : (n - 1) % NREG) + y_base;
#pragma unroll
        for (int sc = 0; sc < NSC; ++sc) {
            __builtin_amdgcn_sched_barrier(0);                            // one super-chunk's sweeps at a time
            float a = fa[sc], bb = fb[sc], c = fc[sc], d = fd[sc];
            const float nrw = -Rw[sc];
            float PN[L], PD[L];
#pragma unroll
            for (int j = 0; j < L; ++j) {
                const float kk = to_f32(__builtin_bit_cast(IO, (unsigned short)(raw[sc][j] & 0xffffu)));
                const float vv = to_f32(__builtin_bit_cast(IO, (unsigned short)(raw[sc][j] >> 16)));
                const float E = fast_exp2(fmaf(kk, LOG2E, nrw));
                const float Ev = E * vv;
                PN[j] = fmaf(cu, Ev, a);
                PD[j] = fmaf(cu, E, bb);
                a = fmaf(gd, a, Ev);
                bb = fmaf(gd, bb, E);
            }
#pragma unroll
            for (int j = L - 1; j >= 0; --j) {
                const float kk = to_f32(__builtin_bit_cast(IO, (unsigned short)(raw[sc][j] & 0xffffu)));
                const float vv = to_f32(__builtin_bit_cast(IO, (unsigned short)(raw[sc][j] >> 16)));
                const float E = fast_exp2(fmaf(kk, LOG2E, nrw));
                const float Ev = E * vv;
                const float out = (PN[j] + c) * fast_rcp(PD[j] + d);
                c = fmaf(gd, c, Ev);
                d = fmaf(gd, d, E);
                lds_put<IO>(yrows, j * WAVE + lane, from_f32<IO>(out));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            int tw = (sc * S + wave) * L;
            asm volatile("" : "+v"(tw));             // as in issue_rows
            const int Cs = C;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int rl = RPI * i + lane / LPR;
                const int rowt = tw + rl;
                const unsigned vo = (rl < L && rowt < T && cq < Cs) ? (unsigned)((rowt * Cs + cq) * (int)sizeof(IO)) : OOB_OFFSET;
                const BufRaw<16>::type val = lds_get16<IO>(yrows, rl * WAVE + (lane % LPR) * EPL);
                BufRaw<16>::template st<CPOL_NT>(val, ry, vo, 0);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // the y rows are read before they are rewritten
        }
    }
}

}  // namespace biwkv_fwd_detail
}  // namespace vrwkv
