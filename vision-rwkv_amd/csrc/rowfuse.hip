// Fused row-wise epilogues of the VRWKV blocks: for every row (token) of N channels
//   y   = LayerNorm(pre(a)) * ln_weight + ln_bias        (LayerNorm optional; pre = identity or relu(.)^2)
//   out = y | sigmoid(other) * y | other + gamma * y      (gamma optional)
// in one pass over memory.  These are the element-wise steps around the WKV operator and the GEMMs that the reference
// runs as separate PyTorch kernels (classification/mmcls_custom/models/backbones/vrwkv.py):
//   :184-186  rwkv = key_norm(rwkv); rwkv = sr * rwkv             -> a = rwkv, other = receptance(xr), LayerNorm, sigmoid gate
//   :256-260  k = square(relu(key(xk))); k = key_norm(k)           -> a = key(xk), pre = relu^2, LayerNorm
//   :261      sigmoid(receptance(xr)) * kv                         -> a = kv, other = receptance(xr), sigmoid gate
//   :300-313  x = x + gamma * ln(att(x)) / x + gamma * att(ln(x))  -> a = branch output, other = x, (LayerNorm,) gamma
// One wave per row of up to 128 16-byte vectors, the four waves of a workgroup per longer row: a thread keeps its vectors
// of the row in registers (read once, every load of a group's rows issued before the first value is used), the mean and
// the variance are reduced in fp32 (two passes over the registers), the result is written once.
//
// Backward (vrwkv_rowfuse_bwd; the reference differentiates the PyTorch ops by autograd): with g the gradient of out,
// z = pre(a), xh = (z - mean) rstd, y = xh w + b (y = z without LayerNorm):
//   gate:      gy = g sigmoid(o),  g_other = g y sigmoid(o) (1 - sigmoid(o))
//   residual:  gy = g gamma,       g_other = g (not written: it is g itself),  g_gamma[c] = sum_rows g y
//   LayerNorm: g_w[c] = sum_rows gy xh,  g_b[c] = sum_rows gy,  gz = rstd (w gy - mean(w gy) - xh mean(w gy xh))
//   pre:       ga = gz 2 relu(a)  (relu^2)  or  gz
// A wave recomputes the row statistics from `a` and keeps the per-channel sums of its lanes' channels in registers; the
// waves of a workgroup add theirs in LDS and write one partial row per gradient, which batch_sum_kernel adds over the
// workgroups in a fixed order.
#include "vrwkv_common.h"

namespace vrwkv {
namespace {

enum { PRE_NONE = 0, PRE_RELU_SQ = 1 };
enum { POST_NONE = 0, POST_SIGMOID_GATE = 1, POST_RESIDUAL = 2 };

// Sum over the 64 lanes, the same value in every lane: four DPP steps inside each row of 16 lanes (quad swaps, half-row
// and row mirrors), then the four row sums through scalar registers.  All lanes must be active.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
    return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float wave_sum(float x) {
    x = dpp_add<0xB1>(x);      // quad_perm [1,0,3,2]
    x = dpp_add<0x4E>(x);      // quad_perm [2,3,0,1]
    x = dpp_add<0x141>(x);     // row_half_mirror
    x = dpp_add<0x140>(x);     // row_mirror
    const int xi = __builtin_bit_cast(int, x);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 0)),
                r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 16)),
                r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 32)),
                r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 48));
    return (r0 + r1) + (r2 + r3);
}

// W waves share a row (1: a wave per row, short rows; 4: the workgroup's four waves, long rows), a thread keeps VPL
// 16-byte vectors of it.  A group takes R rows whose loads are all issued before the first value is used, so a thread
// has 2 x 16 bytes x VPL x R in flight; workgroups are short and many, the dispatcher evens out the load.  R = 2 for
// short rows, but 1 where a wave has a 16-bit row to itself (768 channels, sigmoid gate: 13.4 us with two rows per wave,
// 12.1 us with one; four rows 15.6 us; a resident grid of 1024 workgroups walking the rows: no difference).
template <int VPL, int ES, int W> constexpr int rows_per_group_fwd() { return VPL <= 2 && (ES == 4 || W > 1) ? 2 : 1; }

template <typename IO, int VPL, int W, int PRE, int POST, bool HAS_LN>
__global__ __launch_bounds__(256)
void rowfuse_kernel(const IO* __restrict__ a_, const IO* __restrict__ other_, const IO* __restrict__ lnw_,
                    const IO* __restrict__ lnb_, const IO* __restrict__ gamma_, IO* __restrict__ out_,
                    long long rows, int N, float eps)
{
    constexpr int V = 16 / (int)sizeof(IO);
    constexpr int R = rows_per_group_fwd<VPL, (int)sizeof(IO), W>();
    constexpr int GROUP = WAVE * W;                            // threads per row
    __shared__ float s_red[W > 1 ? 2 * R : 1][4];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const int tid = W == 1 ? lane : (int)threadIdx.x;
    const int nvec = N / V;
    const bool has_gamma = POST == POST_RESIDUAL && gamma_ != nullptr;
    const long long row0 = (W == 1 ? (long long)blockIdx.x * (blockDim.x >> 6) + wave : (long long)blockIdx.x) * R;
    if (row0 >= rows) return;                                 // whole waves (W = 1) or whole workgroups (W = 4) leave
    // the sum over a row's threads, the same value in all of them; `slot` is used once per kernel
    auto group_sum = [&](float v, int slot) -> float {
        v = wave_sum(v);
        if constexpr (W > 1) {
            if (lane == 0) s_red[slot][wave] = v;
            __syncthreads();
            v = (s_red[slot][0] + s_red[slot][1]) + (s_red[slot][2] + s_red[slot][3]);
        }
        return v;
    };
    // every load is issued before the first value is used: the rows and `other` are streamed (non-temporal), the
    // per-channel vectors come from the caches; a vector waits in four registers and is widened where it is used
    nt_u32x4 a_raw[R][VPL], o_raw[R][VPL], w_raw[VPL], b_raw[VPL], g_raw[VPL];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const bool row_ok = row0 + j < rows;                  // uniform over the group
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int vi = tid + GROUP * i;
            a_raw[j][i] = o_raw[j][i] = nt_u32x4{0u, 0u, 0u, 0u};
            if (row_ok && vi < nvec) {
                const size_t off = (size_t)(row0 + j) * N + (size_t)vi * V;
                a_raw[j][i] = load_raw16<true>(a_ + off);
                if (POST != POST_NONE) o_raw[j][i] = load_raw16<true>(other_ + off);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int vi = tid + GROUP * i;
        w_raw[i] = b_raw[i] = g_raw[i] = nt_u32x4{0u, 0u, 0u, 0u};
        if (vi < nvec) {
            const size_t c = (size_t)vi * V;
            if (HAS_LN) { w_raw[i] = load_raw16<false>(lnw_ + c); b_raw[i] = load_raw16<false>(lnb_ + c); }
            if (has_gamma) g_raw[i] = load_raw16<false>(gamma_ + c);
        }
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const long long row = row0 + j;
        if (row >= rows) break;                               // uniform over the group
        float x[VPL][V];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            widen_raw16<IO, V>(a_raw[j][i], x[i]);            // threads past the row hold zeros
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if (PRE == PRE_RELU_SQ) { const float r = fmaxf(x[i][e], 0.f); x[i][e] = r * r; }
                s += x[i][e];
            }
        }
        float mean = 0.f, rstd = 1.f;
        if (HAS_LN) {
            mean = group_sum(s, 2 * j) / (float)N;
            float q = 0.f;
#pragma unroll
            for (int i = 0; i < VPL; ++i)
                if (tid + GROUP * i < nvec) {
#pragma unroll
                    for (int e = 0; e < V; ++e) { const float d = x[i][e] - mean; q = fmaf(d, d, q); }
                }
            rstd = rsqrtf(group_sum(q, 2 * j + 1) / (float)N + eps);
        }
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int vi = tid + GROUP * i;
            if (vi >= nvec) continue;
            const size_t c = (size_t)vi * V;
            float y[V];
            if (HAS_LN) {
                float w[V], b[V];
                widen_raw16<IO, V>(w_raw[i], w);
                widen_raw16<IO, V>(b_raw[i], b);
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = fmaf((x[i][e] - mean) * rstd, w[e], b[e]);
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = x[i][e];
            }
            if (POST == POST_SIGMOID_GATE) {
                float o[V];
                widen_raw16<IO, V>(o_raw[j][i], o);
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] *= fast_rcp(1.f + fast_exp2(-o[e] * LOG2E));
            } else if (POST == POST_RESIDUAL) {
                float o[V], gm[V];
                widen_raw16<IO, V>(o_raw[j][i], o);
                widen_raw16<IO, V>(g_raw[i], gm);
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = has_gamma ? fmaf(gm[e], y[e], o[e]) : o[e] + y[e];
            }
            store_vec_nt<IO, V>(out_ + row * N + c, y);
        }
    }
}

// Backward without LayerNorm and gamma: nothing couples the channels of a row and no parameter gradient exists, a
// plain element-wise pass (runtime switches, all wave-uniform); a wave takes a run of consecutive rows.
template <typename IO, int VPL>
__global__ __launch_bounds__(256)
void rowfuse_bwd_plain_kernel(const IO* __restrict__ a_, const IO* __restrict__ other_, const IO* __restrict__ g_,
                              IO* __restrict__ ga_, IO* __restrict__ go_, long long rows, int N, int pre, int post,
                              int rows_per_wave)
{
    constexpr int V = 16 / (int)sizeof(IO);
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const int nvec = N / V;
    const long long row0 = ((long long)blockIdx.x * (blockDim.x >> 6) + wave) * rows_per_wave;
    for (int rr = 0; rr < rows_per_wave; ++rr) {
        const long long row = row0 + rr;
        if (row >= rows) break;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int vi = lane + WAVE * i;
            if (vi >= nvec) continue;
            const size_t off = (size_t)row * N + (size_t)vi * V;
            float av[V], gv[V], ov[V], go[V], ga[V];
            load_vec<IO, V>(a_ + off, av);
            load_vec<IO, V>(g_ + off, gv);
            if (post == POST_SIGMOID_GATE) load_vec<IO, V>(other_ + off, ov);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float rl = fmaxf(av[e], 0.f);
                const float y = pre == PRE_RELU_SQ ? rl * rl : av[e];
                float gy = gv[e];
                if (post == POST_SIGMOID_GATE) {
                    const float sg = fast_rcp(1.f + fast_exp2(-ov[e] * LOG2E));
                    go[e] = gy * y * sg * (1.f - sg);
                    gy *= sg;
                }
                ga[e] = pre == PRE_RELU_SQ ? gy * 2.f * rl : gy;
            }
            if (post == POST_SIGMOID_GATE) store_vec<IO, V>(go_ + off, go);
            store_vec<IO, V>(ga_ + off, ga);
        }
    }
}

// Backward with LayerNorm and / or gamma (per-channel parameter gradients = sums over the rows).
// Every parameter gradient is a combination of two per-channel sums over the rows, with G = g (g sigmoid(o) under
// the gate) and xh the normalised row (z itself without LayerNorm):
//   S0[c] = sum_rows G,   S1[c] = sum_rows G xh
//   LayerNorm alone, or with the gate:   g_w = S1,        g_b = S0
//   LayerNorm and residual:              g_w = gamma S1,  g_b = gamma S0,  g_gamma = w S1 + b S0
//   residual without LayerNorm:          g_gamma = S1
// so a lane keeps two sums per channel in registers.  A lane owns VPL vectors of V channels; (V, VPL) is picked by the
// host so that the row fills the 64 lanes as well as it can (768 16-bit channels: three 8-byte vectors per lane).
// Rows are dealt out wave by wave over the whole grid, a wave requests its next row before it works on the current
// one.  Up to 12 channels per lane fit 128 registers: workgroups of eight waves, two per compute unit (four waves per
// SIMD); more channels per lane (and the gate, which also keeps the bias): workgroups of four waves, three (two) per
// compute unit.  The waves' sums are added in wave order through LDS, combined into the three gradient rows and
// written as the workgroup's partial rows, which batch_sum_kernel adds over the workgroups in a fixed order.
template <typename IO, int V, int VPL, int POST>
struct BwsShape {
    static constexpr int CH = V * VPL;
    static constexpr bool GATE = POST == POST_SIGMOID_GATE;
    static constexpr bool HEAVY = CH > 12 || (sizeof(IO) == 4 && CH > 8) || (GATE && CH > 8);
    static constexpr int WAVES = HEAVY ? 4 : 8;
    static constexpr int MIN_WAVES_PER_SIMD = !HEAVY ? 4 : (GATE || (sizeof(IO) == 4 && CH > 12)) ? 2 : 3;
    static constexpr int MAX_WG = 256 * (MIN_WAVES_PER_SIMD * 4 / WAVES);   // resident workgroups of the 256 compute units
};
constexpr int BWS_MAX_PARTIAL_ROWS = 768;     // the largest MAX_WG

template <int BYTES> struct Pk;
template <> struct Pk<16> { typedef unsigned int type __attribute__((ext_vector_type(4))); };
template <> struct Pk<8>  { typedef unsigned int type __attribute__((ext_vector_type(2))); };
template <typename IO, int V>
__device__ __forceinline__ void widen_pk(typename Pk<sizeof(IO) * V>::type raw, float (&out)[V]) {
    IO tmp[V];
    __builtin_memcpy(tmp, &raw, sizeof(raw));
#pragma unroll
    for (int e = 0; e < V; ++e) out[e] = to_f32(tmp[e]);
}
template <typename IO, int V>
__device__ __forceinline__ typename Pk<sizeof(IO) * V>::type pack_pk(const float (&in)[V]) {
    using T = typename Pk<sizeof(IO) * V>::type;
    IO tmp[V];
#pragma unroll
    for (int e = 0; e < V; ++e) tmp[e] = from_f32<IO>(in[e]);
    T raw;
    __builtin_memcpy(&raw, tmp, sizeof(raw));
    return raw;
}

template <typename IO, int V, int VPL, int POST, bool HAS_LN>
__global__ __launch_bounds__((WAVE * BwsShape<IO, V, VPL, POST>::WAVES), (BwsShape<IO, V, VPL, POST>::MIN_WAVES_PER_SIMD))
void rowfuse_bwd_sums_kernel(const IO* __restrict__ a_, const IO* __restrict__ other_, const IO* __restrict__ lnw_,
                             const IO* __restrict__ lnb_, const IO* __restrict__ gamma_, const IO* __restrict__ g_,
                             IO* __restrict__ ga_, IO* __restrict__ go_, float* __restrict__ part,
                             long long rows, int N, float eps, int pre)
{
    constexpr int VB = V * (int)sizeof(IO);
    constexpr bool GATE = POST == POST_SIGMOID_GATE;
    constexpr int BWS_WAVES = BwsShape<IO, V, VPL, POST>::WAVES;
    using Raw = typename Pk<VB>::type;
    extern __shared__ float s_red[];                          // [wave][S0, S1][N]
    const int lane = threadIdx.x & (WAVE - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nvec = N / V;
    const bool has_gamma = POST == POST_RESIDUAL && gamma_ != nullptr;
    // per-channel factor of G in the gradient that goes back through the LayerNorm: w, w gamma, or gamma
    float wg[VPL][V], S0[VPL][V], S1[VPL][V];
    Raw b_raw[GATE ? VPL : 1];
    // A row is addressed through a descriptor of exactly its bytes: lanes past the row read zeros and store nothing.
    const unsigned row_bytes = (unsigned)N * (unsigned)sizeof(IO);
    unsigned voff[VPL];
    bool ok[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int vi = lane + WAVE * i;
        ok[i] = vi < nvec;
        voff[i] = (unsigned)vi * VB;
    }
    const long long stride = (long long)gridDim.x * BWS_WAVES;
    long long row = (long long)blockIdx.x * BWS_WAVES + wave;
    Raw a_cur[VPL], g_cur[VPL], o_cur[GATE ? VPL : 1];
    // a row past the end is requested through an empty descriptor: nothing is read
    auto fetch = [&](long long r, Raw (&ar)[VPL], Raw (&gr)[VPL], Raw (&orr)[GATE ? VPL : 1]) {
        const unsigned nb = r < rows ? row_bytes : 0u;
        const size_t eo = r < rows ? (size_t)r * N : 0;
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(a_ + eo, nb), rg = make_rsrc(g_ + eo, nb);
        const __amdgpu_buffer_rsrc_t ro = make_rsrc((GATE ? other_ : a_) + eo, nb);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            ar[i] = BufRaw<VB>::template ld<CPOL_NT>(ra, voff[i], 0);
            gr[i] = BufRaw<VB>::template ld<CPOL_NT>(rg, voff[i], 0);
            if (GATE) orr[i] = BufRaw<VB>::template ld<CPOL_NT>(ro, voff[i], 0);
        }
    };
    // the first row is requested before the per-channel vectors: both are on their way together
    fetch(row, a_cur, g_cur, o_cur);
    {
        // null parameters read a valid one and are replaced by 1: no branches around the loads
        const __amdgpu_buffer_rsrc_t rw = make_rsrc(HAS_LN ? lnw_ : gamma_, row_bytes), rgm = make_rsrc(has_gamma ? gamma_ : lnw_, row_bytes);
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(GATE ? lnb_ : (HAS_LN ? lnw_ : gamma_), row_bytes);
        Raw w_raw[VPL], gm_raw[VPL];
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            w_raw[i] = BufRaw<VB>::ld(rw, voff[i], 0);
            gm_raw[i] = BufRaw<VB>::ld(rgm, voff[i], 0);
            if (GATE) b_raw[i] = BufRaw<VB>::ld(rb, voff[i], 0);
        }
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            float w[V], gm[V];
            widen_pk<IO, V>(w_raw[i], w);
            widen_pk<IO, V>(gm_raw[i], gm);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float wv = HAS_LN ? w[e] : 1.f, gv = has_gamma ? gm[e] : 1.f;
                wg[i][e] = ok[i] ? wv * gv : 0.f;
                S0[i][e] = S1[i][e] = 0.f;
            }
        }
    }
    const float inv_n = 1.f / (float)N;
    // one row: statistics, gradients, sums
    auto process = [&](long long row, const Raw (&a_raw)[VPL], const Raw (&g_raw)[VPL], const Raw (&o_raw)[GATE ? VPL : 1]) {
        const __amdgpu_buffer_rsrc_t rga = make_rsrc(ga_ + (size_t)row * N, row_bytes);
        const __amdgpu_buffer_rsrc_t rgo = make_rsrc((GATE ? go_ : ga_) + (size_t)row * N, row_bytes);
        float z[VPL][V], t[VPL][V];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            widen_pk<IO, V>(a_raw[i], z[i]);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if (pre == PRE_RELU_SQ) { const float r = fmaxf(z[i][e], 0.f); z[i][e] = r * r; }
                s += z[i][e];
            }
        }
        float rstd = 1.f;
        if (HAS_LN) {
            const float mean = wave_sum(s) * inv_n;
            float q = 0.f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const float mi = ok[i] ? mean : 0.f;
#pragma unroll
                for (int e = 0; e < V; ++e) { z[i][e] -= mi; q = fmaf(z[i][e], z[i][e], q); }
            }
            rstd = rsqrtf(wave_sum(q) * inv_n + eps);
        }
        // z becomes xh (normalised) under LayerNorm; t the gradient on xh
        float t1 = 0.f, t2 = 0.f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            float G[V], go[V], o[V], b[V];
            widen_pk<IO, V>(g_raw[i], G);
            if (GATE) { widen_pk<IO, V>(o_raw[i], o); widen_pk<IO, V>(b_raw[i], b); }
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float xh = HAS_LN ? z[i][e] * rstd : z[i][e];
                float Gv = G[e];
                if (GATE) {
                    const float sg = fast_rcp(1.f + fast_exp2(-o[e] * LOG2E));
                    const float y = fmaf(xh, wg[i][e], b[e]);             // the gate always comes with LayerNorm here
                    Gv *= sg;
                    go[e] = Gv * y * (1.f - sg);
                }
                S0[i][e] += Gv;
                S1[i][e] = fmaf(Gv, xh, S1[i][e]);
                const float tt = Gv * wg[i][e];
                if (HAS_LN) { t1 += tt; t2 = fmaf(tt, xh, t2); }
                z[i][e] = xh;
                t[i][e] = tt;
            }
            if (GATE) BufRaw<VB>::template st<CPOL_NT>(pack_pk<IO, V>(go), rgo, voff[i], 0);
        }
        float m1 = 0.f, m2 = 0.f;
        if (HAS_LN) { m1 = wave_sum(t1) * inv_n; m2 = wave_sum(t2) * inv_n; }
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            float ga[V], av[V];
            if (pre == PRE_RELU_SQ) widen_pk<IO, V>(a_raw[i], av);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float gz = HAS_LN ? rstd * (t[i][e] - m1 - z[i][e] * m2) : t[i][e];
                ga[e] = pre == PRE_RELU_SQ ? gz * 2.f * fmaxf(av[e], 0.f) : gz;
            }
            BufRaw<VB>::template st<CPOL_NT>(pack_pk<IO, V>(ga), rga, voff[i], 0);
        }
    };
    // two sets of row registers take turns: one is refilled while the other is worked on (copying a set would wait
    // for its loads)
    Raw a_alt[VPL], g_alt[VPL], o_alt[GATE ? VPL : 1];
    while (row < rows) {
        fetch(row + stride, a_alt, g_alt, o_alt);
        process(row, a_cur, g_cur, o_cur);
        row += stride;
        if (row >= rows) break;
        fetch(row + stride, a_cur, g_cur, o_cur);
        process(row, a_alt, g_alt, o_alt);
        row += stride;
    }
    // the eight waves' sums, added in wave order, give this workgroup's partial gradient rows
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        if (!ok[i]) continue;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            s_red[((size_t)wave * 2 + 0) * N + (lane + WAVE * i) * V + e] = S0[i][e];
            s_red[((size_t)wave * 2 + 1) * N + (lane + WAVE * i) * V + e] = S1[i][e];
        }
    }
    __syncthreads();
    float* prow = part + (size_t)blockIdx.x * 3 * N;
    for (int c = threadIdx.x; c < N; c += WAVE * BWS_WAVES) {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int wv = 0; wv < BWS_WAVES; ++wv) {
            s0 += s_red[((size_t)wv * 2 + 0) * N + c];
            s1 += s_red[((size_t)wv * 2 + 1) * N + c];
        }
        const float w = HAS_LN ? to_f32(lnw_[c]) : 1.f, b = HAS_LN ? to_f32(lnb_[c]) : 0.f;
        const float gm = has_gamma ? to_f32(gamma_[c]) : 1.f;
        prow[c] = HAS_LN ? gm * s1 : 0.f;
        prow[N + c] = HAS_LN ? gm * s0 : 0.f;
        prow[2 * N + c] = has_gamma ? (HAS_LN ? fmaf(w, s1, b * s0) : s1) : 0.f;
    }
}

constexpr int BWD_ROWS_PER_WAVE_PLAIN = 2;   // element-wise only: many short workgroups

static long long bwd_sums_workgroups(long long rows, int waves, int max_wg) {
    const long long n = (rows + waves - 1) / waves;
    return n < max_wg ? n : max_wg;
}

template <typename IO, int V, int VPL, int POST, bool LN>
int launch_bwd_sums_mode(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma,
                         const void* g, void* ga, void* go, float* gparam, float* part, long long rows, int N, int pre,
                         float eps, hipStream_t st) {
    using Shape = BwsShape<IO, V, VPL, POST>;
    const int nwg = (int)bwd_sums_workgroups(rows, Shape::WAVES, Shape::MAX_WG);
    const size_t lds = (size_t)Shape::WAVES * 2 * N * sizeof(float);
    auto kernel = rowfuse_bwd_sums_kernel<IO, V, VPL, POST, LN>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)nwg), dim3(WAVE * Shape::WAVES), lds, st,
                       static_cast<const IO*>(a), static_cast<const IO*>(other), static_cast<const IO*>(lnw),
                       static_cast<const IO*>(lnb), static_cast<const IO*>(gamma), static_cast<const IO*>(g),
                       static_cast<IO*>(ga), static_cast<IO*>(go), part, rows, N, eps, pre);
    const int wide = 3 * N;                                   // gparam: (3, N) = g_weight, g_bias, g_gamma
    hipLaunchKernelGGL(batch_sum_kernel, dim3((wide + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, part, gparam,
                       (const float*)nullptr, (float*)nullptr, nwg, wide);
    return check_launch("rowfuse_bwd");
}

template <typename IO, int V, int VPL>
int launch_bwd_sums(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, const void* g,
                    void* ga, void* go, float* gparam, float* part, long long rows, int N, int pre, int post, float eps,
                    hipStream_t st) {
#define VRWKV_SUMS(POST, LN) return launch_bwd_sums_mode<IO, V, VPL, POST, LN>(a, other, lnw, lnb, gamma, g, ga, go, gparam, part, rows, N, pre, eps, st)
    if (post == POST_SIGMOID_GATE) VRWKV_SUMS(POST_SIGMOID_GATE, true);
    if (post == POST_RESIDUAL && lnw) VRWKV_SUMS(POST_RESIDUAL, true);
    if (post == POST_RESIDUAL) VRWKV_SUMS(POST_RESIDUAL, false);
    VRWKV_SUMS(POST_NONE, true);
#undef VRWKV_SUMS
}

template <typename IO, int VPL>
int launch_bwd_plain(const void* a, const void* other, const void* g, void* ga, void* go, long long rows, int N, int pre,
                     int post, hipStream_t st) {
    const int rows_per_block = 4 * BWD_ROWS_PER_WAVE_PLAIN;
    const long long nblk = (rows + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL((rowfuse_bwd_plain_kernel<IO, VPL>), dim3((unsigned)nblk), dim3(256), 0, st,
                       static_cast<const IO*>(a), static_cast<const IO*>(other), static_cast<const IO*>(g),
                       static_cast<IO*>(ga), static_cast<IO*>(go), rows, N, pre, post, BWD_ROWS_PER_WAVE_PLAIN);
    return check_launch("rowfuse_bwd");
}

template <typename IO>
int launch_bwd_io(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, const void* g,
                  void* ga, void* go, float* gparam, float* part, long long rows, int N, int pre, int post, float eps,
                  hipStream_t st) {
    constexpr int V = 16 / (int)sizeof(IO);
    const int per_lane = (N / V + WAVE - 1) / WAVE;
    const bool sums = lnw != nullptr || (post == POST_RESIDUAL && gamma != nullptr);
    if (sums) {                                               // at most 16 channels per lane (checked by the caller)
#define VRWKV_BWD(V_, VPL) return launch_bwd_sums<IO, V_, VPL>(a, other, lnw, lnb, gamma, g, ga, go, gparam, part, rows, N, pre, post, eps, st)
        if constexpr (sizeof(IO) == 2) {
            // 8-byte vectors where they fill the lanes better than 16-byte ones (192, 768 channels)
            constexpr int V8 = V / 2;
            const int per8 = (N / V8 + WAVE - 1) / WAVE;
            const bool narrow = per8 <= 3 && per8 * V8 < per_lane * V;
            if (narrow) {
                if (per8 <= 1) VRWKV_BWD(V8, 1);
                if (per8 <= 2) VRWKV_BWD(V8, 2);
                VRWKV_BWD(V8, 3);
            }
            if (per_lane <= 1) VRWKV_BWD(V, 1);
            VRWKV_BWD(V, 2);
        } else {
            if (per_lane <= 1) VRWKV_BWD(V, 1);
            if (per_lane <= 2) VRWKV_BWD(V, 2);
            if (per_lane <= 3) VRWKV_BWD(V, 3);
            VRWKV_BWD(V, 4);
        }
#undef VRWKV_BWD
    }
#define VRWKV_BWD(VPL) return launch_bwd_plain<IO, VPL>(a, other, g, ga, go, rows, N, pre, post, st)
    if (per_lane <= 1) VRWKV_BWD(1);
    if (per_lane <= 2) VRWKV_BWD(2);
    if (per_lane <= 4) VRWKV_BWD(4);
    if (per_lane <= 8) VRWKV_BWD(8);
    VRWKV_BWD(16);
#undef VRWKV_BWD
}

template <typename IO, int VPL, int W, int PRE, int POST>
int launch_ln(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, void* out,
              long long rows, int N, float eps, hipStream_t st) {
    constexpr int per_wg = (W == 1 ? 4 : 1) * rows_per_group_fwd<VPL, (int)sizeof(IO), W>();
    if ((rows + per_wg - 1) / per_wg > 0x7fffffffLL) {
        set_error("rowfuse: too many rows (%lld)", rows);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const dim3 block(256), grid((unsigned)((rows + per_wg - 1) / per_wg));
    const IO *pa = static_cast<const IO*>(a), *po = static_cast<const IO*>(other), *pw = static_cast<const IO*>(lnw),
             *pb = static_cast<const IO*>(lnb), *pg = static_cast<const IO*>(gamma);
    IO* pout = static_cast<IO*>(out);
    if (lnw) hipLaunchKernelGGL((rowfuse_kernel<IO, VPL, W, PRE, POST, true>), grid, block, 0, st, pa, po, pw, pb, pg, pout, rows, N, eps);
    else     hipLaunchKernelGGL((rowfuse_kernel<IO, VPL, W, PRE, POST, false>), grid, block, 0, st, pa, po, pw, pb, pg, pout, rows, N, eps);
    return check_launch("rowfuse");
}

template <typename IO, int VPL, int W>
int launch_ops(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, void* out,
               long long rows, int N, int pre, int post, float eps, hipStream_t st) {
#define VRWKV_ROW(PRE, POST) return launch_ln<IO, VPL, W, PRE, POST>(a, other, lnw, lnb, gamma, out, rows, N, eps, st)
    if (pre == PRE_NONE) {
        if (post == POST_NONE) VRWKV_ROW(PRE_NONE, POST_NONE);
        if (post == POST_SIGMOID_GATE) VRWKV_ROW(PRE_NONE, POST_SIGMOID_GATE);
        VRWKV_ROW(PRE_NONE, POST_RESIDUAL);
    }
    if (post == POST_NONE) VRWKV_ROW(PRE_RELU_SQ, POST_NONE);
    if (post == POST_SIGMOID_GATE) VRWKV_ROW(PRE_RELU_SQ, POST_SIGMOID_GATE);
    VRWKV_ROW(PRE_RELU_SQ, POST_RESIDUAL);
#undef VRWKV_ROW
}

template <typename IO>
int launch_io(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, void* out,
              long long rows, int N, int pre, int post, float eps, hipStream_t st) {
    constexpr int V = 16 / (int)sizeof(IO);
    const int nvec = N / V;
    // rows of up to 128 vectors: a wave per row; longer ones: the four waves of a workgroup per row
    if (nvec <= WAVE)     return launch_ops<IO, 1, 1>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    if (nvec <= 2 * WAVE) return launch_ops<IO, 2, 1>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    if (nvec <= 4 * WAVE) return launch_ops<IO, 1, 4>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    if (nvec <= 8 * WAVE) return launch_ops<IO, 2, 4>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    return launch_ops<IO, 4, 4>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" int vrwkv_rowfuse(const void* a, const void* other, const void* ln_weight, const void* ln_bias,
                             const void* gamma, void* out, long long rows, int N, int pre, int post, float eps,
                             int io_dtype, void* hip_stream) {
    if (rows <= 0 || N <= 0 || pre < 0 || pre > 1 || post < 0 || post > 2) {
        set_error("rowfuse: bad arguments (rows=%lld N=%d pre=%d post=%d)", rows, N, pre, post);
        return VRWKV_INVALID_ARG;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("rowfuse: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (!a || !out || (post != POST_NONE && !other) || ((ln_weight == nullptr) != (ln_bias == nullptr))) {
        set_error("rowfuse: null pointer argument (other is required with a gate or a residual; LayerNorm takes weight and bias)");
        return VRWKV_INVALID_ARG;
    }
    const int V = io_dtype == VRWKV_F32 ? 4 : 8;
    if (N % V != 0 || N / V > 16 * WAVE) {
        set_error("rowfuse: N=%d must be a multiple of %d and at most %d", N, V, 16 * WAVE * V);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (rows > 0x7fffffffLL * 4) {
        set_error("rowfuse: too many rows (%lld)", rows);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const uintptr_t all = (uintptr_t)a | (uintptr_t)out | (uintptr_t)other | (uintptr_t)ln_weight | (uintptr_t)ln_bias | (uintptr_t)gamma;
    if (all & 15) {
        set_error("rowfuse: every tensor must be 16-byte aligned");
        return VRWKV_INVALID_ARG;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    switch (io_dtype) {
        case VRWKV_F32:  return launch_io<float>(a, other, ln_weight, ln_bias, gamma, out, rows, N, pre, post, eps, st);
        case VRWKV_BF16: return launch_io<__hip_bfloat16>(a, other, ln_weight, ln_bias, gamma, out, rows, N, pre, post, eps, st);
        case VRWKV_F16:  return launch_io<__half>(a, other, ln_weight, ln_bias, gamma, out, rows, N, pre, post, eps, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}

// Channel sums are kept in registers: the backward with LayerNorm or gamma takes rows of at most 16 channels per lane.
static int rowfuse_bwd_max_n(int) { return 16 * WAVE; }

extern "C" size_t vrwkv_rowfuse_bwd_workspace_bytes(long long rows, int N) {
    if (rows <= 0 || N <= 0) return 0;
    return (size_t)bwd_sums_workgroups(rows, 4, BWS_MAX_PARTIAL_ROWS) * 3 * N * sizeof(float);
}

extern "C" int vrwkv_rowfuse_bwd(const void* a, const void* other, const void* ln_weight, const void* ln_bias,
                                 const void* gamma, const void* gout, void* ga, void* gother, float* gparam,
                                 long long rows, int N, int pre, int post, float eps, int io_dtype,
                                 void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (rows <= 0 || N <= 0 || pre < 0 || pre > 1 || post < 0 || post > 2) {
        set_error("rowfuse_bwd: bad arguments (rows=%lld N=%d pre=%d post=%d)", rows, N, pre, post);
        return VRWKV_INVALID_ARG;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("rowfuse_bwd: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    const bool sums = ln_weight != nullptr || (post == POST_RESIDUAL && gamma != nullptr);
    if (!a || !gout || !ga || (post != POST_NONE && !other) || (post == POST_SIGMOID_GATE && !gother) ||
        ((ln_weight == nullptr) != (ln_bias == nullptr)) || (sums && !gparam)) {
        set_error("rowfuse_bwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    const int V = io_dtype == VRWKV_F32 ? 4 : 8;
    if (N % V != 0 || N / V > 16 * WAVE || (sums && N > rowfuse_bwd_max_n(io_dtype)) || rows > 0x7fffffffLL * 32) {
        set_error("rowfuse_bwd: N=%d must be a multiple of %d, at most %d (%d with LayerNorm or gamma)", N, V,
                  16 * WAVE * V, rowfuse_bwd_max_n(io_dtype));
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const uintptr_t all = (uintptr_t)a | (uintptr_t)other | (uintptr_t)ln_weight | (uintptr_t)ln_bias | (uintptr_t)gamma |
                          (uintptr_t)gout | (uintptr_t)ga | (uintptr_t)gother;
    if (all & 15) {
        set_error("rowfuse_bwd: every tensor must be 16-byte aligned");
        return VRWKV_INVALID_ARG;
    }
    if (sums) {
        const size_t need = vrwkv_rowfuse_bwd_workspace_bytes(rows, N);
        if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3)) {
            set_error("rowfuse_bwd: a 4-byte aligned workspace of %zu bytes is required", need);
            return VRWKV_WORKSPACE_TOO_SMALL;
        }
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* part = static_cast<float*>(workspace);
    switch (io_dtype) {
        case VRWKV_F32:  return launch_bwd_io<float>(a, other, ln_weight, ln_bias, gamma, gout, ga, gother, gparam, part, rows, N, pre, post, eps, st);
        case VRWKV_BF16: return launch_bwd_io<__hip_bfloat16>(a, other, ln_weight, ln_bias, gamma, gout, ga, gother, gparam, part, rows, N, pre, post, eps, st);
        case VRWKV_F16:  return launch_bwd_io<__half>(a, other, ln_weight, ln_bias, gamma, gout, ga, gother, gparam, part, rows, N, pre, post, eps, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
