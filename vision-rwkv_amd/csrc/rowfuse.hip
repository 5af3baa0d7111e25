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
// A wave walks a run of consecutive rows, recomputes the row statistics from `a`, keeps the per-channel sums of its
// lanes' channels in registers; the four waves of a workgroup add theirs in LDS and write one partial row per sum,
// which batch_sum_kernel adds over the workgroups in a fixed order.
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
// has 2 x 16 bytes x VPL x R in flight; workgroups are short and many, the dispatcher evens out the load.
template <int VPL> constexpr int rows_per_group_fwd() { return VPL <= 2 ? 2 : 1; }

template <typename IO, int VPL, int W, int PRE, int POST, bool HAS_LN>
__global__ __launch_bounds__(256)
void rowfuse_kernel(const IO* __restrict__ a_, const IO* __restrict__ other_, const IO* __restrict__ lnw_,
                    const IO* __restrict__ lnb_, const IO* __restrict__ gamma_, IO* __restrict__ out_,
                    long long rows, int N, float eps)
{
    constexpr int V = 16 / (int)sizeof(IO);
    constexpr int R = rows_per_group_fwd<VPL>();
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

// Runtime switches (all wave-uniform) instead of template parameters: the backward has many more combinations.
// SUMS: LayerNorm and / or gamma take part (per-channel vectors and sums in registers); without them the kernel is a
// plain element-wise pass and rows may be longer.
template <typename IO, int VPL, bool SUMS>
__global__ __launch_bounds__(256)
void rowfuse_bwd_kernel(const IO* __restrict__ a_, const IO* __restrict__ other_, const IO* __restrict__ lnw_,
                        const IO* __restrict__ lnb_, const IO* __restrict__ gamma_, const IO* __restrict__ g_,
                        IO* __restrict__ ga_, IO* __restrict__ go_, float* __restrict__ part,
                        long long rows, int N, float eps, int pre, int post, int rows_per_wave)
{
    constexpr int V = 16 / (int)sizeof(IO);
    extern __shared__ float s_red[];                          // [4 waves][3 sums][N] when channel sums are wanted
    const bool has_ln = SUMS && lnw_ != nullptr, has_gamma = SUMS && post == POST_RESIDUAL && gamma_ != nullptr;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const int nvec = N / V;
    constexpr int PV = SUMS ? VPL : 1, PE = SUMS ? V : 1;     // the per-channel arrays exist only with SUMS
    float acc_w[PV][PE], acc_b[PV][PE], acc_g[PV][PE];
    nt_u32x4 w_raw[PV], b_raw[PV], gam_raw[PV];              // the per-channel vectors stay packed, widened per row
#pragma unroll
    for (int i = 0; i < PV; ++i) {
        const int vi = lane + WAVE * i;
        const bool ok = vi < nvec;
#pragma unroll
        for (int e = 0; e < PE; ++e) acc_w[i][e] = acc_b[i][e] = acc_g[i][e] = 0.f;
        w_raw[i] = b_raw[i] = gam_raw[i] = nt_u32x4{0u, 0u, 0u, 0u};
        if constexpr (SUMS) {
            if (ok && has_ln) { w_raw[i] = load_raw16<false>(lnw_ + (size_t)vi * V); b_raw[i] = load_raw16<false>(lnb_ + (size_t)vi * V); }
            if (ok && has_gamma) gam_raw[i] = load_raw16<false>(gamma_ + (size_t)vi * V);
        }
    }
    const long long row0 = ((long long)blockIdx.x * (blockDim.x >> 6) + wave) * rows_per_wave;
    if constexpr (!SUMS) {
        // no LayerNorm, no gamma: nothing couples the channels of a row, one vector at a time
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
        return;
    }
    // The rows of a wave go in batches of RB whose loads (a, the incoming gradient, and `other` where the gate needs it)
    // are all issued before the first value is used; a vector waits in four registers and is widened where it is used.
    constexpr int RB = VPL == 1 ? 4 : VPL == 2 ? 2 : 1;
    const bool need_o = post == POST_SIGMOID_GATE;            // the residual's backward does not read `other`
    for (int rb = 0; rb < rows_per_wave; rb += RB) {
        if (row0 + rb >= rows) break;                         // wave-uniform
        nt_u32x4 a_raw[RB][VPL], g_raw[RB][VPL], o_raw[RB][VPL];
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            const bool row_ok = rb + j < rows_per_wave && row0 + rb + j < rows;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const int vi = lane + WAVE * i;
                a_raw[j][i] = g_raw[j][i] = o_raw[j][i] = nt_u32x4{0u, 0u, 0u, 0u};
                if (row_ok && vi < nvec) {
                    const size_t off = (size_t)(row0 + rb + j) * N + (size_t)vi * V;
                    a_raw[j][i] = load_raw16<true>(a_ + off);
                    g_raw[j][i] = load_raw16<true>(g_ + off);
                    if (need_o) o_raw[j][i] = load_raw16<true>(other_ + off);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            const long long row = row0 + rb + j;
            if (rb + j >= rows_per_wave || row >= rows) break;    // wave-uniform
            float r[VPL][V], z[VPL][V], g[VPL][V];
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                widen_raw16<IO, V>(a_raw[j][i], r[i]);        // lanes past the row hold zeros
                widen_raw16<IO, V>(g_raw[j][i], g[i]);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    if (pre == PRE_RELU_SQ) { r[i][e] = fmaxf(r[i][e], 0.f); z[i][e] = r[i][e] * r[i][e]; }
                    else z[i][e] = r[i][e];
                    s += z[i][e];
                }
            }
            float mean = 0.f, rstd = 1.f;
            if (has_ln) {
                mean = wave_sum(s) / (float)N;
                float q = 0.f;
#pragma unroll
                for (int i = 0; i < VPL; ++i)
                    if (lane + WAVE * i < nvec) {
#pragma unroll
                        for (int e = 0; e < V; ++e) { const float d = z[i][e] - mean; q = fmaf(d, d, q); }
                    }
                rstd = rsqrtf(wave_sum(q) / (float)N + eps);
            }
            // z becomes xh (normalised) under LayerNorm; g becomes gy
            float t1 = 0.f, t2 = 0.f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const int vi = lane + WAVE * i;
                if (vi >= nvec) continue;
                float go[V], o[V], w[V], b[V], gam[V];
                if (need_o) widen_raw16<IO, V>(o_raw[j][i], o);
                widen_raw16<IO, V>(w_raw[SUMS ? i : 0], w);
                widen_raw16<IO, V>(b_raw[SUMS ? i : 0], b);
                widen_raw16<IO, V>(gam_raw[SUMS ? i : 0], gam);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const int pi = SUMS ? i : 0, pe = SUMS ? e : 0;
                    const float xh = has_ln ? (z[i][e] - mean) * rstd : z[i][e];
                    const float y = has_ln ? fmaf(xh, w[e], b[e]) : xh;
                    float gy = g[i][e];
                    if (post == POST_SIGMOID_GATE) {
                        const float sg = fast_rcp(1.f + fast_exp2(-o[e] * LOG2E));
                        go[e] = gy * y * sg * (1.f - sg);
                        gy *= sg;
                    } else if (post == POST_RESIDUAL) {
                        if (has_gamma) { acc_g[pi][pe] = fmaf(gy, y, acc_g[pi][pe]); gy *= gam[e]; }
                    }
                    if (has_ln) {
                        acc_b[pi][pe] += gy;
                        acc_w[pi][pe] = fmaf(gy, xh, acc_w[pi][pe]);
                        const float t = w[e] * gy;
                        t1 += t;
                        t2 = fmaf(t, xh, t2);
                        g[i][e] = t;
                    } else {
                        g[i][e] = gy;
                    }
                    z[i][e] = xh;
                }
                if (post == POST_SIGMOID_GATE) store_vec_nt<IO, V>(go_ + (size_t)row * N + (size_t)vi * V, go);
            }
            float m1 = 0.f, m2 = 0.f;
            if (has_ln) { m1 = wave_sum(t1) / (float)N; m2 = wave_sum(t2) / (float)N; }
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const int vi = lane + WAVE * i;
                if (vi >= nvec) continue;
                float ga[V];
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float gz = has_ln ? rstd * (g[i][e] - m1 - z[i][e] * m2) : g[i][e];
                    ga[e] = pre == PRE_RELU_SQ ? gz * 2.f * r[i][e] : gz;
                }
                store_vec_nt<IO, V>(ga_ + (size_t)row * N + (size_t)vi * V, ga);
            }
        }
    }
    if constexpr (SUMS) {
        // the four waves' channel sums are added in wave order and written as this workgroup's partial rows
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int vi = lane + WAVE * i;
            if (vi >= nvec) continue;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const int c = vi * V + e;
                s_red[((size_t)wave * 3 + 0) * N + c] = acc_w[i][e];
                s_red[((size_t)wave * 3 + 1) * N + c] = acc_b[i][e];
                s_red[((size_t)wave * 3 + 2) * N + c] = acc_g[i][e];
            }
        }
        __syncthreads();
        const int nw = blockDim.x >> 6;
        float* prow = part + (size_t)blockIdx.x * 3 * N;
        for (int idx = threadIdx.x; idx < 3 * N; idx += blockDim.x) {
            float sum = 0.f;
            for (int wv = 0; wv < nw; ++wv) sum += s_red[(size_t)wv * 3 * N + idx];
            prow[idx] = sum;
        }
    }
}

constexpr int BWD_ROWS_PER_WAVE = 8;      // with channel sums: one partial row per 32 rows
constexpr int BWD_ROWS_PER_WAVE_PLAIN = 2;   // element-wise only: more workgroups in flight

template <typename IO, int VPL, bool SUMS>
int launch_bwd_vpl(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, const void* g,
                   void* ga, void* go, float* gparam, float* part, long long rows, int N, int pre, int post, float eps,
                   hipStream_t st) {
    const int rpw = SUMS ? BWD_ROWS_PER_WAVE : BWD_ROWS_PER_WAVE_PLAIN;
    const int rows_per_block = 4 * rpw;
    const long long nblk = (rows + rows_per_block - 1) / rows_per_block;
    const size_t lds = SUMS ? (size_t)4 * 3 * N * sizeof(float) : 0;
    hipLaunchKernelGGL((rowfuse_bwd_kernel<IO, VPL, SUMS>), dim3((unsigned)nblk), dim3(256), lds, st,
                       static_cast<const IO*>(a), static_cast<const IO*>(other), static_cast<const IO*>(lnw),
                       static_cast<const IO*>(lnb), static_cast<const IO*>(gamma), static_cast<const IO*>(g),
                       static_cast<IO*>(ga), static_cast<IO*>(go), part, rows, N, eps, pre, post, rpw);
    if (SUMS) {
        const int wide = 3 * N;                               // gparam: (3, N) = g_weight, g_bias, g_gamma
        hipLaunchKernelGGL(batch_sum_kernel, dim3((wide + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, part, gparam,
                           (const float*)nullptr, (float*)nullptr, (int)nblk, wide);
    }
    return check_launch("rowfuse_bwd");
}

template <typename IO>
int launch_bwd_io(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, const void* g,
                  void* ga, void* go, float* gparam, float* part, long long rows, int N, int pre, int post, float eps,
                  hipStream_t st) {
    constexpr int V = 16 / (int)sizeof(IO);
    const int per_lane = (N / V + WAVE - 1) / WAVE;
    const bool sums = lnw != nullptr || (post == POST_RESIDUAL && gamma != nullptr);
#define VRWKV_BWD(VPL, SUMS) return launch_bwd_vpl<IO, VPL, SUMS>(a, other, lnw, lnb, gamma, g, ga, go, gparam, part, rows, N, pre, post, eps, st)
    if (sums) {                                               // at most 16 channels per lane (checked by the caller)
        if (per_lane <= 1) VRWKV_BWD(1, true);
        if (per_lane <= 2 || V == 8) VRWKV_BWD(2, true);
        VRWKV_BWD(4, true);
    }
    if (per_lane <= 1) VRWKV_BWD(1, false);
    if (per_lane <= 2) VRWKV_BWD(2, false);
    if (per_lane <= 4) VRWKV_BWD(4, false);
    if (per_lane <= 8) VRWKV_BWD(8, false);
    VRWKV_BWD(16, false);
#undef VRWKV_BWD
}

template <typename IO, int VPL, int W, int PRE, int POST>
int launch_ln(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, void* out,
              long long rows, int N, float eps, hipStream_t st) {
    constexpr int per_wg = (W == 1 ? 4 : 1) * rows_per_group_fwd<VPL>();
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
    const long long nblk = (rows + 4 * BWD_ROWS_PER_WAVE - 1) / (4 * BWD_ROWS_PER_WAVE);
    return (size_t)nblk * 3 * N * sizeof(float);
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
