// Element-wise steps of the VRWKV6 spatial mix around the wkv6 operator
// (classification/mmcls_custom/models/backbones/vrwkv6.py:176-212), each in one pass over memory:
//
//  vrwkv_maa_mix        the five data-dependent token mixes of jit_func (:190-194)
//                           out_i = x + (sx - x) * (maa_i + m_i),  i = w, k, v, r, g
//                       from x, the shifted x, the (5, B, T, C) low-rank mix of :183-186 and the five (C,) vectors;
//                       the reference runs three PyTorch kernels per output plus the subtraction.
//  vrwkv_groupnorm_gate jit_func_2 (:205-211): out = GroupNorm(y) * silu(gate), groups of `group` consecutive
//                       channels per token (ln_x = GroupNorm(n_head, C) on a (B*T, C) view), y as the operator
//                       returns it (fp32) or in the I/O type.
//
// Backward of both (the reference differentiates the PyTorch ops by autograd), one pass each plus a fixed-order sum of
// per-workgroup partial rows for the per-channel gradients:
//  vrwkv_maa_mix_bwd         d = sx - x, f_i = maa_i + m_i:  gx = sum_i g_i (1 - f_i),  gsx = sum_i g_i f_i,
//                            gm_i = g_i d,  gmaa_i[c] = sum_rows g_i d
//  vrwkv_groupnorm_gate_bwd  s = silu(gate), yn = xh w + b:  g_gate = g yn s',  gyn = g s,  g_w[c] = sum_rows gyn xh,
//                            g_b[c] = sum_rows gyn,  gy = rstd (w gyn - mean_grp(w gyn) - xh mean_grp(w gyn xh))
#include "vrwkv_common.h"

namespace vrwkv {
namespace {

template <typename IO>
__global__ __launch_bounds__(256)
void maa_mix_kernel(const IO* __restrict__ x_, const IO* __restrict__ sx_, const IO* __restrict__ m_,
                    const float* __restrict__ maa_, IO* __restrict__ o0, IO* __restrict__ o1, IO* __restrict__ o2,
                    IO* __restrict__ o3, IO* __restrict__ o4, long long nvec, int C)
{
    constexpr int V = 16 / (int)sizeof(IO);
    const long long vi = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vi >= nvec) return;
    const size_t e0 = (size_t)vi * V;
    const int c = (int)(e0 % (size_t)C);                      // C % V == 0: a vector stays inside one token
    const size_t n = (size_t)nvec * V;                        // elements per (B, T, C) tensor
    float x[V], d[V];
    load_vec<IO, V>(x_ + e0, x);
    load_vec<IO, V>(sx_ + e0, d);
#pragma unroll
    for (int e = 0; e < V; ++e) d[e] -= x[e];
    IO* outs[5] = {o0, o1, o2, o3, o4};
#pragma unroll
    for (int i = 0; i < 5; ++i) {
        float m[V], a[V], r[V];
        load_vec<IO, V>(m_ + (size_t)i * n + e0, m);
#pragma unroll
        for (int e4 = 0; e4 < V; e4 += 4)
            load_vec<float, 4>(maa_ + (size_t)i * C + c + e4, *reinterpret_cast<float(*)[4]>(&a[e4]));
#pragma unroll
        for (int e = 0; e < V; ++e) r[e] = fmaf(d[e], a[e] + m[e], x[e]);
        store_vec<IO, V>(outs[i] + e0, r);
    }
}

// Eight consecutive elements widened to fp32: one 16-byte vector of a 16-bit type, two of fp32.
template <typename T>
__device__ __forceinline__ void load8(const T* __restrict__ p, float (&out)[8]) {
    if constexpr (sizeof(T) == 4) {
        load_vec<T, 4>(p, *reinterpret_cast<float(*)[4]>(&out[0]));
        load_vec<T, 4>(p + 4, *reinterpret_cast<float(*)[4]>(&out[4]));
    } else {
        load_vec<T, 8>(p, out);
    }
}
template <typename T>
__device__ __forceinline__ void store8(T* __restrict__ p, const float (&in)[8]) {
    if constexpr (sizeof(T) == 4) {
        store_vec<T, 4>(p, *reinterpret_cast<const float(*)[4]>(&in[0]));
        store_vec<T, 4>(p + 4, *reinterpret_cast<const float(*)[4]>(&in[4]));
    } else {
        store_vec<T, 8>(p, in);
    }
}

// One wave per token; a lane owns 8 consecutive channels per step, so a group of 64 channels is 8 neighbouring lanes.
template <typename YT, typename IO, int GL>                   // GL = lanes per group = group / 8
__global__ __launch_bounds__(256)
void groupnorm_gate_kernel(const YT* __restrict__ y_, const IO* __restrict__ g_, const IO* __restrict__ w_,
                           const IO* __restrict__ b_, IO* __restrict__ out_, long long rows, int C, float eps)
{
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + wave;
    if (row >= rows) return;                                  // whole waves leave; there is no barrier below
    const int nchunk = C / 8;                                 // 8-channel pieces in a row; C % (8 GL) == 0
    for (int p0 = 0; p0 < nchunk; p0 += WAVE) {
        const int p = p0 + lane;
        const bool ok = p < nchunk;                           // whole groups: the lanes of a group agree
        const size_t e0 = (size_t)row * C + (size_t)(ok ? p : 0) * 8;
        float y[8];
        load8<YT>(y_ + e0, y);
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s += y[e];
#pragma unroll
        for (int off = 1; off < GL; off <<= 1) s += __shfl_xor(s, off, WAVE);
        const float mean = s / (float)(8 * GL);
        float q = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float dlt = y[e] - mean; q = fmaf(dlt, dlt, q); }
#pragma unroll
        for (int off = 1; off < GL; off <<= 1) q += __shfl_xor(q, off, WAVE);
        const float rstd = rsqrtf(q / (float)(8 * GL) + eps);
        if (!ok) continue;
        const int c = p * 8;
        float g[8], w[8], b[8], r[8];
        load8<IO>(g_ + e0, g);
        load8<IO>(w_ + c, w);
        load8<IO>(b_ + c, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float gate = g[e] * fast_rcp(1.f + fast_exp2(-g[e] * LOG2E));      // silu
            r[e] = fmaf((y[e] - mean) * rstd, w[e], b[e]) * gate;
        }
        store8<IO>(out_ + e0, r);
    }
}

template <typename YT, typename IO>
int launch_gn(const void* y, const void* g, const void* w, const void* b, void* out, long long rows, int C, int group,
              float eps, hipStream_t st) {
    const dim3 block(256), grid((unsigned)((rows + 3) / 4));
    const YT* py = static_cast<const YT*>(y);
    const IO *pg = static_cast<const IO*>(g), *pw = static_cast<const IO*>(w), *pb = static_cast<const IO*>(b);
    IO* po = static_cast<IO*>(out);
    switch (group / 8) {
        case 1:  hipLaunchKernelGGL((groupnorm_gate_kernel<YT, IO, 1>), grid, block, 0, st, py, pg, pw, pb, po, rows, C, eps); break;
        case 2:  hipLaunchKernelGGL((groupnorm_gate_kernel<YT, IO, 2>), grid, block, 0, st, py, pg, pw, pb, po, rows, C, eps); break;
        case 4:  hipLaunchKernelGGL((groupnorm_gate_kernel<YT, IO, 4>), grid, block, 0, st, py, pg, pw, pb, po, rows, C, eps); break;
        case 8:  hipLaunchKernelGGL((groupnorm_gate_kernel<YT, IO, 8>), grid, block, 0, st, py, pg, pw, pb, po, rows, C, eps); break;
        case 16: hipLaunchKernelGGL((groupnorm_gate_kernel<YT, IO, 16>), grid, block, 0, st, py, pg, pw, pb, po, rows, C, eps); break;
        default:
            set_error("groupnorm_gate: group size %d is not 8, 16, 32, 64 or 128", group);
            return VRWKV_UNSUPPORTED_SHAPE;
    }
    return check_launch("groupnorm_gate");
}

constexpr int MB_CX = 32, MB_TY = 8, MB_ROWS = 32;   // maa_mix backward workgroup: 32 channel vectors x 8 row lanes, 32 rows

template <typename IO>
__global__ __launch_bounds__(MB_CX * MB_TY)
void maa_mix_bwd_kernel(const IO* __restrict__ x_, const IO* __restrict__ sx_, const IO* __restrict__ m_,
                        const float* __restrict__ maa_, const IO* __restrict__ g0, const IO* __restrict__ g1,
                        const IO* __restrict__ g2, const IO* __restrict__ g3, const IO* __restrict__ g4,
                        IO* __restrict__ gx_, IO* __restrict__ gsx_, IO* __restrict__ gm_, float* __restrict__ part,
                        long long rows, int C)
{
    constexpr int V = 16 / (int)sizeof(IO);
    __shared__ float s_acc[MB_TY][5][MB_CX * V];
    const int cx = threadIdx.x % MB_CX, ty = threadIdx.x / MB_CX;
    const int c = (blockIdx.x * MB_CX + cx) * V;
    const bool cok = c < C;
    const size_t n = (size_t)rows * C;
    const IO* gs[5] = {g0, g1, g2, g3, g4};
    float maa[5][V], acc[5][V];
#pragma unroll
    for (int i = 0; i < 5; ++i)
#pragma unroll
        for (int e = 0; e < V; ++e) { maa[i][e] = cok ? maa_[(size_t)i * C + c + e] : 0.f; acc[i][e] = 0.f; }
    if (cok) {
#pragma unroll
        for (int k = 0; k < MB_ROWS / MB_TY; ++k) {
            const long long row = (long long)blockIdx.y * MB_ROWS + ty + MB_TY * k;
            if (row >= rows) continue;
            const size_t e0 = (size_t)row * C + c;
            float x[V], d[V], gx[V], gsx[V];
            load_vec<IO, V>(x_ + e0, x);
            load_vec<IO, V>(sx_ + e0, d);
#pragma unroll
            for (int e = 0; e < V; ++e) { d[e] -= x[e]; gx[e] = 0.f; gsx[e] = 0.f; }
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                float m[V], g[V], gm[V];
                load_vec<IO, V>(m_ + (size_t)i * n + e0, m);
                load_vec<IO, V>(gs[i] + e0, g);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float f = maa[i][e] + m[e];
                    gsx[e] = fmaf(g[e], f, gsx[e]);
                    gx[e] = fmaf(g[e], 1.f - f, gx[e]);
                    gm[e] = g[e] * d[e];
                    acc[i][e] += gm[e];
                }
                store_vec<IO, V>(gm_ + (size_t)i * n + e0, gm);
            }
            store_vec<IO, V>(gx_ + e0, gx);
            store_vec<IO, V>(gsx_ + e0, gsx);
        }
    }
#pragma unroll
    for (int i = 0; i < 5; ++i)
#pragma unroll
        for (int e = 0; e < V; ++e) s_acc[ty][i][cx * V + e] = acc[i][e];
    __syncthreads();
    float* prow = part + (size_t)blockIdx.y * 5 * C;
    for (int o = threadIdx.x; o < 5 * MB_CX * V; o += MB_CX * MB_TY) {
        const int i = o / (MB_CX * V), col = o % (MB_CX * V);
        const int cg = blockIdx.x * MB_CX * V + col;
        if (cg >= C) continue;
        float sum = 0.f;
#pragma unroll
        for (int y = 0; y < MB_TY; ++y) sum += s_acc[y][i][col];
        prow[(size_t)i * C + cg] = sum;
    }
}

constexpr int GN_RPW = 8;        // rows a wave walks in the GroupNorm backward (one partial row per 32 rows)
constexpr int GN_STEPS = 2;      // 512-channel steps a row may take there: C <= 1024

template <typename YT, typename IO, int GL>
__global__ __launch_bounds__(256)
void groupnorm_gate_bwd_kernel(const YT* __restrict__ y_, const IO* __restrict__ gate_, const IO* __restrict__ w_,
                               const IO* __restrict__ b_, const IO* __restrict__ g_, YT* __restrict__ gy_,
                               IO* __restrict__ ggate_, float* __restrict__ part, long long rows, int C, float eps)
{
    extern __shared__ float s_red[];                          // [4 waves][2 sums][C]
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const int nchunk = C / 8;
    float w[GN_STEPS][8], b[GN_STEPS][8], acc_w[GN_STEPS][8], acc_b[GN_STEPS][8];
#pragma unroll
    for (int st = 0; st < GN_STEPS; ++st) {
        const int p = st * WAVE + lane;
#pragma unroll
        for (int e = 0; e < 8; ++e) { w[st][e] = 0.f; b[st][e] = 0.f; acc_w[st][e] = 0.f; acc_b[st][e] = 0.f; }
        if (p < nchunk) { load8<IO>(w_ + p * 8, w[st]); load8<IO>(b_ + p * 8, b[st]); }
    }
    const long long row0 = ((long long)blockIdx.x * (blockDim.x >> 6) + wave) * GN_RPW;
    for (int rr = 0; rr < GN_RPW; ++rr) {
        const long long row = row0 + rr;
        if (row >= rows) break;                               // wave-uniform
#pragma unroll
        for (int st = 0; st < GN_STEPS; ++st) {
            const int p = st * WAVE + lane;
            if (st * WAVE >= nchunk) break;                   // wave-uniform
            const bool ok = p < nchunk;                       // whole groups: the lanes of a group agree
            const size_t e0 = (size_t)row * C + (size_t)(ok ? p : 0) * 8;
            float y[8], gt[8], g[8];
            load8<YT>(y_ + e0, y);
            load8<IO>(gate_ + e0, gt);
            load8<IO>(g_ + e0, g);
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) s += y[e];
#pragma unroll
            for (int off = 1; off < GL; off <<= 1) s += __shfl_xor(s, off, WAVE);
            const float mean = s / (float)(8 * GL);
            float q = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) { const float dlt = y[e] - mean; q = fmaf(dlt, dlt, q); }
#pragma unroll
            for (int off = 1; off < GL; off <<= 1) q += __shfl_xor(q, off, WAVE);
            const float rstd = rsqrtf(q / (float)(8 * GL) + eps);
            float t[8], xh[8], gg[8], t1 = 0.f, t2 = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                xh[e] = (y[e] - mean) * rstd;
                const float yn = fmaf(xh[e], w[st][e], b[st][e]);
                const float sg = fast_rcp(1.f + fast_exp2(-gt[e] * LOG2E));
                const float silu = gt[e] * sg;
                gg[e] = g[e] * yn * sg * (1.f + gt[e] * (1.f - sg));
                const float gyn = ok ? g[e] * silu : 0.f;
                acc_b[st][e] += gyn;
                acc_w[st][e] = fmaf(gyn, xh[e], acc_w[st][e]);
                t[e] = w[st][e] * gyn;
                t1 += t[e];
                t2 = fmaf(t[e], xh[e], t2);
            }
#pragma unroll
            for (int off = 1; off < GL; off <<= 1) { t1 += __shfl_xor(t1, off, WAVE); t2 += __shfl_xor(t2, off, WAVE); }
            const float m1 = t1 / (float)(8 * GL), m2 = t2 / (float)(8 * GL);
            if (!ok) continue;
            float gy[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) gy[e] = rstd * (t[e] - m1 - xh[e] * m2);
            store8<YT>(gy_ + e0, gy);
            store8<IO>(ggate_ + e0, gg);
        }
    }
    // the four waves' channel sums are added in wave order and written as this workgroup's partial rows
#pragma unroll
    for (int st = 0; st < GN_STEPS; ++st) {
        const int p = st * WAVE + lane;
        if (p >= nchunk) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            s_red[((size_t)wave * 2 + 0) * C + p * 8 + e] = acc_w[st][e];
            s_red[((size_t)wave * 2 + 1) * C + p * 8 + e] = acc_b[st][e];
        }
    }
    __syncthreads();
    const int nw = blockDim.x >> 6;
    float* prow = part + (size_t)blockIdx.x * 2 * C;
    for (int idx = threadIdx.x; idx < 2 * C; idx += blockDim.x) {
        float sum = 0.f;
        for (int wv = 0; wv < nw; ++wv) sum += s_red[(size_t)wv * 2 * C + idx];
        prow[idx] = sum;
    }
}

template <typename YT, typename IO>
int launch_gn_bwd(const void* y, const void* gate, const void* w, const void* b, const void* g, void* gy, void* ggate,
                  float* gparam, float* part, long long rows, int C, int group, float eps, hipStream_t st) {
    const long long nblk = (rows + 4 * GN_RPW - 1) / (4 * GN_RPW);
    const dim3 block(256), grid((unsigned)nblk);
    const size_t lds = (size_t)4 * 2 * C * sizeof(float);
#define VRWKV_GNB(GL) hipLaunchKernelGGL((groupnorm_gate_bwd_kernel<YT, IO, GL>), grid, block, lds, st, static_cast<const YT*>(y), \
        static_cast<const IO*>(gate), static_cast<const IO*>(w), static_cast<const IO*>(b), static_cast<const IO*>(g), \
        static_cast<YT*>(gy), static_cast<IO*>(ggate), part, rows, C, eps)
    switch (group / 8) {
        case 1:  VRWKV_GNB(1); break;
        case 2:  VRWKV_GNB(2); break;
        case 4:  VRWKV_GNB(4); break;
        case 8:  VRWKV_GNB(8); break;
        case 16: VRWKV_GNB(16); break;
        default:
            set_error("groupnorm_gate_bwd: group size %d is not 8, 16, 32, 64 or 128", group);
            return VRWKV_UNSUPPORTED_SHAPE;
    }
#undef VRWKV_GNB
    const int wide = 2 * C;                                   // gparam: (2, C) = g_weight, g_bias
    hipLaunchKernelGGL(batch_sum_kernel, dim3((wide + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, part, gparam, (const float*)nullptr,
                       (float*)nullptr, (int)nblk, wide);
    return check_launch("groupnorm_gate_bwd");
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" int vrwkv_maa_mix(const void* x, const void* sx, const void* m, const float* maa, void* const* out,
                             long long rows, int C, int io_dtype, void* hip_stream) {
    if (rows <= 0 || C <= 0 || !x || !sx || !m || !maa || !out) {
        set_error("maa_mix: bad arguments (rows=%lld C=%d)", rows, C);
        return VRWKV_INVALID_ARG;
    }
    for (int i = 0; i < 5; ++i)
        if (!out[i]) { set_error("maa_mix: output %d is null", i); return VRWKV_INVALID_ARG; }
    if (io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16 && io_dtype != VRWKV_F32) {
        set_error("maa_mix: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    const int V = io_dtype == VRWKV_F32 ? 4 : 8;
    uintptr_t all = (uintptr_t)x | (uintptr_t)sx | (uintptr_t)m;
    for (int i = 0; i < 5; ++i) all |= (uintptr_t)out[i];
    if (C % V != 0 || ((all | (uintptr_t)maa) & 15)) {
        set_error("maa_mix: C=%d must be a multiple of %d and every tensor 16-byte aligned", C, V);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const long long nvec = rows * (C / V);
    if ((nvec + 255) / 256 > 0x7fffffffLL) { set_error("maa_mix: too many elements"); return VRWKV_UNSUPPORTED_SHAPE; }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    const dim3 block(256), grid((unsigned)((nvec + 255) / 256));
#define VRWKV_MAA(IO) hipLaunchKernelGGL((maa_mix_kernel<IO>), grid, block, 0, st, static_cast<const IO*>(x), \
        static_cast<const IO*>(sx), static_cast<const IO*>(m), maa, static_cast<IO*>(out[0]), static_cast<IO*>(out[1]), \
        static_cast<IO*>(out[2]), static_cast<IO*>(out[3]), static_cast<IO*>(out[4]), nvec, C)
    switch (io_dtype) {
        case VRWKV_F32:  VRWKV_MAA(float); break;
        case VRWKV_BF16: VRWKV_MAA(__hip_bfloat16); break;
        case VRWKV_F16:  VRWKV_MAA(__half); break;
    }
#undef VRWKV_MAA
    return check_launch("maa_mix");
}

extern "C" int vrwkv_groupnorm_gate(const void* y, const void* gate, const void* gn_weight, const void* gn_bias,
                                    void* out, long long rows, int C, int group, float eps, int y_dtype, int io_dtype,
                                    void* hip_stream) {
    if (rows <= 0 || C <= 0 || group <= 0 || !y || !gate || !gn_weight || !gn_bias || !out) {
        set_error("groupnorm_gate: bad arguments (rows=%lld C=%d group=%d)", rows, C, group);
        return VRWKV_INVALID_ARG;
    }
    if ((io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16 && io_dtype != VRWKV_F32) || (y_dtype != VRWKV_F32 && y_dtype != io_dtype)) {
        set_error("groupnorm_gate: gate / out must be fp32, bf16 or fp16 and y fp32 or that same type (got %d, %d)", io_dtype, y_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (C % group != 0 || group % 8 != 0 || rows > 0x7fffffffLL * 4) {
        set_error("groupnorm_gate: C=%d must be a multiple of the group size %d, itself a multiple of 8", C, group);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (((uintptr_t)y | (uintptr_t)gate | (uintptr_t)gn_weight | (uintptr_t)gn_bias | (uintptr_t)out) & 15) {
        set_error("groupnorm_gate: every tensor must be 16-byte aligned");
        return VRWKV_INVALID_ARG;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    if (io_dtype == VRWKV_F32) return launch_gn<float, float>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
    if (io_dtype == VRWKV_BF16) {
        if (y_dtype == VRWKV_F32) return launch_gn<float, __hip_bfloat16>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
        return launch_gn<__hip_bfloat16, __hip_bfloat16>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
    }
    if (y_dtype == VRWKV_F32) return launch_gn<float, __half>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
    return launch_gn<__half, __half>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
}

extern "C" size_t vrwkv_maa_mix_bwd_workspace_bytes(long long rows, int C) {
    if (rows <= 0 || C <= 0) return 0;
    return (size_t)((rows + MB_ROWS - 1) / MB_ROWS) * 5 * C * sizeof(float);
}

extern "C" int vrwkv_maa_mix_bwd(const void* x, const void* sx, const void* m, const float* maa, const void* const* gout,
                                 void* gx, void* gsx, void* gm, float* gmaa, long long rows, int C, int io_dtype,
                                 void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (rows <= 0 || C <= 0 || !x || !sx || !m || !maa || !gout || !gx || !gsx || !gm || !gmaa) {
        set_error("maa_mix_bwd: bad arguments (rows=%lld C=%d)", rows, C);
        return VRWKV_INVALID_ARG;
    }
    if (io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16 && io_dtype != VRWKV_F32) {
        set_error("maa_mix_bwd: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    const int V = io_dtype == VRWKV_F32 ? 4 : 8;
    uintptr_t all = (uintptr_t)x | (uintptr_t)sx | (uintptr_t)m | (uintptr_t)gx | (uintptr_t)gsx | (uintptr_t)gm;
    for (int i = 0; i < 5; ++i) {
        if (!gout[i]) { set_error("maa_mix_bwd: gradient %d is null", i); return VRWKV_INVALID_ARG; }
        all |= (uintptr_t)gout[i];
    }
    const long long nrb = (rows + MB_ROWS - 1) / MB_ROWS;
    if (C % V != 0 || (all & 15) || nrb > 65535) {
        set_error("maa_mix_bwd: C=%d must be a multiple of %d, every tensor 16-byte aligned, rows <= %d", C, V, 65535 * MB_ROWS);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const size_t need = vrwkv_maa_mix_bwd_workspace_bytes(rows, C);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3)) {
        set_error("maa_mix_bwd: a 4-byte aligned workspace of %zu bytes is required", need);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* part = static_cast<float*>(workspace);
    const int ncv = C / V;
    const dim3 block(MB_CX * MB_TY), grid((ncv + MB_CX - 1) / MB_CX, (unsigned)nrb);
#define VRWKV_MAAB(IO) hipLaunchKernelGGL((maa_mix_bwd_kernel<IO>), grid, block, 0, st, static_cast<const IO*>(x), \
        static_cast<const IO*>(sx), static_cast<const IO*>(m), maa, static_cast<const IO*>(gout[0]), \
        static_cast<const IO*>(gout[1]), static_cast<const IO*>(gout[2]), static_cast<const IO*>(gout[3]), \
        static_cast<const IO*>(gout[4]), static_cast<IO*>(gx), static_cast<IO*>(gsx), static_cast<IO*>(gm), part, rows, C)
    switch (io_dtype) {
        case VRWKV_F32:  VRWKV_MAAB(float); break;
        case VRWKV_BF16: VRWKV_MAAB(__hip_bfloat16); break;
        case VRWKV_F16:  VRWKV_MAAB(__half); break;
    }
#undef VRWKV_MAAB
    const int wide = 5 * C;
    hipLaunchKernelGGL(batch_sum_kernel, dim3((wide + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, part, gmaa, (const float*)nullptr,
                       (float*)nullptr, (int)nrb, wide);
    return check_launch("maa_mix_bwd");
}

extern "C" size_t vrwkv_groupnorm_gate_bwd_workspace_bytes(long long rows, int C) {
    if (rows <= 0 || C <= 0) return 0;
    return (size_t)((rows + 4 * GN_RPW - 1) / (4 * GN_RPW)) * 2 * C * sizeof(float);
}

extern "C" int vrwkv_groupnorm_gate_bwd(const void* y, const void* gate, const void* gn_weight, const void* gn_bias,
                                        const void* gout, void* gy, void* ggate, float* gparam, long long rows, int C,
                                        int group, float eps, int y_dtype, int io_dtype,
                                        void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (rows <= 0 || C <= 0 || group <= 0 || !y || !gate || !gn_weight || !gn_bias || !gout || !gy || !ggate || !gparam) {
        set_error("groupnorm_gate_bwd: bad arguments (rows=%lld C=%d group=%d)", rows, C, group);
        return VRWKV_INVALID_ARG;
    }
    if ((io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16 && io_dtype != VRWKV_F32) || (y_dtype != VRWKV_F32 && y_dtype != io_dtype)) {
        set_error("groupnorm_gate_bwd: gate / gradients must be fp32, bf16 or fp16 and y fp32 or that same type (got %d, %d)", io_dtype, y_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (C % group != 0 || group % 8 != 0 || C > GN_STEPS * WAVE * 8 || rows > 0x7fffffffLL * 32) {
        set_error("groupnorm_gate_bwd: C=%d must be a multiple of the group size %d (a multiple of 8) and at most %d",
                  C, group, GN_STEPS * WAVE * 8);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (((uintptr_t)y | (uintptr_t)gate | (uintptr_t)gn_weight | (uintptr_t)gn_bias | (uintptr_t)gout | (uintptr_t)gy | (uintptr_t)ggate) & 15) {
        set_error("groupnorm_gate_bwd: every tensor must be 16-byte aligned");
        return VRWKV_INVALID_ARG;
    }
    const size_t need = vrwkv_groupnorm_gate_bwd_workspace_bytes(rows, C);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3)) {
        set_error("groupnorm_gate_bwd: a 4-byte aligned workspace of %zu bytes is required", need);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* part = static_cast<float*>(workspace);
    if (io_dtype == VRWKV_F32) return launch_gn_bwd<float, float>(y, gate, gn_weight, gn_bias, gout, gy, ggate, gparam, part, rows, C, group, eps, st);
    if (io_dtype == VRWKV_BF16) {
        if (y_dtype == VRWKV_F32) return launch_gn_bwd<float, __hip_bfloat16>(y, gate, gn_weight, gn_bias, gout, gy, ggate, gparam, part, rows, C, group, eps, st);
        return launch_gn_bwd<__hip_bfloat16, __hip_bfloat16>(y, gate, gn_weight, gn_bias, gout, gy, ggate, gparam, part, rows, C, group, eps, st);
    }
    if (y_dtype == VRWKV_F32) return launch_gn_bwd<float, __half>(y, gate, gn_weight, gn_bias, gout, gy, ggate, gparam, part, rows, C, group, eps, st);
    return launch_gn_bwd<__half, __half>(y, gate, gn_weight, gn_bias, gout, gy, ggate, gparam, part, rows, C, group, eps, st);
}
