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
        if constexpr (sizeof(YT) == 4) {
            load_vec<YT, 4>(y_ + e0, *reinterpret_cast<float(*)[4]>(&y[0]));
            load_vec<YT, 4>(y_ + e0 + 4, *reinterpret_cast<float(*)[4]>(&y[4]));
        } else {
            load_vec<YT, 8>(y_ + e0, y);
        }
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
        load_vec<IO, 8>(g_ + e0, g);
        load_vec<IO, 8>(w_ + c, w);
        load_vec<IO, 8>(b_ + c, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float gate = g[e] * fast_rcp(1.f + fast_exp2(-g[e] * LOG2E));      // silu
            r[e] = fmaf((y[e] - mean) * rstd, w[e], b[e]) * gate;
        }
        store_vec<IO, 8>(out_ + e0, r);
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
    if ((io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) || (y_dtype != VRWKV_F32 && y_dtype != io_dtype)) {
        set_error("groupnorm_gate: gate / out must be bf16 or fp16 and y fp32 or that same type (got %d, %d)", io_dtype, y_dtype);
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
    if (io_dtype == VRWKV_BF16) {
        if (y_dtype == VRWKV_F32) return launch_gn<float, __hip_bfloat16>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
        return launch_gn<__hip_bfloat16, __hip_bfloat16>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
    }
    if (y_dtype == VRWKV_F32) return launch_gn<float, __half>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
    return launch_gn<__half, __half>(y, gate, gn_weight, gn_bias, out, rows, C, group, eps, st);
}
