// Fused row-wise epilogues of the VRWKV blocks: for every row (token) of N channels
//   y   = LayerNorm(pre(a)) * ln_weight + ln_bias        (LayerNorm optional; pre = identity or relu(.)^2)
//   out = y | sigmoid(other) * y | other + gamma * y      (gamma optional)
// in one pass over memory.  These are the element-wise steps around the WKV operator and the GEMMs that the reference
// runs as separate PyTorch kernels (classification/mmcls_custom/models/backbones/vrwkv.py):
//   :184-186  rwkv = key_norm(rwkv); rwkv = sr * rwkv             -> a = rwkv, other = receptance(xr), LayerNorm, sigmoid gate
//   :256-260  k = square(relu(key(xk))); k = key_norm(k)           -> a = key(xk), pre = relu^2, LayerNorm
//   :261      sigmoid(receptance(xr)) * kv                         -> a = kv, other = receptance(xr), sigmoid gate
//   :300-313  x = x + gamma * ln(att(x)) / x + gamma * att(ln(x))  -> a = branch output, other = x, (LayerNorm,) gamma
// One wave per row: a lane keeps its 16-byte vectors of the row in registers (read once), the mean and the variance are
// reduced across the wave in fp32 (two passes over the registers), the result is written once.
#include "vrwkv_common.h"

namespace vrwkv {
namespace {

enum { PRE_NONE = 0, PRE_RELU_SQ = 1 };
enum { POST_NONE = 0, POST_SIGMOID_GATE = 1, POST_RESIDUAL = 2 };

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, WAVE);
    return x;
}

template <typename IO, int VPL, int PRE, int POST, bool HAS_LN>
__global__ __launch_bounds__(256)
void rowfuse_kernel(const IO* __restrict__ a_, const IO* __restrict__ other_, const IO* __restrict__ lnw_,
                    const IO* __restrict__ lnb_, const IO* __restrict__ gamma_, IO* __restrict__ out_,
                    long long rows, int N, float eps)
{
    constexpr int V = 16 / (int)sizeof(IO);
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + wave;
    if (row >= rows) return;                                  // whole waves leave; there is no barrier below
    const IO* a = a_ + row * N;
    const int nvec = N / V;
    float x[VPL][V];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int vi = lane + WAVE * i;
        if (vi < nvec) {
            load_vec<IO, V>(a + (size_t)vi * V, x[i]);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if (PRE == PRE_RELU_SQ) { const float r = fmaxf(x[i][e], 0.f); x[i][e] = r * r; }
                s += x[i][e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) x[i][e] = 0.f;
        }
    }
    float mean = 0.f, rstd = 1.f;
    if (HAS_LN) {
        mean = wave_sum(s) / (float)N;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
            if (lane + WAVE * i < nvec) {
#pragma unroll
                for (int e = 0; e < V; ++e) { const float d = x[i][e] - mean; q = fmaf(d, d, q); }
            }
        rstd = rsqrtf(wave_sum(q) / (float)N + eps);
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int vi = lane + WAVE * i;
        if (vi >= nvec) continue;
        const size_t c = (size_t)vi * V;
        float y[V];
        if (HAS_LN) {
            float w[V], b[V];
            load_vec<IO, V>(lnw_ + c, w);
            load_vec<IO, V>(lnb_ + c, b);
#pragma unroll
            for (int e = 0; e < V; ++e) y[e] = fmaf((x[i][e] - mean) * rstd, w[e], b[e]);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) y[e] = x[i][e];
        }
        if (POST != POST_NONE) {
            float o[V];
            load_vec<IO, V>(other_ + row * N + c, o);
            if (POST == POST_SIGMOID_GATE) {
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] *= fast_rcp(1.f + fast_exp2(-o[e] * LOG2E));
            } else {
                float g[V];
                if (gamma_) load_vec<IO, V>(gamma_ + c, g);
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = gamma_ ? fmaf(g[e], y[e], o[e]) : o[e] + y[e];
            }
        }
        store_vec<IO, V>(out_ + row * N + c, y);
    }
}

template <typename IO, int VPL, int PRE, int POST>
int launch_ln(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, void* out,
              long long rows, int N, float eps, hipStream_t st) {
    const dim3 block(256), grid((unsigned)((rows + 3) / 4));
    const IO *pa = static_cast<const IO*>(a), *po = static_cast<const IO*>(other), *pw = static_cast<const IO*>(lnw),
             *pb = static_cast<const IO*>(lnb), *pg = static_cast<const IO*>(gamma);
    IO* pout = static_cast<IO*>(out);
    if (lnw) hipLaunchKernelGGL((rowfuse_kernel<IO, VPL, PRE, POST, true>), grid, block, 0, st, pa, po, pw, pb, pg, pout, rows, N, eps);
    else     hipLaunchKernelGGL((rowfuse_kernel<IO, VPL, PRE, POST, false>), grid, block, 0, st, pa, po, pw, pb, pg, pout, rows, N, eps);
    return check_launch("rowfuse");
}

template <typename IO, int VPL>
int launch_ops(const void* a, const void* other, const void* lnw, const void* lnb, const void* gamma, void* out,
               long long rows, int N, int pre, int post, float eps, hipStream_t st) {
#define VRWKV_ROW(PRE, POST) return launch_ln<IO, VPL, PRE, POST>(a, other, lnw, lnb, gamma, out, rows, N, eps, st)
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
    const int per_lane = (N / V + WAVE - 1) / WAVE;           // 16-byte vectors a lane keeps
    if (per_lane <= 1) return launch_ops<IO, 1>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    if (per_lane <= 2) return launch_ops<IO, 2>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    if (per_lane <= 4) return launch_ops<IO, 4>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    if (per_lane <= 8) return launch_ops<IO, 8>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
    return launch_ops<IO, 16>(a, other, lnw, lnb, gamma, out, rows, N, pre, post, eps, st);
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
