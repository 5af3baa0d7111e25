// Bi-WKV backward for gfx950: gw, gu (C,), gk, gv (B,T,C) from gy.
// Replaces bi_wkv_backward (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:35-47,
// kernel .../cuda_new/bi_wkv_kernel.cu:119-367).
//
// With W[t,i] = e^{k_i - w(|t-i|-1)} (i != t), W[t,t] = e^{u+k_t}, y_t = N_t/D_t and z_t = gy_t/D_t:
//   gv_i = sum_t z_t W[t,i]                     gk_i = sum_t z_t W[t,i] (v_i - y_t)
//   gu   = sum_t z_t W[t,t] (v_t - y_t)         gw   = - sum_t sum_{i!=t} (|t-i|-1) z_t W[t,i] (v_i - y_t)
// so besides the forward states only decayed scans of z_t and z_t*y_t over past and future are
// needed (and, for gw, the same scans weighted by the distance: B' = g (B + A)).
//
// One lane owns one (batch, channel) sequence and walks it three times, lanes of a wave being 64
// adjacent channels (every access is a contiguous 64-channel row segment):
//   pass A (ascending)   past state (a, b, p) before each token            -> workspace
//   pass B (descending)  future state, y_t, z_t; future scans; partial gk, gv; gu, gw partials
//   pass C (ascending)   past scans; final gk, gv; gw partial
// Every running sum is a (mantissa, exponent) pair renormalised at each token, i.e. the
// reference's own stabilised recurrence (bi_wkv_kernel.cu:103-108), so any w, u, k is handled.
// gw and gu are reduced over the batch by a second small kernel (deterministic, no atomics).
// The reference needs 3 scratch tensors and atomicAdd (bi_wkv_kernel.cu:303-304, 415-417);
// here the workspace is 5 floats per element + 2*B*C.
#include "biwkv_bwd_serial.h"
#include "biwkv_bwd_tile.h"

namespace vrwkv {
namespace {

using namespace biwkv_bwd_detail;

template <typename IO>
__global__ __launch_bounds__(64)
void biwkv_bwd_serial_kernel(const float* __restrict__ w_, const float* __restrict__ u_,
                             const IO* __restrict__ k_, const IO* __restrict__ v_, const IO* __restrict__ gy_,
                             IO* __restrict__ gk_, IO* __restrict__ gv_, float* __restrict__ ws,
                             float* __restrict__ gw_part, float* __restrict__ gu_part, int B, int T, int C)
{
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= C) return;
    biwkv_bwd_serial_seq<IO>(w_, u_, k_, v_, gy_, gk_, gv_, ws, gw_part, gu_part, B, T, C, blockIdx.y, c);
}

int validate(int B, int T, int C, int io_dtype) {
    if (B <= 0 || T <= 0 || C <= 0) {
        set_error("biwkv_bwd: B, T, C must be positive (got %d, %d, %d)", B, T, C);
        return VRWKV_INVALID_ARG;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("biwkv_bwd: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (B > 65535 || (long long)B * T * C >= (1LL << 40)) {
        set_error("biwkv_bwd: B must be <= 65535 and B*T*C < 2^40");
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    return VRWKV_OK;
}

// How a call is laid out: L tokens per wave, S waves per workgroup, nSC super-chunks per sequence
// (L = 0: the sequential kernel), and where the pieces of the workspace are (in floats).
struct BwdPlan {
    int L = 0, S = 0, nSC = 1;
    size_t planes = 0, agg1 = 0, agg2 = 0, parts = 0, total = 0;
};

BwdPlan make_bwd_plan(int B, int T, int C) {
    BwdPlan p;
    static const int kL[] = {4, 8, 16, 25, 28};
    const int el = option(OPT_BIWKV_L);                      // tuning override: tokens per wave
    const bool tiled = !option(OPT_BIWKV_BWD_SERIAL) && (long long)T * C < (1LL << 29);   // the option forces the sequential kernel (testing)
    if (tiled) {
        for (int i = 4; i >= 0; --i)
            if ((T + kL[i] - 1) / kL[i] <= BWD_SMAX && (!el || el == kL[i])) p.L = kL[i];   // smallest L that fits: most waves per tile
        if (p.L) {
            p.S = (T + p.L - 1) / p.L;
        } else {
            p.L = 28; p.S = BWD_SMAX;
            p.nSC = (T + p.S * p.L - 1) / (p.S * p.L);
        }
    }
    p.planes = (size_t)5 * B * T * C;                        // sequential form: 5 floats per element
    p.agg1 = (size_t)B * p.nSC * 5 * C;
    p.agg2 = (size_t)B * p.nSC * 8 * C;
    p.parts = (size_t)2 * B * p.nSC * C;
    p.total = p.planes + p.agg1 + p.agg2 + p.parts;
    return p;
}

template <typename IO, int L>
void launch_tiled(const BwdPlan& p, const float* w, const float* u, const IO* k, const IO* v, const IO* gy, IO* gk, IO* gv,
                  float* ws, float* agg1, float* agg2, float* gw_part, float* gu_part, int B, int T, int C, hipStream_t st) {
    BwdGeom geo;
    geo.n_ctile = (C + WAVE - 1) / WAVE;
    geo.nSC = p.nSC;
    geo.n_tiles = B * p.nSC * geo.n_ctile;
    const int per_cu = BWD_SMAX / p.S > 0 ? BWD_SMAX / p.S : 1;
    int grid = biwkv_fwd_detail::num_cus() * per_cu;
    if (grid > geo.n_tiles) grid = geo.n_tiles;
    const dim3 g(grid), blk(p.S * WAVE);
    if (p.nSC == 1) {
        if constexpr (sizeof(IO) == 4) {
            const bool aligned = C % 4 == 0 && (((uintptr_t)k | (uintptr_t)v) & 15) == 0;
            if (aligned && !option(OPT_BIWKV_NO_STAGE)) {
                hipLaunchKernelGGL((biwkv_bwd_tile_kernel<IO, L, 0, true>), g, blk, 0, st, w, u, k, v, gy, gk, gv, ws, agg1, agg2,
                                   gw_part, gu_part, B, T, C, geo);
                return;
            }
        }
        hipLaunchKernelGGL((biwkv_bwd_tile_kernel<IO, L, 0>), g, blk, 0, st, w, u, k, v, gy, gk, gv, ws, agg1, agg2,
                           gw_part, gu_part, B, T, C, geo);
    } else if constexpr (L == 28) {
        hipLaunchKernelGGL((biwkv_bwd_tile_kernel<IO, L, 1>), g, blk, 0, st, w, u, k, v, gy, gk, gv, ws, agg1, agg2,
                           gw_part, gu_part, B, T, C, geo);
        hipLaunchKernelGGL((biwkv_bwd_tile_kernel<IO, L, 2>), g, blk, 0, st, w, u, k, v, gy, gk, gv, ws, agg1, agg2,
                           gw_part, gu_part, B, T, C, geo);
        hipLaunchKernelGGL((biwkv_bwd_tile_kernel<IO, L, 3>), g, blk, 0, st, w, u, k, v, gy, gk, gv, ws, agg1, agg2,
                           gw_part, gu_part, B, T, C, geo);
    }
}

template <typename IO>
int launch(const float* w, const float* u, const void* k, const void* v, const void* gy, float* gw, float* gu,
           void* gk, void* gv, float* ws, int B, int T, int C, hipStream_t st) {
    const BwdPlan p = make_bwd_plan(B, T, C);
    float* agg1 = ws + p.planes;
    float* agg2 = agg1 + p.agg1;
    float* gw_part = agg2 + p.agg2;
    float* gu_part = gw_part + p.parts / 2;
    const IO* kk = static_cast<const IO*>(k);
    const IO* vv = static_cast<const IO*>(v);
    const IO* gg = static_cast<const IO*>(gy);
    IO* ok = static_cast<IO*>(gk);
    IO* ov = static_cast<IO*>(gv);
    switch (p.L) {
        case 4:  launch_tiled<IO, 4>(p, w, u, kk, vv, gg, ok, ov, ws, agg1, agg2, gw_part, gu_part, B, T, C, st); break;
        case 8:  launch_tiled<IO, 8>(p, w, u, kk, vv, gg, ok, ov, ws, agg1, agg2, gw_part, gu_part, B, T, C, st); break;
        case 16: launch_tiled<IO, 16>(p, w, u, kk, vv, gg, ok, ov, ws, agg1, agg2, gw_part, gu_part, B, T, C, st); break;
        case 25: launch_tiled<IO, 25>(p, w, u, kk, vv, gg, ok, ov, ws, agg1, agg2, gw_part, gu_part, B, T, C, st); break;
        case 28: launch_tiled<IO, 28>(p, w, u, kk, vv, gg, ok, ov, ws, agg1, agg2, gw_part, gu_part, B, T, C, st); break;
        default:
            hipLaunchKernelGGL((biwkv_bwd_serial_kernel<IO>), dim3((C + 63) / 64, B), dim3(64), 0, st, w, u,
                               kk, vv, gg, ok, ov, ws, gw_part, gu_part, B, T, C);
    }
    hipLaunchKernelGGL(batch_sum_kernel, dim3((C + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, gw_part, gw, gu_part, gu, B * p.nSC, C);
    return check_launch("biwkv_bwd");
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" size_t vrwkv_biwkv_bwd_workspace_bytes(int B, int T, int C, int io_dtype) {
    if (validate(B, T, C, io_dtype) != VRWKV_OK) return 0;
    return make_bwd_plan(B, T, C).total * sizeof(float);
}

extern "C" int vrwkv_biwkv_bwd(const float* w, const float* u, const void* k, const void* v, const void* gy,
                               float* gw, float* gu, void* gk, void* gv, int B, int T, int C, int io_dtype,
                               void* workspace, size_t workspace_bytes, void* hip_stream) {
    int rc = validate(B, T, C, io_dtype);
    if (rc != VRWKV_OK) return rc;
    if (!w || !u || !k || !v || !gy || !gw || !gu || !gk || !gv) {
        set_error("biwkv_bwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    const size_t need = make_bwd_plan(B, T, C).total * sizeof(float);
    if (!workspace || workspace_bytes < need) {
        set_error("biwkv_bwd: workspace of %zu bytes required (got %zu)", need, workspace ? workspace_bytes : (size_t)0);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    const size_t esz = io_dtype == VRWKV_F32 ? 4 : 2;
    if ((((uintptr_t)k | (uintptr_t)v | (uintptr_t)gy | (uintptr_t)gk | (uintptr_t)gv) & (esz - 1)) ||
        (((uintptr_t)w | (uintptr_t)u | (uintptr_t)gw | (uintptr_t)gu | (uintptr_t)workspace) & 3)) {
        set_error("biwkv_bwd: pointers must be aligned to their element size");
        return VRWKV_INVALID_ARG;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* ws = static_cast<float*>(workspace);
    switch (io_dtype) {
        case VRWKV_F32:  return launch<float>(w, u, k, v, gy, gw, gu, gk, gv, ws, B, T, C, st);
        case VRWKV_BF16: return launch<__hip_bfloat16>(w, u, k, v, gy, gw, gu, gk, gv, ws, B, T, C, st);
        case VRWKV_F16:  return launch<__half>(w, u, k, v, gy, gw, gu, gk, gv, ws, B, T, C, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
