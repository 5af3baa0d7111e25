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

template <typename IO>
int launch(const float* w, const float* u, const void* k, const void* v, const void* gy, float* gw, float* gu,
           void* gk, void* gv, float* ws, int B, int T, int C, hipStream_t st) {
    const size_t plane = (size_t)B * T * C;
    float* gw_part = ws + 5 * plane;
    float* gu_part = gw_part + (size_t)B * C;
    const IO* kk = static_cast<const IO*>(k);
    const IO* vv = static_cast<const IO*>(v);
    const IO* gg = static_cast<const IO*>(gy);
    IO* ok = static_cast<IO*>(gk);
    IO* ov = static_cast<IO*>(gv);
    // sequences that fit one workgroup (8 waves x L tokens) take the tiled kernel
    static const int kL[] = {4, 8, 16, 28};
    int L = 0;
    const char* path = getenv("VRWKV_BIWKV_BWD_PATH");       // "serial" forces the sequential kernel (testing)
    if (!(path && path[0] == 's'))
        for (int i = 3; i >= 0; --i)
            if ((T + kL[i] - 1) / kL[i] <= BWD_SMAX) L = kL[i];   // smallest L that fits: most waves per tile
    if (L) {
        const int S = (T + L - 1) / L;
        const int n_ctile = (C + WAVE - 1) / WAVE;
        const int n_tiles = B * n_ctile;
        const int per_cu = BWD_SMAX / S > 0 ? BWD_SMAX / S : 1;
        int grid = biwkv_fwd_detail::num_cus() * per_cu;
        if (grid > n_tiles) grid = n_tiles;
#define VRWKV_BWD_CASE(LL) case LL: hipLaunchKernelGGL((biwkv_bwd_tile_kernel<IO, LL>), dim3(grid), dim3(S * WAVE), 0, st, \
                           w, u, kk, vv, gg, ok, ov, ws, gw_part, gu_part, B, T, C, n_ctile, n_tiles); break;
        switch (L) { VRWKV_BWD_CASE(4) VRWKV_BWD_CASE(8) VRWKV_BWD_CASE(16) VRWKV_BWD_CASE(28) }
#undef VRWKV_BWD_CASE
    } else {
        hipLaunchKernelGGL((biwkv_bwd_serial_kernel<IO>), dim3((C + 63) / 64, B), dim3(64), 0, st, w, u,
                           kk, vv, gg, ok, ov, ws, gw_part, gu_part, B, T, C);
    }
    hipLaunchKernelGGL(batch_sum_kernel, dim3((C + 15) / 16), dim3(256), 0, st, gw_part, gw, gu_part, gu, B, C);
    return check_launch("biwkv_bwd");
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" size_t vrwkv_biwkv_bwd_workspace_bytes(int B, int T, int C, int io_dtype) {
    if (validate(B, T, C, io_dtype) != VRWKV_OK) return 0;
    return ((size_t)5 * B * T * C + (size_t)2 * B * C) * sizeof(float);
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
    const size_t need = ((size_t)5 * B * T * C + (size_t)2 * B * C) * sizeof(float);
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
