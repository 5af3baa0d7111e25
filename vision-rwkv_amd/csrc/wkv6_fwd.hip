// wkv6 forward entry points.
#include "wkv6_fwd_scalar.h"
#include "wkv6_fwd_chunk.h"
#include <cstdlib>
#include <cstring>

using namespace vrwkv;
using namespace vrwkv::wkv6_detail;

namespace {

int validate(int B, int T, int C, int H, int rkv_dtype, int w_dtype) {
    if (B <= 0 || T <= 0 || C <= 0 || H <= 0) {
        set_error("wkv6_fwd: B, T, C, H must be positive (got %d, %d, %d, %d)", B, T, C, H);
        return VRWKV_INVALID_ARG;
    }
    if (C != H * N) {                                   // assert(H*_N_ == C), wkv6_cuda.cu:350
        set_error("wkv6_fwd: C must equal H*64 (got C=%d, H=%d)", C, H);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    for (int dt : {rkv_dtype, w_dtype})
        if (dt != VRWKV_F32 && dt != VRWKV_BF16 && dt != VRWKV_F16) {
            set_error("wkv6_fwd: unsupported dtype code %d", dt);
            return VRWKV_UNSUPPORTED_DTYPE;
        }
    if (w_dtype != VRWKV_F32 && w_dtype != rkv_dtype) {
        set_error("wkv6_fwd: w must be fp32 or have the dtype of r, k, v");
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if ((long long)B * T * C >= (1LL << 40) || (long long)B * H > 0x7fffffffLL || (long long)T * C >= (1LL << 29)) {
        set_error("wkv6_fwd: tensor too large");
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    return VRWKV_OK;
}

template <typename IO, typename WT>
int launch_scalar(const void* r, const void* k, const void* v, const void* w, const float* u, float* y,
                  int B, int T, int C, int H, bool w_is_ew, hipStream_t st) {
    const dim3 grid(B * H), block(256);
    const IO* rr = static_cast<const IO*>(r);
    const IO* kk = static_cast<const IO*>(k);
    const IO* vv = static_cast<const IO*>(v);
    const WT* ww = static_cast<const WT*>(w);
    if (w_is_ew) {
        hipLaunchKernelGGL((wkv6_fwd_scalar_kernel<IO, WT, 1, true>), grid, block, 0, st, rr, kk, vv, ww, u, y, T, C, H);
        hipLaunchKernelGGL((wkv6_fwd_scalar_kernel<IO, WT, 0, true>), grid, block, 0, st, rr, kk, vv, ww, u, y, T, C, H);
    } else {
        hipLaunchKernelGGL((wkv6_fwd_scalar_kernel<IO, WT, 1, false>), grid, block, 0, st, rr, kk, vv, ww, u, y, T, C, H);
        hipLaunchKernelGGL((wkv6_fwd_scalar_kernel<IO, WT, 0, false>), grid, block, 0, st, rr, kk, vv, ww, u, y, T, C, H);
    }
    return check_launch("wkv6_fwd");
}

// One launch: both passes of a (b,h) sequence side by side in one workgroup, out-of-range sequences
// redone in place by the sequential recurrence.
template <typename IO, typename WT>
int launch_chunked(const void* r, const void* k, const void* v, const void* w, const float* u, float* y,
                   int B, int T, int C, int H, bool w_is_ew, hipStream_t st) {
    const dim3 grid(B * H), block(64 * FW_WAVES);
    const IO* rr = static_cast<const IO*>(r);
    const IO* kk = static_cast<const IO*>(k);
    const IO* vv = static_cast<const IO*>(v);
    const WT* ww = static_cast<const WT*>(w);
    if (w_is_ew)
        hipLaunchKernelGGL((wkv6_fwd_chunk_kernel<IO, WT, true>), grid, block, 0, st, rr, kk, vv, ww, u, y, T, C, H, nullptr);
    else
        hipLaunchKernelGGL((wkv6_fwd_chunk_kernel<IO, WT, false>), grid, block, 0, st, rr, kk, vv, ww, u, y, T, C, H, nullptr);
    return check_launch("wkv6_fwd (chunked)");
}

bool force_scalar() { return option(OPT_WKV6_FWD_SCALAR) != 0; }   // testing override

template <typename IO, typename WT>
int launch_any(const void* r, const void* k, const void* v, const void* w, const float* u, float* y,
               void* ws, int B, int T, int C, int H, bool w_is_ew, hipStream_t st) {
    (void)ws;
    if (force_scalar()) return launch_scalar<IO, WT>(r, k, v, w, u, y, B, T, C, H, w_is_ew, st);
    return launch_chunked<IO, WT>(r, k, v, w, u, y, B, T, C, H, w_is_ew, st);
}

}  // namespace

extern "C" size_t vrwkv_wkv6_fwd_phases_bytes(int B, int T, int H) {
    if (B <= 0 || T <= 0 || H <= 0) return 0;
    return (size_t)B * H * FW_WAVES * ((T + LC - 1) / LC) * FW_STAMP_POINTS * sizeof(unsigned long long);
}

extern "C" int vrwkv_wkv6_fwd_phases(const void* r, const void* k, const void* v, const void* w, const float* u,
                                     float* y, int B, int T, int C, int H, void* stamps, size_t stamp_bytes,
                                     void* hip_stream) {
    int rc = validate(B, T, C, H, VRWKV_BF16, VRWKV_F32);
    if (rc != VRWKV_OK) return rc;
    if (!r || !k || !v || !w || !u || !y || !stamps) {
        set_error("wkv6_fwd_phases: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    if ((((uintptr_t)r | (uintptr_t)k | (uintptr_t)v) & 1) || (((uintptr_t)w | (uintptr_t)u | (uintptr_t)y) & 3) ||
        ((uintptr_t)stamps & 7)) {
        set_error("wkv6_fwd_phases: pointers must be aligned to their element size");
        return VRWKV_INVALID_ARG;
    }
    const size_t need = vrwkv_wkv6_fwd_phases_bytes(B, T, H);
    if (stamp_bytes < need) {
        set_error("wkv6_fwd_phases: stamp buffer of %zu bytes required (got %zu)", need, stamp_bytes);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    hipLaunchKernelGGL((wkv6_fwd_chunk_kernel<__hip_bfloat16, float, false, true>), dim3(B * H), dim3(64 * FW_WAVES), 0,
                       static_cast<hipStream_t>(hip_stream), static_cast<const __hip_bfloat16*>(r),
                       static_cast<const __hip_bfloat16*>(k), static_cast<const __hip_bfloat16*>(v),
                       static_cast<const float*>(w), u, y, T, C, H, static_cast<unsigned long long*>(stamps));
    return check_launch("wkv6_fwd_phases");
}

extern "C" size_t vrwkv_wkv6_fwd_workspace_bytes(int B, int T, int C, int H) {
    (void)B; (void)T; (void)C; (void)H;
    return 0;                                            // no workspace is needed (kept for ABI symmetry)
}

extern "C" int vrwkv_wkv6_fwd(const void* r, const void* k, const void* v, const void* w, const float* u,
                              float* y, int B, int T, int C, int H, int rkv_dtype, int w_dtype, int w_is_ew,
                              void* workspace, size_t workspace_bytes, void* hip_stream) {
    int rc = validate(B, T, C, H, rkv_dtype, w_dtype);
    if (rc != VRWKV_OK) return rc;
    (void)workspace_bytes;
    if (!r || !k || !v || !w || !u || !y) {
        set_error("wkv6_fwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    const size_t esz = rkv_dtype == VRWKV_F32 ? 4 : 2, wsz = w_dtype == VRWKV_F32 ? 4 : 2;
    if ((((uintptr_t)r | (uintptr_t)k | (uintptr_t)v) & (esz - 1)) || ((uintptr_t)w & (wsz - 1)) ||
        (((uintptr_t)u | (uintptr_t)y) & 3)) {
        set_error("wkv6_fwd: pointers must be aligned to their element size");
        return VRWKV_INVALID_ARG;
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    const bool ew = w_is_ew != 0;
    switch (rkv_dtype) {
        case VRWKV_F32:
            return launch_any<float, float>(r, k, v, w, u, y, workspace, B, T, C, H, ew, st);
        case VRWKV_BF16:
            return w_dtype == VRWKV_F32
                       ? launch_any<__hip_bfloat16, float>(r, k, v, w, u, y, workspace, B, T, C, H, ew, st)
                       : launch_any<__hip_bfloat16, __hip_bfloat16>(r, k, v, w, u, y, workspace, B, T, C, H, ew, st);
        case VRWKV_F16:
            return w_dtype == VRWKV_F32
                       ? launch_any<__half, float>(r, k, v, w, u, y, workspace, B, T, C, H, ew, st)
                       : launch_any<__half, __half>(r, k, v, w, u, y, workspace, B, T, C, H, ew, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
