// Entry points of the Bi-WKV forward (argument checks, plan, dtype dispatch); the kernels
// are instantiated per element type in biwkv_fwd_{f32,bf16,f16}.hip.
#include "biwkv_fwd_impl.h"

namespace vrwkv {
namespace biwkv_fwd_detail {
extern template int biwkv_fwd_launch_io<float>(const Plan&, const float*, const float*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
extern template int biwkv_fwd_launch_io<__hip_bfloat16>(const Plan&, const float*, const float*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
extern template int biwkv_fwd_launch_io<__half>(const Plan&, const float*, const float*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
}
namespace {
using namespace biwkv_fwd_detail;

int validate(int B, int T, int C, int io_dtype) {
    if (B <= 0 || T <= 0 || C <= 0) {
        set_error("biwkv_fwd: B, T, C must be positive (got %d, %d, %d)", B, T, C);
        return VRWKV_INVALID_ARG;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("biwkv_fwd: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if ((long long)T * C * 4 >= (1LL << 31) || (long long)B * T * C >= (1LL << 40)) {
        set_error("biwkv_fwd: T*C must stay below 2^29 elements (got T=%d, C=%d)", T, C);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    return VRWKV_OK;
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" size_t vrwkv_biwkv_fwd_workspace_bytes(int B, int T, int C, int io_dtype) {
    if (validate(B, T, C, io_dtype) != VRWKV_OK) return 0;
    const Plan p = make_plan(B, T, C, io_dtype);
    if (!p.multi()) return 0;
    return (size_t)B * p.nSC * NSLOT * C * sizeof(float);
}

extern "C" int vrwkv_biwkv_fwd(const float* w, const float* u, const void* k, const void* v, void* y,
                               int B, int T, int C, int io_dtype,
                               void* workspace, size_t workspace_bytes, void* hip_stream) {
    int rc = validate(B, T, C, io_dtype);
    if (rc != VRWKV_OK) return rc;
    if (!w || !u || !k || !v || !y) {
        set_error("biwkv_fwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    const size_t esz = io_dtype == VRWKV_F32 ? 4 : 2;
    if ((((uintptr_t)k | (uintptr_t)v | (uintptr_t)y) & (esz - 1)) || (((uintptr_t)w | (uintptr_t)u) & 3)) {
        set_error("biwkv_fwd: pointers must be aligned to their element size");
        return VRWKV_INVALID_ARG;
    }
    const Plan p = make_plan(B, T, C, io_dtype);
    if (p.multi()) {
        const size_t need = (size_t)B * p.nSC * NSLOT * C * sizeof(float);
        if (!workspace || workspace_bytes < need) {
            set_error("biwkv_fwd: workspace of %zu bytes required for T=%d (got %zu)", need, T,
                      workspace ? workspace_bytes : (size_t)0);
            return VRWKV_WORKSPACE_TOO_SMALL;
        }
        if ((uintptr_t)workspace & 3) {
            set_error("biwkv_fwd: workspace must be 4-byte aligned");
            return VRWKV_INVALID_ARG;
        }
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* ws = static_cast<float*>(workspace);
    switch (io_dtype) {
        case VRWKV_F32:  return biwkv_fwd_launch_io<float>(p, w, u, k, v, y, ws, B, T, C, st);
        case VRWKV_BF16: return biwkv_fwd_launch_io<__hip_bfloat16>(p, w, u, k, v, y, ws, B, T, C, st);
        case VRWKV_F16:  return biwkv_fwd_launch_io<__half>(p, w, u, k, v, y, ws, B, T, C, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
