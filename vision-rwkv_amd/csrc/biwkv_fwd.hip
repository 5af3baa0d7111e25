// Entry points of the Bi-WKV forward (argument checks, plan, dtype dispatch); the kernels
// are instantiated per element type in biwkv_fwd_{f32,bf16,f16}.hip.
#include "biwkv_fwd_impl.h"
#include <atomic>
#include <mutex>

namespace vrwkv {
namespace biwkv_fwd_detail {
extern template int biwkv_fwd_launch_io<float>(const Plan&, const float*, const float*, const void*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
extern template int biwkv_fwd_launch_io<__hip_bfloat16>(const Plan&, const float*, const float*, const void*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
extern template int biwkv_fwd_launch_io<__half>(const Plan&, const float*, const float*, const void*, const void*, const void*, void*, float*, int, int, int, hipStream_t);
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

// ---- workspace of the entry point that allocates nothing -------------------------------------------------------
// The long-sequence path hands per-super-chunk aggregates from its first kernel to its second through a workspace
// (B * nSC * 6 * C floats).  vrwkv_biwkv_fwd takes it from the caller; vrwkv_biwkv_fwd_static takes this array
// instead, which every GPU the library runs on holds (at its own address) until the process ends.
constexpr size_t kStaticWorkspaceBytes = 4u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticWorkspaceBytes];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device; looked up once per device (the array's name is a host-side
// handle, not an address a kernel can use).
int static_workspace(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("biwkv_fwd_static: cannot identify the current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return VRWKV_INVALID_ARG;
    }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p) {
                set_error("biwkv_fwd_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
                return VRWKV_LAUNCH_FAILED;
            }
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
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

namespace vrwkv {
namespace {

// y <- sigmoid(r) * y in place: the gate as a pass of its own, for the calls whose kernels have no gated variant.
// 16-byte pieces where both tensors allow it (two per thread in flight), single elements for the rest and the tail.
template <typename IO>
__global__ __launch_bounds__(256)
void gate_in_place_kernel(const IO* r_, IO* y_, size_t n, size_t n_vec) {
    constexpr int V = 16 / (int)sizeof(IO);
    const size_t stride = (size_t)gridDim.x * blockDim.x, tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    auto one = [&](size_t i) {
        float rv[V], yv[V];
        load_vec_nt<IO, V>(r_ + i * V, rv);
        load_vec<IO, V>(y_ + i * V, yv);
#pragma unroll
        for (int e = 0; e < V; ++e) yv[e] *= fast_rcp(1.f + fast_exp2(-rv[e] * LOG2E));
        store_vec<IO, V>(y_ + i * V, yv);
    };
    size_t i = tid;
    for (; i + stride < n_vec; i += 2 * stride) {
        float r0[V], y0[V], r1[V], y1[V];
        load_vec_nt<IO, V>(r_ + i * V, r0);
        load_vec<IO, V>(y_ + i * V, y0);
        load_vec_nt<IO, V>(r_ + (i + stride) * V, r1);
        load_vec<IO, V>(y_ + (i + stride) * V, y1);
#pragma unroll
        for (int e = 0; e < V; ++e) {
            y0[e] *= fast_rcp(1.f + fast_exp2(-r0[e] * LOG2E));
            y1[e] *= fast_rcp(1.f + fast_exp2(-r1[e] * LOG2E));
        }
        store_vec<IO, V>(y_ + i * V, y0);
        store_vec<IO, V>(y_ + (i + stride) * V, y1);
    }
    if (i < n_vec) one(i);
    for (size_t j = n_vec * V + tid; j < n; j += stride) {
        const float g = fast_rcp(1.f + fast_exp2(-to_f32(r_[j]) * LOG2E));
        y_[j] = from_f32<IO>(to_f32(y_[j]) * g);
    }
}
template <typename IO>
int launch_gate_in_place(const void* r, void* y, size_t n, hipStream_t st) {
    constexpr int V = 16 / (int)sizeof(IO);
    const bool aligned = (((uintptr_t)r | (uintptr_t)y) & 15) == 0;
    const size_t n_vec = aligned ? n / V : 0;
    const size_t work = n_vec / 2 + (n - n_vec * V) + 1;          // threads that have something to do
    size_t blocks = (work + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL((gate_in_place_kernel<IO>), dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const IO*>(r), static_cast<IO*>(y), n, n_vec);
    return check_launch("biwkv_fwd_gate");
}

// the forward, with the gate when r is given
int biwkv_fwd_common(const char* who, const float* w, const float* u, const void* k, const void* v, const void* r, void* y,
                     int B, int T, int C, int io_dtype, void* workspace, size_t workspace_bytes, void* hip_stream) {
    int rc = validate(B, T, C, io_dtype);
    if (rc != VRWKV_OK) return rc;
    if (!w || !u || !k || !v || !y) {
        set_error("%s: null pointer argument", who);
        return VRWKV_INVALID_ARG;
    }
    const size_t esz = io_dtype == VRWKV_F32 ? 4 : 2;
    if ((((uintptr_t)k | (uintptr_t)v | (uintptr_t)y | (uintptr_t)r) & (esz - 1)) || (((uintptr_t)w | (uintptr_t)u) & 3)) {
        set_error("%s: pointers must be aligned to their element size", who);
        return VRWKV_INVALID_ARG;
    }
    const Plan p = make_plan(B, T, C, io_dtype);
    if (p.multi()) {
        const size_t need = (size_t)B * p.nSC * NSLOT * C * sizeof(float);
        if (!workspace || workspace_bytes < need) {
            set_error("%s: workspace of %zu bytes required for T=%d (got %zu)", who, need, T,
                      workspace ? workspace_bytes : (size_t)0);
            return VRWKV_WORKSPACE_TOO_SMALL;
        }
        if ((uintptr_t)workspace & 3) {
            set_error("%s: workspace must be 4-byte aligned", who);
            return VRWKV_INVALID_ARG;
        }
    }
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* ws = static_cast<float*>(workspace);
    auto go = [&](const void* rr) -> int {
        switch (io_dtype) {
            case VRWKV_F32:  return biwkv_fwd_launch_io<float>(p, w, u, k, v, rr, y, ws, B, T, C, st);
            case VRWKV_BF16: return biwkv_fwd_launch_io<__hip_bfloat16>(p, w, u, k, v, rr, y, ws, B, T, C, st);
            case VRWKV_F16:  return biwkv_fwd_launch_io<__half>(p, w, u, k, v, rr, y, ws, B, T, C, st);
        }
        return VRWKV_UNSUPPORTED_DTYPE;
    };
    rc = go(r);
    if (rc != GATE_NOT_FUSED) return rc;
    rc = go(nullptr);
    if (rc != VRWKV_OK) return rc;
    const size_t n = (size_t)B * T * C;
    switch (io_dtype) {
        case VRWKV_F32:  return launch_gate_in_place<float>(r, y, n, st);
        case VRWKV_BF16: return launch_gate_in_place<__hip_bfloat16>(r, y, n, st);
        default:         return launch_gate_in_place<__half>(r, y, n, st);
    }
}

}  // namespace
}  // namespace vrwkv

extern "C" int vrwkv_biwkv_fwd(const float* w, const float* u, const void* k, const void* v, void* y,
                               int B, int T, int C, int io_dtype,
                               void* workspace, size_t workspace_bytes, void* hip_stream) {
    return biwkv_fwd_common("biwkv_fwd", w, u, k, v, nullptr, y, B, T, C, io_dtype, workspace, workspace_bytes, hip_stream);
}

extern "C" int vrwkv_biwkv_fwd_gate(const float* w, const float* u, const void* k, const void* v, const void* r, void* y,
                                    int B, int T, int C, int io_dtype,
                                    void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (!r) {
        set_error("biwkv_fwd_gate: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    return biwkv_fwd_common("biwkv_fwd_gate", w, u, k, v, r, y, B, T, C, io_dtype, workspace, workspace_bytes, hip_stream);
}

extern "C" size_t vrwkv_biwkv_fwd_static_max_workspace_bytes(void) { return kStaticWorkspaceBytes; }

extern "C" int vrwkv_biwkv_fwd_static(const float* w, const float* u, const void* k, const void* v, void* y,
                                      int B, int T, int C, int io_dtype, void* hip_stream) {
    int rc = validate(B, T, C, io_dtype);
    if (rc != VRWKV_OK) return rc;
    const size_t need = vrwkv_biwkv_fwd_workspace_bytes(B, T, C, io_dtype);
    if (need > kStaticWorkspaceBytes) {
        set_error("biwkv_fwd_static: B=%d, T=%d, C=%d needs a workspace of %zu bytes, the built-in one holds %zu; "
                  "use vrwkv_biwkv_fwd with a caller-owned workspace", B, T, C, need, kStaticWorkspaceBytes);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    void* ws = nullptr;
    rc = static_workspace(&ws);
    if (rc != VRWKV_OK) return rc;
    // every workspace entry the second kernel reads is written by the first one of the same call: nothing to clear
    return vrwkv_biwkv_fwd(w, u, k, v, y, B, T, C, io_dtype, ws, kStaticWorkspaceBytes, hip_stream);
}
