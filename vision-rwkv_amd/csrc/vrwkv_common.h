// Shared host/device helpers for the vrwkv HIP library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <cstdarg>
#include <cstdio>
#include "../../include/vrwkv_hip.h"

namespace vrwkv {

// Thread-local message behind vrwkv_last_error().
void set_error(const char* fmt, ...);
// Returns VRWKV_OK, or VRWKV_LAUNCH_FAILED after recording hipGetLastError()'s text.
int check_launch(const char* what);

constexpr int WAVE = 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float NEG_BIG = -1e38f;   // "empty state" exponent, bi_wkv_kernel.cu:14

#if defined(__HIPCC__)
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(__hip_bfloat16 x) { return __bfloat162float(x); }
__device__ __forceinline__ float to_f32(__half x) { return __half2float(x); }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ __hip_bfloat16 from_f32<__hip_bfloat16>(float x) { return __float2bfloat16(x); }
template <> __device__ __forceinline__ __half from_f32<__half>(float x) { return __float2half(x); }

template <int BYTES> struct RawVec;
template <> struct RawVec<2>  { using type = unsigned short; };
template <> struct RawVec<4>  { using type = unsigned int; };
template <> struct RawVec<8>  { using type = uint2; };
template <> struct RawVec<16> { using type = uint4; };

// One vector load of VEC consecutive elements, widened to fp32.
template <typename IO, int VEC>
__device__ __forceinline__ void load_vec(const IO* __restrict__ p, float (&out)[VEC]) {
    using R = typename RawVec<sizeof(IO) * VEC>::type;
    R raw = *reinterpret_cast<const R*>(p);
    IO tmp[VEC];
    __builtin_memcpy(tmp, &raw, sizeof(raw));
#pragma unroll
    for (int e = 0; e < VEC; ++e) out[e] = to_f32(tmp[e]);
}
template <typename IO, int VEC>
__device__ __forceinline__ void store_vec(IO* __restrict__ p, const float (&in)[VEC]) {
    using R = typename RawVec<sizeof(IO) * VEC>::type;
    IO tmp[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) tmp[e] = from_f32<IO>(in[e]);
    R raw;
    __builtin_memcpy(&raw, tmp, sizeof(raw));
    *reinterpret_cast<R*>(p) = raw;
}
// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it does not wait
// for outstanding global loads/stores (vmcnt), so prefetches stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- raw buffer access (descriptor + 32-bit byte offsets; out-of-range accesses are dropped by the
//      hardware: loads return 0, stores do nothing) -------------------------------------------------
constexpr unsigned OOB_OFFSET = 0x80000000u;   // byte offset no descriptor here reaches
constexpr unsigned CPOL_NT = 2;                // gfx94x/gfx950 cache policy bit: non-temporal (data streamed once)
template <int BYTES> struct BufRaw;
template <> struct BufRaw<2> {
    using type = unsigned short;
    template <unsigned CP = 0> static __device__ __forceinline__ type ld(__amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { return __builtin_amdgcn_raw_buffer_load_b16(r, v, s, CP); }
    template <unsigned CP = 0> static __device__ __forceinline__ void st(type d, __amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { __builtin_amdgcn_raw_buffer_store_b16(d, r, v, s, CP); }
};
template <> struct BufRaw<4> {
    using type = unsigned int;
    template <unsigned CP = 0> static __device__ __forceinline__ type ld(__amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { return __builtin_amdgcn_raw_buffer_load_b32(r, v, s, CP); }
    template <unsigned CP = 0> static __device__ __forceinline__ void st(type d, __amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { __builtin_amdgcn_raw_buffer_store_b32(d, r, v, s, CP); }
};
template <> struct BufRaw<8> {
    typedef unsigned int type __attribute__((ext_vector_type(2)));
    template <unsigned CP = 0> static __device__ __forceinline__ type ld(__amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { return __builtin_amdgcn_raw_buffer_load_b64(r, v, s, CP); }
    template <unsigned CP = 0> static __device__ __forceinline__ void st(type d, __amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { __builtin_amdgcn_raw_buffer_store_b64(d, r, v, s, CP); }
};
template <> struct BufRaw<16> {
    typedef unsigned int type __attribute__((ext_vector_type(4)));
    template <unsigned CP = 0> static __device__ __forceinline__ type ld(__amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { return __builtin_amdgcn_raw_buffer_load_b128(r, v, s, CP); }
    template <unsigned CP = 0> static __device__ __forceinline__ void st(type d, __amdgpu_buffer_rsrc_t r, unsigned v, unsigned s) { __builtin_amdgcn_raw_buffer_store_b128(d, r, v, s, CP); }
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
#endif

}  // namespace vrwkv
