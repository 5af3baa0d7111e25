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
int device_cus();                 // compute units of the current device (256 when the query fails)

// Tuning / testing switches (0 = default behaviour).  Their initial values come from the environment variables
// VRWKV_<NAME IN CAPITALS>, read once per process; vrwkv_set_option changes them afterwards.
enum Option {
    OPT_BIWKV_L,            // tokens per wave of the Bi-WKV forward (4, 8, 16, 28)
    OPT_BIWKV_S,            // waves per workgroup on the long-sequence path
    OPT_BIWKV_GRID,         // persistent grid size
    OPT_BIWKV_NO_STAGE,     // register loads instead of LDS-staged rows
    OPT_BIWKV_NO_RESIDENT,  // two-kernel long-sequence path also where the one-launch kernel applies
    OPT_BIWKV_BWD_SERIAL,   // sequential Bi-WKV backward kernel
    OPT_WKV6_FWD_SCALAR,    // sequential-state wkv6 forward kernel
    OPT_WKV6_BWD_SCALAR,    // sequential wkv6 backward sweeps
    OPT_WKV6_BWD_UNFUSED,   // one launch per wkv6 backward scan
    N_OPTIONS
};
int option(Option o);

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
// A vector of VEC elements fetched now and widened where it is used (it waits in its packed form).
template <typename IO, int VEC>
__device__ __forceinline__ typename RawVec<sizeof(IO) * VEC>::type load_packed(const IO* __restrict__ p) {
    return *reinterpret_cast<const typename RawVec<sizeof(IO) * VEC>::type*>(p);
}
template <typename IO, int VEC>
__device__ __forceinline__ void widen_packed(typename RawVec<sizeof(IO) * VEC>::type raw, float (&out)[VEC]) {
    IO tmp[VEC];
    __builtin_memcpy(tmp, &raw, sizeof(raw));
#pragma unroll
    for (int e = 0; e < VEC; ++e) out[e] = to_f32(tmp[e]);
}
// The same with the non-temporal cache policy, for tensors that are streamed through once (16-byte vectors only).
typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4)));
template <typename IO, int VEC>
__device__ __forceinline__ void load_vec_nt(const IO* __restrict__ p, float (&out)[VEC]) {
    static_assert(sizeof(IO) * VEC == 16, "16-byte vectors");
    const nt_u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4*>(p));
    IO tmp[VEC];
    __builtin_memcpy(tmp, &raw, sizeof(raw));
#pragma unroll
    for (int e = 0; e < VEC; ++e) out[e] = to_f32(tmp[e]);
}
// A 16-byte vector fetched now and widened where it is used (keeps four registers, not VEC, while it waits).
template <bool NT>
__device__ __forceinline__ nt_u32x4 load_raw16(const void* p) {
    return NT ? __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4*>(p)) : *reinterpret_cast<const nt_u32x4*>(p);
}
template <typename IO, int VEC>
__device__ __forceinline__ void widen_raw16(nt_u32x4 raw, float (&out)[VEC]) {
    static_assert(sizeof(IO) * VEC == 16, "16-byte vectors");
    IO tmp[VEC];
    __builtin_memcpy(tmp, &raw, sizeof(raw));
#pragma unroll
    for (int e = 0; e < VEC; ++e) out[e] = to_f32(tmp[e]);
}
template <typename IO, int VEC>
__device__ __forceinline__ void store_vec_nt(IO* __restrict__ p, const float (&in)[VEC]) {
    static_assert(sizeof(IO) * VEC == 16, "16-byte vectors");
    IO tmp[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) tmp[e] = from_f32<IO>(in[e]);
    nt_u32x4 raw;
    __builtin_memcpy(&raw, tmp, sizeof(raw));
    __builtin_nontemporal_store(raw, reinterpret_cast<nt_u32x4*>(p));
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
// ---- per-phase cycle stamps (instrumented build only: -DVRWKV_STAMPS, `make stamps`) ----------------------------
// A wave records the shader clock at numbered points of a tile into a buffer the host registered with
// vrwkv_debug_set_stamp_buffer_<tag>(buffer, n_workgroups): layout [workgroup][wave (8)][tile slot (VRWKV_STAMP_TILES)]
// [point (VRWKV_STAMP_POINTS)]; workgroups beyond the count the buffer was sized for record nothing.
#ifdef VRWKV_STAMPS
constexpr int VRWKV_STAMP_TILES = 4, VRWKV_STAMP_POINTS = 12;
static __device__ unsigned long long* g_stamp_buffer = nullptr;   // one per translation unit (device code is not linked across them)
static __device__ unsigned g_stamp_workgroups = 0;                // workgroups the buffer has room for
// defines vrwkv_debug_set_stamp_buffer_<tag>(device_buffer, n_workgroups) for the translation unit it is used in
#define VRWKV_DEFINE_STAMP_SETTER(tag)                                                                      \
    extern "C" int vrwkv_debug_set_stamp_buffer_##tag(void* device_buffer, unsigned n_workgroups) {          \
        unsigned long long* p = static_cast<unsigned long long*>(device_buffer);                             \
        if (hipMemcpyToSymbol(HIP_SYMBOL(::vrwkv::g_stamp_workgroups), &n_workgroups, sizeof(n_workgroups)) != hipSuccess) return 4; \
        return hipMemcpyToSymbol(HIP_SYMBOL(::vrwkv::g_stamp_buffer), &p, sizeof(p)) == hipSuccess ? 0 : 4;   \
    }
__device__ __forceinline__ void stamp(int wave, int slot, int point) {
    unsigned long long* buf = g_stamp_buffer;
    if (buf && blockIdx.x < g_stamp_workgroups && wave < 8 && slot < VRWKV_STAMP_TILES && point < VRWKV_STAMP_POINTS &&
        (threadIdx.x & 63) == 0) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        buf[(((size_t)blockIdx.x * 8 + wave) * VRWKV_STAMP_TILES + slot) * VRWKV_STAMP_POINTS + point] = __builtin_amdgcn_s_memtime();
    }
}
#define VRWKV_STAMP(wave, slot, point) ::vrwkv::stamp(wave, slot, point)
#else
#define VRWKV_STAMP(wave, slot, point) ((void)0)
#endif

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// out[c] = sum_b part[b*C + c] for up to two (part, out) pairs (the second may be null).  1024 threads = 32 columns
// (one 128-byte piece of a row per half wave) x 32 slices of the batch, sixteen loads of a slice in flight at a time
// (512 partial rows in one round of loads); the slices are added in a fixed order (deterministic).
// Grid: ceil(C / BATCH_SUM_COLS), block: BATCH_SUM_THREADS.
constexpr int BATCH_SUM_THREADS = 1024, BATCH_SUM_COLS = 32, BATCH_SUM_SLICES = BATCH_SUM_THREADS / BATCH_SUM_COLS;
__global__ __launch_bounds__(1024) inline void batch_sum_kernel(const float* __restrict__ part0, float* __restrict__ out0,
                                                                const float* __restrict__ part1, float* __restrict__ out1,
                                                                int B, int C) {
    constexpr int NS = BATCH_SUM_SLICES, U = 16;
    __shared__ float red[2][NS][BATCH_SUM_COLS];
    const int cl = threadIdx.x % BATCH_SUM_COLS, slice = threadIdx.x / BATCH_SUM_COLS;
    const int c = blockIdx.x * BATCH_SUM_COLS + cl;
    float s0 = 0.f, s1 = 0.f;
    if (c < C) {
        int b = slice;
        for (; b + NS * (U - 1) < B; b += NS * U) {
            float t0[U], t1[U];
#pragma unroll
            for (int i = 0; i < U; ++i) {
                t0[i] = part0[(size_t)(b + NS * i) * C + c];
                t1[i] = part1 ? part1[(size_t)(b + NS * i) * C + c] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < U; ++i) { s0 += t0[i]; s1 += t1[i]; }
        }
        for (; b < B; b += NS) {
            s0 += part0[(size_t)b * C + c];
            if (part1) s1 += part1[(size_t)b * C + c];
        }
    }
    red[0][slice][cl] = s0;
    red[1][slice][cl] = s1;
    __syncthreads();
    if (slice == 0 && c < C) {
        float t0 = 0.f, t1 = 0.f;
#pragma unroll
        for (int i = 0; i < NS; ++i) { t0 += red[0][i][cl]; t1 += red[1][i][cl]; }
        out0[c] = t0;
        if (part1) out1[c] = t1;
    }
}
#endif

}  // namespace vrwkv
