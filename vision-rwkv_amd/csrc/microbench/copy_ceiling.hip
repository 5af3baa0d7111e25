// What a kernel that only moves the Bi-WKV forward's bytes reaches on this device: out = f(a, b) element-wise on
// three (64, 196, 768) fp32 tensors -- the traffic of one VRWKV-B call (two reads, one write, 115.6 MB) -- with
//   linear    every workgroup streams a contiguous range, 16 bytes per lane;
//   tile      the forward kernel's access pattern without its arithmetic: a workgroup of 7 waves owns one
//             (batch, 64 channels) tile of 196 token rows, i.e. 256-byte row pieces 3 KB apart, moved as 16-byte
//             pieces, all loads of a tile issued before its stores; persistent (one workgroup per CU) or one
//             workgroup per tile;
// each with plain and with non-temporal cache policy.  Twelve distinct buffer sets are cycled through, as in the
// benchmark, so nothing stays cache-resident from call to call.  Build: make -C vision-rwkv_amd/csrc microbench
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 1; } } while (0)
typedef unsigned u4 __attribute__((ext_vector_type(4)));
constexpr unsigned OOB = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

template <int CP>
__global__ __launch_bounds__(256) void linear_copy(const u4* __restrict__ a, const u4* __restrict__ b, u4* __restrict__ o, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
        u4 x, y;
        if (CP) { x = __builtin_nontemporal_load(a + i); y = __builtin_nontemporal_load(b + i); }
        else { x = a[i]; y = b[i]; }
        if (CP) __builtin_nontemporal_store(x ^ y, o + i); else o[i] = x ^ y;
    }
}

template <int CP>
__global__ __launch_bounds__(448) void tile_copy(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ o,
                                                 int T, int C, int n_tiles, int n_ctile) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned bytes = (unsigned)((size_t)T * C * 4);
    for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int ct = tile % n_ctile, bb = tile / n_ctile;
        const size_t slab = (size_t)bb * T * C;
        const __amdgpu_buffer_rsrc_t ra = rsrc(a + slab, bytes), rb = rsrc(b + slab, bytes), ro = rsrc(o + slab, bytes);
        u4 x[7], y[7];
        unsigned off[7];
#pragma unroll
        for (int i = 0; i < 7; ++i) {                       // 28 rows per wave, 4 rows of 256 bytes per instruction
            const int row = wave * 28 + 4 * i + (lane >> 4), col = ct * 64 + (lane & 15) * 4;
            off[i] = row < T ? (unsigned)((row * C + col) * 4) : OOB;
            x[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, off[i], 0, CP);
            y[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off[i], 0, CP);
        }
#pragma unroll
        for (int i = 0; i < 7; ++i) __builtin_amdgcn_raw_buffer_store_b128(x[i] ^ y[i], ro, off[i], 0, CP);
    }
}

int main() {
    const int B = 64, T = 196, C = 768, NB = 12;
    const size_t n = (size_t)B * T * C;
    std::vector<float*> a(NB), b(NB), o(NB);
    for (int i = 0; i < NB; ++i) {
        CK(hipMalloc(&a[i], n * 4)); CK(hipMalloc(&b[i], n * 4)); CK(hipMalloc(&o[i], n * 4));
        CK(hipMemset(a[i], 1, n * 4)); CK(hipMemset(b[i], 2, n * 4));
    }
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int ncu = prop.multiProcessorCount;
    const double bytes = 3.0 * n * 4;
    auto timeit = [&](const char* name, auto launch) -> int {
        for (int r = 0; r < 3; ++r) for (int i = 0; i < NB; ++i) launch(i);
        CK(hipDeviceSynchronize());
        double best = 1e30, sum = 0;
        for (int rep = 0; rep < 5; ++rep) {
            CK(hipEventRecord(e0, 0));
            for (int r = 0; r < 10; ++r) for (int i = 0; i < NB; ++i) launch(i);
            CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1));
            const double us = ms * 1e3 / (10 * NB);
            best = us < best ? us : best; sum += us;
        }
        const double us = sum / 5;
        printf("%-52s %7.2f us/call (best loop %6.2f)  %6.0f GB/s  %5.1f %% of 8 TB/s\n", name, us, best, bytes / us / 1e3, bytes / us / 1e3 / 80);
        fflush(stdout);
        return 0;
    };
    const int nct = C / 64, nt = B * nct;
    printf("copy ceiling for 2 reads + 1 write of (%d, %d, %d) fp32 = %.1f MB per call, %d CUs\n", B, T, C, bytes / 1e6, ncu);
    if (timeit("linear, plain, 2048 workgroups", [&](int i) { hipLaunchKernelGGL(linear_copy<0>, dim3(2048), dim3(256), 0, 0, (const u4*)a[i], (const u4*)b[i], (u4*)o[i], n / 4); })) return 1;
    if (timeit("linear, non-temporal, 2048 workgroups", [&](int i) { hipLaunchKernelGGL(linear_copy<1>, dim3(2048), dim3(256), 0, 0, (const u4*)a[i], (const u4*)b[i], (u4*)o[i], n / 4); })) return 1;
    if (timeit("linear, non-temporal, 8 workgroups per CU", [&](int i) { hipLaunchKernelGGL(linear_copy<1>, dim3(8 * ncu), dim3(256), 0, 0, (const u4*)a[i], (const u4*)b[i], (u4*)o[i], n / 4); })) return 1;
    if (timeit("tile, plain, one workgroup per tile", [&](int i) { hipLaunchKernelGGL(tile_copy<0>, dim3(nt), dim3(448), 0, 0, a[i], b[i], o[i], T, C, nt, nct); })) return 1;
    if (timeit("tile, non-temporal, one workgroup per tile", [&](int i) { hipLaunchKernelGGL(tile_copy<2>, dim3(nt), dim3(448), 0, 0, a[i], b[i], o[i], T, C, nt, nct); })) return 1;
    if (timeit("tile, non-temporal, persistent (one workgroup per CU)", [&](int i) { hipLaunchKernelGGL(tile_copy<2>, dim3(ncu), dim3(448), 0, 0, a[i], b[i], o[i], T, C, nt, nct); })) return 1;
    return 0;
}
