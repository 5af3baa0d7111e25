// Helpers shared by the chunked matrix-core wkv6 kernels (forward and backward scans) for gfx950: packed bf16
// head / tail splits, DPP moves, the transposing row-sum butterflies and the layout constants of the LDS operands.
#pragma once
#include "vrwkv_common.h"
#include "wkv6_fwd_scalar.h"
#include <type_traits>

namespace vrwkv {
namespace wkv6_detail {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int LC = 32;           // chunk length
constexpr int HN = 64;           // head size
constexpr int PJ = 72;           // row pitch (bf16) of the [token][channel] operand arrays
constexpr int PS = 40;           // row pitch (bf16) of the [channel][token] operand arrays
constexpr float SAFE_DECAY = 60.f;

__device__ __forceinline__ bf16x8 cat8(bf16x4 a, bf16x4 b) {
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
constexpr float LOG2_LOG2E = 0.5287663729448977f;     // log2(log2(e))
// two fp32 values rounded to bf16 in one register (a low, b high), and the halves widened back
__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
__device__ __forceinline__ float bf16_lo(unsigned w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(unsigned w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
__device__ __forceinline__ void st_bf16_pair(__bf16* lo, __bf16* hi, unsigned w) {
    *reinterpret_cast<unsigned short*>(lo) = (unsigned short)w;
    *reinterpret_cast<unsigned short*>(hi) = (unsigned short)(w >> 16);
}

// head/tail split of eight fp32 accumulator values into two packed bf16 operands (two values per conversion)
__device__ __forceinline__ void split8(const float (&x)[8], bf16x8& hi, bf16x8& lo) {
    u32x4 h, l;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const unsigned w = pack_bf16(x[2 * p], x[2 * p + 1]);
        h[p] = w;
        l[p] = pack_bf16(x[2 * p] - bf16_lo(w), x[2 * p + 1] - bf16_hi(w));
    }
    hi = __builtin_bit_cast(bf16x8, h);
    lo = __builtin_bit_cast(bf16x8, l);
}

// DPP move: lane reads `v` of the lane selected by CTRL (0 where there is none).
template <int CTRL>
__device__ __forceinline__ float dpp_get(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// 16 values per lane -> per 16-lane row, the row sums of all 16: lane l ends up with the sum over
// its row of value index 8*(l&1) + 4*((l>>1)&1) + 2*((l>>3)&1) + ((l>>2)&1).  Transposing butterfly:
// at each step a lane keeps one half of its values and hands the other half to its partner.
__device__ __forceinline__ float row_sums16(const float (&p)[16], int lane, int& index) {
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4, b3 = lane & 8;
    float a8[8], a4[4], a2[2];
#pragma unroll
    for (int i = 0; i < 8; ++i) a8[i] = (b0 ? p[8 + i] : p[i]) + dpp_get<0xB1>(b0 ? p[i] : p[8 + i]);     // quad_perm [1,0,3,2]
#pragma unroll
    for (int i = 0; i < 4; ++i) a4[i] = (b1 ? a8[4 + i] : a8[i]) + dpp_get<0x4E>(b1 ? a8[i] : a8[4 + i]); // quad_perm [2,3,0,1]
#pragma unroll
    for (int i = 0; i < 2; ++i) a2[i] = (b3 ? a4[2 + i] : a4[i]) + dpp_get<0x128>(b3 ? a4[i] : a4[2 + i]); // row_ror:8
    const float give = b2 ? a2[0] : a2[1];
    const float from_lo = dpp_get<0x114>(give), from_hi = dpp_get<0x104>(give);   // row_shr:4 (from l-4), row_shl:4 (from l+4)
    const float recv = b2 ? from_lo : from_hi;                            // both moves run with every lane active
    index = (b0 ? 8 : 0) + (b1 ? 4 : 0) + (b3 ? 2 : 0) + (b2 ? 1 : 0);
    return (b2 ? a2[1] : a2[0]) + recv;
}


}  // namespace wkv6_detail
}  // namespace vrwkv
