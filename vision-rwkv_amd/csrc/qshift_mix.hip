// Fused Q-Shift + token-mix prologue: for m = 0..n_mix-1
//   out_m[b,t,c] = x[b,t,c] * mix_m[c] + xx[b,t,c] * (1 - mix_m[c]),   xx = q_shift(x)
// i.e. q_shift (classification/mmcls_custom/models/backbones/vrwkv.py:68-79) and the lerps of
// VRWKV_SpatialMix.jit_func (:160-163, three mixes) / VRWKV_ChannelMix.forward (:248-250, two mixes)
// in one pass: x is read once (plus the neighbouring rows, which hit in cache), the shifted copy,
// its two transposes and the zero-filled buffer of the reference are never materialised.
// Tokens are row-major over the (Hp, Wp) patch grid.  Channel quarter q of width g = int(C*gamma)
// takes its value from the pixel one step left / right / up / down (zero outside the grid);
// channels >= 4g pass through.  q_shift_multihead (vrwkv6.py:75-100) is the same with the quarter
// taken inside every head: pass head_dim = 64 (0 = whole-tensor quarters).
#include "vrwkv_common.h"

namespace vrwkv {
namespace {

template <typename IO, int VEC, int NMIX>
__global__ __launch_bounds__(256)
void qshift_mix_kernel(const IO* __restrict__ x_, const float* __restrict__ mix_, IO* __restrict__ o0, IO* __restrict__ o1,
                       IO* __restrict__ o2, int T, int C, int Hp, int Wp, int shift, int g, int head_dim, int n_grid_tokens)
{
    const int cv = blockIdx.x * blockDim.x + threadIdx.x;       // channel vector
    const int c = cv * VEC;
    if (c >= C) return;
    const int t = blockIdx.y, b = blockIdx.z;
    const size_t row = ((size_t)b * T + t) * C;
    float xs[VEC], xx[VEC];
    load_vec<IO, VEC>(x_ + row + c, xs);
    // direction of this channel vector (host guarantees a vector never straddles a quarter boundary)
    const int cq = head_dim > 0 ? c % head_dim : c;
    const int dir = (g > 0 && cq < 4 * g) ? cq / g : 4;
    bool have = true;
    int ts = t;
    if (t >= n_grid_tokens) {
        // trailing class token (q_shift_multihead with_cls_token): passed through
    } else if (dir < 4) {
        const int yy = t / Wp, xc = t % Wp;
        int sy = yy, sx = xc;
        if (dir == 0) sx = xc - shift; else if (dir == 1) sx = xc + shift;
        else if (dir == 2) sy = yy - shift; else sy = yy + shift;
        have = sx >= 0 && sx < Wp && sy >= 0 && sy < Hp;
        ts = sy * Wp + sx;
    }
    if (have && ts != t) load_vec<IO, VEC>(x_ + ((size_t)b * T + ts) * C + c, xx);
    else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) xx[e] = have ? xs[e] : 0.f;
    }
    IO* outs[3] = {o0, o1, o2};
#pragma unroll
    for (int m = 0; m < NMIX; ++m) {
        float r[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float mu = mix_[(size_t)m * C + c + e];
            r[e] = xs[e] * mu + xx[e] * (1.f - mu);
        }
        store_vec<IO, VEC>(outs[m] + row + c, r);
    }
}

template <typename IO, int VEC>
int launch(const void* x, const float* mix, void* const* out, int n_mix, int B, int T, int C, int Hp, int Wp,
           int shift, int g, int head_dim, int n_grid, hipStream_t st) {
    const int ncv = C / VEC;
    const dim3 block(ncv < 256 ? ((ncv + 63) / 64) * 64 : 256);
    const dim3 grid((ncv + block.x - 1) / block.x, T, B);
    const IO* xx = static_cast<const IO*>(x);
    IO* o0 = static_cast<IO*>(out[0]);
    IO* o1 = n_mix > 1 ? static_cast<IO*>(out[1]) : nullptr;
    IO* o2 = n_mix > 2 ? static_cast<IO*>(out[2]) : nullptr;
    switch (n_mix) {
        case 1: hipLaunchKernelGGL((qshift_mix_kernel<IO, VEC, 1>), grid, block, 0, st, xx, mix, o0, o1, o2, T, C, Hp, Wp, shift, g, head_dim, n_grid); break;
        case 2: hipLaunchKernelGGL((qshift_mix_kernel<IO, VEC, 2>), grid, block, 0, st, xx, mix, o0, o1, o2, T, C, Hp, Wp, shift, g, head_dim, n_grid); break;
        case 3: hipLaunchKernelGGL((qshift_mix_kernel<IO, VEC, 3>), grid, block, 0, st, xx, mix, o0, o1, o2, T, C, Hp, Wp, shift, g, head_dim, n_grid); break;
    }
    return check_launch("qshift_mix");
}

template <typename IO>
int launch_io(const void* x, const float* mix, void* const* out, int n_mix, int B, int T, int C, int Hp, int Wp,
              int shift, int g, int head_dim, int n_grid, bool vec_ok, hipStream_t st) {
    constexpr int V = 16 / sizeof(IO);                  // 16-byte accesses
    const int period = head_dim > 0 ? head_dim : C;
    if (vec_ok && C % V == 0 && g % V == 0 && period % V == 0)
        return launch<IO, V>(x, mix, out, n_mix, B, T, C, Hp, Wp, shift, g, head_dim, n_grid, st);
    return launch<IO, 1>(x, mix, out, n_mix, B, T, C, Hp, Wp, shift, g, head_dim, n_grid, st);
}

}  // namespace
}  // namespace vrwkv

using namespace vrwkv;

extern "C" int vrwkv_qshift_mix(const void* x, const float* mix, void* const* out, int n_mix,
                                int B, int T, int C, int Hp, int Wp, int shift_pixel, int quarter_width,
                                int head_dim, int io_dtype, void* hip_stream) {
    if (B <= 0 || T <= 0 || C <= 0 || Hp <= 0 || Wp <= 0 || n_mix < 1 || n_mix > 3 || shift_pixel < 0) {
        set_error("qshift_mix: bad sizes (B=%d T=%d C=%d Hp=%d Wp=%d n_mix=%d shift=%d)", B, T, C, Hp, Wp, n_mix, shift_pixel);
        return VRWKV_INVALID_ARG;
    }
    const int n_grid = Hp * Wp;
    if (n_grid != T && n_grid != T - 1) {               // at most one trailing class token
        set_error("qshift_mix: Hp*Wp must be T or T-1 (got %d*%d, T=%d)", Hp, Wp, T);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (quarter_width < 0 || head_dim < 0 || (head_dim > 0 && (C % head_dim || 4 * quarter_width > head_dim)) ||
        (head_dim == 0 && 4 * (long long)quarter_width > C)) {
        set_error("qshift_mix: quarter_width=%d does not fit (C=%d, head_dim=%d)", quarter_width, C, head_dim);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (T > 65535 || B > 65535) {
        set_error("qshift_mix: B and T must be <= 65535");
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("qshift_mix: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (!x || !mix || !out) {
        set_error("qshift_mix: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    uintptr_t bits = (uintptr_t)x;
    for (int m = 0; m < n_mix; ++m) {
        if (!out[m]) { set_error("qshift_mix: null output pointer %d", m); return VRWKV_INVALID_ARG; }
        bits |= (uintptr_t)out[m];
    }
    const bool vec_ok = (bits & 15) == 0;
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    switch (io_dtype) {
        case VRWKV_F32:  return launch_io<float>(x, mix, out, n_mix, B, T, C, Hp, Wp, shift_pixel, quarter_width, head_dim, n_grid, vec_ok, st);
        case VRWKV_BF16: return launch_io<__hip_bfloat16>(x, mix, out, n_mix, B, T, C, Hp, Wp, shift_pixel, quarter_width, head_dim, n_grid, vec_ok, st);
        case VRWKV_F16:  return launch_io<__half>(x, mix, out, n_mix, B, T, C, Hp, Wp, shift_pixel, quarter_width, head_dim, n_grid, vec_ok, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
