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
//
// Backward (the reference differentiates the PyTorch ops by autograd): with g_m the gradient of out_m,
//   gx[b,t,c]  = sum_m g_m[b,t,c] mix_m[c]  +  sum_m g_m[b,t',c] (1 - mix_m[c])     t' = the token that reads t
//   gmix_m[c]  = sum_{b,t} g_m[b,t,c] (x[b,t,c] - xx[b,t,c])
// (t' is one step right / left / down / up of t, none at the border; pass-through channels and a trailing class
// token read themselves).  One kernel writes gx and per-(batch, token-chunk) partial sums of gmix, which
// batch_sum_kernel then adds in a fixed order.
#include "vrwkv_common.h"

namespace vrwkv {
namespace {

// Workgroups are dealt round-robin to the 8 XCDs, each with an L2 of its own.  A token's neighbour rows belong to the
// next token chunk of the same image, so the launch is one-dimensional and XCD x takes a contiguous eighth of the
// (channel block, token chunk, image) grid: an image's chunks then share an L2 and the neighbour reads hit in it.
struct Block3 { int x, y, z; };
__device__ __forceinline__ Block3 xcd_block(int gx, int gy, int gz) {
    const int total = gx * gy * gz, id = blockIdx.x;
    const int per = total / 8;
    const int v = (total % 8 == 0) ? (id % 8) * per + id / 8 : id;
    return Block3{v % gx, (v / gx) % gy, v / (gx * gy)};
}

constexpr int QF_CX = 32, QF_TY = 8;   // forward workgroup: 32 channel vectors x 8 token lanes
constexpr int QF_TPT = 4;              // tokens per thread: a workgroup covers up to 32 tokens of 32 channel vectors

// A thread keeps one channel vector's mix values in registers and walks QF_TPT tokens with them; the loads of all its
// tokens (the token itself and the neighbour its channel group points at) are issued before the first value is used.
// x is read with the default cache policy (every row is read again as somebody's neighbour), the outputs are streamed.
template <typename IO, int VEC, int NMIX>
__global__ __launch_bounds__(QF_CX * QF_TY)
void qshift_mix_kernel(const IO* __restrict__ x_, const float* __restrict__ mix_, IO* __restrict__ o0, IO* __restrict__ o1,
                       IO* __restrict__ o2, int T, int C, int Hp, int Wp, int shift, int g, int head_dim, int n_grid_tokens,
                       int tokens_per_wg, int gx, int gy, int gz)
{
    const Block3 blk = xcd_block(gx, gy, gz);
    const int cx = threadIdx.x % QF_CX, ty = threadIdx.x / QF_CX;
    const int c = (blk.x * QF_CX + cx) * VEC;
    if (c >= C) return;                                        // no barrier below
    const int b = blk.z;
    const int t_begin = blk.y * tokens_per_wg, t_end = min(T, t_begin + tokens_per_wg);
    // direction of this channel vector (the host guarantees a vector never straddles a group boundary)
    const int cq = head_dim > 0 ? c % head_dim : c;
    const int dir = (g > 0 && cq < 4 * g) ? cq / g : 4;
    float mu[NMIX][VEC];
#pragma unroll
    for (int m = 0; m < NMIX; ++m)
#pragma unroll
        for (int e = 0; e < VEC; ++e) mu[m][e] = mix_[(size_t)m * C + c + e];
    const size_t slab = (size_t)b * T * C + c;
    float xs[QF_TPT][VEC], xx[QF_TPT][VEC];
    bool have[QF_TPT];
#pragma unroll
    for (int i = 0; i < QF_TPT; ++i) {
        const int t = t_begin + ty + QF_TY * i;
        have[i] = false;
        if (t >= t_end) continue;
        int ts = t;
        have[i] = true;
        if (t < n_grid_tokens && dir < 4) {                    // a trailing class token and channels >= 4g pass through
            const int yy = t / Wp, xc = t % Wp;
            int sy = yy, sx = xc;
            if (dir == 0) sx = xc - shift; else if (dir == 1) sx = xc + shift;
            else if (dir == 2) sy = yy - shift; else sy = yy + shift;
            have[i] = sx >= 0 && sx < Wp && sy >= 0 && sy < Hp;
            ts = have[i] ? sy * Wp + sx : t;                   // outside the grid: read the token itself, masked below
        }
        load_vec<IO, VEC>(x_ + slab + (size_t)t * C, xs[i]);
        load_vec<IO, VEC>(x_ + slab + (size_t)ts * C, xx[i]);
    }
    IO* outs[3] = {o0, o1, o2};
#pragma unroll
    for (int i = 0; i < QF_TPT; ++i) {
        const int t = t_begin + ty + QF_TY * i;
        if (t >= t_end) continue;
#pragma unroll
        for (int e = 0; e < VEC; ++e) xx[i][e] = have[i] ? xx[i][e] : 0.f;      // zero fill outside the grid
#pragma unroll
        for (int m = 0; m < NMIX; ++m) {
            float r[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = xs[i][e] * mu[m][e] + xx[i][e] * (1.f - mu[m][e]);
            if constexpr (sizeof(IO) * VEC == 16) store_vec_nt<IO, VEC>(outs[m] + slab + (size_t)t * C, r);
            else store_vec<IO, VEC>(outs[m] + slab + (size_t)t * C, r);
        }
    }
}

constexpr int QS_TOK = 2;              // tokens a thread has in flight (three or four measure the same)
constexpr int QS_CX = 32, QS_TY = 8;   // backward workgroup: 32 channel vectors x 8 token lanes
constexpr int QS_TCH = 32;             // fewest tokens per workgroup (the workspace holds one partial gmix row per 32 tokens)
constexpr int QS_TARGET_WG = 896;      // workgroups per launch the token chunks are sized for: one round on 256 compute units

// direction of a channel vector and the token offsets of its source (forward) / destination (backward)
__device__ __forceinline__ int qs_dir(int c, int g, int head_dim) {
    const int cq = head_dim > 0 ? c % head_dim : c;
    return (g > 0 && cq < 4 * g) ? cq / g : 4;
}
// token that the forward reads for (t, dir): -1 = zero fill, t itself for pass-through
__device__ __forceinline__ int qs_src(int t, int dir, int Hp, int Wp, int shift, int n_grid) {
    if (t >= n_grid || dir == 4) return t;
    const int yy = t / Wp, xc = t % Wp;
    int sy = yy, sx = xc;
    if (dir == 0) sx = xc - shift; else if (dir == 1) sx = xc + shift;
    else if (dir == 2) sy = yy - shift; else sy = yy + shift;
    return (sx >= 0 && sx < Wp && sy >= 0 && sy < Hp) ? sy * Wp + sx : -1;
}
// token whose forward value was read from (t, dir): the opposite step
__device__ __forceinline__ int qs_dst(int t, int dir, int Hp, int Wp, int shift, int n_grid) {
    if (t >= n_grid || dir == 4) return t;
    const int yy = t / Wp, xc = t % Wp;
    int sy = yy, sx = xc;
    if (dir == 0) sx = xc + shift; else if (dir == 1) sx = xc - shift;
    else if (dir == 2) sy = yy + shift; else sy = yy - shift;
    return (sx >= 0 && sx < Wp && sy >= 0 && sy < Hp) ? sy * Wp + sx : -1;
}

template <typename IO, int VEC, int NMIX>
__global__ __launch_bounds__(QS_CX * QS_TY)
void qshift_mix_bwd_kernel(const IO* __restrict__ x_, const float* __restrict__ mix_, const IO* __restrict__ g0,
                           const IO* __restrict__ g1, const IO* __restrict__ g2, IO* __restrict__ gx_,
                           float* __restrict__ gmix_part, int T, int C, int Hp, int Wp, int shift, int g, int head_dim,
                           int n_grid_tokens, int n_tchunk, int gx, int gz)
{
    __shared__ float s_acc[QS_TY][NMIX][QS_CX * VEC];
    const Block3 blk = xcd_block(gx, n_tchunk, gz);
    const int cx = threadIdx.x % QS_CX, ty = threadIdx.x / QS_CX;
    const int cv = blk.x * QS_CX + cx;
    const int c = cv * VEC;
    const bool cok = c < C;
    const int tc = blk.y, b = blk.z;
    const int dir = qs_dir(cok ? c : 0, g, head_dim);
    const IO* gs[3] = {g0, g1, g2};
    float mu[NMIX][VEC], acc[NMIX][VEC];
#pragma unroll
    for (int m = 0; m < NMIX; ++m)
#pragma unroll
        for (int e = 0; e < VEC; ++e) { mu[m][e] = cok ? mix_[(size_t)m * C + c + e] : 0.f; acc[m][e] = 0.f; }
    const size_t slab = (size_t)b * T * C + c;
    // the chunk's tokens, evened out over the chunks (196 tokens in two chunks: 98 each); a thread takes every eighth,
    // two at a time: the loads of a pair are issued before the first value is used and wait packed
    const int tch = (T + n_tchunk - 1) / n_tchunk;
    const int t_begin = tc * tch, t_end = min(T, t_begin + tch);
    using Packed = typename RawVec<sizeof(IO) * VEC>::type;
    if (cok) {
        for (int t0 = t_begin + ty; t0 < t_end; t0 += QS_TOK * QS_TY) {
            Packed pxs[QS_TOK], pgt[QS_TOK][NMIX], pgd[QS_TOK][NMIX];
            float keep_d[QS_TOK];
            int tt[QS_TOK];
#pragma unroll
            for (int j = 0; j < QS_TOK; ++j) {
                const int t = t0 + QS_TY * j;
                tt[j] = t < t_end ? t : -1;
                const int tl = t < t_end ? t : t_begin;          // a token past the chunk: load a valid one, use nothing
                const int td = qs_dst(tl, dir, Hp, Wp, shift, n_grid_tokens);
                // a neighbour outside the grid is read from the token itself and masked: no divergent branches
                keep_d[j] = td >= 0 ? 1.f : 0.f;
                pxs[j] = load_packed<IO, VEC>(x_ + slab + (size_t)tl * C);
#pragma unroll
                for (int m = 0; m < NMIX; ++m) {
                    pgt[j][m] = load_packed<IO, VEC>(gs[m] + slab + (size_t)tl * C);
                    pgd[j][m] = load_packed<IO, VEC>(gs[m] + slab + (size_t)(td >= 0 ? td : tl) * C);
                }
            }
#pragma unroll
            for (int j = 0; j < QS_TOK; ++j) {
                if (tt[j] < 0) continue;
                float xs[VEC], gx[VEC];
                widen_packed<IO, VEC>(pxs[j], xs);
#pragma unroll
                for (int e = 0; e < VEC; ++e) gx[e] = 0.f;
#pragma unroll
                for (int m = 0; m < NMIX; ++m) {
                    float gt[VEC], gd[VEC];
                    widen_packed<IO, VEC>(pgt[j][m], gt);
                    widen_packed<IO, VEC>(pgd[j][m], gd);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        // out_m[t] = x[t] mu + x[src(t)] (1 - mu):  x[t] reaches out_m[t] with weight mu and out_m[dst(t)]
                        // with weight 1 - mu, so with D = g_m[dst(t)] (0 outside the grid)
                        //   gx[t] += D + (g_m[t] - D) mu,   gmix_m += x[t] (g_m[t] - D)
                        // (the second one is the sum over t of g_m[t] (x[t] - x[src(t)]) re-indexed by the source token)
                        const float D = keep_d[j] * gd[e];
                        const float diff = gt[e] - D;
                        gx[e] += fmaf(diff, mu[m][e], D);
                        acc[m][e] = fmaf(xs[e], diff, acc[m][e]);
                    }
                }
                if constexpr (sizeof(IO) * VEC == 16) store_vec_nt<IO, VEC>(gx_ + slab + (size_t)tt[j] * C, gx);
                else store_vec<IO, VEC>(gx_ + slab + (size_t)tt[j] * C, gx);
            }
        }
    }
    // the eight token lanes' sums of a column are added in a fixed order and written as one partial row
#pragma unroll
    for (int m = 0; m < NMIX; ++m)
#pragma unroll
        for (int e = 0; e < VEC; ++e) s_acc[ty][m][cx * VEC + e] = acc[m][e];
    __syncthreads();
    float* part = gmix_part + ((size_t)b * n_tchunk + tc) * NMIX * C;
    for (int o = threadIdx.x; o < NMIX * QS_CX * VEC; o += QS_CX * QS_TY) {
        const int m = o / (QS_CX * VEC), col = o % (QS_CX * VEC);
        const int cg = blk.x * QS_CX * VEC + col;
        if (cg >= C) continue;
        float sum = 0.f;
#pragma unroll
        for (int y = 0; y < QS_TY; ++y) sum += s_acc[y][m][col];
        part[(size_t)m * C + cg] = sum;
    }
}

template <typename IO, int VEC>
int launch_bwd(const void* x, const float* mix, const void* const* gout, void* gx, float* gmix, float* part, int n_mix,
               int B, int T, int C, int Hp, int Wp, int shift, int g, int head_dim, int n_grid, hipStream_t st) {
    const int ncv = C / VEC;
    const dim3 block(QS_CX * QS_TY);
    const int gbx = (ncv + QS_CX - 1) / QS_CX;
    // Token chunks: as many as give about QS_TARGET_WG workgroups (one round of long-lived workgroups: measured at
    // 64 x 196 x 768 bf16, three mixes, 40 us with 32-token chunks, 30 us with two chunks of 98), at most one per 32
    // tokens (the workspace's row count), at least one.
    const int max_tchunk = (T + QS_TCH - 1) / QS_TCH;
    int n_tchunk = (int)((QS_TARGET_WG + (long long)gbx * B / 2) / ((long long)gbx * B));
    n_tchunk = n_tchunk < 1 ? 1 : n_tchunk > max_tchunk ? max_tchunk : n_tchunk;
    if ((long long)gbx * n_tchunk * B > 0x7fffffffLL) {
        set_error("qshift_mix_bwd: too many workgroups (%d x %d x %d)", gbx, n_tchunk, B);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const dim3 grid((unsigned)gbx * n_tchunk * B);
    const IO* xx = static_cast<const IO*>(x);
    const IO* g0 = static_cast<const IO*>(gout[0]);
    const IO* g1 = n_mix > 1 ? static_cast<const IO*>(gout[1]) : nullptr;
    const IO* g2 = n_mix > 2 ? static_cast<const IO*>(gout[2]) : nullptr;
    IO* pgx = static_cast<IO*>(gx);
    switch (n_mix) {
        case 1: hipLaunchKernelGGL((qshift_mix_bwd_kernel<IO, VEC, 1>), grid, block, 0, st, xx, mix, g0, g1, g2, pgx, part, T, C, Hp, Wp, shift, g, head_dim, n_grid, n_tchunk, gbx, B); break;
        case 2: hipLaunchKernelGGL((qshift_mix_bwd_kernel<IO, VEC, 2>), grid, block, 0, st, xx, mix, g0, g1, g2, pgx, part, T, C, Hp, Wp, shift, g, head_dim, n_grid, n_tchunk, gbx, B); break;
        case 3: hipLaunchKernelGGL((qshift_mix_bwd_kernel<IO, VEC, 3>), grid, block, 0, st, xx, mix, g0, g1, g2, pgx, part, T, C, Hp, Wp, shift, g, head_dim, n_grid, n_tchunk, gbx, B); break;
    }
    // gmix[m][c] = sum over the B * n_tchunk partial rows: the rows are (n_mix * C) wide
    const int wide = n_mix * C;
    hipLaunchKernelGGL(batch_sum_kernel, dim3((wide + BATCH_SUM_COLS - 1) / BATCH_SUM_COLS), dim3(BATCH_SUM_THREADS), 0, st, part, gmix, (const float*)nullptr,
                       (float*)nullptr, B * n_tchunk, wide);
    return check_launch("qshift_mix_bwd");
}

template <typename IO>
int launch_bwd_io(const void* x, const float* mix, const void* const* gout, void* gx, float* gmix, float* part, int n_mix,
                  int B, int T, int C, int Hp, int Wp, int shift, int g, int head_dim, int n_grid, bool vec_ok, hipStream_t st) {
    // four channels per thread: 16-byte accesses of fp32, 8-byte ones of 16-bit elements (eight channels per thread
    // cost 153 registers with three mixes, three waves per SIMD: measured 10-13 % slower)
    constexpr int V = 4;
    const int period = head_dim > 0 ? head_dim : C;
    if (vec_ok && C % V == 0 && g % V == 0 && period % V == 0)
        return launch_bwd<IO, V>(x, mix, gout, gx, gmix, part, n_mix, B, T, C, Hp, Wp, shift, g, head_dim, n_grid, st);
    return launch_bwd<IO, 1>(x, mix, gout, gx, gmix, part, n_mix, B, T, C, Hp, Wp, shift, g, head_dim, n_grid, st);
}

template <typename IO, int VEC>
int launch(const void* x, const float* mix, void* const* out, int n_mix, int B, int T, int C, int Hp, int Wp,
           int shift, int g, int head_dim, int n_grid, hipStream_t st) {
    const int ncv = C / VEC;
    // token chunks of at most QF_TY * QF_TPT tokens, evened out (196 tokens: seven chunks of 28)
    const int n_tchunk = (T + QF_TY * QF_TPT - 1) / (QF_TY * QF_TPT);
    const int tpw = (T + n_tchunk - 1) / n_tchunk;
    const dim3 block(QF_CX * QF_TY);
    const int gx = (ncv + QF_CX - 1) / QF_CX;
    if ((long long)gx * n_tchunk * B > 0x7fffffffLL) {
        set_error("qshift_mix: too many workgroups (%d x %d x %d)", gx, n_tchunk, B);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    const dim3 grid((unsigned)gx * n_tchunk * B);
    const IO* xx = static_cast<const IO*>(x);
    IO* o0 = static_cast<IO*>(out[0]);
    IO* o1 = n_mix > 1 ? static_cast<IO*>(out[1]) : nullptr;
    IO* o2 = n_mix > 2 ? static_cast<IO*>(out[2]) : nullptr;
    switch (n_mix) {
        case 1: hipLaunchKernelGGL((qshift_mix_kernel<IO, VEC, 1>), grid, block, 0, st, xx, mix, o0, o1, o2, T, C, Hp, Wp, shift, g, head_dim, n_grid, tpw, gx, n_tchunk, B); break;
        case 2: hipLaunchKernelGGL((qshift_mix_kernel<IO, VEC, 2>), grid, block, 0, st, xx, mix, o0, o1, o2, T, C, Hp, Wp, shift, g, head_dim, n_grid, tpw, gx, n_tchunk, B); break;
        case 3: hipLaunchKernelGGL((qshift_mix_kernel<IO, VEC, 3>), grid, block, 0, st, xx, mix, o0, o1, o2, T, C, Hp, Wp, shift, g, head_dim, n_grid, tpw, gx, n_tchunk, B); break;
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

extern "C" size_t vrwkv_qshift_mix_bwd_workspace_bytes(int n_mix, int B, int T, int C) {
    if (n_mix < 1 || n_mix > 3 || B <= 0 || T <= 0 || C <= 0) return 0;
    return (size_t)B * ((T + QS_TCH - 1) / QS_TCH) * n_mix * C * sizeof(float);
}

extern "C" int vrwkv_qshift_mix_bwd(const void* x, const float* mix, const void* const* gout, int n_mix,
                                    void* gx, float* gmix, int B, int T, int C, int Hp, int Wp, int shift_pixel,
                                    int quarter_width, int head_dim, int io_dtype,
                                    void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (B <= 0 || T <= 0 || C <= 0 || Hp <= 0 || Wp <= 0 || n_mix < 1 || n_mix > 3 || shift_pixel < 0) {
        set_error("qshift_mix_bwd: bad sizes (B=%d T=%d C=%d Hp=%d Wp=%d n_mix=%d shift=%d)", B, T, C, Hp, Wp, n_mix, shift_pixel);
        return VRWKV_INVALID_ARG;
    }
    const int n_grid = Hp * Wp;
    if (n_grid != T && n_grid != T - 1) {
        set_error("qshift_mix_bwd: Hp*Wp must be T or T-1 (got %d*%d, T=%d)", Hp, Wp, T);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (quarter_width < 0 || head_dim < 0 || (head_dim > 0 && (C % head_dim || 4 * quarter_width > head_dim)) ||
        (head_dim == 0 && 4 * (long long)quarter_width > C)) {
        set_error("qshift_mix_bwd: quarter_width=%d does not fit (C=%d, head_dim=%d)", quarter_width, C, head_dim);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (T > 65535 * QS_TCH || B > 65535) {
        set_error("qshift_mix_bwd: B must be <= 65535 and T <= %d", 65535 * QS_TCH);
        return VRWKV_UNSUPPORTED_SHAPE;
    }
    if (io_dtype != VRWKV_F32 && io_dtype != VRWKV_BF16 && io_dtype != VRWKV_F16) {
        set_error("qshift_mix_bwd: unsupported io_dtype code %d", io_dtype);
        return VRWKV_UNSUPPORTED_DTYPE;
    }
    if (!x || !mix || !gout || !gx || !gmix) {
        set_error("qshift_mix_bwd: null pointer argument");
        return VRWKV_INVALID_ARG;
    }
    uintptr_t bits = (uintptr_t)x | (uintptr_t)gx;
    for (int m = 0; m < n_mix; ++m) {
        if (!gout[m]) { set_error("qshift_mix_bwd: null gradient pointer %d", m); return VRWKV_INVALID_ARG; }
        bits |= (uintptr_t)gout[m];
    }
    const size_t need = vrwkv_qshift_mix_bwd_workspace_bytes(n_mix, B, T, C);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 3)) {
        set_error("qshift_mix_bwd: a 4-byte aligned workspace of %zu bytes is required", need);
        return VRWKV_WORKSPACE_TOO_SMALL;
    }
    const bool vec_ok = (bits & 15) == 0;
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    float* part = static_cast<float*>(workspace);
    switch (io_dtype) {
        case VRWKV_F32:  return launch_bwd_io<float>(x, mix, gout, gx, gmix, part, n_mix, B, T, C, Hp, Wp, shift_pixel, quarter_width, head_dim, n_grid, vec_ok, st);
        case VRWKV_BF16: return launch_bwd_io<__hip_bfloat16>(x, mix, gout, gx, gmix, part, n_mix, B, T, C, Hp, Wp, shift_pixel, quarter_width, head_dim, n_grid, vec_ok, st);
        case VRWKV_F16:  return launch_bwd_io<__half>(x, mix, gout, gx, gmix, part, n_mix, B, T, C, Hp, Wp, shift_pixel, quarter_width, head_dim, n_grid, vec_ok, st);
    }
    return VRWKV_UNSUPPORTED_DTYPE;
}
