/* libvrwkv_hip.so -- C ABI of the MI355X (gfx950) WKV operators for Vision-RWKV.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its kernels on the
 * HIP stream it is given (NULL = the default stream), returns without waiting for them,
 * and never allocates or frees device memory: the caller owns every buffer, including
 * the workspace whose size the *_workspace_bytes functions report.  No exception crosses
 * this boundary; a non-zero status comes with a message in vrwkv_last_error().
 *
 * Layouts are the reference's: k, v, y, r, w_raw, gy, g* are (B,T,C) with C fastest and
 * fully contiguous; per-channel parameters are (C,) -- for wkv6, u is (H,N) = (C,) -- fp32.
 */
#ifndef VRWKV_HIP_H
#define VRWKV_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  Replaces TORCH_CHECK / assert at
 * classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:6-8,
 * .../cuda_new/bi_wkv_kernel.cu:382-384 and .../cuda_v6/wkv6_cuda.cu:350-351. */
enum {
    VRWKV_OK = 0,
    VRWKV_INVALID_ARG = 1,        /* null pointer, non-positive size, misaligned pointer */
    VRWKV_UNSUPPORTED_DTYPE = 2,
    VRWKV_UNSUPPORTED_SHAPE = 3,  /* e.g. C != H*64 for wkv6 */
    VRWKV_LAUNCH_FAILED = 4,      /* hipGetLastError() after a launch */
    VRWKV_WORKSPACE_TOO_SMALL = 5
};

/* Element type of the (B,T,C) tensors. */
enum { VRWKV_F32 = 0, VRWKV_BF16 = 1, VRWKV_F16 = 2 };

int vrwkv_version(void);                 /* major*10000 + minor*100 + patch */
const char* vrwkv_last_error(void);      /* thread-local, never NULL */

/* Tuning / testing switches, process-wide (no counterpart in the reference).  Names: "biwkv_l", "biwkv_s",
 * "biwkv_grid", "biwkv_no_stage", "biwkv_no_resident", "biwkv_bwd_serial", "wkv6_fwd_scalar", "wkv6_bwd_scalar",
 * "wkv6_bwd_unfused"; 0 = default behaviour.  The initial value of <name> is that of the environment variable
 * VRWKV_<NAME> when the library first looks at any switch; the entry points never read the environment afterwards.
 * vrwkv_set_option rejects (VRWKV_INVALID_ARG) a value the plans would ignore: biwkv_l takes 0, 4, 8, 16, 25, 28 (tokens
 * per wave), biwkv_s 0 or 2..8 (waves per workgroup), biwkv_grid 0 or a positive workgroup count, the others 0 or 1. */
int vrwkv_set_option(const char* name, int value);
int vrwkv_get_option(const char* name, int* value);

/* ---- Bi-WKV forward -------------------------------------------------------------------
 * Replaces bi_wkv_forward(w,u,k,v) -> y
 *   (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:23-33,
 *    launcher .../cuda_new/bi_wkv_kernel.cu:370-399) and the legacy
 *   forward(B,T,C,w,u,k,v,y) (.../backbones/cuda/wkv_op.cpp:6-8).
 * w, u: (C,) fp32 (already divided by T by the caller, vrwkv.py:183).
 * k, v, y: (B,T,C) of io_dtype; state and arithmetic are fp32.  No T_MAX and no
 * C >= 32 / B*C % 32 restriction; T*C must stay below 2^29 elements.
 * workspace: needed only for long sequences (see vrwkv_biwkv_fwd_workspace_bytes, which
 * returns 0 when none is); may be NULL when that size is 0. */
size_t vrwkv_biwkv_fwd_workspace_bytes(int B, int T, int C, int io_dtype);
int vrwkv_biwkv_fwd(const float* w, const float* u, const void* k, const void* v, void* y,
                    int B, int T, int C, int io_dtype,
                    void* workspace, size_t workspace_bytes, void* hip_stream);

/* Bi-WKV forward with the receptance gate applied before y is stored: y = sigmoid(r) * wkv(w, u, k, v), i.e. the
 * operator plus the step that follows it in VRWKV_SpatialMix.forward when key_norm is off
 * (classification/mmcls_custom/models/backbones/vrwkv.py:183-186: rwkv = RUN_CUDA(...); rwkv = sr * rwkv).  The
 * reference has no such entry (it runs the gate as PyTorch ops on the stored y); this one saves writing y and reading
 * it back.  r: (B,T,C) of the dtype of k, v; every other argument as vrwkv_biwkv_fwd (same workspace).  The gate runs
 * inside the emitting kernel for 16-byte aligned k, v, y with C a multiple of 16 bytes of elements, on the one-launch
 * path (T <= 224) and, for 16-bit rows, the two-launch path; other calls (unaligned rows, fp32 sequences beyond 224
 * tokens, 16-bit sequences of 225..672 tokens, which a kernel without the gate serves) run vrwkv_biwkv_fwd and then
 * gate y in place -- same result, smaller saving.  Forward only. */
int vrwkv_biwkv_fwd_gate(const float* w, const float* u, const void* k, const void* v, const void* r, void* y,
                         int B, int T, int C, int io_dtype,
                         void* workspace, size_t workspace_bytes, void* hip_stream);

/* Bi-WKV forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as vrwkv_biwkv_fwd,
 * but the long-sequence workspace is an array built into the library (4 MiB of device memory per GPU, held until the
 * process ends) and the call allocates nothing.  Shapes whose workspace (vrwkv_biwkv_fwd_workspace_bytes) exceeds
 * vrwkv_biwkv_fwd_static_max_workspace_bytes() are rejected with VRWKV_WORKSPACE_TOO_SMALL.  All calls on one GPU
 * share that array: calls that may overlap on a GPU (different streams or threads) race; use vrwkv_biwkv_fwd with
 * separate workspaces for those.  The first call on a device looks up the array's device address (hipGetSymbolAddress,
 * which may load the code object): make it outside a stream capture; every later call only launches kernels. */
size_t vrwkv_biwkv_fwd_static_max_workspace_bytes(void);
int vrwkv_biwkv_fwd_static(const float* w, const float* u, const void* k, const void* v, void* y,
                           int B, int T, int C, int io_dtype, void* hip_stream);

/* ---- Bi-WKV backward ------------------------------------------------------------------
 * Replaces bi_wkv_backward(w,u,k,v,gy) -> [gw,gu,gk,gv]
 *   (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:35-47, launcher
 *    .../cuda_new/bi_wkv_kernel.cu:401-443, kernel :119-367) and the legacy
 *   backward(B,T,C,w,u,k,v,gy,gw,gu,gk,gv) (.../backbones/cuda/wkv_op.cpp:9-11).
 * w, u, gw, gu: (C,) fp32, gw and gu already summed over batch and tokens (fully overwritten,
 * no need to zero them); k, v, gy, gk, gv: (B,T,C) of io_dtype.  The workspace (always needed)
 * replaces the three scratch tensors the reference allocates (bi_wkv_kernel.cu:415-417). */
size_t vrwkv_biwkv_bwd_workspace_bytes(int B, int T, int C, int io_dtype);
int vrwkv_biwkv_bwd(const float* w, const float* u, const void* k, const void* v, const void* gy,
                    float* gw, float* gu, void* gk, void* gv, int B, int T, int C, int io_dtype,
                    void* workspace, size_t workspace_bytes, void* hip_stream);

/* ---- wkv6 forward (bidirectional RWKV-6 scan) -----------------------------------------
 * Replaces forward(B,T,C,H,r,k,v,w,u,y)
 *   (classification/mmcls_custom/models/backbones/cuda_v6/wkv6_op.cpp:7-9, launcher
 *    .../cuda_v6/wkv6_cuda.cu:348-353, kernel :6-97).
 * r, k, v: (B,T,C) of rkv_dtype; w: (B,T,C) of w_dtype (fp32, or the dtype of r, k, v);
 * u: (H,64) fp32; y: (B,T,C) fp32, caller-allocated, fully overwritten.  C must be H*64.
 * w_is_ew = 0: w is the raw decay logit and the kernel uses d = exp(-exp(w)), i.e. it folds in
 *              the `ew = -exp(w)` of WKV_6.forward (vrwkv6.py:48);
 * w_is_ew = 1: w already holds ew = -exp(w_raw), as the reference extension receives it.
 * State and accumulation are fp32.  No limit on T (T*C < 2^29).  No workspace is needed: the size
 * function returns 0 and workspace may be NULL (both kept so that every operator has the same shape). */
size_t vrwkv_wkv6_fwd_workspace_bytes(int B, int T, int C, int H);
int vrwkv_wkv6_fwd(const void* r, const void* k, const void* v, const void* w, const float* u,
                   float* y, int B, int T, int C, int H, int rkv_dtype, int w_dtype, int w_is_ew,
                   void* workspace, size_t workspace_bytes, void* hip_stream);

/* Profiling twin of vrwkv_wkv6_fwd (no counterpart in the reference; for benchmarks and tuning): the same kernel
 * for bf16 r, k, v and fp32 raw-logit w, with every wave storing the shader clock at the boundaries of its stages.
 * stamps: device buffer of vrwkv_wkv6_fwd_phases_bytes(B, T, H) bytes, laid out as uint64
 * [B*H][8 waves][ceil(T/32) chunk steps][8 points]: 0 element-wise stage entered, 1 its operands written (before the
 * barrier), 2 behind that barrier, 4 matrix stage entered, 5 y stored and the next decay sums formed (before the
 * barrier), 6 behind that barrier; 3 and 7 unused.  Waves 0-3 are the descending pass, 4-7 the ascending one.  y is
 * written as by vrwkv_wkv6_fwd.  Sequences whose decays fall outside the chunked kernel's range leave later steps
 * unstamped. */
size_t vrwkv_wkv6_fwd_phases_bytes(int B, int T, int H);
int vrwkv_wkv6_fwd_phases(const void* r, const void* k, const void* v, const void* w, const float* u,
                          float* y, int B, int T, int C, int H, void* stamps, size_t stamp_bytes, void* hip_stream);

/* ---- wkv6 backward ---------------------------------------------------------------------
 * Replaces backward(B,T,C,H,r,k,v,w,u,gy,gr,gk,gv,gw,gu)
 *   (classification/mmcls_custom/models/backbones/cuda_v6/wkv6_op.cpp:10-12, launcher
 *    .../cuda_v6/wkv6_cuda.cu:355-362, kernels :99-346), without its T <= 256 limit.
 * r, k, v, w, u as in vrwkv_wkv6_fwd; gy, gr, gk, gv, gw: (B,T,C) fp32, fully overwritten; gw is the
 * gradient w.r.t. the raw decay logit (wkv6_cuda.cu:248,277); gu: (H,64) fp32 already summed over
 * the batch (the reference returns (B,C) and sums in Python, vrwkv6.py:69). */
size_t vrwkv_wkv6_bwd_workspace_bytes(int B, int T, int C, int H);
int vrwkv_wkv6_bwd(const void* r, const void* k, const void* v, const void* w, const float* u,
                   const float* gy, float* gr, float* gk, float* gv, float* gw, float* gu,
                   int B, int T, int C, int H, int rkv_dtype, int w_dtype, int w_is_ew,
                   void* workspace, size_t workspace_bytes, void* hip_stream);

/* ---- fused Q-Shift + token mix (the elementwise step in front of the r/k/v projections) -----
 * Replaces q_shift (classification/mmcls_custom/models/backbones/vrwkv.py:68-79) followed by the
 * lerps x*mix_m + q_shift(x)*(1-mix_m) of VRWKV_SpatialMix.jit_func (:160-163, n_mix = 3) and
 * VRWKV_ChannelMix.forward (:248-250, n_mix = 2); with head_dim = 64 the shift is q_shift_multihead
 * (.../vrwkv6.py:75-100).  The reference has no native code for this step (pure PyTorch ops).
 * x, out[m]: (B,T,C) of io_dtype; mix: (n_mix, C) fp32; tokens row-major over the (Hp,Wp) patch
 * grid, T == Hp*Wp or Hp*Wp + 1 (one trailing class token, passed through).
 * quarter_width = int(C*gamma) (head_dim = 0) or head_dim/4 (per-head quarters). */
int vrwkv_qshift_mix(const void* x, const float* mix, void* const* out, int n_mix,
                     int B, int T, int C, int Hp, int Wp, int shift_pixel, int quarter_width,
                     int head_dim, int io_dtype, void* hip_stream);

/* Backward of vrwkv_qshift_mix (the reference differentiates its PyTorch ops by autograd; no native code):
 * gout[m]: gradients of out[m], (B,T,C) of io_dtype; gx: (B,T,C) of io_dtype; gmix: (n_mix, C) fp32, summed over
 * batch and tokens in a fixed order.  workspace: vrwkv_qshift_mix_bwd_workspace_bytes(n_mix, B, T, C) bytes. */
size_t vrwkv_qshift_mix_bwd_workspace_bytes(int n_mix, int B, int T, int C);
int vrwkv_qshift_mix_bwd(const void* x, const float* mix, const void* const* gout, int n_mix,
                         void* gx, float* gmix, int B, int T, int C, int Hp, int Wp, int shift_pixel,
                         int quarter_width, int head_dim, int io_dtype,
                         void* workspace, size_t workspace_bytes, void* hip_stream);

/* ---- fused row-wise epilogues of the blocks (the elementwise steps behind the operator and the GEMMs) ----
 * For every row of N channels:  y = LayerNorm(pre(a)) (weight, bias; LayerNorm skipped when ln_weight is NULL),
 * out = y (post 0) | sigmoid(other) * y (post 1) | other + gamma * y (post 2, gamma NULL = 1); pre 0 = identity,
 * pre 1 = relu(a)^2.  Replaces, in one pass over memory, the PyTorch-op sequences of
 * classification/mmcls_custom/models/backbones/vrwkv.py:184-186 (key_norm, sr * rwkv), :256-261 (relu^2, key_norm,
 * sigmoid gate) and :300-313 (residual with layer scale, post- or pre-norm).  The reference has no native code here.
 * a, other, out: (rows, N) of io_dtype; ln_weight, ln_bias, gamma: (N,) of io_dtype; all 16-byte aligned;
 * N a multiple of the 4 (fp32) or 8 (16-bit) elements in 16 bytes and at most 1024 such vectors. */
int vrwkv_rowfuse(const void* a, const void* other, const void* ln_weight, const void* ln_bias,
                  const void* gamma, void* out, long long rows, int N, int pre, int post, float eps,
                  int io_dtype, void* hip_stream);

/* Backward of vrwkv_rowfuse (the reference differentiates its PyTorch ops by autograd; no native code).
 * gout: gradient of out; ga: gradient of a; gother: gradient of `other` for the sigmoid gate (for the residual it is
 * gout itself and nothing is written; may be NULL then); gparam: (3, N) fp32 = gradients of ln_weight, ln_bias and
 * gamma summed over the rows in a fixed order (required when LayerNorm or gamma take part; rows unused by the call
 * are zero).  With LayerNorm or gamma N is at most 1024.  workspace: vrwkv_rowfuse_bwd_workspace_bytes(rows, N)
 * bytes, needed only when gparam is. */
size_t vrwkv_rowfuse_bwd_workspace_bytes(long long rows, int N);
int vrwkv_rowfuse_bwd(const void* a, const void* other, const void* ln_weight, const void* ln_bias,
                      const void* gamma, const void* gout, void* ga, void* gother, float* gparam,
                      long long rows, int N, int pre, int post, float eps, int io_dtype,
                      void* workspace, size_t workspace_bytes, void* hip_stream);

/* ---- element-wise steps of the VRWKV6 spatial mix (.../backbones/vrwkv6.py:176-212), one pass each ----
 * vrwkv_maa_mix: the five data-dependent token mixes of jit_func (:190-194),
 *   out[i] = x + (sx - x) * (maa[i] + m[i]),  i = w, k, v, r, g;
 *   x, sx (the shifted x), out[i]: (rows, C) of io_dtype; m: (5, rows, C) of io_dtype (the low-rank mix of :183-186);
 *   maa: (5, C) fp32 (time_maa_w, _k, _v, _r, _g).
 * vrwkv_groupnorm_gate: jit_func_2 (:205-211), out = GroupNorm(y) * silu(gate) with groups of `group` consecutive
 *   channels per row (ln_x = GroupNorm(n_head, C) on the (B*T, C) view); y: (rows, C) fp32 (as the operator returns
 *   it) or io_dtype; gate, out: (rows, C), gn_weight, gn_bias: (C,) of io_dtype (fp32, bf16 or fp16; fp32 only beside an fp32 y).
 * All tensors 16-byte aligned, C a multiple of 8 (4 for fp32 maa_mix).  The reference has no native code here. */
int vrwkv_maa_mix(const void* x, const void* sx, const void* m, const float* maa, void* const* out,
                  long long rows, int C, int io_dtype, void* hip_stream);
int vrwkv_groupnorm_gate(const void* y, const void* gate, const void* gn_weight, const void* gn_bias, void* out,
                         long long rows, int C, int group, float eps, int y_dtype, int io_dtype, void* hip_stream);

/* Backward of the two (the reference differentiates its PyTorch ops by autograd; no native code).
 * vrwkv_maa_mix_bwd: gout[i] gradients of out[i]; gx, gsx: (rows, C), gm: (5, rows, C) of io_dtype; gmaa: (5, C) fp32
 *   summed over the rows in a fixed order; workspace vrwkv_maa_mix_bwd_workspace_bytes(rows, C) bytes.
 * vrwkv_groupnorm_gate_bwd: gout gradient of out (io_dtype); gy in y's type, ggate in io_dtype; gparam: (2, C) fp32 =
 *   gradients of gn_weight and gn_bias; C at most 1024; workspace vrwkv_groupnorm_gate_bwd_workspace_bytes(rows, C). */
size_t vrwkv_maa_mix_bwd_workspace_bytes(long long rows, int C);
int vrwkv_maa_mix_bwd(const void* x, const void* sx, const void* m, const float* maa, const void* const* gout,
                      void* gx, void* gsx, void* gm, float* gmaa, long long rows, int C, int io_dtype,
                      void* workspace, size_t workspace_bytes, void* hip_stream);
size_t vrwkv_groupnorm_gate_bwd_workspace_bytes(long long rows, int C);
int vrwkv_groupnorm_gate_bwd(const void* y, const void* gate, const void* gn_weight, const void* gn_bias,
                             const void* gout, void* gy, void* ggate, float* gparam, long long rows, int C, int group,
                             float eps, int y_dtype, int io_dtype, void* workspace, size_t workspace_bytes,
                             void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* VRWKV_HIP_H */
