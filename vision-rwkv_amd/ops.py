"""Operator boundary: the reference's autograd Functions and RUN_* entry points, backed by
libvrwkv_hip.so.

Mirrors
  WKV / RUN_CUDA(w,u,k,v)                 classification/mmcls_custom/models/backbones/vrwkv.py:29-65
  legacy RUN_CUDA(B,T,C,w,u,k,v)          classification/mae/vrwkv/vrwkv.py:30-90
  WKV_6 / RUN_CUDA_RWKV6(B,T,C,H,r,k,v,w,u)  classification/mmcls_custom/models/backbones/vrwkv6.py:34-73
with the same argument meaning, output dtype rule and error behaviour (RuntimeError for
non-device / non-contiguous tensors).
"""
import ctypes

import torch

from . import _lib

_DT = {torch.float32: _lib.VRWKV_F32, torch.bfloat16: _lib.VRWKV_BF16, torch.float16: _lib.VRWKV_F16}


def _check_input(x, name):
    # CHECK_INPUT of bi_wkv.cpp:6-8
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_out(t, name, shape, dtype, like):
    """A caller-allocated result (the legacy / wkv6 extension interfaces pass them in)."""
    if not (t.is_cuda and t.is_contiguous() and t.device == like.device):
        raise RuntimeError(f"{name} must be a contiguous CUDA tensor on the inputs' device")
    if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
        raise RuntimeError(f"{name} must have shape {tuple(shape)} and dtype {dtype}")
    return t


def _stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


def bi_wkv_forward(w, u, k, v, out=None, gate=None):
    """Extension-level entry (bi_wkv.cpp:23-33): w,u (C,) fp32; k,v (B,T,C) of one dtype
    (fp32, bf16 or fp16); returns y (B,T,C) of that dtype.  State and arithmetic are fp32.
    out: a caller-allocated y (the legacy interface, wkv_op.cpp:6-8).
    gate: None, or the receptance r (B,T,C) of the same dtype: the result is sigmoid(r) * y, the step that follows the
    operator in VRWKV_SpatialMix.forward (vrwkv.py:185-186 without key_norm), applied before y is stored
    (vrwkv_biwkv_fwd_gate; forward only: it has no autograd)."""
    for t, n in ((w, "w"), (u, "u"), (k, "k"), (v, "v")) + (((gate, "gate"),) if gate is not None else ()):
        _check_input(t, n)
    if k.dim() != 3 or v.shape != k.shape or (gate is not None and (gate.shape != k.shape or gate.dtype != k.dtype)):
        raise RuntimeError("k and v (and the gate) must all be (B,T,C) of one dtype")
    B, T, C = k.shape
    if w.numel() != C or u.numel() != C:
        raise RuntimeError("w and u must have C elements")
    if w.dtype != torch.float32 or u.dtype != torch.float32:
        raise RuntimeError("w and u must be float32")
    if k.dtype not in _DT or v.dtype != k.dtype:
        raise RuntimeError("k and v must share one of float32 / bfloat16 / float16")
    L = _lib.lib()
    dt = _DT[k.dtype]
    y = torch.empty_like(k) if out is None else _check_out(out, "y", k.shape, k.dtype, k)
    if y.numel() == 0:
        return y
    ws_bytes = L.vrwkv_biwkv_fwd_workspace_bytes(B, T, C, dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=k.device) if ws_bytes else None
    with torch.cuda.device(k.device):
        tail = (B, T, C, dt, ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(k.device))
        if gate is None:
            _lib.check(L.vrwkv_biwkv_fwd(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), *tail))
        else:
            _lib.check(L.vrwkv_biwkv_fwd_gate(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), gate.data_ptr(),
                                              y.data_ptr(), *tail))
    return y


def bi_wkv_backward(w, u, k, v, gy, out=None):
    """Extension-level entry (bi_wkv.cpp:35-47): w,u (C,) fp32; k,v,gy (B,T,C) of one dtype;
    returns [gw, gu, gk, gv] with gw, gu (C,) fp32 summed over batch and tokens and gk, gv of the
    dtype of k.  out: caller-allocated (gw, gu, gk, gv)."""
    for t, n in ((w, "w"), (u, "u"), (k, "k"), (v, "v"), (gy, "gy")):
        _check_input(t, n)
    if k.dim() != 3 or v.shape != k.shape or gy.shape != k.shape:
        raise RuntimeError("k, v and gy must all be (B,T,C)")
    B, T, C = k.shape
    if w.numel() != C or u.numel() != C or w.dtype != torch.float32 or u.dtype != torch.float32:
        raise RuntimeError("w and u must be float32 with C elements")
    if k.dtype not in _DT or v.dtype != k.dtype or gy.dtype != k.dtype:
        raise RuntimeError("k, v and gy must share one of float32 / bfloat16 / float16")
    L = _lib.lib()
    dt = _DT[k.dtype]
    if out is None:
        gw = torch.empty(C, dtype=torch.float32, device=k.device)
        gu = torch.empty(C, dtype=torch.float32, device=k.device)
        gk = torch.empty_like(k)
        gv = torch.empty_like(k)
    else:
        gw, gu = (_check_out(t, n, (C,), torch.float32, k) for t, n in zip(out[:2], ("gw", "gu")))
        gk, gv = (_check_out(t, n, k.shape, k.dtype, k) for t, n in zip(out[2:], ("gk", "gv")))
    if k.numel() == 0:
        return [gw.zero_(), gu.zero_(), gk, gv]
    ws_bytes = L.vrwkv_biwkv_bwd_workspace_bytes(B, T, C, dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=k.device)
    with torch.cuda.device(k.device):
        _lib.check(L.vrwkv_biwkv_bwd(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), gy.data_ptr(),
                                     gw.data_ptr(), gu.data_ptr(), gk.data_ptr(), gv.data_ptr(),
                                     B, T, C, dt, ws.data_ptr(), ws_bytes, _stream_ptr(k.device)))
    return [gw, gu, gk, gv]


class WKV(torch.autograd.Function):
    """Bi-WKV with the reference's dtype rule: arithmetic in fp32, the result is fp32 unless
    the *parameter* w is half / bfloat16, in which case it has w's dtype (vrwkv.py:31-44).
    When k and v already arrive in that 16-bit dtype they are consumed as they are
    (no up-cast copies, no separate down-cast of y)."""

    @staticmethod
    def forward(ctx, w, u, k, v):
        out_dtype = w.dtype if w.dtype in (torch.half, torch.bfloat16) else torch.float32
        wf = w.float().contiguous()
        uf = u.float().contiguous()
        ctx.save_for_backward(wf, uf, k, v)                # the fp32 copies serve the backward too
        ctx.out_dtype = out_dtype
        if k.dtype == out_dtype and v.dtype == out_dtype:
            return bi_wkv_forward(wf, uf, k.contiguous(), v.contiguous())
        y = bi_wkv_forward(wf, uf, k.float().contiguous(), v.float().contiguous())
        return y if out_dtype == torch.float32 else y.to(out_dtype)

    @staticmethod
    def backward(ctx, gy):
        # vrwkv.py:47-61: gradients in fp32, returned in w's dtype when that is half / bfloat16
        wf, uf, k, v = ctx.saved_tensors
        out_dtype = ctx.out_dtype
        if k.dtype == out_dtype and v.dtype == out_dtype and out_dtype != torch.float32:
            gw, gu, gk, gv = bi_wkv_backward(wf, uf, k.contiguous(), v.contiguous(), gy.to(out_dtype).contiguous())
        else:
            gw, gu, gk, gv = bi_wkv_backward(wf, uf, k.float().contiguous(), v.float().contiguous(),
                                             gy.float().contiguous())
        if out_dtype == torch.float32:
            return (gw, gu, gk, gv)
        gwu = torch.stack((gw, gu)).to(out_dtype)           # one cast for both parameter gradients
        return (gwu[0], gwu[1], gk.to(out_dtype), gv.to(out_dtype))


class _WKVLegacy(torch.autograd.Function):
    """Seven-argument form used by the MAE code (classification/mae/vrwkv/vrwkv.py:30-90)."""

    @staticmethod
    def forward(ctx, B, T, C, w, u, k, v):
        if tuple(k.shape) != (B, T, C):
            raise RuntimeError(f"k has shape {tuple(k.shape)}, expected {(B, T, C)}")
        return WKV.forward(ctx, w, u, k, v)

    @staticmethod
    def backward(ctx, gy):
        return (None, None, None) + tuple(WKV.backward(ctx, gy))


def RUN_CUDA(*args):
    """RUN_CUDA(w, u, k, v) (vrwkv.py:64-65) or legacy RUN_CUDA(B, T, C, w, u, k, v)."""
    if len(args) == 4:
        w, u, k, v = args
        return WKV.apply(w.cuda(), u.cuda(), k.cuda(), v.cuda())
    if len(args) == 7:
        B, T, C, w, u, k, v = args
        return _WKVLegacy.apply(B, T, C, w.cuda(), u.cuda(), k.cuda(), v.cuda())
    raise TypeError("RUN_CUDA takes (w, u, k, v) or (B, T, C, w, u, k, v)")


HEAD_SIZE = 64   # vrwkv6.py:23


def wkv6_forward(B, T, C, H, r, k, v, w, u, w_is_ew=False, out=None):
    """Extension-level entry (wkv6_op.cpp:7-9): r,k,v (B,T,C) fp32/bf16/fp16, w (B,T,C) fp32 or
    that dtype, u (H,64); returns y (B,T,C) fp32.  With w_is_ew=False, w is the raw decay logit
    (the kernel applies d = exp(-exp(w))); with True it is ew = -exp(w_raw) as the reference
    extension receives it."""
    for t, n in ((r, "r"), (k, "k"), (v, "v"), (w, "w"), (u, "u")):
        _check_input(t, n)
    if tuple(r.shape) != (B, T, C) or k.shape != r.shape or v.shape != r.shape or w.shape != r.shape:
        raise RuntimeError("r, k, v, w must all be (B,T,C)")
    if u.numel() != C:
        raise RuntimeError("u must have H*64 = C elements")
    if r.dtype not in _DT or k.dtype != r.dtype or v.dtype != r.dtype:
        raise RuntimeError("r, k, v must share one of float32 / bfloat16 / float16")
    if w.dtype != torch.float32 and w.dtype != r.dtype:
        raise RuntimeError("w must be float32 or have the dtype of r, k, v")
    uf = u if u.dtype == torch.float32 else u.float()
    L = _lib.lib()
    y = (torch.empty((B, T, C), device=r.device, dtype=torch.float32) if out is None
         else _check_out(out, "y", (B, T, C), torch.float32, r))      # the reference passes y in (wkv6_op.cpp:7-9)
    if y.numel() == 0:
        return y
    ws_bytes = L.vrwkv_wkv6_fwd_workspace_bytes(B, T, C, H)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=r.device) if ws_bytes else None
    with torch.cuda.device(r.device):
        _lib.check(L.vrwkv_wkv6_fwd(r.data_ptr(), k.data_ptr(), v.data_ptr(), w.data_ptr(), uf.data_ptr(),
                                    y.data_ptr(), B, T, C, H, _DT[r.dtype], _DT[w.dtype], 1 if w_is_ew else 0,
                                    ws.data_ptr() if ws is not None else None, ws_bytes,
                                    _stream_ptr(r.device)))
    return y


def wkv6_backward(B, T, C, H, r, k, v, w, u, gy, w_is_ew=False, out=None):
    """Extension-level entry (wkv6_op.cpp:10-12): returns (gr, gk, gv, gw) as (B,T,C) fp32 and gu as
    (H,64) fp32 (already summed over the batch); gw is the gradient w.r.t. the raw decay logit."""
    for t, n in ((r, "r"), (k, "k"), (v, "v"), (w, "w"), (u, "u"), (gy, "gy")):
        _check_input(t, n)
    if tuple(r.shape) != (B, T, C) or any(x.shape != r.shape for x in (k, v, w, gy)):
        raise RuntimeError("r, k, v, w, gy must all be (B,T,C)")
    if r.dtype not in _DT or k.dtype != r.dtype or v.dtype != r.dtype:
        raise RuntimeError("r, k, v must share one of float32 / bfloat16 / float16")
    if w.dtype != torch.float32 and w.dtype != r.dtype:
        raise RuntimeError("w must be float32 or have the dtype of r, k, v")
    uf = u if u.dtype == torch.float32 else u.float()
    gyf = gy if gy.dtype == torch.float32 else gy.float()
    L = _lib.lib()
    if out is None:
        mk = lambda: torch.empty((B, T, C), device=r.device, dtype=torch.float32)
        gr, gk, gv, gw = mk(), mk(), mk(), mk()
        gu = torch.empty((H, C // H), device=r.device, dtype=torch.float32)
    else:                                                             # caller-allocated (gr, gk, gv, gw, gu)
        gr, gk, gv, gw = (_check_out(t, n, (B, T, C), torch.float32, r) for t, n in zip(out[:4], ("gr", "gk", "gv", "gw")))
        gu = _check_out(out[4], "gu", (H, C // H), torch.float32, r)
    if gr.numel() == 0:
        return gr, gk, gv, gw, gu.zero_()
    ws_bytes = L.vrwkv_wkv6_bwd_workspace_bytes(B, T, C, H)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=r.device)
    with torch.cuda.device(r.device):
        _lib.check(L.vrwkv_wkv6_bwd(r.data_ptr(), k.data_ptr(), v.data_ptr(), w.data_ptr(), uf.data_ptr(),
                                    gyf.data_ptr(), gr.data_ptr(), gk.data_ptr(), gv.data_ptr(), gw.data_ptr(),
                                    gu.data_ptr(), B, T, C, H, _DT[r.dtype], _DT[w.dtype], 1 if w_is_ew else 0,
                                    ws.data_ptr(), ws_bytes, _stream_ptr(r.device)))
    return gr, gk, gv, gw, gu


class WKV_6(torch.autograd.Function):
    """Bidirectional RWKV-6 scan with the reference's call contract (vrwkv6.py:34-70): contiguous
    (B,T,C) inputs, raw decay logit w, fp32 (B,T,C) result.  The `ew = -exp(w)` tensor the
    reference materialises is folded into the kernel."""

    @staticmethod
    def forward(ctx, B, T, C, H, r, k, v, w, u):
        with torch.no_grad():
            assert HEAD_SIZE == C // H
            ctx.B, ctx.T, ctx.C, ctx.H = B, T, C, H
            assert r.is_contiguous()
            assert k.is_contiguous()
            assert v.is_contiguous()
            assert w.is_contiguous()
            assert u.is_contiguous()
            ctx.save_for_backward(r, k, v, w, u)
            return wkv6_forward(B, T, C, H, r, k, v, w, u)

    @staticmethod
    def backward(ctx, gy):
        # vrwkv6.py:55-70: fp32 gradients, gu summed over the batch and shaped (H, C//H)
        with torch.no_grad():
            assert gy.is_contiguous()
            r, k, v, w, u = ctx.saved_tensors
            gr, gk, gv, gw, gu = wkv6_backward(ctx.B, ctx.T, ctx.C, ctx.H, r, k, v, w, u, gy)
            return (None, None, None, None, gr, gk, gv, gw, gu)


def RUN_CUDA_RWKV6(B, T, C, H, r, k, v, w, u):
    """vrwkv6.py:72-73."""
    return WKV_6.apply(B, T, C, H, r, k, v, w, u)


def q_shift(input, shift_pixel=1, gamma=1 / 4, patch_resolution=None):
    """q_shift of vrwkv.py:68-79 in plain tensor ops (used where gradients are needed)."""
    assert gamma <= 1 / 4
    B, N, C = input.shape
    x = input.transpose(1, 2).reshape(B, C, patch_resolution[0], patch_resolution[1])
    H, W = patch_resolution
    b1, b2, b3, b4 = _shift_bounds(C, gamma)
    out = torch.zeros_like(x)
    out[:, 0:b1, :, shift_pixel:W] = x[:, 0:b1, :, 0:W - shift_pixel]
    out[:, b1:b2, :, 0:W - shift_pixel] = x[:, b1:b2, :, shift_pixel:W]
    out[:, b2:b3, shift_pixel:H, :] = x[:, b2:b3, 0:H - shift_pixel, :]
    out[:, b3:b4, 0:H - shift_pixel, :] = x[:, b3:b4, shift_pixel:H, :]
    out[:, b4:, ...] = x[:, b4:, ...]
    return out.flatten(2).transpose(1, 2)


def _shift_bounds(C, gamma):
    """Upper ends of the four shifted channel groups exactly as the reference cuts them (vrwkv.py:72-76):
    int(C*gamma), int(C*gamma*2), int(C*gamma*3), int(C*gamma*4)."""
    return int(C * gamma), int(C * gamma * 2), int(C * gamma * 3), int(C * gamma * 4)


def _equal_quarters(C, gamma, head_dim):
    """The kernels shift four groups of one width; true when the reference's cuts are of that kind (every
    stock model: C a multiple of 4 with gamma = 1/4, or per-head quarters)."""
    if head_dim:
        return True
    b = _shift_bounds(C, gamma)
    return b == (b[0], 2 * b[0], 3 * b[0], 4 * b[0])


def stack_mixes(mixes, device):
    """The (n_mix, C) fp32 table q_shift_mix hands to the kernel; callers that apply the same mixes again and again
    may build it once and pass it as `mix_table`."""
    return torch.stack([m.detach().reshape(-1).float() for m in mixes]).contiguous().to(device)


def q_shift_mix(x, mixes, shift_pixel=1, gamma=1 / 4, patch_resolution=None, head_dim=0, mix_table=None):
    """One HIP kernel for q_shift + the token-mix lerps: returns [x*m + q_shift(x)*(1-m) for m in mixes]
    (vrwkv.py:160-163 / :248-250).  mixes: 1..3 tensors of C elements.  head_dim=64 gives the per-head
    q_shift_multihead of vrwkv6.py:75-100 (a trailing class token is passed through).  Forward only."""
    _check_input(x, "x")
    if x.dim() != 3 or x.dtype not in _DT:
        raise RuntimeError("x must be (B,T,C) float32 / bfloat16 / float16")
    B, T, C = x.shape
    Hp, Wp = patch_resolution
    if not _equal_quarters(C, gamma, head_dim):
        # unequal channel groups (C*gamma not an integer): the reference's slice copies, then the lerps
        xx = q_shift(x, shift_pixel, gamma, patch_resolution)
        tab = mix_table if mix_table is not None else stack_mixes(mixes, x.device)
        return [(x.float() * m + xx.float() * (1 - m)).to(x.dtype) for m in tab]
    mix = mix_table if mix_table is not None else stack_mixes(mixes, x.device)
    if mix.shape != (len(mixes), C) or mix.dtype != torch.float32 or not mix.is_contiguous() or mix.device != x.device:
        raise RuntimeError("mix_table must be a contiguous float32 (n_mix, C) tensor on x's device")
    if mix.shape[1] != C:
        raise RuntimeError("every mix vector must have C elements")
    outs = [torch.empty_like(x) for _ in mixes]
    if x.numel() == 0:
        return outs
    ptrs = (ctypes.c_void_p * len(outs))(*[o.data_ptr() for o in outs])
    g = head_dim // 4 if head_dim else int(C * gamma)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().vrwkv_qshift_mix(x.data_ptr(), mix.data_ptr(), ptrs, len(outs), B, T, C, Hp, Wp,
                                               shift_pixel, g, head_dim, _DT[x.dtype], _stream_ptr(x.device)))
    return outs


PRE_NONE, PRE_RELU_SQ = 0, 1
POST_NONE, POST_SIGMOID_GATE, POST_RESIDUAL = 0, 1, 2
ROW_FUSE_ENABLED = True      # set False to make row_fuse run the tensor-op sequence everywhere (for comparisons)


def _vec_ok(*tensors):
    """True when every given tensor can be read as it lies in 16-byte pieces (dense and 16-byte aligned)."""
    return all(t is None or (t.is_contiguous() and t.data_ptr() % 16 == 0) for t in tensors)


def row_fuse_tensor_ops(a, other=None, ln_weight=None, ln_bias=None, gamma=None, pre=PRE_NONE, post=POST_NONE, eps=1e-5):
    """The PyTorch-op sequence row_fuse replaces (what the reference runs: vrwkv.py:184-186, :256-261, :300-313);
    used under autograd and wherever the kernel does not apply."""
    y = torch.square(torch.relu(a)) if pre == PRE_RELU_SQ else a
    if ln_weight is not None:
        y = torch.nn.functional.layer_norm(y, (y.shape[-1],), ln_weight, ln_bias, eps)
    if post == POST_SIGMOID_GATE:
        y = torch.sigmoid(other) * y
    elif post == POST_RESIDUAL:
        y = other + (gamma * y if gamma is not None else y)
    return y


class _RowFuse(torch.autograd.Function):
    """row_fuse with a hand-written backward (vrwkv_rowfuse / vrwkv_rowfuse_bwd).  Per-channel inputs arrive in the
    dtype of `a` (the casts outside are differentiated by autograd)."""

    @staticmethod
    def forward(ctx, a, other, ln_weight, ln_bias, gamma, pre, post, eps):
        ctx.save_for_backward(a, other, ln_weight, ln_bias, gamma)
        ctx.meta = (pre, post, eps)
        return _row_fuse_launch(a, other, ln_weight, ln_bias, gamma, pre, post, eps)

    @staticmethod
    def backward(ctx, gout):
        a, other, ln_weight, ln_bias, gamma = ctx.saved_tensors
        pre, post, eps = ctx.meta
        N = a.shape[-1]
        rows = a.numel() // N
        gout = gout.to(a.dtype).contiguous()
        ga = torch.empty_like(a)
        go = torch.empty_like(a) if post == POST_SIGMOID_GATE else None
        sums = ln_weight is not None or (post == POST_RESIDUAL and gamma is not None)
        L = _lib.lib()
        gparam = ws = None
        ws_bytes = 0
        if sums:
            gparam = torch.empty(3, N, dtype=torch.float32, device=a.device)
            ws_bytes = L.vrwkv_rowfuse_bwd_workspace_bytes(rows, N)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
        ptr = lambda t: t.data_ptr() if t is not None else None
        with torch.cuda.device(a.device):
            _lib.check(L.vrwkv_rowfuse_bwd(a.data_ptr(), ptr(other), ptr(ln_weight), ptr(ln_bias), ptr(gamma),
                                           gout.data_ptr(), ga.data_ptr(), ptr(go), ptr(gparam), rows, N, pre, post,
                                           float(eps), _DT[a.dtype], ptr(ws), ws_bytes, _stream_ptr(a.device)))
        g_other = go if post == POST_SIGMOID_GATE else (gout if post == POST_RESIDUAL else None)
        gp = gparam.to(a.dtype) if sums else None            # one cast for the three parameter gradients
        g_w = gp[0] if ln_weight is not None else None
        g_b = gp[1] if ln_bias is not None else None
        g_g = gp[2] if (gamma is not None and post == POST_RESIDUAL) else None
        return ga, g_other, g_w, g_b, g_g, None, None, None


def _row_fuse_launch(a, other, ln_weight, ln_bias, gamma, pre, post, eps):
    out = torch.empty_like(a)
    N = a.shape[-1]
    ptr = lambda t: t.data_ptr() if t is not None else None
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().vrwkv_rowfuse(a.data_ptr(), ptr(other), ptr(ln_weight), ptr(ln_bias), ptr(gamma), out.data_ptr(),
                                            a.numel() // N, N, pre, post, float(eps), _DT[a.dtype], _stream_ptr(a.device)))
    return out


def row_fuse(a, other=None, ln_weight=None, ln_bias=None, gamma=None, pre=PRE_NONE, post=POST_NONE, eps=1e-5):
    """One HIP kernel per row-wise epilogue of a block: out = post(LayerNorm(pre(a))) with pre = identity / relu^2,
    LayerNorm optional, post = identity / sigmoid(other) * y / other + gamma * y; under autograd one backward kernel
    (rows of at most 1024 channels when LayerNorm or gamma take part).  Where the kernels do not apply (not on the
    GPU, row length, alignment) the tensor ops are used instead."""
    tensors = [t for t in (a, other, ln_weight, ln_bias, gamma) if t is not None]
    N = a.shape[-1]
    vec = 4 if a.dtype == torch.float32 else 8
    need_grad = torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    sums = ln_weight is not None or (post == POST_RESIDUAL and gamma is not None)
    fits = (ROW_FUSE_ENABLED and a.is_cuda and a.dtype in _DT and N % vec == 0 and N // vec <= 1024 and a.numel() > 0
            and (other is None or (other.shape == a.shape and other.dtype == a.dtype))
            and not (need_grad and sums and N > 1024))
    if not fits:
        return row_fuse_tensor_ops(a, other, ln_weight, ln_bias, gamma, pre, post, eps)
    if need_grad:
        ac = a.contiguous()
        oc = other.contiguous() if other is not None else None
        par = [p.reshape(-1).to(a.dtype).contiguous() if p is not None else None for p in (ln_weight, ln_bias, gamma)]
        if post != POST_RESIDUAL:
            par[2] = None
        if not _vec_ok(ac, oc, *par) or any(p is not None and p.numel() != N for p in par):
            return row_fuse_tensor_ops(a, other, ln_weight, ln_bias, gamma, pre, post, eps)
        return _RowFuse.apply(ac, oc, par[0], par[1], par[2], pre, post, float(eps))
    a = a.contiguous()
    other = other.contiguous() if other is not None else None
    par = [p.detach().reshape(-1).to(a.dtype).contiguous() if p is not None else None for p in (ln_weight, ln_bias, gamma)]
    if not _vec_ok(a, other, *par):
        return row_fuse_tensor_ops(a, other, ln_weight, ln_bias, gamma, pre, post, eps)
    for p in par:
        if p is not None and p.numel() != N:
            raise RuntimeError("LayerNorm weight, bias and gamma must have one element per channel")
    return _row_fuse_launch(a, other, par[0], par[1], par[2], pre, post, eps)


def maa_mix_tensor_ops(x, sx, m, maas):
    """vrwkv6.py:180, 190-194 as the reference writes them: xx = sx - x; x + xx * (maa_i + m_i)."""
    xx = sx - x
    return [x + xx * (maa + mi) for maa, mi in zip(maas, m.unbind(0))]


class _MaaMix(torch.autograd.Function):
    """maa_mix with a hand-written backward (vrwkv_maa_mix / vrwkv_maa_mix_bwd); the five vectors enter as one (5, C)
    fp32 table built by differentiable tensor ops outside."""

    @staticmethod
    def forward(ctx, x, sx, m, table):
        ctx.save_for_backward(x, sx, m, table)
        return tuple(_maa_mix_launch(x, sx, m, table))

    @staticmethod
    def backward(ctx, *gouts):
        x, sx, m, table = ctx.saved_tensors
        C = x.shape[-1]
        rows = x.numel() // C
        gs = [g.to(x.dtype).contiguous() for g in gouts]
        gx, gsx, gm = torch.empty_like(x), torch.empty_like(x), torch.empty_like(m)
        gmaa = torch.empty_like(table)
        L = _lib.lib()
        ws_bytes = L.vrwkv_maa_mix_bwd_workspace_bytes(rows, C)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
        ptrs = (ctypes.c_void_p * 5)(*[g.data_ptr() for g in gs])
        with torch.cuda.device(x.device):
            _lib.check(L.vrwkv_maa_mix_bwd(x.data_ptr(), sx.data_ptr(), m.data_ptr(), table.data_ptr(), ptrs, gx.data_ptr(),
                                           gsx.data_ptr(), gm.data_ptr(), gmaa.data_ptr(), rows, C, _DT[x.dtype],
                                           ws.data_ptr(), ws_bytes, _stream_ptr(x.device)))
        return gx, gsx, gm, gmaa


def _maa_mix_launch(x, sx, m, table):
    C = x.shape[-1]
    outs = [torch.empty_like(x) for _ in range(5)]
    ptrs = (ctypes.c_void_p * 5)(*[o.data_ptr() for o in outs])
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().vrwkv_maa_mix(x.data_ptr(), sx.data_ptr(), m.data_ptr(), table.data_ptr(), ptrs,
                                            x.numel() // C, C, _DT[x.dtype], _stream_ptr(x.device)))
    return outs


def maa_mix(x, sx, m, maas, maa_table=None):
    """The five data-dependent token mixes of VRWKV6 (vrwkv6.py:190-194) in one HIP kernel: x, sx (the shifted x):
    (B,T,C); m: (5,B,T,C); maas: the five (C,) vectors time_maa_w, _k, _v, _r, _g (or their stacked fp32 table).
    Under autograd one backward kernel; tensor ops when the kernels do not apply."""
    C = x.shape[-1]
    vec = 4 if x.dtype == torch.float32 else 8
    tensors = [x, sx, m] + list(maas)
    need_grad = torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    fits = (ROW_FUSE_ENABLED and x.is_cuda and x.dtype in _DT and C % vec == 0 and x.numel() > 0
            and sx.shape == x.shape and sx.dtype == x.dtype and m.dtype == x.dtype and tuple(m.shape) == (5,) + tuple(x.shape)
            and not (need_grad and x.numel() // C > 65535 * 32))
    if not fits:
        return maa_mix_tensor_ops(x, sx, m, maas)
    xc, sxc, mc = x.contiguous(), sx.contiguous(), m.contiguous()
    if not _vec_ok(xc, sxc, mc):
        return maa_mix_tensor_ops(x, sx, m, maas)
    if need_grad:
        table = torch.stack([a.reshape(-1).float() for a in maas])      # differentiable: the vectors' gradients flow through it
        return list(_MaaMix.apply(xc, sxc, mc, table))
    table = maa_table if maa_table is not None else stack_mixes(maas, x.device)
    if tuple(table.shape) != (5, C) or table.dtype != torch.float32 or not table.is_contiguous():
        raise RuntimeError("maa table must be a contiguous float32 (5, C) tensor")
    return _maa_mix_launch(xc, sxc, mc, table)


def groupnorm_gate_tensor_ops(y, gate, gn_weight, gn_bias, n_groups, eps=1e-5):
    """vrwkv6.py:205-211 and :199: ln_x on the (B*T, C) view, times silu(gate).  The group statistics are written out
    with mean / var instead of torch.nn.functional.group_norm: on a GPU that function's backward returns wrong weight
    and bias gradients for a 2-D input of more than 128 rows (PyTorch 2.10.0+rocm7.0, every dtype: measured against
    the sums written out in float64 and against the CPU), and this function is the path that autograd differentiates
    when the kernels do not apply.  Statistics in fp32 for 16-bit inputs, as the library computes them."""
    C = y.shape[-1]
    x = y.to(gate.dtype).reshape(-1, n_groups, C // n_groups)
    xs = x.float() if x.dtype in (torch.bfloat16, torch.float16) else x
    mean = xs.mean(-1, keepdim=True)
    var = xs.var(-1, unbiased=False, keepdim=True)
    xh = ((xs - mean) * torch.rsqrt(var + eps)).reshape(-1, C)
    yn = (xh * gn_weight + gn_bias).to(gate.dtype)
    return yn.view(gate.shape) * torch.nn.functional.silu(gate)


class _GroupNormGate(torch.autograd.Function):
    """groupnorm_gate with a hand-written backward (vrwkv_groupnorm_gate / vrwkv_groupnorm_gate_bwd)."""

    @staticmethod
    def forward(ctx, y, gate, w, b, group, eps):
        ctx.save_for_backward(y, gate, w, b)
        ctx.meta = (group, eps)
        return _groupnorm_gate_launch(y, gate, w, b, group, eps)

    @staticmethod
    def backward(ctx, gout):
        y, gate, w, b = ctx.saved_tensors
        group, eps = ctx.meta
        C = y.shape[-1]
        rows = y.numel() // C
        gout = gout.to(gate.dtype).contiguous()
        gy, gg = torch.empty_like(y), torch.empty_like(gate)
        gparam = torch.empty(2, C, dtype=torch.float32, device=y.device)
        L = _lib.lib()
        ws_bytes = L.vrwkv_groupnorm_gate_bwd_workspace_bytes(rows, C)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=y.device)
        with torch.cuda.device(y.device):
            _lib.check(L.vrwkv_groupnorm_gate_bwd(y.data_ptr(), gate.data_ptr(), w.data_ptr(), b.data_ptr(), gout.data_ptr(),
                                                  gy.data_ptr(), gg.data_ptr(), gparam.data_ptr(), rows, C, group, float(eps),
                                                  _DT[y.dtype], _DT[gate.dtype], ws.data_ptr(), ws_bytes, _stream_ptr(y.device)))
        return gy, gg, gparam[0].to(w.dtype), gparam[1].to(b.dtype), None, None


def _groupnorm_gate_launch(y, gate, w, b, group, eps):
    C = y.shape[-1]
    out = torch.empty_like(gate)
    with torch.cuda.device(y.device):
        _lib.check(_lib.lib().vrwkv_groupnorm_gate(y.data_ptr(), gate.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(),
                                                   y.numel() // C, C, group, float(eps), _DT[y.dtype], _DT[gate.dtype],
                                                   _stream_ptr(y.device)))
    return out


def groupnorm_gate(y, gate, gn_weight, gn_bias, n_groups, eps=1e-5):
    """GroupNorm(n_groups, C) of every token of y (fp32 as RUN_CUDA_RWKV6 returns it, or gate's dtype) times
    silu(gate), in one HIP kernel (vrwkv6.py:199, 205-211), and one backward kernel under autograd (C <= 1024);
    tensor ops for other shapes."""
    C = y.shape[-1]
    group = C // n_groups if n_groups > 0 and C % n_groups == 0 else 0
    tensors = [y, gate, gn_weight, gn_bias]
    need_grad = torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    fits = (ROW_FUSE_ENABLED and y.is_cuda and gate.dtype in (torch.float32, torch.bfloat16, torch.float16) and y.shape == gate.shape
            and y.dtype in (torch.float32, gate.dtype) and group in (8, 16, 32, 64, 128) and y.numel() > 0
            and not (need_grad and C > 1024))
    if not fits:
        return groupnorm_gate_tensor_ops(y, gate, gn_weight, gn_bias, n_groups, eps)
    yc, gc = y.contiguous(), gate.contiguous()
    if need_grad:
        w, b = gn_weight.to(gate.dtype).contiguous(), gn_bias.to(gate.dtype).contiguous()
    else:
        w, b = gn_weight.detach().to(gate.dtype).contiguous(), gn_bias.detach().to(gate.dtype).contiguous()
    if not _vec_ok(yc, gc, w, b):
        return groupnorm_gate_tensor_ops(y, gate, gn_weight, gn_bias, n_groups, eps)
    if need_grad:
        return _GroupNormGate.apply(yc, gc, w, b, group, float(eps))
    return _groupnorm_gate_launch(yc, gc, w, b, group, eps)


class _QShiftMix(torch.autograd.Function):
    """q_shift + mix lerps with a hand-written backward (vrwkv_qshift_mix / vrwkv_qshift_mix_bwd); the mix vectors
    enter as one (n_mix, C) fp32 table, so whatever produced them (parameters, 1 - parameter, ...) is differentiated
    by autograd outside."""

    @staticmethod
    def forward(ctx, x, table, shift_pixel, gamma, Hp, Wp, head_dim):
        x = x.contiguous()
        table = table.contiguous()
        ctx.save_for_backward(x, table)
        ctx.meta = (shift_pixel, gamma, Hp, Wp, head_dim)
        outs = q_shift_mix(x, [None] * table.shape[0], shift_pixel, gamma, (Hp, Wp), head_dim, mix_table=table)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *gouts):
        x, table = ctx.saved_tensors
        shift_pixel, gamma, Hp, Wp, head_dim = ctx.meta
        B, T, C = x.shape
        n_mix = table.shape[0]
        gs = [g.to(x.dtype).contiguous() for g in gouts]
        gx = torch.empty_like(x)
        gmix = torch.empty_like(table)
        L = _lib.lib()
        ws_bytes = L.vrwkv_qshift_mix_bwd_workspace_bytes(n_mix, B, T, C)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
        ptrs = (ctypes.c_void_p * n_mix)(*[g.data_ptr() for g in gs])
        g = head_dim // 4 if head_dim else int(C * gamma)
        with torch.cuda.device(x.device):
            _lib.check(L.vrwkv_qshift_mix_bwd(x.data_ptr(), table.data_ptr(), ptrs, n_mix, gx.data_ptr(), gmix.data_ptr(),
                                              B, T, C, Hp, Wp, shift_pixel, g, head_dim, _DT[x.dtype],
                                              ws.data_ptr(), ws_bytes, _stream_ptr(x.device)))
        return gx, gmix, None, None, None, None, None


def q_shift_mix_autograd(x, mixes, shift_pixel=1, gamma=1 / 4, patch_resolution=None, head_dim=0):
    """q_shift_mix for training: the same fused forward kernel, and one fused backward kernel in place of autograd
    through the slice copies and lerps.  `mixes` may be parameters or tensors derived from parameters."""
    _check_input(x, "x")
    if x.dim() != 3 or x.dtype not in _DT:
        raise RuntimeError("x must be (B,T,C) float32 / bfloat16 / float16")
    table = torch.stack([m.reshape(-1) for m in mixes]).float()       # one cast, differentiated as one
    Hp, Wp = patch_resolution
    if not _equal_quarters(x.shape[-1], gamma, head_dim):
        xx = q_shift(x, shift_pixel, gamma, patch_resolution)
        return [(x.float() * m + xx.float() * (1 - m)).to(x.dtype) for m in table]
    return list(_QShiftMix.apply(x, table, shift_pixel, gamma, Hp, Wp, head_dim))
