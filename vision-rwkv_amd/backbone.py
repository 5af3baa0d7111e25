"""Plain-PyTorch VRWKV backbone (no mmcv / mmcls) that calls the HIP Bi-WKV through RUN_CUDA.

It exists to time the operator in situ (VRWKV-L forward, benchmark config 4) and mirrors, module
for module and parameter name for parameter name,
classification/mmcls_custom/models/backbones/vrwkv.py:82-432 (identical copy:
classification_internimage/models/vrwkv.py) with the VRWKV-L settings of
classification_internimage/configs/vrwkv_l_22kto1k_384.yaml:10-28.  PatchEmbed is
Conv2d(kernel = stride = patch) + flatten (mmcv's PatchEmbed with these arguments) and the position
embedding is resized bicubically as in detection/mmdet_custom/models/utils/embed.py:6-47.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .ops import (RUN_CUDA, bi_wkv_forward, q_shift, q_shift_mix, q_shift_mix_autograd, stack_mixes, row_fuse, PRE_NONE, PRE_RELU_SQ, POST_NONE, POST_SIGMOID_GATE,
                  POST_RESIDUAL)


def resize_pos_embed(pos_embed, src_shape, dst_shape, mode="bicubic", num_extra_tokens=0):
    """Position table (1, extra + Hs*Ws, C) resampled to the grid dst_shape, extra tokens passed through: the
    interpolation of detection/mmdet_custom/models/utils/embed.py:6-47 (F.interpolate, align_corners=False), which
    the backbones call with no extra tokens (vrwkv.py:411-415)."""
    if tuple(src_shape) == tuple(dst_shape):
        return pos_embed
    _, L, C = pos_embed.shape
    if L != src_shape[0] * src_shape[1] + num_extra_tokens:
        raise RuntimeError(f"pos_embed has {L} tokens, expected {src_shape[0]}*{src_shape[1]}+{num_extra_tokens}")
    extra, grid = pos_embed[:, :num_extra_tokens], pos_embed[:, num_extra_tokens:]
    w = grid.reshape(1, src_shape[0], src_shape[1], C).permute(0, 3, 1, 2)
    w = F.interpolate(w.float(), size=dst_shape, align_corners=False, mode=mode).to(pos_embed.dtype)
    w = torch.flatten(w, 2).transpose(1, 2)
    return torch.cat((extra, w), dim=1) if num_extra_tokens else w


def eval_cached(module, name, params, extra, make):
    """Value derived from parameters (a dtype conversion, a stacked table), kept on the module between forward passes
    without autograd and rebuilt when a parameter was written to (its version counter), moved or cast."""
    key = (extra,) + tuple((p._version, p.dtype, p.device, p.data_ptr()) for p in params)
    slot = module.__dict__.setdefault("_eval_cache", {})
    hit = slot.get(name)
    if hit is None or hit[0] != key:
        hit = (key, make())
        slot[name] = hit
    return hit[1]


def _mix(module, x, mixes, shift_pixel, gamma, patch_resolution, fused, head_dim=0):
    """[x*m + q_shift(x)*(1-m) for m in mixes]: one fused kernel (forward, and backward under autograd); tensor ops
    when `fused` is off or the tensors are not on the GPU."""
    if fused and x.is_cuda:
        if torch.is_grad_enabled() and (x.requires_grad or any(m.requires_grad for m in mixes)):
            return q_shift_mix_autograd(x, mixes, shift_pixel, gamma, patch_resolution, head_dim)
        table = eval_cached(module, "mix_table", mixes, x.device, lambda: stack_mixes(mixes, x.device))
        return q_shift_mix(x.contiguous(), mixes, shift_pixel, gamma, patch_resolution, head_dim, mix_table=table)
    xx = q_shift(x, shift_pixel, gamma, patch_resolution)
    return [x * m + xx * (1 - m) for m in mixes]


class _SplitKLinear(torch.autograd.Function):
    """x @ W^T whose weight gradient g^T x -- a contraction over all B*T tokens into a small (out, in) matrix, which the
    library's GEMM runs as one deep sum on too few workgroups -- is computed as `splits` batched partial products that
    are added in fp32.  Forward and input gradient are the library's plain GEMMs."""

    @staticmethod
    def forward(ctx, x, weight, splits):
        ctx.save_for_backward(x, weight)
        ctx.splits = splits
        return F.linear(x, weight)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        S = ctx.splits
        gx = g @ weight if ctx.needs_input_grad[0] else None
        gw = None
        if ctx.needs_input_grad[1]:
            g2, x2 = g.reshape(-1, g.shape[-1]), x.reshape(-1, x.shape[-1])
            M = g2.shape[0]
            part = torch.bmm(g2.view(S, M // S, -1).transpose(1, 2), x2.view(S, M // S, -1))
            gw = part.sum(0)              # one kernel: the sum of 16-bit values accumulates in fp32 and is rounded once
        return gx, gw, None


class _SplitKMatmul(torch.autograd.Function):
    """x @ W for a parameter matrix W (in, out): the same split of the weight gradient x^T g over the tokens."""

    @staticmethod
    def forward(ctx, x, weight, splits):
        ctx.save_for_backward(x, weight)
        ctx.splits = splits
        return x @ weight

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        S = ctx.splits
        gx = g @ weight.t() if ctx.needs_input_grad[0] else None
        gw = None
        if ctx.needs_input_grad[1]:
            g2, x2 = g.reshape(-1, g.shape[-1]), x.reshape(-1, x.shape[-1])
            M = g2.shape[0]
            part = torch.bmm(x2.view(S, M // S, -1).transpose(1, 2), g2.view(S, M // S, -1))
            gw = part.sum(0)              # accumulated in fp32, rounded once
        return gx, gw, None


class _SplitKBmm(torch.autograd.Function):
    """torch.bmm(x, W) for a stack of parameter matrices W (n, in, out) and x (n, M, in) with M = all B*T tokens: each
    weight gradient x_i^T g_i is split over the tokens like _SplitKMatmul's (the library runs the deep, narrow
    contraction on a handful of workgroups otherwise)."""

    @staticmethod
    def forward(ctx, x, weight, splits):
        ctx.save_for_backward(x, weight)
        ctx.splits = splits
        return torch.bmm(x, weight)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        S = ctx.splits
        gx = torch.bmm(g, weight.transpose(1, 2)) if ctx.needs_input_grad[0] else None
        gw = None
        if ctx.needs_input_grad[1]:
            n, M, _ = x.shape
            x4 = x.reshape(n, S, M // S, x.shape[-1])
            g4 = g.reshape(n, S, M // S, g.shape[-1])
            part = torch.matmul(x4.transpose(2, 3), g4)               # (n, S, in, out)
            gw = part.sum(1)              # accumulated in fp32, rounded once
        return gx, gw, None


def _bmm(x, weight):
    """torch.bmm(x, weight) for stacked low-rank parameter matrices; split weight gradient under autograd with many
    tokens."""
    if (x.is_cuda and torch.is_grad_enabled() and weight.requires_grad and x.dtype == weight.dtype
            and x.dtype in (torch.bfloat16, torch.float16) and weight.dim() == 3 and x.dim() == 3):
        M = x.shape[1]
        if M >= 4096 and M % 8 == 0:
            return _SplitKBmm.apply(x, weight, 8)
    return torch.bmm(x, weight)


def _matmul(x, weight):
    """x @ weight for a low-rank parameter matrix; split weight gradient under autograd with many tokens."""
    if (x.is_cuda and torch.is_grad_enabled() and weight.requires_grad and x.dtype == weight.dtype
            and x.dtype in (torch.bfloat16, torch.float16) and weight.dim() == 2):
        M = x.numel() // x.shape[-1]
        if M >= 4096 and M % 8 == 0:
            return _SplitKMatmul.apply(x, weight, 8)
    return x @ weight


def _proj(linear, x):
    """linear(x) for the bias-free projections of a block; under autograd on the GPU with many tokens the weight gradient
    is split over the tokens (see _SplitKLinear)."""
    w = linear.weight
    hooked = linear._forward_hooks or linear._forward_pre_hooks       # hooks fire only through linear(x)
    if (linear.bias is None and not hooked and x.is_cuda and torch.is_grad_enabled() and w.requires_grad
            and x.dtype == w.dtype and x.dtype in (torch.bfloat16, torch.float16)):
        M = x.numel() // x.shape[-1]
        S = 4 if w.numel() >= (1 << 21) else 8
        if M >= 4096 and M % S == 0:
            return _SplitKLinear.apply(x, w, S)
    return linear(x)


def _layer_norm(ln, x):
    """nn.LayerNorm over the channels through the fused row kernel (forward and backward); tensor ops where it does
    not apply."""
    return row_fuse(x, None, ln.weight, ln.bias, None, PRE_NONE, POST_NONE, ln.eps)


class VRWKV_SpatialMix(nn.Module):
    def __init__(self, n_embd, n_layer, layer_id, channel_gamma=1 / 4, shift_pixel=1, key_norm=False, fused_shift=True):
        super().__init__()
        self.layer_id, self.n_layer, self.n_embd = layer_id, n_layer, n_embd
        self.shift_pixel, self.channel_gamma, self.fused_shift = shift_pixel, channel_gamma, fused_shift
        r01 = layer_id / max(n_layer - 1, 1)
        r10 = 1.0 - layer_id / n_layer
        h = torch.arange(n_embd, dtype=torch.float32)
        self.spatial_decay = nn.Parameter(-5 + 8 * (h / (n_embd - 1)) ** (0.7 + 1.3 * r01))
        zigzag = torch.tensor([(i + 1) % 3 - 1 for i in range(n_embd)], dtype=torch.float32) * 0.5
        self.spatial_first = nn.Parameter(torch.ones(n_embd) * math.log(0.3) + zigzag)
        x = (h / n_embd).reshape(1, 1, n_embd)
        self.spatial_mix_k = nn.Parameter(torch.pow(x, r10))
        self.spatial_mix_v = nn.Parameter(torch.pow(x, r10) + 0.3 * r01)
        self.spatial_mix_r = nn.Parameter(torch.pow(x, 0.5 * r10))
        self.key = nn.Linear(n_embd, n_embd, bias=False)
        self.value = nn.Linear(n_embd, n_embd, bias=False)
        self.receptance = nn.Linear(n_embd, n_embd, bias=False)
        self.key_norm = nn.LayerNorm(n_embd) if key_norm else None
        self.output = nn.Linear(n_embd, n_embd, bias=False)
        self.fused_gate = True     # inference without key_norm: sigmoid(r) * y inside the Bi-WKV kernel

    def forward(self, x, patch_resolution):
        B, T, C = x.shape
        if self.shift_pixel > 0:
            xk, xv, xr = _mix(self, x, [self.spatial_mix_k, self.spatial_mix_v, self.spatial_mix_r], self.shift_pixel,
                              self.channel_gamma, patch_resolution, self.fused_shift)
        else:
            xk = xv = xr = x
        k, v, r = _proj(self.key, xk), _proj(self.value, xv), _proj(self.receptance, xr)
        wd = self.spatial_decay.dtype
        if torch.is_grad_enabled() or k.dtype != (wd if wd in (torch.half, torch.bfloat16) else torch.float32):
            y = RUN_CUDA(self.spatial_decay / T, self.spatial_first / T, k, v)  # vrwkv.py:183
        else:
            # what WKV.forward does with these arguments, the scaled fp32 copies of w and u kept between calls
            w, u = eval_cached(self, "wu", (self.spatial_decay, self.spatial_first), T,
                               lambda: ((self.spatial_decay / T).float().contiguous(),
                                        (self.spatial_first / T).float().contiguous()))
            if self.key_norm is None and self.fused_gate and r.dtype == k.dtype:
                # the receptance gate (vrwkv.py:185-186) applied inside the operator, before y is stored
                return _proj(self.output, bi_wkv_forward(w, u, k.contiguous(), v.contiguous(), gate=r.contiguous()))
            y = bi_wkv_forward(w, u, k.contiguous(), v.contiguous())
        y = y.to(r.dtype)
        # key_norm and the sigmoid gate (vrwkv.py:184-186) in one pass; tensor ops under autograd
        kn = self.key_norm
        y = row_fuse(y, r, kn.weight if kn is not None else None, kn.bias if kn is not None else None, None,
                     PRE_NONE, POST_SIGMOID_GATE, kn.eps if kn is not None else 1e-5)
        return _proj(self.output, y)


class VRWKV_ChannelMix(nn.Module):
    def __init__(self, n_embd, n_layer, layer_id, channel_gamma=1 / 4, shift_pixel=1, hidden_rate=4, key_norm=False,
                 fused_shift=True):
        super().__init__()
        self.shift_pixel, self.channel_gamma, self.fused_shift = shift_pixel, channel_gamma, fused_shift
        r10 = 1.0 - layer_id / n_layer
        x = (torch.arange(n_embd, dtype=torch.float32) / n_embd).reshape(1, 1, n_embd)
        self.spatial_mix_k = nn.Parameter(torch.pow(x, r10))
        self.spatial_mix_r = nn.Parameter(torch.pow(x, r10))
        hidden = hidden_rate * n_embd
        self.key = nn.Linear(n_embd, hidden, bias=False)
        self.key_norm = nn.LayerNorm(hidden) if key_norm else None
        self.receptance = nn.Linear(n_embd, n_embd, bias=False)
        self.value = nn.Linear(hidden, n_embd, bias=False)

    def forward(self, x, patch_resolution):
        if self.shift_pixel > 0:
            xk, xr = _mix(self, x, [self.spatial_mix_k, self.spatial_mix_r], self.shift_pixel, self.channel_gamma,
                          patch_resolution, self.fused_shift)
        else:
            xk = xr = x
        # relu^2 (+ key_norm) and the sigmoid gate (vrwkv.py:256-261), one pass each; tensor ops under autograd
        kn = self.key_norm
        k = row_fuse(_proj(self.key, xk), None, kn.weight if kn is not None else None, kn.bias if kn is not None else None, None,
                     PRE_RELU_SQ, POST_NONE, kn.eps if kn is not None else 1e-5)
        return row_fuse(_proj(self.value, k), _proj(self.receptance, xr), None, None, None, PRE_NONE, POST_SIGMOID_GATE)


class Block(nn.Module):
    def __init__(self, n_embd, n_layer, layer_id, channel_gamma=1 / 4, shift_pixel=1, hidden_rate=4, init_values=None,
                 post_norm=False, key_norm=False, fused_shift=True):
        super().__init__()
        self.layer_id, self.post_norm = layer_id, post_norm
        self.ln1, self.ln2 = nn.LayerNorm(n_embd), nn.LayerNorm(n_embd)
        if layer_id == 0:
            self.ln0 = nn.LayerNorm(n_embd)
        self.att = VRWKV_SpatialMix(n_embd, n_layer, layer_id, channel_gamma, shift_pixel, key_norm, fused_shift)
        self.ffn = VRWKV_ChannelMix(n_embd, n_layer, layer_id, channel_gamma, shift_pixel, hidden_rate, key_norm, fused_shift)
        self.layer_scale = init_values is not None
        if self.layer_scale:
            self.gamma1 = nn.Parameter(init_values * torch.ones(n_embd))
            self.gamma2 = nn.Parameter(init_values * torch.ones(n_embd))

    def forward(self, x, patch_resolution):
        if self.layer_id == 0:
            x = _layer_norm(self.ln0, x)
        g1 = self.gamma1 if self.layer_scale else None
        g2 = self.gamma2 if self.layer_scale else None
        # residual with layer scale (vrwkv.py:300-313): x + gamma * ln(branch(x)) or x + gamma * branch(ln(x)), the
        # scale, the add and the post-norm in one pass; tensor ops under autograd
        if self.post_norm:
            x = row_fuse(self.att(x, patch_resolution), x, self.ln1.weight, self.ln1.bias, g1, PRE_NONE, POST_RESIDUAL, self.ln1.eps)
            x = row_fuse(self.ffn(x, patch_resolution), x, self.ln2.weight, self.ln2.bias, g2, PRE_NONE, POST_RESIDUAL, self.ln2.eps)
        else:
            x = row_fuse(self.att(_layer_norm(self.ln1, x), patch_resolution), x, None, None, g1, PRE_NONE, POST_RESIDUAL)
            x = row_fuse(self.ffn(_layer_norm(self.ln2, x), patch_resolution), x, None, None, g2, PRE_NONE, POST_RESIDUAL)
        return x


class VRWKV(nn.Module):
    """vrwkv.py:322-432 without the mmcv base classes.  With `out_indices` left at None it returns the last feature map
    (B, C, Hp, Wp); with an int or a sequence of layer indices (negative ones count from the end) it returns the tuple
    of those layers' feature maps, as the reference does for the mmdet / mmseg callers (vrwkv.py:368-378, 421-432)."""

    def __init__(self, img_size=224, patch_size=16, in_channels=3, embed_dims=256, depth=12, channel_gamma=1 / 4,
                 shift_pixel=1, post_norm=False, key_norm=False, init_values=None, hidden_rate=4, final_norm=True,
                 interpolate_mode="bicubic", fused_shift=True, out_indices=None):
        super().__init__()
        if out_indices is not None:
            out_indices = [out_indices] if isinstance(out_indices, int) else list(out_indices)
            out_indices = [depth + i if i < 0 else i for i in out_indices]
            for i in out_indices:
                if not 0 <= i <= depth:
                    raise ValueError(f"Invalid out_indices {i}")
        self.out_indices = out_indices
        self.patch_size = patch_size
        self.patch_embed = nn.Conv2d(in_channels, embed_dims, kernel_size=patch_size, stride=patch_size, bias=True)
        self.patch_resolution = (img_size // patch_size, img_size // patch_size)
        self.pos_embed = nn.Parameter(torch.zeros(1, self.patch_resolution[0] * self.patch_resolution[1], embed_dims))
        self.interpolate_mode = interpolate_mode
        self.layers = nn.ModuleList([
            Block(embed_dims, depth, i, channel_gamma, shift_pixel, hidden_rate, init_values, post_norm, key_norm,
                  fused_shift) for i in range(depth)])
        self.final_norm = final_norm
        if final_norm:
            self.ln1 = nn.LayerNorm(embed_dims)

    def load_reference_state_dict(self, state_dict, strict=True):
        """Load a checkpoint written by the reference backbones (vrwkv.py:322-432, vrwkv6.py, the mmdet / mmseg /
        classification_internimage copies).  Their parameter names are the ones used here except for the patch
        embedding, which mmcv's PatchEmbed keeps as `patch_embed.projection.{weight,bias}` (vrwkv.py:351-358);
        whole-model checkpoints carry a `backbone.` prefix and other modules' entries (`head.*`, `neck.*`), which are
        dropped.  A position table trained on another grid replaces this model's table and pre-training grid (it is
        interpolated to the input's grid in forward, as vrwkv.py:411-415 does).  Returns what
        nn.Module.load_state_dict returns."""
        sd = state_dict.get("state_dict", state_dict)
        if any(k.startswith("backbone.") for k in sd):
            sd = {k[len("backbone."):]: v for k, v in sd.items() if k.startswith("backbone.")}
        own = set(self.state_dict().keys())
        out = {}
        for k, v in sd.items():
            k = k.replace("patch_embed.projection.", "patch_embed.")
            if k in own:
                out[k] = v
            elif strict and k.split(".")[0] in {"patch_embed", "pos_embed", "layers", "ln1", "cls_token"}:
                raise KeyError(f"unexpected backbone entry {k!r} in the checkpoint")
        pe = out.get("pos_embed")
        if pe is not None and pe.shape != self.pos_embed.shape:
            n = pe.shape[1]
            side = int(round(n ** 0.5))
            if pe.dim() != 3 or pe.shape[2] != self.pos_embed.shape[2] or side * side != n:
                raise RuntimeError(f"pos_embed of shape {tuple(pe.shape)} does not fit this model")
            self.pos_embed = nn.Parameter(torch.zeros_like(pe, dtype=self.pos_embed.dtype, device=self.pos_embed.device))
            self.patch_resolution = (side, side)
        return self.load_state_dict(out, strict=strict)

    def _pos_embed_for(self, res):
        """Position embedding at grid `res`; in eval mode the interpolated table is computed once per grid
        (the reference re-runs the bicubic resize in every forward, vrwkv.py:411-415)."""
        if self.training or torch.is_grad_enabled():
            return resize_pos_embed(self.pos_embed, self.patch_resolution, res, self.interpolate_mode)
        key = (tuple(res), self.pos_embed._version, self.pos_embed.device, self.pos_embed.dtype)
        if getattr(self, "_pos_cache_key", None) != key:
            self._pos_cache = resize_pos_embed(self.pos_embed.detach(), self.patch_resolution, res, self.interpolate_mode)
            self._pos_cache_key = key
        return self._pos_cache

    def embed(self, img):
        """Patch embedding: (B, 3, H, W) -> (B, Hp*Wp, C) tokens and the patch grid (Hp, Wp)."""
        # kernel = stride = patch: the convolution is one GEMM over the flattened patches
        B, Cin, Hi, Wi = img.shape
        P = self.patch_size
        res = (Hi // P, Wi // P)
        patches = img[:, :, :res[0] * P, :res[1] * P].reshape(B, Cin, res[0], P, res[1], P)
        patches = patches.permute(0, 2, 4, 1, 3, 5).reshape(B, res[0] * res[1], Cin * P * P)
        x = F.linear(patches, self.patch_embed.weight.reshape(self.patch_embed.out_channels, -1), self.patch_embed.bias)
        return x, res

    def forward(self, img):
        x, res = self.embed(img)
        x = x + self._pos_embed_for(res).to(x.dtype)
        B, _, C = x.shape
        outs = []
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            x = layer(x, res)
            if i == last and self.final_norm:
                x = _layer_norm(self.ln1, x)
            if self.out_indices is not None and i in self.out_indices:
                outs.append(x.reshape(B, res[0], res[1], C).permute(0, 3, 1, 2))
        if self.out_indices is not None:
            return tuple(outs)
        return x.reshape(B, res[0], res[1], C).permute(0, 3, 1, 2)


def vrwkv_l(**kw):
    """VRWKV-L as fine-tuned at 384x384: classification_internimage/configs/vrwkv_l_22kto1k_384.yaml:10-28
    (pre-training grid 192/16 = 12x12, interpolated to 24x24; K_NORM defaults to True, config.py:82)."""
    cfg = dict(img_size=192, patch_size=16, embed_dims=1024, depth=24, post_norm=True, init_values=1e-5,
               hidden_rate=4, key_norm=True, final_norm=True)
    cfg.update(kw)
    return VRWKV(**cfg)
