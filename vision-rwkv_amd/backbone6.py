"""Plain-PyTorch VRWKV6 backbone (no mmcv / mmcls) on top of the HIP wkv6 operator.

Mirrors, module for module and parameter name for parameter name (state_dict keys `time_maa_*`,
`time_decay*`, `time_faaaa`, `ln_x`, `spatial_mix_*`), classification/mmcls_custom/models/backbones/vrwkv6.py:
SpatialMix_V6 :103-227 (data-dependent token mix through two low-rank maps, low-rank decay, GroupNorm and
SiLU gate around RUN_CUDA_RWKV6), ChannelMix :230-285, Block :288-343, VRWKV6 :346-478.  The token shift is
q_shift_multihead (:75-100): Q-Shift inside every 64-channel head, an optional class token kept last.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .backbone import VRWKV, eval_cached, _proj, _matmul, _bmm
from .ops import (HEAD_SIZE, RUN_CUDA_RWKV6, q_shift, q_shift_mix, q_shift_mix_autograd, stack_mixes, row_fuse, maa_mix, groupnorm_gate, PRE_NONE, PRE_RELU_SQ, POST_NONE,
                  POST_SIGMOID_GATE, POST_RESIDUAL)


def q_shift_multihead(x, shift_pixel=1, head_dim=HEAD_SIZE, patch_resolution=None, with_cls_token=False):
    """Q-Shift of every head separately: heads are folded into the batch and shifted as C = head_dim images."""
    B, N, C = x.shape
    assert C % head_dim == 0 and head_dim % 4 == 0
    body = x[:, :-1] if with_cls_token else x
    T = body.shape[1]
    heads = body.reshape(B, T, C // head_dim, head_dim).permute(0, 2, 1, 3).reshape(-1, T, head_dim)
    heads = q_shift(heads, shift_pixel, 1 / 4, patch_resolution)
    out = heads.reshape(B, C // head_dim, T, head_dim).permute(0, 2, 1, 3).reshape(B, T, C)
    return torch.cat((out, x[:, -1:]), dim=1) if with_cls_token else out


def _shift_and_mix(module, x, mixes, shift_pixel, patch_resolution, with_cls_token, fused, params):
    """[x*m + shift(x)*(1-m) for m in mixes()]; one HIP kernel (forward, and backward under autograd), tensor ops when
    `fused` is off or off the GPU.  `mixes` is a callable (the vectors may be derived from `params`); at inference
    its stacked fp32 table is kept on the module."""
    if fused and x.is_cuda:
        if torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in params)):
            return q_shift_mix_autograd(x, mixes(), shift_pixel, 1 / 4, patch_resolution, HEAD_SIZE)
        table = eval_cached(module, "mix_table", params, x.device, lambda: stack_mixes(mixes(), x.device))
        return q_shift_mix(x.contiguous(), [None] * table.shape[0], shift_pixel, 1 / 4, patch_resolution,
                           head_dim=HEAD_SIZE, mix_table=table)
    sx = q_shift_multihead(x, shift_pixel, HEAD_SIZE, patch_resolution, with_cls_token)
    return [x * m + sx * (1 - m) for m in mixes()]


def _layer_norm(ln, x):
    """nn.LayerNorm over the channels through the fused row kernel (forward and backward); tensor ops where it does
    not apply."""
    return row_fuse(x, None, ln.weight, ln.bias, None, PRE_NONE, POST_NONE, ln.eps)


class VRWKV_SpatialMix_V6(nn.Module):
    def __init__(self, n_embd, n_head, n_layer, layer_id, shift_pixel=1, key_norm=False, with_cls_token=False,
                 fused_shift=True):
        super().__init__()
        assert n_embd // n_head == HEAD_SIZE
        self.n_embd, self.n_head, self.layer_id = n_embd, n_head, layer_id
        self.shift_pixel, self.with_cls_token, self.fused_shift = shift_pixel, with_cls_token, fused_shift
        r01 = layer_id / max(n_layer - 1, 1)
        r10 = 1.0 - layer_id / n_layer
        ddd = (torch.arange(n_embd, dtype=torch.float32) / n_embd).reshape(1, 1, n_embd)
        self.time_maa_x = nn.Parameter(1.0 - torch.pow(ddd, r10))
        self.time_maa_w = nn.Parameter(1.0 - torch.pow(ddd, r10))
        self.time_maa_k = nn.Parameter(1.0 - torch.pow(ddd, r10))
        self.time_maa_v = nn.Parameter(1.0 - (torch.pow(ddd, r10) + 0.3 * r01))
        self.time_maa_r = nn.Parameter(1.0 - torch.pow(ddd, 0.5 * r10))
        self.time_maa_g = nn.Parameter(1.0 - torch.pow(ddd, 0.5 * r10))
        self.time_maa_w1 = nn.Parameter(torch.empty(n_embd, 32 * 5).uniform_(-1e-4, 1e-4))
        self.time_maa_w2 = nn.Parameter(torch.empty(5, 32, n_embd).uniform_(-1e-4, 1e-4))
        n = torch.arange(n_embd, dtype=torch.float32)
        self.time_decay = nn.Parameter((-6 + 5 * (n / (n_embd - 1)) ** (0.7 + 1.3 * r01)).reshape(1, 1, n_embd))
        self.time_decay_w1 = nn.Parameter(torch.empty(n_embd, 64).uniform_(-1e-4, 1e-4))
        self.time_decay_w2 = nn.Parameter(torch.empty(64, n_embd).uniform_(-1e-4, 1e-4))
        zigzag = torch.tensor([((i + 1) % 3 - 1) * 0.1 for i in range(n_embd)], dtype=torch.float32)
        self.time_faaaa = nn.Parameter((r01 * (1 - n / (n_embd - 1)) + zigzag).reshape(n_head, HEAD_SIZE))
        self.key = nn.Linear(n_embd, n_embd, bias=False)
        self.value = nn.Linear(n_embd, n_embd, bias=False)
        self.receptance = nn.Linear(n_embd, n_embd, bias=False)
        self.gate = nn.Linear(n_embd, n_embd, bias=False)
        self.key_norm = nn.LayerNorm(n_embd) if key_norm else None
        self.output = nn.Linear(n_embd, n_embd, bias=False)
        self.ln_x = nn.GroupNorm(n_head, n_embd, eps=1e-5)

    def forward(self, x, patch_resolution):
        B, T, C = x.shape
        # shift(x) and x + (shift(x) - x) * maa_x = x*(1 - maa_x) + shift(x)*maa_x in one pass over x
        sx, xxx = _shift_and_mix(self, x, lambda: [torch.zeros_like(self.time_maa_x), 1 - self.time_maa_x],
                                 self.shift_pixel, patch_resolution, self.with_cls_token, self.fused_shift,
                                 (self.time_maa_x,))
        lo = torch.tanh(_matmul(xxx, self.time_maa_w1)).view(B * T, 5, -1).transpose(0, 1)
        m = _bmm(lo, self.time_maa_w2).view(5, B, T, C)
        # xw..xg = x + (sx - x) * (time_maa_* + m_*)  (vrwkv6.py:190-194): one pass at inference
        maas = (self.time_maa_w, self.time_maa_k, self.time_maa_v, self.time_maa_r, self.time_maa_g)
        table = None
        if not torch.is_grad_enabled() and x.is_cuda:
            table = eval_cached(self, "maa_table", maas, x.device, lambda: stack_mixes(maas, x.device))
        xw, xk, xv, xr, xg = maa_mix(x, sx, m, maas, table)
        r, k, v = _proj(self.receptance, xr), _proj(self.key, xk), _proj(self.value, xv)
        gate = _proj(self.gate, xg)
        w = self.time_decay + _matmul(torch.tanh(_matmul(xw, self.time_decay_w1)), self.time_decay_w2)
        y = RUN_CUDA_RWKV6(B, T, C, self.n_head, r.contiguous(), k.contiguous(), v.contiguous(),
                           w.contiguous(), self.time_faaaa.float())                  # vrwkv6.py:217 (w as it is: the
        # kernel widens a 16-bit decay logit itself, the same values the reference's `w.float()` holds)
        if self.key_norm is not None:
            y = self.key_norm(y.to(gate.dtype))
        # ln_x over each head's channels, times silu(gate) (vrwkv6.py:199, 205-211): one pass at inference
        y = groupnorm_gate(y, gate, self.ln_x.weight, self.ln_x.bias, self.ln_x.num_groups, self.ln_x.eps)
        return _proj(self.output, y)


class VRWKV_ChannelMix_V6(nn.Module):
    def __init__(self, n_embd, n_head, n_layer, layer_id, shift_pixel=1, hidden_rate=4, key_norm=False,
                 with_cls_token=False, fused_shift=True):
        super().__init__()
        assert n_embd // n_head == HEAD_SIZE
        self.shift_pixel, self.with_cls_token, self.fused_shift = shift_pixel, with_cls_token, fused_shift
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
        xk, xr = _shift_and_mix(self, x, lambda: [self.spatial_mix_k, self.spatial_mix_r], self.shift_pixel,
                                patch_resolution, self.with_cls_token, self.fused_shift,
                                (self.spatial_mix_k, self.spatial_mix_r))
        kn = self.key_norm                                   # relu^2 (+ key_norm), then the sigmoid gate: one pass each
        k = row_fuse(_proj(self.key, xk), None, kn.weight if kn is not None else None, kn.bias if kn is not None else None, None,
                     PRE_RELU_SQ, POST_NONE, kn.eps if kn is not None else 1e-5)
        return row_fuse(_proj(self.value, k), _proj(self.receptance, xr), None, None, None, PRE_NONE, POST_SIGMOID_GATE)


class Block6(nn.Module):
    def __init__(self, n_embd, n_head, n_layer, layer_id, shift_pixel=1, hidden_rate=4, init_values=None,
                 post_norm=False, key_norm=False, with_cls_token=False, fused_shift=True):
        super().__init__()
        self.layer_id, self.post_norm = layer_id, post_norm
        self.ln1, self.ln2 = nn.LayerNorm(n_embd), nn.LayerNorm(n_embd)
        if layer_id == 0:
            self.ln0 = nn.LayerNorm(n_embd)
        self.att = VRWKV_SpatialMix_V6(n_embd, n_head, n_layer, layer_id, shift_pixel, key_norm, with_cls_token, fused_shift)
        self.ffn = VRWKV_ChannelMix_V6(n_embd, n_head, n_layer, layer_id, shift_pixel, hidden_rate, key_norm,
                                       with_cls_token, fused_shift)
        self.layer_scale = init_values is not None
        if self.layer_scale:
            self.gamma1 = nn.Parameter(init_values * torch.ones(n_embd))
            self.gamma2 = nn.Parameter(init_values * torch.ones(n_embd))

    def forward(self, x, patch_resolution):
        if self.layer_id == 0:
            x = _layer_norm(self.ln0, x)
        g1 = self.gamma1 if self.layer_scale else None
        g2 = self.gamma2 if self.layer_scale else None
        if self.post_norm:                                   # scale, add and post-norm in one pass
            x = row_fuse(self.att(x, patch_resolution), x, self.ln1.weight, self.ln1.bias, g1, PRE_NONE, POST_RESIDUAL, self.ln1.eps)
            x = row_fuse(self.ffn(x, patch_resolution), x, self.ln2.weight, self.ln2.bias, g2, PRE_NONE, POST_RESIDUAL, self.ln2.eps)
        else:
            x = row_fuse(self.att(_layer_norm(self.ln1, x), patch_resolution), x, None, None, g1, PRE_NONE, POST_RESIDUAL)
            x = row_fuse(self.ffn(_layer_norm(self.ln2, x), patch_resolution), x, None, None, g2, PRE_NONE, POST_RESIDUAL)
        return x


class VRWKV6(VRWKV):
    """vrwkv6.py:346-478; patch embedding and position table are those of VRWKV.  Returns the last feature
    map (B, C, Hp, Wp), and the class token as well when output_cls_token is set."""

    def __init__(self, img_size=224, patch_size=16, in_channels=3, embed_dims=192, num_heads=3, depth=12,
                 shift_pixel=1, post_norm=False, key_norm=False, init_values=None, hidden_rate=4, final_norm=True,
                 interpolate_mode="bicubic", with_cls_token=False, output_cls_token=False, fused_shift=True):
        super().__init__(img_size=img_size, patch_size=patch_size, in_channels=in_channels, embed_dims=embed_dims,
                         depth=0, final_norm=final_norm, interpolate_mode=interpolate_mode)
        assert with_cls_token or not output_cls_token
        self.with_cls_token, self.output_cls_token = with_cls_token, output_cls_token
        if with_cls_token:
            self.cls_token = nn.Parameter(torch.zeros(1, 1, embed_dims))
        self.layers = nn.ModuleList([
            Block6(embed_dims, num_heads, depth, i, shift_pixel, hidden_rate, init_values, post_norm, key_norm,
                   with_cls_token, fused_shift) for i in range(depth)])

    def forward(self, img):
        x, res = self.embed(img)
        x = x + self._pos_embed_for(res).to(x.dtype)
        B = x.shape[0]
        if self.with_cls_token:
            x = torch.cat((x, self.cls_token.expand(B, -1, -1).to(x.dtype)), dim=1)      # class token last
        for layer in self.layers:
            x = layer(x, res)
        if self.final_norm:
            x = _layer_norm(self.ln1, x)
        C = x.shape[-1]
        patches = x[:, :-1] if self.with_cls_token else x
        fmap = patches.reshape(B, res[0], res[1], C).permute(0, 3, 1, 2)
        return (fmap, x[:, -1]) if self.output_cls_token else fmap


def vrwkv6_b(**kw):
    """VRWKV6-B: classification/configs/vrwkv6/vrwkv6_base_16xb64_in1k.py:11-20."""
    cfg = dict(img_size=224, patch_size=16, embed_dims=768, num_heads=12, depth=12, post_norm=True, init_values=1e-5)
    cfg.update(kw)
    return VRWKV6(**cfg)
