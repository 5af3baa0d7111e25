"""q_shift / q_shift_multihead oracle as explicit index loops.  Test infrastructure only.

q_shift            : classification/mmcls_custom/models/backbones/vrwkv.py:68-79
q_shift_multihead  : classification/mmcls_custom/models/backbones/vrwkv6.py:75-100

Tokens are row-major over the (Hp, Wp) patch grid: t = y*Wp + x.  A channel group
"shifted right" takes its value from the left neighbour (zero in column 0), etc.
"""
import numpy as np


def _source(direction, y, x, Hp, Wp, s):
    """Source pixel of output pixel (y,x) for a shift direction, or None (zero fill)."""
    if direction == 0:      # shift right: out[:, x] = in[:, x-s]
        return (y, x - s) if x - s >= 0 else None
    if direction == 1:      # shift left:  out[:, x] = in[:, x+s]
        return (y, x + s) if x + s < Wp else None
    if direction == 2:      # shift down:  out[y, :] = in[y-s, :]
        return (y - s, x) if y - s >= 0 else None
    if direction == 3:      # shift up:    out[y, :] = in[y+s, :]
        return (y + s, x) if y + s < Hp else None
    return (y, x)           # pass-through


def q_shift_loops(x, shift_pixel, gamma, patch_resolution):
    """x: (B,T,C) -> (B,T,C); channel group q = [int(C*gamma*q), int(C*gamma*(q+1))) moves in direction q."""
    x = np.asarray(x)
    B, T, C = x.shape
    Hp, Wp = patch_resolution
    assert Hp * Wp == T and gamma <= 0.25
    # the reference cuts the channel axis at int(C*gamma), int(C*gamma*2), int(C*gamma*3), int(C*gamma*4)
    # (vrwkv.py:72-76); for C*gamma not an integer the groups are not four equal quarters
    bounds = [int(C * gamma), int(C * gamma * 2), int(C * gamma * 3), int(C * gamma * 4)]
    out = np.zeros_like(x)
    for c in range(C):
        direction = next((d for d, hi in enumerate(bounds) if c < hi), 4)
        for yy in range(Hp):
            for xx in range(Wp):
                src = _source(direction, yy, xx, Hp, Wp, shift_pixel)
                if src is not None:
                    out[:, yy * Wp + xx, c] = x[:, src[0] * Wp + src[1], c]
    return out


def q_shift_multihead_loops(x, shift_pixel, head_dim, patch_resolution, with_cls_token=False):
    """Per-head variant: inside every head of `head_dim` channels, quarter q moves in direction q.
    With a class token it sits LAST in the sequence and is passed through (vrwkv6.py:80-82, 95-97)."""
    x = np.asarray(x)
    B, T, C = x.shape
    Hp, Wp = patch_resolution
    n_tok = T - 1 if with_cls_token else T
    assert Hp * Wp == n_tok and C % head_dim == 0 and head_dim % 4 == 0
    q = head_dim // 4
    out = np.zeros_like(x)
    for c in range(C):
        direction = (c % head_dim) // q
        for yy in range(Hp):
            for xx in range(Wp):
                src = _source(direction, yy, xx, Hp, Wp, shift_pixel)
                if src is not None:
                    out[:, yy * Wp + xx, c] = x[:, src[0] * Wp + src[1], c]
    if with_cls_token:
        out[:, -1, :] = x[:, -1, :]
    return out
