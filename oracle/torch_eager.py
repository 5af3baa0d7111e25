"""The reference recurrences as PyTorch CPU-eager loops over T.  Test infrastructure only.

These are what the benchmark times as its CPU baseline (one vectorised update of
(B,C) / (B,H,N,N) state tensors per token, two passes), and what the GPU parity
tests use as the fp32 sequential reference.  Same mathematics as oracle/biwkv.py
and oracle/wkv6.py; formulas follow
classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:93-108 and
classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:23-96.
"""
import torch

MIN_VALUE = -1e38


@torch.no_grad()
def biwkv_eager(w, u, k, v):
    """w,u (C,), k,v (B,T,C) CPU tensors of one dtype -> y (B,T,C) same dtype."""
    B, T, C = k.shape
    dt = k.dtype
    a = torch.zeros(B, C, dtype=dt)
    b = torch.zeros(B, C, dtype=dt)
    p = torch.full((B, C), MIN_VALUE, dtype=dt)
    A = torch.empty(T, B, C, dtype=dt)
    Bd = torch.empty(T, B, C, dtype=dt)
    P = torch.empty(T, B, C, dtype=dt)
    for t in range(T):
        A[t], Bd[t], P[t] = a, b, p
        kt, vt = k[:, t], v[:, t]
        q = torch.maximum(p - w, kt)
        e1 = torch.exp(p - w - q)
        e2 = torch.exp(kt - q)
        a = e1 * a + e2 * vt
        b = e1 * b + e2
        p = q
    y = torch.empty(B, T, C, dtype=dt)
    c = torch.zeros(B, C, dtype=dt)
    d = torch.zeros(B, C, dtype=dt)
    o = torch.full((B, C), MIN_VALUE, dtype=dt)
    for t in range(T - 1, -1, -1):
        kt, vt = k[:, t], v[:, t]
        uk = u + kt
        m = torch.maximum(torch.maximum(P[t], o), uk)
        ea = torch.exp(P[t] - m)
        ec = torch.exp(o - m)
        eu = torch.exp(uk - m)
        y[:, t] = (ea * A[t] + ec * c + eu * vt) / (ea * Bd[t] + ec * d + eu)
        q = torch.maximum(o - w, kt)
        e1 = torch.exp(o - w - q)
        e2 = torch.exp(kt - q)
        c = e1 * c + e2 * vt
        d = e1 * d + e2
        o = q
    return y


@torch.no_grad()
def wkv6_eager(r, k, v, w_raw, u, H):
    """r,k,v,w_raw (B,T,C), u (H,N) CPU tensors -> y (B,T,C), state (B,H,N,N) per direction."""
    B, T, C = r.shape
    N = C // H
    dt = r.dtype
    r4 = r.view(B, T, H, N)
    k4 = k.view(B, T, H, N)
    v4 = v.view(B, T, H, N)
    d4 = torch.exp(-torch.exp(w_raw)).view(B, T, H, N)
    y = torch.zeros(B, T, H, N, dtype=dt)
    S = torch.zeros(B, H, N, N, dtype=dt)
    for t in range(T - 1, -1, -1):
        y[:, t] = torch.einsum('bhj,bhji->bhi', r4[:, t], S)
        S = d4[:, t].unsqueeze(-1) * S + k4[:, t].unsqueeze(-1) * v4[:, t].unsqueeze(-2)
    S = torch.zeros(B, H, N, N, dtype=dt)
    uu = u.view(1, H, N, 1)
    for t in range(T):
        kv = k4[:, t].unsqueeze(-1) * v4[:, t].unsqueeze(-2)
        y[:, t] += torch.einsum('bhj,bhji->bhi', r4[:, t], uu * kv + S)
        S = d4[:, t].unsqueeze(-1) * S + kv
    return y.view(B, T, C)
