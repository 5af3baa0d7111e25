"""Bi-WKV oracle (float64, NumPy).  Test infrastructure -- see oracle/__init__.py.

Mathematics (per batch b, channel c; w and u are what the caller hands to the
operator, i.e. already divided by T at
classification/mmcls_custom/models/backbones/vrwkv.py:183):

    y[t] = ( sum_{i != t} exp(k[i] - w*(|t-i|-1)) * v[i] + exp(u + k[t]) * v[t] )
         / ( sum_{i != t} exp(k[i] - w*(|t-i|-1))        + exp(u + k[t])        )

This is what the in-chunk recurrence of the reference kernel evaluates
(classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:93-115:
the emit at :95-100 uses the past state before the update at :103-108, so the
nearest neighbour carries decay exponent 0).  The reference adds EPS=1e-6 to the
max-normalised denominator (:16, :100); with every partial state normalised to
its own maximum that changes y by at most 1e-6 relative, and it is left out here.
"""
import numpy as np

MIN_VALUE = -1e38  # bi_wkv_kernel.cu:14


def biwkv_closed(w, u, k, v, channel_block=64):
    """O(T^2) closed form.  w,u: (C,), k,v: (B,T,C) -> y (B,T,C) float64."""
    w = np.asarray(w, np.float64)
    u = np.asarray(u, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    B, T, C = k.shape
    y = np.empty((B, T, C), np.float64)
    t = np.arange(T)
    dist = np.abs(t[:, None] - t[None, :]) - 1          # (T,T); -1 on the diagonal
    eye = np.eye(T, dtype=bool)
    for c0 in range(0, C, channel_block):
        c1 = min(C, c0 + channel_block)
        wc = w[c0:c1]
        uc = u[c0:c1]
        for b in range(B):
            kk = k[b, :, c0:c1]                             # (T,c)
            vv = v[b, :, c0:c1]
            # logit[t,i,c]
            logit = kk[None, :, :] - dist[:, :, None] * wc[None, None, :]
            diag = uc[None, :] + kk                         # (T,c)
            logit[eye] = diag
            m = logit.max(axis=1, keepdims=True)
            e = np.exp(logit - m)
            y[b, :, c0:c1] = (e * vv[None, :, :]).sum(axis=1) / e.sum(axis=1)
    return y


def biwkv_scan(w, u, k, v, dtype=np.float64):
    """Two-pass stabilised recurrence (forward state, then backward state).

    State update = bi_wkv_kernel.cu:103-108, output combine = :95-100, with the
    future state built by a second (descending) pass instead of the kernel's
    subtractive update at :109-113.
    """
    w = np.asarray(w, dtype)
    u = np.asarray(u, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    B, T, C = k.shape
    # forward pass: state before token t
    a = np.zeros((B, C), dtype)
    b = np.zeros((B, C), dtype)
    p = np.full((B, C), MIN_VALUE, dtype)
    A = np.empty((T, B, C), dtype)
    Bd = np.empty((T, B, C), dtype)
    P = np.empty((T, B, C), dtype)
    for t in range(T):
        A[t], Bd[t], P[t] = a, b, p
        kt, vt = k[:, t], v[:, t]
        q = np.maximum(p - w, kt)
        e1 = np.exp(p - w - q)
        e2 = np.exp(kt - q)
        a = e1 * a + e2 * vt
        b = e1 * b + e2
        p = q
    y = np.empty((B, T, C), dtype)
    c = np.zeros((B, C), dtype)
    d = np.zeros((B, C), dtype)
    o = np.full((B, C), MIN_VALUE, dtype)
    for t in range(T - 1, -1, -1):
        kt, vt = k[:, t], v[:, t]
        m = np.maximum(np.maximum(P[t], o), u + kt)
        ea = np.exp(P[t] - m)
        ec = np.exp(o - m)
        eu = np.exp(u + kt - m)
        y[:, t] = (ea * A[t] + ec * c + eu * vt) / (ea * Bd[t] + ec * d + eu)
        q = np.maximum(o - w, kt)
        e1 = np.exp(o - w - q)
        e2 = np.exp(kt - q)
        c = e1 * c + e2 * vt
        d = e1 * d + e2
        o = q
    return y


def biwkv_grads_closed(w, u, k, v, gy):
    """(gw, gu, gk, gv) by torch.autograd through the float64 closed form.

    Follows the contract of bi_wkv_backward
    (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:35-47):
    gw,gu are (C,) summed over batch and tokens; gk,gv are (B,T,C).
    """
    import torch
    w = torch.tensor(np.asarray(w, np.float64), requires_grad=True)
    u = torch.tensor(np.asarray(u, np.float64), requires_grad=True)
    k = torch.tensor(np.asarray(k, np.float64), requires_grad=True)
    v = torch.tensor(np.asarray(v, np.float64), requires_grad=True)
    gy = torch.tensor(np.asarray(gy, np.float64))
    B, T, C = k.shape
    t = torch.arange(T)
    dist = ((t[:, None] - t[None, :]).abs() - 1).to(torch.float64)   # (T,T)
    eye = torch.eye(T, dtype=torch.bool)
    logit = k[:, None, :, :] - dist[None, :, :, None] * w[None, None, None, :]   # (B,t,i,C)
    diag = (u[None, None, :] + k)                                                # (B,T,C)
    logit = torch.where(eye[None, :, :, None], diag[:, :, None, :].expand(B, T, T, C), logit)
    p = torch.softmax(logit, dim=2)
    y = (p * v[:, None, :, :]).sum(dim=2)
    y.backward(gy)
    return (w.grad.numpy(), u.grad.numpy(), k.grad.numpy(), v.grad.numpy())
