"""Bidirectional RWKV-6 (wkv6) oracle, float64 NumPy.  Test infrastructure only.

Contract of the operator (classification/mmcls_custom/models/backbones/vrwkv6.py:34-73):
the caller passes the raw decay logit ``w`` (B,T,C); the Function forms
``ew = -exp(w)`` (:48) and the kernel uses ``d = exp(ew)`` per token and channel
(classification/mmcls_custom/models/backbones/cuda_v6/wkv6_cuda.cu:26).

Per batch b, head h (N = C/H channels), key index j, value index i:

    y_t[i] = sum_j r_t[j] * ( u[h,j] k_t[j] v_t[i] + S_t[j,i] + S'_t[j,i] )
    S_0 = 0,       S_{t+1}  = diag(d_t) S_t  + k_t v_t^T     (ascending,  wkv6_cuda.cu:58-96)
    S'_{T-1} = 0,  S'_{t-1} = diag(d_t) S'_t + k_t v_t^T     (descending, wkv6_cuda.cu:23-57)

both states being used before their update; the bonus u enters once (:85-88).
"""
import numpy as np


def wkv6_scan(r, k, v, w_raw, u, H, dtype=np.float64):
    """Sequential two-direction recurrence.  r,k,v,w_raw: (B,T,C); u: (H,N)."""
    r = np.asarray(r, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    w_raw = np.asarray(w_raw, dtype)
    u = np.asarray(u, dtype)
    B, T, C = r.shape
    N = C // H
    assert N * H == C and u.shape == (H, N)
    r4 = r.reshape(B, T, H, N)
    k4 = k.reshape(B, T, H, N)
    v4 = v.reshape(B, T, H, N)
    d4 = np.exp(-np.exp(w_raw)).reshape(B, T, H, N)
    y = np.zeros((B, T, H, N), dtype)
    S = np.zeros((B, H, N, N), dtype)                 # [j (key), i (value)]
    for t in range(T - 1, -1, -1):                    # descending pass
        y[:, t] = np.einsum('bhj,bhji->bhi', r4[:, t], S)
        S = d4[:, t][..., None] * S + k4[:, t][..., None] * v4[:, t][:, :, None, :]
    S = np.zeros((B, H, N, N), dtype)
    for t in range(T):                                # ascending pass
        kv = k4[:, t][..., None] * v4[:, t][:, :, None, :]
        y[:, t] += np.einsum('bhj,bhji->bhi', r4[:, t], u[None, :, :, None] * kv + S)
        S = d4[:, t][..., None] * S + kv
    return y.reshape(B, T, C)


def wkv6_closed(r, k, v, w_raw, u, H):
    """O(T^2) closed form with cumulative log-decay.

    y_t = sum_j r_t[j] ( u_j k_t[j] v_t + sum_{s != t} (prod_{l strictly between s and t} d_l[j]) k_s[j] v_s )
    """
    r = np.asarray(r, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    ld = -np.exp(np.asarray(w_raw, np.float64))       # log d, (B,T,C)
    u = np.asarray(u, np.float64)
    B, T, C = r.shape
    N = C // H
    y = np.zeros((B, T, C), np.float64)
    cum = np.cumsum(ld, axis=1)                       # inclusive
    cum_ex = cum - ld                                 # exclusive: sum_{l<t}
    for b in range(B):
        for h in range(H):
            sl = slice(h * N, (h + 1) * N)
            rr, kk, vv = r[b, :, sl], k[b, :, sl], v[b, :, sl]
            ci, ce = cum[b, :, sl], cum_ex[b, :, sl]
            A = np.zeros((T, T), np.float64)
            for t in range(T):
                # s < t : sum_{l=s+1}^{t-1} ld_l = cum_ex[t] - cum[s]
                if t > 0:
                    dec = np.exp(ce[t][None, :] - ci[:t])            # (t,N)
                    A[t, :t] = (rr[t][None, :] * kk[:t] * dec).sum(-1)
                # s > t : sum_{l=t+1}^{s-1} ld_l = cum_ex[s] - cum[t]
                if t < T - 1:
                    dec = np.exp(ce[t + 1:] - ci[t][None, :])
                    A[t, t + 1:] = (rr[t][None, :] * kk[t + 1:] * dec).sum(-1)
                A[t, t] = (rr[t] * u[h] * kk[t]).sum()
            y[b, :, sl] = A @ vv
    return y


def wkv6_grads_closed(r, k, v, w_raw, u, H, gy):
    """(gr, gk, gv, gw, gu) by torch.autograd through a float64 closed form.

    Contract of WKV_6.backward (vrwkv6.py:55-70): gr,gk,gv,gw are (B,T,C) with gw
    the gradient w.r.t. the *raw* decay logit (the kernels multiply by ew,
    wkv6_cuda.cu:248,277); gu is summed over the batch and shaped (H,N).
    """
    import torch
    tt = lambda a: torch.tensor(np.asarray(a, np.float64), requires_grad=True)
    r, k, v, w_raw, u = tt(r), tt(k), tt(v), tt(w_raw), tt(u)
    gy = torch.tensor(np.asarray(gy, np.float64))
    B, T, C = r.shape
    N = C // H
    r4, k4, v4 = (x.view(B, T, H, N) for x in (r, k, v))
    ld = (-torch.exp(w_raw)).view(B, T, H, N)
    cum = torch.cumsum(ld, dim=1)
    cum_ex = cum - ld
    # expo[b,t,s,h,j]: t>s -> cum_ex[t]-cum[s];  t<s -> cum_ex[s]-cum[t]
    lo = cum_ex[:, :, None] - cum[:, None, :]          # (B,t,s,H,N), valid for s<t
    hi = cum_ex[:, None, :] - cum[:, :, None]          # valid for s>t
    idx = torch.arange(T)
    lower = (idx[:, None] > idx[None, :])[None, :, :, None, None]
    upper = (idx[:, None] < idx[None, :])[None, :, :, None, None]
    zero = torch.zeros((), dtype=torch.float64)
    dec = torch.where(lower, torch.exp(torch.where(lower, lo, zero)), zero) \
        + torch.where(upper, torch.exp(torch.where(upper, hi, zero)), zero)
    A = torch.einsum('bthj,bshj,btshj->bhts', r4, k4, dec)
    diag = torch.einsum('bthj,hj,bthj->bht', r4, u, k4)
    A = A + torch.diag_embed(diag)
    y = torch.einsum('bhts,bshi->bthi', A, v4).reshape(B, T, C)
    y.backward(gy)
    return tuple(x.grad.numpy() for x in (r, k, v, w_raw, u))
