"""Float64 model of the reference Bi-WKV forward kernel's 32-way token split.  TEST INFRASTRUCTURE ONLY.

The reference kernel (classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:21-116) gives each of
32 lanes a chunk of L = ceil(T/32) consecutive tokens of one (batch, channel) sequence and works in three steps.
This file restates those steps as sums (it is not a line-by-line copy; the kernel carries every sum as a
max-normalised pair, which changes nothing in exact arithmetic, and its EPS = 1e-6 in the normalised denominator is
left out):

  1. per chunk q = [s_q, e_q):   P_q = sum_i e^{k_i - w (e_q - i)} v_i     (weights counted from ONE PAST the chunk end)
                                 F_q = sum_i e^{k_i - w (i - s_q)} v_i     (weights counted from the chunk start)
  2. carries at the chunk start: A_p = sum_{q<p} e^{-w L (p-q-1)} P_q      = sum_{i<s_p} e^{k_i - w (s_p - i)} v_i
                                 C_p = sum_{q>=p} e^{-w L (q-p)} F_q - e^{k_s} v_s = sum_{i>s_p} e^{k_i - w (i - s_p)} v_i
  3. inside the chunk, token by token:
         y_t = (A + C + e^{u + k_t} v_t) / (same with v -> 1)
         A <- e^{-w} A + e^{k_t} v_t ,      C <- e^{w} (C - e^{k_{t+1}} v_{t+1})

The formula the operator is defined by weights a token at distance |t - i| with e^{-w (|t-i| - 1)}; the updates of
step 3 keep exactly that convention, but the carries of step 2 use the exponent |t - i|: every chunk starts from
carries that are e^{-w} times what the formula asks for.  `carry_fix=True` multiplies A_p and C_p by e^{w}.
"""
import numpy as np

TOKEN_SPLIT = 32      # bi_wkv_kernel.cu:17


def biwkv_chunk_carry(w, u, k, v, carry_fix=False, split=TOKEN_SPLIT):
    """w, u: (C,), k, v: (T, C) -> y (T, C), float64 throughout."""
    w = np.asarray(w, np.float64)
    u = np.asarray(u, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    T, C = k.shape
    L = -(-T // split)
    E = np.exp(k)
    starts = [min(p * L, T) for p in range(split)]
    ends = [min(s + L, T) for s in starts]
    P = np.zeros((split, 2, C))
    F = np.zeros((split, 2, C))
    for q, (s, e) in enumerate(zip(starts, ends)):
        for i in range(s, e):
            P[q, 0] += np.exp(-w * (e - i)) * E[i] * v[i]
            P[q, 1] += np.exp(-w * (e - i)) * E[i]
            F[q, 0] += np.exp(-w * (i - s)) * E[i] * v[i]
            F[q, 1] += np.exp(-w * (i - s)) * E[i]
    y = np.zeros((T, C))
    for p, (s, e) in enumerate(zip(starts, ends)):
        if s >= e:
            continue
        A = sum((np.exp(-w * L * (p - q - 1)) * P[q] for q in range(p)), np.zeros((2, C)))
        Cf = sum((np.exp(-w * L * (q - p)) * F[q] for q in range(p, split)), np.zeros((2, C)))
        Cf = Cf - np.stack([E[s] * v[s], E[s]])
        if carry_fix:
            A, Cf = A * np.exp(w), Cf * np.exp(w)
        for t in range(s, e):
            bonus = np.exp(u) * E[t]
            y[t] = (A[0] + Cf[0] + bonus * v[t]) / (A[1] + Cf[1] + bonus)
            A = np.exp(-w) * A + np.stack([E[t] * v[t], E[t]])
            n = (t + 1) % T
            Cf = np.exp(w) * (Cf - np.stack([E[n] * v[n], E[n]]))
    return y
