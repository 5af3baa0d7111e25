"""Writes the golden fixtures in this directory from the float64 closed forms in oracle/.

The reference ships no vectors for the WKV operators, so these are produced here:
inputs are drawn with NumPy's PCG64 from the seeds below, rounded to fp32 (so that a
GPU kernel sees bit-identical inputs), and the expected outputs are float64 results of
the O(T^2) closed forms.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import biwkv, wkv6, qshift  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
f32 = lambda a: np.asarray(a, np.float32)


def baseline_wu(C, T, channels=None):
    """w_c = (-5 + 8 c/(C-1))/T ; u_c = (ln 0.3 + 0.5(((c+1)%3)-1))/T  (benchmark config 0)."""
    c = np.arange(C) if channels is None else np.asarray(channels)
    w = (-5.0 + 8.0 * (c / max(C - 1, 1))) / T
    u = (np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T
    return f32(w), f32(u)


def make_biwkv():
    out = {}
    cases = []
    # (name, B, T, C, seed, kind)
    for T in (1, 2, 3, 31, 32, 33, 65):
        cases.append((f"T{T}_C32", 2, T, 32, 100 + T, "baseline"))
    cases.append(("T196_cfg0sub", 1, 196, 16, 7, "cfg0sub"))
    cases.append(("T40_wide", 1, 40, 32, 11, "wide"))        # large |w|, large |u|
    cases.append(("T50_outlier", 2, 50, 32, 13, "outlier"))  # 8x scaled tokens
    for name, B, T, C, seed, kind in cases:
        rng = np.random.default_rng(seed)
        k = f32(rng.standard_normal((B, T, C)))
        v = f32(rng.standard_normal((B, T, C)))
        if kind == "baseline":
            w, u = baseline_wu(C, T)
        elif kind == "cfg0sub":
            w, u = baseline_wu(192, T, channels=np.arange(0, 192, 12))
        elif kind == "wide":
            w = f32(rng.uniform(-3.0, 6.0, C))
            u = f32(rng.uniform(-6.0, 6.0, C))
        elif kind == "outlier":
            w, u = baseline_wu(C, T)
            mask = rng.random((B, T, 1)) < 0.1
            k = f32(np.where(mask, 8 * k, k))
            v = f32(np.where(mask, 8 * v, v))
        y = biwkv.biwkv_closed(w, u, k, v)
        for nm, arr in (("w", w), ("u", u), ("k", k), ("v", v), ("y", y)):
            out[f"{name}/{nm}"] = arr
    # one gradient case (autograd through the closed form)
    rng = np.random.default_rng(21)
    B, T, C = 2, 19, 8
    k = f32(rng.standard_normal((B, T, C)))
    v = f32(rng.standard_normal((B, T, C)))
    gy = f32(rng.standard_normal((B, T, C)))
    w = f32(rng.uniform(-0.3, 0.3, C))
    u = f32(rng.uniform(-0.5, 0.5, C))
    gw, gu, gk, gv = biwkv.biwkv_grads_closed(w, u, k, v, gy)
    for nm, arr in (("w", w), ("u", u), ("k", k), ("v", v), ("gy", gy),
                    ("gw", gw), ("gu", gu), ("gk", gk), ("gv", gv),
                    ("y", biwkv.biwkv_closed(w, u, k, v))):
        out[f"grad_T19_C8/{nm}"] = arr
    np.savez_compressed(os.path.join(HERE, "biwkv_golden.npz"), **out)


def make_wkv6():
    out = {}
    # (name, B, T, H, N, seed)
    for name, B, T, H, N, seed in (("T1", 1, 1, 1, 64, 1), ("T2", 1, 2, 2, 64, 2), ("T17", 2, 17, 2, 64, 3),
                                   ("T33", 1, 33, 1, 64, 4), ("T70", 1, 70, 2, 64, 5)):
        rng = np.random.default_rng(seed)
        C = H * N
        r, k, v = (f32(rng.standard_normal((B, T, C))) for _ in range(3))
        w_raw = f32(rng.normal(-0.5, 0.5, (B, T, C)))
        u = f32(rng.normal(0.0, 0.1, (H, N)))
        y = wkv6.wkv6_closed(r, k, v, w_raw, u, H)
        for nm, arr in (("r", r), ("k", k), ("v", v), ("w", w_raw), ("u", u), ("y", y)):
            out[f"{name}/{nm}"] = arr
    rng = np.random.default_rng(31)
    B, T, H, N = 1, 9, 1, 64
    C = H * N
    r, k, v = (f32(rng.standard_normal((B, T, C))) for _ in range(3))
    w_raw = f32(rng.normal(-0.5, 0.5, (B, T, C)))
    u = f32(rng.normal(0.0, 0.1, (H, N)))
    gy = f32(rng.standard_normal((B, T, C)))
    gr, gk, gv, gw, gu = wkv6.wkv6_grads_closed(r, k, v, w_raw, u, H, gy)
    for nm, arr in (("r", r), ("k", k), ("v", v), ("w", w_raw), ("u", u), ("gy", gy),
                    ("gr", gr), ("gk", gk), ("gv", gv), ("gw", gw), ("gu", gu),
                    ("y", wkv6.wkv6_closed(r, k, v, w_raw, u, H))):
        out[f"grad_T9/{nm}"] = arr
    np.savez_compressed(os.path.join(HERE, "wkv6_golden.npz"), **out)


def make_qshift():
    out = {}
    rng = np.random.default_rng(41)
    x = f32(rng.standard_normal((2, 3 * 5, 16)))
    out["q/x"] = x
    out["q/y"] = qshift.q_shift_loops(x, 1, 0.25, (3, 5))
    x = f32(rng.standard_normal((1, 4 * 3 + 1, 16)))
    out["mh/x"] = x
    out["mh/y"] = qshift.q_shift_multihead_loops(x, 1, 8, (4, 3), with_cls_token=True)
    np.savez_compressed(os.path.join(HERE, "qshift_golden.npz"), **out)


if __name__ == "__main__":
    make_biwkv()
    make_wkv6()
    make_qshift()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
