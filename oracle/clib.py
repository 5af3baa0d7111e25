"""ctypes loader for the plain-C oracle (oracle/c/libwkv_oracle.so).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "c", "libwkv_oracle.so")
_lib = None


def build(force=False):
    """Compile the C oracle with the Makefile beside it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", os.path.join(_HERE, "c")], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        lib = ctypes.CDLL(_SO)
        fp = ctypes.POINTER(ctypes.c_float)
        dp = ctypes.POINTER(ctypes.c_double)
        lib.oracle_biwkv_fwd.argtypes = [fp, fp, fp, fp, dp, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.oracle_biwkv_fwd.restype = ctypes.c_int
        lib.oracle_wkv6_fwd.argtypes = [fp, fp, fp, fp, fp, dp] + [ctypes.c_int] * 4
        lib.oracle_wkv6_fwd.restype = ctypes.c_int
        lib.oracle_biwkv_bwd.argtypes = [fp] * 5 + [dp] * 4 + [ctypes.c_int] * 3
        lib.oracle_biwkv_bwd.restype = ctypes.c_int
        lib.oracle_wkv6_bwd.argtypes = [fp] * 6 + [dp] * 5 + [ctypes.c_int] * 4
        lib.oracle_wkv6_bwd.restype = ctypes.c_int
        _lib = lib
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def biwkv_fwd(w, u, k, v):
    """fp32 inputs (anything array-like), float64 output (B,T,C)."""
    lib = load()
    w, pw = _f32(w)
    u, pu = _f32(u)
    k, pk = _f32(k)
    v, pv = _f32(v)
    B, T, C = k.shape
    assert w.shape == (C,) and u.shape == (C,) and v.shape == k.shape
    y = np.empty((B, T, C), np.float64)
    rc = lib.oracle_biwkv_fwd(pw, pu, pk, pv, y.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), B, T, C)
    if rc:
        raise RuntimeError(f"oracle_biwkv_fwd failed with status {rc}")
    return y


def wkv6_fwd(r, k, v, w_raw, u, H):
    lib = load()
    r, pr = _f32(r)
    k, pk = _f32(k)
    v, pv = _f32(v)
    w_raw, pw = _f32(w_raw)
    u, pu = _f32(u)
    B, T, C = r.shape
    assert k.shape == r.shape == v.shape == w_raw.shape and u.size == C
    y = np.empty((B, T, C), np.float64)
    rc = lib.oracle_wkv6_fwd(pr, pk, pv, pw, pu, y.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), B, T, C, H)
    if rc:
        raise RuntimeError(f"oracle_wkv6_fwd failed with status {rc}")
    return y


def _dp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def biwkv_bwd(w, u, k, v, gy):
    """(gw, gu, gk, gv) in float64 from the definition (softmax form, O(T^2) per sequence); gw, gu summed over
    batch and tokens."""
    lib = load()
    w, pw = _f32(w)
    u, pu = _f32(u)
    k, pk = _f32(k)
    v, pv = _f32(v)
    gy, pg = _f32(gy)
    B, T, C = k.shape
    assert w.shape == (C,) and u.shape == (C,) and v.shape == k.shape and gy.shape == k.shape
    gw, gu = np.empty(C, np.float64), np.empty(C, np.float64)
    gk, gv = np.empty((B, T, C), np.float64), np.empty((B, T, C), np.float64)
    rc = lib.oracle_biwkv_bwd(pw, pu, pk, pv, pg, _dp(gw), _dp(gu), _dp(gk), _dp(gv), B, T, C)
    if rc:
        raise RuntimeError(f"oracle_biwkv_bwd failed with status {rc}")
    return gw, gu, gk, gv


def wkv6_bwd(r, k, v, w_raw, u, gy, H):
    """(gr, gk, gv, gw, gu) in float64; gw with respect to the raw decay logit, gu (H, N) summed over the batch."""
    lib = load()
    r, pr = _f32(r)
    k, pk = _f32(k)
    v, pv = _f32(v)
    w_raw, pw = _f32(w_raw)
    u, pu = _f32(u)
    gy, pg = _f32(gy)
    B, T, C = r.shape
    assert k.shape == r.shape == v.shape == w_raw.shape == gy.shape and u.size == C and C % H == 0
    outs = [np.empty((B, T, C), np.float64) for _ in range(4)]
    gu = np.empty((H, C // H), np.float64)
    rc = lib.oracle_wkv6_bwd(pr, pk, pv, pw, pu, pg, *[_dp(o) for o in outs], _dp(gu), B, T, C, H)
    if rc:
        raise RuntimeError(f"oracle_wkv6_bwd failed with status {rc}")
    return (*outs, gu)
