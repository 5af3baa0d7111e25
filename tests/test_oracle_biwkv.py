"""Pins the Bi-WKV oracle: independent restatements must agree, and the formula must reduce
to textbook routines in the special cases the mathematics fixes."""
import numpy as np
import pytest

from conftest import load_golden
from oracle import biwkv, clib, torch_eager


def _rand(B, T, C, seed, wlo=-0.5, whi=0.5):
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((B, T, C))
    v = rng.standard_normal((B, T, C))
    w = rng.uniform(wlo, whi, C)
    u = rng.uniform(-1, 1, C)
    return w, u, k, v


@pytest.mark.parametrize("T", [1, 2, 5, 64, 196])
def test_closed_vs_scan(T):
    w, u, k, v = _rand(2, T, 6, T)
    assert np.abs(biwkv.biwkv_closed(w, u, k, v) - biwkv.biwkv_scan(w, u, k, v)).max() < 1e-12


def test_closed_vs_scan_long_with_outliers():
    rng = np.random.default_rng(5)
    T, C = 4150, 3
    k = rng.standard_normal((1, T, C))
    v = rng.standard_normal((1, T, C))
    mask = rng.random((1, T, 1)) < 0.01
    k = np.where(mask, 8 * k, k)
    v = np.where(mask, 8 * v, v)
    w = np.array([-5.0, 0.0, 3.0]) / T
    u = np.array([0.1, -0.2, 0.0]) / T
    assert np.abs(biwkv.biwkv_closed(w, u, k, v) - biwkv.biwkv_scan(w, u, k, v)).max() < 1e-11


def test_c_and_torch_restatements_agree():
    w, u, k, v = _rand(3, 41, 10, 3)
    f = lambda a: a.astype(np.float32)
    ref = biwkv.biwkv_closed(f(w), f(u), f(k), f(v))
    assert np.abs(clib.biwkv_fwd(w, u, k, v) - ref).max() < 1e-12
    import torch
    yt = torch_eager.biwkv_eager(*(torch.tensor(f(a)).double() for a in (w, u, k, v))).numpy()
    assert np.abs(yt - ref).max() < 1e-12


def test_softmax_reduction():
    """w = u = 0: every token sees the same softmax(k)-weighted mean of v."""
    import torch
    _, _, k, v = _rand(2, 37, 5, 9)
    z = np.zeros(5)
    y = biwkv.biwkv_closed(z, z, k, v)
    p = torch.softmax(torch.tensor(k), dim=1).numpy()
    want = (p * v).sum(axis=1, keepdims=True)
    assert np.abs(y - want).max() < 1e-13


def test_single_token_and_big_bonus():
    w, u, k, v = _rand(2, 1, 4, 1)
    assert np.abs(biwkv.biwkv_closed(w, u, k, v) - v).max() < 1e-15
    w, u, k, v = _rand(2, 9, 4, 2)
    y = biwkv.biwkv_scan(w, np.full(4, 80.0), k, v)
    assert np.abs(y - v).max() < 1e-12


def test_strong_decay_three_term_mean():
    """w -> +inf: only t-1, t, t+1 survive (neighbours carry decay exponent 0)."""
    _, u, k, v = _rand(1, 12, 3, 4)
    y = biwkv.biwkv_scan(np.full(3, 500.0), u, k, v)
    T = 12
    for t in range(T):
        num = np.exp(u + k[0, t]) * v[0, t]
        den = np.exp(u + k[0, t])
        for i in (t - 1, t + 1):
            if 0 <= i < T:
                num = num + np.exp(k[0, i]) * v[0, i]
                den = den + np.exp(k[0, i])
        assert np.abs(y[0, t] - num / den).max() < 1e-12


def test_two_tokens_by_hand():
    """T=2: y_0 = (e^{k1} v1 + e^{u+k0} v0)/(e^{k1}+e^{u+k0}); w must not matter."""
    k = np.array([[[0.3], [-1.1]]])
    v = np.array([[[2.0], [5.0]]])
    u = np.array([0.7])
    for w in (-3.0, 0.0, 4.0):
        y = biwkv.biwkv_closed(np.array([w]), u, k, v)
        y0 = (np.exp(-1.1) * 5 + np.exp(1.0) * 2) / (np.exp(-1.1) + np.exp(1.0))
        y1 = (np.exp(0.3) * 2 + np.exp(-0.4) * 5) / (np.exp(0.3) + np.exp(-0.4))
        assert abs(y[0, 0, 0] - y0) < 1e-14 and abs(y[0, 1, 0] - y1) < 1e-14


def test_three_tokens_decay_sign():
    """T=3: the only decayed pair is (0,2) with factor e^{-w}; a wrong sign or an
    off-by-one in |t-i|-1 changes this value."""
    k = np.zeros((1, 3, 1))
    v = np.array([[[1.0], [0.0], [0.0]]])
    w = np.array([np.log(4.0)])
    u = np.array([0.0])
    y = biwkv.biwkv_closed(w, u, k, v)
    assert abs(y[0, 2, 0] - 0.25 / (0.25 + 1 + 1)) < 1e-15
    assert abs(y[0, 1, 0] - 1 / 3) < 1e-15
    assert abs(y[0, 0, 0] - 1 / (1 + 1 + 0.25)) < 1e-15


def test_invariants():
    w, u, k, v = _rand(2, 23, 7, 6)
    y = biwkv.biwkv_closed(w, u, k, v)
    # convexity
    assert (y <= v.max(axis=1, keepdims=True) + 1e-12).all() and (y >= v.min(axis=1, keepdims=True) - 1e-12).all()
    # constant v
    assert np.abs(biwkv.biwkv_closed(w, u, k, np.full_like(v, 1.7)) - 1.7).max() < 1e-13
    # k-shift invariance
    assert np.abs(biwkv.biwkv_closed(w, u, k + 3.3, v) - y).max() < 1e-12
    # reversal symmetry
    yr = biwkv.biwkv_closed(w, u, k[:, ::-1], v[:, ::-1])
    assert np.abs(yr[:, ::-1] - y).max() < 1e-13
    # channel independence
    perm = np.random.default_rng(0).permutation(7)
    yp = biwkv.biwkv_closed(w[perm], u[perm], k[..., perm], v[..., perm])
    assert np.abs(yp - y[..., perm]).max() == 0


def test_golden_fixtures_match_scan_and_c():
    g = load_golden("biwkv_golden")
    assert len(g) >= 10
    for name, a in g.items():
        ys = biwkv.biwkv_scan(a["w"], a["u"], a["k"], a["v"])
        assert np.abs(ys - a["y"]).max() < 1e-11, name
        yc = clib.biwkv_fwd(a["w"], a["u"], a["k"], a["v"])
        assert np.abs(yc - a["y"]).max() < 1e-11, name


def test_gradients_finite_difference_and_identities():
    g = load_golden("biwkv_golden")["grad_T19_C8"]
    w, u, k, v, gy = (g[n].astype(np.float64) for n in ("w", "u", "k", "v", "gy"))
    f = lambda w_, u_, k_, v_: float((biwkv.biwkv_scan(w_, u_, k_, v_) * gy).sum())
    eps = 1e-6
    rng = np.random.default_rng(0)
    for _ in range(5):
        b, t, c = rng.integers(2), rng.integers(19), rng.integers(8)
        kk = k.copy(); kk[b, t, c] += eps
        km = k.copy(); km[b, t, c] -= eps
        assert abs((f(w, u, kk, v) - f(w, u, km, v)) / (2 * eps) - g["gk"][b, t, c]) < 1e-7
        vv = v.copy(); vv[b, t, c] += eps
        vm = v.copy(); vm[b, t, c] -= eps
        assert abs((f(w, u, k, vv) - f(w, u, k, vm)) / (2 * eps) - g["gv"][b, t, c]) < 1e-7
    for c in range(8):
        ww = w.copy(); ww[c] += eps
        wm = w.copy(); wm[c] -= eps
        assert abs((f(ww, u, k, v) - f(wm, u, k, v)) / (2 * eps) - g["gw"][c]) < 1e-6
        uu = u.copy(); uu[c] += eps
        um = u.copy(); um[c] -= eps
        assert abs((f(w, uu, k, v) - f(w, um, k, v)) / (2 * eps) - g["gu"][c]) < 1e-6
    # k -> k + const leaves y unchanged; the weights sum to one
    assert np.abs(g["gk"].sum(axis=1)).max() < 1e-12
    assert np.abs(g["gv"].sum(axis=1) - gy.sum(axis=1)).max() < 1e-12
