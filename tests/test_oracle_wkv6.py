"""Pins the wkv6 oracle."""
import numpy as np
import pytest

from conftest import load_golden
from oracle import wkv6, clib, torch_eager


def _rand(B, T, H, N, seed):
    rng = np.random.default_rng(seed)
    C = H * N
    r, k, v = (rng.standard_normal((B, T, C)) for _ in range(3))
    w = rng.normal(-0.5, 0.5, (B, T, C))
    u = rng.normal(0, 0.1, (H, N))
    return r, k, v, w, u


@pytest.mark.parametrize("T", [1, 2, 3, 20])
def test_scan_vs_closed(T):
    r, k, v, w, u = _rand(2, T, 2, 8, T)
    assert np.abs(wkv6.wkv6_scan(r, k, v, w, u, 2) - wkv6.wkv6_closed(r, k, v, w, u, 2)).max() < 1e-12


def test_c_and_torch_restatements_agree():
    import torch
    r, k, v, w, u = _rand(2, 15, 2, 8, 7)
    f = lambda a: a.astype(np.float32)
    ref = wkv6.wkv6_scan(f(r), f(k), f(v), f(w), f(u), 2)
    assert np.abs(clib.wkv6_fwd(r, k, v, w, u, 2) - ref).max() < 1e-12
    yt = torch_eager.wkv6_eager(*(torch.tensor(f(a)).double() for a in (r, k, v, w, u)), 2).numpy()
    assert np.abs(yt - ref).max() < 1e-12


def test_no_decay_is_linear_attention():
    """d == 1 (w_raw -> -inf): y_t = r_t . (sum_{s != t} k_s v_s^T + diag(u) k_t v_t^T)."""
    r, k, v, _, u = _rand(1, 11, 2, 4, 3)
    H, N = 2, 4
    w = np.full_like(r, -80.0)
    y = wkv6.wkv6_scan(r, k, v, w, u, H)
    r4, k4, v4 = (a.reshape(1, 11, H, N) for a in (r, k, v))
    A = np.einsum('bthj,bshj->bhts', r4, k4)
    Au = np.einsum('bthj,hj,bthj->bht', r4, u, k4)
    eye = np.eye(11, dtype=bool)
    A = np.where(eye, 0.0, A) + np.einsum('bht,ts->bhts', Au, np.eye(11))
    want = np.einsum('bhts,bshi->bthi', A, v4).reshape(1, 11, H * N)
    assert np.abs(y - want).max() < 1e-12


def test_full_decay_three_tokens():
    """d == 0: only s = t-1, t, t+1 contribute (neighbours have an empty decay product)."""
    r, k, v, _, u = _rand(1, 7, 1, 4, 5)
    w = np.full_like(r, 6.0)       # exp(-exp(6)) == 0 in double
    y = wkv6.wkv6_scan(r, k, v, w, u, 1)
    for t in range(7):
        want = (r[0, t] * u[0] * k[0, t]).sum() * v[0, t]
        for s in (t - 1, t + 1):
            if 0 <= s < 7:
                want = want + (r[0, t] * k[0, s]).sum() * v[0, s]
        assert np.abs(y[0, t] - want).max() < 1e-12


def test_decay_applies_strictly_between():
    """T=3, one channel: the (0,2) pair is decayed by d_1 only."""
    r = np.ones((1, 3, 1)); k = np.ones((1, 3, 1))
    v = np.array([[[1.0], [0.0], [0.0]]])
    w = np.log(-np.log(np.array([0.9, 0.5, 0.7]))).reshape(1, 3, 1)   # d = .9 .5 .7
    u = np.array([[2.0]])
    y = wkv6.wkv6_closed(r, k, v, w, u, 1)
    assert abs(y[0, 0, 0] - 2.0) < 1e-14      # bonus only
    assert abs(y[0, 1, 0] - 1.0) < 1e-14      # neighbour, no decay
    assert abs(y[0, 2, 0] - 0.5) < 1e-14      # through d_1
    assert np.abs(wkv6.wkv6_scan(r, k, v, w, u, 1) - y).max() < 1e-14


def test_single_token_heads_reversal():
    r, k, v, w, u = _rand(2, 1, 2, 4, 9)
    y = wkv6.wkv6_scan(r, k, v, w, u, 2)
    r4, k4, v4 = (a.reshape(2, 1, 2, 4) for a in (r, k, v))
    want = (np.einsum('bthj,hj,bthj->bth', r4, u, k4)[..., None] * v4).reshape(2, 1, 8)
    assert np.abs(y - want).max() < 1e-14
    r, k, v, w, u = _rand(2, 13, 2, 4, 10)
    y = wkv6.wkv6_scan(r, k, v, w, u, 2)
    yr = wkv6.wkv6_scan(r[:, ::-1], k[:, ::-1], v[:, ::-1], w[:, ::-1], u, 2)
    assert np.abs(yr[:, ::-1] - y).max() < 1e-12
    # heads are independent: swapping heads swaps outputs
    sw = lambda a: np.concatenate([a[..., 4:], a[..., :4]], axis=-1)
    ys = wkv6.wkv6_scan(sw(r), sw(k), sw(v), sw(w), u[::-1], 2)
    assert np.abs(sw(ys) - y).max() < 1e-13


def test_golden_fixtures_match_scan_and_c():
    g = load_golden("wkv6_golden")
    for name, a in g.items():
        H = a["u"].shape[0]
        ys = wkv6.wkv6_scan(a["r"], a["k"], a["v"], a["w"], a["u"], H)
        assert np.abs(ys - a["y"]).max() < 1e-10, name
        yc = clib.wkv6_fwd(a["r"], a["k"], a["v"], a["w"], a["u"], H)
        assert np.abs(yc - a["y"]).max() < 1e-10, name


def test_gradients_finite_difference():
    g = load_golden("wkv6_golden")["grad_T9"]
    r, k, v, w, u, gy = (g[n].astype(np.float64) for n in ("r", "k", "v", "w", "u", "gy"))
    f = lambda *a: float((wkv6.wkv6_scan(*a, 1) * gy).sum())
    args = [r, k, v, w, u]
    names = ["gr", "gk", "gv", "gw", "gu"]
    rng = np.random.default_rng(1)
    eps = 1e-6
    for ai in range(5):
        for _ in range(4):
            idx = tuple(rng.integers(s) for s in args[ai].shape)
            ap = [a.copy() for a in args]; ap[ai][idx] += eps
            am = [a.copy() for a in args]; am[ai][idx] -= eps
            fd = (f(*ap) - f(*am)) / (2 * eps)
            assert abs(fd - g[names[ai]][idx]) < 1e-6 * max(1.0, abs(fd)), (names[ai], idx)
