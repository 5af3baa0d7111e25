"""Pins the gradient routines of the plain-C oracle (oracle/c/wkv_oracle.c): autograd through the float64 closed
forms on small shapes (including negative and strong decays), central finite differences of the C forward, and the
identities the forward's invariances imply (sum_t gk = 0, sum_t gv = sum_t gy)."""
import numpy as np
import pytest

from oracle import biwkv, clib, wkv6


def _biwkv_case(B, T, C, seed, wlo=-0.03, whi=0.02):
    rng = np.random.default_rng(seed)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    w = rng.uniform(wlo, whi, C).astype(np.float32)
    u = rng.uniform(-0.5, 0.5, C).astype(np.float32)
    return w, u, f(B, T, C), f(B, T, C), f(B, T, C)


@pytest.mark.parametrize("B,T,C,wlo,whi", [(2, 1, 3, -1, 1), (2, 2, 3, -1, 1), (2, 3, 4, -1, 1), (3, 17, 5, -0.3, 0.3),
                                            (2, 40, 6, -0.05, 2.0)])
def test_biwkv_bwd_equals_autograd_through_the_closed_form(B, T, C, wlo, whi):
    w, u, k, v, gy = _biwkv_case(B, T, C, T, wlo, whi)
    got = clib.biwkv_bwd(w, u, k, v, gy)
    want = biwkv.biwkv_grads_closed(w, u, k, v, gy)
    for g, r, name in zip(got, want, ("gw", "gu", "gk", "gv")):
        assert np.allclose(g, r, rtol=1e-10, atol=1e-12), name


def test_biwkv_bwd_finite_differences_and_identities():
    w, u, k, v, gy = _biwkv_case(2, 23, 4, 5)
    gw, gu, gk, gv = clib.biwkv_bwd(w, u, k, v, gy)
    loss = lambda w_, u_, k_, v_: float((clib.biwkv_fwd(w_, u_, k_, v_) * gy).sum())
    h = 1e-3                                     # inputs are fp32: a step that survives the rounding
    for c in range(4):
        e = np.zeros(4, np.float32); e[c] = h
        assert abs((loss(w + e, u, k, v) - loss(w - e, u, k, v)) / (2 * float(e[c])) - gw[c]) <= 2e-4 * max(1, abs(gw[c]))
        assert abs((loss(w, u + e, k, v) - loss(w, u - e, k, v)) / (2 * float(e[c])) - gu[c]) <= 2e-4 * max(1, abs(gu[c]))
    for (b, t, c) in ((0, 0, 0), (1, 22, 3), (0, 11, 2)):
        e = np.zeros_like(k); e[b, t, c] = h
        assert abs((loss(w, u, k + e, v) - loss(w, u, k - e, v)) / (2 * h) - gk[b, t, c]) <= 2e-4
        assert abs((loss(w, u, k, v + e) - loss(w, u, k, v - e)) / (2 * h) - gv[b, t, c]) <= 2e-4
    # y is invariant under k -> k + const and is a weighted mean with weights summing to one
    assert np.abs(gk.sum(1)).max() <= 1e-12
    assert np.allclose(gv.sum(1), gy.astype(np.float64).sum(1), rtol=0, atol=1e-12)


def _wkv6_case(B, T, H, N, seed, wmean=-0.5):
    rng = np.random.default_rng(seed)
    C = H * N
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    w = rng.normal(wmean, 0.5, (B, T, C)).astype(np.float32)
    u = rng.normal(0, 0.3, (H, N)).astype(np.float32)
    return f(B, T, C), f(B, T, C), f(B, T, C), w, u, f(B, T, C)


@pytest.mark.parametrize("B,T,H,N,wmean", [(2, 1, 2, 4, -0.5), (2, 2, 1, 4, -0.5), (2, 3, 2, 4, 0.5), (2, 19, 2, 8, -0.5),
                                            (1, 33, 1, 64, -2.0)])
def test_wkv6_bwd_equals_autograd_through_the_closed_form(B, T, H, N, wmean):
    r, k, v, w, u, gy = _wkv6_case(B, T, H, N, T + N, wmean)
    got = clib.wkv6_bwd(r, k, v, w, u, gy, H)
    want = wkv6.wkv6_grads_closed(r, k, v, w, u, H, gy)
    for g, x, name in zip(got, want, ("gr", "gk", "gv", "gw", "gu")):
        assert np.allclose(g, np.asarray(x).reshape(g.shape), rtol=1e-9, atol=1e-11), name


def test_wkv6_bwd_finite_differences():
    B, T, H, N = 1, 9, 2, 4
    r, k, v, w, u, gy = _wkv6_case(B, T, H, N, 3)
    gr, gk, gv, gw, gu = clib.wkv6_bwd(r, k, v, w, u, gy, H)
    loss = lambda r_, k_, v_, w_, u_: float((clib.wkv6_fwd(r_, k_, v_, w_, u_, H) * gy).sum())
    h = 1e-3
    for (t, c) in ((0, 0), (4, 5), (8, 7)):
        e = np.zeros_like(r); e[0, t, c] = h
        fd = lambda lp, lm: (lp - lm) / (2 * h)
        assert abs(fd(loss(r + e, k, v, w, u), loss(r - e, k, v, w, u)) - gr[0, t, c]) <= 5e-4 * max(1, abs(gr[0, t, c]))
        assert abs(fd(loss(r, k + e, v, w, u), loss(r, k - e, v, w, u)) - gk[0, t, c]) <= 5e-4 * max(1, abs(gk[0, t, c]))
        assert abs(fd(loss(r, k, v + e, w, u), loss(r, k, v - e, w, u)) - gv[0, t, c]) <= 5e-4 * max(1, abs(gv[0, t, c]))
        assert abs(fd(loss(r, k, v, w + e, u), loss(r, k, v, w - e, u)) - gw[0, t, c]) <= 5e-4 * max(1, abs(gw[0, t, c]))
    e = np.zeros_like(u); e[1, 2] = h
    assert abs((loss(r, k, v, w, u + e) - loss(r, k, v, w, u - e)) / (2 * h) - gu[1, 2]) <= 5e-4 * max(1, abs(gu[1, 2]))
    # the first token of the descending order and the last of the ascending one see no state: gw there comes from the
    # other pass alone, and a sequence of one token has no decay gradient at all
    r1, k1, v1, w1, u1, gy1 = _wkv6_case(1, 1, 1, 4, 9)
    assert np.array_equal(clib.wkv6_bwd(r1, k1, v1, w1, u1, gy1, 1)[3], np.zeros((1, 1, 4)))
