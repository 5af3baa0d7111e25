"""Parity of the HIP Bi-WKV backward with autograd through the float64 closed form.

Tolerance: err = max|g - ref| / max(|ref|, rms(ref)) <= 1e-4 (fp32 I/O), 2e-2 (bf16 I/O, ref on the
rounded inputs; two rounded tensors enter each product)."""
import numpy as np
import pytest
import torch

from conftest import load_golden, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import vision_rwkv_amd
    assert torch.cuda.is_available()
    return vision_rwkv_amd


def run(ops, w, u, k, v, gy, dtype=torch.float32):
    dev = "cuda:0"
    t = lambda a, d=torch.float32: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(dev).to(d)
    kt, vt, gt = t(k, dtype), t(v, dtype), t(gy, dtype)
    gw, gu, gk, gv = ops.bi_wkv_backward(t(w), t(u), kt, vt, gt)
    torch.cuda.synchronize()
    f = lambda x: x.float().cpu().numpy()
    return f(gw), f(gu), f(gk), f(gv), f(kt), f(vt), f(gt)


def test_golden_gradient_fixture(ops):
    g = load_golden("biwkv_golden")["grad_T19_C8"]
    gw, gu, gk, gv, *_ = run(ops, g["w"], g["u"], g["k"], g["v"], g["gy"])
    for got, name in ((gw, "gw"), (gu, "gu"), (gk, "gk"), (gv, "gv")):
        assert rel_err(got, g[name]) <= 1e-4, name


@pytest.mark.parametrize("B,T,C,wscale", [(2, 1, 64, 1.0), (3, 37, 70, 1.0), (2, 196, 96, 1.0), (1, 50, 64, 40.0)])
def test_against_autograd_closed_form(ops, B, T, C, wscale):
    from oracle import biwkv
    rng = np.random.default_rng(T + C)
    k = rng.standard_normal((B, T, C)).astype(np.float32)
    v = rng.standard_normal((B, T, C)).astype(np.float32)
    gy = rng.standard_normal((B, T, C)).astype(np.float32)
    w = (rng.uniform(-5, 3, C) / T * wscale).astype(np.float32)
    u = rng.uniform(-1, 1, C).astype(np.float32)
    gw, gu, gk, gv, *_ = run(ops, w, u, k, v, gy)
    rw, ru, rk, rv = biwkv.biwkv_grads_closed(w, u, k, v, gy)
    if T == 1:                                    # gk, gw, gu are exactly zero: absolute check
        assert np.abs(gk).max() <= 1e-6 and np.abs(gw).max() <= 1e-6 and np.abs(gu).max() <= 1e-6
        assert rel_err(gv, rv) <= 1e-4
        return
    assert rel_err(gk, rk) <= 1e-4 and rel_err(gv, rv) <= 1e-4
    assert rel_err(gw, rw) <= 2e-4 and rel_err(gu, ru) <= 1e-4
    # exact identities: k -> k + const leaves y unchanged; the weights sum to one
    assert np.abs(gk.sum(axis=1)).max() <= 1e-4 * np.abs(gk).max() * T ** 0.5
    assert np.abs(gv.sum(axis=1) - gy.sum(axis=1)).max() <= 1e-4 * np.abs(gy).sum(axis=1).max()


def test_bf16_io(ops):
    from oracle import biwkv
    B, T, C = 2, 64, 64
    rng = np.random.default_rng(9)
    k, v, gy = (rng.standard_normal((B, T, C)).astype(np.float32) for _ in range(3))
    w = (rng.uniform(-5, 3, C) / T).astype(np.float32)
    u = rng.uniform(-1, 1, C).astype(np.float32)
    gw, gu, gk, gv, kr, vr, gr = run(ops, w, u, k, v, gy, torch.bfloat16)
    rw, ru, rk, rv = biwkv.biwkv_grads_closed(w, u, kr, vr, gr)
    assert rel_err(gk, rk) <= 2e-2 and rel_err(gv, rv) <= 2e-2
    assert rel_err(gw, rw) <= 1e-3 and rel_err(gu, ru) <= 1e-3


def test_autograd_function_end_to_end(ops):
    """RUN_CUDA(...).backward() against torch.autograd through a float64 dense formula."""
    B, T, C = 2, 23, 64
    g = torch.Generator().manual_seed(3)
    k = torch.randn(B, T, C, generator=g)
    v = torch.randn(B, T, C, generator=g)
    w = (torch.rand(C, generator=g) * 8 - 5) / T
    u = torch.rand(C, generator=g) - 0.5
    gy = torch.randn(B, T, C, generator=g)
    leaves = [t.cuda().requires_grad_(True) for t in (w, u, k, v)]
    y = ops.RUN_CUDA(*leaves)
    y.backward(gy.cuda())
    from oracle import biwkv
    ref = biwkv.biwkv_grads_closed(w.numpy(), u.numpy(), k.numpy(), v.numpy(), gy.numpy())
    for leaf, r in zip(leaves, ref):
        assert rel_err(leaf.grad.cpu().numpy(), r) <= 2e-4


def test_tiled_and_sequential_kernels_full_size(ops, force):
    """VRWKV-B shape, random per-channel w, u: the tiled kernel and the sequential one (forced through the library
    switch), each against the C oracle on every output, and the sum identities that hold at any size."""
    from oracle import clib
    B, T, C = 64, 196, 768
    g = torch.Generator().manual_seed(5)
    k = torch.randn(B, T, C, generator=g).cuda()
    v = torch.randn(B, T, C, generator=g).cuda()
    gy = torch.randn(B, T, C, generator=g).cuda()
    w = ((torch.rand(C, generator=g) * 8 - 5) / T).cuda()
    u = (torch.rand(C, generator=g) - 0.5).cuda()
    got = ops.bi_wkv_backward(w, u, k, v, gy)
    force("biwkv_bwd_serial")
    ref = ops.bi_wkv_backward(w, u, k, v, gy)
    torch.cuda.synchronize()
    f = lambda x: x.cpu().numpy()
    want = clib.biwkv_bwd(f(w), f(u), f(k), f(v), f(gy))
    for a, b, r, name in zip(got, ref, want, ("gw", "gu", "gk", "gv")):
        assert rel_err(f(a), r) <= 1e-4, name
        # the sequential kernel renormalises at every token and is the less accurate of the two
        assert rel_err(f(b), r) <= 5e-4, name
    gk, gv = got[2], got[3]
    assert (gv.sum(1) - gy.sum(1)).abs().max().item() <= 1e-4 * gy.abs().sum(1).max().item()
    assert gk.sum(1).abs().max().item() <= 1e-4 * gk.abs().max().item() * T ** 0.5


@pytest.mark.parametrize("T", [29, 100, 224, 225, 300, 700])
def test_wave_scales_far_apart_and_sequence_lengths(ops, T):
    """k jumps by +-60 between token ranges (every wave gets its own reference exponent, rescaled exactly
    when aggregates cross waves); T = 224 is the longest single-launch case, longer ones take the three-launch
    path (2 and 4 super-chunks)."""
    from oracle import biwkv
    B, C = 2, 64
    rng = np.random.default_rng(T)
    k = rng.standard_normal((B, T, C)).astype(np.float32)
    k[:, T // 3: T // 2] += 60.0
    k[:, T // 2: (2 * T) // 3] -= 60.0
    k[1, 5] += 80.0
    v, gy = (rng.standard_normal((B, T, C)).astype(np.float32) for _ in range(2))
    w = (rng.uniform(-5, 3, C) / T).astype(np.float32)
    u = rng.uniform(-1, 1, C).astype(np.float32)
    gw, gu, gk, gv, *_ = run(ops, w, u, k, v, gy)
    rw, ru, rk, rv = biwkv.biwkv_grads_closed(w, u, k, v, gy)
    assert np.isfinite(gk).all() and np.isfinite(gv).all()
    # where one token outweighs all others, y_t ~ v_i for every t and gk_i = sum_t z_t W[t,i] (v_i - y_t)
    # cancels to ~1e-6 of its terms: fp32 keeps 5e-4 of the tensor's rms there (both kernels), not 1e-4
    assert rel_err(gk, rk) <= 5e-4 and rel_err(gv, rv) <= 5e-4
    assert rel_err(gw, rw) <= 5e-4 and rel_err(gu, ru) <= 5e-4


@pytest.mark.parametrize("T", [196, 500])
def test_growing_weights_with_waves_far_apart(ops, T):
    """Negative w with k = +40 on the first 28 tokens and -40 elsewhere (see the forward's test of that name):
    finite, and equal to the oracle's gradients."""
    from oracle import clib
    B, C = 2, 64
    rng = np.random.default_rng(T + 1)
    k = np.full((B, T, C), -40.0, np.float32)
    k[:, :28] = 40.0
    k += rng.standard_normal((B, T, C)).astype(np.float32)
    v, gy = (rng.standard_normal((B, T, C)).astype(np.float32) for _ in range(2))
    w = (np.array([-0.13, -0.05, -0.02, 0.02] * (C // 4)) * 196.0 / T).astype(np.float32)
    u = np.zeros(C, np.float32)
    gw, gu, gk, gv, *_ = run(ops, w, u, k, v, gy)
    ref = clib.biwkv_bwd(w, u, k, v, gy)
    for got, want, name in zip((gw, gu, gk, gv), ref, ("gw", "gu", "gk", "gv")):
        assert np.isfinite(got).all(), name
        assert rel_err(got, want) <= 5e-4, name


def test_long_sequence_tiled_equals_sequential(ops, force):
    """VRWKV-L at 384x384 (T = 576, three super-chunks): the three-launch tiled path against the sequential
    kernel, the float64 closed form on a slice, and the sum identities."""
    B, T, C = 4, 576, 256
    g = torch.Generator().manual_seed(11)
    k = torch.randn(B, T, C, generator=g).cuda()
    v = torch.randn(B, T, C, generator=g).cuda()
    gy = torch.randn(B, T, C, generator=g).cuda()
    w = ((torch.rand(C, generator=g) * 8 - 5) / T).cuda()
    u = (torch.rand(C, generator=g) - 0.5).cuda()
    got = ops.bi_wkv_backward(w, u, k, v, gy)
    force("biwkv_bwd_serial")
    ref = ops.bi_wkv_backward(w, u, k, v, gy)
    torch.cuda.synchronize()
    for a, b, name in zip(got, ref, ("gw", "gu", "gk", "gv")):
        assert rel_err(a.cpu().numpy(), b.cpu().numpy()) <= 5e-4, name
    from oracle import biwkv
    sl = (slice(0, 1), slice(None), slice(64, 128))
    f = lambda x: x.cpu().numpy()
    _, _, rk, rv = biwkv.biwkv_grads_closed(f(w[64:128]), f(u[64:128]), f(k[sl]), f(v[sl]), f(gy[sl]))
    assert rel_err(f(got[2][sl]), rk) <= 1e-4 and rel_err(f(got[3][sl]), rv) <= 1e-4
    assert (got[3].sum(1) - gy.sum(1)).abs().max().item() <= 1e-4 * gy.abs().sum(1).max().item()
