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
