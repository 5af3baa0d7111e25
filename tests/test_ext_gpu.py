"""The stand-ins for the reference's extension modules (same call signatures, results passed in by the caller where
the reference does so) against the operator entry points the other tests pin to the oracle, and through torch.ops."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import vision_rwkv_amd
    assert torch.cuda.is_available()
    return vision_rwkv_amd


def _biwkv_inputs(B, T, C, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / (C - 1)) / T).to(DEV)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    k, v, gy = (torch.randn(B, T, C, generator=g).to(DEV) for _ in range(3))
    return w, u, k, v, gy


def test_bi_wkv_module_and_torch_ops(ops):
    w, u, k, v, gy = _biwkv_inputs(3, 196, 192, 1)
    y = ops.bi_wkv_forward(w, u, k, v)
    assert torch.equal(ops.ext.bi_wkv.bi_wkv_forward(w, u, k, v), y)
    assert torch.equal(torch.ops.bi_wkv.bi_wkv_forward(w, u, k, v), y)
    ref = ops.bi_wkv_backward(w, u, k, v, gy)
    for got in (ops.ext.bi_wkv.bi_wkv_backward(w, u, k, v, gy), torch.ops.bi_wkv.bi_wkv_backward(w, u, k, v, gy)):
        assert len(got) == 4 and all(torch.equal(a, b) for a, b in zip(got, ref))


@pytest.mark.parametrize("B,T,C", [(3, 196, 192), (2, 500, 64)])
def test_legacy_wkv_module_writes_into_the_callers_tensors(ops, B, T, C):
    """classification/mae/vrwkv/vrwkv.py:46-47, 66-86: y and the gradient buffers are allocated by the caller, gw and
    gu as (B, C) and summed over the batch afterwards."""
    w, u, k, v, gy = _biwkv_inputs(B, T, C, 2)
    y = torch.full((B, T, C), float("nan"), device=DEV)
    assert ops.ext.wkv.forward(B, T, C, w, u, k, v, y) is None
    assert torch.equal(y, ops.bi_wkv_forward(w, u, k, v))
    gw, gu = (torch.full((B, C), float("nan"), device=DEV) for _ in range(2))
    gk, gv = (torch.full((B, T, C), float("nan"), device=DEV) for _ in range(2))
    torch.ops.wkv.backward(B, T, C, w, u, k, v, gy, gw, gu, gk, gv)
    rw, ru, rk, rv = ops.bi_wkv_backward(w, u, k, v, gy)
    assert torch.equal(gw.sum(0), rw) and torch.equal(gu.sum(0), ru) and torch.equal(gk, rk) and torch.equal(gv, rv)
    with pytest.raises(RuntimeError):
        ops.ext.wkv.forward(B, T, C, w, u, k, v, y.half())          # the caller's y must match k's dtype
    with pytest.raises(RuntimeError):
        ops.ext.wkv.forward(B, T + 1, C, w, u, k, v, y)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wkv6_module_takes_ew_and_the_callers_tensors(ops, dtype):
    """vrwkv6.py:48-52, 60-68: the Function forms ew = -exp(w), allocates y, gr, gk, gv, gw (B,T,C) and gu (B,C), and
    sums gu over the batch itself."""
    B, T, H = 3, 100, 2
    C = H * 64
    g = torch.Generator(device="cpu").manual_seed(3)
    r, k, v = (torch.randn(B, T, C, generator=g).to(DEV).to(dtype) for _ in range(3))
    w = (torch.randn(B, T, C, generator=g) * 0.5 - 0.5).to(DEV)
    u = (0.1 * torch.randn(H, 64, generator=g)).to(DEV)
    gy = torch.randn(B, T, C, generator=g).to(DEV)
    ew = (-torch.exp(w)).contiguous()
    y = torch.full((B, T, C), float("nan"), device=DEV)
    ops.ext.wkv6.forward(B, T, C, H, r, k, v, ew, u, y)
    y_raw = ops.wkv6_forward(B, T, C, H, r, k, v, w, u)
    assert (y - y_raw).abs().max() <= 1e-4 * y_raw.abs().max()       # exp(w) formed in torch here, in the kernel there
    gr, gk, gv, gw = (torch.full((B, T, C), float("nan"), device=DEV) for _ in range(4))
    gu = torch.full((B, C), float("nan"), device=DEV)
    torch.ops.wkv6.backward(B, T, C, H, r, k, v, ew, u, gy, gr, gk, gv, gw, gu)
    ref = ops.wkv6_backward(B, T, C, H, r, k, v, w, u, gy)
    for a, b in zip((gr, gk, gv, gw, gu.sum(0).view(H, C // H)), ref):
        assert torch.isfinite(a).all()
        assert (a - b).abs().max() <= 1e-3 * b.abs().max()
    with pytest.raises(RuntimeError):
        ops.ext.wkv6.forward(B, T, C, H, r, k, v, ew, u, y.half())
