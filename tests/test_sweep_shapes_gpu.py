"""Parity at every shape of the dense-prediction sweep the benchmark times: B=2 (the adapters' batch), T in {1024, 4150,
4200} x C in {192, 384, 768, 1024} -- the long-sequence paths with 5 to 19 super-chunks per sequence (forward: aggregate
kernel + emitting kernel with the batched fold of the other super-chunks' table entries; backward: three launches through
the auxiliary tables), which bi_wkv_cuda_forward / bi_wkv_cuda_backward serve in the reference
(classification/mmcls_custom/models/backbones/cuda_new/bi_wkv_kernel.cu:370-443).

  forward   fp32 and bf16 at the full shape against the C oracle's recurrence (O(T) per sequence).
  backward  the kernel runs at the full shape; the oracle's O(T^2) softmax form is evaluated on 64 channels spread over
            the width (channels are independent, and gw, gu are per-channel sums over batch and tokens, so the slice
            is exact for all four outputs); the remaining channels are held to the identities sum_t gk = 0 and
            sum_t gv = sum_t gy.
  beyond    T = 8000 (36 super-chunks: more table entries than one batched fetch holds) for both directions.
Error measure: max|x - ref| / max(|ref|, rms(ref)) (conftest.rel_err)."""
import numpy as np
import pytest
import torch

from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SWEEP_T = (1024, 4150, 4200)
SWEEP_C = (192, 384, 768, 1024)


@pytest.fixture(scope="module")
def ops():
    import vision_rwkv_amd
    assert torch.cuda.is_available()
    return vision_rwkv_amd


def baseline_wu(C, T):
    c = np.arange(C)
    w = ((-5.0 + 8.0 * c / (C - 1)) / T).astype(np.float32)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).astype(np.float32)
    return w, u


def inputs(B, T, C, seed, n, outliers=True):
    """n tensors N(0,1); with outliers 1 % of the (batch, token) rows of the first two are scaled x8 as the
    Mask-RCNN configuration does."""
    rng = np.random.default_rng(seed)
    xs = [rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(n)]
    if outliers:
        mask = rng.random((B, T, 1)) < 0.01
        for x in xs[:2]:
            x *= np.where(mask, 8.0, 1.0).astype(np.float32)
    return xs


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


@pytest.mark.parametrize("C", SWEEP_C)
@pytest.mark.parametrize("T", SWEEP_T)
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 1e-2)])
def test_forward_at_every_sweep_shape(ops, T, C, dtype, tol):
    from oracle import clib
    B = 2
    print(f"fwd sweep cell B={B} T={T} C={C} {dtype}", flush=True)
    k, v = inputs(B, T, C, seed=T + C, n=2)
    w, u = baseline_wu(C, T)
    kd, vd = t(k).to(dtype), t(v).to(dtype)
    y = ops.bi_wkv_forward(t(w), t(u), kd, vd)
    assert y.dtype == dtype and y.shape == (B, T, C)
    f = lambda x: x.float().cpu().numpy()
    ref = clib.biwkv_fwd(w, u, f(kd), f(vd))
    err = rel_err(f(y), ref)
    print(f"  rel_err {err:.3e}")
    assert err <= tol


def _slice_channels(C, n=64):
    return np.unique(np.linspace(0, C - 1, n).round().astype(np.int64))


def _check_backward(ops, B, T, C, dtype, seed, tol_big, tol_sum, outliers=True):
    from oracle import clib
    k, v, gy = inputs(B, T, C, seed=seed, n=3, outliers=outliers)
    w, u = baseline_wu(C, T)
    kd, vd, gd = (t(x).to(dtype) for x in (k, v, gy))
    gw, gu, gk, gv = ops.bi_wkv_backward(t(w), t(u), kd, vd, gd)
    torch.cuda.synchronize()
    assert gk.dtype == dtype and gk.shape == (B, T, C) and gw.shape == (C,)
    f = lambda x: x.float().cpu().numpy()
    cs = _slice_channels(C)
    ref = clib.biwkv_bwd(w[cs], u[cs], f(kd)[:, :, cs], f(vd)[:, :, cs], f(gd)[:, :, cs])
    got = (f(gw)[cs], f(gu)[cs], f(gk)[:, :, cs], f(gv)[:, :, cs])
    errs = {n: rel_err(g, r) for g, r, n in zip(got, ref, ("gw", "gu", "gk", "gv"))}
    print("  ", errs)
    assert errs["gk"] <= tol_big and errs["gv"] <= (tol_big if dtype != torch.float32 else 1e-4), errs
    assert errs["gw"] <= tol_sum and errs["gu"] <= tol_sum, errs
    # every channel, not only the slice: the weights of an output sum to one, and y does not move with k + const
    gk64, gv64, gy64 = gk.double(), gv.double(), gd.double()
    scale = gy64.abs().sum(1).max().item()
    round_off = 1e-4 if dtype == torch.float32 else 4e-3          # bf16 results: T roundings of 2^-9, signs random
    assert (gv64.sum(1) - gy64.sum(1)).abs().max().item() <= round_off * scale
    assert gk64.sum(1).abs().max().item() <= round_off * gk64.abs().sum(1).max().item()
    assert torch.isfinite(gw).all() and torch.isfinite(gu).all()


@pytest.mark.parametrize("C", SWEEP_C)
@pytest.mark.parametrize("T", SWEEP_T)
def test_backward_at_every_sweep_shape(ops, T, C):
    """fp32 on N(0,1) inputs, as the benchmark times it.  Tolerance 1e-4 for all four outputs."""
    print(f"bwd sweep cell B=2 T={T} C={C} fp32", flush=True)
    _check_backward(ops, 2, T, C, torch.float32, seed=7 * T + C, tol_big=1e-4, tol_sum=1e-4, outliers=False)


@pytest.mark.parametrize("T,C", [(1024, 768), (4150, 768), (4200, 192)])
def test_backward_with_outlier_tokens(ops, T, C):
    """1 % of the tokens scaled x8 (the Mask-RCNN configuration's stress): a token with k near +24 outweighs its whole
    neighbourhood, y_t ~ v_i for every t in reach, and gk_i = sum_t z_t W[t,i] (v_i - y_t) cancels to a small fraction
    of its terms -- fp32 keeps 5e-4 of the tensor's rms there (any O(T) evaluation in fp32 does: the difference is formed
    from two running sums); gv, gw, gu stay at 1e-4."""
    print(f"bwd outlier cell B=2 T={T} C={C} fp32", flush=True)
    _check_backward(ops, 2, T, C, torch.float32, seed=5 * T + C, tol_big=5e-4, tol_sum=1e-4, outliers=True)


@pytest.mark.parametrize("T,C", [(1024, 384), (4150, 768), (4200, 1024)])
def test_backward_bf16_at_sweep_shapes(ops, T, C):
    """bf16 k, v, gy (oracle on the rounded inputs): gk, gv carry one bf16 rounding of the result."""
    print(f"bwd sweep cell B=2 T={T} C={C} bf16", flush=True)
    _check_backward(ops, 2, T, C, torch.bfloat16, seed=11 * T + C, tol_big=1e-2, tol_sum=1e-4, outliers=False)


def test_forward_and_backward_beyond_32_super_chunks(ops):
    """T = 8000 is 36 super-chunks of 224 tokens: the emitting kernels fold more table entries than the two batched
    fetches of a tile hold and take the remainder in their loop."""
    from oracle import clib
    B, T, C = 1, 8000, 128
    print(f"long cell B={B} T={T} C={C}", flush=True)
    k, v = inputs(B, T, C, seed=3, n=2)
    w, u = baseline_wu(C, T)
    y = ops.bi_wkv_forward(t(w), t(u), t(k), t(v)).cpu().numpy()
    assert rel_err(y, clib.biwkv_fwd(w, u, k, v)) <= 1e-4
    _check_backward(ops, B, T, C, torch.float32, seed=4, tol_big=1e-4, tol_sum=1e-4, outliers=False)
