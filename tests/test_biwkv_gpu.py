"""Parity of the HIP Bi-WKV forward (through the C ABI) with the CPU oracle.

Tolerance (stated once, used everywhere): err = max|y - ref| / max(|ref|, rms(ref)), i.e.
allclose(rtol, atol = rtol*rms(ref)) -- y is a weighted mean of zero-mean values and crosses
zero, so a pointwise relative error needs a floor.
fp32 I/O: err <= 1e-4;  bf16 / fp16 I/O: err <= 1e-2 (ref evaluated on the rounded inputs).
At the VRWKV-B shape the kernel must also be at least as accurate as the reference recurrence
itself run in fp32 (PyTorch CPU eager), under the stricter floor 1e-2*rms.
"""
import numpy as np
import pytest
import torch

from conftest import load_golden, rel_err

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-4
TOL_16 = 1e-2


@pytest.fixture(scope="module")
def ops():
    import vision_rwkv_amd
    assert torch.cuda.is_available()
    return vision_rwkv_amd


def baseline_wu(C, T):
    c = np.arange(C)
    w = (-5.0 + 8.0 * (c / max(C - 1, 1))) / T
    u = (np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T
    return w.astype(np.float32), u.astype(np.float32)


def run(ops, w, u, k, v, dtype=torch.float32):
    dev = "cuda:0"
    wt = torch.from_numpy(np.ascontiguousarray(w, np.float32)).to(dev)
    ut = torch.from_numpy(np.ascontiguousarray(u, np.float32)).to(dev)
    kt = torch.from_numpy(np.ascontiguousarray(k, np.float32)).to(dev).to(dtype)
    vt = torch.from_numpy(np.ascontiguousarray(v, np.float32)).to(dev).to(dtype)
    y = ops.bi_wkv_forward(wt, ut, kt, vt)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == kt.shape
    return y.float().cpu().numpy(), kt.float().cpu().numpy(), vt.float().cpu().numpy()


def test_golden_fixtures(ops):
    for name, a in load_golden("biwkv_golden").items():
        print("case", name, flush=True)
        y, _, _ = run(ops, a["w"], a["u"], a["k"], a["v"])
        assert rel_err(y, a["y"]) <= TOL_F32, name


@pytest.mark.parametrize("B,T,C", [(1, 196, 192), (64, 196, 768)])
def test_config_shapes_fp32(ops, B, T, C):
    from oracle import clib
    rng = np.random.default_rng(1234)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w, u = baseline_wu(C, T)
    y, _, _ = run(ops, w, u, k, v)
    ref = clib.biwkv_fwd(w, u, k, v)
    assert rel_err(y, ref) <= TOL_F32
    from oracle import torch_eager
    y_eager = torch_eager.biwkv_eager(*(torch.from_numpy(a) for a in (w, u, k, v))).numpy()
    strict, strict_eager = rel_err(y, ref, 1e-2), rel_err(y_eager, ref, 1e-2)
    print(f"strict-floor error: kernel {strict:.2e}, fp32 eager recurrence {strict_eager:.2e}")
    assert strict <= strict_eager


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_config1_16bit(ops, dtype):
    from oracle import clib
    B, T, C = 64, 196, 768
    rng = np.random.default_rng(77)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w, u = baseline_wu(C, T)
    y, kr, vr = run(ops, w, u, k, v, dtype)
    assert rel_err(y, clib.biwkv_fwd(w, u, kr, vr)) <= TOL_16


def test_config2_long_sequence_outliers_bf16(ops):
    """B=2, T=4150, C=768, bf16 I/O, 1% of tokens scaled x8 (long-sequence two-kernel path)."""
    from oracle import clib
    B, T, C = 2, 4150, 768
    rng = np.random.default_rng(2)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    mask = rng.random((B, T, 1)) < 0.01
    k = np.where(mask, 8 * k, k).astype(np.float32)
    v = np.where(mask, 8 * v, v).astype(np.float32)
    w, u = baseline_wu(C, T)
    y, kr, vr = run(ops, w, u, k, v, torch.bfloat16)
    assert rel_err(y, clib.biwkv_fwd(w, u, kr, vr)) <= TOL_16
    y32, _, _ = run(ops, w, u, k, v, torch.float32)
    assert rel_err(y32, clib.biwkv_fwd(w, u, k, v)) <= TOL_F32


@pytest.mark.parametrize("B,T,C", [(3, 1, 64), (2, 5, 33), (1, 197, 100), (2, 300, 1), (1, 577, 96),
                                   (2, 1024, 192), (1, 1500, 70), (5, 64, 1024)])
def test_ragged_shapes(ops, B, T, C):
    from oracle import clib
    rng = np.random.default_rng(B * 1000 + T + C)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w = rng.uniform(-5, 3, C).astype(np.float32) / T
    u = rng.uniform(-1, 1, C).astype(np.float32)
    y, _, _ = run(ops, w, u, k, v)
    assert rel_err(y, clib.biwkv_fwd(w, u, k, v)) <= TOL_F32
    if C % 2 == 0:
        y, kr, vr = run(ops, w, u, k, v, torch.bfloat16)
        assert rel_err(y, clib.biwkv_fwd(w, u, kr, vr)) <= TOL_16


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,T,C", [(2, 225, 64), (1, 384, 128), (2, 448, 72), (1, 449, 64), (2, 576, 128),
                                   (1, 672, 64), (3, 600, 200), (40, 300, 512)])
def test_two_and_three_super_chunks_16bit(ops, B, T, C, dtype):
    """16-bit sequences of 225..672 tokens take the one-launch path that keeps a whole sequence in a workgroup's
    registers (24- or 28-token chunks, two or three super-chunks; 320 sequences walk the persistent loop).  One
    channel tile has parameters outside the plain-sum regime and is redone by the renormalising recurrence."""
    from oracle import clib
    rng = np.random.default_rng(B * 1000 + T + C)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w = rng.uniform(-5, 3, C).astype(np.float32) / T
    u = rng.uniform(-1, 1, C).astype(np.float32) / T
    if C > 64:
        w[C - 3] = 2.5
    y, kr, vr = run(ops, w, u, k, v, dtype)
    assert np.isfinite(y).all()
    assert rel_err(y, clib.biwkv_fwd(w, u, kr, vr)) <= TOL_16


def test_one_launch_and_two_kernel_paths_agree(ops, force):
    """The same 16-bit sequence through the one-launch kernel and through the aggregate + emit kernels: both round
    the same fp32 arithmetic to bf16, so they may differ by an output ulp here and there, no more."""
    B, T, C = 4, 576, 256
    rng = np.random.default_rng(5)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w, u = baseline_wu(C, T)
    y1, _, _ = run(ops, w, u, k, v, torch.bfloat16)
    force("biwkv_no_resident")
    y2, _, _ = run(ops, w, u, k, v, torch.bfloat16)
    assert np.abs(y1 - y2).max() <= 2.0 ** -7 * np.abs(y2).max()
    assert (y1 != y2).mean() < 0.02


def test_very_long_sequence_many_super_chunks(ops):
    """T = 9100 is 41 super-chunks: more than the carry step's on-chip table holds, so it walks the workspace
    directly; a second channel tile has parameters outside the plain-sum regime (its entries must stay untouched)."""
    from oracle import clib
    B, T, C = 1, 9100, 128
    rng = np.random.default_rng(91)
    k = rng.standard_normal((B, T, C), dtype=np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w = rng.uniform(-5, 3, C).astype(np.float32) / T
    u = rng.uniform(-1, 1, C).astype(np.float32)
    w[70] = 3.0
    y, _, _ = run(ops, w, u, k, v)
    assert rel_err(y, clib.biwkv_fwd(w, u, k, v)) <= TOL_F32


@pytest.mark.parametrize("T", [40, 196, 700])
def test_robust_path_extreme_parameters(ops, T):
    """|w| and |u| far outside the plain-sum regime, mixed with benign channels."""
    from oracle import clib
    B, C = 2, 128
    rng = np.random.default_rng(T)
    k = (3 * rng.standard_normal((B, T, C))).astype(np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w = rng.uniform(-2.0, 8.0, C).astype(np.float32)
    u = rng.uniform(-30.0, 30.0, C).astype(np.float32)
    w[::7] = 0.01
    u[::7] = 0.1
    w[3] = 200.0      # three-term regime
    u[5] = 90.0       # y -> v
    y, _, _ = run(ops, w, u, k, v)
    ref = clib.biwkv_fwd(w, u, k, v)
    assert np.isfinite(y).all()
    assert rel_err(y, ref) <= TOL_F32
    assert np.abs(y[..., 5] - v[..., 5]).max() < 1e-6


def test_huge_k_range_stays_finite(ops):
    """k spanning +-60 in one sequence (e^{+-60} is far outside what an unstabilised sum survives)."""
    from oracle import clib
    B, T, C = 1, 196, 64
    rng = np.random.default_rng(3)
    k = rng.uniform(-60, 60, (B, T, C)).astype(np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w, u = baseline_wu(C, T)
    y, _, _ = run(ops, w, u, k, v)
    assert np.isfinite(y).all()
    assert rel_err(y, clib.biwkv_fwd(w, u, k, v)) <= TOL_F32


@pytest.mark.parametrize("T,dtype", [(196, torch.float32), (196, torch.bfloat16), (576, torch.bfloat16), (900, torch.float32)])
def test_growing_weights_with_waves_far_apart_stay_finite(ops, T, dtype):
    """Negative w (weights that grow with distance) together with k = +40 on the first 28 tokens and -40 elsewhere:
    the carried sums grow by up to e^{|w| T} while the light waves raise them by 2^115 to their own scale.  Channels:
    w = -0.13 (growth 2^37 at T=196: the renormalising path), w = -0.05 and -0.02 (plain sums, growth 2^14 / 2^6),
    w = +0.02, and the same spread scaled to the longer sequences."""
    from oracle import clib
    B, C = 2, 64
    rng = np.random.default_rng(T)
    k = np.full((B, T, C), -40.0, np.float32)
    k[:, :28] = 40.0
    k += rng.standard_normal((B, T, C)).astype(np.float32)
    v = rng.standard_normal((B, T, C), dtype=np.float32)
    w = (np.array([-0.13, -0.05, -0.02, 0.02] * (C // 4)) * 196.0 / T).astype(np.float32)
    u = np.zeros(C, np.float32)
    y, kr, vr = run(ops, w, u, k, v, dtype)
    assert np.isfinite(y).all()
    assert rel_err(y, clib.biwkv_fwd(w, u, kr, vr)) <= (TOL_F32 if dtype == torch.float32 else 1e-2)


def test_properties_at_full_size(ops):
    """Size-independent properties at the VRWKV-B shape."""
    B, T, C = 64, 196, 768
    g = torch.Generator(device="cpu").manual_seed(5)
    k = torch.randn(B, T, C, generator=g).cuda()
    v = torch.randn(B, T, C, generator=g).cuda()
    w, u = (torch.from_numpy(a).cuda() for a in baseline_wu(C, T))
    y = ops.bi_wkv_forward(w, u, k, v)
    # convexity
    assert (y <= v.amax(dim=1, keepdim=True) + 1e-5).all() and (y >= v.amin(dim=1, keepdim=True) - 1e-5).all()
    # constant v
    yc = ops.bi_wkv_forward(w, u, k, torch.full_like(v, 1.25))
    assert (yc - 1.25).abs().max().item() < 1e-5
    # k -> k + const
    ys = ops.bi_wkv_forward(w, u, k + 2.5, v)
    assert (ys - y).abs().max().item() < 2e-5
    # token reversal
    yr = ops.bi_wkv_forward(w, u, k.flip(1).contiguous(), v.flip(1).contiguous()).flip(1)
    assert (yr - y).abs().max().item() < 2e-5
    # softmax reduction
    z = torch.zeros_like(w)
    y0 = ops.bi_wkv_forward(z, z, k, v)
    want = (torch.softmax(k.double(), dim=1) * v.double()).sum(dim=1, keepdim=True)
    assert (y0.double() - want).abs().max().item() < 1e-5


def test_non_default_stream_and_determinism(ops):
    B, T, C = 4, 196, 256
    k = torch.randn(B, T, C, device="cuda")
    v = torch.randn(B, T, C, device="cuda")
    w, u = (torch.from_numpy(a).cuda() for a in baseline_wu(C, T))
    y0 = ops.bi_wkv_forward(w, u, k, v)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y1 = ops.bi_wkv_forward(w, u, k, v)
    s.synchronize()
    assert torch.equal(y0, y1)


def test_run_cuda_dtype_rule(ops):
    """RUN_CUDA output dtype follows w.dtype (vrwkv.py:31-44)."""
    B, T, C = 2, 50, 64
    k = torch.randn(B, T, C)
    v = torch.randn(B, T, C)
    w, u = (torch.from_numpy(a) for a in baseline_wu(C, T))
    y = ops.RUN_CUDA(w, u, k, v)                       # CPU tensors are moved by RUN_CUDA
    assert y.is_cuda and y.dtype == torch.float32
    yb = ops.RUN_CUDA(w.bfloat16(), u.bfloat16(), k.bfloat16(), v.bfloat16())
    assert yb.dtype == torch.bfloat16
    ya = ops.RUN_CUDA(w, u, k.bfloat16(), v.bfloat16())  # autocast-like: fp32 parameters
    assert ya.dtype == torch.float32
    yh = ops.RUN_CUDA(w.half(), u.half(), k, v)
    assert yh.dtype == torch.float16
    yl = ops.RUN_CUDA(B, T, C, w, u, k, v)             # legacy seven-argument form
    assert torch.equal(yl, y)


def test_error_behaviour(ops):
    k = torch.randn(2, 8, 64, device="cuda")
    w = torch.zeros(64, device="cuda")
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.bi_wkv_forward(w, w, k.transpose(0, 1), k.transpose(0, 1))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ops.bi_wkv_forward(w.cpu(), w, k, k)
    with pytest.raises(RuntimeError):
        ops.bi_wkv_forward(w[:32].contiguous(), w, k, k)
