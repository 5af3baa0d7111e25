"""Parity of the HIP wkv6 forward (through the C ABI) with the CPU oracle.

Tolerance: err = max|y - ref| / max(|ref|, rms(ref)) <= 1e-3, with ref the sequential recurrence
evaluated in float64 on the same (bf16- or fp32-rounded) inputs.
"""
import numpy as np
import pytest
import torch

from conftest import load_golden, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def ops():
    import vision_rwkv_amd
    assert torch.cuda.is_available()
    return vision_rwkv_amd


def run(ops, r, k, v, w, u, H, dtype=torch.float32, w_dtype=torch.float32):
    dev = "cuda:0"
    t = lambda a, d: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(dev).to(d)
    rt, kt, vt = t(r, dtype), t(k, dtype), t(v, dtype)
    wt, ut = t(w, w_dtype), t(u, torch.float32)
    B, T, C = rt.shape
    y = ops.RUN_CUDA_RWKV6(B, T, C, H, rt, kt, vt, wt, ut)
    torch.cuda.synchronize()
    assert y.dtype == torch.float32 and tuple(y.shape) == (B, T, C)
    f = lambda x: x.float().cpu().numpy()
    return y.cpu().numpy(), f(rt), f(kt), f(vt), f(wt)


def gen(B, T, H, seed, w_mean=-0.5, w_std=0.5):
    rng = np.random.default_rng(seed)
    C = H * 64
    r, k, v = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(3))
    w = rng.normal(w_mean, w_std, (B, T, C)).astype(np.float32)
    u = rng.normal(0.0, 0.1, (H, 64)).astype(np.float32)
    return r, k, v, w, u


def test_golden_fixtures(ops):
    for name, a in load_golden("wkv6_golden").items():
        print("case", name, flush=True)
        H = a["u"].shape[0]
        y, *_ = run(ops, a["r"], a["k"], a["v"], a["w"], a["u"], H)
        assert rel_err(y, a["y"]) <= TOL, name


@pytest.mark.parametrize("B,T,H", [(1, 1, 1), (2, 7, 2), (1, 64, 1), (2, 65, 3), (1, 196, 2), (1, 300, 1)])
def test_shapes_fp32(ops, B, T, H):
    from oracle import clib
    r, k, v, w, u = gen(B, T, H, B * 100 + T)
    y, *_ = run(ops, r, k, v, w, u, H)
    assert rel_err(y, clib.wkv6_fwd(r, k, v, w, u, H)) <= TOL


def test_config3_bf16(ops):
    """B=64, T=196, C=768, H=12, bf16 r,k,v (w fp32): against the sequential recurrence on the
    same bf16-rounded inputs."""
    from oracle import clib
    B, T, H = 64, 196, 12
    r, k, v, w, u = gen(B, T, H, 3)
    y, rr, kr, vr, wr = run(ops, r, k, v, w, u, H, torch.bfloat16)
    assert rel_err(y, clib.wkv6_fwd(rr, kr, vr, wr, u, H)) <= TOL
    y2, rr, kr, vr, wr = run(ops, r, k, v, w, u, H, torch.bfloat16, torch.bfloat16)
    assert rel_err(y2, clib.wkv6_fwd(rr, kr, vr, wr, u, H)) <= TOL


@pytest.mark.parametrize("w_mean", [-8.0, 1.5, 4.0])
def test_extreme_decay(ops, w_mean):
    """d ~ 1 (no decay), strong decay, and d == 0 (only t-1, t, t+1 contribute)."""
    from oracle import clib
    r, k, v, w, u = gen(2, 100, 2, 11, w_mean=w_mean, w_std=0.3)
    y, *_ = run(ops, r, k, v, w, u, 2)
    assert np.isfinite(y).all()
    assert rel_err(y, clib.wkv6_fwd(r, k, v, w, u, 2)) <= TOL


def test_chunked_and_sequential_kernels_agree(ops, force):
    """The matrix-core path and the sequential-state path are independent implementations."""
    r, k, v, w, u = gen(3, 196, 2, 21)
    y_chunk, *_ = run(ops, r, k, v, w, u, 2, torch.bfloat16)
    force("wkv6_fwd_scalar")
    y_seq, *_ = run(ops, r, k, v, w, u, 2, torch.bfloat16)
    assert rel_err(y_chunk, y_seq) <= TOL


def test_mixed_ranges_fall_back_per_sequence(ops):
    """One head with a decay far outside the chunked kernel's range, the other ordinary."""
    from oracle import clib
    r, k, v, w, u = gen(2, 130, 2, 31)
    w[:, :, :64] = 3.0 + 0.2 * w[:, :, :64]
    y, *_ = run(ops, r, k, v, w, u, 2)
    assert np.isfinite(y).all()
    assert rel_err(y, clib.wkv6_fwd(r, k, v, w, u, 2)) <= TOL


def test_reversal_and_head_independence(ops):
    r, k, v, w, u = gen(2, 50, 2, 5)
    y, *_ = run(ops, r, k, v, w, u, 2)
    yr, *_ = run(ops, r[:, ::-1], k[:, ::-1], v[:, ::-1], w[:, ::-1], u, 2)
    assert np.abs(yr[:, ::-1] - y).max() <= 1e-3 * np.sqrt((y ** 2).mean())
    sw = lambda a: np.concatenate([a[..., 64:], a[..., :64]], axis=-1)
    ys, *_ = run(ops, sw(r), sw(k), sw(v), sw(w), u[::-1], 2)
    assert np.abs(sw(ys) - y).max() <= 1e-3 * np.sqrt((y ** 2).mean())


def test_error_behaviour(ops):
    x = torch.randn(1, 4, 64, device="cuda")
    u = torch.zeros(1, 64, device="cuda")
    with pytest.raises(AssertionError):
        ops.RUN_CUDA_RWKV6(1, 4, 64, 2, x, x, x, x, u)           # HEAD_SIZE != C // H
    with pytest.raises(AssertionError):
        ops.RUN_CUDA_RWKV6(1, 4, 64, 1, x.transpose(1, 2).contiguous().transpose(1, 2), x, x, x, u)
    with pytest.raises(RuntimeError):
        ops.wkv6_forward(1, 4, 64, 1, x.cpu(), x, x, x, u)


def test_phase_stamping_entry_point(ops):
    """vrwkv_wkv6_fwd_phases (the chunked kernel writing a shader-clock stamp at six points of every wave's chunk
    steps, which bench.py turns into its per-phase figures): same y as the plain entry point bit for bit, every stamp
    written, and the stamps of a wave in program order -- stage E entered, operands written, behind the barrier, matrix
    stage entered, y stored, behind the barrier -- within a step and from step to step.  Also its argument checks."""
    import ctypes
    lib = ops.lib()
    dev = "cuda:0"
    B, T, H = 3, 200, 2
    C = H * 64
    r, k, v, w, u = gen(B, T, H, 77)
    tt = lambda a, d: torch.from_numpy(a).to(dev).to(d)
    rt, kt, vt, wt, ut = tt(r, torch.bfloat16), tt(k, torch.bfloat16), tt(v, torch.bfloat16), tt(w, torch.float32), tt(u, torch.float32)
    want = ops.RUN_CUDA_RWKV6(B, T, C, H, rt, kt, vt, wt, ut)
    nb = lib.vrwkv_wkv6_fwd_phases_bytes(B, T, H)
    nchunk = (T + 31) // 32
    assert nb == B * H * 8 * nchunk * 8 * 8
    st = torch.zeros(nb // 8, dtype=torch.int64, device=dev)
    y = torch.full((B, T, C), float("nan"), device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    args = (rt.data_ptr(), kt.data_ptr(), vt.data_ptr(), wt.data_ptr(), ut.data_ptr(), y.data_ptr(), B, T, C, H)
    assert lib.vrwkv_wkv6_fwd_phases(*args, st.data_ptr(), nb, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y, want)
    s = st.cpu().numpy().reshape(B * H, 8, nchunk, 8)
    pts = s[..., [0, 1, 2, 4, 5, 6]]
    assert (pts > 0).all()
    assert (np.diff(pts, axis=-1) >= 0).all()                       # inside a step
    assert (s[:, :, 1:, 0] >= s[:, :, :-1, 6]).all()                # from step to step
    # a stamp buffer that is too small, or missing, is refused before anything is launched
    assert lib.vrwkv_wkv6_fwd_phases(*args, st.data_ptr(), nb - 8, stream) == 5
    assert lib.vrwkv_wkv6_fwd_phases(*args, None, nb, stream) == 1
    assert lib.vrwkv_wkv6_fwd_phases_bytes(0, T, H) == 0
