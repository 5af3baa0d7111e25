"""vrwkv_biwkv_fwd_gate: the Bi-WKV forward with the receptance gate applied before y is stored,
y = sigmoid(r) * wkv(w, u, k, v) -- the operator and the step after it in VRWKV_SpatialMix.forward
(classification/mmcls_custom/models/backbones/vrwkv.py:183-186, key_norm off).

Checked against oracle/blocks.row_epilogue(post = sigmoid gate) applied to the C oracle's Bi-WKV recurrence on the same
(rounded) inputs, on every path the entry point has: the one-launch kernel with the gate inside (T <= 224; 25- and
28-token chunks, short sequences), the two-launch path (gate inside the emitting kernel for 16-bit rows, a pass of its
own for fp32 rows), channel tiles redone by the renormalising recurrence, and the calls served without fusion (16-bit
sequences of 225..672 tokens, unaligned rows).  The backbone's use of it: VRWKV-B in eval mode with and without it.
Tolerances as for the operator: err = max|y - ref| / max(|ref|, rms(ref)) <= 1e-4 (fp32 I/O), 1e-2 (16-bit I/O)."""
import numpy as np
import pytest
import torch

from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    import vision_rwkv_amd
    assert torch.cuda.is_available()
    return vision_rwkv_amd


def _case(ops, B, T, C, dtype, seed, w=None, u=None, offset=0):
    from oracle import blocks, clib
    rng = np.random.default_rng(seed)
    k, v, r = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(3))
    r *= 2.0                                                  # gates from 0.02 to 0.98
    c = np.arange(C)
    if w is None:
        w = ((-5.0 + 8.0 * c / max(C - 1, 1)) / T).astype(np.float32)
    if u is None:
        u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).astype(np.float32)

    def dev(a):
        # offset > 0: a view that starts `offset` elements into its allocation (rows no longer 16-byte aligned)
        flat = torch.empty(a.size + offset, dtype=dtype, device=DEV)
        t = flat[offset:].view(a.shape)
        t.copy_(torch.from_numpy(a).to(DEV))
        return t

    kd, vd, rd = dev(k), dev(v), dev(r)
    wt, ut = torch.from_numpy(w).to(DEV), torch.from_numpy(u).to(DEV)
    y = ops.bi_wkv_forward(wt, ut, kd, vd, gate=rd)
    plain = ops.bi_wkv_forward(wt, ut, kd, vd)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == (B, T, C)
    f = lambda x: x.float().cpu().numpy()
    ref = blocks.row_epilogue(clib.biwkv_fwd(w, u, f(kd), f(vd)), f(rd), post=blocks.POST_SIGMOID_GATE).reshape(B, T, C)
    err = rel_err(f(y), ref)
    # and against the operator's own result gated in float64: the fused store rounds once, this rounds twice
    two_step = f(plain).astype(np.float64) / (1.0 + np.exp(-f(rd).astype(np.float64)))
    err2 = rel_err(f(y), two_step)
    print(f"  B={B} T={T} C={C} {dtype}: err {err:.2e}, against the two-step result {err2:.2e}", flush=True)
    assert np.isfinite(f(y)).all()
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    assert err <= tol and err2 <= tol
    return y


@pytest.mark.parametrize("B,T,C,dtype", [
    (3, 196, 192, torch.float32), (2, 196, 768, torch.bfloat16), (2, 197, 256, torch.float16),    # 28- / 25-token chunks
    (2, 180, 128, torch.bfloat16), (2, 100, 256, torch.float32), (5, 33, 64, torch.bfloat16), (1, 7, 64, torch.float32),
    (2, 224, 320, torch.float32)])
def test_gate_inside_the_one_launch_kernel(ops, B, T, C, dtype):
    _case(ops, B, T, C, dtype, seed=B * 1000 + T + C)


@pytest.mark.parametrize("B,T,C,dtype", [
    (2, 1024, 192, torch.float32), (2, 4150, 256, torch.bfloat16), (1, 700, 128, torch.float32),
    (2, 900, 64, torch.float16), (1, 9100, 64, torch.float32)])
def test_gate_on_the_two_launch_path_of_long_sequences(ops, B, T, C, dtype):
    _case(ops, B, T, C, dtype, seed=B * 1000 + T + C)


@pytest.mark.parametrize("T,dtype", [(196, torch.float32), (1000, torch.float32), (196, torch.bfloat16)])
def test_gate_on_tiles_redone_by_the_renormalising_recurrence(ops, T, dtype):
    """Channel tiles with parameters outside the plain-sum regime are emitted by the second walk of the kernel: they
    take the gate there."""
    C = 192
    rng = np.random.default_rng(T)
    w = rng.uniform(-5, 3, C).astype(np.float32) / T
    u = rng.uniform(-1, 1, C).astype(np.float32) / T
    w[70] = 2.5                                               # tile 1 leaves the plain-sum regime
    u[140] = 30.0                                             # and so does tile 2
    _case(ops, 2, T, C, dtype, seed=T + 1, w=w, u=u)


@pytest.mark.parametrize("B,T,C,dtype,offset", [
    (4, 576, 128, torch.bfloat16, 0),     # one-launch kernel for three super-chunks of 16-bit rows: gate as a second pass
    (2, 300, 64, torch.float16, 0),
    (2, 196, 100, torch.float32, 0),      # rows that are no multiple of 16 bytes
    (2, 196, 192, torch.bfloat16, 3),     # tensors that start off a 16-byte boundary
    (2, 1024, 192, torch.float32, 1)])
def test_calls_served_without_fusion_give_the_same_result(ops, B, T, C, dtype, offset):
    _case(ops, B, T, C, dtype, seed=B + T + C, offset=offset)


def test_gate_argument_checks(ops):
    lib = ops.lib()
    w = torch.zeros(64, device=DEV)
    k = torch.zeros(1, 8, 64, device=DEV)
    with pytest.raises(RuntimeError):
        ops.bi_wkv_forward(w, w, k, k, gate=torch.zeros(1, 8, 32, device=DEV))
    with pytest.raises(RuntimeError):
        ops.bi_wkv_forward(w, w, k, k, gate=k.bfloat16())
    assert lib.vrwkv_biwkv_fwd_gate(w.data_ptr(), w.data_ptr(), k.data_ptr(), k.data_ptr(), None, k.data_ptr(),
                                    1, 8, 64, 0, None, 0, None) == 1
    assert b"biwkv_fwd_gate" in lib.vrwkv_last_error()


def test_backbone_inference_with_the_gate_inside_the_operator(ops):
    """VRWKV_SpatialMix.forward without key_norm takes the gated entry point when no gradient is recorded; the model's
    output must agree with the same model run with the gate as a pass of its own (bf16: one rounding fewer per block)."""
    torch.manual_seed(3)
    net = ops.VRWKV(img_size=224, patch_size=16, embed_dims=192, depth=3, post_norm=True, init_values=1e-2).to(DEV).bfloat16().eval()
    img = torch.randn(4, 3, 224, 224, device=DEV, dtype=torch.bfloat16)
    assert all(m.fused_gate for m in net.modules() if hasattr(m, "fused_gate"))
    with torch.no_grad():
        a = net(img).float()
        for m in net.modules():
            if hasattr(m, "fused_gate"):
                m.fused_gate = False
        b = net(img).float()
    assert torch.isfinite(a).all()
    err = (a - b).abs().max().item() / b.abs().max().item()
    print(f"  fused gate against separate gate pass: {err:.2e}")
    assert err <= 2e-2
