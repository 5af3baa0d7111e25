"""Edge cases of the two WKV operators on the GPU: empty batches, one- and two-token sequences, and the
closed forms those reduce to (no oracle call is needed for them: the expected values are textbook).

  Bi-WKV, T = 1: the only weight is the bonus term, so y = v exactly (up to the output rounding).
  Bi-WKV, T = 2: y_0 = (e^{u+k_0} v_0 + e^{k_1} v_1) / (e^{u+k_0} + e^{k_1})  (neighbours have decay exponent 0).
  wkv6,  T = 1: y[i] = (sum_j r[j] u[j] k[j]) v[i] per head.
  wkv6,  T = 2: y_0 = (r_0 . (u k_0)) v_0 + (r_0 . k_1) v_1  (adjacent tokens: empty decay product).
Tolerances: 1e-4 fp32, 1e-2 16-bit I/O (Bi-WKV); 1e-3 (wkv6) of max(|ref|, rms(ref)).
"""
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


@pytest.mark.parametrize("shape", [(0, 196, 768), (4, 0, 64)])
def test_biwkv_empty_inputs(ops, shape):
    C = shape[2]
    w = torch.randn(C, device=DEV, requires_grad=True)
    u = torch.randn(C, device=DEV, requires_grad=True)
    k = torch.randn(*shape, device=DEV, requires_grad=True)
    v = torch.randn(*shape, device=DEV, requires_grad=True)
    y = ops.RUN_CUDA(w, u, k, v)
    assert tuple(y.shape) == shape and y.dtype == torch.float32
    y.sum().backward()
    torch.cuda.synchronize()
    assert k.grad.shape == k.shape and v.grad.shape == v.shape
    assert torch.count_nonzero(w.grad).item() == 0 and torch.count_nonzero(u.grad).item() == 0


@pytest.mark.parametrize("shape", [(0, 196, 128), (2, 0, 64)])
def test_wkv6_empty_inputs(ops, shape):
    B, T, C = shape
    H = C // 64
    r, k, v, w = (torch.randn(*shape, device=DEV, requires_grad=True) for _ in range(4))
    u = torch.randn(H, 64, device=DEV, requires_grad=True)
    y = ops.RUN_CUDA_RWKV6(B, T, C, H, r, k, v, w, u)
    assert tuple(y.shape) == shape and y.dtype == torch.float32
    y.sum().backward()
    torch.cuda.synchronize()
    assert r.grad.shape == r.shape and w.grad.shape == w.shape
    assert tuple(u.grad.shape) == (H, 64) and torch.count_nonzero(u.grad).item() == 0


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 1e-2), (torch.float16, 1e-2)])
@pytest.mark.parametrize("B,C", [(3, 192), (1, 37), (5, 768)])
def test_biwkv_one_and_two_tokens(ops, B, C, dtype, tol):
    g = torch.Generator(device="cpu").manual_seed(B * 1000 + C)
    w = (torch.rand(C, generator=g) * 8 - 5).to(DEV)
    u = torch.randn(C, generator=g).to(DEV)
    for T in (1, 2):
        k = torch.randn(B, T, C, generator=g).to(DEV).to(dtype)
        v = torch.randn(B, T, C, generator=g).to(DEV).to(dtype)
        y = ops.bi_wkv_forward(w / T, u / T, k, v).double().cpu().numpy()
        kd, vd, ud = k.double().cpu().numpy(), v.double().cpu().numpy(), (u / T).double().cpu().numpy()
        if T == 1:
            ref = vd
        else:
            ref = np.empty_like(vd)
            for t in (0, 1):
                a, b = np.exp(ud + kd[:, t]), np.exp(kd[:, 1 - t])
                ref[:, t] = (a * vd[:, t] + b * vd[:, 1 - t]) / (a + b)
        assert rel_err(y, ref) <= tol, (T, rel_err(y, ref))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wkv6_one_and_two_tokens(ops, dtype):
    B, H = 3, 2
    C = H * 64
    g = torch.Generator(device="cpu").manual_seed(7)
    u = (0.1 * torch.randn(H, 64, generator=g)).to(DEV)
    for T in (1, 2):
        r, k, v = (torch.randn(B, T, C, generator=g).to(DEV).to(dtype) for _ in range(3))
        w = (torch.randn(B, T, C, generator=g) * 0.5 - 0.5).to(DEV)
        y = ops.RUN_CUDA_RWKV6(B, T, C, H, r, k, v, w, u).double().cpu().numpy().reshape(B, T, H, 64)
        rd, kd, vd = (x.double().cpu().numpy().reshape(B, T, H, 64) for x in (r, k, v))
        ud = u.double().cpu().numpy()[None]
        ref = np.empty_like(vd)
        for t in range(T):
            ref[:, t] = (rd[:, t] * ud * kd[:, t]).sum(-1, keepdims=True) * vd[:, t]
            if T == 2:
                ref[:, t] += (rd[:, t] * kd[:, 1 - t]).sum(-1, keepdims=True) * vd[:, 1 - t]
        assert rel_err(y, ref) <= 1e-3, (T, rel_err(y, ref))


def test_backward_gradient_sum_identities_full_size(ops):
    """Size-independent identities of the Bi-WKV gradients at the VRWKV-B shape: y is unchanged by k -> k + const, so
    sum_t gk = 0, and the weights of a token's output sum to one, so sum_t gv = sum_t gy (both per (b, c))."""
    B, T, C = 64, 196, 768
    g = torch.Generator(device="cpu").manual_seed(11)
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / (C - 1)) / T).to(DEV)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    k = torch.randn(B, T, C, generator=g).to(DEV)
    v = torch.randn(B, T, C, generator=g).to(DEV)
    gy = torch.randn(B, T, C, generator=g).to(DEV)
    gw, gu, gk, gv = ops.bi_wkv_backward(w, u, k, v, gy)
    scale = gk.abs().sum(1).double()
    assert (gk.double().sum(1).abs() <= 1e-4 * scale + 1e-6).all()
    diff = (gv.double().sum(1) - gy.double().sum(1)).abs()
    assert (diff <= 1e-4 * gy.abs().sum(1).double() + 1e-6).all()
    assert torch.isfinite(gw).all() and torch.isfinite(gu).all()


def _offset_copy(t, n=1):
    """Same values in storage that starts n elements into an allocation: contiguous, but not 16-byte aligned."""
    buf = torch.empty(t.numel() + n, dtype=t.dtype, device=t.device)
    out = buf[n:].view(t.shape)
    out.copy_(t)
    assert out.is_contiguous() and out.data_ptr() % 16 != 0
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,C", [(3, 196, 192), (2, 500, 128)])
def test_biwkv_tensors_that_are_not_16_byte_aligned(ops, B, T, C, dtype):
    """k, v, gy views that start one element into their allocation take the kernels without 16-byte row staging;
    results agree with the aligned call (same arithmetic, other load path): 1e-5 of the tensor's scale."""
    g = torch.Generator(device="cpu").manual_seed(T + C)
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / (C - 1)) / T).to(DEV)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    k, v, gy = (torch.randn(B, T, C, generator=g).to(DEV).to(dtype) for _ in range(3))
    y0 = ops.bi_wkv_forward(w, u, k, v)
    g0 = ops.bi_wkv_backward(w, u, k, v, gy)
    ko, vo, gyo = _offset_copy(k), _offset_copy(v), _offset_copy(gy)
    y1 = ops.bi_wkv_forward(w, u, ko, vo)
    g1 = ops.bi_wkv_backward(w, u, ko, vo, gyo)
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -7
    assert (y1.float() - y0.float()).abs().max() <= tol * y0.float().abs().max()
    for a, b in zip(g1, g0):
        assert (a.float() - b.float()).abs().max() <= max(tol, 1e-4) * b.float().abs().max()


def test_wkv6_tensors_that_are_not_16_byte_aligned(ops):
    B, T, H = 2, 100, 2
    C = H * 64
    g = torch.Generator(device="cpu").manual_seed(3)
    r, k, v = (torch.randn(B, T, C, generator=g).to(DEV).to(torch.bfloat16) for _ in range(3))
    w = (torch.randn(B, T, C, generator=g) * 0.5 - 0.5).to(DEV)
    gy = torch.randn(B, T, C, generator=g).to(DEV)
    u = (0.1 * torch.randn(H, 64, generator=g)).to(DEV)
    y0 = ops.wkv6_forward(B, T, C, H, r, k, v, w, u)
    g0 = ops.wkv6_backward(B, T, C, H, r, k, v, w, u, gy)
    ro, ko, vo, wo, gyo = (_offset_copy(t) for t in (r, k, v, w, gy))
    y1 = ops.wkv6_forward(B, T, C, H, ro, ko, vo, wo, u)
    g1 = ops.wkv6_backward(B, T, C, H, ro, ko, vo, wo, u, gyo)
    assert torch.equal(y1, y0)
    for a, b in zip(g1, g0):
        assert torch.equal(a, b)


def test_tensors_larger_than_4_gib(ops):
    """Maximum sizes: B*T*C*4 bytes beyond 2^32 (7200 x 196 x 768), all four operators.  No oracle run at this size:
    the kernels are deterministic and treat every (b, channel tile) / (b, head) alone, so the last and the first
    batch elements of the big call must equal, bit for bit, a call on those elements alone (which the other tests
    pin to the oracle); a 32-bit offset anywhere would break exactly that.  Plus sum_t gk = 0 and finiteness overall."""
    if torch.cuda.get_device_properties(0).total_memory < 100e9:
        pytest.skip("needs about 50 GB of device memory")
    B, T, C = 7200, 196, 768
    H = C // 64
    assert B * T * C * 4 > 2 ** 32
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / (C - 1)) / T).to(DEV)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    g = torch.Generator(device=DEV).manual_seed(1)
    k, v, gy = (torch.randn(B, T, C, device=DEV, generator=g) for _ in range(3))
    tail, head = slice(B - 3, B), slice(0, 3)
    part = lambda t, s: t[s].contiguous()

    y = ops.bi_wkv_forward(w, u, k, v)
    for s in (tail, head):
        assert torch.equal(y[s], ops.bi_wkv_forward(w, u, part(k, s), part(v, s)))
    assert torch.isfinite(y).all()
    del y
    gw, gu, gk, gv = ops.bi_wkv_backward(w, u, k, v, gy)
    _, _, gk2, gv2 = ops.bi_wkv_backward(w, u, part(k, tail), part(v, tail), part(gy, tail))
    assert torch.equal(gk[tail], gk2) and torch.equal(gv[tail], gv2)
    assert gk.double().sum(1).abs().max().item() <= 1e-3
    assert torch.isfinite(gw).all() and torch.isfinite(gu).all()
    del gk, gv, gk2, gv2
    torch.cuda.empty_cache()

    r = torch.randn(B, T, C, device=DEV, generator=g).bfloat16()
    kb, vb = k.bfloat16(), v.bfloat16()
    del k, v
    wl = torch.randn(B, T, C, device=DEV, generator=g) * 0.5 - 0.5
    u6 = 0.1 * torch.randn(H, 64, device=DEV, generator=g)
    y = ops.wkv6_forward(B, T, C, H, r, kb, vb, wl, u6)
    assert torch.equal(y[tail], ops.wkv6_forward(3, T, C, H, part(r, tail), part(kb, tail), part(vb, tail), part(wl, tail), u6))
    assert torch.isfinite(y).all()
    del y
    big = ops.wkv6_backward(B, T, C, H, r, kb, vb, wl, u6, gy)
    small = ops.wkv6_backward(3, T, C, H, part(r, tail), part(kb, tail), part(vb, tail), part(wl, tail), u6, part(gy, tail))
    for a, b in zip(big[:4], small[:4]):
        assert torch.equal(a[tail], b)
    assert torch.isfinite(big[4]).all()
    del big, small, r, kb, vb, wl, gy
    torch.cuda.empty_cache()


def test_elementwise_kernels_beyond_4_gib(ops):
    """The fused shift + mix, row epilogue, GroupNorm x gate and five-mix kernels on 7200 x 196 x 768 fp32 tensors
    (4.3 GB each): every output row depends on its own batch element only, so the last batch elements must equal,
    bit for bit, a call on those elements alone (pinned against tensor ops by the other tests)."""
    if torch.cuda.get_device_properties(0).total_memory < 100e9:
        pytest.skip("needs about 55 GB of device memory")
    O = ops.ops
    B, T, C = 7200, 196, 768
    g = torch.Generator(device=DEV).manual_seed(2)
    tail = slice(B - 2, B)
    part = lambda t: t[tail].contiguous()
    x, other = (torch.randn(B, T, C, device=DEV, generator=g) for _ in range(2))
    lw, lb = (torch.randn(C, device=DEV, generator=g) for _ in range(2))
    mixes = [torch.rand(C, device=DEV, generator=g) for _ in range(3)]
    with torch.no_grad():
        outs = ops.q_shift_mix(x, mixes, patch_resolution=(14, 14))
        for a, b in zip(outs, ops.q_shift_mix(part(x), mixes, patch_resolution=(14, 14))):
            assert torch.equal(a[tail], b)
        del outs
        r = ops.row_fuse(x, other, lw, lb, post=O.POST_SIGMOID_GATE)
        assert torch.equal(r[tail], ops.row_fuse(part(x), part(other), lw, lb, post=O.POST_SIGMOID_GATE))
        assert torch.isfinite(r).all()
        r = ops.groupnorm_gate(x, other, lw, lb, 12)
        assert torch.equal(r[tail], ops.groupnorm_gate(part(x), part(other), lw, lb, 12))
        assert torch.isfinite(r).all()
        del r
        m = torch.randn(5, B, T, C, device=DEV, generator=g)
        maas = [torch.rand(C, device=DEV, generator=g) for _ in range(5)]
        outs = ops.maa_mix(x, other, m, maas)
        for a, b in zip(outs, ops.maa_mix(part(x), part(other), m[:, tail].contiguous(), maas)):
            assert torch.equal(a[tail], b)
    del outs, m, x, other
    torch.cuda.empty_cache()


def test_concurrent_calls_from_threads_on_their_own_streams(ops):
    """The library keeps no state between calls besides a thread-local error string, and every call brings its own
    workspace: four host threads, each on its own stream, repeat the long-sequence Bi-WKV forward (which uses a
    workspace) and the wkv6 forward, and must reproduce the single-threaded results bit for bit."""
    import threading
    B, T, C, H = 2, 700, 128, 2
    g = torch.Generator(device="cpu").manual_seed(9)
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / (C - 1)) / T).to(DEV)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    sets = []
    for _ in range(4):
        k, v, r = (torch.randn(B, T, C, generator=g).to(DEV) for _ in range(3))
        wl = (torch.randn(B, T, C, generator=g) * 0.5 - 0.5).to(DEV)
        sets.append((k, v, r, wl))
    u6 = (0.1 * torch.randn(H, 64, generator=g)).to(DEV)
    ref = [(ops.bi_wkv_forward(w, u, k, v), ops.wkv6_forward(B, T, C, H, r, k, v, wl, u6)) for k, v, r, wl in sets]
    torch.cuda.synchronize()
    errors = []

    def work(i):
        try:
            k, v, r, wl = sets[i]
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for _ in range(10):
                    y = ops.bi_wkv_forward(w, u, k, v)
                    y6 = ops.wkv6_forward(B, T, C, H, r, k, v, wl, u6)
                st.synchronize()
            if not (torch.equal(y, ref[i][0]) and torch.equal(y6, ref[i][1])):
                errors.append(f"thread {i}: results differ")
        except Exception as e:                                        # noqa: BLE001 - reported below
            errors.append(f"thread {i}: {e!r}")

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=60)
    assert not errors, errors
