"""vrwkv_biwkv_fwd_static -- the Bi-WKV forward that allocates nothing (its long-sequence workspace is an array built
into the library) -- through the C ABI, against vrwkv_biwkv_fwd with a caller-owned workspace: bit-identical results
(same kernels), on two calls in a row, the second with a smaller input, then a short sequence that needs no
workspace, and the rejection of a shape whose workspace exceeds the built-in one."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _inputs(B, T, C, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, T, C, generator=g).to(DEV).to(dtype)
    v = torch.randn(B, T, C, generator=g).to(DEV).to(dtype)
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / max(C - 1, 1)) / T).to(DEV)
    u = ((np.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    return w, u, k, v


def _both(lib, check, w, u, k, v):
    B, T, C = k.shape
    dt = _DT[k.dtype]
    st = torch.cuda.current_stream().cuda_stream
    ws_bytes = lib.vrwkv_biwkv_fwd_workspace_bytes(B, T, C, dt)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=DEV)
    y_ref = torch.full_like(k, float("nan"))
    check(lib.vrwkv_biwkv_fwd(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), y_ref.data_ptr(), B, T, C, dt,
                              ws.data_ptr(), ws_bytes, st))
    y = torch.full_like(k, float("nan"))
    check(lib.vrwkv_biwkv_fwd_static(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), B, T, C, dt, st))
    torch.cuda.synchronize()
    return y, y_ref, ws_bytes


def test_static_workspace_entry_point_matches_the_caller_workspace_one():
    import vision_rwkv_amd as ops
    from vision_rwkv_amd import _lib
    lib = ops.lib()
    assert torch.cuda.is_available()
    cap = lib.vrwkv_biwkv_fwd_static_max_workspace_bytes()
    assert cap == 4 << 20
    # two calls in a row that use the workspace, the second smaller; then one that needs none
    for (B, T, C, dtype, seed) in ((2, 4150, 768, torch.bfloat16, 1), (2, 1024, 192, torch.float32, 2),
                                   (3, 196, 192, torch.float32, 3)):
        print("case", B, T, C, dtype, flush=True)
        w, u, k, v = _inputs(B, T, C, dtype, seed)
        y, y_ref, ws_bytes = _both(lib, _lib.check, w, u, k, v)
        assert (ws_bytes > 0) == (T > 224) and ws_bytes <= cap
        assert torch.isfinite(y.float()).all()
        assert torch.equal(y, y_ref)
    # the first (larger) case again: the array still holds the last call's entries and all of them are rewritten
    w, u, k, v = _inputs(2, 4150, 768, torch.bfloat16, 1)
    y, y_ref, _ = _both(lib, _lib.check, w, u, k, v)
    assert torch.equal(y, y_ref)
    # a shape beyond the built-in workspace is refused with a clear message, and nothing is launched
    B, T, C = 64, 4150, 1024
    assert lib.vrwkv_biwkv_fwd_workspace_bytes(B, T, C, 0) > cap
    w, u, k, v = _inputs(1, 8, 64, torch.float32, 4)
    rc = lib.vrwkv_biwkv_fwd_static(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), k.data_ptr(), B, T, C, 0, None)
    assert rc == 5
    assert b"built-in" in lib.vrwkv_last_error()
