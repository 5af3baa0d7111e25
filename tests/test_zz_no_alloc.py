"""vrwkv_biwkv_fwd_static -- the Bi-WKV forward that allocates nothing (its long-sequence workspace is an array built
into the library) -- through the C ABI, against vrwkv_biwkv_fwd with a caller-owned workspace: bit-identical results
(same kernels), on two calls in a row, the second with a smaller input, then a short sequence that needs no
workspace, and the rejection of a shape whose workspace exceeds the built-in one.  Also: against the CPU oracle, with
the device memory in use unchanged across the call, and recorded into a HIP graph (after a first call outside the
capture, which is where the library looks up the address of its array)."""
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
    torch.cuda.synchronize()
    free_before, allocated_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    check(lib.vrwkv_biwkv_fwd_static(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(), B, T, C, dt, st))
    torch.cuda.synchronize()
    # the call took no device memory, neither through torch's allocator nor behind its back
    assert torch.cuda.memory_allocated() == allocated_before
    assert torch.cuda.mem_get_info()[0] >= free_before
    return y, y_ref, ws_bytes


def test_static_workspace_entry_point_matches_the_caller_workspace_one():
    import vision_rwkv_amd as ops
    from vision_rwkv_amd import _lib
    lib = ops.lib()
    assert torch.cuda.is_available()
    cap = lib.vrwkv_biwkv_fwd_static_max_workspace_bytes()
    assert cap == 4 << 20
    # the first call on a device looks up the built-in array, which makes the library's code object and with it the
    # 4 MiB array resident (once per process); the memory checks in _both apply to the calls after it
    w, u, k, v = _inputs(1, 300, 64, torch.float32, 9)
    _lib.check(lib.vrwkv_biwkv_fwd_static(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), torch.empty_like(k).data_ptr(),
                                          1, 300, 64, 0, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    # two calls in a row that use the workspace, the second smaller; then one that needs none
    for (B, T, C, dtype, seed) in ((2, 4150, 768, torch.bfloat16, 1), (2, 1024, 192, torch.float32, 2),
                                   (3, 196, 192, torch.float32, 3)):
        print("case", B, T, C, dtype, flush=True)
        w, u, k, v = _inputs(B, T, C, dtype, seed)
        y, y_ref, ws_bytes = _both(lib, _lib.check, w, u, k, v)
        assert (ws_bytes > 0) == (T > 224) and ws_bytes <= cap
        assert torch.isfinite(y.float()).all()
        assert torch.equal(y, y_ref)
        if dtype == torch.float32 and T > 224:
            # ... and the shared kernels are right: the CPU oracle's recurrence on the same inputs (fp32 bar 1e-4)
            from oracle import clib
            from conftest import rel_err
            f = lambda x: x.float().cpu().numpy()
            assert rel_err(f(y), clib.biwkv_fwd(f(w), f(u), f(k), f(v))) <= 1e-4
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


def test_static_workspace_entry_point_in_a_graph():
    """The entry point recorded into a HIP graph (it launches kernels only: no allocation, no memset node).  Its first
    call on a device looks up the address of the built-in array and must happen outside a capture, so one call is made
    first; every replay, on new inputs, must reproduce vrwkv_biwkv_fwd with a caller-owned workspace bit for bit."""
    import vision_rwkv_amd as ops
    from vision_rwkv_amd import _lib
    lib = ops.lib()
    for (B, T, C, dtype) in ((2, 1024, 192, torch.float32), (2, 4150, 256, torch.bfloat16)):
        print("graph case", B, T, C, dtype, flush=True)
        dt = _DT[dtype]
        w, u, k, v = _inputs(B, T, C, dtype, 10)
        y = torch.empty_like(k)

        def run():
            st = torch.cuda.current_stream().cuda_stream
            _lib.check(lib.vrwkv_biwkv_fwd_static(w.data_ptr(), u.data_ptr(), k.data_ptr(), v.data_ptr(), y.data_ptr(),
                                                  B, T, C, dt, st))

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):                  # first call outside the capture
            run()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        for rep in range(3):
            _, _, k2, v2 = _inputs(B, T, C, dtype, 20 + rep)
            k.copy_(k2)
            v.copy_(v2)
            graph.replay()
            torch.cuda.synchronize()
            got = y.clone()
            want = ops.bi_wkv_forward(w, u, k2, v2)    # eager work between the replays
            torch.cuda.synchronize()
            assert torch.isfinite(got.float()).all(), rep
            assert torch.equal(got, want), (rep, (got.float() - want.float()).abs().max().item())
