"""HIP graph capture of the operators.  Every entry point only launches kernels on the stream it is given (no
allocation, no memset node, no synchronisation inside the library), so a caller may record it into a graph to hide
the launch cost of the multi-kernel paths.  Each graph here is replayed three times, with new inputs copied into its
buffers and eager work plus a synchronisation between the replays, and every replay must reproduce the eager call on
the same inputs bit for bit (the kernels have no order-dependent sums)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _wu(C, T):
    c = torch.arange(C, dtype=torch.float32)
    w = ((-5 + 8 * c / max(C - 1, 1)) / T).to(DEV)
    u = ((-1.2 + 0.5 * (((c + 1) % 3) - 1)) / T).to(DEV)
    return w, u


def _replay_and_compare(make_inputs, run, n_replays=3):
    """make_inputs(seed) -> tuple of tensors; run(*tensors) -> tuple of result tensors."""
    static_in = [t.clone() for t in make_inputs(0)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up outside the capture, as torch asks
        run(*static_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = run(*static_in)
    for rep in range(n_replays):
        fresh = make_inputs(100 + rep)
        for dst, src in zip(static_in, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        want = run(*fresh)                             # eager work between the replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.isfinite(a.float()).all(), (rep, i)
            assert torch.equal(a, b), (rep, i, (a.float() - b.float()).abs().max().item())


@pytest.mark.parametrize("B,T,C,dtype", [(3, 196, 192, torch.float32),      # one launch
                                          (2, 1024, 192, torch.float32),     # aggregate + emitting kernel, workspace
                                          (2, 4150, 256, torch.bfloat16),    # the same with 19 super-chunks
                                          (4, 576, 128, torch.bfloat16)])    # one-launch kernel for three super-chunks
def test_biwkv_forward_in_a_graph(B, T, C, dtype):
    import vision_rwkv_amd as ops
    w, u = _wu(C, T)

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(B, T, C, generator=g).to(DEV).to(dtype), torch.randn(B, T, C, generator=g).to(DEV).to(dtype))

    print("biwkv forward graph", B, T, C, dtype, flush=True)
    _replay_and_compare(make, lambda k, v: (ops.bi_wkv_forward(w, u, k, v),))


@pytest.mark.parametrize("B,T,C", [(4, 196, 128), (2, 700, 128)])           # tile kernel; three-launch long path
def test_biwkv_backward_in_a_graph(B, T, C):
    import vision_rwkv_amd as ops
    w, u = _wu(C, T)

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        return tuple(torch.randn(B, T, C, generator=g).to(DEV) for _ in range(3))

    print("biwkv backward graph", B, T, C, flush=True)
    _replay_and_compare(make, lambda k, v, gy: tuple(ops.bi_wkv_backward(w, u, k, v, gy)))


def test_wkv6_forward_and_backward_in_a_graph():
    import vision_rwkv_amd as ops
    B, T, H = 2, 196, 2
    C = 64 * H
    u = (torch.randn(H, 64, generator=torch.Generator().manual_seed(5)) * 0.1).to(DEV)

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        r, k, v = (torch.randn(B, T, C, generator=g).to(DEV).bfloat16() for _ in range(3))
        w = (torch.randn(B, T, C, generator=g) * 0.5 - 0.5).to(DEV)
        gy = torch.randn(B, T, C, generator=g).to(DEV)
        return r, k, v, w, gy

    def run(r, k, v, w, gy):
        y = ops.wkv6_forward(B, T, C, H, r, k, v, w, u)
        return (y,) + tuple(ops.wkv6_backward(B, T, C, H, r, k, v, w, u, gy))

    print("wkv6 forward + backward graph", B, T, C, flush=True)
    _replay_and_compare(make, run)
