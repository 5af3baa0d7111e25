"""Stand-ins for the three extension modules the reference compiles at import, with their exact call signatures,
for a checkout that keeps its own autograd Functions and only swaps the `load(...)` line:

    wkv_cuda  = vision_rwkv_amd.ext.bi_wkv    # cuda_new/bi_wkv.cpp:49-57   bi_wkv_forward / bi_wkv_backward
    wkv_cuda  = vision_rwkv_amd.ext.wkv       # cuda/wkv_op.cpp:13-21       forward / backward, results passed in
    wkv6_cuda = vision_rwkv_amd.ext.wkv6      # cuda_v6/wkv6_op.cpp:13-21   forward / backward, results passed in

The same functions are registered as torch.ops.bi_wkv.*, torch.ops.wkv.* and torch.ops.wkv6.* (the reference's
TORCH_LIBRARY blocks) unless another library in the process already owns such a namespace; REGISTERED lists
the namespaces this module defined.

Two things differ from the reference kernels and are invisible to its Python callers, which only ever sum these
buffers over the batch (classification/mae/vrwkv/vrwkv.py:75-86, vrwkv6.py:68): the per-batch gradient buffers
gw, gu of shape (B, C) come back with the batch total in row 0 and zeros elsewhere.
"""
import torch

from . import ops


class bi_wkv:
    """cuda_new/bi_wkv.cpp:23-47."""
    bi_wkv_forward = staticmethod(ops.bi_wkv_forward)
    bi_wkv_backward = staticmethod(ops.bi_wkv_backward)


def _legacy_forward(B, T, C, w, u, k, v, y):
    if tuple(k.shape) != (B, T, C):
        raise RuntimeError(f"k has shape {tuple(k.shape)}, expected {(B, T, C)}")
    ops.bi_wkv_forward(w, u, k, v, out=y)


def _legacy_backward(B, T, C, w, u, k, v, gy, gw, gu, gk, gv):
    if tuple(k.shape) != (B, T, C) or tuple(gw.shape) != (B, C) or tuple(gu.shape) != (B, C):
        raise RuntimeError("k must be (B,T,C) and gw, gu (B,C)")
    if not (gw.is_contiguous() and gu.is_contiguous()):
        raise RuntimeError("gw and gu must be contiguous")
    gw.zero_()
    gu.zero_()
    if B > 0:
        ops.bi_wkv_backward(w, u, k, v, gy, out=(gw[0], gu[0], gk, gv))


class wkv:
    """cuda/wkv_op.cpp:6-11 (fp32 tensors, results written into the caller's y / gw, gu, gk, gv)."""
    forward = staticmethod(_legacy_forward)
    backward = staticmethod(_legacy_backward)


def _wkv6_forward(B, T, C, H, r, k, v, w, u, y):
    ops.wkv6_forward(B, T, C, H, r, k, v, w, u, w_is_ew=True, out=y)


def _wkv6_backward(B, T, C, H, r, k, v, w, u, gy, gr, gk, gv, gw, gu):
    if tuple(gu.shape) != (B, C) or not gu.is_contiguous():
        raise RuntimeError("gu must be a contiguous (B,C) tensor")
    gu.zero_()
    if B > 0:
        ops.wkv6_backward(B, T, C, H, r, k, v, w, u, gy, w_is_ew=True, out=(gr, gk, gv, gw, gu[0].view(H, C // H)))


class wkv6:
    """cuda_v6/wkv6_op.cpp:7-12: w is ew = -exp(w_raw) as WKV_6.forward forms it (vrwkv6.py:48); gw is the gradient
    with respect to w_raw, which is what the reference kernel returns (vrwkv6.py:70 hands it on unchanged)."""
    forward = staticmethod(_wkv6_forward)
    backward = staticmethod(_wkv6_backward)


REGISTERED = []
_libs = []


def _register():
    defs = {
        "bi_wkv": [("bi_wkv_forward(Tensor w, Tensor u, Tensor k, Tensor v) -> Tensor",
                    lambda w, u, k, v: ops.bi_wkv_forward(w, u, k, v)),
                   ("bi_wkv_backward(Tensor w, Tensor u, Tensor k, Tensor v, Tensor gy) -> Tensor[]",
                    lambda w, u, k, v, gy: ops.bi_wkv_backward(w, u, k, v, gy))],
        "wkv": [("forward(int B, int T, int C, Tensor w, Tensor u, Tensor k, Tensor v, Tensor(a!) y) -> ()", _legacy_forward),
                ("backward(int B, int T, int C, Tensor w, Tensor u, Tensor k, Tensor v, Tensor gy, Tensor(a!) gw, "
                 "Tensor(b!) gu, Tensor(c!) gk, Tensor(d!) gv) -> ()", _legacy_backward)],
        "wkv6": [("forward(int B, int T, int C, int H, Tensor r, Tensor k, Tensor v, Tensor w, Tensor u, Tensor(a!) y) -> ()",
                  _wkv6_forward),
                 ("backward(int B, int T, int C, int H, Tensor r, Tensor k, Tensor v, Tensor w, Tensor u, Tensor gy, "
                  "Tensor(a!) gr, Tensor(b!) gk, Tensor(c!) gv, Tensor(d!) gw, Tensor(e!) gu) -> ()", _wkv6_backward)],
    }
    for ns, fns in defs.items():
        try:
            lib = torch.library.Library(ns, "DEF")
            for schema, fn in fns:
                lib.define(schema)
                lib.impl(schema.split("(")[0], fn, "CUDA")
        except RuntimeError:
            continue                                  # the namespace belongs to another library in this process
        _libs.append(lib)                             # registrations live as long as the Library object
        REGISTERED.append(ns)


_register()
