"""ctypes binding of libvrwkv_hip.so (the C ABI declared in include/vrwkv_hip.h).

The library is loaded from this directory; it is never compiled at import time and there
is no fallback: a missing library is a hard error.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libvrwkv_hip.so")

VRWKV_F32, VRWKV_BF16, VRWKV_F16 = 0, 1, 2
STATUS_NAMES = {0: "OK", 1: "INVALID_ARG", 2: "UNSUPPORTED_DTYPE", 3: "UNSUPPORTED_SHAPE",
                4: "LAUNCH_FAILED", 5: "WORKSPACE_TOO_SMALL"}

_lib = None


class VrwkvError(RuntimeError):
    """Non-zero status from the C ABI (mirrors the RuntimeError TORCH_CHECK raises at
    classification/mmcls_custom/models/backbones/cuda_new/bi_wkv.cpp:6-8)."""

    def __init__(self, status, message):
        super().__init__(f"vrwkv status {status} ({STATUS_NAMES.get(status, '?')}): {message}")
        self.status = status


def build(force=True):
    """Compile libvrwkv_hip.so for gfx950 with the Makefile in csrc/ (hipcc cross-compiles
    without a GPU)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True)
    return LIB_PATH


def _declare(lib):
    c = ctypes
    vp, fp, i, sz = c.c_void_p, c.c_void_p, c.c_int, c.c_size_t
    lib.vrwkv_version.argtypes = []
    lib.vrwkv_version.restype = i
    lib.vrwkv_last_error.argtypes = []
    lib.vrwkv_last_error.restype = c.c_char_p
    lib.vrwkv_set_option.argtypes = [c.c_char_p, i]
    lib.vrwkv_set_option.restype = i
    lib.vrwkv_get_option.argtypes = [c.c_char_p, c.POINTER(c.c_int)]
    lib.vrwkv_get_option.restype = i
    lib.vrwkv_biwkv_fwd_workspace_bytes.argtypes = [i, i, i, i]
    lib.vrwkv_biwkv_fwd_workspace_bytes.restype = sz
    lib.vrwkv_biwkv_fwd.argtypes = [fp, fp, vp, vp, vp, i, i, i, i, vp, sz, vp]
    lib.vrwkv_biwkv_fwd.restype = i
    lib.vrwkv_biwkv_fwd_gate.argtypes = [fp, fp, vp, vp, vp, vp, i, i, i, i, vp, sz, vp]
    lib.vrwkv_biwkv_fwd_gate.restype = i
    lib.vrwkv_biwkv_fwd_static_max_workspace_bytes.argtypes = []
    lib.vrwkv_biwkv_fwd_static_max_workspace_bytes.restype = sz
    lib.vrwkv_biwkv_fwd_static.argtypes = [fp, fp, vp, vp, vp, i, i, i, i, vp]
    lib.vrwkv_biwkv_fwd_static.restype = i
    lib.vrwkv_biwkv_bwd_workspace_bytes.argtypes = [i, i, i, i]
    lib.vrwkv_biwkv_bwd_workspace_bytes.restype = sz
    lib.vrwkv_biwkv_bwd.argtypes = [fp, fp, vp, vp, vp, fp, fp, vp, vp, i, i, i, i, vp, sz, vp]
    lib.vrwkv_biwkv_bwd.restype = i
    lib.vrwkv_wkv6_fwd_workspace_bytes.argtypes = [i, i, i, i]
    lib.vrwkv_wkv6_fwd_workspace_bytes.restype = sz
    lib.vrwkv_wkv6_fwd.argtypes = [vp, vp, vp, vp, fp, vp, i, i, i, i, i, i, i, vp, sz, vp]
    lib.vrwkv_wkv6_fwd.restype = i
    lib.vrwkv_wkv6_fwd_phases_bytes.argtypes = [i, i, i]
    lib.vrwkv_wkv6_fwd_phases_bytes.restype = sz
    lib.vrwkv_wkv6_fwd_phases.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, vp, sz, vp]
    lib.vrwkv_wkv6_fwd_phases.restype = i
    lib.vrwkv_wkv6_bwd_workspace_bytes.argtypes = [i, i, i, i]
    lib.vrwkv_wkv6_bwd_workspace_bytes.restype = sz
    lib.vrwkv_wkv6_bwd.argtypes = [vp, vp, vp, vp, fp, fp, fp, fp, fp, fp, fp, i, i, i, i, i, i, i, vp, sz, vp]
    lib.vrwkv_wkv6_bwd.restype = i
    lib.vrwkv_qshift_mix.argtypes = [vp, fp, c.POINTER(c.c_void_p), i, i, i, i, i, i, i, i, i, i, vp]
    lib.vrwkv_qshift_mix.restype = i
    lib.vrwkv_qshift_mix_bwd_workspace_bytes.argtypes = [i, i, i, i]
    lib.vrwkv_qshift_mix_bwd_workspace_bytes.restype = sz
    lib.vrwkv_qshift_mix_bwd.argtypes = [vp, fp, c.POINTER(c.c_void_p), i, vp, fp, i, i, i, i, i, i, i, i, i, vp, sz, vp]
    lib.vrwkv_qshift_mix_bwd.restype = i
    lib.vrwkv_rowfuse.argtypes = [vp, vp, vp, vp, vp, vp, c.c_longlong, i, i, i, c.c_float, i, vp]
    lib.vrwkv_rowfuse.restype = i
    lib.vrwkv_rowfuse_bwd_workspace_bytes.argtypes = [c.c_longlong, i]
    lib.vrwkv_rowfuse_bwd_workspace_bytes.restype = sz
    lib.vrwkv_rowfuse_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, fp, c.c_longlong, i, i, i, c.c_float, i, vp, sz, vp]
    lib.vrwkv_rowfuse_bwd.restype = i
    lib.vrwkv_maa_mix.argtypes = [vp, vp, vp, fp, c.POINTER(c.c_void_p), c.c_longlong, i, i, vp]
    lib.vrwkv_maa_mix.restype = i
    lib.vrwkv_groupnorm_gate.argtypes = [vp, vp, vp, vp, vp, c.c_longlong, i, i, c.c_float, i, i, vp]
    lib.vrwkv_groupnorm_gate.restype = i
    lib.vrwkv_maa_mix_bwd_workspace_bytes.argtypes = [c.c_longlong, i]
    lib.vrwkv_maa_mix_bwd_workspace_bytes.restype = sz
    lib.vrwkv_maa_mix_bwd.argtypes = [vp, vp, vp, fp, c.POINTER(c.c_void_p), vp, vp, vp, fp, c.c_longlong, i, i, vp, sz, vp]
    lib.vrwkv_maa_mix_bwd.restype = i
    lib.vrwkv_groupnorm_gate_bwd_workspace_bytes.argtypes = [c.c_longlong, i]
    lib.vrwkv_groupnorm_gate_bwd_workspace_bytes.restype = sz
    lib.vrwkv_groupnorm_gate_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, fp, c.c_longlong, i, i, c.c_float, i, i, vp, sz, vp]
    lib.vrwkv_groupnorm_gate_bwd.restype = i
    return lib


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
                "or make -C vision-rwkv_amd/csrc); there is no non-HIP fallback")
        _lib = _declare(ctypes.CDLL(LIB_PATH))
    return _lib


def get_option(name):
    """Value of a tuning / testing switch of the library (include/vrwkv_hip.h lists the names)."""
    out = ctypes.c_int(0)
    check(lib().vrwkv_get_option(name.encode(), ctypes.byref(out)))
    return out.value


def set_option(name, value):
    check(lib().vrwkv_set_option(name.encode(), int(value)))


class option:
    """with option("wkv6_fwd_scalar", 1): ...  -- sets a switch for the block and restores it afterwards."""

    def __init__(self, name, value):
        self.name, self.value = name, value

    def __enter__(self):
        self.old = get_option(self.name)
        set_option(self.name, self.value)
        return self

    def __exit__(self, *exc):
        set_option(self.name, self.old)
        return False


def check(status):
    if status != 0:
        raise VrwkvError(status, lib().vrwkv_last_error().decode("utf-8", "replace"))
