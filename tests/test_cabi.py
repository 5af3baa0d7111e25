"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares, and rejects bad arguments with a status and a message before touching the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    import vision_rwkv_amd
    if not os.path.exists(vision_rwkv_amd.LIB_PATH):
        vision_rwkv_amd.build(force=False)
    return vision_rwkv_amd.lib()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "vrwkv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vrwkv_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_symbols()
    assert "vrwkv_biwkv_fwd" in names and "vrwkv_last_error" in names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/vrwkv_hip.h but not exported"


def test_version_and_error_string(lib):
    assert lib.vrwkv_version() >= 100
    assert isinstance(lib.vrwkv_last_error(), bytes)


def test_option_values_are_validated(lib):
    """vrwkv_set_option refuses unknown names and values the plans would silently ignore; accepted values read back."""
    val = ctypes.c_int(-1)
    assert lib.vrwkv_set_option(b"no_such_switch", 1) == 1
    assert lib.vrwkv_get_option(b"no_such_switch", ctypes.byref(val)) == 1
    for name, good, bad in ((b"biwkv_l", (4, 8, 16, 25, 28, 0), (7, 32, -1)), (b"biwkv_s", (2, 8, 0), (1, 9, -3)),
                            (b"biwkv_grid", (64, 0), (-1,)), (b"wkv6_fwd_scalar", (1, 0), (2, -1)),
                            (b"biwkv_bwd_serial", (1, 0), (5,))):
        for v in good:
            assert lib.vrwkv_set_option(name, v) == 0, (name, v)
            assert lib.vrwkv_get_option(name, ctypes.byref(val)) == 0 and val.value == v
        for v in bad:
            assert lib.vrwkv_set_option(name, v) == 1, (name, v)
            assert name in lib.vrwkv_last_error()
            assert lib.vrwkv_get_option(name, ctypes.byref(val)) == 0 and val.value == 0     # unchanged


def test_argument_validation_without_device(lib):
    f = lib.vrwkv_biwkv_fwd
    one = ctypes.c_void_p(16)
    # null pointers
    assert f(None, None, None, None, None, 1, 1, 1, 0, None, 0, None) == 1
    assert b"null" in lib.vrwkv_last_error()
    # non-positive sizes
    assert f(one, one, one, one, one, 0, 4, 4, 0, None, 0, None) == 1
    assert f(one, one, one, one, one, 1, -3, 4, 0, None, 0, None) == 1
    # unknown dtype code
    assert f(one, one, one, one, one, 1, 4, 4, 7, None, 0, None) == 2
    assert b"dtype" in lib.vrwkv_last_error()
    # misaligned tensor pointer
    assert f(one, one, ctypes.c_void_p(18), one, one, 1, 4, 4, 0, None, 0, None) == 1
    # a long sequence needs the workspace the query reports
    need = lib.vrwkv_biwkv_fwd_workspace_bytes(2, 4150, 768, 1)
    assert need > 0
    assert f(one, one, one, one, one, 2, 4150, 768, 1, None, 0, None) == 5
    assert b"workspace" in lib.vrwkv_last_error()
    assert lib.vrwkv_biwkv_fwd_workspace_bytes(64, 196, 768, 0) == 0
    # too large for 32-bit buffer offsets
    assert f(one, one, one, one, one, 1, 1 << 20, 1 << 10, 0, None, 0, None) == 3


def test_elementwise_entry_points_validate_without_device(lib):
    """The fused element-wise entry points reject bad arguments before touching the device."""
    one = ctypes.c_void_p(64)
    rf = lib.vrwkv_rowfuse
    assert rf(None, None, None, None, None, one, 4, 64, 0, 0, 1e-5, 1, None) == 1            # a is null
    assert rf(one, None, None, None, None, one, 4, 64, 0, 1, 1e-5, 1, None) == 1              # gate without `other`
    assert rf(one, None, one, None, None, one, 4, 64, 0, 0, 1e-5, 1, None) == 1               # LayerNorm weight without bias
    assert rf(one, None, None, None, None, one, 4, 60, 0, 0, 1e-5, 1, None) == 3              # N not a multiple of 8 (bf16)
    assert rf(one, None, None, None, None, one, 4, 64, 0, 0, 1e-5, 9, None) == 2              # unknown dtype
    assert rf(one, None, None, None, None, ctypes.c_void_p(72), 4, 64, 0, 0, 1e-5, 1, None) == 1   # misaligned output
    assert rf(one, None, None, None, None, one, 4, 64, 2, 0, 1e-5, 1, None) == 1              # unknown pre
    rb = lib.vrwkv_rowfuse_bwd
    assert lib.vrwkv_rowfuse_bwd_workspace_bytes(100, 768) == 25 * 3 * 768 * 4               # one partial row set per workgroup
    assert lib.vrwkv_rowfuse_bwd_workspace_bytes(1 << 20, 768) == 768 * 3 * 768 * 4         # ... of a grid of at most 768
    assert rb(one, one, None, None, None, one, one, None, None, 4, 64, 0, 1, 1e-5, 1, None, 0, None) == 1     # gate without gother
    assert rb(one, None, one, one, None, one, one, None, None, 4, 64, 0, 0, 1e-5, 1, None, 0, None) == 1      # LayerNorm without gparam
    assert rb(one, None, one, one, None, one, one, None, one, 4, 2048, 0, 0, 1e-5, 1, one, 1 << 20, None) == 3  # channel sums beyond 1024 channels
    assert rb(one, None, one, one, None, one, one, None, one, 4, 64, 0, 0, 1e-5, 1, None, 0, None) == 5       # workspace missing
    mm = lib.vrwkv_maa_mix
    outs = (ctypes.c_void_p * 5)(64, 64, 64, 64, 64)
    assert mm(one, one, one, one, outs, 0, 64, 1, None) == 1                                    # no rows
    assert mm(one, one, one, one, outs, 4, 60, 1, None) == 3                                    # C not a multiple of 8
    outs[3] = None
    assert mm(one, one, one, one, outs, 4, 64, 1, None) == 1                                    # a null output
    qb = lib.vrwkv_qshift_mix_bwd
    gp = (ctypes.c_void_p * 3)(64, 64, 64)
    need = lib.vrwkv_qshift_mix_bwd_workspace_bytes(3, 2, 196, 768)
    assert need == 2 * 7 * 3 * 768 * 4                                                        # one partial row per 32 tokens
    assert qb(one, one, gp, 3, one, one, 2, 196, 768, 14, 14, 1, 192, 0, 1, None, 0, None) == 5     # workspace missing
    assert b"workspace" in lib.vrwkv_last_error()
    assert qb(one, one, gp, 3, one, one, 2, 196, 768, 13, 14, 1, 192, 0, 1, one, need, None) == 3   # grid does not match T
    assert qb(one, one, gp, 4, one, one, 2, 196, 768, 14, 14, 1, 192, 0, 1, one, need, None) == 1   # n_mix out of range
    gp[1] = None
    assert qb(one, one, gp, 3, one, one, 2, 196, 768, 14, 14, 1, 192, 0, 1, one, need, None) == 1   # a null gradient
    gg = lib.vrwkv_groupnorm_gate
    assert gg(one, one, one, one, one, 4, 128, 64, 1e-5, 1, 0, None) == 2                      # fp32 gate beside a bf16 y
    assert gg(one, one, one, one, one, 4, 128, 48, 1e-5, 0, 1, None) == 3                      # C not a multiple of the group
    assert gg(one, one, one, one, one, 4, 96, 24, 1e-5, 0, 1, None) == 3                       # group not 8..128 in powers of two
    assert b"group" in lib.vrwkv_last_error()
    mb = lib.vrwkv_maa_mix_bwd
    gouts = (ctypes.c_void_p * 5)(64, 64, 64, 64, 64)
    assert lib.vrwkv_maa_mix_bwd_workspace_bytes(100, 768) == 4 * 5 * 768 * 4                 # one partial row set per 32 rows
    assert mb(one, one, one, one, gouts, one, one, one, None, 4, 64, 1, None, 0, None) == 1    # gmaa is null
    assert mb(one, one, one, one, gouts, one, one, one, one, 4, 64, 5, None, 0, None) == 2     # unknown dtype
    assert mb(one, one, one, one, gouts, one, one, one, one, 4, 60, 1, None, 0, None) == 3     # C not a multiple of 8
    assert mb(one, one, one, one, gouts, one, one, one, one, 4, 64, 1, None, 0, None) == 5     # workspace missing
    gouts[2] = None
    assert mb(one, one, one, one, gouts, one, one, one, one, 4, 64, 1, one, 1 << 20, None) == 1   # a null gradient
    gb = lib.vrwkv_groupnorm_gate_bwd
    assert lib.vrwkv_groupnorm_gate_bwd_workspace_bytes(100, 768) == 4 * 2 * 768 * 4          # one partial row pair per 32 rows
    assert gb(one, one, one, one, one, one, one, None, 4, 128, 64, 1e-5, 0, 1, None, 0, None) == 1    # gparam is null
    assert gb(one, one, one, one, one, one, one, one, 4, 128, 64, 1e-5, 2, 0, None, 0, None) == 2     # fp32 gate beside an fp16 y
    assert gb(one, one, one, one, one, one, one, one, 4, 2048, 64, 1e-5, 0, 1, None, 0, None) == 3    # more than 1024 channels
    assert gb(one, one, one, one, one, one, one, one, 4, 128, 64, 1e-5, 0, 1, None, 0, None) == 5     # workspace missing


def test_python_boundary_errors_without_device():
    import torch
    import vision_rwkv_amd as ops
    k = torch.randn(2, 8, 64)
    w = torch.zeros(64)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ops.bi_wkv_forward(w, w, k, k)
    with pytest.raises(TypeError):
        ops.RUN_CUDA(w, w, k)


def test_bench_refuses_more_than_one_gpu_and_has_no_cpu_path():
    """bench.py runs on one GPU: --gpus 2 exits with a message instead of a number, and without a GPU the timed path
    refuses to run (nothing falls back to the CPU oracle)."""
    import subprocess
    import sys
    import torch
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr + r.stdout and "{" not in r.stdout
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "1", "--warmup", "1"],
                           capture_output=True, text=True, timeout=300)
        assert r.returncode != 0 and "needs a GPU" in r.stderr and "{" not in r.stdout


def test_extension_module_stand_ins_and_torch_ops_namespaces():
    """The reference's three extension modules (bi_wkv.cpp:49-57, wkv_op.cpp:13-21, wkv6_op.cpp:13-21) have stand-ins
    with the same function names, also reachable through torch.ops."""
    import torch
    import vision_rwkv_amd as ops
    assert set(ops.ext.REGISTERED) == {"bi_wkv", "wkv", "wkv6"}
    for mod, names in ((ops.ext.bi_wkv, ("bi_wkv_forward", "bi_wkv_backward")), (ops.ext.wkv, ("forward", "backward")),
                       (ops.ext.wkv6, ("forward", "backward"))):
        for n in names:
            assert callable(getattr(mod, n))
    assert torch.ops.bi_wkv.bi_wkv_forward is not None and torch.ops.wkv.forward is not None
    assert torch.ops.wkv6.backward is not None
    k = torch.randn(2, 8, 64)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ops.ext.wkv.forward(2, 8, 64, torch.zeros(64), torch.zeros(64), k, k, torch.empty_like(k))
