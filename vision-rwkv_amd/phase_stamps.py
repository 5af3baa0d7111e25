"""Per-phase cycle stamps of the Bi-WKV forward kernels (where the time of a tile goes).

Needs the instrumented library (make -C vision-rwkv_amd/csrc stamps), which records the shader clock (s_memtime) at
numbered points of every tile, per wave.  Runs the forward at one shape, reads the stamps of the last call and prints,
per round of tiles (a workgroup's first, second, ... tile) the mean time spent between consecutive points, and the
kernel's own timeline.

    python vision-rwkv_amd/phase_stamps.py [B T C dtype]        (default 64 196 768 fp32)
"""
import ctypes
import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
TILES, POINTS, WAVES = 4, 12, 8
NAMES = {0: "tile entered", 1: "other super-chunks folded", 2: "rows copied from LDS to registers",
         3: "next tile's loads issued", 4: "aggregate pass, aggregates written to LDS", 5: "workgroup barrier passed",
         6: "carries from the other waves formed", 7: "ascending sweep", 8: "descending sweep up to the first store",
         9: "wait for the next tile's rows", 10: "descending sweep and stores issued"}


def main():
    B, T, C = (int(a) for a in sys.argv[1:4]) if len(sys.argv) >= 4 else (64, 196, 768)
    dtype = {"fp32": torch.float32, "bf16": torch.bfloat16}[sys.argv[4] if len(sys.argv) >= 5 else "fp32"]
    code = 0 if dtype == torch.float32 else 1
    lib = ctypes.CDLL(os.path.join(HERE, "libvrwkv_hip_stamps.so"))
    lib.vrwkv_biwkv_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.vrwkv_biwkv_fwd_workspace_bytes.argtypes = [ctypes.c_int] * 4
    lib.vrwkv_biwkv_fwd.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    set_buffer = getattr(lib, "vrwkv_debug_set_stamp_buffer_" + ("f32" if dtype == torch.float32 else "bf16"))
    set_buffer.argtypes = [ctypes.c_void_p]
    dev = "cuda:0"
    g = torch.Generator().manual_seed(1234)
    c = torch.arange(C, dtype=torch.float64)
    w = ((-5.0 + 8.0 * (c / (C - 1))) / T).float().to(dev)
    u = ((math.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T).float().to(dev)
    NB = 12
    ks = [torch.randn(B, T, C, generator=g).to(dev).to(dtype) for _ in range(NB)]
    vs = [torch.randn(B, T, C, generator=g).to(dev).to(dtype) for _ in range(NB)]
    ys = [torch.empty_like(k) for k in ks]
    wsb = ws_bytes = lib.vrwkv_biwkv_fwd_workspace_bytes(B, T, C, code)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    n_wg = 1024
    buf = torch.zeros(n_wg * WAVES * TILES * POINTS, dtype=torch.int64, device=dev)

    def call(i):
        rc = lib.vrwkv_biwkv_fwd(w.data_ptr(), u.data_ptr(), ks[i].data_ptr(), vs[i].data_ptr(), ys[i].data_ptr(),
                                 B, T, C, code, ws.data_ptr(), wsb, st)
        assert rc == 0, rc

    for _ in range(5):
        for i in range(NB):
            call(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        for i in range(NB):
            call(i)
    e1.record()
    torch.cuda.synchronize()
    us_call = e0.elapsed_time(e1) * 1e3 / (10 * NB)
    assert set_buffer(buf.data_ptr()) == 0
    call(0)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(10):
        call(0)
    e1.record()
    torch.cuda.synchronize()
    us_stamped = e0.elapsed_time(e1) * 1e3 / 10
    set_buffer(None)
    s = buf.cpu().numpy().reshape(n_wg, WAVES, TILES, POINTS).astype(np.float64)
    s[s == 0] = np.nan
    # every XCD has a counter of its own: times are taken relative to the workgroup's own first stamp
    wg0 = np.nanmin(s.reshape(n_wg, -1), axis=1)
    live = ~np.isnan(wg0)
    rel = s - wg0[:, None, None, None]
    span = np.nanmax(rel.reshape(n_wg, -1)[live], axis=1)
    print(f"Bi-WKV forward B={B} T={T} C={C} {dtype}: {us_call:.2f} us per call with the stamps switched off, "
          f"{us_stamped:.2f} us with the stamps written (HIP events, back-to-back calls)")
    print(f"{int(live.sum())} workgroups; first to last stamp of a workgroup: mean {span.mean():.0f} ticks of s_memtime "
          f"(min {span.min():.0f}, max {span.max():.0f}), i.e. about {span.mean() / us_stamped:.0f} ticks per microsecond")
    for r in range(TILES):
        tile = rel[:, :, r, :]
        if np.all(np.isnan(tile[:, :, 0])):
            continue
        n = int(np.sum(~np.isnan(tile[:, :, 0])))
        which = "" if ws_bytes == 0 else (" (aggregate-only kernel)" if r >= 2 else " (emit kernel)")
        print(f"\nround {r % 2 if ws_bytes else r}{which}: {n} waves; tile entered {np.nanmean(tile[:, :, 0]):.0f} ticks after the workgroup's first stamp "
              f"(min {np.nanmin(tile[:, :, 0]):.0f}, max {np.nanmax(tile[:, :, 0]):.0f})")
        prev = 0
        for p in range(1, POINTS):
            if np.all(np.isnan(tile[:, :, p])):
                continue
            d = tile[:, :, p] - tile[:, :, prev]
            print(f"  {prev:2d} -> {p:2d}  {NAMES.get(p, ''):48s} mean {np.nanmean(d):8.0f}  min {np.nanmin(d):8.0f}  max {np.nanmax(d):8.0f}")
            prev = p
        d = tile[:, :, prev] - tile[:, :, 0]
        print(f"  tile total (0 -> {prev})" + " " * 37 + f"mean {np.nanmean(d):8.0f}  min {np.nanmin(d):8.0f}  max {np.nanmax(d):8.0f}")


if __name__ == "__main__":
    main()
