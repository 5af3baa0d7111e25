"""Benchmark of the WKV hot path on one MI355X.

A step = the Bi-WKV forward of one VRWKV-B backbone pass: 12 back-to-back calls (one per
layer) at B=64, T=196, C=768, each on its own pre-generated seeded k, v (12 distinct buffer
sets, 1.4 GB in fp32, so nothing stays cache-resident from call to call).  Inputs are resident
in HBM before the timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--io fp32|bf16] [--no-cpu-baseline] [--no-sweep] ...
"""
import argparse
import math
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
# HBM bytes per launch of the kernel at this shape: rocprofv3 FETCH_SIZE + WRITE_SIZE of this
# command with --calibrate-copy, each scaled by what it reads for that plain copy of known size
# (profiles/biwkv_fwd_vrwkvB_hbm_traffic.md holds the two counter runs and the arithmetic).
MEASURED_TRAFFIC_FP32 = 115_947_000
MEASURED_TRAFFIC_BF16 = 58_172_000
TRAFFIC_SOURCE = "profiles/biwkv_fwd_vrwkvB_hbm_traffic.md"
REPEATS = 5                    # timed loops per figure; the median is reported
LAYERS = 12
B, T, C = 64, 196, 768


def baseline_wu(torch):
    import math
    c = torch.arange(C, dtype=torch.float64)
    w = (-5.0 + 8.0 * (c / (C - 1))) / T
    u = (math.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / T
    return w.float(), u.float()


def median_us(torch, fn, steps, warmup, calls_per_step=1, stream=None):
    """Median over REPEATS timed loops of `steps` steps (HIP events on the stream the kernels run on), in
    microseconds per call; also returns the per-loop values."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    reps = []
    for _ in range(REPEATS):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        reps.append(e0.elapsed_time(e1) * 1e3 / (steps * calls_per_step))
    return sorted(reps)[len(reps) // 2], reps


CACHE_BYTES = 256 << 20       # last-level cache: buffer sets rotated in a timed loop add up to more than this


def rotating(make_set, set_bytes, call, min_sets=6, max_sets=48):
    """fn() that runs `call(*sets[i])` on the next of n pre-generated input sets each time it is invoked, with n chosen
    so that the sets together exceed the last-level cache (no call finds its inputs cache-resident)."""
    n = max(min_sets, min(max_sets, -(-int(1.25 * CACHE_BYTES) // max(1, set_bytes))))
    sets = [make_set(i) for i in range(n)]
    state = {"i": 0}

    def fn():
        a = sets[state["i"]]
        state["i"] = (state["i"] + 1) % n
        return call(*a)
    return fn, sets


def error_report(y, ref):
    """The two error measures of the parity tests, for one output against the float64 oracle."""
    import numpy as np
    y = np.asarray(y, np.float64)
    rms = float(np.sqrt(np.mean(ref * ref)))
    d = np.abs(y - ref)
    return {"metric": "max|y - ref| / max(|ref|, floor)", "max_abs_err": float(d.max()), "rms_ref": round(rms, 5),
            "rel_err_floor_rms": float((d / np.maximum(np.abs(ref), rms)).max()),
            "rel_err_floor_0.01rms": float((d / np.maximum(np.abs(ref), 1e-2 * rms)).max()),
            "reference": "oracle/c (float64 two-pass recurrence) on the same inputs"}


def config2_section(torch, ops, steps, warmup):
    """Dense-prediction shape of the Mask R-CNN backbone: B=2, T=4150 (50 x 83 patches), C=768, bf16 I/O, fp32 state;
    k, v ~ N(0,1) with 1 % of the tokens scaled x8 (all channels of a token).  One call per step."""
    import numpy as np
    from oracle import clib
    Bn, Tn, Cn = 2, 4150, 768
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(2)

    def make(i):
        k = torch.randn(Bn, Tn, Cn, generator=g)
        v = torch.randn(Bn, Tn, Cn, generator=g)
        big = (torch.rand(Bn, Tn, 1, generator=g) < 0.01).float() * 7.0 + 1.0
        return (k * big).to(dev).bfloat16(), (v * big).to(dev).bfloat16()
    c = torch.arange(Cn, dtype=torch.float64)
    w = ((-5.0 + 8.0 * (c / (Cn - 1))) / Tn).float().to(dev)
    u = ((math.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / Tn).float().to(dev)
    fn, sets = rotating(make, 2 * Bn * Tn * Cn * 2, lambda k, v: ops.bi_wkv_forward(w, u, k, v))
    us, reps = median_us(torch, fn, steps, warmup)
    k, v = sets[0]
    y = ops.bi_wkv_forward(w, u, k, v)
    ref = clib.biwkv_fwd(w.cpu().numpy(), u.cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy())
    byt = 3 * Bn * Tn * Cn * 2 + 2 * Cn * 4
    return {"workload": f"Bi-WKV forward B={Bn} T={Tn} C={Cn}, bf16 I/O, fp32 state, 1% of tokens x8, one call per step, "
                        f"{len(sets)} input sets in rotation",
            "us_per_call": round(us, 2), "repeats_us": [round(x, 2) for x in reps],
            "roofline": {"bound": "hbm", "achieved": round(byt / us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(byt / us / 1e3 / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_launch": byt,
                         "traffic": None},
            "error": error_report(y.float().cpu().numpy(), ref)}


def cpu_baseline(torch, n_calls):
    """The reference recurrence as PyTorch CPU-eager fp32 loops (oracle/torch_eager.py), timed on
    a bounded sample of the same workload: n_calls full-shape calls."""
    from oracle import torch_eager
    w, u = baseline_wu(torch)
    g = torch.Generator().manual_seed(1234)
    k = torch.randn(B, T, C, generator=g)
    v = torch.randn(B, T, C, generator=g)
    torch_eager.biwkv_eager(w, u, k[:4], v[:4])          # warm-up
    t0 = time.perf_counter()
    for _ in range(n_calls):
        y = torch_eager.biwkv_eager(w, u, k, v)
    dt = time.perf_counter() - t0
    bytes_alg = 3 * B * T * C * 4 + 2 * C * 4
    return {
        "value": round(n_calls * bytes_alg / dt / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{n_calls} calls at the full shape B={B} T={T} C={C} fp32 "
                  f"(PyTorch CPU eager two-pass recurrence, {dt:.1f} s)",
    }, y


def wkv6_section(torch, ops, steps, warmup, with_cpu):
    """Secondary line of the metric: wkv6 forward at the VRWKV6-B shape (B=64, T=196, C=768, H=12,
    bf16 r,k,v, fp32 w and y).  tokens/s = B*T per call; MFMA figures use the flops the chunked
    kernel issues to the matrix cores (all split-bf16 products counted), end to end."""
    Bw, Tw, Hw = 64, 196, 12
    Cw = Hw * 64
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(4321)
    u = (torch.randn(Hw, 64, generator=g) * 0.1).to(dev)

    def make(i):
        r, k, v = (torch.randn(Bw, Tw, Cw, generator=g).to(dev).bfloat16() for _ in range(3))
        return r, k, v, (torch.randn(Bw, Tw, Cw, generator=g) * 0.5 - 0.5).to(dev)
    fn, sets = rotating(make, Bw * Tw * Cw * (3 * 2 + 4), lambda r, k, v, w: ops.wkv6_forward(Bw, Tw, Cw, Hw, r, k, v, w, u))
    us, reps = median_us(torch, fn, steps, warmup)
    r, k, v, w = sets[0]
    nchunk = (Tw + 31) // 32
    # per chunk step a workgroup of eight waves issues 42 MFMA 16x16x32 per wave, 16384 flop each
    waves, mfma_per_wave_step, mfma_flop, mfma_cycles = 8, 42, 2 * 16 * 16 * 32, 16
    mfma_flops = Bw * Hw * nchunk * waves * mfma_per_wave_step * mfma_flop
    out = {
        "workload": f"wkv6 forward B={Bw} T={Tw} C={Cw} H={Hw}, bf16 r,k,v, fp32 w,y, {len(sets)} input sets in rotation",
        "us_per_call": round(us, 2),
        "repeats_us": [round(x, 2) for x in reps],
        "tokens_per_s": round(Bw * Tw / (us * 1e-6), 1),
        "recurrence_tflops": round(Bw * Tw * Hw * (10 * 64 * 64 + 3 * 64) / (us * 1e-6) / 1e12, 2),
        "mfma_issued_tflops": round(mfma_flops / (us * 1e-6) / 1e12, 2),
        "pct_bf16_mfma_peak_end_to_end": round(100.0 * mfma_flops / (us * 1e-6) / 2.5e15, 3),
    }
    # Matrix-pipe share inside the contraction stage: the library's profiling entry runs the same kernel with the shader
    # clock stamped by every wave on entering and leaving the matrix stage of every chunk step; a wave's 42 MFMAs occupy
    # the pipe for 16 cycles each (measured: a chain of dependent v_mfma_f32_16x16x32_bf16 issues one per 16 cycles).
    try:
        import ctypes
        import numpy as np
        from vision_rwkv_amd import _lib
        L = _lib.lib()
        nb = L.vrwkv_wkv6_fwd_phases_bytes(Bw, Tw, Hw)
        st = torch.zeros(nb // 8, dtype=torch.int64, device=dev)
        y = torch.empty(Bw, Tw, Cw, device=dev)
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        for _ in range(3):
            rc = L.vrwkv_wkv6_fwd_phases(P(r), P(k), P(v), P(w), P(u), P(y), Bw, Tw, Cw, Hw, P(st), nb,
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
            if rc:
                raise RuntimeError(f"vrwkv_wkv6_fwd_phases returned status {rc}")
        torch.cuda.synchronize()
        t = st.cpu().numpy().reshape(Bw * Hw, waves, nchunk, 8).astype(np.float64)
        m_stage, e_stage = t[..., 5] - t[..., 4], t[..., 1] - t[..., 0]
        step = t[:, :, 1:, 0] - t[:, :, :-1, 0]
        busy = mfma_per_wave_step * mfma_cycles
        out["phases"] = {
            "unit": "shader-clock cycles per wave and chunk step (mean over all waves and steps)",
            "matrix_stage": round(float(m_stage.mean()), 1), "elementwise_stage": round(float(e_stage.mean()), 1),
            "whole_step": round(float(step.mean()), 1),
            "mfma_pipe_cycles_per_wave_step": busy,
            "mfma_busy_in_contractions": round(busy / float(m_stage.mean()), 4),
            "mfma_busy_in_contractions_simd": round(min(1.0, 4 * busy / float(step.mean())), 4),
            "note": "mfma_busy_in_contractions = one wave's MFMA pipe cycles / the time it spends in its matrix stage; "
                    "..._simd = the four waves sharing a SIMD (two workgroups per CU) x their MFMA cycles / one step: "
                    "the pipe's busy share while the kernel runs at full occupancy",
        }
    except Exception as e:                                  # the profiling entry is optional; the timing above stands
        out["phases"] = {"error": repr(e)}
    # end to end the operator's arithmetic intensity (issued MFMA flop per mandatory byte) is below the machine
    # balance, so min(MFMA peak, AI x HBM peak) is the HBM leg: report the fraction of it as well
    io_bytes = Bw * Tw * Cw * (3 * r.element_size() + w.element_size() + 4) + u.numel() * 4
    out["roofline"] = {"bound": "hbm", "achieved": round(io_bytes / (us * 1e-6) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                       "frac": round(io_bytes / (us * 1e-6) / 8e12, 4), "algorithmic_bytes_per_launch": io_bytes,
                       "flop_per_byte_issued": round(mfma_flops / io_bytes, 1)}
    if with_cpu:
        from oracle import torch_eager
        bs = 4
        rc, kc, vc, wc = (t[:bs].float().cpu() for t in (r, k, v, w))
        uc = u.cpu()
        torch_eager.wkv6_eager(rc, kc, vc, wc, uc, Hw)              # untimed first call
        reps, dt = 0, 0.0
        t0 = time.perf_counter()
        while dt < 10.0 and reps < 2000:                           # about 10 s of CPU work
            torch_eager.wkv6_eager(rc, kc, vc, wc, uc, Hw)
            reps += 1
            dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(reps * bs * Tw / dt, 1), "unit": "tokens/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{reps} passes over {bs} of the {Bw} batch elements, PyTorch CPU eager "
                                         f"two-pass recurrence, {dt:.1f} s"}
    return out


def backward_section(torch, ops, steps, warmup):
    """Backward of both operators at the same VRWKV-B shapes (Bi-WKV fp32 I/O; wkv6 bf16 r,k,v, fp32 w, gy)."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(99)
    w, u = (t.to(dev) for t in baseline_wu(torch))
    Hw = C // 64
    u6 = (torch.randn(Hw, 64, generator=g) * 0.1).to(dev)

    def timed(fn):
        return median_us(torch, fn, steps, warmup)[0]

    # every figure on input sets in rotation (more than the last-level cache holds between two uses of a set)
    def make_b(i):
        return tuple(torch.randn(B, T, C, generator=g).to(dev) for _ in range(3))
    fn, sets = rotating(make_b, 3 * B * T * C * 4, lambda k, v, gy: ops.bi_wkv_backward(w, u, k, v, gy))
    us_b = timed(fn)
    sets_h = [tuple(t.bfloat16() for t in s_) for s_ in sets]
    del sets, fn
    state = {"i": 0}

    def fn_h():
        k, v, gy = sets_h[state["i"]]
        state["i"] = (state["i"] + 1) % len(sets_h)
        return ops.bi_wkv_backward(w, u, k, v, gy)
    us_bh = timed(fn_h)
    del sets_h

    def make_6(i):
        r6, k6, v6 = (torch.randn(B, T, C, generator=g).to(dev).bfloat16() for _ in range(3))
        return r6, k6, v6, (torch.randn(B, T, C, generator=g) * 0.5 - 0.5).to(dev), torch.randn(B, T, C, generator=g).to(dev)
    fn6, sets6 = rotating(make_6, B * T * C * (3 * 2 + 4 + 4),
                          lambda r6, k6, v6, w6, gy: ops.wkv6_backward(B, T, C, Hw, r6, k6, v6, w6, u6, gy))
    us_6 = timed(fn6)
    del sets6, fn6
    bytes_b = 5 * B * T * C * 4                                  # k, v, gy read; gk, gv written
    return {"biwkv_bwd_us_per_call": round(us_b, 2), "biwkv_bwd_GBps": round(bytes_b / (us_b * 1e-6) / 1e9, 1),
            "biwkv_bwd_pct_hbm_peak": round(100 * bytes_b / (us_b * 1e-6) / 1e9 / HBM_PEAK_GBS, 2),
            "biwkv_bwd_bf16_us_per_call": round(us_bh, 2),
            "biwkv_bwd_bf16_pct_hbm_peak": round(100 * bytes_b / 2 / (us_bh * 1e-6) / 1e9 / HBM_PEAK_GBS, 2),
            "wkv6_bwd_us_per_call": round(us_6, 1), "wkv6_bwd_tokens_per_s": round(B * T / (us_6 * 1e-6), 1)}


def sweep_section(torch, ops, steps, warmup):
    """Dense-prediction caller shapes (adapter backbones run groups of blocks at T = H/16 * W/16 with batch 2):
    Bi-WKV forward and backward, fp32 I/O (forward also bf16), per (T, C); plus the VRWKV-L classification shape
    (batch 32, 384x384 -> T=576, C=1024)."""
    dev = torch.device("cuda:0")
    rows = []
    shapes = [(2, Tn, Cn) for Tn in (1024, 4150, 4200) for Cn in (192, 384, 768, 1024)] + [(32, 576, 1024)]
    for Bn, Tn, Cn in shapes:
        if True:
            g = torch.Generator(device="cpu").manual_seed(Tn + Cn)
            c = torch.arange(Cn, dtype=torch.float32)
            w = ((-5 + 8 * c / (Cn - 1)) / Tn).to(dev)
            u = ((math.log(0.3) + 0.5 * (((c + 1) % 3) - 1)) / Tn).to(dev)

            def timed(fn):
                return median_us(torch, fn, steps, warmup)[0]

            # input sets in rotation, more than the last-level cache holds (the small shapes need many)
            fn, sets = rotating(lambda i: tuple(torch.randn(Bn, Tn, Cn, generator=g).to(dev) for _ in range(3)),
                                3 * Bn * Tn * Cn * 4, lambda k, v, gy: ops.bi_wkv_forward(w, u, k, v))
            us_f = timed(fn)
            state = {"i": 0}

            def fn_b():
                k, v, gy = sets[state["i"]]
                state["i"] = (state["i"] + 1) % len(sets)
                return ops.bi_wkv_backward(w, u, k, v, gy)
            us_b = timed(fn_b)
            sets_h = [(k.bfloat16(), v.bfloat16()) for k, v, _ in sets]
            n_sets = len(sets)
            del sets, fn

            def fn_h():
                kh, vh = sets_h[state["i"] % len(sets_h)]
                state["i"] = (state["i"] + 1) % len(sets_h)
                return ops.bi_wkv_forward(w, u, kh, vh)
            us_h = timed(fn_h)
            del sets_h
            el = Bn * Tn * Cn * 4
            rows.append({"B": Bn, "T": Tn, "C": Cn, "input_sets": n_sets, "fwd_us": round(us_f, 1), "fwd_GBps": round(3 * el / us_f / 1e3, 1),
                         "fwd_bf16_us": round(us_h, 1), "fwd_bf16_GBps": round(3 * el / 2 / us_h / 1e3, 1),
                         "bwd_us": round(us_b, 1), "bwd_GBps": round(5 * el / us_b / 1e3, 1)})
    return rows


def elementwise_section(torch, ops, which="b,l"):
    """The element-wise kernels of a block (q_shift + mixes, the row-wise epilogues, the VRWKV6 mix steps) at the
    VRWKV-B layer shape (64, 196, 768) and the VRWKV-L one (32, 576, 1024), bf16: each timed as calls on rotating
    buffer sets back to back (six sets, more than the last-level cache holds), in us and GB/s of the algorithmic
    bytes against the 8 TB/s HBM figure.  Everything is called through the C ABI (at 15-30 us per kernel the host work
    of the Python wrappers would dominate a per-call figure)."""
    import ctypes
    from vision_rwkv_amd import _lib
    from vision_rwkv_amd import ops as O
    dev = torch.device("cuda:0")
    L = _lib.lib()
    NB = 6
    dt = torch.bfloat16
    es = 2

    def timed(fns, reps=4):
        for f in fns:
            f()
        torch.cuda.synchronize()
        r = []
        for _ in range(REPEATS):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                for f in fns:
                    f()
            e1.record()
            torch.cuda.synchronize()
            r.append(e0.elapsed_time(e1) / (reps * len(fns)) * 1e3)
        return sorted(r)[len(r) // 2]

    out = []
    shapes = {"b": (64, 14, 14, 768), "l": (32, 24, 24, 1024)}
    for (Bn, Hp, Wp, Cn) in [shapes[k] for k in which.split(",") if k in shapes]:
        Tn = Hp * Wp
        n = Bn * Tn * Cn
        g = torch.Generator(device="cpu").manual_seed(Cn)
        xs = [torch.randn(Bn, Tn, Cn, generator=g).to(dev).to(dt) for _ in range(NB)]
        os_ = [torch.randn(Bn, Tn, Cn, generator=g).to(dev).to(dt) for _ in range(NB)]
        gs = [torch.randn(Bn, Tn, Cn, generator=g).to(dev).to(dt) for _ in range(3)]
        mixes = [torch.rand(Cn, generator=g).to(dev) for _ in range(3)]
        tab3 = O.stack_mixes(mixes, dev)
        tab2 = tab3[:2].contiguous()
        lw, lb, gm = (torch.randn(Cn, generator=g).to(dev).to(dt) for _ in range(3))
        rows = []

        def add(name, us, nbytes):
            rows.append({"kernel": name, "us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1),
                         "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 3)})

        def each(f):
            return [(lambda i=i: f(i)) for i in range(NB)]

        st = torch.cuda.current_stream().cuda_stream
        rws = Bn * Tn
        fptr = lambda t: ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_float))
        outs3 = [torch.empty_like(xs[0]) for _ in range(5)]
        optr = {k: (ctypes.c_void_p * k)(*[t.data_ptr() for t in outs3[:k]]) for k in (2, 3, 5)}

        def qs_fwd(i, tab, k):
            _lib.check(L.vrwkv_qshift_mix(xs[i].data_ptr(), fptr(tab), optr[k], k, Bn, Tn, Cn, Hp, Wp, 1, Cn // 4, 0,
                                          _lib.VRWKV_BF16, st))

        def row_fwd(a, o, w_, b_, g_, N, pre, post, out):
            p = lambda t: t.data_ptr() if t is not None else None
            _lib.check(L.vrwkv_rowfuse(a.data_ptr(), p(o), p(w_), p(b_), p(g_), out.data_ptr(), a.numel() // N, N, pre, post,
                                       1e-5, _lib.VRWKV_BF16, st))

        add("q_shift + 3 mixes (1 read, 3 writes)", timed(each(lambda i: qs_fwd(i, tab3, 3))), 4 * n * es)
        add("q_shift + 2 mixes (1 read, 2 writes)", timed(each(lambda i: qs_fwd(i, tab2, 2))), 3 * n * es)
        o1 = outs3[0]
        add("LayerNorm + sigmoid gate (2 reads, 1 write)",
            timed(each(lambda i: row_fwd(xs[i], os_[i], lw, lb, None, Cn, O.PRE_NONE, O.POST_SIGMOID_GATE, o1))), 3 * n * es)
        add("sigmoid gate (2 reads, 1 write)",
            timed(each(lambda i: row_fwd(xs[i], os_[i], None, None, None, Cn, O.PRE_NONE, O.POST_SIGMOID_GATE, o1))), 3 * n * es)
        add("LayerNorm + layer-scaled residual (2 reads, 1 write)",
            timed(each(lambda i: row_fwd(xs[i], os_[i], lw, lb, gm, Cn, O.PRE_NONE, O.POST_RESIDUAL, o1))), 3 * n * es)
        x4 = [torch.randn(Bn, Tn, 4 * Cn, generator=g).to(dev).to(dt) for _ in range(3)]
        o4 = torch.empty_like(x4[0])
        lw4, lb4 = (torch.randn(4 * Cn, generator=g).to(dev).to(dt) for _ in range(2))
        add("relu^2 + LayerNorm on 4C channels (1 read, 1 write)",
            timed([(lambda i=i: row_fwd(x4[i], None, lw4, lb4, None, 4 * Cn, O.PRE_RELU_SQ, O.POST_NONE, o4)) for i in range(3)]),
            2 * 4 * n * es)
        del x4, o4
        m5 = [torch.randn(5, Bn, Tn, Cn, generator=g).to(dev).to(dt) for _ in range(3)]
        mt = O.stack_mixes([torch.rand(Cn, generator=g).to(dev) for _ in range(5)], dev)
        add("VRWKV6 five token mixes (7 reads, 5 writes)",
            timed([(lambda i=i: _lib.check(L.vrwkv_maa_mix(xs[i].data_ptr(), os_[i].data_ptr(), m5[i].data_ptr(), fptr(mt),
                                                           optr[5], rws, Cn, _lib.VRWKV_BF16, st))) for i in range(3)]),
            12 * n * es)
        del m5
        y32 = [torch.randn(Bn, Tn, Cn, generator=g).to(dev) for _ in range(NB)]
        add("VRWKV6 GroupNorm x SiLU gate (fp32 y and gate read, 1 write)",
            timed(each(lambda i: _lib.check(L.vrwkv_groupnorm_gate(y32[i].data_ptr(), os_[i].data_ptr(), lw.data_ptr(),
                                                                   lb.data_ptr(), o1.data_ptr(), rws, Cn, 64, 1e-5,
                                                                   _lib.VRWKV_F32, _lib.VRWKV_BF16, st)))), n * (4 + 2 * es))
        del y32
        ga = torch.empty_like(xs[0])
        go = torch.empty_like(xs[0])
        gparam = torch.empty(3, Cn, dtype=torch.float32, device=dev)
        wsb = L.vrwkv_rowfuse_bwd_workspace_bytes(rws, Cn)
        ws = torch.empty(max(wsb, 1), dtype=torch.uint8, device=dev)

        def row_bwd(i, post, with_ln):
            _lib.check(L.vrwkv_rowfuse_bwd(xs[i].data_ptr(), os_[i].data_ptr(), lw.data_ptr() if with_ln else None,
                                           lb.data_ptr() if with_ln else None,
                                           gm.data_ptr() if post == O.POST_RESIDUAL else None, gs[i % 3].data_ptr(),
                                           ga.data_ptr(), go.data_ptr() if post == O.POST_SIGMOID_GATE else None,
                                           ctypes.cast(gparam.data_ptr(), ctypes.POINTER(ctypes.c_float)), rws, Cn,
                                           O.PRE_NONE, post, 1e-5, _lib.VRWKV_BF16, ws.data_ptr(), wsb, st))

        add("backward of LayerNorm + layer-scaled residual (2 reads, 1 write; + reduction launch)",
            timed(each(lambda i: row_bwd(i, O.POST_RESIDUAL, True))), 3 * n * es)
        add("backward of sigmoid gate (3 reads, 2 writes)",
            timed(each(lambda i: row_bwd(i, O.POST_SIGMOID_GATE, False))), 5 * n * es)
        gx = torch.empty_like(xs[0])
        gmix = torch.empty(3, Cn, dtype=torch.float32, device=dev)
        qwb = L.vrwkv_qshift_mix_bwd_workspace_bytes(3, Bn, Tn, Cn)
        qws = torch.empty(qwb, dtype=torch.uint8, device=dev)
        gptr = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in gs])

        def qs_bwd(i):
            _lib.check(L.vrwkv_qshift_mix_bwd(xs[i].data_ptr(), ctypes.cast(tab3.data_ptr(), ctypes.POINTER(ctypes.c_float)),
                                              gptr, 3, gx.data_ptr(), ctypes.cast(gmix.data_ptr(), ctypes.POINTER(ctypes.c_float)),
                                              Bn, Tn, Cn, Hp, Wp, 1, Cn // 4, 0, _lib.VRWKV_BF16, qws.data_ptr(), qwb, st))

        add("backward of q_shift + 3 mixes (4 reads, 1 write; + reduction launch)", timed(each(qs_bwd)), 5 * n * es)
        out.append({"shape": [Bn, Tn, Cn], "dtype": "bf16", "kernels": rows})
        del xs, os_, gs
    return out


def backbone_section(torch, ops, steps, warmup):
    """VRWKV-L forward (24 blocks, C=1024, 384x384 input -> T=576) at batch 32 in bf16, random weights:
    ms per forward, and the share of it spent in the 24 Bi-WKV calls (timed alone at the same shape)."""
    dev = torch.device("cuda:0")
    Bn, S = 32, 384
    torch.manual_seed(0)
    net = ops.vrwkv_l().to(dev).eval().bfloat16()
    img = torch.randn(Bn, 3, S, S, device=dev, dtype=torch.bfloat16)

    def timed(fn, n, wu):
        for _ in range(wu):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    with torch.no_grad():
        ms_fwd = timed(lambda: net(img), steps, warmup)
        for m in net.modules():
            if hasattr(m, "fused_shift"):
                m.fused_shift = False
        ms_fwd_eager_shift = timed(lambda: net(img), steps, warmup)
        ops.ops.ROW_FUSE_ENABLED = False
        ms_fwd_unfused = timed(lambda: net(img), steps, warmup)
        ops.ops.ROW_FUSE_ENABLED = True
        Tn, Cn = (S // 16) ** 2, 1024
        att = net.layers[0].att
        k = torch.randn(Bn, Tn, Cn, device=dev, dtype=torch.bfloat16)
        v = torch.randn(Bn, Tn, Cn, device=dev, dtype=torch.bfloat16)
        w, u = (att.spatial_decay / Tn).float(), (att.spatial_first / Tn).float()
        ms_wkv = timed(lambda: ops.bi_wkv_forward(w, u, k, v), 24 * steps, 24 * warmup) * 24
        # VRWKV6-B at its training shape (batch 64, 224x224 -> T=196, C=768, 12 heads, 12 blocks)
        B6, H6 = 64, 12
        net6 = ops.vrwkv6_b().to(dev).eval().bfloat16()
        img6 = torch.randn(B6, 3, 224, 224, device=dev, dtype=torch.bfloat16)
        ms6 = timed(lambda: net6(img6), steps, warmup)
        r6, k6, v6 = (torch.randn(B6, 196, 768, device=dev, dtype=torch.bfloat16) for _ in range(3))
        w6 = torch.randn(B6, 196, 768, device=dev) * 0.5 - 0.5
        u6 = torch.randn(H6, 64, device=dev) * 0.1
        ms_wkv6 = timed(lambda: ops.wkv6_forward(B6, 196, 768, H6, r6, k6, v6, w6, u6), 12 * steps, 12 * warmup) * 12
    # VRWKV-B (classification/configs/vrwkv/vrwkv_base_16xb64_in1k.py: 224x224, C=768, 12 blocks, post-norm, layer
    # scale): the inference forward with the receptance gate inside the Bi-WKV kernel and as a pass of its own, then
    # one training forward + backward at the per-GPU batch of 64 through the HIP operators and autograd
    netb = ops.VRWKV(img_size=224, patch_size=16, embed_dims=768, depth=12, post_norm=True, init_values=1e-5).to(dev).bfloat16()
    imgb = torch.randn(64, 3, 224, 224, device=dev, dtype=torch.bfloat16)
    netb.eval()
    with torch.no_grad():
        ms_b_fwd = timed(lambda: netb(imgb), steps, warmup)
        for m in netb.modules():
            if hasattr(m, "fused_gate"):
                m.fused_gate = False
        ms_b_fwd_gate_pass = timed(lambda: netb(imgb), steps, warmup)
        for m in netb.modules():
            if hasattr(m, "fused_gate"):
                m.fused_gate = True
    netb.train()

    def train_step():
        netb.zero_grad(set_to_none=True)
        netb(imgb).float().square().mean().backward()

    ms_train = timed(train_step, max(steps // 2, 3), max(warmup // 4, 3))
    # the same step recorded once as a HIP graph and replayed (every kernel of the build launches on the stream it is
    # given and allocates nothing, so the whole forward + backward can be captured); the gradients of a replay are
    # compared with the eager step's on the same images
    graph_step = {"ms_per_step": None}
    try:
        params = [p for p in netb.parameters() if p.requires_grad]
        train_step()
        torch.cuda.synchronize()
        eager_grads = [p.grad.clone() for p in params]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                train_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        netb.zero_grad(set_to_none=True)
        with torch.cuda.graph(graph):
            netb(imgb).float().square().mean().backward()
        ms_graph = timed(graph.replay, max(steps // 2, 3), 3)
        same = all(torch.equal(p.grad, g) for p, g in zip(params, eager_grads))
        graph_step = {"ms_per_step": round(ms_graph, 3), "images_per_s": round(64 / ms_graph * 1e3, 1),
                      "gradients_equal_the_eager_step": bool(same)}
        del graph
    except Exception as exc:                                   # reported, never fatal for the headline
        graph_step["error"] = f"{type(exc).__name__}: {exc}"[:200]
    del netb
    net6t = ops.vrwkv6_b().to(dev).bfloat16()
    net6t.train()

    def train_step6():
        net6t.zero_grad(set_to_none=True)
        net6t(imgb).float().square().mean().backward()

    ms_train6 = timed(train_step6, max(steps // 2, 3), max(warmup // 4, 3))
    del net6t
    return {"workload": f"VRWKV-L forward, batch {Bn}, {S}x{S}, T={Tn}, C={Cn}, 24 blocks, bf16, random weights",
            "ms_per_forward": round(ms_fwd, 3), "images_per_s": round(Bn / ms_fwd * 1e3, 1),
            "ms_per_forward_unfused_shift": round(ms_fwd_eager_shift, 3),
            "ms_per_forward_all_elementwise_in_pytorch": round(ms_fwd_unfused, 3),
            "biwkv_ms_per_forward": round(ms_wkv, 3), "biwkv_share": round(ms_wkv / ms_fwd, 4),
            "vrwkv_b": {"workload": "VRWKV-B forward, batch 64, 224x224, T=196, C=768, 12 blocks, bf16, random weights, "
                                    "sigmoid(r) gate inside the Bi-WKV kernel (vrwkv_biwkv_fwd_gate)",
                        "ms_per_forward": round(ms_b_fwd, 3), "images_per_s": round(64 / ms_b_fwd * 1e3, 1),
                        "ms_per_forward_gate_as_a_pass_of_its_own": round(ms_b_fwd_gate_pass, 3)},
            "vrwkv_b_train": {"workload": "VRWKV-B forward + backward (no optimizer step), batch 64, 224x224, T=196, C=768, "
                                          "12 blocks, bf16, random weights, Bi-WKV forward and backward on the HIP kernels",
                              "ms_per_step": round(ms_train, 3), "images_per_s": round(64 / ms_train * 1e3, 1),
                              "recorded_as_one_hip_graph_and_replayed": graph_step},
            "vrwkv6_b_train": {"workload": "VRWKV6-B forward + backward (no optimizer step), batch 64, 224x224, T=196, C=768, "
                                           "12 heads, 12 blocks, bf16, random weights, wkv6 forward and backward on the HIP kernels",
                               "ms_per_step": round(ms_train6, 3), "images_per_s": round(64 / ms_train6 * 1e3, 1)},
            "vrwkv6_b": {"workload": "VRWKV6-B forward, batch 64, 224x224, T=196, C=768, 12 heads, 12 blocks, bf16, "
                                     "random weights",
                         "ms_per_forward": round(ms6, 3), "images_per_s": round(B6 / ms6 * 1e3, 1),
                         "wkv6_ms_per_forward": round(ms_wkv6, 3), "wkv6_share": round(ms_wkv6 / ms6, 4)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--io", choices=["fp32", "bf16"], default="fp32")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-wkv6", action="store_true", help="skip the secondary wkv6 measurement")
    ap.add_argument("--no-backbone", action="store_true", help="skip the VRWKV-L whole-forward measurement")
    ap.add_argument("--no-backward", action="store_true", help="skip the backward-kernel measurements")
    ap.add_argument("--no-sweep", action="store_true", help="skip the dense-prediction shape sweep (B=2, long T)")
    ap.add_argument("--no-config2", action="store_true", help="skip the B=2, T=4150, C=768 bf16 measurement")
    ap.add_argument("--no-elementwise", action="store_true", help="skip the element-wise block kernels (q_shift + mix, row epilogues)")
    ap.add_argument("--elementwise-shapes", default="b,l",
                    help="layer shapes of the element-wise section: b = (64, 196, 768), l = (32, 576, 1024)")
    ap.add_argument("--cpu-calls", type=int, default=96)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device copy of a (B,T,C) fp32 tensor (a kernel of known "
                         "traffic, for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every (batch, channel) sequence is "
              "independent, so more GPUs would simply split the batch); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import vision_rwkv_amd as ops
    from vision_rwkv_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    io = torch.float32 if args.io == "fp32" else torch.bfloat16
    esz = 4 if args.io == "fp32" else 2
    w, u = (t.to(dev) for t in baseline_wu(torch))
    g = torch.Generator(device="cpu").manual_seed(1234)
    ks, vs = [], []
    for _ in range(LAYERS):
        ks.append(torch.randn(B, T, C, generator=g).to(dev).to(io))
        vs.append(torch.randn(B, T, C, generator=g).to(dev).to(io))
    ys = [torch.empty_like(k) for k in ks]

    # direct C-ABI calls on torch's current stream (what ops.bi_wkv_forward does, minus the
    # per-call output allocation)
    L = ops.lib()
    dt_code = _lib.VRWKV_F32 if args.io == "fp32" else _lib.VRWKV_BF16
    ws_bytes = L.vrwkv_biwkv_fwd_workspace_bytes(B, T, C, dt_code)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)
    calls = [(w.data_ptr(), u.data_ptr(), ks[i].data_ptr(), vs[i].data_ptr(), ys[i].data_ptr(),
              B, T, C, dt_code, ws.data_ptr() if ws_bytes else None, ws_bytes, stream.cuda_stream)
             for i in range(LAYERS)]
    fwd = L.vrwkv_biwkv_fwd

    def step():
        for a in calls:
            rc = fwd(*a)
            if rc:
                _lib.check(rc)

    if args.calibrate_copy:
        ys[0].float().copy_(ks[0].float()) if args.io != "fp32" else ys[0].copy_(ks[0])
    # W warm-up steps, then REPEATS timed loops of exactly K steps each (HIP events on the stream the kernels run
    # on, device idle on both sides of every loop); the median loop is the reported one
    us_per_launch, reps_us = median_us(torch, step, args.steps, args.warmup, LAYERS, stream)
    ms_per_step = us_per_launch * LAYERS / 1e3
    n_launch = args.steps * LAYERS
    bytes_alg = 3 * B * T * C * esz + 2 * C * 4          # k, v read once, y written once, w and u
    gbs = bytes_alg / (us_per_launch * 1e-6) / 1e9

    out = {
        "metric": "Bi-WKV fwd GB/s (% HBM peak) @VRWKV-B; wkv6 tokens/s (% MFMA peak)",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "io_dtype": args.io,
        "data": "synthetic",
        "config": {"workload": f"Bi-WKV forward, VRWKV-B shape B={B} T={T} C={C}, {args.io} I/O, "
                               f"{LAYERS} back-to-back calls per step on distinct seeded k,v",
                   "io_dtype": args.io, "calls_per_step": LAYERS, "seed": 1234},
        "pct_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "us_per_call": round(us_per_launch, 3),
        "timing": f"median of {REPEATS} loops of {args.steps} steps after {args.warmup} warm-up steps",
        "repeats_us_per_call": [round(x, 3) for x in reps_us],
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_FP32 if args.io == "fp32" else MEASURED_TRAFFIC_BF16 if args.io == "bf16" else None,
            "traffic_source": TRAFFIC_SOURCE if args.io in ("fp32", "bf16") else None,
            "kernel": "biwkv_fwd_kernel (one launch per call)",
            "algorithmic_bytes_per_launch": bytes_alg,
        },
    }
    if args.io == "fp32":
        # the same loop with bf16 tensors (secondary figure; the headline stays the fp32 one)
        kh, vh = [k.bfloat16() for k in ks], [v.bfloat16() for v in vs]
        yh = [torch.empty_like(k) for k in kh]
        calls_h = [(w.data_ptr(), u.data_ptr(), kh[i].data_ptr(), vh[i].data_ptr(), yh[i].data_ptr(),
                    B, T, C, _lib.VRWKV_BF16, None, 0, stream.cuda_stream) for i in range(LAYERS)]

        def step_h():
            for a in calls_h:
                rc = fwd(*a)
                if rc:
                    _lib.check(rc)

        us_h, reps_h = median_us(torch, step_h, args.steps, args.warmup, LAYERS, stream)
        bytes_h = 3 * B * T * C * 2 + 2 * C * 4
        out["bf16_io"] = {"us_per_call": round(us_h, 3), "repeats_us_per_call": [round(x, 3) for x in reps_h],
                          "roofline": {"bound": "hbm", "achieved": round(bytes_h / us_h / 1e3, 1), "peak": HBM_PEAK_GBS,
                                       "unit": "GB/s", "frac": round(bytes_h / us_h / 1e3 / HBM_PEAK_GBS, 4),
                                       "traffic": MEASURED_TRAFFIC_BF16, "traffic_source": TRAFFIC_SOURCE,
                                       "algorithmic_bytes_per_launch": bytes_h}}
        if not args.no_cpu_baseline:
            from oracle import clib
            refh = clib.biwkv_fwd(w.cpu().numpy(), u.cpu().numpy(), kh[0].float().cpu().numpy(), vh[0].float().cpu().numpy())
            out["bf16_io"]["error"] = error_report(yh[0].float().cpu().numpy(), refh)
        del kh, vh, yh
    if not args.no_cpu_baseline:
        # layer 0's output against the float64 C oracle and against the CPU-eager fp32 recurrence the baseline times
        # (both on the same k, v: the first two draws of seed 1234)
        from oracle import clib
        ref = clib.biwkv_fwd(w.cpu().numpy(), u.cpu().numpy(), ks[0].float().cpu().numpy(), vs[0].float().cpu().numpy())
        out["error"] = error_report(ys[0].float().cpu().numpy(), ref)
        out["error"]["tolerance"] = "1e-4 (fp32 I/O), 1e-2 (16-bit I/O) on the floor = rms(ref) measure (tests/conftest.py)"
        cb, y_cpu = cpu_baseline(torch, args.cpu_calls)
        out["cpu_baseline"] = cb
        if args.io == "fp32":
            out["error"]["cpu_eager_fp32_recurrence"] = error_report(y_cpu.numpy(), ref)["rel_err_floor_0.01rms"]
    if not args.no_wkv6:
        out["wkv6"] = wkv6_section(torch, ops, max(args.steps, 10), max(args.warmup // 5, 3), not args.no_cpu_baseline)
    if not args.no_backward:
        out["backward"] = backward_section(torch, ops, 10, 3)
    if not args.no_config2:
        out["config2"] = config2_section(torch, ops, 20, 10)
    if not args.no_sweep:
        out["sweep"] = sweep_section(torch, ops, 10, 3)
    if not args.no_elementwise:
        out["elementwise"] = elementwise_section(torch, ops, args.elementwise_shapes)
    if not args.no_backbone:
        out["backbone"] = backbone_section(torch, ops, 5, 3)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
