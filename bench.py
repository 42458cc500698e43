#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c2|c3|c4|c5|dense_mask|bwd|bwd_f32|bwd_c1|logsoftmax|softmax|softmax_dims2|batched_mul[_f32|_c32|_f64]] [--no-cpu]

A "step" is one dot_product_attention call on synthetic inputs that are already resident in HBM.
The default workload is C3 (bf16 causal prefill, head dim 128, L = 4096), the configuration the
prefill target is quoted on; the other four configurations are measured in the same run and reported under
"configs" in the same JSON line (C5, the decode target, also under "decode"), and the workloads beyond them (dense mask,
gradient, softmax family, batched_mul; GPU leg only) under "next_rows".  Timing is by HIP events on the stream the kernels are launched on.
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "nnlib.jl_amd"))

PEAK = {"bf16": 2516.0, "f16": 2516.0, "f32": 157.3, "f64": 78.6}   # dense MFMA TFLOP/s
HBM_PEAK = 8000.0                                       # GB/s
HBM_BOUND = ("c4", "c5")                                # workloads priced against the HBM roofline
# HBM bytes per launch of each workload's dominant kernel are not measured by this script: they come from
# rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of it, summarised in the file below (which also gives the
# commands and the copy-kernel calibration), and are read from there so that the figure and its source travel together.
MIB = 1 << 20
TRAFFIC_FILE = os.path.join("profiles", "hbm_traffic_fetch_write_size.md")
DOMINANT_KERNEL = {"c1": "flash32_resident", "c2": "flash32_kernel", "c3": "flash16_fast_kernel", "c4": "flash16_kernel",
                   "c5": "decode_split_kernel",
                   # a gradient step is three kernels (dq, dk, dv): every row of the workload whose name contains "bwd"
                   "bwd": "bwd", "bwd_f32": "bwd", "bwd_c1": "bwd", "softmax": "softmax", "logsoftmax": "softmax", "softmax_dims2": "softmax",
                   "batched_mul": "gemm", "batched_mul_f32": "gemm",
                   "dense_mask": "flash16_fast_kernel<false, true"}


def measured_traffic(key):
    """(bytes per step, source) of the workload's kernels from the tracked rocprofv3 summary: the rows of its table
    whose first column is the workload and whose kernel name contains DOMINANT_KERNEL[key], read MiB + written MiB,
    summed over those rows (one row for a one-kernel step; the gradient's three).  (None, None) when the file has no
    such row."""
    total = None
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 6 and cells[0] == key and DOMINANT_KERNEL.get(key, "\0") in cells[1]:
                    total = (total or 0.0) + (float(cells[4]) + float(cells[5])) * MIB
    except (OSError, ValueError):
        return None, None
    return (total, TRAFFIC_FILE) if total is not None else (None, None)


def measured_traffic_fields(key):
    traffic, source = measured_traffic(key)
    return dict(traffic=traffic, traffic_source=source)


ROTATE_BYTES = 1 << 30                                  # input sets rotated until they cover 4x the last-level cache

# name -> description of BASELINE.json's configs
WORKLOADS = {
    "c1": dict(name="C1 self-attention f32 (512,128,4) H=8, weights returned", dtype="f32", E=512, Lq=128, Lkv=128,
               B=4, H=8, causal=False, weights=True, scale=1.0, seed=0x5EED0000),
    "c2": dict(name="C2 causal self-attention f32 (1024,1024,8) H=16, weights returned", dtype="f32", E=1024,
               Lq=1024, Lkv=1024, B=8, H=16, causal=True, weights=True, scale=0.125, seed=0x5EED0001),
    "c3": dict(name="C3 causal prefill bf16 (4096,4096,2) H=32 D=128, weights not materialised", dtype="bf16",
               E=4096, Lq=4096, Lkv=4096, B=2, H=32, causal=True, weights=False, scale=1.0, seed=0x5EED0002),
    "c4": dict(name="C4 cross-attention f16 q(1024,256,4) kv(1024,8192,4) H=16 + bias (8192,256,16,4) + mask (8192,256)",
               dtype="f16", E=1024, Lq=256, Lkv=8192, B=4, H=16, causal=False, weights=False, scale=1.0,
               bias=True, mask=True, seed=0x5EED0003),
    "c5": dict(name="C5 decode bf16 q(4096,1,16) kv(4096,32768,16) H=32 D=128", dtype="bf16", E=4096, Lq=1,
               Lkv=32768, B=16, H=32, causal=False, weights=False, scale=1.0, seed=0x5EED0004),
}


def algorithmic_work(w):
    """(FLOPs, compulsory HBM bytes) of one call: 4*Lq*Lkv*D*H*B FLOP (QK^T and PV; causal counts the
    unmasked triangle only), every input read once and every output written once."""
    E, Lq, Lkv, B, H = w["E"], w["Lq"], w["Lkv"], w["B"], w["H"]
    D = E // H
    es = 4 if w["dtype"] == "f32" else 2
    pairs = Lq * (Lq + 1) // 2 if w["causal"] else Lq * Lkv
    flops = 4 * D * H * B * pairs
    nbytes = es * (E * Lq * B + 2 * E * Lkv * B + E * Lq * B)
    if w["weights"]:
        nbytes += es * Lkv * Lq * H * B
    if w.get("bias"):
        nbytes += es * Lkv * Lq * H * B
    if w.get("mask"):
        nbytes += Lkv * Lq
    if w["causal"] and w["weights"]:
        nbytes += Lq * Lkv   # the dense Bool mask the reference would read
    return flops, nbytes


def f32_products(roof, achieved_tflops, executed_per_counted=1.0):
    """Float32 workloads keep `peak` = the published Float32 matrix peak, but by default their products are issued as six
    bf16 matrix instructions on three bf16 planes per operand: the rate the issued instruction allows for Float32 products
    is the bf16 peak / 6.  `executed_per_counted`: products the kernel executes per product the FLOP count holds."""
    exact = os.environ.get("MI355ATTN_F32_MFMA", "")[:1] == "1"
    roof["products"] = ("v_mfma_f32_32x32x2_f32" if exact else
                        "six v_mfma_f32_32x32x16_bf16 on three bf16 planes per operand (Float32 accuracy)")
    pk = PEAK["f32"] if exact else PEAK["bf16"] / 6.0
    roof["products_peak"] = pk
    roof["products_frac"] = achieved_tflops * executed_per_counted / pk
    roof["products_executed_per_counted"] = executed_per_counted


PREHEAT_S = 1.0     # seconds of the same launches before the counted warm-up (0 = none)


def preheat(step, sync):
    """Time-based pre-heat: the same launch back to back for PREHEAT_S seconds, so that the counted warm-up and
    the timed steps run at the clocks of a sustained run rather than on a GPU coming out of idle.  Returns the
    milliseconds spent.  `--steps` and `--warmup` keep their meaning."""
    if PREHEAT_S <= 0:
        return 0.0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < PREHEAT_S:
        for _ in range(10):
            step()
        sync()
    return (time.perf_counter() - t0) * 1e3


class Runner:
    """Owns the device buffers of one workload and launches it through the C ABI."""

    def __init__(self, key, rotate=None):
        import torch
        import nnlib_amd
        from nnlib_amd import _lib
        self.torch, self.nn, self._lib = torch, nnlib_amd, _lib
        self.lib = _lib.load()
        _lib.check(self.lib.mi_init(0))
        w = self.w = WORKLOADS[key]
        # HBM-bound workloads whose inputs could partly survive in the 256 MiB last-level cache from one
        # launch to the next rotate through several independent input sets (same seed, same values).
        _, nbytes = algorithmic_work(w)
        if rotate is None:
            rotate = key in HBM_BOUND
        self.nsets = max(1, min(4, -(-ROTATE_BYTES // nbytes))) if rotate else 1
        self.sets = [self._make_set() for _ in range(self.nsets)]
        self.q, self.k, self.v, self.bias, self.mask, self.out, self.alpha, self.desc = self.sets[0]
        kern, ws = ctypes.c_int32(0), ctypes.c_size_t(0)
        _lib.check(self.lib.mi_attention_plan(ctypes.byref(self.desc), ctypes.byref(kern), ctypes.byref(ws)))
        self.kernel = _lib.KERNEL_NAMES[kern.value]
        self.ws = torch.empty(max(ws.value, 1), dtype=torch.uint8, device="cuda")
        for st in self.sets:
            st[-1].workspace, st[-1].workspace_bytes = self.ws.data_ptr(), ws.value
        self.calls = 0

    def _make_set(self):
        _lib, w = self._lib, self.w
        dt = w["dtype"]
        E, Lq, Lkv, B, H = w["E"], w["Lq"], w["Lkv"], w["B"], w["H"]
        DA = self.nn.DeviceArray
        q, k, v = DA.empty((E, Lq, B), dt), DA.empty((E, Lkv, B), dt), DA.empty((E, Lkv, B), dt)
        for sid, a in enumerate((q, k, v)):
            sc = w["scale"] if sid < 2 else 1.0
            _lib.check(self.lib.mi_randn_fill(a.ptr, a.code, a.length, w["seed"], sid, sc, None))
        bias = mask = None
        if w.get("bias"):
            bias = DA.empty((Lkv, Lq, H, B), dt)
            _lib.check(self.lib.mi_randn_fill(bias.ptr, bias.code, bias.length, w["seed"], 3, 0.5, None))
        if w.get("mask"):
            mask = DA.empty((Lkv, Lq), "bool")
            _lib.check(self.lib.mi_bernoulli_fill(mask.ptr, mask.length, w["seed"], 4, 0.9, None))
        out = DA.empty((E, Lq, B), dt)
        alpha = DA.empty((Lkv, Lq, H, B), dt) if w["weights"] else None
        d = _lib.mi_attn_desc()
        d.struct_size = ctypes.sizeof(_lib.mi_attn_desc)
        d.dtype = q.code
        d.weights_dtype = q.code
        d.causal = int(w["causal"])
        d.E, d.Ev, d.Lq, d.Lkv, d.H, d.B = E, E, Lq, Lkv, H, B
        d.q, d.k, d.v, d.out = q.ptr, k.ptr, v.ptr, out.ptr
        d.weights = alpha.ptr if alpha is not None else None
        if bias is not None:
            d.bias = bias.ptr
            d.bias_strides = (ctypes.c_int64 * 4)(1, Lkv, Lkv * Lq, Lkv * Lq * H)
        if mask is not None:
            d.mask = mask.ptr
            d.mask_strides = (ctypes.c_int64 * 4)(1, Lkv, 0, 0)
        return (q, k, v, bias, mask, out, alpha, d)

    def step(self):
        d = self.sets[self.calls % self.nsets][-1]
        self.calls += 1
        self._lib.check(self.lib.mi_attention_fwd(ctypes.byref(d), None))

    def time(self, steps, warmup):
        """Average ms per call over `steps` back-to-back launches, HIP events on the launch stream."""
        lib, _lib = self.lib, self._lib
        e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
        _lib.check(lib.mi_event_create(ctypes.byref(e0)))
        _lib.check(lib.mi_event_create(ctypes.byref(e1)))
        self.preheat_ms = preheat(self.step, lambda: _lib.check(lib.mi_device_sync()))
        for _ in range(warmup):
            self.step()
        _lib.check(lib.mi_device_sync())
        t0 = time.perf_counter()
        _lib.check(lib.mi_event_record(e0, None))
        for _ in range(steps):
            self.step()
        _lib.check(lib.mi_event_record(e1, None))
        _lib.check(lib.mi_event_sync(e1))
        _lib.check(lib.mi_device_sync())
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        ms = ctypes.c_float(0)
        _lib.check(lib.mi_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        lib.mi_event_destroy(e0)
        lib.mi_event_destroy(e1)
        return ms.value / steps, wall_ms


def cpu_baseline(runner, budget_s=10.0):
    """The CPU oracle (NNlib's op sequence restated in C, Float32, NNlib's thread policy) timed on a bounded sample
    of the same workload: whole (head, batch) slices of the tensors the GPU was timed on (copied to the host and
    widened to Float32, as the reference's CPU path would see them), as many as fit in about `budget_s` seconds
    (sized from a one-slice-per-thread trial run), scaled to the whole job.  The GEMM slices run on the host's BLAS
    sgemm_ when SciPy's can be bound (what the reference calls, src/gemm.jl:141-149), else on the oracle's own kernel;
    `sample` says which."""
    import numpy as np
    from oracle import oracle as O
    w = runner.w
    E, Lq, Lkv, B, H = w["E"], w["Lq"], w["Lkv"], w["B"], w["H"]
    D = E // H
    cores = min(16, len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1))
    O.lib()
    blas = O.use_host_blas()
    mask = None
    if runner.mask is not None:
        mask = np.asfortranarray(runner.mask.storage.view(Lq, Lkv).cpu().numpy().T.astype(bool))
    if w["causal"]:
        mask = O.make_causal_mask(Lq)

    def host(arr, L, nh, nb):      # heads 0..nh-1 of batch elements 0..nb-1 of an (E, L, B) device array
        t = arr.storage.view(B, L, E)[:nb, :, :nh * D].float().cpu().numpy()
        return np.asfortranarray(t.transpose(2, 1, 0))

    def run(nh, nb):
        q, k, v = host(runner.q, Lq, nh, nb), host(runner.k, Lkv, nh, nb), host(runner.v, Lkv, nh, nb)
        bias = None
        if runner.bias is not None:
            t = runner.bias.storage.view(B, H, Lq, Lkv)[:nb, :nh].float().cpu().numpy()
            bias = np.asfortranarray(t.transpose(3, 2, 1, 0))
        t0 = time.perf_counter()
        O.nnlib_attention_f32(q, k, v, bias, mask, nh, nthreads=cores)
        return time.perf_counter() - t0

    try:
        trial_h = min(H, cores)
        t_trial = run(trial_h, 1)
        slices = H * B
        want = int(max(trial_h, min(slices, trial_h * budget_s / max(t_trial, 1e-6))))
        nh = min(H, want)
        nb = max(1, min(B, want // nh))
        dt = run(nh, nb) if nh * nb > trial_h else t_trial
        n = nh * nb if nh * nb > trial_h else trial_h
    finally:
        O.use_host_blas(False)
    flops, nbytes = algorithmic_work(w)
    full_s = dt * slices / n
    gemm = f"GEMM slices by {blas}" if blas else "GEMM slices by the oracle's own 8x16 SGEMM kernel (no BLAS could be bound)"
    return dict(seconds_sample=dt, seconds_full_job=full_s, cores=cores,
                sample=f"{n} of {slices} (head, batch) slices of the tensors the GPU was timed on ({dt:.1f} s), Float32, "
                       f"{cores} threads over batch slices (NNlib's policy), {gemm}, scaled by {slices / n:.3g}x",
                tflops=flops / full_s / 1e12, gbps=nbytes / full_s / 1e9)


def measure(key, steps, warmup, with_cpu):
    w = WORKLOADS[key]
    r = Runner(key)
    ms, wall_ms = r.time(steps, warmup)
    flops, nbytes = algorithmic_work(w)
    tflops = flops / (ms * 1e-3) / 1e12
    gbps = nbytes / (ms * 1e-3) / 1e9
    # C2 returns its weights: 512 MiB written put its HBM floor (84 us) above the matrix floor of its products on the
    # bf16 planes (3 products executed for the 2 counted: 62 us), so HBM is the roofline that binds it
    hbm_bound = key in HBM_BOUND or (key == "c2" and os.environ.get("MI355ATTN_F32_MFMA", "")[:1] != "1")
    traffic, source = measured_traffic(key)
    if hbm_bound:
        roof = dict(bound="hbm", achieved=gbps, peak=HBM_PEAK, unit="GB/s", frac=gbps / HBM_PEAK, traffic=traffic,
                    traffic_source=source)
        if w["dtype"] == "f32":
            roof["mfma"] = dict(achieved=tflops, peak=PEAK["f32"], unit="TFLOP/s", frac=tflops / PEAK["f32"])
            f32_products(roof["mfma"], tflops, 1.5 if w["weights"] else 1.0)   # weights: QK^T runs in both passes
    else:
        pk = PEAK[w["dtype"]]
        roof = dict(bound="mfma", achieved=tflops, peak=pk, unit="TFLOP/s", frac=tflops / pk, traffic=traffic,
                    traffic_source=source, hbm_frac=gbps / HBM_PEAK)
        if w["dtype"] == "f32":
            f32_products(roof, tflops, 1.5 if w["weights"] else 1.0)
    res = dict(workload=w["name"], kernel=r.kernel, preheat_ms=r.preheat_ms, ms_per_step=ms, wall_ms_per_step=wall_ms, tflops=tflops, gbps=gbps,
               flops_per_step=flops, bytes_per_step=nbytes, roofline=roof)
    if with_cpu:
        c = cpu_baseline(r)
        if hbm_bound:
            res["cpu_baseline"] = dict(value=c["gbps"], unit="GB/s", cores=c["cores"], kind="port", sample=c["sample"],
                                       seconds_sample=c["seconds_sample"])
        else:
            res["cpu_baseline"] = dict(value=c["tflops"], unit="TFLOP/s", cores=c["cores"], kind="port",
                                       sample=c["sample"], seconds_sample=c["seconds_sample"])
    del r
    return res


# ---- the rows built after the five configurations: gradient and softmax family ------------------------

EXTRA = {
    "bwd": "gradient of C3: causal bf16 (4096,4096,2) H=32 D=128, dq + dk + dv from dy and the forward result",
    "dense_mask": "forward call of the C3 shape with a dense Bool mask (4096, 4096), 90 % kept, not causal, weights not materialised; "
                  "the same call without the mask is timed beside it",
    "bwd_f32": "gradient of C2: causal f32 (1024,1024,8) H=16 D=64, dq + dk + dv from dy and the forward result",
    "bwd_c1": "gradient of C1: f32 (512,128,4) H=8 D=64, not causal, dq + dk + dv from dy and the forward result (a call on few workgroups: report us)",
    "logsoftmax": "logsoftmax(x; dims=1), x (4096, 65536) f32 (1 GiB in, 1 GiB out)",
    "softmax_dims2": "softmax(x; dims=2), x (256, 4096, 128) bf16 (256 MiB in, 256 MiB out), reduction over the strided dim",
    "softmax": "softmax(x; dims=1), x (1024, 131072) f32: the logits of C2 (512 MiB in, 512 MiB out)",
    "batched_mul": "batched_mul(A, B), A (2048, 2048, 16), B (2048, 2048, 16) bf16",
    "batched_mul_f32": "batched_mul(A, B), A (1024, 64, 128), B (64, 1024, 128) f32: the score product of C2",
    "batched_mul_c32": "batched_mul(A, B), A and B (1024, 1024, 16) ComplexF32, 8 real FLOP per complex multiply-add",
    "batched_mul_f64": "batched_mul(A, B), A (1024, 1024, 32), B (1024, 1024, 32) Float64",
}


def _event_time(lib, _lib, fn, steps, warmup):
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.check(lib.mi_event_create(ctypes.byref(e0)))
    _lib.check(lib.mi_event_create(ctypes.byref(e1)))
    preheat(fn, lambda: _lib.check(lib.mi_device_sync()))
    for _ in range(warmup):
        fn()
    _lib.check(lib.mi_device_sync())
    _lib.check(lib.mi_event_record(e0, None))
    for _ in range(steps):
        fn()
    _lib.check(lib.mi_event_record(e1, None))
    _lib.check(lib.mi_event_sync(e1))
    ms = ctypes.c_float(0)
    _lib.check(lib.mi_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    lib.mi_event_destroy(e0)
    lib.mi_event_destroy(e1)
    return ms.value / steps


def measure_extra(key, steps, warmup, with_cpu):
    """The JSON line (as a dict) of a workload outside BASELINE.json's five configurations (same fields)."""
    import numpy as np
    import nnlib_amd as nn
    from nnlib_amd import _lib
    lib = _lib.load()
    _lib.check(lib.mi_init(0))
    DA = nn.DeviceArray
    cores = min(16, len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1))
    if key == "dense_mask":
        # a mask that depends on the query (src/attention.jl:122-124): packed into bits by a pre-pass inside the call and
        # applied by the software-pipelined kernel; the step timed is the whole call, pre-pass included
        ms_of = {}
        for name, extra in (("unmasked", {}), ("masked", dict(mask=True))):
            WORKLOADS["_dense_mask"] = dict(WORKLOADS["c3"], causal=False, **extra)
            try:
                r = Runner("_dense_mask", rotate=False)
                ms_of[name], _ = r.time(steps, warmup)
                kernel = r.kernel
                flops, _ = algorithmic_work(r.w)
                del r
            finally:
                del WORKLOADS["_dense_mask"]
        ms = ms_of["masked"]
        val = flops / (ms * 1e-3) / 1e12
        line = dict(metric="attention forward TFLOP/s (all pairs counted)", value=val, unit="TFLOP/s", dtype="bf16",
                    roofline=dict(bound="mfma", achieved=val, peak=PEAK["bf16"], unit="TFLOP/s", frac=val / PEAK["bf16"], **measured_traffic_fields(key)),
                    config=dict(workload=EXTRA[key], kernel=kernel, unmasked_ms_per_step=ms_of["unmasked"],
                                rate_against_unmasked=ms_of["unmasked"] / ms),
                    flops_per_step=flops)
    elif key in ("bwd", "bwd_f32", "bwd_c1"):
        w = WORKLOADS[{"bwd": "c3", "bwd_f32": "c2", "bwd_c1": "c1"}[key]]
        E, L, B, H = w["E"], w["Lq"], w["B"], w["H"]
        D = E // H
        dtn = w["dtype"]
        arrs = [DA.empty((E, L, B), dtn) for _ in range(4)]
        for sid, a in enumerate(arrs):
            _lib.check(lib.mi_randn_fill(a.ptr, a.code, a.length, w["seed"], sid, w["scale"] if sid < 2 else 1.0, None))
        q, k, v, dy = arrs
        cmask = nn.make_causal_mask(q) if w["causal"] else None
        y, _ = nn.dot_product_attention(q, k, v, mask=cmask, nheads=H, return_weights=False,
                                        save_for_backward=True)   # as an AD rule would: the pullback reuses the row statistics
        d = _lib.mi_attn_bwd_desc()
        d.struct_size = ctypes.sizeof(_lib.mi_attn_bwd_desc)
        nn.ops._fill_desc(d.fwd, q, k, v, None, cmask, H, B, E, E, L, L, 0)
        d.fwd.out, d.dout, d.fwd.stats = y.ptr, dy.ptr, y.saved_stats.ptr
        grads = [DA.empty((E, L, B), dtn) for _ in range(3)]
        d.dq, d.dk, d.dv = (g.ptr for g in grads)
        kern, ws = ctypes.c_int32(0), ctypes.c_size_t(0)
        _lib.check(lib.mi_attention_bwd_plan(ctypes.byref(d), ctypes.byref(kern), ctypes.byref(ws)))
        wsbuf = DA.empty((ws.value // 4 + 4,), "f32")
        d.workspace, d.workspace_bytes = wsbuf.ptr, ws.value
        ms = _event_time(lib, _lib, lambda: _lib.check(lib.mi_attention_bwd(ctypes.byref(d), None)), steps, warmup)
        # five products (S, dP, dV, dK, dQ) of 2*D FLOP per unmasked (query, key) pair
        flops = 10 * D * H * B * (L * (L + 1) // 2 if w["causal"] else L * L)
        val = flops / (ms * 1e-3) / 1e12
        line = dict(metric="attention gradient TFLOP/s", value=val, unit="TFLOP/s", dtype=dtn,
                    roofline=dict(bound="mfma", achieved=val, peak=PEAK[dtn], unit="TFLOP/s", frac=val / PEAK[dtn], **measured_traffic_fields(key)),
                    config=dict(workload=EXTRA[key], kernel=_lib.KERNEL_NAMES[kern.value]), flops_per_step=flops)
        # dQ kernel S, dP, dQ; fused dK / dV kernel S, dP, dV, dK (16-bit and Float32 alike)
        per_counted = 7 / 5
        line["roofline"]["products_executed_per_counted"] = per_counted
        if dtn == "f32":
            f32_products(line["roofline"], val, per_counted)
        if with_cpu:
            from oracle import oracle as O
            rng = np.random.default_rng(0)
            nh, nb = (4, 1) if key == "bwd" else (H, 2)          # a bounded sample of whole (head, batch) slices
            a1 = [np.asfortranarray(rng.standard_normal((nh * D, L, nb))) for _ in range(4)]
            t0 = time.perf_counter()
            O.attention_bwd_f64(a1[0], a1[1], a1[2], a1[3], None, O.make_causal_mask(L) if w["causal"] else None, nh)
            dt = time.perf_counter() - t0
            line["cpu_baseline"] = dict(value=flops * nh * nb / (dt * H * B) / 1e12, unit="TFLOP/s", cores=1, kind="port",
                                        sample=f"{nh * nb} of {H * B} (head, batch) slices, forward + gradient oracle in Float64 on one "
                                               f"thread ({dt:.1f} s), scaled by {H * B / (nh * nb):g}x")
    elif key.startswith("batched_mul"):
        if key == "batched_mul":
            dt_name, (m, kk, n, nb) = "bf16", (2048, 2048, 2048, 16)
        elif key == "batched_mul_c32":
            dt_name, (m, kk, n, nb) = "c64", (1024, 1024, 1024, 16)
        elif key == "batched_mul_f64":
            dt_name, (m, kk, n, nb) = "f64", (1024, 1024, 1024, 32)
        else:
            dt_name, (m, kk, n, nb) = "f32", (1024, 64, 1024, 128)
        A, Bm = DA.empty((m, kk, nb), dt_name), DA.empty((kk, n, nb), dt_name)
        C = DA.empty((m, n, nb), dt_name)
        for sid, a in enumerate((A, Bm)):
            if dt_name == "c64":   # a complex array is filled as twice as many Float32 values
                _lib.check(lib.mi_randn_fill(a.ptr, _lib.MI_F32, 2 * a.length, 11, sid, 1.0, None))
            elif dt_name == "f64":   # Float32 values widened (the generator has no Float64 stream)
                tmp = DA.empty(a.dims, "f32")
                _lib.check(lib.mi_randn_fill(tmp.ptr, tmp.code, tmp.length, 11, sid, 1.0, None))
                a.storage.copy_(tmp.storage.double())
            else:
                _lib.check(lib.mi_randn_fill(a.ptr, a.code, a.length, 11, sid, 1.0, None))
        ms = _event_time(lib, _lib, lambda: nn.batched_mul_(C, A, Bm), steps, warmup)
        flops = (8 if dt_name == "c64" else 2) * m * n * kk * nb
        val = flops / (ms * 1e-3) / 1e12
        peak = PEAK["f32"] if dt_name == "c64" else PEAK[dt_name]
        line = dict(metric="batched_mul TFLOP/s", value=val, unit="TFLOP/s", dtype=dt_name,
                    roofline=dict(bound="mfma", achieved=val, peak=peak, unit="TFLOP/s", frac=val / peak, **measured_traffic_fields(key)),
                    config=dict(workload=EXTRA[key]),
                    flops_per_step=flops)
        if dt_name == "f32":
            f32_products(line["roofline"], val)
        es_out = {"bf16": 2, "f32": 4, "c64": 8, "f64": 8}[dt_name]
        line["roofline"]["hbm_frac"] = es_out * (m * kk + kk * n + m * n) * nb / (ms * 1e-3) / 1e9 / HBM_PEAK   # every operand once
        if with_cpu and dt_name not in ("c64", "f64"):
            from oracle import oracle as O
            ns = min(nb, 2 if key == "batched_mul" else 32)
            rng = np.random.default_rng(0)
            Ah = np.asfortranarray(rng.standard_normal((m, kk, ns), dtype=np.float32))
            Bh = np.asfortranarray(rng.standard_normal((kk, n, ns), dtype=np.float32))
            t0 = time.perf_counter()
            O.batched_gemm(Ah, Bh, nthreads=cores)
            dt = time.perf_counter() - t0
            line["cpu_baseline"] = dict(value=2 * m * n * kk * ns / dt / 1e12, unit="TFLOP/s", cores=min(cores, ns), kind="port",
                                        sample=f"{ns} of {nb} slices in Float32, one thread per slice as src/gemm.jl:121-123 ({dt:.1f} s)")
    else:
        if key == "logsoftmax":
            dims, dt_name, shape, op = 1, "f32", (4096, 65536), _lib.MI_LOGSOFTMAX
        elif key == "softmax":
            dims, dt_name, shape, op = 1, "f32", (1024, 131072), _lib.MI_SOFTMAX
        else:
            dims, dt_name, shape, op = 2, "bf16", (256, 4096, 128), _lib.MI_SOFTMAX
        nsets = 2 if key in ("logsoftmax", "softmax") else 4          # rotate past the 256 MiB last-level cache
        xs = [DA.empty(shape, dt_name) for _ in range(nsets)]
        ys = [DA.empty(shape, dt_name) for _ in range(nsets)]
        for x in xs:
            _lib.check(lib.mi_randn_fill(x.ptr, x.code, x.length, 7, 0, 1.0, None))
        inner, n, outer, _ = nn.ops._reduction_geometry(shape, dims)
        state = {"i": 0}

        def fn():
            i = state["i"] = (state["i"] + 1) % nsets
            _lib.check(lib.mi_softmax(op, xs[i].code, xs[i].ptr, ys[i].ptr, inner, n, outer, None))
        ms = _event_time(lib, _lib, fn, steps, warmup)
        nbytes = 2 * xs[0].length * xs[0].itemsize       # one read, one write
        val = nbytes / (ms * 1e-3) / 1e9
        line = dict(metric=f"{key} GB/s", value=val, unit="GB/s", dtype=dt_name,
                    roofline=dict(bound="hbm", achieved=val, peak=HBM_PEAK, unit="GB/s", frac=val / HBM_PEAK, **measured_traffic_fields(key)),
                    config=dict(workload=EXTRA[key]),
                    bytes_per_step=nbytes)
        if with_cpu:
            from oracle import oracle as O
            small = (shape[0], shape[1] // 16) + shape[2:]
            xh = np.asfortranarray(np.random.default_rng(0).standard_normal(small).astype(np.float32))
            t0 = time.perf_counter()
            O.softmax(xh, dims, np.float32, log=(key == "logsoftmax"))
            dt = time.perf_counter() - t0
            line["cpu_baseline"] = dict(value=nbytes / 16 / dt / 1e9, unit="GB/s", cores=1, kind="port",
                                        sample=f"1/16 of the array, Float32 oracle on one thread as the reference's passes are ({dt:.2f} s)")
    line.update(n_gpus=1, steps=steps, warmup=warmup, ms_per_step=ms, higher_is_better=True, scaling="weak", vs_baseline=None,
                data="synthetic")
    return line


def copy_calibration(steps):
    """A plain copy kernel of known size (1 GiB read, 1 GiB written per launch): the reference point
    that the FETCH_SIZE / WRITE_SIZE counters are scaled by when HBM traffic is read with rocprofv3."""
    import torch
    import nnlib_amd
    from nnlib_amd import _lib
    lib = _lib.load()
    _lib.check(lib.mi_init(0))
    n = 1 << 28
    src = nnlib_amd.DeviceArray.zeros((n,), "f32")
    dst = nnlib_amd.DeviceArray.empty((n,), "f32")
    for _ in range(steps):
        _lib.check(lib.mi_convert(dst.ptr, _lib.MI_F32, src.ptr, _lib.MI_F32, n, None))
    _lib.check(lib.mi_device_sync())
    print(json.dumps({"workload": "copy", "kernel": "convert_kernel<F32, F32>", "bytes_read": 4 * n,
                      "bytes_written": 4 * n, "launches": steps}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + sorted(EXTRA) + ["copy"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--preheat", type=float, default=1.0, help="seconds of untimed launches before the counted warm-up")
    ap.add_argument("--no-decode", action="store_true", help="skip the secondary decode measurement")
    args = ap.parse_args()
    globals()["PREHEAT_S"] = args.preheat
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only ((head, batch) pairs are independent problems and shard "
                 "without communication). Run with --gpus 1.")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the attention path has no CPU fallback")

    if args.workload == "copy":
        return copy_calibration(min(args.steps, 10))
    if args.workload in EXTRA:
        print(json.dumps(measure_extra(args.workload, min(args.steps, 50), min(args.warmup, 10), not args.no_cpu)))
        return
    main_res = measure(args.workload, args.steps, args.warmup, not args.no_cpu)
    w = WORKLOADS[args.workload]
    prefill = args.workload not in ("c4", "c5")
    line = {
        "metric": "attention TFLOP/s (prefill)" if prefill else "attention GB/s (HBM-bound)",
        "value": main_res["tflops"] if prefill else main_res["gbps"],
        "unit": "TFLOP/s" if prefill else "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "preheat_ms": main_res["preheat_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": main_res["workload"], "kernel": main_res["kernel"], "E": w["E"], "Lq": w["Lq"],
                   "Lkv": w["Lkv"], "B": w["B"], "nheads": w["H"], "causal": w["causal"]},
        "roofline": main_res["roofline"],
        "flops_per_step": main_res["flops_per_step"], "bytes_per_step": main_res["bytes_per_step"],
    }
    if "cpu_baseline" in main_res:
        line["cpu_baseline"] = main_res["cpu_baseline"]
    if args.workload == "c3" and not args.no_decode:
        # the other four configurations of BASELINE.json in the same line: C5 (the decode target) also under "decode"
        line["configs"] = {}
        for key in ("c1", "c2", "c4", "c5"):
            ksteps = max(5, min(args.steps, 50))
            res = measure(key, ksteps, min(args.warmup, 10), not args.no_cpu)
            hbm = res["roofline"]["bound"] == "hbm"
            entry = {"metric": "attention GB/s" if hbm else "attention TFLOP/s", "value": res["gbps"] if hbm else res["tflops"],
                     "unit": "GB/s" if hbm else "TFLOP/s", "ms_per_step": res["ms_per_step"], "us_per_step": 1e3 * res["ms_per_step"],
                     "tflops": res["tflops"], "gbps": res["gbps"], "steps": ksteps,
                     "dtype": WORKLOADS[key]["dtype"], "config": {"workload": res["workload"], "kernel": res["kernel"]},
                     "roofline": res["roofline"], "flops_per_step": res["flops_per_step"], "bytes_per_step": res["bytes_per_step"]}
            if "cpu_baseline" in res:
                entry["cpu_baseline"] = res["cpu_baseline"]
            line["configs"][key] = entry
        dec = dict(line["configs"]["c5"])
        dec["metric"] = "attention GB/s (decode)"
        line["decode"] = dec
        # the workloads beyond the five configurations (gradient, softmax family, batched_mul), GPU leg only, so that
        # their figures are measured by whoever runs this script and not only quoted
        line["next_rows"] = {}
        for key in EXTRA:
            try:
                res = measure_extra(key, max(5, min(args.steps, 20)), min(args.warmup, 5), False)
                line["next_rows"][key] = {f: res[f] for f in ("metric", "value", "unit", "ms_per_step", "steps", "dtype", "config", "roofline")}
            except Exception as e:   # a failure here must not cost the headline figures above; it is reported, not hidden
                line["next_rows"][key] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(line))
    sys.stdout.flush()


if __name__ == "__main__":
    main()
