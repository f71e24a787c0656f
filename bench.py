#!/usr/bin/env python3
"""Benchmark of the HIPTensor kernel path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the hot path over one batch of synthetic fp32 input
at the metric size, 2^26 elements = (8192, 8192), seed 6:

    x <- x + y      AddNode, in place, both operands full      12 B/elem
    x <- x * y      MulNode, in place                          12 B/elem
    o <- exp(y)     ExpNode                                     8 B/elem
    r <- r + sum_c y[:, c]   (!sum y :axis 1)                   4 B/elem

`value` is the algorithmic bytes of a step divided by its time (GB/s), with all
inputs resident in HBM before the timed region.  Every launch works on a
different buffer set of a ring much larger than the 256 MB Infinity Cache, so
no launch finds its operands cached from the previous one.

Extra fields: per-kernel GB/s, the roofline of the dominant kernel (the
in-place binary kernel) from HIP events recorded on the library's stream, the
GPT-2-small block forward time, and the CPU baseline (the reference's own C
kernels compiled under oracle/_ref when present, else the oracle port) timed
on one host core -- cl-waffe2 runs these kernels single-threaded
(`*num-cores*` = 1, no define-impl passes :lparallel).
"""
from __future__ import annotations

import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N = 1 << 26
SIDE = 8192
HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3
BYTES = {"add": 12 * N, "mul": 12 * N, "exp": 8 * N, "rowsum": 4 * N + 4 * SIDE}
RING = 8  # buffer sets: 8 x (x, y, o) x 256 MiB = 6 GiB
# HBM bytes per launch of the in-place binary kernel at 2^26 elements come from two
# `rocprofv3 --pmc` runs of `bench.py --probe` (FETCH_SIZE, then WRITE_SIZE, KiB per
# dispatch), each scaled by what the same counter reads for the plain copy of 2^26
# floats in the same run.  A process cannot read these counters for itself, so the
# figure is read at run time from the committed summary of those runs.
TRAFFIC_PROFILE = os.path.join("profiles", "ew_metric_2p26_pmc_fetch_write.txt")


def binary_traffic_bytes():
    """(bytes, source) for `roofline.traffic`: the "traffic MB" column of the OpAdd line
    of the committed counter summary, or (None, reason) when it cannot be read."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        for line in open(path):
            if "OpAdd" in line:
                cols = line.split()
                return int(round(float(cols[2]) * 1e6)), f"{TRAFFIC_PROFILE} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --probe`, read at run time)"
    except (OSError, ValueError, IndexError):
        pass
    return None, f"{TRAFFIC_PROFILE} not readable"


def profiler_attached():
    """True when a rocprofiler tool library is preloaded into this process.  Replaying HIP
    graphs under the profiler once ended in a host-side fault inside hipGraphLaunch, so the
    rows are then timed from stream launches only."""
    probe = " ".join(os.environ.get(k, "") for k in ("ROCP_TOOL_LIBRARIES", "LD_PRELOAD", "HSA_TOOLS_LIB",
                                                     "ROCPROFILER_LIBRARY_PATH"))
    return "rocprof" in probe.lower()


def p(t):
    return C.c_void_p(t.ptr)


def gpu_steps(W, steps: int, warmup: int):
    lib = W.lib.get()
    rng = np.random.Generator(np.random.PCG64(6))
    hx = rng.standard_normal(N).astype(np.float32)
    hy = rng.standard_normal(N).astype(np.float32)
    x0, y0 = W.HIPTensor.from_numpy(hx), W.HIPTensor.from_numpy(hy)
    del hx, hy
    ring = []
    for i in range(RING):
        xs, ys, os_ = (W.HIPTensor([N]) for _ in range(3))
        W.lib.check(lib.wf2hip_memcpy_d2d(p(xs), p(x0), 4 * N))
        W.lib.check(lib.wf2hip_memcpy_d2d(p(ys), p(y0), 4 * N))
        ring.append((xs, ys, os_, W.HIPTensor([SIDE])))
    W.lib.synchronize()

    def launch(name, slot):
        xs, ys, os_, rs = ring[slot % RING]
        if name == "add":
            W.lib.check(lib.wf2hip_sadd(N, p(xs), 1, p(ys), 1))
        elif name == "mul":
            W.lib.check(lib.wf2hip_smul(N, p(xs), 1, p(ys), 1))
        elif name == "exp":
            W.lib.check(lib.wf2hip_sexp(N, p(ys), 1, p(os_), 1))
        else:
            W.lib.check(lib.wf2hip_reduce_add_rows_f32(SIDE, SIDE, p(ys), SIDE, p(rs), 1))

    order = ["add", "mul", "exp", "rowsum"]
    slot = 0
    for _ in range(warmup):
        for name in order:
            launch(name, slot)
            slot += 1
    W.lib.synchronize()

    # timed region: exactly K steps, launched back to back, bracketed by a
    # synchronisation and one HIP event on the library's stream at each end
    W.lib.synchronize()
    e0, e1 = W.lib.Event(), W.lib.Event()
    t0 = time.perf_counter()
    e0.record()
    for s in range(steps):
        for name in order:
            launch(name, slot)
            slot += 1
    e1.record()
    W.lib.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    step_ms = e0.elapsed_ms(e1) / steps

    # the same step after the clock has settled: the timed region above starts from an
    # idle GPU and is over in a few milliseconds, while the core clock takes 2-3 ms of
    # load to come down from its boost level.  ~40 ms of the same steps, then 20 timed.
    for s in range(max(1, int(40.0 / max(step_ms, 1e-3)))):
        for name in order:
            launch(name, slot)
            slot += 1
    a, b = W.lib.Event(), W.lib.Event()
    a.record()
    for s in range(20):
        for name in order:
            launch(name, slot)
            slot += 1
    b.record()
    sustained_ms = a.elapsed_ms(b) / 20

    # per-kernel average launch duration: each kernel alone, back to back on the
    # ring (cold operands), event pair around the run
    reps = max(steps, 20)
    per_kernel = {}
    for name in order:
        a, b = W.lib.Event(), W.lib.Event()
        a.record()
        for _ in range(reps):
            launch(name, slot)
            slot += 1
        b.record()
        per_kernel[name] = a.elapsed_ms(b) / reps
    return step_ms, wall_ms / steps, per_kernel, per_kernel["add"], sustained_ms


def counter_probe(W, reps: int = 5):
    """A short fixed sequence for `rocprofv3 --pmc` runs: `reps` launches each of
    a plain copy of known size (2^26 floats: 256 MiB read, 256 MiB written; the
    calibration for FETCH_SIZE / WRITE_SIZE) and of the four metric kernels, each
    on a different buffer set so that no launch finds its data in cache."""
    lib = W.lib.get()
    ring = [(W.HIPTensor([N], initial_element=1.0), W.HIPTensor([N], initial_element=1.0),
             W.HIPTensor([N]), W.HIPTensor([SIDE])) for _ in range(RING)]
    W.lib.synchronize()
    slot = 0
    for name in ("copy", "add", "mul", "exp", "rowsum"):
        for _ in range(reps):
            xs, ys, os_, rs = ring[slot % RING]
            slot += 1
            if name == "copy":
                W.lib.check(lib.wf2hip_scopy(N, p(ys), 1, p(os_), 1))
            elif name == "add":
                W.lib.check(lib.wf2hip_sadd(N, p(xs), 1, p(ys), 1))
            elif name == "mul":
                W.lib.check(lib.wf2hip_smul(N, p(xs), 1, p(ys), 1))
            elif name == "exp":
                W.lib.check(lib.wf2hip_sexp(N, p(ys), 1, p(os_), 1))
            else:
                W.lib.check(lib.wf2hip_reduce_add_rows_f32(SIDE, SIDE, p(ys), SIDE, p(rs), 1))
    W.lib.synchronize()
    print(json.dumps({"probe": "copy, add, mul, exp, rowsum", "launches_each": reps, "elements": N}))


def row_probe(W, reps: int = 5):
    """The launch sequence for `rocprofv3 --pmc` runs of the other kernels of the path: `reps`
    launches each, in the order printed at the end, every launch on another buffer set (cold
    cache).  The first case, a plain copy of 2^26 floats, calibrates FETCH_SIZE / WRITE_SIZE."""
    F = W.functional
    T = W.HIPTensor
    rng = np.random.Generator(np.random.PCG64(6))
    order = []

    def normal(shape, scale=1.0):
        return T.from_numpy((rng.standard_normal(shape) * scale).astype(np.float32))

    def uniform(shape, lo, hi):
        return T.from_numpy(rng.uniform(lo, hi, size=shape).astype(np.float32))

    def run(label, nbytes, make, call, launches=1):
        count = max(2, min(8, -(-(1 << 30) // max(nbytes, 1))))
        ring = [make() for _ in range(count)]
        W.lib.synchronize()
        for i in range(reps):
            call(ring[i % count])
        W.lib.synchronize()
        order.append({"case": label, "launches_per_call": launches, "calls": reps, "algorithmic_bytes": nbytes})
        ring.clear()

    x0 = normal([N])
    run("copy 2^26 (calibration)", 8 * N, lambda: (F.copy(x0), T([N], initial_element=None)),
        lambda s: F.move_(s[1], s[0]))
    for label, fn, lo, hi in (("exp", F.exp, -10.0, 10.0), ("tanh", F.tanh, -10.0, 10.0),
                              ("sin", F.sin, -100.0, 100.0), ("loge", F.loge, 1e-3, 1e3)):
        u0 = uniform([N], lo, hi)
        run(f"{label} 2^26", 8 * N, lambda: (F.copy(u0), T([N], initial_element=None)),
            lambda s, fn=fn: fn(s[0], out=s[1]))
        del u0
    run("GELU 2^26", 8 * N, lambda: (F.copy(x0), T([N], initial_element=None)), lambda s: F.gelu_fused(s[0], out=s[1]))
    del x0
    R, Cn = 4096, 8192
    a0, b0 = normal([R, Cn]), normal([1, Cn])
    yb = b0.view((":broadcast", R), True)
    run("A(4096,8192) += B(1,8192)", 8 * R * Cn + 4 * Cn, lambda: F.copy(a0), lambda s: F.add_(s, yb))
    run("A[:, ::2] *= 0.5", 8 * R * Cn // 2, lambda: F.copy(a0), lambda s: F.mul_(s.view(True, (0, Cn, 2)), 0.5))
    run("copy of A[:, ::2]", 8 * R * Cn // 2, lambda: (F.copy(a0), T([R, Cn // 2], initial_element=None)),
        lambda s: F.move_(s[1], s[0].view(True, (0, Cn, 2))))
    del a0, b0, yb
    a0 = normal([SIDE, SIDE])
    run("transposing copy (8192,8192)", 8 * N, lambda: (F.copy(a0), T([SIDE, SIDE], initial_element=None)),
        lambda s: F.move_(s[1], s[0].permute(1, 0)))
    del a0
    R, Cn = 8192, 4096
    a0 = normal([R, Cn])
    run("row sum (8192,4096), one node", 4 * R * Cn + 4 * R, lambda: (F.copy(a0), T([R, 1])),
        lambda s: F.sum(s[0], axis=1, out=s[1], keepdims=True))
    run("full sum (8192,4096), one node", 4 * R * Cn, lambda: (F.copy(a0), T([1, 1])),
        lambda s: F.sum(s[0], axis=True, out=s[1], keepdims=True), launches=2)
    del a0
    R, Cn = 32768, 1024
    a0 = normal([R, Cn], 3.0)
    run("copy (32768,1024)", 8 * R * Cn, lambda: (F.copy(a0), T([R, Cn], initial_element=None)),
        lambda s: F.move_(s[1], s[0]))
    run("row softmax (32768,1024)", 8 * R * Cn, lambda: (F.copy(a0), T([R, Cn], initial_element=None)),
        lambda s: F.softmax_fused(s[0], out=s[1]))
    del a0
    R, Cn = 65536, 1024
    a0, g0, b0 = normal([R, Cn]), normal([Cn]), normal([Cn])
    run("LayerNorm (65536,1024)", 8 * R * Cn, lambda: (F.copy(a0), T([R, Cn], initial_element=None)),
        lambda s: F.layer_norm_fused(s[0], g0, b0, out=s[1]))
    del a0
    p0 = normal([N])
    run("Adam step 2^26", 28 * N, lambda: (W.optimizers.Adam(F.copy(p0), lr=1e-3), F.copy(p0)), lambda s: s[0].step(s[1]))
    run("SGD step 2^26", 16 * N, lambda: (W.optimizers.SGD(F.copy(p0), lr=1e-3), F.copy(p0)), lambda s: s[0].step(s[1]))
    run("GELU backward 2^26", 12 * N, lambda: (F.copy(p0), F.copy(p0)),
        lambda s: F.activation_backward("gelu", s[0], s[1], in_place=True))
    del p0
    R, Cn = 32768, 1024
    a0 = normal([R, Cn], 3.0)
    y0 = F.softmax_fused(a0)
    run("softmax backward (32768,1024)", 12 * R * Cn, lambda: (F.copy(y0), F.copy(a0)),
        lambda s: F.softmax_backward(s[0], s[1], in_place=True))
    del a0, y0
    R, Cn = 65536, 1024
    a0, g0 = normal([R, Cn]), normal([Cn])
    dg, db = T([Cn], initial_element=None), T([Cn], initial_element=None)
    run("LayerNorm backward (65536,1024)", 12 * R * Cn, lambda: (F.copy(a0), F.copy(a0), T([R, Cn], initial_element=None)),
        lambda s: W.nodes.forward("HIP-LayerNorm-Node-backward", s[0], g0, s[1], s[2], dg, db, 1e-5), launches=3)
    del a0, g0, dg, db
    R, Cn = 32768, 1024
    a0 = normal([R, Cn], 3.0)
    t0 = F.softmax_fused(normal([R, Cn]))
    run("softmax cross entropy (32768,1024)", 16 * R * Cn,
        lambda: (F.copy(a0), F.copy(t0), T([R, Cn], initial_element=None), T([R, Cn], initial_element=None)),
        lambda s: W.nodes.forward("HIP-Softmax-Cross-Entropy-Node", s[0], s[1], s[2], s[3], 1e-7))
    run("softmax cross entropy backward (32768,1024)", 16 * R * Cn, lambda: (F.copy(a0), F.copy(t0), F.copy(t0)),
        lambda s: W.nn.softmax_cross_entropy_backward_fused(s[0], s[1], s[2], in_place=True))
    del a0, t0
    Nb, Cc, Hh, Kk = 32, 64, 56, 3
    img, padded = normal([Nb, Cc, Hh, Hh]), normal([Nb, Cc, Hh + 2, Hh + 2])
    ncol, nim = Nb * Cc * Kk * Kk * Hh * Hh, Nb * Cc * Hh * Hh
    run("unfold (32,64,56,56) 3x3 pad 1", 4 * (ncol + nim), lambda: T([Nb * Hh * Hh, Cc * Kk * Kk], initial_element=None),
        lambda s: W.nodes.forward("HIP-Unfold-Node", img, s, (Kk, Kk), (1, 1), (1, 1)))
    run("Im2ColNode (32,64,58,58) 3x3", 4 * (ncol + nim), lambda: T([Nb, Cc, Kk, Kk, Hh, Hh], initial_element=None),
        lambda s: W.nodes.forward("Im2ColNode", padded, s, (1, 1), (0, 0), (1, 1)))
    back = T([Nb, Cc, Hh + 2, Hh + 2], initial_element=None)
    run("Col2ImNode (32,64,3,3,56,56)", 4 * (ncol + nim), lambda: normal([Nb, Cc, Kk, Kk, Hh, Hh]),
        lambda s: W.nodes.forward("Col2ImNode", s, back, (1, 1), (1, 1), (1, 1)))
    print(json.dumps({"probe_rows": order}))


def matrix_core_probe(W, reps: int = 4):
    """The launch sequence for `rocprofv3 --pmc` runs of the kernels bound by the matrix cores, at the block's
    shapes: `reps` launches each of attention forward (full, then causal), attention backward (causal:
    D, then dQ / dK / dV in one launch), the block's projections and the products of a few rows, printed in order
    at the end."""
    F = W.functional
    T = W.HIPTensor
    rng = np.random.Generator(np.random.PCG64(6))
    B, S, H, hd = 8, 1024, 12, 64
    qkv = T.from_numpy(rng.standard_normal((B, S, 3 * H, hd)).astype(np.float32))
    q, k, v = (qkv.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
    out = T([B, S, H, hd], initial_element=None).permute(0, 2, 1, 3)
    lse = T([B, H, S], initial_element=None)
    dout = T.from_numpy(rng.standard_normal((B, S, H, hd)).astype(np.float32)).permute(0, 2, 1, 3)
    dqkv = T([B, S, 3 * H, hd], initial_element=None)
    dq, dk, dv = (dqkv.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
    for causal in (False, True):
        for _ in range(reps):
            F.attention(q, k, v, out=out, causal=causal, lse=lse)
    for _ in range(reps):
        F.attention_backward(q, k, v, dout, causal=True, dq=dq, dk=dk, dv=dv, out=out, lse=lse)
    # the four projections of the block with their epilogues (bias; bias + residual; bias + GELU), the
    # plain product of the widest one, and a cube
    M = B * S
    names = []
    for m, n, k, bias, res, act in ((M, 2304, 768, True, False, None), (M, 768, 768, True, True, None),
                                    (M, 3072, 768, True, False, "gelu"), (M, 768, 3072, True, True, None),
                                    (M, 3072, 768, False, False, None), (4096, 4096, 4096, False, False, None)):
        a = T.from_numpy(rng.standard_normal((m, k)).astype(np.float32))
        b = T.from_numpy((rng.standard_normal((k, n)) * 0.02).astype(np.float32))
        c = T([m, n], initial_element=None)
        bv = T.from_numpy(rng.standard_normal(n).astype(np.float32)) if bias else None
        rv = T.from_numpy(rng.standard_normal((m, n)).astype(np.float32)) if res else None
        for _ in range(reps):
            F.matmul(a, b, out=c, bias=bv, residual=rv, activation=act)
        names.append(f"matmul {m}x{n}x{k}" + (" + bias" if bias else "") + (" + residual" if res else "") +
                     (" + GELU" if act else ""))
        del a, b, c, bv, rv
    # a few rows against a wide operand: the streaming kernel of 16 rows, and the token projection of 64 rows
    # with the operands exchanged
    for m, n, k, stored in ((16, 8192, 8192, "kn"), (16, 50257, 768, "nk"), (64, 50257, 768, "nk")):
        a = T.from_numpy(rng.standard_normal((m, k)).astype(np.float32))
        w = T.from_numpy((rng.standard_normal((k, n) if stored == "kn" else (n, k)) * 0.02).astype(np.float32))
        c = T([m, n], initial_element=None)
        for _ in range(reps):
            F.matmul(a, w if stored == "kn" else F.t(w), out=c)
        names.append(f"matmul {m}x{n}x{k}, few rows" + (", right operand stored (n, k)" if stored == "nk" else ""))
        del a, w, c
    W.lib.synchronize()
    print(json.dumps({"probe_matrix_cores": ["attention (8,12,1024,64) full", "attention causal",
                                             "attention backward causal (D, then dQ / dK / dV)"] + names,
                      "launches_each": reps}))


def size_probe(W, reps: int = 6):
    """The launch sequence behind profiles/short_kernel_fit.txt: four kernels of the path (plain copy,
    row-broadcast add, row sum as one node, row softmax) at six sizes from 32 MB to 1 GB moved per launch,
    `reps` launches each on a ring of buffer sets larger than the Infinity Cache.  Their durations under
    `rocprofv3 --kernel-trace`, fitted as t = t0 + bytes / rate, separate the fixed cost of a launch (ramp
    and drain) from the rate the kernel streams at."""
    F = W.functional
    T = W.HIPTensor
    rng = np.random.Generator(np.random.PCG64(6))
    cases = []
    for mb in SIZE_PROBE_MB:
        moved = mb << 20
        n = moved // 8                      # elements of a kernel that reads and writes each once
        count = max(2, -(-(768 << 20) // moved) + 1)
        src = T.from_numpy(rng.standard_normal(1 << 22).astype(np.float32))

        def fresh(shape):
            t = T(list(shape), initial_element=None)
            flat = F.reshape(t, -1)
            for lo in range(0, flat.shape[0], 1 << 22):  # fill from the 16 MB sample
                hi = min(lo + (1 << 22), flat.shape[0])
                F.move_(flat.view((lo, hi)), src.view((0, hi - lo)))
            return t

        ring = [(fresh([n]), T([n], initial_element=None)) for _ in range(count)]
        for i in range(reps):
            F.move_(ring[i % count][1], ring[i % count][0])
        cases.append(("copy", moved, n))
        row = fresh([1, 8192]).view((":broadcast", n // 8192), True)
        for i in range(reps):
            F.add_(F.reshape(ring[i % count][0], n // 8192, 8192), row)
        cases.append(("row-broadcast add, rows of 8192", moved, n))
        for i in range(reps):
            F.softmax_fused(F.reshape(ring[i % count][0], n // 1024, 1024), out=F.reshape(ring[i % count][1], n // 1024, 1024))
        cases.append(("row softmax, rows of 1024", moved, n))
        del ring, row
        n4 = moved // 4                     # the row sum reads every element once
        ring = [(fresh([n4 // 4096, 4096]), T([n4 // 4096, 1])) for _ in range(count)]
        for i in range(reps):
            F.sum(ring[i % count][0], axis=1, out=ring[i % count][1], keepdims=True)
        cases.append(("row sum, rows of 4096", moved, n4))
        del ring
        W.lib.synchronize()
    print(json.dumps({"probe_sizes": [{"kernel": k, "bytes": b, "elements": e} for k, b, e in cases],
                      "launches_each": reps}))


SIZE_PROBE_MB = (32, 64, 128, 256, 512, 1024)


def size_fit(trace_csv: str, reps: int = 6) -> str:
    """The table of profiles/short_kernel_fit.txt from the kernel trace (csv) of a `--probe-sizes` run: per kernel
    the median of the last `reps` - 1 launches at each size, the least-squares line t = t0 + bytes / rate through
    the six sizes, and what that line says of a launch that moves 128 MB (2^24 elements read and written)."""
    import csv
    with open(trace_csv, newline="") as f:
        launches = sorted(csv.DictReader(f), key=lambda r: int(r["Start_Timestamp"]))
    runs = []  # consecutive launches of one kernel at one grid: [name, durations in us]
    for r in launches:
        key = (r["Kernel_Name"], r["Grid_Size_X"])
        us = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
        if runs and runs[-1][0] == key:
            runs[-1][1].append(us)
        else:
            runs.append([key, [us]])
    # per size, in launch order: fills and `reps` copies (ew_flat<OpMove>) end where the broadcast row is written
    # (ew_rows<OpMove>); then `reps` row-broadcast adds, `reps` softmaxes, fills, `reps` row sums
    picked = {"copy": [], "row-broadcast add, rows of 8192": [], "row softmax, rows of 1024": [],
              "row sum, rows of 4096": []}
    for i, (key, times) in enumerate(runs):
        name = key[0]
        if "ew_rows<wf2::OpMove" in name and i > 0:
            picked["copy"].append(runs[i - 1][1][-reps:])
        elif "ew_rows<wf2::OpAdd" in name and len(times) == reps:
            picked["row-broadcast add, rows of 8192"].append(times)
        elif "softmax_rows" in name and len(times) == reps:
            picked["row softmax, rows of 1024"].append(times)
        elif "reduce_rows" in name and len(times) == reps:
            picked["row sum, rows of 4096"].append(times)
    lines = []
    for kernel, per_size in picked.items():
        if len(per_size) != len(SIZE_PROBE_MB):
            raise SystemExit(f"bench.py --fit-sizes: {len(per_size)} runs of '{kernel}' in the trace, "
                             f"{len(SIZE_PROBE_MB)} expected")
        x = np.array([mb * float(1 << 20) for mb in SIZE_PROBE_MB])
        t = np.array([float(np.median(times[1:])) for times in per_size])
        slope, t0 = np.polyfit(x, t, 1)           # us per byte, us
        rate = 1.0 / slope / 1e6                  # TB/s
        lines.append(f"{kernel}: t = {t0:.2f} us + bytes / {rate:.2f} TB/s  ({rate / 8.0 * 100:.1f} % of 8 TB/s)")
        for mb, got in zip(SIZE_PROBE_MB, t):
            fit = t0 + mb * float(1 << 20) * slope
            frac = mb * float(1 << 20) / got / 1e6 / 8.0 * 100
            lines.append(f"    {mb:5d} MB  measured {got:8.2f} us ({frac:4.1f} %)   line {fit:8.2f} us   "
                         f"fixed share {t0 / got * 100:4.1f} %")
    return "\n".join(lines)


def row_table(W, reps: int = 10, warm: int = 3, replay: bool = True):
    """One line per kernel of the path at the shape its configuration names:
    average launch time from an event pair on the library's stream, the
    algorithmic bytes (or flop) of one call, and the fraction of the roofline
    that bounds it.  Each call of a row works on another buffer set of a ring
    of at least 1 GiB, so operands are cold with respect to the 256 MB
    Infinity Cache.  `ms` is per call inside a replayed HIP graph of `reps`
    calls after about 15 ms of the same load (the sustained rate), `eager_ms`
    the first `reps` calls issued one by one from this process (host time
    between launches and the clock ramp included).  The rows go through the same host functions a model
    uses (the time of a row that is several nodes is the sum of its launches)."""
    F = W.functional
    T = W.HIPTensor
    rng = np.random.Generator(np.random.PCG64(6))
    rows = {}

    def ring_of(make, nbytes):
        count = max(2, min(16, -(-(1 << 30) // max(nbytes, 1))))
        return [make() for _ in range(count)]

    def uniform(shape, lo, hi):
        return T.from_numpy(rng.uniform(lo, hi, size=shape).astype(np.float32))

    def normal(shape, scale=1.0):
        return T.from_numpy((rng.standard_normal(shape) * scale).astype(np.float32))

    def clone(t):
        return F.copy(t)

    def measure(label, ring, call, work, bound="hbm", note=None):
        for i in range(warm):
            call(ring[i % len(ring)])
        a, b = W.lib.Event(), W.lib.Event()
        a.record()
        for i in range(reps):
            call(ring[(warm + i) % len(ring)])
        b.record()
        eager_ms = a.elapsed_ms(b) / reps
        ms = eager_ms
        if replay:
            # the same `reps` calls recorded once and replayed as one HIP graph: the launch
            # times without the host work between them (Python here, Lisp in the product)
            W.lib.synchronize()
            with W.lib.Graph() as g:
                for i in range(reps):  # results are dropped: the recording keeps their blocks
                    call(ring[i % len(ring)])
            # the core clock dips for some milliseconds when a heavy load starts and then
            # settles: replay about 15 ms of work before the timed replays
            for _ in range(max(1, min(60, int(15.0 / max(reps * eager_ms, 1e-3)) + 1))):
                g.launch()
            a.record()
            for _ in range(3):
                g.launch()
            b.record()
            graph_ms = a.elapsed_ms(b) / (3 * reps)
            # the same calls as stream launches while the GPU is still under that load: a
            # graph separates its kernel nodes by a dependency that costs 1-2 us per node,
            # a stream hides it behind the running kernel when the host keeps ahead
            a.record()
            for i in range(reps):
                call(ring[i % len(ring)])
            b.record()
            hot_ms = a.elapsed_ms(b) / reps
            ms, how = (graph_ms, "graph") if graph_ms <= hot_ms else (hot_ms, "stream")
            g.destroy()
        if bound == "hbm":
            rate, peak, unit = work / ms / 1e6, HBM_PEAK_GBS, "GB/s"
        else:
            rate, peak, unit = work / ms / 1e9, FP32_MFMA_PEAK_TFLOPS, "TFLOP/s"
        rows[label] = {"ms": round(ms, 5), "eager_ms": round(eager_ms, 5), "achieved": round(rate, 1),
                       "unit": unit, "frac": round(rate / peak, 4), "bound": bound}
        if replay:
            rows[label].update(graph_ms=round(graph_ms, 5), stream_ms=round(hot_ms, 5), timed_as=how)
        if note:
            rows[label]["note"] = note
        ring.clear()

    # contiguous (1024, 1024): the reference's own CPU-sized case; 12 MiB per call is
    # launch- and ramp-bound, not bandwidth-bound
    a0, b0 = normal([1024, 1024]), normal([1024, 1024])
    ring = ring_of(lambda: (clone(a0), clone(b0)), 8 << 20)
    measure("add (1024,1024) in place", ring, lambda s: F.add_(s[0], s[1]), 12 << 20)

    # strided / broadcast views on (4096, 8192)
    R, Cn = 4096, 8192
    a0, b0 = normal([R, Cn]), normal([1, Cn])
    ring = ring_of(lambda: clone(a0), 4 * R * Cn)
    yb = b0.view((":broadcast", R), True)
    measure("A(4096,8192) += B(1,8192) row broadcast", ring, lambda s: F.add_(s, yb), 8 * R * Cn + 4 * Cn)
    ring = ring_of(lambda: clone(a0), 4 * R * Cn)
    measure("A[:, 0:8192:2] *= 0.5", ring, lambda s: F.mul_(s.view(True, (0, Cn, 2)), 0.5), 8 * R * Cn // 2,
            note="8 B per element of the slice; the hardware moves every 32-byte sector whole, "
                 "twice these bytes")
    ring = ring_of(lambda: (clone(a0), T([R, Cn // 2], initial_element=None)), 6 * R * Cn)
    measure("copy of A[:, 0:8192:2] into a contiguous tensor", ring,
            lambda s: F.move_(s[1], s[0].view(True, (0, Cn, 2))), 8 * R * Cn // 2,
            note="8 B per element; the reads move every sector whole (2.5x these bytes in all)")
    ring = ring_of(lambda: (clone(a0), T([2048, Cn], initial_element=None)), 4 * R * Cn + 4 * 2048 * Cn)
    measure("C = A[1024:3072] - A[0:2048] (copy node + in-place sub)", ring,
            lambda s: F.sub_(F.move_(s[1], s[0].view((1024, 3072), True)), s[0].view((0, 2048), True)),
            (8 + 12) * 2048 * Cn, note="two launches: MoveTensorNode 8 B/elem, SubNode 12 B/elem")
    del a0, b0, yb

    # the arithmetic nodes on other element types (16-byte vectors, same traffic per byte)
    for dtype, count in (("double", N // 2), ("int32", N), ("uint8", 4 * N)):
        host = (rng.standard_normal(count) * 50).astype(getattr(np, {"double": "float64"}.get(dtype, dtype)))
        x0 = T.from_numpy(host, dtype=dtype)
        del host
        ring = ring_of(lambda: (clone(x0), clone(x0)), 2 * 4 * N)
        measure(f"x += y, :{dtype}, 256 MiB per tensor", ring, lambda s: F.add_(s[0], s[1]), 12 * N)
        del x0
    # the same on a sliced view of an 8-bit tensor: rows that start and end off every 16-byte boundary
    rows8, wide8 = 16384, 16448
    x0 = T.from_numpy(rng.integers(0, 100, (rows8, wide8)).astype(np.uint8), dtype="uint8")
    ring = ring_of(lambda: (clone(x0), clone(x0)), 2 * rows8 * wide8)
    measure("x += y on the window [:, 3:16387] of :uint8 (16384,16448) tensors", ring,
            lambda s: F.add_(s[0].view(True, (3, 16387)), s[1].view(True, (5, 16389))), 3 * rows8 * 16384)
    del x0

    # transposing copy through LDS tiles
    a0 = normal([SIDE, SIDE])
    ring = ring_of(lambda: (clone(a0), T([SIDE, SIDE], initial_element=None)), 8 * N)
    measure("transposing copy (8192,8192)", ring, lambda s: F.move_(s[1], s[0].permute(1, 0)), 8 * N)
    del a0

    # the plain copy: what a kernel with one read and one write stream can reach here
    x0 = normal([N])
    ring = ring_of(lambda: (clone(x0), T([N], initial_element=None)), 8 * N)
    measure("copy 2^26 (one read stream, one write stream: the practical ceiling of the unary rows)", ring,
            lambda s: F.move_(s[1], s[0]), 8 * N)
    del x0

    # unary functions on 2^26 elements in the ranges of the configuration
    for label, fn, lo, hi in (("exp", F.exp, -10.0, 10.0), ("tanh", F.tanh, -10.0, 10.0),
                              ("sin", F.sin, -100.0, 100.0), ("loge", F.loge, 1e-3, 1e3)):
        x0 = uniform([N], lo, hi)
        ring = ring_of(lambda: (clone(x0), T([N], initial_element=None)), 8 * N)
        measure(f"{label} 2^26 in [{lo:g}, {hi:g}]", ring, lambda s, fn=fn: fn(s[0], out=s[1]), 8 * N)
        del x0

    # reductions and softmax
    R, Cn = 8192, 4096
    x0 = normal([R, Cn])
    ring = ring_of(lambda: (clone(x0), T([R, 1])), 4 * R * Cn)
    measure("row sum (8192,4096), !sum as one node", ring,
            lambda s: F.sum(s[0], axis=1, out=s[1], keepdims=True), 4 * R * Cn + 4 * R,
            note="HIP-Sum-Node: out overwritten, no zero fill")
    ring = ring_of(lambda: (clone(x0), T([R, 1])), 4 * R * Cn)
    measure("row sum (8192,4096), node for node", ring,
            lambda s: F.sum_composed(s[0], axis=1, out=s[1], keepdims=True), 4 * R * Cn + 12 * R,
            note="the reference's composition: zero fill of out (MulNode by 0) + AddNode into the stride-0 view")
    ring = ring_of(lambda: (clone(x0), T([1, 1])), 4 * R * Cn)
    measure("full sum (8192,4096), !sum as one node", ring, lambda s: F.sum(s[0], axis=True, out=s[1], keepdims=True),
            4 * R * Cn, note="two launches: partial sums per workgroup, then their sum")
    del x0
    R, Cn = 32768, 1024
    x0 = normal([R, Cn], 3.0)
    ring = ring_of(lambda: (clone(x0), T([R, Cn], initial_element=None)), 8 * R * Cn)
    measure("copy (32768,1024): 268 MB in all, the practical ceiling of the rows that move as much", ring,
            lambda s: F.move_(s[1], s[0]), 8 * R * Cn)
    ring = ring_of(lambda: (clone(x0), T([R, Cn], initial_element=None)), 8 * R * Cn)
    measure("row softmax (32768,1024), one kernel", ring, lambda s: F.softmax_fused(s[0], out=s[1]), 8 * R * Cn)
    ring = ring_of(lambda: clone(x0), 4 * R * Cn)
    measure("row softmax (32768,1024), node for node (!softmax)", ring, lambda s: F.softmax(s), 8 * R * Cn,
            note="mean, sub, exp, sum, div as separate nodes with their temporaries; "
                 "rate quoted on the 8 B/elem of the fused form")
    del x0

    # the callers either side of the path: compare / where, row max and argmax, fused GELU and
    # LayerNorm, optimiser steps
    x0 = normal([N])
    ring = ring_of(lambda: (clone(x0), clone(x0), T([N], initial_element=None)), 12 * N)
    measure("compare x < y -> 1 / 0, 2^26", ring, lambda s: F.compare(s[0], s[1], "<", out=s[2]), 12 * N)
    ring = ring_of(lambda: (clone(x0), T([N], initial_element=None)), 8 * N)
    measure("where x > 0.5 -> 1 / 0 (scalar), 2^26", ring, lambda s: F.where(s[0], ">", 0.5, out=s[1]), 8 * N)
    ring = ring_of(lambda: (clone(x0), T([N], initial_element=None)), 8 * N)
    measure("GELU, one kernel, 2^26", ring, lambda s: F.gelu_fused(s[0], out=s[1]), 8 * N)
    del x0
    R, Cn = 65536, 1024
    x0 = normal([R, Cn])
    ring = ring_of(lambda: clone(x0), 4 * R * Cn)
    measure("row max (65536,1024)", ring, lambda s: F.max(s, axis=1), 4 * R * Cn + 4 * R)
    ring = ring_of(lambda: clone(x0), 4 * R * Cn)
    measure("row argmax (65536,1024)", ring, lambda s: F.argmax(s, axis=1), 4 * R * Cn + 4 * R)
    g0, b0 = normal([Cn]), normal([Cn])
    ring = ring_of(lambda: (clone(x0), T([R, Cn], initial_element=None)), 8 * R * Cn)
    measure("LayerNorm (65536,1024), one kernel", ring, lambda s: F.layer_norm_fused(s[0], g0, b0, out=s[1]),
            8 * R * Cn)
    del x0, g0, b0
    # rows beyond 8192 columns: a workgroup of 1024 threads per row, forward and backward
    R, Cn = 4096, 16384
    x0, g0, b0 = normal([R, Cn]), normal([Cn]), normal([Cn])
    ring = ring_of(lambda: (clone(x0), T([R, Cn], initial_element=None)), 8 * R * Cn)
    measure("LayerNorm (4096,16384), one kernel", ring, lambda s: F.layer_norm_fused(s[0], g0, b0, out=s[1]),
            8 * R * Cn)
    dg0, db0 = T([Cn], initial_element=None), T([Cn], initial_element=None)
    ring = ring_of(lambda: (clone(x0), clone(x0), T([R, Cn], initial_element=None)), 12 * R * Cn)
    measure("LayerNorm backward (4096,16384): dx, dgamma, dbeta (three launches)", ring,
            lambda s: W.nodes.forward("HIP-LayerNorm-Node-backward", s[0], g0, s[1], s[2], dg0, db0, 1e-5),
            12 * R * Cn)
    del x0, g0, b0, dg0, db0
    p0 = normal([N])
    for name, make, per in (("Adam", lambda p: W.optimizers.Adam(p, lr=1e-3), 28), ("SGD", lambda p: W.optimizers.SGD(p, lr=1e-3), 16)):
        ring = ring_of(lambda: (make(clone(p0)), clone(p0)), per * N)
        measure(f"{name} step, 2^26 parameters, one kernel", ring, lambda s: s[0].step(s[1]), per * N)
    del p0

    # the backward kernels of the fused layers
    x0 = normal([N])
    ring = ring_of(lambda: (clone(x0), clone(x0)), 8 * N)
    measure("GELU backward (dout <- dout gelu'(x)), 2^26", ring,
            lambda s: F.activation_backward("gelu", s[0], s[1], in_place=True), 12 * N)
    del x0
    R, Cn = 32768, 1024
    x0 = normal([R, Cn], 3.0)
    y0 = F.softmax_fused(x0)
    ring = ring_of(lambda: (clone(y0), clone(x0)), 8 * R * Cn)
    measure("softmax backward (32768,1024), one kernel", ring, lambda s: F.softmax_backward(s[0], s[1], in_place=True),
            12 * R * Cn)
    del x0, y0
    R, Cn = 65536, 1024
    x0, g0 = normal([R, Cn]), normal([Cn])
    dg, db = T([Cn], initial_element=None), T([Cn], initial_element=None)
    ring = ring_of(lambda: (clone(x0), clone(x0), T([R, Cn], initial_element=None)), 12 * R * Cn)
    measure("LayerNorm backward (65536,1024): dx, dgamma, dbeta (three launches)", ring,
            lambda s: W.nodes.forward("HIP-LayerNorm-Node-backward", s[0], g0, s[1], s[2], dg, db, 1e-5), 12 * R * Cn)
    del x0, g0, dg, db
    # Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:82-126), forward and backward
    R, Cn = 32768, 1024
    x0 = normal([R, Cn], 3.0)
    t0 = F.softmax_fused(normal([R, Cn]))
    ring = ring_of(lambda: (clone(x0), clone(t0), T([R, Cn], initial_element=None), T([R, Cn], initial_element=None)),
                   16 * R * Cn)
    measure("softmax cross entropy (32768,1024), one kernel: z and the loss per element", ring,
            lambda s: W.nodes.forward("HIP-Softmax-Cross-Entropy-Node", s[0], s[1], s[2], s[3], 1e-7), 16 * R * Cn)
    ring = ring_of(lambda: (clone(x0), clone(t0)), 8 * R * Cn)
    measure("softmax cross entropy (32768,1024), node for node", ring,
            lambda s: W.nn.softmax_cross_entropy(s[0], s[1], avoid_overflow=True, reduction=True), 16 * R * Cn,
            note="!softmax (mean, sub, exp, sum, div), then add, loge, mul, mul as separate nodes; "
                 "rate quoted on the 16 B/elem of the fused form")
    ring = ring_of(lambda: (clone(x0), clone(t0), clone(t0)), 12 * R * Cn)
    measure("softmax cross entropy backward (32768,1024), one kernel", ring,
            lambda s: W.nn.softmax_cross_entropy_backward_fused(s[0], s[1], s[2], in_place=True), 16 * R * Cn)
    ring = ring_of(lambda: (clone(x0), clone(t0), clone(t0)), 12 * R * Cn)
    measure("softmax cross entropy backward (32768,1024), node for node", ring,
            lambda s: W.nn.softmax_cross_entropy_backward(s[0], s[1], s[2]), 16 * R * Cn,
            note="sub, mul, div as separate nodes; rate quoted on the 16 B/elem of the fused form")
    del x0, t0
    # unfold of a (32, 64, 56, 56) image for a 3 x 3 convolution with padding 1 (source/nn/im2col.lisp:51-95),
    # and the two nodes it is composed from and differentiated through
    Nb, Cc, Hh, Kk = 32, 64, 56, 3
    img = normal([Nb, Cc, Hh, Hh])
    ncol, nim = Nb * Cc * Kk * Kk * Hh * Hh, Nb * Cc * Hh * Hh
    ring = ring_of(lambda: T([Nb * Hh * Hh, Cc * Kk * Kk], initial_element=None), 4 * ncol)
    measure("unfold (32,64,56,56) 3x3 pad 1, one kernel: the (N h w) x (C kh kw) matrix", ring,
            lambda s: W.nodes.forward("HIP-Unfold-Node", img, s, (Kk, Kk), (1, 1), (1, 1)), 4 * (ncol + nim))
    measure("unfold (32,64,56,56) 3x3 pad 1, node for node", [None],
            lambda s: F.unfold_composed(img, (1, 1), (Kk, Kk), (1, 1), (1, 1)), 4 * (ncol + nim),
            note="padding copy, zero fill of col, Im2ColNode, permuting copy; rate quoted on the bytes of the one-kernel form")
    padded = normal([Nb, Cc, Hh + 2, Hh + 2])
    ring = ring_of(lambda: T([Nb, Cc, Kk, Kk, Hh, Hh], initial_element=None), 4 * ncol)
    measure("Im2ColNode (32,64,58,58) -> (32,64,3,3,56,56), no padding argument", ring,
            lambda s: W.nodes.forward("Im2ColNode", padded, s, (1, 1), (0, 0), (1, 1)), 4 * (ncol + nim))
    ring = ring_of(lambda: T([Nb, Cc, Kk, Kk, Hh, Hh], initial_element=None), 4 * ncol)
    measure("Im2ColNode, padding 1: the walk leaves the last row and column of every plane untouched", ring,
            lambda s: W.nodes.forward("Im2ColNode", padded, s, (1, 1), (1, 1), (1, 1)), 4 * (ncol + nim),
            note="the old values of the elements the walk leaves out are read first (whole lines, four of every seven of col) "
                 "and written back inside whole 16-byte stores; rate quoted on the bytes of the walk alone")
    back = T([Nb, Cc, Hh + 2, Hh + 2], initial_element=None)
    ring = ring_of(lambda: normal([Nb, Cc, Kk, Kk, Hh, Hh]), 4 * ncol)
    measure("Col2ImNode (32,64,3,3,56,56) -> (32,64,58,58)", ring,
            lambda s: W.nodes.forward("Col2ImNode", s, back, (1, 1), (1, 1), (1, 1)), 4 * (ncol + nim))
    del img, padded, back
    # the windows of a 2 x 2 pooling layer on (32,64,112,112): rows of four elements
    R, Cn = 32 * 64 * 56 * 56, 4
    w0 = normal([R, Cn])
    ring = ring_of(lambda: clone(w0), 4 * R * Cn)
    measure("row max (6422528,4): MaxPool2D's !max over its windows", ring, lambda s: F.max(s, axis=1), 4 * R * Cn + 4 * R)
    ring = ring_of(lambda: clone(w0), 4 * R * Cn)
    measure("row mean (6422528,4): AvgPool2D's !mean over its windows", ring, lambda s: F.mean(s, axis=1), 4 * R * Cn + 4 * R)
    top = F.max(w0, axis=1, keepdims=True)
    ring = ring_of(lambda: (clone(w0), T([R, Cn], initial_element=None)), 8 * R * Cn)
    measure("compare (6422528,4) = its row maxima (broadcast): the mask of MaxValue-Node's backward", ring,
            lambda s: F.compare(s[0], top, "=", out=s[1]), 8 * R * Cn + 4 * R)
    del w0, top

    # products on fp32 MFMA, random data
    for m, n, k in ((8192, 8192, 8192), (4096, 4096, 4096), (8192, 2304, 768), (8192, 3072, 768),
                    (8192, 768, 3072), (8192, 768, 768)):
        a0, b0 = normal([m, k]), normal([k, n])
        ring = ring_of(lambda: (clone(a0), clone(b0), T([m, n], initial_element=None)), 4 * (m * k + k * n + m * n))
        measure(f"matmul {m}x{n}x{k}", ring, lambda s: F.matmul(s[0], s[1], out=s[2]), 2.0 * m * n * k,
                bound="mfma")
        del a0, b0
    # the layouts of LinearLayer and of its backward (source/nn/regression.lisp:13-17):
    # x . W^T with W stored (out, in); dW = dY^T . x over a long K with few output tiles
    m, n, k = 8192, 3072, 768
    a0, w0 = normal([m, k]), normal([n, k])
    ring = ring_of(lambda: (clone(a0), clone(w0), T([m, n], initial_element=None)), 4 * (m * k + k * n + m * n))
    measure(f"matmul {m}x{n}x{k}, right operand stored ({n},{k}) (!t)", ring,
            lambda s: F.matmul(s[0], F.t(s[1]), out=s[2]), 2.0 * m * n * k, bound="mfma")
    del a0, w0
    m, n, k = 768, 3072, 8192
    a0, b0 = normal([k, m]), normal([k, n])
    ring = ring_of(lambda: (clone(a0), clone(b0), T([m, n], initial_element=None)), 4 * (m * k + k * n + m * n))
    measure(f"matmul {m}x{n}x{k}, left operand stored ({k},{m}) (!t), split over K", ring,
            lambda s: F.matmul(F.t(s[0]), s[1], out=s[2]), 2.0 * m * n * k, bound="mfma")
    del a0, b0
    # a few rows against a wide operand (a few tokens through a layer): one read of that operand, bound by HBM
    for m, n, k, stored in ((16, 8192, 8192, "kn"), (16, 50257, 768, "nk"), (64, 50257, 768, "nk")):
        a0 = normal([m, k])
        w0 = normal([k, n]) if stored == "kn" else normal([n, k])
        ring = ring_of(lambda: (clone(a0), clone(w0), T([m, n], initial_element=None)), 4 * (m * k + k * n + m * n))
        label = (f"matmul {m}x{n}x{k}, few rows" if stored == "kn" else
                 f"matmul {m}x{n}x{k}, few rows, right operand stored ({n},{k}) (!t): GPT-2's token projection")
        # 2 m flop per 4 bytes of the wide operand: beyond 39 rows (157.3 TFLOP/s / 8 TB/s = 19.7 flop per byte)
        # the matrix cores bound the product, not the one read of the operand
        flop_us = 2.0 * m * n * k / FP32_MFMA_PEAK_TFLOPS / 1e6
        byte_us = 4.0 * (m * k + k * n + m * n) / HBM_PEAK_GBS / 1e3
        measure(label, ring, (lambda s: F.matmul(s[0], s[1], out=s[2])) if stored == "kn" else
                (lambda s: F.matmul(s[0], F.t(s[1]), out=s[2])), 4 * (m * k + k * n + m * n),
                note=(f"at the peaks: {byte_us:.1f} us of HBM traffic, {flop_us:.1f} us of fp32 matrix-core work"
                      + ("; bound by the matrix cores" if flop_us > byte_us else "")))
        if flop_us > byte_us:
            rows[label]["frac_mfma_peak"] = round(flop_us * 1e-3 / rows[label]["ms"], 4)
        del a0, w0
    # class scores: very many rows of ten columns; and one row of 2^24 columns
    for rows_, cols_ in ((1677721, 10), (1, 1 << 24)):
        x0 = normal([rows_, cols_])
        ring = ring_of(lambda: (clone(x0), T([rows_, cols_], initial_element=None)), 8 * rows_ * cols_)
        measure(f"row softmax ({rows_},{cols_}), one kernel" if rows_ > 1 else
                f"row softmax ({rows_},{cols_}): pieces of the row over the grid, one launch", ring,
                lambda s: F.softmax_fused(s[0], out=s[1]), 8 * rows_ * cols_)
        del x0
    B, H, S, hd = 8, 12, 1024, 64
    q0 = normal([B, H, S, hd])
    for causal in (True, False):
        ring = ring_of(lambda: (clone(q0), clone(q0), clone(q0), T([B, H, S, hd], initial_element=None)),
                       16 * B * H * S * hd)
        flop = 4.0 * B * H * S * S * hd * (0.5 if causal else 1.0)
        measure(f"attention (8,12,1024,64) {'causal' if causal else 'full'}", ring,
                lambda s, c=causal: F.attention(s[0], s[1], s[2], out=s[3], causal=c), flop, bound="mfma",
                note="flop of the useful half of the score matrix" if causal else None)
    # the backward of the same attention (two launches: D per query; dQ, dK and dV)
    lse = T([B, H, S], initial_element=None)
    o0 = F.attention(q0, q0, q0, causal=True, lse=lse)
    ring = ring_of(lambda: (clone(q0), clone(q0), clone(q0), clone(q0), T([B, H, S, hd], initial_element=None),
                            T([B, H, S, hd], initial_element=None), T([B, H, S, hd], initial_element=None)),
                   28 * B * H * S * hd)
    measure("attention backward (8,12,1024,64) causal: dQ, dK, dV (two launches)", ring,
            lambda s: F.attention_backward(s[0], s[1], s[2], s[3], causal=True, dq=s[4], dk=s[5], dv=s[6], out=o0, lse=lse),
            10.0 * B * H * S * S * hd * 0.5, bound="mfma",
            note="flop of the useful half of the five products a backward needs at least (the kernel forms seven)")
    del q0, o0, lse
    return rows


def block_forward_ms(W, reps: int = 20, warm: int = 10):
    try:
        gpt2 = importlib.import_module("cl-waffe2_amd.gpt2")
    except ImportError:
        return None
    params = gpt2.make_block_params(seed=5)
    x = gpt2.make_block_input(seed=5)
    dparams = gpt2.to_device(params)
    dx = W.HIPTensor.from_numpy(x)
    mask = gpt2.causal_mask(gpt2.CONFIG["seq"])
    out = {}
    for mode in ("nodes", "fused_matmul_attention", "fused"):
        for _ in range(warm):  # the core clock takes tens of milliseconds of load to settle
            gpt2.block_forward(dx, dparams, mode=mode, mask=mask)
        e0, e1 = W.lib.Event(), W.lib.Event()
        e0.record()
        for _ in range(reps):
            gpt2.block_forward(dx, dparams, mode=mode, mask=mask)
        e1.record()
        out[mode] = e0.elapsed_ms(e1) / reps
        # the same node sequence recorded once and replayed as a HIP graph
        W.lib.synchronize()
        with W.lib.Graph() as g:
            keep = gpt2.block_forward(dx, dparams, mode=mode, mask=mask)
        g.launch()
        e0, e1 = W.lib.Event(), W.lib.Event()
        e0.record()
        for _ in range(reps):
            g.launch()
        e1.record()
        out[mode + "_graph"] = e0.elapsed_ms(e1) / reps
        g.destroy()
        del keep
    # forward keeping what the backward reads, then the backward (every fused node's backward,
    # attention with the probabilities recomputed); stream launches
    dout = W.HIPTensor.from_numpy(np.random.Generator(np.random.PCG64(7)).standard_normal(x.shape).astype(np.float32))

    def train_step():
        saved = {}
        gpt2.block_forward(dx, dparams, mode="fused", saved=saved)
        return gpt2.block_backward(dout, saved, dparams)

    for _ in range(3):
        train_step()
    e0, e1 = W.lib.Event(), W.lib.Event()
    e0.record()
    for _ in range(reps):
        train_step()
    e1.record()
    out["fused_forward_and_backward"] = e0.elapsed_ms(e1) / reps
    # the same training step recorded once and replayed as a HIP graph
    W.lib.synchronize()
    with W.lib.Graph() as g:
        keep = train_step()
    g.launch()
    e0, e1 = W.lib.Event(), W.lib.Event()
    e0.record()
    for _ in range(reps):
        g.launch()
    e1.record()
    out["fused_forward_and_backward_graph"] = e0.elapsed_ms(e1) / reps
    g.destroy()
    del keep
    return out


def cpu_baseline():
    """The same step on one host core over the full 2^26 sample, through the
    reference's compiled C kernels when oracle/_ref is present."""
    from oracle import oracle as O

    O.build()
    use_ref = O.ref() is not None
    rng = np.random.Generator(np.random.PCG64(6))
    x = rng.standard_normal(N).astype(np.float32)
    y = rng.standard_normal(N).astype(np.float32)
    o = np.zeros(N, np.float32)
    r = np.zeros(SIDE, np.float32)
    t0 = time.perf_counter()
    reps = 0
    while reps < 2 or time.perf_counter() - t0 < 10.0:
        O.binary_1d("add", N, x, 1, y, 1, use_ref=use_ref)
        O.binary_1d("mul", N, x, 1, y, 1, use_ref=use_ref)
        O.unary_1d("exp", N, y, 1, o, 1, use_ref=use_ref)
        for row in range(SIDE):  # the reference's schedule: one incx = 0 call per row
            O.binary_1d("add", SIDE, r, 0, y, 1, offx=row, offy=row * SIDE, use_ref=use_ref)
        reps += 1
        if time.perf_counter() - t0 > 30.0:
            break
    dt = (time.perf_counter() - t0) / reps
    gbs = sum(BYTES.values()) / dt / 1e9
    block = cpu_block_forward_ms()
    return {
        "block_fwd_ms": block,
        "value": round(gbs, 3),
        "unit": "GB/s",
        "cores": 1,
        "kind": "reference" if use_ref else "port",
        "sample": f"{reps} full steps at 2^26 elements (add, mul, exp, 8192 row sums), "
                  f"{dt:.2f} s each, 1 thread as in the reference (lparallel off, *num-cores* 1), "
                  f"SLEEF {'from libtorch_cpu.so' if O.sleef_available() else 'absent: libm'}",
    }


def cpu_block_forward_ms():
    """The block forward in binary32 on the host (numpy + its BLAS): the
    reference-equivalent CPU path restated, timed on one thread (what
    cl-waffe2's CPU backend uses for everything but the gemm) and on all cores
    given to this process.  A baseline to read the GPU number against, nothing
    more."""
    try:
        from threadpoolctl import threadpool_limits
    except ImportError:
        return None
    from oracle import gpt2_block_ref as ref
    gpt2 = importlib.import_module("cl-waffe2_amd.gpt2")
    params = gpt2.make_block_params(seed=5)
    x = gpt2.make_block_input(seed=5)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, 16)
    out = {"shape": "B 8, T 1024, D 768, 12 x 64, fp32, numpy", "cores_all": cores}
    for label, threads in (("threads_all", cores), ("threads_1", 1)):
        with threadpool_limits(limits=threads):
            ref.block_forward(x[:1], params, 12, dtype=np.float32)  # warm the BLAS
            t0 = time.perf_counter()
            ref.block_forward(x, params, 12, dtype=np.float32)
            out[label] = round((time.perf_counter() - t0) * 1e3, 1)
    return out


# Short names for the rows of the BASELINE configurations and of the kernels that bound the block, for
# a compact last key of the JSON line: whoever keeps only the end of the line still sees every
# configuration.  name -> the start of the row's label in `rows`.
COMPACT_ROWS = (
    ("cfg1_add", "add (1024,1024)"), ("cfg2_bcast_add", "A(4096,8192) += B"), ("cfg2_stride2_mul", "A[:, 0:8192:2] *= 0.5"),
    ("cfg2_slice_copy", "copy of A[:, 0:8192:2]"), ("cfg2_offset_sub", "C = A[1024:3072]"),
    ("cfg3_exp", "exp 2^26"), ("cfg3_tanh", "tanh 2^26"), ("cfg3_sin", "sin 2^26"), ("cfg3_log", "loge 2^26"),
    ("cfg4_rowsum", "row sum (8192,4096), !sum as one node"), ("cfg4_fullsum", "full sum (8192,4096)"),
    ("cfg4_softmax", "row softmax (32768,1024), one kernel"), ("copy_536MB", "copy 2^26"), ("copy_268MB", "copy (32768,1024)"),
    ("layernorm", "LayerNorm (65536,1024)"), ("layernorm_bwd", "LayerNorm backward (65536"), ("ln_16384", "LayerNorm (4096,16384)"),
    ("ln_16384_bwd", "LayerNorm backward (4096,16384)"), ("u8_window_add", "x += y on the window"), ("adam", "Adam step"),
    ("transpose", "transposing copy"), ("unfold", "unfold (32,64,56,56) 3x3 pad 1, one kernel"),
    ("im2col", "Im2ColNode (32,64,58,58)"), ("im2col_pad", "Im2ColNode, padding 1"), ("col2im", "Col2ImNode"),
    ("mm_8192x2304x768", "matmul 8192x2304x768"), ("mm_8192x3072x768", "matmul 8192x3072x768"),
    ("mm_8192x768x3072", "matmul 8192x768x3072"), ("mm_8192x768x768", "matmul 8192x768x768"), ("mm_4096^3", "matmul 4096x4096x4096"),
    ("mm_dW_splitK", "matmul 768x3072x8192"), ("mm_16x50257x768", "matmul 16x50257x768"), ("mm_64x50257x768", "matmul 64x50257x768"),
    ("attn_causal", "attention (8,12,1024,64) causal"), ("attn_full", "attention (8,12,1024,64) full"),
    ("attn_bwd_causal", "attention backward"),
)


def compact_rows(rows, block):
    """{short name: [ms, fraction of the bounding peak]} for COMPACT_ROWS, plus the fused block forward."""
    out = {}
    for name, start in COMPACT_ROWS:
        for label, row in rows.items():
            if label.startswith(start):
                out[name] = [round(row["ms"], 4), round(row["frac"], 3)]
                break
    if block:
        out["cfg5_block_fused_ms"] = round(block.get("fused_graph", block.get("fused", 0.0)), 4)
        out["cfg5_block_fused_eager_ms"] = round(block.get("fused", 0.0), 4)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-block", action="store_true")
    ap.add_argument("--rows-eager", action="store_true",
                    help="rows: time the eager calls only, no HIP-graph replay (`ms` = `eager_ms`); for kernel traces")
    ap.add_argument("--no-rows", action="store_true",
                    help="skip the table of the other kernels of the path at their configured shapes")
    ap.add_argument("--probe-rows", action="store_true",
                    help="run the launch sequence of the other kernels of the path for rocprofv3 --pmc runs and exit")
    ap.add_argument("--probe-matrix-cores", action="store_true",
                    help="run the launch sequence of the attention kernels and one projection for rocprofv3 --pmc runs and exit")
    ap.add_argument("--probe-sizes", action="store_true",
                    help="run four kernels of the path at six sizes (32 MB ... 1 GB moved) for a rocprofv3 --kernel-trace run and exit")
    ap.add_argument("--fit-sizes", metavar="KERNEL_TRACE_CSV",
                    help="fit t = t0 + bytes / rate to the kernel trace of a --probe-sizes run, print the table and exit (no GPU)")
    ap.add_argument("--probe", action="store_true",
                    help="run the short fixed launch sequence used for rocprofv3 --pmc runs and exit")
    args = ap.parse_args()
    if args.fit_sizes:
        print(size_fit(args.fit_sizes))
        return
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on ONE GPU (no collectives, no sharding); "
                 "--gpus must be 1")

    W = importlib.import_module("cl-waffe2_amd")
    W.lib.init(0)  # raises if libwaffe2-hip.so is missing: there is no CPU fallback
    info = W.lib.device_info()
    if args.probe:
        counter_probe(W)
        return
    if args.probe_rows:
        row_probe(W)
        return
    if args.probe_matrix_cores:
        matrix_core_probe(W)
        return
    if args.probe_sizes:
        size_probe(W)
        return

    step_ms, wall_ms, per_kernel, binary_ms, sustained_ms = gpu_steps(W, args.steps, args.warmup)
    traffic, traffic_source = binary_traffic_bytes()
    total_bytes = sum(BYTES.values())
    value = total_bytes / step_ms / 1e6
    kernels = {k: {"ms": round(v, 5), "GB/s": round(BYTES[k] / v / 1e6, 1),
                   "frac_hbm_peak": round(BYTES[k] / v / 1e6 / HBM_PEAK_GBS, 4)}
               for k, v in per_kernel.items()}
    achieved = BYTES["add"] / binary_ms / 1e6
    result = {
        "metric": "fp32 elem-wise/reduce GB/s (% HBM peak) @2^26 elems; GPT-2 block fwd ms",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_ms, 5),
        "wall_ms_per_step": round(wall_ms, 5),
        "value_sustained": round(total_bytes / sustained_ms / 1e6, 1),
        "ms_per_step_sustained": round(sustained_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "x+=y, x*=y, o=exp(y), row-sum(y) on fp32 (8192,8192)=2^26 elements, N(0,1) seed 6; "
                        "cold-cache ring of 8 buffer sets",
            "elements": N,
            "bytes_per_step": total_bytes,
            "device": info["name"] or info["arch"],
            "arch": info["arch"],
        },
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "kernels": kernels,
        "roofline": {
            "kernel": "ew_flat<OpAdd, ReadDst, NT, wave-contiguous, 4 vectors/thread> (x <- x + y, 2^26 elements)",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "algorithmic_bytes_per_launch": BYTES["add"],
            "avg_launch_ms": round(binary_ms, 5),
        },
    }
    if not args.no_rows:
        replay = not args.rows_eager and not profiler_attached()
        result["rows"] = row_table(W, replay=replay)
        result["rows_timing"] = ("ms = the lower of a HIP-graph replay and of stream launches, both after ~15 ms of the "
                                 "same load; eager_ms = the first calls from an idle GPU" if replay else
                                 "stream launches only (no HIP-graph replay: --rows-eager or a profiler is attached)")
    if not args.no_block:
        blk = block_forward_ms(W)
        if blk is not None:
            flop = 141.7e9
            result["gpt2_block_fwd_ms"] = {k: round(v, 4) for k, v in blk.items()}
            result["gpt2_block_tflops_on_141.7_gflop"] = {
                k: round(flop / v / 1e9, 1) for k, v in blk.items() if "backward" not in k}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    if "rows" in result:  # last, and short
        result["baseline_rows"] = compact_rows(result["rows"], result.get("gpt2_block_fwd_ms"))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
