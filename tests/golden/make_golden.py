#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ from the reference's own C
kernels (cl-waffe2-simd/kernels/cl-waffe2-simd.c) compiled into
oracle/_ref/libwaffe2_simd_ref.so by `make -C oracle ref`.

Run in a container that has the reference checkout; the fixtures are data
(inputs and the outputs the reference kernels produced), small enough to
commit, and are what pins the oracle and the device math where the reference
itself cannot travel.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as O  # noqa: E402

REGIMES = [(1, 1), (1, 0), (2, 1), (1, 3), (2, 2), (3, 0), (0, 1), (0, 0), (0, 2)]
SIZES = [1, 7, 8, 9, 31, 64, 67]
EDGE = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-39, 1.0, -1.0, np.inf, -np.inf, np.nan, 88.72, 88.73,
                 -87.4, -103.9, -104.5, 1e10, -1e10, 3.4e38, 1e6, 1.5e6, 9.01, -9.01, 0.5, 2.0,
                 1e-3, 123456.7, 1e-20, 0.99999994, 1.0000001, 3.1415927, 1.5707964, 6.2831855,
                 102.1, 355.0, 710.0, 1e5, 65536.0, 20.0, -20.0, 0.1], np.float32)
UNARY = {"exp": (-10, 10), "tanh": (-10, 10), "sin": (-100, 100), "cos": (-100, 100),
         "log": (1e-3, 1e3), "sqrt": (0, 1e3), "abs": (-5, 5)}


def main():
    assert O.ref() is not None, "oracle/_ref/libwaffe2_simd_ref.so is missing: run `make -C oracle ref`"
    rng = np.random.Generator(np.random.PCG64(2024))
    out = {}
    # x <- x op y for every (incx, incy) regime incl. incx == 0 accumulation
    for op in ("add", "sub", "mul", "div"):
        for n in SIZES:
            for incx, incy in REGIMES:
                size = max(1, n) * 3 + 1
                x = rng.standard_normal(size).astype(np.float32)
                y = (rng.standard_normal(size) + (1.5 if op in ("mul", "div") and incx == 0 else 0)).astype(np.float32)
                if op in ("mul", "div") and incx == 0:
                    y = rng.uniform(0.9, 1.1, size).astype(np.float32)
                res = x.copy()
                O.binary_1d(op, n, res, incx, y, incy, use_ref=True)
                key = f"bin_{op}_{n}_{incx}_{incy}"
                out[key + "_x"], out[key + "_y"], out[key + "_out"] = x, y, res
    # out <- f(x): the ranges of the transcendental benchmark configuration (n = 2048 + 5 so that the libm tail is hit),
    # edge values, strided in/out, broadcast source
    for op, (lo, hi) in UNARY.items():
        x = rng.uniform(lo, hi, 2053).astype(np.float32)
        res = np.zeros_like(x)
        O.unary_1d(op, x.size, x, 1, res, 1, use_ref=True)
        out[f"un_{op}_range_x"], out[f"un_{op}_range_out"] = x, res
        res = np.zeros(EDGE.size, np.float32)
        with np.errstate(all="ignore"):
            O.unary_1d(op, EDGE.size, EDGE, 1, res, 1, use_ref=True)
        out[f"un_{op}_edge_out"] = res
        for n, incx, inco in [(13, 2, 1), (16, 1, 3), (9, 0, 1)]:
            res = np.full(64, 7.0, np.float32)
            O.unary_1d(op, n, x, incx, res, inco, use_ref=True)
            out[f"un_{op}_{n}_{incx}_{inco}_out"] = res
    out["edge_x"] = EDGE
    for p in (2.0, 3.0, 0.5, 2.5, -1.0):
        x = rng.uniform(0.01, 30.0, 1029).astype(np.float32)
        if p == int(p):
            x[::2] *= -1
        res = np.zeros_like(x)
        O.pow_1d(x.size, x, 1, p, res, 1, use_ref=True)
        out[f"pow_{p}_x"], out[f"pow_{p}_out"] = x, res
    for n, inc in [(1, 1), (5, 1), (8, 1), (67, 1), (40, 3)]:
        x = rng.standard_normal(n * inc + 1).astype(np.float32)
        out[f"max_{n}_{inc}_x"] = x
        out[f"max_{n}_{inc}_out"] = np.float32(O.maxmin_1d("max", n, x, inc, use_ref=True))
        out[f"min_{n}_{inc}_out"] = np.float32(O.maxmin_1d("min", n, x, inc, use_ref=True))
    np.savez_compressed(os.path.join(HERE, "simd_kernels.npz"), **out)
    manifest = {
        "source": "cl-waffe2-simd/kernels/cl-waffe2-simd.c compiled by oracle/Makefile target `ref`",
        "compiler": "ROCm clang -O3 -mavx2 -mfma -flax-vector-conversions=all",
        "sleef": "3.8.0 symbols exported by PyTorch's libtorch_cpu.so (Sleef_*f8_u10avx2, sqrt u05)",
        "seed": "PCG64(2024)",
        "arrays": len(out),
        "regimes": REGIMES,
        "sizes": SIZES,
    }
    with open(os.path.join(HERE, "simd_kernels.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "simd_kernels.npz")), "bytes")


CMP_REGIMES = [(1, 1, 1), (1, 0, 1), (2, 1, 1), (1, 3, 2), (2, 2, 3), (0, 1, 1), (1, 1, 0), (3, 0, 0)]
CMP_EDGE = np.array([0.0, -0.0, 1.0, -1.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, 0.5, 2.0,
                     -2.0, 1.0000001, 0.99999994, 7.0], np.float32)


def compare_goldens():
    """out <- (x OP y) ? then : else for the five predicates, tensor and scalar
    right-hand sides (waffe2_s{eq,lt,le,gt,ge}[_scal]), every stride regime
    incl. a stride-0 `out`, and a table of special values against each other."""
    rng = np.random.Generator(np.random.PCG64(2025))
    out = {}
    for op in O.CMP_OPS:
        for n in (1, 7, 8, 9, 31, 67):
            for incx, incy, inco in CMP_REGIMES:
                size = n * 3 + 1
                # small integers so that equality happens
                x = rng.integers(-3, 4, size).astype(np.float32)
                y = rng.integers(-3, 4, size).astype(np.float32)
                res = np.full(size, 9.0, np.float32)
                O.cmp_1d(op, n, x, incx, y, incy, res, inco, 2.5, -1.5, use_ref=True)
                key = f"cmp_{op}_{n}_{incx}_{incy}_{inco}"
                out[key + "_x"], out[key + "_y"], out[key + "_out"] = x, y, res
                res = np.full(size, 9.0, np.float32)
                O.cmp_scal_1d(op, n, x, incx, res, inco, 1.0, 2.5, -1.5, use_ref=True)
                out[key + "_scal_out"] = res
        # every special value against every other one
        xs = np.repeat(CMP_EDGE, CMP_EDGE.size)
        ys = np.tile(CMP_EDGE, CMP_EDGE.size)
        res = np.zeros(xs.size, np.float32)
        O.cmp_1d(op, xs.size, xs, 1, ys, 1, res, 1, 1.0, 0.0, use_ref=True)
        out[f"cmp_{op}_edge_out"] = res
    out["cmp_edge"] = CMP_EDGE
    np.savez_compressed(os.path.join(HERE, "compare_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "compare_kernels.npz")), "bytes")


UNARY_MORE = {"tan": (-100, 100), "asin": (-1, 1), "acos": (-1, 1), "atan": (-100, 100), "sinh": (-10, 10),
              "cosh": (-10, 10), "log2": (1e-3, 1e3), "log10": (1e-3, 1e3), "log1p": (-0.99, 100)}


def unary_more_goldens():
    """The rest of the SIMD extension's unary list (cl-waffe2-simd.c:650-694):
    range samples with an n % 8 tail, special values, strides, broadcast source."""
    rng = np.random.Generator(np.random.PCG64(2026))
    out = {}
    for op, (lo, hi) in UNARY_MORE.items():
        x = rng.uniform(lo, hi, 2053).astype(np.float32)
        if op == "log1p":
            x[:256] = (rng.uniform(-1, 1, 256) * 10.0 ** rng.uniform(-12, -1, 256)).astype(np.float32)
        res = np.zeros_like(x)
        O.unary_1d(op, x.size, x, 1, res, 1, use_ref=True)
        out[f"un_{op}_range_x"], out[f"un_{op}_range_out"] = x, res
        res = np.zeros(EDGE.size, np.float32)
        with np.errstate(all="ignore"):
            O.unary_1d(op, EDGE.size, EDGE, 1, res, 1, use_ref=True)
        out[f"un_{op}_edge_out"] = res
        for n, incx, inco in [(13, 2, 1), (16, 1, 3), (9, 0, 1)]:
            res = np.full(64, 7.0, np.float32)
            O.unary_1d(op, n, x, incx, res, inco, use_ref=True)
            out[f"un_{op}_{n}_{incx}_{inco}_out"] = res
    out["edge_x"] = EDGE
    np.savez_compressed(os.path.join(HERE, "unary_more_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "unary_more_kernels.npz")), "bytes")


IM2COL_CASES = [  # N, C, H_in, W_in, kernel, stride, padding  (dilation 1)
    (1, 1, 5, 5, (3, 3), (1, 1), (0, 0)),
    (2, 3, 8, 7, (3, 2), (1, 1), (1, 1)),
    (1, 2, 9, 9, (3, 3), (2, 2), (1, 1)),
    (2, 2, 10, 6, (2, 3), (2, 1), (0, 2)),
    (1, 4, 12, 12, (5, 5), (3, 3), (2, 2)),
    (3, 1, 6, 11, (1, 1), (1, 2), (0, 0)),
]


def im2col_geometry(case):
    """The arguments `unfold` hands to Im2ColNode (source/nn/im2col.lisp:51-95):
    output sizes from conv-out-size, the image padded by (pad, pad + out mod stride)."""
    N, Cc, H, W, k, s, p = case
    out = [(size + 2 * p[a] - (k[a] - 1) - 1) // s[a] + 1 for a, size in enumerate((H, W))]
    padded = [size + 2 * p[a] + out[a] % s[a] for a, size in enumerate((H, W))]
    return N, Cc, padded[0], padded[1], out[0], out[1], k[0], k[1]


def im2col_goldens():
    """waffe2_im2col_s_column / waffe2_col2im_s_column (cl-waffe2-simd/kernels/im2col.c)
    on the geometries unfold produces."""
    assert O.im2col_ref_available(), "oracle/_ref/libwaffe2_im2col_ref.so is missing: run `make -C oracle ref`"
    rng = np.random.Generator(np.random.PCG64(2027))
    out = {}
    for idx, case in enumerate(IM2COL_CASES):
        N, Cc, H, W, Ho, Wo, kh, kw = im2col_geometry(case)
        _, _, _, _, k, s, p = case
        im = rng.standard_normal((N, Cc, H, W)).astype(np.float32)
        col = np.full((N, Cc, kh, kw, Ho, Wo), 7.0, np.float32)      # untouched elements keep the 7
        O.im2col(col, im, N, Cc, H, W, Ho, Wo, kh, kw, p, s, (1, 1), use_ref=True)
        out[f"im2col_{idx}_im"], out[f"im2col_{idx}_col"] = im, col
        cin = rng.standard_normal(col.shape).astype(np.float32)
        back = np.full(im.shape, 5.0, np.float32)
        O.col2im(cin, back, N, Cc, H, W, Ho, Wo, kh, kw, p, s, (1, 1), use_ref=True)
        out[f"col2im_{idx}_col"], out[f"col2im_{idx}_im"] = cin, back
    np.savez_compressed(os.path.join(HERE, "im2col_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "im2col_kernels.npz")), "bytes")


TYPED_REGIMES = [(1, 1), (1, 0), (2, 1), (1, 3), (2, 2), (0, 1), (0, 2)]
TYPED_SIZES = [1, 4, 5, 13]


def typed_operands(rng, dtype, size, op, incx):
    """Operands that keep the reference out of its traps: no zero divisors, no
    INT_MIN / -1; everything else (overflow, wrap-around) is fair game."""
    npt = O.DTYPES[dtype][1]
    if dtype == "double":
        x = rng.standard_normal(size)
        y = rng.standard_normal(size) if incx != 0 or op in ("add", "sub") else rng.uniform(0.9, 1.1, size)
        return x.astype(npt), y.astype(npt)
    info = np.iinfo(npt)
    x = rng.integers(info.min, info.max, size, dtype=np.int64, endpoint=True).astype(npt)
    y = rng.integers(info.min, info.max, size, dtype=np.int64, endpoint=True).astype(npt)
    if op == "div":
        small = rng.integers(1, 12, size).astype(npt)
        if info.min < 0:
            small = (small * rng.choice(np.array([1, -1], np.int64), size).astype(npt)).astype(npt)
            x[x == info.min] = info.min + 1
        y = np.where(rng.random(size) < 0.7, small, y).astype(npt)
        y[y == 0] = 3
    return x, y


def typed_goldens():
    """waffe2_d{add,sub,mul,div}, waffe2_{i32,...}{add,sub,mul,div,copy} and
    waffe2_*inv of the compiled reference, every increment regime."""
    assert O.ref() is not None, "oracle/_ref/libwaffe2_simd_ref.so is missing: run `make -C oracle ref`"
    rng = np.random.Generator(np.random.PCG64(2028))
    out = {}
    # per (dtype, op): the cases back to back, `cases` rows = (n, incx, incy, start, size)
    for dtype in O.DTYPES:
        for op in ("add", "sub", "mul", "div", "copy"):
            if dtype == "double" and op == "copy":
                continue  # BLAS dcopy_, not in the compiled kernels
            xs, ys, outs, cases, start = [], [], [], [], 0
            for n in TYPED_SIZES:
                for incx, incy in TYPED_REGIMES:
                    size = n * 3 + 1
                    x, y = typed_operands(rng, dtype, size, op, incx)
                    res = x.copy()
                    O.binary_typed_1d(dtype, op, n, res, incx, y, incy, use_ref=True)
                    xs.append(x), ys.append(y), outs.append(res)
                    cases.append((n, incx, incy, start, size))
                    start += size
            key = f"{dtype}_{op}"
            out[key + "_x"], out[key + "_y"], out[key + "_out"] = (np.concatenate(v) for v in (xs, ys, outs))
            out[key + "_cases"] = np.array(cases, np.int64)
        xs, outs, cases, start = [], [], [], 0
        for n in (1, 5, 64):
            for incx in (1, 2):
                x, _ = typed_operands(rng, dtype, n * 2 + 1, "add", 1)
                if dtype != "double":  # mostly the values whose inverse is not 0; never 0
                    info = np.iinfo(x.dtype)
                    pool = np.array([1, 2, 3, info.max] + ([-1, -2, info.min + 1] if info.min < 0 else []), np.int64)
                    x = np.where(rng.random(x.size) < 0.8, rng.choice(pool, x.size), x.astype(np.int64)).astype(x.dtype)
                    x[x == 0] = 1
                res = x.copy()
                O.inv_typed_1d(dtype, n, res, incx, use_ref=True)
                xs.append(x), outs.append(res)
                cases.append((n, incx, 0, start, x.size))
                start += x.size
        out[f"{dtype}_inv_x"], out[f"{dtype}_inv_out"] = np.concatenate(xs), np.concatenate(outs)
        out[f"{dtype}_inv_cases"] = np.array(cases, np.int64)
    np.savez_compressed(os.path.join(HERE, "typed_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "typed_kernels.npz")), "bytes")


# (n, incx, incy, inco); lanes = 32 bytes / element size
CMP_TYPED_REGIMES = [(1, 1, 1, 1), (5, 1, 1, 1), (40, 1, 1, 1), (70, 1, 1, 1), (13, 2, 1, 1), (37, 1, 3, 2),
                     (40, 1, 1, 0), (33, 2, 3, 0), (9, 3, 2, 1), (70, 1, 0, 1)]


def _cmp_case_defined(dtype, n, incx, incy, inco, scal):
    """The reference builds strided integer lanes by indexing a 4-lane vector up to
    lane 31 (cl-waffe2-simd.c:54-107, 119-141): undefined unless the block part is
    skipped (inco < 1, n < lanes) or every increment is 1."""
    if dtype == "double":
        return True
    lanes = 32 // np.dtype(O.DTYPES[dtype][1]).itemsize
    return inco < 1 or n < lanes or (incx == 1 and inco == 1 and (scal or incy == 1))


def _cmp_child(dtype, op, n, x, incx, y, incy, out, inco, then, els, conn):
    O.cmp_typed_1d(dtype, op, n, x, incx, y, incy, out, inco, then, els, use_ref=True)
    conn.send(out)


def compare_typed_goldens():
    """waffe2_<prefix>{eq,lt,le,gt,ge} and ..._scal of the compiled reference for
    :double and the integer types.  Each case runs in a child process: the compiled
    reference faults or spins on some cases its source leaves undefined; those and
    the undefined ones are left out and counted in `<dtype>_skipped`."""
    import multiprocessing as mp
    assert O.ref() is not None, "oracle/_ref/libwaffe2_simd_ref.so is missing: run `make -C oracle ref`"
    ctx = mp.get_context("fork")
    rng = np.random.Generator(np.random.PCG64(2029))
    out = {}
    for dtype, (code, npt, prefix) in O.DTYPES.items():
        xs, ys, outs, cases, start, skipped = [], [], [], [], 0, 0
        for op_index, op in enumerate(O.CMP_OPS):
            for n, incx, incy, inco in CMP_TYPED_REGIMES:
                for scal in (0, 1):
                    if not _cmp_case_defined(dtype, n, incx, incy, inco, scal):
                        skipped += 1
                        continue
                    size = n * 3 + 1
                    if dtype == "double":
                        x = rng.integers(-3, 4, size).astype(npt)
                        y = rng.integers(-3, 4, size).astype(npt)
                        x[rng.random(size) < 0.1] = np.nan
                        y[rng.random(size) < 0.05] = np.inf
                        then, els = 1.5, -0.25
                    else:
                        info = np.iinfo(npt)
                        pool = np.array([info.min, info.max, 0, 1, 2, info.max // 2, info.max // 2 + 1], np.int64)
                        x = rng.choice(pool, size).astype(npt)
                        y = rng.choice(pool, size).astype(npt)
                        then, els = 3, 5
                    res = np.full(size, 7, npt)
                    yy = y[0].item() if scal else y
                    parent, child = ctx.Pipe(duplex=False)
                    proc = ctx.Process(target=_cmp_child, args=(dtype, op, n, x, incx, yy, incy, res, inco, then, els, child))
                    proc.start()
                    got = parent.recv() if parent.poll(3) else None
                    proc.join(1)
                    if proc.is_alive():
                        proc.kill()
                        proc.join()
                    if got is None:
                        skipped += 1
                        continue
                    xs.append(x), ys.append(y), outs.append(got)
                    cases.append((op_index, n, incx, incy, inco, scal, start, size))
                    start += size
        key = f"{dtype}_cmp"
        if cases:
            out[key + "_x"], out[key + "_y"], out[key + "_out"] = (np.concatenate(v) for v in (xs, ys, outs))
        out[key + "_cases"] = np.array(cases, np.int64).reshape(-1, 8)
        out[key + "_skipped"] = np.array([skipped], np.int64)
        print(dtype, "cases", len(cases), "skipped", skipped, flush=True)
    np.savez_compressed(os.path.join(HERE, "typed_compare_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "typed_compare_kernels.npz")), "bytes")


def _extreme_child(dtype, op, n, x, incx, conn):
    conn.send(O.extreme_typed_1d(dtype, op, n, x, incx, use_ref=True))


def extreme_typed_goldens():
    """waffe2_<prefix>{max,min} of the compiled reference; integer runs with
    incx != 1 that reach the block part are undefined there (strided lanes, see
    _cmp_case_defined) and left out, as is any case the compiled reference does not
    finish."""
    import multiprocessing as mp
    assert O.ref() is not None, "oracle/_ref/libwaffe2_simd_ref.so is missing: run `make -C oracle ref`"
    ctx = mp.get_context("fork")
    rng = np.random.Generator(np.random.PCG64(2030))
    out = {}
    for dtype, (code, npt, prefix) in O.DTYPES.items():
        lanes = 32 // np.dtype(npt).itemsize
        xs, outs, cases, start, skipped = [], [], [], 0, 0
        for op_index, op in enumerate(("max", "min")):
            for n, incx in [(1, 1), (3, 1), (lanes, 1), (2 * lanes + 3, 1), (200, 1), (lanes - 1, 2), (5 * lanes + 1, 3)]:
                if dtype != "double" and incx != 1 and n >= lanes:
                    skipped += 1
                    continue
                size = n * incx + 1
                if dtype == "double":
                    x = (rng.standard_normal(size) * 100).round(1)
                else:
                    info = np.iinfo(npt)
                    x = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
                x = x.astype(npt)
                parent, child = ctx.Pipe(duplex=False)
                proc = ctx.Process(target=_extreme_child, args=(dtype, op, n, x, incx, child))
                proc.start()
                got = parent.recv() if parent.poll(3) else None
                proc.join(1)
                if proc.is_alive():
                    proc.kill()
                    proc.join()
                if got is None:
                    skipped += 1
                    continue
                xs.append(x), outs.append(got)
                cases.append((op_index, n, incx, start, size))
                start += size
        key = f"{dtype}_extreme"
        if cases:
            out[key + "_x"] = np.concatenate(xs)
            out[key + "_out"] = np.array(outs, npt)
        out[key + "_cases"] = np.array(cases, np.int64).reshape(-1, 5)
        out[key + "_skipped"] = np.array([skipped], np.int64)
        print(dtype, "cases", len(cases), "skipped", skipped, flush=True)
    np.savez_compressed(os.path.join(HERE, "typed_extreme_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "typed_extreme_kernels.npz")), "bytes")


def dunary_inputs(rng, op, size):
    """Arguments inside each function's domain, a few special values at the end."""
    if op in ("asin", "acos"):
        x = rng.uniform(-1, 1, size)
    elif op in ("log", "log2", "log10", "sqrt"):
        x = np.exp(rng.uniform(-30, 30, size))
    elif op == "log1p":
        x = np.expm1(rng.uniform(-20, 20, size))
    elif op in ("exp", "sinh", "cosh"):
        x = rng.uniform(-40, 40, size)
    elif op in ("sin", "cos", "tan"):
        x = rng.uniform(-1, 1, size) * 10.0 ** rng.integers(-3, 6, size)
    elif op == "pow":
        x = np.exp(rng.uniform(-5, 5, size))
    else:
        x = rng.uniform(-20, 20, size)
    return x


def dunary_goldens():
    """waffe2_d{sin,...,pow} of the compiled reference: SLEEF u10 on the blocks of
    four, libm on the remainder (both as this image has them)."""
    assert O.ref() is not None, "oracle/_ref/libwaffe2_simd_ref.so is missing: run `make -C oracle ref`"
    rng = np.random.Generator(np.random.PCG64(2031))
    out = {}
    for op in O.DUNARY_OPS:
        xs, outs, cases, start = [], [], [], 0
        for n, incx, inco in [(1, 1, 1), (4, 1, 1), (23, 1, 1), (64, 1, 1), (13, 2, 1), (13, 1, 3), (9, 3, 2), (7, 0, 1)]:
            size = n * 3 + 1
            x = dunary_inputs(rng, op, size)
            res = np.full(size, 7.0)
            O.dunary_1d(op, n, x, incx, res, inco, p=2.5, use_ref=True)
            xs.append(x), outs.append(res)
            cases.append((n, incx, inco, start, size))
            start += size
        out[f"{op}_x"], out[f"{op}_out"] = np.concatenate(xs), np.concatenate(outs)
        out[f"{op}_cases"] = np.array(cases, np.int64)
    np.savez_compressed(os.path.join(HERE, "double_unary_kernels.npz"), **out)
    print("wrote", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "double_unary_kernels.npz")), "bytes")


if __name__ == "__main__":
    if "--im2col-only" in sys.argv:
        im2col_goldens()
    elif "--compare-only" in sys.argv:
        compare_goldens()
    elif "--unary-more-only" in sys.argv:
        unary_more_goldens()
    elif "--typed-only" in sys.argv:
        typed_goldens()
    elif "--typed-compare-only" in sys.argv:
        compare_typed_goldens()
    elif "--typed-extreme-only" in sys.argv:
        extreme_typed_goldens()
    elif "--double-unary-only" in sys.argv:
        dunary_goldens()
    else:
        main()
        compare_goldens()
        unary_more_goldens()
        im2col_goldens()
        typed_goldens()
        compare_typed_goldens()
        extreme_typed_goldens()
        dunary_goldens()
