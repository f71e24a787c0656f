"""ctypes front end of the CPU oracle (``libwaffe2_oracle.so``) and of the
compiled reference kernels (``_ref/libwaffe2_simd_ref.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
CPU-baseline leg of the benchmark.  The product package never imports it.

The oracle restates cl-waffe2's CPUTensor + cl-waffe2-simd path; see the header
of ``waffe2_oracle.c`` for the reference file:line each function follows.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "libwaffe2_oracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libwaffe2_simd_ref.so")

MAX_RANK = 8
MAX_TENSORS = 3

# view kinds of orc_views.kind
KIND_T, KIND_BROADCAST, KIND_OTHER = 0, 1, 2

OPS = {
    "add": 0, "sub": 1, "mul": 2, "div": 3, "move": 4,
    "sin": 16, "cos": 17, "tanh": 18, "log": 19, "exp": 20, "sqrt": 21,
    "abs": 22, "tan": 23, "asin": 24, "acos": 25, "atan": 26, "sinh": 27, "cosh": 28, "log2": 29,
    "log10": 30, "log1p": 31, "pow": 32,
    "sign": 34, "square": 35, "asinh": 36, "acosh": 37, "atanh": 38,
}
UNARY_NAMES = ("sin", "cos", "tanh", "log", "exp", "sqrt", "abs", "tan", "asin", "acos", "atan", "sinh", "cosh",
               "log2", "log10", "log1p")
# nodes that run LispTensor's per-element loop in the reference (no SIMD kernel)
LISP_UNARY_NAMES = ("sign", "square", "asinh", "acosh", "atanh")


class OrcViews(C.Structure):
    _fields_ = [
        ("rank", C.c_int),
        ("ntensors", C.c_int),
        ("shape", C.c_long * MAX_RANK),
        ("stride", (C.c_long * MAX_RANK) * MAX_TENSORS),
        ("kind", (C.c_int * MAX_RANK) * MAX_TENSORS),
        ("first", (C.c_long * MAX_RANK) * MAX_TENSORS),
        ("step", (C.c_long * MAX_RANK) * MAX_TENSORS),
        ("offset", C.c_long * MAX_TENSORS),
    ]


class OrcCall(C.Structure):
    _fields_ = [
        ("n", C.c_long),
        ("off", C.c_long * MAX_TENSORS),
        ("inc", C.c_long * MAX_TENSORS),
    ]


def build(force: bool = False) -> None:
    """Compile the oracle (and ``_ref`` when the reference checkout exists)."""
    if force or not os.path.exists(_ORACLE_SO) or (
        os.path.getmtime(_ORACLE_SO)
        < os.path.getmtime(os.path.join(_HERE, "waffe2_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "oracle"], stdout=subprocess.DEVNULL)
    if force or not os.path.exists(_REF_SO):
        subprocess.call(["make", "-C", _HERE, "ref"], stdout=subprocess.DEVNULL,
                        stderr=subprocess.DEVNULL)


def _torch_cpu_lib() -> str | None:
    import importlib.util

    spec = importlib.util.find_spec("torch")
    if spec is None or spec.origin is None:
        return None
    path = os.path.join(os.path.dirname(spec.origin), "lib", "libtorch_cpu.so")
    return path if os.path.exists(path) else None


_lib = None
_ref = None
_F = C.POINTER(C.c_float)


def _fp(a: np.ndarray, offset: int = 0):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return C.cast(a.ctypes.data + 4 * offset, _F)


def lib():
    """The oracle library, with SLEEF resolved when a provider is present."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_ORACLE_SO):
        build()
    L = C.CDLL(_ORACLE_SO)
    for name in ("add", "sub", "mul", "div"):
        f = getattr(L, "orc_s" + name)
        f.argtypes = [C.c_long, _F, C.c_long, _F, C.c_long]
        f.restype = None
    L.orc_scopy.argtypes = [C.c_long, _F, C.c_long, _F, C.c_long]
    L.orc_scopy.restype = None
    for name in UNARY_NAMES + LISP_UNARY_NAMES:
        f = getattr(L, "orc_s" + name)
        f.argtypes = [C.c_long, _F, C.c_long, _F, C.c_long]
        f.restype = None
    L.orc_spow.argtypes = [C.c_long, _F, C.c_long, C.c_float, _F, C.c_long]
    L.orc_spow.restype = None
    for name in ("max", "min"):
        f = getattr(L, "orc_s" + name)
        f.argtypes = [C.c_long, _F, C.c_long, _F]
        f.restype = None
    L.orc_sinv.argtypes = [C.c_long, _F, C.c_long]
    L.orc_sinv.restype = None
    for name in ("orc_ismax", "orc_ismin"):
        f = getattr(L, name)
        f.argtypes = [C.c_long, _F, C.c_long]
        f.restype = C.c_long
    L.orc_scmp.argtypes = [C.c_int, C.c_long, _F, C.c_long, _F, C.c_long, _F, C.c_long,
                           C.c_float, C.c_float]
    L.orc_scmp.restype = None
    L.orc_scmp_scal.argtypes = [C.c_int, C.c_long, _F, C.c_long, _F, C.c_long, C.c_float,
                                C.c_float, C.c_float]
    L.orc_scmp_scal.restype = None
    L.orc_where_nd.argtypes = [C.c_int, C.POINTER(OrcViews), _F, _F, C.c_float, C.c_float, C.c_float]
    L.orc_where_nd.restype = C.c_long
    L.orc_compare_nd.argtypes = [C.c_int, C.POINTER(OrcViews), _F, _F, _F, C.c_float, C.c_float]
    L.orc_compare_nd.restype = C.c_long
    L.orc_schedule.argtypes = [C.POINTER(OrcViews), C.POINTER(OrcCall), C.c_long]
    L.orc_schedule.restype = C.c_long
    L.orc_node_nd.argtypes = [C.c_int, C.POINTER(OrcViews), _F, _F, C.c_float]
    L.orc_node_nd.restype = C.c_long
    L.orc_sgemm.argtypes = [C.c_char, C.c_char, C.c_long, C.c_long, C.c_long,
                            C.c_float, _F, C.c_long, _F, C.c_long, C.c_float,
                            _F, C.c_long]
    L.orc_sgemm.restype = None
    L.orc_matmul_rowmajor.argtypes = [C.c_int, C.c_int, C.c_long, C.c_long,
                                      C.c_long, _F, C.c_long, _F, C.c_long, _F,
                                      C.c_long]
    L.orc_matmul_rowmajor.restype = None
    L.orc_sleef_open.argtypes = [C.c_char_p]
    L.orc_sleef_open.restype = C.c_int
    L.orc_sleef_available.restype = C.c_int
    tl = _torch_cpu_lib()
    if tl is not None:
        L.orc_sleef_open(tl.encode())
    _lib = L
    return L


def sleef_available() -> bool:
    return bool(lib().orc_sleef_available())


def ref():
    """The reference's own C kernels compiled into ``_ref`` (or None)."""
    global _ref
    if _ref is not None:
        return _ref
    if not os.path.exists(_REF_SO):
        return None
    try:
        R = C.CDLL(_REF_SO)
    except OSError:
        return None
    for name in ("add", "sub", "mul", "div") + UNARY_NAMES:
        f = getattr(R, "waffe2_s" + name)
        f.argtypes = [C.c_long, _F, C.c_long, _F, C.c_long]
        f.restype = None
    R.waffe2_spow.argtypes = [C.c_long, _F, C.c_long, C.c_float, _F, C.c_long]
    R.waffe2_spow.restype = None
    R.waffe2_sinv.argtypes = [C.c_long, _F, C.c_long]
    R.waffe2_sinv.restype = None
    for name in CMP_OPS:
        f = getattr(R, "waffe2_s" + name)
        f.argtypes = [C.c_long, _F, C.c_long, _F, C.c_long, _F, C.c_long, C.c_float, C.c_float]
        f.restype = None
        f = getattr(R, "waffe2_s" + name + "_scal")
        f.argtypes = [C.c_long, _F, C.c_long, _F, C.c_long, C.c_float, C.c_float, C.c_float]
        f.restype = None
    for name in ("max", "min"):
        f = getattr(R, "waffe2_s" + name)
        f.argtypes = [C.c_long, _F, C.c_long, _F]
        f.restype = None
    _ref = R
    return R


# ---------------------------------------------------------------------------
# 1-D kernels on numpy storage (in place on `x`, like the reference)
# ---------------------------------------------------------------------------

def binary_1d(op: str, n: int, x: np.ndarray, incx: int, y: np.ndarray, incy: int,
              offx: int = 0, offy: int = 0, use_ref: bool = False) -> None:
    L = ref() if use_ref else lib()
    name = ("waffe2_s" if use_ref else "orc_s") + op
    getattr(L, name)(n, _fp(x, offx), incx, _fp(y, offy), incy)


def copy_1d(n: int, y: np.ndarray, incy: int, x: np.ndarray, incx: int,
            offy: int = 0, offx: int = 0) -> None:
    lib().orc_scopy(n, _fp(y, offy), incy, _fp(x, offx), incx)


def unary_1d(op: str, n: int, x: np.ndarray, incx: int, out: np.ndarray, inco: int,
             offx: int = 0, offo: int = 0, use_ref: bool = False) -> None:
    L = ref() if use_ref else lib()
    name = ("waffe2_s" if use_ref else "orc_s") + op
    getattr(L, name)(n, _fp(x, offx), incx, _fp(out, offo), inco)


def pow_1d(n: int, x: np.ndarray, incx: int, p: float, out: np.ndarray, inco: int,
           use_ref: bool = False) -> None:
    L = ref() if use_ref else lib()
    name = "waffe2_spow" if use_ref else "orc_spow"
    getattr(L, name)(n, _fp(x), incx, C.c_float(p), _fp(out), inco)


_U64 = C.c_uint64
_im2col_ref = None


def _im2col_lib(use_ref: bool):
    """(library, prefix): the oracle, or the reference's im2col.c compiled into _ref."""
    global _im2col_ref
    if not use_ref:
        L = lib()
        for name in ("orc_im2col", "orc_col2im"):
            getattr(L, name).argtypes = [_F] + [_U64] * 14 + [_F]
            getattr(L, name).restype = None
        return L, "orc_"
    if _im2col_ref is None:
        path = os.path.join(_HERE, "_ref", "libwaffe2_im2col_ref.so")
        if not os.path.exists(path):
            return None, None
        _im2col_ref = C.CDLL(path)
        for name in ("waffe2_im2col_s_column", "waffe2_col2im_s_column"):
            getattr(_im2col_ref, name).argtypes = [_F] + [_U64] * 14 + [_F]
            getattr(_im2col_ref, name).restype = None
    return _im2col_ref, "waffe2_"


def im2col_ref_available() -> bool:
    return _im2col_lib(True)[0] is not None


def im2col(col: np.ndarray, im: np.ndarray, N, Cc, H, W, H_out, W_out, K_H, K_W, pad, stride, dilation,
           use_ref: bool = False) -> None:
    """col[N C K_H K_W H_out W_out] <- im[N C H W] (waffe2_im2col_s_column)."""
    L, pre = _im2col_lib(use_ref)
    f = getattr(L, "orc_im2col" if not use_ref else "waffe2_im2col_s_column")
    f(_fp(col), N, Cc, H, W, H_out, W_out, K_H, K_W, pad[0], pad[1], stride[0], stride[1],
      dilation[0], dilation[1], _fp(im))


def col2im(col: np.ndarray, im: np.ndarray, N, Cc, H, W, H_out, W_out, K_H, K_W, pad, stride, dilation,
           use_ref: bool = False) -> None:
    """im[N C H W] <- sum of col (waffe2_col2im_s_column)."""
    L, pre = _im2col_lib(use_ref)
    f = getattr(L, "orc_col2im" if not use_ref else "waffe2_col2im_s_column")
    f(_fp(col), N, Cc, H, W, H_out, W_out, K_H, K_W, pad[0], pad[1], stride[0], stride[1],
      dilation[0], dilation[1], _fp(im))


def inv_1d(n: int, x: np.ndarray, incx: int, use_ref: bool = False) -> None:
    """x <- 1 / x in place (waffe2_sinv)."""
    (ref().waffe2_sinv if use_ref else lib().orc_sinv)(n, _fp(x), incx)


def argmaxmin_1d(op: str, n: int, x: np.ndarray, incx: int, offx: int = 0) -> int:
    """0-based index of the first largest / smallest element of the run, i.e.
    ``(1- (blas-ismax n x incx))`` as ArgMax-Node uses it."""
    return int(getattr(lib(), "orc_is" + op)(n, _fp(x, offx), incx)) - 1


CMP_OPS = ("eq", "lt", "le", "gt", "ge")  # enum order of orc_scmp / wf2hip compare ops


def cmp_1d(op: str, n: int, x: np.ndarray, incx: int, y: np.ndarray, incy: int, out: np.ndarray,
           inco: int, then: float = 1.0, els: float = 0.0, use_ref: bool = False) -> None:
    """out <- (x OP y) ? then : els (waffe2_s{eq,lt,le,gt,ge})."""
    if use_ref:
        getattr(ref(), "waffe2_s" + op)(n, _fp(x), incx, _fp(y), incy, _fp(out), inco,
                                        C.c_float(then), C.c_float(els))
    else:
        lib().orc_scmp(CMP_OPS.index(op), n, _fp(x), incx, _fp(y), incy, _fp(out), inco,
                       C.c_float(then), C.c_float(els))


def cmp_scal_1d(op: str, n: int, x: np.ndarray, incx: int, out: np.ndarray, inco: int, y: float,
                then: float = 1.0, els: float = 0.0, use_ref: bool = False) -> None:
    """out <- (x OP y) ? then : els with a scalar y (waffe2_s{eq,...}_scal)."""
    if use_ref:
        getattr(ref(), "waffe2_s" + op + "_scal")(n, _fp(x), incx, _fp(out), inco, C.c_float(y),
                                                  C.c_float(then), C.c_float(els))
    else:
        lib().orc_scmp_scal(CMP_OPS.index(op), n, _fp(x), incx, _fp(out), inco, C.c_float(y),
                            C.c_float(then), C.c_float(els))


def where_nd(op: str, views: OrcViews, x: np.ndarray, out: np.ndarray, scal: float,
             then: float = 1.0, els: float = 0.0) -> None:
    rc = lib().orc_where_nd(CMP_OPS.index(op), C.byref(views), _fp(x), _fp(out), C.c_float(scal),
                            C.c_float(then), C.c_float(els))
    assert rc == 0


def compare_nd(op: str, views: OrcViews, x: np.ndarray, y: np.ndarray, out: np.ndarray,
               then: float = 1.0, els: float = 0.0) -> None:
    rc = lib().orc_compare_nd(CMP_OPS.index(op), C.byref(views), _fp(x), _fp(y), _fp(out),
                              C.c_float(then), C.c_float(els))
    assert rc == 0


def maxmin_1d(op: str, n: int, x: np.ndarray, incx: int, use_ref: bool = False) -> float:
    L = ref() if use_ref else lib()
    out = np.zeros(1, np.float32)
    getattr(L, ("waffe2_s" if use_ref else "orc_s") + op)(n, _fp(x), incx, _fp(out))
    return float(out[0])


# ---------------------------------------------------------------------------
# Views / scheduler
# ---------------------------------------------------------------------------

def make_views(shape, tensors) -> OrcViews:
    """``tensors``: list of dicts with keys stride, kind, first, step, offset
    (per-axis lists; see waffe2_oracle.c for their meaning)."""
    v = OrcViews()
    v.rank = len(shape)
    v.ntensors = len(tensors)
    for r, s in enumerate(shape):
        v.shape[r] = int(s)
    for t, d in enumerate(tensors):
        v.offset[t] = int(d.get("offset", 0))
        for r in range(len(shape)):
            v.stride[t][r] = int(d["stride"][r])
            v.kind[t][r] = int(d["kind"][r])
            v.first[t][r] = int(d["first"][r])
            v.step[t][r] = int(d["step"][r])
    return v


def schedule(views: OrcViews, cap: int = 1 << 16):
    """List of (n, offs, incs) 1-D calls the reference's compiled loop makes."""
    buf = (OrcCall * cap)()
    cnt = lib().orc_schedule(C.byref(views), buf, cap)
    out = []
    for i in range(min(cnt, cap)):
        c = buf[i]
        out.append((c.n, tuple(c.off[: views.ntensors]), tuple(c.inc[: views.ntensors])))
    return cnt, out


def node_nd(op: str, views: OrcViews, t0: np.ndarray, t1: np.ndarray, p: float = 0.0) -> None:
    """Run a node over N-D views exactly as the CPU backend would: binary/move
    ops write into ``t0`` (x <- x op y); unary/pow read ``t0`` and write ``t1``."""
    rc = lib().orc_node_nd(OPS[op], C.byref(views), _fp(t0), _fp(t1), C.c_float(p))
    if rc != 0:
        raise ValueError("orc_node_nd rejected the views")


# ---------------------------------------------------------------------------
# gemm
# ---------------------------------------------------------------------------

def sgemm(transa: str, transb: str, m: int, n: int, k: int, alpha: float,
          A: np.ndarray, lda: int, B: np.ndarray, ldb: int, beta: float,
          Cm: np.ndarray, ldc: int) -> None:
    lib().orc_sgemm(transa.encode(), transb.encode(), m, n, k, C.c_float(alpha),
                    _fp(A), lda, _fp(B), ldb, C.c_float(beta), _fp(Cm), ldc)


def matmul_rowmajor(A: np.ndarray, B: np.ndarray, trans_a: bool = False,
                    trans_b: bool = False) -> np.ndarray:
    """Row-major ``op(A) @ op(B)`` through the reference's operand-swapped
    column-major sgemm call (backends/cpu/matrix-ops.lisp:12-112)."""
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    m, k = (A.shape[1], A.shape[0]) if trans_a else A.shape
    k2, n = (B.shape[1], B.shape[0]) if trans_b else B.shape
    assert k == k2
    out = np.zeros((m, n), np.float32)
    lib().orc_matmul_rowmajor(int(trans_a), int(trans_b), m, n, k, _fp(A), A.shape[1],
                              _fp(B), B.shape[1], _fp(out), n)
    return out


# ---- the other element types -------------------------------------------------
DTYPES = {"double": (1, np.float64, "d"), "int32": (2, np.int32, "i32"), "uint32": (3, np.uint32, "u32"),
          "int16": (4, np.int16, "i16"), "uint16": (5, np.uint16, "u16"), "int8": (6, np.int8, "i8"),
          "uint8": (7, np.uint8, "u8")}
TYPED_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "copy": 4}


def binary_typed_1d(dtype: str, op: str, n: int, x: np.ndarray, incx: int, y: np.ndarray, incy: int,
                    offx: int = 0, offy: int = 0, use_ref: bool = False) -> None:
    """x[offx + i incx] <- x[...] op y[offy + i incy] in place, through the oracle's
    restatement or (use_ref) the reference's own waffe2_<prefix><op>; :double
    copies have no reference symbol (BLAS dcopy_) and always take the oracle."""
    code, npt, prefix = DTYPES[dtype]
    assert x.dtype == npt and y.dtype == npt
    size = x.itemsize
    px = C.c_void_p(x.ctypes.data + size * offx)
    py = C.c_void_p(y.ctypes.data + size * offy)
    if use_ref and not (dtype == "double" and op == "copy"):
        fn = getattr(ref(), f"waffe2_{prefix}{op}")
        fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long]
        fn.restype = None
        fn(n, px, incx, py, incy)
        return
    fn = lib().orc_binary_typed
    fn.argtypes = [C.c_int, C.c_int, C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long]
    fn.restype = C.c_int
    assert fn(code, TYPED_OPS[op], n, px, incx, py, incy) == 0


def inv_typed_1d(dtype: str, n: int, x: np.ndarray, incx: int, use_ref: bool = False) -> None:
    code, npt, prefix = DTYPES[dtype]
    assert x.dtype == npt
    px = C.c_void_p(x.ctypes.data)
    if use_ref:
        fn = getattr(ref(), f"waffe2_{prefix}inv")
        fn.argtypes = [C.c_long, C.c_void_p, C.c_long]
        fn.restype = None
        fn(n, px, incx)
        return
    fn = lib().orc_inv_typed
    fn.argtypes = [C.c_int, C.c_long, C.c_void_p, C.c_long]
    fn.restype = C.c_int
    assert fn(code, n, px, incx) == 0


_CTYPES = {"double": C.c_double, "int32": C.c_int32, "uint32": C.c_uint32, "int16": C.c_int16,
           "uint16": C.c_uint16, "int8": C.c_int8, "uint8": C.c_uint8}


def cmp_typed_1d(dtype: str, op: str, n: int, x: np.ndarray, incx: int, y, incy: int, out: np.ndarray, inco: int,
                 then=1, els=0, use_ref: bool = False, offx: int = 0, offy: int = 0, offo: int = 0) -> None:
    """out <- (x OP y) ? then : els for one element type, ``y`` an array
    (waffe2_<prefix><op>) or a number (waffe2_<prefix><op>_scal), through the
    oracle's restatement or (use_ref) the compiled reference."""
    code, npt, prefix = DTYPES[dtype]
    scal = not isinstance(y, np.ndarray)
    assert x.dtype == npt and out.dtype == npt and (scal or y.dtype == npt)
    size = x.itemsize
    px = C.c_void_p(x.ctypes.data + size * offx)
    po = C.c_void_p(out.ctypes.data + size * offo)
    py = None if scal else C.c_void_p(y.ctypes.data + size * offy)
    ct = _CTYPES[dtype]
    if use_ref:
        if scal:
            fn = getattr(ref(), f"waffe2_{prefix}{op}_scal")
            fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long, ct, ct, ct]
            fn.restype = None
            fn(n, px, incx, po, inco, ct(y), ct(then), ct(els))
        else:
            fn = getattr(ref(), f"waffe2_{prefix}{op}")
            fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long, ct, ct]
            fn.restype = None
            fn(n, px, incx, py, incy, po, inco, ct(then), ct(els))
        return
    fn = lib().orc_cmp_typed
    fn.argtypes = [C.c_int, C.c_int, C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long,
                   C.c_int, C.c_double, C.c_double, C.c_double]
    fn.restype = C.c_int
    assert fn(code, CMP_OPS.index(op), n, px, incx, py, 0 if scal else incy, po, inco, int(scal),
              float(y) if scal else 0.0, float(then), float(els)) == 0


def extreme_typed_1d(dtype: str, op: str, n: int, x: np.ndarray, incx: int, use_ref: bool = False, offx: int = 0):
    """The largest (op "max") / smallest ("min") element of the run, as
    waffe2_<prefix>{max,min} leave it in y[0]."""
    code, npt, prefix = DTYPES[dtype]
    assert x.dtype == npt
    out = np.zeros(1, npt)
    px = C.c_void_p(x.ctypes.data + x.itemsize * offx)
    if use_ref:
        fn = getattr(ref(), f"waffe2_{prefix}{op}")
        fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p]
        fn.restype = None
        fn(n, px, incx, C.c_void_p(out.ctypes.data))
    else:
        fn = lib().orc_extreme_typed
        fn.argtypes = [C.c_int, C.c_int, C.c_long, C.c_void_p, C.c_long, C.c_void_p]
        fn.restype = C.c_int
        assert fn(code, int(op == "max"), n, px, incx, C.c_void_p(out.ctypes.data)) == 0
    return out[0]


DUNARY_OPS = ("sin", "cos", "tanh", "log", "exp", "sqrt", "abs", "tan", "asin", "acos", "atan", "sinh", "cosh",
              "log2", "log10", "log1p", "pow")


def dunary_1d(op: str, n: int, x: np.ndarray, incx: int, out: np.ndarray, inco: int, p: float = 0.0,
              use_ref: bool = False, offx: int = 0, offo: int = 0) -> None:
    """out <- f(x) on binary64 runs (waffe2_d<op>; ``pow`` takes the exponent p)."""
    assert x.dtype == np.float64 and out.dtype == np.float64
    px = C.c_void_p(x.ctypes.data + 8 * offx)
    po = C.c_void_p(out.ctypes.data + 8 * offo)
    if use_ref:
        fn = getattr(ref(), f"waffe2_d{op}")
        if op == "pow":
            fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_double, C.c_void_p, C.c_long]
            fn.restype = None
            fn(n, px, incx, p, po, inco)
        else:
            fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long]
            fn.restype = None
            fn(n, px, incx, po, inco)
        return
    fn = lib().orc_dunary
    fn.argtypes = [C.c_int, C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long, C.c_double]
    fn.restype = C.c_int
    assert fn(DUNARY_OPS.index(op), n, px, incx, po, inco, p) >= 0


def gpt2_positional_embedding(ctx: np.ndarray, wte: np.ndarray, wpe: np.ndarray, use_ref: bool = False) -> np.ndarray:
    """GPT2PositionalEmbedding of the reference's GPT-2 example on a freshly allocated (zero) output
    (examples/gpt-2/utils.lisp:19-66): per sentence and position, `waffe2_sadd` of the token's WTE row
    and then of the position's WPE row onto the output row, embedding-size elements each; the token id
    is `(round vocab-index)` of the :float context (ties to even).  ctx: (N, T) float32."""
    n, t = ctx.shape
    dim = wte.shape[1]
    out = np.zeros(n * t * dim, np.float32)
    wte_flat = np.ascontiguousarray(wte, np.float32).ravel()
    wpe_flat = np.ascontiguousarray(wpe, np.float32).ravel()
    for s in range(n):
        for pos in range(t):
            token = int(np.rint(ctx[s, pos]))
            offx = (s * t + pos) * dim
            binary_1d("add", dim, out, 1, wte_flat, 1, offx=offx, offy=token * dim, use_ref=use_ref)
            binary_1d("add", dim, out, 1, wpe_flat, 1, offx=offx, offy=pos * dim, use_ref=use_ref)
    return out.reshape(n, t, dim)
