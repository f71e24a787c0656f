"""ctypes binding of ``libwaffe2-hip.so`` (the C ABI in ``include/waffe2_hip.h``).

Mirrors the role of ``cl-waffe2-simd/shared-object.lisp`` + ``api.lisp`` in the
reference: find the shared object next to the package, load it, declare every
foreign function.  Unlike the reference's soft-failing loader
(``shared-object.lisp:4-13`` warns and returns NIL so that CPUTensor falls back
to LispTensor), a missing library here is an error: there is no CPU fallback
behind the HIP backend.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwaffe2-hip.so")
MAX_RANK = 8

# enum wf2hip_binary_op / wf2hip_unary_op
ADD, SUB, MUL, DIV, MOVE = 0, 1, 2, 3, 4
# enum wf2hip_dtype: the element types served by the *_typed entry points
DTYPE_CODES = {"double": 1, "int32": 2, "uint32": 3, "int16": 4, "uint16": 5, "int8": 6, "uint8": 7}
SIN, COS, TANH, LOG, EXP, SQRT, ABS = 16, 17, 18, 19, 20, 21, 22
TAN, ASIN, ACOS, ATAN, SINH, COSH, LOG2, LOG10, LOG1P = 23, 24, 25, 26, 27, 28, 29, 30, 31
POW, GELU = 32, 40
SIGN, SQUARE, ASINH, ACOSH, ATANH = 34, 35, 36, 37, 38
RELU, SIGMOID, LEAKY_RELU = 41, 42, 43  # fused activation recipes
EQ, LT, LE, GT, GE = 0, 1, 2, 3, 4  # enum wf2hip_compare_op
COMPARE_NAMES = ("eq", "lt", "le", "gt", "ge")
MAXVALUE, MINVALUE, ARGMAX, ARGMIN = 48, 49, 50, 51  # enum wf2hip_select_op

EINVAL = -1
EOVERLAP = -3
EUNSUPPORTED = -4
ECAPTURE = -6


class HIPExtensionMissing(RuntimeError):
    """libwaffe2-hip.so is not built or cannot be loaded."""


class HIPError(RuntimeError):
    """A wf2hip_* call returned a non-zero code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"wf2hip error {code}: {message}")
        self.code = code


class View2(C.Structure):
    """``struct wf2hip_view2``"""

    _fields_ = [
        ("rank", C.c_int32),
        ("reserved", C.c_int32),
        ("shape", C.c_int64 * MAX_RANK),
        ("stride_a", C.c_int64 * MAX_RANK),
        ("stride_b", C.c_int64 * MAX_RANK),
        ("off_a", C.c_int64),
        ("off_b", C.c_int64),
    ]


_P = C.c_void_p
_L = C.c_long
_F = C.c_float
_D = C.c_double


class View3(C.Structure):
    """``struct wf2hip_view3``"""

    _fields_ = [
        ("rank", C.c_int32), ("reserved", C.c_int32),
        ("shape", C.c_int64 * 8), ("stride_a", C.c_int64 * 8), ("stride_b", C.c_int64 * 8),
        ("stride_c", C.c_int64 * 8),
        ("off_a", C.c_int64), ("off_b", C.c_int64), ("off_c", C.c_int64),
    ]


class MatmulDesc(C.Structure):
    """``struct wf2hip_matmul_desc``"""

    _fields_ = [
        ("trans_a", C.c_int32), ("trans_b", C.c_int32), ("activation", C.c_int32), ("causal", C.c_int32),
        ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
        ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
        ("batch", C.c_int64), ("batch2", C.c_int64),
        ("stride_a", C.c_int64), ("stride_a2", C.c_int64), ("stride_b", C.c_int64),
        ("stride_b2", C.c_int64), ("stride_c", C.c_int64), ("stride_c2", C.c_int64),
        ("bias", C.c_void_p), ("residual", C.c_void_p),
        ("ld_residual", C.c_int64), ("stride_residual", C.c_int64), ("stride_residual2", C.c_int64),
        ("alpha", C.c_float), ("reserved", C.c_int32),
    ]


class AttentionDesc(C.Structure):
    """``struct wf2hip_attention_desc``"""

    _fields_ = [
        ("batch", C.c_int64), ("heads", C.c_int64), ("seq", C.c_int64), ("head_dim", C.c_int64),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3),
        ("v_stride", C.c_int64 * 3), ("o_stride", C.c_int64 * 3),
        ("scale", C.c_float), ("causal", C.c_int32),
    ]


_SIGNATURES = {
    "wf2hip_abi_version": ([], C.c_int),
    "wf2hip_init": ([C.c_int], C.c_int),
    "wf2hip_shutdown": ([], C.c_int),
    "wf2hip_last_error": ([], C.c_char_p),
    "wf2hip_device_info": ([C.c_char_p, C.c_size_t], C.c_int),
    "wf2hip_malloc": ([C.POINTER(_P), C.c_size_t], C.c_int),
    "wf2hip_malloc_uninitialized": ([C.POINTER(_P), C.c_size_t], C.c_int),
    "wf2hip_free": ([_P], C.c_int),
    "wf2hip_pool_trim": ([], C.c_int),
    "wf2hip_pool_idle_bytes": ([], C.c_size_t),
    "wf2hip_pool_requests": ([], C.c_size_t),
    "wf2hip_memcpy_h2d": ([_P, _P, C.c_size_t], C.c_int),
    "wf2hip_memcpy_d2h": ([_P, _P, C.c_size_t], C.c_int),
    "wf2hip_memcpy_d2d": ([_P, _P, C.c_size_t], C.c_int),
    "wf2hip_fill_f32": ([_P, C.c_size_t, _F], C.c_int),
    "wf2hip_sync": ([], C.c_int),
    "wf2hip_set_stream": ([_P], C.c_int),
    "wf2hip_get_stream": ([], _P),
    "wf2hip_event_create": ([C.POINTER(_P)], C.c_int),
    "wf2hip_event_record": ([_P], C.c_int),
    "wf2hip_event_elapsed_ms": ([_P, _P, C.POINTER(_F)], C.c_int),
    "wf2hip_event_destroy": ([_P], C.c_int),
    "wf2hip_graph_begin": ([], C.c_int),
    "wf2hip_graph_end": ([C.POINTER(_P)], C.c_int),
    "wf2hip_graph_launch": ([_P], C.c_int),
    "wf2hip_graph_destroy": ([_P], C.c_int),
    "wf2hip_sadd": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_ssub": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_smul": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_sdiv": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_scopy": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_ssin": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_scos": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_stanh": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_slog": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_sexp": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_ssqrt": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_sabs": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_sinv": ([_L, _P, _L], C.c_int),
    "wf2hip_binary_1d_typed": ([C.c_int, C.c_int, _L, _P, _L, _P, _L], C.c_int),
    "wf2hip_binary_nd_typed": ([C.c_int, C.c_int, C.POINTER(View2), _P, _P], C.c_int),
    "wf2hip_inv_1d_typed": ([C.c_int, _L, _P, _L], C.c_int),
    "wf2hip_dcopy": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_stan": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_sasin": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_sacos": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_satan": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_ssinh": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_scosh": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_slog2": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_slog10": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_slog1p": ([_L, _P, _L, _P, _L], C.c_int),
    "wf2hip_spow": ([_L, _P, _L, _F, _P, _L], C.c_int),
    "wf2hip_smax": ([_L, _P, _L, _P], C.c_int),
    "wf2hip_smin": ([_L, _P, _L, _P], C.c_int),
    "wf2hip_binary_nd": ([C.c_int, C.POINTER(View2), _P, _P], C.c_int),
    "wf2hip_unary_nd": ([C.c_int, C.POINTER(View2), _P, _P, _F], C.c_int),
    "wf2hip_set_reduce_mode": ([C.c_int], C.c_int),
    "wf2hip_get_reduce_mode": ([], C.c_int),
    "wf2hip_sum_nd": ([C.POINTER(View2), _P, _P, C.c_float], C.c_int),
    "wf2hip_reduce_add_rows_f32": ([_L, _L, _P, _L, _P, _L], C.c_int),
    "wf2hip_reduce_add_rows_f32_noalloc": ([_L, _L, _P, _L, _P, _L], C.c_int),
    "wf2hip_softmax_rows_f32": ([_L, _L, _P, _L, _P, _L], C.c_int),
    "wf2hip_causal_softmax_f32": ([_L, _L, _P, _P, _F], C.c_int),
    "wf2hip_layernorm_rows_f32": ([_L, _L, _P, _P, _P, _F, _P], C.c_int),
    "wf2hip_softmax_backward_rows_f32": ([_L, _L, _P, _L, _P, _L, _P, _L, _F, _L], C.c_int),
    "wf2hip_layernorm_backward_f32": ([_L, _L, _P, _P, _P, _F, _P, _P, _P], C.c_int),
    "wf2hip_softmax_cross_entropy_f32": ([_L, _L, _P, _P, _F, _P, _P], C.c_int),
    "wf2hip_softmax_cross_entropy_backward_f32": ([_L, _P, C.c_int, _P, _P, _F, _P], C.c_int),
    "wf2hip_activation_backward_nd": ([C.c_int, C.POINTER(View2), _P, _P, _F], C.c_int),
    "wf2hip_sgemm": ([C.c_char, C.c_char, _L, _L, _L, _F, _P, _L, _P, _L, _F, _P, _L], C.c_int),
    "wf2hip_sgemm_strided_batched": (
        [C.c_char, C.c_char, _L, _L, _L, _F, _P, _L, _L, _P, _L, _L, _F, _P, _L, _L, _L],
        C.c_int,
    ),
    "wf2hip_matmul_fused": ([C.POINTER(MatmulDesc), _P, _P, _P], C.c_int),
    "wf2hip_select_nd": ([C.c_int, C.POINTER(View2), _L, _L, _P, _P], C.c_int),
    "wf2hip_where_nd": ([C.c_int, C.POINTER(View2), _P, _P, _F, _F, _F], C.c_int),
    "wf2hip_compare_nd": ([C.c_int, C.POINTER(View3), _P, _P, _P, _F, _F], C.c_int),
    **{f"wf2hip_s{n}": ([_L, _P, _L, _P, _L, _P, _L, _F, _F], C.c_int)
       for n in ("eq", "lt", "le", "gt", "ge")},
    **{f"wf2hip_s{n}_scal": ([_L, _P, _L, _P, _L, _F, _F, _F], C.c_int)
       for n in ("eq", "lt", "le", "gt", "ge")},
    "wf2hip_im2col_f32": ([_P] + [_L] * 14 + [_P], C.c_int),
    "wf2hip_col2im_f32": ([_P] + [_L] * 14 + [_P], C.c_int),
    "wf2hip_unfold_f32": ([_L] * 10 + [_P, _P], C.c_int),
    "wf2hip_sgd_step_f32": ([_L, _P, _P, _F], C.c_int),
    "wf2hip_adam_step_f32": ([_L, _P, _P, _P, _P, _F, _F, _F, _F], C.c_int),
    "wf2hip_embedding_add_f32": ([_L, _L, _L, _P, _P, _L, _P, _L, _P], C.c_int),
    "wf2hip_attention_f32": ([C.POINTER(AttentionDesc), _P, _P, _P, _P], C.c_int),
    "wf2hip_attention_forward_f32": ([C.POINTER(AttentionDesc), _P, _P, _P, _P, _P], C.c_int),
    "wf2hip_attention_backward_f32": ([C.POINTER(AttentionDesc)] + [_P] * 9, C.c_int),
    "wf2hip_sgemm_strided_batched_2d": (
        [C.c_char, C.c_char, _L, _L, _L, _F, _P, _L, _L, _L, _P, _L, _L, _L, _F, _P, _L, _L, _L, _L, _L],
        C.c_int,
    ),
    "wf2hip_dgemm": ([C.c_char, C.c_char, _L, _L, _L, _D, _P, _L, _P, _L, _D, _P, _L], C.c_int),
    "wf2hip_dgemm_strided_batched_2d": (
        [C.c_char, C.c_char, _L, _L, _L, _D, _P, _L, _L, _L, _P, _L, _L, _L, _D, _P, _L, _L, _L, _L, _L],
        C.c_int,
    ),
}

# the reference's own per-dtype names (waffe2_dadd -> wf2hip_dadd, ...): pointers are void* here
for _prefix in ("d", "i32", "u32", "i16", "u16", "i8", "u8"):
    for _op in ("add", "sub", "mul", "div") + (() if _prefix == "d" else ("copy",)):
        _SIGNATURES[f"wf2hip_{_prefix}{_op}"] = ([_L, _P, _L, _P, _L], C.c_int)
    _SIGNATURES[f"wf2hip_{_prefix}inv"] = ([_L, _P, _L], C.c_int)

_SIGNATURES["wf2hip_compare_nd_typed"] = ([C.c_int, C.c_int, C.POINTER(View3), _P, _P, _P, C.c_double, C.c_double], C.c_int)
_SIGNATURES["wf2hip_where_nd_typed"] = ([C.c_int, C.c_int, C.POINTER(View2), _P, _P, C.c_double, C.c_double, C.c_double],
                                       C.c_int)
# waffe2_<prefix>{eq,...} / ..._scal: the scalar and the two constants have the element type
for _prefix, _ctype in (("d", C.c_double), ("i32", C.c_int32), ("u32", C.c_uint32), ("i16", C.c_int16),
                        ("u16", C.c_uint16), ("i8", C.c_int8), ("u8", C.c_uint8)):
    for _op in ("eq", "lt", "le", "gt", "ge"):
        _SIGNATURES[f"wf2hip_{_prefix}{_op}"] = ([_L, _P, _L, _P, _L, _P, _L, _ctype, _ctype], C.c_int)
        _SIGNATURES[f"wf2hip_{_prefix}{_op}_scal"] = ([_L, _P, _L, _P, _L, _ctype, _ctype, _ctype], C.c_int)

_SIGNATURES["wf2hip_select_nd_typed"] = ([C.c_int, C.c_int, C.POINTER(View2), _L, _L, _P, _P], C.c_int)
for _prefix in ("d", "i32", "u32", "i16", "u16", "i8", "u8"):
    for _op in ("max", "min"):
        _SIGNATURES[f"wf2hip_{_prefix}{_op}"] = ([_L, _P, _L, _P], C.c_int)

_SIGNATURES["wf2hip_unary_nd_typed"] = ([C.c_int, C.c_int, C.POINTER(View2), _P, _P, C.c_double], C.c_int)
for _fn in ("sin", "cos", "tanh", "log", "exp", "sqrt", "abs", "tan", "asin", "acos", "atan", "sinh", "cosh",
            "log2", "log10", "log1p"):
    _SIGNATURES[f"wf2hip_d{_fn}"] = ([_L, _P, _L, _P, _L], C.c_int)
_SIGNATURES["wf2hip_dpow"] = ([_L, _P, _L, C.c_double, _P, _L], C.c_int)

EXPORTS = tuple(_SIGNATURES)

_lib = None
_initialised_device = None


def load():
    """Load the shared library and declare its functions (no GPU touched)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HIPExtensionMissing(
            f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()). The HIP backend has no CPU fallback."
        )
    try:
        lib = C.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise HIPExtensionMissing(f"cannot load {LIB_PATH}: {e}") from e
    for name, (argtypes, restype) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    _lib = lib
    return lib


def check(code: int) -> None:
    if code != 0:
        msg = load().wf2hip_last_error()
        raise HIPError(code, msg.decode() if msg else "")


def init(device: int = 0):
    """Initialise the runtime on ``device`` (idempotent) and return the library."""
    global _initialised_device
    lib = load()
    if _initialised_device != device:
        check(lib.wf2hip_init(device))
        _initialised_device = device
    return lib


def get():
    """The initialised library; initialises device 0 on first use."""
    if _initialised_device is None:
        return init(0)
    return _lib


def device_info() -> dict:
    buf = C.create_string_buffer(256)
    check(get().wf2hip_device_info(buf, 256))
    name, arch, cus, mem = buf.value.decode().split("|")
    return {"name": name, "arch": arch, "compute_units": int(cus), "memory_bytes": int(mem)}


def synchronize() -> None:
    check(get().wf2hip_sync())


class Event:
    """HIP event on the library's stream (for timing kernels where they run)."""

    def __init__(self):
        self._h = _P()
        check(get().wf2hip_event_create(C.byref(self._h)))

    def record(self) -> "Event":
        check(get().wf2hip_event_record(self._h))
        return self

    def elapsed_ms(self, stop: "Event") -> float:
        ms = _F()
        check(get().wf2hip_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            if self._h and _lib is not None:
                _lib.wf2hip_event_destroy(self._h)
        except Exception:
            pass


class Graph:
    """A recorded kernel sequence (``wf2hip_graph_*``).

        run()                       # once, so that the pool holds the temporaries
        with Graph() as g:          # record
            out = run()
        g.launch()                  # replay: one launch, no per-node host cost

    Keep the tensors the replay reads or writes (inputs, ``out``) alive while the
    graph is in use."""

    def __init__(self):
        self._h = _P()

    def __enter__(self) -> "Graph":
        check(get().wf2hip_graph_begin())
        return self

    def __exit__(self, exc_type, exc, tb):
        code = get().wf2hip_graph_end(C.byref(self._h))
        if exc_type is None:
            check(code)
        return False

    def launch(self) -> None:
        check(get().wf2hip_graph_launch(self._h))

    def destroy(self) -> None:
        if self._h and _lib is not None:
            _lib.wf2hip_graph_destroy(self._h)
            self._h = _P()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
