/*
 * waffe2_hip.h -- C ABI of libwaffe2-hip.so, the MI355X (gfx950) tensor-kernel
 * library behind cl-waffe2's HIPTensor backend.
 *
 * The library takes the place that cl-waffe2-simd.so plus the system BLAS hold
 * for the CPUTensor backend: a host language (Common Lisp through CFFI, or any
 * FFI) passes element counts, raw DEVICE pointers, offsets and strides.  Every
 * entry point cites the reference interface it replaces (paths relative to the
 * cl-waffe2 checkout).
 *
 * Conventions
 *   - All data pointers are device pointers obtained from wf2hip_malloc (or
 *     any other HIP allocation of the current device).  The entry points
 *     without a dtype argument or prefix take fp32; :double and the integer
 *     element types have the *_typed entry points and the reference's own
 *     per-type names (wf2hip_dadd ... wf2hip_u8ge_scal).
 *   - Strides/increments and offsets are in ELEMENTS.  inc == 0 broadcasts.
 *   - Every function returns 0 on success or a negative WF2HIP_E* code / a
 *     positive hipError_t; wf2hip_last_error() returns a thread-local message.
 *     (The reference's kernels return void and have no error channel.)
 *   - Kernels are enqueued on one stream (created by wf2hip_init; another one
 *     can be adopted with wf2hip_set_stream) and return without waiting; wf2hip_memcpy_d2h, wf2hip_sync and
 *     wf2hip_event_elapsed_ms block.
 *   - The library keeps no pointer after a call returns and never frees or
 *     reallocates a caller's buffer.
 */
#ifndef WAFFE2_HIP_H
#define WAFFE2_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WF2HIP_ABI_VERSION 1
#define WF2HIP_MAX_RANK 8

/* error codes (negative: raised by the library before any launch) */
#define WF2HIP_OK 0
#define WF2HIP_EINVAL (-1)     /* bad rank, negative size, null pointer          */
#define WF2HIP_ENOTINIT (-2)   /* wf2hip_init has not succeeded                  */
#define WF2HIP_EOVERLAP (-3)   /* in-place op on partially overlapping views     */
#define WF2HIP_EUNSUPPORTED (-4)
#define WF2HIP_ENOMEM (-5)
#define WF2HIP_ECAPTURE (-6)   /* not possible during / outside a graph capture    */

/* ---- runtime ----------------------------------------------------------- */
/* No counterpart in cl-waffe2-simd (host memory needs none); the loader
 * pattern it follows is cl-waffe2-simd/shared-object.lisp:4-13 and the
 * allocation hook is AbstractTensor's initialize-instance
 * (source/vm/generic-tensor/tensor.lisp:146-210). */
int wf2hip_abi_version(void);
int wf2hip_init(int device);
int wf2hip_shutdown(void);
const char* wf2hip_last_error(void);
/* "name|gcnArch|CUs|memory bytes" of the initialised device */
int wf2hip_device_info(char* buf, size_t buflen);
/* Zero-initialised device memory: cl-waffe2 relies on fresh tensors being 0
 * (backends/lisp/tensor.lisp:12-28; !sum zero-fills by multiplying by 0,
 * base-impl/reduction.lisp:63). */
int wf2hip_malloc(void** ptr, size_t bytes);
/* Same without the zero fill, for tensors whose first use overwrites them
 * (cl-waffe2's InputTensor temporaries from make-input,
 * source/vm/generic-tensor/tensor.lisp:613-717). */
int wf2hip_malloc_uninitialized(void** ptr, size_t bytes);
/* Returns the block to the library's pool: no synchronisation, the block is
 * recycled in stream order (the steady state cl-waffe2 gets from allocating a
 * compiled model's temporaries once, source/vm/allocation.lisp:121-145).
 * WF2HIP_POOL=0 in the environment makes every free a hipFree. */
int wf2hip_free(void* ptr);
/* Give idle pooled blocks back to the device (synchronises). */
int wf2hip_pool_trim(void);
size_t wf2hip_pool_idle_bytes(void);
/* Number of block requests (wf2hip_malloc, wf2hip_malloc_uninitialized and the library's own scratch) served
 * since the library was loaded, from the pool or from the device: a caller can check that a sequence it
 * means to capture, or an entry point that promises not to allocate, asked for nothing. */
size_t wf2hip_pool_requests(void);
int wf2hip_memcpy_h2d(void* dst, const void* src, size_t bytes);
int wf2hip_memcpy_d2h(void* dst, const void* src, size_t bytes);
int wf2hip_memcpy_d2d(void* dst, const void* src, size_t bytes);
int wf2hip_fill_f32(float* x, size_t n, float value);
int wf2hip_sync(void);
/* Adopt an externally created hipStream_t (NULL = back to the library's own). */
int wf2hip_set_stream(void* hip_stream);
void* wf2hip_get_stream(void);
/* Events on the library's stream, for timing kernels where they run. */
int wf2hip_event_create(void** event);
int wf2hip_event_record(void* event);
int wf2hip_event_elapsed_ms(void* start, void* stop, float* ms);
int wf2hip_event_destroy(void* event);

/* ---- graph capture ------------------------------------------------------- */
/* Record everything enqueued between begin and end into a HIP graph and replay
 * it with one launch: the device-side counterpart of cl-waffe2 compiling a
 * model once and re-running its instruction sequence on every forward
 * (source/vm/generic-tensor/acceptor.lisp:409-508, source/vm/vm.lisp:260).
 * Rules: run the sequence once before capturing (allocations during capture
 * are served from the pool only: WF2HIP_ECAPTURE otherwise); host transfers and
 * wf2hip_sync are refused while capturing; tensors the replay reads or writes
 * (inputs, outputs) must stay allocated for as long as the graph is used; new
 * inputs are written into the same buffers.  wf2hip_graph_destroy waits for
 * the stream; called while another graph is being recorded it returns at once
 * and the graph is destroyed when that recording ends (a live graph keeps its
 * blocks: run the sequence once more before recording it again). */
int wf2hip_graph_begin(void);
int wf2hip_graph_end(void** graph);
int wf2hip_graph_launch(void* graph);
int wf2hip_graph_destroy(void* graph);

/* ---- BLAS-like 1-D kernels (one-for-one with waffe2_s*) ---------------- */
/* x[i*incx] <- x[i*incx] op y[i*incy], i < n.
 * Replaces waffe2_s{add,sub,mul,div} (cl-waffe2-simd.c:153-250; CFFI binding
 * cl-waffe2-simd/api.lisp:63-82).  IEEE binary32, no FMA contraction.
 * incx == 0 makes x[0] an accumulator (x[0] <- x[0] op y[0] op y[incy] ...):
 * add is tree-reduced unless wf2hip_set_reduce_mode(1); the others always run
 * in the reference's sequential order. */
int wf2hip_sadd(long n, float* x, long incx, const float* y, long incy);
int wf2hip_ssub(long n, float* x, long incx, const float* y, long incy);
int wf2hip_smul(long n, float* x, long incx, const float* y, long incy);
int wf2hip_sdiv(long n, float* x, long incx, const float* y, long incy);
/* x[i*incx] <- y[i*incy].  Replaces BLAS scopy_ as called by
 * expand-move-form (source/backends/cpu/arithmetic.lisp:39-61): source first. */
int wf2hip_scopy(long n, const float* y, long incy, float* x, long incx);
/* out[i*inco] <- f(x[i*incx]).  Replaces waffe2_s{sin,cos,tanh,log,exp,sqrt,abs}
 * (cl-waffe2-simd.c:586-706; api.lisp:212-251).  <= 2 ulp from SLEEF u10. */
int wf2hip_ssin(long n, const float* x, long incx, float* out, long inco);
int wf2hip_scos(long n, const float* x, long incx, float* out, long inco);
int wf2hip_stanh(long n, const float* x, long incx, float* out, long inco);
int wf2hip_slog(long n, const float* x, long incx, float* out, long inco);
int wf2hip_sexp(long n, const float* x, long incx, float* out, long inco);
int wf2hip_ssqrt(long n, const float* x, long incx, float* out, long inco);
int wf2hip_sabs(long n, const float* x, long incx, float* out, long inco);
/* The rest of define-math-impl's list (source/backends/cpu/mathematics.lisp:33-53): Tan, ASin,
 * ACos, ATan, SinH, CosH, Log2, Log10, Log1p (cl-waffe2-simd.c:650-694). */
int wf2hip_stan(long n, const float* x, long incx, float* out, long inco);
int wf2hip_sasin(long n, const float* x, long incx, float* out, long inco);
int wf2hip_sacos(long n, const float* x, long incx, float* out, long inco);
int wf2hip_satan(long n, const float* x, long incx, float* out, long inco);
int wf2hip_ssinh(long n, const float* x, long incx, float* out, long inco);
int wf2hip_scosh(long n, const float* x, long incx, float* out, long inco);
int wf2hip_slog2(long n, const float* x, long incx, float* out, long inco);
int wf2hip_slog10(long n, const float* x, long incx, float* out, long inco);
int wf2hip_slog1p(long n, const float* x, long incx, float* out, long inco);
/* x <- 1 / x in place (IEEE division; with incx == 0 the one element is inverted n times, as the
 * reference's loop does).  Replaces waffe2_sinv (cl-waffe2-simd.c:290-302; api.lisp:111-124). */
int wf2hip_sinv(long n, float* x, long incx);
/* out <- x^p.  Replaces waffe2_spow (cl-waffe2-simd.c:708-768; api.lisp:257-273). */
int wf2hip_spow(long n, const float* x, long incx, float p, float* out, long inco);
/* out[0] <- max/min_i x[i*incx].  Replaces waffe2_s{max,min}
 * (cl-waffe2-simd.c:316-365; api.lisp:126-141). */
int wf2hip_smax(long n, const float* x, long incx, float* out);
int wf2hip_smin(long n, const float* x, long incx, float* out);

/* ---- N-D view form: one launch per node -------------------------------- */
/* Replaces the host loops call-with-view emits around the 1-D kernels
 * (source/vm/generic-tensor/call-with-view.lisp:112-229,
 * do-compiled-loop.lisp:76-164): the whole iteration space of a node in one
 * descriptor.  For each axis r: extent shape[r]; stride_a/stride_b are the
 * EFFECTIVE strides of the two tensors (storage stride x view step, 0 for a
 * broadcast axis); off_a/off_b are the start offsets (tensor-initial-offset
 * plus stride x range-nth(view, 0) per axis). */
typedef struct wf2hip_view2 {
  int32_t rank; /* 1..WF2HIP_MAX_RANK */
  int32_t reserved;
  int64_t shape[WF2HIP_MAX_RANK];
  int64_t stride_a[WF2HIP_MAX_RANK];
  int64_t stride_b[WF2HIP_MAX_RANK];
  int64_t off_a;
  int64_t off_b;
} wf2hip_view2;

enum wf2hip_binary_op {
  WF2HIP_ADD = 0, /* AddNode  source/base-impl/arithmetic.lisp:57-103 */
  WF2HIP_SUB = 1, /* SubNode  */
  WF2HIP_MUL = 2, /* MulNode  */
  WF2HIP_DIV = 3, /* DivNode  */
  WF2HIP_MOVE = 4 /* MoveTensorNode source/base-impl/fundamental.lisp:9-43 */
};

enum wf2hip_unary_op {
  WF2HIP_SIN = 16, /* SinNode  source/base-impl/mathematics.lisp:13-120 */
  WF2HIP_COS = 17,
  WF2HIP_TANH = 18,
  WF2HIP_LOG = 19, /* LogENode */
  WF2HIP_EXP = 20,
  WF2HIP_SQRT = 21,
  WF2HIP_ABS = 22,
  WF2HIP_TAN = 23,
  WF2HIP_ASIN = 24,
  WF2HIP_ACOS = 25,
  WF2HIP_ATAN = 26,
  WF2HIP_SINH = 27,
  WF2HIP_COSH = 28,
  WF2HIP_LOG2 = 29,
  WF2HIP_LOG10 = 30,
  WF2HIP_LOG1P = 31,
  WF2HIP_POW = 32, /* ExptNode mathematics.lisp:267-303 */
  WF2HIP_INV = 33, /* 1 / x */
  WF2HIP_SIGN = 34,   /* SignNode: -1, +-0, 1 (CL signum; NaN stays NaN)  mathematics.lisp:131 */
  WF2HIP_SQUARE = 35, /* SquareNode: x * x                               mathematics.lisp:147 */
  WF2HIP_ASINH = 36,  /* ASinHNode, ACosHNode, ATanHNode: the inverse hyperbolic functions */
  WF2HIP_ACOSH = 37,  /* themselves (mathematics.lisp:217-219), not the hyperbolic ones the   */
  WF2HIP_ATANH = 38,  /* SIMD extension binds under these names (cl-waffe2-simd.c:672-679)     */
  WF2HIP_GELU = 40, /* fused tanh-form GELU (nn/activation.lisp:45-66) */
  WF2HIP_RELU = 41, /* fused !relu = x * (x > 0 ? 1 : 0) (nn/activation.lisp:11-25), bit-identical to the two nodes */
  WF2HIP_SIGMOID = 42, /* fused !sigmoid = 1 / (1 + exp(-1 x)) (nn/activation.lisp:27-43), each step rounded as its node */
  WF2HIP_LEAKY_RELU = 43 /* fused !leaky-relu = x * (x >= 0 ? 1 : p) (nn/activation.lisp:68-92); p = negative slope */
};

/* a <- a op b over the view (a = X, the in-place destination; b = Y).
 * Replaces the define-impl forwards of Add/Sub/Mul/Div/MoveTensorNode for
 * CPUTensor (source/backends/cpu/arithmetic.lisp:65-144).
 * Axes where stride_a == 0 and the extent is > 1 make `a` an accumulator:
 * that is how cl-waffe2 expresses !sum / !mean (base-impl/reduction.lisp:5-79).
 * WF2HIP_ADD reduces them in parallel (fp32 tree) unless reduce mode 1 is set;
 * SUB/MUL/DIV use the sequential order of the reference; MOVE keeps the last
 * element written, as a sequential loop would.
 * Returns WF2HIP_EOVERLAP when a and b are different, partially overlapping
 * windows of one buffer (the CPU result then depends on loop order). */
int wf2hip_binary_nd(int op, const wf2hip_view2* v, float* a, const float* b);
/* b <- f(a) over the view (a = X source, b = OUT).  Replaces the
 * define-math-impl forwards and ExptNode (source/backends/cpu/mathematics.lisp:
 * 8-76).  `p` is the exponent for WF2HIP_POW, the negative slope for
 * WF2HIP_LEAKY_RELU and ignored otherwise. */
int wf2hip_unary_nd(int op, const wf2hip_view2* v, const float* a, float* b, float p);

/* ---- the other element types -------------------------------------------- */
/* AddNode / SubNode / MulNode / DivNode / MoveTensorNode and inv for :double,
 * :int32, :uint32, :int16, :uint16, :int8 and :uint8 tensors.  Replace
 * waffe2_d{add,sub,mul,div} (cl-waffe2-simd.c:153-213 instantiated at :247-250),
 * waffe2_{i32,i16,i8,u32,u16,u8}{add,sub,mul,div,copy} (:214-288; api.lisp:63-109),
 * waffe2_{d,i32,...}inv (:290-310) and BLAS dcopy_ (source/backends/cpu/
 * arithmetic.lisp:39-61), same argument order: x[i*incx] <- x[i*incx] OP y[i*incy].
 * Integer arithmetic is C's (promotion to int, truncation on store, unsigned
 * wrap-around, division toward zero); where the reference traps -- a zero
 * divisor, INT_MIN / -1 -- the element becomes 0 / INT_MIN.  The 1-D :double
 * entry points reproduce the reference's remainder loop, which rounds through
 * binary32 (sas_dadd & co. return float, :229-232): the last n % 4 elements of a
 * call, and every element when incx < 1.  The N-D entry point computes every
 * element in binary64.  A destination with stride-0 axes accumulates (what !sum
 * composes): ADD as a tree per destination element -- exact for the integer types,
 * whose sums wrap modulo 2^bits in any order, binary64 partial sums for :double --
 * and SUB / MUL / DIV (or ADD after wf2hip_set_reduce_mode(1)) in the reference's
 * sequential order. */
enum wf2hip_dtype {
  WF2HIP_F64 = 1,
  WF2HIP_I32 = 2,
  WF2HIP_U32 = 3,
  WF2HIP_I16 = 4,
  WF2HIP_U16 = 5,
  WF2HIP_I8 = 6,
  WF2HIP_U8 = 7
};
int wf2hip_binary_1d_typed(int dtype, int op, long n, void* x, long incx, const void* y, long incy);
int wf2hip_binary_nd_typed(int dtype, int op, const wf2hip_view2* v, void* a, const void* b);
int wf2hip_inv_1d_typed(int dtype, long n, void* x, long incx);
int wf2hip_dcopy(long n, const double* y, long incy, double* x, long incx);
int wf2hip_dadd(long n, double* x, long incx, const double* y, long incy);
int wf2hip_dsub(long n, double* x, long incx, const double* y, long incy);
int wf2hip_dmul(long n, double* x, long incx, const double* y, long incy);
int wf2hip_ddiv(long n, double* x, long incx, const double* y, long incy);
int wf2hip_dinv(long n, double* x, long incx);
int wf2hip_i32add(long n, int32_t* x, long incx, const int32_t* y, long incy);
int wf2hip_i32sub(long n, int32_t* x, long incx, const int32_t* y, long incy);
int wf2hip_i32mul(long n, int32_t* x, long incx, const int32_t* y, long incy);
int wf2hip_i32div(long n, int32_t* x, long incx, const int32_t* y, long incy);
int wf2hip_i32copy(long n, int32_t* x, long incx, const int32_t* y, long incy);
int wf2hip_i32inv(long n, int32_t* x, long incx);
int wf2hip_u32add(long n, uint32_t* x, long incx, const uint32_t* y, long incy);
int wf2hip_u32sub(long n, uint32_t* x, long incx, const uint32_t* y, long incy);
int wf2hip_u32mul(long n, uint32_t* x, long incx, const uint32_t* y, long incy);
int wf2hip_u32div(long n, uint32_t* x, long incx, const uint32_t* y, long incy);
int wf2hip_u32copy(long n, uint32_t* x, long incx, const uint32_t* y, long incy);
int wf2hip_u32inv(long n, uint32_t* x, long incx);
int wf2hip_i16add(long n, int16_t* x, long incx, const int16_t* y, long incy);
int wf2hip_i16sub(long n, int16_t* x, long incx, const int16_t* y, long incy);
int wf2hip_i16mul(long n, int16_t* x, long incx, const int16_t* y, long incy);
int wf2hip_i16div(long n, int16_t* x, long incx, const int16_t* y, long incy);
int wf2hip_i16copy(long n, int16_t* x, long incx, const int16_t* y, long incy);
int wf2hip_i16inv(long n, int16_t* x, long incx);
int wf2hip_u16add(long n, uint16_t* x, long incx, const uint16_t* y, long incy);
int wf2hip_u16sub(long n, uint16_t* x, long incx, const uint16_t* y, long incy);
int wf2hip_u16mul(long n, uint16_t* x, long incx, const uint16_t* y, long incy);
int wf2hip_u16div(long n, uint16_t* x, long incx, const uint16_t* y, long incy);
int wf2hip_u16copy(long n, uint16_t* x, long incx, const uint16_t* y, long incy);
int wf2hip_u16inv(long n, uint16_t* x, long incx);
int wf2hip_i8add(long n, int8_t* x, long incx, const int8_t* y, long incy);
int wf2hip_i8sub(long n, int8_t* x, long incx, const int8_t* y, long incy);
int wf2hip_i8mul(long n, int8_t* x, long incx, const int8_t* y, long incy);
int wf2hip_i8div(long n, int8_t* x, long incx, const int8_t* y, long incy);
int wf2hip_i8copy(long n, int8_t* x, long incx, const int8_t* y, long incy);
int wf2hip_i8inv(long n, int8_t* x, long incx);
int wf2hip_u8add(long n, uint8_t* x, long incx, const uint8_t* y, long incy);
int wf2hip_u8sub(long n, uint8_t* x, long incx, const uint8_t* y, long incy);
int wf2hip_u8mul(long n, uint8_t* x, long incx, const uint8_t* y, long incy);
int wf2hip_u8div(long n, uint8_t* x, long incx, const uint8_t* y, long incy);
int wf2hip_u8copy(long n, uint8_t* x, long incx, const uint8_t* y, long incy);
int wf2hip_u8inv(long n, uint8_t* x, long incx);

/* ---- row selection: max / min value and index ----------------------------- */
/* For every row of the `outer` space (a = X, b = OUT, in elements; use rank 1,
 * extent 1 for a single run): OUT <- max / min of the run x[i * incx], i < n, or
 * its index as a uint32.  Replaces the forwards of MaxValue-Node, MinValue-Node,
 * ArgMax-Node and ArgMin-Node (source/backends/cpu/matrix-ops.lisp:240-369), which
 * call waffe2_s{max,min} (cl-waffe2-simd.c:316-365) or BLAS i?max / i?min once
 * per row.  Ties go to the lowest index; NaN elements are never selected. */
enum wf2hip_select_op { WF2HIP_MAXVALUE = 48, WF2HIP_MINVALUE = 49, WF2HIP_ARGMAX = 50, WF2HIP_ARGMIN = 51 };
int wf2hip_select_nd(int op, const wf2hip_view2* outer, long n, long incx, const float* x, void* out);
/* The same on the other element types (dtype: enum wf2hip_dtype, declared with the
 * typed arithmetic below): MaxValue-Node / MinValue-Node for every dtype -- the CPU
 * backend calls waffe2_<prefix>{max,min} per row (source/backends/cpu/matrix-ops.lisp:
 * 323-369; cl-waffe2-simd.c:316-365) -- with OUT of the same dtype, ArgMax-Node /
 * ArgMin-Node for :double only (BLAS idmax / idmin, matrix-ops.lisp:254-266; any other
 * dtype is an error there and WF2HIP_EUNSUPPORTED here).  The 1-D names keep the
 * reference's arguments: out[0] <- the extreme of the n elements. */
int wf2hip_select_nd_typed(int dtype, int op, const wf2hip_view2* outer, long n, long incx, const void* x,
                           void* out);
int wf2hip_dmax(long n, const double* x, long incx, double* out);
int wf2hip_dmin(long n, const double* x, long incx, double* out);
int wf2hip_i32max(long n, const int32_t* x, long incx, int32_t* out);
int wf2hip_i32min(long n, const int32_t* x, long incx, int32_t* out);
int wf2hip_u32max(long n, const uint32_t* x, long incx, uint32_t* out);
int wf2hip_u32min(long n, const uint32_t* x, long incx, uint32_t* out);
int wf2hip_i16max(long n, const int16_t* x, long incx, int16_t* out);
int wf2hip_i16min(long n, const int16_t* x, long incx, int16_t* out);
int wf2hip_u16max(long n, const uint16_t* x, long incx, uint16_t* out);
int wf2hip_u16min(long n, const uint16_t* x, long incx, uint16_t* out);
int wf2hip_i8max(long n, const int8_t* x, long incx, int8_t* out);
int wf2hip_i8min(long n, const int8_t* x, long incx, int8_t* out);
int wf2hip_u8max(long n, const uint8_t* x, long incx, uint8_t* out);
int wf2hip_u8min(long n, const uint8_t* x, long incx, uint8_t* out);

/* ---- compare / where ---------------------------------------------------- */
/* out <- (x OP y) ? then_value : else_value.  OP is ordered: false when an
 * operand is NaN (the reference uses _CMP_*_OQ, avx2.h:179-230). */
enum wf2hip_compare_op { WF2HIP_EQ = 0, WF2HIP_LT = 1, WF2HIP_LE = 2, WF2HIP_GT = 3, WF2HIP_GE = 4 };

/* 1-D forms.  Replace waffe2_s{eq,lt,le,gt,ge} (cl-waffe2-simd.c:385-468;
 * api.lisp:143-175) and waffe2_s{eq,lt,le,gt,ge}_scal (cl-waffe2-simd.c:474-560;
 * api.lisp:177-209), same argument order.  With inco == 0 `out` keeps the last
 * element's result, as the reference's sequential loop leaves it. */
int wf2hip_seq(long n, const float* x, long incx, const float* y, long incy, float* out, long inco,
               float then_value, float else_value);
int wf2hip_slt(long n, const float* x, long incx, const float* y, long incy, float* out, long inco,
               float then_value, float else_value);
int wf2hip_sle(long n, const float* x, long incx, const float* y, long incy, float* out, long inco,
               float then_value, float else_value);
int wf2hip_sgt(long n, const float* x, long incx, const float* y, long incy, float* out, long inco,
               float then_value, float else_value);
int wf2hip_sge(long n, const float* x, long incx, const float* y, long incy, float* out, long inco,
               float then_value, float else_value);
int wf2hip_seq_scal(long n, const float* x, long incx, float* out, long inco, float y,
                    float then_value, float else_value);
int wf2hip_slt_scal(long n, const float* x, long incx, float* out, long inco, float y,
                    float then_value, float else_value);
int wf2hip_sle_scal(long n, const float* x, long incx, float* out, long inco, float y,
                    float then_value, float else_value);
int wf2hip_sgt_scal(long n, const float* x, long incx, float* out, long inco, float y,
                    float then_value, float else_value);
int wf2hip_sge_scal(long n, const float* x, long incx, float* out, long inco, float y,
                    float then_value, float else_value);

/* Three tensors over one iteration space (a = X, b = Y, c = OUT), in elements. */
typedef struct wf2hip_view3 {
  int32_t rank; /* 1..WF2HIP_MAX_RANK */
  int32_t reserved;
  int64_t shape[WF2HIP_MAX_RANK];
  int64_t stride_a[WF2HIP_MAX_RANK];
  int64_t stride_b[WF2HIP_MAX_RANK];
  int64_t stride_c[WF2HIP_MAX_RANK];
  int64_t off_a, off_b, off_c;
} wf2hip_view3;

/* N-D forms, one launch per node.  wf2hip_where_nd replaces the forward of
 * Where-Operation-Node (source/backends/cpu/logical.lisp:37-60; view: a = X,
 * b = OUT), wf2hip_compare_nd that of Compare-Operation-Node (logical.lisp:
 * 62-84).  Stride-0 axes of OUT keep the last element written. */
int wf2hip_where_nd(int op, const wf2hip_view2* v, const float* x, float* out, float scal,
                    float then_value, float else_value);
int wf2hip_compare_nd(int op, const wf2hip_view3* v, const float* x, const float* y, float* out,
                      float then_value, float else_value);

/* Unary math on :double tensors: replace waffe2_d{sin,cos,tan,asin,acos,atan,sinh,cosh,
 * tanh,log,log2,log10,log1p,exp,sqrt,abs} (cl-waffe2-simd.c:586-706, SLEEF u10 on blocks of
 * four, libm on the remainder) and waffe2_dpow (:708-768), same argument order; `op` of the
 * N-D form is an enum wf2hip_unary_op (SIN ... POW), view a = X, b = OUT.  Every element
 * goes through the device math library's binary64 routine: within 2 ulp of SLEEF u10.
 * Other element types have no unary math in the reference either (WF2HIP_EUNSUPPORTED). */
int wf2hip_unary_nd_typed(int dtype, int op, const wf2hip_view2* v, const void* x, void* out, double p);
int wf2hip_dsin(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dcos(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dtanh(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dlog(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dexp(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dsqrt(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dabs(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dtan(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dasin(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dacos(long n, const double* x, long incx, double* out, long inco);
int wf2hip_datan(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dsinh(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dcosh(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dlog2(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dlog10(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dlog1p(long n, const double* x, long incx, double* out, long inco);
int wf2hip_dpow(long n, const double* x, long incx, double p, double* out, long inco);

/* Compare-Operation-Node / Where-Operation-Node on the other element types: x, y,
 * out, the scalar and the two constants all have the element type `dtype`
 * (enum wf2hip_dtype).  Replace waffe2_{d,i32,i16,i8,u32,u16,u8}{eq,lt,le,gt,ge}
 * (cl-waffe2-simd.c:385-468) and ..._scal (:474-560), which the CPU backend calls
 * for every dtype (source/backends/cpu/logical.lisp:26-84).  The N-D forms take
 * the constants as double (exact for every element type here) and compare in the
 * element type's own order.  The 1-D names keep the reference's argument order
 * and its results bit for bit, including this: its 256-bit body orders :uint32 /
 * :uint16 / :uint8 lanes as SIGNED integers (simd/x86_64/avx2.h:198-239 bind the
 * unsigned names to _mm256_cmpgt_epi*), so with inco >= 1 the leading
 * (n / lanes) * lanes elements of a call (lanes = 32 bytes / element size) compare
 * that way and only the remainder as unsigned; with inco < 1 every element takes
 * the scalar loop. */
int wf2hip_compare_nd_typed(int dtype, int op, const wf2hip_view3* v, const void* x, const void* y, void* out,
                            double then_value, double else_value);
int wf2hip_where_nd_typed(int dtype, int op, const wf2hip_view2* v, const void* x, void* out, double scal,
                          double then_value, double else_value);
int wf2hip_deq(long n, const double* x, long incx, const double* y, long incy, double* out, long inco,
               double then_value, double else_value);
int wf2hip_dlt(long n, const double* x, long incx, const double* y, long incy, double* out, long inco,
               double then_value, double else_value);
int wf2hip_dle(long n, const double* x, long incx, const double* y, long incy, double* out, long inco,
               double then_value, double else_value);
int wf2hip_dgt(long n, const double* x, long incx, const double* y, long incy, double* out, long inco,
               double then_value, double else_value);
int wf2hip_dge(long n, const double* x, long incx, const double* y, long incy, double* out, long inco,
               double then_value, double else_value);
int wf2hip_deq_scal(long n, const double* x, long incx, double* out, long inco, double y,
                    double then_value, double else_value);
int wf2hip_dlt_scal(long n, const double* x, long incx, double* out, long inco, double y,
                    double then_value, double else_value);
int wf2hip_dle_scal(long n, const double* x, long incx, double* out, long inco, double y,
                    double then_value, double else_value);
int wf2hip_dgt_scal(long n, const double* x, long incx, double* out, long inco, double y,
                    double then_value, double else_value);
int wf2hip_dge_scal(long n, const double* x, long incx, double* out, long inco, double y,
                    double then_value, double else_value);
int wf2hip_i32eq(long n, const int32_t* x, long incx, const int32_t* y, long incy, int32_t* out, long inco,
               int32_t then_value, int32_t else_value);
int wf2hip_i32lt(long n, const int32_t* x, long incx, const int32_t* y, long incy, int32_t* out, long inco,
               int32_t then_value, int32_t else_value);
int wf2hip_i32le(long n, const int32_t* x, long incx, const int32_t* y, long incy, int32_t* out, long inco,
               int32_t then_value, int32_t else_value);
int wf2hip_i32gt(long n, const int32_t* x, long incx, const int32_t* y, long incy, int32_t* out, long inco,
               int32_t then_value, int32_t else_value);
int wf2hip_i32ge(long n, const int32_t* x, long incx, const int32_t* y, long incy, int32_t* out, long inco,
               int32_t then_value, int32_t else_value);
int wf2hip_i32eq_scal(long n, const int32_t* x, long incx, int32_t* out, long inco, int32_t y,
                    int32_t then_value, int32_t else_value);
int wf2hip_i32lt_scal(long n, const int32_t* x, long incx, int32_t* out, long inco, int32_t y,
                    int32_t then_value, int32_t else_value);
int wf2hip_i32le_scal(long n, const int32_t* x, long incx, int32_t* out, long inco, int32_t y,
                    int32_t then_value, int32_t else_value);
int wf2hip_i32gt_scal(long n, const int32_t* x, long incx, int32_t* out, long inco, int32_t y,
                    int32_t then_value, int32_t else_value);
int wf2hip_i32ge_scal(long n, const int32_t* x, long incx, int32_t* out, long inco, int32_t y,
                    int32_t then_value, int32_t else_value);
int wf2hip_u32eq(long n, const uint32_t* x, long incx, const uint32_t* y, long incy, uint32_t* out, long inco,
               uint32_t then_value, uint32_t else_value);
int wf2hip_u32lt(long n, const uint32_t* x, long incx, const uint32_t* y, long incy, uint32_t* out, long inco,
               uint32_t then_value, uint32_t else_value);
int wf2hip_u32le(long n, const uint32_t* x, long incx, const uint32_t* y, long incy, uint32_t* out, long inco,
               uint32_t then_value, uint32_t else_value);
int wf2hip_u32gt(long n, const uint32_t* x, long incx, const uint32_t* y, long incy, uint32_t* out, long inco,
               uint32_t then_value, uint32_t else_value);
int wf2hip_u32ge(long n, const uint32_t* x, long incx, const uint32_t* y, long incy, uint32_t* out, long inco,
               uint32_t then_value, uint32_t else_value);
int wf2hip_u32eq_scal(long n, const uint32_t* x, long incx, uint32_t* out, long inco, uint32_t y,
                    uint32_t then_value, uint32_t else_value);
int wf2hip_u32lt_scal(long n, const uint32_t* x, long incx, uint32_t* out, long inco, uint32_t y,
                    uint32_t then_value, uint32_t else_value);
int wf2hip_u32le_scal(long n, const uint32_t* x, long incx, uint32_t* out, long inco, uint32_t y,
                    uint32_t then_value, uint32_t else_value);
int wf2hip_u32gt_scal(long n, const uint32_t* x, long incx, uint32_t* out, long inco, uint32_t y,
                    uint32_t then_value, uint32_t else_value);
int wf2hip_u32ge_scal(long n, const uint32_t* x, long incx, uint32_t* out, long inco, uint32_t y,
                    uint32_t then_value, uint32_t else_value);
int wf2hip_i16eq(long n, const int16_t* x, long incx, const int16_t* y, long incy, int16_t* out, long inco,
               int16_t then_value, int16_t else_value);
int wf2hip_i16lt(long n, const int16_t* x, long incx, const int16_t* y, long incy, int16_t* out, long inco,
               int16_t then_value, int16_t else_value);
int wf2hip_i16le(long n, const int16_t* x, long incx, const int16_t* y, long incy, int16_t* out, long inco,
               int16_t then_value, int16_t else_value);
int wf2hip_i16gt(long n, const int16_t* x, long incx, const int16_t* y, long incy, int16_t* out, long inco,
               int16_t then_value, int16_t else_value);
int wf2hip_i16ge(long n, const int16_t* x, long incx, const int16_t* y, long incy, int16_t* out, long inco,
               int16_t then_value, int16_t else_value);
int wf2hip_i16eq_scal(long n, const int16_t* x, long incx, int16_t* out, long inco, int16_t y,
                    int16_t then_value, int16_t else_value);
int wf2hip_i16lt_scal(long n, const int16_t* x, long incx, int16_t* out, long inco, int16_t y,
                    int16_t then_value, int16_t else_value);
int wf2hip_i16le_scal(long n, const int16_t* x, long incx, int16_t* out, long inco, int16_t y,
                    int16_t then_value, int16_t else_value);
int wf2hip_i16gt_scal(long n, const int16_t* x, long incx, int16_t* out, long inco, int16_t y,
                    int16_t then_value, int16_t else_value);
int wf2hip_i16ge_scal(long n, const int16_t* x, long incx, int16_t* out, long inco, int16_t y,
                    int16_t then_value, int16_t else_value);
int wf2hip_u16eq(long n, const uint16_t* x, long incx, const uint16_t* y, long incy, uint16_t* out, long inco,
               uint16_t then_value, uint16_t else_value);
int wf2hip_u16lt(long n, const uint16_t* x, long incx, const uint16_t* y, long incy, uint16_t* out, long inco,
               uint16_t then_value, uint16_t else_value);
int wf2hip_u16le(long n, const uint16_t* x, long incx, const uint16_t* y, long incy, uint16_t* out, long inco,
               uint16_t then_value, uint16_t else_value);
int wf2hip_u16gt(long n, const uint16_t* x, long incx, const uint16_t* y, long incy, uint16_t* out, long inco,
               uint16_t then_value, uint16_t else_value);
int wf2hip_u16ge(long n, const uint16_t* x, long incx, const uint16_t* y, long incy, uint16_t* out, long inco,
               uint16_t then_value, uint16_t else_value);
int wf2hip_u16eq_scal(long n, const uint16_t* x, long incx, uint16_t* out, long inco, uint16_t y,
                    uint16_t then_value, uint16_t else_value);
int wf2hip_u16lt_scal(long n, const uint16_t* x, long incx, uint16_t* out, long inco, uint16_t y,
                    uint16_t then_value, uint16_t else_value);
int wf2hip_u16le_scal(long n, const uint16_t* x, long incx, uint16_t* out, long inco, uint16_t y,
                    uint16_t then_value, uint16_t else_value);
int wf2hip_u16gt_scal(long n, const uint16_t* x, long incx, uint16_t* out, long inco, uint16_t y,
                    uint16_t then_value, uint16_t else_value);
int wf2hip_u16ge_scal(long n, const uint16_t* x, long incx, uint16_t* out, long inco, uint16_t y,
                    uint16_t then_value, uint16_t else_value);
int wf2hip_i8eq(long n, const int8_t* x, long incx, const int8_t* y, long incy, int8_t* out, long inco,
               int8_t then_value, int8_t else_value);
int wf2hip_i8lt(long n, const int8_t* x, long incx, const int8_t* y, long incy, int8_t* out, long inco,
               int8_t then_value, int8_t else_value);
int wf2hip_i8le(long n, const int8_t* x, long incx, const int8_t* y, long incy, int8_t* out, long inco,
               int8_t then_value, int8_t else_value);
int wf2hip_i8gt(long n, const int8_t* x, long incx, const int8_t* y, long incy, int8_t* out, long inco,
               int8_t then_value, int8_t else_value);
int wf2hip_i8ge(long n, const int8_t* x, long incx, const int8_t* y, long incy, int8_t* out, long inco,
               int8_t then_value, int8_t else_value);
int wf2hip_i8eq_scal(long n, const int8_t* x, long incx, int8_t* out, long inco, int8_t y,
                    int8_t then_value, int8_t else_value);
int wf2hip_i8lt_scal(long n, const int8_t* x, long incx, int8_t* out, long inco, int8_t y,
                    int8_t then_value, int8_t else_value);
int wf2hip_i8le_scal(long n, const int8_t* x, long incx, int8_t* out, long inco, int8_t y,
                    int8_t then_value, int8_t else_value);
int wf2hip_i8gt_scal(long n, const int8_t* x, long incx, int8_t* out, long inco, int8_t y,
                    int8_t then_value, int8_t else_value);
int wf2hip_i8ge_scal(long n, const int8_t* x, long incx, int8_t* out, long inco, int8_t y,
                    int8_t then_value, int8_t else_value);
int wf2hip_u8eq(long n, const uint8_t* x, long incx, const uint8_t* y, long incy, uint8_t* out, long inco,
               uint8_t then_value, uint8_t else_value);
int wf2hip_u8lt(long n, const uint8_t* x, long incx, const uint8_t* y, long incy, uint8_t* out, long inco,
               uint8_t then_value, uint8_t else_value);
int wf2hip_u8le(long n, const uint8_t* x, long incx, const uint8_t* y, long incy, uint8_t* out, long inco,
               uint8_t then_value, uint8_t else_value);
int wf2hip_u8gt(long n, const uint8_t* x, long incx, const uint8_t* y, long incy, uint8_t* out, long inco,
               uint8_t then_value, uint8_t else_value);
int wf2hip_u8ge(long n, const uint8_t* x, long incx, const uint8_t* y, long incy, uint8_t* out, long inco,
               uint8_t then_value, uint8_t else_value);
int wf2hip_u8eq_scal(long n, const uint8_t* x, long incx, uint8_t* out, long inco, uint8_t y,
                    uint8_t then_value, uint8_t else_value);
int wf2hip_u8lt_scal(long n, const uint8_t* x, long incx, uint8_t* out, long inco, uint8_t y,
                    uint8_t then_value, uint8_t else_value);
int wf2hip_u8le_scal(long n, const uint8_t* x, long incx, uint8_t* out, long inco, uint8_t y,
                    uint8_t then_value, uint8_t else_value);
int wf2hip_u8gt_scal(long n, const uint8_t* x, long incx, uint8_t* out, long inco, uint8_t y,
                    uint8_t then_value, uint8_t else_value);
int wf2hip_u8ge_scal(long n, const uint8_t* x, long incx, uint8_t* out, long inco, uint8_t y,
                    uint8_t then_value, uint8_t else_value);

/* 0 (default): parallel tree reduction for accumulate-into-stride-0 ADD.
 * 1: the reference's strictly sequential fp32 order (slow; for bit parity). */
int wf2hip_set_reduce_mode(int mode);
int wf2hip_get_reduce_mode(void);

/* ---- reductions and softmax as direct entry points ---------------------- */
/* a <- (sum of b over the axes on which a has stride 0 and an extent above 1)
 * / divisor, one node for what (!sum x :axis ..) and (!mean x :axis ..) compose
 * from a zero fill (MulNode by 0), AddNode into the (:broadcast n) view of
 * `out` and, for !mean, DivNode by the element count
 * (base-impl/reduction.lisp:5-79 and :81-136).  `a` is overwritten: its old
 * content is not read, so it needs no zero fill.  The bits are those of the
 * composition on a zeroed `out`: the sum rounded to binary32 once (reduce mode
 * 0) or added in the reference's sequential binary32 order (reduce mode 1),
 * then an IEEE binary32 division by `divisor` (pass 1 for !sum). */
int wf2hip_sum_nd(const wf2hip_view2* v, float* a, const float* b, float divisor);
/* out[r*inco] <- out[r*inco] + sum_c x[r*ldx + c], r < rows, c < cols.
 * What (!sum x :axis -1) lowers to after its zero-fill
 * (base-impl/reduction.lisp:5-79). */
int wf2hip_reduce_add_rows_f32(long rows, long cols, const float* x, long ldx,
                               float* out, long inco);
/* The same row sums through an entry point that allocates nothing.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  Same arguments, same kernels and bit-identical results as
 * wf2hip_reduce_add_rows_f32; the partial sums of rows that are split over
 * several workgroups go to a 256 KiB static device array (one copy per GPU,
 * held until the process ends) instead of a buffer the library allocates.
 * rows * cols above WF2HIP_NOALLOC_MAX_ELEMENTS returns WF2HIP_EUNSUPPORTED.
 * Every call on a GPU shares that GPU's array: calls that overlap in time on
 * one GPU (two streams, two host threads) race; nothing in the array has to
 * start at zero, each launch writes every partial sum it later reads. */
#define WF2HIP_NOALLOC_MAX_ELEMENTS (1LL << 32)
int wf2hip_reduce_add_rows_f32_noalloc(long rows, long cols, const float* x, long ldx,
                                       float* out, long inco);
/* out[r*ldo + c] <- softmax over c of x[r*ldx + c], max-subtracted.
 * One fused kernel for what !softmax composes from mean/sub/exp/sum/div
 * (source/nn/activation.lisp:126-159). */
int wf2hip_softmax_rows_f32(long rows, long cols, const float* x, long ldx,
                            float* out, long ldo);
/* Causal variant for attention scores: row r of each (seq x seq) matrix keeps
 * columns c <= r; x is (batch, seq, seq) contiguous, scaled by `scale` first. */
int wf2hip_causal_softmax_f32(long batch, long seq, const float* x, float* out,
                              float scale);
/* LayerNorm over the last axis: out = (x - mean)/sqrt(var + eps) * g + b
 * (source/nn/norms.lisp:44-82; examples/gpt-2/utils.lisp:114-127).  Rows beyond
 * 8192 columns run in pieces of 16384 columns over several workgroups: two
 * launches (one where all pieces fit on the device at once and x and out are
 * apart) and 16 bytes per piece of scratch from the library's pool. */
int wf2hip_layernorm_rows_f32(long rows, long cols, const float* x, const float* gamma,
                              const float* beta, float eps, float* out);
/* Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:90-126) over the last axis
 * in one pass: z[r, c] <- softmax over c of x[r, c] (max-subtracted, the bits of
 * wf2hip_softmax_rows_f32; the node saves it for its backward) and
 * loss[r, c] <- -1 * (labels[r, c] * log(z[r, c] + delta)), each operation
 * rounded to binary32 like the nodes of cross-entropy-loss (criterion.lisp:158).
 * All four arrays are contiguous (rows, cols); z and loss overlap neither the
 * inputs nor each other (WF2HIP_EOVERLAP).  The reductions :sum / :mean stay
 * outside the node, as in the reference (criterion.lisp:192-196). */
int wf2hip_softmax_cross_entropy_f32(long rows, long cols, const float* x,
                                     const float* labels, float delta, float* z,
                                     float* loss);

/* ---- backward of the fused layers ------------------------------------------ */
/* The reference differentiates !softmax, LayerNorm and the activations through
 * their node compositions (defnode backward of every node in
 * source/nn/activation.lisp:11-159 and source/nn/norms.lisp:72-82; the gradient
 * of a composition is again a composition, source/vm/nodes/defnode.lisp:383-393).
 * These entries are the backward of the one-kernel forms above, each one pass. */
/* dx[r*lddx + c] <- scale * y[r*ldy + c] * (dy[r*lddy + c] - sum_k dy[r, k] y[r, k]):
 * the gradient of y = softmax(scale * x) over the last axis from the saved output.
 * causal_seq = 0: plain rows.  causal_seq = cols: rows of (seq x seq) matrices whose
 * row r keeps columns c <= r % seq; dy is not read above the diagonal (it may be
 * uninitialised there) and dx is 0 there.  dx may be dy (same pitch). */
int wf2hip_softmax_backward_rows_f32(long rows, long cols, const float* y, long ldy,
                                     const float* dy, long lddy, float* dx, long lddx,
                                     float scale, long causal_seq);
/* The backward of Softmax-Cross-Entropy-Node, sce-diff-static
 * (source/nn/criterion.lisp:82-88, 103-110): dx[i] <- (dy[i] * (z[i] - labels[i])) / batch
 * for i < n, the SubNode, MulNode and DivNode of the reference in one pass with
 * the same binary32 roundings.  `batch` is the second-to-last extent of z as a
 * float.  dy_is_scalar != 0: dy points to ONE float on the device that every
 * element uses (the gradient a !sum or !mean of the loss hands down through its
 * broadcasting view).  dx may be dy or z; it overlaps nothing else. */
int wf2hip_softmax_cross_entropy_backward_f32(long n, const float* dy, int dy_is_scalar,
                                              const float* z, const float* labels,
                                              float batch, float* dx);
/* Gradients of wf2hip_layernorm_rows_f32 from the saved input: with
 * xh = (x - mean) rstd and dyh = dy gamma,
 *   dx = rstd (dyh - mean(dyh) - xh mean(dyh xh)),
 *   dgamma[c] = sum over rows of dy xh,  dbeta[c] = sum over rows of dy.
 * Contiguous (rows, cols) operands of any width: up to 8192 columns one row
 * kernel and two small folds; beyond that (and beyond 2048 columns that are no
 * multiple of 4 or lie off a 16-byte boundary) the row in pieces of 16384
 * columns over several workgroups, three row kernels.  dx may be dy.  Allocates
 * 8 * cols bytes per workgroup of scratch from the library's pool (and 32 bytes
 * per piece for rows in pieces). */
int wf2hip_layernorm_backward_f32(long rows, long cols, const float* x, const float* gamma,
                                  const float* dy, float eps, float* dx, float* dgamma,
                                  float* dbeta);
/* dout <- dout * f'(x) in place, f one of WF2HIP_RELU, WF2HIP_LEAKY_RELU (slope p),
 * WF2HIP_SIGMOID, WF2HIP_GELU (tanh form): the MulNode of the upstream gradient
 * with the derivative recipe of source/nn/activation.lisp:11-92 as one kernel.
 * The view's `a` side describes dout, its `b` side x.  ReLU, leaky ReLU and the
 * sigmoid give the bits of the composed recipe; GELU's derivative is
 * s (1 + x (1 - s) 2 u'), s = sigmoid(2 u), to 1e-6 of |s| + |x s (1 - s) 2 u'|. */
int wf2hip_activation_backward_nd(int op, const wf2hip_view2* v, float* dout, const float* x,
                                  float p);

/* ---- gemm ---------------------------------------------------------------- */
/* Column-major C(m x n) <- alpha op(A) op(B) + beta C with the argument
 * meaning of Fortran sgemm_, scalars by value.  Replaces the BLAS call of
 * expand-gemm-form-column/-row (source/backends/cpu/matrix-ops.lisp:12-212;
 * binding source/backends/cpu/blas-functions.lisp:34-38).  fp32 MFMA. */
int wf2hip_sgemm(char transa, char transb, long m, long n, long k, float alpha,
                 const float* A, long lda, const float* B, long ldb, float beta,
                 float* C, long ldc);
/* Same product for `batch` matrices strideA/strideB/strideC elements apart
 * (stride 0 re-uses one operand): the host loop over batch axes that
 * call-with-view :at-least-dim 2 emits (matrix-ops.lisp:214-237), in one
 * launch. */
int wf2hip_sgemm_strided_batched(char transa, char transb, long m, long n, long k,
                                 float alpha, const float* A, long lda, long strideA,
                                 const float* B, long ldb, long strideB, float beta,
                                 float* C, long ldc, long strideC, long batch);

/* Two batch axes (matrix z = outer * batch + inner; strides *2 belong to the
 * outer axis): heads read in place from a fused (B, T, 3, H, hd) projection
 * have batch strides that do not merge into one. */
int wf2hip_sgemm_strided_batched_2d(char transa, char transb, long m, long n, long k,
                                    float alpha, const float* A, long lda, long strideA,
                                    long strideA2, const float* B, long ldb, long strideB,
                                    long strideB2, float beta, float* C, long ldc, long strideC,
                                    long strideC2, long batch, long batch2);

/* The :double product: Fortran dgemm_ with scalars by value, the other branch
 * of the same expansion (matrix-ops.lisp:12-112 picks sgemm_ or dgemm_ by
 * dtype; blas-functions.lisp:34-38).  On the binary64 matrix cores
 * (v_mfma_f64_16x16x4), 128 x 128 (or 64 x 64) x 16 LDS tiles per workgroup; at
 * most 65535 matrices per call. */
int wf2hip_dgemm(char transa, char transb, long m, long n, long k, double alpha,
                 const double* A, long lda, const double* B, long ldb, double beta,
                 double* C, long ldc);
int wf2hip_dgemm_strided_batched_2d(char transa, char transb, long m, long n, long k,
                                    double alpha, const double* A, long lda, long strideA,
                                    long strideA2, const double* B, long ldb, long strideB,
                                    long strideB2, double beta, double* C, long ldc, long strideC,
                                    long strideC2, long batch, long batch2);

/* ---- fused matmul (extension; no BLAS counterpart) ------------------------- */
/* Row-major C[m,n] = act(alpha * op(A)[m,k] . op(B)[k,n] + bias[n]) + residual[m,n]
 * in one kernel: the bias add, GELU and residual add that cl-waffe2 runs as
 * separate AddNode / !gelu passes after MatMulNode (examples/gpt-2/model.lisp:
 * 109-137), applied in the same order and the same binary32 arithmetic, so the
 * result is bit-identical to the unfused sequence.  The route for it on the
 * Lisp side is define-bypass (source/vm/nodes/symbolic.lisp:118-131).
 * causal 1: only entries with col <= row are needed (attention scores before a
 * causal softmax): tiles wholly above the diagonal are neither computed nor
 * written.  causal 2: op(A) is lower-triangular (causal attention
 * probabilities): the K loop of each row tile stops at its last row.
 * Leading dimensions are row pitches; stride_*2 belong to the outer batch axis. */
typedef struct wf2hip_matmul_desc {
  int32_t trans_a;    /* A stored [k][m] */
  int32_t trans_b;    /* B stored [n][k] */
  int32_t activation; /* 0 none, 1 tanh-form GELU (nn/activation.lisp:45-66) */
  int32_t causal;     /* 0, 1 or 2, see above */
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  int64_t batch, batch2;
  int64_t stride_a, stride_a2, stride_b, stride_b2, stride_c, stride_c2;
  const float* bias;     /* n floats or NULL */
  const float* residual; /* [m][ld_residual] per matrix or NULL */
  int64_t ld_residual, stride_residual, stride_residual2;
  float alpha;
  int32_t reserved;
} wf2hip_matmul_desc;
int wf2hip_matmul_fused(const wf2hip_matmul_desc* desc, const float* A, const float* B, float* C);

/* ---- unfold / fold --------------------------------------------------------- */
/* Col[N C K_H K_W H_out W_out] <- X[N C H W] (X already padded) and its adjoint
 * X <- sum of the columns.  Replace waffe2_im2col_s_column / waffe2_col2im_s_column
 * (cl-waffe2-simd/kernels/im2col.c:63-115, 395-448), same argument order and the
 * same walk: for kernel offset k the positions k, k + stride, ... below
 * dilation * k - pad + stride * out are visited.  Elements of Col the walk does
 * not reach keep their values (with a padding argument the call may read them and
 * store them back unchanged, so Col must be readable and nothing else may write
 * it during the call); col2im overwrites X and accumulates in the
 * reference's order (kernel rows, then kernel columns, ascending).  Geometries
 * whose walk would leave its plane of Col (dilation > 1) return
 * WF2HIP_EUNSUPPORTED.  Tensors in cl-waffe2's default (:column) order. */
int wf2hip_im2col_f32(float* col, long N, long C, long H, long W, long H_out, long W_out, long K_H,
                      long K_W, long pad_h, long pad_w, long stride_h, long stride_w,
                      long dilation_h, long dilation_w, const float* im);
int wf2hip_col2im_f32(const float* col, long N, long C, long H, long W, long H_out, long W_out,
                      long K_H, long K_W, long pad_h, long pad_w, long stride_h, long stride_w,
                      long dilation_h, long dilation_w, float* im);
/* (unfold input dilation kernel-size stride padding) of source/nn/im2col.lisp:51-95
 * with dilation 1 as one kernel: out[(n i j), (c kh kw)], a row-major
 * (N H_out W_out) x (C K_H K_W) matrix, from the unpadded image x[N C H W], with
 * H_out = (H + 2 pad_h - K_H) / stride_h + 1 (conv-out-size, source/nn/pool.lisp:10-17)
 * and W_out likewise.  Bit for bit what the reference's composition leaves in a
 * fresh matrix: the zero padding, Im2ColNode's walk (positions it does not reach
 * hold 0), the permuting copy and the reshape.  Its backward is the reference's own
 * (permute back, wf2hip_col2im_f32, the interior of the padded image).
 * WF2HIP_EUNSUPPORTED when one channel of one output row does not fit the kernel's
 * staging memory (compose it from the nodes then). */
int wf2hip_unfold_f32(long N, long C, long H, long W, long K_H, long K_W, long stride_h,
                      long stride_w, long pad_h, long pad_w, const float* x, float* out);

/* ---- optimiser steps (extension) ------------------------------------------ */
/* One pass per parameter tensor, performing the binary32 operations of the
 * reference's node compositions in the same order, so the result is
 * bit-identical to running those nodes one by one.  Contiguous, non-overlapping
 * buffers of n elements.
 * SGD (source/optimizers/impls/sgd.lisp:18-34): grad <- grad * lr (the reference
 * scales the gradient in place), param <- param - grad.
 * Adam (source/optimizers/impls/adam.lisp:45-117): m <- m + (g - m) * (1 - beta1);
 * v <- v + (1 - beta2) * (g * g - v); param <- param - (m * lr_t) / (eps + sqrt(v)),
 * with lr_t = lr * sqrt(1 - beta2^t) / (1 - beta1^t) computed by the caller
 * (adam-step-lr, adam.lisp:78-92) and 1 - beta rounded to binary32 by the caller. */
int wf2hip_sgd_step_f32(long n, float* param, float* grad, float lr);
int wf2hip_adam_step_f32(long n, float* param, const float* grad, float* m, float* v,
                         float one_minus_beta1, float one_minus_beta2, float lr_t, float eps);

/* ---- attention (extension; no BLAS counterpart) ---------------------------- */
/* O[b,h,i,:] = sum_j softmax_j(scale * Q[b,h,i,:].K[b,h,j,:] (+ causal mask j <= i)) V[b,h,j,:]
 * in one kernel, replacing the node sequence !matmul, scalar multiply, mask add,
 * !softmax, !matmul of cl-waffe2's SelfAttention (examples/gpt-2/utils.lisp:
 * 222-243) without materialising the (batch, heads, seq, seq) scores.  Softmax is
 * the max-subtracted form.  head_dim: a multiple of 4, at most 64 (narrower heads
 * run zero-padded to 64).  Each operand is addressed as
 * base[b * stride[0] + h * stride[1] + i * stride[2] + c], c < head_dim with unit
 * stride, so heads can be read in place from a fused (B, T, 3, H, 64) projection
 * and O written directly as (B, T, H * 64).  Pointers 16-byte aligned, strides
 * multiples of 4 elements; O may not overlap an input (WF2HIP_EOVERLAP).
 * Result: within 1e-5 of the float64 value relative to max |V|. */
typedef struct wf2hip_attention_desc {
  int64_t batch, heads, seq, head_dim;
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3]; /* batch, head, position */
  float scale;    /* multiplies Q.K before the softmax, e.g. 1/sqrt(head_dim) */
  int32_t causal; /* 1: position i attends to j <= i only */
} wf2hip_attention_desc;
int wf2hip_attention_f32(const wf2hip_attention_desc* desc, const float* q, const float* k,
                         const float* v, float* o);
/* The same forward pass that also leaves, per (batch, head, query), the base-2 logarithm
 * of the row sum of exp2(scale log2(e) Q.K) in lse[(b * heads + h) * seq + i] (contiguous;
 * may be NULL): with it the backward pass forms the probabilities of any tile directly. */
int wf2hip_attention_forward_f32(const wf2hip_attention_desc* desc, const float* q, const float* k,
                                 const float* v, float* o, float* lse);
/* dQ, dK, dV of that forward pass from Q, K, V, its output O, the upstream gradient dO and
 * lse, without materialising a (seq, seq) tensor: the backward of the !matmul / !softmax /
 * !matmul chain (MatMulNode's backward, source/base-impl/matrix-ops.lisp:10-15; !softmax's
 * through its composition, source/nn/activation.lisp:126-159) in two launches
 * (D = sum_d dO O per query; then workgroups with queries resident that form dQ and
 * workgroups with keys resident that form dK and dV, handed out longest first).
 * dO is addressed through o_stride; dQ, dK, dV through q_stride, k_stride, v_stride, so they
 * can be windows of one fused-projection gradient.  The gradients may not overlap anything
 * that is read.  Allocates 4 * batch * heads * seq bytes of scratch from the library's pool.
 * Result: within 1e-5 of the float64 gradients relative to the magnitude their last
 * product adds up. */
int wf2hip_attention_backward_f32(const wf2hip_attention_desc* desc, const float* q, const float* k,
                                  const float* v, const float* o, const float* dout,
                                  const float* lse, float* dq, float* dk, float* dv);

/* ---- GPT-2 example: token + position embedding ------------------------------ */
/* out[r, :] <- wte[round(ctx[r]), :] + wpe[r % seq, :] for r < rows (rows = sentences x seq):
 * the GPT2PositionalEmbedding node of examples/gpt-2/utils.lisp:19-110, which the example
 * implements for LispTensor only (a zero fill and two waffe2_sadd calls per position).
 * ctx holds token ids as floats, rounded to nearest (ties to even, as ROUND) and clamped to
 * [0, vocab); wte is (vocab, dim), wpe (n_ctx, dim), out (rows, dim), all contiguous;
 * seq <= n_ctx.  Bit-exact: one binary32 add per element. */
int wf2hip_embedding_add_f32(long rows, long seq, long dim, const float* ctx, const float* wte,
                             long vocab, const float* wpe, long n_ctx, float* out);

#ifdef __cplusplus
}
#endif
#endif /* WAFFE2_HIP_H */
