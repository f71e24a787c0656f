/*
 * waffe2_oracle.c -- CPU restatement of cl-waffe2's CPUTensor + cl-waffe2-simd
 * tensor-kernel path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against (tests, the smoke check and the CPU-baseline leg of the
 * benchmark).  Nothing in the shipped library may call, link or fall back to
 * it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the cl-waffe2 checkout).  The arithmetic is plain C compiled with
 * -ffp-contract=off so that + - * / are single IEEE-754 binary32 operations,
 * exactly as _mm256_{add,sub,mul,div}_ps are in the reference.
 *
 * Third-party arithmetic that is NOT in the reference checkout:
 *   - SLEEF (un-vendored submodule third_party/sleef, no commit pin): the
 *     unary math kernels call Sleef_<f>f8_u10avx2.  The oracle resolves those
 *     very symbols at run time from a library that exports SLEEF 3.8.0
 *     (PyTorch's libtorch_cpu.so); when none is found it falls back to libm in
 *     double precision and orc_sleef_available() returns 0 so that the caller
 *     can say so.
 *   - BLAS sgemm_/scopy_ (system libblas, unpinned; CI installs netlib
 *     reference BLAS): restated here from the published netlib reference
 *     algorithm (column-major, j-l-i loop nest for 'N','N').
 *
 * Pinning status (which independent check covers each function) is recorded
 * in tests/test_oracle_*.py:
 *   orc_s{add,sub,mul,div}, orc_scopy  : golden vectors from the compiled
 *       reference C (tests/golden), numpy IEEE closed form, reference test
 *       vectors 10 op 1 -> 11/9/10/10.
 *   orc_s{exp,log,tanh,sin,sqrt}, orc_spow : golden vectors from the compiled
 *       reference C; float64 truth within 1 ulp; special values.
 *   orc_s{max,min}                     : golden vectors, numpy max/min.
 *   orc_schedule / orc_*_nd            : worked schedules derived by hand from
 *       do-compiled-loop.lisp, exactly-once coverage invariant, brute-force
 *       N-D index walk on random tiny views.
 *   orc_binary_typed, orc_inv_typed    : golden vectors from the compiled
 *       reference C (waffe2_d*, waffe2_{i32,...}*), numpy closed forms (integer
 *       wrap-around, binary64 arithmetic, the binary32 round trip of the tail).
 *   orc_cmp_typed                      : golden vectors from the compiled
 *       reference C (waffe2_{d,i32,...}{eq,...} and ..._scal), numpy closed forms
 *       (the element type's own order on the remainder, the signed order on the
 *       leading blocks of the unsigned types).
 *   orc_dunary                         : golden vectors from the compiled
 *       reference C (waffe2_d{sin,...,pow}, bit for bit where SLEEF resolves);
 *       float64 closed forms (numpy / libm within 1 ulp), special values.
 *   orc_extreme_typed                  : golden vectors from the compiled
 *       reference C (waffe2_{d,i32,...}{max,min}), numpy max / min.
 *   orc_sgemm                          : the reference's integer gemm vectors
 *       (base-impl/t/arithmetic.lisp:120,135,142,148), float64 truth.
 */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))
#define ORC_SIMD 8 /* SIMD_SINGLE_STRIDE, simd/x86_64/avx2.h:26 */

/* ------------------------------------------------------------------ */
/* SLEEF resolution                                                    */
/* ------------------------------------------------------------------ */

typedef float v8f __attribute__((vector_size(32)));
typedef v8f (*sleef_f8_1)(v8f);
typedef v8f (*sleef_f8_2)(v8f, v8f);

static void *g_sleef_handle = NULL;
static int g_sleef_tried = 0;

ORC_API int orc_sleef_open(const char *path) {
  g_sleef_tried = 1;
  g_sleef_handle = dlopen(path, RTLD_NOW | RTLD_GLOBAL);
  if (!g_sleef_handle) return 0;
  if (!dlsym(g_sleef_handle, "Sleef_expf8_u10avx2")) {
    g_sleef_handle = NULL;
    return 0;
  }
  return 1;
}

ORC_API int orc_sleef_available(void) { return g_sleef_handle != NULL; }

static void *sleef_sym(const char *name) {
  if (!g_sleef_handle) return NULL;
  return dlsym(g_sleef_handle, name);
}

/* ------------------------------------------------------------------ */
/* x <- x op y   (cl-waffe2-simd.c:153-250, define_arithmetic_func)     */
/* ------------------------------------------------------------------ */
/* The reference handles incx >= 1 in blocks of 8 (load 8 x, load 8 y,
 * compute, store 8) and everything else -- the n%8 tail, and the whole range
 * when incx <= 0 -- with a sequential scalar loop (:205-212).  incx == 0 is
 * therefore a strictly sequential accumulate into x[0]. */
#define ORC_DEFINE_ARITH(name, OP)                                            \
  ORC_API void orc_s##name(long n, float *x, long incx, const float *y,      \
                           long incy) {                                       \
    long count = 0;                                                           \
    const long simd_end = (n / ORC_SIMD) * ORC_SIMD;                          \
    if (incx >= 1) {                                                          \
      while (count != simd_end) {                                             \
        float vx[ORC_SIMD], vy[ORC_SIMD];                                     \
        for (int i = 0; i < ORC_SIMD; i++) vx[i] = x[(count + i) * incx];     \
        for (int i = 0; i < ORC_SIMD; i++) vy[i] = y[(count + i) * incy];     \
        for (int i = 0; i < ORC_SIMD; i++) vx[i] = vx[i] OP vy[i];            \
        for (int i = 0; i < ORC_SIMD; i++) x[(count + i) * incx] = vx[i];     \
        count += ORC_SIMD;                                                    \
      }                                                                       \
    }                                                                         \
    x += count * incx;                                                        \
    y += count * incy;                                                        \
    while (count != n) {                                                      \
      count += 1;                                                             \
      x[0] = x[0] OP y[0];                                                    \
      x += incx;                                                              \
      y += incy;                                                              \
    }                                                                         \
  }

ORC_DEFINE_ARITH(add, +)
ORC_DEFINE_ARITH(sub, -)
ORC_DEFINE_ARITH(mul, *)
ORC_DEFINE_ARITH(div, /)

/* x <- y strided copy.  backends/cpu/arithmetic.lisp:39-61 passes
 * (n, y, incy, x, incx) to BLAS scopy_, i.e. source first.  Netlib scopy
 * with non-negative increments is a plain strided copy. */
ORC_API void orc_scopy(long n, const float *y, long incy, float *x, long incx) {
  for (long i = 0; i < n; i++) x[i * incx] = y[i * incy];
}

/* ------------------------------------------------------------------ */
/* out <- f(x)   (cl-waffe2-simd.c:586-706, define_math_func)           */
/* ------------------------------------------------------------------ */
/* Blocks of 8 go through SLEEF u10 when incx >= 1; the tail and the whole
 * range when incx <= 0 use libm in double precision, narrowed to float
 * (:636-641: `y[0] = sin(x[0])` with float operands promotes to double). */
static void unary_apply(long n, const float *x, long incx, float *out,
                        long inco, const char *sleef_name,
                        double (*libm_f)(double)) {
  long count = 0;
  const long simd_end = (n / ORC_SIMD) * ORC_SIMD;
  sleef_f8_1 vf = (sleef_f8_1)sleef_sym(sleef_name);
  if (incx >= 1) {
    while (count != simd_end) {
      float in[ORC_SIMD] __attribute__((aligned(32)));
      float res[ORC_SIMD] __attribute__((aligned(32)));
      for (int i = 0; i < ORC_SIMD; i++) in[i] = x[(count + i) * incx];
      if (vf) {
        v8f v;
        memcpy(&v, in, sizeof v);
        v = vf(v);
        memcpy(res, &v, sizeof v);
      } else {
        for (int i = 0; i < ORC_SIMD; i++) res[i] = (float)libm_f((double)in[i]);
      }
      for (int i = 0; i < ORC_SIMD; i++) out[(count + i) * inco] = res[i];
      count += ORC_SIMD;
    }
  }
  x += count * incx;
  out += count * inco;
  while (count != n) {
    count += 1;
    out[0] = (float)libm_f((double)x[0]);
    x += incx;
    out += inco;
  }
}

#define ORC_DEFINE_UNARY(name, sleef, libm)                                  \
  ORC_API void orc_s##name(long n, const float *x, long incx, float *out,   \
                           long inco) {                                      \
    unary_apply(n, x, incx, out, inco, sleef, libm);                         \
  }

/* avx2.h:265,291,308,322,325 and cl-waffe2-simd.c:645,670,685,697,703 */
ORC_DEFINE_UNARY(sin, "Sleef_sinf8_u10avx2", sin)
ORC_DEFINE_UNARY(cos, "Sleef_cosf8_u10avx2", cos)
ORC_DEFINE_UNARY(tanh, "Sleef_tanhf8_u10avx2", tanh)
ORC_DEFINE_UNARY(log, "Sleef_logf8_u10avx2", log)
ORC_DEFINE_UNARY(exp, "Sleef_expf8_u10avx2", exp)
ORC_DEFINE_UNARY(sqrt, "Sleef_sqrtf8_u05avx2", sqrt)
ORC_DEFINE_UNARY(abs, "Sleef_fabsf8_avx2", fabs)
ORC_DEFINE_UNARY(tan, "Sleef_tanf8_u10avx2", tan)
ORC_DEFINE_UNARY(asin, "Sleef_asinf8_u10avx2", asin)
ORC_DEFINE_UNARY(acos, "Sleef_acosf8_u10avx2", acos)
ORC_DEFINE_UNARY(atan, "Sleef_atanf8_u10avx2", atan)
ORC_DEFINE_UNARY(sinh, "Sleef_sinhf8_u10avx2", sinh)
ORC_DEFINE_UNARY(cosh, "Sleef_coshf8_u10avx2", cosh)
ORC_DEFINE_UNARY(log2, "Sleef_log2f8_u10avx2", log2)
ORC_DEFINE_UNARY(log10, "Sleef_log10f8_u10avx2", log10)
ORC_DEFINE_UNARY(log1p, "Sleef_log1pf8_u10avx2", log1p)

/* SignNode, SquareNode, ASinHNode, ACosHNode, ATanHNode have no CPUTensor implementation:
 * they run LispTensor's per-element loop y[offy + incy i] <- f(x[offx + incx i])
 * (source/backends/lisp/mathematics.lisp:11-45) with f = signum, (* x x), asinh, acosh,
 * atanh of Common Lisp (:48,52,:66-68 of the same file).  CL's functions are restated by
 * their definitions: signum keeps +-0 (and NaN), the inverse hyperbolic functions of a
 * single-float are the mathematical ones rounded to binary32, evaluated here in binary64
 * by libm.  PARITY UNPINNED BY THE REFERENCE beyond its own one-point test
 * (mathematical-test-set at x = 1, source/base-impl/t/mathematical.lisp:37-162): no
 * Common Lisp implementation is available to produce vectors; pinned by float64 closed
 * forms (tests/test_oracle_golden.py). */
static float lisp_signum(float x) { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : x); }
#define ORC_DEFINE_LISP_UNARY(name, expr)                                                       \
  ORC_API void orc_s##name(long n, const float *x, long incx, float *out, long inco) {          \
    for (long i = 0; i < n; i++) {                                                              \
      const float v = x[i * incx];                                                              \
      out[i * inco] = (expr);                                                                   \
    }                                                                                           \
  }
ORC_DEFINE_LISP_UNARY(sign, lisp_signum(v))
ORC_DEFINE_LISP_UNARY(square, v * v)
ORC_DEFINE_LISP_UNARY(asinh, (float)asinh((double)v))
ORC_DEFINE_LISP_UNARY(acosh, (float)acosh((double)v))
ORC_DEFINE_LISP_UNARY(atanh, (float)atanh((double)v))

/* out <- x^p  (cl-waffe2-simd.c:708-768; avx2.h:304) */
ORC_API void orc_spow(long n, const float *x, long incx, float p, float *out,
                      long inco) {
  long count = 0;
  const long simd_end = (n / ORC_SIMD) * ORC_SIMD;
  sleef_f8_2 vf = (sleef_f8_2)sleef_sym("Sleef_powf8_u10avx2");
  if (incx >= 1) {
    while (count != simd_end) {
      float in[ORC_SIMD], res[ORC_SIMD];
      for (int i = 0; i < ORC_SIMD; i++) in[i] = x[(count + i) * incx];
      if (vf) {
        v8f v, pv;
        memcpy(&v, in, sizeof v);
        for (int i = 0; i < ORC_SIMD; i++) pv[i] = p;
        v = vf(v, pv);
        memcpy(res, &v, sizeof v);
      } else {
        for (int i = 0; i < ORC_SIMD; i++)
          res[i] = (float)pow((double)in[i], (double)p);
      }
      for (int i = 0; i < ORC_SIMD; i++) out[(count + i) * inco] = res[i];
      count += ORC_SIMD;
    }
  }
  x += count * incx;
  out += count * inco;
  while (count != n) {
    count += 1;
    out[0] = (float)pow((double)x[0], (double)p);
    x += incx;
    out += inco;
  }
}

/* out[0] <- max/min over x  (cl-waffe2-simd.c:316-365).  _mm256_max_ps(a,b)
 * returns b when either operand is NaN; MAX(a,b) = a > b ? a : b. */
#define ORC_DEFINE_MAXMIN(name, CMP)                                          \
  ORC_API void orc_s##name(long n, const float *x, long incx, float *out) {  \
    float best = x[0];                                                        \
    float lanes[ORC_SIMD];                                                    \
    long count = 0;                                                           \
    const long simd_end = (n / ORC_SIMD) * ORC_SIMD;                          \
    for (int i = 0; i < ORC_SIMD; i++) lanes[i] = best;                       \
    while (count != simd_end) {                                               \
      for (int i = 0; i < ORC_SIMD; i++) {                                    \
        float v = x[(count + i) * incx];                                      \
        lanes[i] = (lanes[i] CMP v) ? lanes[i] : v;                           \
      }                                                                       \
      count += ORC_SIMD;                                                      \
    }                                                                         \
    for (int i = 0; i < ORC_SIMD; i++)                                        \
      best = (best CMP lanes[i]) ? best : lanes[i];                           \
    x += count * incx;                                                        \
    while (count != n) {                                                      \
      count += 1;                                                             \
      best = (best CMP x[0]) ? best : x[0];                                   \
      x += incx;                                                              \
    }                                                                         \
    out[0] = best;                                                            \
  }

ORC_DEFINE_MAXMIN(max, >)
ORC_DEFINE_MAXMIN(min, <)

/* ------------------------------------------------------------------ */
/* Loop scheduler                                                      */
/* ------------------------------------------------------------------ */
/* Restates solve-loop-order (vm/generic-tensor/do-compiled-loop.lisp:76-164)
 * with rest-contiguous-p (:46-73) and the emitter call-with-view
 * (call-with-view.lisp:112-229) for kernel rank 1 (element-wise), all tensors
 * sharing one permute order.
 *
 * A tensor axis is described by
 *   stride   the storage stride of the axis in elements
 *            (tensor-stride, utils.lisp:50-67)
 *   kind     0 = T (whole axis), 1 = (:broadcast n), 2 = anything else
 *            (index, slice, stepped slice; view.lisp:120-138)
 *   first    range-nth(view, 0)                 (iterator/range.lisp:74-98)
 *   step     range-nth(view, 1) - range-nth(view, 0)
 * and a tensor by its axes plus tensor-initial-offset.
 *
 * The result is the list of 1-D calls the compiled loop makes:
 *   (n, off_0, inc_0, off_1, inc_1, ...) per call, offsets in elements. */

#define ORC_MAX_RANK 8
#define ORC_MAX_TENSORS 3

typedef struct {
  int rank;
  int ntensors;
  long shape[ORC_MAX_RANK];
  long stride[ORC_MAX_TENSORS][ORC_MAX_RANK];
  int kind[ORC_MAX_TENSORS][ORC_MAX_RANK];
  long first[ORC_MAX_TENSORS][ORC_MAX_RANK];
  long step[ORC_MAX_TENSORS][ORC_MAX_RANK];
  long offset[ORC_MAX_TENSORS];
} orc_views;

typedef struct {
  long n;
  long off[ORC_MAX_TENSORS];
  long inc[ORC_MAX_TENSORS];
} orc_call;

/* rest-contiguous-p: from `rank` on, every view of every tensor is T or
 * broadcast, and within one tensor they all have the same type. */
static int rest_contiguous_p(const orc_views *v, int rank) {
  for (int t = 0; t < v->ntensors; t++) {
    for (int r = rank; r < v->rank; r++) {
      if (v->kind[t][r] != 0 && v->kind[t][r] != 1) return 0;
      if (v->kind[t][r] != v->kind[t][rank]) return 0;
    }
  }
  return 1;
}

typedef void (*orc_emit_fn)(const orc_call *c, void *ctx);

static void emit_rec(const orc_views *v, int rank, long *offsets,
                     orc_emit_fn emit, void *ctx) {
  if (rest_contiguous_p(v, rank)) {
    /* :apply-flatten (do-compiled-loop.lisp:113-137, call-with-view.lisp:
     * 160-195): one call over the product of the remaining extents; stride 1,
     * or 0 for a broadcast tensor.  Offsets add stride*range-nth(0) of every
     * remaining non-broadcast axis (all T here, so zero). */
    orc_call c;
    c.n = 1;
    for (int r = rank; r < v->rank; r++) c.n *= v->shape[r];
    for (int t = 0; t < v->ntensors; t++) {
      long off = offsets[t];
      for (int r = rank; r < v->rank; r++)
        if (v->kind[t][r] != 1) off += v->stride[t][r] * v->first[t][r];
      c.off[t] = off;
      c.inc[t] = (v->kind[t][rank] == 1) ? 0 : 1;
    }
    emit(&c, ctx);
    return;
  }
  if (v->rank - rank == 1) {
    /* :apply (do-compiled-loop.lisp:141-155): the innermost axis as one call
     * with size shape[last], stride = stride*step or 0 if broadcast. */
    orc_call c;
    c.n = v->shape[rank];
    for (int t = 0; t < v->ntensors; t++) {
      int bc = v->kind[t][rank] == 1;
      c.off[t] = offsets[t] + (bc ? 0 : v->stride[t][rank] * v->first[t][rank]);
      c.inc[t] = bc ? 0 : v->stride[t][rank] * v->step[t][rank];
    }
    emit(&c, ctx);
    return;
  }
  /* :batch (call-with-view.lisp:120-159): host loop over this axis; each
   * tensor's offset starts at stride*range-nth(0) and advances by
   * stride*(range-nth(1)-range-nth(0)) unless the axis is broadcast. */
  long local[ORC_MAX_TENSORS];
  for (int t = 0; t < v->ntensors; t++) {
    local[t] = offsets[t];
    if (v->kind[t][rank] != 1) local[t] += v->stride[t][rank] * v->first[t][rank];
  }
  for (long i = 0; i < v->shape[rank]; i++) {
    emit_rec(v, rank + 1, local, emit, ctx);
    for (int t = 0; t < v->ntensors; t++)
      if (v->kind[t][rank] != 1) local[t] += v->stride[t][rank] * v->step[t][rank];
  }
}

typedef struct {
  orc_call *out;
  long cap;
  long count;
} collect_ctx;

static void collect_emit(const orc_call *c, void *p) {
  collect_ctx *ctx = (collect_ctx *)p;
  if (ctx->count < ctx->cap) ctx->out[ctx->count] = *c;
  ctx->count++;
}

/* Returns the number of 1-D calls; writes at most `cap` of them. */
ORC_API long orc_schedule(const orc_views *v, orc_call *out, long cap) {
  collect_ctx ctx = {out, cap, 0};
  long offsets[ORC_MAX_TENSORS];
  for (int t = 0; t < v->ntensors; t++) offsets[t] = v->offset[t];
  if (v->rank == 0) return 0;
  emit_rec(v, 0, offsets, collect_emit, &ctx);
  return ctx.count;
}

/* N-D node execution = schedule + the 1-D kernel per call
 * (backends/cpu/arithmetic.lisp:32-37, 39-61; mathematics.lisp:8-32,55-76). */
typedef struct {
  int op;
  float *a;
  float *b;
  float p;
} exec_ctx;

enum {
  ORC_ADD = 0,
  ORC_SUB,
  ORC_MUL,
  ORC_DIV,
  ORC_MOVE,
  ORC_SIN = 16,
  ORC_COS,
  ORC_TANH,
  ORC_LOG,
  ORC_EXP,
  ORC_SQRT,
  ORC_ABS,
  ORC_TAN,
  ORC_ASIN,
  ORC_ACOS,
  ORC_ATAN,
  ORC_SINH,
  ORC_COSH,
  ORC_LOG2,
  ORC_LOG10,
  ORC_LOG1P,
  ORC_POW = 32
};

static void exec_emit(const orc_call *c, void *p) {
  exec_ctx *e = (exec_ctx *)p;
  float *a = e->a + c->off[0];
  float *b = e->b + c->off[1];
  switch (e->op) {
    case ORC_ADD: orc_sadd(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_SUB: orc_ssub(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_MUL: orc_smul(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_DIV: orc_sdiv(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_MOVE: orc_scopy(c->n, b, c->inc[1], a, c->inc[0]); break;
    /* unary: tensor 0 = x (source), tensor 1 = out */
    case ORC_SIN: orc_ssin(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_COS: orc_scos(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_TANH: orc_stanh(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_LOG: orc_slog(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_EXP: orc_sexp(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_SQRT: orc_ssqrt(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_ABS: orc_sabs(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_TAN: orc_stan(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_ASIN: orc_sasin(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_ACOS: orc_sacos(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_ATAN: orc_satan(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_SINH: orc_ssinh(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_COSH: orc_scosh(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_LOG2: orc_slog2(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_LOG10: orc_slog10(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_LOG1P: orc_slog1p(c->n, a, c->inc[0], b, c->inc[1]); break;
    case ORC_POW: orc_spow(c->n, a, c->inc[0], e->p, b, c->inc[1]); break;
    default: break;
  }
}

/* Binary/move: tensor 0 = x (destination, in place), tensor 1 = y.
 * Unary/pow: tensor 0 = x (source), tensor 1 = out. */
ORC_API long orc_node_nd(int op, const orc_views *v, float *t0, float *t1,
                         float p) {
  exec_ctx e = {op, t0, t1, p};
  long offsets[ORC_MAX_TENSORS];
  collect_ctx unused = {NULL, 0, 0};
  (void)unused;
  if (v->rank == 0 || v->ntensors != 2) return -1;
  for (int t = 0; t < v->ntensors; t++) offsets[t] = v->offset[t];
  emit_rec(v, 0, offsets, exec_emit, &e);
  return 0;
}

/* x <- 1 / x, element after element (cl-waffe2-simd.c:290-302): the literal
 * 1.0 is a double, so the division runs in binary64 and is rounded to binary32
 * (equal to a binary32 division: 53 >= 2 * 24 + 2). */
ORC_API void orc_sinv(long n, float *x, long incx) {
  for (long count = 0; count != n; count++) {
    x[0] = 1.0 / x[0];
    x += incx;
  }
}

/* ------------------------------------------------------------------ */
/* index of the largest / smallest value                               */
/* ------------------------------------------------------------------ */
/* ArgMax-Node / ArgMin-Node call BLAS i?max / i?min
 * (backends/cpu/blas-functions.lisp:16-21, matrix-ops.lisp:240-290): `ismax_` and
 * `ismin_` are OpenBLAS extensions (netlib BLAS only has isamax), the library is
 * whatever `libblas` the host provides and is not part of the reference tree.
 * Restated from their published behaviour: the 1-based position of the first
 * element holding the largest (smallest) value, found with a strict comparison.
 * Pinned by the definition (first occurrence on tie-rich data, numpy.argmax). */
ORC_API long orc_ismax(long n, const float *x, long incx) {
  if (n < 1) return 0;
  long best = 0;
  for (long i = 1; i < n; i++)
    if (x[i * incx] > x[best * incx]) best = i;
  return best + 1;
}

ORC_API long orc_ismin(long n, const float *x, long incx) {
  if (n < 1) return 0;
  long best = 0;
  for (long i = 1; i < n; i++)
    if (x[i * incx] < x[best * incx]) best = i;
  return best + 1;
}

/* ------------------------------------------------------------------ */
/* compare / where                                                     */
/* ------------------------------------------------------------------ */
/* out[i] = (x[i] OP y[i]) ? then : else  (cl-waffe2-simd.c:385-425, define_cmp)
 * and the scalar-right-hand-side form (cl-waffe2-simd.c:474-513, define_scmp).
 * The SIMD predicates are the ordered, quiet ones (avx2.h:179,192,205,218,230:
 * _CMP_EQ_OQ 0, _CMP_LT_OQ 17, _CMP_LE_OQ 18, _CMP_GE_OQ 29, _CMP_GT_OQ 30), i.e. what
 * the C operators of the scalar tail give: false whenever an operand is NaN.
 * With inco < 1 the block-of-8 part is skipped and every element is written
 * through the scalar loop, so a stride-0 `out` ends up holding the last one. */
enum { ORC_EQ = 0, ORC_LT, ORC_LE, ORC_GT, ORC_GE };

static int orc_cmp1(int op, float a, float b) {
  switch (op) {
    case ORC_EQ: return a == b;
    case ORC_LT: return a < b;
    case ORC_LE: return a <= b;
    case ORC_GT: return a > b;
    default: return a >= b;
  }
}

ORC_API void orc_scmp(int op, long n, const float *x, long incx, const float *y, long incy,
                      float *out, long inco, float then_value, float else_value) {
  long count = 0;
  if (inco >= 1) {
    const long blocks_end = (n / 8) * 8;
    for (; count != blocks_end; count += 8) {
      float res[8];
      for (int l = 0; l < 8; l++)
        res[l] = orc_cmp1(op, x[(count + l) * incx], y[(count + l) * incy]) ? then_value : else_value;
      for (int l = 0; l < 8; l++) out[(count + l) * inco] = res[l];
    }
  }
  for (; count != n; count++)
    out[count * inco] = orc_cmp1(op, x[count * incx], y[count * incy]) ? then_value : else_value;
}

ORC_API void orc_scmp_scal(int op, long n, const float *x, long incx, float *out, long inco,
                           float y, float then_value, float else_value) {
  long count = 0;
  if (inco >= 1) {
    const long blocks_end = (n / 8) * 8;
    for (; count != blocks_end; count += 8) {
      float res[8];
      for (int l = 0; l < 8; l++)
        res[l] = orc_cmp1(op, x[(count + l) * incx], y) ? then_value : else_value;
      for (int l = 0; l < 8; l++) out[(count + l) * inco] = res[l];
    }
  }
  for (; count != n; count++)
    out[count * inco] = orc_cmp1(op, x[count * incx], y) ? then_value : else_value;
}

/* Where-Operation-Node / Compare-Operation-Node over N-D views: the schedule of
 * do-compiled-loop with one 1-D call per row (backends/cpu/logical.lisp:37-84). */
typedef struct {
  int op;
  const float *x;
  const float *y;
  float *out;
  float scal, then_value, else_value;
} cmp_ctx;

static void where_emit(const orc_call *c, void *p) {
  cmp_ctx *e = (cmp_ctx *)p;
  orc_scmp_scal(e->op, c->n, e->x + c->off[0], c->inc[0], e->out + c->off[1], c->inc[1], e->scal,
                e->then_value, e->else_value);
}

static void compare_emit(const orc_call *c, void *p) {
  cmp_ctx *e = (cmp_ctx *)p;
  orc_scmp(e->op, c->n, e->x + c->off[0], c->inc[0], e->y + c->off[1], c->inc[1],
           e->out + c->off[2], c->inc[2], e->then_value, e->else_value);
}

/* tensors of `v`: 0 = x, 1 = out */
ORC_API long orc_where_nd(int op, const orc_views *v, const float *x, float *out, float scal,
                          float then_value, float else_value) {
  cmp_ctx e = {op, x, NULL, out, scal, then_value, else_value};
  long offsets[ORC_MAX_TENSORS];
  if (v->rank == 0 || v->ntensors != 2) return -1;
  for (int t = 0; t < v->ntensors; t++) offsets[t] = v->offset[t];
  emit_rec(v, 0, offsets, where_emit, &e);
  return 0;
}

/* tensors of `v`: 0 = x, 1 = y, 2 = out */
ORC_API long orc_compare_nd(int op, const orc_views *v, const float *x, const float *y, float *out,
                            float then_value, float else_value) {
  cmp_ctx e = {op, x, y, out, 0.0f, then_value, else_value};
  long offsets[ORC_MAX_TENSORS];
  if (v->rank == 0 || v->ntensors != 3) return -1;
  for (int t = 0; t < v->ntensors; t++) offsets[t] = v->offset[t];
  emit_rec(v, 0, offsets, compare_emit, &e);
  return 0;
}

/* ------------------------------------------------------------------ */
/* im2col / col2im                                                     */
/* ------------------------------------------------------------------ */
/* cl-waffe2-simd/kernels/im2col.c:63-115 (waffe2_im2col_s_column) and 395-448
 * (waffe2_col2im_s_column): X[N C H W] <-> Col[N C K_H K_W H_out W_out].  The walk
 * over image rows starts at the kernel offset itself and ends below
 * dilation * k - pad + stride * out (evaluated in uint64 like the reference);
 * col2im clears X first and accumulates in loop order. */
typedef unsigned long long orc_u64;

static void orc_unfold_walk(int fold, float *col, orc_u64 N, orc_u64 C, orc_u64 H, orc_u64 W,
                            orc_u64 H_out, orc_u64 W_out, orc_u64 K_H, orc_u64 K_W, orc_u64 pad_h,
                            orc_u64 pad_w, orc_u64 s_h, orc_u64 s_w, orc_u64 d_h, orc_u64 d_w,
                            float *im) {
  for (orc_u64 n = 0; n < N; n++)
    for (orc_u64 kh = 0; kh < K_H; kh++) {
      const orc_u64 h_end = d_h * kh - pad_h + s_h * H_out;
      for (orc_u64 kw = 0; kw < K_W; kw++) {
        const orc_u64 w_end = d_w * kw - pad_w + s_w * W_out;
        orc_u64 i = 0;
        for (orc_u64 y = kh; y < h_end; y += s_h, i++) {
          orc_u64 j = 0;
          for (orc_u64 x = kw; x < w_end; x += s_w, j++)
            for (orc_u64 c = 0; c < C; c++) {
              float *cp = col + ((((n * C + c) * K_H + kh) * K_W + kw) * H_out + i) * W_out + j;
              float *ip = im + ((n * C + c) * H + y) * W + x;
              if (fold)
                *ip += *cp;
              else
                *cp = *ip;
            }
        }
      }
    }
}

ORC_API void orc_im2col(float *col, orc_u64 N, orc_u64 C, orc_u64 H, orc_u64 W, orc_u64 H_out,
                        orc_u64 W_out, orc_u64 K_H, orc_u64 K_W, orc_u64 pad_h, orc_u64 pad_w,
                        orc_u64 s_h, orc_u64 s_w, orc_u64 d_h, orc_u64 d_w, const float *im) {
  orc_unfold_walk(0, col, N, C, H, W, H_out, W_out, K_H, K_W, pad_h, pad_w, s_h, s_w, d_h, d_w,
                  (float *)im);
}

ORC_API void orc_col2im(const float *col, orc_u64 N, orc_u64 C, orc_u64 H, orc_u64 W, orc_u64 H_out,
                        orc_u64 W_out, orc_u64 K_H, orc_u64 K_W, orc_u64 pad_h, orc_u64 pad_w,
                        orc_u64 s_h, orc_u64 s_w, orc_u64 d_h, orc_u64 d_w, float *im) {
  for (orc_u64 i = 0; i < N * C * H * W; i++) im[i] = 0.0f;
  orc_unfold_walk(1, (float *)col, N, C, H, W, H_out, W_out, K_H, K_W, pad_h, pad_w, s_h, s_w, d_h,
                  d_w, im);
}

/* ------------------------------------------------------------------ */
/* sgemm                                                               */
/* ------------------------------------------------------------------ */
/* Column-major C(m x n) <- alpha*op(A)*op(B) + beta*C with Fortran sgemm_
 * argument meaning (backends/cpu/blas-functions.lisp:34-38,
 * backends/cpu/blas.lisp:76-92), restated from the netlib reference BLAS loop
 * nests (fp32 accumulation in the order l = 0..k-1). */
ORC_API void orc_sgemm(char transa, char transb, long m, long n, long k,
                       float alpha, const float *A, long lda, const float *B,
                       long ldb, float beta, float *C, long ldc) {
  const int nota = (transa == 'N' || transa == 'n');
  const int notb = (transb == 'N' || transb == 'n');
  for (long j = 0; j < n; j++) {
    if (nota) {
      for (long i = 0; i < m; i++)
        C[i + j * ldc] = (beta == 0.0f) ? 0.0f : beta * C[i + j * ldc];
      for (long l = 0; l < k; l++) {
        float temp = alpha * (notb ? B[l + j * ldb] : B[j + l * ldb]);
        for (long i = 0; i < m; i++) C[i + j * ldc] += temp * A[i + l * lda];
      }
    } else {
      for (long i = 0; i < m; i++) {
        float temp = 0.0f;
        for (long l = 0; l < k; l++)
          temp += A[l + i * lda] * (notb ? B[l + j * ldb] : B[j + l * ldb]);
        C[i + j * ldc] =
            (beta == 0.0f) ? alpha * temp : alpha * temp + beta * C[i + j * ldc];
      }
    }
  }
}

/* Row-major C[m,n] = A[m,k] . B[k,n] the way expand-gemm-form-column calls
 * it (backends/cpu/matrix-ops.lisp:12-112): operands swapped,
 * sgemm_(transB, transA, n, m, k, 1, B, ldb, A, lda, 0, C, ldc), where the
 * leading dimensions are the last-axis sizes of the untransposed tensors. */
ORC_API void orc_matmul_rowmajor(int trans_a, int trans_b, long m, long n,
                                 long k, const float *A, long lda,
                                 const float *B, long ldb, float *C, long ldc) {
  orc_sgemm(trans_b ? 'C' : 'N', trans_a ? 'C' : 'N', n, m, k, 1.0f, B, ldb, A,
            lda, 0.0f, C, ldc);
}


/* ------------------------------------------------------------------ */
/* The other element types                                             */
/* ------------------------------------------------------------------ */
/* waffe2_d{add,sub,mul,div}: define_arithmetic_func at SIMD_DOUBLE_STRIDE = 4
 * (cl-waffe2-simd.c:153-213, instantiated :247-250).  The vector body handles
 * (n / 4) * 4 elements when incx >= 1 in binary64; the remainder loop calls
 * sas_d{add,sub,mul,div}, declared `float static inline` (:229-232), so those
 * elements are rounded to binary32 on the way back.
 * waffe2_{i32,...}{add,sub,mul,div,copy}: define_arithmetic_scal_func, plain C
 * loops (:214-288).  Integer overflow wraps (two's complement, what the
 * reference's compiled code does); a zero divisor and INT_MIN / -1 trap there
 * and are left to the caller to avoid.
 * dtype codes: 1 double, 2 int32, 3 uint32, 4 int16, 5 uint16, 6 int8, 7 uint8;
 * op codes: 0 add, 1 sub, 2 mul, 3 div, 4 copy. */
static double orc_dop(int op, double a, double b) {
  switch (op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    case 3: return a / b;
    default: return b;
  }
}

#define ORC_INT_LOOP(T, W, U)                                          \
  {                                                                    \
    T *xp = (T *)x;                                                    \
    const T *yp = (const T *)y;                                        \
    for (long c = 0; c < n; c++) {                                     \
      W a = (W)xp[0], b = (W)yp[0];                                    \
      switch (op) {                                                    \
        case 0: xp[0] = (T)(U)((U)a + (U)b); break;                    \
        case 1: xp[0] = (T)(U)((U)a - (U)b); break;                    \
        case 2: xp[0] = (T)(U)((U)a * (U)b); break;                    \
        case 3: xp[0] = (T)(a / b); break;                             \
        default: xp[0] = yp[0]; break;                                 \
      }                                                                \
      xp += incx;                                                      \
      yp += incy;                                                      \
    }                                                                  \
  }

ORC_API int orc_binary_typed(int dtype, int op, long n, void *x, long incx, const void *y, long incy) {
  if (op < 0 || op > 4) return -1;
  switch (dtype) {
    case 1: {
      double *xp = (double *)x;
      const double *yp = (const double *)y;
      long count = 0;
      if (op == 4) { /* dcopy_ (BLAS): no arithmetic */
        for (long c = 0; c < n; c++) xp[c * incx] = yp[c * incy];
        return 0;
      }
      if (incx >= 1) {
        const long simd_end = (n / 4) * 4;
        for (; count < simd_end; count++) xp[count * incx] = orc_dop(op, xp[count * incx], yp[count * incy]);
      }
      xp += count * incx;
      yp += count * incy;
      for (; count < n; count++) {
        xp[0] = (double)(float)orc_dop(op, xp[0], yp[0]); /* sas_d*: float return type */
        xp += incx;
        yp += incy;
      }
      return 0;
    }
    case 2: ORC_INT_LOOP(int32_t, int32_t, uint32_t) return 0;
    case 3: ORC_INT_LOOP(uint32_t, uint32_t, uint32_t) return 0;
    case 4: ORC_INT_LOOP(int16_t, int, unsigned) return 0;
    case 5: ORC_INT_LOOP(uint16_t, int, unsigned) return 0;
    case 6: ORC_INT_LOOP(int8_t, int, unsigned) return 0;
    case 7: ORC_INT_LOOP(uint8_t, int, unsigned) return 0;
    default: return -1;
  }
}

/* waffe2_{d,i32,...}inv: x[0] = 1 / x[0] (cl-waffe2-simd.c:290-310) */
ORC_API int orc_inv_typed(int dtype, long n, void *x, long incx) {
#define ORC_INV(T, ONE)                      \
  {                                          \
    T *xp = (T *)x;                          \
    for (long c = 0; c < n; c++) {           \
      xp[0] = (T)(ONE / xp[0]);              \
      xp += incx;                            \
    }                                        \
    return 0;                                \
  }
  switch (dtype) {
    case 1: ORC_INV(double, 1.0)
    case 2: ORC_INV(int32_t, 1)
    case 3: ORC_INV(uint32_t, 1)
    case 4: ORC_INV(int16_t, 1)
    case 5: ORC_INV(uint16_t, 1)
    case 6: ORC_INV(int8_t, 1)
    case 7: ORC_INV(uint8_t, 1)
    default: return -1;
  }
#undef ORC_INV
}

/* waffe2_{d,i32,i16,i8,u32,u16,u8}{eq,lt,le,gt,ge} and ..._scal
 * (cl-waffe2-simd.c:385-468 define_cmp, :474-560 define_scmp): the block part
 * (inco >= 1, blocks of 32 bytes / element size) compares through the AVX2 lane
 * predicates, the remainder through the C operators.  For the unsigned types the
 * lane predicates are the SIGNED ones (simd/x86_64/avx2.h:198-200 lt, :211-213 gt,
 * :224-226 le = not gt, :237-239 ge = not gt swapped, all on _mm256_cmpgt_epi*);
 * eq is sign-agnostic.  `scal` != 0 selects the scalar right-hand side `ys`. */
#define ORC_CMPV(op, a, b) \
  ((op) == ORC_EQ ? (a) == (b) : (op) == ORC_LT ? (a) < (b) : (op) == ORC_LE ? (a) <= (b) : (op) == ORC_GT ? (a) > (b) : (a) >= (b))

#define ORC_CMP_LOOP(T, S)                                                                     \
  {                                                                                            \
    const T *xp = (const T *)x, *yp = (const T *)y;                                            \
    T *outp = (T *)out;                                                                        \
    const T tv = (T)then_value, ev = (T)else_value, yv = (T)ys;                                \
    const long lanes = 32 / (long)sizeof(T);                                                   \
    long count = 0;                                                                            \
    if (inco >= 1) {                                                                           \
      const long blocks_end = (n / lanes) * lanes;                                             \
      for (; count != blocks_end; count += lanes) {                                            \
        T res[32];                                                                             \
        for (long l = 0; l < lanes; l++) {                                                     \
          const S a = (S)xp[(count + l) * incx];                                               \
          const S b = (S)(scal ? yv : yp[(count + l) * incy]);                                 \
          res[l] = ORC_CMPV(op, a, b) ? tv : ev;                                               \
        }                                                                                      \
        for (long l = 0; l < lanes; l++) outp[(count + l) * inco] = res[l];                    \
      }                                                                                        \
    }                                                                                          \
    for (; count != n; count++) {                                                              \
      const T a = xp[count * incx];                                                            \
      const T b = scal ? yv : yp[count * incy];                                                \
      outp[count * inco] = ORC_CMPV(op, a, b) ? tv : ev;                                       \
    }                                                                                          \
    return 0;                                                                                  \
  }

ORC_API int orc_cmp_typed(int dtype, int op, long n, const void *x, long incx, const void *y, long incy, void *out,
                          long inco, int scal, double ys, double then_value, double else_value) {
  if (op < ORC_EQ || op > ORC_GE) return -1;
  switch (dtype) {
    case 1: ORC_CMP_LOOP(double, double)
    case 2: ORC_CMP_LOOP(int32_t, int32_t)
    case 3: ORC_CMP_LOOP(uint32_t, int32_t)
    case 4: ORC_CMP_LOOP(int16_t, int16_t)
    case 5: ORC_CMP_LOOP(uint16_t, int16_t)
    case 6: ORC_CMP_LOOP(int8_t, int8_t)
    case 7: ORC_CMP_LOOP(uint8_t, int8_t)
    default: return -1;
  }
}

/* waffe2_{d,i32,i16,i8,u32,u16,u8}{max,min} (cl-waffe2-simd.c:316-365, define_maxmin):
 * `lanes` running extremes over blocks of 32 bytes / element size, folded, then the
 * remainder.  Exact for the integer types in any order; for :double the lane
 * operation is _mm256_max_pd / _mm256_min_pd (the second operand when either is
 * NaN) and the folds use MAX / MIN (a > b ? a : b). */
#define ORC_EXTREME_LOOP(T)                                                          \
  {                                                                                  \
    const T *xp = (const T *)x;                                                      \
    const long lanes = 32 / (long)sizeof(T);                                         \
    T lane[32], best = xp[0];                                                        \
    long count = 0;                                                                  \
    const long blocks_end = (n / lanes) * lanes;                                     \
    for (long l = 0; l < lanes; l++) lane[l] = best;                                 \
    for (; count != blocks_end; count += lanes)                                      \
      for (long l = 0; l < lanes; l++) {                                             \
        const T v = xp[(count + l) * incx];                                          \
        lane[l] = is_max ? (lane[l] > v ? lane[l] : v) : (lane[l] < v ? lane[l] : v); \
      }                                                                              \
    for (long l = 0; l < lanes; l++)                                                 \
      best = is_max ? (best > lane[l] ? best : lane[l]) : (best < lane[l] ? best : lane[l]); \
    for (; count != n; count++) {                                                    \
      const T v = xp[count * incx];                                                  \
      best = is_max ? (best > v ? best : v) : (best < v ? best : v);                 \
    }                                                                                \
    ((T *)out)[0] = best;                                                            \
    return 0;                                                                        \
  }

ORC_API int orc_extreme_typed(int dtype, int is_max, long n, const void *x, long incx, void *out) {
  if (n < 1) return -1;
  switch (dtype) {
    case 1: ORC_EXTREME_LOOP(double)
    case 2: ORC_EXTREME_LOOP(int32_t)
    case 3: ORC_EXTREME_LOOP(uint32_t)
    case 4: ORC_EXTREME_LOOP(int16_t)
    case 5: ORC_EXTREME_LOOP(uint16_t)
    case 6: ORC_EXTREME_LOOP(int8_t)
    case 7: ORC_EXTREME_LOOP(uint8_t)
    default: return -1;
  }
}

/* waffe2_d{sin,...} (cl-waffe2-simd.c:586-706 at SIMD_DOUBLE_STRIDE = 4): blocks of four
 * through Sleef_<f>d4_u10avx2 (avx2.h:264-331; sqrt u05, fabs exact) when incx >= 1, the
 * remainder -- and everything when incx < 1 -- through libm.  op: 0 sin 1 cos 2 tanh 3 log
 * 4 exp 5 sqrt 6 abs 7 tan 8 asin 9 acos 10 atan 11 sinh 12 cosh 13 log2 14 log10 15 log1p
 * 16 pow (waffe2_dpow, :708-768, Sleef_powd4_u10avx2 / pow). */
typedef double v4d __attribute__((vector_size(32)));
typedef v4d (*sleef_d4_1)(v4d);
typedef v4d (*sleef_d4_2)(v4d, v4d);

static const char *const orc_dnames[17] = {
    "Sleef_sind4_u10avx2",  "Sleef_cosd4_u10avx2",  "Sleef_tanhd4_u10avx2",  "Sleef_logd4_u10avx2",
    "Sleef_expd4_u10avx2",  "Sleef_sqrtd4_u05avx2", "Sleef_fabsd4_avx2",     "Sleef_tand4_u10avx2",
    "Sleef_asind4_u10avx2", "Sleef_acosd4_u10avx2", "Sleef_atand4_u10avx2",  "Sleef_sinhd4_u10avx2",
    "Sleef_coshd4_u10avx2", "Sleef_log2d4_u10avx2", "Sleef_log10d4_u10avx2", "Sleef_log1pd4_u10avx2",
    "Sleef_powd4_u10avx2"};

static double orc_dlibm(int op, double x, double p) {
  switch (op) {
    case 0: return sin(x);
    case 1: return cos(x);
    case 2: return tanh(x);
    case 3: return log(x);
    case 4: return exp(x);
    case 5: return sqrt(x);
    case 6: return fabs(x);
    case 7: return tan(x);
    case 8: return asin(x);
    case 9: return acos(x);
    case 10: return atan(x);
    case 11: return sinh(x);
    case 12: return cosh(x);
    case 13: return log2(x);
    case 14: return log10(x);
    case 15: return log1p(x);
    default: return pow(x, p);
  }
}

/* returns 1 when the blocks went through SLEEF, 0 when libm stood in, -1 on a bad op */
ORC_API int orc_dunary(int op, long n, const double *x, long incx, double *out, long inco, double p) {
  if (op < 0 || op > 16) return -1;
  void *sym = sleef_sym(orc_dnames[op]);
  long count = 0;
  if (incx >= 1) {
    const long blocks_end = (n / 4) * 4;
    for (; count != blocks_end; count += 4) {
      double in[4], res[4];
      for (int l = 0; l < 4; l++) in[l] = x[(count + l) * incx];
      if (sym) {
        v4d v, pv, r;
        memcpy(&v, in, sizeof v);
        for (int l = 0; l < 4; l++) pv[l] = p;
        r = op == 16 ? ((sleef_d4_2)sym)(v, pv) : ((sleef_d4_1)sym)(v);
        memcpy(res, &r, sizeof r);
      } else {
        for (int l = 0; l < 4; l++) res[l] = orc_dlibm(op, in[l], p);
      }
      for (int l = 0; l < 4; l++) out[(count + l) * inco] = res[l];
    }
  }
  for (; count != n; count++) out[count * inco] = orc_dlibm(op, x[count * incx], p);
  return sym ? 1 : 0;
}

ORC_API int orc_abi_version(void) { return 1; }
