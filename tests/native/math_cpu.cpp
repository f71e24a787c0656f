// CPU build of the device math cores (cl-waffe2_amd/csrc/wf2_math.h) so that
// every binary32 input can be checked on the host.  Test infrastructure.
//
//   wf2cpu_unary(op, n, in, out)        out[i] = f(in[i])
//   wf2cpu_pow(n, in, p, out)
//   wf2cpu_scan(op, first, last, stride, &max_ulp, &worst_bits)
//       walks the binary32 bit patterns first, first+stride, ... <= last and
//       returns the largest error in ulps against libm evaluated in binary64.
//   wf2cpu_fastdiv_mismatches(d, n, count)
//       how many of the numerators n[i] < 2^31, and of the multiples of d and their
//       neighbours up to 2^31 - 1, the multiply-and-shift division gets wrong.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "../../cl-waffe2_amd/csrc/wf2_math.h"
#include "../../cl-waffe2_amd/csrc/wf2_fastdiv.h"

enum { OP_SIN = 16, OP_COS, OP_TANH, OP_LOG, OP_EXP, OP_SQRT, OP_ABS, OP_TAN, OP_ASIN, OP_ACOS, OP_ATAN,
       OP_SINH, OP_COSH, OP_LOG2, OP_LOG10, OP_LOG1P, OP_SIGN = 34, OP_SQUARE, OP_ASINH, OP_ACOSH, OP_ATANH,
       OP_GELU = 40, OP_GELU_GRAD = 44 };

static inline float apply(int op, float x) {
  switch (op) {
    case OP_SIN: return wf2::sinf_(x);
    case OP_COS: return wf2::cosf_(x);
    case OP_TANH: return wf2::tanhf_(x);
    case OP_LOG: return wf2::logf_(x);
    case OP_EXP: return wf2::expf_(x);
    case OP_SQRT: return wf2::sqrtf_(x);
    case OP_ABS: return wf2::absf_(x);
    case OP_TAN: return wf2::tanf_(x);
    case OP_ASIN: return wf2::asinf_(x);
    case OP_ACOS: return wf2::acosf_(x);
    case OP_ATAN: return wf2::atanf_(x);
    case OP_SINH: return wf2::sinhf_(x);
    case OP_COSH: return wf2::coshf_(x);
    case OP_LOG2: return wf2::log2f_(x);
    case OP_LOG10: return wf2::log10f_(x);
    case OP_LOG1P: return wf2::log1pf_(x);
    case OP_GELU: return wf2::gelu_tanh_f(x);
    case OP_GELU_GRAD: return wf2::gelu_tanh_grad_f(x);
    case OP_SIGN: return wf2::signf_(x);
    case OP_SQUARE: return x * x;
    case OP_ASINH: return wf2::asinhf_(x);
    case OP_ACOSH: return wf2::acoshf_(x);
    case OP_ATANH: return wf2::atanhf_(x);
  }
  return 0.0f;
}

static inline double truth(int op, double x) {
  switch (op) {
    case OP_SIN: return sin(x);
    case OP_COS: return cos(x);
    case OP_TANH: return tanh(x);
    case OP_LOG: return log(x);
    case OP_EXP: return exp(x);
    case OP_SQRT: return sqrt(x);
    case OP_ABS: return fabs(x);
    case OP_TAN: return tan(x);
    case OP_ASIN: return asin(x);
    case OP_ACOS: return acos(x);
    case OP_ATAN: return atan(x);
    case OP_SINH: return sinh(x);
    case OP_COSH: return cosh(x);
    case OP_LOG2: return log2(x);
    case OP_LOG10: return log10(x);
    case OP_LOG1P: return log1p(x);
    case OP_SIGN: return x > 0 ? 1.0 : (x < 0 ? -1.0 : x);
    case OP_SQUARE: return x * x;
    case OP_ASINH: return asinh(x);
    case OP_ACOSH: return acosh(x);
    case OP_ATANH: return atanh(x);
    case OP_GELU: {
      // 0.5 (1 + tanh u) == 1 / (1 + exp(-2u)), free of cancellation
      double u = 0.7978845608028654 * (x + 0.044715 * x * x * x);
      return x / (1.0 + exp(-2.0 * u));
    }
  }
  return 0.0;
}

// error of `got` against `want` in units of the binary32 ulp at `want`
static inline double ulp_error(float got, double want) {
  if (isnan(want)) return isnan(got) ? 0.0 : INFINITY;
  float wf = (float)want;
  if (isinf(wf) || wf == 0.0f || isinf(got)) {
    // overflow/underflow boundary: demand the correctly rounded value
    if (got == wf) return 0.0;
    if (isinf(wf) || isinf(got)) return INFINITY;
  }
  double a = fabs((double)wf);
  int e;
  frexp(a, &e);                 // a = m * 2^e, m in [0.5,1)
  int ulp_exp = e - 24;
  if (ulp_exp < -149) ulp_exp = -149;
  return fabs((double)got - want) / ldexp(1.0, ulp_exp);
}

extern "C" {

void wf2cpu_unary(int op, long n, const float* in, float* out) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; i++) out[i] = apply(op, in[i]);
}

void wf2cpu_pow(long n, const float* in, float p, float* out) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; i++) out[i] = wf2::powf_(in[i], p);
}

void wf2cpu_scan(int op, uint32_t first, uint32_t last, uint32_t stride,
                 double* max_ulp, uint32_t* worst_bits) {
  const long count = ((long)last - (long)first) / stride + 1;
  double best = 0.0;
  uint32_t best_bits = first;
#pragma omp parallel
  {
    double local = 0.0;
    uint32_t local_bits = first;
#pragma omp for schedule(static)
    for (long i = 0; i < count; i++) {
      uint32_t b = first + (uint32_t)(i * stride);
      float x;
      memcpy(&x, &b, 4);
      double err = ulp_error(apply(op, x), truth(op, (double)x));
      if (err > local) {
        local = err;
        local_bits = b;
      }
    }
#pragma omp critical
    if (local > best) {
      best = local;
      best_bits = local_bits;
    }
  }
  *max_ulp = best;
  *worst_bits = best_bits;
}

long wf2cpu_fastdiv_mismatches(uint32_t d, const uint32_t* n, long count) {
  const wf2::FastDiv f = wf2::make_fastdiv(d);
  long bad = 0;
  auto check = [&](uint32_t v) {
    uint32_t rem;
    const uint32_t q = wf2::fd_divmod(v, f, &rem);
    if (q != v / d || rem != v % d) bad++;
  };
  for (long i = 0; i < count; i++) check(n[i]);
  // k d - 1, k d, k d + 1 for up to 2^16 values of k spread over the range, the largest included
  const uint64_t top = ((uint64_t)1 << 31) - 1;
  const uint64_t kmax = top / d;
  const uint64_t step = kmax / 65536 + 1;
  for (uint64_t k = 0; k <= kmax; k += step) {
    const uint64_t m = k * d;
    if (m >= 1) check((uint32_t)(m - 1));
    check((uint32_t)m);
    if (m + 1 <= top) check((uint32_t)(m + 1));
  }
  const uint64_t m = kmax * d;
  if (m >= 1) check((uint32_t)(m - 1));
  check((uint32_t)m);
  check((uint32_t)top);
  return bad;
}

}  // extern "C"
