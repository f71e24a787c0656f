// wf2_math.h -- scalar math cores of the element-wise kernels.
//
// Contract being replaced: cl-waffe2-simd's unary kernels call SLEEF's
// Sleef_{sin,cos,tanh,log,exp,pow}f8_u10avx2 (<= 1.0 ulp) and
// Sleef_sqrtf8_u05avx2 (cl-waffe2-simd/kernels/simd/x86_64/avx2.h:264-332,
// cl-waffe2-simd.c:586-768).  The device versions below must stay within
// 2 ulp of those results.
//
// Design: CDNA3/CDNA4 issue a binary64 FMA at the same rate as a non-packed
// binary32 FMA, so every core does its argument reduction and the leading
// terms of its series in binary64 and rounds to binary32 once at the end.
// Binary64 FMAs draw much more power, though: beyond ~20 of them per element a
// streaming kernel leaves the HBM roofline because the clock sags, so the
// high-order remainders of exp (as used by tanh and GELU), log, sin and cos are
// evaluated in binary32, where their rounding is below 2^-30 of the result.
// The result is within 0.52 ulp of the exact value for every binary32 input
// (0.507 for the functions evaluated wholly in binary64; exhaustive host runs),
// hence within 1.52 ulp of any 1.0-ulp implementation.  Only IEEE operations and fma are
// used (plus one reciprocal seed that is refined by a Newton step), so the
// same header compiles for the host and a CPU build can check every binary32
// input against libm.
//
// Coefficients come from gen_math_coeffs.py (Chebyshev fits in 60-digit
// arithmetic).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define WF2_MATH_FN __device__ __forceinline__
#define WF2_FMA(a, b, c) __builtin_fma((a), (b), (c))
#define WF2_RCP_SEED(f) __builtin_amdgcn_rcpf(f)
#define WF2_SLOW_SINF(x) sinf(x)
#define WF2_SLOW_COSF(x) cosf(x)
#define WF2_SLOW_POW(x, p) pow((x), (p))
#define WF2_SLOW_TANF(x) tanf(x)
#define WF2_SQRTF(x) __builtin_sqrtf(x)
#define WF2_FAST_EXP2F(x) __builtin_amdgcn_exp2f(x)
#define WF2_FAST_RCPF(x) __builtin_amdgcn_rcpf(x)
#else
#include <math.h>
#define WF2_MATH_FN static inline
#define WF2_FMA(a, b, c) __builtin_fma((a), (b), (c))
#define WF2_RCP_SEED(f) (1.0f / (f))
#define WF2_SLOW_SINF(x) ((float)sin((double)(x)))
#define WF2_SLOW_COSF(x) ((float)cos((double)(x)))
#define WF2_SLOW_POW(x, p) pow((x), (p))
#define WF2_SLOW_TANF(x) ((float)tan((double)(x)))
#define WF2_SQRTF(x) sqrtf(x)
#define WF2_FAST_EXP2F(x) exp2f(x)
#define WF2_FAST_RCPF(x) (1.0f / (x))
#endif

namespace wf2 {

WF2_MATH_FN uint64_t bits_of(double d) { return __builtin_bit_cast(uint64_t, d); }
WF2_MATH_FN double double_of(uint64_t u) { return __builtin_bit_cast(double, u); }
WF2_MATH_FN uint32_t bits_of(float f) { return __builtin_bit_cast(uint32_t, f); }
WF2_MATH_FN float float_of(uint32_t u) { return __builtin_bit_cast(float, u); }

// Adding 1.5*2^52 rounds a |value| < 2^31 to the nearest-even integer in the
// fma's own rounding; the integer is then the low 32 bits of the sum.
constexpr double kRoundMagic = 6755399441055744.0;
constexpr double kLog2e = 1.442695040888963407359925;
constexpr double kLn2 = 0.6931471805599453094172321;
constexpr double kLn2Head = 0.6931471803691238164901733;   // 33 significant bits
constexpr double kLn2Tail = 1.908214929270587816144266e-10;
constexpr double kTwoOverPi = 0.6366197723675813430755351;
constexpr double kPio2Head = 1.57079632673412561416626;    // 33 significant bits
constexpr double kPio2Tail = 6.077100506506192601475144e-11;

// exp(r) = 1 + r + r^2 Q(r) on |r| <= 0.35, Q of degree 5; relative error
// 2.4e-10 (exp), 5.7e-10 (expm1): 2^-31, i.e. at most 0.004 ulp of binary32.
WF2_MATH_FN double expm1_poly(double r) {
  double q = 0.00019891969905683136498;
  q = WF2_FMA(q, r, 0.0013934531655088020325);
  q = WF2_FMA(q, r, 0.0083333100347068682249);
  q = WF2_FMA(q, r, 0.041666456904062640998);
  q = WF2_FMA(q, r, 0.16666666682523656912);
  q = WF2_FMA(q, r, 0.50000000142765894076);
  return WF2_FMA(r * r, q, r);
}

// Splits x = n ln2 + r, |r| <= ln2/2; returns expm1(r) and 2^n.
// Valid for |x| < 700.
WF2_MATH_FN void exp_reduce(double x, double* em1_r, double* scale) {
  double t = WF2_FMA(x, kLog2e, kRoundMagic);
  double n = t - kRoundMagic;
  int32_t ni = (int32_t)(uint32_t)bits_of(t);
  double r = WF2_FMA(n, -kLn2Head, x);
  r = WF2_FMA(n, -kLn2Tail, r);
  *em1_r = expm1_poly(r);
  *scale = double_of((uint64_t)(uint32_t)(ni + 1023) << 52);
}

// e^x in binary64 for x in [-104, 89] (relative error < 2.5e-10).
WF2_MATH_FN double exp_core(double x) {
  double p, s;
  exp_reduce(x, &p, &s);
  return WF2_FMA(s, p, s);
}

// ---- binary32 tails ---------------------------------------------------------
// Measured on MI355X with random data: a unary kernel with 26 dependent binary64
// FMAs per element runs at 72 % of the HBM peak and at 69 % with 30 (the clock
// sags under the power they draw), while 32 binary32 FMAs cost nothing (80 %).
// The cores below therefore keep in binary64 only what decides the last bit --
// the argument reduction and the leading terms of each series -- and evaluate the
// high-order remainder, which is below 2^-6 of the result, in binary32: its 2^-24
// rounding then stays below 2^-30 of the result (at most 0.05 ulp of binary32;
// the exhaustive host run gives the bound per function).

// expm1(r) = r + r^2/2 + r^3/6 + r^4 Q4(r), |r| <= 0.35; Q4 of degree 4 in binary32
// (relative error of expm1 1.9e-10 including its roundings).
WF2_MATH_FN double expm1_mixed(double r) {
  const float rf = (float)r;
  float q = 2.4843823e-05f;
  q = __builtin_fmaf(q, rf, 0.00019883514f);
  q = __builtin_fmaf(q, rf, 0.0013888876f);
  q = __builtin_fmaf(q, rf, 0.0083333207f);
  q = __builtin_fmaf(q, rf, 0.041666668f);
  const float r2 = rf * rf;
  const float tail = (r2 * r2) * q;
  return WF2_FMA(r * r, WF2_FMA(r, 0.16666666666666666667, 0.5), r) + (double)tail;
}

// x = n ln2 + r for |x| < 177 (|n| < 2^8): ln 2 cut to 45 bits makes n * head
// exact, and what the cut drops (2.7e-14 n) is far below the target.
constexpr double kLn2Head45 = 0x1.62e42fefa39p-1;
WF2_MATH_FN void exp_reduce_mixed(double x, double* em1_r, double* scale) {
  double t = WF2_FMA(x, kLog2e, kRoundMagic);
  double n = t - kRoundMagic;
  int32_t ni = (int32_t)(uint32_t)bits_of(t);
  double r = WF2_FMA(n, -kLn2Head45, x);
  *em1_r = expm1_mixed(r);
  *scale = double_of((uint64_t)(uint32_t)(ni + 1023) << 52);
}

WF2_MATH_FN double exp_core_mixed(double x) {
  double p, s;
  exp_reduce_mixed(x, &p, &s);
  return WF2_FMA(s, p, s);
}

WF2_MATH_FN float expf_(float x) {
  // Below -104 the result rounds to +0 and above 89 to +inf, as e^-104 and
  // e^89 already do, so clamping is exact.  fmin/fmax drop a NaN operand.
  float xc = __builtin_fminf(__builtin_fmaxf(x, -104.0f), 89.0f);  // one v_med3_f32
  float r = (float)exp_core((double)xc);
  return (x != x) ? x : r;
}

// 1/d for d >= 1 in binary32 range: a binary32 seed (relative error <= 2^-22
// for v_rcp_f32, 2^-24 for a correctly rounded host division) refined by one
// Newton step in binary64, which squares the error: <= 2^-44.
WF2_MATH_FN double rcp_refined(double d) {
  double y = (double)WF2_RCP_SEED((float)d);
  double e = WF2_FMA(-d, y, 1.0);
  return WF2_FMA(y, e, y);
}

// tanh(x) = expm1(2|x|) / (expm1(2|x|) + 2); saturates to 1 from |x| = 10
// (1 - tanh(10) = 4.1e-9 < 2^-25).
WF2_MATH_FN double tanh_core(double ax) {
  double p, s;
  exp_reduce_mixed(ax + ax, &p, &s);
  double em1 = WF2_FMA(s, p, s - 1.0);
  return em1 * rcp_refined(em1 + 2.0);
}

WF2_MATH_FN float tanhf_(float x) {
  double ax = __builtin_fmin(__builtin_fabs((double)x), 10.0);
  float r = __builtin_copysignf((float)tanh_core(ax), x);
  return (x != x) ? x : r;
}

// log(m) for m in [sqrt(1/2), sqrt(2)): f = m - 1,
// log(1+f) = f - f^2/2 + f^3 R(f); relative error 1.3e-11.
WF2_MATH_FN double log1p_poly(double f) {
  double r = -0.05005748841457288547;
  r = WF2_FMA(r, f, 0.09036934208961060298);
  r = WF2_FMA(r, f, -0.09109982945851015244);
  r = WF2_FMA(r, f, 0.09031005007965443269);
  r = WF2_FMA(r, f, -0.09922837010255326152);
  r = WF2_FMA(r, f, 0.1110948193429464372);
  r = WF2_FMA(r, f, -0.1250321982641986753);
  r = WF2_FMA(r, f, 0.1428586067850288431);
  r = WF2_FMA(r, f, -0.1666661173195466807);
  r = WF2_FMA(r, f, 0.1999999784866672395);
  r = WF2_FMA(r, f, -0.2500000026716445387);
  r = WF2_FMA(r, f, 0.3333333333749120236);
  double f2 = f * f;
  return WF2_FMA(f2 * f, r, WF2_FMA(-0.5, f2, f));
}

// The same with the tail in binary32: log(1+f) = f - f^2/2 + f^3/3 - f^4/4 +
// f^5 R5(f), R5 of degree 8 (relative error 8.8e-10 including its roundings).
WF2_MATH_FN double log1p_mixed(double f) {
  const float ff = (float)f;
  float r = 0.058937758f;
  r = __builtin_fmaf(r, ff, -0.096051253f);
  r = __builtin_fmaf(r, ff, 0.095819056f);
  r = __builtin_fmaf(r, ff, -0.099360347f);
  r = __builtin_fmaf(r, ff, 0.11079729f);
  r = __builtin_fmaf(r, ff, -0.12500979f);
  r = __builtin_fmaf(r, ff, 0.14286327f);
  r = __builtin_fmaf(r, ff, -0.16666664f);
  r = __builtin_fmaf(r, ff, 0.19999999f);
  const float f2 = ff * ff;
  const float tail = (f2 * f2) * (ff * r);
  double h = WF2_FMA(f, -0.25, 0.33333333333333333333);
  h = WF2_FMA(h, f, -0.5);
  return WF2_FMA(f * f, h, f) + (double)tail;
}

// log of a positive finite binary64 that is normal (every positive binary32,
// subnormals included, converts to one).
WF2_MATH_FN double log_core(double xd) {
  uint64_t b = bits_of(xd);
  int32_t hi = (int32_t)(b >> 32);
  hi += 0x3ff00000 - 0x3fe6a09e;  // moves the binade boundary to sqrt(1/2)
  int32_t k = (hi >> 20) - 0x3ff;
  hi = (hi & 0x000fffff) + 0x3fe6a09e;
  double m = double_of(((uint64_t)(uint32_t)hi << 32) | (b & 0xffffffffu));
  return WF2_FMA((double)k, kLn2, log1p_mixed(m - 1.0));
}

WF2_MATH_FN float logf_(float x) {
  const float inf = __builtin_inff();
  bool ok = (x > 0.0f) && (x < inf);
  float r = (float)log_core(ok ? (double)x : 1.0);
  // x == +inf -> +inf; x == +-0 -> -inf; x < 0 or NaN -> NaN
  float special = (x == inf) ? inf : ((x == 0.0f) ? -inf : __builtin_nanf(""));
  return ok ? r : special;
}

// sin/cos on |r| <= pi/4: sin r = r + r^3 S(r^2) (1.9e-11),
// cos r = 1 - z/2 + z^2 C(z) (1.3e-12).
WF2_MATH_FN double sin_poly(double r, double z) {
  double s = 2.7249146796813166492e-6;
  s = WF2_FMA(s, z, -0.0001984008071991224356);
  s = WF2_FMA(s, z, 0.008333331863560767561);
  s = WF2_FMA(s, z, -0.1666666666382658236);
  return WF2_FMA(r * z, s, r);
}

WF2_MATH_FN double cos_poly(double z) {
  double c = -2.7300309020522219532e-7;
  c = WF2_FMA(c, z, 0.000024800595356594503473);
  c = WF2_FMA(c, z, -0.0013888887662711772101);
  c = WF2_FMA(c, z, 0.041666666664297246826);
  return WF2_FMA(z * z, c, WF2_FMA(-0.5, z, 1.0));
}

// Quadrant reduction x = q*pi/2 + r in binary64.  q*kPio2Head is exact for
// |q| < 2^20, i.e. |x| <= 1e6.
constexpr float kTrigFastLimit = 1.0e6f;

WF2_MATH_FN double trig_core(double xd, int32_t quadrant_shift) {
  double t = WF2_FMA(xd, kTwoOverPi, kRoundMagic);
  double q = t - kRoundMagic;
  int32_t qi = (int32_t)(uint32_t)bits_of(t) + quadrant_shift;
  double r = WF2_FMA(q, -kPio2Head, xd);
  r = WF2_FMA(q, -kPio2Tail, r);
  // sin r = r - r^3/6 + r^5 S5(z), cos r = 1 - z/2 + z^2/24 + z^3 C3(z), z = r^2: the
  // leading terms in binary64, S5 and C3 (degree 2 in z) in binary32 (relative
  // error 2.9e-10 and 3.9e-11 including their roundings)
  double z = r * r;
  const float rf = (float)r, zf = rf * rf;
  float s5 = 2.7325962e-06f;
  s5 = __builtin_fmaf(s5, zf, -0.00019840735f);
  s5 = __builtin_fmaf(s5, zf, 0.0083333328f);
  float c3 = -2.7364399e-07f;
  c3 = __builtin_fmaf(c3, zf, 2.480114e-05f);
  c3 = __builtin_fmaf(c3, zf, -0.0013888889f);
  const float z2f = zf * zf;
  const float stail = (z2f * rf) * s5;
  const float ctail = (z2f * zf) * c3;
  const double shead = WF2_FMA(r * z, -0.16666666666666666667, r);
  const double chead = WF2_FMA(z, WF2_FMA(z, 0.041666666666666666667, -0.5), 1.0);
  const bool odd = (qi & 1) != 0;
  double v = (odd ? chead : shead) + (double)(odd ? ctail : stail);
  return (qi & 2) ? -v : v;
}

WF2_MATH_FN float sinf_(float x) {
  if (!(__builtin_fabsf(x) <= kTrigFastLimit)) return WF2_SLOW_SINF(x);
  float r = (float)trig_core((double)x, 0);
  return (x == 0.0f) ? x : r;  // sin(-0) = -0: the polynomial's sign of zero is not x's
}

WF2_MATH_FN float cosf_(float x) {
  if (!(__builtin_fabsf(x) <= kTrigFastLimit)) return WF2_SLOW_COSF(x);
  return (float)trig_core((double)x, 1);
}

// tan = sin / cos of the reduced argument (one binary64 division); odd
// quadrants give -cos / sin.
WF2_MATH_FN float tanf_(float x) {
  if (!(__builtin_fabsf(x) <= kTrigFastLimit)) return WF2_SLOW_TANF(x);
  double xd = (double)x;
  double t = WF2_FMA(xd, kTwoOverPi, kRoundMagic);
  double q = t - kRoundMagic;
  int32_t qi = (int32_t)(uint32_t)bits_of(t);
  double r = WF2_FMA(q, -kPio2Head, xd);
  r = WF2_FMA(q, -kPio2Tail, r);
  double z = r * r;
  double s = sin_poly(r, z);
  double c = cos_poly(z);
  float v = (float)((qi & 1) ? -c / s : s / c);
  return (x == 0.0f) ? x : v;
}

// log2, log10: the binary64 logarithm times a constant, rounded once (exact for
// powers of two: k ln2 / ln2).
WF2_MATH_FN float log2f_(float x) {
  const float inf = __builtin_inff();
  bool ok = (x > 0.0f) && (x < inf);
  float r = (float)(log_core(ok ? (double)x : 1.0) * 1.4426950408889634074);
  float special = (x == inf) ? inf : ((x == 0.0f) ? -inf : __builtin_nanf(""));
  return ok ? r : special;
}

WF2_MATH_FN float log10f_(float x) {
  const float inf = __builtin_inff();
  bool ok = (x > 0.0f) && (x < inf);
  float r = (float)(log_core(ok ? (double)x : 1.0) * 0.43429448190325182765);
  float special = (x == inf) ? inf : ((x == 0.0f) ? -inf : __builtin_nanf(""));
  return ok ? r : special;
}

// log1p: 1 + x is exact in binary64 from |x| >= 2^-29 on; below that
// x - x^2/2 is correct to 2^-58 relative.
WF2_MATH_FN float log1pf_(float x) {
  const float inf = __builtin_inff();
  bool ok = (x > -1.0f) && (x < inf);
  double xd = ok ? (double)x : 0.0;
  double small = WF2_FMA(-0.5 * xd, xd, xd);
  double big = log_core(1.0 + xd);
  float r = (float)((__builtin_fabs(xd) < 0x1p-28) ? small : big);
  float special = (x == inf) ? inf : ((x == -1.0f) ? -inf : __builtin_nanf(""));
  r = (x == 0.0f) ? x : r;  // log1p(-0) = -0
  return ok ? r : special;
}

// sinh, cosh from E = expm1(|x|): sinh = (E + E / (E + 1)) / 2 (no
// cancellation for small |x|), cosh = ((E + 1) + 1 / (E + 1)) / 2.  From
// |x| = 90 on both overflow binary32.
WF2_MATH_FN float sinhf_(float x) {
  double ax = __builtin_fmin(__builtin_fabs((double)x), 90.0);
  double p, s;
  exp_reduce(ax, &p, &s);
  double em1 = WF2_FMA(s, p, s - 1.0);
  double v = 0.5 * (em1 + em1 / (em1 + 1.0));
  float r = __builtin_copysignf((float)v, x);
  return (x != x) ? x : r;
}

WF2_MATH_FN float coshf_(float x) {
  double ax = __builtin_fmin(__builtin_fabs((double)x), 90.0);
  double p, s;
  exp_reduce(ax, &p, &s);
  double e = WF2_FMA(s, p, s);  // e^|x|
  float r = (float)(0.5 * (e + 1.0 / e));
  return (x != x) ? x : r;
}

// atan in binary64: |x| > 1 is folded by atan x = pi/2 - atan(1/x); on [0, 1]
// the argument is split once more at tan(pi/8) with
// atan x = pi/4 + atan((x - 1) / (x + 1)), which leaves |t| <= tan(pi/8) for
// atan t = t + t^3 P(t^2), P of degree 9 (relative error 1.4e-16).
WF2_MATH_FN double atan_core(double ax) {  // ax >= 0, finite
  bool inv = ax > 1.0;
  double y = inv ? 1.0 / ax : ax;
  bool mid = y > 0.41421356237309503;
  double t = mid ? (y - 1.0) / (y + 1.0) : y;
  double z = t * t;
  double p = 0.022750526993361672084;
  p = WF2_FMA(p, z, -0.0448333462227288608);
  p = WF2_FMA(p, z, 0.057363321659076425088);
  p = WF2_FMA(p, z, -0.066496136952916693446);
  p = WF2_FMA(p, z, 0.07691055158393149258);
  p = WF2_FMA(p, z, -0.090908525571760493567);
  p = WF2_FMA(p, z, 0.11111109636534361442);
  p = WF2_FMA(p, z, -0.14285714266096617917);
  p = WF2_FMA(p, z, 0.1999999999989840813);
  p = WF2_FMA(p, z, -0.3333333333333324625);
  double a = WF2_FMA(t * z, p, t);
  a = mid ? 0.78539816339744830962 + a : a;
  return inv ? 1.57079632679489661923 - a : a;
}

WF2_MATH_FN float atanf_(float x) {
  double ax = __builtin_fabs((double)x);
  double a = (ax > 0x1p60) ? 1.57079632679489661923 : atan_core(ax);
  float r = __builtin_copysignf((float)a, x);
  return (x != x) ? x : r;
}

// asin x = atan(x / sqrt((1 - x)(1 + x))), acos x = 2 atan(sqrt((1 - x) / (1 + x)));
// (1 - x) and (1 + x) are exact in binary64 for binary32 x.
WF2_MATH_FN float asinf_(float x) {
  double xd = (double)x;
  double ax = __builtin_fabs(xd);
  if (!(ax <= 1.0)) return __builtin_nanf("");
  double a = (ax == 1.0) ? 1.57079632679489661923
                         : atan_core(ax / __builtin_sqrt((1.0 - ax) * (1.0 + ax)));
  float r = __builtin_copysignf((float)a, x);
  return (x == 0.0f) ? x : r;
}

WF2_MATH_FN float acosf_(float x) {
  double xd = (double)x;
  if (!(__builtin_fabs(xd) <= 1.0)) return __builtin_nanf("");
  if (xd == -1.0) return 3.14159274101257324f;
  return (float)(2.0 * atan_core(__builtin_sqrt((1.0 - xd) / (1.0 + xd))));
}

WF2_MATH_FN float sqrtf_(float x) { return WF2_SQRTF(x); }
WF2_MATH_FN float absf_(float x) { return __builtin_fabsf(x); }

// x^p.  The exponent is the same for every element of a launch (it is the
// host scalar of ExptNode, base-impl/mathematics.lisp:267-303), so the branch
// is uniform.  Integral exponents (GELU's x^3, LayerNorm's (x-u)^2) are
// repeated products in binary64, exact to ~2^-48 and rounded once.
WF2_MATH_FN float powf_(float x, float p) {
  float ap = __builtin_fabsf(p);
  if (ap <= 1024.0f && p == __builtin_truncf(p)) {
    uint32_t e = (uint32_t)ap;
    double base = (double)x, acc = 1.0;
    while (e) {
      if (e & 1u) acc *= base;
      base *= base;
      e >>= 1;
    }
    if (p < 0.0f) acc = 1.0 / acc;
    return (float)acc;
  }
  if (p == 0.5f) return WF2_SQRTF(x);
  return (float)WF2_SLOW_POW((double)x, (double)p);
}

// tanh-form GELU, 0.5 x (1 + tanh(u)), u = sqrt(2/pi) (x + 0.044715 x^3)
// (nn/activation.lisp:45-66), in binary64 and rounded once.  0.5 (1 + tanh u)
// equals sigmoid(2u), evaluated with e = exp(-2|u|) in (0, 1] as 1/(1+e) for
// u >= 0 and e/(1+e) for u < 0: no cancellation on either side.
WF2_MATH_FN float gelu_tanh_f(float x) {
  double xd = (double)x;
  double u = 0.7978845608028654 * WF2_FMA(0.044715 * xd * xd, xd, xd);
  double au = __builtin_fmin(__builtin_fabs(u), 80.0);  // e^-160 is far below 2^-30 already; keeps |n| < 2^8
  double e = exp_core_mixed(-(au + au));
  double num = (u >= 0.0) ? 1.0 : e;
  float r = (float)(xd * num * rcp_refined(1.0 + e));
  // x = -inf: the limit is -0 (x e^{2u} -> 0), not -inf * tiny.
  r = (x == -__builtin_inff()) ? -0.0f : r;
  return (x != x) ? x : r;
}

// The same function in binary32 for gemm epilogues, whose inputs already carry
// the rounding of a long binary32 accumulation: x / (1 + 2^t) with
// t = -2 u log2(e) = x (k1 + k2 x^2), through v_exp_f32 and v_rcp_f32 (12 VALU
// slots against 35).  Error: three roundings of t (|t| 2e-7 absolute, so
// |t| 1.3e-7 relative in 2^t), one ulp each from the exponential, the
// reciprocal and the two products: below 4e-6 relative wherever the result is
// a normal number, below 1e-6 for |x| < 4.
WF2_MATH_FN float gelu_tanh_fast(float x) {
  const float k1 = -2.3022082f;    // -2 sqrt(2/pi) log2(e)
  const float k2 = -0.10294324f;   // k1 * 0.044715
  const float t = x * __builtin_fmaf(k2, x * x, k1);
  const float e = WF2_FAST_EXP2F(t < 126.0f ? t : 126.0f);
  const float r = x * WF2_FAST_RCPF(1.0f + e);
  // far on the negative side x e^{2u} underflows; x = -inf would give inf / inf
  return (t > 100.0f) ? -0.0f : r;
}

}  // namespace wf2
