// wf2_math.h -- scalar math cores of the element-wise kernels.
//
// Contract being replaced: cl-waffe2-simd's unary kernels call SLEEF's
// Sleef_{sin,cos,tanh,log,exp,pow}f8_u10avx2 (<= 1.0 ulp) and
// Sleef_sqrtf8_u05avx2 (cl-waffe2-simd/kernels/simd/x86_64/avx2.h:264-332,
// cl-waffe2-simd.c:586-768).  The device versions below must stay within
// 2 ulp of those results.
//
// Design: two families.
//  * exp, log, sin, cos, tanh -- the functions of the benchmark configurations, which
//    run over 2^26 elements at the HBM roofline -- are written in binary32 only:
//    Cody-Waite reductions with fma, short polynomials, and double-float
//    (head + tail) arithmetic at the few places that decide the last bit.  A
//    streaming kernel on MI355X keeps its bandwidth with up to ~48 binary32 VALU
//    operations per element and one 16-byte vector per thread; binary64 FMAs draw
//    more power and pull the clock down once the load is sustained (measured: the
//    binary64 forms of sin and tanh 76-79 % of the HBM peak, the binary32 forms
//    80-83 %).  Error below 0.9 ulp for every binary32 input (exhaustive host runs;
//    the bound per function is stated at its definition), hence within 2 ulp of
//    any 1.0-ulp implementation such as SLEEF u10.
//  * everything else does its argument reduction and the leading terms of its
//    series in binary64 (a binary64 FMA issues at the rate of a non-packed
//    binary32 one on CDNA3/CDNA4) and rounds once: within 0.52 ulp.
// Only IEEE operations, fma and ldexp are used (plus one reciprocal seed that is
// refined by a Newton step), so the same header compiles for the host and a CPU
// build can check every binary32 input against libm.
//
// Coefficients come from gen_math_coeffs.py (Chebyshev fits in 60-digit
// arithmetic).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define WF2_MATH_FN __device__ __forceinline__
#define WF2_MATH_COLD static __device__ __attribute__((noinline))
#define WF2_FMA(a, b, c) __builtin_fma((a), (b), (c))
#define WF2_RCP_SEED(f) __builtin_amdgcn_rcpf(f)
#define WF2_SLOW_SINF(x) sinf(x)
#define WF2_SLOW_COSF(x) cosf(x)
#define WF2_SLOW_POW(x, p) pow((x), (p))
#define WF2_SLOW_TANF(x) tanf(x)
#define WF2_SQRTF(x) __builtin_sqrtf(x)
#define WF2_FAST_EXP2F(x) __builtin_amdgcn_exp2f(x)
#define WF2_FAST_RCPF(x) __builtin_amdgcn_rcpf(x)
#define WF2_LDEXPF(x, e) __builtin_ldexpf((x), (e))
#define WF2_FREXP_MANT(x) __builtin_amdgcn_frexp_mantf(x)
#define WF2_FREXP_EXP(x) __builtin_amdgcn_frexp_expf(x)
#else
#include <math.h>
#define WF2_MATH_FN static inline
#define WF2_MATH_COLD static __attribute__((noinline))
#define WF2_FMA(a, b, c) __builtin_fma((a), (b), (c))
#define WF2_RCP_SEED(f) (1.0f / (f))
#define WF2_SLOW_SINF(x) ((float)sin((double)(x)))
#define WF2_SLOW_COSF(x) ((float)cos((double)(x)))
#define WF2_SLOW_POW(x, p) pow((x), (p))
#define WF2_SLOW_TANF(x) ((float)tan((double)(x)))
#define WF2_SQRTF(x) sqrtf(x)
#define WF2_FAST_EXP2F(x) exp2f(x)
#define WF2_FAST_RCPF(x) (1.0f / (x))
#define WF2_LDEXPF(x, e) ldexpf((x), (e))
static inline float wf2_frexp_mant_host(float x) { int e; return frexpf(x, &e); }
static inline int wf2_frexp_exp_host(float x) { int e; (void)frexpf(x, &e); return e; }
#define WF2_FREXP_MANT(x) wf2_frexp_mant_host(x)
#define WF2_FREXP_EXP(x) wf2_frexp_exp_host(x)
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

// ---- binary32 cores -----------------------------------------------------------
// Adding 1.5 * 2^23 rounds |value| < 2^22 to the nearest integer in the fma's own
// rounding; the integer is then the difference of the bit patterns.
constexpr float kRoundMagic32 = 12582912.0f;
constexpr float kLog2e32 = 1.44269502f;
constexpr float kLn2Head32 = 0.693145751953125f;     // 16 significant bits: n * head is exact for |n| < 2^8
constexpr float kLn2Tail32 = 1.428606765330187e-06f;

// exp(r) = 1 + r + r^2 Q(r) on |r| <= 0.3475, Q of degree 5 with binary32
// coefficients fitted one at a time (each rounded, the rest refitted): relative
// error 1.5e-10 for exp and 4.6e-10 for expm1 before the roundings of the
// evaluation.
WF2_MATH_FN float exp_q32(float r) {
  float q = 0.00019738492846954614f;
  q = __builtin_fmaf(q, r, 0.0013933394802734256f);
  q = __builtin_fmaf(q, r, 0.008333572186529636f);
  q = __builtin_fmaf(q, r, 0.041666481643915176f);
  q = __builtin_fmaf(q, r, 0.1666666567325592f);
  return __builtin_fmaf(q, r, 0.5f);
}

// e^x, binary32 only.  x = n ln2 + r; exp(r) = 1 + w, w = r + r^2 Q(r).  The
// roundings of r and of w (each up to a quarter ulp of the result) are recovered
// as tails and added back with the exact remainder of 1 + w, so that one rounding
// decides the result: error below 0.6 ulp.  Below -104 the result rounds to +0
// and above 89 to +inf, as e^-104 and e^89 already do, so clamping is exact;
// fmin / fmax drop a NaN operand.  ldexp rounds once into the subnormals.
// 28 VALU operations.
WF2_MATH_FN float expf_(float x) {
  const float xc = __builtin_fminf(__builtin_fmaxf(x, -104.0f), 89.0f);  // one v_med3_f32
  const float t = __builtin_fmaf(xc, kLog2e32, kRoundMagic32);
  const float n = t - kRoundMagic32;
  const int32_t ni = (int32_t)(bits_of(t) - bits_of(kRoundMagic32));
  const float r1 = __builtin_fmaf(n, -kLn2Head32, xc);  // exact
  const float r = __builtin_fmaf(n, -kLn2Tail32, r1);
  const float rl = __builtin_fmaf(n, -kLn2Tail32, r1 - r);
  const float r2 = r * r, q = exp_q32(r);
  const float wh = __builtin_fmaf(r2, q, r);
  const float wl = __builtin_fmaf(r2, q, r - wh);
  const float y = 1.0f + wh;
  const float yl = ((1.0f - y) + wh) + (wl + rl);
  const float res = WF2_LDEXPF(y + yl, ni);
  return (x != x) ? x : res;
}

// 1/d for d >= 1 in binary32 range: a binary32 seed (relative error <= 2^-22
// for v_rcp_f32, 2^-24 for a correctly rounded host division) refined by one
// Newton step in binary64, which squares the error: <= 2^-44.
WF2_MATH_FN double rcp_refined(double d) {
  double y = (double)WF2_RCP_SEED((float)d);
  double e = WF2_FMA(-d, y, 1.0);
  return WF2_FMA(y, e, y);
}

// tanh(x) = (E - 1) / (E + 1), E = e^{2|x|} = 2^n y, y = 1 + w, as the quotient of
// N = y - c and D = y + c with c = 2^-n: for n = 0 the numerator is expm1(2|x|)
// itself, so small arguments need no branch.  w is carried as head + tail (the tail
// is the rounding error of its last fma), y, N and D are exact two-term sums, and
// the quotient is one Newton-corrected division, so that the only full rounding is
// the last one.  Saturates to 1 from |x| = 10 (1 - tanh(10) = 4.1e-9 < 2^-25).
// 45 VALU operations; error below 0.75 ulp.
WF2_MATH_FN float tanhf_(float x) {
  const float a2 = 2.0f * __builtin_fminf(__builtin_fabsf(x), 10.0f);
  const float t = __builtin_fmaf(a2, kLog2e32, kRoundMagic32);
  const float n = t - kRoundMagic32;
  const int32_t ni = (int32_t)(bits_of(t) - bits_of(kRoundMagic32));  // 0 .. 29
  float r = __builtin_fmaf(n, -kLn2Head32, a2);
  r = __builtin_fmaf(n, -kLn2Tail32, r);
  const float r2 = r * r, q = exp_q32(r);
  const float wh = __builtin_fmaf(r2, q, r);
  const float wl = __builtin_fmaf(r2, q, r - wh);
  const float c = float_of((uint32_t)(127 - ni) << 23);
  // y = 1 + w, N = y - c, D = y + c as exact two-term sums (for n = 0, c = 1 and y >= 1:
  // y - 1 is exact and 1 <= y orders the other sum)
  const float yh = 1.0f + wh, yl = ((1.0f - yh) + wh) + wl;
  const float nh = yh - c, nl = ((yh - nh) - c) + yl;
  const float dh = yh + c, dl = ((yh - dh) + c) + yl;
  const float y0 = WF2_FAST_RCPF(dh);
  const float q0 = nh * y0;
  float rho = __builtin_fmaf(-q0, dh, nh);
  rho = __builtin_fmaf(-q0, dl, rho + nl);
  const float res = __builtin_copysignf(__builtin_fmaf(rho, y0, q0), x);
  return (x != x) ? x : res;
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

// log x = k ln2 + log(1 + f), x = 2^k (1 + f), 1 + f in [sqrt(1/2), sqrt(2)):
// with s = f / (2 + f), log(1 + f) = 2 atanh(s) = 2 s + s R(s^2), and
// 2 s = f - f^2/2 + s f^2/2 exactly, so that f, the dominant term, enters
// unrounded: log(1 + f) = f - (h - s (h + R)), h = f^2/2 (the classical
// arrangement of 4.4BSD's logf).  R of degree 3 in z = s^2 <= 0.0295 (relative
// error 2.4e-11).  v_frexp_* handle subnormal arguments.  36 VALU operations;
// error below 0.87 ulp.
WF2_MATH_FN float logf_(float x) {
  const float inf = __builtin_inff();
  const bool ok = (x > 0.0f) && (x < inf);
  const float xs = ok ? x : 1.0f;
  float m = WF2_FREXP_MANT(xs);  // [0.5, 1)
  int32_t e = WF2_FREXP_EXP(xs);
  const bool low = m < 0.707106769f;
  m = low ? m + m : m;
  e = low ? e - 1 : e;
  const float f = m - 1.0f;
  const float k = (float)e;
  const float d = 2.0f + f;
  const float y0 = WF2_FAST_RCPF(d);
  const float y = __builtin_fmaf(y0, __builtin_fmaf(-d, y0, 1.0f), y0);
  const float s = f * y;
  const float z = s * s;
  float p = 0.23103581368923187f;
  p = __builtin_fmaf(p, z, 0.2856609523296356f);
  p = __builtin_fmaf(p, z, 0.3999979794025421f);
  p = __builtin_fmaf(p, z, 0.6666666865348816f);
  const float R = z * p;
  const float h = (0.5f * f) * f;
  const float u = __builtin_fmaf(s, h + R, k * kLn2Tail32);
  const float r = __builtin_fmaf(k, kLn2Head32, -((h - u) - f));
  // x == +inf -> +inf; x == +-0 -> -inf; x < 0 or NaN -> NaN
  const float special = (x == inf) ? inf : ((x == 0.0f) ? -inf : __builtin_nanf(""));
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

// sin and cos in binary32 for |x| <= 128: |x| = q pi/2 + r, |r| <= pi/4, by a
// three-term Cody-Waite reduction (pi/2 = A + B + C with 17 + 17 + 24 bits, so
// q A is exact for q <= 82); the roundings of the second and third step are
// recovered as a tail rl, and sin(r + rl) = sin r + rl (1 - r^2/2), cos(r + rl) =
// cos r - rl r.  sin r = r + r^3 S(r^2), cos r = 1 - z/2 + z^2 C(z) with S of
// degree 3 and C of degree 2 (relative errors 1.9e-10 and 1.2e-10).  Error below
// 0.75 ulp.  From 128 on the binary64 reduction takes over (to 1e6, 0.52 ulp), then
// the platform's routine.  41 VALU operations on the fast path.
constexpr float kTrigFast32 = 128.0f;
constexpr float kPio2A = 1.5707855224609375f, kPio2B = 1.0804273188114166e-05f, kPio2C = 6.07710062827671e-11f;

// value of sin (shift 0) or cos (shift 1) of |x| = ax <= 128, without the sign of x
WF2_MATH_FN float trig32(float ax, uint32_t shift) {
  const float t = __builtin_fmaf(ax, 0.636619747f, kRoundMagic32);
  const float q = t - kRoundMagic32;
  const uint32_t qi = bits_of(t) + shift;  // low bits: the quadrant
  const float r1 = __builtin_fmaf(q, -kPio2A, ax);  // exact
  const float r2 = __builtin_fmaf(q, -kPio2B, r1);
  const float r2l = __builtin_fmaf(q, -kPio2B, r1 - r2);
  const float r = __builtin_fmaf(q, -kPio2C, r2);
  const float rl = __builtin_fmaf(q, -kPio2C, r2 - r) + r2l;
  const float z = r * r, zl = __builtin_fmaf(r, r, -z);
  float sp = 2.8040192319167545e-06f;
  sp = __builtin_fmaf(sp, z, -0.00019850277749355882f);
  sp = __builtin_fmaf(sp, z, 0.008333372883498669f);
  sp = __builtin_fmaf(sp, z, -0.1666666716337204f);
  float cp = 2.443209450575523e-05f;
  cp = __builtin_fmaf(cp, z, -0.0013887308305129409f);
  cp = __builtin_fmaf(cp, z, 0.04166664555668831f);
  // one rounding decides each value: sin = r + (small), cos = (1 + mh) + (small)
  const float sv = r + __builtin_fmaf(r * z, sp, rl * __builtin_fmaf(z, -0.5f, 1.0f));
  const float ci = __builtin_fmaf(z, cp, -0.5f);
  const float mh = z * ci, ml = __builtin_fmaf(z, ci, -mh);
  const float y = 1.0f + mh;
  const float cv = y + (((1.0f - y) + mh) + __builtin_fmaf(-rl, r, __builtin_fmaf(-0.5f, zl, ml)));
  const float v = (qi & 1u) ? cv : sv;
  return float_of(bits_of(v) ^ ((qi & 2u) << 30));
}

// Arguments beyond the binary32 fast path; kept out of line so that the rare case
// does not swell the streaming kernels (inlined four times per vector it cost them
// two thirds of their bandwidth).
WF2_MATH_COLD float trig_beyond(float x, int32_t quadrant_shift) {
  if (!(__builtin_fabsf(x) <= kTrigFastLimit)) return quadrant_shift ? WF2_SLOW_COSF(x) : WF2_SLOW_SINF(x);
  return (float)trig_core((double)x, quadrant_shift);
}

WF2_MATH_FN float sinf_(float x) {
  const float ax = __builtin_fabsf(x);
  if (__builtin_expect(!(ax <= kTrigFast32), 0)) return trig_beyond(x, 0);
  // sin is odd: -0 stays -0
  return float_of(bits_of(trig32(ax, 0u)) ^ (bits_of(x) & 0x80000000u));
}

WF2_MATH_FN float cosf_(float x) {
  const float ax = __builtin_fabsf(x);
  if (__builtin_expect(!(ax <= kTrigFast32), 0)) return trig_beyond(x, 1);
  return trig32(ax, 1u);
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

// The inverse hyperbolic functions through the binary64 logarithm (0.52 ulp); small
// arguments, where 1 + y would round y away, through their series.
WF2_MATH_FN float asinhf_(float x) {
  const double t = __builtin_fabs((double)x);
  const double t2 = t * t;
  double r;
  if (t < 0x1p-10)
    r = t * WF2_FMA(t2, WF2_FMA(t2, 0.075, -0.16666666666666666667), 1.0);
  else if (t > 0x1p30)
    r = log_core(t) + kLn2;  // sqrt(t^2 + 1) = t to binary64 precision
  else
    r = log_core(t + __builtin_sqrt(t2 + 1.0));
  const float v = __builtin_copysignf((float)r, x);
  return (x != x || __builtin_fabsf(x) == __builtin_inff()) ? x : v;
}

WF2_MATH_FN float acoshf_(float x) {
  if (!(x >= 1.0f)) return __builtin_nanf("");
  if (x == __builtin_inff()) return x;
  const double t = (double)x;
  if (t > 0x1p30) return (float)(log_core(t) + kLn2);
  // (x - 1)(x + 1) is exact in binary64 for a binary32 x; x = 1 gives log(1) = 0
  return (float)log_core(t + __builtin_sqrt((t - 1.0) * (t + 1.0)));
}

WF2_MATH_FN float atanhf_(float x) {
  const double t = __builtin_fabs((double)x);
  if (!(t <= 1.0)) return __builtin_nanf("");
  if (t == 1.0) return __builtin_copysignf(__builtin_inff(), x);
  const double t2 = t * t;
  double r;
  if (t < 0x1p-10)
    r = t * WF2_FMA(t2, WF2_FMA(t2, 0.2, 0.33333333333333333333), 1.0);
  else
    r = 0.5 * log_core((1.0 + t) / (1.0 - t));  // 1 + t and 1 - t are exact
  return __builtin_copysignf((float)r, x);
}

// CL's signum on floats: -1, 1, and the argument itself when it is +-0 or NaN
WF2_MATH_FN float signf_(float x) { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : x); }

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
// (nn/activation.lisp:45-66).  0.5 (1 + tanh u) equals sigmoid(2u), evaluated
// with E = exp(-2|u|) in (0, 1] as 1 / (1 + E) for x >= 0 and E / (1 + E) for
// x < 0: no cancellation on either side.  a = 2|u| log2(e) = |x| (K1 + K2 x^2)
// and its split into an integer and |p| <= 1/2 are formed in binary64 (eight
// operations: a binary32 rounding of a would be multiplied by |a| in the left
// tail, where the result is x e^{-2|u|}); E = 2^-a through the binary32 exp
// polynomial, and the quotient (x or x E) / (1 + E) is one Newton-corrected
// division against 1 + E kept as an exact two-term sum.  Error below 2 ulp
// (exhaustive host run), far inside the reference's own node composition, whose
// 1 + tanh u cancels on the left.  48 VALU operations.
WF2_MATH_FN float gelu_tanh_f(float x) {
  const double K1 = 2.3022081981443249;   // 2 sqrt(2/pi) log2(e)
  const double K2 = 0.10294323958002349;  // K1 * 0.044715
  const float Ln2h = 0.6931471824645996f, Ln2l = -1.9046542121259336e-09f;
  // beyond |x| = 16, E is 0 in binary32; fmin / fmax drop a NaN, which the last line restores
  const float xc = __builtin_fminf(__builtin_fmaxf(x, -16.0f), 16.0f);
  const double xd = (double)xc;
  const double a = __builtin_fabs(xd) * WF2_FMA(K2, xd * xd, K1);  // <= 460
  const double td = a + kRoundMagic;
  const int32_t ni = (int32_t)(uint32_t)bits_of(td);
  const float p = (float)(a - (td - kRoundMagic));  // a = n + p, |p| <= 1/2
  const float r = __builtin_fmaf(p, -Ln2l, p * -Ln2h);
  const float w = __builtin_fmaf(r * r, exp_q32(r), r);
  const float E = WF2_LDEXPF(1.0f + w, -ni);
  const float D = 1.0f + E, Dl = (1.0f - D) + E;  // exact two-term sum
  // the numerator without its factor 2^-n, which is applied last: x E may be a normal
  // number where E alone is subnormal
  const bool right = xc >= 0.0f;
  const float num = right ? xc : __builtin_fmaf(xc, w, xc);
  const float y0 = WF2_FAST_RCPF(D);
  const float q0 = num * y0;
  const float q = __builtin_fmaf(__builtin_fmaf(-q0, Dl, __builtin_fmaf(-q0, D, num)), y0, q0);
  const float res = WF2_LDEXPF(q, right ? 0 : -ni);
  // |x| >= 16 (or NaN): x on the right, -0 on the left (x e^{2u} underflows)
  const float far = (x != x) ? x : __builtin_fmaxf(x, -0.0f);
  return (__builtin_fabsf(x) < 16.0f) ? res : far;
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

// d/dx of the tanh-form GELU, x / (1 + E) with E = 2^t, t = x (k1 + k2 x^2):
//   g'(x) = s (1 + x (1 - s) v),  s = 1 / (1 + E),  v = 2 sqrt(2/pi) (1 + 3 * 0.044715 x^2).
// s and 1 - s are both formed from e = 2^-|t| <= 1 (no cancellation, no overflow):
// (s, 1 - s) = (r, e r) for x >= 0 and (e r, r) for x < 0 with r = 1 / (1 + e).
// Error: three roundings of t (1e-7 |t| absolute in the exponent) and one ulp each
// from v_exp_f32, v_rcp_f32 and the products: below 1e-6 of |s| + |x s (1 - s) v|
// for |x| <= 4 (host sweep: 7.7e-7), growing with |t| in the left tail to 1e-5 at
// x = -10, where g' is 1e-33; g' has a zero near x = -0.75, so no bound relative to
// g' itself exists.  Beyond |x| = 16, e is 0 in binary32: g' = 1 on the right, 0 on
// the left; v_exp_f32 returns 0 below 2^-126, so gradients under about 2^-120 (x < -6.9)
// are flushed to 0.  15 VALU operations.
WF2_MATH_FN float gelu_tanh_grad_f(float x) {
  const float k1 = -2.3022082f;    // -2 sqrt(2/pi) log2(e)
  const float k2 = -0.10294324f;   // k1 * 0.044715
  const float c1 = 1.5957691f;     // 2 sqrt(2/pi)
  const float c2 = 0.21406446f;    // c1 * 3 * 0.044715
  const float xc = __builtin_fminf(__builtin_fmaxf(x, -16.0f), 16.0f);  // drops a NaN, restored below
  const float x2 = xc * xc;
  const float t = xc * __builtin_fmaf(k2, x2, k1);
  const float e = WF2_FAST_EXP2F(-__builtin_fabsf(t));
  const float r = WF2_FAST_RCPF(1.0f + e);
  const float er = e * r;
  const bool right = xc >= 0.0f;
  const float sg = right ? r : er;
  const float cs = right ? er : r;
  const float v = __builtin_fmaf(c2, x2, c1);
  const float res = sg * __builtin_fmaf(xc * cs, v, 1.0f);
  return (x != x) ? x : res;
}

}  // namespace wf2
