"""Regenerates the polynomial coefficients in wf2_math.h.

Each core function is evaluated in binary64 on the device and rounded to
binary32 once at the end, so the fits only need a relative error well below
2^-30.  Chebyshev interpolation in 60-digit arithmetic gives near-minimax
polynomials; the script prints the coefficients (lowest order first) and the
measured maximum relative error of the double-precision evaluation.
"""
import mpmath as mp

mp.mp.dps = 60


def fit(f, a, b, deg):
    c = mp.chebyfit(f, [a, b], deg + 1)  # highest order first
    return [c[len(c) - 1 - i] for i in range(len(c))]


def show(name, coeffs):
    print(f"// {name}")
    for i, c in enumerate(coeffs):
        print(f"  {mp.nstr(c, 19)},  // c{i}")


def horner(coeffs, x):
    acc = mp.mpf(0)
    for c in reversed(coeffs):
        acc = acc * x + mp.mpf(float(c))
    return acc


def maxrel(approx, exact, a, b, n=4001):
    worst = mp.mpf(0)
    for i in range(n):
        x = a + (b - a) * mp.mpf(i) / (n - 1)
        e = exact(x)
        if e == 0:
            continue
        worst = max(worst, abs((approx(x) - e) / e))
    return worst


# exp(r) = 1 + r + r^2 * Q(r),  |r| <= 0.35
def qexp(r):
    return (mp.exp(r) - 1 - r) / (r * r) if r != 0 else mp.mpf(1) / 2


Q = fit(qexp, -0.35, 0.35, 5)
show("EXP_Q: exp(r) = 1 + r + r^2*Q(r), |r| <= 0.35, degree 5", Q)
print("// max rel err exp  :", mp.nstr(maxrel(lambda r: 1 + r + r * r * horner(Q, r), mp.exp, -0.35, 0.35), 5))
print("// max rel err expm1:", mp.nstr(maxrel(lambda r: r + r * r * horner(Q, r), mp.expm1, -0.35, 0.35), 5))

# log(1+f) = f - f^2/2 + f^3 * R(f),  f in [sqrt(1/2)-1, sqrt(2)-1]
LO, HI = mp.sqrt(mp.mpf(1) / 2) - 1 - mp.mpf("1e-6"), mp.sqrt(2) - 1 + mp.mpf("1e-6")


def rlog(f):
    if abs(f) < mp.mpf("1e-12"):
        return mp.mpf(1) / 3
    return (mp.log1p(f) - f + f * f / 2) / f**3


R = fit(rlog, LO, HI, 11)
show("LOG_R: log(1+f) = f - f^2/2 + f^3*R(f), f in [sqrt(.5)-1, sqrt(2)-1], degree 11", R)
print("// max rel err log1p:", mp.nstr(maxrel(lambda f: f - f * f / 2 + f**3 * horner(R, f), mp.log1p, LO, HI), 5))

# sin(r) = r + r^3 * S(r^2); cos(r) = 1 - z/2 + z^2*C(z), |r| <= pi/4 (+slack)
ZMAX = (mp.pi / 4 + mp.mpf("1e-3")) ** 2


def ssin(z):
    if z < mp.mpf("1e-20"):
        return -mp.mpf(1) / 6
    r = mp.sqrt(z)
    return (mp.sin(r) - r) / (r * z)


def ccos(z):
    if z < mp.mpf("1e-14"):
        return mp.mpf(1) / 24
    r = mp.sqrt(z)
    return (mp.cos(r) - 1 + z / 2) / (z * z)


S = fit(ssin, 0, ZMAX, 3)
Cc = fit(ccos, 0, ZMAX, 3)
show("SIN_S: sin(r) = r + r^3*S(r^2), degree 3 in z", S)
show("COS_C: cos(r) = 1 - z/2 + z^2*C(z), degree 3 in z", Cc)
rm = mp.pi / 4 + mp.mpf("1e-3")
print("// max rel err sin:", mp.nstr(maxrel(lambda r: r + r**3 * horner(S, r * r), mp.sin, -rm, rm), 5))
print("// max rel err cos:", mp.nstr(maxrel(lambda r: 1 - r * r / 2 + r**4 * horner(Cc, r * r), mp.cos, -rm, rm), 5))

# pi/2 split for the binary64 Cody-Waite reduction: the head keeps 33
# significant bits so that q*head is exact for |q| < 2^20.
pio2 = mp.pi / 2
head = mp.ldexp(mp.floor(mp.ldexp(pio2, 32)), -32)
tail = pio2 - head
print("// PIO2_HEAD =", mp.nstr(head, 25), " PIO2_TAIL =", mp.nstr(tail, 25))
print("// 2/pi =", mp.nstr(2 / mp.pi, 25), " log2(e) =", mp.nstr(1 / mp.log(2), 25))
ln2 = mp.log(2)
lh = mp.ldexp(mp.floor(mp.ldexp(ln2, 32)), -32)
print("// LN2_HEAD =", mp.nstr(lh, 25), " LN2_TAIL =", mp.nstr(ln2 - lh, 25), " LN2 =", mp.nstr(ln2, 25))

# atan(t) = t + t^3 * P(t^2), |t| <= tan(pi/8)
TAN_PIO8 = mp.tan(mp.pi / 8)


def patan(z):
    if z < mp.mpf("1e-20"):
        return -mp.mpf(1) / 3
    t = mp.sqrt(z)
    return (mp.atan(t) - t) / (t * z)


P = fit(patan, 0, TAN_PIO8 ** 2, 9)
show("ATAN_P: atan(t) = t + t^3*P(t^2), |t| <= tan(pi/8), degree 9 in z", P)
print("// max rel err atan:", mp.nstr(maxrel(lambda t: t + t**3 * horner(P, t * t), mp.atan, mp.mpf("1e-6"), TAN_PIO8), 5))
print("// 1/ln2 =", mp.nstr(1 / mp.log(2), 25), " 1/ln10 =", mp.nstr(1 / mp.log(10), 25),
      " pi/2 =", mp.nstr(mp.pi / 2, 25), " pi/4 =", mp.nstr(mp.pi / 4, 25), " tan(pi/8) =", mp.nstr(TAN_PIO8, 20))


# ---- binary32 tails --------------------------------------------------------------
# The high-order remainders of exp (tanh, GELU), log, sin and cos are evaluated in
# binary32 on the device; the fits below are printed rounded to binary32 and the
# errors are measured with binary32 Horner arithmetic on a binary32 argument.
import numpy as np


def horner32(coeffs, x):
    acc = np.float32(0)
    for c in reversed(coeffs):
        acc = np.float32(acc * np.float32(float(x)) + np.float32(float(c)))
    return mp.mpf(float(acc))


def show32(name, coeffs):
    print(f"// {name}")
    for i, c in enumerate(coeffs):
        print(f"  {float(np.float32(float(c)))!r}f,  // c{i}")


def q4exp(r):
    if abs(r) < mp.mpf("1e-8"):
        return mp.mpf(1) / 24
    return (mp.exp(r) - 1 - r - r * r / 2 - r**3 / 6) / r**4


Q4 = fit(q4exp, -0.35, 0.35, 4)
show32("EXP_Q4: expm1(r) = r + r^2/2 + r^3/6 + r^4*Q4(r), |r| <= 0.35, degree 4", Q4)
print("// max rel err expm1:", mp.nstr(maxrel(lambda r: r + r * r / 2 + r**3 / 6 + r**4 * horner32(Q4, r), mp.expm1,
                                               mp.mpf(-0.35), mp.mpf(0.35)), 5))


def r5log(f):
    if abs(f) < mp.mpf("1e-6"):
        return mp.mpf(1) / 5 - f / 6
    return (mp.log1p(f) - f + f * f / 2 - f**3 / 3 + f**4 / 4) / f**5


R5 = fit(r5log, LO, HI, 8)
show32("LOG_R5: log(1+f) = f - f^2/2 + f^3/3 - f^4/4 + f^5*R5(f), degree 8", R5)
print("// max rel err log1p:", mp.nstr(maxrel(lambda f: f - f * f / 2 + f**3 / 3 - f**4 / 4 + f**5 * horner32(R5, f),
                                               mp.log1p, LO, HI), 5))


def s5sin(z):
    if z < mp.mpf("1e-12"):
        return mp.mpf(1) / 120
    r = mp.sqrt(z)
    return (mp.sin(r) - r + r**3 / 6) / r**5


def c3cos(z):
    if z < mp.mpf("1e-8"):
        return -mp.mpf(1) / 720
    r = mp.sqrt(z)
    return (mp.cos(r) - 1 + z / 2 - z * z / 24) / z**3


S5 = fit(s5sin, 0, ZMAX, 2)
C3 = fit(c3cos, 0, ZMAX, 2)
show32("SIN_S5: sin(r) = r - r^3/6 + r^5*S5(r^2), degree 2 in z", S5)
show32("COS_C3: cos(r) = 1 - z/2 + z^2/24 + z^3*C3(z), degree 2 in z", C3)
print("// max rel err sin:", mp.nstr(maxrel(lambda r: r - r**3 / 6 + r**5 * horner32(S5, r * r), mp.sin,
                                             mp.mpf("1e-3"), rm), 5))
print("// max rel err cos:", mp.nstr(maxrel(lambda r: 1 - r * r / 2 + r**4 / 24 + r**6 * horner32(C3, r * r), mp.cos,
                                             mp.mpf(0), rm), 5))
lh45 = mp.ldexp(mp.floor(mp.ldexp(ln2, 45)), -45)
print("// LN2_HEAD45 =", float(lh45).hex(), " dropped:", mp.nstr(ln2 - lh45, 5))
