// wf2_fastdiv.h -- division of 32-bit indices by a divisor fixed at launch.
//
// For 1 <= d < 2^31 and 0 <= n < 2^31: with p = 31 + ceil(log2 d) and m = ceil(2^p / d)
// (m < 2^32 because d > 2^(ceil(log2 d) - 1)), floor(n / d) = (n m) >> p.  n m / 2^p exceeds
// n / d by n (m d - 2^p) / (d 2^p) < n / 2^p <= 2^31 / (2^31 d) = 1 / d, too little to reach
// the next integer from a quotient whose fractional part is at most (d - 1) / d.
// A multiply-high and a shift where the compiler's expansion of n / d takes about
// twenty instructions.  Compiles for the host as well (the index maps are checked there).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define WF2_FD_FN __host__ __device__ __forceinline__
#else
#define WF2_FD_FN inline
#endif

namespace wf2 {

struct FastDiv {
  uint32_t d, mul, shr;
};

inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  if (d <= 1) {
    f.mul = 0;
    f.shr = 0;
    return f;
  }
  uint32_t lg = 0;
  while (((uint64_t)1 << lg) < d) lg++;  // ceil(log2 d)
  const uint32_t p = 31 + lg;
  f.mul = (uint32_t)((((uint64_t)1 << p) + d - 1) / d);
  f.shr = p - 32;
  return f;
}

WF2_FD_FN uint32_t mulhi_u32(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umulhi(a, b);
#else
  return (uint32_t)(((uint64_t)a * b) >> 32);
#endif
}

// n / f.d for n < 2^31
WF2_FD_FN uint32_t fd_div(uint32_t n, const FastDiv& f) { return f.d == 1 ? n : (mulhi_u32(n, f.mul) >> f.shr); }

// quotient, and the remainder through *rem
WF2_FD_FN uint32_t fd_divmod(uint32_t n, const FastDiv& f, uint32_t* rem) {
  const uint32_t q = fd_div(n, f);
  *rem = n - q * f.d;
  return q;
}

}  // namespace wf2
