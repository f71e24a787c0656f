// optim.hip -- optimiser steps as one pass over the parameter.
//
// cl-waffe2's optimisers are compositions of element-wise nodes:
//   SGD   (optimizers/impls/sgd.lisp:18-34)   grad *= lr ; param -= grad
//   Adam  (optimizers/impls/adam.lisp:45-117) m += (g - m) (1 - b1)
//                                             v += (1 - b2) (g g - v)
//                                             param -= (m lr_t) / (eps + sqrt v)
// which on the node path means a dozen launches and about 100 bytes of traffic
// per parameter.  The kernels here perform the same binary32 operations in the
// same order (each one rounded, no contraction), so the result is bit-identical
// to the node sequence, with 16 (SGD) or 28 (Adam) bytes per parameter.
// HBM-bound.
#include "wf2_common.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void adam1(float& p, float g, float& m, float& v, float omb1, float omb2,
                                      float lr_t, float eps) {
  m = m + (g - m) * omb1;
  v = v + omb2 * (g * g - v);
  p = p - (m * lr_t) / (eps + __builtin_sqrtf(v));
}

// VEC: four 16-byte vectors per thread and stream (2^26 parameters: one 65 %, two 76 %, four 78 %,
// eight 67 % of the HBM peak), all loads issued before the arithmetic; NT: streaming hint for tensors far beyond the Infinity Cache.
template <bool VEC, bool NT, bool FULL = false>
__global__ __launch_bounds__(kBlock) void adam_kernel(float* __restrict__ p, const float* __restrict__ g,
                                                      float* __restrict__ m, float* __restrict__ v,
                                                      size_t n, float omb1, float omb2, float lr_t,
                                                      float eps) {
  if (VEC) {
    constexpr int U = 4;
    const size_t nvec = n / 4;
    // each wavefront on 1 KB of its own per access and stream
    const size_t base = ((size_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * kWave * U +
                        (threadIdx.x & (kWave - 1));
    f4 pv[U], gv[U], mv[U], vv[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        pv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<f4*>(p) + i) : reinterpret_cast<f4*>(p)[i];
        gv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<const f4*>(g) + i)
                   : reinterpret_cast<const f4*>(g)[i];
        mv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<f4*>(m) + i) : reinterpret_cast<f4*>(m)[i];
        vv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<f4*>(v) + i) : reinterpret_cast<f4*>(v)[i];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          float pe = pv[u][c], me = mv[u][c], ve = vv[u][c];
          adam1(pe, gv[u][c], me, ve, omb1, omb2, lr_t, eps);
          pv[u][c] = pe;
          mv[u][c] = me;
          vv[u][c] = ve;
        }
        if (NT) {
          __builtin_nontemporal_store(pv[u], reinterpret_cast<f4*>(p) + i);
          __builtin_nontemporal_store(mv[u], reinterpret_cast<f4*>(m) + i);
          __builtin_nontemporal_store(vv[u], reinterpret_cast<f4*>(v) + i);
        } else {
          reinterpret_cast<f4*>(p)[i] = pv[u];
          reinterpret_cast<f4*>(m)[i] = mv[u];
          reinterpret_cast<f4*>(v)[i] = vv[u];
        }
      }
    }
    if (!FULL && blockIdx.x == 0 && threadIdx.x < (n & 3)) {
      const size_t j = nvec * 4 + threadIdx.x;
      adam1(p[j], g[j], m[j], v[j], omb1, omb2, lr_t, eps);
    }
  } else {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) adam1(p[i], g[i], m[i], v[i], omb1, omb2, lr_t, eps);
  }
}

// VEC: four 16-byte vectors per lane and stream, wave-contiguous, loads first
// (the shape measured best for x <- x op y); NT as above.
template <bool VEC, bool NT, bool FULL = false>
__global__ __launch_bounds__(kBlock) void sgd_kernel(float* __restrict__ p, float* __restrict__ g,
                                                     size_t n, float lr) {
  if (VEC) {
    constexpr int U = 4;
    const size_t nvec = n / 4;
    const size_t base = ((size_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * kWave * U +
                        (threadIdx.x & (kWave - 1));
    f4 pv[U], gv[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        pv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<f4*>(p) + i) : reinterpret_cast<f4*>(p)[i];
        gv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<f4*>(g) + i) : reinterpret_cast<f4*>(g)[i];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        gv[u] = gv[u] * lr;
        pv[u] = pv[u] - gv[u];
        if (NT) {
          __builtin_nontemporal_store(gv[u], reinterpret_cast<f4*>(g) + i);
          __builtin_nontemporal_store(pv[u], reinterpret_cast<f4*>(p) + i);
        } else {
          reinterpret_cast<f4*>(g)[i] = gv[u];
          reinterpret_cast<f4*>(p)[i] = pv[u];
        }
      }
    }
    if (!FULL && blockIdx.x == 0 && threadIdx.x < (n & 3)) {
      const size_t j = nvec * 4 + threadIdx.x;
      g[j] = g[j] * lr;
      p[j] = p[j] - g[j];
    }
  } else {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) {
      g[i] = g[i] * lr;
      p[i] = p[i] - g[i];
    }
  }
}

static bool disjoint(const float* a, const float* b, size_t n) { return a + n <= b || b + n <= a; }
static bool aligned16(const void* q) { return ((uintptr_t)q & 15u) == 0; }

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_adam_step_f32(long n, float* param, const float* grad, float* m, float* v,
                                 float one_minus_beta1, float one_minus_beta2, float lr_t, float eps) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  if (n == 0) return 0;
  if (!param || !grad || !m || !v) return fail(WF2HIP_EINVAL, "null tensor pointer");
  const float* all[4] = {param, grad, m, v};
  for (int a = 0; a < 4; a++)
    for (int b = a + 1; b < 4; b++)
      if (!disjoint(all[a], all[b], (size_t)n))
        return fail(WF2HIP_EOVERLAP, "adam step: parameter, gradient and moments must not overlap");
  const bool vec = aligned16(param) && aligned16(grad) && aligned16(m) && aligned16(v);
  const int64_t nvec = n / 4 > 0 ? n / 4 : 1;
  const int64_t blocks = vec ? ceil_div(nvec, (int64_t)kBlock * 4) : ceil_div(n, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many elements for one launch");
  hipStream_t st = rt().stream;
  const bool streaming = (int64_t)n * 28 >= ((int64_t)192 << 20);
  // every workgroup full: no bounds tests, so all sixteen loads of a thread are issued before its first
  // wait (2^26 parameters with two vectors per thread and stream: 315.4 -> 304.2 us)
  if (vec && streaming && n % (4 * kBlock * 4) == 0)
    adam_kernel<true, true, true><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, m, v, (size_t)n,
                                                                      one_minus_beta1, one_minus_beta2, lr_t, eps);
  else if (vec && streaming)
    adam_kernel<true, true><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, m, v, (size_t)n,
                                                                one_minus_beta1, one_minus_beta2, lr_t, eps);
  else if (vec)
    adam_kernel<true, false><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, m, v, (size_t)n,
                                                                 one_minus_beta1, one_minus_beta2, lr_t, eps);
  else
    adam_kernel<false, false><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, m, v, (size_t)n,
                                                                  one_minus_beta1, one_minus_beta2, lr_t, eps);
  return after_launch("adam_kernel");
}

WF2_API int wf2hip_sgd_step_f32(long n, float* param, float* grad, float lr) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  if (n == 0) return 0;
  if (!param || !grad) return fail(WF2HIP_EINVAL, "null tensor pointer");
  if (!disjoint(param, grad, (size_t)n))
    return fail(WF2HIP_EOVERLAP, "sgd step: parameter and gradient must not overlap");
  const bool vec = aligned16(param) && aligned16(grad);
  const int64_t nvec = n / 4 > 0 ? n / 4 : 1;
  const int64_t blocks = vec ? ceil_div(nvec, (int64_t)kBlock * 4) : ceil_div(n, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many elements for one launch");
  hipStream_t st = rt().stream;
  const bool streaming = (int64_t)n * 16 >= ((int64_t)192 << 20);
  // (the form without bounds tests that Adam gains 3 points from measures 0.5 - 1.5 points lower here)
  if (vec && streaming)
    sgd_kernel<true, true><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, (size_t)n, lr);
  else if (vec)
    sgd_kernel<true, false><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, (size_t)n, lr);
  else
    sgd_kernel<false, false><<<(uint32_t)blocks, kBlock, 0, st>>>(param, grad, (size_t)n, lr);
  return after_launch("sgd_kernel");
}
