// dgemm.hip -- MatMulNode on :double tensors.
//
// The CPU backend sends :double products to BLAS dgemm_ (source/backends/cpu/
// matrix-ops.lisp:12-112 expands to sgemm_ or dgemm_ by dtype; binding
// blas-functions.lisp:34-38).  This is the same contract as wf2hip_sgemm --
// column-major C(m x n) <- alpha op(A) op(B) + beta C, scalars by value -- on
// binary64 with FMA accumulation.  It is a plain LDS-tiled kernel on the vector
// ALUs (64 x 64 outputs per workgroup, 4 x 4 per thread, K in steps of 16): the
// :double path is there so that models keep running on the device, the tuned
// matrix-core kernels are the :float ones in gemm.hip.
#include "wf2_common.h"

namespace wf2 {

struct DgemmParams {
  const double* A;
  const double* B;
  double* C;
  int64_t m, n, k, lda, ldb, ldc;
  int64_t sA, sB, sC, sA2, sB2, sC2;  // batch strides: inner / outer level
  uint32_t batch_inner;
  double alpha, beta;
};

constexpr int kDT = 64;   // tile edge
constexpr int kDK = 16;   // K step

template <bool TA, bool TB>
__global__ __launch_bounds__(kBlock) void dgemm_kernel(DgemmParams p) {
  __shared__ double As[kDK][kDT + 1];
  __shared__ double Bs[kDK][kDT + 1];
  const uint32_t bi = blockIdx.z % p.batch_inner, bo = blockIdx.z / p.batch_inner;
  const double* A = p.A + (int64_t)bi * p.sA + (int64_t)bo * p.sA2;
  const double* B = p.B + (int64_t)bi * p.sB + (int64_t)bo * p.sB2;
  double* C = p.C + (int64_t)bi * p.sC + (int64_t)bo * p.sC2;
  const int64_t i0 = (int64_t)blockIdx.x * kDT, j0 = (int64_t)blockIdx.y * kDT;
  const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
  double acc[4][4] = {};
  for (int64_t k0 = 0; k0 < p.k; k0 += kDK) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      // op(A)(i, kk): consecutive threads along the axis that is contiguous in memory
      const int i = TA ? (t >> 4) + 16 * r : (t & 63);
      const int kk = TA ? (t & 15) : (t >> 6) + 4 * r;
      const int64_t gi = i0 + i, gk = k0 + kk;
      double v = 0.0;
      if (gi < p.m && gk < p.k) v = TA ? A[gk + gi * p.lda] : A[gi + gk * p.lda];
      As[kk][i] = v;
      // op(B)(kk, j)
      const int j = TB ? (t & 63) : (t >> 4) + 16 * r;
      const int kb = TB ? (t >> 6) + 4 * r : (t & 15);
      const int64_t gj = j0 + j, gkb = k0 + kb;
      double w = 0.0;
      if (gj < p.n && gkb < p.k) w = TB ? B[gj + gkb * p.ldb] : B[gkb + gj * p.ldb];
      Bs[kb][j] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kDK; kk++) {
      double a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        a[u] = As[kk][tx + 16 * u];
        b[u] = Bs[kk][ty + 16 * u];
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[u][v] = __builtin_fma(a[u], b[v], acc[u][v]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < 4; u++)
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int64_t gi = i0 + tx + 16 * u, gj = j0 + ty + 16 * v;
      if (gi < p.m && gj < p.n) {
        double* c = C + gi + gj * p.ldc;
        *c = p.beta == 0.0 ? p.alpha * acc[u][v] : p.alpha * acc[u][v] + p.beta * *c;
      }
    }
}

static bool dn(char c) { return c == 'N' || c == 'n'; }
static bool dt(char c) { return c == 'T' || c == 't' || c == 'C' || c == 'c'; }

static int dgemm_batched2(char transa, char transb, long m, long n, long k, double alpha, const double* A, long lda,
                          long strideA, long strideA2, const double* B, long ldb, long strideB, long strideB2,
                          double beta, double* C, long ldc, long strideC, long strideC2, long batch, long batch2) {
  WF2_TRY(require_init());
  if (!(dn(transa) || dt(transa)) || !(dn(transb) || dt(transb))) return fail(WF2HIP_EINVAL, "trans must be N, T or C");
  if (m < 0 || n < 0 || k < 0 || batch < 0 || batch2 < 0) return fail(WF2HIP_EINVAL, "negative dimension");
  const long rows_a = dn(transa) ? m : k, rows_b = dn(transb) ? k : n;
  if (lda < (rows_a > 1 ? rows_a : 1) || ldb < (rows_b > 1 ? rows_b : 1) || ldc < (m > 1 ? m : 1))
    return fail(WF2HIP_EINVAL, "leading dimension too small (lda %ld ldb %ld ldc %ld)", lda, ldb, ldc);
  if (m == 0 || n == 0 || batch == 0 || batch2 == 0) return 0;
  if (!A || !B || !C) return fail(WF2HIP_EINVAL, "null matrix pointer");
  if ((int64_t)batch * batch2 > 65535) return fail(WF2HIP_EUNSUPPORTED, "more than 65535 matrices in one batch");
  DgemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.m = m; p.n = n; p.k = k;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.sA = strideA; p.sB = strideB; p.sC = strideC;
  p.sA2 = strideA2; p.sB2 = strideB2; p.sC2 = strideC2;
  p.batch_inner = (uint32_t)batch;
  p.alpha = alpha; p.beta = beta;
  const int64_t gx = ceil_div(m, kDT), gy = ceil_div(n, kDT);
  if (gx >= ((int64_t)1 << 31) || gy > 65535) return fail(WF2HIP_EUNSUPPORTED, "matrix too large for one launch");
  dim3 grid((uint32_t)gx, (uint32_t)gy, (uint32_t)(batch * batch2));
  hipStream_t st = rt().stream;
  const bool ta = !dn(transa), tb = !dn(transb);
  if (ta && tb) dgemm_kernel<true, true><<<grid, kBlock, 0, st>>>(p);
  else if (ta) dgemm_kernel<true, false><<<grid, kBlock, 0, st>>>(p);
  else if (tb) dgemm_kernel<false, true><<<grid, kBlock, 0, st>>>(p);
  else dgemm_kernel<false, false><<<grid, kBlock, 0, st>>>(p);
  return after_launch("dgemm_kernel");
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_dgemm(char transa, char transb, long m, long n, long k, double alpha, const double* A, long lda,
                         const double* B, long ldb, double beta, double* C, long ldc) {
  return dgemm_batched2(transa, transb, m, n, k, alpha, A, lda, 0, 0, B, ldb, 0, 0, beta, C, ldc, 0, 0, 1, 1);
}

WF2_API int wf2hip_dgemm_strided_batched_2d(char transa, char transb, long m, long n, long k, double alpha,
                                            const double* A, long lda, long strideA, long strideA2, const double* B,
                                            long ldb, long strideB, long strideB2, double beta, double* C, long ldc,
                                            long strideC, long strideC2, long batch, long batch2) {
  return dgemm_batched2(transa, transb, m, n, k, alpha, A, lda, strideA, strideA2, B, ldb, strideB, strideB2, beta, C,
                        ldc, strideC, strideC2, batch, batch2);
}
