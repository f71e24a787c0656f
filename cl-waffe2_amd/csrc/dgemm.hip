// dgemm.hip -- MatMulNode on :double tensors.
//
// The CPU backend sends :double products to BLAS dgemm_ (source/backends/cpu/
// matrix-ops.lisp:12-112 expands to sgemm_ or dgemm_ by dtype; binding
// blas-functions.lisp:34-38).  This is the same contract as wf2hip_sgemm --
// column-major C(m x n) <- alpha op(A) op(B) + beta C, scalars by value -- on
// binary64 on the matrix cores (v_mfma_f64_16x16x4, fused multiply-add).  It is a
// plain LDS-tiled kernel (128 x 128 or 64 x 64 outputs per workgroup, a quarter
// per wavefront, K in steps of 16 with the next step prefetched into registers): the :double path is there so that
// models keep running on the device, the tuned kernels are the :float ones in
// gemm.hip.
#include <algorithm>

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
  int64_t kslice;  // > 0: blockIdx.z names a slice of K of this length (a single product split over K)
};

typedef double d4 __attribute__((ext_vector_type(4)));

constexpr int kDK = 16;   // K step

// TILE x TILE outputs per workgroup of four wavefronts (2 x 2), TILE / 2 squared per wavefront as
// (TILE / 32)^2 matrix-core tiles.  The next K step's operands are fetched into registers while the
// current one is multiplied out of LDS.
template <bool TA, bool TB, int TILE>
__global__ __launch_bounds__(kBlock) void dgemm_kernel(DgemmParams p) {
  constexpr int NT = TILE / 32;              // matrix-core tiles per wavefront and dimension
  constexpr int PER = TILE * kDK / kBlock;   // elements of each operand per thread and K step
  __shared__ double As[kDK][TILE + 1];
  __shared__ double Bs[kDK][TILE + 1];
  const uint32_t bi = blockIdx.z % p.batch_inner, bo = blockIdx.z / p.batch_inner;
  const double* A = p.A + (int64_t)bi * p.sA + (int64_t)bo * p.sA2;
  const double* B = p.B + (int64_t)bi * p.sB + (int64_t)bo * p.sB2;
  double* C = p.C + (int64_t)bi * p.sC + (int64_t)bo * p.sC2;
  int64_t kbeg = 0, kend = p.k;
  if (p.kslice > 0) {  // batch_inner is the slice count and only sC is set: slice z writes its own m x n plane
    kbeg = (int64_t)blockIdx.z * p.kslice;
    kend = kbeg + p.kslice < p.k ? kbeg + p.kslice : p.k;
  }
  const int64_t i0 = (int64_t)blockIdx.x * TILE, j0 = (int64_t)blockIdx.y * TILE;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wr = (wave & 1) * (TILE / 2), wc = (wave >> 1) * (TILE / 2);
  const int l16 = lane & 15, lq = lane >> 4;
  // op(A)(i, kk) and op(B)(kk, j): consecutive threads along the axis that is contiguous in memory
  auto a_pos = [&](int r, int& i, int& kk) {
    const int e = t + kBlock * r;
    if (TA) { kk = e % kDK; i = e / kDK; } else { i = e % TILE; kk = e / TILE; }
  };
  auto b_pos = [&](int r, int& j, int& kk) {
    const int e = t + kBlock * r;
    if (TB) { j = e % TILE; kk = e / TILE; } else { kk = e % kDK; j = e / kDK; }
  };
  double ra[PER], rb[PER];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int r = 0; r < PER; r++) {
      int i, kk;
      a_pos(r, i, kk);
      const int64_t gi = i0 + i, gk = k0 + kk;
      ra[r] = (gi < p.m && gk < kend) ? (TA ? A[gk + gi * p.lda] : A[gi + gk * p.lda]) : 0.0;
      int j, kb;
      b_pos(r, j, kb);
      const int64_t gj = j0 + j, gkb = k0 + kb;
      rb[r] = (gj < p.n && gkb < kend) ? (TB ? B[gj + gkb * p.ldb] : B[gkb + gj * p.ldb]) : 0.0;
    }
  };
  d4 acc[NT][NT] = {};
  if (kend > kbeg) fetch(kbeg);
  for (int64_t k0 = kbeg; k0 < kend; k0 += kDK) {
#pragma unroll
    for (int r = 0; r < PER; r++) {
      int i, kk, j, kb;
      a_pos(r, i, kk);
      As[kk][i] = ra[r];
      b_pos(r, j, kb);
      Bs[kb][j] = rb[r];
    }
    __syncthreads();
    if (k0 + kDK < kend) fetch(k0 + kDK);
#pragma unroll
    for (int kk = 0; kk < kDK; kk += 4) {
      // v_mfma_f64_16x16x4: D(16 x 16) += L(16 x 4) R(4 x 16); lane l supplies L[l%16][l/16] and
      // R[l/16][l%16] and holds D[l/16 + 4 r][l%16] in register r (rows interleaved, unlike the
      // binary32 forms).  L is taken from op(B) and R from op(A), so that D is the transposed
      // output tile and l%16 runs along C's contiguous (row) index.
      double a[NT], b[NT];
#pragma unroll
      for (int u = 0; u < NT; u++) {
        a[u] = As[kk + lq][wr + 16 * u + l16];
        b[u] = Bs[kk + lq][wc + 16 * u + l16];
      }
#pragma unroll
      for (int u = 0; u < NT; u++)
#pragma unroll
        for (int v = 0; v < NT; v++)
          acc[u][v] = __builtin_amdgcn_mfma_f64_16x16x4f64(b[v], a[u], acc[u][v], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < NT; u++)
#pragma unroll
    for (int v = 0; v < NT; v++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int64_t gi = i0 + wr + 16 * u + l16, gj = j0 + wc + 16 * v + lq + 4 * r;
        if (gi < p.m && gj < p.n) {
          double* c = C + gi + gj * p.ldc;
          const double x = acc[u][v][r];
          *c = p.beta == 0.0 ? p.alpha * x : p.alpha * x + p.beta * *c;
        }
      }
}

template <int TILE>
static void launch_dgemm(const DgemmParams& p, bool ta, bool tb, dim3 grid, hipStream_t st) {
  if (ta && tb) dgemm_kernel<true, true, TILE><<<grid, kBlock, 0, st>>>(p);
  else if (ta) dgemm_kernel<true, false, TILE><<<grid, kBlock, 0, st>>>(p);
  else if (tb) dgemm_kernel<false, true, TILE><<<grid, kBlock, 0, st>>>(p);
  else dgemm_kernel<false, false, TILE><<<grid, kBlock, 0, st>>>(p);
}

// C <- beta C + the sum of the `splits` planes of a product split over K (planes packed m x n, already
// scaled by alpha): a wavefront per output element, lane l adds planes l, l + 64, ... and the lanes meet by
// shuffles -- a fixed order.
__global__ __launch_bounds__(kBlock) void dgemm_fold(const double* __restrict__ partials, int splits, int64_t m,
                                                     int64_t n, double beta, double* __restrict__ C, int64_t ldc) {
  const int64_t e = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (e >= m * n) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t plane = m * n;
  double acc = 0.0;
  for (int s = lane; s < splits; s += kWave) acc += partials[(int64_t)s * plane + e];
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) {
    const int64_t j = e / m, i = e - j * m;
    double* c = C + i + j * ldc;
    *c = beta == 0.0 ? acc : beta * *c + acc;
  }
}

bool try_dgemm_small_batch(bool ta, bool tb, long m, long n, long k, double alpha, const double* A, long lda, long sA,
                           long sA2, const double* B, long ldb, long sB, long sB2, double beta, double* C, long ldc,
                           long sC, long sC2, long batch, long batch2, int* rc);  // gemm_skinny.hip

// up to 16 planes: an output element per thread, the planes added in order
__global__ __launch_bounds__(kBlock) void dgemm_fold_few(const double* __restrict__ partials, int splits, int64_t m,
                                                         int64_t n, double beta, double* __restrict__ C, int64_t ldc) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= m * n) return;
  const int64_t plane = m * n;
  double acc = 0.0;
  for (int s = 0; s < splits; s++) acc += partials[(int64_t)s * plane + e];
  const int64_t j = e / m, i = e - j * m;
  double* c = C + i + j * ldc;
  *c = beta == 0.0 ? acc : beta * *c + acc;
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
  {  // many small matrices: an output element per thread or wavefront
    int rc = 0;
    if (try_dgemm_small_batch(!dn(transa), !dn(transb), m, n, k, alpha, A, lda, strideA, strideA2, B, ldb, strideB,
                              strideB2, beta, C, ldc, strideC, strideC2, batch, batch2, &rc))
      return rc;
  }
  DgemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.m = m; p.n = n; p.k = k;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.sA = strideA; p.sB = strideB; p.sC = strideC;
  p.sA2 = strideA2; p.sB2 = strideB2; p.sC2 = strideC2;
  p.batch_inner = (uint32_t)batch;
  p.alpha = alpha; p.beta = beta;
  p.kslice = 0;
  hipStream_t st = rt().stream;
  const bool ta = !dn(transa), tb = !dn(transb);
  // A single product with few output tiles over a long K ((10 x 1048576) . (1048576 x 10) ran 66 ms on one
  // workgroup): slices of K of at least 512, as many as keep four workgroups per compute unit, each into a
  // plane of its own, folded in a fixed order afterwards.
  const int64_t small_tiles = ceil_div(m, 64) * ceil_div(n, 64);
  // (K of 512 ... 2047, a layer applied to a few hundred rows: slices of at least 256)
  if (batch == 1 && batch2 == 1 && k >= 512 && small_tiles < (int64_t)rt().num_cus) {
    int64_t splits = std::min<int64_t>(k / (k >= 2048 ? 512 : 256), 4 * (int64_t)rt().num_cus / small_tiles);
    splits = std::min<int64_t>(splits, 4096);
    const int64_t kslice = ceil_div(ceil_div(k, splits), (int64_t)kDK) * kDK;
    splits = ceil_div(k, kslice);
    void* scratch = nullptr;
    int held_up = 0;
    if (splits >= 2 && !scratch_block(&scratch, (size_t)splits * m * n * sizeof(double), &held_up) && held_up)
      return held_up;
    if (scratch) {
      DgemmParams q = p;
      q.C = static_cast<double*>(scratch);
      q.ldc = m;
      q.sA = q.sB = q.sA2 = q.sB2 = q.sC2 = 0;
      q.sC = (int64_t)m * n;
      q.batch_inner = (uint32_t)splits;
      q.beta = 0.0;
      q.kslice = kslice;
      dim3 grid((uint32_t)ceil_div(m, 64), (uint32_t)ceil_div(n, 64), (uint32_t)splits);
      launch_dgemm<64>(q, ta, tb, grid, st);
      int rc = after_launch("dgemm_kernel");
      if (rc == 0) {
        if (splits <= 16)
          dgemm_fold_few<<<(uint32_t)ceil_div((int64_t)m * n, (int64_t)kBlock), kBlock, 0, st>>>(
              static_cast<const double*>(scratch), (int)splits, m, n, beta, C, ldc);
        else
          dgemm_fold<<<(uint32_t)ceil_div((int64_t)m * n, kBlock / kWave), kBlock, 0, st>>>(
              static_cast<const double*>(scratch), (int)splits, m, n, beta, C, ldc);
        rc = after_launch("dgemm_fold");
      }
      (void)wf2hip_free(scratch);  // stream order keeps it alive for the launches above
      return rc;
    }
  }
  // 128 x 128 tiles once they fill the chip twice over, 64 x 64 below that
  const int64_t big = ceil_div(m, 128) * ceil_div(n, 128) * batch * batch2;
  const int tile = big >= 2 * (int64_t)rt().num_cus ? 128 : 64;
  const int64_t gx = ceil_div(m, tile), gy = ceil_div(n, tile);
  if (gx >= ((int64_t)1 << 31) || gy > 65535) return fail(WF2HIP_EUNSUPPORTED, "matrix too large for one launch");
  dim3 grid((uint32_t)gx, (uint32_t)gy, (uint32_t)(batch * batch2));
  if (tile == 128) launch_dgemm<128>(p, ta, tb, grid, st);
  else launch_dgemm<64>(p, ta, tb, grid, st);
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
