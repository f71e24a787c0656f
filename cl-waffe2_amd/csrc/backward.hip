// backward.hip -- the row kernels of the backward pass: softmax (plain and causal)
// and LayerNorm gradients, each one pass over its rows.
//
// cl-waffe2 differentiates these layers through their node compositions
// (source/nn/activation.lisp:126-159, source/nn/norms.lisp:72-82): some twenty
// element-wise and reduction passes per layer.  Here a wavefront holds the row of
// the saved tensor and the row of the upstream gradient in registers, forms the
// row statistics with shuffles and writes the gradient once:
//   softmax    dx = scale y (dy - sum_j dy y)                      12 bytes per element
//   LayerNorm  dx = rstd (dyh - mean(dyh) - xh mean(dyh xh)),      12 bytes per element
//              dgamma = sum_rows dy xh, dbeta = sum_rows dy         (+ the partial sums)
//   softmax cross entropy  dx = (dy (z - labels)) / batch          16 bytes per element
// with xh = (x - mean) rstd and dyh = dy gamma.  All are HBM-bound.
#include <algorithm>

#include "wf2_common.h"
#include "wf2_fastdiv.h"
#include "wf2_rows.h"

namespace wf2 {

__device__ __forceinline__ int64_t ceil_div_dev(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- softmax ------------------------------------------------------------------------------------
// One wavefront per row.  With causal_seq > 0 row r holds (r % causal_seq) + 1 entries:
// what lies above the diagonal is neither read (dy may be uninitialised there, e.g. the
// skipped tiles of a triangular product) nor left unwritten (dx is 0 there).
template <int NV, bool VEC, bool NT>
__global__ __launch_bounds__(kBlock) void softmax_bwd_rows_wave(const float* __restrict__ y, int64_t ldy,
                                                                const float* dy, int64_t lddy,  // dx may be dy
                                                                float* dx, int64_t lddx,
                                                                int64_t nrows, int64_t ncols, int64_t causal_seq,
                                                                float scale) {
  const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= nrows) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t valid = causal_seq > 0 ? (row % causal_seq) + 1 : ncols;
  RowRegs<NV, VEC, NT> a, b;
  a.load(y + row * ldy, valid, lane, 0.0f);
  b.load(dy + row * lddy, valid, lane, 0.0f);
  float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int g = 0; g < NV; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) part[c] = __builtin_fmaf(b.v[g][c], a.v[g][c], part[c]);
  const float dot = (float)wave_sum(((double)part[0] + (double)part[1]) + ((double)part[2] + (double)part[3]));
#pragma unroll
  for (int g = 0; g < NV; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const bool in = RowRegs<NV, VEC, NT>::col(g, c, lane) < valid;
      const float t = scale * (a.v[g][c] * (b.v[g][c] - dot));
      a.v[g][c] = in ? t : 0.0f;
    }
  a.store(dx + row * lddx, ncols, lane);
}

// Many rows of at most 64 columns (class scores): a wavefront per row leaves most lanes idle ((1677721, 10):
// 292 us).  A workgroup takes 128 adjacent rows (64 beyond 32 columns): y and dy, one contiguous run each, are staged into LDS in
// storage order (row r at r * (ncols | 1), the odd pitch keeps a wavefront's rows on different banks), thread
// r works through row r, and dx is written in storage order.  Rows must be adjacent (pitch == ncols) in all
// three.
constexpr int kTinyCols = 64;
constexpr int kTinyFloats = 128 * 33;  // >= 64 * 65
// rows per workgroup: up to four rounds of 128 rows on rows of at most 8 columns (a group of 128 rows of two
// columns is 1 KB per tensor: the launch rate bounds the kernels)
__host__ __device__ static inline int tiny_bwd_rows_per_group(int ncols) {
  if (ncols > 32) return 64;
  if (ncols > 8) return 128;
  const int rounds = 33 / (ncols | 1);
  return 128 * (rounds > 4 ? 4 : rounds);
}

// VEC: y, dy and dx are 16-byte aligned: the runs are staged in 16-byte vectors.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void softmax_bwd_rows_tiny(const float* __restrict__ y, const float* dy,  // dx may be dy
                                                                float* dx, int64_t nrows, int ncols, float scale,
                                                                FastDiv by_c) {
  __shared__ float ty[kTinyFloats];
  __shared__ float td[kTinyFloats];
  const int pitch = ncols | 1, group = tiny_bwd_rows_per_group(ncols);
  const int64_t row0 = (int64_t)blockIdx.x * group;
  if (row0 >= nrows) return;  // a grid sized for other groups must not index past the rows
  const int rows_here = (int)(nrows - row0 < group ? nrows - row0 : group);
  const uint32_t cells = (uint32_t)rows_here * (uint32_t)ncols;
  const int64_t base = row0 * ncols;
  constexpr int U = 4;
  typedef float f4 __attribute__((ext_vector_type(4)));
  const uint32_t whole = VEC ? cells / 4 : 0;
  if constexpr (VEC) {
    for (uint32_t q0 = threadIdx.x; q0 < whole; q0 += kBlock * 2) {
      f4 a[2], b[2];
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const bool live = q0 + u * kBlock < whole;
        a[u] = live ? *reinterpret_cast<const f4*>(y + base + 4 * (int64_t)(q0 + u * kBlock)) : f4{0.f, 0.f, 0.f, 0.f};
        b[u] = live ? *reinterpret_cast<const f4*>(dy + base + 4 * (int64_t)(q0 + u * kBlock)) : f4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < 2; u++)
        if (q0 + u * kBlock < whole) {
          uint32_t col;
          uint32_t row = fd_divmod(4 * (q0 + u * kBlock), by_c, &col);
#pragma unroll
          for (int c = 0; c < 4; c++) {
            ty[row * pitch + col] = a[u][c];
            td[row * pitch + col] = b[u][c];
            if (++col == (uint32_t)ncols) {
              col = 0;
              row++;
            }
          }
        }
    }
  }
  for (uint32_t e0 = 4 * whole + threadIdx.x; e0 < cells; e0 += kBlock * U) {
    float a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bool live = e0 + u * kBlock < cells;
      a[u] = live ? y[base + e0 + u * kBlock] : 0.0f;
      b[u] = live ? dy[base + e0 + u * kBlock] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < U; u++)
      if (e0 + u * kBlock < cells) {
        uint32_t col;
        const uint32_t row = fd_divmod(e0 + u * kBlock, by_c, &col);
        ty[row * pitch + col] = a[u];
        td[row * pitch + col] = b[u];
      }
  }
  __syncthreads();
  for (int mine = threadIdx.x; mine < rows_here; mine += kBlock) {
    float* a = ty + mine * pitch;
    const float* b = td + mine * pitch;
    double acc = 0.0;
    for (int j = 0; j < ncols; j++) acc += (double)(b[j] * a[j]);
    const float dot = (float)acc;
    for (int j = 0; j < ncols; j++) a[j] = scale * (a[j] * (b[j] - dot));
  }
  __syncthreads();
  if constexpr (VEC) {
    for (uint32_t q = threadIdx.x; q < whole; q += kBlock) {
      uint32_t col;
      uint32_t row = fd_divmod(4 * q, by_c, &col);
      f4 v;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        v[c] = ty[row * pitch + col];
        if (++col == (uint32_t)ncols) {
          col = 0;
          row++;
        }
      }
      *reinterpret_cast<f4*>(dx + base + 4 * (int64_t)q) = v;
    }
  }
  for (uint32_t e = 4 * whole + threadIdx.x; e < cells; e += kBlock) {
    uint32_t col;
    const uint32_t row = fd_divmod(e, by_c, &col);
    dx[base + e] = ty[row * pitch + col];
  }
}

// Rows beyond the register tile: a workgroup per row, two passes (the second one from the L2).
__global__ __launch_bounds__(kBlock) void softmax_bwd_rows_block(const float* __restrict__ y, int64_t ldy,
                                                                 const float* dy, int64_t lddy,  // dx may be dy
                                                                 float* dx, int64_t lddx,
                                                                 int64_t ncols, int64_t causal_seq, float scale) {
  __shared__ double lds[kWavesPerBlock];
  __shared__ float stat;
  const int64_t row = blockIdx.x;
  const int64_t valid = causal_seq > 0 ? (row % causal_seq) + 1 : ncols;
  const float* yr = y + row * ldy;
  const float* dr = dy + row * lddy;
  float* xr = dx + row * lddx;
  double acc = 0.0;
  for (int64_t c = threadIdx.x; c < valid; c += kBlock) acc += (double)(dr[c] * yr[c]);
  const double total = block_sum(acc, lds);
  if (threadIdx.x == 0) stat = (float)total;
  __syncthreads();
  const float dot = stat;
  for (int64_t c = threadIdx.x; c < ncols; c += kBlock) xr[c] = c < valid ? scale * (yr[c] * (dr[c] - dot)) : 0.0f;
}

// Rows of 2049 ... 32768 columns: a workgroup of 1024 threads per row with y and dy in registers
// (thread t holds columns t, t + 1024, ...), one read of each and one write; the two-pass form
// above reads both rows twice ((4096, 50257): 832 us).
constexpr int kLongBlock = 1024;

template <int E>
__global__ __launch_bounds__(kLongBlock) void softmax_bwd_rows_long(const float* __restrict__ y, int64_t ldy,
                                                                    const float* dy, int64_t lddy,  // dx may be dy
                                                                    float* dx, int64_t lddx, int64_t ncols,
                                                                    float scale) {
  __shared__ double lds[kLongBlock / kWave];
  const float* yr = y + (int64_t)blockIdx.x * ldy;
  const float* dr = dy + (int64_t)blockIdx.x * lddy;
  float a[E], b[E];
  float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int k = 0; k < E; k++) {
    const int64_t c = (int64_t)k * kLongBlock + threadIdx.x;
    a[k] = c < ncols ? yr[c] : 0.0f;
    b[k] = c < ncols ? dr[c] : 0.0f;
  }
#pragma unroll
  for (int k = 0; k < E; k++) part[k & 3] = __builtin_fmaf(b[k], a[k], part[k & 3]);
  const double w = wave_sum(((double)part[0] + (double)part[1]) + ((double)part[2] + (double)part[3]));
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = w;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int i = 0; i < kLongBlock / kWave; i++) total += lds[i];
  const float dot = (float)total;
  float* xr = dx + (int64_t)blockIdx.x * lddx;
#pragma unroll
  for (int k = 0; k < E; k++) {
    const int64_t c = (int64_t)k * kLongBlock + threadIdx.x;
    if (c < ncols) xr[c] = scale * (a[k] * (b[k] - dot));
  }
}

// Rows beyond 32768 columns, or a few long rows that would leave most compute units without a workgroup:
// the row in pieces of 8192 columns, a workgroup of 1024 threads each.  The first kernel leaves every piece's
// sum of dy y in binary64, the second adds the pieces of its row in a fixed order and writes its piece of dx.
constexpr int kSplitE = 8;
constexpr int64_t kSplitPiece = (int64_t)kLongBlock * kSplitE;

__global__ __launch_bounds__(kLongBlock) void softmax_bwd_split_dot(const float* __restrict__ y, int64_t ldy,
                                                                    const float* __restrict__ dy, int64_t lddy,
                                                                    int64_t ncols, uint32_t pieces,
                                                                    double* __restrict__ pdot) {
  __shared__ double lds[kLongBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const float* yr = y + (int64_t)row * ldy;
  const float* dr = dy + (int64_t)row * lddy;
  const int64_t c0 = (int64_t)piece * kSplitPiece + threadIdx.x;
  float a[kSplitE], b[kSplitE];
#pragma unroll
  for (int k = 0; k < kSplitE; k++) {
    const int64_t c = c0 + (int64_t)k * kLongBlock;
    a[k] = c < ncols ? yr[c] : 0.0f;
    b[k] = c < ncols ? dr[c] : 0.0f;
  }
  float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int k = 0; k < kSplitE; k++) part[k & 3] = __builtin_fmaf(b[k], a[k], part[k & 3]);
  const double w = wave_sum(((double)part[0] + (double)part[1]) + ((double)part[2] + (double)part[3]));
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = w;
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
    for (int i = 0; i < kLongBlock / kWave; i++) total += lds[i];
    pdot[blockIdx.x] = total;
  }
}

__global__ __launch_bounds__(kLongBlock) void softmax_bwd_split_apply(const float* __restrict__ y, int64_t ldy,
                                                                      const float* dy, int64_t lddy,  // dx may be dy
                                                                      float* dx, int64_t lddx, int64_t ncols,
                                                                      uint32_t pieces,
                                                                      const double* __restrict__ pdot, float scale) {
  __shared__ double lds[kLongBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  double s = 0.0;
  for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock) s += pdot[row * pieces + i];
  s = wave_sum(s);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = s;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int i = 0; i < kLongBlock / kWave; i++) total += lds[i];
  const float dot = (float)total;
  const float* yr = y + (int64_t)row * ldy;
  const float* dr = dy + (int64_t)row * lddy;
  float* xr = dx + (int64_t)row * lddx;
  const int64_t c0 = (int64_t)piece * kSplitPiece + threadIdx.x;
  float a[kSplitE], b[kSplitE];
#pragma unroll
  for (int k = 0; k < kSplitE; k++) {
    const int64_t c = c0 + (int64_t)k * kLongBlock;
    a[k] = c < ncols ? yr[c] : 0.0f;
    b[k] = c < ncols ? dr[c] : 0.0f;
  }
#pragma unroll
  for (int k = 0; k < kSplitE; k++) {
    const int64_t c = c0 + (int64_t)k * kLongBlock;
    if (c < ncols) xr[c] = scale * (a[k] * (b[k] - dot));
  }
}

template <bool VEC, bool NT>
static int launch_softmax_bwd(int nv, const float* y, int64_t ldy, const float* dy, int64_t lddy, float* dx,
                              int64_t lddx, int64_t nrows, int64_t ncols, int64_t causal_seq, float scale) {
  const uint32_t blocks = (uint32_t)ceil_div(nrows, kWavesPerBlock);
  hipStream_t st = rt().stream;
#define WF2_CASE(N)                                                                                            \
  case N:                                                                                                      \
    softmax_bwd_rows_wave<N, VEC, NT><<<blocks, kBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, nrows, ncols,      \
                                                                 causal_seq, scale);                           \
    break;
  switch (nv) {
    WF2_CASE(1)
    WF2_CASE(2)
    WF2_CASE(3)
    WF2_CASE(4)
    WF2_CASE(5)
    WF2_CASE(6)
    WF2_CASE(7)
    WF2_CASE(8)
    default: return fail(WF2HIP_EINVAL, "bad register tile");
  }
#undef WF2_CASE
  return after_launch("softmax_bwd_rows_wave");
}

// ---- LayerNorm ----------------------------------------------------------------------------------
// A wavefront walks rows wave, wave + W, wave + 2 W, ... (W = wavefronts of the grid, so that
// the grid reads a contiguous band of rows at a time), keeps gamma and its share of the two
// column sums in registers, and the four wavefronts of a workgroup fold their shares through
// LDS into one row of `partial` ([workgroup][2][ncols]: dgamma, then dbeta); two small kernels
// then add the workgroups' rows in binary64.  Row statistics as in the forward kernel: the
// mean from binary64 sums, deviations and squares in binary32 with four partial sums per lane.
template <int NV, bool VEC, bool NT>
__global__ __launch_bounds__(kBlock) void layernorm_bwd_rows(const float* __restrict__ x,
                                                             const float* __restrict__ gamma,
                                                             const float* dy, float eps,  // dx may be dy
                                                             float* dx, float* __restrict__ partial,
                                                             int64_t nrows, int64_t ncols) {
  __shared__ float fold[kWavesPerBlock][NV * kWave * 4];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t stride = (int64_t)gridDim.x * kWavesPerBlock;
  RowRegs<NV, VEC, false> g;
  g.load(gamma, ncols, lane, 0.0f);
  float dg[NV][4], db[NV][4];
#pragma unroll
  for (int i = 0; i < NV; i++)
#pragma unroll
    for (int c = 0; c < 4; c++) dg[i][c] = db[i][c] = 0.0f;
  const float inv_n = 1.0f / (float)ncols;
  // the loads of the wavefront's next row are issued before the arithmetic of this one
  int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  RowRegs<NV, VEC, NT> xr, dr, xn, dn;
  if (row < nrows) {
    xr.load(x + row * ncols, ncols, lane, 0.0f);
    dr.load(dy + row * ncols, ncols, lane, 0.0f);
  }
  for (; row < nrows; row += stride) {
    const int64_t next = row + stride;
    if (next < nrows) {  // uniform over the wavefront
      xn.load(x + next * ncols, ncols, lane, 0.0f);
      dn.load(dy + next * ncols, ncols, lane, 0.0f);
    }
    double sum = 0.0;
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) sum += (double)xr.v[i][c];
    const float mean = (float)(wave_sum(sum) / (double)ncols);
    float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const bool in = RowRegs<NV, VEC, NT>::col(i, c, lane) < ncols;
        const float d = in ? xr.v[i][c] - mean : 0.0f;
        xr.v[i][c] = d;
        sq[c] = __builtin_fmaf(d, d, sq[c]);
      }
    const double var = wave_sum(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3])) / (double)ncols;
    const float rstd = (float)(1.0 / __builtin_sqrt(var + (double)eps));
    // xh, dyh and the two row means
    float s1[2] = {0.0f, 0.0f}, s2[2] = {0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float xh = xr.v[i][c] * rstd;
        const float d = dr.v[i][c];
        xr.v[i][c] = xh;
        dg[i][c] = __builtin_fmaf(d, xh, dg[i][c]);
        db[i][c] += d;
        const float dyh = d * g.v[i][c];
        dr.v[i][c] = dyh;
        s1[c & 1] += dyh;
        s2[c & 1] = __builtin_fmaf(dyh, xh, s2[c & 1]);
      }
    const float m1 = (float)wave_sum((double)s1[0] + (double)s1[1]) * inv_n;
    const float m2 = (float)wave_sum((double)s2[0] + (double)s2[1]) * inv_n;
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) dr.v[i][c] = rstd * ((dr.v[i][c] - m1) - xr.v[i][c] * m2);
    dr.store(dx + row * ncols, ncols, lane);
    xr = xn;
    dr = dn;
  }
  // fold the four wavefronts' column sums, dgamma first, then dbeta through the same LDS
#pragma unroll
  for (int which = 0; which < 2; which++) {
    if (which == 1) __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int64_t cc = RowRegs<NV, VEC, NT>::col(i, c, lane);
        fold[wave][cc] = which == 0 ? dg[i][c] : db[i][c];
      }
    __syncthreads();
    float* out = partial + ((int64_t)blockIdx.x * 2 + which) * ncols;
    for (int64_t cc = threadIdx.x; cc < ncols; cc += kBlock)
      out[cc] = (fold[0][cc] + fold[1][cc]) + (fold[2][cc] + fold[3][cc]);
  }
}

// Very many rows of at most 64 columns: a wavefront per row leaves most lanes idle ((1677721, 10): 1.4 ms).
// A workgroup walks groups of 128 adjacent rows (64 beyond 32 columns): x and dy, one contiguous run each, are
// staged into LDS in storage order (odd pitch), thread r works through row r (the formulas of layernorm_bwd_rows:
// the mean from a binary64 sum, deviations and squares in binary32) and leaves xh in place of x and the row's
// rstd and two means beside it; threads 0 .. ncols - 1 then add their column's dy xh and dy over the group's rows
// into registers, and all threads write dx in storage order.  A workgroup's column sums go to its row of
// `partial`, folded like the other kernels'.
__global__ __launch_bounds__(kBlock) void layernorm_bwd_tiny(const float* __restrict__ x, const float* __restrict__ gamma,
                                                             const float* dy, float eps,  // dx may be dy
                                                             float* dx, float* __restrict__ partial, int64_t nrows,
                                                             int ncols, FastDiv by_c) {
  __shared__ float tx[kTinyFloats];
  __shared__ float td[kTinyFloats];
  __shared__ float row_rstd[128], row_m1[128], row_m2[128];
  // groups of 128 rows (64 beyond 32 columns) whatever the width
  const int pitch = ncols | 1, group = ncols <= 32 ? 128 : 64;
  const int64_t ngroups = (nrows + group - 1) / group;
  const float inv_n = 1.0f / (float)ncols;
  float dg = 0.0f, db = 0.0f;  // threads 0 .. ncols - 1: the column sums over this workgroup's rows
  constexpr int U = 4;
  for (int64_t grp = blockIdx.x; grp < ngroups; grp += gridDim.x) {
    const int64_t row0 = grp * group;
    const int rows_here = (int)(nrows - row0 < group ? nrows - row0 : group);
    const uint32_t cells = (uint32_t)rows_here * (uint32_t)ncols;
    const int64_t base = row0 * ncols;
    __syncthreads();  // the previous group has been written out
    for (uint32_t e0 = threadIdx.x; e0 < cells; e0 += kBlock * U) {
      float a[U], b[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const bool live = e0 + u * kBlock < cells;
        a[u] = live ? x[base + e0 + u * kBlock] : 0.0f;
        b[u] = live ? dy[base + e0 + u * kBlock] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < U; u++)
        if (e0 + u * kBlock < cells) {
          uint32_t col;
          const uint32_t row = fd_divmod(e0 + u * kBlock, by_c, &col);
          tx[row * pitch + col] = a[u];
          td[row * pitch + col] = b[u];
        }
    }
    __syncthreads();
    for (int mine = threadIdx.x; mine < rows_here; mine += kBlock) {
      float* xr = tx + mine * pitch;
      const float* dr = td + mine * pitch;
      double sum = 0.0;
      for (int j = 0; j < ncols; j++) sum += (double)xr[j];
      const float mean = (float)(sum / (double)ncols);
      float sq = 0.0f;
      for (int j = 0; j < ncols; j++) {
        const float d = xr[j] - mean;
        xr[j] = d;
        sq = __builtin_fmaf(d, d, sq);
      }
      const float rstd = (float)(1.0 / __builtin_sqrt((double)sq / (double)ncols + (double)eps));
      float s1 = 0.0f, s2 = 0.0f;
      for (int j = 0; j < ncols; j++) {
        const float xh = xr[j] * rstd;
        xr[j] = xh;
        const float dyh = dr[j] * gamma[j];
        s1 += dyh;
        s2 = __builtin_fmaf(dyh, xh, s2);
      }
      row_rstd[mine] = rstd;
      row_m1[mine] = s1 * inv_n;
      row_m2[mine] = s2 * inv_n;
    }
    __syncthreads();
    if ((int)threadIdx.x < ncols) {
      for (int r = 0; r < rows_here; r++) {
        const float d = td[r * pitch + threadIdx.x];
        dg = __builtin_fmaf(d, tx[r * pitch + threadIdx.x], dg);
        db += d;
      }
    }
    for (uint32_t e = threadIdx.x; e < cells; e += kBlock) {
      uint32_t col;
      const uint32_t row = fd_divmod(e, by_c, &col);
      const float dyh = td[row * pitch + col] * gamma[col];
      dx[base + e] = row_rstd[row] * ((dyh - row_m1[row]) - tx[row * pitch + col] * row_m2[row]);
    }
  }
  if ((int)threadIdx.x < ncols) {
    partial[((int64_t)blockIdx.x * 2 + 0) * ncols + threadIdx.x] = dg;
    partial[((int64_t)blockIdx.x * 2 + 1) * ncols + threadIdx.x] = db;
  }
}

// Rows of 2049 ... 8192 columns: a workgroup per row, thread t holding the NG 16-byte vectors
// (g 256 + t) 4 ... of x, dy and gamma and its share of the two column sums in registers; the
// row statistics meet in LDS (three exchanges per row).  Workgroup b walks rows b, b + B, ...
// and leaves its column sums in row b of `partial`, folded like the narrower kernel's.  Same
// formulas as above: the mean from binary64 sums, deviations and squares in binary32.
template <int NG, bool NT>
__global__ __launch_bounds__(kBlock) void layernorm_bwd_wide(const float* __restrict__ x,
                                                             const float* __restrict__ gamma,
                                                             const float* dy, float eps,  // dx may be dy
                                                             float* dx, float* __restrict__ partial,
                                                             int64_t nrows, int64_t ncols) {
  constexpr int kWaves = kBlock / kWave;
  __shared__ double red[2][kWaves];
  const int wave = threadIdx.x / kWave;
  // sum of v (and w) over the workgroup, in every thread; a fixed order
  auto all_sum2 = [&](double v, double w, double* out_w) -> double {
    v = wave_sum(v);
    w = wave_sum(w);
    __syncthreads();  // the previous exchange has been read
    if ((threadIdx.x & (kWave - 1)) == 0) {
      red[0][wave] = v;
      red[1][wave] = w;
    }
    __syncthreads();
    double tv = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    double tw = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
#pragma unroll
    for (int i = 4; i < kWaves; i += 4) {
      tv += (red[0][i] + red[0][i + 1]) + (red[0][i + 2] + red[0][i + 3]);
      tw += (red[1][i] + red[1][i + 1]) + (red[1][i + 2] + red[1][i + 3]);
    }
    *out_w = tw;
    return tv;
  };
  bool in[NG];
  f4 g[NG], dg[NG], db[NG];
#pragma unroll
  for (int i = 0; i < NG; i++) {
    const int64_t c = ((int64_t)i * kBlock + threadIdx.x) * 4;
    in[i] = c < ncols;  // ncols is a multiple of 4: a vector is wholly inside or outside
    g[i] = in[i] ? *reinterpret_cast<const f4*>(gamma + c) : f4{0.f, 0.f, 0.f, 0.f};
    dg[i] = db[i] = f4{0.f, 0.f, 0.f, 0.f};
  }
  const float inv_n = 1.0f / (float)ncols;
  for (int64_t row = blockIdx.x; row < nrows; row += gridDim.x) {
    f4 xr[NG], dr[NG];
#pragma unroll
    for (int i = 0; i < NG; i++) {
      const int64_t at = row * ncols + ((int64_t)i * kBlock + threadIdx.x) * 4;
      xr[i] = dr[i] = f4{0.f, 0.f, 0.f, 0.f};
      if (in[i]) {
        const f4* px = reinterpret_cast<const f4*>(x + at);
        const f4* pd = reinterpret_cast<const f4*>(dy + at);
        xr[i] = NT ? __builtin_nontemporal_load(px) : *px;
        dr[i] = NT ? __builtin_nontemporal_load(pd) : *pd;
      }
    }
    double sum = 0.0, unused;
#pragma unroll
    for (int i = 0; i < NG; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) sum += (double)xr[i][c];
    const float mean = (float)(all_sum2(sum, 0.0, &unused) / (double)ncols);
    float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < NG; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float d = in[i] ? xr[i][c] - mean : 0.0f;
        xr[i][c] = d;
        sq[c] = __builtin_fmaf(d, d, sq[c]);
      }
    const double var =
        all_sum2(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3]), 0.0, &unused) / (double)ncols;
    const float rstd = (float)(1.0 / __builtin_sqrt(var + (double)eps));
    float s1[2] = {0.0f, 0.0f}, s2[2] = {0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < NG; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float xh = xr[i][c] * rstd;
        const float d = dr[i][c];
        xr[i][c] = xh;
        dg[i][c] = __builtin_fmaf(d, xh, dg[i][c]);
        db[i][c] += d;
        const float dyh = d * g[i][c];
        dr[i][c] = dyh;
        s1[c & 1] += dyh;
        s2[c & 1] = __builtin_fmaf(dyh, xh, s2[c & 1]);
      }
    double t2;
    const double t1 = all_sum2((double)s1[0] + (double)s1[1], (double)s2[0] + (double)s2[1], &t2);
    const float m1 = (float)t1 * inv_n, m2 = (float)t2 * inv_n;
#pragma unroll
    for (int i = 0; i < NG; i++) {
      if (!in[i]) continue;
      f4 r;
#pragma unroll
      for (int c = 0; c < 4; c++) r[c] = rstd * ((dr[i][c] - m1) - xr[i][c] * m2);
      f4* q = reinterpret_cast<f4*>(dx + row * ncols + ((int64_t)i * kBlock + threadIdx.x) * 4);
      if (NT)
        __builtin_nontemporal_store(r, q);
      else
        *q = r;
    }
  }
  float* out = partial + (int64_t)blockIdx.x * 2 * ncols;
#pragma unroll
  for (int i = 0; i < NG; i++) {
    if (!in[i]) continue;
    const int64_t c = ((int64_t)i * kBlock + threadIdx.x) * 4;
    *reinterpret_cast<f4*>(out + c) = dg[i];
    *reinterpret_cast<f4*>(out + ncols + c) = db[i];
  }
}

// Rows of 8193 ... 16384 columns, 16-byte aligned, at least a row per compute unit: layernorm_bwd_wide's row
// per 1024-thread workgroup with the next row's loads issued before the current row is reduced.  One such
// workgroup fills a compute unit, and its sixteen wavefronts move through a row in step (load, three exchanges,
// store), so without the second set of registers nothing is in flight while a row is reduced.  The registers
// come from the two column sums, which live in LDS instead (2 x 16384 floats, each element read and written by
// the one thread that owns the column).  Same formulas, same order of accumulation, same layout of `partial`.
constexpr int kLongNG = 4;  // vectors per thread of the kLongBlock = 1024 threads
constexpr int kLongCols = kLongBlock * kLongNG * 4;
constexpr size_t kLongLdsBytes = 2 * (size_t)kLongCols * sizeof(float) + 4 * (kLongBlock / kWave) * sizeof(double);

template <bool NT>
__global__ __launch_bounds__(kLongBlock) void layernorm_bwd_long(const float* __restrict__ x,
                                                                 const float* __restrict__ gamma,
                                                                 const float* dy, float eps,  // dx may be dy
                                                                 float* dx, float* __restrict__ partial,
                                                                 uint32_t nrows, int64_t ncols) {  // rows are counted in 32 bits: the SALU compares no wider
  constexpr int kWaves = kLongBlock / kWave, NG = kLongNG;
  extern __shared__ double long_lds[];
  double* red = long_lds;                                          // two buffers of [2][kWaves], used in turn
  f4* acc = reinterpret_cast<f4*>(long_lds + 4 * kWaves);         // [2][NG][kLongBlock]: dgamma, dbeta
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  int turn = 0;
  // Sums of v and w over the workgroup, in every thread, in a fixed order.  The barrier waits for this
  // wavefront's LDS traffic only (__syncthreads would also wait for the loads of the next row, which is what
  // they are issued early to avoid); two buffers in turn, so a wavefront that runs ahead into the next exchange
  // writes where nobody still reads (it has passed this barrier, so everyone has finished the exchange before).
  // Lane l reads the partial of wavefront l mod 16 and four butterfly steps leave the total in every lane.
  auto all_sum2 = [&](double v, double w, double* out_w) -> double {
    static_assert(kWaves == 16, "the butterfly below folds sixteen partials");
    v = wave_sum(v);
    w = wave_sum(w);
    double* buf = red + turn * 2 * kWaves;
    turn ^= 1;
    if (lane == 0) {
      buf[wave] = v;
      buf[kWaves + wave] = w;
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    double tv = buf[lane & (kWaves - 1)], tw = buf[kWaves + (lane & (kWaves - 1))];
#pragma unroll
    for (int o = kWaves / 2; o > 0; o >>= 1) {
      tv += __shfl_xor(tv, o);
      tw += __shfl_xor(tw, o);
    }
    *out_w = tw;
    return tv;
  };
  auto all_sum = [&](double v) -> double {
    v = wave_sum(v);
    double* buf = red + turn * 2 * kWaves;
    turn ^= 1;
    if (lane == 0) buf[wave] = v;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    double tv = buf[lane & (kWaves - 1)];
#pragma unroll
    for (int o = kWaves / 2; o > 0; o >>= 1) tv += __shfl_xor(tv, o);
    return tv;
  };
  bool in[NG];
  f4 g[NG];
#pragma unroll
  for (int i = 0; i < NG; i++) {
    const int64_t c = ((int64_t)i * kLongBlock + threadIdx.x) * 4;
    in[i] = c < ncols;  // ncols is a multiple of 4: a vector is wholly inside or outside
    g[i] = in[i] ? *reinterpret_cast<const f4*>(gamma + c) : f4{0.f, 0.f, 0.f, 0.f};
    acc[i * kLongBlock + threadIdx.x] = f4{0.f, 0.f, 0.f, 0.f};
    acc[(NG + i) * kLongBlock + threadIdx.x] = f4{0.f, 0.f, 0.f, 0.f};
  }
  const float inv_n = 1.0f / (float)ncols;
  // A row of x, dy or dx is a buffer of ncols floats: loads take a scalar descriptor, one 32-bit lane offset and
  // a scalar offset per vector (no 64-bit address per load held in registers), a lane past the end of the row
  // reads zeros and its store is dropped.  No branch around a load, so the loads are straight-line code and
  // the wait for this row's registers can leave the next row's loads in flight.
  constexpr int kRawBuffer = 0x00020000;  // dword 3 of a raw buffer descriptor: 32-bit data, no swizzle, no stride
  constexpr int kAux = NT ? 2 : 0;        // the nt bit
  const uint32_t lane_off = threadIdx.x * 16;
  auto row_of = [&](const float* base, uint32_t row) {  // a row past the last one: an empty buffer
    const bool there = row < nrows;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base + (int64_t)(there ? row : 0u) * ncols), 0,
                                             there ? (int)(ncols * 4) : 0, kRawBuffer);
  };
  // (issued for the row after the last one too, where it reads nothing: with the same instructions on every
  // path the compiler's wait before a row's first use counts exactly the loads issued after it)
  auto load = [&](f4 (&xr)[NG], f4 (&dr)[NG], uint32_t row) {
    const __amdgpu_buffer_rsrc_t rx = row_of(x, row), rd = row_of(dy, row);
#pragma unroll
    for (int i = 0; i < NG; i++) {
      xr[i] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(rx, lane_off, i * kLongBlock * 16, kAux));
      dr[i] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(rd, lane_off, i * kLongBlock * 16, kAux));
    }
  };
  auto reduce_row = [&](f4 (&xr)[NG], f4 (&dr)[NG], uint32_t row) {
    double sum = 0.0;
#pragma unroll
    for (int i = 0; i < NG; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) sum += (double)xr[i][c];
    const float mean = (float)(all_sum(sum) / (double)ncols);
    float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < NG; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float d = in[i] ? xr[i][c] - mean : 0.0f;
        xr[i][c] = d;
        sq[c] = __builtin_fmaf(d, d, sq[c]);
      }
    const double var = all_sum(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3])) / (double)ncols;
    const float rstd = (float)(1.0 / __builtin_sqrt(var + (double)eps));
    float s1[2] = {0.0f, 0.0f}, s2[2] = {0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < NG; i++) {
      f4 dg = acc[i * kLongBlock + threadIdx.x], db = acc[(NG + i) * kLongBlock + threadIdx.x];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float xh = xr[i][c] * rstd;
        const float d = dr[i][c];
        xr[i][c] = xh;
        dg[c] = __builtin_fmaf(d, xh, dg[c]);
        db[c] += d;
        const float dyh = d * g[i][c];
        dr[i][c] = dyh;
        s1[c & 1] += dyh;
        s2[c & 1] = __builtin_fmaf(dyh, xh, s2[c & 1]);
      }
      acc[i * kLongBlock + threadIdx.x] = dg;
      acc[(NG + i) * kLongBlock + threadIdx.x] = db;
    }
    double t2;
    const double t1 = all_sum2((double)s1[0] + (double)s1[1], (double)s2[0] + (double)s2[1], &t2);
    const float m1 = (float)t1 * inv_n, m2 = (float)t2 * inv_n;
#pragma unroll
    for (int i = 0; i < NG; i++) {
      f4 r;
#pragma unroll
      for (int c = 0; c < 4; c++) r[c] = rstd * ((dr[i][c] - m1) - xr[i][c] * m2);
      if (in[i]) {
        f4* q = reinterpret_cast<f4*>(dx + (int64_t)row * ncols + ((int64_t)i * kLongBlock + threadIdx.x) * 4);
        if (NT)
          __builtin_nontemporal_store(r, q);
        else
          *q = r;
      }
    }
  };
  const uint32_t step = gridDim.x;  // rows + step stays below 2^32: the host keeps rows below 2^31
  f4 xa[NG], da[NG], xb[NG], db_[NG];
  uint32_t row = blockIdx.x;
  load(xa, da, row);
  while (row < nrows) {
    load(xb, db_, row + step);
    reduce_row(xa, da, row);
    row += step;
    if (row >= nrows) break;
    load(xa, da, row + step);
    reduce_row(xb, db_, row);
    row += step;
  }
  float* out = partial + (int64_t)blockIdx.x * 2 * ncols;
#pragma unroll
  for (int i = 0; i < NG; i++) {
    if (!in[i]) continue;
    const int64_t c = ((int64_t)i * kLongBlock + threadIdx.x) * 4;
    *reinterpret_cast<f4*>(out + c) = acc[i * kLongBlock + threadIdx.x];
    *reinterpret_cast<f4*>(out + ncols + c) = acc[(NG + i) * kLongBlock + threadIdx.x];
  }
}

// Rows beyond 8192 columns, and rows beyond 2048 that cannot be read with 16-byte loads: the row in
// pieces of 16384 columns.  layernorm_bwd_piece_sums reads x, dy and gamma once and leaves, per piece,
// S_p = sum x, Q_p = sum (x - a_p)^2, D_p = sum gamma dy and C_p = sum gamma dy (x - a_p) about the
// piece's own a_p = (float)(S_p / n_p); the row's sums follow from them without a pass that knows the
// mean: sum gamma dy (x - mean) = sum_p [C_p + (a_p - mean) D_p].  layernorm_bwd_piece_apply folds them
// per row and writes dx, 512 threads on a quarter of a piece each.  Its workgroup (quarter, group) walks
// rows group, group + G, ... and leaves its column sums in row `group` of `partial`, folded like the narrower kernels' (with one group they are
// dgamma and dbeta themselves).  The formulas of layernorm_bwd_rows.
template <bool VEC>
__global__ __launch_bounds__(kPieceBlock) void layernorm_bwd_piece_sums(const float* __restrict__ x,
                                                                       const float* __restrict__ gamma,
                                                                       const float* __restrict__ dy, int64_t ncols,
                                                                       uint32_t pieces, double* __restrict__ psum,
                                                                       double* __restrict__ pdev,
                                                                       double* __restrict__ pd, double* __restrict__ pc) {
  __shared__ double lds[2 * kPieceBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const int64_t c0 = (int64_t)piece * kPieceCols;
  const int64_t left = ncols - c0;
  const int64_t n = left < kPieceCols ? left : kPieceCols;
  PieceRegs<VEC> xr, dr, g;
  xr.load(x + (int64_t)row * ncols + c0, left, 0.0f);
  dr.load(dy + (int64_t)row * ncols + c0, left, 0.0f);
  g.load(gamma + c0, left, 0.0f);
  double sum = 0.0;
  float s1[2] = {0.0f, 0.0f};
#pragma unroll
  for (int k = 0; k < kPieceE; k++) {
    sum += (double)xr.v[k];
    dr.v[k] *= g.v[k];
    s1[k & 1] += dr.v[k];
  }
  double d_total;
  const double total = piece_sum2(sum, (double)s1[0] + (double)s1[1], lds, &d_total);
  const float a = (float)(total / (double)n);
  float sq[2] = {0.0f, 0.0f}, s2[2] = {0.0f, 0.0f};
#pragma unroll
  for (int k = 0; k < kPieceE; k++) {
    const float d = PieceRegs<VEC>::col(k) < left ? xr.v[k] - a : 0.0f;
    sq[k & 1] = __builtin_fmaf(d, d, sq[k & 1]);
    s2[k & 1] = __builtin_fmaf(dr.v[k], d, s2[k & 1]);
  }
  double c_total;
  const double dev = piece_sum2((double)sq[0] + (double)sq[1], (double)s2[0] + (double)s2[1], lds, &c_total);
  if (threadIdx.x == 0) {
    psum[blockIdx.x] = total;
    pdev[blockIdx.x] = dev;
    pd[blockIdx.x] = d_total;
    pc[blockIdx.x] = c_total;
  }
}

// five registers per element: 512 threads on 4096 columns, so that two workgroups per compute unit
// cover each other's exchanges
constexpr int kApplyBlock = 512;
constexpr int kApplyE = 8;
constexpr int64_t kApplyCols = (int64_t)kApplyBlock * kApplyE;

template <bool VEC>
__global__ __launch_bounds__(kApplyBlock) void layernorm_bwd_piece_apply(const float* __restrict__ x,
                                                                        const float* __restrict__ gamma,
                                                                        const float* dy,  // dx may be dy
                                                                        float eps, float* dx, float* __restrict__ out_g,
                                                                        float* __restrict__ out_b, int64_t nrows,
                                                                        int64_t ncols, uint32_t pieces,
                                                                        const double* __restrict__ psum,
                                                                        const double* __restrict__ pdev,
                                                                        const double* __restrict__ pd,
                                                                        const double* __restrict__ pc) {
  __shared__ double lds[2 * kApplyBlock / kWave];
  const uint32_t piece = blockIdx.x;
  const int64_t c0 = (int64_t)piece * kApplyCols;
  const int64_t left = ncols - c0;
  typedef PieceRegs<VEC, kApplyBlock, kApplyE> Regs;
  Regs g, dg, db;
  g.load(gamma + c0, left, 0.0f);
#pragma unroll
  for (int k = 0; k < kApplyE; k++) dg.v[k] = db.v[k] = 0.0f;
  for (int64_t row = blockIdx.y; row < nrows; row += gridDim.y) {
    Regs xr, dr;
    xr.load(x + row * ncols + c0, left, 0.0f);
    dr.load(dy + row * ncols + c0, left, 0.0f);
    const double* rs = psum + row * pieces;
    const double* rq = pdev + row * pieces;
    const double* rd = pd + row * pieces;
    const double* rc = pc + row * pieces;
    double s = 0.0, d_sum = 0.0;
    for (uint32_t i = threadIdx.x; i < pieces; i += kApplyBlock) {
      s += rs[i];
      d_sum += rd[i];
    }
    double t1;
    const double mean = piece_sum2<kApplyBlock>(s, d_sum, lds, &t1) / (double)ncols;
    double q = 0.0, c_sum = 0.0;
    for (uint32_t i = threadIdx.x; i < pieces; i += kApplyBlock) {
      const int64_t l = ncols - (int64_t)i * kPieceCols;
      const double n = (double)(l < kPieceCols ? l : kPieceCols);
      const double mu = rs[i] / n;
      const double a = (double)(float)mu;
      q += rq[i] + n * ((mu - mean) * (mu - mean) - (mu - a) * (mu - a));
      c_sum += rc[i] + (a - mean) * rd[i];
    }
    double t2;
    const double var = piece_sum2<kApplyBlock>(q, c_sum, lds, &t2) / (double)ncols;
    const float meanf = (float)mean;
    const double rstd64 = 1.0 / __builtin_sqrt((var > 0.0 ? var : 0.0) + (double)eps);
    const float rstd = (float)rstd64;
    const float m1 = (float)(t1 / (double)ncols), m2 = (float)(t2 * rstd64 / (double)ncols);
#pragma unroll
    for (int k = 0; k < kApplyE; k++) {
      const float xh = Regs::col(k) < left ? (xr.v[k] - meanf) * rstd : 0.0f;
      const float d = dr.v[k];
      dg.v[k] = __builtin_fmaf(d, xh, dg.v[k]);
      db.v[k] += d;
      xr.v[k] = rstd * ((d * g.v[k] - m1) - xh * m2);
    }
    xr.store(dx + row * ncols + c0, left);
  }
  dg.store(out_g + (int64_t)blockIdx.y * 2 * ncols + c0, left);
  db.store(out_b + (int64_t)blockIdx.y * 2 * ncols + c0, left);
}

// Column sums of the workgroups' rows in two small steps, so that the first has enough
// workgroups to pull the few megabytes of `partial` at speed: the rows are cut into kFoldGroups
// groups; workgroup (x, g) adds the rows of group g for 64 of the 2 ncols columns (its four
// wavefronts take every fourth row, eight loads in flight each) into level2[g][.] in binary64;
// the second step adds the kFoldGroups rows of level2 and rounds once.
constexpr int kFoldGroups = 16;
__global__ __launch_bounds__(kBlock) void layernorm_bwd_fold1(const float* __restrict__ partial, int64_t nparts,
                                                              int64_t width, double* __restrict__ level2) {
  __shared__ double lds[kWavesPerBlock][kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t col = (int64_t)blockIdx.x * kWave + lane;  // 0 .. width - 1, width = 2 ncols
  const int64_t per = ceil_div_dev(nparts, kFoldGroups);
  const int64_t first = (int64_t)blockIdx.y * per;
  const int64_t last = first + per < nparts ? first + per : nparts;
  double acc = 0.0;
  if (col < width) {
    int64_t w = first + wave;
    for (; w + 7 * kWavesPerBlock < last; w += 8 * kWavesPerBlock) {
      float t[8];
#pragma unroll
      for (int u = 0; u < 8; u++) t[u] = partial[(w + u * kWavesPerBlock) * width + col];
#pragma unroll
      for (int u = 0; u < 8; u++) acc += (double)t[u];
    }
    for (; w < last; w += kWavesPerBlock) acc += (double)partial[w * width + col];
  }
  lds[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && col < width)
    level2[(int64_t)blockIdx.y * width + col] = (lds[0][lane] + lds[1][lane]) + (lds[2][lane] + lds[3][lane]);
}

// `groups` rows (at most kFoldGroups) of 2 ncols sums each: binary64 ones from the first step, or
// the kernels' own binary32 rows when there are few enough of them to skip that step.
template <typename T>
__global__ __launch_bounds__(kWave) void layernorm_bwd_fold2(const T* __restrict__ level2, int groups, int64_t ncols,
                                                             float* __restrict__ dgamma, float* __restrict__ dbeta) {
  const int64_t col = (int64_t)blockIdx.x * kWave + threadIdx.x;
  if (col >= 2 * ncols) return;
  double t[kFoldGroups];
#pragma unroll
  for (int g = 0; g < kFoldGroups; g++) t[g] = g < groups ? (double)level2[(int64_t)g * 2 * ncols + col] : 0.0;
  double acc = 0.0;
#pragma unroll
  for (int g = 0; g < kFoldGroups; g++) acc += t[g];
  if (col < ncols)
    dgamma[col] = (float)acc;
  else
    dbeta[col - ncols] = (float)acc;
}

template <bool VEC, bool NT>
static int launch_layernorm_bwd(int nv, uint32_t blocks, const float* x, const float* gamma, const float* dy,
                                float eps, float* dx, float* partial, int64_t nrows, int64_t ncols) {
  hipStream_t st = rt().stream;
#define WF2_CASE(N)                                                                                              \
  case N:                                                                                                        \
    layernorm_bwd_rows<N, VEC, NT><<<blocks, kBlock, 0, st>>>(x, gamma, dy, eps, dx, partial, nrows, ncols);      \
    break;
  switch (nv) {
    WF2_CASE(1)
    WF2_CASE(2)
    WF2_CASE(3)
    WF2_CASE(4)
    WF2_CASE(5)
    WF2_CASE(6)
    WF2_CASE(7)
    WF2_CASE(8)
    default: return fail(WF2HIP_EUNSUPPORTED, "LayerNorm backward: rows longer than 2048 are not built");
  }
#undef WF2_CASE
  return after_launch("layernorm_bwd_rows");
}

// ---- softmax cross entropy ----------------------------------------------------------------------
// sce-diff-static of Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:82-88, 103-110): the
// SubNode, MulNode and DivNode of dx = (dy (z - labels)) / batch in one pass, every operation
// rounded to binary32 as those nodes round them.  BCAST: dy is one number (the gradient that a
// !sum or !mean of the loss hands down through its broadcasting view).  Four 16-byte vectors per
// thread and stream, all loads issued before the arithmetic.
__device__ __forceinline__ float xent_grad(float dy, float z, float label, float batch) {
  return (dy * (z - label)) / batch;
}

template <bool VEC, bool NT, bool BCAST, bool FULL = false>
__global__ __launch_bounds__(kBlock) void xent_bwd_kernel(const float* dy, const float* z,  // dx may be dy or z
                                                          const float* __restrict__ labels, float* dx, size_t n,
                                                          float batch) {
  const float d0 = BCAST ? dy[0] : 0.0f;
  if (VEC) {
    constexpr int U = 4;
    const size_t nvec = n / 4;
    const size_t base = ((size_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * kWave * U + (threadIdx.x & (kWave - 1));
    f4 dv[U], zv[U], tv[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        if (!BCAST) dv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<const f4*>(dy) + i) : reinterpret_cast<const f4*>(dy)[i];
        zv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<const f4*>(z) + i) : reinterpret_cast<const f4*>(z)[i];
        tv[u] = NT ? __builtin_nontemporal_load(reinterpret_cast<const f4*>(labels) + i) : reinterpret_cast<const f4*>(labels)[i];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        f4 r;
#pragma unroll
        for (int c = 0; c < 4; c++) r[c] = xent_grad(BCAST ? d0 : dv[u][c], zv[u][c], tv[u][c], batch);
        if (NT)
          __builtin_nontemporal_store(r, reinterpret_cast<f4*>(dx) + i);
        else
          reinterpret_cast<f4*>(dx)[i] = r;
      }
    }
    if (!FULL && blockIdx.x == 0 && threadIdx.x < (n & 3)) {
      const size_t j = nvec * 4 + threadIdx.x;
      dx[j] = xent_grad(BCAST ? d0 : dy[j], z[j], labels[j], batch);
    }
  } else {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) dx[i] = xent_grad(BCAST ? d0 : dy[i], z[i], labels[i], batch);
  }
}

template <bool BCAST>
static int launch_xent_bwd(const float* dy, const float* z, const float* labels, float* dx, int64_t n, float batch) {
  const bool vec = aligned16(z) && aligned16(labels) && aligned16(dx) && (BCAST || aligned16(dy));
  const int64_t nvec = n / 4 > 0 ? n / 4 : 1;
  const int64_t blocks = vec ? ceil_div(nvec, (int64_t)kBlock * 4) : ceil_div(n, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many elements for one launch");
  hipStream_t st = rt().stream;
  const bool streaming = n * (BCAST ? 12 : 16) >= ((int64_t)192 << 20);
  // every workgroup full: no bounds tests, so a thread's loads are all issued before its first wait
  if (vec && streaming && n % (4 * kBlock * 4) == 0)
    xent_bwd_kernel<true, true, BCAST, true><<<(uint32_t)blocks, kBlock, 0, st>>>(dy, z, labels, dx, (size_t)n, batch);
  else if (vec && streaming)
    xent_bwd_kernel<true, true, BCAST><<<(uint32_t)blocks, kBlock, 0, st>>>(dy, z, labels, dx, (size_t)n, batch);
  else if (vec)
    xent_bwd_kernel<true, false, BCAST><<<(uint32_t)blocks, kBlock, 0, st>>>(dy, z, labels, dx, (size_t)n, batch);
  else
    xent_bwd_kernel<false, false, BCAST><<<(uint32_t)blocks, kBlock, 0, st>>>(dy, z, labels, dx, (size_t)n, batch);
  return after_launch("xent_bwd_kernel");
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_softmax_backward_rows_f32(long rows, long cols, const float* y, long ldy, const float* dy,
                                             long lddy, float* dx, long lddx, float scale, long causal_seq) {
  WF2_TRY(require_init());
  if (rows < 0 || cols < 0 || causal_seq < 0) return fail(WF2HIP_EINVAL, "negative extent");
  if (rows == 0 || cols == 0) return 0;
  if (!y || !dy || !dx) return fail(WF2HIP_EINVAL, "null pointer");
  if (ldy < cols || lddy < cols || lddx < cols) return fail(WF2HIP_EINVAL, "row pitch smaller than the row");
  if (causal_seq > 0 && causal_seq != cols)
    return fail(WF2HIP_EINVAL, "causal softmax backward takes square (seq, seq) matrices: cols %ld, seq %ld", cols,
                causal_seq);
  if (rows >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows");
  // dx may be dy (in place, row by row) but must not overlap anything else
  const float* ylo = y;
  const float* yhi = y + (rows - 1) * (int64_t)ldy + cols;
  const float* dlo = dy;
  const float* dhi = dy + (rows - 1) * (int64_t)lddy + cols;
  const float* xlo = dx;
  const float* xhi = dx + (rows - 1) * (int64_t)lddx + cols;
  if (xlo < yhi && ylo < xhi) return fail(WF2HIP_EOVERLAP, "softmax backward: dx overlaps y");
  if (xlo < dhi && dlo < xhi && !(dx == dy && lddx == lddy))
    return fail(WF2HIP_EOVERLAP, "softmax backward: dx overlaps dy without being dy");
  if (cols <= kTinyCols && causal_seq == 0 && rows >= 16384 && ldy == cols && lddy == cols && lddx == cols) {
    const uint32_t groups = (uint32_t)ceil_div((int64_t)rows, tiny_bwd_rows_per_group((int)cols));
    if (aligned16(y) && aligned16(dy) && aligned16(dx))
      softmax_bwd_rows_tiny<true><<<groups, kBlock, 0, rt().stream>>>(y, dy, dx, rows, (int)cols, scale,
                                                                        make_fastdiv((uint32_t)cols));
    else
      softmax_bwd_rows_tiny<false><<<groups, kBlock, 0, rt().stream>>>(y, dy, dx, rows, (int)cols, scale,
                                                                         make_fastdiv((uint32_t)cols));
    return after_launch("softmax_bwd_rows_tiny");
  }
  int nv = pick_nv(cols);
  if (nv == 0 || nv > 8) {
    hipStream_t st = rt().stream;
    const int64_t pieces = ceil_div((int64_t)cols, kSplitPiece);
    if (causal_seq == 0 && (cols > 32 * kLongBlock || (pieces >= 2 && rows < rt().num_cus)) &&
        rows * pieces < ((int64_t)1 << 31)) {
      void* pdot = nullptr;
      int held_up = 0;
      if (!scratch_block(&pdot, (size_t)(rows * pieces) * sizeof(double), &held_up)) {
        if (held_up) return held_up;
      } else {
        const uint32_t grid = (uint32_t)(rows * pieces);
        softmax_bwd_split_dot<<<grid, kLongBlock, 0, st>>>(y, ldy, dy, lddy, cols, (uint32_t)pieces,
                                                           static_cast<double*>(pdot));
        int rc = after_launch("softmax_bwd_split_dot");
        if (rc == 0) {
          softmax_bwd_split_apply<<<grid, kLongBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, cols, (uint32_t)pieces,
                                                               static_cast<const double*>(pdot), scale);
          rc = after_launch("softmax_bwd_split_apply");
        }
        (void)wf2hip_free(pdot);  // stream order keeps it alive for the launches above
        return rc;
      }
    }
    if (causal_seq == 0 && cols <= 32 * kLongBlock) {  // beyond: y and dy of a row exceed the registers of 1024 threads
      if (cols <= 4 * kLongBlock)
        softmax_bwd_rows_long<4><<<(uint32_t)rows, kLongBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, cols, scale);
      else if (cols <= 8 * kLongBlock)
        softmax_bwd_rows_long<8><<<(uint32_t)rows, kLongBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, cols, scale);
      else if (cols <= 16 * kLongBlock)
        softmax_bwd_rows_long<16><<<(uint32_t)rows, kLongBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, cols, scale);
      else
        softmax_bwd_rows_long<32><<<(uint32_t)rows, kLongBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, cols, scale);
      return after_launch("softmax_bwd_rows_long");
    }
    softmax_bwd_rows_block<<<(uint32_t)rows, kBlock, 0, st>>>(y, ldy, dy, lddy, dx, lddx, cols, causal_seq, scale);
    return after_launch("softmax_bwd_rows_block");
  }
  const bool vec = aligned16(y) && aligned16(dy) && aligned16(dx) && ldy % 4 == 0 && lddy % 4 == 0 && lddx % 4 == 0;
  const bool streaming = (int64_t)rows * cols * 12 >= ((int64_t)192 << 20);
  if (vec && streaming) return launch_softmax_bwd<true, true>(nv, y, ldy, dy, lddy, dx, lddx, rows, cols, causal_seq, scale);
  if (vec) return launch_softmax_bwd<true, false>(nv, y, ldy, dy, lddy, dx, lddx, rows, cols, causal_seq, scale);
  return launch_softmax_bwd<false, false>(nv, y, ldy, dy, lddy, dx, lddx, rows, cols, causal_seq, scale);
}

WF2_API int wf2hip_layernorm_backward_f32(long rows, long cols, const float* x, const float* gamma, const float* dy,
                                          float eps, float* dx, float* dgamma, float* dbeta) {
  WF2_TRY(require_init());
  if (rows < 0 || cols < 0) return fail(WF2HIP_EINVAL, "negative extent");
  if (cols == 0) return 0;
  if (!gamma || !dgamma || !dbeta) return fail(WF2HIP_EINVAL, "null pointer");
  if (rows == 0) {  // empty sums
    WF2_TRY(wf2hip_fill_f32(dgamma, (size_t)cols, 0.0f));
    return wf2hip_fill_f32(dbeta, (size_t)cols, 0.0f);
  }
  if (!x || !dy || !dx) return fail(WF2HIP_EINVAL, "null pointer");
  int nv = pick_nv(cols);
  // seven groups only where they fill the tile: rows of 1537 ... 1791 columns run at 2.1 TB/s on the
  // guarded seven-group tile and at 3.9 TB/s on the guarded eight-group one ((32768, 1600))
  if (nv == 7 && cols != 7 * kWave * 4) nv = 8;
  const bool wide = nv == 0 || nv > 8;  // more than 2048 columns: a workgroup per row
  const bool vec = aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(gamma) && cols % 4 == 0;
  const bool long_rows = wide && vec && cols > 8192 && cols <= 16384 && rows >= rt().num_cus && rows < ((int64_t)1 << 31);  // 1024 threads per row
  const bool in_pieces = wide && (cols > 8192 || !vec) && !long_rows;
  const int64_t total = (int64_t)rows * cols;
  if ((x < dx + total && dx < x + total) || (dgamma < dbeta + cols && dbeta < dgamma + cols))
    return fail(WF2HIP_EOVERLAP, "LayerNorm backward: dx overlaps x, or dgamma overlaps dbeta");
  if (dy < dx + total && dx < dy + total && dx != dy)
    return fail(WF2HIP_EOVERLAP, "LayerNorm backward: dx overlaps dy without being dy");
  // two workgroups per compute unit, at most one wavefront per row: (65536, 1024) runs at 74 % of
  // the HBM peak (both small folds included), 66 % with one workgroup per unit, 65 - 67 % with
  // three to eight (more rows of `partial` to write and fold)
  const bool tiny = cols <= kTinyCols && rows >= 16384;
  const int64_t pieces = ceil_div((int64_t)cols, kPieceCols);
  if (in_pieces && (rows * pieces >= ((int64_t)1 << 31) || pieces >= ((int64_t)1 << 31)))
    return fail(WF2HIP_EUNSUPPORTED, "too many row pieces for one launch");
  // in pieces: enough row groups for two workgroups of 512 threads per compute unit
  const int64_t quarters = ceil_div((int64_t)cols, kApplyCols);
  const int64_t blocks = in_pieces ? std::min<int64_t>({(int64_t)rows, ceil_div(2 * (int64_t)std::max(rt().num_cus, 1), quarters), 65535})
                         : long_rows ? std::min<int64_t>(rows, (int64_t)std::max(rt().num_cus, 1))
                         : wide  ? std::min<int64_t>(rows, 2 * (int64_t)std::max(rt().num_cus, 1))
                         : tiny ? std::min<int64_t>(ceil_div((int64_t)rows, (int64_t)(cols <= 32 ? 128 : 64)),
                                                    4 * (int64_t)std::max(rt().num_cus, 1))
                              : std::min<int64_t>(ceil_div(rows, kWavesPerBlock), 2 * (int64_t)std::max(rt().num_cus, 1));
  // few enough rows of column sums go to the last fold as they are; one row is the result itself
  const bool direct = in_pieces && blocks == 1;
  const bool two_folds = blocks > kFoldGroups;
  const size_t partial_bytes = direct ? 0 : (size_t)blocks * 2 * cols * sizeof(float);
  const size_t level2_bytes = two_folds ? (size_t)kFoldGroups * 2 * cols * sizeof(double) : 0;
  void* partial = nullptr;
  if (!direct) WF2_TRY(wf2hip_malloc_uninitialized(&partial, partial_bytes + level2_bytes));  // partial_bytes is a multiple of 8
  double* level2 = reinterpret_cast<double*>(static_cast<char*>(partial) + partial_bytes);
  const bool streaming = total * 12 >= ((int64_t)192 << 20);
  int rc;
  if (in_pieces) {
    hipStream_t st = rt().stream;
    void* stats = nullptr;  // four binary64 values per (row, piece)
    const size_t np = (size_t)(rows * pieces);
    rc = wf2hip_malloc_uninitialized(&stats, np * 4 * sizeof(double));
    if (rc != 0) {
      if (partial) (void)wf2hip_free(partial);
      return rc;
    }
    double* psum = static_cast<double*>(stats);
    double *pdev = psum + np, *pd = psum + 2 * np, *pc = psum + 3 * np;
    float* out_g = direct ? dgamma : static_cast<float*>(partial);
    float* out_b = direct ? dbeta : static_cast<float*>(partial) + cols;
    const uint32_t grid = (uint32_t)np;
    const dim3 grid2((uint32_t)quarters, (uint32_t)blocks);
    if (vec)
      layernorm_bwd_piece_sums<true><<<grid, kPieceBlock, 0, st>>>(x, gamma, dy, cols, (uint32_t)pieces, psum, pdev, pd, pc);
    else
      layernorm_bwd_piece_sums<false><<<grid, kPieceBlock, 0, st>>>(x, gamma, dy, cols, (uint32_t)pieces, psum, pdev, pd, pc);
    rc = after_launch("layernorm_bwd_piece_sums");
    if (rc == 0) {
      if (vec)
        layernorm_bwd_piece_apply<true><<<grid2, kApplyBlock, 0, st>>>(x, gamma, dy, eps, dx, out_g, out_b, rows, cols,
                                                                      (uint32_t)pieces, psum, pdev, pd, pc);
      else
        layernorm_bwd_piece_apply<false><<<grid2, kApplyBlock, 0, st>>>(x, gamma, dy, eps, dx, out_g, out_b, rows, cols,
                                                                       (uint32_t)pieces, psum, pdev, pd, pc);
      rc = after_launch("layernorm_bwd_piece_apply");
    }
    (void)wf2hip_free(stats);  // stream order keeps it alive for the launches above
    if (direct) return rc;
  } else if (tiny) {
    layernorm_bwd_tiny<<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(x, gamma, dy, eps, dx, (float*)partial, rows, (int)cols,
                                                                     make_fastdiv((uint32_t)cols));
    rc = after_launch("layernorm_bwd_tiny");
  } else if (long_rows) {
    hipStream_t st = rt().stream;
    static bool configured = false;
    rc = 0;
    if (!configured) {
      rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&layernorm_bwd_long<true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLongLdsBytes),
                     "hipFuncSetAttribute(layernorm_bwd_long)");
      if (rc == 0)
        rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&layernorm_bwd_long<false>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLongLdsBytes),
                       "hipFuncSetAttribute(layernorm_bwd_long)");
      configured = rc == 0;
    }
    if (rc != 0) {
      (void)wf2hip_free(partial);
      return rc;
    }
    if (streaming)
      layernorm_bwd_long<true><<<(uint32_t)blocks, kLongBlock, kLongLdsBytes, st>>>(x, gamma, dy, eps, dx, (float*)partial, (uint32_t)rows, cols);
    else
      layernorm_bwd_long<false><<<(uint32_t)blocks, kLongBlock, kLongLdsBytes, st>>>(x, gamma, dy, eps, dx, (float*)partial, (uint32_t)rows, cols);
    rc = after_launch("layernorm_bwd_long");
  } else if (wide) {
    hipStream_t st = rt().stream;
    const int ng = (int)ceil_div(cols, (int64_t)kBlock * 4);
#define WF2_WIDE(NG_)                                                                                              \
  if (streaming)                                                                                                   \
    layernorm_bwd_wide<NG_, true><<<(uint32_t)blocks, kBlock, 0, st>>>(x, gamma, dy, eps, dx, (float*)partial, rows, cols); \
  else                                                                                                             \
    layernorm_bwd_wide<NG_, false><<<(uint32_t)blocks, kBlock, 0, st>>>(x, gamma, dy, eps, dx, (float*)partial, rows, cols);
    if (ng <= 3) {
      WF2_WIDE(3)
    } else if (ng <= 4) {
      WF2_WIDE(4)
    } else if (ng <= 6) {
      WF2_WIDE(6)
    } else {
      WF2_WIDE(8)
    }
#undef WF2_WIDE
    rc = after_launch("layernorm_bwd_wide");
  } else if (vec && streaming)
    rc = launch_layernorm_bwd<true, true>(nv, (uint32_t)blocks, x, gamma, dy, eps, dx, (float*)partial, rows, cols);
  else if (vec)
    rc = launch_layernorm_bwd<true, false>(nv, (uint32_t)blocks, x, gamma, dy, eps, dx, (float*)partial, rows, cols);
  else
    rc = launch_layernorm_bwd<false, false>(nv, (uint32_t)blocks, x, gamma, dy, eps, dx, (float*)partial, rows, cols);
  if (rc == 0 && two_folds) {
    const uint32_t strips = (uint32_t)ceil_div(2 * (int64_t)cols, kWave);
    layernorm_bwd_fold1<<<dim3(strips, kFoldGroups), kBlock, 0, rt().stream>>>((const float*)partial, blocks,
                                                                              2 * (int64_t)cols, level2);
    rc = after_launch("layernorm_bwd_fold1");
  }
  if (rc == 0) {
    const uint32_t grid = (uint32_t)ceil_div(2 * (int64_t)cols, kWave);
    if (two_folds)
      layernorm_bwd_fold2<double><<<grid, kWave, 0, rt().stream>>>(level2, kFoldGroups, cols, dgamma, dbeta);
    else
      layernorm_bwd_fold2<float><<<grid, kWave, 0, rt().stream>>>((const float*)partial, (int)blocks, cols, dgamma, dbeta);
    rc = after_launch("layernorm_bwd_fold2");
  }
  (void)wf2hip_free(partial);  // stream order keeps it alive for the launches above
  return rc;
}

WF2_API int wf2hip_softmax_cross_entropy_backward_f32(long n, const float* dy, int dy_is_scalar, const float* z,
                                                      const float* labels, float batch, float* dx) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  if (n == 0) return 0;
  if (!dy || !z || !labels || !dx) return fail(WF2HIP_EINVAL, "null pointer");
  // dx may be dy or z (element for element); any other overlap would race
  auto meets = [&](const float* a, int64_t na) { return a < dx + n && dx < a + na; };
  if (meets(labels, n)) return fail(WF2HIP_EOVERLAP, "softmax cross entropy backward: dx overlaps labels");
  if (meets(z, n) && dx != z) return fail(WF2HIP_EOVERLAP, "softmax cross entropy backward: dx overlaps z without being z");
  if (dy_is_scalar ? meets(dy, 1) : (meets(dy, n) && dx != dy))
    return fail(WF2HIP_EOVERLAP, "softmax cross entropy backward: dx overlaps dy without being dy");
  return dy_is_scalar ? launch_xent_bwd<true>(dy, z, labels, dx, n, batch)
                      : launch_xent_bwd<false>(dy, z, labels, dx, n, batch);
}
