// reduce.hip -- accumulation into stride-0 destinations (cl-waffe2's !sum /
// !mean), max/min, and the fused row kernels (softmax, causal softmax,
// LayerNorm).
//
// cl-waffe2 has no reduction node: (!sum x :axis k) zero-fills `out`, views it
// with (:broadcast n) on the reduced axes and runs AddNode into that view
// (source/base-impl/reduction.lisp:5-79), so the CPU kernel is called with
// incx == 0 and adds sequentially into one float (cl-waffe2-simd.c:159,
// 205-212).  On the GPU the same node becomes a parallel reduction:
// wavefront shuffles inside a 64-lane wave, LDS across the four waves of a
// workgroup, and a second tiny pass when a row has to be split over
// workgroups.  Partial sums are kept in binary64 (binary64 adds issue at the
// binary32 rate on CDNA) and rounded once, so the result is closer to the
// exact sum than the reference's own sequential binary32 order; reduce mode 1
// reproduces that order exactly for bit-parity checks.
//
// All kernels here are HBM-bound: 4 bytes read per element reduced, 8 bytes
// per element for softmax/LayerNorm (one read, one write).
#include <algorithm>

#include "wf2_common.h"
#include "wf2_fastdiv.h"
#include "wf2_math.h"
#include "wf2_view.h"
#include "wf2_rows.h"

namespace wf2 {

constexpr int kMaxOuter = WF2HIP_MAX_RANK - 1;

// What a reduction leaves in its destination.  Accumulating (AddNode into a
// stride-0 view): dst + total, rounded once.  Overwriting (the one-node form of
// !sum / !mean): total rounded to binary32, then divided by `divisor` in binary32
// -- the bits the reference's zero fill, AddNode and DivNode by the element
// count produce from a zero destination; the old content of dst is not read.
struct Commit {
  int32_t overwrite;
  float divisor;
  __device__ __forceinline__ void operator()(float* dst, double total) const {
    *dst = overwrite ? (float)total / divisor : (float)((double)*dst + total);
  }
};

// ---- row reduction: a[row] += sum_c b[row, c] ---------------------------------
struct RowRedParams {
  float* a;
  const float* b;
  int64_t n0;       // reduced (innermost, contiguous) extent
  uint32_t nrows;
  int32_t nouter;
  uint32_t oshape[kMaxOuter];  // kept axes, innermost of them first
  int64_t oa[kMaxOuter];
  int64_t ob[kMaxOuter];
  uint32_t splits;  // workgroups per row
  int64_t seg;      // elements per split (multiple of 4)
  double* partials; // nrows*splits, used when splits > 1
  Commit commit;
};

__device__ __forceinline__ void row_offsets(const RowRedParams& p, uint32_t row, int64_t* aoff,
                                            int64_t* boff) {
  int64_t ao = 0, bo = 0;
  uint32_t rem = row;
  for (int i = 0; i < p.nouter; i++) {
    uint32_t idx;
    if (i == p.nouter - 1) {
      idx = rem;
    } else {
      uint32_t q = rem / p.oshape[i];
      idx = rem - q * p.oshape[i];
      rem = q;
    }
    ao += (int64_t)idx * p.oa[i];
    bo += (int64_t)idx * p.ob[i];
  }
  *aoff = ao;
  *boff = bo;
}

// Sum of b[lo, hi) by `nthreads` cooperating threads; `t` is this thread's
// rank among them.  VEC == 4 needs b + lo 16-byte aligned.
template <int VEC, bool NT = false>
__device__ __forceinline__ double strided_sum(const float* __restrict__ b, int64_t lo, int64_t hi,
                                              int t, int nthreads) {
  double acc0 = 0.0, acc1 = 0.0;
  if constexpr (VEC == 4) {
    int64_t nvec = (hi - lo) / 4;
    const f4* bv = reinterpret_cast<const f4*>(b + lo);
    int64_t i = t;
    for (; i + nthreads < nvec; i += 2 * (int64_t)nthreads) {
      f4 v0 = NT ? __builtin_nontemporal_load(bv + i) : bv[i];
      f4 v1 = NT ? __builtin_nontemporal_load(bv + i + nthreads) : bv[i + nthreads];
      acc0 += ((double)v0.x + (double)v0.y) + ((double)v0.z + (double)v0.w);
      acc1 += ((double)v1.x + (double)v1.y) + ((double)v1.z + (double)v1.w);
    }
    if (i < nvec) {
      f4 v0 = NT ? __builtin_nontemporal_load(bv + i) : bv[i];
      acc0 += ((double)v0.x + (double)v0.y) + ((double)v0.z + (double)v0.w);
    }
    for (int64_t c = lo + nvec * 4 + t; c < hi; c += nthreads) acc1 += (double)b[c];
  } else {
    for (int64_t c = lo + t; c < hi; c += nthreads) acc0 += (double)b[c];
  }
  return acc0 + acc1;
}

// One workgroup per (row, split).
template <int VEC, bool NT = false>
__global__ __launch_bounds__(kBlock) void reduce_rows_block(RowRedParams p) {
  __shared__ double lds[kWavesPerBlock];
  const uint32_t row = blockIdx.x / p.splits;
  const uint32_t split = blockIdx.x - row * p.splits;
  int64_t aoff, boff;
  row_offsets(p, row, &aoff, &boff);
  int64_t lo = (int64_t)split * p.seg;
  int64_t hi = lo + p.seg < p.n0 ? lo + p.seg : p.n0;
  double v = strided_sum<VEC, NT>(p.b + boff, lo, hi, threadIdx.x, kBlock);
  double total = block_sum(v, lds);
  if (threadIdx.x == 0) {
    if (p.splits == 1)
      p.commit(p.a + aoff, total);
    else
      p.partials[(int64_t)row * p.splits + split] = total;
  }
}

// Streaming form for footprints far beyond the Infinity Cache: 512 threads per
// (row, split), two unguarded non-temporal 16-byte loads per thread and batch
// (measured: 4-5 % more bandwidth than the 256-thread form above, which in turn
// beats one wavefront per row and 1024-thread workgroups).
constexpr int kStreamBlock = 512;
__global__ __launch_bounds__(kStreamBlock) void reduce_rows_stream(RowRedParams p) {
  __shared__ double lds[kStreamBlock / kWave];
  const uint32_t row = blockIdx.x / p.splits;
  const uint32_t split = blockIdx.x - row * p.splits;
  int64_t aoff, boff;
  row_offsets(p, row, &aoff, &boff);
  const int64_t lo = (int64_t)split * p.seg;
  const int64_t hi = lo + p.seg < p.n0 ? lo + p.seg : p.n0;
  const float* b = p.b + boff;
  const f4* bv = reinterpret_cast<const f4*>(b + lo);
  constexpr int64_t kBatch = 2 * kStreamBlock;  // vectors per batch
  const int64_t nfull = ((hi - lo) / 4) / kBatch * kBatch;
  double acc0 = 0.0, acc1 = 0.0;
  for (int64_t i = threadIdx.x; i < nfull; i += kBatch) {
    f4 v0 = __builtin_nontemporal_load(bv + i);
    f4 v1 = __builtin_nontemporal_load(bv + i + kStreamBlock);
    acc0 += ((double)v0.x + (double)v0.y) + ((double)v0.z + (double)v0.w);
    acc1 += ((double)v1.x + (double)v1.y) + ((double)v1.z + (double)v1.w);
  }
  double v = acc0 + acc1;
  if (lo + nfull * 4 < hi) v += strided_sum<4, true>(b, lo + nfull * 4, hi, threadIdx.x, kStreamBlock);
  v = wave_sum(v);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
#pragma unroll
    for (int i = 0; i < kStreamBlock / kWave; i++) total += lds[i];
    if (p.splits == 1)
      p.commit(p.a + aoff, total);
    else
      p.partials[(int64_t)row * p.splits + split] = total;
  }
}

// One wavefront per row, four rows per workgroup.
template <int VEC, bool NT = false>
__global__ __launch_bounds__(kBlock) void reduce_rows_wave(RowRedParams p) {
  const uint32_t row = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (row >= p.nrows) return;
  int64_t aoff, boff;
  row_offsets(p, row, &aoff, &boff);
  double v = strided_sum<VEC, NT>(p.b + boff, 0, p.n0, threadIdx.x & (kWave - 1), kWave);
  v = wave_sum(v);
  if ((threadIdx.x & (kWave - 1)) == 0) p.commit(p.a + aoff, v);
}

// Rows of at most 512 elements (vector loads): four rows per wavefront, their loads
// issued together -- a wavefront with one row of 256 has 1 KB in flight, which holds
// the row sums of (262144, 256) at 46 % of the HBM peak.
template <bool NT>
__global__ __launch_bounds__(kBlock) void reduce_rows_short(RowRedParams p) {
  constexpr int RW = 4;
  const int64_t row0 = ((int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * RW;
  if (row0 >= p.nrows) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t nvec = p.n0 / 4;  // <= 128
  f4 v[RW][2];
  int64_t aoff[RW], boff[RW];
#pragma unroll
  for (int w = 0; w < RW; w++) {
    const int64_t row = row0 + w < p.nrows ? row0 + w : p.nrows - 1;
    row_offsets(p, (uint32_t)row, &aoff[w], &boff[w]);
    const f4* bv = reinterpret_cast<const f4*>(p.b + boff[w]);
#pragma unroll
    for (int k = 0; k < 2; k++) {
      const int64_t i = lane + k * kWave;
      v[w][k] = f4{0.f, 0.f, 0.f, 0.f};
      if (i < nvec) v[w][k] = NT ? __builtin_nontemporal_load(bv + i) : bv[i];
    }
  }
#pragma unroll
  for (int w = 0; w < RW; w++) {
    double acc = (((double)v[w][0].x + (double)v[w][0].y) + ((double)v[w][0].z + (double)v[w][0].w)) +
                 (((double)v[w][1].x + (double)v[w][1].y) + ((double)v[w][1].z + (double)v[w][1].w));
    for (int64_t c = nvec * 4 + lane; c < p.n0; c += kWave) acc += (double)p.b[boff[w] + c];
    acc = wave_sum(acc);
    if (lane == 0 && row0 + w < p.nrows) p.commit(p.a + aoff[w], acc);
  }
}

// Rows of at most 32 elements, adjacent in memory (AvgPool2D's !mean over windows of k-h k-w
// elements, source/nn/pool.lisp:95-105): a thread per row.  The workgroup's 256 rows are one
// contiguous run, read by consecutive lanes into LDS (rows padded to an odd pitch) and added
// from there in index order, in binary64; a wavefront per four rows left (6422528, 4) at 770 us.
__global__ __launch_bounds__(kBlock) void reduce_rows_tiny(RowRedParams p, FastDiv by_n) {
  extern __shared__ float tiny_tile[];
  const uint32_t n = (uint32_t)p.n0, pitch = n | 1u;
  const uint32_t row0 = blockIdx.x * kBlock;
  const uint32_t rows_here = p.nrows - row0 < (uint32_t)kBlock ? p.nrows - row0 : (uint32_t)kBlock;
  const uint32_t count = rows_here * n;
  const float* src = p.b + (int64_t)row0 * n;
  auto place = [&](uint32_t e) { const uint32_t r = fd_div(e, by_n); return r * pitch + (e - r * n); };
  if (((uintptr_t)src & 15u) == 0) {
    // the run in 16-byte vectors (a workgroup's run of 256 rows starts on a multiple of 16 bytes), four in
    // flight per thread; the elements of a vector are placed one by one
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4* vsrc = reinterpret_cast<const f4*>(src);
    const uint32_t whole = count / 4;
    for (uint32_t q0 = threadIdx.x; q0 < whole; q0 += 4 * kBlock) {
      f4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) v[u] = q0 + u * kBlock < whole ? vsrc[q0 + u * kBlock] : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (q0 + u * kBlock < whole) {
          uint32_t r = fd_div((q0 + u * kBlock) * 4, by_n), c = (q0 + u * kBlock) * 4 - r * n;
#pragma unroll
          for (int i = 0; i < 4; i++) {
            tiny_tile[r * pitch + c] = v[u][i];
            if (++c == n) {
              c = 0;
              r++;
            }
          }
        }
    }
    for (uint32_t e = whole * 4 + threadIdx.x; e < count; e += kBlock) tiny_tile[place(e)] = src[e];
  } else {
    uint32_t e = threadIdx.x;
    for (; e + 7 * kBlock < count; e += 8 * kBlock) {  // eight loads in flight per thread
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = src[e + u * kBlock];
#pragma unroll
      for (int u = 0; u < 8; u++) tiny_tile[place(e + u * kBlock)] = v[u];
    }
    for (; e < count; e += kBlock) tiny_tile[place(e)] = src[e];
  }
  __syncthreads();
  if (threadIdx.x >= rows_here) return;
  const float* row = tiny_tile + threadIdx.x * pitch;
  double acc = 0.0;
  for (uint32_t c = 0; c < n; c++) acc += (double)row[c];
  p.commit(p.a + (int64_t)(row0 + threadIdx.x) * p.oa[0], acc);
}

// Rows of exactly four floats, 16-byte aligned (2 x 2 pooling windows): the row is one vector load, four
// rows per thread in flight, no LDS; the same sum in index order, in binary64.
__global__ __launch_bounds__(kBlock) void reduce_rows_vec4(RowRedParams p) {
  constexpr int U = 4;
  typedef float f4 __attribute__((ext_vector_type(4)));
  const f4* src = reinterpret_cast<const f4*>(p.b);
  const uint32_t first = blockIdx.x * (kBlock * U) + threadIdx.x;
  f4 r[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t row = first + u * kBlock;
    r[u] = row < p.nrows ? src[row] : f4{0.f, 0.f, 0.f, 0.f};
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t row = first + u * kBlock;
    if (row >= p.nrows) continue;
    double acc = 0.0;
#pragma unroll
    for (int c = 0; c < 4; c++) acc += (double)r[u][c];
    p.commit(p.a + (int64_t)row * p.oa[0], acc);
  }
}

// Folds the partial sums of a row in a fixed order.  This launch depends on the one
// before it, so its own latency is all that counts: a thread issues its (up to 16)
// loads together instead of one after the other (full sum of 2^25 elements: 25.0 ->
// 23.4 us over both launches; finishing inside the first launch, by the workgroup that
// arrives last, needs a device-scope release per workgroup and took 114 us).
__global__ __launch_bounds__(kBlock) void reduce_rows_finish(RowRedParams p) {
  __shared__ double lds[kWavesPerBlock];
  constexpr int U = 16;
  const uint32_t row = blockIdx.x;
  int64_t aoff, boff;
  row_offsets(p, row, &aoff, &boff);
  const double* src = p.partials + (int64_t)row * p.splits;
  double t = 0.0;
  for (uint32_t base = 0; base < p.splits; base += kBlock * U) {
    double v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t i = base + u * kBlock + threadIdx.x;
      v[u] = i < p.splits ? src[i] : 0.0;
    }
#pragma unroll
    for (int u = 0; u < U; u++) t += v[u];
  }
  double total = block_sum(t, lds);
  if (threadIdx.x == 0) p.commit(p.a + aoff, total);
}

// ---- generic accumulation: one wavefront per destination element ----------------
struct AccParams {
  float* a;
  const float* b;
  int32_t nk, nr;                       // kept / reduced axis counts
  int64_t nout, nred;
  int64_t kshape[WF2HIP_MAX_RANK], ka[WF2HIP_MAX_RANK], kb[WF2HIP_MAX_RANK];
  int64_t rshape[WF2HIP_MAX_RANK], rb[WF2HIP_MAX_RANK];  // outermost first
  Commit commit;
};

__device__ __forceinline__ void kept_offsets(const AccParams& p, int64_t out, int64_t* aoff,
                                             int64_t* boff) {
  int64_t ao = 0, bo = 0, rem = out;
  for (int i = p.nk - 1; i >= 0; i--) {
    int64_t q = rem / p.kshape[i];
    int64_t idx = rem - q * p.kshape[i];
    rem = q;
    ao += idx * p.ka[i];
    bo += idx * p.kb[i];
  }
  *aoff = ao;
  *boff = bo;
}

__device__ __forceinline__ int64_t reduced_offset(const AccParams& p, int64_t j) {
  int64_t off = 0, rem = j;
  for (int i = p.nr - 1; i >= 0; i--) {
    int64_t q = rem / p.rshape[i];
    int64_t idx = rem - q * p.rshape[i];
    rem = q;
    off += idx * p.rb[i];
  }
  return off;
}

__global__ __launch_bounds__(kBlock) void accumulate_generic(AccParams p) {
  const int64_t out = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  if (out >= p.nout) return;
  int64_t aoff, boff;
  kept_offsets(p, out, &aoff, &boff);
  const int lane = threadIdx.x & (kWave - 1);
  double acc = 0.0;
  for (int64_t j = lane; j < p.nred; j += kWave) acc += (double)p.b[boff + reduced_offset(p, j)];
  acc = wave_sum(acc);
  if (lane == 0) p.commit(p.a + aoff, acc);
}

// Few destinations, each the sum of a long reduced index space that is neither one row nor a
// stack of rows (the per-channel sums of an (N, C, H, W) tensor: sixty-four destinations of
// N H W terms each): `splits` workgroups per destination walk ranges of the reduced indices,
// their sums folded in a fixed order by a second launch.  A wavefront per destination takes
// 950 us for the (32, 64, 56, 56) case.  The reduced index space is below 2^31 here.
__device__ __forceinline__ int64_t reduced_offset32(const AccParams& p, uint32_t j) {
  int64_t off = 0;
  uint32_t rem = j;
  for (int i = p.nr - 1; i > 0; i--) {
    const uint32_t extent = (uint32_t)p.rshape[i];
    const uint32_t q = rem / extent;
    off += (int64_t)(rem - q * extent) * p.rb[i];
    rem = q;
  }
  return off + (int64_t)rem * p.rb[0];
}

__global__ __launch_bounds__(kBlock) void accumulate_partial(AccParams p, uint32_t splits, uint32_t seg,
                                                             double* __restrict__ scratch) {
  __shared__ double lds[kWavesPerBlock];
  const uint32_t out = blockIdx.x / splits, split = blockIdx.x - out * splits;
  int64_t aoff, boff;
  kept_offsets(p, out, &aoff, &boff);
  const float* src = p.b + boff;
  const uint32_t lo = split * seg;
  const uint32_t hi = lo + seg < (uint32_t)p.nred ? lo + seg : (uint32_t)p.nred;
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  uint32_t j = lo + threadIdx.x;
  for (; j + 3 * kBlock < hi; j += 4 * kBlock) {  // four loads in flight
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) v[u] = src[reduced_offset32(p, j + u * kBlock)];
#pragma unroll
    for (int u = 0; u < 4; u++) acc[u] += (double)v[u];
  }
  for (; j < hi; j += kBlock) acc[0] += (double)src[reduced_offset32(p, j)];
  const double total = block_sum((acc[0] + acc[1]) + (acc[2] + acc[3]), lds);
  if (threadIdx.x == 0) {
    if (splits == 1)
      p.commit(p.a + aoff, total);
    else
      scratch[(int64_t)out * splits + split] = total;
  }
}

__global__ __launch_bounds__(kBlock) void accumulate_partial_fold(AccParams p, uint32_t splits,
                                                                  const double* __restrict__ scratch) {
  const int64_t out = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (out >= p.nout) return;
  int64_t aoff, boff;
  kept_offsets(p, out, &aoff, &boff);
  double total = 0.0;
  for (uint32_t s2 = 0; s2 < splits; s2++) total += scratch[out * splits + s2];
  p.commit(p.a + aoff, total);
}

// ---- column form: the kept axis is the contiguous one ----------------------------
// a[c] += sum_j b[j, c] (sums over the batch axes: bias gradients, !sum :axis 0).  A
// wavefront per destination element would read with the row pitch as its stride
// (column sums of (8192, 8192): 7 % of the HBM peak); here a workgroup owns 256
// columns x a range of the reduced index space, each lane adds four columns of four
// rows per step in binary64, and the ranges' partial sums are folded in a fixed order
// by a second launch (scratch from the pool).
struct ColRedParams {
  AccParams acc;     // nk == 1: the kept axis is the last, contiguous one
  int64_t ncols;
  int64_t seg;       // reduced indices per split
  uint32_t splits;
  double* scratch;   // splits x ncols, unused when splits == 1
};

template <bool NT>
__global__ __launch_bounds__(kBlock) void reduce_cols_partial(ColRedParams q) {
  typedef f4 f4u __attribute__((aligned(4)));
  __shared__ double lds[3][kWave][4];
  const AccParams& p = q.acc;
  const int cx = threadIdx.x & (kWave - 1), ry = threadIdx.x / kWave;  // 64 column lanes x 4 row phases
  const uint32_t ctiles = (uint32_t)((q.ncols + 255) / 256);
  const uint32_t ctile = blockIdx.x % ctiles;
  const uint32_t split = blockIdx.x / ctiles;
  const int64_t c = (int64_t)ctile * 256 + 4 * cx;
  const int64_t lo = (int64_t)split * q.seg;
  const int64_t hi = lo + q.seg < p.nred ? lo + q.seg : p.nred;
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  if (c + 4 <= q.ncols) {
    int64_t j = lo + ry;
    for (; j + 12 < hi; j += 16) {  // four rows in flight per lane
      f4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const f4u* src = reinterpret_cast<const f4u*>(p.b + reduced_offset(p, j + 4 * u) + c);
        v[u] = NT ? __builtin_nontemporal_load(src) : *src;
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        acc[0] += (double)v[u].x;
        acc[1] += (double)v[u].y;
        acc[2] += (double)v[u].z;
        acc[3] += (double)v[u].w;
      }
    }
    for (; j < hi; j += 4) {
      const f4 v = *reinterpret_cast<const f4u*>(p.b + reduced_offset(p, j) + c);
      acc[0] += (double)v.x;
      acc[1] += (double)v.y;
      acc[2] += (double)v.z;
      acc[3] += (double)v.w;
    }
  } else {
    for (int64_t j = lo + ry; j < hi; j += 4) {
      const float* row = p.b + reduced_offset(p, j);
#pragma unroll
      for (int k = 0; k < 4; k++)
        if (c + k < q.ncols) acc[k] += (double)row[c + k];
    }
  }
  if (ry > 0) {
#pragma unroll
    for (int k = 0; k < 4; k++) lds[ry - 1][cx][k] = acc[k];
  }
  __syncthreads();
  if (ry == 0) {
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const double total = acc[k] + lds[0][cx][k] + lds[1][cx][k] + lds[2][cx][k];
      if (c + k < q.ncols) {
        if (q.splits == 1)
          p.commit(p.a + c + k, total);
        else
          q.scratch[(int64_t)split * q.ncols + c + k] = total;
      }
    }
  }
}

// Narrow dense matrices (bias gradients of a layer with few outputs: the column sums of
// (N h w, C_out) or (N, classes)): up to 128 columns, rows adjacent in memory.  The 256-column
// tiles above leave most lanes without a column, and below 64 columns the kept axis was handed
// to the wavefront-per-output kernel, which walks a column with the row pitch as its stride
// ((4194304, 4): 30 ms).  Here the workgroup reads k = 256 / ncols whole rows per step, one
// contiguous run of k ncols floats: thread t adds column t mod ncols of every k-th row in
// binary64, eight loads in flight, and the k threads of a column meet in LDS in a fixed order.
__global__ __launch_bounds__(kBlock) void reduce_cols_narrow(ColRedParams q) {
  __shared__ double lds[kBlock];
  const AccParams& p = q.acc;
  const uint32_t ncols = (uint32_t)q.ncols;
  const uint32_t k = kBlock / ncols;  // rows per step
  const uint32_t phase = threadIdx.x / ncols, col = threadIdx.x - phase * ncols;
  const int64_t lo = (int64_t)blockIdx.x * q.seg;
  const int64_t hi = lo + q.seg < p.nred ? lo + q.seg : p.nred;
  double acc = 0.0;
  if (phase < k) {
    const float* src = p.b + col;
    int64_t j = lo + phase;
    for (; j + 7 * (int64_t)k < hi; j += 8 * (int64_t)k) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = src[(j + u * (int64_t)k) * ncols];
#pragma unroll
      for (int u = 0; u < 8; u++) acc += (double)v[u];
    }
    for (; j < hi; j += k) acc += (double)src[j * ncols];
  }
  lds[threadIdx.x] = acc;
  __syncthreads();
  if (threadIdx.x < ncols) {
    double total = lds[threadIdx.x];
    for (uint32_t r = 1; r < k; r++) total += lds[r * ncols + threadIdx.x];
    if (q.splits == 1)
      p.commit(p.a + threadIdx.x, total);
    else
      q.scratch[(int64_t)blockIdx.x * ncols + threadIdx.x] = total;
  }
}

// Folds the splits' partial sums: 64 columns per workgroup, its four wavefronts take every
// fourth split with eight loads in flight, then meet in LDS -- a fixed order.  (One thread per
// column walking all splits in turn waits for memory once per split: 32 us for 128 splits of
// 768 columns, 4 us this way.)
__global__ __launch_bounds__(kBlock) void reduce_cols_finish(ColRedParams q) {
  __shared__ double lds[kWavesPerBlock][kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t c = (int64_t)blockIdx.x * kWave + lane;
  double acc = 0.0;
  if (c < q.ncols) {
    uint32_t s = (uint32_t)wave;
    for (; s + 7 * kWavesPerBlock < q.splits; s += 8 * kWavesPerBlock) {
      double t[8];
#pragma unroll
      for (int u = 0; u < 8; u++) t[u] = q.scratch[(int64_t)(s + u * kWavesPerBlock) * q.ncols + c];
#pragma unroll
      for (int u = 0; u < 8; u++) acc += t[u];
    }
    for (; s < q.splits; s += kWavesPerBlock) acc += q.scratch[(int64_t)s * q.ncols + c];
  }
  lds[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && c < q.ncols)
    q.acc.commit(q.acc.a + c, (lds[0][lane] + lds[1][lane]) + (lds[2][lane] + lds[3][lane]));
}

static int launch_col_reduce(const AccParams& p, int64_t ncols, bool narrow = false) {
  ColRedParams q;
  q.acc = p;
  q.ncols = ncols;
  const int64_t ctiles = narrow ? 1 : ceil_div(ncols, 256);
  const int64_t target = (int64_t)rt().num_cus * 8;
  int64_t splits = ceil_div(target, ctiles);
  // at least 64 reduced indices per workgroup (64 steps of whole rows in the narrow form)
  const int64_t least = narrow ? 64 * (kBlock / ncols) : 64;
  if (splits > p.nred / least) splits = p.nred / least;
  if (splits < 1) splits = 1;
  q.seg = ceil_div(ceil_div(p.nred, splits), 16) * 16;
  splits = ceil_div(p.nred, q.seg);
  q.splits = (uint32_t)splits;
  q.scratch = nullptr;
  if (ctiles * splits >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
  void* scratch = nullptr;
  if (splits > 1) {
    // no block to be had (out of memory): one workgroup per column tile instead
    int held_up = 0;
    if (!scratch_block(&scratch, (size_t)(splits * ncols) * sizeof(double), &held_up)) {
      if (held_up) return held_up;
      splits = 1;
      q.splits = 1;
      q.seg = p.nred;
    } else {
      q.scratch = static_cast<double*>(scratch);
    }
  }
  hipStream_t st = rt().stream;
  if (narrow)
    reduce_cols_narrow<<<(uint32_t)splits, kBlock, 0, st>>>(q);
  else if (p.nred * ncols * 4 >= ((int64_t)192 << 20))
    reduce_cols_partial<true><<<(uint32_t)(ctiles * splits), kBlock, 0, st>>>(q);
  else
    reduce_cols_partial<false><<<(uint32_t)(ctiles * splits), kBlock, 0, st>>>(q);
  int rc = after_launch("reduce_cols_partial");
  if (rc == 0 && splits > 1) {
    reduce_cols_finish<<<(uint32_t)ceil_div(ncols, kWave), kBlock, 0, st>>>(q);
    rc = after_launch("reduce_cols_finish");
  }
  // the block goes back to the pool; later work on the same stream that reuses it is
  // ordered after these launches
  if (scratch) (void)wf2hip_free(scratch);
  return rc;
}

// The reference's order: for one destination element, visit the reduced index
// space in row-major order and apply a <- a op b in binary32 each time.
template <class F>
__global__ __launch_bounds__(kBlock) void accumulate_sequential(AccParams p, F f) {
  const int64_t out = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (out >= p.nout) return;
  int64_t aoff, boff;
  kept_offsets(p, out, &aoff, &boff);
  // overwriting: the reference's zero fill leaves +0 (or -0, which the first add absorbs)
  float acc = p.commit.overwrite ? 0.0f : p.a[aoff];
  const int64_t inner = p.rshape[p.nr - 1];
  const int64_t inner_stride = p.rb[p.nr - 1];
  const int64_t outer = p.nred / inner;
  for (int64_t o = 0; o < outer; o++) {
    int64_t base = boff + reduced_offset(p, o * inner);
    for (int64_t i = 0; i < inner; i++) acc = f(acc, p.b[base + i * inner_stride]);
  }
  p.a[aoff] = p.commit.overwrite ? acc / p.commit.divisor : acc;
}

struct SeqAdd { __device__ __forceinline__ float operator()(float d, float s) const { return d + s; } };
struct SeqSub { __device__ __forceinline__ float operator()(float d, float s) const { return d - s; } };
struct SeqMul { __device__ __forceinline__ float operator()(float d, float s) const { return d * s; } };
struct SeqDiv { __device__ __forceinline__ float operator()(float d, float s) const { return d / s; } };

static void split_axes(const Space& s, AccParams* p) {
  p->nk = p->nr = 0;
  p->nout = p->nred = 1;
  for (int r = 0; r < s.rank; r++) {
    if (s.sa[r] == 0 && s.shape[r] > 1) {
      p->rshape[p->nr] = s.shape[r];
      p->rb[p->nr] = s.sb[r];
      p->nr++;
      p->nred *= s.shape[r];
    } else {
      p->kshape[p->nk] = s.shape[r];
      p->ka[p->nk] = s.sa[r];
      p->kb[p->nk] = s.sb[r];
      p->nk++;
      p->nout *= s.shape[r];
    }
  }
}


// `partials` holds at least kPartialCapacity / 2 binary64 sums: the library's
// own buffer, or the static array of the allocation-free entry point.
static int launch_row_reduce(const Space& s, float* a, const float* b, double* partials, Commit commit) {
  const int last = s.rank - 1;
  RowRedParams p;
  p.commit = commit;
  p.a = a + s.off_a;
  p.b = b + s.off_b;
  p.n0 = s.shape[last];
  p.nouter = s.rank - 1;
  int64_t nrows = 1;
  bool vec_ok = aligned16(p.b);
  for (int i = 0; i < p.nouter; i++) {
    int r = last - 1 - i;
    p.oshape[i] = (uint32_t)s.shape[r];
    p.oa[i] = s.sa[r];
    p.ob[i] = s.sb[r];
    nrows *= s.shape[r];
    if (s.sb[r] % 4 != 0) vec_ok = false;
  }
  p.nrows = (uint32_t)nrows;
  p.partials = partials;
  p.splits = 1;
  p.seg = p.n0;
  hipStream_t st = rt().stream;
  const int64_t target_blocks = (int64_t)rt().num_cus * 8;
  if (p.n0 <= 32 && p.nouter == 1 && p.ob[0] == p.n0 && nrows >= 4 * target_blocks) {
    if (p.n0 == 4 && aligned16(p.b)) {
      reduce_rows_vec4<<<(uint32_t)ceil_div(nrows, (int64_t)kBlock * 4), kBlock, 0, st>>>(p);
      return after_launch("reduce_rows_vec4");
    }
    reduce_rows_tiny<<<(uint32_t)ceil_div(nrows, kBlock), kBlock, (size_t)kBlock * (p.n0 | 1) * sizeof(float), st>>>(
        p, make_fastdiv((uint32_t)p.n0));
    return after_launch("reduce_rows_tiny");
  }
  if (p.n0 < 2048 && nrows * 1 >= 1) {
    // short rows: a wavefront each
    if (nrows >= target_blocks || p.n0 < 8192) {
      uint32_t blocks = (uint32_t)ceil_div(nrows, kWavesPerBlock);
      if (vec_ok && p.n0 <= 512 && nrows >= 4 * target_blocks) {
        const uint32_t short_blocks = (uint32_t)ceil_div(nrows, kWavesPerBlock * 4);
        if (nrows * p.n0 * 4 >= ((int64_t)192 << 20))
          reduce_rows_short<true><<<short_blocks, kBlock, 0, st>>>(p);
        else
          reduce_rows_short<false><<<short_blocks, kBlock, 0, st>>>(p);
        return after_launch("reduce_rows_short");
      }
      // nontemporal loads beyond the Infinity Cache: (65536, 1024) 40.8 us against 44.4 us
      if (vec_ok && nrows * p.n0 * 4 >= ((int64_t)192 << 20))
        reduce_rows_wave<4, true><<<blocks, kBlock, 0, st>>>(p);
      else if (vec_ok)
        reduce_rows_wave<4><<<blocks, kBlock, 0, st>>>(p);
      else
        reduce_rows_wave<1><<<blocks, kBlock, 0, st>>>(p);
      return after_launch("reduce_rows_wave");
    }
  }
  if (nrows < target_blocks) {
    // segments of at least 8192 elements, about 16 workgroups per compute unit: the full
    // sum of 2^25 elements runs 21.4 us in 2048 segments and 20.7 us in 4096
    int64_t by_work = ceil_div(p.n0, 8192);
    int64_t by_fill = ceil_div(2 * target_blocks, nrows);
    int64_t by_cap = (kPartialCapacity / 2) / nrows;
    int64_t splits = by_work < by_fill ? by_work : by_fill;
    if (splits > by_cap) splits = by_cap;
    if (splits < 1) splits = 1;
    int64_t seg = ceil_div(ceil_div(p.n0, splits), 1024) * 1024;
    splits = ceil_div(p.n0, seg);
    p.splits = (uint32_t)splits;
    p.seg = seg;
  }
  int64_t blocks = nrows * p.splits;
  if (blocks >= ((int64_t)1 << 31))
    return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
  // From 16 MiB on, rows (or row segments) of 4096 elements and more go through the streaming
  // kernel; shorter ones, which do not fill one of its 4096-element batches, through the
  // 256-thread kernel.  Kernel durations on operands that are not in a cache, (32768, 2048):
  // 42.1 us against 67.1 us through the streaming kernel; (16384, 4096): 39.2 us streaming
  // against 45.5 us; (8192, 4096): 21.6 us against 24.4 us; (4096, 4096): 13.0 us against
  // 24.6 us; (2048, 4096): 8.6 us against 13.8 us.  On operands the Infinity Cache holds the
  // two are within 10 % of each other up to 32 MiB and the streaming kernel ahead beyond
  // ((4096, 4096): 8.1 us against 11.9 us).  WF2HIP_ROWSUM_STREAM_MB moves the threshold.
  const int64_t bytes = nrows * p.n0 * 4;
  static const int64_t stream_from = [] {
    const char* e = getenv("WF2HIP_ROWSUM_STREAM_MB");
    return (int64_t)(e ? atoi(e) : 16) << 20;
  }();
  if (vec_ok && p.seg >= 4096 && bytes >= stream_from)
    reduce_rows_stream<<<(uint32_t)blocks, kStreamBlock, 0, st>>>(p);
  else if (vec_ok && bytes >= ((int64_t)192 << 20))  // nontemporal loads: (32768, 2048) 39.0 us against 41.7 us
    reduce_rows_block<4, true><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  else if (vec_ok)
    reduce_rows_block<4><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  else
    reduce_rows_block<1><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  WF2_TRY(after_launch("reduce_rows_block"));
  if (p.splits > 1) {
    reduce_rows_finish<<<(uint32_t)nrows, kBlock, 0, st>>>(p);
    WF2_TRY(after_launch("reduce_rows_finish"));
  }
  return 0;
}

// a <- a op b where `a` has broadcast (stride-0) axes.  `s` is normalised.
// `row_partials` replaces the library's partial-sum buffer for the row form.
// may_allocate == false: only the paths that need no scratch beyond row_partials (the row form, the
// sequential form and the wavefront-per-destination form) -- what the allocation-free entry point may use.
static int launch_accumulate_with(int op, const Space& s, float* a, const float* b, double* row_partials,
                                  Commit commit = Commit{0, 1.0f}, bool may_allocate = true) {
  hipStream_t st = rt().stream;
  const bool sequential = op != WF2HIP_ADD || rt().reduce_mode == 1;
  AccParams p;
  p.commit = commit;
  p.a = a + s.off_a;
  p.b = b + s.off_b;
  split_axes(s, &p);
  if (sequential) {
    if (p.nout >= ((int64_t)1 << 31) * kBlock)
      return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
    uint32_t blocks = (uint32_t)ceil_div(p.nout, kBlock);
    switch (op) {
      case WF2HIP_ADD: accumulate_sequential<SeqAdd><<<blocks, kBlock, 0, st>>>(p, SeqAdd{}); break;
      case WF2HIP_SUB: accumulate_sequential<SeqSub><<<blocks, kBlock, 0, st>>>(p, SeqSub{}); break;
      case WF2HIP_MUL: accumulate_sequential<SeqMul><<<blocks, kBlock, 0, st>>>(p, SeqMul{}); break;
      case WF2HIP_DIV: accumulate_sequential<SeqDiv><<<blocks, kBlock, 0, st>>>(p, SeqDiv{}); break;
      default: return fail(WF2HIP_EINVAL, "op %d cannot accumulate", op);
    }
    return after_launch("accumulate_sequential");
  }
  // Row form: the only reduced axis is the innermost one and b is contiguous
  // along it; every other axis is kept.
  const int last = s.rank - 1;
  bool row_form = s.sa[last] == 0 && s.sb[last] == 1 && p.nr == 1 &&
                  p.nout < ((int64_t)1 << 31);
  for (int r = 0; r < last; r++)
    if (s.shape[r] >= ((int64_t)1 << 32)) row_form = false;
  if (row_form) return launch_row_reduce(s, a, b, row_partials, commit);
  if (!may_allocate) {
    int64_t blocks = ceil_div(p.nout, kWavesPerBlock);
    if (blocks >= ((int64_t)1 << 31))
      return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
    accumulate_generic<<<(uint32_t)blocks, kBlock, 0, st>>>(p);
    return after_launch("accumulate_generic");
  }
  // column form: the only kept axis is the last one, contiguous on both sides
  if (p.nk == 1 && s.sa[last] == 1 && s.sb[last] == 1 && s.shape[last] <= 128 && p.nr == 1 &&
      p.rb[0] == s.shape[last] && p.nred >= 16)
    return launch_col_reduce(p, s.shape[last], true);  // a dense narrow matrix
  if (p.nk == 1 && s.sa[last] == 1 && s.sb[last] == 1 && s.shape[last] >= 64 && p.nred >= 2)
    return launch_col_reduce(p, s.shape[last]);
  {
    // few destinations with long sums: ranges of the reduced indices to several workgroups each
    const int64_t target = (int64_t)rt().num_cus * 8;
    if (p.nout < target && p.nred >= 32768 && p.nred < ((int64_t)1 << 31) - 4 * kBlock) {
      int64_t splits = std::min<int64_t>(ceil_div(p.nred, 16384), ceil_div(2 * target, p.nout));
      const int64_t seg = ceil_div(ceil_div(p.nred, splits), kBlock) * kBlock;
      splits = ceil_div(p.nred, seg);
      void* scratch = nullptr;
      int held_up = 0;
      if (splits > 1 && !scratch_block(&scratch, (size_t)(splits * p.nout) * sizeof(double), &held_up) && held_up)
        return held_up;
      if (scratch) {
        accumulate_partial<<<(uint32_t)(p.nout * splits), kBlock, 0, st>>>(p, (uint32_t)splits, (uint32_t)seg,
                                                                          static_cast<double*>(scratch));
        int rc = after_launch("accumulate_partial");
        if (rc == 0) {
          accumulate_partial_fold<<<(uint32_t)ceil_div(p.nout, kBlock), kBlock, 0, st>>>(
              p, (uint32_t)splits, static_cast<const double*>(scratch));
          rc = after_launch("accumulate_partial_fold");
        }
        (void)wf2hip_free(scratch);  // stream order keeps it alive for the launches above
        return rc;
      }
    }
  }
  int64_t blocks = ceil_div(p.nout, kWavesPerBlock);
  if (blocks >= ((int64_t)1 << 31))
    return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
  accumulate_generic<<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  return after_launch("accumulate_generic");
}

int launch_accumulate(int op, const Space& s, float* a, const float* b) {
  return launch_accumulate_with(op, s, a, b, reinterpret_cast<double*>(rt().partials));
}

// ---- max / min ------------------------------------------------------------------
template <bool IsMax>
__global__ __launch_bounds__(kBlock) void maxmin_pass(const float* __restrict__ x, int64_t n,
                                                      int64_t incx, float* __restrict__ out) {
  __shared__ float lds[kWavesPerBlock];
  float best = x[0];
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    float v = x[i * incx];
    best = IsMax ? fmaxf(best, v) : fminf(best, v);
  }
  best = IsMax ? wave_max(best) : wave_min(best);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < kWavesPerBlock; i++) best = IsMax ? fmaxf(best, lds[i]) : fminf(best, lds[i]);
    out[blockIdx.x] = best;
  }
}

template <bool IsMax>
static int launch_maxmin(long n, const float* x, long incx, float* out) {
  if (n <= 0) return fail(WF2HIP_EINVAL, "max/min of an empty range");
  if (!x || !out) return fail(WF2HIP_EINVAL, "null pointer");
  hipStream_t st = rt().stream;
  int64_t blocks = ceil_div(n, kBlock * 16);
  if (blocks > 1024) blocks = 1024;
  if (blocks == 1) {
    maxmin_pass<IsMax><<<1, kBlock, 0, st>>>(x, n, incx, out);
    return after_launch("maxmin");
  }
  float* partial = rt().partials;
  maxmin_pass<IsMax><<<(uint32_t)blocks, kBlock, 0, st>>>(x, n, incx, partial);
  WF2_TRY(after_launch("maxmin pass 1"));
  maxmin_pass<IsMax><<<1, kBlock, 0, st>>>(partial, blocks, 1, out);
  return after_launch("maxmin pass 2");
}

// ---- fused row kernels: one wavefront per row, the row held in registers (RowRegs, wf2_rows.h) ----
// softmax over the first `valid` columns of a row; columns valid..ncols-1 of
// the output are set to 0 (used by the causal form).
// RW rows per wavefront: with one or two vectors per lane and row a wavefront that
// takes a single row has 1 - 2 KB in flight and leaves the memory system idle (rows
// of 256: 68 % of the HBM peak for softmax, 53 % for LayerNorm at 2^26 elements); the
// rows' loads are all issued first and their reductions interleave.
//
// XENT: the cross entropy of Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:90-126,
// 158) in the same pass.  The softmax z goes to `out` (the node saves it for its backward)
// and loss = -1 (labels log(z + delta)), each operation rounded to binary32 as the nodes
// of cross-entropy-loss round them, goes to xe.loss; labels and loss are rows of ncols.
struct Xent {
  const float* labels;
  float* loss;
  float delta;
};

__device__ __forceinline__ float xent_term(float label, float z, float delta) {
  return -1.0f * (label * logf_(z + delta));
}

template <int NV, bool VEC, bool NT, int RW = 1, bool XENT = false>
__global__ __launch_bounds__(kBlock) void softmax_rows_wave(const float* __restrict__ x, int64_t ldx,
                                                            float* __restrict__ out, int64_t ldo,
                                                            int64_t nrows, int64_t ncols,
                                                            int64_t causal_seq, float scale, Xent xe) {
  const int64_t row0 = ((int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * RW;
  if (row0 >= nrows) return;
  const int lane = threadIdx.x & (kWave - 1);
  const float ninf = -__builtin_inff();
  RowRegs<NV, VEC, NT> r[RW];
  RowRegs<NV, VEC, NT> t[XENT ? RW : 1];
  int64_t valid[RW];
#pragma unroll
  for (int w = 0; w < RW; w++) {
    const int64_t row = row0 + w < nrows ? row0 + w : nrows - 1;  // a repeated last row is computed and not stored
    valid[w] = causal_seq > 0 ? (row % causal_seq) + 1 : ncols;
    r[w].load(x + row * ldx, valid[w], lane, ninf);
  }
  if (XENT) {
#pragma unroll
    for (int w = 0; w < RW; w++) {
      const int64_t row = row0 + w < nrows ? row0 + w : nrows - 1;
      t[w].load(xe.labels + row * ncols, ncols, lane, 0.0f);
    }
  }
#pragma unroll
  for (int w = 0; w < RW; w++) {
    float m = ninf;
#pragma unroll
    for (int g = 0; g < NV; g++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        if (causal_seq > 0) {
          // binary32 product, like a MulNode; padding stays -inf whatever the sign of scale
          bool in = RowRegs<NV, VEC, NT>::col(g, c, lane) < valid[w];
          r[w].v[g][c] = in ? r[w].v[g][c] * scale : ninf;
        }
        m = fmaxf(m, r[w].v[g][c]);
      }
    m = wave_max(m);
    // exp(x - max) in binary32 through v_exp_f32: 2^(d log2 e) with the rounding
    // error of the product folded back, so what remains is the rounding of d
    // itself (|d| 2^-24 relative: 5e-7 at d = -10, 4e-6 at the underflow edge)
    // and the instruction's own ulp.  The binary64 body this replaces cost 21
    // VALU slots per element against 12 and left the kernel ALU-bound once the
    // clock settles (65 % of the HBM peak at (32768, 1024)).  Clamping d at -160
    // makes padding (-inf) and everything below the denormals an exact 0.
    float sum = 0.0f;
#pragma unroll
    for (int g = 0; g < NV; g++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const float d = fmaxf(r[w].v[g][c] - m, -160.0f);
        const float t = d * 1.44269502f;
        float tl = __builtin_fmaf(d, 1.44269502f, -t);
        tl = __builtin_fmaf(d, 1.92596299e-8f, tl);
        const float e = __builtin_amdgcn_exp2f(t);
        const float ed = __builtin_fmaf(e, tl * 0.693147182f, e);
        r[w].v[g][c] = ed;
        sum += ed;
      }
    const double total = wave_sum((double)sum);
    const float inv = (float)(1.0 / total);
#pragma unroll
    for (int g = 0; g < NV; g++)
#pragma unroll
      for (int c = 0; c < 4; c++) r[w].v[g][c] *= inv;
  }
#pragma unroll
  for (int w = 0; w < RW; w++)
    if (row0 + w < nrows) r[w].store(out + (row0 + w) * ldo, ncols, lane);
  if (XENT) {
#pragma unroll
    for (int w = 0; w < RW; w++) {
#pragma unroll
      for (int g = 0; g < NV; g++)
#pragma unroll
        for (int c = 0; c < 4; c++) t[w].v[g][c] = xent_term(t[w].v[g][c], r[w].v[g][c], xe.delta);
      if (row0 + w < nrows) t[w].store(xe.loss + (row0 + w) * ncols, ncols, lane);
    }
  }
}

// Rows of 769 ... 1024 columns: two wavefronts per row, each holding half of it (two
// vectors per lane), two rows per workgroup; maxima and sums of the halves meet in
// LDS.  Twice the wavefronts of the one-per-row form at half the registers and half
// the arithmetic between a wavefront's loads and its stores: (32768, 1024) 44.5 ->
// 43.1 us, where a plain copy of the same rows by one wavefront each takes 43.9 us.
template <bool VEC, bool NT, bool XENT = false>
__global__ __launch_bounds__(kBlock) void softmax_rows_pair(const float* __restrict__ x, int64_t ldx,
                                                            float* __restrict__ out, int64_t ldo,
                                                            int64_t nrows, int64_t ncols,
                                                            int64_t causal_seq, float scale, Xent xe) {
  constexpr int NVH = 2;
  constexpr int64_t kHalf = (int64_t)NVH * kWave * 4;  // 512 columns
  __shared__ float lmax[kWavesPerBlock];
  __shared__ double lsum[kWavesPerBlock];
  const int w = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), half = w & 1;
  const int64_t row_raw = (int64_t)blockIdx.x * 2 + (w >> 1);
  const int64_t row = row_raw < nrows ? row_raw : nrows - 1;  // a repeated last row is computed and not stored
  const float ninf = -__builtin_inff();
  const int64_t valid = causal_seq > 0 ? (row % causal_seq) + 1 : ncols;
  auto part = [&](int64_t n) { n -= half * kHalf; return n < 0 ? (int64_t)0 : (n > kHalf ? kHalf : n); };
  const int64_t valid_here = part(valid);
  RowRegs<NVH, VEC, NT> r, t;
  r.load(x + row * ldx + half * kHalf, valid_here, lane, ninf);
  if (XENT) t.load(xe.labels + row * ncols + half * kHalf, part(ncols), lane, 0.0f);
  float m = ninf;
#pragma unroll
  for (int g = 0; g < NVH; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      if (causal_seq > 0) {
        const bool in = RowRegs<NVH, VEC, NT>::col(g, c, lane) < valid_here;
        r.v[g][c] = in ? r.v[g][c] * scale : ninf;
      }
      m = fmaxf(m, r.v[g][c]);
    }
  m = wave_max(m);
  if (lane == 0) lmax[w] = m;
  __syncthreads();
  m = fmaxf(lmax[w & ~1], lmax[w | 1]);
  float sum = 0.0f;
#pragma unroll
  for (int g = 0; g < NVH; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      // the exponential of softmax_rows_wave
      const float d = fmaxf(r.v[g][c] - m, -160.0f);
      const float t = d * 1.44269502f;
      float tl = __builtin_fmaf(d, 1.44269502f, -t);
      tl = __builtin_fmaf(d, 1.92596299e-8f, tl);
      const float e = __builtin_amdgcn_exp2f(t);
      const float ed = __builtin_fmaf(e, tl * 0.693147182f, e);
      r.v[g][c] = ed;
      sum += ed;
    }
  const double total_here = wave_sum((double)sum);
  if (lane == 0) lsum[w] = total_here;
  __syncthreads();
  const float inv = (float)(1.0 / (lsum[w & ~1] + lsum[w | 1]));
#pragma unroll
  for (int g = 0; g < NVH; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) r.v[g][c] *= inv;
  if (row_raw < nrows) r.store(out + row * ldo + half * kHalf, part(ncols), lane);
  if (XENT) {
#pragma unroll
    for (int g = 0; g < NVH; g++)
#pragma unroll
      for (int c = 0; c < 4; c++) t.v[g][c] = xent_term(t.v[g][c], r.v[g][c], xe.delta);
    if (row_raw < nrows) t.store(xe.loss + row * ncols + half * kHalf, part(ncols), lane);
  }
}

// Rows of 4097 ... 65536 columns (a vocabulary: the logits of a language model): a workgroup of
// 1024 threads per row, thread t holding columns t, t + 1024, ... in registers, so the row is read
// once and written once; maxima and sums meet in LDS.  The three-pass form above reads the row three
// times from wherever it lies (reads that hit the L2 cost the memory system what misses cost):
// (4096, 50257) 982 us.  The exponential of softmax_rows_wave.
constexpr int kLongBlock = 1024;

// Thread t holds the vectors t, t + 1024, ... of four consecutive columns each.  A row of an odd length (a
// vocabulary of 50257) starts wherever the row before it ends, so the vectors are read and written as
// unaligned 16-byte accesses (one instruction each on this hardware); the last columns of a row whose length
// is no multiple of four go one by one.  Against a thread holding columns t, t + 1024, ... one by one: a quarter
// of the memory instructions and no spills at 52 elements per thread -- (1024, 50257) 110 -> 95 us, with the
// cross entropy 256 -> 176 us; (1024, 65536) 192 -> 139 and 547 -> 259 us; (8192, 8192) level, with the cross
// entropy 194 -> 183 us.
template <int E4, bool XENT>
__global__ __launch_bounds__(kLongBlock) void softmax_rows_long(const float* __restrict__ x, int64_t ldx,
                                                                 float* __restrict__ out, int64_t ldo, int64_t ncols,
                                                                 Xent xe) {
  __shared__ float lmax[kLongBlock / kWave];
  __shared__ double lsum[kLongBlock / kWave];
  const float* xr = x + (int64_t)blockIdx.x * ldx;
  const float ninf = -__builtin_inff();
  const int64_t whole = ncols / 4;  // vectors wholly inside the row
  f4 v[E4];
  float m = ninf;
#pragma unroll
  for (int k = 0; k < E4; k++) {
    const int64_t j = (int64_t)k * kLongBlock + threadIdx.x;
    v[k] = f4{ninf, ninf, ninf, ninf};
    if (j < whole) {
      __builtin_memcpy(&v[k], xr + 4 * j, 16);
    } else if (j == whole) {
#pragma unroll
      for (int c = 0; c < 3; c++)
        if (4 * j + c < ncols) v[k][c] = xr[4 * j + c];
    }
    m = fmaxf(fmaxf(m, fmaxf(v[k][0], v[k][1])), fmaxf(v[k][2], v[k][3]));
  }
  m = wave_max(m);
  if ((threadIdx.x & (kWave - 1)) == 0) lmax[threadIdx.x / kWave] = m;
  __syncthreads();
  m = lmax[0];
#pragma unroll
  for (int w = 1; w < kLongBlock / kWave; w++) m = fmaxf(m, lmax[w]);
  float sum = 0.0f;
#pragma unroll
  for (int k = 0; k < E4; k++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const float d = fmaxf(v[k][c] - m, -160.0f);
      const float t = d * 1.44269502f;
      float tl = __builtin_fmaf(d, 1.44269502f, -t);
      tl = __builtin_fmaf(d, 1.92596299e-8f, tl);
      const float e = __builtin_amdgcn_exp2f(t);
      const float ed = __builtin_fmaf(e, tl * 0.693147182f, e);
      v[k][c] = ed;
      sum += ed;
    }
  const double part = wave_sum((double)sum);
  if ((threadIdx.x & (kWave - 1)) == 0) lsum[threadIdx.x / kWave] = part;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int w = 0; w < kLongBlock / kWave; w++) total += lsum[w];
  const float inv = (float)(1.0 / total);
  float* orow = out + (int64_t)blockIdx.x * ldo;
#pragma unroll
  for (int k = 0; k < E4; k++) {
    const int64_t j = (int64_t)k * kLongBlock + threadIdx.x;
    v[k] *= inv;
    if (j < whole) {
      __builtin_memcpy(orow + 4 * j, &v[k], 16);
    } else if (j == whole) {
#pragma unroll
      for (int c = 0; c < 3; c++)
        if (4 * j + c < ncols) orow[4 * j + c] = v[k][c];
    }
  }
  if (XENT) {
    const float* lrow = xe.labels + (int64_t)blockIdx.x * ncols;
    float* srow = xe.loss + (int64_t)blockIdx.x * ncols;
#pragma unroll
    for (int k = 0; k < E4; k++) {
      const int64_t j = (int64_t)k * kLongBlock + threadIdx.x;
      if (j < whole) {
        f4 lab, r;
        __builtin_memcpy(&lab, lrow + 4 * j, 16);
#pragma unroll
        for (int c = 0; c < 4; c++) r[c] = xent_term(lab[c], v[k][c], xe.delta);
        __builtin_memcpy(srow + 4 * j, &r, 16);
      } else if (j == whole) {
#pragma unroll
        for (int c = 0; c < 3; c++)
          if (4 * j + c < ncols) srow[4 * j + c] = xent_term(lrow[4 * j + c], v[k][c], xe.delta);
      }
    }
  }
}

// Rows beyond 65536 columns, or a few long rows that would leave most compute units without a workgroup
// ((1, 16777216): 62 ms on one workgroup): the row in pieces of 16384 columns, a workgroup of 1024 threads
// each.  softmax_split_stats leaves every piece's maximum m_p and s_p = sum exp(x - m_p) (its 16 elements
// per thread in registers, one read); softmax_split_apply folds the pieces of its row -- M = max m_p,
// S = sum s_p exp(m_p - M) in binary64, in a fixed order -- and writes exp(x - M) / S: two reads and a
// write of the row.  The exponential of softmax_rows_wave.
constexpr int kSplitE = 16;
constexpr int64_t kSplitPiece = (int64_t)kLongBlock * kSplitE;

__device__ __forceinline__ float exp_below_max(float v, float m) {
  const float d = fmaxf(v - m, -160.0f);
  const float t = d * 1.44269502f;
  float tl = __builtin_fmaf(d, 1.44269502f, -t);
  tl = __builtin_fmaf(d, 1.92596299e-8f, tl);
  const float e = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(e, tl * 0.693147182f, e);
}

__device__ __forceinline__ float long_block_max(float m, float* lmax) {
  m = wave_max(m);
  __syncthreads();  // lmax may still be read from an earlier use
  if ((threadIdx.x & (kWave - 1)) == 0) lmax[threadIdx.x / kWave] = m;
  __syncthreads();
  m = lmax[0];
#pragma unroll
  for (int w = 1; w < kLongBlock / kWave; w++) m = fmaxf(m, lmax[w]);
  return m;
}

__device__ __forceinline__ double long_block_sum(double s, double* lsum) {
  s = wave_sum(s);
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) lsum[threadIdx.x / kWave] = s;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int w = 0; w < kLongBlock / kWave; w++) total += lsum[w];
  return total;
}

__global__ __launch_bounds__(kLongBlock) void softmax_split_stats(const float* __restrict__ x, int64_t ldx,
                                                                  int64_t ncols, uint32_t pieces,
                                                                  float* __restrict__ pmax,
                                                                  double* __restrict__ psum) {
  __shared__ float lmax[kLongBlock / kWave];
  __shared__ double lsum[kLongBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const float* xr = x + (int64_t)row * ldx;
  const int64_t c0 = (int64_t)piece * kSplitPiece + threadIdx.x;
  const float ninf = -__builtin_inff();
  float v[kSplitE];
  float m = ninf;
#pragma unroll
  for (int k = 0; k < kSplitE; k++) {
    const int64_t c = c0 + (int64_t)k * kLongBlock;
    v[k] = c < ncols ? xr[c] : ninf;
    m = fmaxf(m, v[k]);
  }
  m = long_block_max(m, lmax);
  float sum = 0.0f;
#pragma unroll
  for (int k = 0; k < kSplitE; k++) sum += exp_below_max(v[k], m);
  const double total = long_block_sum((double)sum, lsum);
  if (threadIdx.x == 0) {
    pmax[blockIdx.x] = m;
    psum[blockIdx.x] = total;
  }
}

template <bool XENT>
__global__ __launch_bounds__(kLongBlock) void softmax_split_apply(const float* x, int64_t ldx,  // out may be x
                                                                  float* out, int64_t ldo, int64_t ncols,
                                                                  uint32_t pieces, const float* __restrict__ pmax,
                                                                  const double* __restrict__ psum, Xent xe) {
  __shared__ float lmax[kLongBlock / kWave];
  __shared__ double lsum[kLongBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const float ninf = -__builtin_inff();
  float m = ninf;
  for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock) m = fmaxf(m, pmax[row * pieces + i]);
  m = long_block_max(m, lmax);
  double s = 0.0;
  for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock)
    s += psum[row * pieces + i] * (double)exp_below_max(pmax[row * pieces + i], m);
  const float inv = (float)(1.0 / long_block_sum(s, lsum));
  const float* xr = x + (int64_t)row * ldx;
  float* orow = out + (int64_t)row * ldo;
  const int64_t c0 = (int64_t)piece * kSplitPiece + threadIdx.x;
  float v[kSplitE];
#pragma unroll
  for (int k = 0; k < kSplitE; k++) {
    const int64_t c = c0 + (int64_t)k * kLongBlock;
    v[k] = c < ncols ? xr[c] : ninf;
  }
  float lab[XENT ? kSplitE : 1];
  if (XENT) {
#pragma unroll
    for (int k = 0; k < kSplitE; k++) {
      const int64_t c = c0 + (int64_t)k * kLongBlock;
      lab[k] = c < ncols ? xe.labels[(int64_t)row * ncols + c] : 0.0f;
    }
  }
#pragma unroll
  for (int k = 0; k < kSplitE; k++) {
    const int64_t c = c0 + (int64_t)k * kLongBlock;
    v[k] = exp_below_max(v[k], m) * inv;
    if (c < ncols) orow[c] = v[k];
  }
  if (XENT) {
#pragma unroll
    for (int k = 0; k < kSplitE; k++) {
      const int64_t c = c0 + (int64_t)k * kLongBlock;
      if (c < ncols) xe.loss[(int64_t)row * ncols + c] = xent_term(lab[k], v[k], xe.delta);
    }
  }
}

// A few very long rows in ONE launch: a workgroup of 1024 threads holds a piece of 65536 columns in registers,
// leaves the piece's maximum and sum, waits until every piece of the launch has done so, folds its row's pieces
// like softmax_split_apply and writes its share -- one read and one write of the row where the two launches
// above read it twice.
//
// The wait needs every workgroup of the grid on the device at the same time: the host launches this form only
// when the grid is no larger than what the device holds at once (one such workgroup per compute unit).  Even
// so a workgroup never waits without bound: after kMeetSpins polls it stops waiting and works out the row's
// maximum and sum from the row itself -- which is why x and out must not overlap here.  The two counters are
// left at zero by the last workgroup to pass, for the next launch; launches of this kernel that overlap in
// time on one device (several streams) would share them and must not happen: the library launches on one stream.
constexpr int kOneE = 64;
constexpr int64_t kOnePiece = (int64_t)kLongBlock * kOneE;
constexpr uint32_t kMeetSpins = 1u << 20;  // about a second
__device__ unsigned int g_softmax_meet[2];  // [0]: pieces that left their statistics, [1]: workgroups past the wait

template <bool XENT>
__global__ __launch_bounds__(kLongBlock) void softmax_one_launch(const float* __restrict__ x, int64_t ldx,
                                                                 float* __restrict__ out, int64_t ldo, int64_t ncols,
                                                                 uint32_t pieces, float* pmax, double* psum,
                                                                 uint32_t spins, Xent xe) {
  __shared__ float lmax[kLongBlock / kWave];
  __shared__ double lsum[kLongBlock / kWave];
  __shared__ int met;
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const float* xr = x + (int64_t)row * ldx;
  const int64_t c0 = (int64_t)piece * kOnePiece;
  const float ninf = -__builtin_inff();
  // thread t holds the 16-byte vectors (g 1024 + t) 4 of the piece (16-byte aligned rows, ncols a multiple of 4)
  float v[kOneE];
  const uint32_t first = threadIdx.x * 4;                            // within the piece
  const uint32_t left = (uint32_t)((ncols - c0 < kOnePiece ? ncols - c0 : kOnePiece));  // columns of this piece
  const float* xp = xr + c0;
  float m = ninf;
#pragma unroll
  for (int g = 0; g < kOneE / 4; g++) {
    f4 t = {ninf, ninf, ninf, ninf};
    if (first + g * 4 * kLongBlock < left) t = __builtin_nontemporal_load(reinterpret_cast<const f4*>(xp + first + g * 4 * kLongBlock));
    v[4 * g] = t.x; v[4 * g + 1] = t.y; v[4 * g + 2] = t.z; v[4 * g + 3] = t.w;
  }
  // exponentials once, against the thread's own maximum (no exchange between the loads and this pass): the
  // output is e_k exp(m_thread - M) / S
#pragma unroll
  for (int k = 0; k < kOneE; k++) m = fmaxf(m, v[k]);
  float sum = 0.0f;
#pragma unroll
  for (int k = 0; k < kOneE; k++) {
    v[k] = exp_below_max(v[k], m);
    sum += v[k];
  }
  const float mine = m;
  m = long_block_max(mine, lmax);
  const double total = long_block_sum((double)sum * (double)exp_below_max(mine, m), lsum);
  if (threadIdx.x == 0) {
    // The statistics go to memory past the caches (device-scope atomic stores), are waited for, and only then
    // is the arrival counted: the order a release would give, without its write-back of the whole L2 (2.6 us
    // per workgroup here).  The readers below use device-scope loads, which no stale cache line serves.
    __hip_atomic_store(&pmax[blockIdx.x], m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&psum[blockIdx.x], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __hip_atomic_fetch_add(&g_softmax_meet[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t polls = 0;
    while (__hip_atomic_load(&g_softmax_meet[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gridDim.x && polls < spins) {
      __builtin_amdgcn_s_sleep(8);
      polls++;
    }
    met = __hip_atomic_load(&g_softmax_meet[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= gridDim.x;
  }
  __syncthreads();
  float big = ninf;
  double s = 0.0;
  if (met) {
    // the fold of softmax_split_apply; the statistics were written by other workgroups during this launch:
    // read them past the caches this compute unit may hold stale lines in
    for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock)
      big = fmaxf(big, __hip_atomic_load(&pmax[row * pieces + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    big = long_block_max(big, lmax);
    for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock)
      s += __hip_atomic_load(&psum[row * pieces + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) *
           (double)exp_below_max(__hip_atomic_load(&pmax[row * pieces + i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), big);
  } else {
    // gave up waiting: the row's maximum and sum from the row itself (x is not written by this launch)
    for (int64_t c = threadIdx.x; c < ncols; c += kLongBlock) big = fmaxf(big, xr[c]);
    big = long_block_max(big, lmax);
    float part = 0.0f;
    for (int64_t c = threadIdx.x; c < ncols; c += kLongBlock) part += exp_below_max(xr[c], big);
    s = (double)part;
  }
  const float factor = exp_below_max(mine, big) * (float)(1.0 / long_block_sum(s, lsum));
  float* op = out + (int64_t)row * ldo + c0;
#pragma unroll
  for (int g = 0; g < kOneE / 4; g++) {
    f4 t;
#pragma unroll
    for (int c = 0; c < 4; c++) t[c] = v[4 * g + c] * factor;
    if (first + g * 4 * kLongBlock < left) {
      __builtin_nontemporal_store(t, reinterpret_cast<f4*>(op + first + g * 4 * kLongBlock));
      if constexpr (XENT) {  // labels and loss are packed (rows, ncols)
        const int64_t at = (int64_t)row * ncols + c0 + first + g * 4 * kLongBlock;
        const f4 lab = __builtin_nontemporal_load(reinterpret_cast<const f4*>(xe.labels + at));
        f4 l;
#pragma unroll
        for (int c = 0; c < 4; c++) l[c] = xent_term(lab[c], t[c], xe.delta);
        __builtin_nontemporal_store(l, reinterpret_cast<f4*>(xe.loss + at));
      }
    }
  }
  if (threadIdx.x == 0) {
    const unsigned int before = __hip_atomic_fetch_add(&g_softmax_meet[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before + 1 == gridDim.x) {  // everyone has arrived and is past the wait: zero for the next launch
      __hip_atomic_store(&g_softmax_meet[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&g_softmax_meet[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <int NV, bool VEC, bool NT, int RW = 1>
__global__ __launch_bounds__(kBlock) void layernorm_rows_wave(const float* __restrict__ x,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta,
                                                              float eps, float* __restrict__ out,
                                                              int64_t nrows, int64_t ncols) {
  const int64_t row0 = ((int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * RW;
  if (row0 >= nrows) return;
  const int lane = threadIdx.x & (kWave - 1);
  RowRegs<NV, VEC, NT> r[RW];
  RowRegs<NV, VEC, false> g, b;
#pragma unroll
  for (int w = 0; w < RW; w++) r[w].load(x + (row0 + w < nrows ? row0 + w : nrows - 1) * ncols, ncols, lane, 0.0f);
  g.load(gamma, ncols, lane, 0.0f);
  b.load(beta, ncols, lane, 0.0f);
#pragma unroll
  for (int w = 0; w < RW; w++) {
    if constexpr (RW > 1) {
      // rows of at most 512 columns: binary32 statistics (each lane adds at most eight
      // terms, the wavefront folds 64 partial sums as a tree: relative error of the
      // mean and the variance below 1e-6), a third of the instructions of the binary64 form
      float sum = 0.0f;
#pragma unroll
      for (int i = 0; i < NV; i++)
#pragma unroll
        for (int c = 0; c < 4; c++) sum += r[w].v[i][c];
      const float mean = wave_sum32(sum) / (float)ncols;
      float sq = 0.0f;
#pragma unroll
      for (int i = 0; i < NV; i++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          bool in = RowRegs<NV, VEC, NT>::col(i, c, lane) < ncols;
          float d = in ? r[w].v[i][c] - mean : 0.0f;
          sq = __builtin_fmaf(d, d, sq);
        }
      const float var = wave_sum32(sq) / (float)ncols;
      const float rstd = (float)(1.0 / __builtin_sqrt((double)var + (double)eps));
#pragma unroll
      for (int i = 0; i < NV; i++)
#pragma unroll
        for (int c = 0; c < 4; c++)
          r[w].v[i][c] = __builtin_fmaf((r[w].v[i][c] - mean) * rstd, g.v[i][c], b.v[i][c]);
    } else {
      // longer rows: the mean from binary64 sums; deviations, their squares (four
      // partial sums per lane, folded in binary64) and the output in binary32 -- two
      // binary64 operations per element where the all-binary64 form had twelve (same
      // bandwidth, (65536, 1024) at 77.5 % of the HBM peak, for less power; fetching gamma
      // and beta only after the statistics frees 24 registers and runs slower, 75.8 %)
      double sum = 0.0;
#pragma unroll
      for (int i = 0; i < NV; i++)
#pragma unroll
        for (int c = 0; c < 4; c++) sum += (double)r[w].v[i][c];
      const double mean = wave_sum(sum) / (double)ncols;
      const float meanf = (float)mean;
      float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int i = 0; i < NV; i++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const bool in = RowRegs<NV, VEC, NT>::col(i, c, lane) < ncols;
          const float d = in ? r[w].v[i][c] - meanf : 0.0f;
          r[w].v[i][c] = d;
          sq[c] = __builtin_fmaf(d, d, sq[c]);
        }
      const double var = wave_sum(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3])) / (double)ncols;
      const float rstd = (float)(1.0 / __builtin_sqrt(var + (double)eps));
#pragma unroll
      for (int i = 0; i < NV; i++)
#pragma unroll
        for (int c = 0; c < 4; c++) r[w].v[i][c] = __builtin_fmaf(r[w].v[i][c] * rstd, g.v[i][c], b.v[i][c]);
    }
  }
#pragma unroll
  for (int w = 0; w < RW; w++)
    if (row0 + w < nrows) r[w].store(out + (row0 + w) * ncols, ncols, lane);
}

// Rows beyond the register tile (2048 columns): a workgroup per row, three passes
// over the row (sum, squared deviations, output); the second and third come from
// the L2 the first one filled.  Same arithmetic as the wavefront form.
__global__ __launch_bounds__(kBlock) void layernorm_rows_block(const float* __restrict__ x,
                                                               const float* __restrict__ gamma,
                                                               const float* __restrict__ beta, float eps,
                                                               float* __restrict__ out, int64_t ncols) {
  __shared__ double lds[kWavesPerBlock];
  __shared__ double stat;
  const float* xr = x + (int64_t)blockIdx.x * ncols;
  float* outr = out + (int64_t)blockIdx.x * ncols;
  double sum = 0.0;
  for (int64_t c = threadIdx.x; c < ncols; c += kBlock) sum += (double)xr[c];
  double total = block_sum(sum, lds);
  if (threadIdx.x == 0) stat = total / (double)ncols;
  __syncthreads();
  const double mean = stat;
  double sq = 0.0;
  for (int64_t c = threadIdx.x; c < ncols; c += kBlock) {
    const double d = (double)xr[c] - mean;
    sq += d * d;
  }
  __syncthreads();  // everyone has read `stat` and is done with `lds`
  total = block_sum(sq, lds);
  if (threadIdx.x == 0) stat = 1.0 / __builtin_sqrt(total / (double)ncols + (double)eps);
  __syncthreads();
  const double rstd = stat;
  for (int64_t c = threadIdx.x; c < ncols; c += kBlock)
    outr[c] = (float)(((double)xr[c] - mean) * rstd * (double)gamma[c] + (double)beta[c]);
}

// Rows of 8196 ... 65536 columns (multiples of 4), at least one per compute unit: a workgroup of 1024
// threads per row, thread t holding the E / 4 16-byte vectors (g 1024 + t) 4 of the row in registers --
// one read and one write.  The arithmetic of layernorm_rows_wide.
template <int E, bool NT>
__global__ __launch_bounds__(kPieceBlock) void layernorm_rows_long(const float* __restrict__ x,
                                                                  const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta, float eps,
                                                                  float* __restrict__ out, int64_t ncols) {
  __shared__ double lds[2 * kPieceBlock / kWave];
  const int64_t base = (int64_t)blockIdx.x * ncols;
  f4 v[E / 4];
  bool in[E / 4];
#pragma unroll
  for (int g = 0; g < E / 4; g++) {
    const int64_t c = ((int64_t)g * kPieceBlock + threadIdx.x) * 4;
    in[g] = c < ncols;
    v[g] = f4{0.f, 0.f, 0.f, 0.f};
    if (in[g]) {
      const f4* q = reinterpret_cast<const f4*>(x + base + c);
      v[g] = NT ? __builtin_nontemporal_load(q) : *q;
    }
  }
  double sum = 0.0, unused;
#pragma unroll
  for (int g = 0; g < E / 4; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) sum += (double)v[g][c];
  const float mean = (float)(piece_sum2(sum, 0.0, lds, &unused) / (double)ncols);
  float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int g = 0; g < E / 4; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const float d = in[g] ? v[g][c] - mean : 0.0f;
      v[g][c] = d;
      sq[c] = __builtin_fmaf(d, d, sq[c]);
    }
  const double var =
      piece_sum2(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3]), 0.0, lds, &unused) / (double)ncols;
  const float rstd = (float)(1.0 / __builtin_sqrt(var + (double)eps));
#pragma unroll
  for (int g = 0; g < E / 4; g++) {
    if (!in[g]) continue;
    const int64_t c = ((int64_t)g * kPieceBlock + threadIdx.x) * 4;
    const f4 gm = *reinterpret_cast<const f4*>(gamma + c);
    const f4 bt = *reinterpret_cast<const f4*>(beta + c);
    f4 r;
#pragma unroll
    for (int k = 0; k < 4; k++) r[k] = __builtin_fmaf(v[g][k] * rstd, gm[k], bt[k]);
    f4* q = reinterpret_cast<f4*>(out + base + c);
    if (NT)
      __builtin_nontemporal_store(r, q);
    else
      *q = r;
  }
}

// Rows beyond 8192 columns: the row in pieces of 16384 columns (layernorm_piece_stats), then every
// piece folds its row's statistics and writes its share of the output: two reads and a write of the
// row, on as many workgroups as there are pieces ((1, 16777216) on 1024 of them where the three-pass
// kernel above has one).
template <bool VEC>
__global__ __launch_bounds__(kPieceBlock) void layernorm_piece_apply(const float* __restrict__ x,
                                                                    const float* __restrict__ gamma,
                                                                    const float* __restrict__ beta, float eps,
                                                                    float* __restrict__ out, int64_t ncols,
                                                                    uint32_t pieces, const double* __restrict__ psum,
                                                                    const double* __restrict__ pdev) {
  __shared__ double lds[2 * kPieceBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const int64_t c0 = (int64_t)piece * kPieceCols;
  const int64_t left = ncols - c0;
  PieceRegs<VEC> r, g, b;
  r.load(x + (int64_t)row * ncols + c0, left, 0.0f);
  g.load(gamma + c0, left, 0.0f);
  b.load(beta + c0, left, 0.0f);
  float mean, rstd;
  piece_row_stats(psum + (int64_t)row * pieces, pdev + (int64_t)row * pieces, pieces, ncols, eps, lds, &mean, &rstd);
#pragma unroll
  for (int k = 0; k < kPieceE; k++) r.v[k] = __builtin_fmaf((r.v[k] - mean) * rstd, g.v[k], b.v[k]);
  r.store(out + (int64_t)row * ncols + c0, left);
}

// A few very long rows in ONE launch, like softmax_one_launch: a workgroup of 1024 threads holds a piece of
// 65536 columns in registers, leaves the piece's sum S_p and squared deviations Q_p about a_p = (float)(S_p / n_p),
// waits -- bounded -- until every piece of the launch has, folds its row's pieces as layernorm_piece_apply does
// and writes its share: one read and one write of the row.  The same conditions: every workgroup of the grid on
// the device at once, x and out apart (a workgroup that gives up waiting reads the row itself), one stream.
__device__ unsigned int g_layernorm_meet[2];

__global__ __launch_bounds__(kLongBlock) void layernorm_one_launch(const float* __restrict__ x,
                                                                   const float* __restrict__ gamma,
                                                                   const float* __restrict__ beta, float eps,
                                                                   float* __restrict__ out, int64_t ncols, uint32_t pieces,
                                                                   double* psum, double* pdev, uint32_t spins) {
  __shared__ double lsum[kLongBlock / kWave];
  __shared__ int met;
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const float* xr = x + (int64_t)row * ncols;
  const int64_t c0 = (int64_t)piece * kOnePiece;
  float v[kOneE];
  const uint32_t first = threadIdx.x * 4;
  const uint32_t left = (uint32_t)((ncols - c0 < kOnePiece ? ncols - c0 : kOnePiece));
  const float* xp = xr + c0;
#pragma unroll
  for (int g = 0; g < kOneE / 4; g++) {
    f4 t = {0.f, 0.f, 0.f, 0.f};
    if (first + g * 4 * kLongBlock < left) t = __builtin_nontemporal_load(reinterpret_cast<const f4*>(xp + first + g * 4 * kLongBlock));
    v[4 * g] = t.x; v[4 * g + 1] = t.y; v[4 * g + 2] = t.z; v[4 * g + 3] = t.w;
  }
  double sum = 0.0;
#pragma unroll
  for (int k = 0; k < kOneE; k++) sum += (double)v[k];
  const double total = long_block_sum(sum, lsum);
  const float a = (float)(total / (double)left);
  float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int g = 0; g < kOneE / 4; g++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const float d = first + g * 4 * kLongBlock < left ? v[4 * g + c] - a : 0.0f;
      sq[c] = __builtin_fmaf(d, d, sq[c]);
    }
  const double dev = long_block_sum(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3]), lsum);
  if (threadIdx.x == 0) {
    // statistics past the caches, waited for, then the arrival (see softmax_one_launch)
    __hip_atomic_store(&psum[blockIdx.x], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&pdev[blockIdx.x], dev, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __hip_atomic_fetch_add(&g_layernorm_meet[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t polls = 0;
    while (__hip_atomic_load(&g_layernorm_meet[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gridDim.x && polls < spins) {
      __builtin_amdgcn_s_sleep(8);
      polls++;
    }
    met = __hip_atomic_load(&g_layernorm_meet[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= gridDim.x;
  }
  __syncthreads();
  double mean, var;
  if (met) {
    const double* rs = psum + (int64_t)row * pieces;
    const double* rq = pdev + (int64_t)row * pieces;
    double s = 0.0;
    for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock)
      s += __hip_atomic_load(&rs[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    mean = long_block_sum(s, lsum) / (double)ncols;
    double q = 0.0;
    for (uint32_t i = threadIdx.x; i < pieces; i += kLongBlock) {
      const int64_t l = ncols - (int64_t)i * kOnePiece;
      const double n = (double)(l < kOnePiece ? l : kOnePiece);
      const double mu = __hip_atomic_load(&rs[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) / n;
      const double ap = (double)(float)mu;
      q += __hip_atomic_load(&rq[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + n * ((mu - mean) * (mu - mean) - (mu - ap) * (mu - ap));
    }
    var = long_block_sum(q, lsum) / (double)ncols;
  } else {
    // gave up waiting: the row's statistics from the row itself (x is not written by this launch)
    double s = 0.0;
    for (int64_t c = threadIdx.x; c < ncols; c += kLongBlock) s += (double)xr[c];
    mean = long_block_sum(s, lsum) / (double)ncols;
    double q = 0.0;
    for (int64_t c = threadIdx.x; c < ncols; c += kLongBlock) {
      const double d = (double)xr[c] - mean;
      q += d * d;
    }
    var = long_block_sum(q, lsum) / (double)ncols;
  }
  const float meanf = (float)mean;
  const float rstd = (float)(1.0 / __builtin_sqrt((var > 0.0 ? var : 0.0) + (double)eps));
  float* op = out + (int64_t)row * ncols + c0;
#pragma unroll
  for (int g = 0; g < kOneE / 4; g++) {
    const uint32_t at = first + g * 4 * kLongBlock;
    if (at < left) {
      const f4 gm = *reinterpret_cast<const f4*>(gamma + c0 + at);
      const f4 bt = *reinterpret_cast<const f4*>(beta + c0 + at);
      f4 t;
#pragma unroll
      for (int c = 0; c < 4; c++) t[c] = __builtin_fmaf((v[4 * g + c] - meanf) * rstd, gm[c], bt[c]);
      __builtin_nontemporal_store(t, reinterpret_cast<f4*>(op + at));
    }
  }
  if (threadIdx.x == 0) {
    const unsigned int before = __hip_atomic_fetch_add(&g_layernorm_meet[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before + 1 == gridDim.x) {  // everyone has arrived and is past the wait: zero for the next launch
      __hip_atomic_store(&g_layernorm_meet[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&g_layernorm_meet[1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// Rows of 2049 ... 8192 columns that are a multiple of 4: a workgroup per row with the row in
// registers (thread t holds the NG 16-byte vectors (g 256 + t) 4 ...), one read and one write
// where the three-pass form above reads the row three times ((8192, 4096): 82 us).  The
// arithmetic of the wavefront form: the mean from binary64 sums, deviations, squares and the
// output in binary32; the statistics meet in LDS.
template <int NG, bool NT>
__global__ __launch_bounds__(kBlock) void layernorm_rows_wide(const float* __restrict__ x,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta, float eps,
                                                              float* __restrict__ out, int64_t ncols) {
  __shared__ double red[2][kWavesPerBlock];
  const int wave = threadIdx.x / kWave;
  const int64_t base = (int64_t)blockIdx.x * ncols;
  bool in[NG];
  f4 r[NG];
#pragma unroll
  for (int i = 0; i < NG; i++) {
    const int64_t c = ((int64_t)i * kBlock + threadIdx.x) * 4;
    in[i] = c < ncols;  // a vector is wholly inside or outside
    r[i] = f4{0.f, 0.f, 0.f, 0.f};
    if (in[i]) {
      const f4* p = reinterpret_cast<const f4*>(x + base + c);
      r[i] = NT ? __builtin_nontemporal_load(p) : *p;
    }
  }
  double sum = 0.0;
#pragma unroll
  for (int i = 0; i < NG; i++)
#pragma unroll
    for (int c = 0; c < 4; c++) sum += (double)r[i][c];
  sum = wave_sum(sum);
  if ((threadIdx.x & (kWave - 1)) == 0) red[0][wave] = sum;
  __syncthreads();
  const float meanf = (float)(((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) / (double)ncols);
  float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < NG; i++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const float d = in[i] ? r[i][c] - meanf : 0.0f;
      r[i][c] = d;
      sq[c] = __builtin_fmaf(d, d, sq[c]);
    }
  const double part = wave_sum(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3]));
  if ((threadIdx.x & (kWave - 1)) == 0) red[1][wave] = part;
  __syncthreads();
  const double var = ((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) / (double)ncols;
  const float rstd = (float)(1.0 / __builtin_sqrt(var + (double)eps));
#pragma unroll
  for (int i = 0; i < NG; i++) {
    if (!in[i]) continue;
    const int64_t c = ((int64_t)i * kBlock + threadIdx.x) * 4;
    const f4 g = *reinterpret_cast<const f4*>(gamma + c);
    const f4 b = *reinterpret_cast<const f4*>(beta + c);
    f4 o;
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = __builtin_fmaf(r[i][k] * rstd, g[k], b[k]);
    f4* q = reinterpret_cast<f4*>(out + base + c);
    if (NT)
      __builtin_nontemporal_store(o, q);
    else
      *q = o;
  }
}

template <bool VEC, bool NT, bool XENT>
static int launch_softmax_wave(int nv, uint32_t blocks, const float* x, int64_t ldx, float* out,
                               int64_t ldo, int64_t nrows, int64_t ncols, int64_t causal_seq,
                               float scale, Xent xe) {
  hipStream_t st = rt().stream;
#define WF2_SOFTMAX_CASE(N)                                                                            \
  case N:                                                                                              \
    softmax_rows_wave<N, VEC, NT, 1, XENT><<<blocks, kBlock, 0, st>>>(x, ldx, out, ldo, nrows, ncols,   \
                                                                      causal_seq, scale, xe);          \
    break;
  if (nv == 4) {
    softmax_rows_pair<VEC, NT, XENT><<<(uint32_t)ceil_div(nrows, 2), kBlock, 0, st>>>(
        x, ldx, out, ldo, nrows, ncols, causal_seq, scale, xe);
    return after_launch("softmax_rows_pair");
  }
  switch (nv) {
    case 1:
      softmax_rows_wave<1, VEC, NT, 4, XENT><<<(uint32_t)ceil_div(nrows, kWavesPerBlock * 4), kBlock, 0, st>>>(
          x, ldx, out, ldo, nrows, ncols, causal_seq, scale, xe);
      break;
    case 2:
      softmax_rows_wave<2, VEC, NT, 2, XENT><<<(uint32_t)ceil_div(nrows, kWavesPerBlock * 2), kBlock, 0, st>>>(
          x, ldx, out, ldo, nrows, ncols, causal_seq, scale, xe);
      break;
    WF2_SOFTMAX_CASE(3)
    WF2_SOFTMAX_CASE(4)
    WF2_SOFTMAX_CASE(5)
    WF2_SOFTMAX_CASE(6)
    WF2_SOFTMAX_CASE(7)
    WF2_SOFTMAX_CASE(8)
    WF2_SOFTMAX_CASE(12)
    WF2_SOFTMAX_CASE(16)
    default: return fail(WF2HIP_EINVAL, "bad register tile");
  }
#undef WF2_SOFTMAX_CASE
  return after_launch("softmax_rows_wave");
}

// xe == nullptr: the plain softmax.  Otherwise the cross-entropy epilogue as well
// (no causal form; labels and loss are contiguous rows of ncols).
// ---- rows of at most 64 columns (class scores: softmax over 10 classes) -----------------------------
// A wavefront per row -- or per four rows -- leaves most lanes idle on such rows ((1677721, 10): softmax 361
// us, 11 % of what its bytes take).  Here a workgroup takes 256 adjacent rows (up to 1024 of a few columns, 128 beyond 32 columns): their storage, one contiguous
// run, is staged into LDS in storage order (row r at r * (ncols | 1): the odd pitch keeps the 64 rows of a
// wavefront on different banks), thread r works through row r there, and the run is written back in storage
// order.  Rows must be adjacent in x and in every output (pitch == ncols).
constexpr int kTinyCols = 64;
constexpr int kTinyFloats = 256 * 33;  // >= 128 * 65
// rows per workgroup: as many whole rounds of 256 rows (at most four) as the tile holds -- rows of two columns
// in groups of 256 are 2 KB of work per workgroup, and the launch rate bounds the kernel ((8388608, 2): 55 us)
__host__ __device__ static inline int tiny_fwd_rows_per_group(int ncols) {
  if (ncols > 32) return 128;
  if (ncols > 8) return 256;  // (1677721, 10): 26 us in groups of 256, 30 us in groups of 768
  const int rounds = 33 / (ncols | 1);
  return 256 * (rounds > 4 ? 4 : rounds);
}
enum { kTinySoftmax = 0, kTinyXent = 1, kTinyLayerNorm = 2 };

struct TinyRows {
  const float* x;
  float* out;
  const float* aux0;  // Xent: labels; LayerNorm: gamma
  const float* aux1;  // LayerNorm: beta
  float* loss;        // Xent
  float param;        // Xent: delta; LayerNorm: eps
  int64_t nrows;
  int ncols;
};

// VEC: x and every output are 16-byte aligned: the run is staged in 16-byte vectors (a group's run starts on
// a multiple of 16 bytes: 256 or 128 rows), the last partial vector of a ragged last group element by element.
template <int MODE, bool VEC>
__global__ __launch_bounds__(kBlock) void rows_tiny(TinyRows a, FastDiv by_c) {
  __shared__ float tile[kTinyFloats];
  const int ncols = a.ncols, pitch = ncols | 1, group = tiny_fwd_rows_per_group(ncols);
  const int64_t row0 = (int64_t)blockIdx.x * group;
  if (row0 >= a.nrows) return;  // a grid sized for other groups must not index past the rows
  const int rows_here = (int)(a.nrows - row0 < group ? a.nrows - row0 : group);
  const uint32_t cells = (uint32_t)rows_here * (uint32_t)ncols;
  const int64_t base = row0 * ncols;
  constexpr int U = 4;
  typedef float f4 __attribute__((ext_vector_type(4)));
  if constexpr (VEC) {
    const uint32_t whole = cells / 4;
    for (uint32_t q0 = threadIdx.x; q0 < whole; q0 += kBlock * U) {
      f4 v[U];
#pragma unroll
      for (int u = 0; u < U; u++)
        v[u] = q0 + u * kBlock < whole ? *reinterpret_cast<const f4*>(a.x + base + 4 * (int64_t)(q0 + u * kBlock))
                                       : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < U; u++)
        if (q0 + u * kBlock < whole) {
          uint32_t col;
          uint32_t row = fd_divmod(4 * (q0 + u * kBlock), by_c, &col);
#pragma unroll
          for (int c = 0; c < 4; c++) {
            tile[row * pitch + col] = v[u][c];
            if (++col == (uint32_t)ncols) {
              col = 0;
              row++;
            }
          }
        }
    }
    for (uint32_t e = 4 * whole + threadIdx.x; e < cells; e += kBlock) {
      uint32_t col;
      const uint32_t row = fd_divmod(e, by_c, &col);
      tile[row * pitch + col] = a.x[base + e];
    }
  } else {
    for (uint32_t e0 = threadIdx.x; e0 < cells; e0 += kBlock * U) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; u++) v[u] = e0 + u * kBlock < cells ? a.x[base + e0 + u * kBlock] : 0.0f;
#pragma unroll
      for (int u = 0; u < U; u++)
        if (e0 + u * kBlock < cells) {
          uint32_t col;
          const uint32_t row = fd_divmod(e0 + u * kBlock, by_c, &col);
          tile[row * pitch + col] = v[u];
        }
    }
  }
  __syncthreads();
  for (int mine = threadIdx.x; mine < rows_here; mine += kBlock) {
    float* r = tile + mine * pitch;
    if constexpr (MODE == kTinyLayerNorm) {
      // the statistics of layernorm_bwd_tiny, operation for operation, so that the backward's xh is the
      // forward's: the mean from a binary64 sum, deviations and their squares in binary32
      double sum = 0.0;
      for (int j = 0; j < ncols; j++) sum += (double)r[j];
      const float mean = (float)(sum / (double)ncols);
      float sq = 0.0f;
      for (int j = 0; j < ncols; j++) {
        const float d = r[j] - mean;
        r[j] = d;
        sq = __builtin_fmaf(d, d, sq);
      }
      const float rstd = (float)(1.0 / __builtin_sqrt((double)sq / (double)ncols + (double)a.param));
      for (int j = 0; j < ncols; j++) r[j] = __builtin_fmaf(r[j] * rstd, a.aux0[j], a.aux1[j]);
    } else {
      float m = -__builtin_inff();
      for (int j = 0; j < ncols; j++) m = fmaxf(m, r[j]);
      double total = 0.0;
      for (int j = 0; j < ncols; j++) {  // the exponential of softmax_rows_wave
        const float d = fmaxf(r[j] - m, -160.0f);
        const float t = d * 1.44269502f;
        float tl = __builtin_fmaf(d, 1.44269502f, -t);
        tl = __builtin_fmaf(d, 1.92596299e-8f, tl);
        const float e = __builtin_amdgcn_exp2f(t);
        const float ed = __builtin_fmaf(e, tl * 0.693147182f, e);
        r[j] = ed;
        total += (double)ed;
      }
      const float inv = (float)(1.0 / total);
      for (int j = 0; j < ncols; j++) r[j] *= inv;
    }
  }
  __syncthreads();
  auto finish = [&](uint32_t e, float z, float lab) {
    a.out[base + e] = z;
    if constexpr (MODE == kTinyXent) a.loss[base + e] = xent_term(lab, z, a.param);
  };
  if constexpr (VEC) {
    const uint32_t whole = cells / 4;
    for (uint32_t q = threadIdx.x; q < whole; q += kBlock) {
      f4 lab = {0.f, 0.f, 0.f, 0.f};
      if constexpr (MODE == kTinyXent) lab = *reinterpret_cast<const f4*>(a.aux0 + base + 4 * (int64_t)q);
      uint32_t col;
      uint32_t row = fd_divmod(4 * q, by_c, &col);
      f4 z, loss;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        z[c] = tile[row * pitch + col];
        if constexpr (MODE == kTinyXent) loss[c] = xent_term(lab[c], z[c], a.param);
        if (++col == (uint32_t)ncols) {
          col = 0;
          row++;
        }
      }
      *reinterpret_cast<f4*>(a.out + base + 4 * (int64_t)q) = z;
      if constexpr (MODE == kTinyXent) *reinterpret_cast<f4*>(a.loss + base + 4 * (int64_t)q) = loss;
    }
    for (uint32_t e = 4 * whole + threadIdx.x; e < cells; e += kBlock) {
      uint32_t col;
      const uint32_t row = fd_divmod(e, by_c, &col);
      finish(e, tile[row * pitch + col], MODE == kTinyXent ? a.aux0[base + e] : 0.0f);
    }
  } else {
    for (uint32_t e0 = threadIdx.x; e0 < cells; e0 += kBlock * U) {
      float lab[U];
#pragma unroll
      for (int u = 0; u < U; u++)
        lab[u] = (MODE == kTinyXent && e0 + u * kBlock < cells) ? a.aux0[base + e0 + u * kBlock] : 0.0f;
#pragma unroll
      for (int u = 0; u < U; u++)
        if (e0 + u * kBlock < cells) {
          uint32_t col;
          const uint32_t row = fd_divmod(e0 + u * kBlock, by_c, &col);
          finish(e0 + u * kBlock, tile[row * pitch + col], lab[u]);
        }
    }
  }
}

// at least this many rows: below it the wavefront forms already finish within a launch's floor
constexpr int64_t kTinyMinRows = 16384;

static int64_t layernorm_one_launch_capacity() {
  static const int64_t capacity = [] {
    int held = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&held, layernorm_one_launch, kLongBlock, 0) != hipSuccess) {
      (void)hipGetLastError();
      return (int64_t)0;
    }
    return (int64_t)held * rt().num_cus;
  }();
  return capacity;
}

// How many workgroups of softmax_one_launch the device holds at once (0: the form is not used).
static int64_t softmax_one_launch_capacity() {
  static const int64_t capacity = [] {
    int plain = 0, xent = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&plain, softmax_one_launch<false>, kLongBlock, 0) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&xent, softmax_one_launch<true>, kLongBlock, 0) != hipSuccess) {
      (void)hipGetLastError();
      return (int64_t)0;
    }
    return (int64_t)std::min(plain, xent) * rt().num_cus;
  }();
  return capacity;
}

template <bool XENT>
static int softmax_dispatch_as(int64_t nrows, int64_t ncols, const float* x, int64_t ldx, float* out,
                               int64_t ldo, int64_t causal_seq, float scale, Xent xe) {
  if (ncols <= kTinyCols && ldx == ncols && ldo == ncols && causal_seq == 0 && nrows >= kTinyMinRows &&
      ceil_div(nrows, 128) < ((int64_t)1 << 31)) {
    TinyRows a{x, out, xe.labels, nullptr, xe.loss, xe.delta, nrows, (int)ncols};
    const uint32_t groups = (uint32_t)ceil_div(nrows, tiny_fwd_rows_per_group((int)ncols));
    if (aligned16(x) && aligned16(out) && (!XENT || (aligned16(xe.labels) && aligned16(xe.loss))))
      rows_tiny<XENT ? kTinyXent : kTinySoftmax, true><<<groups, kBlock, 0, rt().stream>>>(a, make_fastdiv((uint32_t)ncols));
    else
      rows_tiny<XENT ? kTinyXent : kTinySoftmax, false><<<groups, kBlock, 0, rt().stream>>>(a, make_fastdiv((uint32_t)ncols));
    return after_launch("rows_tiny");
  }
  const int nv = pick_nv(ncols);
  if (nv == 0) {
    if (causal_seq > 0) return fail(WF2HIP_EUNSUPPORTED, "causal softmax rows longer than 4096");
    if (nrows >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows");
    hipStream_t st = rt().stream;
    const int64_t pieces = ceil_div(ncols, kSplitPiece);
    if (ncols > 64 * kLongBlock || (pieces >= 2 && nrows < rt().num_cus)) {
      if (nrows * pieces >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many row pieces for one launch");
      // one launch when every workgroup of it is on the device at once, and x and out are apart
      const int64_t big_pieces = ceil_div(ncols, kOnePiece);
      const float* x_end = x + (nrows - 1) * ldx + ncols;
      const float* out_end = out + (nrows - 1) * ldo + ncols;
      static const bool one_env = [] {
        const char* e = getenv("WF2HIP_SOFTMAX_ONE_LAUNCH");
        return !e || atoi(e) != 0;
      }();
      // testing knob, read at every call: with 0 polls every workgroup takes the path of one that gave up waiting
      const char* spins_env = getenv("WF2HIP_MEET_SPINS");
      const uint32_t meet_spins = spins_env ? (uint32_t)atol(spins_env) : kMeetSpins;
      const bool vec = aligned16(x) && aligned16(out) && ldx % 4 == 0 && ldo % 4 == 0 && ncols % 4 == 0;
      const bool xent_ok = !XENT || (aligned16(xe.labels) && aligned16(xe.loss));
      if (one_env && vec && xent_ok && nrows * big_pieces <= softmax_one_launch_capacity() && (x_end <= out || out_end <= x)) {
        void* stats = nullptr;
        WF2_TRY(wf2hip_malloc_uninitialized(&stats, (size_t)(nrows * big_pieces) * (sizeof(double) + sizeof(float))));
        double* psum = static_cast<double*>(stats);
        float* pmax = reinterpret_cast<float*>(psum + nrows * big_pieces);
        const uint32_t grid = (uint32_t)(nrows * big_pieces);
        softmax_one_launch<XENT><<<grid, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, (uint32_t)big_pieces, pmax, psum, meet_spins, xe);
        const int rc = after_launch("softmax_one_launch");
        (void)wf2hip_free(stats);  // stream order keeps it alive for the launch above
        return rc;
      }
      void* stats = nullptr;  // nrows x pieces sums (binary64), then as many maxima
      WF2_TRY(wf2hip_malloc_uninitialized(&stats, (size_t)(nrows * pieces) * (sizeof(double) + sizeof(float))));
      double* psum = static_cast<double*>(stats);
      float* pmax = reinterpret_cast<float*>(psum + nrows * pieces);
      const uint32_t grid = (uint32_t)(nrows * pieces);
      softmax_split_stats<<<grid, kLongBlock, 0, st>>>(x, ldx, ncols, (uint32_t)pieces, pmax, psum);
      int rc = after_launch("softmax_split_stats");
      if (rc == 0) {
        softmax_split_apply<XENT><<<grid, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, (uint32_t)pieces, pmax, psum, xe);
        rc = after_launch("softmax_split_apply");
      }
      (void)wf2hip_free(stats);  // stream order keeps it alive for the launches above
      return rc;
    }
    if (ncols <= 8 * kLongBlock)
      softmax_rows_long<2, XENT><<<(uint32_t)nrows, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, xe);
    else if (ncols <= 16 * kLongBlock)
      softmax_rows_long<4, XENT><<<(uint32_t)nrows, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, xe);
    else if (ncols <= 32 * kLongBlock)
      softmax_rows_long<8, XENT><<<(uint32_t)nrows, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, xe);
    else if (ncols <= 52 * kLongBlock)  // GPT-2's vocabulary of 50257 without the register spills of 64
      softmax_rows_long<13, XENT><<<(uint32_t)nrows, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, xe);
    else
      softmax_rows_long<16, XENT><<<(uint32_t)nrows, kLongBlock, 0, st>>>(x, ldx, out, ldo, ncols, xe);
    return after_launch("softmax_rows_long");
  }
  int64_t blocks = ceil_div(nrows, kWavesPerBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows");
  bool vec = aligned16(x) && aligned16(out) && ldx % 4 == 0 && ldo % 4 == 0;
  if (XENT) vec = vec && aligned16(xe.labels) && aligned16(xe.loss) && ncols % 4 == 0;
  const bool streaming = nrows * ncols * (XENT ? 16 : 8) >= ((int64_t)192 << 20);
  if (vec && streaming)
    return launch_softmax_wave<true, true, XENT>(nv, (uint32_t)blocks, x, ldx, out, ldo, nrows, ncols,
                                                 causal_seq, scale, xe);
  if (vec)
    return launch_softmax_wave<true, false, XENT>(nv, (uint32_t)blocks, x, ldx, out, ldo, nrows, ncols,
                                                  causal_seq, scale, xe);
  return launch_softmax_wave<false, false, XENT>(nv, (uint32_t)blocks, x, ldx, out, ldo, nrows, ncols,
                                                 causal_seq, scale, xe);
}

static int softmax_dispatch(int64_t nrows, int64_t ncols, const float* x, int64_t ldx, float* out,
                            int64_t ldo, int64_t causal_seq, float scale) {
  if (nrows < 0 || ncols < 0) return fail(WF2HIP_EINVAL, "negative extent");
  if (nrows == 0 || ncols == 0) return 0;
  if (!x || !out) return fail(WF2HIP_EINVAL, "null pointer");
  if (ldx < ncols || ldo < ncols) return fail(WF2HIP_EINVAL, "row pitch smaller than the row");
  return softmax_dispatch_as<false>(nrows, ncols, x, ldx, out, ldo, causal_seq, scale, Xent{nullptr, nullptr, 0.0f});
}

template <bool VEC, bool NT>
static int launch_layernorm_wave(int nv, uint32_t blocks, const float* x, const float* g,
                                 const float* b, float eps, float* out, int64_t nrows,
                                 int64_t ncols) {
  hipStream_t st = rt().stream;
#define WF2_LN_CASE(N)                                                                            \
  case N:                                                                                         \
    layernorm_rows_wave<N, VEC, NT><<<blocks, kBlock, 0, st>>>(x, g, b, eps, out, nrows, ncols);   \
    break;
  switch (nv) {
    case 1:
      layernorm_rows_wave<1, VEC, NT, 4><<<(uint32_t)ceil_div(nrows, kWavesPerBlock * 4), kBlock, 0, st>>>(
          x, g, b, eps, out, nrows, ncols);
      break;
    case 2:
      layernorm_rows_wave<2, VEC, NT, 2><<<(uint32_t)ceil_div(nrows, kWavesPerBlock * 2), kBlock, 0, st>>>(
          x, g, b, eps, out, nrows, ncols);
      break;
    WF2_LN_CASE(3)
    WF2_LN_CASE(4)
    WF2_LN_CASE(5)
    WF2_LN_CASE(6)
    WF2_LN_CASE(7)
    WF2_LN_CASE(8)
    default: return fail(WF2HIP_EUNSUPPORTED, "LayerNorm rows longer than 2048 are not supported");
  }
#undef WF2_LN_CASE
  return after_launch("layernorm_rows_wave");
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_smax(long n, const float* x, long incx, float* out) {
  WF2_TRY(require_init());
  return launch_maxmin<true>(n, x, incx, out);
}

WF2_API int wf2hip_smin(long n, const float* x, long incx, float* out) {
  WF2_TRY(require_init());
  return launch_maxmin<false>(n, x, incx, out);
}

namespace wf2 {
int binary_nd(int op, Space s, float* a, const float* b);  // elementwise.hip
}

WF2_API int wf2hip_reduce_add_rows_f32(long rows, long cols, const float* x, long ldx, float* out,
                                       long inco) {
  WF2_TRY(require_init());
  if (rows < 0 || cols < 0) return fail(WF2HIP_EINVAL, "negative extent");
  Space s;
  s.rank = 2;
  s.shape[0] = rows;
  s.shape[1] = cols;
  s.sa[0] = inco;
  s.sa[1] = 0;
  s.sb[0] = ldx;
  s.sb[1] = 1;
  s.off_a = s.off_b = 0;
  s.total = (int64_t)rows * cols;
  return binary_nd(WF2HIP_ADD, s, out, x);
}

// a <- (sum of b over the axes where a's stride is 0) / divisor, in one node.
WF2_API int wf2hip_sum_nd(const wf2hip_view2* v, float* a, const float* b, float divisor) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(load_space(v, &s));
  if (s.total == 0) return 0;
  if (!a || !b) return fail(WF2HIP_EINVAL, "null tensor pointer");
  if (!(divisor != 0.0f)) return fail(WF2HIP_EINVAL, "divisor must not be zero");
  normalise(&s);
  if (hazardous_overlap(s, a, b)) return fail(WF2HIP_EOVERLAP, "sum into a window that overlaps its source");
  if (!has_broadcast_axis(s, s.sa)) {
    // nothing is reduced (every reduced axis has extent 1, so the divisor of !mean is 1)
    if (divisor != 1.0f)
      return fail(WF2HIP_EUNSUPPORTED, "wf2hip_sum_nd with a divisor needs at least one reduced axis");
    return binary_nd(WF2HIP_MOVE, s, a, b);
  }
  return launch_accumulate_with(WF2HIP_ADD, s, a, b, reinterpret_cast<double*>(rt().partials), Commit{1, divisor});
}

// ---- row sums without any allocation ---------------------------------------------
// For callers that cannot allocate device memory (code under graph capture, tight
// serving loops, harnesses that forbid it): the partial sums of rows split over
// several workgroups live in a static device array instead of a buffer the library
// allocates.  Every device holds its own copy of the array at its own address, which
// wf2hip_init looks up once per device; host code only ever uses that address.
constexpr int64_t kStaticPartials = kPartialCapacity / 2;  // binary64 sums, 256 KiB
constexpr int kMaxDevices = 64;
static __device__ __align__(256) double scratch[kStaticPartials];
static double* g_scratch_ptr[kMaxDevices];

namespace wf2 {
// Called by wf2hip_init with `device` current.
int reduce_setup_device(int device) {
  if (device < 0 || device >= kMaxDevices)
    return fail(WF2HIP_EUNSUPPORTED, "device ordinal %d beyond the %d this library keeps state for", device,
                kMaxDevices);
  if (g_scratch_ptr[device]) return 0;
  double* ptr = nullptr;
  WF2_TRY(check_hip(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)"));
  if (!ptr) return fail(WF2HIP_EINVAL, "hipGetSymbolAddress(scratch) returned a null address");
  g_scratch_ptr[device] = ptr;
  return 0;
}
}  // namespace wf2

WF2_API int wf2hip_reduce_add_rows_f32_noalloc(long rows, long cols, const float* x, long ldx, float* out,
                                               long inco) {
  WF2_TRY(require_init());
  if (rows < 0 || cols < 0) return fail(WF2HIP_EINVAL, "negative extent");
  if ((int64_t)rows > WF2HIP_NOALLOC_MAX_ELEMENTS || (int64_t)cols > WF2HIP_NOALLOC_MAX_ELEMENTS ||
      (rows > 0 && (int64_t)cols > WF2HIP_NOALLOC_MAX_ELEMENTS / rows))
    return fail(WF2HIP_EUNSUPPORTED,
                "wf2hip_reduce_add_rows_f32_noalloc: %ld x %ld elements exceed the maximum of %lld this "
                "entry point accepts; use wf2hip_reduce_add_rows_f32",
                rows, cols, (long long)WF2HIP_NOALLOC_MAX_ELEMENTS);
  if (rows == 0 || cols == 0) return 0;
  if (!x || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  const int device = rt().device;
  double* partials = device >= 0 && device < kMaxDevices ? g_scratch_ptr[device] : nullptr;
  if (!partials) return fail(WF2HIP_ENOTINIT, "the static scratch of device %d was not set up by wf2hip_init", device);
  Space s;
  s.rank = 2;
  s.shape[0] = rows;
  s.shape[1] = cols;
  s.sa[0] = inco;
  s.sa[1] = 0;
  s.sb[0] = ldx;
  s.sb[1] = 1;
  s.off_a = s.off_b = 0;
  s.total = (int64_t)rows * cols;
  normalise(&s);
  if (hazardous_overlap(s, out, x))
    return fail(WF2HIP_EOVERLAP, "row sums into a window that overlaps the source");
  // cols == 1 leaves no reduced axis: a plain strided add, which uses no scratch
  if (!has_broadcast_axis(s, s.sa)) return binary_nd(WF2HIP_ADD, s, out, x);
  return launch_accumulate_with(WF2HIP_ADD, s, out, x, partials, Commit{0, 1.0f}, false);
}

WF2_API int wf2hip_softmax_rows_f32(long rows, long cols, const float* x, long ldx, float* out,
                                    long ldo) {
  WF2_TRY(require_init());
  return softmax_dispatch(rows, cols, x, ldx, out, ldo, 0, 1.0f);
}

WF2_API int wf2hip_softmax_cross_entropy_f32(long rows, long cols, const float* x, const float* labels, float delta,
                                             float* z, float* loss) {
  WF2_TRY(require_init());
  if (rows < 0 || cols < 0) return fail(WF2HIP_EINVAL, "negative extent");
  if (rows == 0 || cols == 0) return 0;
  if (!x || !labels || !z || !loss) return fail(WF2HIP_EINVAL, "null pointer");
  const int64_t n = (int64_t)rows * cols;
  auto meet = [n](const float* a, const float* b) { return a < b + n && b < a + n; };
  if (meet(z, x) || meet(z, labels) || meet(z, loss) || meet(loss, x) || meet(loss, labels))
    return fail(WF2HIP_EOVERLAP, "softmax cross entropy: z and loss must overlap neither the inputs nor each other");
  return softmax_dispatch_as<true>(rows, cols, x, cols, z, cols, 0, 1.0f, Xent{labels, loss, delta});
}

WF2_API int wf2hip_causal_softmax_f32(long batch, long seq, const float* x, float* out,
                                      float scale) {
  WF2_TRY(require_init());
  if (batch < 0 || seq < 0) return fail(WF2HIP_EINVAL, "negative extent");
  return softmax_dispatch((int64_t)batch * seq, seq, x, seq, out, seq, seq > 0 ? seq : 0, scale);
}

WF2_API int wf2hip_layernorm_rows_f32(long rows, long cols, const float* x, const float* gamma,
                                      const float* beta, float eps, float* out) {
  WF2_TRY(require_init());
  if (rows < 0 || cols < 0) return fail(WF2HIP_EINVAL, "negative extent");
  if (rows == 0 || cols == 0) return 0;
  if (!x || !gamma || !beta || !out) return fail(WF2HIP_EINVAL, "null pointer");
  if (cols <= kTinyCols && rows >= kTinyMinRows) {
    TinyRows a{x, out, gamma, beta, nullptr, eps, rows, (int)cols};
    const uint32_t groups = (uint32_t)ceil_div((int64_t)rows, tiny_fwd_rows_per_group((int)cols));
    if (aligned16(x) && aligned16(out))
      rows_tiny<kTinyLayerNorm, true><<<groups, kBlock, 0, rt().stream>>>(a, make_fastdiv((uint32_t)cols));
    else
      rows_tiny<kTinyLayerNorm, false><<<groups, kBlock, 0, rt().stream>>>(a, make_fastdiv((uint32_t)cols));
    return after_launch("rows_tiny");
  }
  int nv = pick_nv(cols);
  if (nv == 0 || nv > 8) {
    if (rows >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows");
    hipStream_t st = rt().stream;
    if (cols <= 8192 && cols % 4 == 0 && aligned16(x) && aligned16(out) && aligned16(gamma) && aligned16(beta)) {
      const bool nt = (int64_t)rows * cols * 8 >= ((int64_t)192 << 20);
      const int ng = (int)ceil_div(cols, (int64_t)kBlock * 4);
#define WF2_WIDE(NG_)                                                                                      \
  if (nt)                                                                                                  \
    layernorm_rows_wide<NG_, true><<<(uint32_t)rows, kBlock, 0, st>>>(x, gamma, beta, eps, out, cols);      \
  else                                                                                                     \
    layernorm_rows_wide<NG_, false><<<(uint32_t)rows, kBlock, 0, st>>>(x, gamma, beta, eps, out, cols);
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
      return after_launch("layernorm_rows_wide");
    }
    const bool aligned = cols % 4 == 0 && aligned16(x) && aligned16(out) && aligned16(gamma) && aligned16(beta);
    if (cols > 8192 && cols <= 64 * (int64_t)kPieceBlock && aligned && rows >= rt().num_cus) {
      const bool nt = (int64_t)rows * cols * 8 >= ((int64_t)192 << 20);
#define WF2_LONG(E_)                                                                                       \
  if (nt)                                                                                                  \
    layernorm_rows_long<E_, true><<<(uint32_t)rows, kPieceBlock, 0, st>>>(x, gamma, beta, eps, out, cols); \
  else                                                                                                     \
    layernorm_rows_long<E_, false><<<(uint32_t)rows, kPieceBlock, 0, st>>>(x, gamma, beta, eps, out, cols);
      if (cols <= 16 * (int64_t)kPieceBlock) {
        WF2_LONG(16)
      } else if (cols <= 32 * (int64_t)kPieceBlock) {
        WF2_LONG(32)
      } else if (cols <= 48 * (int64_t)kPieceBlock) {
        WF2_LONG(48)
      } else {
        WF2_LONG(64)
      }
#undef WF2_LONG
      return after_launch("layernorm_rows_long");
    }
    if (cols > 8192) {
      const int64_t pieces = ceil_div((int64_t)cols, kPieceCols);
      if (rows * pieces >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many row pieces for one launch");
      // one launch when every workgroup of it is on the device at once, and x and out are apart
      const int64_t big_pieces = ceil_div((int64_t)cols, kOnePiece);
      const float* x_end = x + (int64_t)rows * cols;
      const float* out_end = out + (int64_t)rows * cols;
      static const bool one_env = [] {
        const char* e = getenv("WF2HIP_LAYERNORM_ONE_LAUNCH");
        return !e || atoi(e) != 0;
      }();
      // (below 2^22 elements the meeting costs more than the second launch: (100, 20000) 15.7 against 12.8 us)
      if (one_env && aligned && (int64_t)rows * cols >= ((int64_t)1 << 22) && rows * big_pieces <= layernorm_one_launch_capacity() &&
          (x_end <= out || out_end <= x)) {
        const char* spins_env = getenv("WF2HIP_MEET_SPINS");  // testing knob, read at every call
        const uint32_t meet_spins = spins_env ? (uint32_t)atol(spins_env) : kMeetSpins;
        void* stats = nullptr;
        WF2_TRY(wf2hip_malloc_uninitialized(&stats, (size_t)(rows * big_pieces) * 2 * sizeof(double)));
        double* psum = static_cast<double*>(stats);
        double* pdev = psum + rows * big_pieces;
        layernorm_one_launch<<<(uint32_t)(rows * big_pieces), kLongBlock, 0, st>>>(x, gamma, beta, eps, out, cols,
                                                                                  (uint32_t)big_pieces, psum, pdev, meet_spins);
        const int rc = after_launch("layernorm_one_launch");
        (void)wf2hip_free(stats);  // stream order keeps it alive for the launch above
        return rc;
      }
      void* stats = nullptr;  // rows x pieces sums, then as many sums of squared deviations
      WF2_TRY(wf2hip_malloc_uninitialized(&stats, (size_t)(rows * pieces) * 2 * sizeof(double)));
      double* psum = static_cast<double*>(stats);
      double* pdev = psum + rows * pieces;
      const uint32_t grid = (uint32_t)(rows * pieces);
      const bool vec = aligned;
      if (vec)
        layernorm_piece_stats<true><<<grid, kPieceBlock, 0, st>>>(x, cols, (uint32_t)pieces, psum, pdev);
      else
        layernorm_piece_stats<false><<<grid, kPieceBlock, 0, st>>>(x, cols, (uint32_t)pieces, psum, pdev);
      int rc = after_launch("layernorm_piece_stats");
      if (rc == 0) {
        if (vec)
          layernorm_piece_apply<true><<<grid, kPieceBlock, 0, st>>>(x, gamma, beta, eps, out, cols, (uint32_t)pieces, psum, pdev);
        else
          layernorm_piece_apply<false><<<grid, kPieceBlock, 0, st>>>(x, gamma, beta, eps, out, cols, (uint32_t)pieces, psum, pdev);
        rc = after_launch("layernorm_piece_apply");
      }
      (void)wf2hip_free(stats);  // stream order keeps it alive for the launches above
      return rc;
    }
    layernorm_rows_block<<<(uint32_t)rows, kBlock, 0, st>>>(x, gamma, beta, eps, out, cols);
    return after_launch("layernorm_rows_block");
  }
  int64_t blocks = ceil_div(rows, kWavesPerBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows");
  const bool vec = aligned16(x) && aligned16(out) && aligned16(gamma) && aligned16(beta) &&
                   cols % 4 == 0;
  const bool streaming = (int64_t)rows * cols * 8 >= ((int64_t)192 << 20);
  if (vec && streaming)
    return launch_layernorm_wave<true, true>(nv, (uint32_t)blocks, x, gamma, beta, eps, out, rows, cols);
  if (vec)
    return launch_layernorm_wave<true, false>(nv, (uint32_t)blocks, x, gamma, beta, eps, out, rows, cols);
  return launch_layernorm_wave<false, false>(nv, (uint32_t)blocks, x, gamma, beta, eps, out, rows, cols);
}
