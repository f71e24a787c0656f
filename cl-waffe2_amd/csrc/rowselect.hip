// rowselect.hip -- largest / smallest value of a row and where it sits.
//
// MaxValue-Node, MinValue-Node, ArgMax-Node and ArgMin-Node
// (source/base-impl/matrix-ops.lisp:197-470) reduce the trailing run of A and
// write one element per row of OUT; the CPU backend calls waffe2_s{max,min} or
// BLAS i?max / i?min once per row
// (source/backends/cpu/matrix-ops.lisp:240-369).  Here a node is one launch: a
// wavefront per short row, a workgroup per long row, and (row, split)
// workgroups plus a small second pass when there are too few rows to fill the
// chip.  HBM-bound: 4 bytes per element.
//
// Ties go to the lowest index (the first occurrence, what a sequential scan
// with a strict comparison finds); NaN elements are never selected; a row of
// NaNs gives -inf / +inf and index 0.
#include <math.h>

#include "wf2_common.h"
#include "wf2_fastdiv.h"
#include "wf2_view.h"

namespace wf2 {

constexpr int kSelMaxOuter = WF2HIP_MAX_RANK;

template <class T>
struct Best {
  T v;
  uint32_t i;
};

// the value no element loses against: -inf / +inf, or the end of the integer range
template <class T, bool IsMax>
__device__ __forceinline__ T worst() {
  if constexpr (__is_floating_point(T)) {
    return IsMax ? (T)-INFINITY : (T)INFINITY;
  } else {
    constexpr bool is_signed = (T)(-1) < (T)0;
    constexpr T lo = is_signed ? (T)((T)1 << (sizeof(T) * 8 - 1)) : (T)0;
    return IsMax ? lo : (T)~lo;
  }
}

template <bool IsMax, class T>
__device__ __forceinline__ bool better(T v, uint32_t i, const Best<T>& b) {
  return IsMax ? (v > b.v || (v == b.v && i < b.i)) : (v < b.v || (v == b.v && i < b.i));
}

template <class T>
__device__ __forceinline__ T shuffle_xor(T v, int o) {
  if constexpr (sizeof(T) < 4)
    return (T)__shfl_xor((int)v, o);
  else
    return __shfl_xor(v, o);
}

template <bool IsMax, class T>
__device__ __forceinline__ Best<T> wave_best(Best<T> b) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const T ov = shuffle_xor(b.v, o);
    const uint32_t oi = __shfl_xor(b.i, o);
    if (better<IsMax>(ov, oi, b)) {
      b.v = ov;
      b.i = oi;
    }
  }
  return b;
}

template <class T>
struct SelParams {
  const T* x;
  void* out;        // T for value ops, uint32_t for index ops
  int64_t n, incx;  // the reduced run
  uint32_t nrows;
  int32_t nouter;
  uint32_t oshape[kSelMaxOuter];  // kept axes, innermost of them first
  int64_t ox[kSelMaxOuter], oo[kSelMaxOuter];
  int32_t want_index;
  uint32_t splits;  // workgroups per row
  int64_t seg;      // elements per split (multiple of the 16-byte vector)
  Best<T>* partials;  // nrows * splits
};

template <class T>
__device__ __forceinline__ void sel_offsets(const SelParams<T>& p, uint32_t row, int64_t* xoff, int64_t* ooff) {
  int64_t xo = 0, oo = 0;
  uint32_t rem = row;
  for (int i = 0; i < p.nouter; i++) {
    uint32_t idx;
    if (i == p.nouter - 1) {
      idx = rem;
    } else {
      const uint32_t q = rem / p.oshape[i];
      idx = rem - q * p.oshape[i];
      rem = q;
    }
    xo += (int64_t)idx * p.ox[i];
    oo += (int64_t)idx * p.oo[i];
  }
  *xoff = xo;
  *ooff = oo;
}

// best of x[lo, hi) seen by thread `t` of `nthreads`; a lane scans increasing
// indices with a strict comparison, so it keeps the first occurrence
template <bool IsMax, bool VEC, class T>
__device__ __forceinline__ Best<T> scan(const T* __restrict__ x, int64_t incx, int64_t lo, int64_t hi, int t,
                                        int nthreads) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  constexpr int N = 16 / (int)sizeof(T);
  struct alignas(16) Pack { T v[N]; };
  Best<T> b = {worst<T, IsMax>(), 0u};
  if (VEC) {  // incx == 1, x + lo 16-byte aligned
    const int64_t nvec = (hi - lo) / N;
    const f4* xv = reinterpret_cast<const f4*>(x + lo);
    auto take = [&](const f4& raw, uint32_t at) {
      const Pack v = __builtin_bit_cast(Pack, raw);
#pragma unroll
      for (int k = 0; k < N; k++)
        if (IsMax ? v.v[k] > b.v : v.v[k] < b.v) { b.v = v.v[k]; b.i = at + k; }
    };
    int64_t i = t;
    for (; i + nthreads < nvec; i += 2 * (int64_t)nthreads) {  // two loads in flight
      const f4 v0 = __builtin_nontemporal_load(xv + i);
      const f4 v1 = __builtin_nontemporal_load(xv + i + nthreads);
      take(v0, (uint32_t)(lo + N * i));
      take(v1, (uint32_t)(lo + N * (i + nthreads)));
    }
    if (i < nvec) take(__builtin_nontemporal_load(xv + i), (uint32_t)(lo + N * i));
    for (int64_t c = lo + nvec * N + t; c < hi; c += nthreads) {
      const T v = x[c];
      if (IsMax ? v > b.v : v < b.v) { b.v = v; b.i = (uint32_t)c; }
    }
  } else {
    for (int64_t c = lo + t; c < hi; c += nthreads) {
      const T v = x[c * incx];
      if (IsMax ? v > b.v : v < b.v) { b.v = v; b.i = (uint32_t)c; }
    }
  }
  return b;
}

template <class T>
__device__ __forceinline__ void emit(const SelParams<T>& p, int64_t ooff, const Best<T>& b) {
  if (p.want_index)
    static_cast<uint32_t*>(p.out)[ooff] = b.i;
  else
    static_cast<T*>(p.out)[ooff] = b.v;
}

// one wavefront per row, four rows per workgroup
template <bool IsMax, bool VEC, class T>
__global__ __launch_bounds__(kBlock) void select_rows_wave(SelParams<T> p) {
  const uint32_t row = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= p.nrows) return;
  int64_t xoff, ooff;
  sel_offsets(p, row, &xoff, &ooff);
  Best<T> b = scan<IsMax, VEC>(p.x + xoff, p.incx, 0, p.n, threadIdx.x & (kWave - 1), kWave);
  b = wave_best<IsMax>(b);
  if ((threadIdx.x & (kWave - 1)) == 0) emit(p, ooff, b);
}

// four short rows (at most one 16-byte vector per lane) per wavefront: their loads are
// issued together; a wavefront with one row of 256 floats has 1 KB in flight
// ((262144, 256): 46 % of the HBM peak)
template <bool IsMax, bool VEC, class T>
__global__ __launch_bounds__(kBlock) void select_rows_wave4(SelParams<T> p) {
  constexpr int RW = 4;
  const uint32_t row0 = (blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * RW;
  if (row0 >= p.nrows) return;
  const int lane = threadIdx.x & (kWave - 1);
  Best<T> b[RW];
  int64_t ooff[RW];
#pragma unroll
  for (int w = 0; w < RW; w++) {
    const uint32_t row = row0 + w < p.nrows ? row0 + w : p.nrows - 1;
    int64_t xoff;
    sel_offsets(p, row, &xoff, &ooff[w]);
    b[w] = scan<IsMax, VEC>(p.x + xoff, p.incx, 0, p.n, lane, kWave);
  }
#pragma unroll
  for (int w = 0; w < RW; w++) {
    b[w] = wave_best<IsMax>(b[w]);
    if (lane == 0 && row0 + w < p.nrows) emit(p, ooff[w], b[w]);
  }
}

// Rows of a few elements (pooling windows: MaxPool2D takes the maximum of rows of k-h k-w
// elements, source/nn/pool.lisp:83-93), adjacent in memory: a thread per row.  The workgroup's
// 256 rows are one contiguous run, read by consecutive lanes into LDS (rows padded to an odd
// pitch) and scanned from there; a wavefront per four rows left (6422528, 4) at 970 us.
constexpr int kTinyRowBytes = 128;  // rows up to 32 four-byte elements

template <bool IsMax, class T>
__global__ __launch_bounds__(kBlock) void select_rows_tiny(SelParams<T> p, FastDiv by_n) {
  extern __shared__ __align__(16) unsigned char tiny_lds[];
  T* tile = reinterpret_cast<T*>(tiny_lds);
  const uint32_t n = (uint32_t)p.n, pitch = n | 1u;
  const uint32_t row0 = blockIdx.x * kBlock;
  const uint32_t rows_here = p.nrows - row0 < (uint32_t)kBlock ? p.nrows - row0 : (uint32_t)kBlock;
  const uint32_t count = rows_here * n;
  const T* src = p.x + (int64_t)row0 * n;
  auto place = [&](uint32_t e) { const uint32_t r = fd_div(e, by_n); return r * pitch + (e - r * n); };
  if (((uintptr_t)src & 15u) == 0) {
    // the run in 16-byte vectors (a workgroup's run of 256 rows starts on a multiple of 16 bytes), four in
    // flight per thread; the elements of a vector are placed one by one
    constexpr int N = 16 / (int)sizeof(T);
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    union Vec {
      u4 q;
      T v[N];
    };
    const u4* vsrc = reinterpret_cast<const u4*>(src);
    const uint32_t whole = count / N;
    for (uint32_t q0 = threadIdx.x; q0 < whole; q0 += 4 * kBlock) {
      Vec v[4];
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (q0 + u * kBlock < whole) v[u].q = vsrc[q0 + u * kBlock];
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (q0 + u * kBlock < whole) {
          uint32_t r = fd_div((q0 + u * kBlock) * N, by_n), c = (q0 + u * kBlock) * N - r * n;
#pragma unroll
          for (int i = 0; i < N; i++) {
            tile[r * pitch + c] = v[u].v[i];
            if (++c == n) {
              c = 0;
              r++;
            }
          }
        }
    }
    for (uint32_t e = whole * N + threadIdx.x; e < count; e += kBlock) tile[place(e)] = src[e];
  } else {
    uint32_t e = threadIdx.x;
    for (; e + 7 * kBlock < count; e += 8 * kBlock) {  // eight loads in flight per thread
      T v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = src[e + u * kBlock];
#pragma unroll
      for (int u = 0; u < 8; u++) tile[place(e + u * kBlock)] = v[u];
    }
    for (; e < count; e += kBlock) tile[place(e)] = src[e];
  }
  __syncthreads();
  if (threadIdx.x >= rows_here) return;
  Best<T> b = {worst<T, IsMax>(), 0u};
  const T* row = tile + threadIdx.x * pitch;
  for (uint32_t c = 0; c < n; c++) {  // increasing indices, strict comparison: the first occurrence stays
    const T v = row[c];
    if (IsMax ? v > b.v : v < b.v) { b.v = v; b.i = c; }
  }
  emit(p, (int64_t)(row0 + threadIdx.x) * p.oo[0], b);
}

// Rows of exactly 16 bytes (2 x 2 pooling windows of :float), 16-byte aligned: the row is one vector load,
// four rows per thread in flight, no LDS ((6422528, 4) :float inside a replayed graph: 19 us, half the time
// of select_rows_tiny).
template <bool IsMax, class T>
__global__ __launch_bounds__(kBlock) void select_rows_vec16(SelParams<T> p) {
  constexpr int N = 16 / (int)sizeof(T);
  constexpr int U = 4;
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  union Row {
    u4 q;
    T v[N];
  };
  const u4* src = reinterpret_cast<const u4*>(p.x);
  const uint32_t first = blockIdx.x * (kBlock * U) + threadIdx.x;
  Row r[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t row = first + u * kBlock;
    if (row < p.nrows) r[u].q = src[row];
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t row = first + u * kBlock;
    if (row >= p.nrows) continue;
    Best<T> b = {worst<T, IsMax>(), 0u};
#pragma unroll
    for (int c = 0; c < N; c++) {  // increasing indices, strict comparison: the first occurrence stays
      const T v = r[u].v[c];
      if (IsMax ? v > b.v : v < b.v) { b.v = v; b.i = (uint32_t)c; }
    }
    emit(p, (int64_t)row * p.oo[0], b);
  }
}

// one workgroup per (row, split)
template <bool IsMax, bool VEC, class T>
__global__ __launch_bounds__(kBlock) void select_rows_block(SelParams<T> p) {
  __shared__ Best<T> lds[kBlock / kWave];
  const uint32_t row = blockIdx.x / p.splits;
  const uint32_t split = blockIdx.x - row * p.splits;
  int64_t xoff, ooff;
  sel_offsets(p, row, &xoff, &ooff);
  const int64_t lo = (int64_t)split * p.seg;
  const int64_t hi = lo + p.seg < p.n ? lo + p.seg : p.n;
  Best<T> b = scan<IsMax, VEC>(p.x + xoff, p.incx, lo, hi, threadIdx.x, kBlock);
  b = wave_best<IsMax>(b);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = b;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kBlock / kWave; w++)
      if (better<IsMax>(lds[w].v, lds[w].i, b)) b = lds[w];
    if (p.splits == 1)
      emit(p, ooff, b);
    else
      p.partials[(int64_t)row * p.splits + split] = b;
  }
}

template <bool IsMax, class T>
__global__ __launch_bounds__(kBlock) void select_rows_finish(SelParams<T> p) {
  __shared__ Best<T> lds[kBlock / kWave];
  const uint32_t row = blockIdx.x;
  int64_t xoff, ooff;
  sel_offsets(p, row, &xoff, &ooff);
  Best<T> b = {worst<T, IsMax>(), 0u};
  for (uint32_t s = threadIdx.x; s < p.splits; s += kBlock) {
    const Best<T> c = p.partials[(int64_t)row * p.splits + s];
    if (better<IsMax>(c.v, c.i, b)) b = c;
  }
  b = wave_best<IsMax>(b);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = b;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kBlock / kWave; w++)
      if (better<IsMax>(lds[w].v, lds[w].i, b)) b = lds[w];
    emit(p, ooff, b);
  }
}

template <bool IsMax, bool VEC, class T>
static int launch_select(SelParams<T>& p) {
  hipStream_t st = rt().stream;
  const int64_t target = (int64_t)rt().num_cus * 8;
  if (p.n * (int64_t)sizeof(T) <= kTinyRowBytes && p.incx == 1 && p.nouter == 1 && p.ox[0] == p.n &&
      p.nrows >= 4 * target) {
    if (p.n * (int64_t)sizeof(T) == 16 && ((uintptr_t)p.x & 15u) == 0) {
      select_rows_vec16<IsMax, T><<<(uint32_t)ceil_div(p.nrows, kBlock * 4), kBlock, 0, st>>>(p);
      return after_launch("select_rows_vec16");
    }
    const uint32_t blocks = (uint32_t)ceil_div(p.nrows, kBlock);
    const size_t bytes = (size_t)kBlock * ((size_t)p.n | 1u) * sizeof(T);
    select_rows_tiny<IsMax, T><<<blocks, kBlock, bytes, st>>>(p, make_fastdiv((uint32_t)p.n));
    return after_launch("select_rows_tiny");
  }
  if (p.n <= (int64_t)kWave * (16 / (int64_t)sizeof(T)) && p.nrows >= 4 * target) {
    const uint32_t blocks = (uint32_t)ceil_div(p.nrows, (kBlock / kWave) * 4);
    select_rows_wave4<IsMax, VEC, T><<<blocks, kBlock, 0, st>>>(p);
    return after_launch("select_rows_wave4");
  }
  if (p.n <= 2048 || (p.n < 8192 && p.nrows >= target)) {
    const uint32_t blocks = (uint32_t)ceil_div(p.nrows, kBlock / kWave);
    select_rows_wave<IsMax, VEC, T><<<blocks, kBlock, 0, st>>>(p);
    return after_launch("select_rows_wave");
  }
  p.splits = 1;
  p.seg = p.n;
  if (p.nrows < target) {
    int64_t by_work = ceil_div(p.n, 16384);
    int64_t by_fill = ceil_div(target, p.nrows);
    int64_t by_cap = (int64_t)(kPartialCapacity * sizeof(float) / sizeof(Best<T>)) / p.nrows;
    int64_t splits = by_work < by_fill ? by_work : by_fill;
    if (splits > by_cap) splits = by_cap;
    if (splits < 1) splits = 1;
    const int64_t seg = ceil_div(ceil_div(p.n, splits), 1024) * 1024;
    p.splits = (uint32_t)ceil_div(p.n, seg);
    p.seg = seg;
  }
  const int64_t blocks = (int64_t)p.nrows * p.splits;
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows for one launch");
  select_rows_block<IsMax, VEC, T><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  WF2_TRY(after_launch("select_rows_block"));
  if (p.splits > 1) {
    select_rows_finish<IsMax, T><<<p.nrows, kBlock, 0, st>>>(p);
    WF2_TRY(after_launch("select_rows_finish"));
  }
  return 0;
}

template <class T>
static int select_nd(int op, const wf2hip_view2* outer, long n, long incx, const T* x, void* out) {
  WF2_TRY(require_init());
  if (op < WF2HIP_MAXVALUE || op > WF2HIP_ARGMIN) return fail(WF2HIP_EINVAL, "unknown selection op %d", op);
  Space s;
  WF2_TRY(load_space(outer, &s));
  if (n < 0) return fail(WF2HIP_EINVAL, "negative run length");
  if (s.total == 0) return 0;
  if (n == 0) return fail(WF2HIP_EINVAL, "cannot select from an empty run");
  if (!x || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  if (n >= ((int64_t)1 << 32)) return fail(WF2HIP_EUNSUPPORTED, "run longer than 2^32 - 1 elements");
  if (s.total >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many rows");
  // a stride-0 axis of OUT keeps what the sequential loop writes last
  for (int r = 0; r < s.rank; r++)
    if (s.sb[r] == 0 && s.shape[r] > 1) {
      s.off_a += s.sa[r] * (s.shape[r] - 1);
      s.shape[r] = 1;
    }
  normalise(&s);
  SelParams<T> p;
  p.want_index = op == WF2HIP_ARGMAX || op == WF2HIP_ARGMIN;
  p.x = x + s.off_a;
  p.out = static_cast<char*>(out) + (p.want_index ? 4 : (int64_t)sizeof(T)) * s.off_b;
  p.n = n;
  p.incx = incx;
  p.nouter = s.rank;
  int64_t nrows = 1;
  constexpr int64_t N = 16 / (int64_t)sizeof(T);
  bool vec = incx == 1 && ((uintptr_t)p.x & 15u) == 0;
  for (int i = 0; i < s.rank; i++) {
    const int r = s.rank - 1 - i;
    if (s.shape[r] >= ((int64_t)1 << 32)) return fail(WF2HIP_EUNSUPPORTED, "axis too long");
    p.oshape[i] = (uint32_t)s.shape[r];
    p.ox[i] = s.sa[r];
    p.oo[i] = s.sb[r];
    nrows *= s.shape[r];
    if (s.shape[r] > 1 && s.sa[r] % N != 0) vec = false;
  }
  p.nrows = (uint32_t)nrows;
  p.splits = 1;
  p.seg = n;
  p.partials = reinterpret_cast<Best<T>*>(rt().partials);
  const bool is_max = op == WF2HIP_MAXVALUE || op == WF2HIP_ARGMAX;
  if (is_max) return vec ? launch_select<true, true>(p) : launch_select<true, false>(p);
  return vec ? launch_select<false, true>(p) : launch_select<false, false>(p);
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_select_nd(int op, const wf2hip_view2* outer, long n, long incx, const float* x, void* out) {
  return select_nd<float>(op, outer, n, incx, x, out);
}

// MaxValue-Node / MinValue-Node on every dtype (the CPU backend calls
// waffe2_<prefix>{max,min} per row, backends/cpu/matrix-ops.lisp:336-369), ArgMax-Node /
// ArgMin-Node on :double (BLAS idmax / idmin, :240-283; other dtypes are an error there too)
WF2_API int wf2hip_select_nd_typed(int dtype, int op, const wf2hip_view2* outer, long n, long incx, const void* x,
                                   void* out) {
  const bool index = op == WF2HIP_ARGMAX || op == WF2HIP_ARGMIN;
  if (index && dtype != WF2HIP_F64)
    return fail(WF2HIP_EUNSUPPORTED, "argmax / argmin support :float and :double only");
  switch (dtype) {
    case WF2HIP_F64: return select_nd<double>(op, outer, n, incx, (const double*)x, out);
    case WF2HIP_I32: return select_nd<int32_t>(op, outer, n, incx, (const int32_t*)x, out);
    case WF2HIP_U32: return select_nd<uint32_t>(op, outer, n, incx, (const uint32_t*)x, out);
    case WF2HIP_I16: return select_nd<int16_t>(op, outer, n, incx, (const int16_t*)x, out);
    case WF2HIP_U16: return select_nd<uint16_t>(op, outer, n, incx, (const uint16_t*)x, out);
    case WF2HIP_I8: return select_nd<int8_t>(op, outer, n, incx, (const int8_t*)x, out);
    case WF2HIP_U8: return select_nd<uint8_t>(op, outer, n, incx, (const uint8_t*)x, out);
    default: return fail(WF2HIP_EINVAL, "unknown element type %d (:float has its own entry point)", dtype);
  }
}

// waffe2_<prefix>{max,min}(n, x, incx, y): y[0] <- the extreme of the run (cl-waffe2-simd.c:316-365)
#define WF2_DEFINE_TYPED_EXTREME(prefix, T)                                                    \
  WF2_API int wf2hip_##prefix##max(long n, const T* x, long incx, T* out) {                  \
    wf2hip_view2 one = {};                                                                    \
    one.rank = 1;                                                                             \
    one.shape[0] = 1;                                                                         \
    return select_nd<T>(WF2HIP_MAXVALUE, &one, n, incx, x, out);                              \
  }                                                                                           \
  WF2_API int wf2hip_##prefix##min(long n, const T* x, long incx, T* out) {                  \
    wf2hip_view2 one = {};                                                                    \
    one.rank = 1;                                                                             \
    one.shape[0] = 1;                                                                         \
    return select_nd<T>(WF2HIP_MINVALUE, &one, n, incx, x, out);                              \
  }
WF2_DEFINE_TYPED_EXTREME(d, double)
WF2_DEFINE_TYPED_EXTREME(i32, int32_t)
WF2_DEFINE_TYPED_EXTREME(u32, uint32_t)
WF2_DEFINE_TYPED_EXTREME(i16, int16_t)
WF2_DEFINE_TYPED_EXTREME(u16, uint16_t)
WF2_DEFINE_TYPED_EXTREME(i8, int8_t)
WF2_DEFINE_TYPED_EXTREME(u8, uint8_t)
