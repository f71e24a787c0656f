// typed.hip -- the element types of cl-waffe2 other than :float -- :double, :int32,
// :uint32, :int16, :uint16, :int8, :uint8: AddNode / SubNode / MulNode / DivNode /
// MoveTensorNode and inv (below), accumulation into broadcast destinations (!sum),
// Compare- / Where-Operation-Node, and unary math on :double, each introduced by its
// own section comment.  MaxValue / MinValue / ArgMax / ArgMin live in rowselect.hip.
//
// Reference: waffe2_d{add,sub,mul,div} (the AVX2 macro of
// cl-waffe2-simd.c:153-213 instantiated at :247-250), the scalar loops
// waffe2_{i32,i16,i8,u32,u16,u8}{add,sub,mul,div,copy} (:214-288), dcopy_ from
// BLAS for :double moves (source/backends/cpu/arithmetic.lisp:39-61) and
// waffe2_{d,i32,...}inv (:290-310).
//
// Integer semantics are C's: int8 / int16 operands are promoted to int and the
// result is truncated on the store, unsigned types wrap, signed division
// truncates toward zero.  The reference traps (SIGFPE) on a zero divisor and on
// INT_MIN / -1; a GPU cannot, so those elements become 0 and INT_MIN.
//
// :double has one quirk in the reference that the 1-D entry point reproduces:
// the scalar remainder of the AVX2 macro goes through `sas_dadd` & co., which
// are declared to return float (cl-waffe2-simd.c:229-232), so the last n % 4
// elements of a call -- and every element when incx < 1, which skips the vector
// body -- are rounded to binary32 and widened again.  The N-D entry point has
// no notion of "calls" and computes every element in binary64, which is what
// the reference's vector body does.
//
// These are bandwidth kernels like their :float counterparts: 16-byte vectors
// when both runs are contiguous (or y is one value) and on the rows of sliced
// views of the 8- and 16-bit types, tiles through LDS for transposing passes,
// one element per lane with four in flight otherwise.  A destination with incx = 0 accumulates in the
// reference's order on one lane.
#include <math.h>

#include <type_traits>

#include "wf2_common.h"
#include "wf2_view.h"

namespace wf2 {

template <class T>
struct Wide { using type = T; };
template <> struct Wide<int8_t> { using type = int; };
template <> struct Wide<uint8_t> { using type = int; };
template <> struct Wide<int16_t> { using type = int; };
template <> struct Wide<uint16_t> { using type = int; };

template <class T>
constexpr bool kIsInt = !__is_floating_point(T);

template <class T, int OP>
__device__ __forceinline__ T apply(T a, T b) {
  using W = typename Wide<T>::type;
  const W x = (W)a, y = (W)b;
  if constexpr (OP == WF2HIP_ADD) {
    if constexpr (kIsInt<T> && sizeof(W) == 4 && (W)(-1) < (W)0)  // signed: wrap, as x86 does
      return (T)(int32_t)((uint32_t)x + (uint32_t)y);
    else
      return (T)(x + y);
  } else if constexpr (OP == WF2HIP_SUB) {
    if constexpr (kIsInt<T> && sizeof(W) == 4 && (W)(-1) < (W)0)
      return (T)(int32_t)((uint32_t)x - (uint32_t)y);
    else
      return (T)(x - y);
  } else if constexpr (OP == WF2HIP_MUL) {
    if constexpr (kIsInt<T> && sizeof(W) == 4 && (W)(-1) < (W)0)
      return (T)(int32_t)((uint32_t)x * (uint32_t)y);
    else
      return (T)(x * y);
  } else if constexpr (OP == WF2HIP_DIV) {
    if constexpr (kIsInt<T>) {
      if (y == 0) return (T)0;
      if constexpr ((W)(-1) < (W)0) {
        if (sizeof(T) == 4 && x == (W)INT32_MIN && y == (W)-1) return (T)x;
      }
      return (T)(x / y);
    } else {
      return (T)(x / y);
    }
  } else {
    return b;  // MOVE
  }
}

// the reference's scalar remainder for :double: through binary32
template <class T>
__device__ __forceinline__ T through_float(T v) {
  if constexpr (__is_same(T, double)) return (double)(float)v;
  return v;
}

template <class T, int N>
struct alignas(16) Pack { T v[N]; };

// Four 8-bit or two 16-bit elements per 32-bit word, add / sub / mul modulo the
// element width: the same bits as widening to int, operating and truncating
// (signed or not), in a fraction of the instructions -- per-byte unpacking
// holds the 8-bit kernels at 64 % of the HBM peak, these forms at the 32-bit rate.
template <class T, int OP>
constexpr bool kWordOp = kIsInt<T> && sizeof(T) < 4 && (OP == WF2HIP_ADD || OP == WF2HIP_SUB || OP == WF2HIP_MUL);

template <int BYTES, int OP>
__device__ __forceinline__ uint32_t apply_word(uint32_t a, uint32_t b) {
  typedef unsigned short us2 __attribute__((ext_vector_type(2)));
  if constexpr (BYTES == 2) {
    const us2 x = __builtin_bit_cast(us2, a), y = __builtin_bit_cast(us2, b);
    if constexpr (OP == WF2HIP_ADD) return __builtin_bit_cast(uint32_t, (us2)(x + y));
    if constexpr (OP == WF2HIP_SUB) return __builtin_bit_cast(uint32_t, (us2)(x - y));
    return __builtin_bit_cast(uint32_t, (us2)(x * y));
  } else {
    constexpr uint32_t H = 0x80808080u;
    if constexpr (OP == WF2HIP_ADD) return ((a & ~H) + (b & ~H)) ^ ((a ^ b) & H);
    if constexpr (OP == WF2HIP_SUB) return ((a | H) - (b & ~H)) ^ ((a ^ ~b) & H);
    // low bytes: the low byte of a 16-bit product depends on the low bytes only;
    // high bytes: (a >> 8) * (b with its low byte cleared) = (ah * bh) << 8 modulo 2^16
    const us2 x = __builtin_bit_cast(us2, a), y = __builtin_bit_cast(us2, b);
    const us2 lo = (us2)(x * y) & (unsigned short)0x00ff;
    const us2 hi = (us2)((us2)(x >> (unsigned short)8) * (us2)(y & (unsigned short)0xff00));
    return __builtin_bit_cast(uint32_t, (us2)(lo | hi));
  }
}

// contiguous x, y contiguous (or one value): 16 bytes per lane and access, four
// accesses per lane issued before the first use, each wavefront on 4 KB of its
// own per stream, nontemporal from 192 MiB of traffic on -- the shape measured
// best for the :float kernel x <- x op y (82 % of the HBM peak at 2^26 elements;
// one access per lane without the nontemporal hint: 72 %).
template <class T, int OP, bool BCAST, bool NT>
__global__ __launch_bounds__(kBlock) void typed_flat(T* __restrict__ x, const T* __restrict__ y, size_t nvec) {
  constexpr int N = 16 / sizeof(T);
  constexpr int U = 4;
  using P = Pack<T, N>;
  typedef float f4 __attribute__((ext_vector_type(4)));
  const unsigned wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const size_t base = ((size_t)blockIdx.x * (kBlock / kWave) + wave) * kWave * U + lane;
  // the loaded vectors stay float4 values up to their use: converted to element
  // arrays where they are loaded, the narrow types lose the nontemporal hint
  auto load = [](const T* p, size_t i) {
    const f4* q = reinterpret_cast<const f4*>(p) + i;
    return NT ? __builtin_nontemporal_load(q) : *q;
  };
  T s = T(0);
  if (BCAST) s = y[0];
  // Two shapes of one body.  Predicated per vector (FULL = false): a branch and a
  // dozen instructions between the load pairs; that spacing measures best when the
  // arithmetic is a few instructions (x <- x + y on 256 MiB per tensor: 122 us; with the
  // eight loads back to back: 127 us).  Branch-free (FULL = true) for a wavefront whose
  // 4 KB lie inside the run: the scheduler starts on each vector as it arrives, which
  // hides the longer arithmetic of the 8- and 16-bit types (123 us against 131 us).
  auto body = [&](auto full) {
    constexpr bool FULL = decltype(full)::value;
    f4 a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        if (OP != WF2HIP_MOVE) a[u] = load(x, i);
        if (!BCAST) b[u] = load(y, i);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        P r;
        if constexpr (kWordOp<T, OP>) {
          typedef uint32_t u4 __attribute__((ext_vector_type(4)));
          u4 aw = __builtin_bit_cast(u4, a[u]), bw, rw;
          if (BCAST) {
            uint32_t w = sizeof(T) == 1 ? (uint32_t)(uint8_t)s * 0x01010101u : (uint32_t)(uint16_t)s * 0x00010001u;
            bw = (u4){w, w, w, w};
          } else {
            bw = __builtin_bit_cast(u4, b[u]);
          }
#pragma unroll
          for (int k = 0; k < 4; k++) rw[k] = apply_word<(int)sizeof(T), OP>(aw[k], bw[k]);
          r = __builtin_bit_cast(P, rw);
        } else {
          const P pa = __builtin_bit_cast(P, a[u]), pb = __builtin_bit_cast(P, b[u]);
#pragma unroll
          for (int k = 0; k < N; k++) {
            const T yv = BCAST ? s : pb.v[k];
            r.v[k] = apply<T, OP>(OP != WF2HIP_MOVE ? pa.v[k] : yv, yv);
          }
        }
        f4* q = reinterpret_cast<f4*>(x) + i;
        if (NT)
          __builtin_nontemporal_store(__builtin_bit_cast(f4, r), q);
        else
          *q = __builtin_bit_cast(f4, r);
      }
    }
  };
  constexpr bool kBranchFree = kIsInt<T> && sizeof(T) < 4 && OP != WF2HIP_MOVE;
  if (kBranchFree && base - lane + (size_t)kWave * U <= nvec)
    body(std::true_type{});
  else
    body(std::false_type{});
}

// any increments (incx != 0): elements first..n-1; those from `exact_end` on go
// through binary32 when T is double (the reference's remainder loop)
template <class T, int OP>
__global__ __launch_bounds__(kBlock) void typed_strided(T* x, int64_t incx, const T* y, int64_t incy, int64_t first,
                                                        int64_t n, int64_t exact_end) {
  constexpr int U = 4;
  const int64_t step = (int64_t)gridDim.x * kBlock * U;
  for (int64_t base = first + (int64_t)blockIdx.x * kBlock * U + threadIdx.x; base < n; base += step) {
    T a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t i = base + (int64_t)u * kBlock;
      if (i < n) {
        a[u] = OP != WF2HIP_MOVE ? x[i * incx] : T(0);
        b[u] = y[i * incy];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t i = base + (int64_t)u * kBlock;
      if (i < n) {
        T r = apply<T, OP>(a[u], b[u]);
        if (OP != WF2HIP_MOVE && i >= exact_end) r = through_float(r);
        x[i * incx] = r;
      }
    }
  }
}

// incx == 0: x[0] <- x[0] op y[i], i = 0..n-1, in that order (one lane)
template <class T, int OP>
__global__ void typed_sequential(T* x, const T* y, int64_t incy, int64_t n) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  T acc = x[0];
  for (int64_t i = 0; i < n; i++) {
    acc = apply<T, OP>(acc, y[i * incy]);
    if (OP != WF2HIP_MOVE) acc = through_float(acc);
  }
  x[0] = acc;
}

struct TypedGen {
  int32_t rank;
  int64_t total;
  int64_t shape[WF2HIP_MAX_RANK];
  int64_t sd[WF2HIP_MAX_RANK];
  int64_t ss[WF2HIP_MAX_RANK];
};

template <class T, int OP>
__global__ __launch_bounds__(kBlock) void typed_generic(T* dst, const T* src, TypedGen p) {
  constexpr int U = 4;
  const int64_t step = (int64_t)gridDim.x * kBlock * U;
  for (int64_t base = (int64_t)blockIdx.x * kBlock * U + threadIdx.x; base < p.total; base += step) {
    int64_t doff[U], soff[U];
    T a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      int64_t rem = base + (int64_t)u * kBlock;
      if (rem >= p.total) rem = p.total - 1;
      int64_t d = 0, q = 0;
      for (int r = p.rank - 1; r > 0; r--) {
        const int64_t quot = rem / p.shape[r];
        const int64_t idx = rem - quot * p.shape[r];
        rem = quot;
        d += idx * p.sd[r];
        q += idx * p.ss[r];
      }
      doff[u] = d + rem * p.sd[0];
      soff[u] = q + rem * p.ss[0];
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bool live = base + (int64_t)u * kBlock < p.total;
      a[u] = (OP != WF2HIP_MOVE && live) ? dst[doff[u]] : T(0);
      b[u] = live ? src[soff[u]] : T(0);
    }
#pragma unroll
    for (int u = 0; u < U; u++)
      if (base + (int64_t)u * kBlock < p.total) dst[doff[u]] = apply<T, OP>(a[u], b[u]);
  }
}

template <class T>
__global__ __launch_bounds__(kBlock) void typed_inv(T* x, int64_t incx, int64_t n) {
  if (incx == 0) {  // the reference's loop inverts the one element n times
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    T v = x[0];
    for (int64_t i = 0; i < n; i++) v = apply<T, WF2HIP_DIV>(T(1), v);
    x[0] = v;
    return;
  }
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step)
    x[i * incx] = apply<T, WF2HIP_DIV>(T(1), x[i * incx]);
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

static uint32_t grid_for(int64_t n, int per_thread) {
  int64_t want = ceil_div(n, (int64_t)kBlock * per_thread);
  int64_t cap = (int64_t)rt().num_cus * 64;
  if (want < 1) want = 1;
  return (uint32_t)(want < cap ? want : cap);
}

// `quirk`: reproduce the binary32 rounding of the reference's remainder loop (:double only)
template <class T, int OP>
static int run_1d(int64_t n, T* x, int64_t incx, const T* y, int64_t incy, bool quirk) {
  hipStream_t st = rt().stream;
  if (incx == 0) {
    if (OP == WF2HIP_MOVE) {  // the last write wins
      typed_strided<T, OP><<<1, kBlock, 0, st>>>(x, 0, y + (n - 1) * incy, 0, 0, 1, 1);
      return after_launch("typed_strided");
    }
    if (!quirk && __is_same(T, double))
      return fail(WF2HIP_EUNSUPPORTED, "reductions of :double tensors go through the 1-D entry point");
    typed_sequential<T, OP><<<1, kWave, 0, st>>>(x, y, incy, n);
    return after_launch("typed_sequential");
  }
  constexpr int N = 16 / (int)sizeof(T);
  // the reference's vector body covers (n / 4) * 4 elements when incx >= 1
  const int64_t exact_end = (!quirk || !__is_same(T, double) || OP == WF2HIP_MOVE) ? n : (incx >= 1 ? (n / 4) * 4 : 0);
  int64_t done = 0;
  if (incx == 1 && (incy == 1 || incy == 0) && aligned16(x) && (incy == 0 || aligned16(y))) {
    const int64_t nvec = (exact_end < n ? exact_end : n) / N;
    if (nvec > 0) {
      const int64_t blocks = ceil_div(nvec, kBlock * 4);
      if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "run too long for one launch");
      const int streams = (OP != WF2HIP_MOVE ? 2 : 1) + (incy == 0 ? 0 : 1);
      const bool nt = nvec * 16 * streams >= ((int64_t)192 << 20);
      if (incy == 0 && nt)
        typed_flat<T, OP, true, true><<<(uint32_t)blocks, kBlock, 0, st>>>(x, y, (size_t)nvec);
      else if (incy == 0)
        typed_flat<T, OP, true, false><<<(uint32_t)blocks, kBlock, 0, st>>>(x, y, (size_t)nvec);
      else if (nt)
        typed_flat<T, OP, false, true><<<(uint32_t)blocks, kBlock, 0, st>>>(x, y, (size_t)nvec);
      else
        typed_flat<T, OP, false, false><<<(uint32_t)blocks, kBlock, 0, st>>>(x, y, (size_t)nvec);
      WF2_TRY(after_launch("typed_flat"));
      done = nvec * N;
    }
  }
  if (done < n) {
    typed_strided<T, OP><<<grid_for(n - done, 4), kBlock, 0, st>>>(x, incx, y, incy, done, n, exact_end);
    return after_launch("typed_strided");
  }
  return 0;
}

template <class T>
static int dispatch_1d(int op, int64_t n, T* x, int64_t incx, const T* y, int64_t incy, bool quirk) {
  switch (op) {
    case WF2HIP_ADD: return run_1d<T, WF2HIP_ADD>(n, x, incx, y, incy, quirk);
    case WF2HIP_SUB: return run_1d<T, WF2HIP_SUB>(n, x, incx, y, incy, quirk);
    case WF2HIP_MUL: return run_1d<T, WF2HIP_MUL>(n, x, incx, y, incy, quirk);
    case WF2HIP_DIV: return run_1d<T, WF2HIP_DIV>(n, x, incx, y, incy, quirk);
    case WF2HIP_MOVE: return run_1d<T, WF2HIP_MOVE>(n, x, incx, y, incy, quirk);
    default: return fail(WF2HIP_EINVAL, "unknown binary op %d", op);
  }
}

// Transposing passes: dst has stride 1 along its last axis I, src along another axis J.  A 64 x 64 tile is
// read with lanes running along J, parked in LDS (pitch 65) and written with lanes running along I: both
// sides in whole lines, where an element per lane leaves one of them at a stride ((8192, 8192) transposed:
// :double 414 us, :int32 329 us, :uint8 272 us).
struct TypedTile {
  int64_t ni, nj, d_j, s_i;  // extents of I and J, dst stride along J, src stride along I
  uint32_t tiles_i, tiles_j;
  int32_t nouter;
  uint32_t oshape[WF2HIP_MAX_RANK];
  int64_t odst[WF2HIP_MAX_RANK], osrc[WF2HIP_MAX_RANK];
};

template <class T, int OP>
__global__ __launch_bounds__(kBlock) void typed_tile(T* dst, const T* src, TypedTile p) {
  constexpr int kEdge = 64;
  __shared__ T tile[kEdge][kEdge + 1];
  uint32_t rem = blockIdx.x / p.tiles_i;
  const int64_t i0 = (int64_t)(blockIdx.x - rem * p.tiles_i) * kEdge;
  const uint32_t tj = rem % p.tiles_j;
  rem /= p.tiles_j;
  const int64_t j0 = (int64_t)tj * kEdge;
  int64_t doff = 0, soff = 0;
  for (int i = 0; i < p.nouter; i++) {
    const uint32_t q = rem / p.oshape[i];
    const uint32_t idx = rem - q * p.oshape[i];
    rem = q;
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  const int tx = threadIdx.x & (kEdge - 1), ty = threadIdx.x / kEdge;
  constexpr int kRows = kBlock / kEdge;  // rows of the tile per pass
  {
    T v[kEdge / kRows];
#pragma unroll
    for (int q = 0; q < kEdge / kRows; q++) {
      const int64_t i = i0 + ty + q * kRows, j = j0 + tx;
      v[q] = (i < p.ni && j < p.nj) ? src[soff + i * p.s_i + j] : T(0);
    }
#pragma unroll
    for (int q = 0; q < kEdge / kRows; q++) tile[ty + q * kRows][tx] = v[q];
  }
  __syncthreads();
  T old[kEdge / kRows];
#pragma unroll
  for (int q = 0; q < kEdge / kRows; q++) {
    const int64_t i = i0 + tx, j = j0 + ty + q * kRows;
    old[q] = (OP != WF2HIP_MOVE && i < p.ni && j < p.nj) ? dst[doff + j * p.d_j + i] : T(0);
  }
#pragma unroll
  for (int q = 0; q < kEdge / kRows; q++) {
    const int64_t i = i0 + tx, j = j0 + ty + q * kRows;
    if (i < p.ni && j < p.nj) dst[doff + j * p.d_j + i] = apply<T, OP>(old[q], tile[tx][ty + q * kRows]);
  }
}

template <class T, int OP>
static bool try_typed_tile(const Space& s, T* a, const T* b, int* rc) {
  const int last = s.rank - 1;
  if (s.rank < 2 || s.sa[last] != 1 || s.sb[last] <= 1) return false;
  int J = -1;
  for (int r = 0; r < last; r++)
    if (s.sb[r] == 1 && s.sa[r] > 0) J = r;
  if (J < 0 || s.shape[last] < 16 || s.shape[J] < 16) return false;
  TypedTile p;
  p.ni = s.shape[last];
  p.nj = s.shape[J];
  p.d_j = s.sa[J];
  p.s_i = s.sb[last];
  p.tiles_i = (uint32_t)ceil_div(p.ni, (int64_t)64);
  p.tiles_j = (uint32_t)ceil_div(p.nj, (int64_t)64);
  p.nouter = 0;
  int64_t blocks = (int64_t)p.tiles_i * p.tiles_j;
  for (int r = last - 1; r >= 0; r--) {
    if (r == J) continue;
    if (s.shape[r] >= ((int64_t)1 << 32)) return false;
    p.oshape[p.nouter] = (uint32_t)s.shape[r];
    p.odst[p.nouter] = s.sa[r];
    p.osrc[p.nouter] = s.sb[r];
    p.nouter++;
    blocks *= s.shape[r];
  }
  if (blocks >= ((int64_t)1 << 31)) return false;
  typed_tile<T, OP><<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(a + s.off_a, b + s.off_b, p);
  *rc = after_launch("typed_tile");
  return true;
}

// Sliced views of the 8- and 16-bit types: both sides have stride 1 along the last axis, rows of `len`
// elements at any pitch and any (element-aligned) start.  An element per lane moves 64 or 128 bytes per
// wavefront and access; here a lane takes 16 bytes of the destination row: `lanes` (a power of two up to
// 256) lanes share a row, the elements before the row's first 16-byte boundary and after its last one
// go one to a lane, the vectors between them are read and written whole.  The source row starts wherever
// it starts: its vectors are read at element alignment, which the hardware serves.
struct TypedRows {
  int64_t len, nrows;
  uint32_t lane_shift;  // log2(lanes)
  int32_t nouter;
  uint32_t oshape[WF2HIP_MAX_RANK];  // innermost outer axis first
  int64_t odst[WF2HIP_MAX_RANK], osrc[WF2HIP_MAX_RANK];
};

template <class T, int OP, bool NT>
__global__ __launch_bounds__(kBlock) void typed_rows(T* dst, const T* src, TypedRows p) {
  constexpr int N = 16 / (int)sizeof(T);
  constexpr int U = 4;
  using P = Pack<T, N>;
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const uint32_t lanes = 1u << p.lane_shift;
  const uint32_t sub = threadIdx.x & (lanes - 1);
  const int64_t rows_per_pass = (int64_t)gridDim.x * (kBlock >> p.lane_shift);
  for (int64_t row = (int64_t)blockIdx.x * (kBlock >> p.lane_shift) + (threadIdx.x >> p.lane_shift); row < p.nrows;
       row += rows_per_pass) {
  int64_t doff = 0, soff = 0;
  {
    uint64_t rem = (uint64_t)row;
    for (int i = 0; i < p.nouter; i++) {
      const uint64_t q = rem / p.oshape[i];
      const int64_t idx = (int64_t)(rem - q * p.oshape[i]);
      rem = q;
      doff += idx * p.odst[i];
      soff += idx * p.osrc[i];
    }
  }
  T* d = dst + doff;
  const T* s = src + soff;
  int64_t head = (int64_t)((16 - ((uintptr_t)d & 15)) & 15) / (int64_t)sizeof(T);
  if (head > p.len) head = p.len;
  const int64_t nvec = (p.len - head) / N;
  const int64_t tail0 = head + nvec * N;
  if (blockIdx.y == 0) {
    // at most N - 1 elements on either side of the vectors
    const int64_t loose = head + (p.len - tail0);
    for (int64_t e = sub; e < loose; e += lanes) {
      const int64_t i = e < head ? e : tail0 + (e - head);
      const T yv = s[i];
      d[i] = apply<T, OP>(OP != WF2HIP_MOVE ? d[i] : yv, yv);
    }
  }
  const int64_t step = (int64_t)lanes * gridDim.y;
  for (int64_t v0 = (int64_t)blockIdx.y * lanes + sub; v0 < nvec; v0 += step * U) {
    u4 a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t v = v0 + u * step;
      if (v < nvec) {
        if (OP != WF2HIP_MOVE) {
          const u4* q = reinterpret_cast<const u4*>(d + head + v * N);
          a[u] = NT ? __builtin_nontemporal_load(q) : *q;
        }
        __builtin_memcpy(&b[u], s + head + v * N, 16);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t v = v0 + u * step;
      if (v < nvec) {
        u4 r;
        if constexpr (OP == WF2HIP_MOVE) {
          r = b[u];
        } else if constexpr (kWordOp<T, OP>) {
#pragma unroll
          for (int k = 0; k < 4; k++) r[k] = apply_word<(int)sizeof(T), OP>(a[u][k], b[u][k]);
        } else {
          const P pa = __builtin_bit_cast(P, a[u]), pb = __builtin_bit_cast(P, b[u]);
          P pr;
#pragma unroll
          for (int k = 0; k < N; k++) pr.v[k] = apply<T, OP>(pa.v[k], pb.v[k]);
          r = __builtin_bit_cast(u4, pr);
        }
        u4* q = reinterpret_cast<u4*>(d + head + v * N);
        if (NT)
          __builtin_nontemporal_store(r, q);
        else
          *q = r;
      }
    }
  }
  }
}

template <class T, int OP>
static bool try_typed_rows(const Space& s, T* a, const T* b, int* rc) {
  const int last = s.rank - 1;
  if (sizeof(T) > 2 || s.rank < 2 || s.sa[last] != 1 || s.sb[last] != 1) return false;
  constexpr int N = 16 / (int)sizeof(T);
  const int64_t len = s.shape[last];
  if (len < 4 * N) return false;  // rows under 64 bytes: mostly loose elements
  TypedRows p;
  p.len = len;
  p.nrows = s.total / len;
  p.nouter = 0;
  for (int r = last - 1; r >= 0; r--) {
    if (s.shape[r] >= ((int64_t)1 << 32)) return false;
    p.oshape[p.nouter] = (uint32_t)s.shape[r];
    p.odst[p.nouter] = s.sa[r];
    p.osrc[p.nouter] = s.sb[r];
    p.nouter++;
  }
  const int64_t vecs = ceil_div(len, (int64_t)N);
  p.lane_shift = 0;
  while (p.lane_shift < 8 && ((int64_t)1 << p.lane_shift) < vecs) p.lane_shift++;
  const int64_t lanes = (int64_t)1 << p.lane_shift;
  // at most 64 workgroups per compute unit and position along the row: a workgroup then walks several rows
  int64_t gx = ceil_div(p.nrows, (int64_t)kBlock / lanes);
  if (gx > (int64_t)rt().num_cus * 64) gx = (int64_t)rt().num_cus * 64;
  // along a long row: workgroups of four vectors per lane, as many as fill the device with few rows
  int64_t gy = ceil_div(vecs, lanes * 4);
  const int64_t fill = ceil_div((int64_t)rt().num_cus * 16, gx);
  if (gy > fill) gy = fill;
  if (gy > 65535) gy = 65535;
  if (gy < 1) gy = 1;
  // far beyond the Infinity Cache: the destination's side nontemporal, as in the contiguous kernels
  if (s.total * (int64_t)sizeof(T) * (OP != WF2HIP_MOVE ? 3 : 2) >= ((int64_t)192 << 20))
    typed_rows<T, OP, true><<<dim3((uint32_t)gx, (uint32_t)gy), kBlock, 0, rt().stream>>>(a + s.off_a, b + s.off_b, p);
  else
    typed_rows<T, OP, false><<<dim3((uint32_t)gx, (uint32_t)gy), kBlock, 0, rt().stream>>>(a + s.off_a, b + s.off_b, p);
  *rc = after_launch("typed_rows");
  return true;
}

template <class T, int OP>
static int run_generic(const Space& s, T* a, const T* b) {
  int rc = 0;
  if (try_typed_rows<T, OP>(s, a, b, &rc)) return rc;
  if (try_typed_tile<T, OP>(s, a, b, &rc)) return rc;
  TypedGen p;
  p.rank = s.rank;
  p.total = s.total;
  for (int r = 0; r < s.rank; r++) {
    p.shape[r] = s.shape[r];
    p.sd[r] = s.sa[r];
    p.ss[r] = s.sb[r];
  }
  typed_generic<T, OP><<<grid_for(s.total, 4), kBlock, 0, rt().stream>>>(a + s.off_a, b + s.off_b, p);
  return after_launch("typed_generic");
}

// the :float path's test, in elements of `size` bytes
static bool typed_overlap(const Space& s, const void* a, const void* b, size_t size) {
  const int64_t bytes = (const char*)b - (const char*)a;
  if (bytes % (int64_t)size == 0) return hazardous_overlap_at(s, bytes / (int64_t)size);
  // bases that are not a whole number of elements apart: plain interval test
  int64_t alo, ahi, blo, bhi;
  extent_of(s, s.sa, s.off_a, &alo, &ahi);
  extent_of(s, s.sb, s.off_b, &blo, &bhi);
  const char* a0 = (const char*)a + alo * (int64_t)size;
  const char* a1 = (const char*)a + (ahi + 1) * (int64_t)size;
  const char* b0 = (const char*)b + blo * (int64_t)size;
  const char* b1 = (const char*)b + (bhi + 1) * (int64_t)size;
  return !(a1 <= b0 || b1 <= a0);
}

// ---- accumulation into a broadcast destination (what !sum composes) ------------
// a[kept] <- a[kept] OP b[kept, reduced] over every reduced index.  Integer sums
// wrap modulo 2^bits whatever the order, so ADD runs as a tree per destination
// (one workgroup each) and is exact; :double ADD is the same tree in binary64
// (within a few ulp of the reference's sequential order).  The other operations
// keep the reference's order: one lane per destination walks the reduced indices
// row-major.
struct TypedAcc {
  int32_t nk, nr;  // kept / reduced axis counts
  int64_t nout, nred;
  int64_t kshape[WF2HIP_MAX_RANK], ka[WF2HIP_MAX_RANK], kb[WF2HIP_MAX_RANK];
  int64_t rshape[WF2HIP_MAX_RANK], rb[WF2HIP_MAX_RANK];  // outermost first
};

__device__ __forceinline__ void acc_kept(const TypedAcc& p, int64_t out, int64_t* aoff, int64_t* boff) {
  int64_t ao = 0, bo = 0, rem = out;
  for (int i = p.nk - 1; i >= 0; i--) {
    const int64_t q = rem / p.kshape[i];
    const int64_t idx = rem - q * p.kshape[i];
    rem = q;
    ao += idx * p.ka[i];
    bo += idx * p.kb[i];
  }
  *aoff = ao;
  *boff = bo;
}

__device__ __forceinline__ int64_t acc_reduced(const TypedAcc& p, int64_t j) {
  int64_t off = 0, rem = j;
  for (int i = p.nr - 1; i >= 0; i--) {
    const int64_t q = rem / p.rshape[i];
    const int64_t idx = rem - q * p.rshape[i];
    rem = q;
    off += idx * p.rb[i];
  }
  return off;
}

template <class T>
struct SumOf { using type = uint32_t; };  // wrap-around sums of every integer type
template <> struct SumOf<double> { using type = double; };

template <class T>
__global__ __launch_bounds__(kBlock) void typed_accumulate_add(T* a, const T* b, TypedAcc p) {
  using S = typename SumOf<T>::type;
  __shared__ S lds[kBlock / kWave];
  const int64_t out = blockIdx.x;
  int64_t aoff, boff;
  acc_kept(p, out, &aoff, &boff);
  S acc = S(0);
  // consecutive threads take consecutive reduced indices: a unit stride on the innermost
  // reduced axis coalesces, and a single long axis keeps all 256 threads busy
  if (p.nr == 1) {
    for (int64_t j = threadIdx.x; j < p.nred; j += kBlock) acc += (S)b[boff + j * p.rb[0]];
  } else {
    for (int64_t j = threadIdx.x; j < p.nred; j += kBlock) acc += (S)b[boff + acc_reduced(p, j)];
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    S total = lds[0];
#pragma unroll
    for (int w = 1; w < kBlock / kWave; w++) total += lds[w];
    a[aoff] = (T)((S)a[aoff] + total);
  }
}

// Many destinations, few terms each (sums over a short trailing axis: (2097152, 4) rows): a thread
// per destination adds its terms in index order.  A workgroup per destination takes 1.3 ms for
// those two million sums of four.
template <class T>
__global__ __launch_bounds__(kBlock) void typed_accumulate_thread(T* a, const T* b, TypedAcc p) {
  using S = typename SumOf<T>::type;
  const int64_t out = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (out >= p.nout) return;
  int64_t aoff, boff;
  acc_kept(p, out, &aoff, &boff);
  S acc = S(0);
  if (p.nr == 1) {
    for (int64_t j = 0; j < p.nred; j++) acc += (S)b[boff + j * p.rb[0]];
  } else {
    for (int64_t j = 0; j < p.nred; j++) acc += (S)b[boff + acc_reduced(p, j)];
  }
  a[aoff] = (T)((S)a[aoff] + acc);
}

// Column form: the only kept axis is contiguous on both sides (sums over the leading
// axes).  A thread owns one destination column, consecutive threads consecutive columns,
// so every reduced index is one coalesced row segment; the reduced indices are split
// over `splits` workgroups per 256 columns and folded by typed_accumulate_fold.
template <class T>
__global__ __launch_bounds__(kBlock) void typed_accumulate_cols(T* a, const T* b, TypedAcc p, int64_t ncols,
                                                                uint32_t splits, int64_t seg,
                                                                typename SumOf<T>::type* partials) {
  using S = typename SumOf<T>::type;
  const uint32_t ctiles = (uint32_t)((ncols + kBlock - 1) / kBlock);
  const uint32_t ctile = blockIdx.x % ctiles, split = blockIdx.x / ctiles;
  const int64_t c = (int64_t)ctile * kBlock + threadIdx.x;
  if (c >= ncols) return;
  const int64_t lo = (int64_t)split * seg;
  const int64_t hi = lo + seg < p.nred ? lo + seg : p.nred;
  S acc0 = S(0), acc1 = S(0), acc2 = S(0), acc3 = S(0);
  int64_t j = lo;
  for (; j + 3 < hi; j += 4) {  // four rows in flight per thread
    const T v0 = b[acc_reduced(p, j) + c], v1 = b[acc_reduced(p, j + 1) + c];
    const T v2 = b[acc_reduced(p, j + 2) + c], v3 = b[acc_reduced(p, j + 3) + c];
    acc0 += (S)v0;
    acc1 += (S)v1;
    acc2 += (S)v2;
    acc3 += (S)v3;
  }
  for (; j < hi; j++) acc0 += (S)b[acc_reduced(p, j) + c];
  const S total = (acc0 + acc1) + (acc2 + acc3);
  if (splits == 1)
    a[c] = (T)((S)a[c] + total);
  else
    partials[(int64_t)split * ncols + c] = total;
}

// Narrow dense matrices (at most 128 columns, rows adjacent in memory): the 256-column tiles above leave most
// lanes without a column ((131072, 64) :double: 518 us).  The workgroup reads k = 256 / ncols whole rows per
// step, one contiguous run: thread t adds column t mod ncols of every k-th row with eight loads in flight, and
// the k threads of a column meet in LDS in a fixed order.
template <class T>
__global__ __launch_bounds__(kBlock) void typed_accumulate_cols_narrow(T* a, const T* b, int64_t nred, uint32_t ncols,
                                                                       uint32_t splits, int64_t seg,
                                                                       typename SumOf<T>::type* partials) {
  using S = typename SumOf<T>::type;
  __shared__ S lds[kBlock];
  const uint32_t k = kBlock / ncols;  // rows per step
  const uint32_t phase = threadIdx.x / ncols, col = threadIdx.x - phase * ncols;
  const int64_t lo = (int64_t)blockIdx.x * seg;
  const int64_t hi = lo + seg < nred ? lo + seg : nred;
  S acc = S(0);
  if (phase < k) {
    const T* src = b + col;
    int64_t j = lo + phase;
    for (; j + 7 * (int64_t)k < hi; j += 8 * (int64_t)k) {
      T v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = src[(j + u * (int64_t)k) * ncols];
#pragma unroll
      for (int u = 0; u < 8; u++) acc += (S)v[u];
    }
    for (; j < hi; j += k) acc += (S)src[j * ncols];
  }
  lds[threadIdx.x] = acc;
  __syncthreads();
  if (threadIdx.x < ncols) {
    S total = lds[threadIdx.x];
    for (uint32_t r = 1; r < k; r++) total += lds[r * ncols + threadIdx.x];
    if (splits == 1)
      a[threadIdx.x] = (T)((S)a[threadIdx.x] + total);
    else
      partials[(int64_t)blockIdx.x * ncols + threadIdx.x] = total;
  }
}

// Folds the splits' partial sums: 64 columns per workgroup, its four wavefronts take every fourth split with
// eight loads in flight, then meet in LDS -- a fixed order.  (One thread per column walking all splits in
// turn waits for memory once per split.)
template <class T>
__global__ __launch_bounds__(kBlock) void typed_accumulate_cols_fold(T* a, int64_t ncols, uint32_t splits,
                                                                     const typename SumOf<T>::type* partials) {
  using S = typename SumOf<T>::type;
  constexpr int kWaves = kBlock / kWave;
  __shared__ S lds[kWaves][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t c = (int64_t)blockIdx.x * kWave + lane;
  S acc = S(0);
  if (c < ncols) {
    uint32_t sp = (uint32_t)wave;
    for (; sp + 7 * kWaves < splits; sp += 8 * kWaves) {
      S t[8];
#pragma unroll
      for (int u = 0; u < 8; u++) t[u] = partials[(int64_t)(sp + u * kWaves) * ncols + c];
#pragma unroll
      for (int u = 0; u < 8; u++) acc += t[u];
    }
    for (; sp < splits; sp += kWaves) acc += partials[(int64_t)sp * ncols + c];
  }
  lds[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && c < ncols) {
    S total = lds[0][lane];
#pragma unroll
    for (int w = 1; w < kWaves; w++) total += lds[w][lane];
    a[c] = (T)((S)a[c] + total);
  }
}

// Few destinations, long reductions: `splits` workgroups per destination each sum a
// contiguous range of the reduced index space into `partials`, a second launch folds
// them in a fixed order (deterministic for :double, exact for the integer types).
template <class T>
__global__ __launch_bounds__(kBlock) void typed_accumulate_partial(const T* b, TypedAcc p, uint32_t splits, int64_t seg,
                                                                   typename SumOf<T>::type* partials) {
  using S = typename SumOf<T>::type;
  __shared__ S lds[kBlock / kWave];
  const int64_t out = blockIdx.x / splits;
  const uint32_t split = blockIdx.x - (uint32_t)out * splits;
  int64_t aoff, boff;
  acc_kept(p, out, &aoff, &boff);
  const int64_t lo = (int64_t)split * seg;
  const int64_t hi = lo + seg < p.nred ? lo + seg : p.nred;
  S acc = S(0);
  if (p.nr == 1) {
    for (int64_t j = lo + threadIdx.x; j < hi; j += kBlock) acc += (S)b[boff + j * p.rb[0]];
  } else {
    for (int64_t j = lo + threadIdx.x; j < hi; j += kBlock) acc += (S)b[boff + acc_reduced(p, j)];
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    S total = lds[0];
#pragma unroll
    for (int w = 1; w < kBlock / kWave; w++) total += lds[w];
    partials[blockIdx.x] = total;
  }
}

template <class T>
__global__ __launch_bounds__(kWave) void typed_accumulate_fold(T* a, TypedAcc p, uint32_t splits,
                                                               const typename SumOf<T>::type* partials) {
  using S = typename SumOf<T>::type;
  const int64_t out = (int64_t)blockIdx.x * kWave + threadIdx.x;
  if (out >= p.nout) return;
  int64_t aoff, boff;
  acc_kept(p, out, &aoff, &boff);
  S total = S(0);
  for (uint32_t s = 0; s < splits; s++) total += partials[out * splits + s];
  a[aoff] = (T)((S)a[aoff] + total);
}

template <class T, int OP>
__global__ __launch_bounds__(kBlock) void typed_accumulate_sequential(T* a, const T* b, TypedAcc p) {
  const int64_t out = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (out >= p.nout) return;
  int64_t aoff, boff;
  acc_kept(p, out, &aoff, &boff);
  T acc = a[aoff];
  const int64_t inner = p.rshape[p.nr - 1], inner_stride = p.rb[p.nr - 1];
  const int64_t outer = p.nred / inner;
  for (int64_t o = 0; o < outer; o++) {
    const int64_t base = boff + acc_reduced(p, o * inner);
    for (int64_t i = 0; i < inner; i++) acc = apply<T, OP>(acc, b[base + i * inner_stride]);
  }
  a[aoff] = acc;
}

// `s` is normalised and has at least one broadcast axis in `a`
template <class T>
static int run_accumulate(int op, const Space& s, T* a, const T* b) {
  TypedAcc p;
  p.nk = p.nr = 0;
  p.nout = p.nred = 1;
  for (int r = 0; r < s.rank; r++) {
    if (s.sa[r] == 0 && s.shape[r] > 1) {
      p.rshape[p.nr] = s.shape[r];
      p.rb[p.nr] = s.sb[r];
      p.nr++;
      p.nred *= s.shape[r];
    } else {
      p.kshape[p.nk] = s.shape[r];
      p.ka[p.nk] = s.sa[r];
      p.kb[p.nk] = s.sb[r];
      p.nk++;
      p.nout *= s.shape[r];
    }
  }
  hipStream_t st = rt().stream;
  T* ap = a + s.off_a;
  const T* bp = b + s.off_b;
  if (op == WF2HIP_ADD && rt().reduce_mode == 0) {
    if (p.nout >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
    using S = typename SumOf<T>::type;
    const int64_t target = (int64_t)rt().num_cus * 8;
    const int last = s.rank - 1;
    // a dense matrix of at most 128 columns with at least 64 steps of whole rows
    const bool narrow = p.nk == 1 && p.nr == 1 && s.sa[last] == 1 && s.sb[last] == 1 && s.shape[last] <= 128 &&
                        p.rb[0] == s.shape[last] && p.nred >= 64 * (kBlock / s.shape[last]);
    if (narrow || (p.nk == 1 && s.sa[last] == 1 && s.sb[last] == 1 && s.shape[last] >= 64 && p.nred >= 2)) {
      const int64_t ncols = s.shape[last];
      const int64_t ctiles = narrow ? 1 : ceil_div(ncols, kBlock);
      int64_t splits = ceil_div(target, ctiles);
      const int64_t least = narrow ? 64 * (kBlock / ncols) : 32;  // reduced indices per workgroup
      if (splits > p.nred / least) splits = p.nred / least;
      if (splits < 1) splits = 1;
      int64_t seg = ceil_div(p.nred, splits);
      splits = ceil_div(p.nred, seg);
      void* scratch = nullptr;
      int held_up = 0;
      if (splits > 1 && !scratch_block(&scratch, (size_t)(splits * ncols) * sizeof(S), &held_up)) {
        if (held_up) return held_up;
        splits = 1;
        seg = p.nred;
      }
      if (ctiles * splits < ((int64_t)1 << 31)) {
        if (narrow)
          typed_accumulate_cols_narrow<T><<<(uint32_t)splits, kBlock, 0, st>>>(ap, bp, p.nred, (uint32_t)ncols,
                                                                             (uint32_t)splits, seg, static_cast<S*>(scratch));
        else
          typed_accumulate_cols<T><<<(uint32_t)(ctiles * splits), kBlock, 0, st>>>(ap, bp, p, ncols, (uint32_t)splits, seg,
                                                                                 static_cast<S*>(scratch));
        int rc = after_launch("typed_accumulate_cols");
        if (rc == 0 && splits > 1) {
          typed_accumulate_cols_fold<T><<<(uint32_t)ceil_div(ncols, kWave), kBlock, 0, st>>>(ap, ncols, (uint32_t)splits,
                                                                                         static_cast<const S*>(scratch));
          rc = after_launch("typed_accumulate_cols_fold");
        }
        if (scratch) (void)wf2hip_free(scratch);  // stream order keeps it alive for the launches above
        return rc;
      }
      if (scratch) (void)wf2hip_free(scratch);
    }
    const int64_t capacity = (int64_t)(kPartialCapacity * sizeof(float) / sizeof(S));
    if (p.nout < target && p.nred >= 2 * 16384 && p.nout <= capacity / 2) {
      int64_t splits = ceil_div(p.nred, 16384);
      const int64_t by_fill = ceil_div(target, p.nout), by_cap = capacity / p.nout;
      if (splits > by_fill) splits = by_fill;
      if (splits > by_cap) splits = by_cap;
      const int64_t seg = ceil_div(p.nred, splits);
      splits = ceil_div(p.nred, seg);
      S* partials = reinterpret_cast<S*>(rt().partials);
      typed_accumulate_partial<T><<<(uint32_t)(p.nout * splits), kBlock, 0, st>>>(bp, p, (uint32_t)splits, seg, partials);
      WF2_TRY(after_launch("typed_accumulate_partial"));
      typed_accumulate_fold<T><<<(uint32_t)ceil_div(p.nout, kWave), kWave, 0, st>>>(ap, p, (uint32_t)splits, partials);
      return after_launch("typed_accumulate_fold");
    }
    if (p.nred <= 128 && p.nout >= 64 * target) {
      typed_accumulate_thread<T><<<(uint32_t)ceil_div(p.nout, kBlock), kBlock, 0, st>>>(ap, bp, p);
      return after_launch("typed_accumulate_thread");
    }
    typed_accumulate_add<T><<<(uint32_t)p.nout, kBlock, 0, st>>>(ap, bp, p);
    return after_launch("typed_accumulate_add");
  }
  const int64_t blocks = ceil_div(p.nout, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
  switch (op) {
    case WF2HIP_ADD: typed_accumulate_sequential<T, WF2HIP_ADD><<<(uint32_t)blocks, kBlock, 0, st>>>(ap, bp, p); break;
    case WF2HIP_SUB: typed_accumulate_sequential<T, WF2HIP_SUB><<<(uint32_t)blocks, kBlock, 0, st>>>(ap, bp, p); break;
    case WF2HIP_MUL: typed_accumulate_sequential<T, WF2HIP_MUL><<<(uint32_t)blocks, kBlock, 0, st>>>(ap, bp, p); break;
    case WF2HIP_DIV: typed_accumulate_sequential<T, WF2HIP_DIV><<<(uint32_t)blocks, kBlock, 0, st>>>(ap, bp, p); break;
    default: return fail(WF2HIP_EINVAL, "op %d cannot accumulate", op);
  }
  return after_launch("typed_accumulate_sequential");
}

template <class T>
static int dispatch_nd(int op, Space s, T* a, const T* b) {
  if (s.total == 0) return 0;
  if (!a || !b) return fail(WF2HIP_EINVAL, "null tensor pointer");
  normalise(&s);
  if (typed_overlap(s, a, b, sizeof(T)))
    return fail(WF2HIP_EOVERLAP,
                "in-place op on partially overlapping windows of one buffer; copy one operand first");
  if (has_broadcast_axis(s, s.sa)) {
    if (op != WF2HIP_MOVE) return run_accumulate<T>(op, s, a, b);
    for (int r = 0; r < s.rank; r++)  // the last write wins
      if (s.sa[r] == 0 && s.shape[r] > 1) {
        s.off_b += s.sb[r] * (s.shape[r] - 1);
        s.shape[r] = 1;
      }
    s.total = 1;
    for (int r = 0; r < s.rank; r++) s.total *= s.shape[r];
    normalise(&s);
  }
  if (s.rank == 1 && s.sa[0] != 0)
    return dispatch_1d<T>(op, s.total, a + s.off_a, s.sa[0], b + s.off_b, s.sb[0], false);
  switch (op) {
    case WF2HIP_ADD: return run_generic<T, WF2HIP_ADD>(s, a, b);
    case WF2HIP_SUB: return run_generic<T, WF2HIP_SUB>(s, a, b);
    case WF2HIP_MUL: return run_generic<T, WF2HIP_MUL>(s, a, b);
    case WF2HIP_DIV: return run_generic<T, WF2HIP_DIV>(s, a, b);
    case WF2HIP_MOVE: return run_generic<T, WF2HIP_MOVE>(s, a, b);
    default: return fail(WF2HIP_EINVAL, "unknown binary op %d", op);
  }
}

// ---- compare / where ----------------------------------------------------------
// out <- (x OP y) ? then : else with all three of one element type
// (cl-waffe2-simd.c:385-468 define_cmp, :474-560 define_scmp with a scalar y).
// The reference's AVX2 body orders the lanes of the unsigned types as signed
// integers (simd/x86_64/avx2.h:198-200, 211-213, 224-226, 237-239: _mm256_cmpgt_epi*
// under the u32 / u16 / u8 names) while its scalar remainder compares them as
// unsigned; `signed_end` is the number of leading elements the 1-D entry points
// order that way to reproduce it.  The N-D entry points always compare in the
// element type's own order.
template <class T>
constexpr T sign_bit_of() {
  if constexpr (kIsInt<T>) {
    if constexpr (!((T)(-1) < (T)0)) return (T)((T)1 << (sizeof(T) * 8 - 1));
  }
  return (T)0;
}
template <class T>
constexpr T kSignBit = sign_bit_of<T>();

template <class T>
__device__ __forceinline__ bool holds_t(int op, T a, T b) {
  switch (op) {
    case WF2HIP_EQ: return a == b;
    case WF2HIP_LT: return a < b;
    case WF2HIP_LE: return a <= b;
    case WF2HIP_GT: return a > b;
    default: return a >= b;
  }
}

// x XOR bias with bias = the sign bit turns the unsigned order into the signed one
template <class T>
__device__ __forceinline__ T biased(T v, T bias) {
  if constexpr (kIsInt<T>)
    return (T)(v ^ bias);
  else
    return v;
}

// x, (y,) out contiguous and 16-byte aligned: the layout of typed_flat
template <class T, bool SCAL, bool NT>
__global__ __launch_bounds__(kBlock) void typed_cmp_flat(const T* __restrict__ x, const T* __restrict__ y,
                                                         T* __restrict__ out, size_t nvec, size_t signed_vecs, int op,
                                                         T ys, T then_value, T else_value) {
  constexpr int N = 16 / sizeof(T);
  constexpr int U = 4;
  using P = Pack<T, N>;
  typedef float f4 __attribute__((ext_vector_type(4)));
  const unsigned wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const size_t base = ((size_t)blockIdx.x * (kBlock / kWave) + wave) * kWave * U + lane;
  auto load = [](const T* p, size_t i) {
    const f4* q = reinterpret_cast<const f4*>(p) + i;
    return NT ? __builtin_nontemporal_load(q) : *q;
  };
  auto body = [&](auto full) {
    constexpr bool FULL = decltype(full)::value;
    f4 a[U], b[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        a[u] = load(x, i);
        if (!SCAL) b[u] = load(y, i);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t i = base + (size_t)u * kWave;
      if (FULL || i < nvec) {
        const T bias = i < signed_vecs ? kSignBit<T> : (T)0;
        const P pa = __builtin_bit_cast(P, a[u]), pb = __builtin_bit_cast(P, b[u]);
        const T yb = biased(ys, bias);
        P r;
#pragma unroll
        for (int k = 0; k < N; k++)
          r.v[k] = holds_t<T>(op, biased(pa.v[k], bias), SCAL ? yb : biased(pb.v[k], bias)) ? then_value : else_value;
        f4* q = reinterpret_cast<f4*>(out) + i;
        if (NT)
          __builtin_nontemporal_store(__builtin_bit_cast(f4, r), q);
        else
          *q = __builtin_bit_cast(f4, r);
      }
    }
  };
  constexpr bool kBranchFree = sizeof(T) < 4;
  if (kBranchFree && base - lane + (size_t)kWave * U <= nvec)
    body(std::true_type{});
  else
    body(std::false_type{});
}

template <class T>
struct TypedCmp {
  const T* x;
  const T* y;
  T* out;
  int32_t rank, op;
  int64_t total, signed_end;
  int64_t shape[WF2HIP_MAX_RANK], sa[WF2HIP_MAX_RANK], sb[WF2HIP_MAX_RANK], sc[WF2HIP_MAX_RANK];
  T ys, then_value, else_value;
};

// any strides, one element per thread, innermost axis fastest
template <class T, bool SCAL>
__global__ __launch_bounds__(kBlock) void typed_cmp_generic(TypedCmp<T> p) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= p.total) return;
  int64_t rem = i, ao = 0, bo = 0, co = 0;
  for (int r = p.rank - 1; r > 0; r--) {
    const int64_t q = rem / p.shape[r];
    const int64_t idx = rem - q * p.shape[r];
    rem = q;
    ao += idx * p.sa[r];
    bo += idx * p.sb[r];
    co += idx * p.sc[r];
  }
  ao += rem * p.sa[0];
  bo += rem * p.sb[0];
  co += rem * p.sc[0];
  const T bias = i < p.signed_end ? kSignBit<T> : (T)0;
  const T b = SCAL ? p.ys : p.y[bo];
  p.out[co] = holds_t<T>(p.op, biased(p.x[ao], bias), biased(b, bias)) ? p.then_value : p.else_value;
}

// `signed_end` counts elements of the (rank-1) space in iteration order; 0 for N-D calls
template <class T, bool SCAL>
static int run_cmp(int op, Space3 s, const T* x, const T* y, T* out, T ys, T then_value, T else_value,
                   int64_t signed_end) {
  if (op < WF2HIP_EQ || op > WF2HIP_GE) return fail(WF2HIP_EINVAL, "unknown compare op %d", op);
  if (s.total == 0) return 0;
  if (!x || !out || (!SCAL && !y)) return fail(WF2HIP_EINVAL, "null tensor pointer");
  if (SCAL) {
    y = x;
    for (int r = 0; r < s.rank; r++) s.sb[r] = s.sa[r];
    s.off_b = s.off_a;
  }
  // a stride-0 axis of `out` keeps what the sequential loop writes last (its scalar
  // loop, which compares in the element type's own order)
  for (int r = 0; r < s.rank; r++)
    if (s.sc[r] == 0 && s.shape[r] > 1) {
      s.off_a += s.sa[r] * (s.shape[r] - 1);
      s.off_b += s.sb[r] * (s.shape[r] - 1);
      s.shape[r] = 1;
      signed_end = 0;
    }
  normalise3(&s);
  if (hazardous3(s, out, s.sa, s.off_a, x) || hazardous3(s, out, s.sb, s.off_b, y))
    return fail(WF2HIP_EOVERLAP, "compare writes into a window that partially overlaps an input");
  hipStream_t st = rt().stream;
  const T* xp = x + s.off_a;
  const T* yp = y + s.off_b;
  T* op_ = out + s.off_c;
  constexpr int N = 16 / (int)sizeof(T);
  int64_t done = 0;
  const bool flat = s.rank == 1 && s.total >= N && s.sa[0] == 1 && s.sb[0] == 1 && s.sc[0] == 1 &&
                    (((uintptr_t)xp | (uintptr_t)yp | (uintptr_t)op_) & 15u) == 0;
  if (flat) {
    const int64_t nvec = s.total / N;
    const int64_t blocks = ceil_div(nvec, (int64_t)kBlock * 4);
    if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
    const size_t signed_vecs = (size_t)(signed_end / N);  // a multiple of 2 N elements by construction
    if (nvec * 16 * (SCAL ? 2 : 3) >= ((int64_t)192 << 20))
      typed_cmp_flat<T, SCAL, true><<<(uint32_t)blocks, kBlock, 0, st>>>(xp, yp, op_, (size_t)nvec, signed_vecs, op, ys,
                                                                        then_value, else_value);
    else
      typed_cmp_flat<T, SCAL, false><<<(uint32_t)blocks, kBlock, 0, st>>>(xp, yp, op_, (size_t)nvec, signed_vecs, op, ys,
                                                                         then_value, else_value);
    WF2_TRY(after_launch("typed_cmp_flat"));
    done = nvec * N;
    if (done == s.total) return 0;
  }
  TypedCmp<T> p;
  p.rank = s.rank;
  p.op = op;
  for (int r = 0; r < s.rank; r++) {
    p.shape[r] = s.shape[r];
    p.sa[r] = s.sa[r];
    p.sb[r] = s.sb[r];
    p.sc[r] = s.sc[r];
  }
  // after the vector kernel only the tail of a rank-1 run is left
  p.x = xp + done * s.sa[0];
  p.y = yp + done * s.sb[0];
  p.out = op_ + done * s.sc[0];
  if (done > 0) p.shape[0] = s.total - done;
  p.total = s.total - done;
  p.signed_end = signed_end > done ? signed_end - done : 0;
  p.ys = ys;
  p.then_value = then_value;
  p.else_value = else_value;
  const int64_t blocks = ceil_div(p.total, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
  typed_cmp_generic<T, SCAL><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  return after_launch("typed_cmp_generic");
}

// the reference's 1-D kernels: the leading (n / lanes) * lanes elements go through
// its 256-bit body when inco >= 1 (lanes = 32 bytes / element size)
template <class T, bool SCAL>
static int cmp_1d(int op, long n, const T* x, long incx, const T* y, long incy, T* out, long inco, T ys,
                  T then_value, T else_value) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  Space3 s;
  s.rank = 1;
  s.shape[0] = n;
  s.sa[0] = incx;
  s.sb[0] = SCAL ? incx : incy;
  s.sc[0] = inco;
  s.total = n;
  constexpr long lanes = 32 / (long)sizeof(T);
  const int64_t signed_end = (kSignBit<T> != (T)0 && inco >= 1) ? (n / lanes) * lanes : 0;
  return run_cmp<T, SCAL>(op, s, x, y, out, ys, then_value, else_value, signed_end);
}

// ---- :double unary math --------------------------------------------------------
// out <- f(x) for :double tensors (waffe2_d{sin,...}, cl-waffe2-simd.c:586-706; pow :708-768).
// The reference mixes SLEEF u10 (blocks of four) and libm (remainder), so its own
// results vary within an ulp from element to element; here every element goes
// through the device math library's binary64 routine.

template <int OP>
__device__ __forceinline__ double dmath(double x, double p) {
  if constexpr (OP == WF2HIP_SIN) return ::sin(x);
  else if constexpr (OP == WF2HIP_COS) return ::cos(x);
  else if constexpr (OP == WF2HIP_TANH) return ::tanh(x);
  else if constexpr (OP == WF2HIP_LOG) return ::log(x);
  else if constexpr (OP == WF2HIP_EXP) return ::exp(x);
  else if constexpr (OP == WF2HIP_SQRT) return ::sqrt(x);
  else if constexpr (OP == WF2HIP_ABS) return ::fabs(x);
  else if constexpr (OP == WF2HIP_TAN) return ::tan(x);
  else if constexpr (OP == WF2HIP_ASIN) return ::asin(x);
  else if constexpr (OP == WF2HIP_ACOS) return ::acos(x);
  else if constexpr (OP == WF2HIP_ATAN) return ::atan(x);
  else if constexpr (OP == WF2HIP_SINH) return ::sinh(x);
  else if constexpr (OP == WF2HIP_COSH) return ::cosh(x);
  else if constexpr (OP == WF2HIP_LOG2) return ::log2(x);
  else if constexpr (OP == WF2HIP_LOG10) return ::log10(x);
  else if constexpr (OP == WF2HIP_LOG1P) return x == 0.0 ? x : ::log1p(x);  // keeps the sign of -0
  else if constexpr (OP == WF2HIP_POW) return ::pow(x, p);
  else if constexpr (OP == WF2HIP_SIGN) return x > 0.0 ? 1.0 : (x < 0.0 ? -1.0 : x);
  else if constexpr (OP == WF2HIP_SQUARE) return x * x;
  else if constexpr (OP == WF2HIP_ASINH) return ::asinh(x);
  else if constexpr (OP == WF2HIP_ACOSH) return ::acosh(x);
  else if constexpr (OP == WF2HIP_ATANH) return ::atanh(x);
  else return 1.0 / x;  // WF2HIP_INV
}

// x and out contiguous, 16-byte aligned: two elements per access, four accesses per lane
template <int OP, bool NT>
__global__ __launch_bounds__(kBlock) void dunary_flat(const double* __restrict__ x, double* __restrict__ out, size_t nvec,
                                                      double p) {
  typedef double d2 __attribute__((ext_vector_type(2)));
  constexpr int U = 4;
  const unsigned wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const size_t base = ((size_t)blockIdx.x * (kBlock / kWave) + wave) * kWave * U + lane;
  const d2* xv = reinterpret_cast<const d2*>(x);
  d2* ov = reinterpret_cast<d2*>(out);
  d2 a[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const size_t i = base + (size_t)u * kWave;
    if (i < nvec) a[u] = NT ? __builtin_nontemporal_load(xv + i) : xv[i];
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const size_t i = base + (size_t)u * kWave;
    if (i < nvec) {
      d2 r;
      r.x = dmath<OP>(a[u].x, p);
      r.y = dmath<OP>(a[u].y, p);
      if (NT)
        __builtin_nontemporal_store(r, ov + i);
      else
        ov[i] = r;
    }
  }
}

template <int OP>
__global__ __launch_bounds__(kBlock) void dunary_generic(double* dst, const double* src, TypedGen g, double p) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= g.total) return;
  int64_t rem = i, d = 0, q = 0;
  for (int r = g.rank - 1; r > 0; r--) {
    const int64_t quot = rem / g.shape[r];
    const int64_t idx = rem - quot * g.shape[r];
    rem = quot;
    d += idx * g.sd[r];
    q += idx * g.ss[r];
  }
  d += rem * g.sd[0];
  q += rem * g.ss[0];
  dst[d] = dmath<OP>(src[q], p);
}

// `s`: a = X (source), b = OUT
template <int OP>
static int run_dunary(Space s, const double* x, double* out, double p) {
  if (s.total == 0) return 0;
  if (!x || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  // a stride-0 axis of OUT keeps what the sequential loop writes last
  for (int r = 0; r < s.rank; r++)
    if (s.sb[r] == 0 && s.shape[r] > 1) {
      s.off_a += s.sa[r] * (s.shape[r] - 1);
      s.shape[r] = 1;
    }
  s.total = 1;
  for (int r = 0; r < s.rank; r++) s.total *= s.shape[r];
  normalise(&s);
  if (typed_overlap(s, x, out, sizeof(double)))
    return fail(WF2HIP_EOVERLAP, "out partially overlaps x; copy one of them first");
  hipStream_t st = rt().stream;
  const double* xp = x + s.off_a;
  double* op_ = out + s.off_b;
  int64_t done = 0;
  if (s.rank == 1 && s.sa[0] == 1 && s.sb[0] == 1 && s.total >= 2 && aligned16(xp) && aligned16(op_)) {
    const int64_t nvec = s.total / 2;
    const int64_t blocks = ceil_div(nvec, (int64_t)kBlock * 4);
    if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
    if (nvec * 32 >= ((int64_t)192 << 20))
      dunary_flat<OP, true><<<(uint32_t)blocks, kBlock, 0, st>>>(xp, op_, (size_t)nvec, p);
    else
      dunary_flat<OP, false><<<(uint32_t)blocks, kBlock, 0, st>>>(xp, op_, (size_t)nvec, p);
    WF2_TRY(after_launch("dunary_flat"));
    done = nvec * 2;
    if (done == s.total) return 0;
  }
  TypedGen g;
  g.rank = s.rank;
  for (int r = 0; r < s.rank; r++) {
    g.shape[r] = s.shape[r];
    g.sd[r] = s.sb[r];
    g.ss[r] = s.sa[r];
  }
  if (done > 0) g.shape[0] = s.total - done;  // the odd last element of a flat run
  g.total = s.total - done;
  const int64_t blocks = ceil_div(g.total, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
  dunary_generic<OP><<<(uint32_t)blocks, kBlock, 0, st>>>(op_ + done * s.sb[0], xp + done * s.sa[0], g, p);
  return after_launch("dunary_generic");
}

static int dispatch_dunary(int op, const Space& s, const double* x, double* out, double p) {
  switch (op) {
#define WF2_DUNARY_CASE(OP) case OP: return run_dunary<OP>(s, x, out, p);
    WF2_DUNARY_CASE(WF2HIP_SIN) WF2_DUNARY_CASE(WF2HIP_COS) WF2_DUNARY_CASE(WF2HIP_TANH) WF2_DUNARY_CASE(WF2HIP_LOG)
    WF2_DUNARY_CASE(WF2HIP_EXP) WF2_DUNARY_CASE(WF2HIP_SQRT) WF2_DUNARY_CASE(WF2HIP_ABS) WF2_DUNARY_CASE(WF2HIP_TAN)
    WF2_DUNARY_CASE(WF2HIP_ASIN) WF2_DUNARY_CASE(WF2HIP_ACOS) WF2_DUNARY_CASE(WF2HIP_ATAN) WF2_DUNARY_CASE(WF2HIP_SINH)
    WF2_DUNARY_CASE(WF2HIP_COSH) WF2_DUNARY_CASE(WF2HIP_LOG2) WF2_DUNARY_CASE(WF2HIP_LOG10)
    WF2_DUNARY_CASE(WF2HIP_LOG1P) WF2_DUNARY_CASE(WF2HIP_POW) WF2_DUNARY_CASE(WF2HIP_SIGN)
    WF2_DUNARY_CASE(WF2HIP_SQUARE) WF2_DUNARY_CASE(WF2HIP_ASINH) WF2_DUNARY_CASE(WF2HIP_ACOSH)
    WF2_DUNARY_CASE(WF2HIP_ATANH)
#undef WF2_DUNARY_CASE
    default: return fail(WF2HIP_EINVAL, "unary op %d has no :double kernel", op);
  }
}

static int dunary_1d(int op, long n, const double* x, long incx, double* out, long inco, double p) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  Space s;
  s.rank = 1;
  s.shape[0] = n;
  s.sa[0] = incx;
  s.sb[0] = inco;
  s.total = n;
  return dispatch_dunary(op, s, x, out, p);
}

}  // namespace wf2

using namespace wf2;

#define WF2_FOR_DTYPE(dtype, ...)                                                     \
  switch (dtype) {                                                                      \
    case WF2HIP_F64: { using T = double; __VA_ARGS__; }                                        \
    case WF2HIP_I32: { using T = int32_t; __VA_ARGS__; }                                       \
    case WF2HIP_U32: { using T = uint32_t; __VA_ARGS__; }                                      \
    case WF2HIP_I16: { using T = int16_t; __VA_ARGS__; }                                       \
    case WF2HIP_U16: { using T = uint16_t; __VA_ARGS__; }                                      \
    case WF2HIP_I8: { using T = int8_t; __VA_ARGS__; }                                         \
    case WF2HIP_U8: { using T = uint8_t; __VA_ARGS__; }                                        \
    default: return fail(WF2HIP_EINVAL, "unknown element type %d (:float has its own entry points)", dtype); \
  }

static size_t dtype_width(int dtype) {
  switch (dtype) {
    case WF2HIP_F64: return 8;
    case WF2HIP_I32: case WF2HIP_U32: return 4;
    case WF2HIP_I16: case WF2HIP_U16: return 2;
    case WF2HIP_I8: case WF2HIP_U8: return 1;
    default: return 0;
  }
}

WF2_API int wf2hip_binary_1d_typed(int dtype, int op, long n, void* x, long incx, const void* y, long incy) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative length");
  if (n == 0) return 0;
  if (!x || !y) return fail(WF2HIP_EINVAL, "null tensor pointer");
  // The kernels read y while other lanes write x.  Two runs over one buffer are only safe when
  // they are the same run (x <- x op x); anything else depends on the order of the writes, which
  // the N-D entry point refuses as well.
  {
    const size_t width = dtype_width(dtype);
    if (width == 0) return fail(WF2HIP_EINVAL, "unknown element type %d (:float has its own entry points)", dtype);
    auto span = [&](const void* base, long inc, uintptr_t* lo, uintptr_t* hi) {
      const int64_t reach = (int64_t)(n - 1) * inc * (int64_t)width;
      const uintptr_t b = (uintptr_t)base;
      *lo = reach < 0 ? b + reach : b;
      *hi = (reach < 0 ? b : b + reach) + width;
    };
    uintptr_t xlo, xhi, ylo, yhi;
    span(x, incx, &xlo, &xhi);
    span(y, incy, &ylo, &yhi);
    const bool same_run = x == y && incx == incy;
    if (xlo < yhi && ylo < xhi && !same_run)
      return fail(WF2HIP_EOVERLAP, "in-place op between overlapping runs of one buffer; copy one operand first");
  }
  WF2_FOR_DTYPE(dtype, return dispatch_1d<T>(op, n, (T*)x, incx, (const T*)y, incy, true));
}

WF2_API int wf2hip_binary_nd_typed(int dtype, int op, const wf2hip_view2* v, void* a, const void* b) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(load_space(v, &s));
  WF2_FOR_DTYPE(dtype, return dispatch_nd<T>(op, s, (T*)a, (const T*)b));
}

WF2_API int wf2hip_inv_1d_typed(int dtype, long n, void* x, long incx) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative length");
  if (n == 0) return 0;
  if (!x) return fail(WF2HIP_EINVAL, "null tensor pointer");
  WF2_FOR_DTYPE(dtype, {
    typed_inv<T><<<incx == 0 ? 1u : grid_for(n, 1), kBlock, 0, rt().stream>>>((T*)x, incx, n);
    return after_launch("typed_inv");
  });
}

// The reference's own names, one per element type: waffe2_dadd -> wf2hip_dadd, ...
#define WF2_TYPED_ARITH(prefix, T, code)                                                               \
  WF2_API int wf2hip_##prefix##add(long n, T* x, long incx, const T* y, long incy) {                   \
    return wf2hip_binary_1d_typed(code, WF2HIP_ADD, n, x, incx, y, incy);                              \
  }                                                                                                    \
  WF2_API int wf2hip_##prefix##sub(long n, T* x, long incx, const T* y, long incy) {                   \
    return wf2hip_binary_1d_typed(code, WF2HIP_SUB, n, x, incx, y, incy);                              \
  }                                                                                                    \
  WF2_API int wf2hip_##prefix##mul(long n, T* x, long incx, const T* y, long incy) {                   \
    return wf2hip_binary_1d_typed(code, WF2HIP_MUL, n, x, incx, y, incy);                              \
  }                                                                                                    \
  WF2_API int wf2hip_##prefix##div(long n, T* x, long incx, const T* y, long incy) {                   \
    return wf2hip_binary_1d_typed(code, WF2HIP_DIV, n, x, incx, y, incy);                              \
  }                                                                                                    \
  WF2_API int wf2hip_##prefix##inv(long n, T* x, long incx) { return wf2hip_inv_1d_typed(code, n, x, incx); }

#define WF2_TYPED_FAMILY(prefix, T, code)                                                              \
  WF2_TYPED_ARITH(prefix, T, code)                                                                     \
  WF2_API int wf2hip_##prefix##copy(long n, T* x, long incx, const T* y, long incy) {                  \
    return wf2hip_binary_1d_typed(code, WF2HIP_MOVE, n, x, incx, y, incy);                             \
  }

WF2_TYPED_ARITH(d, double, WF2HIP_F64)
// :double moves are dcopy_ in the reference (source/backends/cpu/arithmetic.lisp:39-61): BLAS argument order
WF2_API int wf2hip_dcopy(long n, const double* src, long incsrc, double* dst, long incdst) {
  return wf2hip_binary_1d_typed(WF2HIP_F64, WF2HIP_MOVE, n, dst, incdst, src, incsrc);
}
WF2_TYPED_FAMILY(i32, int32_t, WF2HIP_I32)
WF2_TYPED_FAMILY(u32, uint32_t, WF2HIP_U32)
WF2_TYPED_FAMILY(i16, int16_t, WF2HIP_I16)
WF2_TYPED_FAMILY(u16, uint16_t, WF2HIP_U16)
WF2_TYPED_FAMILY(i8, int8_t, WF2HIP_I8)
WF2_TYPED_FAMILY(u8, uint8_t, WF2HIP_U8)

WF2_API int wf2hip_compare_nd_typed(int dtype, int op, const wf2hip_view3* v, const void* x, const void* y, void* out,
                                    double then_value, double else_value) {
  WF2_TRY(require_init());
  Space3 s;
  WF2_TRY(load_space3(v, &s));
  WF2_FOR_DTYPE(dtype, return (run_cmp<T, false>(op, s, (const T*)x, (const T*)y, (T*)out, (T)0, (T)then_value,
                                                 (T)else_value, 0)));
}

WF2_API int wf2hip_where_nd_typed(int dtype, int op, const wf2hip_view2* v, const void* x, void* out, double scal,
                                  double then_value, double else_value) {
  WF2_TRY(require_init());
  Space two;
  WF2_TRY(load_space(v, &two));
  Space3 s;
  s.rank = two.rank;
  s.total = two.total;
  for (int r = 0; r < two.rank; r++) {
    s.shape[r] = two.shape[r];
    s.sa[r] = s.sb[r] = two.sa[r];
    s.sc[r] = two.sb[r];
  }
  s.off_a = s.off_b = two.off_a;
  s.off_c = two.off_b;
  WF2_FOR_DTYPE(dtype, return (run_cmp<T, true>(op, s, (const T*)x, nullptr, (T*)out, (T)scal, (T)then_value,
                                                (T)else_value, 0)));
}

// the reference's own names: waffe2_<prefix>{eq,lt,le,gt,ge} and ..._scal
#define WF2_DEFINE_TYPED_CMP(prefix, T, name, OP)                                                                  \
  WF2_API int wf2hip_##prefix##name(long n, const T* x, long incx, const T* y, long incy, T* out, long inco,      \
                                    T then_value, T else_value) {                                                  \
    return cmp_1d<T, false>(OP, n, x, incx, y, incy, out, inco, (T)0, then_value, else_value);                    \
  }                                                                                                                \
  WF2_API int wf2hip_##prefix##name##_scal(long n, const T* x, long incx, T* out, long inco, T y, T then_value,  \
                                           T else_value) {                                                         \
    return cmp_1d<T, true>(OP, n, x, incx, nullptr, 0, out, inco, y, then_value, else_value);                     \
  }
#define WF2_DEFINE_TYPED_CMPS(prefix, T)          \
  WF2_DEFINE_TYPED_CMP(prefix, T, eq, WF2HIP_EQ)  \
  WF2_DEFINE_TYPED_CMP(prefix, T, lt, WF2HIP_LT)  \
  WF2_DEFINE_TYPED_CMP(prefix, T, le, WF2HIP_LE)  \
  WF2_DEFINE_TYPED_CMP(prefix, T, gt, WF2HIP_GT)  \
  WF2_DEFINE_TYPED_CMP(prefix, T, ge, WF2HIP_GE)

WF2_DEFINE_TYPED_CMPS(d, double)
WF2_DEFINE_TYPED_CMPS(i32, int32_t)
WF2_DEFINE_TYPED_CMPS(u32, uint32_t)
WF2_DEFINE_TYPED_CMPS(i16, int16_t)
WF2_DEFINE_TYPED_CMPS(u16, uint16_t)
WF2_DEFINE_TYPED_CMPS(i8, int8_t)
WF2_DEFINE_TYPED_CMPS(u8, uint8_t)

// OUT <- f(X) on a :double tensor (view: a = X, b = OUT); `p` is the exponent of WF2HIP_POW
WF2_API int wf2hip_unary_nd_typed(int dtype, int op, const wf2hip_view2* v, const void* x, void* out, double p) {
  WF2_TRY(require_init());
  if (dtype != WF2HIP_F64)
    return fail(WF2HIP_EUNSUPPORTED, "unary math exists for :float and :double only (element type %d)", dtype);
  Space s;
  WF2_TRY(load_space(v, &s));
  return dispatch_dunary(op, s, (const double*)x, (double*)out, p);
}

#define WF2_DEFINE_DUNARY(name, OP)                                                           \
  WF2_API int wf2hip_d##name(long n, const double* x, long incx, double* out, long inco) {    \
    return dunary_1d(OP, n, x, incx, out, inco, 0.0);                                        \
  }
WF2_DEFINE_DUNARY(sin, WF2HIP_SIN)
WF2_DEFINE_DUNARY(cos, WF2HIP_COS)
WF2_DEFINE_DUNARY(tanh, WF2HIP_TANH)
WF2_DEFINE_DUNARY(log, WF2HIP_LOG)
WF2_DEFINE_DUNARY(exp, WF2HIP_EXP)
WF2_DEFINE_DUNARY(sqrt, WF2HIP_SQRT)
WF2_DEFINE_DUNARY(abs, WF2HIP_ABS)
WF2_DEFINE_DUNARY(tan, WF2HIP_TAN)
WF2_DEFINE_DUNARY(asin, WF2HIP_ASIN)
WF2_DEFINE_DUNARY(acos, WF2HIP_ACOS)
WF2_DEFINE_DUNARY(atan, WF2HIP_ATAN)
WF2_DEFINE_DUNARY(sinh, WF2HIP_SINH)
WF2_DEFINE_DUNARY(cosh, WF2HIP_COSH)
WF2_DEFINE_DUNARY(log2, WF2HIP_LOG2)
WF2_DEFINE_DUNARY(log10, WF2HIP_LOG10)
WF2_DEFINE_DUNARY(log1p, WF2HIP_LOG1P)
WF2_API int wf2hip_dpow(long n, const double* x, long incx, double p, double* out, long inco) {
  return dunary_1d(WF2HIP_POW, n, x, incx, out, inco, p);
}
