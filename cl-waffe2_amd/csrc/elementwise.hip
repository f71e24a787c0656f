// elementwise.hip -- fp32 element-wise kernels over offset/stride/broadcast
// views: a <- a op b, a <- b (copy), out <- f(x).
//
// Reference semantics: cl-waffe2-simd.c:153-250 (x[i*incx] <- x[i*incx] op
// y[i*incy], in place in x), :586-768 (out <- f(x), out <- x^p), BLAS scopy
// for MoveTensorNode (source/backends/cpu/arithmetic.lisp:39-61,125-144).
// The reference reaches N-D views by wrapping those 1-D kernels in host loops
// (call-with-view.lisp:112-229) -- thousands of calls for a row-broadcast or a
// sliced operand; here a node is ONE launch over the normalised space.
//
// All of these are HBM-bound (8 or 12 bytes per element against a handful of
// VALU instructions), so the kernels are organised around 16-byte coalesced
// accesses: the "rows" kernel walks an innermost contiguous axis with float4
// loads, several independent loads in flight per thread, and resolves the
// outer axes (arbitrary strides, broadcast, slices) once per thread; the
// "tile" kernel turns a transposed operand into coalesced reads AND writes
// through an LDS tile; the "generic" kernel covers what is left.
//
// Arithmetic is IEEE binary32 with contraction disabled at build time
// (-ffp-contract=off) so a+b, a*b ... are bit-identical to _mm256_*_ps.
#include "wf2_common.h"
#include "wf2_fastdiv.h"
#include "wf2_math.h"
#include "wf2_view.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));

// Streaming hint: a node whose footprint is far beyond the 256 MB Infinity
// Cache gains ~10-15 % of HBM bandwidth when its loads and stores are marked
// non-temporal (measured on MI355X: 5.3 -> 6.2 TB/s for x += y at 2^26);
// smaller nodes keep the default policy so that the next node finds their
// output in cache.
constexpr int64_t kStreamingBytes = (int64_t)192 << 20;

// Four consecutive floats as one access.  The vector type is declared 4-byte
// aligned: gfx950 runs with unaligned access enabled, so the compiler still emits a
// single global_load / global_store_dwordx4 and the hardware takes any float
// address.  Views that start an odd number of elements into their storage
// (x[1:], A[:, 1:4097]) therefore use the vector kernels like aligned ones
// (x[1:] += y at 2^26: 70 % of the HBM peak through scalar accesses).
typedef f4 f4u __attribute__((aligned(4)));

template <bool NT>
__device__ __forceinline__ f4 load4(const float* p) {
  if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const f4u*>(p));
  return *reinterpret_cast<const f4u*>(p);
}

template <bool NT>
__device__ __forceinline__ void store4(float* p, f4 v) {
  if constexpr (NT)
    __builtin_nontemporal_store(v, reinterpret_cast<f4u*>(p));
  else
    *reinterpret_cast<f4u*>(p) = v;
}

// ---- functors: operator()(dst_value, src_value) ---------------------------
struct OpAdd { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float d, float s) const { return d + s; } };
struct OpSub { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float d, float s) const { return d - s; } };
struct OpMul { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float d, float s) const { return d * s; } };
struct OpDiv { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float d, float s) const { return d / s; } };
struct OpMove { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float, float s) const { return s; } };
struct OpSin { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return sinf_(s); } };
struct OpCos { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return cosf_(s); } };
struct OpTanh { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return tanhf_(s); } };
struct OpLog { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return logf_(s); } };
struct OpExp { static constexpr int kFlatU = 1; __device__ __forceinline__ float operator()(float, float s) const { return expf_(s); } };
struct OpSqrt { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float, float s) const { return sqrtf_(s); } };
struct OpAbs { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float, float s) const { return absf_(s); } };
struct OpTan { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return tanf_(s); } };
struct OpASin { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return asinf_(s); } };
struct OpACos { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return acosf_(s); } };
struct OpATan { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return atanf_(s); } };
struct OpSinH { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return sinhf_(s); } };
struct OpCosH { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return coshf_(s); } };
struct OpLog2 { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return log2f_(s); } };
struct OpLog10 { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return log10f_(s); } };
struct OpLog1p { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return log1pf_(s); } };
struct OpSign { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float, float s) const { return signf_(s); } };
struct OpSquare { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float, float s) const { return s * s; } };
struct OpASinH { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return asinhf_(s); } };
struct OpACosH { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return acoshf_(s); } };
struct OpATanH { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return atanhf_(s); } };
struct OpInv { static constexpr int kFlatU = 4; __device__ __forceinline__ float operator()(float, float s) const { return 1.0f / s; } };
struct OpGelu { static constexpr int kFlatU = 2; __device__ __forceinline__ float operator()(float, float s) const { return gelu_tanh_f(s); } };
// The activation recipes of nn/activation.lisp as single kernels; each performs
// the binary32 operations of its node sequence in the same order, so the result
// is bit-identical to running the nodes (8 bytes per element instead of 20-36).
struct OpRelu {
  static constexpr int kFlatU = 4;
  __device__ __forceinline__ float operator()(float, float s) const { return s * (s > 0.0f ? 1.0f : 0.0f); }
};
struct OpLeakyRelu {
  static constexpr int kFlatU = 4;
  float slope;
  __device__ __forceinline__ float operator()(float, float s) const { return s * (s >= 0.0f ? 1.0f : slope); }
};
struct OpSigmoid {
  static constexpr int kFlatU = 2;
  __device__ __forceinline__ float operator()(float, float s) const {
    const float e = expf_(-1.0f * s);
    return 1.0f / (1.0f + e);
  }
};
// dOUT <- dOUT f'(X) for the same activations: the MulNode of the upstream gradient with
// the derivative recipe (A>scal for ReLU, A>=scal with slope for leaky ReLU, s (1 - s) with
// s recomputed for the sigmoid -- each the binary32 operations of that composition in the
// same order, so bit-identical to it) in one pass, 12 bytes per element.
struct OpReluGrad {
  static constexpr int kFlatU = 4;
  __device__ __forceinline__ float operator()(float d, float s) const { return d * (s > 0.0f ? 1.0f : 0.0f); }
};
struct OpLeakyReluGrad {
  static constexpr int kFlatU = 4;
  float slope;
  __device__ __forceinline__ float operator()(float d, float s) const { return d * (s >= 0.0f ? 1.0f : slope); }
};
struct OpSigmoidGrad {
  static constexpr int kFlatU = 4;
  __device__ __forceinline__ float operator()(float d, float s) const {
    const float e = expf_(-1.0f * s);
    const float sg = 1.0f / (1.0f + e);
    return d * (sg * (1.0f + -1.0f * sg));  // (!sub 1 s) is 1 + (-1 s)
  }
};
struct OpGeluGrad {
  static constexpr int kFlatU = 4;
  __device__ __forceinline__ float operator()(float d, float s) const { return d * gelu_tanh_grad_f(s); }
};
struct OpPow {
  static constexpr int kFlatU = 2;
  float p;
  __device__ __forceinline__ float operator()(float, float s) const { return powf_(s, p); }
};

// (x OP y) ? then : else with a scalar y: Where-Operation-Node's kernel
// (cl-waffe2-simd.c:474-513).  All five predicates are the ordered ones: false
// when x or y is NaN.
struct OpWhere {
  static constexpr int kFlatU = 4;
  int op;
  float y, then_value, else_value;
  __device__ __forceinline__ float operator()(float, float s) const {
    bool t;
    switch (op) {
      case WF2HIP_EQ: t = s == y; break;
      case WF2HIP_LT: t = s < y; break;
      case WF2HIP_LE: t = s <= y; break;
      case WF2HIP_GT: t = s > y; break;
      default: t = s >= y; break;
    }
    return t ? then_value : else_value;
  }
};

// ---- flat kernel -------------------------------------------------------------
// Both tensors one contiguous run (or src a single broadcast value): the node
// the reference flattens to a single 1-D call (do-compiled-loop.lisp:113-137).
// Workgroups live for ~2 us each at this size, so the prologue is kept to a
// handful of instructions: no index decomposition, no runtime layout flags.
// Each thread issues all its 16-byte loads before the first use.
// LAYOUT 0: the four accesses of a thread are a workgroup-width apart (every
// load instruction of the workgroup covers 4 KB contiguous); LAYOUT 1: each
// wavefront owns 4 KB contiguous per stream.  Measured at 2^26 elements with
// cold operands: three streams (x <- x op y) 6.66 TB/s with layout 1 against
// 6.59 with layout 0; two streams (copy, unary) 6.45 with layout 0 against 6.25.
// Functors with a long binary64 body (transcendentals) take two vectors per
// thread instead of four: measured 4-7 % faster at 2^26 (exp 5.91 -> 6.36 TB/s).
struct FlatEdges {
  int head, tail;
};
struct NoEdges {};

template <class F, bool ReadDst, bool SrcBroadcast, bool NT, int LAYOUT, int kFlatU, class Edges = NoEdges>
__global__ __launch_bounds__(kBlock) void ew_flat(float* __restrict__ dst,
                                                  const float* __restrict__ src, size_t nvec, F f, Edges edges = Edges()) {
  // the elements before the first whole vector of the body and after the last one (the
  // aligned, whole-vector case is a kernel of its own without this prologue)
  if constexpr (__is_same(Edges, FlatEdges)) {
    const int head = edges.head, tail = edges.tail;
    if (blockIdx.x == 0 && (int)threadIdx.x < head + tail) {
      const int t = threadIdx.x;
      const ptrdiff_t at = t < head ? (ptrdiff_t)t - head : (ptrdiff_t)(4 * nvec) + (t - head);
      const float a = ReadDst ? dst[at] : 0.0f;
      dst[at] = f(a, SrcBroadcast ? src[0] : src[at]);
    }
  }
  size_t base;
  if (LAYOUT == 0) {
    base = (size_t)blockIdx.x * kBlock * kFlatU + threadIdx.x;
  } else {
    const unsigned wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
    base = ((size_t)blockIdx.x * (kBlock / kWave) + wave) * kWave * kFlatU + lane;
  }
  constexpr unsigned step = LAYOUT == 0 ? kBlock : kWave;
  f4 dv[kFlatU], sv[kFlatU];
  float sb = 0.0f;
  if (SrcBroadcast) sb = src[0];
  // Two-stream forms (copy, unary, scalar operand): a workgroup that lies wholly
  // inside the array runs without per-lane bounds checks, so that all loads are
  // issued back to back (+4 % at 2^26: copy 6.10 -> 6.33 TB/s).  The
  // three-stream form x <- x op y is the other way round on MI355X: the
  // per-access predicated form below, in which the compiler spaces the four
  // load pairs with the bounds logic, measured 6.62 TB/s against 6.33 unguarded.
  constexpr bool kThreeStreams = ReadDst && !SrcBroadcast;
  const bool full = ((size_t)blockIdx.x + 1) * kBlock * kFlatU <= nvec;
  if (!kThreeStreams && full) {
#pragma unroll
    for (int u = 0; u < kFlatU; u++) {
      size_t i = base + (size_t)u * step;
      if (ReadDst) dv[u] = load4<NT>(dst + 4 * i);
      if (!SrcBroadcast) sv[u] = load4<NT>(src + 4 * i);
    }
#pragma unroll
    for (int u = 0; u < kFlatU; u++) {
      size_t i = base + (size_t)u * step;
      f4 a = ReadDst ? dv[u] : f4{0.f, 0.f, 0.f, 0.f};
      f4 b = SrcBroadcast ? f4{sb, sb, sb, sb} : sv[u];
      f4 r;
      r.x = f(a.x, b.x);
      r.y = f(a.y, b.y);
      r.z = f(a.z, b.z);
      r.w = f(a.w, b.w);
      store4<NT>(dst + 4 * i, r);
    }
    return;
  }
#pragma unroll
  for (int u = 0; u < kFlatU; u++) {
    size_t i = base + (size_t)u * step;
    if (i < nvec) {
      if (ReadDst) dv[u] = load4<NT>(dst + 4 * i);
      if (!SrcBroadcast) sv[u] = load4<NT>(src + 4 * i);
    }
  }
#pragma unroll
  for (int u = 0; u < kFlatU; u++) {
    size_t i = base + (size_t)u * step;
    if (i < nvec) {
      f4 a = ReadDst ? dv[u] : f4{0.f, 0.f, 0.f, 0.f};
      f4 b = SrcBroadcast ? f4{sb, sb, sb, sb} : sv[u];
      f4 r;
      r.x = f(a.x, b.x);
      r.y = f(a.y, b.y);
      r.z = f(a.z, b.z);
      r.w = f(a.w, b.w);
      store4<NT>(dst + 4 * i, r);
    }
  }
}

// ---- rows kernel ------------------------------------------------------------
constexpr int kMaxOuter = WF2HIP_MAX_RANK - 1;

struct RowsParams {
  float* dst;
  const float* src;
  int64_t n0;     // extent of the innermost (contiguous) axis
  uint32_t nrows; // product of the outer extents
  int32_t src_inner;  // 1: src contiguous along the inner axis, 0: broadcast
  int32_t nouter;
  int32_t tpr_log2;  // threads that share one row segment
  uint32_t chunks_per_row;
  uint32_t oshape[kMaxOuter];  // outer axes, innermost of them first
  int64_t odst[kMaxOuter];
  int64_t osrc[kMaxOuter];
};

template <class F, bool ReadDst, int VEC, int U, bool NT = false>
__global__ __launch_bounds__(kBlock) void ew_rows(RowsParams p, F f) {
  const int tpr = 1 << p.tpr_log2;
  const int rpb = kBlock >> p.tpr_log2;
  const int lane = threadIdx.x & (tpr - 1);
  const int sub = threadIdx.x >> p.tpr_log2;
  const uint32_t rblock = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk = blockIdx.x - rblock * p.chunks_per_row;
  const uint32_t row = rblock * rpb + sub;
  if (row >= p.nrows) return;

  int64_t doff = 0, soff = 0;
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
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  float* __restrict__ d = p.dst + doff;
  const float* __restrict__ s = p.src + soff;
  const int64_t col0 = (int64_t)chunk * U * tpr * VEC + (int64_t)lane * VEC;

  if constexpr (VEC == 4) {
    f4 dv[U], sv[U];
    float sb = 0.0f;
    if (!p.src_inner) sb = s[0];
    // Segments wholly inside the row take the unguarded path (see ew_flat).
    const bool full = ((int64_t)chunk + 1) * U * tpr * 4 <= p.n0;
    if (full) {
      if (p.src_inner) {
#pragma unroll
        for (int u = 0; u < U; u++) {
          int64_t col = col0 + (int64_t)u * tpr * 4;
          if constexpr (ReadDst) dv[u] = load4<NT>(d + col);
          sv[u] = load4<NT>(s + col);
        }
      } else {
#pragma unroll
        for (int u = 0; u < U; u++) {
          int64_t col = col0 + (int64_t)u * tpr * 4;
          if constexpr (ReadDst) dv[u] = load4<NT>(d + col);
          sv[u] = f4{sb, sb, sb, sb};
        }
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        int64_t col = col0 + (int64_t)u * tpr * 4;
        f4 a = ReadDst ? dv[u] : f4{0.f, 0.f, 0.f, 0.f};
        f4 r;
        r.x = f(a.x, sv[u].x);
        r.y = f(a.y, sv[u].y);
        r.z = f(a.z, sv[u].z);
        r.w = f(a.w, sv[u].w);
        store4<NT>(d + col, r);
      }
      return;
    }
    for (int u = 0; u < U; u++) {
      int64_t col = col0 + (int64_t)u * tpr * 4;
      if (col + 4 <= p.n0) {
        f4 a = ReadDst ? load4<NT>(d + col) : f4{0.f, 0.f, 0.f, 0.f};
        f4 b = p.src_inner ? load4<NT>(s + col) : f4{sb, sb, sb, sb};
        f4 r;
        r.x = f(a.x, b.x);
        r.y = f(a.y, b.y);
        r.z = f(a.z, b.z);
        r.w = f(a.w, b.w);
        store4<NT>(d + col, r);
      } else if (col < p.n0) {  // ragged end of the row
        for (int64_t c = col; c < p.n0; c++) {
          float a = ReadDst ? d[c] : 0.0f;
          float b = p.src_inner ? s[c] : sb;
          d[c] = f(a, b);
        }
      }
    }
  } else {
    float dv[U], sv[U];
    float sb = 0.0f;
    if (!p.src_inner) sb = s[0];
#pragma unroll
    for (int u = 0; u < U; u++) {
      int64_t col = col0 + (int64_t)u * tpr;
      if (col < p.n0) {
        if constexpr (ReadDst) dv[u] = d[col];
        if (p.src_inner) sv[u] = s[col];
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      int64_t col = col0 + (int64_t)u * tpr;
      if (col < p.n0) {
        float a = ReadDst ? dv[u] : 0.0f;
        float b = p.src_inner ? sv[u] : sb;
        d[col] = f(a, b);
      }
    }
  }
}

// ---- rows shorter than one deep pass ---------------------------------------------
// ew_rows gives a thread four vectors of one row; a row of fewer than 16 vectors per
// thread position leaves it with one, and one 16-byte access in flight per lane holds
// x += row / x *= column on (65536, 1024) at 72 - 75 % of the HBM peak.  Here the four
// vectors of a thread come from four rows (rpb rows apart, so that each pass of the
// workgroup still covers consecutive rows), all loaded before the first store.
template <class F, bool ReadDst, bool NT>
__global__ __launch_bounds__(kBlock) void ew_rows_short(RowsParams p, F f) {
  constexpr int UR = 4;
  const int tpr = 1 << p.tpr_log2;
  const int rpb = kBlock >> p.tpr_log2;
  const int lane = threadIdx.x & (tpr - 1);
  const int sub = threadIdx.x >> p.tpr_log2;
  const uint32_t rblock = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk = blockIdx.x - rblock * p.chunks_per_row;
  const int64_t col = ((int64_t)chunk * tpr + lane) * 4;
  if (col >= p.n0) return;
  float* d[UR];
  const float* s[UR];
  bool live[UR];
#pragma unroll
  for (int u = 0; u < UR; u++) {
    const uint64_t row = ((uint64_t)rblock * UR + u) * rpb + sub;
    live[u] = row < p.nrows;
    int64_t doff = 0, soff = 0;
    uint32_t rem = live[u] ? (uint32_t)row : 0u;
    for (int i = 0; i < p.nouter; i++) {
      uint32_t idx;
      if (i == p.nouter - 1) {
        idx = rem;
      } else {
        uint32_t q = rem / p.oshape[i];
        idx = rem - q * p.oshape[i];
        rem = q;
      }
      doff += (int64_t)idx * p.odst[i];
      soff += (int64_t)idx * p.osrc[i];
    }
    d[u] = p.dst + doff;
    s[u] = p.src + soff;
  }
  if (col + 4 <= p.n0) {
    f4 dv[UR], sv[UR];
#pragma unroll
    for (int u = 0; u < UR; u++) {
      if (live[u]) {
        if constexpr (ReadDst) dv[u] = load4<NT>(d[u] + col);
        if (p.src_inner) {
          sv[u] = load4<NT>(s[u] + col);
        } else {
          const float sb = s[u][0];
          sv[u] = f4{sb, sb, sb, sb};
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UR; u++) {
      if (live[u]) {
        const f4 a = ReadDst ? dv[u] : f4{0.f, 0.f, 0.f, 0.f};
        f4 r;
        r.x = f(a.x, sv[u].x);
        r.y = f(a.y, sv[u].y);
        r.z = f(a.z, sv[u].z);
        r.w = f(a.w, sv[u].w);
        store4<NT>(d[u] + col, r);
      }
    }
    return;
  }
  for (int u = 0; u < UR; u++) {  // ragged end of the rows
    if (!live[u]) continue;
    for (int64_t c = col; c < p.n0; c++) {
      const float a = ReadDst ? d[u][c] : 0.0f;
      const float b = p.src_inner ? s[u][c] : s[u][0];
      d[u][c] = f(a, b);
    }
  }
}

// ---- stride-2 kernel -----------------------------------------------------------
// x <- x op y where x takes every second element of its rows (a [::2] slice) and
// y is a scalar per row, contiguous, or another [::2] slice.  Stores that fill
// half of each 32-byte sector cost a read-modify-write in the memory system:
// measured on the slice of (4096, 8192), 4-byte stores 52.6 us however the loads
// are shaped, whole 16-byte vectors 41.3 us.  So each thread loads one aligned
// float4 of the row's storage, applies the op to the two lanes the view selects
// and stores the vector whole: the lanes in between are written back as read.
// That is only sound when no other row of the launch owns those in-between
// elements (the launcher checks that the rows' storage intervals are disjoint)
// and for vectors wholly inside the row's interval; the first and last vector of a
// row fall back to single elements.  All work of the library is ordered on one
// stream, so nothing else writes the in-between elements meanwhile.
template <class F, bool NT, int SS>
__global__ __launch_bounds__(kBlock) void ew_stride2(RowsParams p, F f) {
  const uint32_t row = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk = blockIdx.x - row * p.chunks_per_row;
  int64_t doff = 0, soff = 0;
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
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  float* d = p.dst + doff;
  const float* s = p.src + soff;
  const int a = (int)(((uintptr_t)d >> 2) & 3);  // floats between the vector boundary below d and d
  const int64_t span = 2 * p.n0 - 1;              // storage interval of the row: [0, span)
  const int64_t rel0 = ((int64_t)chunk * kBlock + threadIdx.x) * 4 - a;
  if (rel0 >= span) return;
  const int first = a & 1;                        // lanes first and first + 2 hold view elements
  const int64_t i0 = (rel0 + first) >> 1;         // their indices along the row (i0, i0 + 1)
  constexpr int ss = SS;  // 0: one value per row (read through the scalar unit), 1, 2
  if (rel0 >= 0 && rel0 + 4 <= span) {
    f4 v = load4<NT>(d + rel0);
    const float y0 = s[i0 * ss], y1 = s[(i0 + 1) * ss];
    if (first == 0) {
      v.x = f(v.x, y0);
      v.z = f(v.z, y1);
    } else {
      v.y = f(v.y, y0);
      v.w = f(v.w, y1);
    }
    store4<NT>(d + rel0, v);
    return;
  }
  for (int e = first; e < 4; e += 2) {
    const int64_t pos = rel0 + e;
    if (pos >= 0 && pos < span) d[pos] = f(d[pos], s[(pos >> 1) * ss]);
  }
}

// ---- stride-2 source into contiguous rows -------------------------------------
// x <- x op y (or x <- f(y)) where y takes every second element of its rows and x is
// contiguous: the copy cl-waffe2 makes of a [::2] slice before any out-of-place
// op on it.  Each thread reads the 32 contiguous bytes that hold its four source
// elements as two aligned float4 loads (every fetched sector is used in full by
// the wavefront; with 4-byte gathers the slice copy of (4096, 8192) sits at 70 %
// of the sector traffic's roofline) and writes one float4.  `odd` says whether the
// wanted elements are lanes 1, 3 or 0, 2 of the vectors; the launcher only takes
// rows whose storage starts 0 or 1 floats past a 16-byte boundary.
template <class F, bool ReadDst, bool NT>
__global__ __launch_bounds__(kBlock) void ew_gather2(RowsParams p, F f, int odd) {
  constexpr int U = 2;
  const uint32_t row = blockIdx.x / p.chunks_per_row;
  const uint32_t chunk = blockIdx.x - row * p.chunks_per_row;
  int64_t doff = 0, soff = 0;
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
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  float* d = p.dst + doff;
  const float* s = p.src + soff - odd;  // 16-byte aligned
  const int64_t nvec = p.n0 / 4;
  f4 lo[U], hi[U], old[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const int64_t v = ((int64_t)chunk * U + u) * kBlock + threadIdx.x;
    if (v < nvec) {
      lo[u] = load4<NT>(s + 8 * v);
      hi[u] = load4<NT>(s + 8 * v + 4);
      if (ReadDst) old[u] = load4<NT>(d + 4 * v);
    }
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const int64_t v = ((int64_t)chunk * U + u) * kBlock + threadIdx.x;
    if (v < nvec) {
      f4 y = odd ? f4{lo[u].y, lo[u].w, hi[u].y, hi[u].w} : f4{lo[u].x, lo[u].z, hi[u].x, hi[u].z};
      f4 o;
      o.x = f(ReadDst ? old[u].x : 0.0f, y.x);
      o.y = f(ReadDst ? old[u].y : 0.0f, y.y);
      o.z = f(ReadDst ? old[u].z : 0.0f, y.z);
      o.w = f(ReadDst ? old[u].w : 0.0f, y.w);
      store4<NT>(d + 4 * v, o);
    }
  }
  // the last n0 % 4 elements of the row
  if (chunk == 0 && threadIdx.x < (p.n0 & 3)) {
    const int64_t c = nvec * 4 + threadIdx.x;
    d[c] = f(ReadDst ? d[c] : 0.0f, s[2 * c + odd]);
  }
}

// ---- generic kernel -----------------------------------------------------------
struct GenParams {
  float* dst;
  const float* src;
  int32_t rank;
  int64_t total;
  int64_t shape[WF2HIP_MAX_RANK];
  int64_t sd[WF2HIP_MAX_RANK];
  int64_t ss[WF2HIP_MAX_RANK];
};

// Element per lane with the offsets rebuilt from the linear index.  Each thread
// takes kGenU elements a workgroup-width apart and issues all their loads before
// the first store: with one 4-byte access in flight per lane a strided view is
// latency-bound (measured on the column-stride-2 slice of (4096, 8192): 53 us with
// one element per thread).
constexpr int kGenU = 4;

template <class F, bool ReadDst, class Index>
__global__ __launch_bounds__(kBlock) void ew_generic(GenParams p, F f) {
  const Index total = (Index)p.total;
  const Index step = (Index)gridDim.x * kBlock * kGenU;
  for (Index base = (Index)blockIdx.x * kBlock * kGenU + threadIdx.x; base < total; base += step) {
    int64_t doff[kGenU], soff[kGenU];
    float a[kGenU], b[kGenU];
#pragma unroll
    for (int u = 0; u < kGenU; u++) {
      Index rem = base + (Index)u * kBlock;
      if (rem >= total) rem = total - 1;  // offsets stay inside the view; the access is skipped below
      int64_t d = 0, q = 0;
      for (int r = p.rank - 1; r > 0; r--) {
        Index extent = (Index)p.shape[r];
        Index quot = rem / extent;
        Index idx = rem - quot * extent;
        rem = quot;
        d += (int64_t)idx * p.sd[r];
        q += (int64_t)idx * p.ss[r];
      }
      doff[u] = d + (int64_t)rem * p.sd[0];
      soff[u] = q + (int64_t)rem * p.ss[0];
    }
#pragma unroll
    for (int u = 0; u < kGenU; u++) {
      const bool live = base + (Index)u * kBlock < total;
      a[u] = (ReadDst && live) ? p.dst[doff[u]] : 0.0f;
      b[u] = live ? p.src[soff[u]] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < kGenU; u++)
      if (base + (Index)u * kBlock < total) p.dst[doff[u]] = f(a[u], b[u]);
  }
}

// ---- tile kernel: dst contiguous along one axis, src along another ------------
// dst[..., j, ..., i] <- f(dst, src) where dst has stride 1 along axis I (the
// innermost) and src has stride 1 along another axis J.  A 64x64 tile is read
// with threads running along J (coalesced for src), parked in LDS, and written
// with threads running along I (coalesced for dst).  The +1 padding keeps the
// column reads free of LDS bank conflicts.
constexpr int kTile = 64;

struct TileParams {
  float* dst;
  const float* src;
  int64_t ni, nj;        // extents of axis I and J
  int64_t d_j;           // dst stride along J   (dst stride along I is 1)
  int64_t s_i;           // src stride along I   (src stride along J is 1)
  uint32_t tiles_i, tiles_j;
  uint32_t band;         // tiles_i / 8 when that divides, else 0 (see tile_position)
  int32_t nouter;
  uint32_t oshape[kMaxOuter];
  int64_t odst[kMaxOuter];
  int64_t osrc[kMaxOuter];
};

// Which tile a workgroup takes.  Workgroups go to the eight XCDs round robin
// (id modulo 8), each with an L2 of its own, so the order is chosen per XCD:
// XCD x owns the band of tiles_i / 8 tiles x * band .. along I, walks it with I
// fastest, and steps along J alternately from the two ends towards the middle.
// The tiles resident on one XCD then read and write runs of band * tile bytes
// between them, the eight XCDs stay on different parts of every row, and the
// two column windows in flight keep moving relative to each other instead of
// sitting a fixed power of two apart.  Transposing copy, 128 x 128 tiles, % of
// the HBM peak with I fastest over the whole grid -> this order:
// (8192, 8192) 75.1 -> 79.1, (16384, 4096) 61.8 -> 73.9, (4096, 16384) 71.0 -> 75.0,
// (8192, 1024) 63.6 -> 74.4, (8192, 3072) 66.6 -> 72.8; 64 x 64 tiles 56.6 -> 71.2.
// J fastest, 8 x 8 super tiles, bands along J, one contiguous chunk of the
// linear order per XCD, a per-XCD skew along J and strides of a half or a
// quarter of tiles_j along J all measured lower.  Without a band (tiles_i not a
// multiple of 8) the order is I fastest over the whole grid.
__device__ __forceinline__ void tile_position(const TileParams& p, uint32_t bid, uint32_t& ti, uint32_t& tj,
                                              uint32_t& rem) {
  if (p.band != 0) {
    const uint32_t r = bid >> 3;
    ti = (bid & 7) * p.band + r % p.band;
    uint32_t q = r / p.band;
    rem = q / p.tiles_j;
    q -= rem * p.tiles_j;
    tj = (q & 1) ? p.tiles_j - 1 - (q >> 1) : (q >> 1);
  } else {
    ti = bid % p.tiles_i;
    bid /= p.tiles_i;
    tj = bid % p.tiles_j;
    rem = bid / p.tiles_j;
  }
}

template <class F, bool ReadDst, bool VEC, bool NT = false>
__global__ __launch_bounds__(kBlock) void ew_tile(TileParams p, F f) {
  __shared__ float tile[kTile][kTile + 1];
  uint32_t ti, tj, rem;
  tile_position(p, blockIdx.x, ti, tj, rem);
  int64_t doff = 0, soff = 0;
  for (int i = 0; i < p.nouter; i++) {
    uint32_t q = rem / p.oshape[i];
    uint32_t idx = rem - q * p.oshape[i];
    rem = q;
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  const int64_t i0 = (int64_t)ti * kTile;
  const int64_t j0 = (int64_t)tj * kTile;
  if constexpr (VEC) {
    // 16-byte global accesses on both sides (extents and strides are multiples
    // of 4, checked on the host); the transposition itself goes through LDS
    // with 32-bit accesses at a pitch of 65 floats (at most 2-way conflicts).
    const int q4 = (threadIdx.x & 15) * 4;  // 0,4,..,60 along the contiguous axis
    const int rr = threadIdx.x >> 4;        // 0..15
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
      const int r = rr + 16 * pass;
      const int64_t i = i0 + r, j = j0 + q4;
      if (i < p.ni && j < p.nj) {
        f4 v = load4<NT>(p.src + soff + i * p.s_i + j);
        tile[r][q4 + 0] = v.x;
        tile[r][q4 + 1] = v.y;
        tile[r][q4 + 2] = v.z;
        tile[r][q4 + 3] = v.w;
      }
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
      const int r = rr + 16 * pass;
      const int64_t i = i0 + q4, j = j0 + r;
      if (i < p.ni && j < p.nj) {
        float* dp = p.dst + doff + j * p.d_j + i;
        f4 a = ReadDst ? load4<NT>(dp) : f4{0.f, 0.f, 0.f, 0.f};
        f4 o;
        o.x = f(a.x, tile[q4 + 0][r]);
        o.y = f(a.y, tile[q4 + 1][r]);
        o.z = f(a.z, tile[q4 + 2][r]);
        o.w = f(a.w, tile[q4 + 3][r]);
        store4<NT>(dp, o);
      }
    }
  } else {
    const int tx = threadIdx.x & (kTile - 1);  // 0..63
    const int ty = threadIdx.x >> 6;           // 0..3
    // read: tx runs along J (src contiguous), rows of the tile are I
    for (int r = ty; r < kTile; r += kBlock / kTile) {
      int64_t i = i0 + r, j = j0 + tx;
      if (i < p.ni && j < p.nj) tile[r][tx] = p.src[soff + i * p.s_i + j];
    }
    __syncthreads();
    // write: tx runs along I (dst contiguous), rows are J
    for (int r = ty; r < kTile; r += kBlock / kTile) {
      int64_t i = i0 + tx, j = j0 + r;
      if (i < p.ni && j < p.nj) {
        float* dp = p.dst + doff + j * p.d_j + i;
        float a = ReadDst ? *dp : 0.0f;
        *dp = f(a, tile[tx][r]);
      }
    }
  }
}

// The same exchange on 128 x 128 tiles for large operands: a workgroup then
// touches 512 contiguous bytes per row on both sides.  Measured for plain tiled
// copies of (8192, 8192): 256-byte runs 70 % of the HBM peak, 512-byte runs and
// longer 80 %.  32 lanes cover a row, a wavefront two neighbouring rows, the
// workgroup THREADS / 32 rows per pass; LDS element (a, b) lives at a * 129 + b
// (at most 2-way bank conflicts; the LDS moves 15 % of what it could here).
constexpr int kBigTile = 128;
constexpr int kBigTileFloats = kBigTile * (kBigTile + 1) + 4;

template <class F, bool ReadDst, bool NT, int THREADS>
__global__ __launch_bounds__(THREADS) void ew_tile128(TileParams p, F f) {
  constexpr int kRowLanes = kBigTile / 4;         // 32 lanes x 4 floats
  constexpr int kRows = THREADS / kRowLanes;      // rows per pass
  constexpr int kPasses = kBigTile / kRows;
  constexpr int kPitch = kBigTile + 1;
  extern __shared__ float big_tile[];
  uint32_t ti, tj, rem;
  tile_position(p, blockIdx.x, ti, tj, rem);
  int64_t doff = 0, soff = 0;
  for (int i = 0; i < p.nouter; i++) {
    uint32_t q = rem / p.oshape[i];
    uint32_t idx = rem - q * p.oshape[i];
    rem = q;
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  const int64_t i0 = (int64_t)ti * kBigTile;
  const int64_t j0 = (int64_t)tj * kBigTile;
  const int q4 = (threadIdx.x % kRowLanes) * 4;  // position along the contiguous axis
  const int r0 = threadIdx.x / kRowLanes;        // row within a pass
  f4 v[kPasses];
#pragma unroll
  for (int pass = 0; pass < kPasses; pass++) {
    const int64_t i = i0 + r0 + pass * kRows, j = j0 + q4;
    v[pass] = f4{0.f, 0.f, 0.f, 0.f};
    if (i < p.ni && j < p.nj) v[pass] = load4<NT>(p.src + soff + i * p.s_i + j);
  }
#pragma unroll
  for (int pass = 0; pass < kPasses; pass++) {
    float* t = big_tile + (r0 + pass * kRows) * kPitch + q4;
    t[0] = v[pass].x;
    t[1] = v[pass].y;
    t[2] = v[pass].z;
    t[3] = v[pass].w;
  }
  __syncthreads();
  f4 a[kPasses];
#pragma unroll
  for (int pass = 0; pass < kPasses; pass++) {
    const int64_t i = i0 + q4, j = j0 + r0 + pass * kRows;
    a[pass] = f4{0.f, 0.f, 0.f, 0.f};
    if (ReadDst && i < p.ni && j < p.nj) a[pass] = load4<NT>(p.dst + doff + j * p.d_j + i);
  }
#pragma unroll
  for (int pass = 0; pass < kPasses; pass++) {
    const int r = r0 + pass * kRows;
    const int64_t i = i0 + q4, j = j0 + r;
    if (i < p.ni && j < p.nj) {
      f4 o;
      o.x = f(a[pass].x, big_tile[(q4 + 0) * kPitch + r]);
      o.y = f(a[pass].y, big_tile[(q4 + 1) * kPitch + r]);
      o.z = f(a[pass].z, big_tile[(q4 + 2) * kPitch + r]);
      o.w = f(a[pass].w, big_tile[(q4 + 3) * kPitch + r]);
      store4<NT>(p.dst + doff + j * p.d_j + i, o);
    }
  }
}

// Sixteen wavefronts per tile: the 66 KB tile allows two workgroups per compute
// unit whatever their width, so a wide workgroup is what puts enough loads in
// flight (transposing copy of (8192, 8192): 256 threads 104.1 us, 512 100.1 us,
// 1024 94.8 us).
constexpr int kBigTileThreads = 1024;

template <class F, bool ReadDst, bool NT>
static int launch_tile128(const TileParams& p, uint32_t blocks, F f) {
  constexpr int bytes = kBigTileFloats * (int)sizeof(float);
  static bool configured = false;  // per instantiation
  if (!configured) {
    WF2_TRY(check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&ew_tile128<F, ReadDst, NT, kBigTileThreads>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, bytes),
                      "hipFuncSetAttribute(ew_tile128)"));
    configured = true;
  }
  ew_tile128<F, ReadDst, NT, kBigTileThreads><<<blocks, kBigTileThreads, bytes, rt().stream>>>(p, f);
  return 0;
}

// ---- narrow tile kernel: the source's contiguous axis is short ---------------------------------------
// (N, 12) -> (12, N), NHWC -> NCHW of images: the axis J along which src is contiguous has fewer than 32
// elements.  A 64 x 64 tile would leave most of its lanes idle, and an element per lane reads every line of
// src once per element of J ((1398101, 12) transposed: 126 us).  Here a workgroup takes `tl` positions of
// dst's contiguous axis I with the whole of J: src is walked in storage order (whole lines when its rows are
// adjacent), dst is written in 16-byte vectors, and LDS (element (j, i) at j * (tl + 4) + i) sits between
// them.  tl is 512 for up to 15 elements of J and 256 for up to 31: at most 32 KB of LDS.  (The mirrored
// case -- dst contiguous along the short axis -- is served well by an element per lane: dst is then written
// in storage order and neighbouring wavefronts use up the lines of src.)
constexpr int kNarrowMax = 31;
constexpr int kNarrowFloats = 8064;  // >= 15 * 516 and 31 * 260

// VECSRC: src's rows are adjacent (s_i == nj) and 16-byte aligned: its run is read in 16-byte vectors.
template <class F, bool ReadDst, bool VEC, bool VECSRC>
__global__ __launch_bounds__(kBlock) void ew_tile_narrow(TileParams p, F f, FastDiv by_nj, int tl) {
  __shared__ __attribute__((aligned(16))) float tile[kNarrowFloats];
  const int pitch = tl + 4;
  uint32_t rem = blockIdx.x / p.tiles_i;
  const int64_t i0 = (int64_t)(blockIdx.x - rem * p.tiles_i) * tl;
  int64_t doff = 0, soff = 0;
  for (int i = 0; i < p.nouter; i++) {
    uint32_t q = rem / p.oshape[i];
    uint32_t idx = rem - q * p.oshape[i];
    rem = q;
    doff += (int64_t)idx * p.odst[i];
    soff += (int64_t)idx * p.osrc[i];
  }
  const int nj = (int)p.nj;
  const int live = (int)(p.ni - i0 < tl ? p.ni - i0 : tl);  // positions of I in this tile
  const uint32_t cells = (uint32_t)live * (uint32_t)nj;
  float* dst = p.dst + doff;
  const float* src = p.src + soff;
  constexpr int U = 4;
  uint32_t staged = 0;  // cells already in LDS
  if constexpr (VECSRC) {
    const uint32_t whole = cells / 4;
    const f4* vsrc = reinterpret_cast<const f4*>(src + i0 * p.s_i);
    for (uint32_t q0 = threadIdx.x; q0 < whole; q0 += kBlock * U) {
      f4 v[U];
#pragma unroll
      for (int u = 0; u < U; u++) v[u] = q0 + u * kBlock < whole ? vsrc[q0 + u * kBlock] : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < U; u++)
        if (q0 + u * kBlock < whole) {
          uint32_t j;
          uint32_t i = fd_divmod(4 * (q0 + u * kBlock), by_nj, &j);
          const float c4[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
          for (int c = 0; c < 4; c++) {
            tile[j * pitch + i] = c4[c];
            if (++j == (uint32_t)nj) {
              j = 0;
              i++;
            }
          }
        }
    }
    staged = 4 * whole;
  }
  // src (i, j) at i * s_i + j  ->  LDS
  for (uint32_t e0 = staged + threadIdx.x; e0 < cells; e0 += kBlock * U) {
    float v[U];
    uint32_t i[U], j[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t e = e0 + u * kBlock;
      i[u] = fd_divmod(e < cells ? e : 0u, by_nj, &j[u]);
      v[u] = e < cells ? src[(i0 + i[u]) * p.s_i + j[u]] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < U; u++)
      if (e0 + u * kBlock < cells) tile[j[u] * pitch + i[u]] = v[u];
  }
  __syncthreads();
  // LDS -> dst (j, i) at j * d_j + i
  const uint32_t per_row = (uint32_t)tl / 4;
  const uint32_t vecs = (uint32_t)nj * per_row;
  for (uint32_t q = threadIdx.x; q < vecs; q += kBlock) {
    const uint32_t j = q / per_row;  // tl / 4 is a power of two
    const int i4 = (int)(q - j * per_row) * 4;
    if (i4 >= live) continue;
    float* dp = dst + (int64_t)j * p.d_j + i0 + i4;
    const float* t = tile + j * pitch + i4;
    if (VEC && i4 + 4 <= live) {
      const f4 a = ReadDst ? *reinterpret_cast<const f4*>(dp) : f4{0.f, 0.f, 0.f, 0.f};
      const f4 b = *reinterpret_cast<const f4*>(t);
      f4 o;
      o.x = f(a.x, b.x);
      o.y = f(a.y, b.y);
      o.z = f(a.z, b.z);
      o.w = f(a.w, b.w);
      *reinterpret_cast<f4*>(dp) = o;
    } else {
      for (int u = 0; u < 4 && i4 + u < live; u++) dp[u] = f(ReadDst ? dp[u] : 0.0f, t[u]);
    }
  }
}

// ---- dispatch -------------------------------------------------------------------
static inline int ilog2_ceil(int64_t v) {
  int l = 0;
  while (((int64_t)1 << l) < v) l++;
  return l;
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <class F, bool ReadDst>
static int launch_rows(const Space& s, float* dst, const float* src, F f) {
  const int last = s.rank - 1;
  RowsParams p;
  p.dst = dst + s.off_a;
  p.src = src + s.off_b;
  p.n0 = s.shape[last];
  p.src_inner = (int32_t)s.sb[last];
  p.nouter = s.rank - 1;
  int64_t nrows = 1;
  for (int i = 0; i < p.nouter; i++) {
    int r = last - 1 - i;
    p.oshape[i] = (uint32_t)s.shape[r];
    p.odst[i] = s.sa[r];
    p.osrc[i] = s.sb[r];
    nrows *= s.shape[r];
  }
  p.nrows = (uint32_t)nrows;
  const int vec = p.n0 >= 4 ? 4 : 1;  // any row start: the vector accesses need no alignment
  const int64_t n0v = ceil_div(p.n0, vec);
  int tl = ilog2_ceil(n0v);
  if (tl > 8) tl = 8;
  p.tpr_log2 = tl;
  const int tpr = 1 << tl;
  const int rpb = kBlock >> tl;
  const bool deep = p.n0 >= (int64_t)tpr * vec * 4;
  const int u = deep ? 4 : 1;
  const int64_t chunks = ceil_div(p.n0, (int64_t)tpr * vec * u);
  const int64_t blocks = ceil_div(nrows, rpb) * chunks;
  if (blocks <= 0 || blocks >= ((int64_t)1 << 31))
    return fail(WF2HIP_EUNSUPPORTED, "iteration space too large for one launch");
  p.chunks_per_row = (uint32_t)chunks;
  hipStream_t st = rt().stream;
  const int64_t streams = 1 + (ReadDst ? 1 : 0) + (p.src_inner ? 1 : 0);
  const bool streaming = s.total * 4 * streams >= kStreamingBytes;
  if (vec == 4 && deep && streaming)
    ew_rows<F, ReadDst, 4, 4, true><<<(uint32_t)blocks, kBlock, 0, st>>>(p, f);
  else if (vec == 4 && deep)
    ew_rows<F, ReadDst, 4, 4><<<(uint32_t)blocks, kBlock, 0, st>>>(p, f);
  else if (vec == 4) {  // chunks were counted with one vector per thread
    const int64_t short_blocks = ceil_div(nrows, (int64_t)rpb * 4) * chunks;
    if (streaming)
      ew_rows_short<F, ReadDst, true><<<(uint32_t)short_blocks, kBlock, 0, st>>>(p, f);
    else
      ew_rows_short<F, ReadDst, false><<<(uint32_t)short_blocks, kBlock, 0, st>>>(p, f);
  }
  else if (deep)
    ew_rows<F, ReadDst, 1, 4><<<(uint32_t)blocks, kBlock, 0, st>>>(p, f);
  else
    ew_rows<F, ReadDst, 1, 1><<<(uint32_t)blocks, kBlock, 0, st>>>(p, f);
  return after_launch("ew_rows");
}

// Rank-1, unit-stride destination, source unit-stride or broadcast: the flat kernel.
template <class F, bool ReadDst>
static bool try_launch_flat(const Space& s, float* dst, const float* src, F f, int* rc) {
  float* d = dst + s.off_a;
  const float* q = src + s.off_b;
  const bool bcast = s.sb[0] == 0;
  // The vector body starts where dst reaches a 256-byte boundary, so that the 1 KB a
  // wavefront stores per access covers whole cache lines: x[1:] += y at 2^26 runs at 70 %
  // of the HBM peak with dst 4 or 16 bytes past such a boundary, 82 % with only the loads
  // misaligned.  The up to 63 elements before the body and the up to three after its last
  // whole vector are done by the first workgroup.
  const int64_t head = (int64_t)((64 - (((uintptr_t)d >> 2) & 63)) & 63);  // elements up to the next 256-byte boundary
  d += head;
  if (!bcast) q += head;
  const size_t nvec = (size_t)((s.total - head) / 4);
  const int64_t tail = s.total - head - (int64_t)nvec * 4;
  // vectors per thread: 4 for x <- x op y (three streams), 2 for functors with
  // a long binary64 body, 1 for the light two-stream forms (copy, fill, scalar
  // operand, sqrt, abs) -- each the best of a sweep at 2^26 on MI355X.
  constexpr int u3 = 4;
  constexpr int u2 = F::kFlatU == 2 ? 2 : 1;
  const int64_t streams = 1 + (ReadDst ? 1 : 0) + (bcast ? 0 : 1);
  const bool nt = s.total * 4 * streams >= kStreamingBytes;
  hipStream_t st = rt().stream;
  const bool three = ReadDst && !bcast;
  const int64_t blocks = ceil_div((int64_t)nvec, kBlock * (three ? u3 : u2));
  if (blocks >= ((int64_t)1 << 31)) return false;
  const uint32_t grid = (uint32_t)blocks;
  const FlatEdges edges{(int)head, (int)tail};
  const bool plain = head == 0 && tail == 0;
#define WF2_FLAT(BC, NTV, LAY, UV)                                                                   \
  do {                                                                                               \
    if (plain)                                                                                       \
      ew_flat<F, ReadDst, BC, NTV, LAY, UV><<<grid, kBlock, 0, st>>>(d, q, nvec, f);                 \
    else                                                                                             \
      ew_flat<F, ReadDst, BC, NTV, LAY, UV, FlatEdges><<<grid, kBlock, 0, st>>>(d, q, nvec, f, edges); \
  } while (0)
  if (bcast) {
    if (nt)
      WF2_FLAT(true, true, 0, u2);
    else
      WF2_FLAT(true, false, 0, u2);
  } else if (ReadDst) {
    if (nt)
      WF2_FLAT(false, true, 1, u3);
    else
      WF2_FLAT(false, false, 1, u3);
  } else {
    if (nt)
      WF2_FLAT(false, true, 0, u2);
    else
      WF2_FLAT(false, false, 0, u2);
  }
#undef WF2_FLAT
  *rc = after_launch("ew_flat");
  return true;
}

template <class F, bool ReadDst>
static int launch_generic(const Space& s, float* dst, const float* src, F f) {
  GenParams p;
  p.dst = dst + s.off_a;
  p.src = src + s.off_b;
  p.rank = s.rank;
  p.total = s.total;
  for (int r = 0; r < s.rank; r++) {
    p.shape[r] = s.shape[r];
    p.sd[r] = s.sa[r];
    p.ss[r] = s.sb[r];
  }
  int64_t want = ceil_div(s.total, kBlock * kGenU);
  int64_t cap = (int64_t)rt().num_cus * 64;
  uint32_t blocks = (uint32_t)(want < cap ? want : cap);
  hipStream_t st = rt().stream;
  if (s.total < ((int64_t)1 << 31))
    ew_generic<F, ReadDst, uint32_t><<<blocks, kBlock, 0, st>>>(p, f);
  else
    ew_generic<F, ReadDst, int64_t><<<blocks, kBlock, 0, st>>>(p, f);
  return after_launch("ew_generic");
}

// dst stride 1 on the last axis; src stride 1 on another axis J whose dst
// stride is positive; both extents large enough for a tile to pay off.
template <class F, bool ReadDst>
static bool try_launch_tile(const Space& s, float* dst, const float* src, F f, int* rc) {
  const int last = s.rank - 1;
  if (s.rank < 2 || s.sa[last] != 1 || s.sb[last] <= 1) return false;
  int J = -1;
  for (int r = 0; r < last; r++)
    if (s.sb[r] == 1 && s.sa[r] > 0) J = r;
  if (J < 0) return false;
  const bool narrow = s.shape[J] <= kNarrowMax && s.shape[last] >= 256;
  if (!narrow && (s.shape[last] < 32 || s.shape[J] < 16)) return false;  // an element per lane serves a short dst axis
  TileParams p;
  p.dst = dst + s.off_a;
  p.src = src + s.off_b;
  p.ni = s.shape[last];
  p.nj = s.shape[J];
  p.d_j = s.sa[J];
  p.s_i = s.sb[last];
  p.tiles_i = (uint32_t)ceil_div(p.ni, kTile);
  p.tiles_j = (uint32_t)ceil_div(p.nj, kTile);
  p.band = p.tiles_i % 8 == 0 ? p.tiles_i / 8 : 0;
  p.nouter = 0;
  int64_t blocks = (int64_t)p.tiles_i * p.tiles_j;
  for (int r = last - 1; r >= 0; r--) {
    if (r == J) continue;
    p.oshape[p.nouter] = (uint32_t)s.shape[r];
    p.odst[p.nouter] = s.sa[r];
    p.osrc[p.nouter] = s.sb[r];
    p.nouter++;
    blocks *= s.shape[r];
  }
  if (narrow) {
    const int tl = p.nj <= 15 ? 512 : 256;
    const int64_t tiles = ceil_div(p.ni, tl);
    int64_t nblocks = tiles;
    for (int i = 0; i < p.nouter; i++) nblocks *= p.oshape[i];
    if (nblocks >= ((int64_t)1 << 31)) return false;
    p.tiles_i = (uint32_t)tiles;
    bool v16 = aligned16(p.dst) && p.d_j % 4 == 0;  // 16-byte accesses on dst
    for (int i = 0; i < p.nouter; i++)
      if (p.odst[i] % 4 != 0) v16 = false;
    const FastDiv by_nj = make_fastdiv((uint32_t)p.nj);
    bool vsrc = aligned16(p.src) && p.s_i == p.nj;  // a tile's rows of src are one run, on a multiple of 16 bytes
    for (int i = 0; i < p.nouter; i++)
      if (p.osrc[i] % 4 != 0) vsrc = false;
    if (v16 && vsrc)
      ew_tile_narrow<F, ReadDst, true, true><<<(uint32_t)nblocks, kBlock, 0, rt().stream>>>(p, f, by_nj, tl);
    else if (v16)
      ew_tile_narrow<F, ReadDst, true, false><<<(uint32_t)nblocks, kBlock, 0, rt().stream>>>(p, f, by_nj, tl);
    else if (vsrc)
      ew_tile_narrow<F, ReadDst, false, true><<<(uint32_t)nblocks, kBlock, 0, rt().stream>>>(p, f, by_nj, tl);
    else
      ew_tile_narrow<F, ReadDst, false, false><<<(uint32_t)nblocks, kBlock, 0, rt().stream>>>(p, f, by_nj, tl);
    *rc = after_launch("ew_tile_narrow");
    return true;
  }
  if (blocks >= ((int64_t)1 << 31)) return false;
  bool vec = aligned16(p.dst) && aligned16(p.src) && p.ni % 4 == 0 && p.nj % 4 == 0 &&
             p.d_j % 4 == 0 && p.s_i % 4 == 0;
  for (int i = 0; i < p.nouter; i++)
    if (p.odst[i] % 4 != 0 || p.osrc[i] % 4 != 0) vec = false;
  const bool streaming = s.total * 4 * (ReadDst ? 3 : 2) >= kStreamingBytes;
  if (vec && p.ni >= kBigTile && p.nj >= kBigTile && s.total >= ((int64_t)1 << 22)) {
    p.tiles_i = (uint32_t)ceil_div(p.ni, kBigTile);
    p.tiles_j = (uint32_t)ceil_div(p.nj, kBigTile);
    p.band = p.tiles_i % 8 == 0 ? p.tiles_i / 8 : 0;
    int64_t big_blocks = (int64_t)p.tiles_i * p.tiles_j;
    for (int i = 0; i < p.nouter; i++) big_blocks *= p.oshape[i];
    int lrc = streaming ? launch_tile128<F, ReadDst, true>(p, (uint32_t)big_blocks, f)
                        : launch_tile128<F, ReadDst, false>(p, (uint32_t)big_blocks, f);
    *rc = lrc != 0 ? lrc : after_launch("ew_tile128");
    return true;
  }
  if (vec && streaming)
    ew_tile<F, ReadDst, true, true><<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(p, f);
  else if (vec)
    ew_tile<F, ReadDst, true><<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(p, f);
  else
    ew_tile<F, ReadDst, false><<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(p, f);
  *rc = after_launch("ew_tile");
  return true;
}

// In-place ops on a [::2] slice whose rows occupy disjoint storage intervals.
template <class F, bool ReadDst>
static bool try_launch_stride2(const Space& s, float* dst, const float* src, F f, int* rc) {
  if constexpr (!ReadDst) {
    return false;
  } else {
    const int last = s.rank - 1;
    const int64_t n0 = s.shape[last];
    if (s.sa[last] != 2 || s.sb[last] < 0 || s.sb[last] > 2 || n0 < 128) return false;
    if (s.rank - 1 > kMaxOuter) return false;
    // rows must not interleave: sorted by stride, each outer axis steps over
    // everything the axes below it cover
    int order[WF2HIP_MAX_RANK];
    int nouter = 0;
    for (int r = 0; r < last; r++) {
      if (s.shape[r] == 1) continue;
      if (s.sa[r] <= 0 || s.shape[r] >= ((int64_t)1 << 32)) return false;
      order[nouter++] = r;
    }
    for (int i = 1; i < nouter; i++)
      for (int j = i; j > 0 && s.sa[order[j]] < s.sa[order[j - 1]]; j--) {
        int t = order[j];
        order[j] = order[j - 1];
        order[j - 1] = t;
      }
    int64_t extent = 2 * n0 - 1;
    for (int i = 0; i < nouter; i++) {
      if (s.sa[order[i]] < extent) return false;
      extent += (s.shape[order[i]] - 1) * s.sa[order[i]];
    }
    RowsParams p;
    p.dst = dst + s.off_a;
    p.src = src + s.off_b;
    p.n0 = n0;
    p.src_inner = (int32_t)s.sb[last];
    p.nouter = 0;
    p.tpr_log2 = 8;
    int64_t nrows = 1;
    for (int r = last - 1; r >= 0; r--) {
      p.oshape[p.nouter] = (uint32_t)s.shape[r];
      p.odst[p.nouter] = s.sa[r];
      p.osrc[p.nouter] = s.sb[r];
      p.nouter++;
      nrows *= s.shape[r];
    }
    const int64_t chunks = ceil_div(ceil_div(2 * n0 - 1 + 3, 4), kBlock);
    if (nrows * chunks >= ((int64_t)1 << 31)) return false;
    p.nrows = (uint32_t)nrows;
    p.chunks_per_row = (uint32_t)chunks;
    const uint32_t blocks = (uint32_t)(nrows * chunks);
    const bool nt = s.total * 16 >= kStreamingBytes;
    hipStream_t st = rt().stream;
    switch ((int)s.sb[last] * 2 + (nt ? 1 : 0)) {
      case 0: ew_stride2<F, false, 0><<<blocks, kBlock, 0, st>>>(p, f); break;
      case 1: ew_stride2<F, true, 0><<<blocks, kBlock, 0, st>>>(p, f); break;
      case 2: ew_stride2<F, false, 1><<<blocks, kBlock, 0, st>>>(p, f); break;
      case 3: ew_stride2<F, true, 1><<<blocks, kBlock, 0, st>>>(p, f); break;
      case 4: ew_stride2<F, false, 2><<<blocks, kBlock, 0, st>>>(p, f); break;
      default: ew_stride2<F, true, 2><<<blocks, kBlock, 0, st>>>(p, f); break;
    }
    *rc = after_launch("ew_stride2");
    return true;
  }
}

// Contiguous destination rows, source rows of stride 2.
template <class F, bool ReadDst>
static bool try_launch_gather2(const Space& s, float* dst, const float* src, F f, int* rc) {
  const int last = s.rank - 1;
  const int64_t n0 = s.shape[last];
  if (s.sa[last] != 1 || s.sb[last] != 2 || n0 < 128 || s.rank - 1 > kMaxOuter) return false;
  RowsParams p;
  p.dst = dst + s.off_a;
  p.src = src + s.off_b;
  const int lead = (int)(((uintptr_t)p.src >> 2) & 3);  // floats past a 16-byte boundary
  if (lead > 1 || !aligned16(p.dst)) return false;
  p.n0 = n0;
  p.src_inner = 2;
  p.nouter = 0;
  p.tpr_log2 = 8;
  int64_t nrows = 1;
  for (int r = last - 1; r >= 0; r--) {
    if (s.shape[r] >= ((int64_t)1 << 32)) return false;
    if (s.shape[r] > 1 && (s.sa[r] % 4 != 0 || s.sb[r] % 4 != 0)) return false;  // every row as aligned as the first
    p.oshape[p.nouter] = (uint32_t)s.shape[r];
    p.odst[p.nouter] = s.sa[r];
    p.osrc[p.nouter] = s.sb[r];
    p.nouter++;
    nrows *= s.shape[r];
  }
  const int64_t chunks = ceil_div(n0 / 4 > 0 ? n0 / 4 : 1, (int64_t)kBlock * 2);
  if (nrows * chunks >= ((int64_t)1 << 31)) return false;
  p.nrows = (uint32_t)nrows;
  p.chunks_per_row = (uint32_t)chunks;
  const uint32_t blocks = (uint32_t)(nrows * chunks);
  const bool nt = s.total * (ReadDst ? 16 : 12) >= kStreamingBytes;
  if (nt)
    ew_gather2<F, ReadDst, true><<<blocks, kBlock, 0, rt().stream>>>(p, f, lead);
  else
    ew_gather2<F, ReadDst, false><<<blocks, kBlock, 0, rt().stream>>>(p, f, lead);
  *rc = after_launch("ew_gather2");
  return true;
}

// `s` describes dst through (sa, off_a) and src through (sb, off_b); dst has
// no broadcast axis.
// The destination's unit-stride axis moved to the end (x^T += y): an elementwise pass may visit its index
// space in any order as long as no destination element is visited twice, which holds when the axes sorted by
// stride each step over everything the smaller ones cover.  False when there is nothing to move.
static bool dst_unit_axis_last(const Space& s, Space* out) {
  const int last = s.rank - 1;
  if (s.rank < 2 || s.sa[last] == 1) return false;
  int unit = -1;
  for (int r = 0; r < last; r++)
    if (s.sa[r] == 1 && s.shape[r] >= 16) unit = r;
  if (unit < 0) return false;
  int order[WF2HIP_MAX_RANK];
  for (int r = 0; r < s.rank; r++) {
    if (s.sa[r] <= 0) return false;
    order[r] = r;
  }
  for (int i = 1; i < s.rank; i++)
    for (int j = i; j > 0 && s.sa[order[j]] < s.sa[order[j - 1]]; j--) {
      const int t = order[j];
      order[j] = order[j - 1];
      order[j - 1] = t;
    }
  int64_t covered = 1;  // elements spanned by the axes so far
  for (int i = 0; i < s.rank; i++) {
    const int r = order[i];
    if (s.sa[r] < covered) return false;
    covered = s.sa[r] * (s.shape[r] - 1) + covered;
  }
  *out = s;
  int w = 0;
  for (int r = 0; r < s.rank; r++) {
    if (r == unit) continue;
    out->shape[w] = s.shape[r];
    out->sa[w] = s.sa[r];
    out->sb[w] = s.sb[r];
    w++;
  }
  out->shape[w] = s.shape[unit];
  out->sa[w] = s.sa[unit];
  out->sb[w] = s.sb[unit];
  normalise(out);
  return true;
}

template <class F, bool ReadDst>
static int launch_elementwise(const Space& s_in, float* dst, const float* src, F f) {
  Space turned;
  const Space& s = dst_unit_axis_last(s_in, &turned) ? turned : s_in;
  const int last = s.rank - 1;
  int64_t nrows = s.total / (s.shape[last] ? s.shape[last] : 1);
  bool rows_ok = s.sa[last] == 1 && (s.sb[last] == 1 || s.sb[last] == 0) &&
                 nrows < ((int64_t)1 << 31);
  for (int r = 0; r < last; r++)
    if (s.shape[r] >= ((int64_t)1 << 32)) rows_ok = false;
  if (rows_ok && s.rank == 1 && s.total >= (1 << 16)) {
    int rc = 0;
    if (try_launch_flat<F, ReadDst>(s, dst, src, f, &rc)) return rc;
  }
  if (rows_ok) return launch_rows<F, ReadDst>(s, dst, src, f);
  int rc = 0;
  if (try_launch_tile<F, ReadDst>(s, dst, src, f, &rc)) return rc;
  if (try_launch_stride2<F, ReadDst>(s, dst, src, f, &rc)) return rc;
  if (try_launch_gather2<F, ReadDst>(s, dst, src, f, &rc)) return rc;
  return launch_generic<F, ReadDst>(s, dst, src, f);
}

// For ops that overwrite dst (copy, unary) a broadcast dst axis means "the
// last write wins", exactly what the reference's sequential loops leave
// behind: keep only the last index of such axes.
static void keep_last_write(Space* s) {
  for (int r = 0; r < s->rank; r++) {
    if (s->sa[r] == 0 && s->shape[r] > 1) {
      s->off_b += s->sb[r] * (s->shape[r] - 1);
      s->shape[r] = 1;
    }
  }
  s->total = 1;
  for (int r = 0; r < s->rank; r++) s->total *= s->shape[r];
  normalise(s);
}

int launch_accumulate(int op, const Space& s, float* a, const float* b);  // reduce.hip

int binary_nd(int op, Space s, float* a, const float* b) {
  if (op < WF2HIP_ADD || op > WF2HIP_MOVE) return fail(WF2HIP_EINVAL, "unknown binary op %d", op);
  if (s.total == 0) return 0;
  if (!a || !b) return fail(WF2HIP_EINVAL, "null tensor pointer");
  normalise(&s);
  if (hazardous_overlap(s, a, b))
    return fail(WF2HIP_EOVERLAP,
                "in-place op on partially overlapping windows of one buffer; "
                "copy one operand first");
  if (has_broadcast_axis(s, s.sa)) {
    if (op != WF2HIP_MOVE) return launch_accumulate(op, s, a, b);
    keep_last_write(&s);
  }
  switch (op) {
    case WF2HIP_ADD: return launch_elementwise<OpAdd, true>(s, a, b, OpAdd{});
    case WF2HIP_SUB: return launch_elementwise<OpSub, true>(s, a, b, OpSub{});
    case WF2HIP_MUL: return launch_elementwise<OpMul, true>(s, a, b, OpMul{});
    case WF2HIP_DIV: return launch_elementwise<OpDiv, true>(s, a, b, OpDiv{});
    default: return launch_elementwise<OpMove, false>(s, a, b, OpMove{});
  }
}

// dout (the `a` side, updated in place) <- dout f'(x) with x on the `b` side.
int activation_backward_nd(int op, Space s, float* dout, const float* x, float p) {
  if (s.total == 0) return 0;
  if (!dout || !x) return fail(WF2HIP_EINVAL, "null tensor pointer");
  normalise(&s);
  if (hazardous_overlap(s, dout, x))
    return fail(WF2HIP_EOVERLAP, "activation backward between partially overlapping windows");
  if (has_broadcast_axis(s, s.sa))
    return fail(WF2HIP_EINVAL, "activation backward: the gradient may not be a broadcast view");
  switch (op) {
    case WF2HIP_GELU: return launch_elementwise<OpGeluGrad, true>(s, dout, x, OpGeluGrad{});
    case WF2HIP_RELU: return launch_elementwise<OpReluGrad, true>(s, dout, x, OpReluGrad{});
    case WF2HIP_SIGMOID: return launch_elementwise<OpSigmoidGrad, true>(s, dout, x, OpSigmoidGrad{});
    case WF2HIP_LEAKY_RELU: return launch_elementwise<OpLeakyReluGrad, true>(s, dout, x, OpLeakyReluGrad{p});
    default: return fail(WF2HIP_EINVAL, "activation backward: op %d is not an activation", op);
  }
}

// x = source (described by the view's `a` side), out = destination (`b` side).
int unary_nd(int op, Space s, const float* x, float* out, float p) {
  if (s.total == 0) return 0;
  if (!x || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  // launch_elementwise wants dst on the `a` side
  for (int r = 0; r < s.rank; r++) {
    int64_t t = s.sa[r];
    s.sa[r] = s.sb[r];
    s.sb[r] = t;
  }
  int64_t t = s.off_a;
  s.off_a = s.off_b;
  s.off_b = t;
  normalise(&s);
  if (hazardous_overlap(s, out, x))
    return fail(WF2HIP_EOVERLAP, "unary op between partially overlapping windows");
  if (has_broadcast_axis(s, s.sa)) keep_last_write(&s);
  switch (op) {
    case WF2HIP_SIN: return launch_elementwise<OpSin, false>(s, out, x, OpSin{});
    case WF2HIP_COS: return launch_elementwise<OpCos, false>(s, out, x, OpCos{});
    case WF2HIP_TANH: return launch_elementwise<OpTanh, false>(s, out, x, OpTanh{});
    case WF2HIP_LOG: return launch_elementwise<OpLog, false>(s, out, x, OpLog{});
    case WF2HIP_EXP: return launch_elementwise<OpExp, false>(s, out, x, OpExp{});
    case WF2HIP_SQRT: return launch_elementwise<OpSqrt, false>(s, out, x, OpSqrt{});
    case WF2HIP_ABS: return launch_elementwise<OpAbs, false>(s, out, x, OpAbs{});
    case WF2HIP_TAN: return launch_elementwise<OpTan, false>(s, out, x, OpTan{});
    case WF2HIP_ASIN: return launch_elementwise<OpASin, false>(s, out, x, OpASin{});
    case WF2HIP_ACOS: return launch_elementwise<OpACos, false>(s, out, x, OpACos{});
    case WF2HIP_ATAN: return launch_elementwise<OpATan, false>(s, out, x, OpATan{});
    case WF2HIP_SINH: return launch_elementwise<OpSinH, false>(s, out, x, OpSinH{});
    case WF2HIP_COSH: return launch_elementwise<OpCosH, false>(s, out, x, OpCosH{});
    case WF2HIP_LOG2: return launch_elementwise<OpLog2, false>(s, out, x, OpLog2{});
    case WF2HIP_LOG10: return launch_elementwise<OpLog10, false>(s, out, x, OpLog10{});
    case WF2HIP_LOG1P: return launch_elementwise<OpLog1p, false>(s, out, x, OpLog1p{});
    case WF2HIP_INV: return launch_elementwise<OpInv, false>(s, out, x, OpInv{});
    case WF2HIP_SIGN: return launch_elementwise<OpSign, false>(s, out, x, OpSign{});
    case WF2HIP_SQUARE: return launch_elementwise<OpSquare, false>(s, out, x, OpSquare{});
    case WF2HIP_ASINH: return launch_elementwise<OpASinH, false>(s, out, x, OpASinH{});
    case WF2HIP_ACOSH: return launch_elementwise<OpACosH, false>(s, out, x, OpACosH{});
    case WF2HIP_ATANH: return launch_elementwise<OpATanH, false>(s, out, x, OpATanH{});
    case WF2HIP_GELU: return launch_elementwise<OpGelu, false>(s, out, x, OpGelu{});
    case WF2HIP_RELU: return launch_elementwise<OpRelu, false>(s, out, x, OpRelu{});
    case WF2HIP_SIGMOID: return launch_elementwise<OpSigmoid, false>(s, out, x, OpSigmoid{});
    case WF2HIP_LEAKY_RELU: return launch_elementwise<OpLeakyRelu, false>(s, out, x, OpLeakyRelu{p});
    case WF2HIP_POW: return launch_elementwise<OpPow, false>(s, out, x, OpPow{p});
    default: return fail(WF2HIP_EINVAL, "unknown unary op %d", op);
  }
}

// out <- (x OP scal) ? then : else; x on the view's `a` side, out on `b`.
int where_nd(int op, Space s, const float* x, float* out, float scal, float then_value,
             float else_value) {
  if (op < WF2HIP_EQ || op > WF2HIP_GE) return fail(WF2HIP_EINVAL, "unknown compare op %d", op);
  if (s.total == 0) return 0;
  if (!x || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  for (int r = 0; r < s.rank; r++) {
    int64_t t = s.sa[r];
    s.sa[r] = s.sb[r];
    s.sb[r] = t;
  }
  int64_t t = s.off_a;
  s.off_a = s.off_b;
  s.off_b = t;
  normalise(&s);
  if (hazardous_overlap(s, out, x))
    return fail(WF2HIP_EOVERLAP, "compare between partially overlapping windows");
  if (has_broadcast_axis(s, s.sa)) keep_last_write(&s);
  return launch_elementwise<OpWhere, false>(s, out, x, OpWhere{op, scal, then_value, else_value});
}

// x[0] <- 1 / x[0], n times over: what the reference's loop does to a stride-0 run
__global__ void inv_repeated(float* x, long n) {
  float v = *x;
  for (long i = 0; i < n; i++) v = 1.0f / v;
  *x = v;
}

static int space_1d(long n, long inca, long incb, Space* s) {
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  s->rank = 1;
  s->shape[0] = n;
  s->sa[0] = inca;
  s->sb[0] = incb;
  s->off_a = s->off_b = 0;
  s->total = n;
  return 0;
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_binary_nd(int op, const wf2hip_view2* v, float* a, const float* b) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(load_space(v, &s));
  return binary_nd(op, s, a, b);
}

WF2_API int wf2hip_unary_nd(int op, const wf2hip_view2* v, const float* a, float* b, float p) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(load_space(v, &s));
  return unary_nd(op, s, a, b, p);
}

WF2_API int wf2hip_activation_backward_nd(int op, const wf2hip_view2* v, float* dout, const float* x, float p) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(load_space(v, &s));
  return activation_backward_nd(op, s, dout, x, p);
}

#define WF2_DEFINE_BINARY_1D(name, OP)                                                   \
  WF2_API int wf2hip_s##name(long n, float* x, long incx, const float* y, long incy) {  \
    WF2_TRY(require_init());                                                             \
    Space s;                                                                             \
    WF2_TRY(space_1d(n, incx, incy, &s));                                                \
    return binary_nd(OP, s, x, y);                                                       \
  }

WF2_DEFINE_BINARY_1D(add, WF2HIP_ADD)
WF2_DEFINE_BINARY_1D(sub, WF2HIP_SUB)
WF2_DEFINE_BINARY_1D(mul, WF2HIP_MUL)
WF2_DEFINE_BINARY_1D(div, WF2HIP_DIV)

WF2_API int wf2hip_scopy(long n, const float* y, long incy, float* x, long incx) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(space_1d(n, incx, incy, &s));
  return binary_nd(WF2HIP_MOVE, s, x, y);
}

#define WF2_DEFINE_UNARY_1D(name, OP)                                                        \
  WF2_API int wf2hip_s##name(long n, const float* x, long incx, float* out, long inco) {    \
    WF2_TRY(require_init());                                                                 \
    Space s;                                                                                 \
    WF2_TRY(space_1d(n, incx, inco, &s));                                                    \
    return unary_nd(OP, s, x, out, 0.0f);                                                    \
  }

WF2_DEFINE_UNARY_1D(sin, WF2HIP_SIN)
WF2_DEFINE_UNARY_1D(cos, WF2HIP_COS)
WF2_DEFINE_UNARY_1D(tanh, WF2HIP_TANH)
WF2_DEFINE_UNARY_1D(log, WF2HIP_LOG)
WF2_DEFINE_UNARY_1D(exp, WF2HIP_EXP)
WF2_DEFINE_UNARY_1D(sqrt, WF2HIP_SQRT)
WF2_DEFINE_UNARY_1D(abs, WF2HIP_ABS)
WF2_DEFINE_UNARY_1D(tan, WF2HIP_TAN)
WF2_DEFINE_UNARY_1D(asin, WF2HIP_ASIN)
WF2_DEFINE_UNARY_1D(acos, WF2HIP_ACOS)
WF2_DEFINE_UNARY_1D(atan, WF2HIP_ATAN)
WF2_DEFINE_UNARY_1D(sinh, WF2HIP_SINH)
WF2_DEFINE_UNARY_1D(cosh, WF2HIP_COSH)
WF2_DEFINE_UNARY_1D(log2, WF2HIP_LOG2)
WF2_DEFINE_UNARY_1D(log10, WF2HIP_LOG10)
WF2_DEFINE_UNARY_1D(log1p, WF2HIP_LOG1P)

WF2_API int wf2hip_spow(long n, const float* x, long incx, float p, float* out, long inco) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(space_1d(n, incx, inco, &s));
  return unary_nd(WF2HIP_POW, s, x, out, p);
}

WF2_API int wf2hip_where_nd(int op, const wf2hip_view2* v, const float* x, float* out, float scal,
                            float then_value, float else_value) {
  WF2_TRY(require_init());
  Space s;
  WF2_TRY(load_space(v, &s));
  return where_nd(op, s, x, out, scal, then_value, else_value);
}

#define WF2_DEFINE_WHERE_1D(name, OP)                                                            \
  WF2_API int wf2hip_s##name##_scal(long n, const float* x, long incx, float* out, long inco,   \
                                    float y, float then_value, float else_value) {              \
    WF2_TRY(require_init());                                                                     \
    Space s;                                                                                     \
    WF2_TRY(space_1d(n, incx, inco, &s));                                                        \
    return where_nd(OP, s, x, out, y, then_value, else_value);                                   \
  }

WF2_DEFINE_WHERE_1D(eq, WF2HIP_EQ)
WF2_DEFINE_WHERE_1D(lt, WF2HIP_LT)
WF2_DEFINE_WHERE_1D(le, WF2HIP_LE)
WF2_DEFINE_WHERE_1D(gt, WF2HIP_GT)
WF2_DEFINE_WHERE_1D(ge, WF2HIP_GE)

// x <- 1 / x in place.  Replaces waffe2_sinv (cl-waffe2-simd.c:290-302).
WF2_API int wf2hip_sinv(long n, float* x, long incx) {
  WF2_TRY(require_init());
  if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");
  if (n == 0) return 0;
  if (!x) return fail(WF2HIP_EINVAL, "null tensor pointer");
  if (incx == 0) {
    inv_repeated<<<1, 1, 0, rt().stream>>>(x, n);
    return after_launch("inv_repeated");
  }
  Space s;
  WF2_TRY(space_1d(n, incx, incx, &s));
  return unary_nd(WF2HIP_INV, s, x, x, 0.0f);
}
