// compare.hip -- out <- (x OP y) ? then : else over three tensors.
//
// Compare-Operation-Node (source/base-impl/logical.lisp:35-62) compares two
// tensors element by element and writes one of two constants; the CPU backend
// runs it as one waffe2_s{eq,lt,le,gt,ge} call per row
// (source/backends/cpu/logical.lisp:62-84, cl-waffe2-simd.c:385-468).  Here the
// node is one launch: a 16-byte-vector kernel when all three views collapse to
// contiguous runs, an index-decomposing kernel otherwise.  HBM-bound: 12 bytes
// per element (two reads, one write).  The scalar right-hand side
// (Where-Operation-Node) is an element-wise functor in elementwise.hip.
#include "wf2_common.h"
#include "wf2_fastdiv.h"
#include "wf2_view.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bool holds(int op, float a, float b) {
  switch (op) {
    case WF2HIP_EQ: return a == b;
    case WF2HIP_LT: return a < b;
    case WF2HIP_LE: return a <= b;
    case WF2HIP_GT: return a > b;
    default: return a >= b;
  }
}

// all three contiguous and 16-byte aligned.  Three streams, like x <- x + y:
// each wavefront owns 4 KB contiguous per stream and every thread issues its four
// 16-byte loads per operand before the first use (the layout that measured best
// for three-stream kernels, see elementwise.hip).
template <bool NT>
__global__ __launch_bounds__(kBlock) void compare_flat(const float* __restrict__ x,
                                                       const float* __restrict__ y,
                                                       float* __restrict__ out, size_t n, int op,
                                                       float then_value, float else_value) {
  constexpr int U = 4;
  const size_t nvec = n / 4;
  const f4* xv = reinterpret_cast<const f4*>(x);
  const f4* yv = reinterpret_cast<const f4*>(y);
  f4* ov = reinterpret_cast<f4*>(out);
  const unsigned wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const size_t base = ((size_t)blockIdx.x * (kBlock / kWave) + wave) * kWave * U + lane;
  f4 a[U], b[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const size_t i = base + (size_t)u * kWave;
    if (i < nvec) {
      a[u] = NT ? __builtin_nontemporal_load(xv + i) : xv[i];
      b[u] = NT ? __builtin_nontemporal_load(yv + i) : yv[i];
    }
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const size_t i = base + (size_t)u * kWave;
    if (i < nvec) {
      f4 r;
      r.x = holds(op, a[u].x, b[u].x) ? then_value : else_value;
      r.y = holds(op, a[u].y, b[u].y) ? then_value : else_value;
      r.z = holds(op, a[u].z, b[u].z) ? then_value : else_value;
      r.w = holds(op, a[u].w, b[u].w) ? then_value : else_value;
      if (NT)
        __builtin_nontemporal_store(r, ov + i);
      else
        ov[i] = r;
    }
  }
  // the last n % 4 elements
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const size_t i = nvec * 4 + threadIdx.x;
    out[i] = holds(op, x[i], y[i]) ? then_value : else_value;
  }
}

struct Cmp3Params {
  const float* x;
  const float* y;
  float* out;
  int32_t rank, op;
  int64_t total;
  int64_t shape[WF2HIP_MAX_RANK], sa[WF2HIP_MAX_RANK], sb[WF2HIP_MAX_RANK], sc[WF2HIP_MAX_RANK];
  float then_value, else_value;
};

// any strides: one element per thread, innermost axis fastest so that unit
// inner strides stay coalesced
__global__ __launch_bounds__(kBlock) void compare_generic(Cmp3Params p) {
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
  p.out[co] = holds(p.op, p.x[ao], p.y[bo]) ? p.then_value : p.else_value;
}

// Rows: the innermost axis has unit stride in `out` and unit or zero stride in x and y
// (windows of matrices, a row or a column compared against a matrix).  A thread takes
// one 16-byte vector of four rows, all loads before the first store; the vector type
// needs no alignment (see elementwise.hip).  The index-decomposing kernel below ran
// two column windows of (8192, 8192) at 48 % of the HBM peak.
struct CmpRows {
  const float* x;
  const float* y;
  float* out;
  int64_t n0;
  int32_t x_inner, y_inner;  // 1 or 0 (one value per row)
  int32_t nouter, op;
  uint32_t nrows, chunks;
  uint32_t oshape[WF2HIP_MAX_RANK];  // outer axes, innermost of them first
  int64_t ox[WF2HIP_MAX_RANK], oy[WF2HIP_MAX_RANK], oo[WF2HIP_MAX_RANK];
  float then_value, else_value;
};

template <bool NT>
__global__ __launch_bounds__(kBlock) void compare_rows(CmpRows p) {
  typedef f4 f4u __attribute__((aligned(4)));
  constexpr int UR = 4;
  const uint32_t rblock = blockIdx.x / p.chunks;
  const uint32_t chunk = blockIdx.x - rblock * p.chunks;
  const int64_t col = ((int64_t)chunk * kBlock + threadIdx.x) * 4;
  if (col >= p.n0) return;
  const float *xr[UR], *yr[UR];
  float* orow[UR];
  bool live[UR];
#pragma unroll
  for (int u = 0; u < UR; u++) {
    const uint64_t row = (uint64_t)rblock * UR + u;
    live[u] = row < p.nrows;
    uint32_t rem = live[u] ? (uint32_t)row : 0u;
    int64_t xo = 0, yo = 0, oo = 0;
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
      yo += (int64_t)idx * p.oy[i];
      oo += (int64_t)idx * p.oo[i];
    }
    xr[u] = p.x + xo;
    yr[u] = p.y + yo;
    orow[u] = p.out + oo;
  }
  auto pick = [&](float a, float b) { return holds(p.op, a, b) ? p.then_value : p.else_value; };
  if (col + 4 <= p.n0) {
    f4 a[UR], b[UR];
#pragma unroll
    for (int u = 0; u < UR; u++) {
      if (!live[u]) continue;
      if (p.x_inner) {
        const f4u* q = reinterpret_cast<const f4u*>(xr[u] + col);
        a[u] = NT ? __builtin_nontemporal_load(q) : *q;
      } else {
        const float v = xr[u][0];
        a[u] = f4{v, v, v, v};
      }
      if (p.y_inner) {
        const f4u* q = reinterpret_cast<const f4u*>(yr[u] + col);
        b[u] = NT ? __builtin_nontemporal_load(q) : *q;
      } else {
        const float v = yr[u][0];
        b[u] = f4{v, v, v, v};
      }
    }
#pragma unroll
    for (int u = 0; u < UR; u++) {
      if (!live[u]) continue;
      const f4 r = {pick(a[u].x, b[u].x), pick(a[u].y, b[u].y), pick(a[u].z, b[u].z), pick(a[u].w, b[u].w)};
      f4u* q = reinterpret_cast<f4u*>(orow[u] + col);
      if (NT)
        __builtin_nontemporal_store(r, q);
      else
        *q = r;
    }
    return;
  }
  for (int u = 0; u < UR; u++) {  // ragged end of the rows
    if (!live[u]) continue;
    for (int64_t c = col; c < p.n0; c++)
      orow[u][c] = pick(p.x_inner ? xr[u][c] : xr[u][0], p.y_inner ? yr[u][c] : yr[u][0]);
  }
}

// Short rows: matrices whose rows are a few elements long and adjacent in `out` (the windows of a
// pooling layer against their maxima: MaxValue-Node's backward compares (rows, k-h k-w) with a
// (rows, 1) tensor broadcast along the row, base-impl/matrix-ops.lisp:330-334).  compare_rows
// gives a workgroup four rows, which leaves all but one of its threads idle on rows of four
// elements ((6422528, 4): 1.78 ms).  Here a thread takes one 16-byte vector of the flat output,
// U of them kBlock apart, whatever row they fall in: row and column from a division by the row
// length turned into a multiplication (wf2_fastdiv.h; total below 2^31).
struct CmpShort {
  const float* x;
  const float* y;
  float* out;
  uint32_t nvec, total;      // 16-byte vectors of out (the last one may be partial); elements
  FastDiv by_n0;             // the row length
  int64_t ox, oy;            // row strides of x and y
  int32_t x_inner, y_inner;  // 1 or 0 (one value per row)
  int32_t op;
  float then_value, else_value;
};

// ALIGNED: the row length is a multiple of 4, so a thread's vector lies in one row.
template <bool NT, bool ALIGNED>
__global__ __launch_bounds__(kBlock) void compare_short_rows(CmpShort p) {
  typedef f4 f4u __attribute__((aligned(4)));
  constexpr int U = 4;
  f4 a[U], b[U];
  bool live[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t v = (blockIdx.x * U + u) * kBlock + threadIdx.x;
    live[u] = v < p.nvec;
    if (!live[u]) continue;
    const uint32_t e = v * 4;
    if (ALIGNED) {
      uint32_t col;
      const uint32_t row = fd_divmod(e, p.by_n0, &col);
      const float* xr = p.x + (int64_t)row * p.ox;
      const float* yr = p.y + (int64_t)row * p.oy;
      if (p.x_inner) {
        const f4u* q = reinterpret_cast<const f4u*>(xr + col);
        a[u] = NT ? __builtin_nontemporal_load(q) : *q;
      } else {
        const float s = xr[0];
        a[u] = f4{s, s, s, s};
      }
      if (p.y_inner) {
        const f4u* q = reinterpret_cast<const f4u*>(yr + col);
        b[u] = NT ? __builtin_nontemporal_load(q) : *q;
      } else {
        const float s = yr[0];
        b[u] = f4{s, s, s, s};
      }
    } else {  // the four elements may lie in two rows (or four, with rows of one to three elements)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        uint32_t col;
        const uint32_t at = e + c < p.total ? e + c : p.total - 1;
        const uint32_t row = fd_divmod(at, p.by_n0, &col);
        a[u][c] = p.x[(int64_t)row * p.ox + (p.x_inner ? col : 0)];
        b[u][c] = p.y[(int64_t)row * p.oy + (p.y_inner ? col : 0)];
      }
    }
  }
  auto pick = [&](float l, float r) { return holds(p.op, l, r) ? p.then_value : p.else_value; };
#pragma unroll
  for (int u = 0; u < U; u++) {
    if (!live[u]) continue;
    const uint32_t v = (blockIdx.x * U + u) * kBlock + threadIdx.x;
    const f4 r = {pick(a[u].x, b[u].x), pick(a[u].y, b[u].y), pick(a[u].z, b[u].z), pick(a[u].w, b[u].w)};
    if (ALIGNED || v * 4 + 4 <= p.total) {
      f4* q = reinterpret_cast<f4*>(p.out) + v;
      if (NT)
        __builtin_nontemporal_store(r, q);
      else
        *q = r;
    } else {
      for (uint32_t c = 0; v * 4 + c < p.total; c++) p.out[v * 4 + c] = r[c];
    }
  }
}

int compare_nd(int op, Space3 s, const float* x, const float* y, float* out, float then_value,
               float else_value) {
  if (op < WF2HIP_EQ || op > WF2HIP_GE) return fail(WF2HIP_EINVAL, "unknown compare op %d", op);
  if (s.total == 0) return 0;
  if (!x || !y || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  // a stride-0 axis of `out` keeps what the sequential loop writes last
  for (int r = 0; r < s.rank; r++)
    if (s.sc[r] == 0 && s.shape[r] > 1) {
      s.off_a += s.sa[r] * (s.shape[r] - 1);
      s.off_b += s.sb[r] * (s.shape[r] - 1);
      s.shape[r] = 1;
    }
  normalise3(&s);
  if (hazardous3(s, out, s.sa, s.off_a, x) || hazardous3(s, out, s.sb, s.off_b, y))
    return fail(WF2HIP_EOVERLAP, "compare writes into a window that partially overlaps an input");
  hipStream_t st = rt().stream;
  const float* xp = x + s.off_a;
  const float* yp = y + s.off_b;
  float* op_ = out + s.off_c;
  const bool flat = s.rank == 1 && (s.total == 1 || (s.sa[0] == 1 && s.sb[0] == 1 && s.sc[0] == 1)) &&
                    (((uintptr_t)xp | (uintptr_t)yp | (uintptr_t)op_) & 15u) == 0;
  if (flat) {
    const int64_t nvec = s.total / 4;
    const int64_t blocks = ceil_div(nvec > 0 ? nvec : 1, (int64_t)kBlock * 4);
    if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
    if (s.total * 12 >= ((int64_t)192 << 20))
      compare_flat<true><<<(uint32_t)blocks, kBlock, 0, st>>>(xp, yp, op_, (size_t)s.total, op,
                                                              then_value, else_value);
    else
      compare_flat<false><<<(uint32_t)blocks, kBlock, 0, st>>>(xp, yp, op_, (size_t)s.total, op,
                                                               then_value, else_value);
    return after_launch("compare_flat");
  }
  const int last = s.rank - 1;
  bool rows_ok = s.rank >= 2 && s.sc[last] == 1 && (s.sa[last] == 1 || s.sa[last] == 0) &&
                 (s.sb[last] == 1 || s.sb[last] == 0) && s.shape[last] >= 4;
  int64_t nrows = 1;
  for (int r = 0; r < last; r++) {
    if (s.shape[r] >= ((int64_t)1 << 32)) rows_ok = false;
    nrows *= s.shape[r];
  }
  const bool short_rows = s.rank == 2 && s.sc[last] == 1 && (s.sa[last] == 1 || s.sa[last] == 0) &&
                          (s.sb[last] == 1 || s.sb[last] == 0) && s.shape[last] < 1024 && s.sc[0] == s.shape[last] &&
                          s.total < ((int64_t)1 << 31) - 4 && ((uintptr_t)op_ & 15u) == 0;
  if (short_rows) {
    CmpShort q;
    q.x = xp;
    q.y = yp;
    q.out = op_;
    q.nvec = (uint32_t)ceil_div(s.total, 4);
    q.total = (uint32_t)s.total;
    q.by_n0 = make_fastdiv((uint32_t)s.shape[last]);
    q.ox = s.sa[0];
    q.oy = s.sb[0];
    q.x_inner = (int32_t)s.sa[last];
    q.y_inner = (int32_t)s.sb[last];
    q.op = op;
    q.then_value = then_value;
    q.else_value = else_value;
    const uint32_t short_blocks = (uint32_t)ceil_div((int64_t)q.nvec, (int64_t)kBlock * 4);
    if (s.shape[last] % 4 != 0)
      compare_short_rows<false, false><<<short_blocks, kBlock, 0, st>>>(q);
    else if (s.total * 12 >= ((int64_t)192 << 20))
      compare_short_rows<true, true><<<short_blocks, kBlock, 0, st>>>(q);
    else
      compare_short_rows<false, true><<<short_blocks, kBlock, 0, st>>>(q);
    return after_launch("compare_short_rows");
  }
  if (rows_ok && nrows < ((int64_t)1 << 32)) {
    CmpRows q;
    q.x = xp;
    q.y = yp;
    q.out = op_;
    q.n0 = s.shape[last];
    q.x_inner = (int32_t)s.sa[last];
    q.y_inner = (int32_t)s.sb[last];
    q.op = op;
    q.nouter = last;
    for (int i = 0; i < last; i++) {
      const int r = last - 1 - i;
      q.oshape[i] = (uint32_t)s.shape[r];
      q.ox[i] = s.sa[r];
      q.oy[i] = s.sb[r];
      q.oo[i] = s.sc[r];
    }
    q.nrows = (uint32_t)nrows;
    q.chunks = (uint32_t)ceil_div(q.n0, (int64_t)kBlock * 4);
    q.then_value = then_value;
    q.else_value = else_value;
    const int64_t row_blocks = ceil_div(nrows, 4) * q.chunks;
    if (row_blocks < ((int64_t)1 << 31)) {
      if (s.total * 12 >= ((int64_t)192 << 20))
        compare_rows<true><<<(uint32_t)row_blocks, kBlock, 0, st>>>(q);
      else
        compare_rows<false><<<(uint32_t)row_blocks, kBlock, 0, st>>>(q);
      return after_launch("compare_rows");
    }
  }
  Cmp3Params p;
  p.x = xp;
  p.y = yp;
  p.out = op_;
  p.rank = s.rank;
  p.op = op;
  p.total = s.total;
  for (int r = 0; r < s.rank; r++) {
    p.shape[r] = s.shape[r];
    p.sa[r] = s.sa[r];
    p.sb[r] = s.sb[r];
    p.sc[r] = s.sc[r];
  }
  p.then_value = then_value;
  p.else_value = else_value;
  const int64_t blocks = ceil_div(s.total, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "iteration space too large");
  compare_generic<<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  return after_launch("compare_generic");
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_compare_nd(int op, const wf2hip_view3* v, const float* x, const float* y,
                              float* out, float then_value, float else_value) {
  WF2_TRY(require_init());
  Space3 s;
  WF2_TRY(load_space3(v, &s));
  return compare_nd(op, s, x, y, out, then_value, else_value);
}

#define WF2_DEFINE_COMPARE_1D(name, OP)                                                          \
  WF2_API int wf2hip_s##name(long n, const float* x, long incx, const float* y, long incy,       \
                             float* out, long inco, float then_value, float else_value) {        \
    WF2_TRY(require_init());                                                                     \
    if (n < 0) return fail(WF2HIP_EINVAL, "negative element count");                             \
    Space3 s;                                                                                    \
    s.rank = 1;                                                                                  \
    s.shape[0] = n;                                                                              \
    s.sa[0] = incx;                                                                              \
    s.sb[0] = incy;                                                                              \
    s.sc[0] = inco;                                                                              \
    s.total = n;                                                                                 \
    return compare_nd(OP, s, x, y, out, then_value, else_value);                                 \
  }

WF2_DEFINE_COMPARE_1D(eq, WF2HIP_EQ)
WF2_DEFINE_COMPARE_1D(lt, WF2HIP_LT)
WF2_DEFINE_COMPARE_1D(le, WF2HIP_LE)
WF2_DEFINE_COMPARE_1D(gt, WF2HIP_GT)
WF2_DEFINE_COMPARE_1D(ge, WF2HIP_GE)
