// im2col.hip -- unfold / fold for convolution and pooling.
//
// Im2ColNode copies X[N C H W] (already padded by the caller) into
// Col[N C k-h k-w h-out w-out]; Col2ImNode, its backward, adds the columns back
// into X (source/base-impl/unfold.lisp; CPU forwards
// source/backends/cpu/im2col.lisp, kernels cl-waffe2-simd/kernels/im2col.c:
// 63-115 and 395-448 for float, column order).
//
// The reference's loops are kept to the letter, quirks included:
//   for kh, kw:  y runs kh, kh + s_h, ... while y < d_h kh - pad_h + s_h h_out
//                x runs kw, kw + s_w, ... while x < d_w kw - pad_w + s_w w_out
//                col[n c kh kw i j] = im[n c y x]          (i, j count the steps)
// i.e. the dilation and padding arguments only move the end of the walk, and
// with pad > 0 the last rows / columns of a (kh, kw) plane are left untouched.
// Geometries for which that walk would leave its plane of `col` or the image
// (possible with dilation > 1) make the result of the sequential loop depend on
// write order and are refused.
//
// im2col: a workgroup stages the image rows of a band of output rows in LDS and
// writes the band of every (kh, kw) plane from there (im2col_lds); im2col_flat,
// which gathers from im through the caches, where there is no reuse to gain
// (k <= stride) or the rows do not fit; im2col_kernel beyond 2^31 elements.
// col2im: im is the sum, over kh then kw ascending (the reference's order of
// accumulation, so the binary32 result is identical), of the col elements that
// land on it: gathered per element of im, no atomics (col2im_gather; col2im_single
// where windows do not overlap; col2im_kernel beyond 2^31 elements).
// HBM-bound: 4 (k-h k-w h-out w-out + H W) bytes per image plane.
#include <algorithm>

#include "wf2_common.h"
#include "wf2_fastdiv.h"

namespace wf2 {

struct UnfoldParams {
  const float* src;
  float* dst;
  uint32_t N, C, H, W, H_out, W_out, K_H, K_W, s_h, s_w;
  uint32_t count_h[32], count_w[32];  // steps of the walk per kernel row / column
  int64_t total;
};

// col[n c kh kw i j] <- im[n c kh + i s_h, kw + j s_w] for i < count_h[kh], j < count_w[kw]
__global__ __launch_bounds__(kBlock) void im2col_kernel(UnfoldParams p) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= p.total) return;
  int64_t rem = t;
  const uint32_t j = rem % p.W_out; rem /= p.W_out;
  const uint32_t i = rem % p.H_out; rem /= p.H_out;
  const uint32_t kw = rem % p.K_W; rem /= p.K_W;
  const uint32_t kh = rem % p.K_H; rem /= p.K_H;
  const int64_t nc = rem;  // n * C + c
  if (i >= p.count_h[kh] || j >= p.count_w[kw]) return;  // not reached by the reference's walk
  const uint32_t y = kh + i * p.s_h, x = kw + j * p.s_w;
  p.dst[t] = p.src[(nc * p.H + y) * p.W + x];
}

// im[n c y x] <- sum over kh, kw ascending of col[n c kh kw (y - kh)/s_h (x - kw)/s_w]
__global__ __launch_bounds__(kBlock) void col2im_kernel(UnfoldParams p) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= p.total) return;
  int64_t rem = t;
  const uint32_t x = rem % p.W; rem /= p.W;
  const uint32_t y = rem % p.H; rem /= p.H;
  const int64_t nc = rem;
  float acc = 0.0f;
  for (uint32_t kh = 0; kh < p.K_H && kh <= y; kh++) {
    const uint32_t dy = y - kh;
    const uint32_t i = dy / p.s_h;
    if (i * p.s_h != dy || i >= p.count_h[kh]) continue;
    for (uint32_t kw = 0; kw < p.K_W && kw <= x; kw++) {
      const uint32_t dx = x - kw;
      const uint32_t j = dx / p.s_w;
      if (j * p.s_w != dx || j >= p.count_w[kw]) continue;
      acc += p.src[(((nc * p.K_H + kh) * p.K_W + kw) * p.H_out + i) * p.W_out + j];
    }
  }
  p.dst[t] = acc;
}

// The same two maps for tensors below 2^31 elements, in 32-bit index arithmetic with the
// divisions by extents turned into multiplications on the host (wf2_fastdiv.h).
struct Unfold32 {
  const float* src;
  float* dst;
  uint32_t H, W, H_out, W_out, K_H, K_W, s_h, s_w;
  uint32_t d_h, d_w, pad_h, pad_w;
  uint32_t total;          // elements of the destination
  uint32_t plane_elems;    // H_out * W_out
  FastDiv by_plane, by_w_out, by_kw, by_kh;  // im2col: col index -> (n c) kh kw i j
  FastDiv by_w, by_h, by_sh, by_sw;          // col2im: im index -> (n c) y x; steps of the walk
};

// Where the reference's walk of kernel offset k stops: y < d k - pad + s out (im2col.c:75-80).
__device__ __forceinline__ uint32_t walk_end(uint32_t d, uint32_t k, uint32_t pad, uint32_t s, uint32_t out) {
  return d * k + s * out - pad;  // the host has refused geometries where this would be negative
}

// im2col: U elements of col per thread, kBlock apart, so that the lanes of a wavefront read
// (with a unit stride along W) and write consecutive addresses: four consecutive elements per
// lane and one 16-byte store measured no better, because a lane's four loads then lie 16
// bytes from its neighbour's and the L1 handles nine times the accesses (231 MB of col from a
// (32, 64, 58, 58) image, 3 x 3: 73 us).  The first element is decoded in full; the others
// follow by adding kBlock to the position in mixed radix, which costs additions and compares
// where a decode costs eight quarter-rate integer multiplications.
struct ColCursor {
  uint32_t nc, kh, kw, i, j;  // position in col[(n c) kh kw i j]
};

struct ColStep {  // kBlock = ((dnc K_H + dkh) K_W + dkw) plane + di W_out + dj
  uint32_t dnc, dkh, dkw, di, dj;
};

__device__ __forceinline__ ColCursor cursor_at(const Unfold32& p, uint32_t e) {
  ColCursor c;
  uint32_t r;
  const uint32_t plane = fd_divmod(e, p.by_plane, &r);
  c.i = fd_divmod(r, p.by_w_out, &c.j);
  const uint32_t rest = fd_divmod(plane, p.by_kw, &c.kw);
  c.nc = fd_divmod(rest, p.by_kh, &c.kh);
  return c;
}

__device__ __forceinline__ void cursor_advance(const Unfold32& p, const ColStep& d, ColCursor& c) {
  uint32_t carry;
  c.j += d.dj;
  carry = c.j >= p.W_out;
  c.j -= carry ? p.W_out : 0;
  c.i += d.di + carry;
  carry = c.i >= p.H_out;
  c.i -= carry ? p.H_out : 0;
  c.kw += d.dkw + carry;
  carry = c.kw >= p.K_W;
  c.kw -= carry ? p.K_W : 0;
  c.kh += d.dkh + carry;
  carry = c.kh >= p.K_H;
  c.kh -= carry ? p.K_H : 0;
  c.nc += d.dnc + carry;
}

// Workgroup b takes chunk (b mod 8) * per_xcd + b / 8: workgroups are dealt to the eight XCDs in
// turn and each XCD has its own L2, so an XCD walks a contiguous range of col and the K_H K_W
// planes that re-read one image plane find it in that XCD's L2.
// M24: every factor of the index products is below 2^24 (one-pass multiplications).
template <int U, bool M24>
__global__ __launch_bounds__(kBlock) void im2col_flat(Unfold32 p, ColStep d, uint32_t per_xcd) {
  const uint32_t chunk = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
  const uint32_t e0 = chunk * (kBlock * U) + threadIdx.x;
  if ((blockIdx.x >> 3) >= per_xcd || e0 >= p.total) return;
  auto mul = [](uint32_t a, uint32_t b) -> uint32_t { return M24 ? __umul24(a, b) : a * b; };
  ColCursor c = cursor_at(p, e0);
  float v[U];
  bool on[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t y = c.kh + mul(c.i, p.s_h), x = c.kw + mul(c.j, p.s_w);
    // what the reference's walk does not reach stays as it was
    on[u] = e0 + u * kBlock < p.total && y < walk_end(p.d_h, c.kh, p.pad_h, p.s_h, p.H_out) &&
            x < walk_end(p.d_w, c.kw, p.pad_w, p.s_w, p.W_out);
    if (on[u]) v[u] = p.src[mul(mul(c.nc, p.H) + y, p.W) + x];
    if (u + 1 < U) cursor_advance(p, d, c);
  }
#pragma unroll
  for (int u = 0; u < U; u++)
    if (on[u]) p.dst[e0 + u * kBlock] = v[u];
}

// im2col through LDS: a workgroup owns `band_rows` output rows of one image plane (n c), reads
// the image rows they touch once (they are adjacent in memory: one contiguous run) and writes the
// band of all K_H K_W planes of col from LDS, lanes on consecutive addresses on both sides.
// Reads that hit the L2 cost the memory system about what reads from HBM cost (the flat kernel
// above takes as long as a copy of col, 79 us for the 231 MB of a (32, 64, 58, 58) image with a
// 3 x 3 kernel, although it fetches only the 28 MB of the image from HBM), so the K_H K_W-fold
// reuse has to happen inside the workgroup.
// VEC: every band of every plane of col starts on a 16-byte boundary: a lane takes four consecutive
// elements and they leave in one 16-byte nontemporal store (single stores where the walk skips one of them).
// SAME (VEC only): without dilation the walk of every kernel offset takes the same steps (i s_h < s_h H_out -
// pad_h whatever kh is, and likewise along W), so which elements of a vector are reached is worked out once per
// vector, not once per vector and plane.
// HOLES (with SAME): the walk along W stops hole_w elements short of the end of every row of col, and what it
// does not reach keeps its value.  Stores that leave four bytes of a 128-byte line out are merged by the memory
// system at about half the rate of whole lines, so the workgroup reads those elements of its band of every plane
// first (kHolesPerThread per thread at most, in flight while the image rows are staged), keeps them in LDS behind
// the tile -- [plane][row of the band][hole_w], which is the order they come in along the band -- and writes them
// back inside whole 16-byte stores.  Nothing else writes them during the launch: a band of a plane belongs to
// one workgroup.  (The padded walk of a (32, 64, 58, 58) image, 3 x 3: 71 us against 94 with single stores
// around them and 47 without a padding argument; the reads fetch whole 128-byte lines, four of every seven of
// col, and the kernel moves those bytes at the rate it moves the others.)
constexpr int kHolesPerThread = 4;

template <bool VEC, bool SAME, bool HOLES>
__device__ __forceinline__ void im2col_band(float* tile, const Unfold32& p, uint32_t bands, uint32_t band_rows,
                                            uint32_t tile_floats, uint32_t hole_w) {
  const uint32_t nc = blockIdx.x / bands, band = blockIdx.x - nc * bands;
  const uint32_t i0 = band * band_rows;
  const uint32_t rows_here = p.H_out - i0 < band_rows ? p.H_out - i0 : band_rows;
  const uint32_t y0 = i0 * p.s_h;
  if (y0 >= p.H) return;  // uniform; the walk of no kernel row reaches this band
  const uint32_t want = (rows_here - 1) * p.s_h + p.K_H;
  const uint32_t need = want < p.H - y0 ? want : p.H - y0;
  const float* src = p.src + ((size_t)nc * p.H + y0) * p.W;
  float* holes = tile + tile_floats;
  float old[kHolesPerThread];
  if constexpr (HOLES) {
    const uint32_t per_plane = rows_here * hole_w, holes_here = p.K_H * p.K_W * per_plane;
#pragma unroll
    for (int u = 0; u < kHolesPerThread; u++) {
      const uint32_t idx = threadIdx.x + u * kBlock;
      old[u] = 0.0f;
      if (idx < holes_here) {
        const uint32_t plane = idx / per_plane, slot = idx - plane * per_plane;
        const uint32_t il = hole_w == 1 ? slot : slot / hole_w, h = slot - il * hole_w;
        // rows the walk along H does not reach are left alone altogether
        if ((i0 + il) * p.s_h < walk_end(1, 0, p.pad_h, p.s_h, p.H_out))
          old[u] = p.dst[((size_t)nc * p.K_H * p.K_W + plane) * p.plane_elems + (i0 + il) * p.W_out + p.W_out - hole_w + h];
      }
    }
  }
  {  // eight loads in flight per thread
    const uint32_t count = need * p.W;
    uint32_t e = threadIdx.x;
    for (; e + 7 * kBlock < count; e += 8 * kBlock) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = src[e + u * kBlock];
#pragma unroll
      for (int u = 0; u < 8; u++) tile[e + u * kBlock] = v[u];
    }
    for (; e < count; e += kBlock) tile[e] = src[e];
  }
  if constexpr (HOLES) {
#pragma unroll
    for (int u = 0; u < kHolesPerThread; u++) holes[threadIdx.x + u * kBlock] = old[u];
  }
  __syncthreads();
  const uint32_t band_elems = rows_here * p.W_out;
  if constexpr (SAME) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int NV = 4;  // vectors per thread and pass
    const uint32_t end_h = walk_end(1, 0, p.pad_h, p.s_h, p.H_out), end_w = walk_end(1, 0, p.pad_w, p.s_w, p.W_out);
    for (uint32_t base = 0; base < band_elems; base += 4 * kBlock * NV) {
      uint32_t toff[NV][4];  // tile offset of element c of vector u for kh = kw = 0
      // bit c: element c of vector u lies inside the band and both walks; bit 4 + c: inside the band and the
      // walk along H but beyond the one along W (its old value is staged); from bit 8: how many such elements
      // of the band come before the vector
      uint32_t reached[NV];
#pragma unroll
      for (int u = 0; u < NV; u++) {
        const uint32_t e = base + 4 * (threadIdx.x + u * kBlock);
        const bool live = e < band_elems;
        uint32_t j;
        uint32_t il = fd_divmod(live ? e : 0, p.by_w_out, &j);
        reached[u] = 0;
        if constexpr (HOLES) reached[u] = (il * hole_w + (j > p.W_out - hole_w ? j - (p.W_out - hole_w) : 0)) << 8;
#pragma unroll
        for (int c = 0; c < 4; c++) {
          toff[u][c] = il * p.s_h * p.W + j * p.s_w;
          if (live && e + c < band_elems && (i0 + il) * p.s_h < end_h) reached[u] |= (j * p.s_w < end_w ? 1u : 16u) << c;
          if (++j == p.W_out) {
            j = 0;
            il++;
          }
        }
      }
      for (uint32_t plane = 0; plane < p.K_H * p.K_W; plane++) {
        const uint32_t kh = plane / p.K_W, kw = plane - kh * p.K_W;
        float* dst = p.dst + ((size_t)nc * p.K_H * p.K_W + plane) * p.plane_elems + i0 * p.W_out + base;
        const uint32_t shift = kh * p.W + kw;
        const uint32_t staged0 = tile_floats + plane * rows_here * hole_w;
#pragma unroll
        for (int u = 0; u < NV; u++) {
          float* d = dst + 4 * (threadIdx.x + u * kBlock);
          if (HOLES ? ((reached[u] | reached[u] >> 4) & 15u) == 15u : (reached[u] & 15u) == 15u) {
            // one gather for reached elements (from the image rows) and staged ones (behind them)
            uint32_t at = staged0 + (reached[u] >> 8);
            f4 v;
#pragma unroll
            for (int c = 0; c < 4; c++) {
              if constexpr (HOLES) {
                const bool staged = reached[u] >> (4 + c) & 1;
                v[c] = tile[staged ? at : toff[u][c] + shift];
                at += staged;
              } else {
                v[c] = tile[toff[u][c] + shift];
              }
            }
            __builtin_nontemporal_store(v, reinterpret_cast<f4*>(d));
          } else {
            // around what the walk leaves as it was: single stores
#pragma unroll
            for (int c = 0; c < 4; c++)
              if (reached[u] >> c & 1) d[c] = tile[toff[u][c] + shift];
          }
        }
      }
    }
    return;
  }
  if constexpr (VEC) {
    // A thread's vectors (four consecutive elements of the band) are the same in every (kh, kw) plane:
    // their positions in the band and in the tile are worked out once, and a plane costs four LDS reads,
    // a few additions and one store per vector.  Planes the walk covers whole (no padding argument) skip
    // the tests; elsewhere the elements the walk does not reach are stored one by one around the hole.
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int NV = 8;  // vectors per thread and pass
    for (uint32_t base = 0; base < band_elems; base += 4 * kBlock * NV) {
      uint32_t toff[NV][4];   // tile offset of element c of vector u for kh = kw = 0
      uint32_t xs[NV][4], ys[NV][4];
      bool live[NV];
#pragma unroll
      for (int u = 0; u < NV; u++) {
        const uint32_t e = base + 4 * (threadIdx.x + u * kBlock);
        live[u] = e < band_elems;
        uint32_t j;
        uint32_t il = fd_divmod(live[u] ? e : 0, p.by_w_out, &j);
#pragma unroll
        for (int c = 0; c < 4; c++) {
          ys[u][c] = (i0 + il) * p.s_h;
          xs[u][c] = j * p.s_w;
          toff[u][c] = (ys[u][c] - y0) * p.W + xs[u][c];
          if (++j == p.W_out) {
            j = 0;
            il++;
          }
        }
      }
      for (uint32_t kh = 0; kh < p.K_H; kh++) {
        const uint32_t end_h = walk_end(p.d_h, kh, p.pad_h, p.s_h, p.H_out);
        for (uint32_t kw = 0; kw < p.K_W; kw++) {
          const uint32_t end_w = walk_end(p.d_w, kw, p.pad_w, p.s_w, p.W_out);
          float* dst = p.dst + (((size_t)nc * p.K_H + kh) * p.K_W + kw) * p.plane_elems + i0 * p.W_out + base;
          const uint32_t shift = kh * p.W + kw;
          // the whole band of this plane is reached: the last element of the band lies inside both walks
          // (a band is a whole number of vectors: a vector lies inside it or outside)
          const bool whole = kh + (i0 + rows_here - 1) * p.s_h < end_h && kw + (p.W_out - 1) * p.s_w < end_w;
          if (whole) {
#pragma unroll
            for (int u = 0; u < NV; u++) {
              if (!live[u]) continue;
              f4 v;
#pragma unroll
              for (int c = 0; c < 4; c++) v[c] = tile[toff[u][c] + shift];
              __builtin_nontemporal_store(v, reinterpret_cast<f4*>(dst + 4 * (threadIdx.x + u * kBlock)));
            }
          } else {
#pragma unroll
            for (int u = 0; u < NV; u++) {
              if (!live[u]) continue;
              const uint32_t e = base + 4 * (threadIdx.x + u * kBlock);
              f4 v;
              bool on[4];
#pragma unroll
              for (int c = 0; c < 4; c++) {
                on[c] = e + c < band_elems && kh + ys[u][c] < end_h && kw + xs[u][c] < end_w;
                v[c] = on[c] ? tile[toff[u][c] + shift] : 0.0f;
              }
              float* d = dst + 4 * (threadIdx.x + u * kBlock);
              if (on[0] && on[1] && on[2] && on[3]) {
                __builtin_nontemporal_store(v, reinterpret_cast<f4*>(d));
              } else {
                // around what the walk leaves as it was: single stores
#pragma unroll
                for (int c = 0; c < 4; c++)
                  if (on[c]) d[c] = v[c];
              }
            }
          }
        }
      }
    }
    return;
  }
  for (uint32_t kh = 0; kh < p.K_H; kh++) {
    const uint32_t end_h = walk_end(p.d_h, kh, p.pad_h, p.s_h, p.H_out);
    for (uint32_t kw = 0; kw < p.K_W; kw++) {
      const uint32_t end_w = walk_end(p.d_w, kw, p.pad_w, p.s_w, p.W_out);
      float* dst = p.dst + (((size_t)nc * p.K_H + kh) * p.K_W + kw) * p.plane_elems + i0 * p.W_out;
      for (uint32_t e = threadIdx.x; e < band_elems; e += kBlock) {
        uint32_t j;
        const uint32_t il = fd_divmod(e, p.by_w_out, &j);
        const uint32_t y = kh + (i0 + il) * p.s_h, x = kw + j * p.s_w;
        // what the reference's walk does not reach stays as it was
        if (y < end_h && x < end_w) dst[e] = tile[(y - y0) * p.W + x];
      }
    }
  }
}

// (four wavefronts per SIMD: the general form sits at the edge of 128 registers)
template <bool VEC, bool SAME = false>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4, 8))) void im2col_lds(Unfold32 p, uint32_t bands, uint32_t band_rows) {
  extern __shared__ float tile[];  // the image rows y0 ..., W floats each
  im2col_band<VEC, SAME, false>(tile, p, bands, band_rows, 0, 0);
}

__global__ __launch_bounds__(kBlock)
void im2col_lds_holes(Unfold32 p, uint32_t bands, uint32_t band_rows, uint32_t tile_floats, uint32_t hole_w) {
  extern __shared__ float tile[];  // the image rows, then the staged old values
  im2col_band<true, true, true>(tile, p, bands, band_rows, tile_floats, hole_w);
}

// col2im: U elements of im per thread, kBlock apart; the kernel offsets are walked kh ascending,
// then kw ascending (the reference's order of accumulation), and every load of a thread is
// issued before its first addition.  A term the walk does not produce enters as +0, which
// leaves a sum that started at +0 unchanged.  The step i along H depends on kh alone and the
// step j along W on kw alone, so an element costs K_H + K_W divisions, not K_H K_W.
// KH, KW > 0: the kernel extents, loops unrolled; 0: extents from p, one element per thread.
// UNIT: both strides are 1.
template <int KH, int KW, bool UNIT, int U>
__global__ __launch_bounds__(kBlock) void col2im_gather(Unfold32 p) {
  const uint32_t k_h = KH > 0 ? KH : p.K_H, k_w = KW > 0 ? KW : p.K_W;
  // kernel row kh reaches (y, .) at step i when y = kh + i s_h and the walk gets that far
  auto step_h = [&](uint32_t y, uint32_t kh, uint32_t* at) -> bool {
    if (kh > y) return false;
    const uint32_t dy = y - kh;
    const uint32_t i = UNIT ? dy : fd_div(dy, p.by_sh);
    *at = i * p.W_out;
    return (UNIT || i * p.s_h == dy) && i < p.H_out && y < walk_end(p.d_h, kh, p.pad_h, p.s_h, p.H_out);
  };
  auto step_w = [&](uint32_t x, uint32_t kw, uint32_t* at) -> bool {
    if (kw > x) return false;
    const uint32_t dx = x - kw;
    const uint32_t j = UNIT ? dx : fd_div(dx, p.by_sw);
    *at = j;
    return (UNIT || j * p.s_w == dx) && j < p.W_out && x < walk_end(p.d_w, kw, p.pad_w, p.s_w, p.W_out);
  };
  if (KH > 0) {
    constexpr int NH = KH > 0 ? KH : 1, NW = KW > 0 ? KW : 1;
    float v[U][NH][NW];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t t = (blockIdx.x * U + u) * kBlock + threadIdx.x;
      uint32_t x, y;
      const uint32_t row = fd_divmod(t, p.by_w, &x);
      const uint32_t nc = fd_divmod(row, p.by_h, &y);
      const float* src = p.src + (size_t)nc * (NH * NW) * p.plane_elems;
      uint32_t ai[NH], aj[NW];
      bool oh[NH], ow[NW];
#pragma unroll
      for (int kh = 0; kh < NH; kh++) oh[kh] = t < p.total && step_h(y, kh, &ai[kh]);
#pragma unroll
      for (int kw = 0; kw < NW; kw++) ow[kw] = step_w(x, kw, &aj[kw]);
#pragma unroll
      for (int kh = 0; kh < NH; kh++)
#pragma unroll
        for (int kw = 0; kw < NW; kw++)
          v[u][kh][kw] = (oh[kh] && ow[kw]) ? src[(kh * NW + kw) * p.plane_elems + ai[kh] + aj[kw]] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const uint32_t t = (blockIdx.x * U + u) * kBlock + threadIdx.x;
      float acc = 0.0f;
#pragma unroll
      for (int kh = 0; kh < NH; kh++)
#pragma unroll
        for (int kw = 0; kw < NW; kw++) acc += v[u][kh][kw];
      if (t < p.total) p.dst[t] = acc;
    }
  } else {
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= p.total) return;
    uint32_t x, y;
    const uint32_t row = fd_divmod(t, p.by_w, &x);
    const uint32_t nc = fd_divmod(row, p.by_h, &y);
    const float* src = p.src + (size_t)nc * k_h * k_w * p.plane_elems;
    float acc = 0.0f;
    for (uint32_t kh = 0; kh < k_h && kh <= y; kh++) {
      uint32_t ai, aj;
      if (!step_h(y, kh, &ai)) continue;
      const float* rowp = src + kh * k_w * p.plane_elems + ai;
      for (uint32_t kw = 0; kw < k_w && kw <= x; kw++)
        if (step_w(x, kw, &aj)) acc += rowp[kw * p.plane_elems + aj];
    }
    p.dst[t] = acc;
  }
}

// col2im when the windows do not overlap (K_H <= s_h and K_W <= s_w, as in pooling): an element
// of im belongs to at most one window, so it is one load, not a sum.  FAST: the strides are
// powers of two (shifts instead of divisions) and every factor of the index products is below
// 2^24 (one-pass multiplications); the index arithmetic is what bounds this kernel.
template <bool FAST, int U>
__global__ __launch_bounds__(kBlock) void col2im_single(Unfold32 p, uint32_t log_sh, uint32_t log_sw) {
  auto mul = [](uint32_t a, uint32_t b) -> uint32_t { return FAST ? __umul24(a, b) : a * b; };
  float v[U];
#pragma unroll
  for (int u = 0; u < U; u++) {  // the loads of a thread are all issued before its stores
    const uint32_t t = (blockIdx.x * U + u) * kBlock + threadIdx.x;
    uint32_t x, y, kh, kw, i, j;
    const uint32_t row = fd_divmod(t, p.by_w, &x);
    const uint32_t nc = fd_divmod(row, p.by_h, &y);
    if (FAST) {
      i = y >> log_sh;
      kh = y & (p.s_h - 1);
      j = x >> log_sw;
      kw = x & (p.s_w - 1);
    } else {
      i = fd_divmod(y, p.by_sh, &kh);
      j = fd_divmod(x, p.by_sw, &kw);
    }
    const bool on = t < p.total && kh < p.K_H && kw < p.K_W && i < p.H_out && j < p.W_out &&
                    y < walk_end(p.d_h, kh, p.pad_h, p.s_h, p.H_out) &&
                    x < walk_end(p.d_w, kw, p.pad_w, p.s_w, p.W_out);
    v[u] = 0.0f;
    if (on) v[u] += p.src[mul(mul(mul(nc, p.K_H) + kh, p.K_W) + kw, p.plane_elems) + mul(i, p.W_out) + j];
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t t = (blockIdx.x * U + u) * kBlock + threadIdx.x;
    if (t < p.total) p.dst[t] = v[u];
  }
}

static int make_params(long N, long C, long H, long W, long H_out, long W_out, long K_H, long K_W,
                       long pad_h, long pad_w, long stride_h, long stride_w, long dilation_h,
                       long dilation_w, UnfoldParams* p) {
  if (N < 0 || C < 0 || H < 0 || W < 0 || H_out < 0 || W_out < 0 || K_H < 1 || K_W < 1 || pad_h < 0 ||
      pad_w < 0 || stride_h < 1 || stride_w < 1 || dilation_h < 1 || dilation_w < 1)
    return fail(WF2HIP_EINVAL, "im2col: negative extent or non-positive kernel / stride / dilation");
  if (K_H > 32 || K_W > 32) return fail(WF2HIP_EUNSUPPORTED, "im2col: kernels up to 32 x 32");
  const long limit = (long)1 << 31;
  if (N * C >= limit || H >= limit || W >= limit || H_out >= limit || W_out >= limit)
    return fail(WF2HIP_EUNSUPPORTED, "im2col: extent beyond 2^31");
  p->N = N; p->C = C; p->H = H; p->W = W; p->H_out = H_out; p->W_out = W_out;
  p->K_H = K_H; p->K_W = K_W; p->s_h = stride_h; p->s_w = stride_w;
  for (int axis = 0; axis < 2; axis++) {
    const long K = axis ? K_W : K_H, d = axis ? dilation_w : dilation_h, pad = axis ? pad_w : pad_h;
    const long s = axis ? stride_w : stride_h, out = axis ? W_out : H_out, size = axis ? W : H;
    for (long k = 0; k < K; k++) {
      const long end = d * k - pad + s * out;  // the reference evaluates this in uint64
      if (end < 0) return fail(WF2HIP_EUNSUPPORTED, "im2col: padding larger than the walk");
      const long steps = end > k ? (end - k + s - 1) / s : 0;
      if (steps > out)
        return fail(WF2HIP_EUNSUPPORTED,
                    "im2col: the walk of kernel offset %ld takes %ld steps but the plane has %ld "
                    "(dilation > 1 is not reproducible)", k, steps, out);
      if (steps > 0 && k + (steps - 1) * s >= size)
        return fail(WF2HIP_EINVAL, "im2col: the walk leaves the image (pass the padded image)");
      (axis ? p->count_w : p->count_h)[k] = (uint32_t)steps;
    }
  }
  return 0;
}

// The 32-bit form of a validated geometry; false when an index would not fit.
static bool make_unfold32(long N, long C, long H, long W, long H_out, long W_out, long K_H, long K_W, long pad_h,
                          long pad_w, long stride_h, long stride_w, long dilation_h, long dilation_w, Unfold32* q) {
  const int64_t limit = (int64_t)1 << 31;
  const int64_t n_im = (int64_t)N * C * H * W, n_col = (int64_t)N * C * K_H * K_W * H_out * W_out;
  // the ends of the walks are formed in 32 bits too
  const int64_t end_h = dilation_h * (K_H - 1) + stride_h * H_out, end_w = dilation_w * (K_W - 1) + stride_w * W_out;
  if (n_im >= limit || n_col >= limit || end_h >= limit || end_w >= limit || pad_h >= limit || pad_w >= limit)
    return false;
  q->H = (uint32_t)H; q->W = (uint32_t)W; q->H_out = (uint32_t)H_out; q->W_out = (uint32_t)W_out;
  q->K_H = (uint32_t)K_H; q->K_W = (uint32_t)K_W; q->s_h = (uint32_t)stride_h; q->s_w = (uint32_t)stride_w;
  q->d_h = (uint32_t)dilation_h; q->d_w = (uint32_t)dilation_w; q->pad_h = (uint32_t)pad_h; q->pad_w = (uint32_t)pad_w;
  q->plane_elems = (uint32_t)(H_out * W_out);
  q->by_plane = make_fastdiv(q->plane_elems);
  q->by_w_out = make_fastdiv(q->W_out);
  q->by_kw = make_fastdiv(q->K_W);
  q->by_kh = make_fastdiv(q->K_H);
  q->by_w = make_fastdiv(q->W);
  q->by_h = make_fastdiv(q->H);
  q->by_sh = make_fastdiv(q->s_h);
  q->by_sw = make_fastdiv(q->s_w);
  return true;
}

template <bool UNIT>
static void launch_col2im(const Unfold32& q, hipStream_t st) {
  auto blocks = [&](int u) { return (uint32_t)ceil_div((int64_t)q.total, (int64_t)kBlock * u); };
  if (q.K_H == q.K_W && q.K_H == 1)
    col2im_gather<1, 1, UNIT, 4><<<blocks(4), kBlock, 0, st>>>(q);
  else if (q.K_H == q.K_W && q.K_H == 2)
    col2im_gather<2, 2, UNIT, 4><<<blocks(4), kBlock, 0, st>>>(q);
  else if (q.K_H == q.K_W && q.K_H == 3)
    col2im_gather<3, 3, UNIT, (UNIT ? 1 : 4)><<<blocks(UNIT ? 1 : 4), kBlock, 0, st>>>(q);
  else if (q.K_H == q.K_W && q.K_H == 5)
    col2im_gather<5, 5, UNIT, (UNIT ? 1 : 2)><<<blocks(UNIT ? 1 : 2), kBlock, 0, st>>>(q);
  else if (q.K_H == q.K_W && q.K_H == 7)
    col2im_gather<7, 7, UNIT, 1><<<blocks(1), kBlock, 0, st>>>(q);
  else
    col2im_gather<0, 0, UNIT, 1><<<blocks(1), kBlock, 0, st>>>(q);
}

// ---- unfold as one kernel -----------------------------------------------------------------------
// (unfold input dilation kernel-size stride padding) of source/nn/im2col.lisp:51-95 composes a
// zero-padded copy of the image, Im2ColNode into a zeroed col[N C kh kw i j], a permuting copy to
// (N i j C kh kw) and a reshape to [(N h-out w-out) (C k-h k-w)]: four passes over tensors of
// col's size.  Here the matrix is written once, from image rows staged in LDS:
//   out[(n i j), (c kh kw)] = reached(i, j) ? padded[n c, kh + i s_h, kw + j s_w] : 0
// with `padded` zero outside the image and reached(i, j) what Im2ColNode's walk visits
// (dilation 1: i s_h + pad_h < s_h h-out and j s_w + pad_w < s_w w-out, whatever kh and kw are).
// A workgroup owns `band` output rows i of one image n and `cc` channels: its part of the matrix
// is, per (i, j), a run of cc K_H K_W consecutive floats (the whole band is one run when it owns
// every channel).  Two small tables in LDS turn the position in the run, and the position (i, j),
// into offsets into the staged tile.
struct UnfoldFused {
  const float* src;
  float* dst;
  uint32_t C, H, W, H_out, W_out, K_H, K_W, s_h, s_w, pad_h, pad_w;
  uint32_t band, bands, cc, chunks;  // output rows per workgroup, channels per workgroup
  uint32_t TR, TW;                   // rows and columns of the staged tile per channel
  uint32_t Q;                        // C K_H K_W
  FastDiv by_kk, by_kw, by_w_out, by_plane, by_tw;  // K_H K_W, K_W, W_out, TR TW, TW
};

// VEC: runs are whole 16-byte vectors on 16-byte boundaries (cc K_H K_W and C K_H K_W multiples of 4, dst
// aligned): a lane then owns NQ vectors of four consecutive entries and the matrix leaves in 16-byte
// nontemporal stores, a quarter of the store instructions of the element form.
template <int NQ, bool VEC = false>  // entries (VEC: vectors) of a run per lane: cc K_H K_W <= 64 NQ (256 NQ)
__global__ __launch_bounds__(kBlock) void unfold_kernel(UnfoldFused p) {
  extern __shared__ float lds[];
  const uint32_t KK = p.K_H * p.K_W;
  const uint32_t plane = p.TR * p.TW;
  float* tile = lds;                                                   // [cc][TR][TW]
  uint32_t* qoff = reinterpret_cast<uint32_t*>(lds + p.cc * plane);    // [cc KK]
  uint32_t* roff = qoff + p.cc * KK;                                   // [band W_out]
  const uint32_t chunk = blockIdx.x % p.chunks;
  const uint32_t rest = blockIdx.x / p.chunks;
  const uint32_t band = rest % p.bands, n = rest / p.bands;
  const uint32_t c0 = chunk * p.cc;
  const uint32_t cc = p.C - c0 < p.cc ? p.C - c0 : p.cc;
  const uint32_t run = cc * KK;
  const uint32_t i0 = band * p.band;
  const uint32_t rows_here = p.H_out - i0 < p.band ? p.H_out - i0 : p.band;
  const uint32_t R = rows_here * p.W_out;
  constexpr uint32_t kSkipped = 0xffffffffu;
  for (uint32_t q = threadIdx.x; q < run; q += kBlock) {
    uint32_t r, kw;
    const uint32_t c = fd_divmod(q, p.by_kk, &r);
    const uint32_t kh = fd_divmod(r, p.by_kw, &kw);
    qoff[q] = (c * p.TR + kh) * p.TW + kw;
  }
  for (uint32_t r = threadIdx.x; r < R; r += kBlock) {
    uint32_t j;
    const uint32_t il = fd_divmod(r, p.by_w_out, &j);
    const bool reached = (i0 + il) * p.s_h + p.pad_h < p.s_h * p.H_out && j * p.s_w + p.pad_w < p.s_w * p.W_out;
    roff[r] = reached ? il * p.s_h * p.TW + j * p.s_w : kSkipped;
  }
  // the tile: rows i0 s_h - pad_h ... of the image, columns -pad_w ..., zero outside the image
  const int32_t y_first = (int32_t)(i0 * p.s_h) - (int32_t)p.pad_h;
  const float* img = p.src + ((size_t)n * p.C + c0) * p.H * p.W;
  auto fetch = [&](uint32_t e) -> float {
    uint32_t r, tx;
    const uint32_t c = fd_divmod(e, p.by_plane, &r);
    const uint32_t ty = fd_divmod(r, p.by_tw, &tx);
    const int32_t y = y_first + (int32_t)ty, x = (int32_t)tx - (int32_t)p.pad_w;
    const bool inside = y >= 0 && y < (int32_t)p.H && x >= 0 && x < (int32_t)p.W;
    return inside ? img[((size_t)c * p.H + y) * p.W + x] : 0.0f;
  };
  {  // eight loads in flight per thread
    const uint32_t count = cc * plane;
    uint32_t e = threadIdx.x;
    for (; e + 7 * kBlock < count; e += 8 * kBlock) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = fetch(e + u * kBlock);
#pragma unroll
      for (int u = 0; u < 8; u++) tile[e + u * kBlock] = v[u];
    }
    for (; e < count; e += kBlock) tile[e] = fetch(e);
  }
  __syncthreads();
  float* out = p.dst + ((size_t)n * p.H_out + i0) * p.W_out * p.Q + (size_t)c0 * KK;
  // A wavefront owns the positions r = wave, wave + 4, ...; its lanes sweep the run, NQ entries
  // each, whose tile offsets stay in registers: an element is one LDS read and one store.
  const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if constexpr (VEC) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    uint32_t off[NQ][4];
#pragma unroll
    for (int m = 0; m < NQ; m++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const uint32_t qc = 4 * (lane + m * kWave) + c;
        off[m][c] = qc < run ? qoff[qc] : 0;
      }
    for (uint32_t r = wave; r < R; r += kBlock / kWave) {
      const uint32_t ro = roff[r];  // uniform over the wavefront
      float* row = out + (size_t)r * p.Q;
      f4 v[NQ];
#pragma unroll
      for (int m = 0; m < NQ; m++)
#pragma unroll
        for (int c = 0; c < 4; c++) v[m][c] = ro == kSkipped ? 0.0f : tile[off[m][c] + ro];
#pragma unroll
      for (int m = 0; m < NQ; m++) {
        const uint32_t qc = 4 * (lane + m * kWave);
        if (qc < run) __builtin_nontemporal_store(v[m], reinterpret_cast<f4*>(row + qc));
      }
    }
  } else {
  uint32_t off[NQ];
#pragma unroll
  for (int m = 0; m < NQ; m++) {
    const uint32_t qc = lane + m * kWave;
    off[m] = qc < run ? qoff[qc] : 0;
  }
  for (uint32_t r = wave; r < R; r += kBlock / kWave) {
    const uint32_t ro = roff[r];  // uniform over the wavefront
    float* row = out + (size_t)r * p.Q;
    float v[NQ];
#pragma unroll
    for (int m = 0; m < NQ; m++) v[m] = ro == kSkipped ? 0.0f : tile[off[m] + ro];
#pragma unroll
    for (int m = 0; m < NQ; m++) {
      const uint32_t qc = lane + m * kWave;
      if (qc < run) row[qc] = v[m];
    }
  }
  }
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_im2col_f32(float* col, long N, long C, long H, long W, long H_out, long W_out,
                              long K_H, long K_W, long pad_h, long pad_w, long stride_h,
                              long stride_w, long dilation_h, long dilation_w, const float* im) {
  WF2_TRY(require_init());
  UnfoldParams p;
  WF2_TRY(make_params(N, C, H, W, H_out, W_out, K_H, K_W, pad_h, pad_w, stride_h, stride_w,
                      dilation_h, dilation_w, &p));
  p.total = (int64_t)N * C * K_H * K_W * H_out * W_out;
  if (p.total == 0) return 0;
  if (!col || !im) return fail(WF2HIP_EINVAL, "null tensor pointer");
  p.src = im;
  p.dst = col;
  Unfold32 q;
  if (make_unfold32(N, C, H, W, H_out, W_out, K_H, K_W, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, &q)) {
    q.src = im;
    q.dst = col;
    q.total = (uint32_t)p.total;
    // the band of output rows whose image rows fit 16 KB of LDS, so that eight workgroups share a
    // compute unit and the loading of one overlaps the storing of the others (48 KB where K_H
    // image rows need more)
    const int64_t lds_floats = (int64_t)K_H * W * 4 <= (16 << 10) ? (16 << 10) / 4 : (48 << 10) / 4;
    const int64_t rows_fit = W > 0 ? lds_floats / W : 0;  // image rows
    if (rows_fit >= K_H && K_H * K_W > stride_h * stride_w) {  // some reuse of the image to gain from
      int64_t band_rows = std::min<int64_t>((rows_fit - K_H) / stride_h + 1, H_out);
      // at least two workgroups per compute unit where the planes are few
      const int64_t planes = (int64_t)N * C;
      const int64_t cus = std::max(rt().num_cus, 1);
      while (band_rows > 8 && planes * ceil_div(H_out, band_rows) < 2 * cus) band_rows = (band_rows + 1) / 2;
      const int64_t bands = ceil_div(H_out, band_rows);
      const int64_t tile_rows = std::min<int64_t>((band_rows - 1) * stride_h + K_H, H);
      if (planes * bands < ((int64_t)1 << 31)) {
        static const char* vec_env = getenv("WF2HIP_UNFOLD_VEC");  // testing knob: 0 = stores of single elements
        const bool vec = ((uintptr_t)col % 16) == 0 && (H_out * W_out) % 4 == 0 && (band_rows * W_out) % 4 == 0 &&
                         !(vec_env && vec_env[0] == '0');
        bool untouched = false;  // does the walk leave elements of col as they were?
        for (long k = 0; k < K_H; k++) untouched |= (long)p.count_h[k] < H_out;
        for (long k = 0; k < K_W; k++) untouched |= (long)p.count_w[k] < W_out;
        const bool same = vec && untouched && dilation_h == 1 && dilation_w == 1;
        const int64_t hole_w = W_out - (int64_t)p.count_w[0];  // without dilation: of every kw
        static const char* holes_env = getenv("WF2HIP_IM2COL_HOLES");  // testing knob: 0 = single stores around them
        const bool holes = same && hole_w > 0 && hole_w < W_out &&
                           K_H * K_W * band_rows * hole_w <= (int64_t)kHolesPerThread * kBlock &&
                           !(holes_env && holes_env[0] == '0');
        if (holes)
          im2col_lds_holes<<<(uint32_t)(planes * bands), kBlock,
                             ((size_t)tile_rows * W + kHolesPerThread * kBlock) * sizeof(float), rt().stream>>>(
              q, (uint32_t)bands, (uint32_t)band_rows, (uint32_t)(tile_rows * W), (uint32_t)hole_w);
        else if (same)
          im2col_lds<true, true><<<(uint32_t)(planes * bands), kBlock, (size_t)tile_rows * W * sizeof(float), rt().stream>>>(
              q, (uint32_t)bands, (uint32_t)band_rows);
        else if (vec)
          im2col_lds<true><<<(uint32_t)(planes * bands), kBlock, (size_t)tile_rows * W * sizeof(float), rt().stream>>>(
              q, (uint32_t)bands, (uint32_t)band_rows);
        else
          im2col_lds<false><<<(uint32_t)(planes * bands), kBlock, (size_t)tile_rows * W * sizeof(float), rt().stream>>>(
              q, (uint32_t)bands, (uint32_t)band_rows);
        return after_launch("im2col_lds");
      }
    }
    constexpr int U = 4;  // 8 and 16 measure the same
    const uint32_t per_xcd = (uint32_t)ceil_div(ceil_div(p.total, (int64_t)kBlock * U), 8);
    ColStep d;  // kBlock in the mixed radix of col's index
    uint32_t rest = kBlock / q.plane_elems, in_plane = kBlock % q.plane_elems;
    d.di = in_plane / q.W_out;
    d.dj = in_plane % q.W_out;
    d.dkw = rest % q.K_W;
    rest /= q.K_W;
    d.dkh = rest % q.K_H;
    d.dnc = rest / q.K_H;
    const int64_t u24 = (int64_t)1 << 24;
    const bool m24 = (int64_t)N * C * H < u24 && W < u24 && H_out < u24 && W_out < u24 && stride_h < u24 && stride_w < u24;
    if (m24)
      im2col_flat<U, true><<<per_xcd * 8, kBlock, 0, rt().stream>>>(q, d, per_xcd);
    else
      im2col_flat<U, false><<<per_xcd * 8, kBlock, 0, rt().stream>>>(q, d, per_xcd);
    return after_launch("im2col_flat");
  }
  const int64_t blocks = ceil_div(p.total, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "im2col: too many elements");
  im2col_kernel<<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(p);
  return after_launch("im2col_kernel");
}

WF2_API int wf2hip_col2im_f32(const float* col, long N, long C, long H, long W, long H_out,
                              long W_out, long K_H, long K_W, long pad_h, long pad_w, long stride_h,
                              long stride_w, long dilation_h, long dilation_w, float* im) {
  WF2_TRY(require_init());
  UnfoldParams p;
  WF2_TRY(make_params(N, C, H, W, H_out, W_out, K_H, K_W, pad_h, pad_w, stride_h, stride_w,
                      dilation_h, dilation_w, &p));
  p.total = (int64_t)N * C * H * W;
  if (p.total == 0) return 0;
  if (!col || !im) return fail(WF2HIP_EINVAL, "null tensor pointer");
  p.src = col;
  p.dst = im;
  const int64_t blocks = ceil_div(p.total, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "col2im: too many elements");
  Unfold32 q;
  if (make_unfold32(N, C, H, W, H_out, W_out, K_H, K_W, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, &q)) {
    q.src = col;
    q.dst = im;
    q.total = (uint32_t)p.total;
    if (K_H <= stride_h && K_W <= stride_w && !(stride_h == 1 && stride_w == 1)) {
      auto pow2 = [](long v) { return (v & (v - 1)) == 0; };
      auto log2 = [](long v) { uint32_t l = 0; while ((1L << l) < v) l++; return l; };
      const int64_t u24 = (int64_t)1 << 24;
      const bool fast = pow2(stride_h) && pow2(stride_w) && (int64_t)N * C * K_H * K_W < u24 &&
                        (int64_t)H_out * W_out < u24;
      const uint32_t blocks4 = (uint32_t)ceil_div(p.total, (int64_t)kBlock * 4);  // 16 per thread: slower
      if (fast)
        col2im_single<true, 4><<<blocks4, kBlock, 0, rt().stream>>>(q, log2(stride_h), log2(stride_w));
      else
        col2im_single<false, 4><<<blocks4, kBlock, 0, rt().stream>>>(q, 0, 0);
    }
    else if (stride_h == 1 && stride_w == 1)
      launch_col2im<true>(q, rt().stream);
    else
      launch_col2im<false>(q, rt().stream);
    return after_launch("col2im_gather");
  }
  col2im_kernel<<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(p);
  return after_launch("col2im_kernel");
}

WF2_API int wf2hip_unfold_f32(long N, long C, long H, long W, long K_H, long K_W, long stride_h, long stride_w,
                              long pad_h, long pad_w, const float* x, float* out) {
  WF2_TRY(require_init());
  if (N < 0 || C < 0 || H < 0 || W < 0 || K_H < 1 || K_W < 1 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0)
    return fail(WF2HIP_EINVAL, "unfold: negative extent or non-positive kernel / stride");
  if (H + 2 * pad_h < K_H || W + 2 * pad_w < K_W) return fail(WF2HIP_EINVAL, "unfold: kernel larger than the padded image");
  const long H_out = (H + 2 * pad_h - K_H) / stride_h + 1, W_out = (W + 2 * pad_w - K_W) / stride_w + 1;
  const int64_t limit = (int64_t)1 << 31;
  const int64_t Q = (int64_t)C * K_H * K_W, rows = (int64_t)N * H_out * W_out;
  if (rows == 0 || Q == 0) return 0;
  if (!x || !out) return fail(WF2HIP_EINVAL, "null tensor pointer");
  if (Q >= limit || H_out * W_out >= limit || (int64_t)H * W >= limit || stride_h * H_out + pad_h >= limit ||
      stride_w * W_out + pad_w >= limit)
    return fail(WF2HIP_EUNSUPPORTED, "unfold: extent beyond 2^31");
  {  // out must not overlap x
    const float* xe = x + (int64_t)N * C * H * W;
    const float* oe = out + rows * Q;
    if (x < oe && out < xe) return fail(WF2HIP_EOVERLAP, "unfold: the matrix overlaps the image");
  }
  UnfoldFused p;
  p.src = x; p.dst = out;
  p.C = (uint32_t)C; p.H = (uint32_t)H; p.W = (uint32_t)W; p.H_out = (uint32_t)H_out; p.W_out = (uint32_t)W_out;
  p.K_H = (uint32_t)K_H; p.K_W = (uint32_t)K_W; p.s_h = (uint32_t)stride_h; p.s_w = (uint32_t)stride_w;
  p.pad_h = (uint32_t)pad_h; p.pad_w = (uint32_t)pad_w;
  p.Q = (uint32_t)Q;
  const int64_t KK = K_H * K_W;
  const int64_t TW = (W_out - 1) * stride_w + K_W;
  // The split into bands of output rows and chunks of channels, among those whose tile and tables
  // fit 60 KB of LDS.  Measured on (32, 64, 56, 56) with a 3 x 3 kernel (231 MB written): runs whose
  // length is not a multiple of 64 bytes double the time (104 us against 55 us), more than 32 KB
  // of LDS per workgroup costs a fifth (66 us), idle lanes at the end of a run and the image rows
  // that neighbouring bands both read cost little.
  if (KK > 1024) return fail(WF2HIP_EUNSUPPORTED, "unfold: kernels up to 1024 elements");
  auto tile_rows = [&](int64_t b) { return (b - 1) * stride_h + K_H; };
  auto lds_floats = [&](int64_t b, int64_t c) { return c * tile_rows(b) * TW + c * KK + b * W_out; };
  const int64_t ceiling = (60 << 10) / 4, roomy = (32 << 10) / 4;
  int64_t band = 0, cc = 0;
  double best = 0.0;
  for (int64_t b = std::max<int64_t>(1, std::min<int64_t>(256 / W_out, H_out)); b >= 1; b = b > 1 ? (b + 1) / 2 : 0) {
    const int64_t most = std::min<int64_t>({C, 1024 / KK, (ceiling - b * W_out) / (tile_rows(b) * TW + KK)});
    for (int64_t c = most; c >= 1; c--) {
      const int64_t whole = C / c, last = C - whole * c;  // chunks of c channels and a shorter one
      const int64_t slots = whole * ceil_div(c * KK, kWave) + (last ? ceil_div(last * KK, kWave) : 0);
      const double lanes = (double)Q / (double)(slots * kWave);
      const double reads = (double)(tile_rows(b) * TW) / (double)(b * W_out * KK);
      const bool aligned = (c * KK) % 16 == 0 || c == C;
      const double score = lanes * (aligned ? 1.0 : 0.5) * (lds_floats(b, c) <= roomy ? 1.0 : 0.85) / (1.0 + 0.3 * reads);
      if (band == 0 || score > best * 1.02) {  // near ties go to the longer run, tried first
        best = score;
        band = b;
        cc = c;
      }
    }
  }
  if (band == 0)
    return fail(WF2HIP_EUNSUPPORTED, "unfold: one channel of one output row needs more than 60 KB of LDS (compose it from nodes)");
  p.band = (uint32_t)band;
  p.bands = (uint32_t)ceil_div(H_out, band);
  p.cc = (uint32_t)cc;
  p.chunks = (uint32_t)ceil_div(C, cc);
  p.TR = (uint32_t)tile_rows(band);
  p.TW = (uint32_t)TW;
  p.by_kk = make_fastdiv((uint32_t)KK);
  p.by_kw = make_fastdiv(p.K_W);
  p.by_w_out = make_fastdiv(p.W_out);
  p.by_plane = make_fastdiv(p.TR * p.TW);
  p.by_tw = make_fastdiv(p.TW);
  const int64_t blocks = (int64_t)N * p.bands * p.chunks;
  if (blocks >= limit) return fail(WF2HIP_EUNSUPPORTED, "unfold: too many workgroups");
  const size_t bytes = (size_t)lds_floats(band, cc) * sizeof(float);
  hipStream_t st = rt().stream;
  static const char* vec_env = getenv("WF2HIP_UNFOLD_VEC");  // testing knob: 0 = stores of single elements
  const bool vec = (cc * KK) % 4 == 0 && ((int64_t)C * KK) % 4 == 0 && ((uintptr_t)out % 16) == 0 &&
                   !(vec_env && vec_env[0] == '0');
  if (vec) {
    const int64_t vecs_per_lane = ceil_div(cc * KK, (int64_t)kWave * 4);
#define WF2_VCASE(NQ_)                                                                                           \
  if (vecs_per_lane <= NQ_) {                                                                                    \
    static bool configured = false;                                                                              \
    if (!configured) {                                                                                           \
      WF2_TRY(check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&unfold_kernel<NQ_, true>),            \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 64 << 10),              \
                        "hipFuncSetAttribute(unfold_kernel)"));                                                  \
      configured = true;                                                                                         \
    }                                                                                                            \
    unfold_kernel<NQ_, true><<<(uint32_t)blocks, kBlock, bytes, st>>>(p);                                        \
    return after_launch("unfold_kernel");                                                                        \
  }
    WF2_VCASE(1)
    WF2_VCASE(2)
    WF2_VCASE(3)
    WF2_VCASE(4)
#undef WF2_VCASE
  }
  const int64_t per_lane = ceil_div(cc * KK, kWave);
#define WF2_CASE(NQ_)                                                                                            \
  if (per_lane <= NQ_) {                                                                                         \
    static bool configured = false;                                                                              \
    if (!configured) {                                                                                           \
      WF2_TRY(check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&unfold_kernel<NQ_>),                  \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 64 << 10),              \
                        "hipFuncSetAttribute(unfold_kernel)"));                                                  \
      configured = true;                                                                                         \
    }                                                                                                            \
    unfold_kernel<NQ_><<<(uint32_t)blocks, kBlock, bytes, st>>>(p);                                              \
    return after_launch("unfold_kernel");                                                                        \
  }
  WF2_CASE(1)
  WF2_CASE(2)
  WF2_CASE(3)
  WF2_CASE(4)
  WF2_CASE(6)
  WF2_CASE(8)
  WF2_CASE(12)
  WF2_CASE(16)
#undef WF2_CASE
  return fail(WF2HIP_EINVAL, "unfold: bad run length");
}
