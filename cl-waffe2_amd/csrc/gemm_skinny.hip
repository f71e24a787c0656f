// gemm_skinny.hip -- MatMulNode when the left operand of the row-major product has at most 64 rows
// (a few tokens through a Linear layer: x (rows, k) . W, W being (k, cols) or the (cols, k) storage that
// `(!matmul x (!t w))` hands to sgemm_, source/backends/cpu/matrix-ops.lisp:12-112).
//
// Such a product is one read of W.  The tiled kernel of gemm.hip pads the rows to its 128 x 128 tile, so
// its matrix cores and LDS do the work of 128 rows whatever the row count and W streams at 1.4 - 1.7 TB/s
// ((1 ... 64, 8192) . (8192, 8192): 155 - 175 us).  Here a wavefront owns 16 CB columns of the output
// (CB = 4 blocks; eight halve x's share of the requests but cost more in registers than that returns:
// 32 rows of 8192 x 8192 74 -> 97 us, 64 rows 124 -> 164 us) and a slice of K and feeds
// v_mfma_f32_16x16x4 straight from global memory, 16 steps of K at a time:
//   W operand, lane (kk = lane / 16, jj = lane % 16):
//     (cols, k) storage: CB 16-byte loads, W[j0 + 16 b + jj][k0 + 4 kk ... + 3], b = 0 .. CB - 1
//     (k, cols) storage: CB 16-byte loads, W[k0 + 4 kk + s][j0 + 64 h + 4 jj ... + 3], s = 0 .. 3, h < CB / 4
//   x operand: one 16-byte load per 16 rows, x[16 t + jj][k0 + 4 kk ... + 3]
//   the product for step s (k = k0 + 4 kk + s on lane group kk) and column block b adds into the 16 x 16
//   tile D of rows 16 t ... and columns j0 + 16 b + jj, or j0 + 64 (b / 4) + 4 jj + b % 4 (columns
//   interleaved by four, so that a lane's four tiles are four neighbouring columns).
// The four wavefronts of a workgroup take a quarter of the workgroup's slice of K each and meet in LDS;
// with several slices of K over the grid each writes a plane of its own and skinny_finish adds the planes
// in a fixed order.  alpha, beta, bias, activation and residual are applied once, at the end.
#include <algorithm>

#include "wf2_common.h"
#include "wf2_fastdiv.h"
#include "wf2_math.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));

struct SkinnyParams {
  const float* W;
  const float* X;
  float* C;             // row-major rows x cols, pitch ldc
  int64_t ldw, ldx, ldc;
  int32_t rows;
  int64_t cols;
  int32_t k;
  int32_t kslice;       // K per workgroup, a multiple of 64
  uint32_t cgroups;     // groups of 16 CB columns
  uint32_t gsplit;      // slices of K over the grid
  float* partial;       // gsplit planes of rows x cols (packed) when gsplit > 1
  float alpha, beta;
  const float* bias;      // cols floats or null
  const float* residual;  // rows x cols, pitch ldres, or null
  int64_t ldres;
  int32_t activation;     // 0 none, 1 tanh-form GELU
};

__device__ __forceinline__ void skinny_finish_store(const SkinnyParams& p, int row, int64_t col, float acc) {
  float* c = p.C + (int64_t)row * p.ldc + col;
  float v = p.alpha * acc;
  if (p.beta != 0.0f) v += p.beta * *c;
  if (p.bias) v += p.bias[col];
  if (p.activation == 1) v = gelu_tanh_fast(v);
  if (p.residual) v += p.residual[(int64_t)row * p.ldres + col];
  *c = v;
}

// TW: W stored (cols, k), k contiguous; otherwise (k, cols), columns contiguous.  MT tiles of 16 rows,
// CB blocks of 16 columns.
// ALIGNED (the (k, cols) storage only): W's rows are 16-byte aligned and cols is a multiple of 4.  Otherwise
// W is read element by element, lane jj taking columns j0 + 16 b + jj (64-byte runs), and the tiles hold those
// columns.
template <bool TW, int MT, int CB, bool ALIGNED = true>
__global__ __launch_bounds__(kBlock) void sgemm_skinny_kernel(SkinnyParams p) {
  static_assert(ALIGNED || (!TW && CB == 4), "the element-by-element form exists for the (k, cols) storage");
  __shared__ float meet[MT * CB * 4 * kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int kk = lane >> 4, jj = lane & 15;
  const uint32_t ks = blockIdx.x / p.cgroups, cg = blockIdx.x - ks * p.cgroups;
  const int64_t j0 = (int64_t)cg * (16 * CB);
  const int quarter = p.kslice / 4;
  const int kbeg = (int)ks * p.kslice + wave * quarter;
  const int kend = kbeg + quarter < p.k ? kbeg + quarter : p.k;
  const f4 zero = {0.f, 0.f, 0.f, 0.f};
  f4 acc[MT][CB];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int b = 0; b < CB; b++) acc[t][b] = zero;

  // row pointers (columns / rows past the end read a valid address and are not stored)
  const float* wrow[CB];
  if (TW) {
#pragma unroll
    for (int b = 0; b < CB; b++) {
      int64_t j = j0 + 16 * b + jj;
      if (j >= p.cols) j = p.cols - 1;
      wrow[b] = p.W + j * p.ldw + 4 * kk;
    }
  } else if (!ALIGNED) {
#pragma unroll
    for (int b = 0; b < CB; b++) {
      int64_t j = j0 + 16 * b + jj;
      if (j >= p.cols) j = p.cols - 1;
      wrow[b] = p.W + (int64_t)(4 * kk) * p.ldw + j;
    }
  } else {
#pragma unroll
    for (int h = 0; h < CB / 4; h++) {
      int64_t j = j0 + 64 * h + 4 * jj;
      if (j + 3 >= p.cols) j = p.cols - 4;  // cols is a multiple of 4 (host)
#pragma unroll
      for (int s = 0; s < 4; s++) wrow[4 * h + s] = p.W + (int64_t)(4 * kk + s) * p.ldw + j;
    }
  }
  const float* xrow[MT];
  bool xlive[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int i = 16 * t + jj;
    xlive[t] = i < p.rows;
    xrow[t] = p.X + (int64_t)(xlive[t] ? i : 0) * p.ldx + 4 * kk;
  }

  // NB fetches of 16 steps in flight per wavefront; fetches past the end of the slice load nothing and multiply
  // zeros, so the loop runs in whole rounds of NB.  Three from 17 rows on ((32, 8192) . (8192, 8192): 75 -> 69 us;
  // at 64 rows no change).  (Four in flight, or 128 columns per wavefront to halve x's share of the requests, left
  // (16, 8192) . (8192, 8192) on operands in no cache at 59 us.)
  constexpr int NB = MT >= 2 ? 3 : 2;
  f4 wv[NB][CB], xv[NB][MT];
  auto fetch = [&](int k0, int buf) {
    const bool in = k0 + 4 * kk < kend;  // k and the slices are multiples of 4: a vector is wholly in or out
#pragma unroll
    for (int q = 0; q < CB; q++) {
      if (TW) {
        wv[buf][q] = in ? *reinterpret_cast<const f4*>(wrow[q] + k0) : zero;
      } else if (ALIGNED) {
        wv[buf][q] = in ? *reinterpret_cast<const f4*>(wrow[q] + (int64_t)k0 * p.ldw) : zero;
      } else {  // q is the step s; component b is column block b
#pragma unroll
        for (int b = 0; b < 4; b++) wv[buf][q][b] = in ? wrow[b][(int64_t)(k0 + q) * p.ldw] : 0.0f;
      }
    }
#pragma unroll
    for (int t = 0; t < MT; t++) xv[buf][t] = (in && xlive[t]) ? *reinterpret_cast<const f4*>(xrow[t] + k0) : zero;
  };
  // The same for 16 steps wholly inside the wavefront's part of K: no test, so no branch around a load.  With
  // branches the compiler's wait before a buffer's first use cannot count the loads issued after it and
  // waits for all of them -- the fetches meant to stay in flight included.  (Rows of x beyond the matrix read
  // row 0 and feed accumulator rows that are never stored.)
  auto fetch_full = [&](int k0, int buf) {
#pragma unroll
    for (int q = 0; q < CB; q++) {
      if (TW) {
        wv[buf][q] = *reinterpret_cast<const f4*>(wrow[q] + k0);
      } else if (ALIGNED) {
        wv[buf][q] = *reinterpret_cast<const f4*>(wrow[q] + (int64_t)k0 * p.ldw);
      } else {
#pragma unroll
        for (int b = 0; b < 4; b++) wv[buf][q][b] = wrow[b][(int64_t)(k0 + q) * p.ldw];
      }
    }
#pragma unroll
    for (int t = 0; t < MT; t++) xv[buf][t] = *reinterpret_cast<const f4*>(xrow[t] + k0);
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int b = 0; b < CB; b++) {
        // (k, cols) storage: block b = 4 h + c is component c of the load (s, h)
        const float w = TW ? wv[buf][b][s] : wv[buf][4 * (b / 4) + s][b % 4];
#pragma unroll
        for (int t = 0; t < MT; t++)
          acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[buf][t][s], w, acc[t][b], 0, 0, 0);
      }
  };
  if (kbeg < kend) {
#pragma unroll
    for (int b = 0; b < NB - 1; b++) fetch(kbeg + 16 * b, b);
    int k0 = kbeg;
    for (; k0 + 16 * (2 * NB - 1) <= kend; k0 += 16 * NB) {  // every fetch of the round is whole
#pragma unroll
      for (int b = 0; b < NB; b++) {
        fetch_full(k0 + 16 * (b + NB - 1), (b + NB - 1) % NB);
        multiply(b);
      }
    }
    for (; k0 < kend; k0 += 16 * NB) {
#pragma unroll
      for (int b = 0; b < NB; b++) {
        fetch(k0 + 16 * (b + NB - 1), (b + NB - 1) % NB);
        multiply(b);
      }
    }
  }

  // the four quarters of K meet in wavefront 0, in the order 1, 2, 3
  for (int w = 1; w < kBlock / kWave; w++) {
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int b = 0; b < CB; b++)
#pragma unroll
          for (int r = 0; r < 4; r++) meet[((t * CB + b) * 4 + r) * kWave + lane] = acc[t][b][r];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int b = 0; b < CB; b++)
#pragma unroll
          for (int r = 0; r < 4; r++) acc[t][b][r] += meet[((t * CB + b) * 4 + r) * kWave + lane];
    }
    __syncthreads();
  }
  if (wave != 0) return;
  // D[4 (lane / 16) + r][lane % 16] of tile (t, b) in register r
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int row = 16 * t + 4 * kk + r;
      if (row >= p.rows) continue;
#pragma unroll
      for (int b = 0; b < CB; b++) {
        const int64_t col = (TW || !ALIGNED) ? j0 + 16 * b + jj : j0 + 64 * (b / 4) + 4 * jj + b % 4;
        if (col >= p.cols) continue;
        if (p.gsplit == 1)
          skinny_finish_store(p, row, col, acc[t][b][r]);
        else
          p.partial[((int64_t)ks * p.rows + row) * p.cols + col] = acc[t][b][r];
      }
    }
}

// W stored (cols, k) and at most 32 rows: the same product with W fetched as whole lines.  In the kernel above a
// lane's 16-byte load covers a quarter of 64 bytes of its row, so a fetch touches 64 bytes of 64 rows and the
// other half of every 128-byte line is asked for a step later (rocprofv3: 1.39 x the operand fetched, (16, 8192)
// . (8192, 8192)^T 69 us against 51 us for the other storage).  Here eight lanes cover 128 bytes of a row (32
// steps of K), a load instruction eight rows, and the wavefront's 64 x 32 piece goes through a region of LDS of
// its own (row pitch 36 floats) from which every lane reads the 16 bytes the matrix-core layout wants: rows
// 16 b + lane % 16, steps 16 h + 4 (lane / 16) ... + 3.  No barrier: a wavefront's LDS accesses execute in order.
template <int MT>
__global__ __launch_bounds__(kBlock) void sgemm_skinny_lines_kernel(SkinnyParams p) {
  constexpr int kPitch = 36, kPiece = 64 * kPitch;  // floats
  __shared__ __attribute__((aligned(16))) float lds[(kBlock / kWave) * kPiece];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int kk = lane >> 4, jj = lane & 15;
  const int lrow = lane >> 3, lk = (lane & 7) * 4;  // the loading layout: row within eight, step within 32
  const uint32_t ks = blockIdx.x / p.cgroups, cg = blockIdx.x - ks * p.cgroups;
  const int64_t j0 = (int64_t)cg * 64;
  const int quarter = p.kslice / 4;  // a multiple of 32
  const int kbeg = (int)ks * p.kslice + wave * quarter;
  const int kend = kbeg + quarter < p.k ? kbeg + quarter : p.k;
  float* piece = lds + wave * kPiece;
  const f4 zero = {0.f, 0.f, 0.f, 0.f};
  f4 acc[MT][4];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int b = 0; b < 4; b++) acc[t][b] = zero;
  const float* wrow[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    int64_t j = j0 + 8 * q + lrow;
    if (j >= p.cols) j = p.cols - 1;  // read, not stored
    wrow[q] = p.W + j * p.ldw + lk;
  }
  const float* xrow[MT];
  bool xlive[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int i = 16 * t + jj;
    xlive[t] = i < p.rows;
    xrow[t] = p.X + (int64_t)(xlive[t] ? i : 0) * p.ldx + 4 * kk;
  }
  f4 wv[2][8], xv[2][MT][2];
  auto fetch = [&](int k0, int buf) {
    const bool in = k0 + lk < kend;  // k and the slices are multiples of 4: a vector is wholly in or out
#pragma unroll
    for (int q = 0; q < 8; q++) wv[buf][q] = in ? *reinterpret_cast<const f4*>(wrow[q] + k0) : zero;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const bool xin = k0 + 16 * h + 4 * kk < kend;
#pragma unroll
      for (int t = 0; t < MT; t++)
        xv[buf][t][h] = (xin && xlive[t]) ? *reinterpret_cast<const f4*>(xrow[t] + k0 + 16 * h) : zero;
    }
  };
  auto fetch_full = [&](int k0, int buf) {  // 32 steps wholly inside: no branch around a load (see above)
#pragma unroll
    for (int q = 0; q < 8; q++) wv[buf][q] = *reinterpret_cast<const f4*>(wrow[q] + k0);
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int t = 0; t < MT; t++) xv[buf][t][h] = *reinterpret_cast<const f4*>(xrow[t] + k0 + 16 * h);
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 8; q++) *reinterpret_cast<f4*>(piece + (8 * q + lrow) * kPitch + lk) = wv[buf][q];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int h = 0; h < 2; h++) {
      f4 w[4];
#pragma unroll
      for (int b = 0; b < 4; b++) w[b] = *reinterpret_cast<const f4*>(piece + (16 * b + jj) * kPitch + 16 * h + 4 * kk);
#pragma unroll
      for (int s = 0; s < 4; s++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int t = 0; t < MT; t++)
            acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[buf][t][h][s], w[b][s], acc[t][b], 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();
  };
  if (kbeg < kend) {
    int k0 = kbeg;
    fetch(k0, 0);
    // (from 17 rows on: (32, 8192) . (8192, 8192)^T 74.7 -> 71.9 us; with one tile of rows the loads this keeps
    // in flight slow the kernel down, 58.8 -> 65.6 us at 16 rows)
    for (; MT >= 2 && k0 + 96 <= kend; k0 += 64) {  // the next two pieces are whole
      fetch_full(k0 + 32, 1);
      multiply(0);
      fetch_full(k0 + 64, 0);
      multiply(1);
    }
    for (; k0 < kend; k0 += 64) {  // fetches past the end load nothing and multiply zeros
      fetch(k0 + 32, 1);
      multiply(0);
      fetch(k0 + 64, 0);
      multiply(1);
    }
  }
  // the four quarters of K meet in wavefront 0, in the order 1, 2, 3 (through the first piece of LDS)
  float* meet = lds;
  for (int w = 1; w < kBlock / kWave; w++) {
    __syncthreads();
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int r = 0; r < 4; r++) meet[((t * 4 + b) * 4 + r) * kWave + lane] = acc[t][b][r];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int r = 0; r < 4; r++) acc[t][b][r] += meet[((t * 4 + b) * 4 + r) * kWave + lane];
    }
  }
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int row = 16 * t + 4 * kk + r;
      if (row >= p.rows) continue;
#pragma unroll
      for (int b = 0; b < 4; b++) {
        const int64_t col = j0 + 16 * b + jj;
        if (col >= p.cols) continue;
        if (p.gsplit == 1)
          skinny_finish_store(p, row, col, acc[t][b][r]);
        else
          p.partial[((int64_t)ks * p.rows + row) * p.cols + col] = acc[t][b][r];
      }
    }
}

// The same product with a workgroup of ONE wavefront per 16 CB columns (rows of W) and slice of K.  The kernel
// above hands a workgroup 64 columns, so GPT-2's token projection (50257 columns) is 786 workgroups, all
// resident at once, three on most compute units and four on some, with nothing to even them out, and over
// K = 768 each of their wavefronts runs three iterations before the four meet in LDS.  1571 one-wavefront
// workgroups of 32 columns are dealt out as compute units fall free.  Each keeps KSTEPS steps of 32 of K in flight per buffer (8 KB of W with CB = 2, KSTEPS = 2); x
// comes from the L2 cache, once per workgroup (16 columns per wavefront read x as often as W and run 15 %
// slower).  No meeting in LDS: a wavefront covers its slice of K alone.
template <int MT, int CB, int KSTEPS>
__global__ __launch_bounds__(kWave) void sgemm_skinny_wave_kernel(SkinnyParams p) {
  constexpr int kPitch = 36;
  __shared__ __attribute__((aligned(16))) float piece[KSTEPS][16 * CB * kPitch];
  const int lane = threadIdx.x;
  const int kk = lane >> 4, jj = lane & 15;
  const int lrow = lane >> 3, lk = (lane & 7) * 4;  // the loading layout: row within eight, step within 32
  const uint32_t ks = blockIdx.x / p.cgroups, cg = blockIdx.x - ks * p.cgroups;
  const int64_t j0 = (int64_t)cg * 16 * CB;
  const int kbeg = (int)ks * p.kslice;
  const int kend = kbeg + p.kslice < p.k ? kbeg + p.kslice : p.k;
  const f4 zero = {0.f, 0.f, 0.f, 0.f};
  f4 acc[MT][CB];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int b = 0; b < CB; b++) acc[t][b] = zero;
  const float* wrow[2 * CB];
#pragma unroll
  for (int q = 0; q < 2 * CB; q++) {
    int64_t j = j0 + 8 * q + lrow;
    if (j >= p.cols) j = p.cols - 1;  // read, not stored
    wrow[q] = p.W + j * p.ldw + lk;
  }
  const float* xrow[MT];
  bool xlive[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) {
    const int i = 16 * t + jj;
    xlive[t] = i < p.rows;
    xrow[t] = p.X + (int64_t)(xlive[t] ? i : 0) * p.ldx + 4 * kk;
  }
  f4 wv[2][KSTEPS][2 * CB], xv[2][KSTEPS][MT][2];
  auto fetch = [&](int k0, int buf) {
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
      const int kq = k0 + 32 * s;
      const bool in = kq + lk < kend;  // k and the slices are multiples of 4: a vector is wholly in or out
#pragma unroll
      for (int q = 0; q < 2 * CB; q++)
        wv[buf][s][q] = in ? __builtin_nontemporal_load(reinterpret_cast<const f4*>(wrow[q] + kq)) : zero;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const bool xin = kq + 16 * h + 4 * kk < kend;
#pragma unroll
        for (int t = 0; t < MT; t++)
          xv[buf][s][t][h] = (xin && xlive[t]) ? *reinterpret_cast<const f4*>(xrow[t] + kq + 16 * h) : zero;
      }
    }
  };
  // The same for a chunk that lies wholly inside [kbeg, kend): no test and so no branch around a load.  With
  // branches the compiler's wait before a buffer's first use cannot count the loads issued after it and
  // waits for all of them, the other buffer's included, which undoes the double buffering.  (Rows of x beyond
  // the matrix read row 0 and feed accumulator rows that are never stored.)
  auto fetch_full = [&](int k0, int buf) {
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
      const int kq = k0 + 32 * s;
#pragma unroll
      for (int q = 0; q < 2 * CB; q++)
        wv[buf][s][q] = __builtin_nontemporal_load(reinterpret_cast<const f4*>(wrow[q] + kq));
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int t = 0; t < MT; t++) xv[buf][s][t][h] = *reinterpret_cast<const f4*>(xrow[t] + kq + 16 * h);
    }
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int s = 0; s < KSTEPS; s++)
#pragma unroll
      for (int q = 0; q < 2 * CB; q++) *reinterpret_cast<f4*>(&piece[s][(8 * q + lrow) * kPitch + lk]) = wv[buf][s][q];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int s = 0; s < KSTEPS; s++)
#pragma unroll
      for (int h = 0; h < 2; h++) {
        f4 w[CB];
#pragma unroll
        for (int b = 0; b < CB; b++) w[b] = *reinterpret_cast<const f4*>(&piece[s][(16 * b + jj) * kPitch + 16 * h + 4 * kk]);
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
          for (int b = 0; b < CB; b++)
#pragma unroll
            for (int t = 0; t < MT; t++)
              acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[buf][s][t][h][e], w[b][e], acc[t][b], 0, 0, 0);
      }
    __builtin_amdgcn_wave_barrier();
  };
  if (kbeg < kend) {
    int k0 = kbeg;
    fetch(k0, 0);
    for (; k0 + 96 * KSTEPS <= kend; k0 += 64 * KSTEPS) {  // the next two chunks are whole
      fetch_full(k0 + 32 * KSTEPS, 1);
      multiply(0);
      fetch_full(k0 + 64 * KSTEPS, 0);
      multiply(1);
    }
    for (; k0 < kend; k0 += 64 * KSTEPS) {  // fetches past the end load nothing and multiply zeros
      fetch(k0 + 32 * KSTEPS, 1);
      multiply(0);
      fetch(k0 + 64 * KSTEPS, 0);
      multiply(1);
    }
  }
  // D[4 (lane / 16) + r][lane % 16] of tile (t, b) in register r
#pragma unroll
  for (int b = 0; b < CB; b++) {
    const int64_t col = j0 + 16 * b + jj;
    if (col >= p.cols) continue;
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int row = 16 * t + 4 * kk + r;
        if (row >= p.rows) continue;
        if (p.gsplit == 1)
          skinny_finish_store(p, row, col, acc[t][b][r]);
        else
          p.partial[((int64_t)ks * p.rows + row) * p.cols + col] = acc[t][b][r];
      }
  }
}

// the slices' planes added in the order 0, 1, ..., then alpha, beta, bias, activation, residual
__global__ __launch_bounds__(kBlock) void sgemm_skinny_finish(SkinnyParams p) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t plane = (int64_t)p.rows * p.cols;
  if (e >= plane) return;
  float acc = 0.0f;
  for (uint32_t s = 0; s < p.gsplit; s++) acc += p.partial[(int64_t)s * plane + e];
  const int row = (int)(e / p.cols);
  skinny_finish_store(p, row, e - (int64_t)row * p.cols, acc);
}

// many slices (a few outputs over a very long K): a wavefront per output element, lane l adds planes l, l + 64,
// ... in binary64 and the lanes meet by shuffles -- a fixed order
__global__ __launch_bounds__(kBlock) void sgemm_skinny_finish_wide(SkinnyParams p) {
  const int64_t e = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  const int64_t plane = (int64_t)p.rows * p.cols;
  if (e >= plane) return;
  const int lane = threadIdx.x & (kWave - 1);
  double acc = 0.0;
  for (uint32_t s = (uint32_t)lane; s < p.gsplit; s += kWave) acc += (double)p.partial[(int64_t)s * plane + e];
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) {
    const int row = (int)(e / p.cols);
    skinny_finish_store(p, row, e - (int64_t)row * p.cols, (float)acc);
  }
}

static inline bool aligned16(const void* q) { return ((uintptr_t)q & 15u) == 0; }

// Row-major C (rows x cols) = act(alpha x . W + beta C + bias) + residual.  `w_is_cols_by_k`: W stored
// (cols, k) with pitch ldw, else (k, cols).  Returns false (nothing launched) when the shape or the
// alignment is not the kernel's; *rc holds the result of the launches otherwise.
bool try_sgemm_skinny(bool w_is_cols_by_k, long rows, long cols, long k, float alpha, const float* W, long ldw,
                      const float* X, long ldx, float beta, float* C, long ldc, const float* bias,
                      const float* residual, long ldres, int activation, int* rc) {
  // 33 ... 64 rows keep the matrix cores busy about half the time here: ahead of the tiled kernel (with its
  // slices of K) only on a large W ((64, 768) . (768, 50304): 92 against 111 us; (768, 2304): 18.1 against 14.6)
  if (rows > 32 && (int64_t)k * cols < ((int64_t)1 << 25)) return false;
  // a wide operand, or a narrow one over a long K ((1 x 4194304) . (4194304 x 1): the slices of K fill the grid)
  if (rows < 1 || rows > 64 || (cols < 256 && k < 8192) || cols < 1 || k < 64 || k % 4 != 0 || k >= (1L << 30))
    return false;
  if (!aligned16(X) || ldx % 4 != 0) return false;
  const bool w_aligned = aligned16(W) && ldw % 4 == 0 && (w_is_cols_by_k || cols % 4 == 0);
  if (w_is_cols_by_k && !w_aligned) return false;
  SkinnyParams p;
  p.W = W;
  p.X = X;
  p.C = C;
  p.ldw = ldw;
  p.ldx = ldx;
  p.ldc = ldc;
  p.rows = (int32_t)rows;
  p.cols = cols;
  p.k = (int32_t)k;
  const int mt = rows <= 16 ? 1 : (rows <= 32 ? 2 : 4);
  const int cb = 4;
  p.cgroups = (uint32_t)ceil_div((int64_t)cols, (int64_t)(16 * cb));
  // about two workgroups per compute unit (on operands that are not in any cache, (16, 8192) . (8192, 8192):
  // 58.5 us with two, 62.4 with four, 70.1 with sixteen: longer slices, fewer planes), every wavefront at
  // least four steps of 16.  Tried without gain: two neighbouring vectors per lane for the (cols, k) storage,
  // so that the four lanes of a row use up a 128-byte line in one step (76 against 74 us); a group of columns
  // per wavefront with the whole K instead of quarters of K (GPT-2's token projection 48.3 against 49.6 us,
  // everything else slower).
  int64_t gsplit = (int64_t)rt().num_cus * 2 / p.cgroups;
  // W stored along k, at most 32 rows, and enough columns to fill the device without slicing K (from 32768
  // columns on): a wavefront per 32 columns.  GPT-2's token projection, 1 / 16 / 32 rows: 30.6 / 33.8 / 50.9 us
  // against 40.9 / 42.7 / 58.5 us; with slices of K ((8192, 8192)^T) the workgroups of four wavefronts above
  // are level or ahead (32 rows: 75 against 86 us) and keep the work.
  static const bool wave_env = [] {
    const char* e = getenv("WF2HIP_SKINNY_WAVE");
    return !e || atoi(e) != 0;
  }();
  const bool by_wave = w_is_cols_by_k && mt <= 2 && wave_env && cols >= (int64_t)128 * rt().num_cus;
  if (by_wave) {
    p.cgroups = (uint32_t)ceil_div((int64_t)cols, (int64_t)32);
    gsplit = 1;
  }
  if (gsplit > k / 256) gsplit = k / 256;
  if (gsplit < 1) gsplit = 1;
  // (128: a quarter per wavefront then starts on a 128-byte line of W's rows where those are stored along k)
  p.kslice = (int32_t)(ceil_div(ceil_div((int64_t)k, gsplit), (int64_t)128) * 128);
  gsplit = ceil_div((int64_t)k, (int64_t)p.kslice);
  p.gsplit = (uint32_t)gsplit;
  p.partial = nullptr;
  p.alpha = alpha;
  p.beta = beta;
  p.bias = bias;
  p.residual = residual;
  p.ldres = ldres;
  p.activation = activation;
  const int64_t blocks = (int64_t)p.cgroups * gsplit;
  if (blocks >= ((int64_t)1 << 31)) return false;
  void* scratch = nullptr;
  if (gsplit > 1) {
    if (!scratch_block(&scratch, (size_t)(gsplit * rows * cols) * sizeof(float), rc)) return *rc != 0;
    p.partial = static_cast<float*>(scratch);
  }
  hipStream_t st = rt().stream;
#define WF2_SKINNY(TW_)                                                                         \
  do {                                                                                          \
    if (mt == 1) sgemm_skinny_kernel<TW_, 1, 4><<<(uint32_t)blocks, kBlock, 0, st>>>(p);        \
    else if (mt == 2) sgemm_skinny_kernel<TW_, 2, 4><<<(uint32_t)blocks, kBlock, 0, st>>>(p);   \
    else sgemm_skinny_kernel<TW_, 4, 4><<<(uint32_t)blocks, kBlock, 0, st>>>(p);                \
  } while (0)
  if (by_wave && mt == 1)
    sgemm_skinny_wave_kernel<1, 2, 2><<<(uint32_t)blocks, kWave, 0, st>>>(p);
  else if (by_wave)
    sgemm_skinny_wave_kernel<2, 2, 2><<<(uint32_t)blocks, kWave, 0, st>>>(p);
  else if (w_is_cols_by_k && mt == 1)
    sgemm_skinny_lines_kernel<1><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  else if (w_is_cols_by_k && mt == 2)
    sgemm_skinny_lines_kernel<2><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  else if (w_is_cols_by_k)
    WF2_SKINNY(true);
  else if (w_aligned)
    WF2_SKINNY(false);
  else if (mt == 1)
    sgemm_skinny_kernel<false, 1, 4, false><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  else if (mt == 2)
    sgemm_skinny_kernel<false, 2, 4, false><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
  else
    sgemm_skinny_kernel<false, 4, 4, false><<<(uint32_t)blocks, kBlock, 0, st>>>(p);
#undef WF2_SKINNY
  *rc = after_launch("sgemm_skinny_kernel");
  if (*rc == 0 && gsplit > 16) {
    sgemm_skinny_finish_wide<<<(uint32_t)ceil_div((int64_t)rows * cols, (int64_t)(kBlock / kWave)), kBlock, 0, st>>>(p);
    *rc = after_launch("sgemm_skinny_finish_wide");
  } else if (*rc == 0 && gsplit > 1) {
    sgemm_skinny_finish<<<(uint32_t)ceil_div((int64_t)rows * cols, (int64_t)kBlock), kBlock, 0, st>>>(p);
    *rc = after_launch("sgemm_skinny_finish");
  }
  if (scratch) (void)wf2hip_free(scratch);  // stream order keeps it alive for the launches above
  return true;
}

// ---- a small output over a long K, both operands stored K-major -----------------------------------------
// out (rows x cols) = sum over k of L[k][i] R[k][j] with rows x cols <= 512 and thousands of k: the weight
// gradient of a convolution with few channels (dY^T . col: (N h w, O)^T . (N h w, C kh kw); the first layer of
// the MNIST example is 4 x 9 outputs over K = 173056).  The tiled kernel spends a 128 x 128 tile's work per
// slice of K on them (240 us for 5 MFLOP).  Here the grid splits K; a workgroup stages 64 rows of L and of R at
// a time into LDS (both are contiguous runs when the rows are adjacent), thread t owns outputs t and t + 256
// in registers, and every workgroup leaves a plane of partial sums that the split-K fold adds in a
// fixed order.
struct TinyOutParams {
  const float* L;  // (k, rows), pitch ldl
  const float* R;  // (k, cols), pitch ldr
  int64_t ldl, ldr, k, kslice;
  int32_t rows, cols, chunk;  // chunk: rows of K per LDS stage
  float alpha;
  float* partial;  // gridDim.x planes of rows x cols, row-major
};

template <int U>
__global__ __launch_bounds__(kBlock) void sgemm_tiny_out_kernel(TinyOutParams p, FastDiv by_rows, FastDiv by_cols) {
  extern __shared__ float stage[];
  float* ls = stage;                            // chunk x rows
  float* rs = stage + (size_t)p.chunk * p.rows;  // chunk x cols
  const int64_t kbeg = (int64_t)blockIdx.x * p.kslice;
  const int64_t kend = kbeg + p.kslice < p.k ? kbeg + p.kslice : p.k;
  const uint32_t outputs = (uint32_t)p.rows * (uint32_t)p.cols;
  uint32_t li[U], rj[U];
  float acc[U];
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t o = threadIdx.x + u * kBlock;
    uint32_t j;
    const uint32_t i = fd_divmod(o < outputs ? o : 0u, by_cols, &j);
    li[u] = i;
    rj[u] = j;
    acc[u] = 0.0f;
  }
  for (int64_t k0 = kbeg; k0 < kend; k0 += p.chunk) {
    const uint32_t live = (uint32_t)(kend - k0 < p.chunk ? kend - k0 : p.chunk);
    __syncthreads();  // the previous stage has been read
    for (uint32_t e = threadIdx.x; e < live * (uint32_t)p.rows; e += kBlock) {
      uint32_t i;
      const uint32_t kk = fd_divmod(e, by_rows, &i);
      ls[e] = p.L[(k0 + kk) * p.ldl + i];
    }
    for (uint32_t e = threadIdx.x; e < live * (uint32_t)p.cols; e += kBlock) {
      uint32_t j;
      const uint32_t kk = fd_divmod(e, by_cols, &j);
      rs[e] = p.R[(k0 + kk) * p.ldr + j];
    }
    __syncthreads();
    for (uint32_t kk = 0; kk < live; kk++) {
      const float* lrow = ls + kk * p.rows;
      const float* rrow = rs + kk * p.cols;
#pragma unroll
      for (int u = 0; u < U; u++) acc[u] = __builtin_fmaf(lrow[li[u]], rrow[rj[u]], acc[u]);
    }
  }
  float* plane = p.partial + (size_t)blockIdx.x * outputs;
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t o = threadIdx.x + u * kBlock;
    if (o < outputs) plane[o] = p.alpha * acc[u];
  }
}

// Returns false (nothing launched) when the shape is not the kernel's.  On success *planes partial planes
// of rows x cols (row-major, scaled by alpha) lie at *partial (pool memory, to be folded and freed by the
// caller).
bool try_sgemm_tiny_out(long rows, long cols, long k, float alpha, const float* L, long ldl, const float* R, long ldr,
                        float** partial, long* planes, int* rc) {
  // up to two outputs per thread: with more, the two LDS reads per multiply-add cost more than the tiled
  // kernel's padding ((32 x 75) outputs over K = 65536: 257 us here, 160 us tiled)
  if (rows < 1 || cols < 1 || rows * cols > 2 * kBlock || rows + cols > 192 || k < 8192) return false;
  TinyOutParams p;
  p.L = L;
  p.R = R;
  p.ldl = ldl;
  p.ldr = ldr;
  p.k = k;
  p.rows = (int32_t)rows;
  p.cols = (int32_t)cols;
  p.chunk = 64;
  p.alpha = alpha;
  // about four workgroups per compute unit, each at least four stages
  int64_t groups = std::min<int64_t>((int64_t)rt().num_cus * 4, k / (4 * p.chunk));
  if (groups < 1) groups = 1;
  p.kslice = ceil_div(ceil_div((int64_t)k, groups), (int64_t)p.chunk) * p.chunk;
  groups = ceil_div((int64_t)k, p.kslice);
  void* scratch = nullptr;
  if (!scratch_block(&scratch, (size_t)(groups * rows * cols) * sizeof(float), rc)) return *rc != 0;
  p.partial = static_cast<float*>(scratch);
  const size_t lds = (size_t)p.chunk * (rows + cols) * sizeof(float);
  const FastDiv by_rows = make_fastdiv((uint32_t)rows), by_cols = make_fastdiv((uint32_t)cols);
  hipStream_t st = rt().stream;
  const int per_thread = (int)ceil_div((int64_t)rows * cols, (int64_t)kBlock);
  if (per_thread <= 1) sgemm_tiny_out_kernel<1><<<(uint32_t)groups, kBlock, lds, st>>>(p, by_rows, by_cols);
  else sgemm_tiny_out_kernel<2><<<(uint32_t)groups, kBlock, lds, st>>>(p, by_rows, by_cols);
  *rc = after_launch("sgemm_tiny_out_kernel");
  *partial = p.partial;
  *planes = (long)groups;
  return true;
}

// ---- many small matrices -----------------------------------------------------------------------------
// A batch of products whose outputs are a few elements each (65535 x (8 x 8) . (8 x 8): 0.49 ms as one 128 x 128
// tile per matrix; 256 x (1 x 4096) . (4096 x 1): 0.23 ms).  One output element per thread, or per wavefront
// from K = 128 on (lanes along K, meeting by shuffles in binary64); the operands of neighbouring outputs are
// the same few lines.  Column-major terms, as sgemm_: C(i, j) at i + j ldc.
template <class T>
struct SmallBatchParams {
  const T* A;
  const T* B;
  T* C;
  int64_t lda, ldb, ldc, sA, sA2, sB, sB2, sC, sC2;
  int32_t m, n, k, ta, tb;
  uint32_t batch_inner;
  int64_t outputs;  // m n batch batch2
  T alpha, beta;
};

__device__ __forceinline__ float small_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double small_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <class T, bool WAVE>
__global__ __launch_bounds__(kBlock) void sgemm_small_batch_kernel(SmallBatchParams<T> p, FastDiv by_m, FastDiv by_n) {
  const int64_t o = WAVE ? (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave
                         : (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (o >= p.outputs) return;
  uint32_t i, j;
  uint32_t rest = fd_divmod((uint32_t)o, by_m, &i);
  const uint32_t z = fd_divmod(rest, by_n, &j);
  const uint32_t bi = z % p.batch_inner, bo = z / p.batch_inner;
  const T* a = p.A + (int64_t)bi * p.sA + (int64_t)bo * p.sA2 + (p.ta ? (int64_t)i * p.lda : (int64_t)i);
  const T* b = p.B + (int64_t)bi * p.sB + (int64_t)bo * p.sB2 + (p.tb ? (int64_t)j : (int64_t)j * p.ldb);
  const int64_t astep = p.ta ? 1 : p.lda, bstep = p.tb ? p.ldb : 1;
  T* c = p.C + (int64_t)bi * p.sC + (int64_t)bo * p.sC2 + i + (int64_t)j * p.ldc;
  if (WAVE) {
    const int lane = threadIdx.x & (kWave - 1);
    T part = T(0);
    for (int kk = lane; kk < p.k; kk += kWave) part = small_fma(a[kk * astep], b[kk * bstep], part);
    double acc = (double)part;
#pragma unroll
    for (int s = kWave / 2; s > 0; s >>= 1) acc += __shfl_xor(acc, s);
    if (lane == 0) *c = p.beta == T(0) ? p.alpha * (T)acc : p.alpha * (T)acc + p.beta * *c;
  } else {
    T acc = T(0);
    for (int kk = 0; kk < p.k; kk++) acc = small_fma(a[kk * astep], b[kk * bstep], acc);
    *c = p.beta == T(0) ? p.alpha * acc : p.alpha * acc + p.beta * *c;
  }
}

// Returns false (nothing launched) when the batch is not of this kind.
template <class T>
static bool try_small_batch(bool ta, bool tb, long m, long n, long k, T alpha, const T* A, long lda, long sA, long sA2,
                            const T* B, long ldb, long sB, long sB2, T beta, T* C, long ldc, long sC, long sC2,
                            long batch, long batch2, int* rc) {
  const int64_t nb = (int64_t)batch * batch2, outputs = (int64_t)m * n * nb;
  // outputs of at most 16 x 16 (4096 x (32 x 32) . (32 x 32): 39 us tiled, 86 us here), enough of them to fill
  // the chip with threads or, from K = 128 on, with wavefronts; K within a few thousand
  if (nb < 64 || m * n > 256 || k < 1 || k > 8192 || outputs >= ((int64_t)1 << 31) ||
      outputs < (k >= 128 ? 256 : 16384))
    return false;
  SmallBatchParams<T> p;
  p.A = A; p.B = B; p.C = C;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.sA = sA; p.sA2 = sA2; p.sB = sB; p.sB2 = sB2; p.sC = sC; p.sC2 = sC2;
  p.m = (int32_t)m; p.n = (int32_t)n; p.k = (int32_t)k;
  p.ta = ta; p.tb = tb;
  p.batch_inner = (uint32_t)batch;
  p.outputs = outputs;
  p.alpha = alpha; p.beta = beta;
  const FastDiv by_m = make_fastdiv((uint32_t)m), by_n = make_fastdiv((uint32_t)n);
  hipStream_t st = rt().stream;
  if (k >= 128)
    sgemm_small_batch_kernel<T, true><<<(uint32_t)ceil_div(outputs, (int64_t)(kBlock / kWave)), kBlock, 0, st>>>(p, by_m, by_n);
  else
    sgemm_small_batch_kernel<T, false><<<(uint32_t)ceil_div(outputs, (int64_t)kBlock), kBlock, 0, st>>>(p, by_m, by_n);
  *rc = after_launch("sgemm_small_batch_kernel");
  return true;
}

bool try_sgemm_small_batch(bool ta, bool tb, long m, long n, long k, float alpha, const float* A, long lda, long sA,
                           long sA2, const float* B, long ldb, long sB, long sB2, float beta, float* C, long ldc,
                           long sC, long sC2, long batch, long batch2, int* rc) {
  return try_small_batch<float>(ta, tb, m, n, k, alpha, A, lda, sA, sA2, B, ldb, sB, sB2, beta, C, ldc, sC, sC2, batch,
                                batch2, rc);
}

bool try_dgemm_small_batch(bool ta, bool tb, long m, long n, long k, double alpha, const double* A, long lda, long sA,
                           long sA2, const double* B, long ldb, long sB, long sB2, double beta, double* C, long ldc,
                           long sC, long sC2, long batch, long batch2, int* rc) {
  return try_small_batch<double>(ta, tb, m, n, k, alpha, A, lda, sA, sA2, B, ldb, sB, sB2, beta, C, ldc, sC, sC2, batch,
                                 batch2, rc);
}

}  // namespace wf2
