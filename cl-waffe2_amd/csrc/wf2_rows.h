// wf2_rows.h -- what the row kernels share (reduce.hip, backward.hip): wavefront and
// workgroup reductions in a fixed order, and the register tile that holds one row
// per wavefront.
#pragma once

#include "wf2_common.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kWavesPerBlock = kBlock / kWave;

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

__device__ __forceinline__ float wave_sum32(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o));
  return v;
}

// Sum over the workgroup in a fixed order; valid in thread 0.
__device__ __forceinline__ double block_sum(double v, double* lds) {
  v = wave_sum(v);
  const int w = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[w] = v;
  __syncthreads();
  double t = 0.0;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < kWavesPerBlock; i++) t += lds[i];
  }
  return t;
}

// ---- fused row kernels: one wavefront per row, the row held in registers --------
// Lane l of the wave owns NV groups of 4 consecutive columns, group g starting
// at column (g*64 + l)*4 (16-byte coalesced) or, when the row cannot be read
// with 16-byte loads, columns (g*4 + c)*64 + l.
template <int NV, bool VEC, bool NT = false>
struct RowRegs {
  float v[NV][4];

  __device__ __forceinline__ static int64_t col(int g, int c, int lane) {
    return VEC ? ((int64_t)(g * kWave + lane) * 4 + c) : ((int64_t)(g * 4 + c) * kWave + lane);
  }

  __device__ __forceinline__ void load(const float* __restrict__ row, int64_t ncols, int lane,
                                       float fill) {
    if (VEC && ncols == (int64_t)NV * kWave * 4) {
      // the row fills the register tile exactly: unguarded loads, all in flight
#pragma unroll
      for (int g = 0; g < NV; g++) {
        const f4* q = reinterpret_cast<const f4*>(row + col(g, 0, lane));
        f4 t = NT ? __builtin_nontemporal_load(q) : *q;
        v[g][0] = t.x; v[g][1] = t.y; v[g][2] = t.z; v[g][3] = t.w;
      }
      return;
    }
#pragma unroll
    for (int g = 0; g < NV; g++) {
      if (VEC && col(g, 3, lane) < ncols) {
        f4 t = *reinterpret_cast<const f4*>(row + col(g, 0, lane));
        v[g][0] = t.x; v[g][1] = t.y; v[g][2] = t.z; v[g][3] = t.w;
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          int64_t cc = col(g, c, lane);
          v[g][c] = cc < ncols ? row[cc] : fill;
        }
      }
    }
  }

  __device__ __forceinline__ void store(float* __restrict__ row, int64_t ncols, int lane) const {
    if (VEC && ncols == (int64_t)NV * kWave * 4) {
#pragma unroll
      for (int g = 0; g < NV; g++) {
        f4 t = {v[g][0], v[g][1], v[g][2], v[g][3]};
        f4* q = reinterpret_cast<f4*>(row + col(g, 0, lane));
        if (NT)
          __builtin_nontemporal_store(t, q);
        else
          *q = t;
      }
      return;
    }
#pragma unroll
    for (int g = 0; g < NV; g++) {
      if (VEC && col(g, 3, lane) < ncols) {
        f4 t = {v[g][0], v[g][1], v[g][2], v[g][3]};
        *reinterpret_cast<f4*>(row + col(g, 0, lane)) = t;
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          int64_t cc = col(g, c, lane);
          if (cc < ncols) row[cc] = v[g][c];
        }
      }
    }
  }
};

// ---- rows in pieces: a workgroup of 1024 threads holds 16384 columns of a row in registers ----
// For rows too long for one workgroup's registers, and for a few long rows that would
// leave most compute units without a workgroup.  Thread t owns the 16-byte vectors
// (g 1024 + t) 4 of the piece, or, when the row cannot be read with 16-byte loads, the
// columns k 1024 + t.  (A kernel that needs more registers per element runs fewer threads
// on fewer columns: BLOCK, E.)
constexpr int kPieceBlock = 1024;
constexpr int kPieceE = 16;
constexpr int64_t kPieceCols = (int64_t)kPieceBlock * kPieceE;

template <bool VEC, int BLOCK = kPieceBlock, int E = kPieceE>
struct PieceRegs {
  float v[E];

  // column of element k, counted from the start of the piece
  __device__ __forceinline__ static int64_t col(int k) {
    return VEC ? ((int64_t)((k >> 2) * BLOCK + (int)threadIdx.x) * 4 + (k & 3))
               : ((int64_t)k * BLOCK + threadIdx.x);
  }

  // `left`: columns from the start of the piece to the end of the row (a multiple of 4 when VEC)
  __device__ __forceinline__ void load(const float* piece, int64_t left, float fill) {
    if constexpr (VEC) {
#pragma unroll
      for (int g = 0; g < E / 4; g++) {
        f4 t = {fill, fill, fill, fill};
        if (col(g * 4) < left) t = *reinterpret_cast<const f4*>(piece + col(g * 4));
        v[g * 4 + 0] = t.x; v[g * 4 + 1] = t.y; v[g * 4 + 2] = t.z; v[g * 4 + 3] = t.w;
      }
    } else {
#pragma unroll
      for (int k = 0; k < E; k++) v[k] = col(k) < left ? piece[col(k)] : fill;
    }
  }

  __device__ __forceinline__ void store(float* piece, int64_t left) const {
    if constexpr (VEC) {
#pragma unroll
      for (int g = 0; g < E / 4; g++) {
        const f4 t = {v[g * 4 + 0], v[g * 4 + 1], v[g * 4 + 2], v[g * 4 + 3]};
        if (col(g * 4) < left) *reinterpret_cast<f4*>(piece + col(g * 4)) = t;
      }
    } else {
#pragma unroll
      for (int k = 0; k < E; k++)
        if (col(k) < left) piece[col(k)] = v[k];
    }
  }
};

// Sums of v and w over a workgroup of BLOCK threads, in every thread; a fixed order.
// lds: 2 x BLOCK / 64 doubles.
template <int BLOCK = kPieceBlock>
__device__ __forceinline__ double piece_sum2(double v, double w, double* lds, double* out_w) {
  constexpr int kWaves = BLOCK / kWave;
  v = wave_sum(v);
  w = wave_sum(w);
  __syncthreads();  // an earlier exchange has been read
  if ((threadIdx.x & (kWave - 1)) == 0) {
    lds[threadIdx.x / kWave] = v;
    lds[kWaves + threadIdx.x / kWave] = w;
  }
  __syncthreads();
  double tv = 0.0, tw = 0.0;
#pragma unroll
  for (int i = 0; i < kWaves; i++) {
    tv += lds[i];
    tw += lds[kWaves + i];
  }
  *out_w = tw;
  return tv;
}

// Every piece's sum S_p and the squares of its deviations Q_p about a_p = (float)(S_p / n_p):
// the arithmetic of the one-workgroup kernels (a binary64 sum, deviations and squares in
// binary32), per piece.
template <bool VEC>
__global__ __launch_bounds__(kPieceBlock) void layernorm_piece_stats(const float* __restrict__ x, int64_t ncols,
                                                                    uint32_t pieces, double* __restrict__ psum,
                                                                    double* __restrict__ pdev) {
  __shared__ double lds[2 * kPieceBlock / kWave];
  const uint32_t row = blockIdx.x / pieces, piece = blockIdx.x - row * pieces;
  const int64_t left = ncols - (int64_t)piece * kPieceCols;
  const int64_t n = left < kPieceCols ? left : kPieceCols;
  PieceRegs<VEC> r;
  r.load(x + (int64_t)row * ncols + (int64_t)piece * kPieceCols, left, 0.0f);
  double sum = 0.0, unused;
#pragma unroll
  for (int k = 0; k < kPieceE; k++) sum += (double)r.v[k];
  const double total = piece_sum2(sum, 0.0, lds, &unused);
  const float a = (float)(total / (double)n);
  float sq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int k = 0; k < kPieceE; k++) {
    const float d = PieceRegs<VEC>::col(k) < left ? r.v[k] - a : 0.0f;
    sq[k & 3] = __builtin_fmaf(d, d, sq[k & 3]);
  }
  const double dev = piece_sum2(((double)sq[0] + (double)sq[1]) + ((double)sq[2] + (double)sq[3]), 0.0, lds, &unused);
  if (threadIdx.x == 0) {
    psum[blockIdx.x] = total;
    pdev[blockIdx.x] = dev;
  }
}

// Mean and 1 / sqrt(variance + eps) of a row from its pieces, in every thread:
// sum (x - mean)^2 = sum_p [Q_p - n_p (mu_p - a_p)^2 + n_p (mu_p - mean)^2], mu_p = S_p / n_p.
__device__ __forceinline__ void piece_row_stats(const double* __restrict__ psum, const double* __restrict__ pdev,
                                                uint32_t pieces, int64_t ncols, float eps, double* lds,
                                                float* mean_out, float* rstd_out) {
  double s = 0.0, unused;
  for (uint32_t i = threadIdx.x; i < pieces; i += kPieceBlock) s += psum[i];
  const double mean = piece_sum2(s, 0.0, lds, &unused) / (double)ncols;
  double q = 0.0;
  for (uint32_t i = threadIdx.x; i < pieces; i += kPieceBlock) {
    const int64_t left = ncols - (int64_t)i * kPieceCols;
    const double n = (double)(left < kPieceCols ? left : kPieceCols);
    const double mu = psum[i] / n;
    const double a = (double)(float)mu;
    q += pdev[i] + n * ((mu - mean) * (mu - mean) - (mu - a) * (mu - a));
  }
  const double var = piece_sum2(q, 0.0, lds, &unused) / (double)ncols;
  *mean_out = (float)mean;
  *rstd_out = (float)(1.0 / __builtin_sqrt((var > 0.0 ? var : 0.0) + (double)eps));
}

// Register tiles: NV groups of 256 columns per wavefront.  Sizes 3, 5, 6 and 12
// make rows of 768, 1280, 1536 and 3072 columns (transformer widths) fill the tile
// exactly, which selects the unguarded load path; 7 holds rows of 1600.
inline int pick_nv(int64_t ncols) {
  static const int sizes[] = {1, 2, 3, 4, 5, 6, 7, 8, 12, 16};
  for (int nv : sizes)
    if ((int64_t)nv * kWave * 4 >= ncols) return nv;
  return 0;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace wf2
