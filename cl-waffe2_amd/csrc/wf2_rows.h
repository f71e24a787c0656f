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
