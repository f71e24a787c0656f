// gemm.hip -- fp32 gemm on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32).
//
// Replaces the BLAS sgemm_ call behind MatMulNode
// (source/backends/cpu/matrix-ops.lisp:12-237; binding
// source/backends/cpu/blas-functions.lisp:34-38).  The public entry keeps
// sgemm_'s column-major argument meaning so the Lisp side ports unchanged
// (expand-gemm-form-column swaps operands: sgemm_(transB, transA, n, m, k, 1,
// B, ldb, A, lda, 0, C, ldc) for a row-major C = A.B).
//
// Internally everything is row-major.  A column-major C(m x n, ldc) is the
// row-major matrix Cr[n][m]; Cr = op(B)^T . op(A)^T, so the LEFT row-major
// operand comes from B and the RIGHT one from A:
//   transb 'N'  ->  left  stored [rows][k]   (k innermost)
//   transb 'T'  ->  left  stored [k][rows]   (rows innermost)
//   transa 'N'  ->  right stored [k][cols]   (cols innermost)
//   transa 'T'  ->  right stored [cols][k]   (k innermost)
// cl-waffe2's plain row-major matmul lands on (left k-innermost, right
// cols-innermost), where both global reads are contiguous.
//
// Tiling: 128x128 (or 128x64) per workgroup, K-step 32, 4 wavefronts in 2x2,
// each owning 2x2 (or 2x1) MFMA tiles of 32x32 (64 or 32 accumulator registers).
// Operand tiles are staged global -> registers -> LDS with two LDS buffers, so
// one barrier per K-step; a k-innermost tile is kept [128][32+4] and read back
// with one 128-bit LDS load per four MFMA steps (the +4 pad makes eight
// consecutive lanes cover all 32 banks), an x-innermost tile is kept [32][128]
// and read with conflict-free 32-bit loads.  Within a group of 8 k values,
// MFMA step s takes k = s from lanes 0-31 and k = 4+s from lanes 32-63 for
// both operands, which is what makes the 128-bit read usable.
//
// Bound: fp32 MFMA peak (157.3 TFLOP/s on MI355X); 2 m n k flop per product.
#include <stdlib.h>

#include <type_traits>

#include "wf2_common.h"
#include "wf2_dma.h"
#include "wf2_math.h"
#include "wf2_view.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int BK = 32;
constexpr int KPITCH = BK + 4;  // row pitch of a k-innermost LDS tile (36: b128 reads of 8 lanes cover all 32 banks)

struct GemmParams {
  const float* L;  // left operand  (rows = M)
  const float* R;  // right operand (cols = N)
  float* C;
  int64_t M, N, K;
  int64_t ldl, ldr, ldc;
  int64_t sL, sR, sC;     // strides of the inner batch axis
  int64_t sL2, sR2, sC2;  // strides of the outer batch axis
  uint32_t batch_inner;   // blockIdx.y = outer * batch_inner + inner
  float alpha, beta;
  uint32_t tiles_m, tiles_n;
  // fused epilogue (row-major terms): C = act(alpha acc + bias[col]) + residual
  const float* bias;       // N floats or null
  const float* residual;   // laid out like C (own pitch and batch strides) or null
  int64_t ldres, sRes, sRes2;
  int32_t activation;      // 0 none, 1 tanh-form GELU
  // 1: only tiles that touch the lower triangle (col <= row) are computed;
  // 2: the left operand is lower-triangular (L[i][l] = 0 for l > i), so the
  //    K loop of a row tile stops at its last row
  int32_t causal;
  int32_t pair_ok;  // C (and residual) rows allow 8-byte stores at even columns
  // 1: the tile (i, j) is stored at C[j * ldc + i] (bias indexed by i, residual laid out like C): the product
  // was handed over with its operands exchanged; 2: the same, and C / residual allow 16-byte accesses along i
  int32_t transposed;
};

// Loads this thread's share of a ROWS x BK operand tile into registers
// (ROWS/32 float4 per thread).
// KIN: operand stored [x][k] (k innermost) else [k][x].
// FAST: 16-byte loads (pointer, pitch and extents checked on the host).  Rows or
// columns beyond the matrix are clamped to its last ones instead of zeroed:
// they only feed accumulators that are never stored.  KGUARD: the tile may
// reach beyond K, where operands must read as zero; the main loop runs without
// it and has no branches.
template <bool KIN, bool FAST, int ROWS, bool KGUARD>
__device__ __forceinline__ void load_tile(const float* __restrict__ base, int64_t ld, int64_t x0,
                                          int64_t k0, int64_t X, int64_t K, f4 (&reg)[ROWS / 32]) {
  const int t = threadIdx.x;
#pragma unroll
  for (int j = 0; j < ROWS / 32; j++) {
    const int f = t + kBlock * j;  // float4 slot
    int64_t x, k;
    if (KIN) {
      x = x0 + (f >> 3);
      k = k0 + (f & 7) * 4;
    } else {
      k = k0 + f / (ROWS / 4);
      x = x0 + (f % (ROWS / 4)) * 4;
    }
    f4 v = {0.f, 0.f, 0.f, 0.f};
    if (FAST) {
      const int64_t xc = KIN ? (x < X ? x : X - 1) : (x < X ? x : X - 4);
      if (!KGUARD || k < K)
        v = *reinterpret_cast<const f4*>(KIN ? base + xc * ld + k : base + k * ld + xc);
    } else {
      float e[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; c++) {
        int64_t xx = KIN ? x : x + c;
        int64_t kk = KIN ? k + c : k;
        if (xx < X && kk < K) e[c] = KIN ? base[xx * ld + kk] : base[kk * ld + xx];
      }
      v = f4{e[0], e[1], e[2], e[3]};
    }
    reg[j] = v;
  }
}

template <bool KIN, int ROWS>
__device__ __forceinline__ void store_tile(float* __restrict__ lds, const f4 (&reg)[ROWS / 32]) {
  const int t = threadIdx.x;
#pragma unroll
  for (int j = 0; j < ROWS / 32; j++) {
    const int f = t + kBlock * j;
    float* dst = KIN ? lds + (f >> 3) * KPITCH + (f & 7) * 4
                     : lds + (f / (ROWS / 4)) * ROWS + (f % (ROWS / 4)) * 4;
    *reinterpret_cast<f4*>(dst) = reg[j];
  }
}

// Fragment for MFMA steps s = 0..3 of k-group `kb` (0, 8, 16 or 24): frag[s] is the
// operand value for row/col (x0 + lane%32) at k = kb + 4*(lane/32) + s.
template <bool KIN, int ROWS>
__device__ __forceinline__ void read_frag(const float* __restrict__ lds, int x0, int kb, int lane,
                                          float (&frag)[4]) {
  const int xi = x0 + (lane & 31);
  const int half = lane >> 5;
  if (KIN) {
    f4 v = *reinterpret_cast<const f4*>(lds + xi * KPITCH + kb + half * 4);
    frag[0] = v.x; frag[1] = v.y; frag[2] = v.z; frag[3] = v.w;
  } else {
#pragma unroll
    for (int s = 0; s < 4; s++) frag[s] = lds[(kb + half * 4 + s) * ROWS + xi];
  }
}

// Which output tile and which matrix of the batch a workgroup owns.
// Tile order: consecutive workgroups land on different XCDs (round robin),
// so each XCD gets a contiguous band of tiles, walked column-major in groups
// of 8 row-tiles so that neighbours share operand panels in that XCD's L2.
// Triangular problems have cheap and expensive tiles, and workgroups start in
// dispatch order (x fastest): there the linear workgroup number is re-read as
// (tile rank, matrix) with the matrix index fastest and the most expensive tile
// rank first, so every CU works through expensive tiles early and fills up
// with cheap ones (longest-processing-time-first).
__device__ __forceinline__ void map_tile(const GemmParams& p, bool triangular, uint32_t* tm,
                                         uint32_t* tn, uint32_t* batch_index) {
  const uint32_t ntiles = p.tiles_m * p.tiles_n;
  uint32_t pid = blockIdx.x;
  *batch_index = blockIdx.y;
  if (triangular) {
    const uint32_t linear = blockIdx.y * ntiles + blockIdx.x;
    *batch_index = linear % gridDim.y;
    pid = ntiles - 1 - linear / gridDim.y;  // large tile rows (long K loops) first
  } else {
    const uint32_t xcds = 8;
    const uint32_t per = ntiles / xcds;
    if (per > 0 && pid < per * xcds) pid = (pid % xcds) * per + pid / xcds;
  }
  const uint32_t group = 8;
  const uint32_t width = group * p.tiles_n;
  const uint32_t gid = pid / width;
  const uint32_t first_m = gid * group;
  const uint32_t gsize = (p.tiles_m - first_m) < group ? (p.tiles_m - first_m) : group;
  *tm = first_m + (pid % width) % gsize;
  *tn = (pid % width) / gsize;
}

// One output element: C = act(alpha acc + beta C + bias) + residual; the caller
// fetches bias and residual (once per column, and in batches) so that the
// loads are not strung out one dependent access per element.
// FUSED: 0 plain, 1 bias / residual / triangular skipping, 2 the same plus an
// activation.  The activation's binary64 body is long; keeping it out of the
// instantiations that never apply it shortens their epilogues by ~12 us at
// 8192 x 2304 x 768 (48 inlined copies that every element had to branch around).
template <int FUSED>
__device__ __forceinline__ float finish_value(const GemmParams& p, float accv, float cold,
                                              float biasv, float resv) {
  float v = p.alpha * accv;
  if (p.beta != 0.0f) v += p.beta * cold;
  if constexpr (FUSED) {
    if (p.bias) v += biasv;
    if (FUSED == 2 && p.activation == 1) v = gelu_tanh_fast(v);
    if (p.residual) v += resv;
  }
  return v;
}

// TM x TN MFMA tiles (32x32) per wavefront, wavefronts 2 x 2: the workgroup
// tile is (64 TM) x (64 TN).  2x2 -> 128x128 (64 accumulator registers), 2x1
// -> 128x64 for narrow outputs and for shapes whose 128x128 tiling would leave
// a partial last round of workgroups.
template <bool LKIN, bool RKIN, bool FAST, int TM, int TN, int FUSED>
__global__ __launch_bounds__(kBlock) void sgemm_kernel(GemmParams p) {
  constexpr int BMt = 64 * TM, BNt = 64 * TN;
  constexpr int LFLOATS = LKIN ? BMt * KPITCH : BK * BMt;
  constexpr int RFLOATS = RKIN ? BNt * KPITCH : BK * BNt;
  // two stages of both operand tiles: up to 73.7 KB, beyond the static limit
  extern __shared__ __attribute__((aligned(16))) float smem[];
  auto ldsL = [&](int stage) { return smem + stage * LFLOATS; };
  auto ldsR = [&](int stage) { return smem + 2 * LFLOATS + stage * RFLOATS; };

  uint32_t tm, tn, batch_index;
  map_tile(p, FUSED && p.causal, &tm, &tn, &batch_index);

  const int64_t m0 = (int64_t)tm * BMt;
  const int64_t n0 = (int64_t)tn * BNt;
  if (FUSED && p.causal == 1 && n0 > m0 + BMt - 1) return;  // tile wholly above the diagonal
  const uint32_t zo = batch_index / p.batch_inner;
  const uint32_t zi = batch_index - zo * p.batch_inner;
  const float* L = p.L + (int64_t)zo * p.sL2 + (int64_t)zi * p.sL;
  const float* R = p.R + (int64_t)zo * p.sR2 + (int64_t)zi * p.sR;
  float* C = p.C + (int64_t)zo * p.sC2 + (int64_t)zi * p.sC;

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int wm = (wave >> 1) * 32 * TM;
  const int wn = (wave & 1) * 32 * TN;

  f16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  f4 regL[BMt / 32], regR[BNt / 32];
  int64_t klimit = p.K;
  if (FUSED && p.causal == 2 && m0 + BMt < klimit) klimit = m0 + BMt;
  const int64_t ksteps = (klimit + BK - 1) / BK;
  load_tile<LKIN, FAST, BMt, true>(L, p.ldl, m0, 0, p.M, p.K, regL);
  load_tile<RKIN, FAST, BNt, true>(R, p.ldr, n0, 0, p.N, p.K, regR);
  store_tile<LKIN, BMt>(ldsL(0), regL);
  store_tile<RKIN, BNt>(ldsR(0), regR);
  __syncthreads();

  for (int64_t ks = 0; ks < ksteps; ks++) {
    const int cur = (int)(ks & 1);
    const bool more = ks + 1 < ksteps;
    if (more) {
      if ((ks + 2) * BK <= p.K) {
        load_tile<LKIN, FAST, BMt, false>(L, p.ldl, m0, (ks + 1) * BK, p.M, p.K, regL);
        load_tile<RKIN, FAST, BNt, false>(R, p.ldr, n0, (ks + 1) * BK, p.N, p.K, regR);
      } else {
        load_tile<LKIN, FAST, BMt, true>(L, p.ldl, m0, (ks + 1) * BK, p.M, p.K, regL);
        load_tile<RKIN, FAST, BNt, true>(R, p.ldr, n0, (ks + 1) * BK, p.N, p.K, regR);
      }
    }
    // fragments of k-group g+1 are fetched from LDS while the matrix cores work
    // on group g
    float a[2][TM][4], b[2][TN][4];
#pragma unroll
    for (int i = 0; i < TM; i++) read_frag<LKIN, BMt>(ldsL(cur), wm + i * 32, 0, lane, a[0][i]);
#pragma unroll
    for (int j = 0; j < TN; j++) read_frag<RKIN, BNt>(ldsR(cur), wn + j * 32, 0, lane, b[0][j]);
#pragma unroll
    for (int g = 0; g < BK / 8; g++) {
      if (g + 1 < BK / 8) {
#pragma unroll
        for (int i = 0; i < TM; i++)
          read_frag<LKIN, BMt>(ldsL(cur), wm + i * 32, 8 * (g + 1), lane, a[(g + 1) & 1][i]);
#pragma unroll
        for (int j = 0; j < TN; j++)
          read_frag<RKIN, BNt>(ldsR(cur), wn + j * 32, 8 * (g + 1), lane, b[(g + 1) & 1][j]);
      }
#pragma unroll
      for (int s = 0; s < 4; s++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[g & 1][i][s], b[g & 1][j][s],
                                                             acc[i][j], 0, 0, 0);
    }
    if (more) {
      // The other buffer was last read in iteration ks-1, and every wave has
      // passed the barrier that ended it.
      store_tile<LKIN, BMt>(ldsL(cur ^ 1), regL);
      store_tile<RKIN, BNt>(ldsR(cur ^ 1), regR);
    }
    __syncthreads();
  }

  // D layout of v_mfma_f32_32x32x2_f32: register r of lane l holds
  // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32x32 tile.
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int64_t col = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int64_t row = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < p.M && col < p.N) {
          float* c = C + row * p.ldc + col;
          float v = p.alpha * acc[i][j][r];
          if (p.beta != 0.0f) v += p.beta * *c;
          if constexpr (FUSED) {
            if (p.bias) v += p.bias[col];
            if (FUSED == 2 && p.activation == 1) v = gelu_tanh_fast(v);
            if (p.residual)
              v += p.residual[(int64_t)zo * p.sRes2 + (int64_t)zi * p.sRes + row * p.ldres + col];
          }
          *c = v;
        }
      }
    }
}

// ---- streaming variant: global -> LDS without passing through registers ------------
// For the common case (left operand k-innermost, 16-byte aligned operands, K a
// multiple of 32) the operand tiles are fetched with global_load_lds_dwordx4:
// each wavefront instruction moves 64 x 16 bytes straight into 1 KB of LDS, so the
// K loop holds no staging registers, no ds_write and no address branches.
// Measured on 4096^3 (cycles the CUs are busy / cycles the matrix cores need):
// 82 % with register staging, 91 % with this kernel.  What made the difference,
// in order: (1) LDS writes issued by the wavefronts themselves cost ~12 cycles of
// CU time each, the DMA path ~8 per KB less; (2) the compiler folds a software
// prefetch of the fragments back into load-wait-use unless the order is pinned
// with sched_group_barrier, which leaves the LDS latency of every k-group exposed;
// (3) the barrier sits before the last k-group, so the first fragments of the next
// K-step are fetched under that group's MFMAs.
//
// LDS layouts (64 banks of 4 bytes: a 128-bit read is conflict-free when 16
// consecutive lanes cover 256 distinct bytes modulo 256):
//   k-innermost tile  [rows][32], no padding; the eight 16-byte slots of a row are
//                     permuted: slot = chunk ^ ((row / 2) % 8).  The DMA writes
//                     lane l of an instruction to byte 16 l, so the permutation is
//                     applied to the global address each lane reads.
//   x-innermost tile  [32][128]: MFMA tile j of a wavefront takes columns
//                     2 c + j (c = lane % 32), so one 64-bit read serves both
//                     tiles and the output is stored as 8-byte pairs.
//                     [32][64] (narrow tile): groups of four k-rows are kept 1152
//                     bytes apart so the two half-waves hit different banks.
//                     [32][192] (128 x 192 tile): columns 0-63 of a wavefront's 96
//                     are shared by tiles 0 and 1 as above, 64-95 belong to tile 2.
//   tall layout       the four wavefronts are stacked along M (32 rows x 32 TN columns
//                     each, TN = 3: a 128 x 96 tile, which divides N = 768 and 2304
//                     into whole tiles and 8192 x 768 outputs into exactly two tiles
//                     per CU).  x-innermost right tile: [3 column blocks][32 k][32];
//                     every DMA instruction fills eight k-rows of a block, stored in
//                     the order 0 4 1 5 2 6 3 7, so that the value lane l needs for
//                     k = 8 g + 4 (l / 32) + s sits at float 64 s + l of the
//                     instruction's 1 KB: plain conflict-free 32-bit reads.
template <bool RKIN, int TN, bool TALL = false>
struct DmaLayout {
  static constexpr int BNt = TALL ? 32 * TN : 64 * TN;
  static constexpr int LFLOATS = 128 * BK;
  // instructions per workgroup and K-step for the right operand, rows each covers
  static constexpr int R_INSTRS = BNt * BK / 256;  // 64 pieces of 16 bytes each
  static constexpr int R_INSTR_PITCH = (!RKIN && TN == 1 && !TALL) ? 288 : 256;  // floats
  static constexpr int RFLOATS = R_INSTRS * R_INSTR_PITCH;
  static constexpr int STAGE = LFLOATS + RFLOATS;
  static constexpr size_t LDS_BYTES = 2 * (size_t)STAGE * sizeof(float);
};

template <bool RKIN, int TN, int FUSED, bool TALL = false>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void sgemm_dma_kernel(
    GemmParams p) {  // two workgroups per CU: at most 256 registers per lane
  using Lay = DmaLayout<RKIN, TN, TALL>;
  constexpr int MI = TALL ? 1 : 2;  // 32-row MFMA tiles per wavefront along M
  constexpr int BMt = 128, BNt = Lay::BNt;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  auto ldsL = [&](int stage) { return smem + stage * Lay::STAGE; };
  auto ldsR = [&](int stage) { return smem + stage * Lay::STAGE + Lay::LFLOATS; };

  uint32_t tm, tn, batch_index;
  map_tile(p, FUSED && p.causal, &tm, &tn, &batch_index);
  const int64_t m0 = (int64_t)tm * BMt;
  const int64_t n0 = (int64_t)tn * BNt;
  if (FUSED && p.causal == 1 && n0 > m0 + BMt - 1) return;  // tile wholly above the diagonal
  const uint32_t zo = batch_index / p.batch_inner;
  const uint32_t zi = batch_index - zo * p.batch_inner;
  const float* L = p.L + (int64_t)zo * p.sL2 + (int64_t)zi * p.sL;
  const float* R = p.R + (int64_t)zo * p.sR2 + (int64_t)zi * p.sR;
  float* C = p.C + (int64_t)zo * p.sC2 + (int64_t)zi * p.sC;

  const int lane = threadIdx.x & (kWave - 1);
  // uniform per wavefront: keeps the LDS destinations of the DMA instructions on the scalar unit
  // (worth 1.5-2 % on every shape)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;
  const int wm = TALL ? wave * 32 : (wave >> 1) * 64;
  const int wn = TALL ? 0 : (wave & 1) * 32 * TN;

  // Global source of every 16-byte piece this lane moves per K-step: a base per operand that is the same
  // for the whole workgroup and moves along K on the scalar unit, plus a byte offset per lane and
  // instruction that never changes (32 bits: the host checks that a tile's rows span less than 4 GB).
  // With the address in this form -- scalar base, 32-bit lane offset -- a load costs the matrix cores about
  // 5 cycles of issue; with a 64-bit address per lane it costs 26, and the 64-bit add that forms it 10 more
  // (measured between back-to-back MFMAs: seven or eight loads per K-step were 8 % of the loop).
  // Rows / columns beyond the matrix are clamped to its last ones: they only feed accumulators that are
  // never stored.
  constexpr int LI = 4;                   // left-operand instructions per wavefront
  constexpr int RI = Lay::R_INSTRS / 4;   // right-operand instructions per wavefront
  uint32_t offL[LI], offR[RI];
#pragma unroll
  for (int j = 0; j < LI; j++) {
    const int row = (wave * LI + j) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int64_t gr = m0 + row;
    gr = gr < p.M ? gr : p.M - 1;
    offL[j] = (uint32_t)(((gr - m0) * p.ldl + chunk * 4) * (int64_t)sizeof(float));
  }
#pragma unroll
  for (int j = 0; j < RI; j++) {
    const int q = wave * RI + j;
    if (RKIN) {
      const int row = q * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      int64_t gn = n0 + row;
      gn = gn < p.N ? gn : p.N - 1;
      offR[j] = (uint32_t)(((gn - n0) * p.ldr + chunk * 4) * (int64_t)sizeof(float));
    } else if (TALL) {
      // instruction q: column block q / 4, k-rows 8 (q % 4) + {0 4 1 5 2 6 3 7}[lane / 8]
      const int slot = lane >> 3;
      const int krow = 8 * (q & 3) + (slot >> 1) + 4 * (slot & 1);
      int64_t gn = n0 + 32 * (q >> 2) + 4 * (lane & 7);
      gn = gn < p.N ? gn : p.N - 4;
      offR[j] = (uint32_t)(((int64_t)krow * p.ldr + (gn - n0)) * (int64_t)sizeof(float));
    } else {
      constexpr int CPR = BNt / 4;  // 16-byte pieces per k-row; LDS keeps [k][BNt] densely
      const int piece = q * 64 + lane;
      const int krow = piece / CPR;
      int64_t gn = n0 + (piece % CPR) * 4;
      gn = gn < p.N ? gn : p.N - 4;
      offR[j] = (uint32_t)(((int64_t)krow * p.ldr + (gn - n0)) * (int64_t)sizeof(float));
    }
  }
  const float* nextL = L + m0 * p.ldl;                          // K-step the next fetch reads
  const float* nextR = RKIN ? R + n0 * p.ldr : R + n0;
  const int64_t stepR = RKIN ? (int64_t)BK : (int64_t)BK * p.ldr;
  const uint32_t lds0 = lds_address(smem);
  auto fetch = [&](int stage) {
#pragma unroll
    for (int j = 0; j < LI; j++)
      dma16(lds0 + (uint32_t)((stage * Lay::STAGE + (wave * LI + j) * 256) * sizeof(float)), offL[j], nextL);
#pragma unroll
    for (int j = 0; j < RI; j++)
      dma16(lds0 + (uint32_t)((stage * Lay::STAGE + Lay::LFLOATS + (wave * RI + j) * Lay::R_INSTR_PITCH) * sizeof(float)),
            offR[j], nextR);
    nextL += BK;
    nextR += stepR;
  };

  f16v acc[MI][TN];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  int lrow[MI], lswz[MI], rrow[TN], rswz[TN];
#pragma unroll
  for (int i = 0; i < MI; i++) {
    lrow[i] = wm + i * 32 + col;
    lswz[i] = (lrow[i] >> 1) & 7;
  }
#pragma unroll
  for (int j = 0; j < TN; j++) {
    rrow[j] = wn + j * 32 + col;
    rswz[j] = (rrow[j] >> 1) & 7;
  }

  // fragments of k-group g (k = 8 g + 4 half + s, s = 0..3) into buffer `buf`
  float a[2][MI][4], b[2][TN][4];
  auto read_frags = [&](int stage, int g, int buf) {
    const float* sl = ldsL(stage);
    const float* sr = ldsR(stage);
#pragma unroll
    for (int i = 0; i < MI; i++) {
      const f4 v = *reinterpret_cast<const f4*>(sl + lrow[i] * BK + ((2 * g + half) ^ lswz[i]) * 4);
      a[buf][i][0] = v.x; a[buf][i][1] = v.y; a[buf][i][2] = v.z; a[buf][i][3] = v.w;
    }
    if constexpr (RKIN) {
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const f4 v = *reinterpret_cast<const f4*>(sr + rrow[j] * BK + ((2 * g + half) ^ rswz[j]) * 4);
        b[buf][j][0] = v.x; b[buf][j][1] = v.y; b[buf][j][2] = v.z; b[buf][j][3] = v.w;
      }
    } else if constexpr (TALL) {
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++) b[buf][j][s4] = sr[(4 * j + g) * 256 + 64 * s4 + lane];
    } else if constexpr (TN >= 2) {
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++) {
        const float* krow = sr + (8 * g + 4 * half + s4) * BNt + wn;
        const f2 v = *reinterpret_cast<const f2*>(krow + 2 * col);
        b[buf][0][s4] = v.x;
        b[buf][1][s4] = v.y;
        if (TN == 3) b[buf][TN - 1][s4] = krow[64 + col];
      }
    } else {
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++) {
        const int k = 8 * g + 4 * half + s4;
        b[buf][0][s4] = sr[(k >> 2) * Lay::R_INSTR_PITCH + (k & 3) * 64 + wn + col];
      }
    }
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
      for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[buf][i][s4], b[buf][j][s4], acc[i][j], 0, 0, 0);
  };
  // keeps the LDS reads of the next k-group among the first MFMAs of this one
  auto pin_order = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
    if (TALL) {
      // 4 TN MFMAs; LDS reads of the next group: one 128-bit read for the left
      // fragment, and for the right one TN 128-bit reads (k-innermost) or 2 TN
      // ds_read2st64_b32 (the compiler pairs the 4 TN 32-bit reads).  All of them
      // go among the first MFMAs, the rest of the group runs without.
      // A read right before the group's first MFMA would sit in front of the wait
      // for the fragments that MFMA needs, so an MFMA leads.
      constexpr int NR = 1 + (RKIN ? TN : 2 * TN);
#pragma unroll
      for (int q = 0; q < NR; q++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * TN - NR, 0);
    } else {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        __builtin_amdgcn_sched_group_barrier(0x008, TN, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // LDS read
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * TN, 0);
    }
#endif
  };

  int64_t klimit = p.K;
  if (FUSED && p.causal == 2 && m0 + BMt < klimit) klimit = m0 + BMt;
  const int ksteps = (int)(klimit / BK);  // K and the tile height are multiples of BK

  // One K-step on the stage `cur` (a constant after inlining: the loop below is unrolled by two, so every LDS
  // address is a register fixed for the kernel plus an immediate and the loop holds no vector-ALU
  // instruction at all -- each one costs the matrix cores 5 - 12 cycles of issue).
  auto k_step = [&](auto cur_c, bool more) {
    constexpr int cur = decltype(cur_c)::value;
    // the other stage was last read before the barrier of the previous step
    if (more) fetch(cur ^ 1);
    read_frags(cur, 1, 1); multiply(0); pin_order();
    read_frags(cur, 2, 0); multiply(1); pin_order();
    read_frags(cur, 3, 1); multiply(0); pin_order();
    // every fragment of this stage is in registers and this wavefront's part of
    // the next stage has landed
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (more) read_frags(cur ^ 1, 0, 0);
    multiply(1); pin_order();
  };
  fetch(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  read_frags(0, 0, 0);
  int ks = 0;
  for (; ks + 2 <= ksteps; ks += 2) {
    k_step(std::integral_constant<int, 0>{}, true);
    k_step(std::integral_constant<int, 1>{}, ks + 2 < ksteps);
  }
  if (ks < ksteps) k_step(std::integral_constant<int, 0>{}, false);

  // D layout of v_mfma_f32_32x32x2_f32: register r of lane l holds
  // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32x32 tile.
  const int64_t res_base = (int64_t)zo * p.sRes2 + (int64_t)zi * p.sRes;
  if constexpr (RKIN && TN == 1 && !TALL) {
    if (p.transposed) {
      // The output of a product with few rows, computed with the operands exchanged so that the long
      // operand is the one with 128 rows per tile (gemm.hip, sgemm_batched2): the 128 x 64 tile is turned
      // over in LDS (the stages are free once every wavefront has passed the last barrier of the K loop:
      // none reads LDS after it) and leaves in runs along its 128 rows, which are contiguous in C.
      constexpr int TP = BMt + 1;  // pitch of a tile column: lanes hold 32 consecutive columns
      float* turn = smem;
#pragma unroll
      for (int i = 0; i < MI; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          turn[(wn + col) * TP + wm + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3)] = acc[i][0][r];
      __syncthreads();
      const float* res = (FUSED && p.residual) ? p.residual + res_base : nullptr;
      // thread t: rows 4 (t % 32) ... + 3 of columns t / 32, t / 32 + 8, ...
      const int r4 = 4 * (threadIdx.x & 31);
      const int64_t gi = m0 + r4;
      float bias4[4] = {0.f, 0.f, 0.f, 0.f};
      if (FUSED && p.bias) {
#pragma unroll
        for (int c = 0; c < 4; c++) bias4[c] = gi + c < p.M ? p.bias[gi + c] : 0.f;
      }
      for (int cj = threadIdx.x >> 5; cj < BNt; cj += kBlock / 32) {
        const int64_t gj = n0 + cj;
        if (gj >= p.N || gi >= p.M) continue;
        float* c_out = C + gj * p.ldc + gi;
        const float* r_in = res ? res + gj * p.ldres + gi : nullptr;
        float v[4];
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = turn[cj * TP + r4 + c];
        if (p.transposed == 2 && gi + 3 < p.M) {
          f4 old = {0.f, 0.f, 0.f, 0.f}, rs = {0.f, 0.f, 0.f, 0.f};
          if (p.beta != 0.0f) old = *reinterpret_cast<const f4*>(c_out);
          if (r_in) rs = *reinterpret_cast<const f4*>(r_in);
          f4 o;
#pragma unroll
          for (int c = 0; c < 4; c++) o[c] = finish_value<FUSED>(p, v[c], old[c], bias4[c], rs[c]);
          *reinterpret_cast<f4*>(c_out) = o;
        } else {
#pragma unroll
          for (int c = 0; c < 4; c++)
            if (gi + c < p.M)
              c_out[c] = finish_value<FUSED>(p, v[c], p.beta != 0.0f ? c_out[c] : 0.f, bias4[c], r_in ? r_in[c] : 0.f);
        }
      }
      return;
    }
  }
  const bool pairs = !TALL && !RKIN && TN >= 2 && p.pair_ok;
  const float* res = (FUSED && p.residual) ? p.residual + res_base : nullptr;
  if constexpr (!TALL) {
    // The same for the 2 x 2 wavefront layouts: tiles wholly inside the output
    // take an epilogue without guards, with one 64-bit multiply per lane and, per
    // 32-row block, every load ahead of the first store.
    if (p.beta == 0.0f && m0 + BMt <= p.M && n0 + BNt <= p.N) {
      constexpr bool INTER = !RKIN && TN >= 2;  // tiles 0 and 1 own columns 2 c, 2 c + 1
      const int64_t row0 = m0 + wm + 4 * half;
      if (INTER && p.pair_ok) {
        float* cl = C + row0 * p.ldc + n0 + wn + 2 * col;
        const float* rl = res ? res + row0 * p.ldres + n0 + wn + 2 * col : nullptr;
        float bias0 = 0.f, bias1 = 0.f, bias2 = 0.f;
        if (FUSED && p.bias) {
          bias0 = p.bias[n0 + wn + 2 * col];
          bias1 = p.bias[n0 + wn + 2 * col + 1];
          if (TN == 3) bias2 = p.bias[n0 + wn + 64 + col];
        }
#pragma unroll
        for (int i = 0; i < MI; i++) {
          f2 rs[16];
          float rs2[16];
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int64_t ro = (int64_t)(32 * i + 8 * (r >> 2) + (r & 3));
            rs[r] = rl ? *reinterpret_cast<const f2*>(rl + ro * p.ldres) : f2{0.f, 0.f};
            if (TN == 3) rs2[r] = rl ? rl[ro * p.ldres + 64 - col] : 0.f;
          }
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int64_t ro = (int64_t)(32 * i + 8 * (r >> 2) + (r & 3));
            f2 v;
            v.x = finish_value<FUSED>(p, acc[i][0][r], 0.f, bias0, rs[r].x);
            v.y = finish_value<FUSED>(p, acc[i][TN >= 2 ? 1 : 0][r], 0.f, bias1, rs[r].y);
            *reinterpret_cast<f2*>(cl + ro * p.ldc) = v;
            if (TN == 3)
              cl[ro * p.ldc + 64 - col] = finish_value<FUSED>(p, acc[i][TN - 1][r], 0.f, bias2, rs2[r]);
          }
#if defined(__HIP_DEVICE_COMPILE__)
          __builtin_amdgcn_sched_barrier(0);
#endif
        }
        return;
      }
      if (!INTER) {
        float* cl = C + row0 * p.ldc + n0 + wn + col;
        const float* rl = res ? res + row0 * p.ldres + n0 + wn + col : nullptr;
        float biasv[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) biasv[j] = (FUSED && p.bias) ? p.bias[n0 + wn + j * 32 + col] : 0.f;
#pragma unroll
        for (int i = 0; i < MI; i++) {
          float rs[TN][16];
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
              rs[j][r] = rl ? rl[(int64_t)(32 * i + 8 * (r >> 2) + (r & 3)) * p.ldres + 32 * j] : 0.f;
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
              cl[(int64_t)(32 * i + 8 * (r >> 2) + (r & 3)) * p.ldc + 32 * j] =
                  finish_value<FUSED>(p, acc[i][j][r], 0.f, biasv[j], rs[j][r]);
#if defined(__HIP_DEVICE_COMPILE__)
          __builtin_amdgcn_sched_barrier(0);
#endif
        }
        return;
      }
    }
  }
  if (pairs) {
    const int64_t c0 = n0 + wn + 2 * col;  // even; N is a multiple of 4 here
    if (c0 < p.N) {
      float bias0 = 0.f, bias1 = 0.f;
      if (FUSED && p.bias) {
        bias0 = p.bias[c0];
        bias1 = p.bias[c0 + 1];
      }
#pragma unroll
      for (int i = 0; i < MI; i++)
#pragma unroll
        for (int h = 0; h < 2; h++) {  // eight rows at a time: loads first, then arithmetic and stores
          f2 old[8], rs[8];
#pragma unroll
          for (int q = 0; q < 8; q++) {
            const int r = 8 * h + q;
            const int64_t row = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
            old[q] = f2{0.f, 0.f};
            rs[q] = f2{0.f, 0.f};
            if (row < p.M) {
              if (p.beta != 0.0f) old[q] = *reinterpret_cast<const f2*>(C + row * p.ldc + c0);
              if (res) rs[q] = *reinterpret_cast<const f2*>(res + row * p.ldres + c0);
            }
          }
#pragma unroll
          for (int q = 0; q < 8; q++) {
            const int r = 8 * h + q;
            const int64_t row = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
            if (row < p.M) {
              f2 v;
              v.x = finish_value<FUSED>(p, acc[i][0][r], old[q].x, bias0, rs[q].x);
              v.y = finish_value<FUSED>(p, acc[i][TN >= 2 ? 1 : 0][r], old[q].y, bias1, rs[q].y);
              *reinterpret_cast<f2*>(C + row * p.ldc + c0) = v;
            }
          }
#if defined(__HIP_DEVICE_COMPILE__)
          __builtin_amdgcn_sched_barrier(0);
#endif
        }
    }
    if (TN < 3) return;
  }
  if constexpr (TALL) {
    // Tiles wholly inside the output (all of them when 128 | M and 96 | N): no
    // per-element guards, one 64-bit multiply per lane (register r of a lane is
    // 8 (r / 4) + r % 4 rows below the lane's first row: a constant times the
    // pitch, computed on the scalar unit), and all loads of the epilogue (bias,
    // residual) before the first store -- loads and stores share one counter on
    // this hardware, so a load issued after stores is only known to have landed
    // once those stores have drained.  Measured at 8192 x 2304 x 768 with a bias:
    // 238 us with the guarded loop below, 225 us without a bias.
    if (p.beta == 0.0f && m0 + BMt <= p.M && n0 + BNt <= p.N) {
      const int64_t row0 = m0 + wm + 4 * half;
      float* cl = C + row0 * p.ldc + n0 + col;
      const float* rl = res ? res + row0 * p.ldres + n0 + col : nullptr;
      float biasv[TN], rs[TN][16];
#pragma unroll
      for (int j = 0; j < TN; j++) {
        biasv[j] = (FUSED && p.bias) ? p.bias[n0 + j * 32 + col] : 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++)
          rs[j][r] = rl ? rl[(int64_t)(8 * (r >> 2) + (r & 3)) * p.ldres + 32 * j] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          cl[(int64_t)(8 * (r >> 2) + (r & 3)) * p.ldc + 32 * j] =
              finish_value<FUSED>(p, acc[0][j][r], 0.f, biasv[j], rs[j][r]);
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      if (pairs && j < 2) continue;  // stored above
      // tiles 0 and 1 of an n-innermost right operand own interleaved columns
      const int64_t cc = (!TALL && !RKIN && TN >= 2)
                             ? (j < 2 ? n0 + wn + 2 * col + j : n0 + wn + 64 + col)
                             : n0 + wn + j * 32 + col;
      if (cc >= p.N) continue;
      const float biasv = (FUSED && p.bias) ? p.bias[cc] : 0.f;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        float old[8], rs[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
          const int r = 8 * h + q;
          const int64_t row = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
          old[q] = 0.f;
          rs[q] = 0.f;
          if (row < p.M) {
            if (p.beta != 0.0f) old[q] = C[row * p.ldc + cc];
            if (res) rs[q] = res[row * p.ldres + cc];
          }
        }
#pragma unroll
        for (int q = 0; q < 8; q++) {
          const int r = 8 * h + q;
          const int64_t row = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
          if (row < p.M) C[row * p.ldc + cc] = finish_value<FUSED>(p, acc[i][j][r], old[q], biasv, rs[q]);
        }
#if defined(__HIP_DEVICE_COMPILE__)
        __builtin_amdgcn_sched_barrier(0);
#endif
      }
    }
}

static inline bool aligned16(const void* q) { return ((uintptr_t)q & 15u) == 0; }

static bool is_n(char c) { return c == 'N' || c == 'n'; }
static bool is_t(char c) { return c == 'T' || c == 't' || c == 'C' || c == 'c'; }

template <bool LK, bool RK, bool FAST, int TM, int TN, int FUSED>
static int launch_kernel(const GemmParams& p, dim3 grid, hipStream_t st) {
  constexpr int lfloats = LK ? 64 * TM * KPITCH : BK * 64 * TM;
  constexpr int rfloats = RK ? 64 * TN * KPITCH : BK * 64 * TN;
  constexpr size_t bytes = 2 * (size_t)(lfloats + rfloats) * sizeof(float);
  static bool configured = false;  // per instantiation
  if (!configured) {
    WF2_TRY(check_hip(
        hipFuncSetAttribute(reinterpret_cast<const void*>(&sgemm_kernel<LK, RK, FAST, TM, TN, FUSED>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes),
        "hipFuncSetAttribute(sgemm_kernel)"));
    configured = true;
  }
  sgemm_kernel<LK, RK, FAST, TM, TN, FUSED><<<grid, kBlock, bytes, st>>>(p);
  return 0;
}

template <bool RK, int TN, int FUSED, bool TALL>
static int launch_dma_kernel(const GemmParams& p, dim3 grid, hipStream_t st) {
  constexpr size_t bytes = DmaLayout<RK, TN, TALL>::LDS_BYTES;
  static bool configured = false;  // per instantiation
  if (!configured) {
    WF2_TRY(check_hip(
        hipFuncSetAttribute(reinterpret_cast<const void*>(&sgemm_dma_kernel<RK, TN, FUSED, TALL>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes),
        "hipFuncSetAttribute(sgemm_dma_kernel)"));
    configured = true;
  }
  sgemm_dma_kernel<RK, TN, FUSED, TALL><<<grid, kBlock, bytes, st>>>(p);
  return 0;
}

// TN = 1, 2, 3: 128 x 64, 128 x 128, 128 x 192 output tiles; TALL with TN = 3: 128 x 96
template <int TN, bool TALL = false>
static int launch_dma(const GemmParams& p, bool rkin, dim3 grid, hipStream_t st) {
  const int fused = p.activation ? 2 : ((p.bias || p.residual || p.causal) ? 1 : 0);
  if (rkin) {
    if (fused == 2) return launch_dma_kernel<true, TN, 2, TALL>(p, grid, st);
    if (fused == 1) return launch_dma_kernel<true, TN, 1, TALL>(p, grid, st);
    return launch_dma_kernel<true, TN, 0, TALL>(p, grid, st);
  }
  if (fused == 2) return launch_dma_kernel<false, TN, 2, TALL>(p, grid, st);
  if (fused == 1) return launch_dma_kernel<false, TN, 1, TALL>(p, grid, st);
  return launch_dma_kernel<false, TN, 0, TALL>(p, grid, st);
}

template <bool LK, bool RK, int TM, int TN>
static int launch_variant(const GemmParams& p, bool fast, dim3 grid, hipStream_t st) {
  // the plain product keeps a lean epilogue; bias / activation / residual /
  // triangular skipping live in a separate instantiation
  const bool fused = p.bias || p.residual || p.activation || p.causal;
  if (fused) {
    if (fast) return launch_kernel<LK, RK, true, TM, TN, 2>(p, grid, st);
    return launch_kernel<LK, RK, false, TM, TN, 2>(p, grid, st);
  }
  if (fast) return launch_kernel<LK, RK, true, TM, TN, 0>(p, grid, st);
  return launch_kernel<LK, RK, false, TM, TN, 0>(p, grid, st);
}

template <int TM, int TN>
static int launch_layout(const GemmParams& p, bool lkin, bool rkin, bool fast, dim3 grid,
                         hipStream_t st) {
  if (lkin && rkin) return launch_variant<true, true, TM, TN>(p, fast, grid, st);
  if (lkin) return launch_variant<true, false, TM, TN>(p, fast, grid, st);
  if (rkin) return launch_variant<false, true, TM, TN>(p, fast, grid, st);
  return launch_variant<false, false, TM, TN>(p, fast, grid, st);
}

// Workgroups are spread evenly over the CUs, and the ones resident on a CU
// share its matrix cores, so the launch takes about as long as the busiest CU:
// ceil(tiles / CUs) tiles, one after the other.
static double busiest_cu_tiles(int64_t tiles) {
  const int64_t cus = rt().num_cus;
  return (double)((tiles + cus - 1) / cus);
}

struct Epilogue {
  const float* bias = nullptr;
  const float* residual = nullptr;
  int64_t ldres = 0, sRes = 0, sRes2 = 0;
  int activation = 0;
  int causal = 0;
};

// What the folds of a split-K run add after the sum (row-major terms, as the product's own epilogue):
// act(sum + beta C + bias[col]) + residual[row][col]; the column-major element (i, j) is row j, column i.
struct FoldEpilogue {
  const float* bias;
  const float* residual;
  int64_t ldres;
  int32_t activation;
};

__device__ __forceinline__ void fold_store(float* c, float acc, float beta, const FoldEpilogue& ep, int64_t i, int64_t j) {
  float v = beta == 0.0f ? acc : beta * *c + acc;
  if (ep.bias) v += ep.bias[i];
  if (ep.activation == 1) v = gelu_tanh_fast(v);
  if (ep.residual) v += ep.residual[j * ep.ldres + i];
  *c = v;
}

// C[b] <- beta C[b] + sum over the `splits` partial products of a split-K run (column-major; the partial
// of slice s and matrix b is the packed m x n plane s * batch + b, already scaled by alpha);
// blockIdx.y is the matrix of the batch
__global__ __launch_bounds__(kBlock) void splitk_fold(const float* __restrict__ partials, int splits, int64_t m,
                                                      int64_t n, float beta, float* __restrict__ C, int64_t ldc,
                                                      int64_t strideC, FoldEpilogue ep) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= m * n) return;
  const int64_t j = e / m, i = e - j * m;
  const int64_t plane = m * n, step = plane * gridDim.y;
  partials += (int64_t)blockIdx.y * plane;
  float acc = 0.0f;
  for (int s = 0; s < splits; s++) acc += partials[(int64_t)s * step + e];
  fold_store(C + (int64_t)blockIdx.y * strideC + i + j * ldc, acc, beta, ep, i, j);
}

// More than 16 partial products: a wavefront per output element, lane l adds slices l, l + 64, ...
// in binary64 with eight loads in flight, the lanes meet by shuffles -- a fixed order.
__global__ __launch_bounds__(kBlock) void splitk_fold_wide(const float* __restrict__ partials, int splits, int64_t m,
                                                           int64_t n, float beta, float* __restrict__ C, int64_t ldc,
                                                           int64_t strideC, FoldEpilogue ep) {
  const int64_t e = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (e >= m * n) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t plane = m * n, step = plane * gridDim.y;
  partials += (int64_t)blockIdx.y * plane;
  double acc = 0.0;
  int s = lane;
  for (; s + 7 * kWave < splits; s += 8 * kWave) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) v[u] = partials[(int64_t)(s + u * kWave) * step + e];
#pragma unroll
    for (int u = 0; u < 8; u++) acc += (double)v[u];
  }
  for (; s < splits; s += kWave) acc += (double)partials[(int64_t)s * step + e];
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) {
    const int64_t j = e / m, i = e - j * m;
    fold_store(C + (int64_t)blockIdx.y * strideC + i + j * ldc, (float)acc, beta, ep, i, j);
  }
}

int sgemm_batched2(char transa, char transb, long m, long n, long k, float alpha, const float* A,
                   long lda, long strideA, long strideA2, const float* B, long ldb, long strideB,
                   long strideB2, float beta, float* C, long ldc, long strideC, long strideC2,
                   long batch, long batch2, const Epilogue& ep = Epilogue());

int binary_nd(int op, Space s, float* a, const float* b);  // elementwise.hip
bool try_sgemm_skinny(bool w_is_cols_by_k, long rows, long cols, long k, float alpha, const float* W, long ldw,
                      const float* X, long ldx, float beta, float* C, long ldc, const float* bias,
                      const float* residual, long ldres, int activation, int* rc);  // gemm_skinny.hip
bool try_sgemm_tiny_out(long rows, long cols, long k, float alpha, const float* L, long ldl, const float* R, long ldr,
                        float** partial, long* planes, int* rc);  // gemm_skinny.hip
bool try_sgemm_small_batch(bool ta, bool tb, long m, long n, long k, float alpha, const float* A, long lda, long sA,
                           long sA2, const float* B, long ldb, long sB, long sB2, float beta, float* C, long ldc,
                           long sC, long sC2, long batch, long batch2, int* rc);  // gemm_skinny.hip

// Products with few output tiles and a long K (weight gradients: 768 x 3072 outputs over K = 8192 are
// 144 tiles for 256 compute units) run as `splits` products over slices of K, the slices as the outer
// batch level of one launch, folded in a fixed order afterwards.  One batch level of such products
// ((12, 3, 100000) . (12, 100000, 3)) is split the same way.
static bool try_split_k(char transa, char transb, long m, long n, long k, float alpha, const float* A, long lda,
                        long strideA, const float* B, long ldb, long strideB, float beta, float* C, long ldc,
                        long strideC, long batch, const Epilogue& ep, int* rc) {
  static thread_local bool splitting = false;  // the slices themselves are not split again
  struct Guard {
    bool& flag;
    explicit Guard(bool& f) : flag(f) { flag = true; }
    ~Guard() { flag = false; }
  };
  const int64_t tiles = ceil_div(m, 128) * ceil_div(n, 128) * batch;
  const int64_t cus = rt().num_cus;
  if (splitting || tiles >= cus || m < 1 || n < 1) return false;
  long splits = 0, kc = 0;
  if (k < 2048) {
    // A short K with few tiles (a few hundred rows through a layer: (256 x 768) . (768 x 2304) is 36 tiles
    // of 48 steps each, one workgroup on a compute unit in seven): equal slices of at least 128 that bring
    // the launch to about half the compute units -- more slices cost in the fold what they save ((256 x 768)
    // . (768 x 2304) with its bias: 30.5 us whole, 22.6 us in 3 slices, 28.3 us in 6), and from a quarter
    // of the compute units in tiles on the whole product is as fast ((512 x 768) . (768 x 2304): 31.9 / 33.5 us).
    // Slices of at least 256 keep the streaming kernel; where those leave the launch below a quarter of the
    // compute units, slices of at least 128 ((128 x 768) . (768 x 2304): 3 slices 19.6 us, 6 slices 16.6 us).
    // Single products only (the layers of a model).
    if (batch != 1 || k < 512 || tiles > cus / 4) return false;
    const long want = (cus / 2 + tiles / 2) / tiles;
    auto equal_slices = [&](long least) {
      for (long cand = std::min<long>(want, k / least); cand >= 2; cand--)
        if (k % (cand * 32) == 0) return cand;
      return 0L;
    };
    splits = equal_slices(256);
    if (splits * tiles < cus / 4) splits = equal_slices(128);
    if (splits == 0) return false;
    kc = k / splits;
  }
  Guard guard(splitting);
  // Equal slices where K allows it.  Few output tiles and a very long K (the weight gradient of a layer
  // with few outputs: (10 x N) . (N x 256) over a batch of 65536 ran 150 us on 16 slices): as many slices
  // of at least 512 as keep the launch within four workgroups per compute unit.
  // (shorter slices, 256 and then 128, where those of 512 leave the launch below a quarter of the compute
  // units: (96 x 3072) . (3072 x 768), 6 tiles: 36 us in 4 slices, 20 us in 24)
  // Where the powers of two leave most compute units idle, any count of equal slices will do: the weight
  // gradient of a convolution over K = 43264 = 2^8 13^2 (one tile) ran as 8 slices, 106 us; 52 divide it too.
  if (splits == 0 && batch == 1)
    for (long least : {512L, 256L, 128L}) {
      for (int cand : {1024, 512, 256, 128, 64, 32, 16, 8, 4, 2})
        if (k % ((long)cand * 32) == 0 && k / cand >= least && tiles * cand <= 4 * cus) {
          splits = cand;
          break;
        }
      if (splits * tiles < cus / 2) {
        const long most = std::min<long>(std::min<long>(k / least, (long)(4 * cus / tiles)), 1024);
        for (long cand = most; cand > splits && cand >= 2; cand--)
          if (k % (cand * 32) == 0) {
            splits = cand;
            break;
          }
      }
      if (splits) kc = k / splits;
      if (splits * tiles >= cus / 4) break;
    }
  long rest = 0;  // length of a shorter last slice
  if (splits == 0) {
    // any K ((127 x 100000) . (100000 x 127) ran 5.9 ms as one product): slices of a multiple of 32, the
    // last one shorter, in a launch of its own
    long most = std::min<long>(k / 512, (long)(4 * cus / tiles));
    most = std::min<long>(most, 1024);
    if (most < 2) return false;
    kc = ceil_div(ceil_div(k, most), 32L) * 32;
    splits = k / kc;
    rest = k - splits * kc;
    if (splits + (rest ? 1 : 0) < 2) return false;
  }
  const long planes = splits + (rest ? 1 : 0);
  const int64_t plane = (int64_t)m * n;
  void* scratch = nullptr;
  if (!scratch_block(&scratch, (size_t)(planes * batch * plane) * sizeof(float), rc)) return *rc != 0;
  float* part = static_cast<float*>(scratch);
  const long sa = is_n(transa) ? kc * lda : kc;  // op(A) is m x k: a K slice starts kc columns / rows further
  const long sb = is_n(transb) ? kc : kc * ldb;
  *rc = sgemm_batched2(transa, transb, m, n, kc, alpha, A, lda, strideA, sa, B, ldb, strideB, sb, 0.0f, part, m,
                       (long)plane, (long)(plane * batch), batch, splits);
  if (*rc == 0 && rest)
    *rc = sgemm_batched2(transa, transb, m, n, rest, alpha, A + splits * sa, lda, strideA, 0, B + splits * sb, ldb,
                         strideB, 0, 0.0f, part + splits * batch * plane, m, (long)plane, 0, batch, 1);
  if (*rc == 0) {
    const FoldEpilogue fe{ep.bias, ep.residual, ep.ldres, ep.activation};
    if (planes <= 16) {
      const dim3 grid((uint32_t)ceil_div(plane, (int64_t)kBlock), (uint32_t)batch);
      splitk_fold<<<grid, kBlock, 0, rt().stream>>>(part, (int)planes, m, n, beta, C, ldc, strideC, fe);
    } else {
      const dim3 grid((uint32_t)ceil_div(plane, (int64_t)(kBlock / kWave)), (uint32_t)batch);
      splitk_fold_wide<<<grid, kBlock, 0, rt().stream>>>(part, (int)planes, m, n, beta, C, ldc, strideC, fe);
    }
    *rc = after_launch("splitk_fold");
  }
  (void)wf2hip_free(scratch);  // stream order keeps it alive for the launches above
  return true;
}

int sgemm_batched2(char transa, char transb, long m, long n, long k, float alpha, const float* A,
                   long lda, long strideA, long strideA2, const float* B, long ldb, long strideB,
                   long strideB2, float beta, float* C, long ldc, long strideC, long strideC2,
                   long batch, long batch2, const Epilogue& ep) {
  if (!(is_n(transa) || is_t(transa)) || !(is_n(transb) || is_t(transb)))
    return fail(WF2HIP_EINVAL, "trans must be N, T or C");
  if (m < 0 || n < 0 || k < 0 || batch < 0 || batch2 < 0)
    return fail(WF2HIP_EINVAL, "negative dimension");
  // sgemm_'s own leading-dimension rules (column-major)
  const long rows_a = is_n(transa) ? m : k;
  const long rows_b = is_n(transb) ? k : n;
  if (lda < (rows_a > 1 ? rows_a : 1) || ldb < (rows_b > 1 ? rows_b : 1) || ldc < (m > 1 ? m : 1))
    return fail(WF2HIP_EINVAL, "leading dimension too small (lda %ld ldb %ld ldc %ld)", lda, ldb,
                ldc);
  if (m == 0 || n == 0 || batch == 0 || batch2 == 0) return 0;
  if (!A || !B || !C) return fail(WF2HIP_EINVAL, "null matrix pointer");
  if ((int64_t)batch * batch2 > 65535)
    return fail(WF2HIP_EUNSUPPORTED, "more than 65535 matrices in one batch");
  // many small matrices: an output element per thread or wavefront
  if (!ep.bias && !ep.residual && ep.activation == 0 && ep.causal == 0) {
    int rc = 0;
    if (try_sgemm_small_batch(!is_n(transa), !is_n(transb), m, n, k, alpha, A, lda, strideA, strideA2, B, ldb, strideB,
                              strideB2, beta, C, ldc, strideC, strideC2, batch, batch2, &rc))
      return rc;
  }
  // 33 ... 64 rows of the row-major product against a weight stored (cols, k) (`(!matmul x (!t w))`: a few
  // dozen tokens against the token table): the few-rows kernel below feeds the matrix cores from global
  // memory and keeps them busy about a third of the time at this height, and the tiled kernels pad the rows
  // to 128.  With the operands exchanged the weight is the operand with 128 rows per tile and the tokens are
  // the 64 columns of a 128 x 64 tile, nothing padded; the streaming kernel turns each tile over in LDS on the
  // way out ((64, 768) . (50257, 768)^T: 96 -> 62 us; with few tiles the slices of K below come first).
  static const char* turn_env = getenv("WF2HIP_GEMM_TURN_ROWS");  // testing knob: least number of rows, 0 = never
  const long turn_from = turn_env ? atol(turn_env) : 33;
  const bool turned = turn_from > 0 && n >= turn_from && n <= 64 && m >= 1024 && is_n(transb) && !is_n(transa) &&
                      ep.causal == 0 && k % BK == 0 && k >= 256 && aligned16(A) && aligned16(B) && lda % 4 == 0 &&
                      ldb % 4 == 0 && lda < ((long)1 << 22) && ldb < ((long)1 << 22) && strideA % 4 == 0 &&
                      strideB % 4 == 0 && strideA2 % 4 == 0 && strideB2 % 4 == 0;
  // at most 64 rows in the row-major product (a few tokens through a layer): one read of the other operand
  if (!turned && batch == 1 && batch2 == 1 && n <= 64 && is_n(transb) && ep.causal == 0) {
    int rc = 0;
    if (try_sgemm_skinny(!is_n(transa), n, m, k, alpha, A, lda, B, ldb, beta, C, ldc, ep.bias, ep.residual, ep.ldres,
                         ep.activation, &rc))
      return rc;
  }
  // a small output over a long K with both operands stored K-major (the weight gradient of a convolution
  // with few channels): partial planes by slices of K, folded like the split-K planes
  if (batch == 1 && batch2 == 1 && is_n(transa) && !is_n(transb) && ep.causal == 0) {
    int rc = 0;
    float* part = nullptr;
    long planes = 0;
    if (try_sgemm_tiny_out(n, m, k, alpha, B, ldb, A, lda, &part, &planes, &rc)) {
      if (rc == 0) {
        const FoldEpilogue fe{ep.bias, ep.residual, ep.ldres, ep.activation};
        const dim3 grid((uint32_t)ceil_div((int64_t)m * n, (int64_t)(kBlock / kWave)), 1);
        splitk_fold_wide<<<grid, kBlock, 0, rt().stream>>>(part, (int)planes, m, n, beta, C, ldc, 0, fe);
        rc = after_launch("splitk_fold");
      }
      (void)wf2hip_free(part);  // stream order keeps it alive for the launches above
      return rc;
    }
  }
  // x^T . dY (weight gradients): the left operand of the row-major product arrives stored
  // (k, rows), which only the register-staged kernel reads.  One transposing pass over it
  // (k x rows elements) puts the product on the streaming kernel.
  if (batch == 1 && batch2 == 1 && !is_n(transb) && k >= 1024 && k % BK == 0 && n >= 128 && m >= 128 &&
      aligned16(A) && aligned16(B) && lda % 4 == 0 && ldb % 4 == 0 && (is_n(transa) ? m % 4 == 0 : true)) {
    void* turned = nullptr;
    int held_up = 0;
    if (!scratch_block(&turned, (size_t)k * n * sizeof(float), &held_up) && held_up) return held_up;
    if (turned) {
      Space sp;  // dst (k x n column-major): (kk, j) at kk + j k; src (n x k): j + kk ldb
      sp.rank = 2;
      sp.shape[0] = n;
      sp.shape[1] = k;
      sp.sa[0] = k;
      sp.sa[1] = 1;
      sp.sb[0] = 1;
      sp.sb[1] = ldb;
      sp.total = (int64_t)k * n;
      int rc = binary_nd(WF2HIP_MOVE, sp, static_cast<float*>(turned), B);
      if (rc == 0)
        rc = sgemm_batched2(transa, 'N', m, n, k, alpha, A, lda, 0, 0, static_cast<const float*>(turned), k, 0, 0,
                            beta, C, ldc, 0, 0, 1, 1, ep);
      (void)wf2hip_free(turned);  // stream order keeps it alive for the launches above
      return rc;
    }
  }
  // (the fused epilogue of a single product goes into the fold; batches with one keep the plain route)
  if (batch2 == 1 && batch <= 65535 && ep.causal == 0 && (batch == 1 || (!ep.bias && !ep.residual && ep.activation == 0))) {
    int rc = 0;
    if (try_split_k(transa, transb, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch, ep,
                    &rc))
      return rc;
  }

  if (turned) {
    GemmParams p;
    p.L = A;  // the weight: m rows of k
    p.R = B;  // the tokens: n rows of k, the columns of the turned product
    p.C = C;
    p.M = m;
    p.N = n;
    p.K = k;
    p.ldl = lda;
    p.ldr = ldb;
    p.ldc = ldc;
    p.sL = strideA;
    p.sR = strideB;
    p.sC = strideC;
    p.sL2 = strideA2;
    p.sR2 = strideB2;
    p.sC2 = strideC2;
    p.batch_inner = (uint32_t)batch;
    p.alpha = alpha;
    p.beta = beta;
    p.bias = ep.bias;
    p.residual = ep.residual;
    p.ldres = ep.ldres;
    p.sRes = ep.sRes;
    p.sRes2 = ep.sRes2;
    p.activation = ep.activation;
    p.causal = 0;
    p.pair_ok = 0;
    auto by4 = [](int64_t v) { return (v & 3) == 0; };
    const bool vec4 = ((uintptr_t)C % 16 == 0) && by4(ldc) && by4(strideC) && by4(strideC2) &&
                      (!ep.residual || (((uintptr_t)ep.residual % 16 == 0) && by4(ep.ldres) && by4(ep.sRes) && by4(ep.sRes2)));
    p.transposed = vec4 ? 2 : 1;
    p.tiles_m = (uint32_t)ceil_div(p.M, 128);
    p.tiles_n = 1;
    WF2_TRY((launch_dma<1>(p, true, dim3(p.tiles_m, (uint32_t)((int64_t)batch * batch2)), rt().stream)));
    return after_launch("sgemm_dma_kernel");
  }

  GemmParams p;
  // row-major view: Cr[n][m] = Left[n][k] . Right[k][m]
  p.L = B;
  p.R = A;
  p.C = C;
  p.M = n;
  p.N = m;
  p.K = k;
  p.ldl = ldb;
  p.ldr = lda;
  p.ldc = ldc;
  p.sL = strideB;
  p.sR = strideA;
  p.sC = strideC;
  p.sL2 = strideB2;
  p.sR2 = strideA2;
  p.sC2 = strideC2;
  p.batch_inner = (uint32_t)batch;
  p.alpha = alpha;
  p.beta = beta;
  p.bias = ep.bias;
  p.residual = ep.residual;
  p.ldres = ep.ldres;
  p.sRes = ep.sRes;
  p.sRes2 = ep.sRes2;
  p.activation = ep.activation;
  p.causal = ep.causal;
  p.transposed = 0;
  const bool lkin = is_n(transb);   // left stored [rows][k]
  const bool rkin = !is_n(transa);  // right stored [cols][k]
  bool fast = aligned16(A) && aligned16(B) && lda % 4 == 0 && ldb % 4 == 0 && strideA % 4 == 0 &&
              strideB % 4 == 0 && strideA2 % 4 == 0 && strideB2 % 4 == 0;
  // every 4-wide load must be wholly inside or wholly outside the matrix
  fast = fast && (lkin ? k % 4 == 0 : p.M % 4 == 0) && (rkin ? k % 4 == 0 : p.N % 4 == 0);

  // 8-byte output stores: even pitch and batch strides, 8-byte aligned bases
  auto even = [](int64_t v) { return (v & 1) == 0; };
  p.pair_ok = ((uintptr_t)C % 8 == 0) && even(ldc) && even(strideC) && even(strideC2) &&
              (!ep.residual || (((uintptr_t)ep.residual % 8 == 0) && even(ep.ldres) &&
                                even(ep.sRes) && even(ep.sRes2)));
  // global -> LDS streaming kernel: left operand k-innermost, whole K-steps
  // (with only a few K-steps per tile the set-up of the streaming kernel costs more
  // than it saves: 96 x 1024x1024x64 runs in 187 us staged, 243 us streamed)
  // (the streaming kernel addresses a tile's rows by 32-bit byte offsets from a base of the workgroup)
  const bool pitch32 = lda < ((long)1 << 22) && ldb < ((long)1 << 22);
  bool dma = fast && lkin && k % BK == 0 && k >= 256 && pitch32;
  if (const char* force = getenv("WF2HIP_GEMM_STREAM"))  // testing knob: 0 never, 1 whenever possible
    dma = force[0] == '1' ? (fast && lkin && k % BK == 0 && k > 0 && pitch32) : false;

  // Tile choice: time ~ tiles on the busiest CU x tile width / efficiency.
  // Measured per unit of work 128x128 is about 6 % ahead of 128x64 (which
  // re-reads one operand from LDS twice as often but keeps three workgroups on a
  // CU), so what decides is how evenly the tile count divides over the CUs
  // (8192 x 768 outputs: 768 or 384 tiles on 256 CUs).  A width that leaves one
  // tile per CU loses the overlap of one workgroup's prologue and epilogue with
  // another's K loop.  The 128x192 tile of the streaming kernel matches the
  // others back to back but ran 25 % slower between other kernels (8192 x 2304
  // x 768: 316 us against 245 us), so it is only reachable through the knob.
  const int64_t nb = (int64_t)batch * batch2;
  // The 128x96 tile (streaming kernel only) exists for widths 128 and 64 leave
  // ragged: N = 768 gives 8 whole tiles per row of tiles, 8192 x 768 outputs two
  // tiles per CU, 8192 x 2304 six.
  const int widths[3] = {64, 128, 96};
  // (over a short K the narrow tile is level with the others per unit of work -- it pays the start and the
  // end of a tile more often, and more, shorter tiles hide those better: 8192 x 768 x 768 75 us in 128 x 64
  // tiles, three per compute unit, against 78 us in 128 x 96 tiles, two per unit)
  const double eff[3] = {p.K <= 1024 ? 0.99 : 0.94, 1.0, 0.97};
  int width = 128;
  double best = 0.0;
  for (int c = 0; c < (dma ? 3 : 2); c++) {
    const int64_t tiles = ceil_div(p.M, 128) * ceil_div(p.N, widths[c]) * nb;
    const double rounds = busiest_cu_tiles(tiles);
    const double cost = rounds * widths[c] / (eff[c] * (rounds < 2.0 ? 0.85 : 1.0));
    if (c == 0 || cost < best) {
      best = cost;
      width = widths[c];
    }
  }
  if (const char* force = getenv("WF2HIP_GEMM_TILE")) {  // tuning knob: n(arrow), w(ide), x(tra wide), t(all)
    width = force[0] == 'n' ? 64 : (force[0] == 'x' && dma ? 192 : (force[0] == 't' && dma ? 96 : 128));
  }
  p.tiles_m = (uint32_t)ceil_div(p.M, 128);
  p.tiles_n = (uint32_t)ceil_div(p.N, width);
  const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many tiles");
  dim3 grid((uint32_t)blocks, (uint32_t)nb);
  hipStream_t st = rt().stream;
  if (dma) {
    if (width == 64)
      WF2_TRY((launch_dma<1>(p, rkin, grid, st)));
    else if (width == 128)
      WF2_TRY((launch_dma<2>(p, rkin, grid, st)));
    else if (width == 96)
      WF2_TRY((launch_dma<3, true>(p, rkin, grid, st)));
    else
      WF2_TRY((launch_dma<3>(p, rkin, grid, st)));
    return after_launch("sgemm_dma_kernel");
  }
  if (width == 64)
    WF2_TRY((launch_layout<2, 1>(p, lkin, rkin, fast, grid, st)));
  else
    WF2_TRY((launch_layout<2, 2>(p, lkin, rkin, fast, grid, st)));
  return after_launch("sgemm_kernel");
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_sgemm(char transa, char transb, long m, long n, long k, float alpha,
                         const float* A, long lda, const float* B, long ldb, float beta, float* C,
                         long ldc) {
  WF2_TRY(require_init());
  return sgemm_batched2(transa, transb, m, n, k, alpha, A, lda, 0, 0, B, ldb, 0, 0, beta, C, ldc, 0,
                        0, 1, 1);
}

WF2_API int wf2hip_sgemm_strided_batched(char transa, char transb, long m, long n, long k,
                                         float alpha, const float* A, long lda, long strideA,
                                         const float* B, long ldb, long strideB, float beta,
                                         float* C, long ldc, long strideC, long batch) {
  WF2_TRY(require_init());
  return sgemm_batched2(transa, transb, m, n, k, alpha, A, lda, strideA, 0, B, ldb, strideB, 0,
                        beta, C, ldc, strideC, 0, batch, 1);
}

WF2_API int wf2hip_sgemm_strided_batched_2d(char transa, char transb, long m, long n, long k,
                                            float alpha, const float* A, long lda, long strideA,
                                            long strideA2, const float* B, long ldb, long strideB,
                                            long strideB2, float beta, float* C, long ldc,
                                            long strideC, long strideC2, long batch, long batch2) {
  WF2_TRY(require_init());
  return sgemm_batched2(transa, transb, m, n, k, alpha, A, lda, strideA, strideA2, B, ldb, strideB,
                        strideB2, beta, C, ldc, strideC, strideC2, batch, batch2);
}

// Row-major C[m,n] = act(alpha A.B + bias) + residual: the operand swap of
// expand-gemm-form-column done here, so that bias is per output column.
WF2_API int wf2hip_matmul_fused(const wf2hip_matmul_desc* d, const float* A, const float* B,
                                float* C) {
  WF2_TRY(require_init());
  if (!d) return fail(WF2HIP_EINVAL, "null descriptor");
  if (d->activation < 0 || d->activation > 1) return fail(WF2HIP_EINVAL, "unknown activation");
  if (d->causal < 0 || d->causal > 2) return fail(WF2HIP_EINVAL, "unknown causal mode");
  if (d->causal == 1 && d->m != d->n)
    return fail(WF2HIP_EINVAL, "lower-triangular output needs a square product");
  if (d->causal == 2 && d->m != d->k)
    return fail(WF2HIP_EINVAL, "a lower-triangular left operand must be square");
  if (d->residual && d->ld_residual < d->n)
    return fail(WF2HIP_EINVAL, "residual pitch smaller than the row");
  Epilogue ep;
  ep.bias = d->bias;
  ep.residual = d->residual;
  ep.ldres = d->ld_residual;
  ep.sRes = d->stride_residual;
  ep.sRes2 = d->stride_residual2;
  ep.activation = d->activation;
  ep.causal = d->causal;
  return sgemm_batched2(d->trans_b ? 'C' : 'N', d->trans_a ? 'C' : 'N', d->n, d->m, d->k, d->alpha,
                        B, d->ldb, d->stride_b, d->stride_b2, A, d->lda, d->stride_a, d->stride_a2,
                        0.0f, C, d->ldc, d->stride_c, d->stride_c2, d->batch, d->batch2, ep);
}
