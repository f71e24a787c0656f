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

#include "wf2_common.h"
#include "wf2_math.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));
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
};

// Loads this thread's share of a ROWS x BK operand tile into registers
// (ROWS/32 float4 per thread).
// KIN: operand stored [x][k] (k innermost) else [k][x].
// FAST: 16-byte loads (pointer, pitch and extents checked on the host).
template <bool KIN, bool FAST, int ROWS>
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
      if (x < X && k < K) v = *reinterpret_cast<const f4*>(KIN ? base + x * ld + k : base + k * ld + x);
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

// TM x TN MFMA tiles (32x32) per wavefront, wavefronts 2 x 2: the workgroup
// tile is (64 TM) x (64 TN).  2x2 -> 128x128 (64 accumulator registers), 2x1
// -> 128x64 for narrow outputs and for shapes whose 128x128 tiling would leave
// a partial last round of workgroups.
template <bool LKIN, bool RKIN, bool FAST, int TM, int TN, bool FUSED>
__global__ __launch_bounds__(kBlock) void sgemm_kernel(GemmParams p) {
  constexpr int BMt = 64 * TM, BNt = 64 * TN;
  constexpr int LFLOATS = LKIN ? BMt * KPITCH : BK * BMt;
  constexpr int RFLOATS = RKIN ? BNt * KPITCH : BK * BNt;
  // two stages of both operand tiles: up to 73.7 KB, beyond the static limit
  extern __shared__ __attribute__((aligned(16))) float smem[];
  auto ldsL = [&](int stage) { return smem + stage * LFLOATS; };
  auto ldsR = [&](int stage) { return smem + 2 * LFLOATS + stage * RFLOATS; };

  // Tile order: consecutive workgroups land on different XCDs (round robin),
  // so give each XCD a contiguous band of tiles, and walk a band column-major
  // in groups of 8 row-tiles so neighbours share operand panels in that L2.
  const uint32_t ntiles = p.tiles_m * p.tiles_n;
  uint32_t pid = blockIdx.x;
  // Triangular problems have cheap and expensive tiles, and workgroups start
  // in dispatch order (x fastest).  Re-read the linear workgroup number as
  // (tile rank, matrix) with the matrix index fastest and the most expensive
  // tile rank first: every CU then works through expensive tiles early and
  // fills up with cheap ones (longest-processing-time-first).
  uint32_t batch_index = blockIdx.y;
  if (FUSED && p.causal) {
    const uint32_t linear = blockIdx.y * ntiles + blockIdx.x;
    batch_index = linear % gridDim.y;
    pid = ntiles - 1 - linear / gridDim.y;  // large tile rows (long K loops) first
  }
  {
    const uint32_t xcds = 8;
    const uint32_t per = ntiles / xcds;
    if (!(FUSED && p.causal) && per > 0 && pid < per * xcds) pid = (pid % xcds) * per + pid / xcds;
  }
  const uint32_t group = 8;
  const uint32_t width = group * p.tiles_n;
  const uint32_t gid = pid / width;
  const uint32_t first_m = gid * group;
  const uint32_t gsize = (p.tiles_m - first_m) < group ? (p.tiles_m - first_m) : group;
  const uint32_t tm = first_m + (pid % width) % gsize;
  const uint32_t tn = (pid % width) / gsize;

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
  load_tile<LKIN, FAST, BMt>(L, p.ldl, m0, 0, p.M, p.K, regL);
  load_tile<RKIN, FAST, BNt>(R, p.ldr, n0, 0, p.N, p.K, regR);
  store_tile<LKIN, BMt>(ldsL(0), regL);
  store_tile<RKIN, BNt>(ldsR(0), regR);
  __syncthreads();

  for (int64_t ks = 0; ks < ksteps; ks++) {
    const int cur = (int)(ks & 1);
    if (ks + 1 < ksteps) {
      load_tile<LKIN, FAST, BMt>(L, p.ldl, m0, (ks + 1) * BK, p.M, p.K, regL);
      load_tile<RKIN, FAST, BNt>(R, p.ldr, n0, (ks + 1) * BK, p.N, p.K, regR);
    }
#pragma unroll
    for (int kb = 0; kb < BK; kb += 8) {
      float a[TM][4], b[TN][4];
#pragma unroll
      for (int i = 0; i < TM; i++) read_frag<LKIN, BMt>(ldsL(cur), wm + i * 32, kb, lane, a[i]);
#pragma unroll
      for (int j = 0; j < TN; j++) read_frag<RKIN, BNt>(ldsR(cur), wn + j * 32, kb, lane, b[j]);
#pragma unroll
      for (int s = 0; s < 4; s++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
    }
    if (ks + 1 < ksteps) {
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
            if (p.activation == 1) v = gelu_tanh_f(v);
            if (p.residual)
              v += p.residual[(int64_t)zo * p.sRes2 + (int64_t)zi * p.sRes + row * p.ldres + col];
          }
          *c = v;
        }
      }
    }
}

static inline bool aligned16(const void* q) { return ((uintptr_t)q & 15u) == 0; }

static bool is_n(char c) { return c == 'N' || c == 'n'; }
static bool is_t(char c) { return c == 'T' || c == 't' || c == 'C' || c == 'c'; }

template <bool LK, bool RK, bool FAST, int TM, int TN, bool FUSED>
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

template <bool LK, bool RK, int TM, int TN>
static int launch_variant(const GemmParams& p, bool fast, dim3 grid, hipStream_t st) {
  // the plain product keeps a lean epilogue; bias / activation / residual /
  // triangular skipping live in a separate instantiation
  const bool fused = p.bias || p.residual || p.activation || p.causal;
  if (fused) {
    if (fast) return launch_kernel<LK, RK, true, TM, TN, true>(p, grid, st);
    return launch_kernel<LK, RK, false, TM, TN, true>(p, grid, st);
  }
  if (fast) return launch_kernel<LK, RK, true, TM, TN, false>(p, grid, st);
  return launch_kernel<LK, RK, false, TM, TN, false>(p, grid, st);
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

int sgemm_batched2(char transa, char transb, long m, long n, long k, float alpha, const float* A,
                   long lda, long strideA, long strideA2, const float* B, long ldb, long strideB,
                   long strideB2, float beta, float* C, long ldc, long strideC, long strideC2,
                   long batch, long batch2, const Epilogue& ep = Epilogue()) {
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
  const bool lkin = is_n(transb);   // left stored [rows][k]
  const bool rkin = !is_n(transa);  // right stored [cols][k]
  bool fast = aligned16(A) && aligned16(B) && lda % 4 == 0 && ldb % 4 == 0 && strideA % 4 == 0 &&
              strideB % 4 == 0 && strideA2 % 4 == 0 && strideB2 % 4 == 0;
  // every 4-wide load must be wholly inside or wholly outside the matrix
  fast = fast && (lkin ? k % 4 == 0 : p.M % 4 == 0) && (rkin ? k % 4 == 0 : p.N % 4 == 0);

  // Tile choice: time ~ tiles on the busiest CU x work per tile.
  // The narrow tile does 10 % less work per cycle (one operand is re-read from
  // LDS twice as often) but wastes nothing on N <= 64 and evens out the last
  // round.
  const int64_t nb = (int64_t)batch * batch2;
  const int64_t tiles_wide = ceil_div(p.M, 128) * ceil_div(p.N, 128) * nb;
  const int64_t tiles_narrow = ceil_div(p.M, 128) * ceil_div(p.N, 64) * nb;
  const double cost_wide = busiest_cu_tiles(tiles_wide) * 1.0;
  const double cost_narrow = busiest_cu_tiles(tiles_narrow) * 0.5 / 0.9;
  bool narrow = cost_narrow < cost_wide;
  if (const char* force = getenv("WF2HIP_GEMM_TILE")) narrow = force[0] == 'n';  // tuning knob
  p.tiles_m = (uint32_t)ceil_div(p.M, 128);
  p.tiles_n = (uint32_t)ceil_div(p.N, narrow ? 64 : 128);
  const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n;
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "too many tiles");
  dim3 grid((uint32_t)blocks, (uint32_t)nb);
  hipStream_t st = rt().stream;
  if (narrow)
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
