// attention.hip -- scaled dot-product attention for heads up to 64 wide in one
// kernel on the CDNA4 fp32 matrix cores (v_mfma_f32_32x32x2_f32).
//
// cl-waffe2 composes attention from nodes: !matmul Q K^T, a scalar multiply,
// !softmax, !matmul with V (examples/gpt-2/utils.lisp:222-243), i.e. two
// batched sgemm_ calls and about ten element-wise / reduction passes over a
// (batch, heads, T, T) tensor.  This kernel produces the same O = softmax(scale
// Q K^T + mask) V without ever writing that tensor: HBM traffic drops from
// O(T^2) to O(T) per head and the causal half of the products is skipped.
//
// Work split: one workgroup per (batch, head, block of 128 queries), four
// wavefronts of 32 queries each; keys/values stream through LDS in blocks of
// 64 (two stages filled by global -> LDS loads, one barrier per block).  Everything is computed transposed so
// that a lane owns one query:
//   S^T = K . Q^T      A operand = K fragment (LDS, conflict-free 128-bit reads),
//                      B operand = Q fragment (registers for the whole kernel,
//                      pre-multiplied by scale * log2 e)
//   O^T += V^T . P^T   A operand = V fragment (LDS, conflict-free 64-bit reads: one accumulator
//                      owns the even head dimensions, the other the odd ones),
//                      B operand = P^T, which is exactly the S^T accumulator
//                      after exp2: accumulator register i of a lane holds key
//                      8 (i/4) + 4 (lane/32) + i%4 of its query, and MFMA step i
//                      takes contraction index "lane/32" from each half, so the
//                      two halves simply contribute different keys and V is
//                      fetched for the matching key.  No shuffle, no LDS round
//                      trip for P.
// The running maximum needs one cross-half exchange per key block; the running
// sum is kept per half and combined once at the end.
//
// Bound: fp32 MFMA (4 T^2 d flop per head dense, half of that causal).
// Numerics: products and sums in binary32 on the matrix cores, exponentials by
// v_exp_f32 (about 1 ulp) on max-subtracted arguments; the result agrees with
// the float64 closed form to ~1e-6 relative to max|V|.
#include <type_traits>

#include "wf2_common.h"
#include "wf2_dma.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kHeadDim = 64;
constexpr int kQBlock = 128;         // queries per workgroup
constexpr int kKBlock = 64;          // keys per LDS stage
constexpr int kRowFloats = kHeadDim;  // LDS rows are unpadded: the global -> LDS path writes 1 KB runs
constexpr int kStageFloats = 2 * kKBlock * kRowFloats;
constexpr size_t kAttnLdsBytes = 2 * (size_t)kStageFloats * sizeof(float);  // 65,536 B

struct AttnParams {
  const float* q;
  const float* k;
  const float* v;
  float* o;
  int64_t qs[3], ks[3], vs[3], os[3];  // element strides: batch, head, position
  int32_t batch, heads, seq;
  int32_t head_dim;  // <= 64, multiple of 4; columns beyond it are treated as zero
  int32_t qblocks;
  int32_t causal;
  float scale_log2e;
  float* lse;  // optional: log2 of the row sums of exp2(scores), (batch * heads, seq); what the backward needs
};

// How far the maximum a row's exponentials are taken against may lag behind the row's true maximum
// (log2 units): the reference only moves when a block holds a score more than this above it, so after
// the first blocks the accumulator is almost never rescaled.  Exponentials then reach 2^8 at most --
// any reference gives the same quotient, and binary32 has the range.
constexpr float kMaxLag = 8.0f;

__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void attention_kernel(
    AttnParams p) {  // two workgroups per CU: at most 256 registers per lane
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr int kKeyFloats = kKBlock * kRowFloats;  // one tile: 64 rows of 64 floats

  // longest query blocks first: with a causal mask block qb needs qb+1 key spans
  const int nbh = p.batch * p.heads;
  const int rank = blockIdx.x / nbh;
  const int bh = blockIdx.x - rank * nbh;
  const int qb = p.qblocks - 1 - rank;
  const int b = bh / p.heads;
  const int h = bh - b * p.heads;

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // uniform: DMA destinations, trip counts and
                                                                         // the causal skipping stay on the scalar unit
  const int half = lane >> 5;
  const int col = lane & 31;

  // With a causal mask the wavefronts of a workgroup walk 2 qb + 1, 2 qb + 1, 2 qb + 2, 2 qb + 2 key
  // blocks.  Wavefront w of every workgroup sits on SIMD w, so every second workgroup hands its
  // queries out in reverse: the two workgroups that share a compute unit then load its SIMDs evenly.
  const int part = (p.causal && (blockIdx.x & 1)) ? 3 - wave : wave;
  const int q_first = qb * kQBlock + part * 32;  // first query of this wavefront
  const int query = q_first + col;
  const int query_ld = query < p.seq ? query : p.seq - 1;

  const float* qp = p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)query_ld * p.qs[2];
  const float* kp = p.k + b * p.ks[0] + h * p.ks[1];
  const float* vp = p.v + b * p.vs[0] + h * p.vs[1];

  // Q fragment: qf[4 j + r] = Q[query][8 j + 4 half + r] * scale * log2(e)
  float qf[32];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    f4 t = {0.f, 0.f, 0.f, 0.f};
    if (8 * j + 4 * half < p.head_dim) t = *reinterpret_cast<const f4*>(qp + 8 * j + 4 * half);
    qf[4 * j + 0] = t.x * p.scale_log2e;
    qf[4 * j + 1] = t.y * p.scale_log2e;
    qf[4 * j + 2] = t.z * p.scale_log2e;
    qf[4 * j + 3] = t.w * p.scale_log2e;
  }

  // key blocks this workgroup walks
  const int q_last_block = min(qb * kQBlock + kQBlock, p.seq) - 1;
  const int key_end = p.causal ? q_last_block + 1 : p.seq;
  const int nkb = (key_end + kKBlock - 1) / kKBlock;
  const int q_last_wave = q_first + 31;

  f16v o0 = {0}, o1 = {0};
  float m = -INFINITY;  // the maximum the exponentials are taken against (log2 domain), shared by both halves
  float lsum = 0.f;     // running sum of this half's keys

  // Key / value blocks go global -> LDS without passing through registers: one
  // instruction moves 64 x 16 bytes into 1 KB of LDS (four rows).  The 16-byte
  // slots of a row are permuted through the address each lane reads from:
  //   keys    slot = chunk ^ (row % 16), so that the 128-bit fragment reads of 16
  //           consecutive rows cover all 64 banks;
  //   values  the two 128-byte halves of a row are swapped when (row / 4) is odd:
  //           the half-waves read rows 4 apart and then hit different banks.
  // A block's base address stays on the scalar unit; per lane there are only the four byte offsets
  // of its pieces (wf2_dma.h).  Rows beyond the sequence are clamped (their scores are masked later):
  // only the last block of a ragged sequence computes offsets of its own.  Chunks beyond head_dim
  // are not loaded and stay zero from the clear below.
  const uint32_t lds0 = lds_address(smem);
  const int drow = lane >> 4, dslot = lane & 15;
  uint32_t koff[4], voff[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int row = (wave * 4 + j) * 4 + drow;
    koff[j] = (uint32_t)((row * p.ks[2] + (dslot ^ (row & 15)) * 4) * (int64_t)sizeof(float));
    voff[j] = (uint32_t)((row * p.vs[2] + (dslot ^ (((row >> 2) & 1) << 3)) * 4) * (int64_t)sizeof(float));
  }
  const bool whole_rows = p.head_dim == kHeadDim;
  auto fetch = [&](bool values, int stage, int key0) {
    const float* base = values ? vp + (int64_t)key0 * p.vs[2] : kp + (int64_t)key0 * p.ks[2];
    const uint32_t dst = lds0 + (uint32_t)((stage * kStageFloats + (values ? kKeyFloats : 0) + wave * 1024) * sizeof(float));
    const bool ragged = key0 + kKBlock > p.seq;
    if (whole_rows && !ragged) {
#pragma unroll
      for (int j = 0; j < 4; j++) dma16(dst + j * 1024, values ? voff[j] : koff[j], base);
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int row = (wave * 4 + j) * 4 + drow;
        const int chunk = values ? dslot ^ (((row >> 2) & 1) << 3) : dslot ^ (row & 15);
        const int last = p.seq - 1 - key0;  // >= 0: key0 < seq
        const int64_t r = row < last ? row : last;
        const uint32_t off = (uint32_t)((r * (values ? p.vs[2] : p.ks[2]) + chunk * 4) * (int64_t)sizeof(float));
        if (chunk * 4 < p.head_dim) dma16(dst + j * 1024, off, base);
      }
    }
  };
  if (p.head_dim < kHeadDim) {
    for (int i = threadIdx.x; i < 2 * kStageFloats / 4; i += kBlock)
      reinterpret_cast<f4*>(smem)[i] = f4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
  }

  // LDS addresses of the fragments, fixed for the kernel: everything that depends on the block or the
  // stage is an immediate, so the loop holds no address arithmetic (a vector-ALU instruction costs the
  // matrix cores 5 - 12 cycles of issue).
  //   keys    row col (and 32 + col), 16-byte slot (2 j + half) ^ (col % 16) for contraction group j
  //   values  row 4 half + ..., floats 2 col, 2 col + 1 with the halves swapped for the upper half-wave
  const float* kfrag[8];
#pragma unroll
  for (int j = 0; j < 8; j++) kfrag[j] = smem + col * kRowFloats + (((2 * j + half) ^ (col & 15)) * 4);
  const float* vfrag = smem + kKeyFloats + 4 * half * kRowFloats + ((2 * col) ^ (half << 5));

  // S^T of one key block: two 32 x 32 tiles (keys 0-31 and 32-63 of the block).  The fragments of
  // contraction group j + 1 are on their way while the matrix cores work on group j.
  auto scores = [&](int stage, f16v& s0, f16v& s1) {
    const int so = stage * kStageFloats;
    f4 ka[2], kb[2];
    ka[0] = *reinterpret_cast<const f4*>(kfrag[0] + so);
    kb[0] = *reinterpret_cast<const f4*>(kfrag[0] + so + 32 * kRowFloats);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      if (j + 1 < 8) {
        ka[(j + 1) & 1] = *reinterpret_cast<const f4*>(kfrag[j + 1] + so);
        kb[(j + 1) & 1] = *reinterpret_cast<const f4*>(kfrag[j + 1] + so + 32 * kRowFloats);
      }
      const f4 k0 = ka[j & 1], k1 = kb[j & 1];
      if (j == 0) {
        const f16v zero = {0};
        s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.x, qf[0], zero, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.x, qf[0], zero, 0, 0, 0);
      } else {
        s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.x, qf[4 * j + 0], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.x, qf[4 * j + 0], s1, 0, 0, 0);
      }
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.y, qf[4 * j + 1], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.y, qf[4 * j + 1], s1, 0, 0, 0);
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.z, qf[4 * j + 2], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.z, qf[4 * j + 2], s1, 0, 0, 0);
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.w, qf[4 * j + 3], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.w, qf[4 * j + 3], s1, 0, 0, 0);
#if defined(__HIP_DEVICE_COMPILE__)
      // the two reads of the next group go among this group's first MFMAs
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 6, 0);
#endif
    }
  };
  // masks, running softmax statistics, P = exp2(S - m) in place.  Per score: a share of a three-way
  // maximum, a subtraction, an exponential and an addition; the accumulator is rescaled only when the
  // reference maximum moves (kMaxLag), which a branch the whole wavefront takes or skips decides.
  auto normalise = [&](int key0, f16v& s0, f16v& s1) {
    // register i of tile t holds key key0 + 32 t + 8 (i/4) + 4 half + i%4
    const bool edge = (p.causal && key0 + kKBlock - 1 > q_first) || key0 + kKBlock > p.seq;
    if (edge) {
      const int limit = p.causal ? min(query, p.seq - 1) : p.seq - 1;  // last visible key
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int key = key0 + 8 * (i >> 2) + 4 * half + (i & 3);
        if (key > limit) s0[i] = -INFINITY;
        if (key + 32 > limit) s1[i] = -INFINITY;
      }
    }
    float mloc = fmaxf(s0[0], s1[0]);
#pragma unroll
    for (int i = 1; i < 16; i++) mloc = fmaxf(fmaxf(mloc, s0[i]), s1[i]);  // v_max3_f32
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    // key 0 is visible to every query, so the reference is finite from the first block on
    if (__any(mloc > m + kMaxLag)) {
      const float mnew = mloc > m + kMaxLag ? mloc : m;
      const float alpha = __builtin_amdgcn_exp2f(m - mnew);
      m = mnew;
      lsum *= alpha;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        o0[i] *= alpha;
        o1[i] *= alpha;
      }
    }
    float ps[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 16; i++) {
      s0[i] = __builtin_amdgcn_exp2f(s0[i] - m);
      s1[i] = __builtin_amdgcn_exp2f(s1[i] - m);
      ps[i & 3] += s0[i];
      ps[i & 3] += s1[i];
    }
    lsum += (ps[0] + ps[1]) + (ps[2] + ps[3]);
  };
  // O^T += V^T . P^T.  Accumulator o0 owns the even head dimensions, o1 the odd
  // ones: a lane then needs V[key][2 col] and V[key][2 col + 1], one 64-bit read
  // (half as many LDS instructions as two tiles of 32 consecutive dimensions).
  typedef float f2 __attribute__((ext_vector_type(2)));
  auto accumulate = [&](int stage, const f16v& s0, const f16v& s1) {
    const float* sv = vfrag + stage * kStageFloats;
    // register i <-> key 8 (i/4) + i%4 (+ 4 half, in vfrag) of each 32-key tile
    f2 va[2], vb[2];
    va[0] = *reinterpret_cast<const f2*>(sv);
    vb[0] = *reinterpret_cast<const f2*>(sv + 32 * kRowFloats);
#pragma unroll
    for (int i = 0; i < 16; i++) {
      if (i + 1 < 16) {
        const int key = 8 * ((i + 1) >> 2) + ((i + 1) & 3);
        va[(i + 1) & 1] = *reinterpret_cast<const f2*>(sv + key * kRowFloats);
        vb[(i + 1) & 1] = *reinterpret_cast<const f2*>(sv + (32 + key) * kRowFloats);
      }
      const f2 v0 = va[i & 1], v1 = vb[i & 1];
      o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(v0.x, s0[i], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(v0.y, s0[i], o1, 0, 0, 0);
      o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(v1.x, s1[i], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(v1.y, s1[i], o1, 0, 0, 0);
#if defined(__HIP_DEVICE_COMPILE__)
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
#endif
    }
  };

  // Software pipeline over key blocks: the scores of block kb + 1 are formed before
  // the softmax of block kb, then P V of block kb follows.  Keys are therefore staged one block
  // further ahead than values:
  //   top of iteration kb   fetch K(kb + 2) into the stage K(kb) left (its scores
  //                         were formed before the last barrier), V(kb + 1) into
  //                         the stage V(kb - 1) left
  //   body                  scores of kb + 1 from K(kb + 1), softmax of kb, P V of
  //                         kb from V(kb)
  //   end                   wait for this wavefront's fetches, barrier
  // The loop is unrolled by two, so that stages are constants and the scores of consecutive blocks
  // alternate between two pairs of accumulators instead of being copied.
  f16v sa0, sa1, sb0, sb1;
  auto block = [&](auto parity, int kb, f16v& c0, f16v& c1, f16v& n0, f16v& n1) {
    constexpr int par = decltype(parity)::value;  // kb % 2
    const int key0 = kb * kKBlock;
    if (kb + 2 < nkb) fetch(false, par, key0 + 2 * kKBlock);
    if (kb + 1 < nkb) fetch(true, par ^ 1, key0 + kKBlock);
    // a wavefront whose queries all precede a key block has nothing to add there
    const bool active = !(p.causal && key0 > q_last_wave);
    const bool next_active = kb + 1 < nkb && !(p.causal && key0 + kKBlock > q_last_wave);
    if (next_active) scores(par ^ 1, n0, n1);  // implies active
    if (active) {
      normalise(key0, c0, c1);
      accumulate(par, c0, c1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's fetches have landed
    __syncthreads();
  };
  fetch(false, 0, 0);
  fetch(true, 0, 0);
  if (nkb > 1) fetch(false, 1, kKBlock);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  scores(0, sa0, sa1);
  __syncthreads();  // every wavefront has read K(0) before its stage is refilled
  int kb = 0;
  for (; kb + 2 <= nkb; kb += 2) {
    block(std::integral_constant<int, 0>{}, kb, sa0, sa1, sb0, sb1);
    block(std::integral_constant<int, 1>{}, kb + 1, sb0, sb1, sa0, sa1);
  }
  if (kb < nkb) block(std::integral_constant<int, 0>{}, kb, sa0, sa1, sb0, sb1);

  const float total = lsum + __shfl_xor(lsum, 32);
  const float inv = 1.0f / total;
  if (p.lse != nullptr && half == 0 && query < p.seq)
    p.lse[(int64_t)bh * p.seq + query] = m + __builtin_amdgcn_logf(total);  // v_log_f32: log2
  if (query < p.seq) {
    float* op = p.o + b * p.os[0] + h * p.os[1] + (int64_t)query * p.os[2];
    // register i of o0 / o1 holds head dimension 2 r / 2 r + 1, r = 8 (i/4) + 4 half + i%4:
    // four consecutive registers of both make eight consecutive dimensions
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const int d0 = 16 * g + 8 * half;
      f4 a = {o0[4 * g] * inv, o1[4 * g] * inv, o0[4 * g + 1] * inv, o1[4 * g + 1] * inv};
      f4 c = {o0[4 * g + 2] * inv, o1[4 * g + 2] * inv, o0[4 * g + 3] * inv, o1[4 * g + 3] * inv};
      if (d0 < p.head_dim) *reinterpret_cast<f4*>(op + d0) = a;
      if (d0 + 4 < p.head_dim) *reinterpret_cast<f4*>(op + d0 + 4) = c;
    }
  }
}

// ---- backward ---------------------------------------------------------------------------------
// dQ, dK, dV of O = softmax(scale Q K^T + mask) V from Q, K, V, dO and two numbers per query
// the forward pass leaves behind or that are cheap to form: L = log2 sum_j exp2(scores) (so that
// P = exp2(S - L) needs no second pass over the keys) and D = sum_d dO O = sum_j P dP.  Per tile
//   S = scale log2e Q K^T,  P = exp2(S - L),  dP = dO V^T,  dS = P (dP - D),
//   dQ += scale dS K,   dK += scale dS^T Q,   dV += P^T dO,
// and no (seq, seq) tensor is ever written.  One body serves both kinds of workgroup of the launch:
//   KEYS = false  a lane owns a QUERY (Q and dO rows in registers), key / value tiles stream
//                 through LDS, the accumulator is dQ            (the forward kernel's frame);
//   KEYS = true   a lane owns a KEY (K and V rows in registers), query / dO tiles stream, the
//                 accumulators are dK and dV; L and D of the streamed queries come with the tile.
// Either way the two score-shaped tiles are (streamed tile) . (resident rows)^T, whose accumulator
// registers are exactly the B operand of (streamed tile)^T . (scores), as in the forward kernel,
// so dS and P never leave the registers either.  Seven products in all where five are the
// minimum: S and dP are formed by both launches.
// Both streamed tiles use the key layout of the forward kernel (16-byte slots XOR row % 16); the
// 64-bit reads of the accumulation step go through the same permutation.
struct AttnBwdParams {
  const float* q;
  const float* k;
  const float* v;
  const float* dout;
  const float* lse;    // (batch * heads, seq), log2 domain, from the forward kernel
  const float* delta;  // (batch * heads, seq)
  float* dq;
  float* dk;
  float* dv;
  int64_t qs[3], ks[3], vs[3], os[3];  // dq, dk, dv are addressed like q, k, v; dout like o
  int32_t batch, heads, seq, head_dim;
  int32_t rblocks;  // blocks of 128 resident rows per head
  int32_t causal;
  float scale_log2e, scale;
};

constexpr int kBwdStageFloats = 2 * kKBlock * kRowFloats;  // two tiles of 64 rows
constexpr int kBwdStatFloats = 2 * kKBlock;                // L and D of 64 streamed queries
constexpr size_t kAttnBwdLdsBytes = 2 * (size_t)(kBwdStageFloats + kBwdStatFloats) * sizeof(float);  // 66,560 B

// D[b, h, t] = sum_d dO[b, h, t, d] O[b, h, t, d]; sixteen lanes per row.
__global__ __launch_bounds__(kBlock) void attention_delta_kernel(const float* __restrict__ o,
                                                                 const float* __restrict__ dout, int64_t s0,
                                                                 int64_t s1, int64_t s2, int32_t heads, int32_t seq,
                                                                 int32_t head_dim, int64_t rows,
                                                                 float* __restrict__ delta) {
  const int64_t gid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t row = gid >> 4;
  const int sub = (int)(gid & 15);
  float acc = 0.0f;
  if (row < rows && sub * 4 < head_dim) {
    const int64_t bh = row / seq;
    const int64_t t = row - bh * seq;
    const int64_t b = bh / heads;
    const int64_t h = bh - b * heads;
    const int64_t off = b * s0 + h * s1 + t * s2 + sub * 4;
    const f4 x = *reinterpret_cast<const f4*>(o + off);
    const f4 y = *reinterpret_cast<const f4*>(dout + off);
    acc = __builtin_fmaf(x.x, y.x, __builtin_fmaf(x.y, y.y, __builtin_fmaf(x.z, y.z, x.w * y.w)));
  }
#pragma unroll
  for (int d = 8; d > 0; d >>= 1) acc += __shfl_xor(acc, d);
  if (row < rows && sub == 0) delta[row] = acc;
}

template <bool KEYS>
__device__ __forceinline__ void attention_bwd_body(const AttnBwdParams& p, const int rank, const int bh) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* const stats = smem + 2 * kBwdStageFloats;  // [stage][L: 64, D: 64]

  // rank 0 is the longest: the last query block walks the most key tiles, the first key block the most query tiles
  const int rb = KEYS ? rank : p.rblocks - 1 - rank;
  const int b = bh / p.heads;
  const int h = bh - b * p.heads;

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int half = lane >> 5;
  const int col = lane & 31;

  const int r_first = rb * kQBlock + wave * 32;  // first resident row of this wavefront
  const int row = r_first + col;                 // this lane's query (KEYS false) or key (KEYS true)
  const int row_ld = row < p.seq ? row : p.seq - 1;

  const float* res1 = KEYS ? p.k + b * p.ks[0] + h * p.ks[1] + (int64_t)row_ld * p.ks[2]
                           : p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)row_ld * p.qs[2];
  const float* res2 = KEYS ? p.v + b * p.vs[0] + h * p.vs[1] + (int64_t)row_ld * p.vs[2]
                           : p.dout + b * p.os[0] + h * p.os[1] + (int64_t)row_ld * p.os[2];
  const float* str1 = KEYS ? p.q + b * p.qs[0] + h * p.qs[1] : p.k + b * p.ks[0] + h * p.ks[1];
  const float* str2 = KEYS ? p.dout + b * p.os[0] + h * p.os[1] : p.v + b * p.vs[0] + h * p.vs[1];
  const int64_t pitch1 = KEYS ? p.qs[2] : p.ks[2];
  const int64_t pitch2 = KEYS ? p.os[2] : p.vs[2];
  const float* lse = p.lse + (int64_t)bh * p.seq;
  const float* delta = p.delta + (int64_t)bh * p.seq;

  // resident fragments: a[4 j + r] = X[row][8 j + 4 half + r]; the first one carries scale * log2(e)
  float a1[32], a2[32];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    f4 t = {0.f, 0.f, 0.f, 0.f}, u = {0.f, 0.f, 0.f, 0.f};
    if (8 * j + 4 * half < p.head_dim) {
      t = *reinterpret_cast<const f4*>(res1 + 8 * j + 4 * half);
      u = *reinterpret_cast<const f4*>(res2 + 8 * j + 4 * half);
    }
    a1[4 * j + 0] = t.x * p.scale_log2e;
    a1[4 * j + 1] = t.y * p.scale_log2e;
    a1[4 * j + 2] = t.z * p.scale_log2e;
    a1[4 * j + 3] = t.w * p.scale_log2e;
    a2[4 * j + 0] = u.x;
    a2[4 * j + 1] = u.y;
    a2[4 * j + 2] = u.z;
    a2[4 * j + 3] = u.w;
  }
  float l_res = 0.f, d_res = 0.f;
  if (!KEYS) {
    l_res = lse[row_ld];
    d_res = delta[row_ld];
  }

  // streamed tiles of 64 rows: keys 0 .. diagonal (KEYS false), queries diagonal .. end (KEYS true)
  const int tiles = (p.seq + kKBlock - 1) / kKBlock;
  int t_begin = 0, t_end = tiles;
  if (p.causal) {
    if (KEYS) {
      t_begin = (rb * kQBlock) / kKBlock;
    } else {
      const int key_end = min(rb * kQBlock + kQBlock, p.seq);
      t_end = (key_end + kKBlock - 1) / kKBlock;
    }
  }

  // The tiles go global -> LDS through scalar-base loads (wf2_dma.h): a base per stream that is the same
  // for the workgroup, per lane the four byte offsets of its pieces in each stream.  Only a ragged last
  // tile (rows clamped to the sequence) and heads narrower than 64 compute offsets of their own.
  const uint32_t lds0 = lds_address(smem);
  const int drow = lane >> 4, dslot = lane & 15;
  uint32_t off1[4], off2[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int r = (wave * 4 + j) * 4 + drow;
    const int chunk = dslot ^ (r & 15);
    off1[j] = (uint32_t)((r * pitch1 + chunk * 4) * (int64_t)sizeof(float));
    off2[j] = (uint32_t)((r * pitch2 + chunk * 4) * (int64_t)sizeof(float));
  }
  const bool whole_rows = p.head_dim == kHeadDim;
  float stat_value = 0.f;
  auto fetch = [&](int stage, int tile) {
    const int row0 = tile * kKBlock;
    const float* b1 = str1 + (int64_t)row0 * pitch1;
    const float* b2 = str2 + (int64_t)row0 * pitch2;
    const uint32_t d1 = lds0 + (uint32_t)((stage * kBwdStageFloats + wave * 1024) * sizeof(float));
    const uint32_t d2 = d1 + (uint32_t)(kKBlock * kRowFloats * sizeof(float));
    if (whole_rows && row0 + kKBlock <= p.seq) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        dma16(d1 + j * 1024, off1[j], b1);
        dma16(d2 + j * 1024, off2[j], b2);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int r = (wave * 4 + j) * 4 + drow;
        const int chunk = dslot ^ (r & 15);
        const int last = p.seq - 1 - row0;  // >= 0
        const int64_t rr = r < last ? r : last;
        if (chunk * 4 < p.head_dim) {
          dma16(d1 + j * 1024, (uint32_t)((rr * pitch1 + chunk * 4) * (int64_t)sizeof(float)), b1);
          dma16(d2 + j * 1024, (uint32_t)((rr * pitch2 + chunk * 4) * (int64_t)sizeof(float)), b2);
        }
      }
    }
    if (KEYS && wave < 2) {  // L (wavefront 0) and D (wavefront 1) of the tile's 64 queries, parked in a register
      int srow = row0 + lane;
      srow = srow < p.seq ? srow : p.seq - 1;
      stat_value = wave == 0 ? lse[srow] : delta[srow];
    }
  };
  // ... and written to LDS only after the arithmetic of the current tile, so that waiting for that
  // load does not also wait for the tile loads issued before it
  auto publish = [&](int stage) {
    if (KEYS && wave < 2) stats[stage * kBwdStatFloats + wave * kKBlock + lane] = stat_value;
  };
  if (p.head_dim < kHeadDim) {
    for (int i = threadIdx.x; i < 2 * kBwdStageFloats / 4; i += kBlock)
      reinterpret_cast<f4*>(smem)[i] = f4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
  }

  f16v g1a = {0}, g1b = {0};  // dQ (KEYS false) or dK (KEYS true): even / odd head dimensions
  f16v g2a = {0}, g2b = {0};  // dV (KEYS true)
  typedef float f2 __attribute__((ext_vector_type(2)));

  // LDS addresses of the fragments, fixed for the kernel (stage, sub-tile and register index enter as
  // immediates, so the tile loop holds no address arithmetic):
  //   products against the resident rows   row col of the sub-tile, 16-byte slot (2 j + half) ^ (col % 16)
  //   products that accumulate gradients   row 4 half + e (e the part of the register's row that is a
  //                                        constant), floats 2 (col % 2) of slot (col / 2) ^ ((e + 4 half) % 16)
  const float* sfrag[8];
#pragma unroll
  for (int j = 0; j < 8; j++) sfrag[j] = smem + col * kRowFloats + (((2 * j + half) ^ (col & 15)) * 4);
  const float* gfrag[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    const int e = 8 * (q >> 2) + (q & 3);  // (row of register i) % 16 - 4 half, for i % 8 == q
    gfrag[q] = smem + 4 * half * kRowFloats + (((col >> 1) ^ (e + 4 * half)) * 4) + 2 * (col & 1);
  }
  const float* sthalf = stats + 4 * half;

  auto compute = [&](auto stage_c, int tile) {
    constexpr int stage = decltype(stage_c)::value;
    constexpr int so = stage * kBwdStageFloats;               // tile 1 of the stage; tile 2 follows it
    constexpr int t2 = kKBlock * kRowFloats;
    const float* st = sthalf + stage * kBwdStatFloats;
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const int s_first = tile * kKBlock + 32 * t;  // first streamed row of this 32-row sub-tile
      bool active = s_first < p.seq;
      if (p.causal) active = active && (KEYS ? s_first + 31 >= r_first : s_first <= r_first + 31);
      if (!active) continue;  // uniform over the wavefront
      f16v sc, dp;
      {
        // the fragments of contraction group j + 1 are on their way while the matrix cores work on group j
        f4 xa[2], xb[2];
        xa[0] = *reinterpret_cast<const f4*>(sfrag[0] + so + 32 * t * kRowFloats);
        xb[0] = *reinterpret_cast<const f4*>(sfrag[0] + so + t2 + 32 * t * kRowFloats);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          if (j + 1 < 8) {
            xa[(j + 1) & 1] = *reinterpret_cast<const f4*>(sfrag[j + 1] + so + 32 * t * kRowFloats);
            xb[(j + 1) & 1] = *reinterpret_cast<const f4*>(sfrag[j + 1] + so + t2 + 32 * t * kRowFloats);
          }
          const f4 x1 = xa[j & 1], x2 = xb[j & 1];
          if (j == 0) {
            const f16v zero = {0};
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.x, a1[0], zero, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.x, a2[0], zero, 0, 0, 0);
          } else {
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.x, a1[4 * j + 0], sc, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.x, a2[4 * j + 0], dp, 0, 0, 0);
          }
          sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.y, a1[4 * j + 1], sc, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.y, a2[4 * j + 1], dp, 0, 0, 0);
          sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.z, a1[4 * j + 2], sc, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.z, a2[4 * j + 2], dp, 0, 0, 0);
          sc = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.w, a1[4 * j + 3], sc, 0, 0, 0);
          dp = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.w, a2[4 * j + 3], dp, 0, 0, 0);
#if defined(__HIP_DEVICE_COMPILE__)
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 6, 0);
#endif
        }
      }
      // register i holds streamed row s_first + 8 (i/4) + 4 half + i%4 against resident row `row`.
      // Only sub-tiles on the diagonal or past the end of the sequence hold hidden pairs; the others take
      // four vector instructions per pair (subtract, exponential, subtract, multiply).
      const bool edge = s_first + 32 > p.seq ||
                        (p.causal && !(KEYS ? r_first + 31 <= s_first : s_first + 31 <= r_first));
#pragma unroll
      for (int g = 0; g < 4; g++) {
        f4 lvals = {l_res, l_res, l_res, l_res}, dvals = {d_res, d_res, d_res, d_res};
        if (KEYS) {
          lvals = *reinterpret_cast<const f4*>(st + 32 * t + 8 * g);
          dvals = *reinterpret_cast<const f4*>(st + kKBlock + 32 * t + 8 * g);
        }
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const int i = 4 * g + c;
          float pe = __builtin_amdgcn_exp2f(sc[i] - lvals[c]);
          if (edge) {
            const int srow = s_first + 8 * g + 4 * half + c;
            const int query = KEYS ? srow : row;
            const int key = KEYS ? row : srow;
            const bool visible = srow < p.seq && (!p.causal || key <= query);
            pe = visible ? pe : 0.f;
          }
          sc[i] = pe;
          dp[i] = pe * (dp[i] - dvals[c]);
        }
      }
      // (streamed tile)^T . dS and, with resident keys, (dO tile)^T . P
      {
        f2 ya[2], yb[2];
        ya[0] = *reinterpret_cast<const f2*>(gfrag[0] + so + 32 * t * kRowFloats);
        if (KEYS) yb[0] = *reinterpret_cast<const f2*>(gfrag[0] + so + t2 + 32 * t * kRowFloats);
#pragma unroll
        for (int i = 0; i < 16; i++) {
          if (i + 1 < 16) {
            // register i + 1: row 32 t + 8 ((i+1)/4) + (i+1)%4 + 4 half, address register ((i+1)/4 % 2) 4 + (i+1)%4
            const int n = i + 1;
            const int q = 4 * ((n >> 2) & 1) + (n & 3);
            const int imm = (32 * t + 8 * (n >> 2) + (n & 3)) * kRowFloats;
            ya[n & 1] = *reinterpret_cast<const f2*>(gfrag[q] + so + imm);
            if (KEYS) yb[n & 1] = *reinterpret_cast<const f2*>(gfrag[q] + so + t2 + imm);
          }
          const f2 x1 = ya[i & 1];
          g1a = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.x, dp[i], g1a, 0, 0, 0);
          g1b = __builtin_amdgcn_mfma_f32_32x32x2f32(x1.y, dp[i], g1b, 0, 0, 0);
          if (KEYS) {
            const f2 x2 = yb[i & 1];
            g2a = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.x, sc[i], g2a, 0, 0, 0);
            g2b = __builtin_amdgcn_mfma_f32_32x32x2f32(x2.y, sc[i], g2b, 0, 0, 0);
          }
#if defined(__HIP_DEVICE_COMPILE__)
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, KEYS ? 2 : 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, KEYS ? 3 : 1, 0);
#endif
        }
      }
    }
  };

  // two stages: the next tile is fetched while this one is worked on; one barrier per tile.  The loop is
  // unrolled by two so that a tile's stage is a constant.
  auto step = [&](auto stage_c, int tile) {
    constexpr int stage = decltype(stage_c)::value;
    const bool more = tile + 1 < t_end;
    if (more) fetch(stage ^ 1, tile + 1);
    compute(stage_c, tile);
    if (more) publish(stage ^ 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's fetches have landed
    __syncthreads();
  };
  fetch(0, t_begin);
  publish(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int tile = t_begin;
  for (; tile + 2 <= t_end; tile += 2) {
    step(std::integral_constant<int, 0>{}, tile);
    step(std::integral_constant<int, 1>{}, tile + 1);
  }
  if (tile < t_end) step(std::integral_constant<int, 0>{}, tile);

  auto write = [&](float* out, const f16v& ea, const f16v& eb, float factor) {
    // register i of ea / eb holds head dimension 2 r / 2 r + 1, r = 8 (i/4) + 4 half + i%4
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const int d0 = 16 * g + 8 * half;
      f4 x = {ea[4 * g] * factor, eb[4 * g] * factor, ea[4 * g + 1] * factor, eb[4 * g + 1] * factor};
      f4 y = {ea[4 * g + 2] * factor, eb[4 * g + 2] * factor, ea[4 * g + 3] * factor, eb[4 * g + 3] * factor};
      if (d0 < p.head_dim) *reinterpret_cast<f4*>(out + d0) = x;
      if (d0 + 4 < p.head_dim) *reinterpret_cast<f4*>(out + d0 + 4) = y;
    }
  };
  if (row < p.seq) {
    if (KEYS) {
      write(p.dk + b * p.ks[0] + h * p.ks[1] + (int64_t)row * p.ks[2], g1a, g1b, p.scale);
      write(p.dv + b * p.vs[0] + h * p.vs[1] + (int64_t)row * p.vs[2], g2a, g2b, 1.0f);
    } else {
      write(p.dq + b * p.qs[0] + h * p.qs[1] + (int64_t)row * p.qs[2], g1a, g1b, p.scale);
    }
  }
}

// Both kinds of workgroup in one launch, handed out by rank (longest first), keys-resident before
// queries-resident within a rank (128 against 96 MFMAs per sub-tile): 2 x 768 workgroups of very unequal
// length at (8, 12, 1024) leave a much shorter tail than two launches of 768 that each end with the compute
// units that drew the longest workgroups finishing alone.
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void attention_bwd_kernel(
    AttnBwdParams p) {  // two workgroups per CU: at most 256 registers per lane
  const int nbh = p.batch * p.heads;
  const int group = blockIdx.x / nbh;
  const int bh = blockIdx.x - group * nbh;
  // Without a mask every workgroup of a kind is as long as the others: one kind after the other then (two
  // code bodies resident side by side cost 4 % in instruction fetches and have no tail to make up for).
  const bool keys = p.causal ? (group & 1) == 0 : group < p.rblocks;
  const int rank = p.causal ? group >> 1 : (keys ? group : group - p.rblocks);
  if (keys)
    attention_bwd_body<true>(p, rank, bh);
  else
    attention_bwd_body<false>(p, rank, bh);
}

// [lo, hi) in elements touched through (batch, head, position) strides
static void extent3(const float* base, const int64_t (&s)[3], int64_t nb, int64_t nh, int64_t nt,
                    int64_t head_dim, const float** lo, const float** hi) {
  *lo = base;
  *hi = base + (nb - 1) * s[0] + (nh - 1) * s[1] + (nt - 1) * s[2] + head_dim;
}

}  // namespace wf2

using namespace wf2;

// Checks shared by the forward and the backward entry: extents, alignment, strides.  `ptrs` are the
// tensors addressed through q / k / v / o strides, in that order (nullptr entries are skipped).
static int load_attention_desc(const wf2hip_attention_desc* d, const void* const (&ptrs)[4], int64_t (&qs)[3],
                               int64_t (&ks)[3], int64_t (&vs)[3], int64_t (&os)[3]) {
  if (d->head_dim < 4 || d->head_dim > kHeadDim || d->head_dim % 4 != 0)
    return fail(WF2HIP_EUNSUPPORTED, "attention: head_dim %ld (multiples of 4 up to 64 are built)",
                (long)d->head_dim);
  if (d->batch < 0 || d->heads < 0 || d->seq < 0)
    return fail(WF2HIP_EINVAL, "attention: negative extent");
  if (d->seq > (1 << 24) || d->batch * d->heads > (1 << 20))
    return fail(WF2HIP_EUNSUPPORTED, "attention: extents beyond one launch");
  if (d->causal != 0 && d->causal != 1) return fail(WF2HIP_EINVAL, "attention: causal must be 0 or 1");
  const int64_t* strides[4] = {d->q_stride, d->k_stride, d->v_stride, d->o_stride};
  int64_t* dst[4] = {qs, ks, vs, os};
  for (int t = 0; t < 4; t++) {
    if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16 != 0)
      return fail(WF2HIP_EINVAL, "attention: operands must be 16-byte aligned");
    for (int a = 0; a < 3; a++) {
      if (strides[t][a] < 0 || strides[t][a] % 4 != 0)
        return fail(WF2HIP_EINVAL, "attention: strides must be non-negative multiples of 4 elements");
      dst[t][a] = strides[t][a];
    }
  }
  return 0;
}

WF2_API int wf2hip_attention_forward_f32(const wf2hip_attention_desc* d, const float* q, const float* k,
                                         const float* v, float* o, float* lse) {
  WF2_TRY(require_init());
  if (!d || !q || !k || !v || !o) return fail(WF2HIP_EINVAL, "attention: null argument");
  AttnParams p;
  p.q = q; p.k = k; p.v = v; p.o = o;
  p.lse = lse;
  const void* const ptrs[4] = {q, k, v, o};
  WF2_TRY(load_attention_desc(d, ptrs, p.qs, p.ks, p.vs, p.os));
  if (d->batch == 0 || d->heads == 0 || d->seq == 0) return 0;
  // the output must be a dense-enough set of rows of its own: no two (batch, head,
  // position) triples may share storage, and it may not alias an input
  if (p.os[2] < d->head_dim && d->seq > 1) return fail(WF2HIP_EINVAL, "attention: output rows overlap");
  const float *olo, *ohi;
  extent3(o, p.os, d->batch, d->heads, d->seq, d->head_dim, &olo, &ohi);
  const float* ins[3] = {q, k, v};
  const int64_t(*ist[3])[3] = {&p.qs, &p.ks, &p.vs};
  for (int t = 0; t < 3; t++) {
    const float *lo, *hi;
    extent3(ins[t], *ist[t], d->batch, d->heads, d->seq, d->head_dim, &lo, &hi);
    if (lo < ohi && olo < hi) return fail(WF2HIP_EOVERLAP, "attention: output overlaps an input");
  }
  if (lse != nullptr) {
    const float* llo = lse;
    const float* lhi = lse + d->batch * d->heads * d->seq;
    if (llo < ohi && olo < lhi) return fail(WF2HIP_EOVERLAP, "attention: the row statistics overlap the output");
  }
  p.batch = (int32_t)d->batch;
  p.heads = (int32_t)d->heads;
  p.seq = (int32_t)d->seq;
  p.head_dim = (int32_t)d->head_dim;
  p.qblocks = (int32_t)ceil_div(d->seq, kQBlock);
  p.causal = d->causal;
  p.scale_log2e = d->scale * 1.44269504088896340736f;
  const int64_t blocks = (int64_t)p.qblocks * p.batch * p.heads;
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "attention: too many workgroups");
  static bool configured = false;
  if (!configured) {
    WF2_TRY(check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)kAttnLdsBytes),
                      "hipFuncSetAttribute(attention_kernel)"));
    configured = true;
  }
  attention_kernel<<<(uint32_t)blocks, kBlock, kAttnLdsBytes, rt().stream>>>(p);
  return after_launch("attention_kernel");
}

WF2_API int wf2hip_attention_f32(const wf2hip_attention_desc* d, const float* q, const float* k,
                                 const float* v, float* o) {
  return wf2hip_attention_forward_f32(d, q, k, v, o, nullptr);
}

WF2_API int wf2hip_attention_backward_f32(const wf2hip_attention_desc* d, const float* q, const float* k,
                                          const float* v, const float* o, const float* dout, const float* lse,
                                          float* dq, float* dk, float* dv) {
  WF2_TRY(require_init());
  if (!d || !q || !k || !v || !o || !dout || !lse || !dq || !dk || !dv)
    return fail(WF2HIP_EINVAL, "attention backward: null argument");
  AttnBwdParams p;
  p.q = q; p.k = k; p.v = v; p.dout = dout; p.lse = lse;
  p.dq = dq; p.dk = dk; p.dv = dv;
  const void* const ptrs[4] = {q, k, v, o};
  WF2_TRY(load_attention_desc(d, ptrs, p.qs, p.ks, p.vs, p.os));
  const void* const more[6] = {dout, dq, dk, dv, lse, nullptr};
  for (int t = 0; t < 4; t++)
    if (reinterpret_cast<uintptr_t>(more[t]) % 16 != 0)
      return fail(WF2HIP_EINVAL, "attention backward: operands must be 16-byte aligned");
  if (d->batch == 0 || d->heads == 0 || d->seq == 0) return 0;
  // gradients are addressed like the tensors they belong to; their rows may not share storage,
  // and none of them may overlap anything that is read
  const float* outs[3] = {dq, dk, dv};
  const int64_t(*ost[3])[3] = {&p.qs, &p.ks, &p.vs};
  const float* ins[5] = {q, k, v, o, dout};
  const int64_t(*ist[5])[3] = {&p.qs, &p.ks, &p.vs, &p.os, &p.os};
  for (int t = 0; t < 3; t++) {
    if ((*ost[t])[2] < d->head_dim && d->seq > 1)
      return fail(WF2HIP_EINVAL, "attention backward: gradient rows overlap");
    const float *olo, *ohi;
    extent3(outs[t], *ost[t], d->batch, d->heads, d->seq, d->head_dim, &olo, &ohi);
    for (int u = 0; u < 5; u++) {
      const float *lo, *hi;
      extent3(ins[u], *ist[u], d->batch, d->heads, d->seq, d->head_dim, &lo, &hi);
      if (lo < ohi && olo < hi) return fail(WF2HIP_EOVERLAP, "attention backward: a gradient overlaps an input");
    }
    const float* lhi = lse + d->batch * d->heads * d->seq;
    if (lse < ohi && olo < lhi) return fail(WF2HIP_EOVERLAP, "attention backward: a gradient overlaps the row statistics");
    for (int u = t + 1; u < 3; u++)
      if (outs[t] == outs[u]) return fail(WF2HIP_EOVERLAP, "attention backward: two gradients share storage");
  }
  p.batch = (int32_t)d->batch;
  p.heads = (int32_t)d->heads;
  p.seq = (int32_t)d->seq;
  p.head_dim = (int32_t)d->head_dim;
  p.rblocks = (int32_t)ceil_div(d->seq, kQBlock);
  p.causal = d->causal;
  p.scale = d->scale;
  p.scale_log2e = d->scale * 1.44269504088896340736f;
  const int64_t blocks = (int64_t)p.rblocks * p.batch * p.heads;
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "attention backward: too many workgroups");
  if (2 * blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "attention backward: too many workgroups");
  static bool configured = false;
  if (!configured) {
    WF2_TRY(check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_bwd_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kAttnBwdLdsBytes),
                      "hipFuncSetAttribute(attention_bwd_kernel)"));
    configured = true;
  }
  const int64_t rows = d->batch * d->heads * d->seq;
  if (ceil_div(rows * 16, kBlock) >= ((int64_t)1 << 31))
    return fail(WF2HIP_EUNSUPPORTED, "attention backward: too many rows for one launch");
  void* delta = nullptr;
  WF2_TRY(wf2hip_malloc_uninitialized(&delta, (size_t)rows * sizeof(float)));
  p.delta = static_cast<const float*>(delta);
  hipStream_t st = rt().stream;
  attention_delta_kernel<<<(uint32_t)ceil_div(rows * 16, kBlock), kBlock, 0, st>>>(
      o, dout, p.os[0], p.os[1], p.os[2], p.heads, p.seq, p.head_dim, rows, static_cast<float*>(delta));
  int rc = after_launch("attention_delta_kernel");
  if (rc == 0) {
    attention_bwd_kernel<<<(uint32_t)(2 * blocks), kBlock, kAttnBwdLdsBytes, st>>>(p);
    rc = after_launch("attention_bwd_kernel");
  }
  (void)wf2hip_free(delta);  // stream order keeps it alive for the launches above
  return rc;
}
