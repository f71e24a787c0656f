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
#include "wf2_common.h"

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
};

__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void attention_kernel(
    AttnParams p) {  // two workgroups per CU: at most 256 registers per lane
  extern __shared__ __attribute__((aligned(16))) float smem[];
  auto lds_k = [&](int stage) { return smem + stage * kStageFloats; };
  auto lds_v = [&](int stage) { return smem + stage * kStageFloats + kKBlock * kRowFloats; };

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

  const int q_first = qb * kQBlock + wave * 32;  // first query of this wavefront
  const int query = q_first + col;
  const int query_ld = query < p.seq ? query : p.seq - 1;

  const float* qp = p.q + b * p.qs[0] + h * p.qs[1] + (int64_t)query_ld * p.qs[2];
  const float* kp = p.k + b * p.ks[0] + h * p.ks[1];
  const float* vp = p.v + b * p.vs[0] + h * p.vs[1];
  (void)kp;
  (void)vp;  // only the device pass reads them (global -> LDS builtin)

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
  float m = -INFINITY;  // running maximum (log2 domain), shared by both halves
  float lsum = 0.f;     // running sum of this half's keys

  // Key / value blocks go global -> LDS without passing through registers: one
  // instruction moves 64 x 16 bytes into 1 KB of LDS (four rows).  The 16-byte
  // slots of a row are permuted through the address each lane reads from:
  //   keys    slot = chunk ^ (row % 16), so that the 128-bit fragment reads of 16
  //           consecutive rows cover all 64 banks;
  //   values  the two 128-byte halves of a row are swapped when (row / 4) is odd:
  //           the half-waves read rows 4 apart and then hit different banks.
  // Rows beyond the sequence are clamped (their scores are masked later); chunks
  // beyond head_dim are not loaded and stay zero from the clear below.
  auto fetch = [&](bool values, int stage, int key0) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int q4 = wave * 4 + j;
      const int row = q4 * 4 + (lane >> 4);
      const int slot = lane & 15;
      int key = key0 + row;
      key = key < p.seq ? key : p.seq - 1;
      const int chunk = values ? slot ^ (((row >> 2) & 1) << 3) : slot ^ (row & 15);
      const float* src = values ? vp + (int64_t)key * p.vs[2] : kp + (int64_t)key * p.ks[2];
      float* dst = (values ? lds_v(stage) : lds_k(stage)) + q4 * 256;
      if (chunk * 4 < p.head_dim) __builtin_amdgcn_global_load_lds(src + chunk * 4, dst, 16, 0, 0);
    }
#endif
  };
  if (p.head_dim < kHeadDim) {
    for (int i = threadIdx.x; i < 2 * kStageFloats / 4; i += kBlock)
      reinterpret_cast<f4*>(smem)[i] = f4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
  }

  const int kswz = col & 15;     // rows col and 32 + col share it
  const int vswap = half << 5;   // keys read by the upper half-wave have (key / 4) odd

  // S^T of one key block: two 32 x 32 tiles (keys 0-31 and 32-63 of the block)
  auto scores = [&](const float* sk, f16v& s0, f16v& s1) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      s0[i] = 0.f;
      s1[i] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int slot = ((2 * j + half) ^ kswz) * 4;
      f4 k0 = *reinterpret_cast<const f4*>(sk + col * kRowFloats + slot);
      f4 k1 = *reinterpret_cast<const f4*>(sk + (32 + col) * kRowFloats + slot);
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.x, qf[4 * j + 0], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.x, qf[4 * j + 0], s1, 0, 0, 0);
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.y, qf[4 * j + 1], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.y, qf[4 * j + 1], s1, 0, 0, 0);
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.z, qf[4 * j + 2], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.z, qf[4 * j + 2], s1, 0, 0, 0);
      s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.w, qf[4 * j + 3], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.w, qf[4 * j + 3], s1, 0, 0, 0);
    }
  };
  // masks, running softmax statistics, P = exp2(S - max) in place
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
    float mloc = s0[0];
#pragma unroll
    for (int i = 1; i < 16; i++) mloc = fmaxf(mloc, s0[i]);
#pragma unroll
    for (int i = 0; i < 16; i++) mloc = fmaxf(mloc, s1[i]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    const float mnew = fmaxf(m, mloc);
    // key 0 is visible to every query, so mnew is finite from the first block on
    const float alpha = __builtin_amdgcn_exp2f(m - mnew);
    m = mnew;
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      s0[i] = __builtin_amdgcn_exp2f(s0[i] - mnew);
      s1[i] = __builtin_amdgcn_exp2f(s1[i] - mnew);
      psum += s0[i] + s1[i];
    }
    lsum = lsum * alpha + psum;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      o0[i] *= alpha;
      o1[i] *= alpha;
    }
  };
  // O^T += V^T . P^T.  Accumulator o0 owns the even head dimensions, o1 the odd
  // ones: a lane then needs V[key][2 col] and V[key][2 col + 1], one 64-bit read
  // (half as many LDS instructions as two tiles of 32 consecutive dimensions).
  typedef float f2 __attribute__((ext_vector_type(2)));
  auto accumulate = [&](const float* sv, const f16v& s0, const f16v& s1) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int key = 8 * (i >> 2) + 4 * half + (i & 3);
      const f2 v0 = *reinterpret_cast<const f2*>(sv + key * kRowFloats + ((2 * col) ^ vswap));
      const f2 v1 = *reinterpret_cast<const f2*>(sv + (32 + key) * kRowFloats + ((2 * col) ^ vswap));
      o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(v0.x, s0[i], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(v0.y, s0[i], o1, 0, 0, 0);
      o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(v1.x, s1[i], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(v1.y, s1[i], o1, 0, 0, 0);
    }
  };

  // Software pipeline over key blocks: while the vector units work through the
  // softmax of block kb, the matrix cores already form the scores of block
  // kb + 1; then P V of block kb follows.  Keys are therefore staged one block
  // further ahead than values:
  //   top of iteration kb   fetch K(kb + 2) into the stage K(kb) left (its scores
  //                         were formed before the last barrier), V(kb + 1) into
  //                         the stage V(kb - 1) left
  //   body                  scores of kb + 1 from K(kb + 1), softmax of kb, P V of
  //                         kb from V(kb)
  //   end                   wait for this wavefront's fetches, barrier
  fetch(false, 0, 0);
  fetch(true, 0, 0);
  if (nkb > 1) fetch(false, 1, kKBlock);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  f16v n0, n1;  // scores of the next block
  scores(lds_k(0), n0, n1);
  __syncthreads();  // every wavefront has read K(0) before its stage is refilled

  for (int kb = 0; kb < nkb; kb++) {
    const int key0 = kb * kKBlock;
    if (kb + 2 < nkb) fetch(false, kb & 1, key0 + 2 * kKBlock);
    if (kb + 1 < nkb) fetch(true, (kb + 1) & 1, key0 + kKBlock);
    // a wavefront whose queries all precede a key block has nothing to add there
    const bool active = !(p.causal && key0 > q_last_wave);
    const bool next_active = kb + 1 < nkb && !(p.causal && key0 + kKBlock > q_last_wave);
    f16v s0 = n0, s1 = n1;
    if (next_active) {  // implies active
      scores(lds_k((kb + 1) & 1), n0, n1);
      normalise(key0, s0, s1);
      accumulate(lds_v(kb & 1), s0, s1);
    } else if (active) {
      normalise(key0, s0, s1);
      accumulate(lds_v(kb & 1), s0, s1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's fetches have landed
    __syncthreads();
  }

  const float total = lsum + __shfl_xor(lsum, 32);
  const float inv = 1.0f / total;
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

// [lo, hi) in elements touched through (batch, head, position) strides
static void extent3(const float* base, const int64_t (&s)[3], int64_t nb, int64_t nh, int64_t nt,
                    int64_t head_dim, const float** lo, const float** hi) {
  *lo = base;
  *hi = base + (nb - 1) * s[0] + (nh - 1) * s[1] + (nt - 1) * s[2] + head_dim;
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_attention_f32(const wf2hip_attention_desc* d, const float* q, const float* k,
                                 const float* v, float* o) {
  WF2_TRY(require_init());
  if (!d || !q || !k || !v || !o) return fail(WF2HIP_EINVAL, "attention: null argument");
  if (d->head_dim < 4 || d->head_dim > kHeadDim || d->head_dim % 4 != 0)
    return fail(WF2HIP_EUNSUPPORTED, "attention: head_dim %ld (multiples of 4 up to 64 are built)",
                (long)d->head_dim);
  if (d->batch < 0 || d->heads < 0 || d->seq < 0)
    return fail(WF2HIP_EINVAL, "attention: negative extent");
  if (d->batch == 0 || d->heads == 0 || d->seq == 0) return 0;
  if (d->seq > (1 << 24) || d->batch * d->heads > (1 << 20))
    return fail(WF2HIP_EUNSUPPORTED, "attention: extents beyond one launch");
  if (d->causal != 0 && d->causal != 1) return fail(WF2HIP_EINVAL, "attention: causal must be 0 or 1");
  AttnParams p;
  p.q = q; p.k = k; p.v = v; p.o = o;
  const int64_t* strides[4] = {d->q_stride, d->k_stride, d->v_stride, d->o_stride};
  int64_t* dst[4] = {p.qs, p.ks, p.vs, p.os};
  const void* ptrs[4] = {q, k, v, o};
  for (int t = 0; t < 4; t++) {
    if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16 != 0)
      return fail(WF2HIP_EINVAL, "attention: operands must be 16-byte aligned");
    for (int a = 0; a < 3; a++) {
      if (strides[t][a] < 0 || strides[t][a] % 4 != 0)
        return fail(WF2HIP_EINVAL, "attention: strides must be non-negative multiples of 4 elements");
      dst[t][a] = strides[t][a];
    }
  }
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
