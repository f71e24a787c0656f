// embedding.hip -- token + position embedding lookup of the GPT-2 example.
//
// examples/gpt-2/utils.lisp:19-110 defines GPT2PositionalEmbedding for LispTensor only:
// per (sentence, position) it zeroes the output row, then adds WTE[round(ctx)] and WPE[position]
// to it with two waffe2_sadd calls of embedding-size elements, i.e.
//   out[n, t, :] = (0 + wte[round(ctx[n, t]), :]) + wpe[t, :]
// in binary32 (the sum with 0 is exact).  One launch here: a gather of rows, 4 bytes written per
// element (HBM-bound; the tables are small and stay in cache).  Token ids arrive as floats
// (the example feeds :float tensors) and are rounded to nearest, ties to even, as Common Lisp's
// ROUND does; ids outside the table are clamped to its ends (the reference reads out of bounds).
#include "wf2_common.h"

namespace wf2 {

typedef float f4 __attribute__((ext_vector_type(4)));

template <bool VEC>
__global__ __launch_bounds__(kBlock) void embedding_add_kernel(const float* __restrict__ ctx,
                                                               const float* __restrict__ wte,
                                                               const float* __restrict__ wpe,
                                                               float* __restrict__ out, int64_t rows, int64_t seq,
                                                               int64_t dim, int64_t vocab) {
  const int64_t per_row = VEC ? dim / 4 : dim;
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= rows * per_row) return;
  const int64_t row = i / per_row;
  const int64_t c = (i - row * per_row) * (VEC ? 4 : 1);
  const float id = ctx[row];
  const float nearest = __builtin_rintf(id);  // ties to even
  const int64_t token = !(nearest >= 0.0f) ? 0 : (nearest >= (float)vocab ? vocab - 1 : (int64_t)nearest);  // NaN -> 0
  const int64_t pos = row % seq;
  if (VEC) {
    const f4 a = *reinterpret_cast<const f4*>(wte + token * dim + c);
    const f4 b = *reinterpret_cast<const f4*>(wpe + pos * dim + c);
    *reinterpret_cast<f4*>(out + row * dim + c) = a + b;
  } else {
    out[row * dim + c] = wte[token * dim + c] + wpe[pos * dim + c];
  }
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_embedding_add_f32(long rows, long seq, long dim, const float* ctx, const float* wte,
                                     long vocab, const float* wpe, long n_ctx, float* out) {
  WF2_TRY(require_init());
  if (rows < 0 || seq < 0 || dim < 0 || vocab < 0 || n_ctx < 0) return fail(WF2HIP_EINVAL, "embedding: negative extent");
  if (rows == 0 || dim == 0) return 0;
  if (!ctx || !wte || !wpe || !out) return fail(WF2HIP_EINVAL, "embedding: null pointer");
  if (seq < 1 || rows % seq != 0) return fail(WF2HIP_EINVAL, "embedding: rows %ld is not a multiple of the sentence length %ld", rows, seq);
  if (seq > n_ctx) return fail(WF2HIP_EINVAL, "embedding: sentence length %ld beyond the %ld positions of wpe", seq, n_ctx);
  if (vocab < 1) return fail(WF2HIP_EINVAL, "embedding: empty token table");
  const float* olo = out;
  const float* ohi = out + (int64_t)rows * dim;
  if ((wte < ohi && olo < wte + (int64_t)vocab * dim) || (wpe < ohi && olo < wpe + (int64_t)n_ctx * dim) ||
      (ctx < ohi && olo < ctx + rows))
    return fail(WF2HIP_EOVERLAP, "embedding: the output overlaps an input");
  const bool vec = dim % 4 == 0 && ((uintptr_t)wte | (uintptr_t)wpe | (uintptr_t)out) % 16 == 0;
  const int64_t items = (int64_t)rows * (vec ? dim / 4 : dim);
  const int64_t blocks = ceil_div(items, kBlock);
  if (blocks >= ((int64_t)1 << 31)) return fail(WF2HIP_EUNSUPPORTED, "embedding: too many elements for one launch");
  if (vec)
    embedding_add_kernel<true><<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(ctx, wte, wpe, out, rows, seq, dim, vocab);
  else
    embedding_add_kernel<false><<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(ctx, wte, wpe, out, rows, seq, dim, vocab);
  return after_launch("embedding_add_kernel");
}
