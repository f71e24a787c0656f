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
// im2col: one thread per written element of col, gathers from im.
// col2im: im is the sum, over kh then kw ascending (the reference's order of
// accumulation, so the binary32 result is identical), of the col elements that
// land on it: one thread per element of im, no atomics.
// HBM-bound: about 4 (k-h k-w + 1) bytes per image element.
#include "wf2_common.h"

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
  col2im_kernel<<<(uint32_t)blocks, kBlock, 0, rt().stream>>>(p);
  return after_launch("col2im_kernel");
}
