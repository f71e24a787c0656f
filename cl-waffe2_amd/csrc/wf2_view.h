// wf2_view.h -- host-side normalisation of a two-tensor iteration space.
//
// cl-waffe2 hands a kernel per-axis (offset, size, stride) triplets
// (ViewInstruction, source/vm/generic-tensor/view.lisp:50-69) and wraps the
// 1-D kernel in host loops (call-with-view.lisp:112-229).  Here the whole
// space arrives in one wf2hip_view2 and is reduced to the fewest axes that
// describe the same address pattern, so that one launch covers the node.
#pragma once

#include <stdint.h>
#include <initializer_list>

#include "wf2_common.h"

namespace wf2 {

struct Space {
  int rank = 0;                       // >= 1 after normalise() unless empty
  int64_t shape[WF2HIP_MAX_RANK];     // outermost first
  int64_t sa[WF2HIP_MAX_RANK];
  int64_t sb[WF2HIP_MAX_RANK];
  int64_t off_a = 0, off_b = 0;
  int64_t total = 0;
};

// Validates the descriptor and copies it.  total == 0 means nothing to do.
inline int load_space(const wf2hip_view2* v, Space* s) {
  if (!v) return fail(WF2HIP_EINVAL, "null view descriptor");
  if (v->rank < 1 || v->rank > WF2HIP_MAX_RANK)
    return fail(WF2HIP_EINVAL, "view rank %d outside 1..%d", v->rank, WF2HIP_MAX_RANK);
  s->rank = v->rank;
  s->total = 1;
  for (int r = 0; r < v->rank; r++) {
    if (v->shape[r] < 0) return fail(WF2HIP_EINVAL, "negative extent on axis %d", r);
    s->shape[r] = v->shape[r];
    s->sa[r] = v->stride_a[r];
    s->sb[r] = v->stride_b[r];
    s->total *= v->shape[r];
  }
  if (v->off_a < 0 || v->off_b < 0) return fail(WF2HIP_EINVAL, "negative offset");
  s->off_a = v->off_a;
  s->off_b = v->off_b;
  return 0;
}

// Drops extent-1 axes and merges neighbours that are one linear run for both
// tensors (stride_outer == stride_inner * extent_inner, which also merges
// 0/0 broadcast pairs).
inline void normalise(Space* s) {
  int w = 0;
  for (int r = 0; r < s->rank; r++) {
    if (s->shape[r] == 1) continue;
    s->shape[w] = s->shape[r];
    s->sa[w] = s->sa[r];
    s->sb[w] = s->sb[r];
    w++;
  }
  if (w == 0) {  // a single element
    s->shape[0] = 1;
    s->sa[0] = 0;
    s->sb[0] = 0;
    w = 1;
  }
  s->rank = w;
  int out = 0;
  for (int r = 1; r < s->rank; r++) {
    bool merge = s->sa[out] == s->sa[r] * s->shape[r] && s->sb[out] == s->sb[r] * s->shape[r];
    if (merge) {
      s->shape[out] *= s->shape[r];
      s->sa[out] = s->sa[r];
      s->sb[out] = s->sb[r];
    } else {
      out++;
      s->shape[out] = s->shape[r];
      s->sa[out] = s->sa[r];
      s->sb[out] = s->sb[r];
    }
  }
  s->rank = out + 1;
}

// Lowest and highest element offset a strided window touches.
inline void extent_of(const Space& s, const int64_t* stride, int64_t off, int64_t* lo,
                      int64_t* hi) {
  *lo = off;
  *hi = off;
  for (int r = 0; r < s.rank; r++) {
    int64_t span = stride[r] * (s.shape[r] - 1);
    if (span >= 0)
      *hi += span;
    else
      *lo += span;
  }
}

// True when the two windows may touch a common element without being the
// same element-for-element mapping.  `delta` = (base of b - base of a) in
// elements; the windows start at off_a and delta + off_b.
inline bool hazardous_overlap_at(const Space& s, int64_t delta) {
  int64_t alo, ahi, blo, bhi;
  extent_of(s, s.sa, s.off_a, &alo, &ahi);
  extent_of(s, s.sb, s.off_b + delta, &blo, &bhi);
  if (ahi < blo || bhi < alo) return false;
  // Interleaved lattices (the even against the odd elements of one buffer): every
  // address of a window is its start plus a multiple of g = gcd of all strides of
  // both windows, so starts that differ modulo g never meet.
  int64_t g = 0;
  for (int r = 0; r < s.rank; r++) {
    if (s.shape[r] <= 1) continue;
    for (int64_t v : {s.sa[r], s.sb[r]}) {
      if (v < 0) v = -v;
      while (v != 0) {
        int64_t t = g % v;
        g = v;
        v = t;
      }
    }
  }
  const int64_t starts = s.off_a - (s.off_b + delta);
  if (g > 1 && starts % g != 0) return false;
  bool same_strides = true;
  for (int r = 0; r < s.rank; r++)
    if (s.sa[r] != s.sb[r]) same_strides = false;
  if (!same_strides) return true;
  if (starts == 0) return false;  // identical mapping: every element depends on itself only
  // One window is the other moved by `starts` elements (x[:, :h] against x[:, h:]): they
  // share an element iff starts = sum k_r stride_r with |k_r| < extent_r.  With nested
  // strides (each larger than everything the axes below it span) only the two
  // neighbouring multiples of a stride can work at each level, so the search is exact;
  // otherwise stay on the safe side.
  int order[WF2HIP_MAX_RANK];
  int n = 0;
  for (int r = 0; r < s.rank; r++)
    if (s.shape[r] > 1 && s.sa[r] != 0) order[n++] = r;
  auto mag = [&](int r) { return s.sa[r] < 0 ? -s.sa[r] : s.sa[r]; };
  for (int i = 1; i < n; i++)
    for (int j = i; j > 0 && mag(order[j]) > mag(order[j - 1]); j--) {
      const int t = order[j];
      order[j] = order[j - 1];
      order[j - 1] = t;
    }
  int64_t below = 0;
  for (int i = n - 1; i >= 0; i--) {
    if (mag(order[i]) <= below) return true;  // not nested
    below += mag(order[i]) * (s.shape[order[i]] - 1);
  }
  struct Search {
    const Space& s;
    const int* order;
    int n;
    bool hits(int64_t rem, int level) const {
      if (level == n) return rem == 0;
      const int r = order[level];
      const int64_t stride = s.sa[r];
      int64_t q = rem / stride;  // truncated; the neighbours q - 1, q, q + 1 cover floor and ceiling
      for (int64_t k = q - 1; k <= q + 1; k++) {
        const int64_t a = k < 0 ? -k : k;
        if (a < s.shape[r] && hits(rem - k * stride, level + 1)) return true;
      }
      return false;
    }
  };
  return Search{s, order, n}.hits(starts, 0);
}

inline bool hazardous_overlap(const Space& s, const float* a, const float* b) {
  return hazardous_overlap_at(s, b - a);
}

inline bool has_broadcast_axis(const Space& s, const int64_t* stride) {
  for (int r = 0; r < s.rank; r++)
    if (stride[r] == 0 && s.shape[r] > 1) return true;
  return false;
}


// ---- three tensors over one iteration space (compare: a = X, b = Y, c = OUT) ----
struct Space3 {
  int rank = 0;
  int64_t shape[WF2HIP_MAX_RANK];
  int64_t sa[WF2HIP_MAX_RANK], sb[WF2HIP_MAX_RANK], sc[WF2HIP_MAX_RANK];
  int64_t off_a = 0, off_b = 0, off_c = 0;
  int64_t total = 0;
};

inline void normalise3(Space3* s) {
  int w = 0;
  for (int r = 0; r < s->rank; r++) {
    if (s->shape[r] == 1) continue;
    s->shape[w] = s->shape[r];
    s->sa[w] = s->sa[r];
    s->sb[w] = s->sb[r];
    s->sc[w] = s->sc[r];
    w++;
  }
  if (w == 0) {
    s->shape[0] = 1;
    s->sa[0] = s->sb[0] = s->sc[0] = 0;
    w = 1;
  }
  s->rank = w;
  int out = 0;
  for (int r = 1; r < s->rank; r++) {
    const bool merge = s->sa[out] == s->sa[r] * s->shape[r] && s->sb[out] == s->sb[r] * s->shape[r] &&
                       s->sc[out] == s->sc[r] * s->shape[r];
    if (merge) {
      s->shape[out] *= s->shape[r];
    } else {
      out++;
      s->shape[out] = s->shape[r];
    }
    s->sa[out] = s->sa[r];
    s->sb[out] = s->sb[r];
    s->sc[out] = s->sc[r];
  }
  s->rank = out + 1;
  s->total = 1;
  for (int r = 0; r < s->rank; r++) s->total *= s->shape[r];
}

// lowest / highest element a strided window touches
inline void span_of(const Space3& s, const int64_t* stride, int64_t off, int64_t* lo, int64_t* hi) {
  *lo = *hi = off;
  for (int r = 0; r < s.rank; r++) {
    const int64_t span = stride[r] * (s.shape[r] - 1);
    if (span >= 0)
      *hi += span;
    else
      *lo += span;
  }
}

// `out` may coincide with an input element for element (in-place compare);
// any other overlap makes the result depend on the order of the writes
template <class T>
inline bool hazardous3(const Space3& s, const T* out, const int64_t* sin, int64_t off_in, const T* in) {
  int64_t olo, ohi, ilo, ihi;
  span_of(s, s.sc, s.off_c, &olo, &ohi);
  span_of(s, sin, off_in, &ilo, &ihi);
  if (out + ohi < in + ilo || in + ihi < out + olo) return false;
  if (out + s.off_c != in + off_in) return true;
  for (int r = 0; r < s.rank; r++)
    if (s.sc[r] != sin[r]) return true;
  return false;
}

inline int load_space3(const wf2hip_view3* v, Space3* s) {
  if (!v) return fail(WF2HIP_EINVAL, "null view descriptor");
  if (v->rank < 1 || v->rank > WF2HIP_MAX_RANK)
    return fail(WF2HIP_EINVAL, "view rank %d outside 1..%d", v->rank, WF2HIP_MAX_RANK);
  s->rank = v->rank;
  s->total = 1;
  for (int r = 0; r < v->rank; r++) {
    if (v->shape[r] < 0) return fail(WF2HIP_EINVAL, "negative extent on axis %d", r);
    s->shape[r] = v->shape[r];
    s->sa[r] = v->stride_a[r];
    s->sb[r] = v->stride_b[r];
    s->sc[r] = v->stride_c[r];
    s->total *= v->shape[r];
  }
  if (v->off_a < 0 || v->off_b < 0 || v->off_c < 0) return fail(WF2HIP_EINVAL, "negative offset");
  s->off_a = v->off_a;
  s->off_b = v->off_b;
  s->off_c = v->off_c;
  return 0;
}


}  // namespace wf2
