// Host-side tensor layout algebra: size/stride collapsing, overlap test,
// index-width selection and the joint iteration space of several operands.
// Pure C++ (no HIP) so it can be exercised on a machine without a GPU.
//
// Behaviour follows lib/THC/THCTensorInfo.cuh:76-278 (collapse, linear index
// -> offset in logical row-major order) and lib/THC/THCTensorTypeUtils.cu
// :164-245 (overlap test, 32-bit eligibility); the code is written for this
// engine, whose kernels want a *joint* description of all operands.
#pragma once
#include <algorithm>
#include <cstdint>
#include <utility>

namespace thc {

constexpr int kMaxDims = 25;  // lib/THC/THCTensorInfo.cuh:10

struct Layout {
  int dims = 0;
  int64_t size[kMaxDims];
  int64_t stride[kMaxDims];

  int64_t numel() const {
    if (dims == 0) return 0;
    int64_t n = 1;
    for (int i = 0; i < dims; ++i) n *= size[i];
    return n;
  }
  bool contiguous() const { return dims == 1 && stride[0] == 1; }
};

inline Layout make_layout(int nDim, const long* size, const long* stride) {
  Layout l;
  l.dims = nDim;
  for (int i = 0; i < nDim; ++i) {
    l.size[i] = size[i];
    l.stride[i] = stride[i];
  }
  return l;
}

// Merge runs of dims that address memory like one longer dim; drop size-1
// dims. `excludeDim` (if >= 0) is kept as it is, never merged with either
// neighbour. Returns the new position of excludeDim (or -1 / 0 as the
// reference does for the degenerate cases).
inline int collapse(Layout& l, int excludeDim = -1) {
  if (l.dims == 0) return -1;
  int64_t ns[kMaxDims], nt[kMaxDims];
  int n = 0;            // dims emitted so far, innermost first
  int where = -1;       // emitted slot of excludeDim
  bool open = false;    // is slot n-1 allowed to absorb an outer dim?
  for (int i = l.dims - 1; i >= 0; --i) {
    const bool excl = (i == excludeDim);
    if (!excl && l.size[i] == 1) continue;
    if (!excl && open && l.stride[i] == ns[n - 1] * nt[n - 1]) {
      ns[n - 1] *= l.size[i];
      continue;
    }
    ns[n] = l.size[i];
    nt[n] = l.stride[i];
    if (excl) where = n;
    open = !excl;
    ++n;
  }
  if (n == 0) {  // every dim had size 1: a single point
    l.dims = 1;
    l.size[0] = 1;
    l.stride[0] = 1;
    return 0;
  }
  l.dims = n;
  for (int i = 0; i < n; ++i) {
    l.size[i] = ns[n - 1 - i];
    l.stride[i] = nt[n - 1 - i];
  }
  return where < 0 ? -1 : n - 1 - where;
}

// True when two distinct logical indices can address the same element.
inline bool overlapping(const Layout& l) {
  std::pair<int64_t, int64_t> d[kMaxDims];  // (stride, size)
  int n = 0;
  for (int i = 0; i < l.dims; ++i)
    if (l.size[i] > 1) d[n++] = {l.stride[i], l.size[i]};
  if (n == 0) return false;
  std::sort(d, d + n);  // ascending stride: d[0] is the innermost
  if (d[0].first < 1) return true;
  for (int i = 1; i < n; ++i)
    if (d[i].first < d[i - 1].first * d[i - 1].second) return true;
  return false;
}

// Offset of the element with logical (row-major) linear index `lin`.
inline int64_t linear_to_offset(const Layout& l, int64_t lin) {
  int64_t off = 0;
  for (int i = l.dims - 1; i >= 0; --i) {
    off += (lin % l.size[i]) * l.stride[i];
    lin /= l.size[i];
  }
  return off;
}

inline int64_t last_offset(const Layout& l) {
  int64_t off = 0;
  for (int i = 0; i < l.dims; ++i) off += (l.size[i] - 1) * l.stride[i];
  return off;
}

// 32-bit index arithmetic is used when both the element count and the
// largest element offset stay below 2^31, so that every intermediate of the
// signed/unsigned kernel arithmetic (including grid-stride increments and the
// multiply-shift division) is exact. The reference draws the line at
// UINT_MAX (THCTensorTypeUtils.cu:221-245) and lets `linearIndex += gridDim.x
// * blockDim.x` wrap; this engine switches one bit earlier.
constexpr int64_t kIndex32Limit = int64_t(1) << 31;
inline bool fits_32bit(const Layout& l) {
  if (l.dims == 0) return true;
  return l.numel() < kIndex32Limit && last_offset(l) < kIndex32Limit &&
         last_offset(l) > -kIndex32Limit;
}

// Joint iteration space of `n` operands that share one logical shape.
// After the call every operand has the same `dims`/`size`, and dim i was
// merged into dim i+1 only where every operand allowed it. Size-1 dims are
// dropped. With `reorder`, the dims are first sorted so that operand 0 (the
// output) walks its memory in increasing-address order: a pointwise op may
// visit the index space in any order as long as all operands are relabelled
// alike, and this turns "every operand transposed the same way" into plain
// contiguous runs. Returns false if the shapes differ (then the operands can
// only be paired by logical linear index).
inline bool joint_collapse(int n, Layout* ops, bool reorder = false) {
  const int nd = ops[0].dims;
  for (int k = 1; k < n; ++k) {
    if (ops[k].dims != nd) return false;
    for (int i = 0; i < nd; ++i)
      if (ops[k].size[i] != ops[0].size[i]) return false;
  }
  // surviving dims, outermost first
  int order[kMaxDims];
  int cnt = 0;
  for (int i = 0; i < nd; ++i)
    if (ops[0].size[i] != 1) order[cnt++] = i;
  if (reorder) {
    auto mag = [&](int d) {
      int64_t st = ops[0].stride[d];
      return st < 0 ? -st : st;
    };
    std::stable_sort(order, order + cnt, [&](int a, int b) { return mag(a) > mag(b); });
  }
  int64_t ns[kMaxDims];
  int64_t nt[4][kMaxDims];
  int m = 0;
  for (int j = cnt - 1; j >= 0; --j) {
    const int i = order[j];
    const int64_t sz = ops[0].size[i];
    bool merge = m > 0;
    for (int k = 0; merge && k < n; ++k)
      merge = ops[k].stride[i] == ns[m - 1] * nt[k][m - 1];
    if (merge) {
      ns[m - 1] *= sz;
    } else {
      ns[m] = sz;
      for (int k = 0; k < n; ++k) nt[k][m] = ops[k].stride[i];
      ++m;
    }
  }
  if (m == 0) {
    ns[0] = 1;
    for (int k = 0; k < n; ++k) nt[k][0] = 1;
    m = 1;
  }
  for (int k = 0; k < n; ++k) {
    ops[k].dims = m;
    for (int i = 0; i < m; ++i) {
      ops[k].size[i] = ns[m - 1 - i];
      ops[k].stride[i] = nt[k][m - 1 - i];
    }
  }
  return true;
}

}  // namespace thc
