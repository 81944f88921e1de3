// Do two strided views share an element?  Host-side arithmetic for the entry points' alias checks.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace srt {

// Up to three dimensions (extent, stride in bytes; strides are non-negative) over a base address.
struct StridedView {
  uintptr_t base;
  size_t es;               // element size in bytes
  long long extent[3];
  long long stride[3];     // bytes
  uintptr_t lo() const { return base; }
  uintptr_t hi() const {   // one past the last byte of the last element
    long long last = 0;
    for (int d = 0; d < 3; ++d) last += (extent[d] - 1) * stride[d];
    return base + (uintptr_t)last + es;
  }
};

// strides in elements, extents all >= 1
inline StridedView make_view(const void* base, size_t es, long long e0, long long s0, long long e1, long long s1, long long e2,
                             long long s2) {
  StridedView v;
  v.base = reinterpret_cast<uintptr_t>(base);
  v.es = es;
  v.extent[0] = e0; v.extent[1] = e1; v.extent[2] = e2;
  v.stride[0] = s0 * (long long)es; v.stride[1] = s1 * (long long)es; v.stride[2] = s2 * (long long)es;
  return v;
}

inline bool spans_overlap(const StridedView& a, const StridedView& b) { return a.lo() < b.hi() && b.lo() < a.hi(); }

// With pitch P: every dimension of the view either moves by a multiple of P, or belongs to the "inner"
// part, whose bytes all lie in [base mod P, base mod P + inner span) without crossing a multiple of P.
// Returns false when the view does not decompose that way.
inline bool inner_interval(const StridedView& v, long long P, long long* from, long long* to) {
  long long inner_last = 0;
  for (int d = 0; d < 3; ++d) {
    if (v.extent[d] <= 1) continue;
    if (v.stride[d] >= P) {
      if (v.stride[d] % P != 0) return false;
    } else {
      inner_last += (v.extent[d] - 1) * v.stride[d];
    }
  }
  *from = (long long)(v.base % (uintptr_t)P);
  *to = *from + inner_last + (long long)v.es;
  return *to <= P;
}

// true: provably no common element.  false: they may share one (not a proof that they do).
// The proof: some pitch P -- one of the views' own strides -- for which both views decompose as above
// into intervals of [0, P) that do not meet.  Column slices of one wide row-major buffer (P = the row
// pitch) and interleaved batches (P = the batch stride) are the cases it is meant for.
inline bool views_disjoint(const StridedView& a, const StridedView& b) {
  if (!spans_overlap(a, b)) return true;
  const StridedView* both[2] = {&a, &b};
  for (const StridedView* v : both) {
    for (int d = 0; d < 3; ++d) {
      const long long P = v->stride[d];
      if (v->extent[d] <= 1 || P <= 0) continue;
      long long a0, a1, b0, b1;
      if (inner_interval(a, P, &a0, &a1) && inner_interval(b, P, &b0, &b1) && (a1 <= b0 || b1 <= a0)) return true;
    }
  }
  return false;
}

// true: provably a common element.  Proved for the plain case only: with some pitch P both views are dense rows
// (unit-stride inner dimension) under a single outer dimension of stride exactly P, their byte ranges inside the
// pitch meet, and so do their ranges of rows.
inline bool views_alias(const StridedView& a, const StridedView& b) {
  if (a.base == b.base) return true;
  if (a.es != b.es || !spans_overlap(a, b)) return false;
  auto rows_of = [](const StridedView& v, long long* P, long long* cols) {
    int outer = -1, inner = -1;
    for (int d = 0; d < 3; ++d) {
      if (v.extent[d] <= 1) continue;
      if (v.stride[d] == (long long)v.es && inner < 0) inner = d;
      else if (outer < 0) outer = d;
      else return false;
    }
    if (outer < 0) return false;
    *P = v.stride[outer];
    *cols = inner < 0 ? 1 : v.extent[inner];
    return *P >= *cols * (long long)v.es;
  };
  long long Pa, Pb, ca, cb;
  if (!rows_of(a, &Pa, &ca) || !rows_of(b, &Pb, &cb) || Pa != Pb) return false;
  long long a0, a1, b0, b1;
  if (!inner_interval(a, Pa, &a0, &a1) || !inner_interval(b, Pa, &b0, &b1)) return false;
  if (a1 <= b0 || b1 <= a0 || (a0 - b0) % (long long)a.es != 0) return false;
  const long long ra = (long long)(a.base / (uintptr_t)Pa), rb = (long long)(b.base / (uintptr_t)Pa);
  long long ea = 1, eb = 1;
  for (int d = 0; d < 3; ++d) {
    if (a.extent[d] > 1 && a.stride[d] == Pa) ea = a.extent[d];
    if (b.extent[d] > 1 && b.stride[d] == Pa) eb = b.extent[d];
  }
  return ra < rb + eb && rb < ra + ea;
}

}  // namespace srt
