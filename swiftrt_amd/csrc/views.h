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

// With pitch P: every dimension of the view either moves by a multiple of P, or belongs to the "inner" part.  The
// bytes of the view then lie, modulo P, in the circular interval [start, start + len) of [0, P) (it may wrap past P:
// nothing here depends on where a buffer happens to lie relative to a multiple of its pitch).  Returns false when
// the view does not decompose that way (a stride above P that is no multiple of it, or an inner part longer than P).
inline bool residue_interval(const StridedView& v, long long P, long long* start, long long* len) {
  long long inner_last = 0;
  for (int d = 0; d < 3; ++d) {
    if (v.extent[d] <= 1) continue;
    if (v.stride[d] >= P) {
      if (v.stride[d] % P != 0) return false;
    } else {
      inner_last += (v.extent[d] - 1) * v.stride[d];
    }
  }
  *start = (long long)(v.base % (uintptr_t)P);
  *len = inner_last + (long long)v.es;
  return *len <= P;
}

// Do the circular intervals [a0, a0 + la) and [b0, b0 + lb) of [0, P) keep apart?  (la, lb <= P)
inline bool circular_apart(long long a0, long long la, long long b0, long long lb, long long P) {
  const long long d = ((b0 - a0) % P + P) % P;   // b's start, counted from a's
  return d >= la && d + lb <= P;
}

// true: provably no common element.  false: they may share one (not a proof that they do).
// The proof: some pitch P -- one of the views' own strides -- for which both views decompose as above
// into circular intervals of [0, P) that do not meet.  Column slices of one wide row-major buffer (P = the row
// pitch) and interleaved batches (P = the batch stride) are the cases it is meant for.  The verdict depends on
// the difference of the two base addresses only.
inline bool views_disjoint(const StridedView& a, const StridedView& b) {
  if (!spans_overlap(a, b)) return true;
  const StridedView* both[2] = {&a, &b};
  for (const StridedView* v : both) {
    for (int d = 0; d < 3; ++d) {
      const long long P = v->stride[d];
      if (v->extent[d] <= 1 || P <= 0) continue;
      long long a0, la, b0, lb;
      if (residue_interval(a, P, &a0, &la) && residue_interval(b, P, &b0, &lb) && circular_apart(a0, la, b0, lb, P)) return true;
    }
  }
  return false;
}

// true: provably a common element.  Proved for the plain case only: with some pitch P both views are dense rows
// (unit-stride inner dimension) under a single outer dimension of stride exactly P.  Counted from a's first byte,
// b starts q whole pitches and r bytes further (0 <= r < P): row j of b meets row q + j of a when r lies inside a's
// row, and row q + j + 1 of a when b's row runs past the end of the pitch.
inline bool views_alias(const StridedView& a, const StridedView& b) {
  if (a.base == b.base) return true;
  if (a.es != b.es || !spans_overlap(a, b)) return false;
  auto rows_of = [](const StridedView& v, long long* P, long long* cols, long long* rows) {
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
    *rows = v.extent[outer];
    return *P >= *cols * (long long)v.es;
  };
  long long Pa, Pb, ca, cb, ea, eb;
  if (!rows_of(a, &Pa, &ca, &ea) || !rows_of(b, &Pb, &cb, &eb) || Pa != Pb) return false;
  const long long P = Pa, wa = ca * (long long)a.es, wb = cb * (long long)b.es;
  const long long delta = a.base <= b.base ? (long long)(b.base - a.base) : -(long long)(a.base - b.base);
  long long q = delta / P, r = delta % P;
  if (r < 0) { r += P; q -= 1; }                       // floor division
  if (r % (long long)a.es != 0) return false;          // (elements that only straddle one another: left to the other verdicts)
  auto rows_meet = [&](long long first) {              // rows first .. first + eb - 1 of a's numbering against 0 .. ea - 1
    return first <= ea - 1 && first + eb - 1 >= 0;
  };
  if (r < wa && rows_meet(q)) return true;
  if (r + wb > P && rows_meet(q + 1)) return true;
  return false;
}

}  // namespace srt
