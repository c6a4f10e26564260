// Finding a row's sequence in a flattened step. A step holds B sequences; sequence b owns rows cu[b] .. cu[b+1]-1
// and has ctx[b] tokens after the step, so its first row sits at position ctx[b] - (cu[b+1] - cu[b]).
#pragma once
#include "common.h"

struct RowSeq {
  int b;     // sequence of the row
  int j;     // the row's index inside its portion
  int qlen;  // rows of the portion
  int pos;   // the row's position in its sequence (< 0: a padded row)
};

__device__ __forceinline__ RowSeq row_seq(const int* __restrict__ cu, const int* __restrict__ ctx, int B, int t) {
  int lo = 0, hi = B;
  while (hi - lo > 1) {  // the last b with cu[b] <= t (empty sequences share a boundary and are skipped)
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  RowSeq r;
  r.b = lo;
  r.qlen = cu[lo + 1] - cu[lo];
  r.j = t - cu[lo];
  r.pos = (t < cu[B]) ? ctx[lo] - r.qlen + r.j : -1;
  return r;
}
