// Host-side layout analysis: per-tensor collapse, self-overlap test, and the
// joint collapse of same-shaped operands that lets a pointwise kernel walk
// all of them with one index decomposition.
#include <algorithm>
#include <climits>

#include "internal.h"

// Per-tensor collapse.  Rule of src/lib/THClReduceApplyUtils.h:67-170: going
// from the innermost dimension outwards, size-1 dims (and `reduceDim`, which
// counts as size 1) vanish, and a dim merges into the run inside it when its
// stride equals that run's size*stride.
Layout thcl_collapse(const THClTensor *t, int reduceDim) {
  Layout L;
  L.offset = t->storageOffset;
  long sz[THCL_MAX_DIMS], st[THCL_MAX_DIMS];
  int k = 0;  // innermost first
  for (int d = t->nDimension - 1; d >= 0; d--) {
    long s = (d == reduceDim) ? 1 : t->size[d];
    if (s == 1) continue;
    if (k > 0 && t->stride[d] == sz[k - 1] * st[k - 1]) {
      sz[k - 1] *= s;
    } else {
      sz[k] = s;
      st[k] = t->stride[d];
      k++;
    }
  }
  if (k == 0) {  // a single point
    L.dims = 1;
    L.sizes[0] = 1;
    L.strides[0] = 1;
    return L;
  }
  L.dims = k;
  for (int i = 0; i < k; i++) {
    L.sizes[i] = sz[k - 1 - i];
    L.strides[i] = st[k - 1 - i];
  }
  return L;
}

// Does any element of the view alias another?  (src/lib/THClReduceApplyUtils.cpp:69-121)
// Dims of size > 1 ordered by stride: overlap iff the smallest stride is < 1
// or some stride is smaller than the extent of the next-smaller dim.
bool thcl_overlapping(const THClTensor *t) {
  struct SS {
    long size, stride;
  } v[THCL_MAX_DIMS];
  int k = 0;
  for (int d = 0; d < t->nDimension; d++)
    if (t->size[d] > 1) v[k++] = {t->size[d], t->stride[d]};
  if (k == 0) return false;
  std::sort(v, v + k, [](const SS &a, const SS &b) { return a.stride < b.stride; });
  if (v[0].stride < 1) return true;
  for (int i = 1; i < k; i++)
    if (v[i].stride < v[i - 1].size * v[i - 1].stride) return true;
  return false;
}

// Largest element offset and the element count both below 2^32
// (src/lib/THClReduceApplyUtils.cpp:9-30).
bool thcl_fits_32bit(const THClTensor *t) {
  long n = 1, maxoff = 0;
  for (int d = 0; d < t->nDimension; d++) {
    n *= t->size[d];
    maxoff += (t->size[d] - 1) * t->stride[d];
  }
  return n < (long)UINT_MAX && maxoff < (long)UINT_MAX;
}

JointLayout thcl_joint_collapse(int n, THClTensor *const *t) {
  JointLayout J;
  long sz[THCL_MAX_DIMS];
  long st[3][THCL_MAX_DIMS];
  int k = -1;
  for (int i = 0; i < n; i++) {
    int ki = 0;
    for (int d = 0; d < t[i]->nDimension; d++) {
      if (t[i]->size[d] == 1) continue;
      if (i == 0) sz[ki] = t[i]->size[d];
      else if (ki >= k || sz[ki] != t[i]->size[d]) return J;  // shapes differ
      st[i][ki] = t[i]->stride[d];
      ki++;
    }
    if (i == 0) k = ki;
    else if (ki != k) return J;
  }
  J.valid = true;
  if (k == 0) {
    J.dims = 1;
    J.sizes[0] = 1;
    for (int i = 0; i < n; i++) J.strides[i][0] = 1;
    return J;
  }
  // order by the written operand's stride, largest first
  int perm[THCL_MAX_DIMS];
  for (int d = 0; d < k; d++) perm[d] = d;
  std::stable_sort(perm, perm + k, [&](int a, int b) { return st[0][a] > st[0][b]; });
  // merge from the innermost dim outwards
  long msz[THCL_MAX_DIMS], mst[3][THCL_MAX_DIMS];
  int m = 0;  // innermost first
  for (int p = k - 1; p >= 0; p--) {
    int d = perm[p];
    bool merge = (m > 0);
    for (int i = 0; merge && i < n; i++)
      if (st[i][d] != msz[m - 1] * mst[i][m - 1]) merge = false;
    if (merge) {
      msz[m - 1] *= sz[d];
    } else {
      msz[m] = sz[d];
      for (int i = 0; i < n; i++) mst[i][m] = st[i][d];
      m++;
    }
  }
  J.dims = m;
  for (int j = 0; j < m; j++) {
    J.sizes[j] = msz[m - 1 - j];
    for (int i = 0; i < n; i++) J.strides[i][j] = mst[i][m - 1 - j];
  }
  return J;
}

// ------------------------------------------------------------ test hooks ---
