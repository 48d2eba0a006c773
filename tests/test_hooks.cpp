// Test-only C entry points over the library's internal host logic (layout rules, expression
// rewrite, apply planning, index division, matrix-product planning).  Not part of the shipped
// library: the CPU test suite links this file with the library's object files into a library of
// its own (tests/conftest.py), and the sanitizer driver compiles the layout / rewrite part with
// g++ (THCL_HOOKS_PLANNERS undefined).
#include <cstring>
#include <string>

#include "internal.h"

extern "C" {
static void dbg_header(THClTensor &h, int nd, long *sz, long *st, long off) {
  h = THClTensor{};
  h.size = sz;
  h.stride = st;
  h.nDimension = nd;
  h.storageOffset = off;
}
int thcl_dbg_collapse(int nd, long *sizes, long *strides, int reduce_dim, long *out_sizes, long *out_strides) {
  THClTensor h;
  dbg_header(h, nd, sizes, strides, 0);
  Layout L = thcl_collapse(&h, reduce_dim);
  for (int d = 0; d < L.dims; d++) {
    out_sizes[d] = L.sizes[d];
    out_strides[d] = L.strides[d];
  }
  return L.dims;
}
int thcl_dbg_overlapping(int nd, long *sizes, long *strides) {
  THClTensor h;
  dbg_header(h, nd, sizes, strides, 0);
  return thcl_overlapping(&h) ? 1 : 0;
}
// n operands, each with `nd[i]` dims stored at row i of the [n][25] arrays;
// returns the joint dim count (-1: shapes differ) and the joint sizes/strides.
int thcl_dbg_joint_collapse(int n, const int *nd, long *sizes, long *strides, long *out_sizes, long *out_strides) {
  THClTensor h[3];
  THClTensor *tp[3];
  for (int i = 0; i < n; i++) {
    dbg_header(h[i], nd[i], sizes + i * THCL_MAX_DIMS, strides + i * THCL_MAX_DIMS, 0);
    tp[i] = &h[i];
  }
  JointLayout J = thcl_joint_collapse(n, tp);
  if (!J.valid) return -1;
  for (int d = 0; d < J.dims; d++) {
    out_sizes[d] = J.sizes[d];
    for (int i = 0; i < n; i++) out_strides[i * THCL_MAX_DIMS + d] = J.strides[i][d];
  }
  return J.dims;
}
// the rewritten text of a user expression
int thcl_dbg_rewrite_expr(const char *expr, int ntensors, char *buf, size_t buflen) {
  try {
    std::string r = thcl_rewrite_expr(expr, ntensors);
    if (r.size() + 1 > buflen) return -1;
    memcpy(buf, r.c_str(), r.size() + 1);
    return (int)r.size();
  } catch (const std::exception &) {
    return -1;
  }
}

#ifdef THCL_HOOKS_PLANNERS
// a compile of the generated source for a named architecture (no device needed)
int thcl_dbg_compile_expr_family(const char *expr, int ntensors, int family, const char *arch, size_t *code_bytes) {
  try {
    std::string src = thcl_expr_source(thcl_rewrite_expr(expr, ntensors), ntensors, family);
    return thcl_rt_compile_check(src.c_str(), arch, code_bytes);
  } catch (const std::exception &) {
    return -2;
  }
}
int thcl_dbg_compile_expr(const char *expr, int ntensors, const char *arch, size_t *code_bytes) {
  return thcl_dbg_compile_expr_family(expr, ntensors, -1, arch, code_bytes);
}

// Which kernel family a call with these views would launch, and its grid (-1: rejected).
// Views are rows of [n][25] arrays; misalign[i] = bytes by which operand i's storage misses a
// 16-byte boundary.
int thcl_dbg_plan_kind(int n, const int *nd, long *sizes, long *strides, const long *offsets, const int *misalign,
                       unsigned *grid) {
  THClTensor hdr[3];
  THClStorage st[3];
  ApplyCall call;
  call.n = n;
  for (int i = 0; i < n; i++) {
    hdr[i] = THClTensor{};
    st[i] = THClStorage{};
    st[i].wrapper = (void *)(uintptr_t)(0x10000000ull * (i + 1) + (unsigned)misalign[i]);
    st[i].size = 1l << 40;
    hdr[i].size = sizes + i * THCL_MAX_DIMS;
    hdr[i].stride = strides + i * THCL_MAX_DIMS;
    hdr[i].nDimension = nd[i];
    hdr[i].storageOffset = offsets[i];
    hdr[i].storage = &st[i];
    call.t[i] = &hdr[i];
  }
  try {
    return thcl_apply_classify(call, grid);
  } catch (const std::exception &) {
    return -1;
  }
}

// n / d the way the kernels compute it (multiply, shift)
unsigned thcl_dbg_divide(unsigned n, long d) { return thcl_host_divide(n, d); }

void thcl_dbg_gemm_plan(long m, long n, long k, int cus, int *bm, int *bn, int *ksplit, int *kchunk, int *tail_tiles, int *tail_split) {
  thcl_gemm_plan(m, n, k, cus, bm, bn, ksplit, kchunk, tail_tiles, tail_split);
}
#endif
}
