// Randomised driver for the host-only parts of the library (layout collapse,
// overlap test, joint collapse, expression rewriting), meant to be built with
// -fsanitize=address,undefined and linked with layout.cpp and expr.cpp only.
// Every collapsed layout is checked against the original by walking all elements.
#include <algorithm>
#include <array>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "internal.h"

// what the two sources need from the rest of the library
void thcl_throw(const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  throw std::runtime_error(buf);
}
std::string thcl_apply_config_defines() { return ""; }
extern "C" int thcl_rt_compile_check(const char *, const char *, size_t *) { return 0; }

extern "C" {
int thcl_dbg_collapse(int nd, long *sizes, long *strides, int reduce_dim, long *out_sizes, long *out_strides);
int thcl_dbg_overlapping(int nd, long *sizes, long *strides);
int thcl_dbg_joint_collapse(int n, const int *nd, long *sizes, long *strides, long *out_sizes, long *out_strides);
int thcl_dbg_rewrite_expr(const char *expr, int ntensors, char *buf, size_t buflen);
}

static long offset_of(long lin, int nd, const long *sz, const long *st) {
  long off = 0;
  for (int d = nd - 1; d >= 0; d--) {
    off += (lin % sz[d]) * st[d];
    lin /= sz[d];
  }
  return off;
}

static int fail(const char *what, unsigned long it) {
  fprintf(stderr, "host_fuzz: %s failed at iteration %lu\n", what, it);
  return 1;
}

int main(int argc, char **argv) {
  const unsigned long iters = argc > 1 ? strtoul(argv[1], nullptr, 10) : 20000;
  std::mt19937_64 rng(12345);
  auto pick = [&](long lo, long hi) { return lo + (long)(rng() % (unsigned long)(hi - lo + 1)); };
  for (unsigned long it = 0; it < iters; it++) {
    // a view built the way narrow / select / transpose / expand build them
    const int nd = (int)pick(1, 6);
    long sz[THCL_MAX_DIMS], st[THCL_MAX_DIMS];
    long run = 1;
    for (int d = nd - 1; d >= 0; d--) {
      sz[d] = pick(1, 5);
      const int kind = (int)pick(0, 9);
      st[d] = kind == 0 ? 0 : kind == 1 ? run * pick(2, 3) : run;  // expanded, strided, dense
      run = (st[d] ? st[d] : run) * sz[d];
    }
    for (int s = 0; s < 2; s++) {
      const int a = (int)pick(0, nd - 1), b = (int)pick(0, nd - 1);
      std::swap(sz[a], sz[b]);
      std::swap(st[a], st[b]);
    }
    long n = 1;
    for (int d = 0; d < nd; d++) n *= sz[d];
    long osz[THCL_MAX_DIMS], ost[THCL_MAX_DIMS];
    const int cd = thcl_dbg_collapse(nd, sz, st, -1, osz, ost);
    if (cd < 1 || cd > nd) return fail("collapse: dim count", it);
    long cn = 1;
    for (int d = 0; d < cd; d++) cn *= osz[d];
    if (cn != n) return fail("collapse: element count", it);
    for (long i = 0; i < n; i++)
      if (offset_of(i, nd, sz, st) != offset_of(i, cd, osz, ost)) return fail("collapse: offsets", it);
    // overlap test against brute force; a "no" from it must be right (a "yes" may be conservative)
    {
      std::vector<long> seen;
      bool dup = false;
      for (long i = 0; i < n && !dup; i++) {
        const long o = offset_of(i, nd, sz, st);
        for (long p : seen) dup = dup || p == o;
        seen.push_back(o);
      }
      if (!thcl_dbg_overlapping(nd, sz, st) && dup) return fail("overlap: missed an alias", it);
    }
    // joint collapse of two or three operands of the same shape
    {
      const int ops = (int)pick(2, 3);
      int nds[3] = {nd, nd, nd};
      long js[3 * THCL_MAX_DIMS], jt[3 * THCL_MAX_DIMS], jos[THCL_MAX_DIMS], jot[3 * THCL_MAX_DIMS];
      for (int o = 0; o < ops; o++) {
        long r = 1;
        for (int d = nd - 1; d >= 0; d--) {
          js[o * THCL_MAX_DIMS + d] = sz[d];
          jt[o * THCL_MAX_DIMS + d] = (o == 0) ? st[d] : (pick(0, 7) == 0 ? 0 : r);
          r *= sz[d] * (pick(0, 5) == 0 ? 2 : 1);
        }
      }
      const int jd = thcl_dbg_joint_collapse(ops, nds, js, jt, jos, jot);
      if (jd < 1 || jd > nd) return fail("joint collapse: dim count", it);
      // the joint order may differ from the operands' own (dims are sorted by the written
      // operand's stride), so compare the sets of offset tuples
      std::vector<std::array<long, 3>> want(n), got(n);
      for (long i = 0; i < n; i++)
        for (int o = 0; o < 3; o++) {
          want[i][o] = o < ops ? offset_of(i, nd, js + o * THCL_MAX_DIMS, jt + o * THCL_MAX_DIMS) : 0;
          got[i][o] = o < ops ? offset_of(i, jd, jos, jot + o * THCL_MAX_DIMS) : 0;
        }
      std::sort(want.begin(), want.end());
      std::sort(got.begin(), got.end());
      if (want != got) return fail("joint collapse: offsets", it);
    }
    // expression rewriting: any text in, bounded text out, no stray reads
    {
      static const char *const words[] = {"x", "y", "z", "exp", "max", "min", "sqrt", "*out", "*in1", "*in2", "xy", "x1",
                                          "_x", "1000", "1.5f", "+", "-", "*", "/", "=", "(", ")", ";", " ", ",", "?", ":",
                                          "<", "expx", "maxy", "\t", "0x1p3", "e", "E", "1e", "1e5", ".", "x.y", "\"", "'"};
      std::string e;
      const int len = (int)pick(0, 24);
      for (int i = 0; i < len; i++) e += words[rng() % (sizeof words / sizeof *words)];
      std::vector<char> buf(16 * e.size() + 64);
      const int ntensors = (int)pick(1, 3);
      const int r = thcl_dbg_rewrite_expr(e.c_str(), ntensors, buf.data(), buf.size());
      if (r >= 0 && (size_t)r != strlen(buf.data())) return fail("rewrite: length", it);
    }
  }
  printf("host_fuzz: %lu iterations ok\n", iters);
  return 0;
}
