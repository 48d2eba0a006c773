// Random walk over the tensor / storage bookkeeping of the library (tensor.cpp,
// state.cpp) linked against the host-memory runtime stand-in (host_rt_stub.cpp), meant
// for -fsanitize=address,undefined.  A small model of each view (offset, sizes,
// strides, following Torch's rules: narrow src/lib/THClTensor.cpp:389-407, select
// :409-431, transpose :433-449, unfold :451-498, squeeze :500-548) is kept beside the
// real header and compared after every step; element reads go through get1d..get4d
// and through the storage.  At the end everything is freed and the stand-in must hold
// no buffer.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "thcl_hip.h"
#include "thcl_rt.h"

struct View {
  THClTensor *t;
  long off;
  std::vector<long> sz, st;
};

static int g_errors = 0;
static void on_error(const char *, void *) { g_errors++; }
static std::mt19937_64 rng(2024);
static long pick(long lo, long hi) { return lo + (long)(rng() % (unsigned long)(hi - lo + 1)); }

static bool same(THClState *S, const View &v) {
  if (THClTensor_nDimension(S, v.t) != (int)v.sz.size()) return false;
  if (THClTensor_storageOffset(S, v.t) != v.off) return false;
  for (size_t d = 0; d < v.sz.size(); d++)
    if (THClTensor_size(S, v.t, (int)d) != v.sz[d] || THClTensor_stride(S, v.t, (int)d) != v.st[d]) return false;
  return true;
}

static long nelem(const View &v) {
  long n = v.sz.empty() ? 0 : 1;
  for (long s : v.sz) n *= s;
  return n;
}

// the element at linear index `lin` read through the storage, and through getNd where there is one
static bool elements_agree(THClState *S, const View &v) {
  const long n = nelem(v);
  THClStorage *stg = THClTensor_storage(S, v.t);
  for (long lin = 0; lin < n; lin++) {
    long idx[8], r = lin, off = v.off;
    for (int d = (int)v.sz.size() - 1; d >= 0; d--) {
      idx[d] = r % v.sz[d];
      r /= v.sz[d];
      off += idx[d] * v.st[d];
    }
    if (off < 0 || off >= THClStorage_size(S, stg)) return false;
    const float want = THClStorage_get(S, stg, off);
    float got = want;
    switch (v.sz.size()) {
      case 1: got = THClTensor_get1d(S, v.t, idx[0]); break;
      case 2: got = THClTensor_get2d(S, v.t, idx[0], idx[1]); break;
      case 3: got = THClTensor_get3d(S, v.t, idx[0], idx[1], idx[2]); break;
      case 4: got = THClTensor_get4d(S, v.t, idx[0], idx[1], idx[2], idx[3]); break;
      default: break;
    }
    if (got != want) return false;
  }
  return true;
}

static int fail(const char *what, unsigned long it) {
  fprintf(stderr, "host_tensor_walk: %s (iteration %lu, last error: %s)\n", what, it,
          THClLastError() ? THClLastError() : "none");
  return 1;
}

int main(int argc, char **argv) {
  const unsigned long iters = argc > 1 ? strtoul(argv[1], nullptr, 10) : 5000;
  THClState state;
  memset(&state, 0, sizeof state);
  THClState *S = &state;
  THClInit(S);
  THClSetErrorHandler(on_error, nullptr);
  std::vector<View> pool;
  auto fresh = [&]() {
    View v;
    const int nd = (int)pick(1, 4);
    for (int d = 0; d < nd; d++) v.sz.push_back(pick(1, 5));
    v.st.assign(nd, 1);
    for (int d = nd - 2; d >= 0; d--) v.st[d] = v.st[d + 1] * v.sz[d + 1];
    v.off = 0;
    THLongStorage *ls = THLongStorage_newWithSize(nd);
    for (int d = 0; d < nd; d++) THLongStorage_set(ls, d, v.sz[d]);
    v.t = THClTensor_newWithSize(S, (int)pick(0, 1), ls, nullptr);
    THLongStorage_free(ls);
    THClStorage *stg = THClTensor_storage(S, v.t);
    for (long i = 0; i < THClStorage_size(S, stg); i++) THClStorage_set(S, stg, i, (float)(pick(0, 1000)));
    return v;
  };
  for (unsigned long it = 0; it < iters; it++) {
    if (pool.size() < 3) pool.push_back(fresh());
    const size_t which = (size_t)pick(0, (long)pool.size() - 1);
    View src = pool[which];
    const int nd = (int)src.sz.size();
    const int op = (int)pick(0, 11);
    const int errors_before = g_errors;
    View out = src;
    bool made = false, expect_error = false;
    switch (op) {
      case 0: {  // narrow, sometimes out of range
        const int d = (int)pick(0, nd - 1);
        const long first = pick(0, src.sz[d]), len = pick(1, src.sz[d] + 1);
        expect_error = first + len > src.sz[d];
        out.t = THClTensor_newNarrow(S, src.t, d, first, len);
        out.off += first * src.st[d];
        out.sz[d] = len;
        made = true;
        break;
      }
      case 1: {  // select
        if (nd < 2) continue;
        const int d = (int)pick(0, nd - 1);
        const long i = pick(0, src.sz[d]);
        expect_error = i >= src.sz[d];
        out.t = THClTensor_newSelect(S, src.t, d, i);
        out.off += i * src.st[d];
        out.sz.erase(out.sz.begin() + d);
        out.st.erase(out.st.begin() + d);
        made = true;
        break;
      }
      case 2: {  // transpose
        const int a = (int)pick(0, nd - 1), b = (int)pick(0, nd);
        expect_error = b >= nd;
        out.t = THClTensor_newTranspose(S, src.t, a, b);
        if (!expect_error) {
          std::swap(out.sz[a], out.sz[b]);
          std::swap(out.st[a], out.st[b]);
        }
        made = true;
        break;
      }
      case 3: {  // unfold
        if (nd >= 4) continue;
        const int d = (int)pick(0, nd - 1);
        const long len = pick(1, src.sz[d] + 1), step = pick(1, 3);
        expect_error = len > src.sz[d];
        out.t = THClTensor_newUnfold(S, src.t, d, len, step);
        if (!expect_error) {
          out.sz.push_back(len);
          out.st.push_back(src.st[d]);
          out.sz[d] = (src.sz[d] - len) / step + 1;
          out.st[d] = src.st[d] * step;
        }
        made = true;
        break;
      }
      case 4: {  // squeeze into a new header
        out.t = THClTensor_newWithTensor(S, src.t);
        THClTensor_squeeze(S, out.t, src.t);
        std::vector<long> sz, st;
        for (int d = 0; d < nd; d++)
          if (src.sz[d] != 1) {
            sz.push_back(src.sz[d]);
            st.push_back(src.st[d]);
          }
        if (sz.empty()) {  // all ones: one dim of size 1 stays
          sz.push_back(1);
          st.push_back(1);
          if (nd > 0) st[0] = THClTensor_stride(S, out.t, 0);
        }
        out.sz = sz;
        out.st = st;
        made = true;
        break;
      }
      case 5: {  // clone: dense copy with equal elements in index order
        out.t = THClTensor_newClone(S, src.t);
        out.off = 0;
        out.st.assign(nd, 1);
        for (int d = nd - 2; d >= 0; d--) out.st[d] = out.st[d + 1] * out.sz[d + 1];
        if (THClTensor_storage(S, out.t) == THClTensor_storage(S, src.t)) return fail("clone shares storage", it);
        const long n = nelem(src);
        for (long lin = 0; lin < n; lin++) {
          long r = lin, off = src.off;
          for (int d = nd - 1; d >= 0; d--) {
            off += (r % src.sz[d]) * src.st[d];
            r /= src.sz[d];
          }
          if (THClStorage_get(S, THClTensor_storage(S, out.t), lin) != THClStorage_get(S, THClTensor_storage(S, src.t), off))
            return fail("clone: elements", it);
        }
        made = true;
        break;
      }
      case 6: {  // newContiguous: same header retained when already dense
        THClTensor *c = THClTensor_newContiguous(S, src.t);
        if (THClTensor_isContiguous(S, src.t) != (c == src.t)) return fail("newContiguous identity", it);
        if (!THClTensor_isContiguous(S, c)) return fail("newContiguous not dense", it);
        THClTensor_free(S, c);
        continue;
      }
      case 7: {  // resize in place: same element count keeps the storage, a larger one grows it
        View &v = pool[which];
        if (!THClTensor_isContiguous(S, v.t) || v.off != 0) continue;
        THClStorage *before = THClTensor_storage(S, v.t);
        const long a = pick(1, 6), b = pick(1, 6);
        THClTensor_resize2d(S, v.t, a, b);
        v.sz = {a, b};
        v.st = {b, 1};
        if (THClTensor_storage(S, v.t) != before) return fail("resize replaced the storage object", it);
        if (THClStorage_size(S, before) < a * b) return fail("resize did not grow the storage", it);
        if (!same(S, v)) return fail("resize2d header", it);
        continue;
      }
      case 8: {  // set: header copy sharing the storage
        out.t = THClTensor_newv2(S, THClTensor_getDevice(S, src.t));
        THClTensor_set(S, out.t, src.t);
        made = true;
        break;
      }
      case 9: {  // element writes through setNd land where the model says
        if (nd > 4 || nelem(src) == 0) continue;
        long idx[4] = {0, 0, 0, 0}, off = src.off;
        for (int d = 0; d < nd; d++) {
          idx[d] = pick(0, src.sz[d] - 1);
          off += idx[d] * src.st[d];
        }
        const float v = (float)pick(2000, 3000);
        if (nd == 1) THClTensor_set1d(S, src.t, idx[0], v);
        if (nd == 2) THClTensor_set2d(S, src.t, idx[0], idx[1], v);
        if (nd == 3) THClTensor_set3d(S, src.t, idx[0], idx[1], idx[2], v);
        if (nd == 4) THClTensor_set4d(S, src.t, idx[0], idx[1], idx[2], idx[3], v);
        if (THClStorage_get(S, THClTensor_storage(S, src.t), off) != v) return fail("setNd landed elsewhere", it);
        continue;
      }
      case 10: {  // retain / free pairs leave the count where it was
        const int rc = src.t->refcount;
        THClTensor_retain(S, src.t);
        THClTensor_free(S, src.t);
        if (src.t->refcount != rc) return fail("retain/free", it);
        continue;
      }
      default: {  // drop one
        THClTensor_free(S, src.t);
        pool.erase(pool.begin() + (long)which);
        continue;
      }
    }
    if (made) {
      if (expect_error) {
        if (g_errors == errors_before) return fail("an out-of-range view raised no error", it);
        if (out.t) THClTensor_free(S, out.t);
        THClClearError();
        if (!same(S, src)) return fail("a failed view changed its source", it);
        continue;
      }
      if (g_errors != errors_before || !out.t) return fail("a valid view raised an error", it);
      if (!same(S, out)) return fail("view header differs from the model", it);
      if (!elements_agree(S, out)) return fail("view elements differ from the storage", it);
      if (pool.size() < 12) pool.push_back(out);
      else THClTensor_free(S, out.t);
    }
  }
  for (View &v : pool) THClTensor_free(S, v.t);
  size_t live = 0;
  for (int d = 0; d < 2; d++)
    if (state.clByDevice && state.clByDevice[d]) {
      size_t b = 0;
      thcl_rt_memory_stats(state.clByDevice[d], &b, nullptr, nullptr, nullptr);
      live += b;
    }
  THClShutdown(S);
  if (live != 0) return fail("buffers left after freeing every tensor", iters);
  printf("host_tensor_walk: %lu iterations ok, %d expected errors\n", iters, g_errors);
  return 0;
}
