// TEST INFRASTRUCTURE ONLY.  A host-memory stand-in for the runtime layer
// (include/thcl_rt.h) plus the two device operations tensor.cpp needs, so that the
// tensor / storage / state bookkeeping (tensor.cpp, state.cpp) can be linked into a
// plain C++ program and run under AddressSanitizer without a device.  Nothing in the
// library links or loads this file; the library itself has no host path.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>

#include "internal.h"

struct thcl_rt {
  thcl_rt_props props;
  std::map<void *, size_t> live;
  float host_word[4];
  void *scratch;
};
struct thcl_rt_timer { int unused; };

static thcl_rt *g_rt[2] = {nullptr, nullptr};
static std::string g_err;

extern "C" {
int thcl_rt_device_count(void) { return 2; }
thcl_rt *thcl_rt_get(int device) {
  if (device < 0 || device >= 2) {
    g_err = "no such device";
    return nullptr;
  }
  if (!g_rt[device]) {
    thcl_rt *rt = new thcl_rt();
    memset(&rt->props, 0, sizeof rt->props);
    snprintf(rt->props.name, sizeof rt->props.name, "host stub %d", device);
    snprintf(rt->props.arch, sizeof rt->props.arch, "none");
    rt->props.compute_units = 4;
    rt->props.wavefront = 64;
    rt->props.max_threads_per_block = 1024;
    rt->props.total_mem = (size_t)1 << 30;
    rt->scratch = calloc(1, 65536);
    g_rt[device] = rt;
  }
  return g_rt[device];
}
void thcl_rt_release_all(void) {
  for (auto &rt : g_rt) {
    if (!rt) continue;
    for (auto &kv : rt->live) free(kv.first);  // the library frees what it allocated; leftovers are reported below
    if (!rt->live.empty()) fprintf(stderr, "host_rt_stub: %zu buffers still allocated at shutdown\n", rt->live.size());
    free(rt->scratch);
    delete rt;
    rt = nullptr;
  }
}
const thcl_rt_props *thcl_rt_get_props(thcl_rt *rt) { return &rt->props; }
const char *thcl_rt_error(void) { return g_err.c_str(); }
void *thcl_rt_malloc(thcl_rt *rt, size_t bytes) {
  void *p = malloc(bytes ? bytes : 1);   // exact size: the sanitizer sees every overrun
  if (p) rt->live[p] = bytes;
  return p;
}
int thcl_rt_free(thcl_rt *rt, void *dptr) {
  if (!dptr) return 0;
  auto it = rt->live.find(dptr);
  if (it == rt->live.end()) {
    g_err = "free of an unknown buffer";
    return -1;
  }
  rt->live.erase(it);
  free(dptr);
  return 0;
}
int thcl_rt_empty_cache(thcl_rt *) { return 0; }
void thcl_rt_memory_stats(thcl_rt *rt, size_t *live_bytes, size_t *cached_bytes, unsigned long long *device_mallocs,
                          unsigned long long *reused) {
  size_t b = 0;
  for (auto &kv : rt->live) b += kv.second;
  if (live_bytes) *live_bytes = b;
  if (cached_bytes) *cached_bytes = 0;
  if (device_mallocs) *device_mallocs = rt->live.size();
  if (reused) *reused = 0;
}
int thcl_rt_memcpy_h2d(thcl_rt *, void *dst, const void *src, size_t bytes) { memcpy(dst, src, bytes); return 0; }
int thcl_rt_memcpy_d2h(thcl_rt *, void *dst, const void *src, size_t bytes) { memcpy(dst, src, bytes); return 0; }
int thcl_rt_copy_converted(thcl_rt *, void *, void *, size_t, int, int) { return -1; }
int thcl_rt_memcpy_d2d(thcl_rt *, void *dst, const void *src, size_t bytes) { memmove(dst, src, bytes); return 0; }
void *thcl_rt_stream(thcl_rt *) { return nullptr; }
int thcl_rt_sync(thcl_rt *) { return 0; }
void *thcl_rt_scratch(thcl_rt *rt, size_t *bytes) {
  if (bytes) *bytes = 65536;
  return rt->scratch;
}
void *thcl_rt_host_alloc(size_t bytes) { return malloc(bytes ? bytes : 1); }
int thcl_rt_host_free(void *ptr) { free(ptr); return 0; }
float *thcl_rt_host_word(thcl_rt *rt) { return rt->host_word; }
float *thcl_rt_host_word_device(thcl_rt *rt) { return rt->host_word; }
unsigned *thcl_rt_fault_word_device(thcl_rt *rt) { return (unsigned *)rt->host_word + 32; }
int thcl_rt_check_fault(thcl_rt *) { return 0; }
float *thcl_rt_tagged_word_device(thcl_rt *rt) { return rt->host_word + 40; }
float *thcl_rt_mailbox_device(thcl_rt *rt) { return rt->host_word; }
const float *thcl_rt_mailbox_host(thcl_rt *rt, size_t *floats) { if (floats) *floats = 0; return rt->host_word; }
unsigned thcl_rt_next_tag(thcl_rt *) { return 1u; }
int thcl_rt_await_tagged(thcl_rt *, unsigned, float *value) { *value = 0.f; return 0; }
thcl_rt_timer *thcl_rt_timer_new(thcl_rt *) { return new thcl_rt_timer(); }
int thcl_rt_timer_start(thcl_rt_timer *) { return 0; }
int thcl_rt_timer_stop(thcl_rt_timer *) { return 0; }
float thcl_rt_timer_ms(thcl_rt_timer *) { return 0.f; }
void thcl_rt_timer_free(thcl_rt_timer *t) { delete t; }

// dst = src, element by element in index order (what the strided copy kernel computes)
void THClTensor_copy(THClState *, THClTensor *dst, THClTensor *src) {
  long n = 1;
  for (int d = 0; d < dst->nDimension; d++) n *= dst->size[d];
  if (dst->nDimension == 0 && !dst->storage) n = 0;
  auto at = [](THClTensor *t, long lin) {
    long off = t->storageOffset;
    for (int d = t->nDimension - 1; d >= 0; d--) {
      off += (lin % t->size[d]) * t->stride[d];
      lin /= t->size[d];
    }
    return (float *)t->storage->wrapper + off;
  };
  for (long i = 0; i < n; i++) *at(dst, i) = *at(src, i);
}
}

void thcl_reduce_static_setup(int) {}  // device-side set-up of the reduction kernels: nothing to do on the host

void thcl_fill_contig(thcl_rt *, float *dst, float value, long n) {
  for (long i = 0; i < n; i++) dst[i] = value;
}
