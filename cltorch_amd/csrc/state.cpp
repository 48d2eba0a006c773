// Error plumbing, library state and the bundled stand-ins for the few Torch7
// `TH` host types the C ABI mentions.
#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "internal.h"

// ---------------------------------------------------------------- errors ---
namespace {
thread_local std::string g_last_error;
thread_local bool g_has_error = false;
THClErrorHandler g_handler = nullptr;
void *g_handler_data = nullptr;
}  // namespace

thread_local int ThclGuardScope::depth = 0;

// ---------------------------------------------------------------- profiling ---
// The reference's `cltorch.setProfiling(1)` / `dumpProfiling()` report OpenCL
// event timings per kernel (src/init.cpp:149-178).  Here every launch made
// while profiling is on sits between two HIP events on the library's stream
// and is booked under the entry point that made it.
namespace {
struct ProfRecord {
  const char *entry;
  thcl_rt_timer *timer;
};
std::vector<ProfRecord> g_prof_records;
bool g_prof_on = false;
thread_local const char *tl_entry = "";
thread_local thcl_rt_timer *tl_open = nullptr;  // started, waiting for the launch it will time

void prof_open(thcl_rt *rt) {
  if (!g_prof_on || tl_open) return;
  tl_open = thcl_rt_timer_new(rt);
  if (tl_open) thcl_rt_timer_start(tl_open);
}
void prof_close(thcl_rt *rt) {
  if (!tl_open) return;
  thcl_rt_timer_stop(tl_open);
  g_prof_records.push_back({tl_entry, tl_open});
  tl_open = nullptr;
  prof_open(rt);  // an entry point may launch again
}
}  // namespace

void thcl_profile_enter(const char *entry) {
  tl_entry = entry;
  if (tl_open) {  // opened by the previous call but never followed by a launch
    thcl_rt_timer_free(tl_open);
    tl_open = nullptr;
  }
}

void thcl_throw(const char *fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  throw ThclError(buf);
}

void thcl_report(const char *msg) {
  g_last_error = msg;
  g_has_error = true;
  if (g_handler) g_handler(g_last_error.c_str(), g_handler_data);
}

void thcl_clear_error() { g_has_error = false; }

extern "C" {

void THClSetErrorHandler(THClErrorHandler handler, void *data) {
  g_handler = handler;
  g_handler_data = data;
}
const char *THClLastError(void) { return g_has_error ? g_last_error.c_str() : nullptr; }
void THClClearError(void) { g_has_error = false; }

// ------------------------------------------------------------ TH stand-ins ---
#ifndef THCL_EXTERNAL_TH
THLongStorage *THLongStorage_newWithSize(long size) {
  auto *s = (THLongStorage *)calloc(1, sizeof(THLongStorage));
  s->data = size > 0 ? (long *)calloc((size_t)size, sizeof(long)) : nullptr;
  s->size = size > 0 ? size : 0;
  s->refcount = 1;
  s->flag = 1 | 2 | 4;
  return s;
}
void THLongStorage_free(THLongStorage *s) {
  if (!s) return;
  if (--s->refcount > 0) return;
  if (s->flag & 4) free(s->data);
  free(s);
}
void THLongStorage_set(THLongStorage *s, long i, long v) {
  if (s && i >= 0 && i < s->size) s->data[i] = v;
}
long THLongStorage_get(const THLongStorage *s, long i) { return (s && i >= 0 && i < s->size) ? s->data[i] : 0; }

static void host_shape(long **osz, long **ost, int nd, const long *size, const long *stride) {
  *osz = (long *)malloc(sizeof(long) * (nd > 0 ? nd : 1));
  *ost = (long *)malloc(sizeof(long) * (nd > 0 ? nd : 1));
  long z = 1;
  for (int d = nd - 1; d >= 0; d--) {
    (*osz)[d] = size[d];
    (*ost)[d] = (stride && stride[d] >= 0) ? stride[d] : z;
    z = (*osz)[d] * (*ost)[d];
  }
}
static long host_extent(int nd, const long *sz, const long *st) {
  if (nd <= 0) return 0;
  long e = 1;
  for (int d = 0; d < nd; d++) {
    if (sz[d] == 0) return 0;
    e += (sz[d] - 1) * st[d];
  }
  return e;
}

THFloatTensor *THFloatTensor_newWithSize(THLongStorage *size, THLongStorage *stride) {
  auto *t = (THFloatTensor *)calloc(1, sizeof(THFloatTensor));
  t->nDimension = size ? (int)size->size : 0;
  host_shape(&t->size, &t->stride, t->nDimension, size ? size->data : nullptr, stride ? stride->data : nullptr);
  long n = host_extent(t->nDimension, t->size, t->stride);
  t->storage = (THFloatStorage *)calloc(1, sizeof(THFloatStorage));
  t->storage->data = n > 0 ? (float *)calloc((size_t)n, sizeof(float)) : nullptr;
  t->storage->size = n;
  t->storage->refcount = 1;
  t->storage->flag = 1 | 2 | 4;
  t->refcount = 1;
  t->flag = 1;
  return t;
}
THFloatTensor *THFloatTensor_newWithData(float *data, long storageSize, long storageOffset, int nDimension,
                                         const long *size, const long *stride) {
  auto *t = (THFloatTensor *)calloc(1, sizeof(THFloatTensor));
  t->nDimension = nDimension;
  host_shape(&t->size, &t->stride, nDimension, size, stride);
  t->storage = (THFloatStorage *)calloc(1, sizeof(THFloatStorage));
  t->storage->data = data;
  t->storage->size = storageSize;
  t->storage->refcount = 1;
  t->storage->flag = 1;  // borrowed memory: no FREEMEM
  t->storageOffset = storageOffset;
  t->refcount = 1;
  t->flag = 1;
  return t;
}
void THFloatTensor_free(THFloatTensor *t) {
  if (!t) return;
  if (--t->refcount > 0) return;
  if (t->storage && --t->storage->refcount <= 0) {
    if (t->storage->flag & 4) free(t->storage->data);
    free(t->storage);
  }
  free(t->size);
  free(t->stride);
  free(t);
}
long THFloatTensor_nElement(const THFloatTensor *t) {
  if (t->nDimension <= 0) return 0;
  long n = 1;
  for (int d = 0; d < t->nDimension; d++) n *= t->size[d];
  return n;
}
THLongTensor *THLongTensor_newWithSize(THLongStorage *size, THLongStorage *stride) {
  auto *t = (THLongTensor *)calloc(1, sizeof(THLongTensor));
  t->nDimension = size ? (int)size->size : 0;
  host_shape(&t->size, &t->stride, t->nDimension, size ? size->data : nullptr, stride ? stride->data : nullptr);
  long n = host_extent(t->nDimension, t->size, t->stride);
  t->storage = THLongStorage_newWithSize(n);
  t->refcount = 1;
  t->flag = 1;
  return t;
}
void THLongTensor_free(THLongTensor *t) {
  if (!t) return;
  if (--t->refcount > 0) return;
  THLongStorage_free(t->storage);
  free(t->size);
  free(t->stride);
  free(t);
}
long THLongTensor_nElement(const THLongTensor *t) {
  if (t->nDimension <= 0) return 0;
  long n = 1;
  for (int d = 0; d < t->nDimension; d++) n *= t->size[d];
  return n;
}
#endif  // THCL_EXTERNAL_TH

// ------------------------------------------------------------------ state ---
void THCl_initializeState(THClState *state) {
  memset(state, 0, sizeof(*state));
}

void THClSetAllowNonGpus(THClState *state, int allowNonGpus) { state->allowNonGpus = allowNonGpus; }

void THClInit(THClState *state) {
  THCL_GUARD_BEGIN
  if (state->initialized) return;
  int n = thcl_rt_device_count();
  THCL_CHECK(n > 0, "no HIP device is visible: this backend has no CPU fallback");
  state->allocatedDevices = n;
  state->currentDevice = 0;
  state->scratchSpaceByDevice = (THClScratchSpace **)calloc((size_t)n, sizeof(THClScratchSpace *));
  state->deviceInfoByDevice = (void **)calloc((size_t)n, sizeof(void *));
  state->clByDevice = (thcl_rt **)calloc((size_t)n, sizeof(thcl_rt *));
  state->initialized = 1;
  THCL_GUARD_END()
}

void THClShutdown(THClState *state) {
  if (!state->initialized) return;
  for (int d = 0; d < state->allocatedDevices; d++) free(state->scratchSpaceByDevice[d]);
  free(state->scratchSpaceByDevice);
  free(state->deviceInfoByDevice);
  free(state->clByDevice);
  state->scratchSpaceByDevice = nullptr;
  state->deviceInfoByDevice = nullptr;
  state->clByDevice = nullptr;
  state->initialized = 0;
  thcl_rt_release_all();
}

int THClState_getNumDevices(THClState *state) { return state->allocatedDevices; }

void THClState_setDevice(THClState *state, int device) {
  THCL_GUARD_BEGIN
  THCL_CHECK(device >= 0 && device < state->allocatedDevices, "device %d out of range [0,%d)", device,
             state->allocatedDevices);
  state->currentDevice = device;
  THCL_GUARD_END()
}
int THClState_getDevice(THClState *state) { return state->currentDevice; }

struct thcl_rt *THClState_getClv2(THClState *state, int device) {
  THCL_GUARD_BEGIN
  return thcl_ctx(state, device);
  THCL_GUARD_END(nullptr)
}

struct THClScratchSpace *THClState_getDeviceScratchSpace(THClState *state, int device, int stream) {
  THCL_GUARD_BEGIN
  (void)stream;
  thcl_ctx(state, device);  // opens the device on first use
  return state->scratchSpaceByDevice[device];
  THCL_GUARD_END(nullptr)
}

size_t THClState_getDeviceScratchSpaceSize(THClState *state, int device) {
  THCL_GUARD_BEGIN
  size_t b = 0;
  thcl_rt_scratch(thcl_ctx(state, device), &b);
  return b;
  THCL_GUARD_END(0)
}

struct thcl_rt *THClState_getCl(THClState *state) { return THClState_getClv2(state, state->currentDevice); }
struct thcl_rt *THClState_getClAndDevice(THClState *state, int *p_device) {
  if (p_device) *p_device = state->currentDevice;
  return THClState_getClv2(state, state->currentDevice);
}
struct THClScratchSpace *THClState_getCurrentDeviceScratchSpace(THClState *state) {
  return THClState_getDeviceScratchSpace(state, state->currentDevice, 0);
}
size_t THClState_getCurrentDeviceScratchSpaceSize(THClState *state) {
  return THClState_getDeviceScratchSpaceSize(state, state->currentDevice);
}

void THClState_synchronize(THClState *state) {
  THCL_GUARD_BEGIN
  for (int d = 0; d < state->allocatedDevices; d++)
    if (state->clByDevice[d]) THCL_CHECK(thcl_rt_sync(state->clByDevice[d]) == 0, "%s", thcl_rt_error());
  THCL_GUARD_END()
}

}  // extern "C"

thcl_rt *thcl_ctx(THClState *state, int device) {
  THCL_CHECK(state && state->initialized, "THClInit has not been called");
  THCL_CHECK(device >= 0 && device < state->allocatedDevices, "device %d out of range [0,%d)", device,
             state->allocatedDevices);
  if (!state->clByDevice[device]) {
    thcl_rt *rt = thcl_rt_get(device);
    THCL_CHECK(rt != nullptr, "cannot open device %d: %s", device, thcl_rt_error());
    thcl_reduce_static_setup(device);
    state->clByDevice[device] = rt;
    state->deviceInfoByDevice[device] = (void *)thcl_rt_get_props(rt);
    auto *sp = (THClScratchSpace *)calloc(1, sizeof(THClScratchSpace));
    sp->wrapper = thcl_rt_scratch(rt, nullptr);
    sp->data = thcl_rt_host_word(rt);
    state->scratchSpaceByDevice[device] = sp;
  }
  prof_open(state->clByDevice[device]);
  return state->clByDevice[device];
}

void thcl_after_launch(THClState *state, thcl_rt *rt) {
  prof_close(rt);
  if (state->addFinish) THCL_CHECK(thcl_rt_sync(rt) == 0, "%s", thcl_rt_error());
}

void thcl_check_same_device(THClState *state, int n, ...) {
  // reference: src/lib/THClTensor.cpp:844-873 (all operands on one device)
  (void)state;
  va_list ap;
  va_start(ap, n);
  int dev = -1;
  bool ok = true;
  for (int i = 0; i < n; i++) {
    THClTensor *t = va_arg(ap, THClTensor *);
    if (!t) continue;
    int d = t->storage ? t->storage->device : t->device;
    if (dev < 0) dev = d;
    else if (d != dev) ok = false;
  }
  va_end(ap);
  THCL_CHECK(ok, "tensors are on different devices");
}

extern "C" {
// `cltorch.setProfiling(on)` (src/init.cpp:166-178)
void THClState_setProfiling(THClState *state, int on) {
  (void)state;
  g_prof_on = on != 0;
}
// `cltorch.dumpProfiling()` (src/init.cpp:149-157): waits for the device, writes one
// line per entry point -- launches, total and mean milliseconds -- into `buf`
// (always NUL-terminated within `cap`), forgets the records, and returns the
// number of characters the full report needs.
long THClState_dumpProfiling(THClState *state, char *buf, long cap) {
  THCL_GUARD_BEGIN
  for (int d = 0; d < state->allocatedDevices; d++)
    if (state->clByDevice[d]) THCL_CHECK(thcl_rt_sync(state->clByDevice[d]) == 0, "%s", thcl_rt_error());
  std::map<std::string, std::pair<long, double>> agg;
  for (auto &r : g_prof_records) {
    auto &a = agg[r.entry];
    a.first += 1;
    a.second += (double)thcl_rt_timer_ms(r.timer);
    thcl_rt_timer_free(r.timer);
  }
  g_prof_records.clear();
  std::vector<std::pair<std::string, std::pair<long, double>>> rows(agg.begin(), agg.end());
  std::sort(rows.begin(), rows.end(), [](const auto &x, const auto &y) { return x.second.second > y.second.second; });
  std::string out = "entry point, launches, total ms, mean ms\n";
  char line[256];
  for (auto &r : rows) {
    snprintf(line, sizeof(line), "%s, %ld, %.4f, %.4f\n", r.first.c_str(), r.second.first, r.second.second,
             r.second.second / (double)r.second.first);
    out += line;
  }
  if (buf && cap > 0) {
    const size_t n = out.size() < (size_t)cap - 1 ? out.size() : (size_t)cap - 1;
    memcpy(buf, out.data(), n);
    buf[n] = 0;
  }
  return (long)out.size();
  THCL_GUARD_END(-1)
}
}  // extern "C"
