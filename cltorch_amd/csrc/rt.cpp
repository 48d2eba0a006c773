// Thin HIP runtime layer behind thcl_rt.h: device contexts, buffers, the
// in-order stream, the hipRTC kernel cache and event timers.
#include "thcl_rt.h"

#include "host_copiers.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>
#include <pthread.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <chrono>
#include <cstring>
#include <condition_variable>
#include <functional>
#include <map>
#include <unordered_map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

struct thcl_rt_kernel {
  hipFunction_t fn = nullptr;
};

// one compiled source: its code object and the entry points looked up so far
struct RtModule {
  hipModule_t module = nullptr;
  std::map<std::string, thcl_rt_kernel *> entries;
};

struct thcl_rt {
  int device = -1;
  hipStream_t stream = nullptr;
  void *scratch = nullptr;
  size_t scratch_bytes = 0;
  float *host_word = nullptr;
  float *host_word_dev = nullptr;  // the same words as the device addresses them
  unsigned tag = 0;                // last tag handed out for the tagged word pair
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  thcl_rt_props props{};
  std::map<std::string, RtModule *> modules;
  // block cache of thcl_rt_malloc / thcl_rt_free
  std::unordered_map<void *, size_t> live;     // blocks handed out: pointer -> allocated bytes
  std::multimap<size_t, void *> cached;        // released blocks by size
  size_t cached_bytes = 0, live_bytes = 0, cache_limit = 0;
  unsigned long long device_mallocs = 0, cache_hits = 0;
  // page-locked staging buffers of the large copies from and to ordinary host memory (made at the first such copy)
  void *stage[3] = {nullptr, nullptr, nullptr};
  hipEvent_t stage_done[3] = {nullptr, nullptr, nullptr};
  // small uploads leave through a ring of page-locked slots and do not wait for their DMA
  char *ring = nullptr;
  hipEvent_t ring_done[16] = {};
  thcl_host::UploadRing ring_state;
};

struct thcl_rt_timer {
  thcl_rt *rt;
  hipEvent_t a, b;
};

namespace {
constexpr int kMaxDevices = 64;
constexpr size_t kScratchBytes = 8u << 20;
constexpr size_t kMailboxFloats = 16384;   // behind the 64 pinned words: room for a small tensor on its way to the host
thcl_rt *g_ctx[kMaxDevices] = {nullptr};
std::mutex g_mu;
// What the embedding process allows the host side to do; both are read when the first context is opened.
int g_copy_threads = 1;          // THCL_HOST_COPY_THREADS (0: the library starts no thread)
long g_scalar_spin_us = 2000;    // THCL_SCALAR_SPIN_US: how long a scalar-returning call polls before it waits for the stream (0: never polls)
thread_local std::string g_err;

int fail(const char *what, hipError_t e) {
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return -1;
}
#define RT_CHECK(call)                                  \
  do {                                                  \
    hipError_t e_ = (call);                             \
    if (e_ != hipSuccess) return fail(#call, e_);       \
  } while (0)

struct DeviceGuard {
  int prev = -1;
  explicit DeviceGuard(int d) {
    if (hipGetDevice(&prev) != hipSuccess) prev = -1;
    if (prev != d) (void)hipSetDevice(d);
  }
};
}  // namespace

extern "C" {

const char *thcl_rt_error(void) { return g_err.c_str(); }

int thcl_rt_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

thcl_rt *thcl_rt_get(int device) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (device < 0 || device >= kMaxDevices) {
    g_err = "device index out of range";
    return nullptr;
  }
  if (g_ctx[device]) return g_ctx[device];
  int n = thcl_rt_device_count();
  if (device >= n) {
    g_err = "no such HIP device: " + std::to_string(device) + " (visible: " + std::to_string(n) + ")";
    return nullptr;
  }
  hipError_t e = hipSetDevice(device);
  if (e != hipSuccess) {
    fail("hipSetDevice", e);
    return nullptr;
  }
  auto *rt = new thcl_rt();
  rt->device = device;
  hipDeviceProp_t p;
  e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) {
    fail("hipGetDeviceProperties", e);
    delete rt;
    return nullptr;
  }
  snprintf(rt->props.name, sizeof(rt->props.name), "%s", p.name);
  snprintf(rt->props.arch, sizeof(rt->props.arch), "%s", p.gcnArchName);
  // The kernels are built for gfx950 only, and their hand-overs between blocks (relaxed device-scope atomics plus
  // waits for store acknowledgements) rely on that chip's cache rules: another device is refused, not tried.
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    g_err = std::string("device ") + std::to_string(device) + " is a " + p.gcnArchName + ": this library is built for gfx950 (MI355X) only";
    delete rt;
    return nullptr;
  }
  rt->props.compute_units = p.multiProcessorCount;
  rt->props.wavefront = p.warpSize;
  rt->props.max_threads_per_block = p.maxThreadsPerBlock;
  rt->props.clock_khz = p.clockRate;
  rt->props.lds_bytes_per_block = (int)p.sharedMemPerBlock;
  rt->props.total_mem = p.totalGlobalMem;
  e = hipStreamCreateWithFlags(&rt->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    fail("hipStreamCreateWithFlags", e);
    delete rt;
    return nullptr;
  }
  e = hipMalloc(&rt->scratch, kScratchBytes);
  if (e == hipSuccess) e = hipMemset(rt->scratch, 0, kScratchBytes);
  if (e == hipSuccess) e = hipHostMalloc((void **)&rt->host_word, (64 + kMailboxFloats) * sizeof(float), hipHostMallocMapped);
  if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&rt->host_word_dev, rt->host_word, 0);
  if (e == hipSuccess) e = hipDeviceSynchronize();
  if (e != hipSuccess) {
    fail("scratch allocation", e);
    delete rt;
    return nullptr;
  }
  rt->scratch_bytes = kScratchBytes;
  rt->cache_limit = rt->props.total_mem / 2;
  if (const char *mb = getenv("THCL_ALLOC_CACHE_MB")) rt->cache_limit = (size_t)strtoull(mb, nullptr, 10) << 20;
  g_copy_threads = thcl_host::copy_threads_setting();
  if (const char *us = getenv("THCL_SCALAR_SPIN_US")) {
    char *end = nullptr;
    const long v = strtol(us, &end, 10);
    if (end != us && v >= 0) g_scalar_spin_us = v;
  }
  g_ctx[device] = rt;
  return rt;
}

void thcl_rt_release_all(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  for (int d = 0; d < kMaxDevices; d++) {
    thcl_rt *rt = g_ctx[d];
    if (!rt) continue;
    DeviceGuard g(d);
    (void)hipStreamSynchronize(rt->stream);
    for (auto &kv : rt->modules) {
      for (auto &e : kv.second->entries) delete e.second;
      if (kv.second->module) (void)hipModuleUnload(kv.second->module);
      delete kv.second;
    }
    for (auto &kv : rt->cached) (void)hipFree(kv.second);
    for (auto &kv : rt->live) (void)hipFree(kv.first);
    (void)hipFree(rt->scratch);
    (void)hipFree(rt->workspace);
    (void)hipHostFree(rt->host_word);
    for (int i = 0; i < 3; i++) {
      if (rt->stage[i]) (void)hipHostFree(rt->stage[i]);
      if (rt->stage_done[i]) (void)hipEventDestroy(rt->stage_done[i]);
    }
    if (rt->ring) (void)hipHostFree(rt->ring);
    for (auto &e : rt->ring_done)
      if (e) (void)hipEventDestroy(e);
    (void)hipStreamDestroy(rt->stream);
    delete rt;
    g_ctx[d] = nullptr;
  }
  thcl_host::HostCopiers::shutdown();   // joined: nothing of this library keeps running once the contexts are gone
}

const thcl_rt_props *thcl_rt_get_props(thcl_rt *rt) { return &rt->props; }

// Device blocks are cached.  Every launch and copy of a context goes through its
// one in-order stream, so a block released by the host can be handed to the
// next request at once: whatever was queued on the old owner's behalf runs
// before anything the new owner queues.  That removes the stream wait and the
// hipFree (itself a device-wide wait) from every tensor release -- measured:
// a 64 MiB temporary cost 61 us around a 10 us kernel before, 12 us now.
// A request takes the smallest cached block that fits and is at most a
// quarter larger; nothing is split.  The cache holds at most `cache_limit`
// bytes (half the device's memory, or THCL_ALLOC_CACHE_MB; 0 turns caching
// off) and is emptied when hipMalloc fails.
static size_t round_request(size_t bytes) {
  if (bytes < 4) bytes = 4;
  const size_t g = bytes <= (1u << 20) ? 512 : (64u << 10);
  return (bytes + g - 1) / g * g;
}
static void drop_cached(thcl_rt *rt) {
  if (rt->cached.empty()) return;
  (void)hipStreamSynchronize(rt->stream);  // queued work may still use the blocks
  for (auto &kv : rt->cached) (void)hipFree(kv.second);
  rt->cached.clear();
  rt->cached_bytes = 0;
}

void *thcl_rt_malloc(thcl_rt *rt, size_t bytes) {
  DeviceGuard g(rt->device);
  const size_t want = round_request(bytes);
  auto it = rt->cached.lower_bound(want);
  if (it != rt->cached.end() && it->first <= want + want / 4) {
    void *p = it->second;
    rt->live[p] = it->first;
    rt->live_bytes += it->first;
    rt->cached_bytes -= it->first;
    rt->cached.erase(it);
    rt->cache_hits++;
    return p;
  }
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, want);
  if (e != hipSuccess) {  // give the cache back to the driver and try once more
    (void)hipGetLastError();
    drop_cached(rt);
    e = hipMalloc(&p, want);
  }
  if (e != hipSuccess) {
    fail("hipMalloc", e);
    return nullptr;
  }
  rt->device_mallocs++;
  rt->live[p] = want;
  rt->live_bytes += want;
  return p;
}

int thcl_rt_free(thcl_rt *rt, void *dptr) {
  if (!dptr) return 0;
  DeviceGuard g(rt->device);
  auto it = rt->live.find(dptr);
  if (it == rt->live.end()) {  // not from thcl_rt_malloc: release it the slow way
    RT_CHECK(hipStreamSynchronize(rt->stream));
    RT_CHECK(hipFree(dptr));
    return 0;
  }
  const size_t size = it->second;
  rt->live.erase(it);
  rt->live_bytes -= size;
  if (rt->cached_bytes + size <= rt->cache_limit) {
    rt->cached.emplace(size, dptr);
    rt->cached_bytes += size;
    return 0;
  }
  RT_CHECK(hipStreamSynchronize(rt->stream));
  RT_CHECK(hipFree(dptr));
  return 0;
}

int thcl_rt_empty_cache(thcl_rt *rt) {
  DeviceGuard g(rt->device);
  drop_cached(rt);
  return 0;
}

void thcl_rt_memory_stats(thcl_rt *rt, size_t *live_bytes, size_t *cached_bytes, unsigned long long *device_mallocs,
                          unsigned long long *cache_hits) {
  if (live_bytes) *live_bytes = rt->live_bytes;
  if (cached_bytes) *cached_bytes = rt->cached_bytes;
  if (device_mallocs) *device_mallocs = rt->device_mallocs;
  if (cache_hits) *cache_hits = rt->cache_hits;
}

static int check_fault(thcl_rt *rt);

// ---- large copies from and to ordinary (pageable) host memory -------------------------------------------
// The driver moves such memory through a staging area of its own, one thread copying: 256 MiB come back at
// 10-18 GB/s and go out at 30, against 57 GB/s both ways for page-locked memory, and its time for 256 KiB to 1 MiB
// jumps about (256 KiB: 115 us, 512 KiB: 35 us; 1 MiB up: 47 or 221 us from run to run).  From kStagedFrom bytes up
// the copy is cut into pieces that travel through three page-locked buffers of this library: the DMA of one piece
// runs while a few host threads move the piece before it between its buffer and the caller's memory (256 MiB:
// 50 GB/s back into touched memory, 41-46 into a new array, 48-52 out; 256 KiB: 27 us).  The threads and the piece
// loops live in host_copiers.h; THCL_HOST_COPY_THREADS=0 keeps the library from starting any thread, and float
// copies then go the driver's way.
namespace {
using thcl_host::HostCopiers;
using thcl_host::kStageBytes;
using thcl_host::kStages;
constexpr size_t kStagedFrom = 2u << 10;   // (64 KiB up: 39 -> 18 us, 4 KiB: 18 -> 14 us; a few bytes stay with the driver)

// page-locked memory (this library's or anybody's) goes the direct way
bool host_memory_is_pagelocked(const void *p) {
  hipPointerAttribute_t a;
  memset(&a, 0, sizeof(a));
  if (hipPointerGetAttributes(&a, p) != hipSuccess) {
    (void)hipGetLastError();   // ordinary memory is unknown to the runtime: that is the answer, not an error
    return false;
  }
  return a.type == hipMemoryTypeHost;
}

int stage_ready(thcl_rt *rt) {
  for (int i = 0; i < kStages; i++) {
    if (!rt->stage[i]) RT_CHECK(hipHostMalloc(&rt->stage[i], kStageBytes, hipHostMallocDefault));
    if (!rt->stage_done[i]) RT_CHECK(hipEventCreateWithFlags(&rt->stage_done[i], hipEventDisableTiming));
  }
  return 0;
}

// the DMA side of the piece loops: the context's stream, its three staging buffers and their events
struct StreamDma {
  thcl_rt *rt;
  char *dev;
  void *stage(int b) { return rt->stage[b]; }
  int wait(int b) {
    RT_CHECK(hipEventSynchronize(rt->stage_done[b]));
    return 0;
  }
  int to_device(size_t off, int b, size_t bytes) {
    RT_CHECK(hipMemcpyAsync(dev + off, rt->stage[b], bytes, hipMemcpyHostToDevice, rt->stream));
    RT_CHECK(hipEventRecord(rt->stage_done[b], rt->stream));
    return 0;
  }
  int to_host(int b, size_t off, size_t bytes) {
    RT_CHECK(hipMemcpyAsync(rt->stage[b], dev + off, bytes, hipMemcpyDeviceToHost, rt->stream));
    RT_CHECK(hipEventRecord(rt->stage_done[b], rt->stream));
    return 0;
  }
  int drain() {
    RT_CHECK(hipStreamSynchronize(rt->stream));
    return 0;
  }
};

// to_device: host -> staging (threads) -> device (DMA); otherwise device -> staging (DMA) -> host (threads)
int staged_copy(thcl_rt *rt, char *dev, char *host, size_t bytes, bool to_device) {
  if (stage_ready(rt) != 0) return -1;
  HostCopiers &copiers = HostCopiers::get();
  StreamDma dma{rt, dev};
  const size_t piece = thcl_host::staged_piece_bytes(bytes);
  if (to_device)
    return thcl_host::staged_upload(dma, bytes, 1, piece, [&](void *st, size_t first, size_t n) { copiers.copy(st, host + first, n); });
  return thcl_host::staged_download(dma, bytes, 1, piece, [&](size_t first, void *st, size_t n) { copiers.copy(host + first, st, n); });
}
// host elements of another type <-> device floats, converted by the host threads on the way through the buffers
extern "C++" {
template <class T>
int staged_convert(thcl_rt *rt, float *dev, T *host, size_t count, bool to_device) {
  if (stage_ready(rt) != 0) return -1;
  HostCopiers &copiers = HostCopiers::get();
  StreamDma dma{rt, (char *)dev};
  const size_t piece = thcl_host::converted_piece_elems(count);
  if (to_device)
    return thcl_host::staged_upload(dma, count, sizeof(float), piece, [&](void *stage, size_t first, size_t n) {
      float *st = (float *)stage;
      const T *from = host + first;
      copiers.run(n, [&](size_t i0, size_t i1) {
        for (size_t i = i0; i < i1; i++) st[i] = (float)from[i];
      });
    });
  return thcl_host::staged_download(dma, count, sizeof(float), piece, [&](size_t first, void *stage, size_t n) {
    const float *st = (const float *)stage;
    T *to = host + first;
    copiers.run(n, [&](size_t i0, size_t i1) {
      for (size_t i = i0; i < i1; i++) to[i] = (T)st[i];
    });
  });
}
}  // extern "C++"
}  // namespace

int thcl_rt_copy_converted(thcl_rt *rt, void *dev, void *host, size_t count, int kind, int to_device) {
  if (!count) return 0;
  DeviceGuard g(rt->device);
  int rc;
  switch (kind) {
    case THCL_RT_U8: rc = staged_convert(rt, (float *)dev, (unsigned char *)host, count, to_device != 0); break;
    case THCL_RT_I8: rc = staged_convert(rt, (float *)dev, (char *)host, count, to_device != 0); break;
    case THCL_RT_I16: rc = staged_convert(rt, (float *)dev, (short *)host, count, to_device != 0); break;
    case THCL_RT_I32: rc = staged_convert(rt, (float *)dev, (int *)host, count, to_device != 0); break;
    case THCL_RT_I64: rc = staged_convert(rt, (float *)dev, (long *)host, count, to_device != 0); break;
    case THCL_RT_F64: rc = staged_convert(rt, (float *)dev, (double *)host, count, to_device != 0); break;
    default: g_err = "thcl_rt_copy_converted: unknown element kind"; return -1;
  }
  if (rc != 0) return rc;
  if (to_device) return 0;
  RT_CHECK(hipStreamSynchronize(rt->stream));
  return check_fault(rt);
}

// Uploads of up to 64 KiB: the bytes are copied into the next of 16 page-locked slots and their DMA is queued on the
// stream; the call returns without waiting for it (the caller's memory is free again, and whatever uses the
// destination is queued behind the DMA).  A slot is waited for only when the ring comes round to it while its DMA is
// still pending.  4 KiB: 14 us with the wait, 5 us without.
constexpr size_t kRingSlot = 64u << 10;
constexpr unsigned kRingSlots = thcl_host::UploadRing::kSlots;
static int ring_upload(thcl_rt *rt, void *dst, const void *src, size_t bytes) {
  if (!rt->ring) {   // the events first, the buffer last: a ring that exists is complete
    for (unsigned i = 0; i < kRingSlots; i++)
      if (!rt->ring_done[i]) RT_CHECK(hipEventCreateWithFlags(&rt->ring_done[i], hipEventDisableTiming));
    RT_CHECK(hipHostMalloc((void **)&rt->ring, kRingSlot * kRingSlots, hipHostMallocDefault));
  }
  bool must_wait;
  const unsigned slot = rt->ring_state.take(&must_wait);
  if (must_wait) RT_CHECK(hipEventSynchronize(rt->ring_done[slot]));
  char *at = rt->ring + (size_t)slot * kRingSlot;
  memcpy(at, src, bytes);
  RT_CHECK(hipMemcpyAsync(dst, at, bytes, hipMemcpyHostToDevice, rt->stream));
  RT_CHECK(hipEventRecord(rt->ring_done[slot], rt->stream));
  return 0;
}

int thcl_rt_memcpy_h2d(thcl_rt *rt, void *dst, const void *src, size_t bytes) {
  if (!bytes) return 0;
  DeviceGuard g(rt->device);
  if (bytes <= kRingSlot) return ring_upload(rt, dst, src, bytes);
  if (bytes >= kStagedFrom && g_copy_threads > 0 && !host_memory_is_pagelocked(src)) return staged_copy(rt, (char *)dst, (char *)src, bytes, true);
  RT_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, rt->stream));
  RT_CHECK(hipStreamSynchronize(rt->stream));
  return 0;
}

// Word of the pinned block that kernels raise when they meet something the host should hear about
// (an index outside its range).  Looked at whenever the host has waited for the stream.
constexpr int kFaultWord = 32;
static int check_fault(thcl_rt *rt) {
  volatile unsigned *w = (volatile unsigned *)(rt->host_word + kFaultWord);
  const unsigned what = *w;
  if (what == 0u) return 0;
  *w = 0u;
  if (what == 2u) {
    g_err = "scan: the blocks of a single-pass scan did not run at the same time (a wait inside the kernel ran out); "
            "the result of that scan is not valid";
    return -3;
  }
  g_err = "index out of range: an indexing kernel met an index outside 1..size of the indexed dimension "
          "(that entry moved nothing; reported at the first wait after the launch)";
  return -3;
}

int thcl_rt_memcpy_d2h(thcl_rt *rt, void *dst, const void *src, size_t bytes) {
  if (!bytes) return 0;
  DeviceGuard g(rt->device);
  if (bytes >= kStagedFrom && g_copy_threads > 0 && !host_memory_is_pagelocked(dst)) {
    if (staged_copy(rt, (char *)src, (char *)dst, bytes, false) != 0) return -1;
    RT_CHECK(hipStreamSynchronize(rt->stream));
    return check_fault(rt);
  }
  RT_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, rt->stream));
  RT_CHECK(hipStreamSynchronize(rt->stream));
  return check_fault(rt);
}

int thcl_rt_memcpy_d2d(thcl_rt *rt, void *dst, const void *src, size_t bytes) {
  if (!bytes) return 0;
  DeviceGuard g(rt->device);
  RT_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, rt->stream));
  return 0;
}

void *thcl_rt_stream(thcl_rt *rt) { return (void *)rt->stream; }

int thcl_rt_sync(thcl_rt *rt) {
  DeviceGuard g(rt->device);
  RT_CHECK(hipStreamSynchronize(rt->stream));
  return check_fault(rt);
}

unsigned *thcl_rt_fault_word_device(thcl_rt *rt) { return (unsigned *)(rt->host_word_dev + kFaultWord); }
int thcl_rt_check_fault(thcl_rt *rt) { return check_fault(rt); }

// A pinned pair of words {value, tag} that a kernel fills with one 8-byte store, so the host can pick a
// scalar up as soon as it lands instead of waiting for the stream's completion signal.
constexpr int kTaggedWord = 40;  // 8-byte aligned
float *thcl_rt_tagged_word_device(thcl_rt *rt) { return rt->host_word_dev + kTaggedWord; }
float *thcl_rt_mailbox_device(thcl_rt *rt) { return rt->host_word_dev + 64; }
const float *thcl_rt_mailbox_host(thcl_rt *rt, size_t *floats) {
  if (floats) *floats = kMailboxFloats;
  return rt->host_word + 64;
}
unsigned thcl_rt_next_tag(thcl_rt *rt) {
  if (++rt->tag == 0u) ++rt->tag;
  return rt->tag;
}
int thcl_rt_await_tagged(thcl_rt *rt, unsigned tag, float *value) {
  volatile unsigned long long *w = (volatile unsigned long long *)(rt->host_word + kTaggedWord);
  // poll for up to 2 ms (a reduction of 2^28 elements takes 0.15 ms; THCL_SCALAR_SPIN_US sets another limit, 0 none at
  // all), then wait for the stream the ordinary way
  const auto t0 = std::chrono::steady_clock::now();
  while (g_scalar_spin_us > 0) {
    for (int i = 0; i < 64; i++) {
      const unsigned long long pair = *w;
      if ((unsigned)(pair >> 32) == tag) {
        const unsigned bits = (unsigned)pair;
        memcpy(value, &bits, sizeof(bits));
        return check_fault(rt);
      }
    }
    if (std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(g_scalar_spin_us)) break;
  }
  const int rc = thcl_rt_sync(rt);
  const unsigned long long pair = *w;
  const unsigned bits = (unsigned)pair;
  memcpy(value, &bits, sizeof(bits));
  if (rc == 0 && (unsigned)(pair >> 32) != tag) {
    g_err = "the kernel that was to hand a scalar to the host did not leave it";
    return -4;
  }
  return rc;
}

void *thcl_rt_scratch(thcl_rt *rt, size_t *bytes) {
  if (bytes) *bytes = rt->scratch_bytes;
  return rt->scratch;
}

void *thcl_rt_host_alloc(size_t bytes) {
  void *p = nullptr;
  hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault);
  if (e != hipSuccess) {
    g_err = std::string("hipHostMalloc: ") + hipGetErrorString(e);
    (void)hipGetLastError();
    return nullptr;
  }
  return p;
}
int thcl_rt_host_free(void *ptr) {
  if (!ptr) return 0;
  hipError_t e = hipHostFree(ptr);
  if (e != hipSuccess) {
    g_err = std::string("hipHostFree: ") + hipGetErrorString(e);
    return -1;
  }
  return 0;
}

float *thcl_rt_host_word(thcl_rt *rt) { return rt->host_word; }
float *thcl_rt_host_word_device(thcl_rt *rt) { return rt->host_word_dev; }

void *thcl_rt_workspace(thcl_rt *rt, size_t bytes) {
  if (bytes <= rt->workspace_bytes) return rt->workspace;
  DeviceGuard g(rt->device);
  if (rt->workspace) {
    // queued kernels may still use the old block
    if (hipStreamSynchronize(rt->stream) != hipSuccess || hipFree(rt->workspace) != hipSuccess) {
      g_err = "releasing the workspace failed";
      return nullptr;
    }
    rt->workspace = nullptr;
    rt->workspace_bytes = 0;
  }
  size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
  hipError_t e = hipMalloc(&rt->workspace, want);
  if (e != hipSuccess) {
    fail("hipMalloc(workspace)", e);
    rt->workspace = nullptr;
    return nullptr;
  }
  rt->workspace_bytes = want;
  return rt->workspace;
}

static int rtc_compile(const char *source, const char *arch, std::vector<char> &code) {
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, "thcl_user_expr.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) {
    g_err = std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r);
    return -1;
  }
  std::string archopt = std::string("--offload-arch=") + arch;
  // Contraction stays off so a*b+c rounds twice like the host arithmetic it is
  // compared with; packed fp32 instructions are kept out of the generated code,
  // as in the library's own build.
  const char *opts[] = {archopt.c_str(), "-O3", "-ffp-contract=off", "-std=c++17",
                        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  int nopts = (int)(sizeof(opts) / sizeof(opts[0]));
  r = hiprtcCompileProgram(prog, nopts, opts);
  if (r != HIPRTC_SUCCESS) {
    size_t ls = 0;
    hiprtcGetProgramLogSize(prog, &ls);
    std::string log(ls + 1, '\0');
    if (ls) hiprtcGetProgramLog(prog, &log[0]);
    g_err = std::string("expression failed to compile: ") + hiprtcGetErrorString(r) + "\n" + log.c_str();
    hiprtcDestroyProgram(&prog);
    return -1;
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  code.resize(cs);
  hiprtcGetCode(prog, code.data());
  hiprtcDestroyProgram(&prog);
  return 0;
}

int thcl_rt_compile_check(const char *source, const char *arch, size_t *code_bytes) {
  std::vector<char> code;
  int rc = rtc_compile(source, arch, code);
  if (rc == 0 && code_bytes) *code_bytes = code.size();
  return rc;
}

// Optional on-disk cache of compiled code objects, for processes that meet the
// same expressions again: THCL_KERNEL_CACHE_DIR names a directory; a file per
// (source text, architecture, compiler version) holds the code object.  Off
// when the variable is unset.  Files are written under a temporary name and
// renamed, so concurrent processes never read a partial file.
static std::string disk_cache_path(const char *source, const std::string &arch) {
  const char *dir = getenv("THCL_KERNEL_CACHE_DIR");
  if (!dir || !dir[0]) return std::string();
  int major = 0, minor = 0;
  hiprtcVersion(&major, &minor);
  unsigned long long h = 1469598103934665603ull;  // FNV-1a over everything that shapes the code
  auto mix = [&](const char *p) {
    for (; *p; p++) h = (h ^ (unsigned char)*p) * 1099511628211ull;
    h = (h ^ 0xffu) * 1099511628211ull;
  };
  mix(source);
  mix(arch.c_str());
  mix("-O3 -ffp-contract=off -std=c++17 -packed-fp32-ops");
  char name[96];
  snprintf(name, sizeof(name), "/thcl_%016llx_%zu_rtc%d.%d.hsaco", h, strlen(source), major, minor);
  return std::string(dir) + name;
}
static bool disk_cache_read(const std::string &path, std::vector<char> &code) {
  if (path.empty()) return false;
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) return false;
  fseek(f, 0, SEEK_END);
  const long n = ftell(f);
  fseek(f, 0, SEEK_SET);
  bool ok = n > 0;
  if (ok) {
    code.resize((size_t)n);
    ok = fread(code.data(), 1, (size_t)n, f) == (size_t)n;
  }
  fclose(f);
  return ok;
}
static void disk_cache_write(const std::string &path, const std::vector<char> &code) {
  if (path.empty()) return;
  char suffix[48];
  snprintf(suffix, sizeof(suffix), ".tmp%ld", (long)getpid());
  const std::string tmp = path + suffix;
  FILE *f = fopen(tmp.c_str(), "wb");
  if (!f) return;  // an unwritable cache directory only costs the next process a compile
  const bool ok = fwrite(code.data(), 1, code.size(), f) == code.size();
  fclose(f);
  if (!ok || rename(tmp.c_str(), path.c_str()) != 0) remove(tmp.c_str());
}

int thcl_rt_kernel_cached(thcl_rt *rt, const char *key) { return rt->modules.count(key) ? 1 : 0; }

// Modules are cached by `key`, entry points by (key, entry): one source holds
// several kernels and each call names the one it needs.
thcl_rt_kernel *thcl_rt_kernel_get(thcl_rt *rt, const char *key, const char *source, const char *entry) {
  DeviceGuard g(rt->device);
  RtModule *mod = nullptr;
  auto it = rt->modules.find(key);
  if (it != rt->modules.end()) {
    mod = it->second;
  } else {
    std::vector<char> code;
    // strip feature suffixes such as ":sramecc+:xnack-" from the device's arch name
    std::string arch = rt->props.arch;
    size_t colon = arch.find(':');
    if (colon != std::string::npos) arch = arch.substr(0, colon);
    const std::string cached = disk_cache_path(source, arch);
    hipError_t e = hipErrorInvalidValue;
    mod = new RtModule();
    if (disk_cache_read(cached, code)) e = hipModuleLoadData(&mod->module, code.data());
    if (e != hipSuccess) {  // nothing cached, or a file this runtime cannot load: compile
      (void)hipGetLastError();
      if (rtc_compile(source, arch.c_str(), code) != 0) {
        delete mod;
        return nullptr;
      }
      e = hipModuleLoadData(&mod->module, code.data());
      if (e == hipSuccess) disk_cache_write(cached, code);
    }
    if (e != hipSuccess) {
      fail("loading runtime-compiled code", e);
      delete mod;
      return nullptr;
    }
    rt->modules[key] = mod;
  }
  auto fit = mod->entries.find(entry);
  if (fit != mod->entries.end()) return fit->second;
  auto *k = new thcl_rt_kernel();
  hipError_t e = hipModuleGetFunction(&k->fn, mod->module, entry);
  if (e != hipSuccess) {
    fail((std::string("entry point not found in runtime-compiled code: ") + entry).c_str(), e);
    delete k;
    return nullptr;
  }
  mod->entries[entry] = k;
  return k;
}

int thcl_rt_launch(thcl_rt *rt, thcl_rt_kernel *k, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                   unsigned by, unsigned bz, unsigned lds_bytes, void *params, size_t params_bytes) {
  DeviceGuard g(rt->device);
  size_t sz = params_bytes;
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, params, HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz,
                    HIP_LAUNCH_PARAM_END};
  RT_CHECK(hipModuleLaunchKernel(k->fn, gx, gy, gz, bx, by, bz, lds_bytes, rt->stream, nullptr, config));
  return 0;
}

thcl_rt_timer *thcl_rt_timer_new(thcl_rt *rt) {
  DeviceGuard g(rt->device);
  auto *t = new thcl_rt_timer();
  t->rt = rt;
  if (hipEventCreate(&t->a) != hipSuccess || hipEventCreate(&t->b) != hipSuccess) {
    delete t;
    return nullptr;
  }
  return t;
}
int thcl_rt_timer_start(thcl_rt_timer *t) {
  RT_CHECK(hipEventRecord(t->a, t->rt->stream));
  return 0;
}
int thcl_rt_timer_stop(thcl_rt_timer *t) {
  RT_CHECK(hipEventRecord(t->b, t->rt->stream));
  return 0;
}
float thcl_rt_timer_ms(thcl_rt_timer *t) {
  float ms = -1.f;
  if (hipEventSynchronize(t->b) != hipSuccess) return -1.f;
  if (hipEventElapsedTime(&ms, t->a, t->b) != hipSuccess) return -1.f;
  return ms;
}
void thcl_rt_timer_free(thcl_rt_timer *t) {
  if (!t) return;
  (void)hipEventDestroy(t->a);
  (void)hipEventDestroy(t->b);
  delete t;
}

}  // extern "C"
