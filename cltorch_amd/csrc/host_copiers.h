// Host side of the large copies between ordinary (pageable) host memory and the device: a few threads that move
// slices of one buffer side by side, and the loops that cut a copy into pieces travelling through three page-locked
// staging buffers, the DMA of one piece running while the threads move the piece before it.  Nothing here names the
// GPU runtime: the DMA is a policy object, so the same loops run in the CPU test suite against host memory under
// the thread and address sanitizers.
//
// What it replaces: the reference moves whole storages through a host mirror with one blocking transfer
// (src/lib/THClTensorCopy.cpp:18-36,70-91, src/lib/THClStorage.cpp:225-234).
#pragma once

#include <pthread.h>

#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace thcl_host {

constexpr size_t kStageBytes = 16u << 20;
constexpr int kStages = 3;

// THCL_HOST_COPY_THREADS: how many copier threads the process may start.  0: none at all (copies of float data go
// the driver's own way, conversions run on the calling thread); unset: 8 on 16 or more hardware threads, half of
// them on 4 to 15, else 1.  Read once, when the first device context is opened.
inline int copy_threads_setting() {
  static const int value = [] {
    if (const char *s = getenv("THCL_HOST_COPY_THREADS")) {
      char *end = nullptr;
      const long v = strtol(s, &end, 10);
      if (end != s && v >= 0) return (int)(v > 64 ? 64 : v);
    }
    const unsigned n = std::thread::hardware_concurrency();
    return (int)(n >= 16 ? 8 : (n >= 4 ? n / 2 : 1));
  }();
  return value;
}

// A handful of threads that copy slices of one buffer side by side; made at the first large copy, then asleep.
class HostCopiers {
 public:
  // the process-wide pool; `threads` counts only when this call creates it
  static HostCopiers &get(int threads = copy_threads_setting()) {
    // A forked child has none of the threads, so it starts over (the parent's object is left alone: its mutexes
    // may be held by threads that do not exist in the child).
    static std::once_flag at_fork;
    std::call_once(at_fork, [] { pthread_atfork(nullptr, nullptr, [] { pool() = nullptr; }); });
    std::lock_guard<std::mutex> lk(pool_mu());
    if (!pool()) pool() = new HostCopiers(threads);
    return *pool();
  }
  // stops and joins the threads (before the library's code may be unmapped); the next get() starts new ones
  static void shutdown() {
    HostCopiers *p;
    {
      std::lock_guard<std::mutex> lk(pool_mu());
      p = pool();
      pool() = nullptr;
    }
    delete p;
  }
  explicit HostCopiers(int threads) {
    const unsigned n = threads < 0 ? 0u : (unsigned)threads;
    for (unsigned i = 0; i < n; i++) threads_.emplace_back([this, i, n] { work(i, n); });
  }
  ~HostCopiers() {
    {
      std::lock_guard<std::mutex> lock(mu_);
      stop_ = true;
      generation_++;
    }
    wake_.notify_all();
    for (auto &t : threads_) t.join();
  }
  HostCopiers(const HostCopiers &) = delete;
  HostCopiers &operator=(const HostCopiers &) = delete;
  size_t threads() const { return threads_.size(); }

  // f(first, last) over [0, n) cut into one range per thread (whole pages); short ranges and pools without
  // threads run on the caller
  void run(size_t n, const std::function<void(size_t, size_t)> &f) {
    if (n < (1u << 18) || threads_.empty()) {   // not worth waking anybody
      f(0, n);
      return;
    }
    std::lock_guard<std::mutex> one_caller(callers_);   // copies of two host threads take turns
    std::unique_lock<std::mutex> lock(mu_);
    n_ = n;
    f_ = &f;
    pending_ = (int)threads_.size();
    generation_++;
    wake_.notify_all();
    done_.wait(lock, [this] { return pending_ == 0; });
  }
  void copy(void *dst, const void *src, size_t bytes) {
    if (bytes < (1u << 20)) {
      memcpy(dst, src, bytes);
      return;
    }
    run(bytes, [&](size_t a, size_t b) { memcpy((char *)dst + a, (const char *)src + a, b - a); });
  }

 private:
  static HostCopiers *&pool() {
    static HostCopiers *p = nullptr;
    return p;
  }
  static std::mutex &pool_mu() {
    static std::mutex m;
    return m;
  }
  void work(unsigned me, unsigned n) {
    unsigned seen = 0;
    for (;;) {
      size_t count;
      const std::function<void(size_t, size_t)> *f;
      {
        std::unique_lock<std::mutex> lock(mu_);
        wake_.wait(lock, [&] { return generation_ != seen; });
        if (stop_) return;
        seen = generation_;
        count = n_;
        f = f_;
      }
      const size_t per = ((count + n - 1) / n + 4095) / 4096 * 4096;   // whole pages (of bytes) per thread
      const size_t from = (size_t)me * per;
      if (from < count) (*f)(from, count - from < per ? count : from + per);
      {
        std::lock_guard<std::mutex> lock(mu_);
        if (--pending_ == 0) done_.notify_one();
      }
    }
  }
  std::mutex mu_, callers_;
  std::condition_variable wake_, done_;
  std::vector<std::thread> threads_;
  size_t n_ = 0;
  const std::function<void(size_t, size_t)> *f_ = nullptr;
  unsigned generation_ = 0;
  int pending_ = 0;
  bool stop_ = false;
};

// A quarter of the copy per piece, between 2 and 16 MiB: small copies still overlap their halves, large ones keep
// the per-piece costs (an event wait, a wake-up of the copiers) small.
inline size_t staged_piece_bytes(size_t bytes) {
  size_t piece = (bytes / 4 + (1u << 20) - 1) >> 20 << 20;
  if (piece < (2u << 20)) piece = 2u << 20;
  if (piece > kStageBytes) piece = kStageBytes;
  return piece;
}
// In elements of the converted copies: a quarter of the copy, 512 Ki to 4 Mi floats
inline size_t converted_piece_elems(size_t count) {
  size_t piece = (count / 4 + (1u << 18) - 1) >> 18 << 18;
  if (piece < (1u << 19)) piece = 1u << 19;
  if (piece > kStageBytes / sizeof(float)) piece = kStageBytes / sizeof(float);
  return piece;
}

// The piece loop.  `units` of `unit` device bytes each move in pieces of `piece` units.  Dma provides
//   void *stage(int b)                                      the b-th staging buffer
//   int wait(int b)                                         until the last DMA that used buffer b is done
//   int to_device(size_t dev_byte_off, int b, size_t bytes) queue buffer -> device and mark the buffer busy
//   int to_host(int b, size_t dev_byte_off, size_t bytes)   queue device -> buffer and mark the buffer busy
//   int drain()                                             wait for everything queued
// (0 = ok).  host_to_stage(stage, first_unit, units) / stage_to_host(first_unit, stage, units) move one piece
// between the caller's memory and a buffer.  On an error the queue is drained before returning, so no DMA still
// points at a buffer or at the caller's memory.
template <class Dma, class In>
int staged_upload(Dma &dma, size_t units, size_t unit, size_t piece, In host_to_stage) {
  const size_t pieces = (units + piece - 1) / piece;
  auto len = [&](size_t c) { return c + 1 < pieces ? piece : units - c * piece; };
  for (size_t c = 0; c < pieces; c++) {
    const int b = (int)(c % kStages);
    int rc = c >= (size_t)kStages ? dma.wait(b) : 0;   // the buffer's last piece has left
    if (rc == 0) {
      host_to_stage(dma.stage(b), c * piece, len(c));
      rc = dma.to_device(c * piece * unit, b, len(c) * unit);
    }
    if (rc != 0) {
      (void)dma.drain();
      return rc;
    }
  }
  return dma.drain();
}
template <class Dma, class Out>
int staged_download(Dma &dma, size_t units, size_t unit, size_t piece, Out stage_to_host) {
  const size_t pieces = (units + piece - 1) / piece;
  auto len = [&](size_t c) { return c + 1 < pieces ? piece : units - c * piece; };
  int rc = 0;
  for (size_t c = 0; rc == 0 && c < pieces && c < (size_t)kStages; c++) rc = dma.to_host((int)c, c * piece * unit, len(c) * unit);
  for (size_t c = 0; rc == 0 && c < pieces; c++) {
    const int b = (int)(c % kStages);
    rc = dma.wait(b);
    if (rc != 0) break;
    stage_to_host(c * piece, dma.stage(b), len(c));
    const size_t next = c + kStages;
    if (next < pieces) rc = dma.to_host(b, next * piece * unit, len(next) * unit);
  }
  if (rc != 0) (void)dma.drain();
  return rc;
}

// Small uploads leave through a ring of page-locked slots without waiting for their DMA: which slot is next, and
// whether it has to be waited for first.
struct UploadRing {
  static constexpr unsigned kSlots = 16;
  unsigned next = 0;
  bool used[kSlots] = {};
  // the slot to use now; *must_wait: its previous DMA may still be pending
  unsigned take(bool *must_wait) {
    const unsigned slot = next;
    next = (slot + 1) % kSlots;
    *must_wait = used[slot];
    used[slot] = true;
    return slot;
  }
};

}  // namespace thcl_host
