// CPU driver for cltorch_amd/csrc/host_copiers.h: the copier threads, the piece loops of the staged copies and the
// upload ring, with host memory standing in for the device and a DMA that finishes late (a helper thread per
// transfer would hide ordering mistakes; here a transfer is only carried out when the loop waits for it or drains,
// so a piece whose buffer is reused too early is seen as wrong bytes).  Built by tests/test_host_sanitizers.py
// under the thread sanitizer and under the address + undefined-behaviour sanitizers.
#include <sys/wait.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#include "host_copiers.h"

using namespace thcl_host;

#define CHECK(c)                                                     \
  do {                                                               \
    if (!(c)) {                                                      \
      printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c);          \
      return 1;                                                      \
    }                                                                \
  } while (0)

// "device" = a host array; transfers are queued and carried out lazily, in order
struct LazyDma {
  std::vector<char> &dev;
  std::vector<std::vector<char>> &bufs = shared_bufs();   // one set for the whole run: 48 MiB that need not be mapped again and again
  static std::vector<std::vector<char>> &shared_bufs() {
    static std::vector<std::vector<char>> b(kStages, std::vector<char>(kStageBytes));
    return b;
  }
  struct Op { bool up; int b; size_t off, bytes; };
  std::vector<Op> queue;
  size_t done = 0;
  int last_use[kStages];
  int fail_at = -1, ops = 0;
  explicit LazyDma(std::vector<char> &d) : dev(d) {
    for (int &u : last_use) u = -1;
  }
  void *stage(int b) { return bufs[b].data(); }
  void carry(size_t upto) {
    for (; done < upto; done++) {
      const Op &o = queue[done];
      if (o.up) memcpy(dev.data() + o.off, bufs[o.b].data(), o.bytes);
      else memcpy(bufs[o.b].data(), dev.data() + o.off, o.bytes);
    }
  }
  int wait(int b) {
    if (last_use[b] >= 0) carry((size_t)last_use[b] + 1);
    return 0;
  }
  int push(bool up, int b, size_t off, size_t bytes) {
    if (ops++ == fail_at) return -7;
    if (off + bytes > dev.size() || bytes > kStageBytes) return -9;
    queue.push_back({up, b, off, bytes});
    last_use[b] = (int)queue.size() - 1;
    return 0;
  }
  int to_device(size_t off, int b, size_t bytes) { return push(true, b, off, bytes); }
  int to_host(int b, size_t off, size_t bytes) { return push(false, b, off, bytes); }
  int drain() {
    carry(queue.size());
    return 0;
  }
};

static uint32_t mix(uint64_t i) { return (uint32_t)((i * 0x9E3779B97F4A7C15ull) >> 29); }

static int round_trip_bytes(HostCopiers &pool, size_t bytes) {
  std::vector<char> host(bytes), dev(bytes, 0), back(bytes, 0);
  for (size_t i = 0; i < bytes; i++) host[i] = (char)mix(i);
  {
    LazyDma dma(dev);
    const size_t piece = staged_piece_bytes(bytes);
    CHECK(staged_upload(dma, bytes, 1, piece, [&](void *st, size_t first, size_t n) { pool.copy(st, host.data() + first, n); }) == 0);
    CHECK(dev == host);
  }
  {
    LazyDma dma(dev);
    const size_t piece = staged_piece_bytes(bytes);
    CHECK(staged_download(dma, bytes, 1, piece, [&](size_t first, void *st, size_t n) { pool.copy(back.data() + first, st, n); }) == 0);
    CHECK(dma.done == dma.queue.size());   // nothing left pending
    CHECK(back == host);
  }
  return 0;
}

template <class T>
static int round_trip_converted(HostCopiers &pool, size_t count) {
  std::vector<T> host(count), back(count);
  std::vector<char> dev(count * sizeof(float), 0);
  for (size_t i = 0; i < count; i++) host[i] = (T)(mix(i) % 200);
  LazyDma up(dev);
  const size_t piece = converted_piece_elems(count);
  CHECK(staged_upload(up, count, sizeof(float), piece, [&](void *stage, size_t first, size_t n) {
          float *st = (float *)stage;
          const T *from = host.data() + first;
          pool.run(n, [&](size_t a, size_t b) { for (size_t i = a; i < b; i++) st[i] = (float)from[i]; });
        }) == 0);
  const float *d = (const float *)dev.data();
  for (size_t i = 0; i < count; i++) CHECK(d[i] == (float)host[i]);
  LazyDma down(dev);
  CHECK(staged_download(down, count, sizeof(float), piece, [&](size_t first, void *stage, size_t n) {
          const float *st = (const float *)stage;
          T *to = back.data() + first;
          pool.run(n, [&](size_t a, size_t b) { for (size_t i = a; i < b; i++) to[i] = (T)st[i]; });
        }) == 0);
  CHECK(back == host);
  return 0;
}

static int pool_checks(int threads, bool heavy) {
  HostCopiers pool(threads);
  CHECK((int)pool.threads() == threads);
  // every index of [0, n) is visited exactly once, on both sides of the wake-up threshold and of page multiples
  const size_t lens[] = {0, 1, 4095, (1u << 18) - 1, 1u << 18, (1u << 18) + 1, (1u << 20) - 1, 1u << 20, (1u << 20) + 4097, 5000000};
  for (size_t n : lens) {
    std::vector<unsigned char> hits(n, 0);
    pool.run(n, [&](size_t a, size_t b) { for (size_t i = a; i < b; i++) hits[i]++; });
    for (size_t i = 0; i < n; i++) CHECK(hits[i] == 1);
  }
  // two callers at once take turns
  std::vector<char> a(3 << 20, 1), b(3 << 20, 2), da(3 << 20), db(3 << 20);
  std::thread t1([&] { for (int r = 0; r < 20; r++) pool.copy(da.data(), a.data(), a.size()); });
  std::thread t2([&] { for (int r = 0; r < 20; r++) pool.copy(db.data(), b.data(), b.size()); });
  t1.join();
  t2.join();
  CHECK(da == a && db == b);
  // copies: every piece boundary of the staged loops (2 MiB pieces up to three and past three buffers, 16 MiB pieces)
  const size_t sizes[] = {2048, 65536, (2u << 20) - 1, 2u << 20, (2u << 20) + 1, (6u << 20) - 3, 6u << 20, (6u << 20) + 5, (8u << 20) + 1};
  for (size_t s : sizes) CHECK(round_trip_bytes(pool, s) == 0);
  CHECK(round_trip_converted<double>(pool, 65536) == 0);
  CHECK(round_trip_converted<long>(pool, (1u << 19) + 1) == 0);
  CHECK(round_trip_converted<unsigned char>(pool, (3u << 19) + 17) == 0);
  if (heavy) {   // pieces of more than 2 MiB, and of the full 16
    CHECK(round_trip_bytes(pool, (20u << 20) + 12345) == 0);
    CHECK(round_trip_bytes(pool, (64u << 20) + 1) == 0);
    CHECK(round_trip_converted<short>(pool, (9u << 20) + 3) == 0);
  }
  // a DMA that fails in the middle: the loop drains what it queued and reports the failure
  {
    const size_t bytes = 20u << 20;
    std::vector<char> host(bytes, 5), dev(bytes, 0);
    LazyDma dma(dev);
    dma.fail_at = 2;
    CHECK(staged_upload(dma, bytes, 1, staged_piece_bytes(bytes), [&](void *st, size_t first, size_t n) { pool.copy(st, host.data() + first, n); }) == -7);
    CHECK(dma.done == dma.queue.size());
    LazyDma dma2(dev);
    dma2.fail_at = 3;   // the request that refills the first buffer
    std::vector<char> back(bytes);
    CHECK(staged_download(dma2, bytes, 1, staged_piece_bytes(bytes), [&](size_t first, void *st, size_t n) { pool.copy(back.data() + first, st, n); }) == -7);
    CHECK(dma2.done == dma2.queue.size());
  }
  return 0;
}

int main() {
  CHECK(staged_piece_bytes(2048) == (2u << 20) && staged_piece_bytes(40u << 20) == (10u << 20) && staged_piece_bytes(1u << 30) == kStageBytes);
  CHECK(converted_piece_elems(65536) == (1u << 19) && converted_piece_elems(1u << 28) == kStageBytes / 4);
  // the upload ring comes round after 16 uploads and only then asks to wait
  {
    UploadRing ring;
    bool w;
    for (unsigned i = 0; i < 16; i++) {
      CHECK(ring.take(&w) == i && !w);
    }
    for (unsigned i = 0; i < 40; i++) {
      CHECK(ring.take(&w) == i % 16 && w);
    }
  }
  for (int threads : {0, 1, 3, 8}) CHECK(pool_checks(threads, threads == 3) == 0);
  // the process-wide pool: shutdown joins, the next get() starts over; a forked child starts its own
  HostCopiers &p = HostCopiers::get(4);
  CHECK(p.threads() == 4);
  std::vector<char> src(4 << 20, 7), dst(4 << 20, 0);
  p.copy(dst.data(), src.data(), src.size());
  CHECK(dst == src);
  fflush(stdout);
  const pid_t child = fork();
  if (child == 0) {
    HostCopiers &q = HostCopiers::get(2);
    std::vector<char> d2(4 << 20, 0);
    q.copy(d2.data(), src.data(), src.size());
    _exit(d2 == src && q.threads() == 2 ? 0 : 3);
  }
  int status = 0;
  CHECK(waitpid(child, &status, 0) == child && WIFEXITED(status) && WEXITSTATUS(status) == 0);
  HostCopiers::shutdown();
  HostCopiers &again = HostCopiers::get(2);
  CHECK(again.threads() == 2);
  std::fill(dst.begin(), dst.end(), 0);
  again.copy(dst.data(), src.data(), src.size());
  CHECK(dst == src);
  HostCopiers::shutdown();
  printf("host copiers ok\n");
  return 0;
}
