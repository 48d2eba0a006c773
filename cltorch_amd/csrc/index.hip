// Indexed movement: indexSelect / indexCopy / indexFill along a dimension,
// gather / scatter / scatterFill, maskedSelect / maskedCopy.
//
// What it replaces (reference): src/lib/THClTensorIndex.cpp:16-330 (one thread
// per slice position looping over the whole index vector), src/lib/THClGather.cpp,
// src/lib/THClScatter.cpp (one thread per index element, per-element div/mod
// over every dim) and src/lib/THClTensorMasked.cpp:126-246 (maskedSelect through
// boost::compute, maskedCopy left unimplemented).
//
// Indices are 1-based floats held in a ClTensor, the reference's convention.
// The indexed tensor is taken as dense [O][N][I] around the dimension; one
// thread moves one unit (4 adjacent floats along I where alignment allows), so
// accesses coalesce along I and the index vector is read from cache.  An index
// outside 1..N (or NaN) moves nothing and raises a pinned flag word that the
// host reports as "index out of range" at its next wait for the stream (the
// reference reads or writes out of bounds; Torch's CPU path raises at once).
// All of it is bound by HBM.
#include <hip/hip_runtime.h>

#include <cstring>

#include "apply_device.h"
#include "internal.h"

namespace {

constexpr int kThreads = 256;

struct IndexParams {
  float *a;            // the tensor indexed along its dim: [O][N][I]
  float *b;            // the other one: [O][M][I]
  const float *index;  // [M] (select / copy / fill) or [O][M][I] (gather / scatter)
  int *winner;         // indexCopy: for every target slice, the last position of the index vector naming it
  unsigned *fault;     // pinned word the host looks at after its next wait: set when an index is out of range
  ThclDivisor units_i, m;  // units along I, entries along the dim
  thcl_u32 total;      // units in [O][M][I]
  thcl_u32 N, M, I;
  float value;
};

enum Mode { SELECT = 0, COPY = 1, FILL = 2, GATHER = 3, SCATTER = 4, SCATTER_FILL = 5 };

// Called by the lanes that met a bad index (inside their branch): one of them sets the pinned word, so a wave full
// of bad entries sends one store over the link to host memory, not 64.
__device__ __forceinline__ void raise_fault(unsigned *word) {
  const unsigned long long here = __builtin_amdgcn_ballot_w64(true);
  if ((int)__lane_id() == __ffsll((long long)here) - 1) *word = 1u;
}

// For duplicate targets the sequential CPU loop leaves the last source slice;
// winner[j] = max position i with index[i] == j + 1 reproduces that in parallel.
__global__ __launch_bounds__(kThreads) void index_winner(IndexParams P) {
  const thcl_u32 i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= P.M) return;
  const long j = (long)P.index[i] - 1;
  if (j >= 0 && j < (long)P.N) atomicMax(P.winner + j, (int)i);
  else raise_fault(P.fault);
}

template <int MODE, int VEC>
__global__ __launch_bounds__(kThreads) void index_move(IndexParams P) {
  typedef typename ThclVec<VEC == 4 ? 4 : 2>::T V4;  // only used when VEC == 4
  const thcl_u32 e = blockIdx.x * kThreads + threadIdx.x;
  if (e >= P.total) return;
  // e -> (o, i, unit along I)
  const thcl_u32 q = thcl_div(e, P.units_i);
  const thcl_u32 ku = e - q * P.units_i.d;
  const thcl_u32 o = thcl_div(q, P.m);
  const thcl_u32 i = q - o * P.m.d;
  const thcl_u64 k = (thcl_u64)ku * VEC;
  const thcl_u64 boff = ((thcl_u64)o * P.M + i) * P.I + k;  // position in [O][M][I]
  if (MODE == GATHER || MODE == SCATTER || MODE == SCATTER_FILL) {
    // one index per element
#pragma unroll
    for (int c = 0; c < VEC; c++) {
      const long j = (long)P.index[boff + c] - 1;
      if (j < 0 || j >= (long)P.N) {
        raise_fault(P.fault);
        continue;
      }
      const thcl_u64 aoff = ((thcl_u64)o * P.N + (thcl_u64)j) * P.I + k + c;
      if (MODE == GATHER) P.b[boff + c] = P.a[aoff];
      else if (MODE == SCATTER) P.a[aoff] = P.b[boff + c];
      else P.a[aoff] = P.value;
    }
    return;
  }
  const long j = (long)P.index[i] - 1;
  if (j < 0 || j >= (long)P.N) {
    if (ku == 0 && o == 0) raise_fault(P.fault);  // once per bad entry, not once per unit of its slice
    return;
  }
  if (MODE == COPY && P.winner[j] != (int)i) return;
  const thcl_u64 aoff = ((thcl_u64)o * P.N + (thcl_u64)j) * P.I + k;
  if (VEC == 4) {
    if (MODE == SELECT) __builtin_nontemporal_store(*(const V4 *)(P.a + aoff), (V4 *)(P.b + boff));
    else if (MODE == COPY) *(V4 *)(P.a + aoff) = __builtin_nontemporal_load((const V4 *)(P.b + boff));
    else {
      V4 v;
      v[0] = v[1] = v[2] = v[3] = P.value;
      *(V4 *)(P.a + aoff) = v;
    }
  } else {
    if (MODE == SELECT) P.b[boff] = P.a[aoff];
    else if (MODE == COPY) P.a[aoff] = P.b[boff];
    else P.a[aoff] = P.value;
  }
}

// The same movement one element per lane (inner sizes that are no multiple of 4, or unaligned tensors), eight
// elements per thread: the index entries, then the elements are all requested before the first is stored, since a
// thread's chain of index, element and store would otherwise leave too little in flight (8192 x 8191 rows selected:
// 2.4 TB/s with one element per thread).  Lanes past the end repeat the last element and store nothing.
template <int MODE>
__global__ __launch_bounds__(kThreads) void index_move_by_element(IndexParams P) {
  constexpr int U = 8;
  const thcl_u32 base = blockIdx.x * (kThreads * U) + threadIdx.x;
  thcl_u64 aoff[U], boff[U];
  bool ok[U];
  long j[U];
  thcl_u32 slice[U];
  // a thread's elements are 256 apart, so most of them lie in the slice of the first: the position is split by
  // division only where the inner index runs over
  thcl_u32 ku_prev = 0, o_prev = 0, i_prev = 0;
#pragma unroll
  for (int k = 0; k < U; k++) {
    const thcl_u32 e = base + k * kThreads, ec = e < P.total ? e : P.total - 1;
    thcl_u32 ku, o, i;
    if (k > 0 && e < P.total && ku_prev + kThreads < P.units_i.d) {
      ku = ku_prev + kThreads;
      o = o_prev;
      i = i_prev;
    } else {
      const thcl_u32 q = thcl_div(ec, P.units_i);
      ku = ec - q * P.units_i.d;
      o = thcl_div(q, P.m);
      i = q - o * P.m.d;
    }
    ku_prev = ku;
    o_prev = o;
    i_prev = i;
    slice[k] = i;
    j[k] = (long)P.index[i] - 1;
    ok[k] = e < P.total;
    boff[k] = ((thcl_u64)o * P.M + i) * P.I + ku;
    aoff[k] = (thcl_u64)o * P.N * P.I + ku;   // the slice's part is added once its index is known
    if (ku != 0 || o != 0) slice[k] |= 0x80000000u;   // only the first element of a slice reports a bad entry
  }
#pragma unroll
  for (int k = 0; k < U; k++) {
    const bool in = j[k] >= 0 && j[k] < (long)P.N;
    if (!in && ok[k] && !(slice[k] & 0x80000000u)) raise_fault(P.fault);
    ok[k] = ok[k] && in;
    aoff[k] += (thcl_u64)(in ? j[k] : 0) * P.I;
  }
  if (MODE == COPY) {
    int w[U];
#pragma unroll
    for (int k = 0; k < U; k++) w[k] = P.winner[ok[k] ? j[k] : 0];
#pragma unroll
    for (int k = 0; k < U; k++) ok[k] = ok[k] && w[k] == (int)(slice[k] & 0x7fffffffu);
  }
  if (MODE == FILL) {
#pragma unroll
    for (int k = 0; k < U; k++)
      if (ok[k]) P.a[aoff[k]] = P.value;
    return;
  }
  float v[U];
#pragma unroll
  for (int k = 0; k < U; k++) v[k] = (MODE == SELECT) ? P.a[aoff[k]] : P.b[boff[k]];
#pragma unroll
  for (int k = 0; k < U; k++) {
    if (!ok[k]) continue;
    if (MODE == SELECT) P.b[boff[k]] = v[k];
    else P.a[aoff[k]] = v[k];
  }
}

__global__ __launch_bounds__(kThreads) void fill_int(int *p, int v, thcl_u32 n) {
  const thcl_u32 i = blockIdx.x * kThreads + threadIdx.x;
  if (i < n) p[i] = v;
}

// ---------------------------------------------------------------- masked ---
// Stream compaction in three passes over blocks of kChunk elements: count the
// selected elements of every block, turn the counts into offsets (one block,
// the list is short), then every block derives its elements' ranks and moves them.
// The first pass also leaves the mask as one bit per element, so the last pass
// reads 1/32 of the mask's bytes and finds ranks by counting bits, with no
// exchange between threads.
//
// Bit layout: a chunk is 4 steps of 1024 elements; in a step thread t holds elements
// 4t .. 4t+3.  Word [chunk][step][wave][e] has bit l set when element e of lane l of
// that wave is selected.
constexpr int kPer = 16, kChunk = kThreads * kPer;
constexpr int kMaskPer = 4, kMaskStep = kThreads * kMaskPer, kMaskSteps = kChunk / kMaskStep, kMaskWaves = kThreads / 64;
constexpr int kWordsPerStep = kMaskWaves * kMaskPer, kWordsPerChunk = kMaskSteps * kWordsPerStep;

struct MaskParams {
  const float *mask;
  const float *src;   // select: [n] values; copy: the packed source
  float *dst;         // select: packed output; copy: [n] destination
  unsigned *counts;   // per block, then exclusive offsets inside the block's group of 4096
  unsigned *groups;   // per group of 4096 blocks: total, then exclusive offset; groups[ngroups] = grand total
  thcl_u32 ngroups;
  unsigned long long *bits;  // [nblocks][kWordsPerChunk]
  thcl_u64 n;
  thcl_u32 nblocks;
  thcl_u64 src_len;   // copy: elements available in src
  unsigned *ticket;   // arrival counter of the group blocks, zero between launches
  unsigned long long *host_total;  // pinned host word pair (device address) that receives {grand total, tag} in one store
  unsigned host_tag;
};

template <bool VEC>
__global__ __launch_bounds__(kThreads) void mask_count(MaskParams P) {
  __shared__ unsigned lds[kMaskWaves];
  const thcl_u64 chunk0 = (thcl_u64)blockIdx.x * kChunk;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  float m[kMaskSteps][kMaskPer];
  if (VEC && chunk0 + kChunk <= P.n) {
    // a whole chunk (the same for every thread of the block): the loads go out together, nothing between them
#pragma unroll
    for (int step = 0; step < kMaskSteps; step++) {
      const thcl_u64 first = chunk0 + (thcl_u64)step * kMaskStep + (thcl_u64)threadIdx.x * kMaskPer;
      const thcl_f4 v = __builtin_nontemporal_load((const thcl_f4 *)(P.mask + first));
#pragma unroll
      for (int e = 0; e < kMaskPer; e++) m[step][e] = v[e];
    }
  } else {
#pragma unroll
    for (int step = 0; step < kMaskSteps; step++) {
      const thcl_u64 first = chunk0 + (thcl_u64)step * kMaskStep + (thcl_u64)threadIdx.x * kMaskPer;
#pragma unroll
      for (int e = 0; e < kMaskPer; e++) m[step][e] = (first + e < P.n) ? P.mask[first + e] : 0.0f;
    }
  }
  unsigned c = 0;                // the wave's selected elements (the same in every lane)
  unsigned long long mine = 0;   // lane 4 * step + e keeps word (step, e) of this wave
#pragma unroll
  for (int step = 0; step < kMaskSteps; step++) {
#pragma unroll
    for (int e = 0; e < kMaskPer; e++) {
      const unsigned long long b = __ballot(m[step][e] != 0.0f);
      c += (unsigned)__popcll(b);
      if (lane == step * kMaskPer + e) mine = b;
    }
  }
  if (lane < kMaskSteps * kMaskPer)
    P.bits[(thcl_u64)blockIdx.x * kWordsPerChunk + (lane / kMaskPer) * kWordsPerStep + wave * kMaskPer + lane % kMaskPer] = mine;
  if (lane == 0) lds[wave] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned total = 0;
#pragma unroll
    for (int w = 0; w < kMaskWaves; w++) total += lds[w];
    P.counts[blockIdx.x] = total;
  }
}

// Block counts -> exclusive offsets in two levels, one launch.  A block of 1024
// threads turns 4096 adjacent counts into offsets within the group (4 per thread, one
// 16-byte access) and publishes the group's total; the block that arrives last turns
// the group totals into group offsets, leaves the grand total behind them and hands it
// to the host through a pinned word (the host only has to wait for the stream).
// The hand-over between the group blocks is the one of the column reductions: totals
// stored with device-scope stores (written through to where all XCDs meet), the storing
// wave waits for their acknowledgement, then takes a ticket; the last arrival reads with
// loads that bypass the caches.
constexpr int kGroup = 4096;

__device__ __forceinline__ unsigned block1024_exclusive(unsigned v, unsigned *lds, unsigned *total) {
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  unsigned incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned up = __shfl_up(incl, d, 64);
    if (lane >= d) incl += up;
  }
  if (lane == 63) lds[wave] = incl;
  __syncthreads();
  unsigned before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < 1024 / 64; w++) {
    if (w < wave) before += lds[w];
    all += lds[w];
  }
  __syncthreads();  // lds may be reused
  *total = all;
  return before + incl - v;
}

__global__ __launch_bounds__(1024) void mask_scan_groups(MaskParams P) {
  __shared__ unsigned lds[1024 / 64];
  const thcl_u64 i0 = (thcl_u64)blockIdx.x * kGroup + (thcl_u64)threadIdx.x * 4;
  unsigned v[4];
#pragma unroll
  for (int k = 0; k < 4; k++) v[k] = (i0 + k < P.nblocks) ? P.counts[i0 + k] : 0u;
  unsigned total;
  unsigned run = block1024_exclusive(v[0] + v[1] + v[2] + v[3], lds, &total);
#pragma unroll
  for (int k = 0; k < 4; k++) {
    if (i0 + k < P.nblocks) P.counts[i0 + k] = run;
    run += v[k];
  }
  __shared__ unsigned s_last;
  if (threadIdx.x == 0) {
    __hip_atomic_store(P.groups + blockIdx.x, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned t = atomicAdd(P.ticket, 1u);
    s_last = (t == gridDim.x - 1) ? 1u : 0u;
  }
  __syncthreads();
  if (!s_last) return;
  unsigned carry = 0;
  for (thcl_u32 g0 = 0; g0 < P.ngroups; g0 += 1024) {
    const thcl_u32 g = g0 + threadIdx.x;
    const unsigned v = g < P.ngroups ? __atomic_load_n(P.groups + g, __ATOMIC_RELAXED) : 0u;
    unsigned gtotal;
    const unsigned excl = block1024_exclusive(v, lds, &gtotal);
    if (g < P.ngroups) P.groups[g] = carry + excl;
    carry += gtotal;
  }
  if (threadIdx.x == 0) {
    P.groups[P.ngroups] = carry;
    __hip_atomic_store(P.host_total, (unsigned long long)carry | ((unsigned long long)P.host_tag << 32), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
    *P.ticket = 0u;
  }
}

// COPY false: dst[rank] = src[i] for selected i.  COPY true: dst[i] = src[rank].
// VEC: the full-length operand (src when selecting, dst when copying) allows 16-byte accesses.
// A block takes a chunk, 4 steps of 1024 elements with 4 consecutive elements per thread.
// Every wave reads the chunk's 64 bit words, one per lane; a shuffle scan of their
// population counts gives the rank in front of every (step, wave), and an element's rank
// adds the set bits of earlier lanes (4 words) and of earlier elements of its own lane.
// The chunk's selected elements are adjacent in the packed tensor: they pass through LDS,
// so the packed side is read or written as one run, and every global read of the block is
// requested before the first one is waited for.  When copying into a chunk with an eighth
// or more of its elements selected, whole 16-byte groups of dst are rewritten instead of
// single elements.
template <bool COPY, bool VEC>
__global__ __launch_bounds__(kThreads) void mask_move(MaskParams P) {
  __shared__ float stage[kChunk];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const unsigned long long below = (1ull << lane) - 1ull;
  const thcl_u64 chunk0 = (thcl_u64)blockIdx.x * kChunk;
  const thcl_u64 block_rank = (thcl_u64)P.counts[blockIdx.x] + (thcl_u64)P.groups[blockIdx.x / kGroup];
  const unsigned long long word = P.bits[(thcl_u64)blockIdx.x * kWordsPerChunk + lane];  // kWordsPerChunk == 64
  // exclusive prefix of the words' population counts, in word order = (step, wave, e) order
  const unsigned pc = (unsigned)__popcll(word);
  unsigned incl = pc;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned up = __shfl_up(incl, d, 64);
    if (lane >= d) incl += up;
  }
  const unsigned excl = incl - pc;
  const unsigned chunk_total = __shfl(incl, 63, 64);
  if (chunk_total == 0) return;  // uniform over the block
  const bool groups16 = COPY && VEC && chunk_total >= kChunk / 8;

  // a vector that is not whole (at most one in the tensor) is requested from the start of the
  // tensor instead (n >= 4 when VEC) and its elements are handled one by one below
  thcl_f4 x[kMaskSteps];
  if (VEC && (!COPY || groups16)) {
    const float *full = COPY ? P.dst : P.src;
#pragma unroll
    for (int step = 0; step < kMaskSteps; step++) {
      thcl_u64 first = chunk0 + (thcl_u64)step * kMaskStep + (thcl_u64)threadIdx.x * kMaskPer;
      if (first + kMaskPer > P.n) first = 0;
      x[step] = COPY ? *(const thcl_f4 *)(full + first) : __builtin_nontemporal_load((const thcl_f4 *)(full + first));
    }
  }
  if (COPY) {
    // the chunk's run of the packed source, as far as the source reaches
    for (unsigned j = threadIdx.x; j < chunk_total; j += kThreads)
      stage[j] = (block_rank + j < P.src_len) ? P.src[block_rank + j] : 0.0f;
    __syncthreads();
  }
#pragma unroll
  for (int step = 0; step < kMaskSteps; step++) {
    const int w0 = step * kWordsPerStep + wave * kMaskPer;   // this wave's first word of the step
    unsigned long long b[kMaskPer];
#pragma unroll
    for (int e = 0; e < kMaskPer; e++) b[e] = __shfl(word, w0 + e, 64);
    unsigned rank = __shfl(excl, w0, 64);   // inside the chunk
#pragma unroll
    for (int e = 0; e < kMaskPer; e++) rank += (unsigned)__popcll(b[e] & below);
    const thcl_u64 first = chunk0 + (thcl_u64)step * kMaskStep + (thcl_u64)threadIdx.x * kMaskPer;
    const bool whole = first + kMaskPer <= P.n;
    if (!COPY) {
#pragma unroll
      for (int e = 0; e < kMaskPer; e++) {
        if ((b[e] >> lane) & 1ull) stage[rank++] = (VEC && whole) ? x[step][e] : P.src[first + e];
      }
    } else if (groups16 && whole) {
      thcl_f4 d = x[step];
      bool any = false;
#pragma unroll
      for (int e = 0; e < kMaskPer; e++) {
        if ((b[e] >> lane) & 1ull) {
          if (block_rank + rank < P.src_len) {
            d[e] = stage[rank];
            any = true;
          }
          rank++;
        }
      }
      if (any) *(thcl_f4 *)(P.dst + first) = d;
    } else {
#pragma unroll
      for (int e = 0; e < kMaskPer; e++) {
        if ((b[e] >> lane) & 1ull) {
          if (block_rank + rank < P.src_len) P.dst[first + e] = stage[rank];
          rank++;
        }
      }
    }
  }
  if (!COPY) {
    __syncthreads();
    for (unsigned j = threadIdx.x; j < chunk_total; j += kThreads) P.dst[block_rank + j] = stage[j];
  }
}

void check(const char *what) {
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "%s launch failed: %s", what, hipGetErrorString(e));
}
bool aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }

struct Dense {  // a dense stand-in for a tensor that kernels write or read
  THClState *state;
  THClTensor *orig, *t;
  bool write_back;
  Dense(THClState *s, THClTensor *x, bool load, bool store) : state(s), orig(x), t(x), write_back(false) {
    if (!THClTensor_isContiguous(s, x)) {
      if (load) {
        t = THClTensor_newContiguous(s, x);
      } else {
        t = THClTensor_newv2(s, THClTensor_getDevice(s, x));
        THClTensor_resizeAs(s, t, x);
      }
      write_back = store;
    }
  }
  void finish() {
    if (t != orig) {
      if (write_back) THClTensor_freeCopyTo(state, t, orig);
      else THClTensor_free(state, t);
      t = orig;
    }
  }
  ~Dense() {
    if (t == orig) return;
    try {
      THClTensor_free(state, t);  // error path: drop the stand-in
    } catch (...) {  // a destructor must not throw
    }
  }
};

template <int MODE>
void launch_move(hipStream_t stream, IndexParams &P, bool vec_ok) {
  const bool vec = vec_ok && MODE != GATHER && MODE != SCATTER && MODE != SCATTER_FILL && (P.I % 4 == 0) &&
                   aligned16(P.a) && (MODE == FILL || aligned16(P.b));
  const thcl_u64 units_i = vec ? P.I / 4 : P.I;
  const thcl_u64 total = (thcl_u64)units_i * P.M * (P.total /* O */);
  THCL_CHECK(total < (1ull << 31), THCL_DIM_WARNING);
  P.units_i = thcl_make_divisor((long)units_i);
  P.m = thcl_make_divisor((long)P.M);
  P.total = (thcl_u32)total;
  if (total == 0) return;
  const dim3 grid((unsigned)((total + kThreads - 1) / kThreads)), block(kThreads);
  if (vec) hipLaunchKernelGGL((index_move<MODE, 4>), grid, block, 0, stream, P);
  else if constexpr (MODE == SELECT || MODE == COPY || MODE == FILL)
    hipLaunchKernelGGL((index_move_by_element<MODE>), dim3((unsigned)((total + kThreads * 8 - 1) / (kThreads * 8))), block, 0, stream, P);
  else hipLaunchKernelGGL((index_move<MODE, 1>), grid, block, 0, stream, P);
  check("index kernel");
}

// sizes of `t` around `dim`
void split_dims(THClTensor *t, int dim, long &O, long &N, long &I) {
  O = I = 1;
  for (int d = 0; d < dim; d++) O *= t->size[d];
  for (int d = dim + 1; d < t->nDimension; d++) I *= t->size[d];
  N = t->size[dim];
}

void index_checks(THClState *state, THClTensor *indices, THClTensor *t, int dim) {
  THCL_ARGCHECK(indices->nDimension == 1, 3, "expecting vector of indices");
  THCL_ARGCHECK(t->nDimension > 0, 2, "Source tensor is empty");
  THCL_ARGCHECK(dim >= 0 && dim < t->nDimension, 4, "Indexing dim is out of bounds");
  (void)state;
}
}  // namespace

extern "C" {

// res = src with its `dim` replaced by the slices index names (src/lib/THClTensorIndex.cpp:186-256)
void THClTensor_indexSelect(THClState *state, THClTensor *res_, THClTensor *src, int dim, THClTensor *indices) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, res_, src, indices);
  index_checks(state, indices, src, dim);
  THCL_CHECK(res_ != src, "result and source must be different tensors");
  const long M = indices->size[0];
  long osz[THCL_MAX_DIMS];
  for (int d = 0; d < src->nDimension; d++) osz[d] = (d == dim) ? M : src->size[d];
  THLongStorage shape;
  memset(&shape, 0, sizeof(shape));
  shape.data = osz;
  shape.size = src->nDimension;
  THClTensor_resize(state, res_, &shape, nullptr);
  Dense s(state, src, true, false), r(state, res_, false, true), ix(state, indices, true, false);
  long O, N, I;
  split_dims(src, dim, O, N, I);
  THCL_CHECK(N < (1l << 31) && M < (1l << 31) && I < (1l << 31) && O < (1l << 31), THCL_DIM_WARNING);
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, src));
  IndexParams P;
  memset(&P, 0, sizeof(P));
  P.fault = thcl_rt_fault_word_device(rt);
  P.a = thcl_dptr(s.t);
  P.b = thcl_dptr(r.t);
  P.index = thcl_dptr(ix.t);
  P.N = (thcl_u32)N;
  P.M = (thcl_u32)M;
  P.I = (thcl_u32)I;
  P.total = (thcl_u32)O;
  if (O * M * I > 0) launch_move<SELECT>((hipStream_t)thcl_rt_stream(rt), P, true);
  thcl_after_launch(state, rt);
  s.finish();
  ix.finish();
  r.finish();
  THCL_GUARD_END()
}

// res[.., index[i], ..] = src[.., i, ..]; for a repeated target the last i wins, as in
// the sequential CPU loop (src/lib/THClTensorIndex.cpp:32-88)
void THClTensor_indexCopy(THClState *state, THClTensor *res_, int dim, THClTensor *indices, THClTensor *src) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, res_, src, indices);
  index_checks(state, indices, src, dim);
  THCL_ARGCHECK(dim < res_->nDimension, 4, "Indexing dim is out of bounds");
  THCL_ARGCHECK(indices->size[0] == src->size[dim], 4, "length of src.size[dim] is not equal to length of indices");
  THCL_ARGCHECK(res_->nDimension == src->nDimension, 2, "result and source differ in dimensions");
  for (int d = 0; d < src->nDimension; d++)
    if (d != dim) THCL_ARGCHECK(res_->size[d] == src->size[d], 2, "result and source sizes differ outside the indexed dim");
  THCL_CHECK(res_ != src, "result and source must be different tensors");
  Dense s(state, src, true, false), r(state, res_, true, true), ix(state, indices, true, false);
  long O, N, I, M = indices->size[0];
  split_dims(res_, dim, O, N, I);
  THCL_CHECK(N < (1l << 31) && M < (1l << 31) && I < (1l << 31) && O < (1l << 31), THCL_DIM_WARNING);
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, res_));
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  IndexParams P;
  memset(&P, 0, sizeof(P));
  P.fault = thcl_rt_fault_word_device(rt);
  P.a = thcl_dptr(r.t);
  P.b = thcl_dptr(s.t);
  P.index = thcl_dptr(ix.t);
  P.N = (thcl_u32)N;
  P.M = (thcl_u32)M;
  P.I = (thcl_u32)I;
  P.total = (thcl_u32)O;
  if (O * M * I > 0 && N > 0) {
    P.winner = (int *)thcl_rt_workspace(rt, (size_t)N * sizeof(int));
    THCL_CHECK(P.winner != nullptr, "%s", thcl_rt_error());
    hipLaunchKernelGGL(fill_int, dim3((unsigned)((N + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, P.winner, -1,
                       (thcl_u32)N);
    hipLaunchKernelGGL(index_winner, dim3((unsigned)((M + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, P);
    check("index winners");
    launch_move<COPY>(stream, P, true);
  }
  thcl_after_launch(state, rt);
  s.finish();
  ix.finish();
  r.finish();
  THCL_GUARD_END()
}

// (src/lib/THClTensorIndex.cpp:104-168)
void THClTensor_indexFill(THClState *state, THClTensor *res_, int dim, THClTensor *indices, float val) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, res_, indices);
  THCL_ARGCHECK(indices->nDimension == 1, 3, "Index is supposed to be a vector");
  THCL_ARGCHECK(res_->nDimension > 0, 2, "Source tensor is empty");
  THCL_ARGCHECK(dim >= 0 && dim < res_->nDimension, 4, "Indexing dim is out of bounds");
  Dense r(state, res_, true, true), ix(state, indices, true, false);
  long O, N, I, M = indices->size[0];
  split_dims(res_, dim, O, N, I);
  THCL_CHECK(N < (1l << 31) && M < (1l << 31) && I < (1l << 31) && O < (1l << 31), THCL_DIM_WARNING);
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, res_));
  IndexParams P;
  memset(&P, 0, sizeof(P));
  P.fault = thcl_rt_fault_word_device(rt);
  P.a = thcl_dptr(r.t);
  P.index = thcl_dptr(ix.t);
  P.N = (thcl_u32)N;
  P.M = (thcl_u32)M;
  P.I = (thcl_u32)I;
  P.total = (thcl_u32)O;
  P.value = val;
  if (O * M * I > 0) launch_move<FILL>((hipStream_t)thcl_rt_stream(rt), P, true);
  thcl_after_launch(state, rt);
  ix.finish();
  r.finish();
  THCL_GUARD_END()
}

// host index vectors: uploaded as floats, like the reference (src/lib/THClTensorIndex.cpp:16-30,90-102,170-184)
static THClTensor *upload_indices(THClState *state, int device, THLongTensor *indices) {
  THCL_ARGCHECK(indices->nDimension == 1, 3, "expecting vector of indices");
  THClTensor *t = THClTensor_newWithSize1d(state, device, indices->size[0]);
  THClTensor_copyLong(state, t, indices);
  return t;
}
void THClTensor_indexSelect_long(THClState *state, THClTensor *res_, THClTensor *src, int dim, THLongTensor *indices) {
  THCL_GUARD_BEGIN
  THClTensor *ix = upload_indices(state, THClTensor_getDevice(state, src), indices);
  THClTensor_indexSelect(state, res_, src, dim, ix);
  THClTensor_free(state, ix);
  THCL_GUARD_END()
}
void THClTensor_indexCopy_long(THClState *state, THClTensor *res_, int dim, THLongTensor *indices, THClTensor *src) {
  THCL_GUARD_BEGIN
  THClTensor *ix = upload_indices(state, THClTensor_getDevice(state, src), indices);
  THClTensor_indexCopy(state, res_, dim, ix, src);
  THClTensor_free(state, ix);
  THCL_GUARD_END()
}
void THClTensor_indexFill_long(THClState *state, THClTensor *res_, int dim, THLongTensor *indices, float val) {
  THCL_GUARD_BEGIN
  THClTensor *ix = upload_indices(state, THClTensor_getDevice(state, res_), indices);
  THClTensor_indexFill(state, res_, dim, ix, val);
  THClTensor_free(state, ix);
  THCL_GUARD_END()
}

// ------------------------------------------------------- gather / scatter ---
static void gather_scatter_checks(THClState *state, THClTensor *full, THClTensor *index, THClTensor *other, long dim) {
  const int nd = index->nDimension;
  THCL_ARGCHECK(nd >= 1, 2, "index tensor is empty");
  THCL_ARGCHECK(full->nDimension == nd, 2, "All tensors should have same number of dims");
  THCL_ARGCHECK(other == nullptr || other->nDimension == nd, 4, "All tensors should have same number of dims");
  THCL_ARGCHECK(dim >= 0 && dim < nd, 4, "dim out of bounds");
  for (int d = 0; d < nd; d++) {
    if (d != dim)
      THCL_CHECK(full->size[d] == index->size[d],
                 "index tensor must have same dimensions as source tensor, but dimension %d doesnt match", d);
    if (other) THCL_CHECK(other->size[d] == index->size[d], "index and value tensors differ in dimension %d", d);
  }
  (void)state;
}

static void run_gather_scatter(THClState *state, int mode, THClTensor *full, THClTensor *index, THClTensor *other,
                               long dim, float value) {
  long O, N, I;
  split_dims(full, (int)dim, O, N, I);
  const long M = index->size[dim];
  THCL_CHECK(N < (1l << 31) && M < (1l << 31) && I < (1l << 31) && O < (1l << 31), THCL_DIM_WARNING);
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, full));
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  IndexParams P;
  memset(&P, 0, sizeof(P));
  P.fault = thcl_rt_fault_word_device(rt);
  P.a = thcl_dptr(full);
  P.b = other ? thcl_dptr(other) : nullptr;
  P.index = thcl_dptr(index);
  P.N = (thcl_u32)N;
  P.M = (thcl_u32)M;
  P.I = (thcl_u32)I;
  P.total = (thcl_u32)O;
  P.value = value;
  if (O * M * I > 0) {
    if (mode == GATHER) launch_move<GATHER>(stream, P, false);
    else if (mode == SCATTER) launch_move<SCATTER>(stream, P, false);
    else launch_move<SCATTER_FILL>(stream, P, false);
  }
  thcl_after_launch(state, rt);
}

// self[i][j][k] = src[index[i][j][k]][j][k] for dim 0, likewise for the others
// (src/lib/THClGather.cpp:17-78); self takes the index tensor's shape
void THClTensor_gather(THClState *state, THClTensor *self, THClTensor *src, long dim, THClTensor *index) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, src, index);
  gather_scatter_checks(state, src, index, nullptr, dim);
  THCL_CHECK(self != src && self != index, "result cannot alias the source or the index");
  THClTensor_resizeAs(state, self, index);
  Dense s(state, src, true, false), r(state, self, false, true), ix(state, index, true, false);
  run_gather_scatter(state, GATHER, s.t, ix.t, r.t, dim, 0.f);
  s.finish();
  ix.finish();
  r.finish();
  THCL_GUARD_END()
}
// self[index[i][j][k]][j][k] = src[i][j][k]; targets named twice keep either writer
// (src/lib/THClScatter.cpp:15-80)
void THClTensor_scatter(THClState *state, THClTensor *self, long dim, THClTensor *index, THClTensor *src) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, src, index);
  gather_scatter_checks(state, self, index, src, dim);
  THCL_ARGCHECK(self != index, 1, "self cannot alias index");
  THCL_ARGCHECK(self != src, 1, "self cannot alias src");
  Dense s(state, src, true, false), r(state, self, true, true), ix(state, index, true, false);
  run_gather_scatter(state, SCATTER, r.t, ix.t, s.t, dim, 0.f);
  s.finish();
  ix.finish();
  r.finish();
  THCL_GUARD_END()
}
void THClTensor_scatterFill(THClState *state, THClTensor *self, long dim, THClTensor *index, float val) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, self, index);
  gather_scatter_checks(state, self, index, nullptr, dim);
  THCL_ARGCHECK(self != index, 1, "self cannot alias index");
  Dense r(state, self, true, true), ix(state, index, true, false);
  run_gather_scatter(state, SCATTER_FILL, r.t, ix.t, nullptr, dim, val);
  ix.finish();
  r.finish();
  THCL_GUARD_END()
}

// ------------------------------------------------------------- masked ---
// per-chunk counts, group offsets and the grand total are 32-bit words
constexpr long kMaskMaxElements = 1l << 32;
constexpr int kMaskTicket = 8;     // word of the context's scratch block (words 1..63 are free for such counters)
static unsigned *mask_prefix(THClState *state, thcl_rt *rt, MaskParams &P, long n) {
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  const long nb = (n + kChunk - 1) / kChunk;
  THCL_CHECK(n < kMaskMaxElements, THCL_DIM_WARNING);
  P.n = (thcl_u64)n;
  P.nblocks = (thcl_u32)nb;
  // the bit words first (8-byte aligned), then the counts and the group totals
  const long ng = (nb + kGroup - 1) / kGroup;
  P.ngroups = (thcl_u32)ng;
  const size_t bit_bytes = (size_t)nb * kWordsPerChunk * sizeof(unsigned long long);
  char *w = (char *)thcl_rt_workspace(rt, bit_bytes + (size_t)(nb + ng + 1) * sizeof(unsigned));
  THCL_CHECK(w != nullptr, "%s", thcl_rt_error());
  P.bits = (unsigned long long *)w;
  P.counts = (unsigned *)(w + bit_bytes);
  P.groups = P.counts + nb;
  if (aligned16(P.mask)) hipLaunchKernelGGL(mask_count<true>, dim3((unsigned)nb), dim3(kThreads), 0, stream, P);
  else hipLaunchKernelGGL(mask_count<false>, dim3((unsigned)nb), dim3(kThreads), 0, stream, P);
  check("mask count");
  P.ticket = (unsigned *)thcl_rt_scratch(rt, nullptr) + kMaskTicket;
  P.host_total = (unsigned long long *)thcl_rt_tagged_word_device(rt);
  P.host_tag = thcl_rt_next_tag(rt);
  hipLaunchKernelGGL(mask_scan_groups, dim3((unsigned)ng), dim3(1024), 0, stream, P);
  check("mask offsets");
  (void)state;
  return P.counts;
}

static long read_total(thcl_rt *rt, const MaskParams &P) {
  // the last group block left {count, tag} in the pinned pair: the host picks it up as soon as it lands
  float as_float = 0.f;
  THCL_CHECK(thcl_rt_await_tagged(rt, P.host_tag, &as_float) == 0, "%s", thcl_rt_error());
  unsigned total;
  memcpy(&total, &as_float, sizeof(total));
  return (long)total;
}

// tensor = the elements of src whose mask entry is non-zero, in order, as a vector
// (src/lib/THClTensorMasked.cpp:193-246)
void THClTensor_maskedSelect(THClState *state, THClTensor *tensor, THClTensor *src, THClTensor *mask) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, tensor, src, mask);
  const long n = THClTensor_nElement(state, mask);
  THCL_ARGCHECK(n == THClTensor_nElement(state, src), 2, "sizes do not match");
  THCL_CHECK(n < kMaskMaxElements, "maskedSelect takes at most 2^32 - 1 elements (the mask has %ld): its offsets are 32-bit", n);
  THCL_CHECK(tensor != src && tensor != mask, "result cannot alias the source or the mask");
  const int device = THClTensor_getDevice(state, src);
  if (tensor->nDimension < 0 && !tensor->storage) tensor->device = device;
  if (n == 0) {
    THClTensor_resize1d(state, tensor, 0);
    return;
  }
  Dense s(state, src, true, false), m(state, mask, true, false);
  thcl_rt *rt = thcl_ctx(state, device);
  MaskParams P;
  memset(&P, 0, sizeof(P));
  P.mask = thcl_dptr(m.t);
  P.src = thcl_dptr(s.t);
  mask_prefix(state, rt, P, n);
  const long total = read_total(rt, P);  // the one synchronising step: the result's size
  THClTensor_resize1d(state, tensor, total);
  if (total > 0) {
    Dense r(state, tensor, false, true);
    P.dst = thcl_dptr(r.t);
    if (aligned16(P.src) && n >= 4)
      hipLaunchKernelGGL((mask_move<false, true>), dim3(P.nblocks), dim3(kThreads), 0, (hipStream_t)thcl_rt_stream(rt), P);
    else
      hipLaunchKernelGGL((mask_move<false, false>), dim3(P.nblocks), dim3(kThreads), 0, (hipStream_t)thcl_rt_stream(rt), P);
    check("masked select");
    thcl_after_launch(state, rt);
    r.finish();
  }
  s.finish();
  m.finish();
  THCL_GUARD_END()
}

// tensor[i] = next element of src, for every i whose mask entry is non-zero
// (declared at src/lib/THClTensorMath.h:113; the reference's body stops at
// THError("Not implemented"), src/lib/THClTensorMasked.cpp:126-191)
void THClTensor_maskedCopy(THClState *state, THClTensor *tensor, THClTensor *mask, THClTensor *src) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, tensor, src, mask);
  const long n = THClTensor_nElement(state, mask);
  THCL_ARGCHECK(n == THClTensor_nElement(state, tensor), 2, "mask and tensor must have the same number of elements");
  THCL_CHECK(n < kMaskMaxElements, "maskedCopy takes at most 2^32 - 1 elements (the mask has %ld): its offsets are 32-bit", n);
  THCL_CHECK(tensor != src && tensor != mask, "tensor cannot alias the source or the mask");
  if (n == 0) return;
  Dense s(state, src, true, false), m(state, mask, true, false), r(state, tensor, true, true);
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, tensor));
  MaskParams P;
  memset(&P, 0, sizeof(P));
  P.mask = thcl_dptr(m.t);
  P.src = thcl_dptr(s.t);
  P.dst = thcl_dptr(r.t);
  P.src_len = (thcl_u64)THClTensor_nElement(state, src);
  mask_prefix(state, rt, P, n);
  if (aligned16(P.dst))
    hipLaunchKernelGGL((mask_move<true, true>), dim3(P.nblocks), dim3(kThreads), 0, (hipStream_t)thcl_rt_stream(rt), P);
  else
    hipLaunchKernelGGL((mask_move<true, false>), dim3(P.nblocks), dim3(kThreads), 0, (hipStream_t)thcl_rt_stream(rt), P);
  check("masked copy");
  const long total = read_total(rt, P);
  thcl_after_launch(state, rt);
  s.finish();
  m.finish();
  r.finish();
  THCL_ARGCHECK(total <= (long)P.src_len, 2, "source nElements must be == mask `1` elements");
  THCL_GUARD_END()
}

}  // extern "C"
