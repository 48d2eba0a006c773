// Reductions: whole tensor -> scalar, and along one dimension (sum, prod,
// max, min; max/min also report positions).
//
// What it replaces (reference): THClTensor_reduceAll's one- or two-pass
// kernels that run on at most 4 work-groups (src/lib/THClReduceAll.cpp:225-272,
// src/lib/THClGeneral.cpp:16-17), THClTensor_reduceDim's two kernels
// (src/lib/THClReduce.cl:30-111) and the (value, index) kernels of
// src/lib/THClTensorMathTransformReduce.cl:17-102.
//
// Numerics follow Torch7's CPU path: sums and products accumulate in fp64 and
// round to fp32 once; max/min propagate NaN (the first one wins) and resolve
// ties to the lowest position.  Every combine order is fixed by the launch
// shape, so results are reproducible run to run; no floating-point atomics.
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cmath>
#include <cstring>

#include "apply_device.h"
#include "internal.h"

namespace {

// a 16-byte read that only needs the alignment of its elements (rows of a view start anywhere)
typedef thcl_f4 rd_f4 __attribute__((aligned(4)));


constexpr int kThreads = 256;
constexpr int kWave = 64;

// scratch block layout (bytes)
constexpr size_t kTicketOff = 0;            // 4096 uint32 tickets: [0] whole-tensor reductions, [64..] column tiles
constexpr size_t kPartialOff = 16384;       // partials
constexpr unsigned kColTicket0 = 64, kColTickets = 4096 - 64;
constexpr size_t kResultSlot = 256;         // tail reserved for scalar results

// --------------------------------------------------------------- combiners ---
template <int KIND>
struct Acc;  // accumulator type + combine rule for value-only reductions

template <>
struct Acc<RED_SUM> {
  typedef double T;
  static __device__ __forceinline__ T init() { return 0.0; }
  static __device__ __forceinline__ T lift(float x, float) { return (double)x; }
  static __device__ __forceinline__ T comb(T a, T b) { return a + b; }
  static __device__ __forceinline__ float lower(T a) { return (float)a; }
};
template <>
struct Acc<RED_PROD> {
  typedef double T;
  static __device__ __forceinline__ T init() { return 1.0; }
  static __device__ __forceinline__ T lift(float x, float) { return (double)x; }
  static __device__ __forceinline__ T comb(T a, T b) { return a * b; }
  static __device__ __forceinline__ float lower(T a) { return (float)a; }
};
template <>
struct Acc<RED_MAX> {
  typedef float T;
  static __device__ __forceinline__ T init() { return -INFINITY; }
  static __device__ __forceinline__ T lift(float x, float) { return x; }
  // NaN on either side gives NaN
  static __device__ __forceinline__ T comb(T a, T b) { return ((b > a) | (b != b)) ? b : a; }
  static __device__ __forceinline__ float lower(T a) { return a; }
};
template <>
struct Acc<RED_MIN> {
  typedef float T;
  static __device__ __forceinline__ T init() { return INFINITY; }
  static __device__ __forceinline__ T lift(float x, float) { return x; }
  static __device__ __forceinline__ T comb(T a, T b) { return ((b < a) | (b != b)) ? b : a; }
  static __device__ __forceinline__ float lower(T a) { return a; }
};

// Sums of a modified element (fp64 like every sum), and the all / any truth
// reductions as min / max over 0 / 1.
struct AccSum {
  typedef double T;
  static __device__ __forceinline__ T init() { return 0.0; }
  static __device__ __forceinline__ T comb(T a, T b) { return a + b; }
  static __device__ __forceinline__ float lower(T a) { return (float)a; }
};
template <>
struct Acc<RED_SUM_NE0> : AccSum {
  static __device__ __forceinline__ T lift(float x, float) { return x != 0.0f ? 1.0 : 0.0; }
};
template <>
struct Acc<RED_SUM_ABS> : AccSum {
  static __device__ __forceinline__ T lift(float x, float) { return (double)fabsf(x); }
};
template <>
struct Acc<RED_SUM_SQ> : AccSum {
  static __device__ __forceinline__ T lift(float x, float) { return (double)x * (double)x; }
};
template <>
struct Acc<RED_SUM_POW> : AccSum {
  static __device__ __forceinline__ T lift(float x, float e) { return pow(fabs((double)x), (double)e); }
};
template <>
struct Acc<RED_ALL> {
  typedef float T;
  static __device__ __forceinline__ T init() { return 1.0f; }
  static __device__ __forceinline__ T lift(float x, float) { return (int)x != 0 ? 1.0f : 0.0f; }
  static __device__ __forceinline__ T comb(T a, T b) { return fminf(a, b); }
  static __device__ __forceinline__ float lower(T a) { return a; }
};
template <>
struct Acc<RED_ANY> {
  typedef float T;
  static __device__ __forceinline__ T init() { return 0.0f; }
  static __device__ __forceinline__ T lift(float x, float) { return (int)x != 0 ? 1.0f : 0.0f; }
  static __device__ __forceinline__ T comb(T a, T b) { return fmaxf(a, b); }
  static __device__ __forceinline__ float lower(T a) { return a; }
};

// (value, position) pairs for max/min along a dim.  Order-independent rule
// equal to the sequential "replace when !(x <= cur), stop at the first NaN":
// NaN beats any number, the earlier NaN beats a later one, equal values keep
// the lower position.
struct VI {
  float v;
  int i;
};
template <int KIND>
__device__ __forceinline__ VI vi_init() {
  VI r;
  r.v = (KIND == RED_MAX) ? -INFINITY : INFINITY;
  r.i = 0x7fffffff;
  return r;
}
template <int KIND>
__device__ __forceinline__ VI vi_comb(VI cur, VI x) {
  // straight-line form (no short-circuit): the compiler turns && / || chains
  // into exec-mask branches, which cost more than the arithmetic
  const bool xn = x.v != x.v, cn = cur.v != cur.v;
  const bool better = (KIND == RED_MAX) ? (x.v > cur.v) : (x.v < cur.v);
  const bool same = (x.v == cur.v) | (xn & cn);
  const bool take = (!cn & (xn | better)) | (same & (x.i < cur.i));
  VI r;
  r.v = take ? x.v : cur.v;
  r.i = take ? x.i : cur.i;
  return r;
}

__device__ __forceinline__ double shfl_xor_t(double v, int m) { return __shfl_xor(v, m, kWave); }
__device__ __forceinline__ float shfl_xor_t(float v, int m) { return __shfl_xor(v, m, kWave); }
__device__ __forceinline__ VI shfl_xor_t(VI v, int m) {
  VI r;
  r.v = __shfl_xor(v.v, m, kWave);
  r.i = __shfl_xor(v.i, m, kWave);
  return r;
}

// butterfly over the `width` lanes (power of two <= 64) a lane belongs to
template <int KIND, class T>
__device__ __forceinline__ T group_reduce(T v, int width) {
  for (int m = width >> 1; m > 0; m >>= 1) v = Acc<KIND>::comb(v, shfl_xor_t(v, m));
  return v;
}
template <int KIND>
__device__ __forceinline__ VI group_reduce_vi(VI v, int width) {
  for (int m = width >> 1; m > 0; m >>= 1) v = vi_comb<KIND>(v, shfl_xor_t(v, m));
  return v;
}

// whole-block reduce; result valid in thread 0
template <int KIND, class T>
__device__ __forceinline__ T block_reduce(T v, T *lds) {
  v = group_reduce<KIND, T>(v, kWave);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();  // lds may still be read by a previous round
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    T r = lds[0];
    for (int w = 1; w < kThreads / kWave; w++) r = Acc<KIND>::comb(r, lds[w]);
    v = r;
  }
  return v;
}

// loads that bypass the non-coherent per-CU cache (partials written by other blocks)
__device__ __forceinline__ double load_fresh(const double *p) {
  return __longlong_as_double((long long)__atomic_load_n((const unsigned long long *)p, __ATOMIC_RELAXED));
}
__device__ __forceinline__ float load_fresh(const float *p) {
  return __uint_as_float(__atomic_load_n((const unsigned *)p, __ATOMIC_RELAXED));
}

// Partials that other blocks of the same launch will read: written through to
// device scope (no dirty line stays in this XCD's L2) and read back with
// device-scope loads.
__device__ __forceinline__ void store_shared(double *p, double v) {
  __hip_atomic_store((unsigned long long *)p, (unsigned long long)__double_as_longlong(v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_shared(float *p, float v) {
  __hip_atomic_store((unsigned *)p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_shared(VI *p, VI v) {
  const unsigned long long bits = (unsigned long long)__float_as_uint(v.v) | ((unsigned long long)(unsigned)v.i << 32);
  __hip_atomic_store((unsigned long long *)p, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ VI load_fresh(const VI *p) {
  const unsigned long long bits = __atomic_load_n((const unsigned long long *)p, __ATOMIC_RELAXED);
  VI r;
  r.v = __uint_as_float((unsigned)bits);
  r.i = (int)(unsigned)(bits >> 32);
  return r;
}

// ------------------------------------------------------------- reduce all ---
struct ReduceAllParams {
  const float *in;
  thcl_u64 n;
  void *partials;
  unsigned *ticket;
  float *out;
  float exponent;        // p of the |x|^p sum
  unsigned host_tag;     // non-zero: `out` is a pinned host word pair that receives {result, tag} in one 8-byte store
  ThclGenericOperand L;  // strided input only
};

// Publishing a block's partial: a device-scope atomic exchange lands at the
// level every XCD sees, and its return value tells this thread it has landed.
// That avoids a release fence, which on this chip writes back the whole L2 of
// the XCD and cost ~45 ns per block when measured.
//
// What each step of the hand-over relies on (the language's memory model
// gives relaxed atomics no ordering; this is correct by the hardware's rules):
//  1. The eight XCDs' L2 caches are not coherent with one another, so a
//     device-scope read-modify-write is performed where all XCDs meet (memory
//     side), and the instruction returns its old value only after that.
//  2. The ticket's increment is made data-dependent on the exchange's return
//     (empty volatile asm): the wave issues in order and must wait for the
//     return (s_waitcnt vmcnt) before it can issue the ticket operation.
//  3. Read-modify-writes on one address are totally ordered: the block that
//     draws the last ticket knows every other block's ticket, hence (1, 2)
//     every other block's exchange, has been performed.
//  4. It reads the slots with system-scope atomic loads, which bypass the
//     per-CU cache and the L2, after the ticket has returned (a branch on the
//     flag in LDS behind a barrier; loads are not issued speculatively).
// It would break on hardware that returns a device-scope atomic before it is
// performed for all XCDs, or lets such loads hit a stale cache line.
__device__ __forceinline__ unsigned publish(double *slot, double v) {
  return (unsigned)atomicExch((unsigned long long *)slot, (unsigned long long)__double_as_longlong(v));
}
__device__ __forceinline__ unsigned publish(float *slot, float v) {
  return atomicExch((unsigned *)slot, __float_as_uint(v));
}

// Last block to arrive (integer ticket) folds the per-block partials in block
// order and writes the scalar; the ticket is left at zero for the next launch.
// Order of events per block: partial exchanged -> its return observed -> ticket
// taken.  The last block therefore takes its ticket after every partial has
// landed, and reads them with device-scope atomic loads.
template <int KIND>
__device__ __forceinline__ void finish_all(typename Acc<KIND>::T blockval, const ReduceAllParams &P,
                                           typename Acc<KIND>::T *lds) {
  typedef typename Acc<KIND>::T T;
  T *partials = (T *)P.partials;
  __shared__ unsigned s_last;
  if (threadIdx.x == 0) {
    const unsigned landed = publish(&partials[blockIdx.x], blockval);
    unsigned inc = 1u;
    asm volatile("" : "+v"(inc) : "v"(landed));  // the increment depends on the exchange's return
    const unsigned t = atomicAdd(P.ticket, inc);
    s_last = (t == gridDim.x - 1) ? 1u : 0u;
  }
  __syncthreads();
  if (!s_last) return;
  T v = Acc<KIND>::init();
  for (unsigned i = threadIdx.x; i < gridDim.x; i += kThreads)
    v = Acc<KIND>::comb(v, load_fresh(&partials[i]));
  v = block_reduce<KIND, T>(v, lds);
  if (threadIdx.x == 0) {
    const float r = Acc<KIND>::lower(v);
    if (P.host_tag) {
      // result and tag travel together, so a host that polls the pair sees both or neither
      const unsigned long long pair = (unsigned long long)__float_as_uint(r) | ((unsigned long long)P.host_tag << 32);
      __hip_atomic_store((unsigned long long *)P.out, pair, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    } else {
      P.out[0] = r;
    }
    *P.ticket = 0u;
  }
}

// One of a thread's running values over a dense stream of float4 loads.
template <int KIND>
struct Chain {
  typedef typename Acc<KIND>::T T;
  T acc = Acc<KIND>::init();
  __device__ __forceinline__ void take4(thcl_f4 v, float e) {
#pragma unroll
    for (int c = 0; c < 4; c++) acc = Acc<KIND>::comb(acc, Acc<KIND>::lift(v[c], e));
  }
  __device__ __forceinline__ T value() const { return acc; }
};
// Max and min: the extremum of the numbers with the three-operand instruction
// (it skips quiet NaNs), and whether a NaN went by with one unordered compare
// per two elements, folded in scalar registers.  One vector instruction per
// element where Acc's rule takes three.  The instruction is written out
// because fmaxf() puts a canonicalising v_max in front of every loaded operand.
template <bool MAX>
struct ChainExtremum {
  typedef float T;
  float acc = MAX ? -INFINITY : INFINITY;
  bool nan = false;
  static __device__ __forceinline__ float three(float a, float b, float c) {
    float r;
    if (MAX) asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    else asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
  }
  __device__ __forceinline__ void take4(thcl_f4 v, float) {
    acc = three(acc, v[0], v[1]);
    acc = three(acc, v[2], v[3]);
    nan |= __builtin_isunordered(v[0], v[1]) | __builtin_isunordered(v[2], v[3]);
  }
  __device__ __forceinline__ T value() const { return nan ? __builtin_nanf("") : acc; }
};
template <>
struct Chain<RED_MAX> : ChainExtremum<true> {};
template <>
struct Chain<RED_MIN> : ChainExtremum<false> {};

template <int KIND>
__global__ __launch_bounds__(kThreads) void reduce_all_dense(ReduceAllParams P) {
  typedef typename Acc<KIND>::T T;
  __shared__ T lds[kThreads / kWave];
  constexpr int U = 4;
  Chain<KIND> chain[U];
  // 16-byte aligned body as float4, unaligned head/tail as scalars
  const uintptr_t addr = (uintptr_t)P.in;
  thcl_u64 head = ((16 - (addr & 15)) & 15) / 4;
  if (head > P.n) head = P.n;
  const thcl_u64 n4 = (P.n - head) >> 2;
  const thcl_f4 *in4 = (const thcl_f4 *)(P.in + head);
  const thcl_u64 tile = (thcl_u64)kThreads * U, all = (thcl_u64)gridDim.x * tile;
  thcl_u64 base = (thcl_u64)blockIdx.x * tile + threadIdx.x;
  // whole tiles: U loads issued back to back with nothing conditional between them
  for (; base + (U - 1) * kThreads < n4; base += all) {
    thcl_f4 v[U];
#pragma unroll
    for (int k = 0; k < U; k++) v[k] = __builtin_nontemporal_load(in4 + base + (thcl_u64)k * kThreads);
#pragma unroll
    for (int k = 0; k < U; k++) chain[k].take4(v[k], P.exponent);
  }
  for (; base < n4; base += kThreads) chain[0].take4(in4[base], P.exponent);  // the one ragged tile
  T acc0 = chain[0].value();
  if (blockIdx.x == 0) {
    const thcl_u64 tail0 = head + (n4 << 2);
    for (thcl_u64 i = threadIdx.x; i < head; i += kThreads) acc0 = Acc<KIND>::comb(acc0, Acc<KIND>::lift(P.in[i], P.exponent));
    for (thcl_u64 i = tail0 + threadIdx.x; i < P.n; i += kThreads)
      acc0 = Acc<KIND>::comb(acc0, Acc<KIND>::lift(P.in[i], P.exponent));
  }
  T v = Acc<KIND>::comb(Acc<KIND>::comb(acc0, chain[1].value()), Acc<KIND>::comb(chain[2].value(), chain[3].value()));
  v = block_reduce<KIND, T>(v, lds);
  finish_all<KIND>(v, P, lds);
}

// VEC 4: the view's innermost run is dense, a multiple of 4 long and 16-byte aligned in every row, so it is
// walked in units of four elements (P.n and P.L count units; one index decomposition and one load per unit).
template <int KIND, int VEC>
__global__ __launch_bounds__(kThreads) void reduce_all_strided(ReduceAllParams P) {
  typedef typename Acc<KIND>::T T;
  __shared__ T lds[kThreads / kWave];
  const thcl_u64 all = (thcl_u64)gridDim.x * kThreads;
  thcl_u64 i = (thcl_u64)blockIdx.x * kThreads + threadIdx.x;
  T acc;
  if (VEC == 4) {
    constexpr int FLY = 8;
    Chain<KIND> chain[FLY];
    for (; i + (FLY - 1) * all < P.n; i += FLY * all) {
      thcl_f4 v[FLY];
#pragma unroll
      for (int k = 0; k < FLY; k++)
        v[k] = __builtin_nontemporal_load((const rd_f4 *)(P.in + thcl_generic_offset((thcl_u32)(i + k * all), P.L)));
#pragma unroll
      for (int k = 0; k < FLY; k++) chain[k].take4(v[k], P.exponent);
    }
    for (; i < P.n; i += all) chain[0].take4(*(const rd_f4 *)(P.in + thcl_generic_offset((thcl_u32)i, P.L)), P.exponent);
    acc = chain[0].value();
#pragma unroll
    for (int k = 1; k < FLY; k++) acc = Acc<KIND>::comb(acc, chain[k].value());
  } else {
    acc = Acc<KIND>::init();
    constexpr int FLY = 8;  // independent loads per thread and turn
    for (; i + (FLY - 1) * all < P.n; i += FLY * all) {
      float v[FLY];
#pragma unroll
      for (int k = 0; k < FLY; k++) v[k] = P.in[thcl_generic_offset((thcl_u32)(i + k * all), P.L)];
#pragma unroll
      for (int k = 0; k < FLY; k++) acc = Acc<KIND>::comb(acc, Acc<KIND>::lift(v[k], P.exponent));
    }
    for (; i < P.n; i += all)
      acc = Acc<KIND>::comb(acc, Acc<KIND>::lift(P.in[thcl_generic_offset((thcl_u32)i, P.L)], P.exponent));
  }
  acc = block_reduce<KIND, T>(acc, lds);
  finish_all<KIND>(acc, P, lds);
}

// sum of a[i] * b[i] over two dense arrays: products and the running sum in fp64
__global__ __launch_bounds__(kThreads) void dot_dense(ReduceAllParams P, const float *other) {
  __shared__ double lds[kThreads / kWave];
  constexpr int U = 4;
  double acc[U] = {0.0, 0.0, 0.0, 0.0};
  {
    const thcl_u64 n4 = P.n >> 2, tile = (thcl_u64)kThreads * U;
    const rd_f4 *a4 = (const rd_f4 *)P.in, *b4 = (const rd_f4 *)other;   // dense arrays that may start at any element
    thcl_u64 base = (thcl_u64)blockIdx.x * tile + threadIdx.x;
    // whole tiles: 2 * U loads issued back to back with nothing conditional between them
    for (; base + (U - 1) * kThreads < n4; base += (thcl_u64)gridDim.x * tile) {
      thcl_f4 x[U], y[U];
#pragma unroll
      for (int k = 0; k < U; k++) {
        x[k] = __builtin_nontemporal_load(a4 + base + (thcl_u64)k * kThreads);
        y[k] = __builtin_nontemporal_load(b4 + base + (thcl_u64)k * kThreads);
      }
#pragma unroll
      for (int k = 0; k < U; k++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[k] += (double)x[k][c] * (double)y[k][c];
    }
    for (; base < n4; base += kThreads) {  // the one ragged tile
      const thcl_f4 x = a4[base], y = b4[base];
#pragma unroll
      for (int c = 0; c < 4; c++) acc[0] += (double)x[c] * (double)y[c];
    }
    if (blockIdx.x == 0)
      for (thcl_u64 i = (n4 << 2) + threadIdx.x; i < P.n; i += kThreads) acc[0] += (double)P.in[i] * (double)other[i];
  }
  double v = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  v = block_reduce<RED_SUM, double>(v, lds);
  finish_all<RED_SUM>(v, P, lds);
}

// ------------------------------------------------------- reduce along dim ---
struct ReduceDimParams {
  const float *in;       // first element of the view
  float *out;            // dense, one value per slice (NULL while writing partials)
  float *idx_f32;        // dense 1-based positions as fp32, or NULL
  long long *idx_i64;    // dense 1-based positions as int64, or NULL
  void *partials;        // [split][nslices] when the reduction length is split over blocks
  unsigned *ticket;      // one arrival counter per column tile (split > 1), zero between launches
  thcl_u32 nslices;      // output elements
  thcl_u32 nunits;       // slices / VEC (column kernel)
  thcl_u32 R;            // reduction length
  thcl_u32 rstride;      // elements between consecutive reduced elements
  thcl_u32 split;        // blocks sharing one slice's reduction (column kernel)
  thcl_u32 fused;        // split > 1: the last block of a tile folds its partials (else a second kernel does)
  thcl_u32 rows_per_split;
  thcl_u32 ub_log2;      // column kernel: a wave spans 2^ub_log2 units side by side and 64 >> ub_log2 rows
  float exponent;        // p of the |x|^p sum
  ThclGenericOperand L;  // layout of the slice starts (the view without `dim`)
};

template <int KIND, bool ARG>
struct Slot;  // what a thread carries
template <int KIND>
struct Slot<KIND, false> {
  typedef typename Acc<KIND>::T T;
  static __device__ __forceinline__ T init() { return Acc<KIND>::init(); }
  static __device__ __forceinline__ T take(T cur, float x, int, float e) { return Acc<KIND>::comb(cur, Acc<KIND>::lift(x, e)); }
  static __device__ __forceinline__ T seal(T acc, int, bool) { return acc; }
  static __device__ __forceinline__ T comb(T a, T b) { return Acc<KIND>::comb(a, b); }
  static __device__ __forceinline__ T reduce(T v, int width) { return group_reduce<KIND, T>(v, width); }
  static __device__ __forceinline__ void store(const ReduceDimParams &P, thcl_u32 s, T v) { P.out[s] = Acc<KIND>::lower(v); }
};
template <int KIND>
struct Slot<KIND, true> {
  typedef VI T;
  static __device__ __forceinline__ T init() { return vi_init<KIND>(); }
  // For a thread that meets positions in increasing order: replace when
  // !(x <= cur) (max) unless cur is already NaN.  Five instructions where the
  // order-free rule takes ten; an element equal to the start value is never
  // taken, which seal() repairs.
  static __device__ __forceinline__ T take(T cur, float x, int i, float) {
    const bool beats = (KIND == RED_MAX) ? !(x <= cur.v) : !(x >= cur.v);
    const bool take = beats & (cur.v == cur.v);
    VI r;
    r.v = take ? x : cur.v;
    r.i = take ? i : cur.i;
    return r;
  }
  // After the thread's last element: if nothing was ever taken, every element
  // equalled the start value and the first position met is the answer.
  static __device__ __forceinline__ T seal(T acc, int first, bool any) {
    if (any & (acc.i == 0x7fffffff)) acc.i = first;
    return acc;
  }
  static __device__ __forceinline__ T comb(T a, T b) { return vi_comb<KIND>(a, b); }
  static __device__ __forceinline__ T reduce(T v, int width) { return group_reduce_vi<KIND>(v, width); }
  static __device__ __forceinline__ void store(const ReduceDimParams &P, thcl_u32 s, T v) {
    P.out[s] = v.v;
    if (P.idx_f32) P.idx_f32[s] = (float)(v.i + 1);
    if (P.idx_i64) P.idx_i64[s] = (long long)v.i + 1;
  }
};

// Reduced dim is dense in memory: LPR lanes walk one slice, VEC floats each.
// LPR in {1, 8, 64, 256}; a block holds 256/LPR slices.  blockIdx.y cuts long slices
// into pieces of rows_per_split elements (a multiple of 4) that leave partials.
template <int KIND, bool ARG, int LPR, int VEC>
__global__ __launch_bounds__(kThreads) void reduce_rows(ReduceDimParams P) {
  typedef Slot<KIND, ARG> S;
  typedef typename S::T T;
  constexpr int ROWS = kThreads / LPR;
  __shared__ T lds[kThreads / kWave];
  const int sub = threadIdx.x % LPR, row_in_block = threadIdx.x / LPR;
  const thcl_u32 ngroups = (P.nslices + ROWS - 1) / ROWS;
  const thcl_u32 r0 = blockIdx.y * P.rows_per_split;
  const thcl_u32 len = (P.R - r0 < P.rows_per_split) ? (P.R - r0) : P.rows_per_split;
  for (thcl_u32 g = blockIdx.x; g < ngroups; g += gridDim.x) {
    const thcl_u32 s = g * ROWS + row_in_block;
    T acc = S::init();
    if (s < P.nslices) {
      const float *row = P.in + thcl_generic_offset(s, P.L) + r0;
      if (VEC == 4) {
        const rd_f4 *row4 = (const rd_f4 *)row;
        const thcl_u32 r4 = len >> 2;
        constexpr int FLY = 4;  // independent loads issued before any is consumed
        thcl_u32 i = sub;
        for (; i + (FLY - 1) * LPR < r4; i += FLY * LPR) {
          thcl_f4 v[FLY];
#pragma unroll
          for (int f = 0; f < FLY; f++) v[f] = __builtin_nontemporal_load(row4 + i + f * LPR);
#pragma unroll
          for (int f = 0; f < FLY; f++)
#pragma unroll
            for (int c = 0; c < 4; c++) acc = S::take(acc, v[f][c], (int)(r0 + (i + f * LPR) * 4 + c), P.exponent);
        }
        for (; i < r4; i += LPR) {
          const thcl_f4 v = __builtin_nontemporal_load(row4 + i);
#pragma unroll
          for (int c = 0; c < 4; c++) acc = S::take(acc, v[c], (int)(r0 + i * 4 + c), P.exponent);
        }
        if (len & 3u)   // the last one to three elements of a slice whose length is no multiple of 4
          for (thcl_u32 e = (r4 << 2) + sub; e < len; e += LPR) acc = S::take(acc, row[e], (int)(r0 + e), P.exponent);
      } else {
        constexpr int FLY = 4;
        thcl_u32 i = sub;
        for (; i + (FLY - 1) * LPR < len; i += FLY * LPR) {
          float v[FLY];
#pragma unroll
          for (int f = 0; f < FLY; f++) v[f] = row[i + f * LPR];
#pragma unroll
          for (int f = 0; f < FLY; f++) acc = S::take(acc, v[f], (int)(r0 + i + f * LPR), P.exponent);
        }
        for (; i < len; i += LPR) acc = S::take(acc, row[i], (int)(r0 + i), P.exponent);
      }
      // the first position this thread met
      if (VEC == 4) {
        const thcl_u32 r4 = len >> 2;
        acc = S::seal(acc, (int)(r0 + ((thcl_u32)sub < r4 ? (thcl_u32)sub * 4 : (r4 << 2) + sub)), (thcl_u32)sub < r4 || (r4 << 2) + sub < len);
      } else {
        acc = S::seal(acc, (int)(r0 + sub), (thcl_u32)sub < len);
      }
    }
    if (LPR <= kWave) {
      acc = S::reduce(acc, LPR);
      if (sub == 0 && s < P.nslices) {
        if (P.split > 1) ((T *)P.partials)[(thcl_u64)blockIdx.y * P.nslices + s] = acc;
        else S::store(P, s, acc);
      }
    } else {
      acc = S::reduce(acc, kWave);
      const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
      __syncthreads();
      if (lane == 0) lds[wave] = acc;
      __syncthreads();
      if (threadIdx.x == 0) {
        T r = lds[0];
        for (int w = 1; w < kThreads / kWave; w++) r = S::comb(r, lds[w]);
        if (P.split > 1) ((T *)P.partials)[(thcl_u64)blockIdx.y * P.nslices + s] = r;
        else S::store(P, s, r);
      }
    }
  }
}

// Reduced dim dense and short (at most 2048 elements, a multiple of 4, 16-byte aligned slices): 2^lpr_log2 lanes
// share a slice, PER float4 each, and FLY = 8 / PER passes of the block's slices are requested before any is
// consumed, so a lane has 8 loads in flight whatever the slice length.  reduce_rows keeps one pass in flight, which
// leaves short slices waiting on memory (2^22 x 16 along dim 2: 71 us, bound 39).
template <int KIND, bool ARG, int LPRL2, int PER>
__global__ __launch_bounds__(kThreads) void reduce_rows_short(ReduceDimParams P) {
  typedef Slot<KIND, ARG> S;
  typedef typename S::T T;
  constexpr int FLY = 8 / PER;
  constexpr thcl_u32 lpr = 1u << LPRL2, rows = (thcl_u32)kThreads >> LPRL2;  // lanes per slice, slices per pass
  const thcl_u32 sub = threadIdx.x & (lpr - 1), rib = threadIdx.x >> LPRL2;
  const thcl_u32 r4 = P.R >> 2;
  const thcl_u32 npass = (P.nslices + rows - 1) / rows;
  for (thcl_u32 p0 = blockIdx.x * FLY; p0 < npass; p0 += gridDim.x * FLY) {
    thcl_f4 v[FLY][PER];
#pragma unroll
    for (int f = 0; f < FLY; f++) {
      // every load is issued: slices and lanes past the end read the last slice / the slice's last float4 again
      // (a branch around a load makes the compiler wait for the loads before it)
      thcl_u32 s = (p0 + f) * rows + rib;
      if (s >= P.nslices) s = P.nslices - 1;
      const rd_f4 *row4 = (const rd_f4 *)(P.in + thcl_generic_offset(s, P.L));
#pragma unroll
      for (int k = 0; k < PER; k++) {
        thcl_u32 i = sub + (thcl_u32)k * lpr;
        if (i >= r4) i = r4 - 1;
        v[f][k] = __builtin_nontemporal_load(row4 + i);
      }
    }
#pragma unroll
    for (int f = 0; f < FLY; f++) {
      const thcl_u32 s = (p0 + f) * rows + rib;
      const bool in = p0 + f < npass && s < P.nslices;
      T acc = S::init();
      if (in) {
#pragma unroll
        for (int k = 0; k < PER; k++) {
          const thcl_u32 i = sub + (thcl_u32)k * lpr;
          if (i < r4) {
#pragma unroll
            for (int c = 0; c < 4; c++) acc = S::take(acc, v[f][k][c], (int)(i * 4 + c), P.exponent);
          }
        }
        acc = S::seal(acc, (int)(sub * 4), sub < r4);
      }
      acc = S::reduce(acc, (int)lpr);
      if (in && sub == 0) S::store(P, s, acc);
    }
  }
}

// Reduced dim is strided: lanes lie along the slices (UB lanes x VEC adjacent
// slices; UB = 64 unless the slices are fewer, then the wave's other lanes take
// further rows), the 4 waves of a block interleave over the reduced dim and meet in
// LDS; blockIdx.y splits long reductions, leaving partials for the finisher.
// GEOM 6 fixes the wave's geometry at compile time (64 units x 1 row); 0 reads it from the launch.
template <int KIND, bool ARG, int VEC, int GEOM>
__global__ __launch_bounds__(kThreads) void reduce_cols(ReduceDimParams P) {
  typedef Slot<KIND, ARG> S;
  typedef typename S::T T;
  constexpr int WAVES = kThreads / kWave;
  constexpr bool NARROW = GEOM != 6;   // several rows across the wave
  __shared__ T lds[WAVES][kWave * VEC];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const thcl_u32 ubl = GEOM ? (thcl_u32)GEOM : P.ub_log2;
  const thcl_u32 UB = 1u << ubl, RL = (thcl_u32)kWave >> ubl;
  const thcl_u32 ul = lane & (UB - 1), rl = (thcl_u32)lane >> ubl;
  const thcl_u32 ntiles = (P.nunits + UB - 1) / UB;
  const thcl_u32 r_begin = blockIdx.y * P.rows_per_split;
  thcl_u32 r_end = r_begin + P.rows_per_split;
  if (r_end > P.R) r_end = P.R;
  const thcl_u32 RSTEP = WAVES * RL;  // rows between a lane's consecutive elements
  for (thcl_u32 tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const thcl_u32 u = tile * UB + ul;
    T acc[VEC];
#pragma unroll
    for (int c = 0; c < VEC; c++) acc[c] = S::init();
    if (u < P.nunits) {
      // a unit is VEC adjacent slices; the innermost slice dim counts units
      thcl_u64 off;
      {
        thcl_u32 i = u;
        off = 0;
        for (int d = P.L.dims - 1; d > 0; d--) {
          const thcl_u32 q = thcl_div(i, P.L.size[d]);
          const thcl_u32 r = i - q * P.L.size[d].d;
          off += (thcl_u64)((d == P.L.dims - 1) ? r * VEC : r) * P.L.stride[d];
          i = q;
        }
        // one inner dim of any length: the last unit is moved back to end with the dim, and gives some slices a
        // second time, from the same rows in the same order
        if (VEC > 1 && P.L.dims == 1 && i * VEC + VEC > P.nslices) off += (thcl_u64)(P.nslices - VEC) * P.L.stride[0];
        else off += (thcl_u64)((P.L.dims == 1) ? i * VEC : i) * P.L.stride[0];
      }
      // this wave takes rows r_begin + wave, + WAVES, ...; FLY of them are loaded
      // before any is consumed, the address advances by a constant step
      constexpr int FLY = 4;   // (batches of 8 rows: the arg-max of 4096 x 16384 along dim 1 took 41.5 us against 40.0, sums the same)
      thcl_u32 r = r_begin + wave * RL + rl;
      const float *ptr = P.in + off + (thcl_u64)r * P.rstride;
      const thcl_u64 step = (thcl_u64)RSTEP * P.rstride;
      if (VEC == 4) {
        // whole batches of FLY rows: the next batch is requested before the current one
        // is consumed, so the wave always has loads in flight
        if (r + (FLY - 1) * RSTEP < r_end) {
          thcl_f4 v[FLY], w[FLY];
          auto fetch = [&](thcl_f4 (&x)[FLY]) {
#pragma unroll
            for (int f = 0; f < FLY; f++) {
              x[f] = __builtin_nontemporal_load((const rd_f4 *)ptr);
              ptr += step;
            }
          };
          auto consume = [&](const thcl_f4 (&x)[FLY]) {
#pragma unroll
            for (int f = 0; f < FLY; f++)
#pragma unroll
              for (int c = 0; c < 4; c++) acc[c] = S::take(acc[c], x[f][c], (int)(r + f * RSTEP), P.exponent);
            r += FLY * RSTEP;
          };
          fetch(v);
          // two batches per turn, each requested while the other is consumed
          while (r + (3 * FLY - 1) * RSTEP < r_end) {
            fetch(w);
            consume(v);
            fetch(v);
            consume(w);
          }
          if (r + (2 * FLY - 1) * RSTEP < r_end) {
            fetch(w);
            consume(v);
            consume(w);
          } else {
            consume(v);
          }
        }
      } else {
        for (; r + (FLY - 1) * RSTEP < r_end; r += FLY * RSTEP) {
          float v[FLY];
#pragma unroll
          for (int f = 0; f < FLY; f++) {
            v[f] = *ptr;
            ptr += step;
          }
#pragma unroll
          for (int f = 0; f < FLY; f++) acc[0] = S::take(acc[0], v[f], (int)(r + f * RSTEP), P.exponent);
        }
      }
      for (; r < r_end; r += RSTEP) {
        if (VEC == 4) {
          const thcl_f4 v0 = *(const rd_f4 *)ptr;
#pragma unroll
          for (int c = 0; c < 4; c++) acc[c] = S::take(acc[c], v0[c], (int)r, P.exponent);
        } else {
          acc[0] = S::take(acc[0], *ptr, (int)r, P.exponent);
        }
        ptr += step;
      }
#pragma unroll
      for (int c = 0; c < VEC; c++)
        acc[c] = S::seal(acc[c], (int)(r_begin + wave * RL + rl), r_begin + wave * RL + rl < r_end);
    }
    // the wave's row lanes of one unit meet first (lanes UB apart)
    if (NARROW) {
      for (thcl_u32 m = UB; m < (thcl_u32)kWave; m <<= 1) {
#pragma unroll
        for (int c = 0; c < VEC; c++) acc[c] = S::comb(acc[c], shfl_xor_t(acc[c], (int)m));
      }
    }
    __syncthreads();
    if (rl == 0) {
#pragma unroll
      for (int c = 0; c < VEC; c++) lds[wave][ul * VEC + c] = acc[c];
    }
    __syncthreads();
    if (wave == 0 && rl == 0 && u < P.nunits) {
#pragma unroll
      for (int c = 0; c < VEC; c++) {
        T r = lds[0][ul * VEC + c];
        for (int w = 1; w < WAVES; w++) r = S::comb(r, lds[w][ul * VEC + c]);
        const thcl_u32 s = ((VEC > 1 && P.L.dims == 1 && u * VEC + VEC > P.nslices) ? P.nslices - VEC : u * VEC) + c;
        if (P.split > 1) store_shared((T *)P.partials + (thcl_u64)blockIdx.y * P.nslices + s, r);
        else S::store(P, s, r);
      }
    }
  }
  if (P.split == 1 || !P.fused) return;
  // Short splits (one tile per block column, gridDim.x == ntiles): the
  // block that arrives last at its tile folds the tile's partials in split
  // order.  Wave 0 wrote this block's partials with device-scope stores,
  // which write through to where all XCDs meet and leave nothing dirty in
  // this XCD's L2; s_waitcnt vmcnt(0) returns when those stores have been
  // acknowledged there; the same wave then takes the ticket (it issues in
  // order), and the last arrival reads with loads that bypass the caches.
  // The stores and the ticket must stay in one wave: another wave's stores
  // would need a barrier before the ticket.  A release-acquire ticket
  // (__ATOMIC_ACQ_REL at device scope) instead of this sequence was measured:
  // it writes back the whole L2 and cost 5.6-8.7 us on 18-44 us launches.
  __shared__ unsigned s_last;
  if (wave == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (lane == 0) {
      const unsigned t = atomicAdd(P.ticket + blockIdx.x, 1u);
      s_last = (t == P.split - 1) ? 1u : 0u;
    }
  }
  __syncthreads();
  if (!s_last) return;
  // J = UB * VEC slices (a power of two, at most 256) share the block's threads: kThreads / J threads walk a slice's
  // partials side by side (split index `parts` apart, up to 8 loads requested together), meet in LDS and are folded in
  // order of their first split index
  const T *partials = (const T *)P.partials;
  const thcl_u32 J = UB * VEC, parts = (thcl_u32)kThreads / J;
  const thcl_u32 j = threadIdx.x % J, part = threadIdx.x / J;
  const thcl_u32 sj = blockIdx.x * J + j;
  const bool live = sj < P.nslices;
  T t = S::init();
  if (live) {
    constexpr int B = 8;
    thcl_u32 k = part;
    for (; k + (B - 1) * parts < P.split; k += B * parts) {
      T v[B];
#pragma unroll
      for (int b = 0; b < B; b++) v[b] = load_fresh(partials + (thcl_u64)(k + b * parts) * P.nslices + sj);
#pragma unroll
      for (int b = 0; b < B; b++) t = S::comb(t, v[b]);
    }
    for (; k < P.split; k += parts) t = S::comb(t, load_fresh(partials + (thcl_u64)k * P.nslices + sj));
  }
  T *meet = &lds[0][0];   // kThreads entries
  meet[part * J + j] = t;
  __syncthreads();
  if (part == 0 && live) {
    T r = meet[j];
    for (thcl_u32 g = 1; g < parts; g++) r = S::comb(r, meet[g * J + j]);
    S::store(P, sj, r);
  }
  if (threadIdx.x == 0) P.ticket[blockIdx.x] = 0u;
}

// Reduced dim is strided and short (R <= 32): a thread owns a unit of VEC adjacent slices and
// walks all of R itself, 4 rows requested at a time; adjacent threads read adjacent units.
template <int KIND, bool ARG, int VEC>
__global__ __launch_bounds__(kThreads) void reduce_cols_short(ReduceDimParams P) {
  typedef Slot<KIND, ARG> S;
  typedef typename S::T T;
  for (thcl_u32 u = blockIdx.x * kThreads + threadIdx.x; u < P.nunits; u += gridDim.x * kThreads) {
    thcl_u64 off = 0;
    {
      thcl_u32 i = u;
      for (int d = P.L.dims - 1; d > 0; d--) {
        const thcl_u32 q = thcl_div(i, P.L.size[d]);
        const thcl_u32 r = i - q * P.L.size[d].d;
        off += (thcl_u64)((d == P.L.dims - 1) ? r * VEC : r) * P.L.stride[d];
        i = q;
      }
      if (VEC > 1 && P.L.dims == 1 && i * VEC + VEC > P.nslices) off += (thcl_u64)(P.nslices - VEC) * P.L.stride[0];
      else off += (thcl_u64)((P.L.dims == 1) ? i * VEC : i) * P.L.stride[0];
    }
    const thcl_u32 s0 = (VEC > 1 && P.L.dims == 1 && u * VEC + VEC > P.nslices) ? P.nslices - VEC : u * VEC;
    const float *ptr = P.in + off;
    T acc[VEC];
#pragma unroll
    for (int c = 0; c < VEC; c++) acc[c] = S::init();
    constexpr int FLY = 4;
    thcl_u32 r = 0;
    for (; r + FLY <= P.R; r += FLY) {
      float x[FLY][VEC];
#pragma unroll
      for (int f = 0; f < FLY; f++) {
        if (VEC == 4) {
          const thcl_f4 v = __builtin_nontemporal_load((const rd_f4 *)(ptr + (thcl_u64)(r + f) * P.rstride));
#pragma unroll
          for (int c = 0; c < VEC; c++) x[f][c] = v[c];
        } else {
          x[f][0] = ptr[(thcl_u64)(r + f) * P.rstride];
        }
      }
#pragma unroll
      for (int f = 0; f < FLY; f++)
#pragma unroll
        for (int c = 0; c < VEC; c++) acc[c] = S::take(acc[c], x[f][c], (int)(r + f), P.exponent);
    }
    for (; r < P.R; r++) {
      if (VEC == 4) {
        const thcl_f4 v = *(const rd_f4 *)(ptr + (thcl_u64)r * P.rstride);
#pragma unroll
        for (int c = 0; c < VEC; c++) acc[c] = S::take(acc[c], v[c], (int)r, P.exponent);
      } else {
        acc[0] = S::take(acc[0], ptr[(thcl_u64)r * P.rstride], (int)r, P.exponent);
      }
    }
#pragma unroll
    for (int c = 0; c < VEC; c++) S::store(P, s0 + c, S::seal(acc[c], 0, P.R > 0));
  }
}

// Folds the [split][nslices] partials.  A block owns 16 adjacent slices; its 16
// thread groups walk the split index 16 apart (each read is a 128-byte run),
// then the groups meet in LDS and are folded in split order.
constexpr int kFinSlices = 16, kFinParts = kThreads / kFinSlices;
template <int KIND, bool ARG>
__global__ __launch_bounds__(kThreads) void reduce_cols_finish(ReduceDimParams P) {
  typedef Slot<KIND, ARG> S;
  typedef typename S::T T;
  __shared__ T lds[kFinParts][kFinSlices];
  const T *partials = (const T *)P.partials;
  const int sl = threadIdx.x % kFinSlices, part = threadIdx.x / kFinSlices;
  const thcl_u32 s = blockIdx.x * kFinSlices + sl;
  T r = S::init();
  if (s < P.nslices) {
    constexpr int B = 8;   // partials requested together (one after the other a long split of one slice took 24 us)
    thcl_u32 k = part;
    for (; k + (B - 1) * kFinParts < P.split; k += B * kFinParts) {
      T v[B];
#pragma unroll
      for (int b = 0; b < B; b++) v[b] = partials[(thcl_u64)(k + b * kFinParts) * P.nslices + s];
#pragma unroll
      for (int b = 0; b < B; b++) r = S::comb(r, v[b]);
    }
    for (; k < P.split; k += kFinParts) r = S::comb(r, partials[(thcl_u64)k * P.nslices + s]);
  }
  lds[part][sl] = r;
  __syncthreads();
  if (part == 0 && s < P.nslices) {
    // group g holds splits g, g+16, ...: folding groups in order keeps sums
    // reproducible and, for positions, the combine rule is order-independent
    T t = lds[0][sl];
    for (int g = 1; g < kFinParts; g++) t = S::comb(t, lds[g][sl]);
    S::store(P, s, t);
  }
}

// ------------------------------------------------------------ host helpers ---

void fill_operand(ThclGenericOperand &o, const Layout &L) {
  memset(&o, 0, sizeof(o));
  o.dims = L.dims;
  for (int d = 0; d < L.dims; d++) {
    THCL_CHECK(L.strides[d] >= 0 && L.strides[d] < (1l << 32) && L.sizes[d] < (1l << 31), THCL_DIM_WARNING);
    o.size[d] = thcl_make_divisor(L.sizes[d]);
    o.stride[d] = (thcl_u32)L.strides[d];
  }
}

float init_value(ThclReduce kind) {
  switch (kind) {
    case RED_PROD: return 1.f;
    case RED_ALL: return 1.f;
    case RED_MAX: return -INFINITY;
    case RED_MIN: return INFINITY;
    default: return 0.f;  // every sum, and any
  }
}

void check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "%s launch failed: %s", what, hipGetErrorString(e));
}

// walk: 0 dense, 1 strided one element at a time, 4 strided in units of four
template <int KIND>
void launch_all(int walk, unsigned grid, hipStream_t stream, const ReduceAllParams &P) {
  if (walk == 0) hipLaunchKernelGGL(reduce_all_dense<KIND>, dim3(grid), dim3(kThreads), 0, stream, P);
  else if (walk == 4) hipLaunchKernelGGL((reduce_all_strided<KIND, 4>), dim3(grid), dim3(kThreads), 0, stream, P);
  else hipLaunchKernelGGL((reduce_all_strided<KIND, 1>), dim3(grid), dim3(kThreads), 0, stream, P);
}

template <int KIND, bool ARG>
void launch_dim(bool rows, int lpr, int vec, dim3 grid, hipStream_t stream, const ReduceDimParams &P) {
  dim3 block(kThreads);
  if (rows && lpr == -2) {  // short dense slices: vec carries the float4 per lane
#define SHORT_CASE(L2, PER) hipLaunchKernelGGL((reduce_rows_short<KIND, ARG, L2, PER>), grid, block, 0, stream, P)
    if (P.ub_log2 == 0) SHORT_CASE(0, 1);
    else if (P.ub_log2 == 2) SHORT_CASE(2, 1);
    else if (P.ub_log2 == 4) SHORT_CASE(4, 1);
    else if (vec == 1) SHORT_CASE(6, 1);
    else if (vec == 2) SHORT_CASE(6, 2);
    else if (vec == 4) SHORT_CASE(6, 4);
    else SHORT_CASE(6, 8);
#undef SHORT_CASE
  } else if (rows) {
#define ROWS_CASE(L, V) \
  if (lpr == L && vec == V) { hipLaunchKernelGGL((reduce_rows<KIND, ARG, L, V>), grid, block, 0, stream, P); return; }
    ROWS_CASE(1, 1) ROWS_CASE(1, 4) ROWS_CASE(8, 1) ROWS_CASE(8, 4) ROWS_CASE(64, 1) ROWS_CASE(64, 4) ROWS_CASE(256, 1) ROWS_CASE(256, 4)
#undef ROWS_CASE
    thcl_throw("internal: no row-reduction kernel for lanes=%d vec=%d", lpr, vec);
  } else if (lpr < 0) {  // short reduced dim: a thread per unit
    if (vec == 4) hipLaunchKernelGGL((reduce_cols_short<KIND, ARG, 4>), grid, block, 0, stream, P);
    else hipLaunchKernelGGL((reduce_cols_short<KIND, ARG, 1>), grid, block, 0, stream, P);
  } else {
    // fewer than 64 units across the wave: the geometry is read from the launch (fixing 32 or 16 units at compile
    // time measured the same or 5 % slower)
#define COLS_CASE(V, G) hipLaunchKernelGGL((reduce_cols<KIND, ARG, V, G>), grid, block, 0, stream, P)
    if (vec == 4) {
      if (P.ub_log2 == 6) COLS_CASE(4, 6);
      else COLS_CASE(4, 0);
    } else {
      if (P.ub_log2 == 6) COLS_CASE(1, 6);
      else COLS_CASE(1, 0);
    }
#undef COLS_CASE
  }
}

template <int KIND, bool ARG>
void launch_finish(unsigned grid, hipStream_t stream, const ReduceDimParams &P) {
  hipLaunchKernelGGL((reduce_cols_finish<KIND, ARG>), dim3(grid), dim3(kThreads), 0, stream, P);
}

bool aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
}  // namespace

// ----------------------------------------------------------------- reduce all
// Tickets and partials of the entry point that allocates nothing live in this
// array instead of the context's scratch block: 256 bytes of tickets, then
// kStaticSlots 8-byte partials.  Every device the library runs on holds its own
// copy, zero at load; the kernels leave the ticket at zero when they finish.
constexpr size_t kStaticTicketBytes = 256;
constexpr long kStaticSlots = 2048;
constexpr size_t kStaticScratchBytes = kStaticTicketBytes + (size_t)kStaticSlots * sizeof(double);
constexpr int kStaticMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
namespace {
// the array's address on each device (hipGetSymbolAddress); in host code the name `scratch` is not one
void *g_static_scratch[kStaticMaxDevices] = {nullptr};
}  // namespace

// Called once per device when its context is opened; makes that device current for the look-up.
void thcl_reduce_static_setup(int device) {
  THCL_CHECK(device >= 0 && device < kStaticMaxDevices, "device %d out of range", device);
  if (g_static_scratch[device]) return;
  int prev = -1;
  hipError_t e = hipGetDevice(&prev);
  if (e == hipSuccess && prev != device) e = hipSetDevice(device);  // each device holds its own copy at its own address
  THCL_CHECK(e == hipSuccess, "making device %d current: %s", device, hipGetErrorString(e));
  void *ptr = nullptr;
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e == hipSuccess && ptr != nullptr) e = hipMemset(ptr, 0, kStaticScratchBytes);
  if (prev >= 0 && prev != device) (void)hipSetDevice(prev);
  THCL_CHECK(e == hipSuccess && ptr != nullptr, "static scratch of device %d (hipGetSymbolAddress / clearing it): %s", device,
             hipGetErrorString(e));
  g_static_scratch[device] = ptr;
}

namespace {
// where one whole-tensor reduction keeps its tickets and partials
struct ReduceAllScratch {
  unsigned *ticket;
  void *partials;
  long slots;  // 8-byte partials
};

void reduce_all_launch(thcl_rt *rt, ThclReduce kind, THClTensor *src, long n, float *out, float exponent,
                       const ReduceAllScratch &S, unsigned host_tag = 0);
}  // namespace

void thcl_reduce_all(THClState *state, ThclReduce kind, THClTensor *src, float *out, float exponent, unsigned host_tag) {
  const long n = THClTensor_nElement(state, src);
  THCL_CHECK(src->nDimension <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  int device = THClTensor_getDevice(state, src);
  thcl_rt *rt = thcl_ctx(state, device);
  if (n == 0) {  // nothing to fold: the identity element
    thcl_fill_contig(rt, out, init_value(kind), 1);
    thcl_after_launch(state, rt);
    return;
  }
  THCL_CHECK(src->storage && src->storage->wrapper, "tensor has no device storage");
  size_t sbytes = 0;
  char *block = (char *)thcl_rt_scratch(rt, &sbytes);
  ReduceAllScratch S;
  S.ticket = (unsigned *)(block + kTicketOff);
  S.partials = block + kPartialOff;
  S.slots = (long)((sbytes - kPartialOff - kResultSlot) / sizeof(double));
  reduce_all_launch(rt, kind, src, n, out, exponent, S, host_tag);
  thcl_after_launch(state, rt);
}

// The same reduction with its tickets and partials in the static array: no device memory is
// requested or released, no event is created, nothing is booked by the profiler.  The device's
// context must already be open (opening one allocates).
void thcl_reduce_all_noalloc(THClState *state, ThclReduce kind, THClTensor *src, float *out) {
  const long n = THClTensor_nElement(state, src);
  THCL_CHECK(src->nDimension <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  THCL_CHECK(n <= THCL_NOALLOC_MAX_ELEMENTS,
             "this entry point takes at most %ld elements (the tensor has %ld): use the allocating form",
             (long)THCL_NOALLOC_MAX_ELEMENTS, n);
  const int device = THClTensor_getDevice(state, src);
  THCL_CHECK(state && state->initialized && device >= 0 && device < state->allocatedDevices && device < kStaticMaxDevices &&
                 state->clByDevice[device] != nullptr && g_static_scratch[device] != nullptr,
             "device %d has not been opened yet, and opening it allocates: make any other call on it first", device);
  thcl_rt *rt = state->clByDevice[device];
  if (n == 0) {
    thcl_fill_contig(rt, out, init_value(kind), 1);
  } else {
    THCL_CHECK(src->storage && src->storage->wrapper, "tensor has no device storage");
    char *block = (char *)g_static_scratch[device];
    ReduceAllScratch S;
    S.ticket = (unsigned *)block;
    S.partials = block + kStaticTicketBytes;
    S.slots = kStaticSlots;
    reduce_all_launch(rt, kind, src, n, out, 0.f, S);
  }
  if (state->addFinish) THCL_CHECK(thcl_rt_sync(rt) == 0, "%s", thcl_rt_error());
}

namespace {
void reduce_all_launch(thcl_rt *rt, ThclReduce kind, THClTensor *src, long n, float *out, float exponent,
                       const ReduceAllScratch &S, unsigned host_tag) {
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  ReduceAllParams P;
  memset(&P, 0, sizeof(P));
  P.in = thcl_dptr(src);
  P.n = (thcl_u64)n;
  P.partials = S.partials;
  P.ticket = S.ticket;
  P.out = out;
  P.exponent = exponent;
  P.host_tag = host_tag;
  // The order in which elements are folded is free, so the view is walked in memory order: dims sorted
  // by stride and merged.  A transposed or permuted view of a whole block of memory becomes dense.
  Layout walk;
  {
    THClTensor *one[1] = {src};
    const JointLayout J = thcl_joint_collapse(1, one);
    walk.dims = J.dims;
    for (int d = 0; d < J.dims; d++) {
      walk.sizes[d] = J.sizes[d];
      walk.strides[d] = J.strides[0][d];
    }
  }
  const bool dense = walk.contiguous();
  const int cus = thcl_rt_get_props(rt)->compute_units;
  long want;
  int how = 0;
  if (dense) {
    want = (n / 4 + kThreads * 4 - 1) / (kThreads * 4);
  } else {
    THCL_CHECK(n < (1l << 31), THCL_DIM_WARNING);
    // units of four when every row of the innermost dim is a dense, 16-byte aligned run of a multiple of 4
    const int last = walk.dims - 1;
    const bool vec4 = walk.dims >= 1 && walk.strides[last] == 1 && walk.sizes[last] % 4 == 0;   // the units' 16-byte reads need no alignment
    if (vec4) {
      walk.sizes[last] /= 4;
      walk.strides[last] = 4;
      P.n = (thcl_u64)(n / 4);
      how = 4;
    } else {
      how = 1;
    }
    fill_operand(P.L, walk);
    want = ((long)P.n + kThreads * 8 - 1) / (kThreads * 8);
  }
  // Every block costs about 10 ns at the end (its partial and its ticket go through one point of the memory
  // system), so the grid is as small as keeps HBM busy: two blocks per CU from 128 MiB up, one below (2^22
  // elements: 10.5 -> 7.1 us), two for walks in units of four, four for walks one element at a time
  // (measured with 1 to 12 blocks per CU: the half rows of an 8192^2 matrix 39 -> 27 us with 2 instead of 8).
  long cap = (long)cus * (dense ? ((size_t)n * sizeof(float) >= (size_t)cus * 2 * 262144 ? 2 : 1) : (how == 4 ? 2 : 4));
  if (cap > S.slots) cap = S.slots;
  unsigned grid = (unsigned)(want < 1 ? 1 : (want > cap ? cap : want));
  switch (kind) {
    case RED_SUM: launch_all<RED_SUM>(how, grid, stream, P); break;
    case RED_PROD: launch_all<RED_PROD>(how, grid, stream, P); break;
    case RED_MAX: launch_all<RED_MAX>(how, grid, stream, P); break;
    case RED_MIN: launch_all<RED_MIN>(how, grid, stream, P); break;
    case RED_SUM_NE0: launch_all<RED_SUM_NE0>(how, grid, stream, P); break;
    case RED_SUM_ABS: launch_all<RED_SUM_ABS>(how, grid, stream, P); break;
    case RED_SUM_SQ: launch_all<RED_SUM_SQ>(how, grid, stream, P); break;
    case RED_SUM_POW: launch_all<RED_SUM_POW>(how, grid, stream, P); break;
    case RED_ALL: launch_all<RED_ALL>(how, grid, stream, P); break;
    case RED_ANY: launch_all<RED_ANY>(how, grid, stream, P); break;
  }
  check_launch("reduce-all");
}
}  // namespace

// One device scalar to the pinned {value, tag} pair the host polls.
__global__ void scalar_to_host(const float *src, unsigned long long *pair, unsigned tag) {
  const unsigned long long w = (unsigned long long)__float_as_uint(*src) | ((unsigned long long)tag << 32);
  __hip_atomic_store(pair, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
void thcl_scalar_to_host(THClState *state, thcl_rt *rt, const float *src, unsigned host_tag) {
  hipLaunchKernelGGL(scalar_to_host, dim3(1), dim3(1), 0, (hipStream_t)thcl_rt_stream(rt), src,
                     (unsigned long long *)thcl_rt_tagged_word_device(rt), host_tag);
  check_launch("scalar to host");
  thcl_after_launch(state, rt);
}

// A small dense tensor to the page-locked mailbox, then the tagged pair: the host picks it up as soon as the tag
// lands (4 KiB: 23 us through the runtime's copy and its wait for the stream, 11 us this way).  One block: every
// thread's stores are pushed out to the system before the barrier, the tag follows the barrier.
__global__ __launch_bounds__(1024) void small_to_host(const float *src, float *box, unsigned n, unsigned long long *pair, unsigned tag) {
  for (unsigned i = threadIdx.x; i < n; i += 1024) box[i] = src[i];
  __threadfence_system();
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(pair, (unsigned long long)tag << 32, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
void thcl_small_to_host(THClState *state, thcl_rt *rt, const float *src, long n, unsigned host_tag) {
  hipLaunchKernelGGL(small_to_host, dim3(1), dim3(1024), 0, (hipStream_t)thcl_rt_stream(rt), src, thcl_rt_mailbox_device(rt), (unsigned)n,
                     (unsigned long long *)thcl_rt_tagged_word_device(rt), host_tag);
  check_launch("small tensor to host");
  thcl_after_launch(state, rt);
}

// out[0] = sum a[i] * b[i], both dense with n elements
void thcl_dot_dense(THClState *state, thcl_rt *rt, const float *a, const float *b, long n, float *out, unsigned host_tag) {
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  if (n == 0) {
    thcl_fill_contig(rt, out, 0.f, 1);
    thcl_after_launch(state, rt);
    return;
  }
  size_t sbytes = 0;
  char *sblock = (char *)thcl_rt_scratch(rt, &sbytes);
  ReduceAllParams P;
  memset(&P, 0, sizeof(P));
  P.in = a;
  P.n = (thcl_u64)n;
  P.partials = sblock + kPartialOff;
  P.ticket = (unsigned *)(sblock + kTicketOff);
  P.out = out;
  P.host_tag = host_tag;
  // units of four, read with 16-byte loads that need no alignment (vectors starting at odd elements: 2.1 -> 6.5 TB/s)
  const long want = (n / 4 + kThreads * 4 - 1) / (kThreads * 4);
  // one block per CU below 128 MiB of operands, two above (every block costs about 10 ns at the end)
  const long cus = thcl_rt_get_props(rt)->compute_units;
  long cap = cus * ((size_t)n * 2 * sizeof(float) >= (size_t)cus * 2 * 262144 ? 2 : 1);
  const long max_partials = (long)((sbytes - kPartialOff - kResultSlot) / sizeof(double));
  if (cap > max_partials) cap = max_partials;
  const unsigned grid = (unsigned)(want < 1 ? 1 : (want > cap ? cap : want));
  hipLaunchKernelGGL(dot_dense, dim3(grid), dim3(kThreads), 0, stream, P, b);
  check_launch("dot");
  thcl_after_launch(state, rt);
}

// ------------------------------------------------------------ reduce along dim
void thcl_reduce_dim(THClState *state, ThclReduce kind, THClTensor *values, THClTensor *indices_f32,
                     int64_t *idx_i64_dev, THClTensor *src, long dim, float exponent) {
  thcl_check_same_device(state, 3, values, indices_f32, src);
  THCL_CHECK(src->nDimension <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  if (src->nDimension <= 0) return;  // nothing to reduce (src/lib/THClReduce.cpp:234-237)
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 3, "dimension out of range");
  THCL_CHECK(values != src && indices_f32 != src, "result and source must be different tensors");
  THCL_CHECK(src->storage && src->storage->wrapper, "tensor has no device storage");
  const bool arg = (kind == RED_MAX || kind == RED_MIN) && (indices_f32 != nullptr || idx_i64_dev != nullptr);
  const int device = THClTensor_getDevice(state, src);
  thcl_rt *rt = thcl_ctx(state, device);
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);

  // outputs take the source's shape with size 1 along dim (src/lib/THClReduce.cpp:258-262)
  long osz[THCL_MAX_DIMS];
  long nslices = 1;
  for (int d = 0; d < src->nDimension; d++) {
    osz[d] = (d == dim) ? 1 : src->size[d];
    nslices *= osz[d];
  }
  THLongStorage oshape;
  memset(&oshape, 0, sizeof(oshape));
  oshape.data = osz;
  oshape.size = src->nDimension;
  if (values->nDimension < 0 && !values->storage) values->device = device;
  THClTensor_resize(state, values, &oshape, nullptr);
  if (indices_f32) {
    if (indices_f32->nDimension < 0 && !indices_f32->storage) indices_f32->device = device;
    THClTensor_resize(state, indices_f32, &oshape, nullptr);
  }
  const long R = src->size[dim];
  THCL_CHECK(nslices < (1l << 31) && R < (1l << 31), THCL_DIM_WARNING);
  THCL_CHECK(thcl_fits_32bit(src), THCL_DIM_WARNING);
  // a dimension of size 1: every slice is its one element, at position 1
  if (R == 1 && idx_i64_dev == nullptr && (kind == RED_SUM || kind == RED_PROD || kind == RED_MAX || kind == RED_MIN)) {
    THClTensor_copy(state, values, src);
    if (indices_f32) THClTensor_fill(state, indices_f32, 1.0f);
    return;
  }

  // kernels write dense outputs; strided destinations get a dense stand-in
  THClTensor *vdense = values, *idense = indices_f32;
  ThclTemp v_hold(state, nullptr), i_hold(state, nullptr);
  if (!THClTensor_isContiguous(state, values)) {
    v_hold.t = vdense = THClTensor_newv2(state, device);
    THClTensor_resize(state, vdense, &oshape, nullptr);
  }
  if (indices_f32 && !THClTensor_isContiguous(state, indices_f32)) {
    i_hold.t = idense = THClTensor_newv2(state, device);
    THClTensor_resize(state, idense, &oshape, nullptr);
  }

  // one slice and no positions asked for: the whole view folds into one number, which the reduce-all kernels do in
  // one launch (a row of 2^26 elements: 59 us as a split row reduction with its second launch, 42 us this way)
  if (nslices == 1 && !arg) {
    thcl_reduce_all(state, kind, src, thcl_dptr(vdense), exponent);
    if (vdense != values) v_hold.give_to(values);
    return;
  }

  ReduceDimParams P;
  memset(&P, 0, sizeof(P));
  P.in = thcl_dptr(src);
  P.out = thcl_dptr(vdense);
  P.idx_f32 = idense ? thcl_dptr(idense) : nullptr;
  P.idx_i64 = (long long *)idx_i64_dev;
  P.nslices = (thcl_u32)nslices;
  P.R = (thcl_u32)R;
  P.rstride = (thcl_u32)src->stride[dim];
  P.split = 1;
  P.rows_per_split = P.R;
  P.exponent = exponent;
  Layout L = thcl_collapse(src, (int)dim);
  fill_operand(P.L, L);

  size_t sbytes = 0;
  char *sblock = (char *)thcl_rt_scratch(rt, &sbytes);
  P.partials = sblock + kPartialOff;
  P.ticket = (unsigned *)(sblock + kTicketOff) + kColTicket0;
  const long partial_cap = (long)((sbytes - kPartialOff - kResultSlot) / 8);  // 8-byte entries
  const int cus = thcl_rt_get_props(rt)->compute_units;

  const bool rows = (src->stride[dim] == 1) || R == 1;
  int lpr = 0, vec = 1;
  dim3 grid(1, 1, 1);
  if (rows) {
    // lanes per slice: a whole block for long slices, a thread for the shortest ones
    lpr = R >= 2048 ? 256 : (R >= 128 ? 64 : (R > 16 ? 8 : 1));
    // 16-byte reads that need no alignment: a slice may start at any element, and from 64 elements up it may have any
    // length (the last one to three elements are taken singly)
    const bool v4 = (R % 4 == 0) || R >= 64;
    vec = v4 ? 4 : 1;
    if (v4 && R % 4 == 0 && R <= 2048 && R > 1) {
      // short dense slices: enough lanes for one float4 each up to 256 elements, then 2, 4 or 8 float4 per lane
      const long r4 = R / 4;
      unsigned l2 = 0;
      while ((1l << l2) < r4 && l2 < 6) l2 += 2;   // 1, 4, 16 or 64 lanes
      int per = 1;
      while ((long)per * 64 < r4) per *= 2;
      P.ub_log2 = l2;
      lpr = -2;
      vec = per;
      const long slices_per_pass = kThreads >> l2, passes = (nslices + slices_per_pass - 1) / slices_per_pass;
      const long fly = 8 / per, blocks = (passes + fly - 1) / fly;
      grid.x = (unsigned)(blocks > (1l << 22) ? (1l << 22) : blocks);
    } else {
    const long groups = (nslices + (kThreads / lpr) - 1) / (kThreads / lpr);
    grid.x = (unsigned)(groups > (1l << 22) ? (1l << 22) : groups);
    // few long slices: cut them into pieces of at least 8192 elements until the chip is full
    if (lpr == 256 && groups < (long)cus * 4) {
      long split = ((long)cus * 8 + groups - 1) / groups;
      if (split > R / 8192) split = R / 8192;
      if (split > 1024) split = 1024;
      if (split * nslices > partial_cap) split = partial_cap / nslices;
      if (split > 1) {
        long rps = ((R + split - 1) / split + 1023) / 1024 * 1024;  // whole passes of the block's 256 x 4 elements
        split = (R + rps - 1) / rps;
        if (split > 1) {
          P.split = (thcl_u32)split;
          P.rows_per_split = (thcl_u32)rps;
          grid.y = (unsigned)split;
          // (folding the pieces in the same launch, the last arrival at a ticket per slice, measured slower: these
          // blocks live for a microsecond or two, and a write-through, its acknowledgement and an atomic at the end
          // of each keep its CU slot twice as long: 64 x 2^20 41.4 -> 46.6 us, 16 x 2^22 44.2 -> 52.0)
        }
      }
    }
    }
  } else {
    const int last = L.dims - 1;
    // units of 4 columns, read without alignment; a single inner dim may have any length from 8 up (its last unit
    // is moved back to end with it)
    const bool v4 = L.strides[last] == 1 && (L.sizes[last] % 4 == 0 || (L.dims == 1 && L.sizes[last] >= 8));
    vec = v4 ? 4 : 1;
    if (v4) P.L.size[last] = thcl_make_divisor((L.sizes[last] + 3) / 4);
    P.nunits = (thcl_u32)((nslices + vec - 1) / vec);
    // a short reduced dim with enough slices to fill the chip: a thread per unit, no exchange
    if (R <= 32 && (long)P.nunits >= (long)cus * 1024) {
      lpr = -1;
      const long blocks = ((long)P.nunits + kThreads - 1) / kThreads;
      grid.x = (unsigned)(blocks > (1l << 22) ? (1l << 22) : blocks);
    } else {
    // Geometry of a wave: 2^ub_log2 units side by side, 64 >> ub_log2 rows.  Fewer units than lanes: the spare lanes
    // take further rows.  Otherwise the widest tile that still gives every CU a block without splitting the reduced
    // dim, down to 16 units (256 bytes of each row): partials and their fold cost more than the narrower runs
    // (4096x16384 along dim 1: 64 units and 16 splits 46.5 us, 16 units and no split 39.9; 4096x8192: 26.5 -> 22.8),
    // as long as a lane still walks 16 rows or more.  With 4-byte units a narrower tile would read less than
    // 256 bytes of a row, so those keep the full wave.
    unsigned ub_log2 = 6;
    while (ub_log2 > 0 && (1u << (ub_log2 - 1)) >= P.nunits) ub_log2--;
    // (a run of 256 or 512 bytes that does not start on a 128-byte line touches one line more than it fills:
    // rows whose pitch is no multiple of 128 bytes keep the full kibibyte)
    if (vec == 4 && src->stride[dim] % 32 == 0 && aligned16(P.in)) {
      while (ub_log2 > 4 && ((long)P.nunits + (1l << ub_log2) - 1) >> ub_log2 < (long)cus &&
             R / ((kThreads / kWave) * (long)(kWave >> (ub_log2 - 1))) >= 16)
        ub_log2--;
    }
    P.ub_log2 = ub_log2;
    const long ub = 1l << ub_log2, row_lanes = kWave >> ub_log2;
    const long tiles = (P.nunits + ub - 1) / ub;
    // a block per CU: split the reduced dim when the tiles are fewer (every extra split is another partial per slice)
    long split = 1;
    // (two per CU for very tall slices walked one element per lane, which keep less in flight per wave:
    // 2^24 x 3 along dim 1 3.7 -> 5.2 TB/s; with 16-byte units a second block per CU costs 10 %)
    const bool more = vec == 1 && R >= (1l << 22);
    const long target = (long)cus * (more ? 2 : 1);
    if (tiles < target) {
      split = (target + tiles - 1) / tiles;
      const long max_by_rows = (R + 32 * row_lanes - 1) / (32 * row_lanes);  // at least 32 rows per lane
      if (split > max_by_rows) split = max_by_rows;
      if (split > (more ? 512 : 256)) split = more ? 512 : 256;
      if (split * nslices > partial_cap) split = partial_cap / nslices;
      if (split < 1) split = 1;
    }
    long rps = (R + split - 1) / split;
    split = (R + rps - 1) / rps;
    P.split = (thcl_u32)split;
    P.rows_per_split = (thcl_u32)rps;
    // One block folding a tile's partials is quick while each of its threads has few of them to fetch (the tile's
    // slices share the block's 256 threads); beyond 64 a thread the fold is left to a second, chip-wide kernel.
    P.fused = (split > 1 && split * ub * vec <= 64 * (long)kThreads && tiles <= (long)kColTickets) ? 1u : 0u;
    grid.x = (unsigned)(tiles > (1l << 20) ? (1l << 20) : tiles);
    grid.y = (unsigned)split;
    }
  }

#define DISPATCH(K)                                                       \
  if (arg) launch_dim<K, true>(rows, lpr, vec, grid, stream, P);          \
  else launch_dim<K, false>(rows, lpr, vec, grid, stream, P);             \
  check_launch("reduce-dim");                                             \
  if (P.split > 1 && !P.fused) {                                          \
    unsigned fg = (unsigned)((nslices + kFinSlices - 1) / kFinSlices);    \
    if (arg) launch_finish<K, true>(fg, stream, P);                       \
    else launch_finish<K, false>(fg, stream, P);                          \
    check_launch("reduce-dim finish");                                    \
  }
#define DISPATCH_VALUES(K)                                                \
  launch_dim<K, false>(rows, lpr, vec, grid, stream, P);                  \
  check_launch("reduce-dim");                                             \
  if (P.split > 1 && !P.fused) {                                          \
    unsigned fg = (unsigned)((nslices + kFinSlices - 1) / kFinSlices);    \
    launch_finish<K, false>(fg, stream, P);                               \
    check_launch("reduce-dim finish");                                    \
  }
  switch (kind) {
    case RED_SUM: DISPATCH(RED_SUM) break;
    case RED_PROD: DISPATCH(RED_PROD) break;
    case RED_MAX: DISPATCH(RED_MAX) break;
    case RED_MIN: DISPATCH(RED_MIN) break;
    case RED_SUM_NE0: DISPATCH_VALUES(RED_SUM_NE0) break;
    case RED_SUM_ABS: DISPATCH_VALUES(RED_SUM_ABS) break;
    case RED_SUM_SQ: DISPATCH_VALUES(RED_SUM_SQ) break;
    case RED_SUM_POW: DISPATCH_VALUES(RED_SUM_POW) break;
    default: thcl_throw("internal: reduction kind %d does not run along a dimension", (int)kind);
  }
#undef DISPATCH_VALUES
#undef DISPATCH
  thcl_after_launch(state, rt);
  if (vdense != values) v_hold.give_to(values);
  if (idense != indices_f32) i_hold.give_to(indices_f32);
}
