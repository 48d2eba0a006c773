// Inclusive scans along one dimension: cumsum, cumprod.
//
// What it replaces (reference): THClTensor_scanDim and its two kernels
// (src/lib/THClTensorMathScan.cpp:27-156, THClTensorMathScan.cl), which walk
// every row with one thread (outer dims) or 16 threads (innermost dim).
//
// The tensor is taken as dense [O][R][I] (outer, scanned, inner).  Numerics
// follow Torch7's CPU path: the running value is fp64 and every output is its
// rounding to fp32.  The kernels:
//   * scan_seq: one thread per (o, i) walks r; adjacent threads are adjacent in
//     i, so accesses coalesce whenever I is not tiny.
//   * scan_row: I == 1 and long rows; a block walks the row 1024 elements at a
//     time with a block-wide fp64 prefix in each step.
//   * scan_short_rows: I == 1 and many short rows; 1 to 64 lanes share a row
//     and adjacent lane groups take adjacent rows.
//   * scan_wave_rows: I == 1 and many aligned rows of 1024 to 8191 elements; a
//     wave per row with the next 1024 elements requested ahead.
//   * scan_strip: I > 1 with fewer columns than the chip has threads; a block
//     walks 32 or 64 columns, 64 to 256 rows a step.
//   * scan_chain: I == 1 and rows too few for a block each, 2^24 elements and more:
//     one pass by blocks that run together and hand their chunk totals on.
// When O * I alone cannot fill the chip otherwise, R is cut into S segments and the
// scan becomes three passes: segment totals, an exclusive scan of the totals, then
// the scan proper with each segment's carry-in.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <cstdlib>
#include <cstring>

#include "apply_device.h"
#include "internal.h"

namespace {

// a 16-byte access that only needs the alignment of its elements (rows of odd length start anywhere)
typedef thcl_f4 sc_f4u __attribute__((aligned(4)));


constexpr int kThreads = 256;
constexpr int kWave = 64;
// Rows that are cut into segments go through in windows of this many input bytes: totals pass and scan pass of a
// window run back to back, so the second read is served by the memory-side cache (256 MiB on this chip; windows of
// 128, 192 and 256 MiB measured within 4 % of each other, 64 MiB 12 % slower).
constexpr unsigned long long kScanWindowBytes = 256ull << 20;
constexpr int kScanSegment = 8192;

struct ScanParams {
  const float *in;
  float *out;
  double *totals;  // [O][S][I]: segment totals, turned into carries in place
  thcl_u64 O, R, I;
  thcl_u64 S, seg;  // segments per scanned line and their length
  thcl_u64 block0;  // scan_row: the first (row, segment) pair of this launch (long inputs go window by window)
  thcl_u32 own_carry;  // scan_row, PHASE 1: totals still hold totals; a block folds the ones ahead of it itself
  double *ahead_in;    // own_carry: what the row of this launch's first segment has accumulated in earlier launches
  double *ahead_out;   // own_carry: the launch's last block leaves its row's running value here for the next launch
};

template <bool PROD>
struct Op {
  static __device__ __forceinline__ double identity() { return PROD ? 1.0 : 0.0; }
  static __device__ __forceinline__ double comb(double a, double b) { return PROD ? a * b : a + b; }
};

// PHASE 0: segment totals only.  PHASE 1: the scan, seeded with the carry when S > 1.
template <bool PROD, int PHASE>
__global__ __launch_bounds__(kThreads) void scan_seq(ScanParams P) {
  const thcl_u64 t = (thcl_u64)blockIdx.x * kThreads + threadIdx.x;
  if (t >= P.O * P.S * P.I) return;
  const thcl_u64 i = t % P.I, s = (t / P.I) % P.S, o = t / (P.I * P.S);
  const thcl_u64 r0 = s * P.seg;
  thcl_u64 r1 = r0 + P.seg;
  if (r1 > P.R) r1 = P.R;
  const thcl_u64 first = (o * P.R + r0) * P.I + i;
  const float *src = P.in + first;
  float *dst = P.out + first;
  double acc = Op<PROD>::identity();
  if (PHASE == 1 && P.S > 1) acc = P.totals[t];
  constexpr int FLY = 8;  // independent loads in flight per thread
  thcl_u64 r = r0;
  for (; r + FLY <= r1; r += FLY) {
    float v[FLY];
#pragma unroll
    for (int k = 0; k < FLY; k++) v[k] = __builtin_nontemporal_load(src + (thcl_u64)k * P.I);
    src += (thcl_u64)FLY * P.I;
#pragma unroll
    for (int k = 0; k < FLY; k++) {
      acc = Op<PROD>::comb(acc, (double)v[k]);
      if (PHASE == 1) __builtin_nontemporal_store((float)acc, dst + (thcl_u64)k * P.I);
    }
    if (PHASE == 1) dst += (thcl_u64)FLY * P.I;
  }
  for (; r < r1; r++) {
    acc = Op<PROD>::comb(acc, (double)*src);
    src += P.I;
    if (PHASE == 1) {
      *dst = (float)acc;
      dst += P.I;
    }
  }
  if (PHASE == 0) P.totals[t] = acc;
}

// totals[o][s][i] -> combination of totals[o][0..s-1][i] (exclusive), one thread per (o, i)
template <bool PROD>
__global__ __launch_bounds__(kThreads) void scan_carries(ScanParams P) {
  const thcl_u64 t = (thcl_u64)blockIdx.x * kThreads + threadIdx.x;
  if (t >= P.O * P.I) return;
  const thcl_u64 i = t % P.I, o = t / P.I;
  double *p = P.totals + o * P.S * P.I + i;
  double acc = Op<PROD>::identity();
  for (thcl_u64 s = 0; s < P.S; s++) {
    const double v = *p;
    *p = acc;
    acc = Op<PROD>::comb(acc, v);
    p += P.I;
  }
}

// Same, for few lines with many segments: a wave per (o, i) line, 512 segments
// per step (8 consecutive ones per lane, loaded together) with a shuffle scan
// over the lanes, instead of one thread walking thousands of dependent loads.
template <bool PROD>
__global__ __launch_bounds__(kWave) void scan_carries_wave(ScanParams P) {
  constexpr int PER = 8;
  const thcl_u64 line = blockIdx.x;
  const thcl_u64 i = line % P.I, o = line / P.I;
  double *p = P.totals + o * P.S * P.I + i;
  const int lane = threadIdx.x;
  double carry = Op<PROD>::identity();
  for (thcl_u64 base = 0; base < P.S; base += (thcl_u64)kWave * PER) {
    const thcl_u64 s0 = base + (thcl_u64)lane * PER;
    double v[PER];
#pragma unroll
    for (int k = 0; k < PER; k++) v[k] = s0 + k < P.S ? p[(s0 + k) * P.I] : Op<PROD>::identity();
    double mine = v[0];
#pragma unroll
    for (int k = 1; k < PER; k++) mine = Op<PROD>::comb(mine, v[k]);
    double incl = mine;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const double up = __shfl_up(incl, d, kWave);
      if (lane >= d) incl = Op<PROD>::comb(up, incl);
    }
    double excl = __shfl_up(incl, 1, kWave);
    if (lane == 0) excl = Op<PROD>::identity();
    double run = Op<PROD>::comb(carry, excl);  // everything ahead of this lane's first segment
#pragma unroll
    for (int k = 0; k < PER; k++) {
      if (s0 + k < P.S) p[(s0 + k) * P.I] = run;
      run = Op<PROD>::comb(run, v[k]);
    }
    carry = Op<PROD>::comb(carry, __shfl(incl, kWave - 1, kWave));
  }
}

template <bool PROD>
__device__ __forceinline__ double wave_inclusive(double v) {
  const int lane = threadIdx.x % kWave;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const double up = __shfl_up(v, d, kWave);
    if (lane >= d) v = Op<PROD>::comb(up, v);
  }
  return v;
}

// I == 1: block (o, s) walks its segment of row o.  A step covers UNR runs of
// 1024 elements; in each run a thread holds 4 consecutive elements (one 16-byte
// access), so every wave reads whole lines, and the UNR runs share one pair of
// barriers and keep UNR loads in flight per thread.
// VEC: rows are 16-byte aligned and a multiple of 4 long; otherwise whole groups of 4 still move as 16 bytes, through
// accesses that need no alignment, and only a row's last group goes element by element
template <bool PROD, int PHASE, bool VEC>
__global__ __launch_bounds__(kThreads) void scan_row(ScanParams P) {
  typedef typename std::conditional<VEC, thcl_f4, sc_f4u>::type LT;
  constexpr int WAVES = kThreads / kWave, PER = 4, RUN = kThreads * PER, UNR = 4, STEP = RUN * UNR;
  __shared__ double wave_tot[UNR][WAVES];
  const thcl_u64 bid = P.block0 + blockIdx.x;
  const thcl_u64 o = bid / P.S, s = bid % P.S;
  const thcl_u64 r0 = s * P.seg;
  thcl_u64 r1 = r0 + P.seg;
  if (r1 > P.R) r1 = P.R;
  const float *row = P.in + o * P.R;
  float *orow = P.out + o * P.R;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  double carry = Op<PROD>::identity();
  if (PHASE == 1 && P.S > 1) {
    if (P.own_carry) {
      // Everything ahead of this segment in its row.  Segments of earlier launches arrive as one value (left by
      // the previous launch's last block) when the row began before this launch; the totals of this launch's
      // segments are folded in a fixed order (thread t takes totals t, t + 256, ..., then lanes, then waves).
      const double *tot = P.totals + o * P.S;
      const thcl_u64 row_first = o * P.S;                                   // the row's first (row, segment) pair
      const thcl_u64 from = row_first < P.block0 ? P.block0 - row_first : 0;  // first segment that is this launch's
      double mine = Op<PROD>::identity();
      if (threadIdx.x == 0 && from > 0) mine = *P.ahead_in;
      for (thcl_u64 k = from + threadIdx.x; k < s; k += kThreads) mine = Op<PROD>::comb(mine, tot[k]);
#pragma unroll
      for (int d = kWave / 2; d > 0; d >>= 1) mine = Op<PROD>::comb(mine, __shfl_xor(mine, d, kWave));
      if (lane == 0) wave_tot[0][wave] = mine;
      __syncthreads();
#pragma unroll
      for (int w = 0; w < WAVES; w++) carry = Op<PROD>::comb(carry, wave_tot[0][w]);
      __syncthreads();
    } else {
      carry = P.totals[bid];
    }
  }
  // one step over x (4 runs of 1024 elements starting at base); FULL: every element is inside the segment
  auto work = [&](float (&x)[UNR][PER], thcl_u64 base, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    double a[UNR][PER], incl[UNR];
#pragma unroll
    for (int u = 0; u < UNR; u++) {
      a[u][0] = (double)x[u][0];
#pragma unroll
      for (int c = 1; c < PER; c++) a[u][c] = Op<PROD>::comb(a[u][c - 1], (double)x[u][c]);
      incl[u] = wave_inclusive<PROD>(a[u][PER - 1]);
    }
    __syncthreads();  // wave_tot of the previous step has been read
    if (lane == kWave - 1) {
#pragma unroll
      for (int u = 0; u < UNR; u++) wave_tot[u][wave] = incl[u];
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < UNR; u++) {
      double before = carry;  // everything ahead of this thread's first element of run u
#pragma unroll
      for (int w = 0; w < WAVES; w++) {
        if (w < wave) before = Op<PROD>::comb(before, wave_tot[u][w]);
        carry = Op<PROD>::comb(carry, wave_tot[u][w]);
      }
      if (PHASE == 1) {
        // lanes ahead in this wave: the exclusive prefix is the neighbour's inclusive one
        const double prev = __shfl_up(incl[u], 1, kWave);
        if (lane > 0) before = Op<PROD>::comb(before, prev);
        const thcl_u64 j = base + (thcl_u64)u * RUN + (thcl_u64)threadIdx.x * PER;
        if (FULL || j + PER <= r1) {
          thcl_f4 v;
#pragma unroll
          for (int c = 0; c < PER; c++) v[c] = (float)Op<PROD>::comb(before, a[u][c]);
          __builtin_nontemporal_store(v, (LT *)(orow + j));
        } else {
#pragma unroll
          for (int c = 0; c < PER; c++)
            if (j + c < r1) orow[j + c] = (float)Op<PROD>::comb(before, a[u][c]);
        }
      }
    }
  };
  thcl_u64 base = r0;
  if (base + STEP <= r1) {
    // Whole steps: the next step's loads are issued before this step's work and carry
    // no bounds tests, so they stay in flight across the step's two barriers.
    auto fetch = [&](float (&x)[UNR][PER], thcl_u64 at) {
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        // the totals pass reads with ordinary loads, which leave the window in the memory-side cache for the
        // scan pass that follows it; the scan pass streams
        const LT *src = (const LT *)(row + at + (thcl_u64)u * RUN + (thcl_u64)threadIdx.x * PER);
        const thcl_f4 v = PHASE == 0 ? *src : __builtin_nontemporal_load(src);
#pragma unroll
        for (int c = 0; c < PER; c++) x[u][c] = v[c];
      }
    };
    float x[UNR][PER], xn[UNR][PER];
    fetch(x, base);
    for (; base + 2 * STEP <= r1; base += STEP) {
      fetch(xn, base + STEP);
      work(x, base, std::true_type());
#pragma unroll
      for (int u = 0; u < UNR; u++)
#pragma unroll
        for (int c = 0; c < PER; c++) x[u][c] = xn[u][c];
    }
    work(x, base, std::true_type());
    base += STEP;
  }
  for (; base < r1; base += STEP) {
    float x[UNR][PER];
#pragma unroll
    for (int u = 0; u < UNR; u++) {
      const thcl_u64 j = base + (thcl_u64)u * RUN + (thcl_u64)threadIdx.x * PER;
      if (j + PER <= r1) {
        const thcl_f4 v = __builtin_nontemporal_load((const LT *)(row + j));
#pragma unroll
        for (int c = 0; c < PER; c++) x[u][c] = v[c];
      } else {
#pragma unroll
        for (int c = 0; c < PER; c++) x[u][c] = (j + c < r1) ? row[j + c] : (PROD ? 1.0f : 0.0f);
      }
    }
    work(x, base, std::false_type());
  }
  if (PHASE == 0 && threadIdx.x == 0) P.totals[bid] = carry;
  // the row's running value at the end of this launch, for the launch that continues the row
  if (PHASE == 1 && P.own_carry && blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *P.ahead_out = carry;
}

// I > 1 with too few columns for a thread per column: a block walks a strip of 4 * TC columns
// down its segment of R, (256 / TC) * 8 rows a step.  A thread holds 8 consecutive rows of 4
// adjacent columns (one 16-byte access per row; the TC threads that share a row read 16 * TC
// contiguous bytes), so 256 / TC rows per column are combined side by side: thread totals, a
// shuffle scan over the row groups of a wave, the 4 waves' totals through LDS, then the rows are
// finished from the registers.  One barrier a step; the rows of the next two steps are requested before
// this step's work (two steps ahead instead of one: 108 -> 103 us on 4096 x 16384).  TC = 16 for wide tensors that
// have a strip of 64 columns for every CU, else 8; with 4 to 28 columns TC = 1, 2, 4 or 8 covers the whole
// width and consecutive rows are adjacent in memory, so a step reads one contiguous run.  PHASE 0 leaves the segment's
// totals, PHASE 1 scans (from the segment's carry when the lines are cut into segments).
// ANY: the width need not be a multiple of 4 nor the rows 16-byte aligned (narrow tensors only): a thread's up to 4
// columns are read and written one element each, columns past the width are dead.
template <bool PROD, int TC, int PHASE, bool ANY = false, bool HALF = false>
__global__ __launch_bounds__(kThreads) void scan_strip(ScanParams P) {
  // rows per thread: 8; 2 on the narrowest strips, where a thread's 8 rows would be 128 or 256 contiguous
  // bytes read 16 at a time (measured 0.6 TB/s on 4 columns against 2.0 with 2 rows); HALF: 4, for launches of
  // one block per CU (8192 x 8192: 104 -> 90 us, 4096 x 16384: 98 -> 88; with two blocks per CU or half a
  // block 8 rows stay ahead: 2048 x 32768 99 against 102 us, 16384 x 4096 126 against 138)
  constexpr int K = HALF ? 4 : (TC >= 4 && !ANY) ? 8 : 2;  // element-wise strips: lanes that share an instruction stay 2 rows apart
  constexpr int WAVES = kThreads / kWave, ROWS = kThreads / TC * K, CW = TC * 4;
  __shared__ double wave_tot[2][WAVES][CW];
  const thcl_u64 strips = ((P.I + 3) / 4 + TC - 1) / TC;
  const thcl_u64 strip = blockIdx.x % strips, seg_id = (blockIdx.x / strips) % P.S, o = blockIdx.x / (strips * P.S);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int tc = threadIdx.x % TC, tr = threadIdx.x / TC;
  const thcl_u64 col = (strip * TC + tc) * 4;
  const bool live = col < P.I;
  const int ncols = !ANY ? 4 : (!live ? 0 : (P.I - col < 4 ? (int)(P.I - col) : 4));  // this thread's columns inside the width
  const thcl_u64 first = o * P.R * P.I + (live ? col : 0);
  const float *src = P.in + first;
  float *dst = P.out + first;
  const float fill = PROD ? 1.0f : 0.0f;
  const thcl_u64 rbegin = seg_id * P.seg;
  const thcl_u64 rend = (rbegin + P.seg < P.R) ? rbegin + P.seg : P.R;
  // rows past the end are read from the last row (so that every load is issued) and replaced
  auto fetch = [&](thcl_f4 (&x)[K], thcl_u64 r0) {
#pragma unroll
    for (int k = 0; k < K; k++) {
      const thcl_u64 r = r0 + (thcl_u64)tr * K + k;
      const float *at = src + (r < rend ? r : rend - 1) * P.I;
      if (!ANY) {
        x[k] = __builtin_nontemporal_load((const thcl_f4 *)at);
      } else {
        // dead columns read the thread's first column again (an address inside the tensor) and become the identity
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const float v = at[c < ncols ? c : 0];
          x[k][c] = c < ncols ? v : fill;
        }
      }
    }
  };
  double *tot = P.totals + (o * P.S + seg_id) * P.I + (live ? col : 0);
  double carry[4];
#pragma unroll
  for (int c = 0; c < 4; c++) carry[c] = (PHASE == 1 && P.S > 1 && c < ncols) ? tot[c] : Op<PROD>::identity();
  // one step: the 256 / TC * K rows from r0, held in x
  auto step = [&](thcl_f4 (&x)[K], thcl_u64 r0, int buf) {
#pragma unroll
    for (int k = 0; k < K; k++)
      if (r0 + (thcl_u64)tr * K + k >= rend) x[k] = thcl_f4{fill, fill, fill, fill};
    double incl[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
      double t = (double)x[0][c];
#pragma unroll
      for (int k = 1; k < K; k++) t = Op<PROD>::comb(t, (double)x[k][c]);
      // the row groups of this wave sit TC lanes apart
#pragma unroll
      for (int d = TC; d < kWave; d <<= 1) {
        const double up = __shfl_up(t, d, kWave);
        if (lane >= d) t = Op<PROD>::comb(up, t);
      }
      incl[c] = t;
    }
    if (lane >= kWave - TC) {
#pragma unroll
      for (int c = 0; c < 4; c++) wave_tot[buf][wave][tc * 4 + c] = incl[c];
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 4; c++) {
      double before = carry[c];
#pragma unroll
      for (int w = 0; w < WAVES; w++) {
        const double wt = wave_tot[buf][w][tc * 4 + c];
        if (w < wave) before = Op<PROD>::comb(before, wt);
        carry[c] = Op<PROD>::comb(carry[c], wt);
      }
      const double prev = __shfl_up(incl[c], TC, kWave);
      if (lane >= TC) before = Op<PROD>::comb(before, prev);
      incl[c] = before;  // from here on: the running value of column c
    }
    if (PHASE == 1) {
#pragma unroll
      for (int k = 0; k < K; k++) {
        thcl_f4 v;
#pragma unroll
        for (int c = 0; c < 4; c++) {
          incl[c] = Op<PROD>::comb(incl[c], (double)x[k][c]);
          v[c] = (float)incl[c];
        }
        const thcl_u64 r = r0 + (thcl_u64)tr * K + k;
        if (!ANY) {
          if (live && r < rend) __builtin_nontemporal_store(v, (thcl_f4 *)(dst + r * P.I));
        } else if (r < rend) {
#pragma unroll
          for (int c = 0; c < 4; c++)
            if (c < ncols) dst[r * P.I + c] = v[c];
        }
      }
    }
  };
  // three sets of registers take turns: while one step is worked on, the rows of the next two are on their way
  // (six steps a round: the register sets come round every three, the two LDS buffers every two)
  thcl_f4 xa[K], xb[K], xc[K];
  fetch(xa, rbegin);
  fetch(xb, rbegin + ROWS);
  thcl_u64 r0 = rbegin;
  for (;;) {
    fetch(xc, r0 + 2 * ROWS);
    __builtin_amdgcn_sched_barrier(0);
    step(xa, r0, 0);
    r0 += ROWS;
    if (r0 >= rend) break;
    fetch(xa, r0 + 2 * ROWS);
    __builtin_amdgcn_sched_barrier(0);
    step(xb, r0, 1);
    r0 += ROWS;
    if (r0 >= rend) break;
    fetch(xb, r0 + 2 * ROWS);
    __builtin_amdgcn_sched_barrier(0);
    step(xc, r0, 0);
    r0 += ROWS;
    if (r0 >= rend) break;
    fetch(xc, r0 + 2 * ROWS);
    __builtin_amdgcn_sched_barrier(0);
    step(xa, r0, 1);
    r0 += ROWS;
    if (r0 >= rend) break;
    fetch(xa, r0 + 2 * ROWS);
    __builtin_amdgcn_sched_barrier(0);
    step(xb, r0, 0);
    r0 += ROWS;
    if (r0 >= rend) break;
    fetch(xb, r0 + 2 * ROWS);
    __builtin_amdgcn_sched_barrier(0);
    step(xc, r0, 1);
    r0 += ROWS;
    if (r0 >= rend) break;
  }
  if (PHASE == 0 && tr == 0 && live) {
#pragma unroll
    for (int c = 0; c < 4; c++)
      if (c < ncols) tot[c] = carry[c];
  }
}

// I == 1 and short rows: G lanes (a power of two <= 64) share a row, 4
// consecutive elements per lane per step; a block holds 256 / G rows.  No LDS:
// the prefix over a row's lanes is a shuffle scan of width G.
template <bool PROD, int G, bool VEC>
__global__ __launch_bounds__(kThreads) void scan_short_rows(ScanParams P) {
  typedef typename std::conditional<VEC, thcl_f4, sc_f4u>::type LT;
  constexpr int PER = 4, ROWS = kThreads / G;
  const int sub = threadIdx.x % G;
  const thcl_u64 o = (thcl_u64)blockIdx.x * ROWS + threadIdx.x / G;
  const bool live = o < P.O;   // dead groups still take part in the shuffles of their wave
  const float *row = P.in + (live ? o : 0) * P.R;
  float *orow = P.out + (live ? o : 0) * P.R;
  double carry = Op<PROD>::identity();
  for (thcl_u64 base = 0; base < P.R; base += G * PER) {
    const thcl_u64 j = base + (thcl_u64)sub * PER;
    float x[PER];
    if (live && j + PER <= P.R) {
      const thcl_f4 v = __builtin_nontemporal_load((const LT *)(row + j));
#pragma unroll
      for (int c = 0; c < PER; c++) x[c] = v[c];
    } else {
#pragma unroll
      for (int c = 0; c < PER; c++) x[c] = (live && j + c < P.R) ? row[j + c] : (PROD ? 1.0f : 0.0f);
    }
    double a[PER];
    a[0] = (double)x[0];
#pragma unroll
    for (int c = 1; c < PER; c++) a[c] = Op<PROD>::comb(a[c - 1], (double)x[c]);
    double incl = a[PER - 1];
#pragma unroll
    for (int d = 1; d < G; d <<= 1) {
      const double up = __shfl_up(incl, d, G);
      if (sub >= d) incl = Op<PROD>::comb(up, incl);
    }
    double before = carry;
    if (G > 1) {
      const double prev = __shfl_up(incl, 1, G);
      if (sub > 0) before = Op<PROD>::comb(before, prev);
      carry = Op<PROD>::comb(carry, __shfl(incl, G - 1, G));
    } else {
      carry = Op<PROD>::comb(carry, incl);
    }
    if (live) {
      if (j + PER <= P.R) {
        thcl_f4 v;
#pragma unroll
        for (int c = 0; c < PER; c++) v[c] = (float)Op<PROD>::comb(before, a[c]);
        __builtin_nontemporal_store(v, (LT *)(orow + j));
      } else {
#pragma unroll
        for (int c = 0; c < PER; c++)
          if (j + c < P.R) orow[j + c] = (float)Op<PROD>::comb(before, a[c]);
      }
    }
  }
}

// I == 1, many rows of 1024 elements or more, 16-byte aligned: a wave per row, no LDS and no barrier.  A batch is
// 4 steps of 256 elements (4 consecutive ones per lane); the next batch is requested before the current one is
// worked on, so a wave always has 4 KiB on its way.  The running value crosses steps through a shuffle.
template <bool PROD>
__global__ __launch_bounds__(kThreads) void scan_wave_rows(ScanParams P) {
  constexpr int PER = 4, UNR = 4, STEP = kWave * PER, BATCH = STEP * UNR;
  const int lane = threadIdx.x % kWave;
  const thcl_u64 o = (thcl_u64)blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (o >= P.O) return;  // whole waves
  const float *row = P.in + o * P.R + (thcl_u64)lane * PER;
  float *orow = P.out + o * P.R + (thcl_u64)lane * PER;
  double carry = Op<PROD>::identity();
  auto fetch = [&](thcl_f4 (&x)[UNR], thcl_u64 base) {
#pragma unroll
    for (int u = 0; u < UNR; u++) x[u] = __builtin_nontemporal_load((const thcl_f4 *)(row + base + (thcl_u64)u * STEP));
  };
  // one step: 256 elements from `base`, this lane's four in x
  auto step = [&](const thcl_f4 &x, thcl_u64 base) {
    double a[PER];
    a[0] = (double)x[0];
#pragma unroll
    for (int c = 1; c < PER; c++) a[c] = Op<PROD>::comb(a[c - 1], (double)x[c]);
    const double incl = wave_inclusive<PROD>(a[PER - 1]);
    double before = carry;
    const double prev = __shfl_up(incl, 1, kWave);
    if (lane > 0) before = Op<PROD>::comb(before, prev);
    carry = Op<PROD>::comb(carry, __shfl(incl, kWave - 1, kWave));
    thcl_f4 v;
#pragma unroll
    for (int c = 0; c < PER; c++) v[c] = (float)Op<PROD>::comb(before, a[c]);
    return v;
  };
  thcl_u64 base = 0;
  if (BATCH <= P.R) {
    thcl_f4 x[UNR], xn[UNR];
    fetch(x, 0);
    for (; base + 2 * BATCH <= P.R; base += BATCH) {
      fetch(xn, base + BATCH);
#pragma unroll
      for (int u = 0; u < UNR; u++)
        __builtin_nontemporal_store(step(x[u], base + (thcl_u64)u * STEP), (thcl_f4 *)(orow + base + (thcl_u64)u * STEP));
#pragma unroll
      for (int u = 0; u < UNR; u++) x[u] = xn[u];
    }
#pragma unroll
    for (int u = 0; u < UNR; u++)
      __builtin_nontemporal_store(step(x[u], base + (thcl_u64)u * STEP), (thcl_f4 *)(orow + base + (thcl_u64)u * STEP));
    base += BATCH;
  }
  // what is left of the row (R is a multiple of 4: a lane's four elements are inside or outside together)
  const float fill = PROD ? 1.0f : 0.0f;
  for (; base < P.R; base += STEP) {
    const bool in = base + (thcl_u64)lane * PER < P.R;
    thcl_f4 x = {fill, fill, fill, fill};
    if (in) x = *(const thcl_f4 *)(row + base);
    const thcl_f4 v = step(x, base);
    if (in) *(thcl_f4 *)(orow + base) = v;
  }
}

// Long rows, too few to fill the chip with a block each, in one pass over memory (8 bytes an element where the three
// passes move 12): a launch whose blocks all run at the same time (two per CU) walks the rows in rounds.  Every row is
// cut into chunks of 8192 elements (its last one may be short), the chunks of all rows are numbered in memory order,
// and in round r block b owns chunk r * G + b, so a round is one run of G chunks.  A block keeps three chunks in
// registers: the one it scans, the next one, whose total it has already published, and the one after, on its way
// from memory.  What lies ahead of a chunk is its row's value at the start of the round (published by the last block
// of the round before, and used when the row began before this round) combined with the totals of the round's chunks
// in front of it in the same row; both were published a whole round
// earlier, so the block that needs them hardly ever waits, and no block waits for anything published later than its
// own position in the row: the waits cannot form a cycle.
// A total travels as one 8-byte word whose bit pattern is the double itself; all ones means "not there yet".  That
// pattern cannot be a total: it is a NaN whose low mantissa bits are set, and sums and products of values converted
// from float keep the 29 low bits of every NaN they meet at zero.  Stores and loads of the words are relaxed atomics
// at device scope (the value is its own flag, nothing else has to be ordered with it).
// Waits are bounded: after `spin_limit` polls a thread raises the fault word and goes on with what it has, so every
// wave leaves the kernel whatever happens, and the host reports the launch as failed at its next wait.
struct ChainParams {
  const float *in;
  float *out;
  thcl_u64 R;                    // elements of a row, a multiple of 4; both pointers 16-byte aligned
  thcl_u64 total;                // elements of all rows
  thcl_u32 cpr, nchunks;         // chunks per row (the last one may be short), chunks of all rows
  unsigned long long *totals;    // [rounds][G]
  unsigned long long *carries;   // [rounds + 1]
  thcl_u32 rounds;
  thcl_u32 spin_limit;
  thcl_u32 mute;                 // a block that publishes nothing (tests of the give-up path; no block otherwise)
  unsigned *fault;
};
constexpr unsigned long long kChainNotYet = ~0ull;
constexpr int kChainSteps = 2;                       // steps of 4096 elements per chunk
constexpr thcl_u64 kChainChunk = kChainSteps * 4096;
constexpr thcl_u64 kChainFrom = 1ull << 24;          // rows from this length up (2^24: 34.5 us against 36.8 for the three passes, 2^28: 400 against 504)

__global__ __launch_bounds__(kThreads) void scan_chain_init(unsigned long long *words, thcl_u64 count) {
  const thcl_u64 i = (thcl_u64)blockIdx.x * kThreads + threadIdx.x;
  if (i < count) words[i] = kChainNotYet;
}

template <bool PROD>
__global__ __launch_bounds__(kThreads) void scan_chain(ChainParams P) {
  constexpr int WAVES = kThreads / kWave, PER = 4, RUN = kThreads * PER, UNR = 4, STEP = RUN * UNR, SPC = kChainSteps;
  __shared__ double wave_tot[UNR][WAVES];
  __shared__ double fold[2][WAVES];
  const thcl_u32 G = gridDim.x, b = blockIdx.x;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const thcl_u64 last_group = P.total - PER;
  // chunk q of the whole tensor: where it starts, where its row ends, and which chunk is its row's first
  // (a chunk past the last one holds nothing and stands for a row of its own)
  auto place = [&](thcl_u64 q, thcl_u64 &base, thcl_u64 &lim) {
    if (q >= P.nchunks) {
      base = lim = P.total;
      return (thcl_u32)q;
    }
    const thcl_u32 row = (thcl_u32)q / P.cpr, cin = (thcl_u32)q - row * P.cpr;
    base = (thcl_u64)row * P.R + (thcl_u64)cin * kChainChunk;
    lim = (thcl_u64)row * P.R + P.R;
    return row * P.cpr;
  };
  bool gave_up = false;   // this thread has met a wait that did not end: it does not wait again
  auto await = [&](const unsigned long long *p) {
    unsigned long long bits = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    thcl_u32 spins = 0;
    while (bits == kChainNotYet && !gave_up) {
      if (++spins > P.spin_limit) {
        gave_up = true;
        *P.fault = 2u;
        break;
      }
      __builtin_amdgcn_s_sleep(2);
      bits = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return __builtin_bit_cast(double, bits);
  };
  auto publish = [&](unsigned long long *p, double v) {
    if (b == P.mute) return;
    __hip_atomic_store(p, __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // block-wide combination in a fixed order: lanes by butterfly, then the waves in order
  // (two values at a time: one pair of barriers serves a chunk's total and what lies ahead of another chunk)
  auto block_fold = [&](double &p, double &q) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
      p = Op<PROD>::comb(p, __shfl_xor(p, d, kWave));
      q = Op<PROD>::comb(q, __shfl_xor(q, d, kWave));
    }
    if (lane == 0) {
      fold[0][wave] = p;
      fold[1][wave] = q;
    }
    __syncthreads();
    p = fold[0][0];
    q = fold[1][0];
#pragma unroll
    for (int w = 1; w < WAVES; w++) {
      p = Op<PROD>::comb(p, fold[0][w]);
      q = Op<PROD>::comb(q, fold[1][w]);
    }
    __syncthreads();
  };
  typedef float Chunk[SPC][UNR][PER];
  // every load is issued: groups past the end of the row read its last group again and count as the identity below
  auto fetch = [&](Chunk &x, thcl_u64 chunk) {
    thcl_u64 base, lim;
    place(chunk, base, lim);
    base += (thcl_u64)threadIdx.x * PER;
#pragma unroll
    for (int st = 0; st < SPC; st++)
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const thcl_u64 j = base + (thcl_u64)st * STEP + (thcl_u64)u * RUN;
        const thcl_f4 v = __builtin_nontemporal_load((const thcl_f4 *)(P.in + (j < lim ? j : last_group)));
#pragma unroll
        for (int c = 0; c < PER; c++) x[st][u][c] = v[c];
      }
  };
  const float fill = PROD ? 1.0f : 0.0f;
  auto chunk_partial = [&](const Chunk &x, thcl_u64 chunk) {   // this thread's part of a chunk's total
    thcl_u64 base, lim;
    place(chunk, base, lim);
    base += (thcl_u64)threadIdx.x * PER;
    double t = Op<PROD>::identity();
#pragma unroll
    for (int st = 0; st < SPC; st++)
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const bool in = base + (thcl_u64)st * STEP + (thcl_u64)u * RUN < lim;
#pragma unroll
        for (int c = 0; c < PER; c++) t = Op<PROD>::comb(t, (double)(in ? x[st][u][c] : fill));
      }
    return t;
  };
  // the scan of one chunk from its registers, `carry` being everything ahead of it (as in scan_row)
  auto scan_chunk = [&](const Chunk &x, thcl_u64 chunk, double carry) {
    thcl_u64 first, lim;
    place(chunk, first, lim);
#pragma unroll
    for (int st = 0; st < SPC; st++) {
      const thcl_u64 base = first + (thcl_u64)st * STEP;
      double a[UNR][PER], incl[UNR];
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const bool in = base + (thcl_u64)u * RUN + (thcl_u64)threadIdx.x * PER < lim;
        a[u][0] = (double)(in ? x[st][u][0] : fill);
#pragma unroll
        for (int c = 1; c < PER; c++) a[u][c] = Op<PROD>::comb(a[u][c - 1], (double)(in ? x[st][u][c] : fill));
        incl[u] = wave_inclusive<PROD>(a[u][PER - 1]);
      }
      __syncthreads();  // wave_tot of the previous step has been read
      if (lane == kWave - 1) {
#pragma unroll
        for (int u = 0; u < UNR; u++) wave_tot[u][wave] = incl[u];
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        double before = carry;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
          if (w < wave) before = Op<PROD>::comb(before, wave_tot[u][w]);
          carry = Op<PROD>::comb(carry, wave_tot[u][w]);
        }
        const double prev = __shfl_up(incl[u], 1, kWave);
        if (lane > 0) before = Op<PROD>::comb(before, prev);
        const thcl_u64 j = base + (thcl_u64)u * RUN + (thcl_u64)threadIdx.x * PER;
        if (j < lim) {
          thcl_f4 v;
#pragma unroll
          for (int c = 0; c < PER; c++) v[c] = (float)Op<PROD>::comb(before, a[u][c]);
          __builtin_nontemporal_store(v, (thcl_f4 *)(P.out + j));
        }
      }
    }
  };
  double tot_cur;   // this block's total of the chunk it scans next
  auto peek = [&](const unsigned long long *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
  auto round = [&](Chunk &cur, Chunk &next, Chunk &far, thcl_u32 r) {
    // what lies ahead of this round's chunk was published a round ago: its words are requested first, so that their
    // trip through memory runs beside the work on the next chunk's total, and they are looked at after it
    // (of this chunk's own row only: the round's chunks from the row's first one on, and the value at the start of
    // the round when the row began before it)
    thcl_u64 unused0, unused1;
    const thcl_u64 round_first = (thcl_u64)r * G;
    const thcl_u32 row_first = place(round_first + b, unused0, unused1);
    const thcl_u32 k_lo = row_first > round_first ? (thcl_u32)(row_first - round_first) : 0u;
    const bool began_before = r > 0 && row_first < round_first;
    const thcl_u32 k0 = threadIdx.x, k1 = threadIdx.x + kThreads;
    const bool take0 = k0 >= k_lo && k0 < b, take1 = k1 >= k_lo && k1 < b, takec = threadIdx.x == 0 && began_before;
    const unsigned long long *row = P.totals + round_first;
    unsigned long long w0 = 0, w1 = 0, wc = 0;
    if (take0) w0 = peek(row + k0);
    if (take1) w1 = peek(row + k1);
    if (takec) wc = peek(P.carries + r);
    fetch(far, (thcl_u64)(r + 2) * G + b);
    __builtin_amdgcn_sched_barrier(0);
    double tot_next = chunk_partial(next, (thcl_u64)(r + 1) * G + b);
    double mine = Op<PROD>::identity();
    if (takec) mine = wc != kChainNotYet ? __builtin_bit_cast(double, wc) : await(P.carries + r);
    if (take0) mine = Op<PROD>::comb(mine, w0 != kChainNotYet ? __builtin_bit_cast(double, w0) : await(row + k0));
    if (take1) mine = Op<PROD>::comb(mine, w1 != kChainNotYet ? __builtin_bit_cast(double, w1) : await(row + k1));
    block_fold(tot_next, mine);
    const double ahead = mine;
    if (threadIdx.x == 0 && r + 1 < P.rounds) publish(P.totals + (thcl_u64)(r + 1) * G + b, tot_next);
    if (b == G - 1 && threadIdx.x == 0) publish(P.carries + r + 1, Op<PROD>::comb(ahead, tot_cur));
    scan_chunk(cur, (thcl_u64)r * G + b, ahead);
    tot_cur = tot_next;
  };
  Chunk xa, xb, xc;
  fetch(xa, b);
  fetch(xb, (thcl_u64)G + b);
  {
    double none = Op<PROD>::identity();
    tot_cur = chunk_partial(xa, b);
    block_fold(tot_cur, none);
  }
  if (threadIdx.x == 0) publish(P.totals + b, tot_cur);
  for (thcl_u32 r = 0;;) {
    round(xa, xb, xc, r);
    if (++r >= P.rounds) break;
    round(xb, xc, xa, r);
    if (++r >= P.rounds) break;
    round(xc, xa, xb, r);
    if (++r >= P.rounds) break;
  }
}

template <bool PROD, int G>
void launch_short(hipStream_t stream, const ScanParams &P, bool vec) {
  const dim3 grid((unsigned)((P.O + kThreads / G - 1) / (kThreads / G))), block(kThreads);
  if (vec) hipLaunchKernelGGL((scan_short_rows<PROD, G, true>), grid, block, 0, stream, P);
  else hipLaunchKernelGGL((scan_short_rows<PROD, G, false>), grid, block, 0, stream, P);
}

template <bool PROD>
void run_short(hipStream_t stream, const ScanParams &P, bool vec) {
  // lanes per row: enough to cover the row in one step, at most a wave
  int g = 1;
  while (g < kWave && (thcl_u64)g * 4 < P.R) g <<= 1;
  switch (g) {
    case 1: launch_short<PROD, 1>(stream, P, vec); break;
    case 2: launch_short<PROD, 2>(stream, P, vec); break;
    case 4: launch_short<PROD, 4>(stream, P, vec); break;
    case 8: launch_short<PROD, 8>(stream, P, vec); break;
    case 16: launch_short<PROD, 16>(stream, P, vec); break;
    case 32: launch_short<PROD, 32>(stream, P, vec); break;
    default: launch_short<PROD, 64>(stream, P, vec); break;
  }
}

void check(const char *what) {
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "%s launch failed: %s", what, hipGetErrorString(e));
}

template <bool PROD>
void launch_carries(hipStream_t stream, const ScanParams &P) {
  const thcl_u64 lines = P.O * P.I;
  if (lines < 4096 && P.S >= 32)
    hipLaunchKernelGGL((scan_carries_wave<PROD>), dim3((unsigned)lines), dim3(kWave), 0, stream, P);
  else
    hipLaunchKernelGGL((scan_carries<PROD>), dim3((unsigned)((lines + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, P);
  check("scan carries");
}

// The single-pass scan of rows that are too few to fill the chip with a block each.  The grid is what the chip holds at one time (the
// occupancy the runtime reports for the kernel, at most two blocks per CU); the launches of a context run in order on
// its one stream, so nothing of the library's competes for the CUs, and should another client of the GPU keep blocks
// from starting, the kernel's bounded waits end the launch with an error report instead of a result.
// False: not started (the kernel does not fit a CU), and the caller takes the three passes.
template <bool PROD>
bool run_chain(thcl_rt *rt, hipStream_t stream, const ScanParams &S) {
  static int per_cu = -1;   // blocks of scan_chain a CU holds at a time, at most 2
  static thcl_u32 spin_limit = 1u << 23, mute = ~0u;   // some seconds of polling before a wait gives up
  if (per_cu < 0) {
    int nb = 0, nbp = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, scan_chain<false>, kThreads, 0) != hipSuccess) nb = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nbp, scan_chain<true>, kThreads, 0) != hipSuccess) nbp = 0;
    if (nbp < nb) nb = nbp;
    (void)hipGetLastError();
    per_cu = nb > 2 ? 2 : nb;
    // for tests of the give-up path: how often a wait polls before it gives up, and a block that publishes nothing
    if (const char *e = getenv("THCL_SCAN_CHAIN_SPINS")) spin_limit = (thcl_u32)strtoul(e, nullptr, 10);
    if (const char *e = getenv("THCL_SCAN_CHAIN_MUTE")) mute = (thcl_u32)strtoul(e, nullptr, 10);
  }
  if (per_cu <= 0) return false;
  const thcl_u32 G = (thcl_u32)(thcl_rt_get_props(rt)->compute_units * per_cu);
  const thcl_u64 cpr = (S.R + kChainChunk - 1) / kChainChunk;
  if (cpr * S.O >= (1ull << 31)) return false;
  ChainParams C;
  C.in = S.in;
  C.out = S.out;
  C.R = S.R;
  C.total = S.O * S.R;
  C.cpr = (thcl_u32)cpr;
  C.nchunks = (thcl_u32)(cpr * S.O);
  C.rounds = (C.nchunks + G - 1) / G;
  C.spin_limit = spin_limit;
  C.mute = mute;
  C.fault = thcl_rt_fault_word_device(rt);
  const thcl_u64 words = (thcl_u64)C.rounds * G + C.rounds + 1;
  C.totals = (unsigned long long *)thcl_rt_workspace(rt, (size_t)words * sizeof(unsigned long long));
  THCL_CHECK(C.totals != nullptr, "%s", thcl_rt_error());
  C.carries = C.totals + (thcl_u64)C.rounds * G;
  hipLaunchKernelGGL(scan_chain_init, dim3((unsigned)((words + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, C.totals, words);
  hipLaunchKernelGGL(scan_chain<PROD>, dim3(G), dim3(kThreads), 0, stream, C);
  check("scan");
  return true;
}

template <bool PROD>
void run_scan(hipStream_t stream, ScanParams &P, bool rows, bool vec) {
  if (rows) {
    const dim3 block(kThreads);
    const thcl_u64 blocks = P.O * P.S;
    if (P.S > 1) {
      // Cut rows are read twice (totals, then the scan with each segment's carry-in).  The input goes through
      // in windows of 256 MiB, totals pass and scan pass back to back per window, so the second read comes out of
      // the memory-side cache instead of HBM (measured on plain kernels: a 128 MiB window re-read and copied in
      // 35 us after an ordinary read of it, 50 us cold; nothing gained after a nontemporal read).  2^28 elements:
      // 570 us in three chip-wide passes, 498 us this way.  A segment's carry-in is folded from the totals by
      // its own block, which saves a launch per window.
      thcl_u64 per_window = (kScanWindowBytes / sizeof(float) + P.seg - 1) / P.seg;
      if (per_window < 1) per_window = 1;
      P.own_carry = 1;
      double *ahead = P.totals + blocks;   // one slot per window, after the totals
      thcl_u64 w = 0;
      for (thcl_u64 b0 = 0; b0 < blocks; b0 += per_window, w++) {
        const thcl_u64 nb = blocks - b0 < per_window ? blocks - b0 : per_window;
        const dim3 grid((unsigned)nb);
        P.block0 = b0;
        P.ahead_in = ahead + w;       // written by the previous window's last block (its own slot 0 is never read)
        P.ahead_out = ahead + w + 1;
        if (vec) hipLaunchKernelGGL((scan_row<PROD, 0, true>), grid, block, 0, stream, P);
        else hipLaunchKernelGGL((scan_row<PROD, 0, false>), grid, block, 0, stream, P);
        if (vec) hipLaunchKernelGGL((scan_row<PROD, 1, true>), grid, block, 0, stream, P);
        else hipLaunchKernelGGL((scan_row<PROD, 1, false>), grid, block, 0, stream, P);
      }
      check("scan");
    } else {
      const dim3 grid((unsigned)blocks);
      if (vec) hipLaunchKernelGGL((scan_row<PROD, 1, true>), grid, block, 0, stream, P);
      else hipLaunchKernelGGL((scan_row<PROD, 1, false>), grid, block, 0, stream, P);
      check("scan");
    }
  } else {
    const thcl_u64 threads = P.O * P.S * P.I;
    const dim3 grid((unsigned)((threads + kThreads - 1) / kThreads)), block(kThreads);
    if (P.S > 1) {
      hipLaunchKernelGGL((scan_seq<PROD, 0>), grid, block, 0, stream, P);
      check("scan totals");
      launch_carries<PROD>(stream, P);
    }
    hipLaunchKernelGGL((scan_seq<PROD, 1>), grid, block, 0, stream, P);
    check("scan");
  }
}
}  // namespace

// self = inclusive scan of src along `dim` (0-based).  Operands that are not
// dense go through dense stand-ins, as in the reference
// (src/lib/THClTensorMathScan.cpp:127-142).
void thcl_scan_dim(THClState *state, bool prod, THClTensor *self, THClTensor *src, long dim) {
  thcl_check_same_device(state, 2, self, src);
  THCL_ARGCHECK(src->nDimension > 0, 2, "cannot scan an empty tensor");
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 3, "dimension out of range");
  if (src->size[dim] == 1) {  // every line has one element: the scan is the source itself
    if (self != src) {
      THClTensor_resizeAs(state, self, src);
      THClTensor_copy(state, self, src);
    }
    return;
  }
  ThclTemp src_hold(state, THClTensor_newContiguous(state, src));  // before resizing self: they may be the same tensor
  THClTensor *srcc = src_hold.t;
  THClTensor_resizeAs(state, self, src);
  ThclTemp self_hold(state, nullptr);
  THClTensor *selfc = self;
  if (!THClTensor_isContiguous(state, self)) {
    self_hold.t = selfc = THClTensor_newv2(state, THClTensor_getDevice(state, self));
    THClTensor_resizeAs(state, selfc, self);
  }
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, src));
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);

  ScanParams P;
  memset(&P, 0, sizeof(P));
  P.in = thcl_dptr(srcc);
  P.out = thcl_dptr(selfc);
  P.O = P.I = 1;
  for (int d = 0; d < dim; d++) P.O *= (thcl_u64)src->size[d];
  for (int d = (int)dim + 1; d < src->nDimension; d++) P.I *= (thcl_u64)src->size[d];
  P.R = (thcl_u64)src->size[dim];
  const thcl_u64 total = P.O * P.R * P.I;
  if (total > 0) {
    const long cus = thcl_rt_get_props(rt)->compute_units;
    // innermost scans: long rows (or few of them) take a block per row segment,
    // many short rows take a lane group per row
    const bool aligned = ((((uintptr_t)P.in) | ((uintptr_t)P.out)) & 15u) == 0;
    // enough aligned rows of 1024 to 8191 elements for a wave each (16 per CU).  Measured against the lane-group kernel
    // without prefetch: 65536 x 1024 85 -> 82 us, 4096 x 4100 34 -> 27 us; on longer rows a block per row wins
    // (4096 x 16384: 95 us against 105).
    const bool waverows = P.I == 1 && P.R >= 1024 && P.R < 8192 && P.R % 4 == 0 && aligned && P.O >= (thcl_u64)cus * 16;
    const bool shortrows = !waverows && P.I == 1 && P.R > 1 && (P.R < 1024 || (P.R < 8192 && P.O >= (thcl_u64)cus * 16));
    const bool rows = (P.I == 1 && P.R >= 1024) && !shortrows && !waverows;
    // cut R into segments until the launch fills the chip; a segment keeps
    // enough elements to amortise the extra pass
    // Outer scans with too few columns for a thread each: strips of 32 columns in one pass, when there
    // is a strip for every other CU and the lines are long enough to amortise a block's start.  On 256
    // CUs, 2^26 elements: 16384 columns 4.9 TB/s against 3.7 in three passes, 8192 columns 5.2,
    // 4096 columns (128 strips) 4.2 against 3.8, 2048 columns 2.5 against 3.7.
    const bool few_lines = !rows && !shortrows && !waverows && P.I % 4 == 0 && aligned && P.O * P.I < (thcl_u64)cus * 512;
    thcl_u64 strips = P.O * ((P.I / 4 + 7) / 8);
    bool strip = few_lines && P.R >= 1024 && strips * 2 >= (thcl_u64)cus && strips < (1ull << 31);
    // A handful of columns (4 to 28): the thread-per-column kernel would read 16 to 112 bytes per row
    // and line segment.  Strips as wide as the tensor read whole runs of rows instead; the lines are
    // cut into segments (three passes) to fill the chip.  2^26 elements in rows of 4 / 8 / 16 columns:
    // 0.8 -> 2.0, 1.7 -> 2.1, 2.5 -> 3.0 TB/s.
    // Widths that are no multiple of 4, or rows that are not 16-byte aligned, take the same strips one element
    // at a time (2^20 x 3: 106 us with a thread per column, 30 us this way; 2^18 x 27: 37 us).
    int strip_tc = 8;
    // strips of 64 columns (runs of 256 bytes) when those still give every CU a block: 4096 x 16384 104 -> 98 us,
    // 2048 x 32768 118 -> 99 us
    // (unless they leave the CUs unevenly loaded where the narrower strips do not: 4096 x 20480 is 320 strips of 64
    // columns, two rounds of blocks on 256 CUs for 1.25 rounds of work, 157 us against 146 in 640 strips of 32)
    if (strip && P.O * ((P.I / 4 + 15) / 16) >= (thcl_u64)cus) {
      const thcl_u64 wide = P.O * ((P.I / 4 + 15) / 16);
      auto balance = [&](thcl_u64 blocks) { return (double)blocks / (double)((blocks + cus - 1) / cus * cus); };
      if (balance(wide) * 1.08 >= balance(strips)) {
        strip_tc = 16;
        strips = wide;
      }
    }
    bool narrow = false, narrow_any = false;
    // (from 1.5 million elements per tensor slice up: below that the three launches of the strips cost more than the
    // thread-per-column walk, 20000 x 8: 42 us against 10)
    const bool few_narrow = !rows && !shortrows && !waverows && P.I > 1 && P.I <= 28 && P.R >= 16384 && P.R * P.I >= (3ull << 19) &&
                            P.O * P.I < (thcl_u64)cus * 512;
    if (!strip && few_narrow) {
      const thcl_u64 quads = (P.I + 3) / 4;
      strip_tc = quads <= 1 ? 1 : (quads <= 2 ? 2 : (quads <= 4 ? 4 : 8));
      strips = P.O;
      strip = narrow = true;
      narrow_any = !(P.I % 4 == 0 && aligned);
    }
    thcl_u64 S = 1;
    if (narrow) {
      const thcl_u64 want = (thcl_u64)cus * 8;  // blocks
      if (P.O < want) S = (want + P.O - 1) / P.O;
      // a few steps of the block at least (a step of the element-wise strips is 2 rows per thread)
      const thcl_u64 most = narrow_any ? P.R / (thcl_u64)(kThreads / strip_tc * 2 * 8) : P.R / 4096;
      if (S > most) S = most;
    } else if (shortrows || waverows || strip) {
      S = 1;
    } else if (rows) {
      // Segments cost a second read of the input (12 bytes an element instead of 8), which pays
      // only while the rows alone leave most of the chip idle: 1024 rows of 65536 elements run at
      // 5.3 TB/s in one pass on 256 CUs and at 3.5 TB/s in two segments each.
      const thcl_u64 want = (thcl_u64)cus * 8;  // blocks
      if (P.O < (thcl_u64)cus * 3) S = (want + P.O - 1) / P.O;
      const thcl_u64 most = P.R / 4096;
      if (S > most) S = most;
    } else {
      const thcl_u64 want = (thcl_u64)cus * 512;  // threads
      if (P.O * P.I < want) S = (want + P.O * P.I - 1) / (P.O * P.I);
      const thcl_u64 most = P.R / 32;
      if (S > most) S = most;
    }
    if (S < 1) S = 1;
    thcl_u64 seg = (P.R + S - 1) / S;
    if (rows) seg = (seg + 4095) / 4096 * 4096;  // whole steps, so vector accesses stay aligned
    // Cut rows take segments of 8192 elements (two steps of a block) when that still leaves several blocks per CU:
    // measured best for the windowed passes (2^28 elements: 8192 -> 497 us, 16384 -> 514, 32768 -> 520, 4096 -> 605),
    // whatever the window.
    if (rows && S > 1 && seg > (thcl_u64)kScanSegment && total >= (thcl_u64)cus * 8 * kScanSegment) {
      seg = (thcl_u64)kScanSegment;
    }
    S = (P.R + seg - 1) / seg;
    P.S = S;
    P.seg = seg;
    THCL_CHECK(P.O * P.S < (1ull << 31) && (P.O * P.S * P.I + kThreads - 1) / kThreads < (1ull << 31), THCL_DIM_WARNING);
    // one hand-over slot per window and one more (run_scan walks the same windows)
    const thcl_u64 per_window = (kScanWindowBytes / sizeof(float) + seg - 1) / seg;
    const thcl_u64 windows = rows && S > 1 ? (P.O * S + per_window - 1) / per_window + 1 : 0;
    if (S > 1) P.totals = (double *)thcl_rt_workspace(rt, (size_t)(P.O * P.S * P.I + windows) * sizeof(double));
    THCL_CHECK(S == 1 || P.totals != nullptr, "%s", thcl_rt_error());
    const bool vec = (rows || shortrows) && (P.R % 4 == 0) && aligned;
    if (waverows) {
      const thcl_u64 blocks = (P.O + kThreads / kWave - 1) / (kThreads / kWave);
      THCL_CHECK(blocks < (1ull << 31), THCL_DIM_WARNING);
      if (prod) hipLaunchKernelGGL(scan_wave_rows<true>, dim3((unsigned)blocks), dim3(kThreads), 0, stream, P);
      else hipLaunchKernelGGL(scan_wave_rows<false>, dim3((unsigned)blocks), dim3(kThreads), 0, stream, P);
      check("scan");
    } else if (shortrows) {
      THCL_CHECK(P.O < (1ull << 31), THCL_DIM_WARNING);
      if (prod) run_short<true>(stream, P, vec);
      else run_short<false>(stream, P, vec);
      check("scan");
    } else if (strip) {
      const dim3 grid((unsigned)(strips * P.S)), block(kThreads);
      // one block on (nearly) every CU and two on none: four rows a thread instead of eight (with 1.125 to 1.375
      // blocks per CU the CUs that hold two set the time and prefer eight rows: 4096 x 10240 84 us against 89)
      const bool strip_half = !narrow && strip_tc >= 8 && strips * P.S * 5 >= (thcl_u64)cus * 4 && strips * P.S <= (thcl_u64)cus;
#define STRIP_CASE(PR, TC_, PH)                                                                               \
  if (narrow_any) hipLaunchKernelGGL((scan_strip<PR, TC_, PH, true>), grid, block, 0, stream, P);              \
  else if (strip_half && TC_ >= 8) hipLaunchKernelGGL((scan_strip<PR, (TC_ >= 8 ? TC_ : 8), PH, false, true>), grid, block, 0, stream, P); \
  else hipLaunchKernelGGL((scan_strip<PR, TC_, PH, false>), grid, block, 0, stream, P);
#define STRIP_PHASE(PH)                                                                                        \
  switch (strip_tc * 2 + (prod ? 1 : 0)) {                                                                     \
    case 2: STRIP_CASE(false, 1, PH) break;                                                                    \
    case 3: STRIP_CASE(true, 1, PH) break;                                                                     \
    case 4: STRIP_CASE(false, 2, PH) break;                                                                    \
    case 5: STRIP_CASE(true, 2, PH) break;                                                                     \
    case 8: STRIP_CASE(false, 4, PH) break;                                                                    \
    case 9: STRIP_CASE(true, 4, PH) break;                                                                     \
    case 16: STRIP_CASE(false, 8, PH) break;                                                                   \
    case 17: STRIP_CASE(true, 8, PH) break;                                                                    \
    case 32: STRIP_CASE(false, 16, PH) break;                                                                  \
    default: STRIP_CASE(true, 16, PH) break;                                                                   \
  }
      if (P.S > 1) {
        STRIP_PHASE(0)
        check("scan totals");
        if (prod) launch_carries<true>(stream, P);
        else launch_carries<false>(stream, P);
      }
      STRIP_PHASE(1)
#undef STRIP_PHASE
#undef STRIP_CASE
      check("scan");
    } else if (rows && vec && P.S > 1 && total >= kChainFrom && (prod ? run_chain<true>(rt, stream, P) : run_chain<false>(rt, stream, P))) {
      // rows too few to fill the chip, 2^24 elements and more: a single pass
    } else if (prod) {
      run_scan<true>(stream, P, rows, vec);
    } else {
      run_scan<false>(stream, P, rows, vec);
    }
    thcl_after_launch(state, rt);
  }
  if (selfc != self) self_hold.give_to(self);
}

extern "C" {
// (src/lib/THClTensorMathScan.cpp:144-156)
void THClTensor_cumsum(THClState *state, THClTensor *self, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  thcl_scan_dim(state, false, self, src, dim);
  THCL_GUARD_END()
}
void THClTensor_cumprod(THClState *state, THClTensor *self, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  thcl_scan_dim(state, true, self, src, dim);
  THCL_GUARD_END()
}
}
