// Level-1 / level-2 contractions: dot, matrix-vector (addmv), rank-1 update (addr).
//
// What it replaces (reference): THClTensor_dot / addmv / addr
// (src/lib/THClTensorMathBlas.cpp:17-105,216-277) and the clBLAS calls behind
// THClBlas_dot / gemv / ger (src/lib/THClBlas.cpp:149-347).
//
// All three are bound by HBM: gemv reads the matrix once (4 bytes per 2
// flops), so the kernels are streaming reductions, with fp64 accumulators
// like the other sums of this library.  The rank-1 update is a pointwise
// operator over the matrix: a dedicated kernel when the matrix has unit stride
// along one dim, otherwise the apply engine with the vectors as stride-0 views.
#include <hip/hip_runtime.h>

#include <cstring>

#include "apply_device.h"
#include "internal.h"

namespace {

// a 16-byte read that only needs the alignment of its elements (columns of a view start anywhere)
typedef thcl_f4 rd_f4 __attribute__((aligned(4)));


constexpr int kThreads = 256;
constexpr int kWave = 64;

// Column-major A (m x n, leading dimension lda), BLAS meaning of the rest.
struct GemvParams {
  const float *a;
  const float *x;
  float *y;
  double *partials;  // [split][outputs] when the contraction is split over blocks
  thcl_u32 m, n;
  thcl_u64 lda;
  long incx, incy;
  float alpha, beta;
  thcl_u32 split, per_split;  // blocks sharing one output's contraction, and the length each takes
  thcl_u32 outputs;           // n for 't', m for 'n'
  thcl_u32 ub_log2;           // 'n' kernel: a wave spans 2^ub_log2 units of outputs and 64 >> ub_log2 columns
};

__device__ __forceinline__ void store_result(const GemvParams &P, thcl_u32 i, double acc) {
  float *yp = P.y + (long)i * P.incy;
  const float scaled = (float)((double)P.alpha * acc);
  *yp = (P.beta == 0.f) ? scaled : P.beta * *yp + scaled;  // beta == 0: y is not read (BLAS rule)
}

// trans = 't': y[j] = alpha * dot(A[:, j], x) + beta * y[j].  Column j is m
// contiguous floats; LPR lanes walk it (1, 8, 64 or a whole block).  blockIdx.y cuts
// long columns into pieces of per_split elements (a multiple of 4) that leave partials.
// VEC 0: one element at a time (incx != 1); 1: units of four, m a multiple of 4; 2: units of four and the last m % 4
template <int LPR, int VEC>
__global__ __launch_bounds__(kThreads) void gemv_t(GemvParams P) {
  constexpr int COLS = kThreads / LPR;
  __shared__ double lds[kThreads / kWave];
  const int sub = threadIdx.x % LPR;
  const thcl_u32 j = blockIdx.x * COLS + threadIdx.x / LPR;
  const thcl_u32 i0 = blockIdx.y * P.per_split;
  const thcl_u32 len = (P.m - i0 < P.per_split) ? (P.m - i0) : P.per_split;
  double acc = 0.0;
  if (j < P.n) {
    const float *col = P.a + (thcl_u64)j * P.lda + i0;
    if (VEC) {  // incx == 1
      const rd_f4 *c4 = (const rd_f4 *)col, *x4 = (const rd_f4 *)(P.x + i0);
      const thcl_u32 m4 = len >> 2;
      constexpr int FLY = 4;
      thcl_u32 i = sub;
      // groups of FLY loads; the next group is requested before the current one is used
      auto fetch = [&](thcl_f4 (&v)[FLY], thcl_f4 (&w)[FLY], thcl_u32 at) {
#pragma unroll
        for (int f = 0; f < FLY; f++) {
          v[f] = __builtin_nontemporal_load(c4 + at + f * LPR);
          w[f] = x4[at + f * LPR];
        }
      };
      auto use = [&](const thcl_f4 (&v)[FLY], const thcl_f4 (&w)[FLY]) {
#pragma unroll
        for (int f = 0; f < FLY; f++)
#pragma unroll
          for (int c = 0; c < 4; c++) acc += (double)v[f][c] * (double)w[f][c];
      };
      if (i + (FLY - 1) * LPR < m4) {
        thcl_f4 v[FLY], w[FLY], vn[FLY], wn[FLY];
        fetch(v, w, i);
        for (; i + (2 * FLY - 1) * LPR < m4; i += FLY * LPR) {
          fetch(vn, wn, i + FLY * LPR);
          use(v, w);
#pragma unroll
          for (int f = 0; f < FLY; f++) {
            v[f] = vn[f];
            w[f] = wn[f];
          }
        }
        use(v, w);
        i += FLY * LPR;
      }
      for (; i < m4; i += LPR) {
        const thcl_f4 v = c4[i], w = x4[i];
#pragma unroll
        for (int c = 0; c < 4; c++) acc += (double)v[c] * (double)w[c];
      }
      if (VEC == 2)
        for (thcl_u32 e = (m4 << 2) + sub; e < len; e += LPR) acc += (double)col[e] * (double)P.x[i0 + e];   // the last len % 4
    } else {
      for (thcl_u32 i = sub; i < len; i += LPR) acc += (double)col[i] * (double)P.x[(long)(i0 + i) * P.incx];
    }
  }
  // fold the LPR lanes of a column
#pragma unroll
  for (int d = (LPR < kWave ? LPR : kWave) >> 1; d > 0; d >>= 1) acc += __shfl_xor(acc, d, kWave);
  if (LPR <= kWave) {
    if (sub == 0 && j < P.n) {
      if (P.split > 1) P.partials[(thcl_u64)blockIdx.y * P.n + j] = acc;
      else store_result(P, j, acc);
    }
  } else {
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) lds[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0 && j < P.n) {
      double r = lds[0];
      for (int w = 1; w < kThreads / kWave; w++) r += lds[w];
      if (P.split > 1) P.partials[(thcl_u64)blockIdx.y * P.n + j] = r;
      else store_result(P, j, r);
    }
  }
}

// trans = 'n': y[i] = alpha * sum_j A[i + j*lda] * x[j] + beta * y[i].  Lanes lie
// along i (VEC rows each; with fewer than 64 units of rows the wave's other lanes take
// further columns), the 4 waves of a block interleave over j and meet in
// LDS; blockIdx.y splits long contractions, leaving partials for gemv_finish.
template <int VEC>
__global__ __launch_bounds__(kThreads) void gemv_n(GemvParams P) {
  constexpr int WAVES = kThreads / kWave;
  __shared__ double lds[WAVES][kWave * VEC];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const thcl_u32 UB = 1u << P.ub_log2, RL = kWave >> P.ub_log2;
  const thcl_u32 ul = lane & (UB - 1), rl = lane >> P.ub_log2;
  const thcl_u32 JSTEP = WAVES * RL;  // columns between a lane's consecutive elements
  const thcl_u32 units = (P.m + VEC - 1) / VEC;
  const thcl_u32 u = blockIdx.x * UB + ul;
  const thcl_u32 j0 = blockIdx.y * P.per_split;
  thcl_u32 j1 = j0 + P.per_split;
  if (j1 > P.n) j1 = P.n;
  // m no multiple of VEC: the last unit is moved back to end with the column; it computes some rows a second time and
  // stores only its own
  const thcl_u32 row0 = (VEC > 1 && u * VEC + VEC > P.m) ? P.m - VEC : u * VEC;
  double acc[VEC];
#pragma unroll
  for (int c = 0; c < VEC; c++) acc[c] = 0.0;
  if (u < units) {
    constexpr int FLY = 4;
    thcl_u32 j = j0 + wave * RL + rl;
    const float *ptr = P.a + (thcl_u64)j * P.lda + (thcl_u64)row0;
    const thcl_u64 step = (thcl_u64)JSTEP * P.lda;
    for (; j + (FLY - 1) * JSTEP < j1; j += FLY * JSTEP) {
      float xs[FLY];
      if (VEC == 4) {
        thcl_f4 v[FLY];
#pragma unroll
        for (int f = 0; f < FLY; f++) {
          v[f] = __builtin_nontemporal_load((const rd_f4 *)ptr);
          xs[f] = P.x[(long)(j + f * JSTEP) * P.incx];
          ptr += step;
        }
#pragma unroll
        for (int f = 0; f < FLY; f++)
#pragma unroll
          for (int c = 0; c < 4; c++) acc[c] += (double)v[f][c] * (double)xs[f];
      } else {
        float v[FLY];
#pragma unroll
        for (int f = 0; f < FLY; f++) {
          v[f] = *ptr;
          xs[f] = P.x[(long)(j + f * JSTEP) * P.incx];
          ptr += step;
        }
#pragma unroll
        for (int f = 0; f < FLY; f++) acc[0] += (double)v[f] * (double)xs[f];
      }
    }
    for (; j < j1; j += JSTEP) {
      const double xj = (double)P.x[(long)j * P.incx];
      if (VEC == 4) {
        const thcl_f4 v = *(const rd_f4 *)ptr;
#pragma unroll
        for (int c = 0; c < 4; c++) acc[c] += (double)v[c] * xj;
      } else {
        acc[0] += (double)*ptr * xj;
      }
      ptr += step;
    }
  }
  // the wave's column lanes of one unit meet first (lanes UB apart)
  for (thcl_u32 d = UB; d < (thcl_u32)kWave; d <<= 1) {
#pragma unroll
    for (int c = 0; c < VEC; c++) acc[c] += __shfl_xor(acc[c], (int)d, kWave);
  }
  if (rl == 0) {
#pragma unroll
    for (int c = 0; c < VEC; c++) lds[wave][ul * VEC + c] = acc[c];
  }
  __syncthreads();
  if (wave == 0 && rl == 0 && u < units) {
#pragma unroll
    for (int c = 0; c < VEC; c++) {
      double r = lds[0][ul * VEC + c];
      for (int w = 1; w < WAVES; w++) r += lds[w][ul * VEC + c];
      const thcl_u32 i = row0 + c;
      if (i >= u * VEC) {
        if (P.split > 1) P.partials[(thcl_u64)blockIdx.y * P.m + i] = r;
        else store_result(P, i, r);
      }
    }
  }
}

// folds the [split][outputs] partials in split order
__global__ __launch_bounds__(kThreads) void gemv_finish(GemvParams P) {
  const thcl_u32 i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= P.outputs) return;
  double r = 0.0;
  for (thcl_u32 k = 0; k < P.split; k++) r += P.partials[(thcl_u64)k * P.outputs + i];
  store_result(P, i, r);
}

void check(const char *what) {
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "%s launch failed: %s", what, hipGetErrorString(e));
}
bool aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }

// 1-d vector as an (rows x cols) view that repeats it along the other dim
// Rank-1 update of a matrix whose lines are contiguous: a[l][c] = beta * a[l][c] + alpha * u[l] * v[c]
// with c along the contiguous dim.  A thread owns 4 adjacent columns (one 16-byte access) and 2 lines,
// both reads in flight together (16384^2: 337 us with 8 lines a thread, 328 with 4, 321 with 2, 372 with 1).  UFIRST: the product is
// (alpha * u[l]) * v[c], otherwise (alpha * v[c]) * u[l] -- the association of the operator string
// the generic path would compile, so both paths give the same bits.
constexpr int kRank1Lines = 2;
struct Rank1Params {
  float *a;
  const float *u, *v;
  thcl_u64 lines, cols, pitch;
  unsigned gx;   // blocks along the columns; the grid is one-dimensional, columns fastest
  long incu, incv;
  float beta, alpha;
};
template <bool UFIRST>
__global__ __launch_bounds__(kThreads) void rank1_update(Rank1Params P) {
  constexpr int LINES = kRank1Lines, LANES = 64, GROUPS = kThreads / LANES;
  const unsigned by = blockIdx.x / P.gx, bx = blockIdx.x - by * P.gx;
  const thcl_u64 c = ((thcl_u64)bx * LANES + threadIdx.x % LANES) * 4;
  const thcl_u64 l0 = (thcl_u64)by * (GROUPS * LINES) + threadIdx.x / LANES;
  if (c >= P.cols) return;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; e++) v[e] = P.v[(long)(c + e) * P.incv];
  thcl_f4 a[LINES];
  float u[LINES];
#pragma unroll
  for (int k = 0; k < LINES; k++) {
    thcl_u64 l = l0 + (thcl_u64)k * GROUPS;
    if (l >= P.lines) l = P.lines - 1;  // read again, not stored
    a[k] = __builtin_nontemporal_load((const thcl_f4 *)(P.a + l * P.pitch + c));
    u[k] = P.u[(long)l * P.incu];
  }
#pragma unroll
  for (int k = 0; k < LINES; k++) {
    const thcl_u64 l = l0 + (thcl_u64)k * GROUPS;
    if (l >= P.lines) break;
    thcl_f4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float prod = UFIRST ? (P.alpha * u[k]) * v[e] : (P.alpha * v[e]) * u[k];
      r[e] = (P.beta == 1.f) ? a[k][e] + prod : P.beta * a[k][e] + prod;
    }
    __builtin_nontemporal_store(r, (thcl_f4 *)(P.a + l * P.pitch + c));
  }
}

// true when the update ran here; false: the caller takes the generic pointwise path
bool rank1_fast(THClState *state, thcl_rt *rt, float *a, thcl_u64 lines, thcl_u64 cols, thcl_u64 pitch, const float *u, long incu,
                const float *v, long incv, float beta, float alpha, bool ufirst) {
  if (cols % 4 != 0 || pitch % 4 != 0 || (((uintptr_t)a) & 15u) != 0 || pitch < cols) return false;
  const thcl_u64 gx = (cols / 4 + 63) / 64, gy = (lines + 4 * kRank1Lines - 1) / (4 * kRank1Lines);
  if (gx * gy >= (1ull << 31)) return false;
  Rank1Params P;
  P.a = a;
  P.u = u;
  P.v = v;
  P.lines = lines;
  P.cols = cols;
  P.pitch = pitch;
  P.gx = (unsigned)gx;
  P.incu = incu;
  P.incv = incv;
  P.beta = beta;
  P.alpha = alpha;
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  if (ufirst) hipLaunchKernelGGL(rank1_update<true>, dim3((unsigned)(gx * gy)), dim3(kThreads), 0, stream, P);
  else hipLaunchKernelGGL(rank1_update<false>, dim3((unsigned)(gx * gy)), dim3(kThreads), 0, stream, P);
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "rank-1 update launch failed: %s", hipGetErrorString(e));
  thcl_after_launch(state, rt);
  return true;
}

THClTensor *expanded(THClState *state, THClTensor *vec, long rows, long cols, bool along_rows) {
  long sz[2] = {rows, cols};
  long st[2] = {along_rows ? vec->stride[0] : 0, along_rows ? 0 : vec->stride[0]};
  THLongStorage sizes, strides;
  memset(&sizes, 0, sizeof(sizes));
  memset(&strides, 0, sizeof(strides));
  sizes.data = sz;
  sizes.size = 2;
  strides.data = st;
  strides.size = 2;
  return THClTensor_newWithStorage(state, vec->storage->device, vec->storage, vec->storageOffset, &sizes, &strides);
}
}  // namespace

extern "C" {

// y = alpha * op(A) * x + beta * y on column-major A (m x n, lda); BLAS argument
// meaning, operands given as tensors whose storage + offset mark the first element
// (src/lib/THClBlas.h:26-30, src/lib/THClBlas.cpp:199-262)
void THClBlas_gemv(THClState *state, char trans, long m, long n, float alpha, THClTensor *a, long lda, THClTensor *x,
                   long incx, float beta, THClTensor *y, long incy) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, a, x, y);
  THCL_CHECK(a->storage && x->storage && y->storage, "gemv operands need device storage");
  const bool t = (trans == 't' || trans == 'T');
  THCL_ARGCHECK(t || trans == 'n' || trans == 'N', 2, "trans must be 'n' or 't'");
  THCL_ARGCHECK(m >= 0 && n >= 0 && m < (1l << 31) && n < (1l << 31), 3, THCL_DIM_WARNING);
  if (n == 1) lda = m;  // a single column: any leading dimension does (src/lib/THClBlas.cpp:201-202)
  THCL_ARGCHECK(lda >= (m > 1 ? m : 1), 7, "lda must be at least m");
  const long outputs = t ? n : m;
  if (outputs == 0) return;
  thcl_rt *rt = thcl_ctx(state, y->storage->device);
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  GemvParams P;
  memset(&P, 0, sizeof(P));
  P.a = thcl_dptr(a);
  P.x = thcl_dptr(x);
  P.y = thcl_dptr(y);
  P.m = (thcl_u32)m;
  P.n = (thcl_u32)n;
  P.lda = (thcl_u64)lda;
  P.incx = incx;
  P.incy = incy;
  P.alpha = alpha;
  P.beta = beta;
  P.split = 1;
  P.per_split = (thcl_u32)(t ? m : n);
  P.outputs = (thcl_u32)outputs;
  const long cus = thcl_rt_get_props(rt)->compute_units;
  const bool whole_units = (m % 4 == 0);   // units of four rows; their 16-byte reads need no alignment
  if (t) {
    const bool vec = incx == 1;
    // few long columns: cut them into pieces of at least 8192 elements until the chip is full
    if (m >= 2048 && n < cus * 4) {
      long split = (cus * 8 + n - 1) / n;
      if (split > m / 8192) split = m / 8192;
      if (split > 1024) split = 1024;
      if (split > 1) {
        const long per = ((m + split - 1) / split + 1023) / 1024 * 1024;
        split = (m + per - 1) / per;
        if (split > 1) {
          P.split = (thcl_u32)split;
          P.per_split = (thcl_u32)per;
          P.partials = (double *)thcl_rt_workspace(rt, (size_t)split * (size_t)n * sizeof(double));
          THCL_CHECK(P.partials != nullptr, "%s", thcl_rt_error());
        }
      }
    }
#define GEMV_T(L)                                                                                        \
  {                                                                                                      \
    const dim3 grid((unsigned)((n + (kThreads / L) - 1) / (kThreads / L)), P.split);                     \
    if (vec && whole_units) hipLaunchKernelGGL((gemv_t<L, 1>), grid, dim3(kThreads), 0, stream, P);     \
    else if (vec) hipLaunchKernelGGL((gemv_t<L, 2>), grid, dim3(kThreads), 0, stream, P);                \
    else hipLaunchKernelGGL((gemv_t<L, 0>), grid, dim3(kThreads), 0, stream, P);                         \
  }
    // a whole block per column only while columns are few: with 2048 columns or more a wave per column
    // measured 3-5 % faster on columns of 4096 to 65536 elements (no barrier, no exchange through LDS)
    if (m >= 2048 && n < cus * 8) GEMV_T(256) else if (m >= 128) GEMV_T(64) else if (m > 16) GEMV_T(8) else GEMV_T(1)
#undef GEMV_T
    check("gemv");
    if (P.split > 1) {
      hipLaunchKernelGGL(gemv_finish, dim3((unsigned)((n + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, P);
      check("gemv finish");
    }
  } else {
    const int vecw = m >= 4 ? 4 : 1;   // units of four rows, the last one moved back when m is no multiple of 4
    const long units = (m + vecw - 1) / vecw;
    // fewer units than lanes: the wave's spare lanes take further columns
    unsigned ub_log2 = 6;
    while (ub_log2 > 0 && (1l << (ub_log2 - 1)) >= units) ub_log2--;
    P.ub_log2 = ub_log2;
    const long ub = 1l << ub_log2, col_lanes = kWave >> ub_log2;
    const long tiles = (units + ub - 1) / ub;
    const long target = cus * 4;
    long split = 1;
    if (tiles < target) {
      split = (target + tiles - 1) / tiles;
      const long most = (n + 32 * col_lanes - 1) / (32 * col_lanes);  // at least 32 columns per lane
      if (split > most) split = most;
      if (split > 256) split = 256;
      if (split < 1) split = 1;
    }
    long per = (n + split - 1) / split;
    if (per < 1) per = 1;
    split = n > 0 ? (n + per - 1) / per : 1;
    P.split = (thcl_u32)split;
    P.per_split = (thcl_u32)per;
    if (split > 1) {
      P.partials = (double *)thcl_rt_workspace(rt, (size_t)split * (size_t)m * sizeof(double));
      THCL_CHECK(P.partials != nullptr, "%s", thcl_rt_error());
    }
    const dim3 grid((unsigned)tiles, (unsigned)split);
    if (vecw == 4) hipLaunchKernelGGL((gemv_n<4>), grid, dim3(kThreads), 0, stream, P);
    else hipLaunchKernelGGL((gemv_n<1>), grid, dim3(kThreads), 0, stream, P);
    check("gemv");
    if (split > 1) {
      hipLaunchKernelGGL(gemv_finish, dim3((unsigned)((m + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, P);
      check("gemv finish");
    }
  }
  thcl_after_launch(state, rt);
  THCL_GUARD_END()
}

// A += alpha * x * y^T on column-major A (m x n, lda)
// (src/lib/THClBlas.h:32-35, src/lib/THClBlas.cpp:264-347)
void THClBlas_ger(THClState *state, long m, long n, float alpha, THClTensor *x, long incx, THClTensor *y, long incy,
                  THClTensor *a, long lda) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, a, x, y);
  THCL_CHECK(a->storage && x->storage && y->storage, "ger operands need device storage");
  if (n == 1) lda = m;
  if (m == 0 || n == 0) return;
  // views over the three storages: A as (n x m) with strides (lda, 1); x along the unit dim, y along the other
  long asz[2] = {n, m}, ast[2] = {lda, 1}, xst[2] = {0, incx}, yst[2] = {incy, 0};
  THLongStorage sizes, sa, sx, sy;
  memset(&sizes, 0, sizeof(sizes));
  sa = sx = sy = sizes;
  sizes.data = asz;
  sa.data = ast;
  sx.data = xst;
  sy.data = yst;
  sizes.size = sa.size = sx.size = sy.size = 2;
  const int dev = a->storage->device;
  THClTensor *av = THClTensor_newWithStorage(state, dev, a->storage, a->storageOffset, &sizes, &sa);
  THClTensor *xv = THClTensor_newWithStorage(state, dev, x->storage, x->storageOffset, &sizes, &sx);
  THClTensor *yv = THClTensor_newWithStorage(state, dev, y->storage, y->storageOffset, &sizes, &sy);
  ApplyCall c;
  c.n = 3;
  c.t[0] = av;
  c.t[1] = xv;
  c.t[2] = yv;
  c.val[0] = alpha;
  try {
    thcl_apply_expr(state, "*out += val1 * *in1 * *in2", c);
  } catch (...) {
    THClTensor_free(state, av);
    THClTensor_free(state, xv);
    THClTensor_free(state, yv);
    throw;
  }
  THClTensor_free(state, av);
  THClTensor_free(state, xv);
  THClTensor_free(state, yv);
  THCL_GUARD_END()
}

// (src/lib/THClTensorMathBlas.cpp:17-41); products and the running sum are fp64
float THClTensor_dot(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, self, src);
  const long n = THClTensor_nElement(state, self);
  THCL_ARGCHECK(n == THClTensor_nElement(state, src), 2, "sizes do not match");
  if (n == 0) return 0.f;
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, self));
  // The order of the products is free: same-shaped views that are dense when walked in memory order
  // (both transposed or permuted alike) are multiplied where they lie; others through dense stand-ins.
  THClTensor *pair[2] = {self, src};
  const JointLayout J = thcl_joint_collapse(2, pair);
  const bool in_place = J.valid && J.dims == 1 && J.strides[0][0] == 1 && J.strides[1][0] == 1;
  ThclTemp a(state, in_place ? nullptr : THClTensor_newContiguous(state, self));
  ThclTemp b(state, in_place ? nullptr : THClTensor_newContiguous(state, src));
  const unsigned tag = thcl_rt_next_tag(rt);
  thcl_dot_dense(state, rt, thcl_dptr(in_place ? self : a.t), thcl_dptr(in_place ? src : b.t), n, thcl_rt_tagged_word_device(rt), tag);
  float result = 0.f;
  THCL_CHECK(thcl_rt_await_tagged(rt, tag, &result) == 0, "%s", thcl_rt_error());
  return result;
  THCL_GUARD_END(0.f)
}

// dot of n elements at x[xoffset + i * incx] and y[yoffset + i * incy]; the two "wrappers" are what
// storage->wrapper holds, device addresses of the storages' first elements
// (src/lib/THClBlas.cpp:149-213, where they are the storages' buffer objects)
float THClBlas_dot(THClState *state, long n, void *xwrapper, long xoffset, long incx, void *ywrapper, long yoffset,
                   long incy) {
  THCL_GUARD_BEGIN
  if (n <= 0) return 0.f;
  if (n == 1) incx = incy = 1;
  THCL_CHECK(n <= INT32_MAX && incx <= INT32_MAX && incy <= INT32_MAX,
             "dot only supports n, incx and incy up to signed integer limits: %d", INT32_MAX);
  THCL_CHECK(xwrapper && ywrapper && xoffset >= 0 && yoffset >= 0 && incx > 0 && incy > 0, "dot: invalid operand");
  const int device = THClState_getDevice(state);
  // borrowed views: storages that are not reference-counted and own nothing
  THClStorage sx, sy;
  memset(&sx, 0, sizeof(sx));
  sx.device = device;
  sx.cl = thcl_ctx(state, device);
  sy = sx;
  sx.wrapper = xwrapper;
  sx.size = xoffset + (n - 1) * incx + 1;
  sy.wrapper = ywrapper;
  sy.size = yoffset + (n - 1) * incy + 1;
  ThclTemp x(state, THClTensor_newWithStorage1d(state, device, &sx, xoffset, n, incx));
  ThclTemp y(state, THClTensor_newWithStorage1d(state, device, &sy, yoffset, n, incy));
  return THClTensor_dot(state, x.t, y.t);
  THCL_GUARD_END(0.f)
}

// r_ = beta * t + alpha * mat * vec  (src/lib/THClTensorMathBlas.cpp:43-105)
void THClTensor_addmv(THClState *state, THClTensor *r_, float beta, THClTensor *t, float alpha, THClTensor *mat,
                      THClTensor *vec) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 4, r_, t, mat, vec);
  THCL_CHECK(mat->nDimension == 2 && vec->nDimension == 1, "matrix and vector expected");
  THCL_CHECK(mat->size[1] == vec->size[0], "size mismatch");
  THCL_CHECK(t->nDimension == 1 && t->size[0] == mat->size[0], "size mismatch");
  if (r_ != t) {
    THClTensor_resizeAs(state, r_, t);
    THClTensor_copy(state, r_, t);
  }
  if (mat->stride[0] == 1 && mat->stride[1] >= (mat->size[0] > 1 ? mat->size[0] : 1)) {
    THClBlas_gemv(state, 'n', mat->size[0], mat->size[1], alpha, mat, mat->stride[1], vec, vec->stride[0], beta, r_,
                  r_->stride[0]);
  } else if (mat->stride[1] == 1 && mat->stride[0] >= (mat->size[1] > 1 ? mat->size[1] : 1)) {
    THClBlas_gemv(state, 't', mat->size[1], mat->size[0], alpha, mat, mat->stride[0], vec, vec->stride[0], beta, r_,
                  r_->stride[0]);
  } else {
    ThclTemp cmat(state, THClTensor_newContiguous(state, mat));
    THClBlas_gemv(state, 't', mat->size[1], mat->size[0], alpha, cmat.t, cmat.t->stride[0], vec, vec->stride[0], beta, r_,
                  r_->stride[0]);
  }
  THCL_GUARD_END()
}

// r_ = beta * t + alpha * vec1 (x) vec2  (src/lib/THClTensorMathBlas.cpp:216-277).
// One pointwise pass over r_ with the vectors as stride-0 views; the reference
// scales r_ in one launch and calls ger in a second.
void THClTensor_addr(THClState *state, THClTensor *r_, float beta, THClTensor *t, float alpha, THClTensor *vec1,
                     THClTensor *vec2) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 4, r_, t, vec1, vec2);
  THCL_CHECK(vec1->nDimension == 1 && vec2->nDimension == 1, "vector and vector expected");
  THCL_CHECK(t->nDimension == 2, "size mismatch");
  THCL_CHECK(t->size[0] == vec1->size[0] && t->size[1] == vec2->size[0], "size mismatch");
  if (r_ != t) {
    THClTensor_resizeAs(state, r_, t);
    THClTensor_copy(state, r_, t);
  }
  if (r_->size[0] == 0 || r_->size[1] == 0) return;
  {
    // the generic path's operator is beta * out + (alpha * vec1[i]) * vec2[j]
    thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, r_));
    const long rows = r_->size[0], cols = r_->size[1];
    if (r_->stride[1] == 1 && r_->stride[0] >= cols && cols > 1 &&
        rank1_fast(state, rt, thcl_dptr(r_), (thcl_u64)rows, (thcl_u64)cols, (thcl_u64)r_->stride[0], thcl_dptr(vec1), vec1->stride[0],
                   thcl_dptr(vec2), vec2->stride[0], beta, alpha, true))
      return;
    if (r_->stride[0] == 1 && r_->stride[1] >= rows && rows > 1 &&
        rank1_fast(state, rt, thcl_dptr(r_), (thcl_u64)cols, (thcl_u64)rows, (thcl_u64)r_->stride[1], thcl_dptr(vec2), vec2->stride[0],
                   thcl_dptr(vec1), vec1->stride[0], beta, alpha, false))
      return;
  }
  THClTensor *v1 = expanded(state, vec1, r_->size[0], r_->size[1], true);
  THClTensor *v2 = expanded(state, vec2, r_->size[0], r_->size[1], false);
  ApplyCall c;
  c.n = 3;
  c.t[0] = r_;
  c.t[1] = v1;
  c.t[2] = v2;
  c.val[0] = beta;
  c.val[1] = alpha;
  try {
    if (beta == 1.f) thcl_apply_expr(state, "*out += val2 * *in1 * *in2", c);
    else thcl_apply_expr(state, "*out = val1 * *out + val2 * *in1 * *in2", c);
  } catch (...) {
    THClTensor_free(state, v1);
    THClTensor_free(state, v2);
    throw;
  }
  THClTensor_free(state, v1);
  THClTensor_free(state, v2);
  THCL_GUARD_END()
}

}  // extern "C"
