// Device side of the pointwise apply engine.  This text is compiled twice: by
// hipcc for the fixed operators, and at run time by hipRTC with a user
// expression wrapped into an operator struct.  It therefore includes nothing
// and uses only built-in types.
//
// What it replaces: the templated OpenCL kernel THClTensor_pointwiseApplyD
// (reference: src/lib/THClApply.cl:47-102), one work-item per element with a
// `%`,`/` chain per operand and per dimension.  Here:
//   * contiguous operands move as 128-bit vectors, several in flight per lane;
//   * same-shaped strided operands share one index decomposition (joint
//     layout), done per 4-element unit when the innermost run allows it, with
//     multiply-shift division;
//   * operands of different shapes fall back to one decomposition per operand.
//
// An operator is a struct with
//   static constexpr int NT;   // tensors it touches (1..3), operand 0 is written
//   static __device__ void run(float &o, float a, float b, float v1, float v2, float p1, float p2);
// `o` holds operand 0's old value on entry; loads whose value the operator
// never reads are removed by the compiler, so write-only operators (fill,
// copy) cost no read of operand 0.
#ifndef THCL_APPLY_DEVICE_H
#define THCL_APPLY_DEVICE_H

#define THCL_APPLY_THREADS 256
// units per lane and tile, per kernel family (measured on MI355X: dense kernels stream
// fastest with one 128-bit unit per lane and a very large grid; strided scalar
// kernels gain from several independent loads in flight)
#define THCL_CONTIG_UNROLL 1
#ifndef THCL_CONTIG_S_UNROLL
#define THCL_CONTIG_S_UNROLL 4
#endif
// Dense vector kernel: floats per lane and lanes per block by tensor count.
// Measured on MI355X at 2^28 elements: two-operand kernels stream fastest with
// one-wave blocks of 128-bit lanes (+4.7 % over 256-thread blocks), three-operand
// kernels with one-wave blocks of 64-bit lanes (+6 %); one-operand kernels (fill)
// keep 256-thread blocks because a grid of one-wave blocks outruns the dispatcher.
#define THCL_CONTIG_W_FOR(NT) ((NT) >= 3 ? 2 : 4)
#define THCL_CONTIG_THREADS_FOR(NT) ((NT) >= 2 ? 64 : 256)
#ifndef THCL_JOINT_V4_UNROLL
#define THCL_JOINT_V4_UNROLL 1
#endif
#ifndef THCL_JOINT_S_UNROLL
#define THCL_JOINT_S_UNROLL 8
#endif
#ifndef THCL_GENERIC_UNROLL
#define THCL_GENERIC_UNROLL 4
#endif
#define THCL_JOINT_MAX_DIMS 8
#define THCL_GENERIC_MAX_DIMS 25

typedef float thcl_f4 __attribute__((ext_vector_type(4)));
typedef unsigned int thcl_u32;
typedef unsigned long long thcl_u64;

// n / d for n < 2^31 by multiply-high and shift (d >= 1).
struct ThclDivisor {
  thcl_u32 d, magic, shift, pad;
};
__device__ __forceinline__ thcl_u32 thcl_div(thcl_u32 n, const ThclDivisor &dv) {
  return (__umulhi(n, dv.magic) + n) >> dv.shift;
}
#ifndef __HIPCC_RTC__
// host side: magic = floor(2^32 * (2^shift - d) / d) + 1 with 2^shift >= d
inline ThclDivisor thcl_make_divisor(long d) {
  ThclDivisor r;
  r.d = (thcl_u32)d;
  unsigned shift = 0;
  while (shift < 32 && (1ull << shift) < (unsigned long long)d) shift++;
  const unsigned long long magic =
      ((1ull << 32) * ((1ull << shift) - (unsigned long long)d)) / (unsigned long long)d + 1;
  r.magic = (thcl_u32)magic;
  r.shift = shift;
  r.pad = 0;
  return r;
}
#endif

struct ThclContigParams {
  float *p[3];
  const float *pt[2];
  float val[2];
  thcl_u64 n;       // elements
  thcl_u64 ntiles;  // tiles of THREADS*UNROLL units
};

struct ThclJointParams {
  float *p[3];
  const float *pt[2];
  float val[2];
  thcl_u32 nunits;  // units = n / VEC
  thcl_u32 ntiles;
  int dims;
  ThclDivisor size[THCL_JOINT_MAX_DIMS];       // in units along the innermost dim
  thcl_u32 stride[3][THCL_JOINT_MAX_DIMS];     // in elements
};

struct ThclGenericOperand {
  int dims;
  int pad;
  ThclDivisor size[THCL_GENERIC_MAX_DIMS];
  thcl_u32 stride[THCL_GENERIC_MAX_DIMS];
  thcl_u32 pad2;
};
struct ThclGenericParams {
  float *p[3];
  const float *pt[2];
  float val[2];
  thcl_u32 n;
  thcl_u32 ntiles;
  ThclGenericOperand op[3];
};

// OpenCL's pown(x, n): x to an integer power by repeated squaring (what the reference's pow uses
// for integral exponents, src/lib/THClTensorMath2.cpp:22-61); user expressions reach it as pown().
__device__ __forceinline__ float thcl_pown(float x, int n) {
  float r = 1.0f, b = x;
  unsigned e = n < 0 ? (unsigned)(-(long long)n) : (unsigned)n;
  while (e) { if (e & 1u) r *= b; b *= b; e >>= 1; }
  return n < 0 ? 1.0f / r : r;
}

template <class Op>
__device__ __forceinline__ void thcl_apply_one(float &o, float a, float b, float v1, float v2, float p1, float p2) {
  Op::run(o, a, b, v1, v2, p1, p2);
}

// Streaming accesses: every element is touched once per launch, so loads and
// stores carry the nontemporal hint (measured +10% on transposing tiles, +5-8%
// on dense streams).
template <class V>
__device__ __forceinline__ V thcl_ld(const V *p) {
  return __builtin_nontemporal_load(p);
}
template <class V>
__device__ __forceinline__ void thcl_st(V v, V *p) {
  __builtin_nontemporal_store(v, p);
}

// A unit of an input: 4 adjacent floats, or one float repeated (stride-0 innermost dim).
template <class V>
__device__ __forceinline__ V thcl_ld_unit(const float *p, bool same) {
  if (same) {
    const float x = *p;
    V v;
    v[0] = x;
    v[1] = x;
    v[2] = x;
    v[3] = x;
    return v;
  }
  return thcl_ld((const V *)p);
}

// ------------------------------------------------------------ contiguous ---
// All operands dense and 16-byte aligned.  A tile is THREADS*UNROLL float4
// units; lane l of a block touches units l, l+THREADS, ... so every wave reads
// whole 1 KiB lines.  Loads of a tile are issued before any arithmetic.
template <int W>
struct ThclVec;
template <>
struct ThclVec<4> {
  typedef float T __attribute__((ext_vector_type(4)));
};
template <>
struct ThclVec<2> {
  typedef float T __attribute__((ext_vector_type(2)));
};

template <class Op, int NT>
__device__ __forceinline__ void thcl_apply_contig_v4(const ThclContigParams &P) {
  constexpr int W = THCL_CONTIG_W_FOR(NT), T = THCL_CONTIG_THREADS_FOR(NT), U = THCL_CONTIG_UNROLL;
  typedef typename ThclVec<W>::T VT;
  const float p1 = P.pt[0] ? *P.pt[0] : 0.f;
  const float p2 = P.pt[1] ? *P.pt[1] : 0.f;
  const float v1 = P.val[0], v2 = P.val[1];
  const thcl_u64 nv = P.n / W;
  VT *ov = (VT *)P.p[0];
  const VT *av = (const VT *)P.p[1];
  const VT *bv = (const VT *)P.p[2];
  for (thcl_u64 tile = blockIdx.x; tile < P.ntiles; tile += gridDim.x) {
    const thcl_u64 base = tile * (T * U) + threadIdx.x;
    VT o[U], a[U], b[U];
    if (base + (U - 1) * T < nv) {
#pragma unroll
      for (int k = 0; k < U; k++) {
        const thcl_u64 i = base + (thcl_u64)k * T;
        o[k] = __builtin_nontemporal_load(ov + i);
        if (NT > 1) a[k] = __builtin_nontemporal_load(av + i);
        if (NT > 2) b[k] = __builtin_nontemporal_load(bv + i);
      }
#pragma unroll
      for (int k = 0; k < U; k++) {
#pragma unroll
        for (int c = 0; c < W; c++) {
          float oo = o[k][c];
          thcl_apply_one<Op>(oo, NT > 1 ? a[k][c] : 0.f, NT > 2 ? b[k][c] : 0.f, v1, v2, p1, p2);
          o[k][c] = oo;
        }
      }
#pragma unroll
      for (int k = 0; k < U; k++) __builtin_nontemporal_store(o[k], ov + base + (thcl_u64)k * T);
    } else {
#pragma unroll
      for (int k = 0; k < U; k++) {
        const thcl_u64 i = base + (thcl_u64)k * T;
        if (i < nv) {
          VT x = ov[i], y, z;
          if (NT > 1) y = av[i];
          if (NT > 2) z = bv[i];
#pragma unroll
          for (int c = 0; c < W; c++) {
            float oo = x[c];
            thcl_apply_one<Op>(oo, NT > 1 ? y[c] : 0.f, NT > 2 ? z[c] : 0.f, v1, v2, p1, p2);
            x[c] = oo;
          }
          ov[i] = x;
        }
      }
    }
  }
  // the last n % W elements
  const thcl_u64 rem = P.n % W;
  if (blockIdx.x == 0 && threadIdx.x < rem) {
    const thcl_u64 i = nv * W + threadIdx.x;
    float oo = P.p[0][i];
    thcl_apply_one<Op>(oo, NT > 1 ? P.p[1][i] : 0.f, NT > 2 ? P.p[2][i] : 0.f, v1, v2, p1, p2);
    P.p[0][i] = oo;
  }
}

// Dense operands whose addresses are not all 16-byte aligned: one dword per
// lane, still whole lines per wave.
template <class Op, int NT>
__device__ __forceinline__ void thcl_apply_contig_s(const ThclContigParams &P) {
  const float p1 = P.pt[0] ? *P.pt[0] : 0.f;
  const float p2 = P.pt[1] ? *P.pt[1] : 0.f;
  const float v1 = P.val[0], v2 = P.val[1];
  for (thcl_u64 tile = blockIdx.x; tile < P.ntiles; tile += gridDim.x) {
    const thcl_u64 base = tile * (THCL_APPLY_THREADS * THCL_CONTIG_S_UNROLL) + threadIdx.x;
    float o[THCL_CONTIG_S_UNROLL], a[THCL_CONTIG_S_UNROLL], b[THCL_CONTIG_S_UNROLL];
    // Every load is issued: lanes past the end read the last element again and store nothing.  (A test
    // around the loads makes the compiler wait for each group before it issues the next.)
#pragma unroll
    for (int k = 0; k < THCL_CONTIG_S_UNROLL; k++) {
      thcl_u64 i = base + (thcl_u64)k * THCL_APPLY_THREADS;
      if (i >= P.n) i = P.n - 1;
      o[k] = thcl_ld(P.p[0] + i);
      if (NT > 1) a[k] = thcl_ld(P.p[1] + i);
      if (NT > 2) b[k] = thcl_ld(P.p[2] + i);
    }
#pragma unroll
    for (int k = 0; k < THCL_CONTIG_S_UNROLL; k++) {
      const thcl_u64 i = base + (thcl_u64)k * THCL_APPLY_THREADS;
      if (i < P.n) {
        float oo = o[k];
        thcl_apply_one<Op>(oo, NT > 1 ? a[k] : 0.f, NT > 2 ? b[k] : 0.f, v1, v2, p1, p2);
        thcl_st(oo, P.p[0] + i);
      }
    }
  }
}

// ------------------------------------------------------- joint strided ---
// Operands share sizes; dims were ordered by the written operand's stride and
// merged on the host.  A unit is VEC consecutive elements of the innermost
// dim (VEC = 4 needs unit stride there plus 16-byte aligned rows).
template <class Op, int NT, int VEC, int U>
__device__ __forceinline__ void thcl_apply_joint(const ThclJointParams &P) {
  const float p1 = P.pt[0] ? *P.pt[0] : 0.f;
  const float p2 = P.pt[1] ? *P.pt[1] : 0.f;
  const float v1 = P.val[0], v2 = P.val[1];
  for (thcl_u32 tile = blockIdx.x; tile < P.ntiles; tile += gridDim.x) {
    const thcl_u32 base = tile * (THCL_APPLY_THREADS * U) + threadIdx.x;
    thcl_u64 off[U][3];
#pragma unroll
    for (int k = 0; k < U; k++) {
      thcl_u32 u = base + k * THCL_APPLY_THREADS;
      if (u >= P.nunits) u = P.nunits - 1;  // lanes past the end read the last unit again and store nothing
      thcl_u64 o0 = 0, o1 = 0, o2 = 0;
      for (int d = P.dims - 1; d > 0; d--) {
        const thcl_u32 q = thcl_div(u, P.size[d]);
        const thcl_u32 r = u - q * P.size[d].d;
        const thcl_u32 rr = (d == P.dims - 1) ? r * VEC : r;
        o0 += (thcl_u64)rr * P.stride[0][d];
        if (NT > 1) o1 += (thcl_u64)rr * P.stride[1][d];
        if (NT > 2) o2 += (thcl_u64)rr * P.stride[2][d];
        u = q;
      }
      const thcl_u32 r0 = (P.dims == 1) ? u * VEC : u;
      off[k][0] = o0 + (thcl_u64)r0 * P.stride[0][0];
      off[k][1] = o1 + (thcl_u64)r0 * P.stride[1][0];
      off[k][2] = o2 + (thcl_u64)r0 * P.stride[2][0];
    }
    if (VEC == 4) {
      // an input whose innermost stride is 0 repeats one value along the unit
      const bool same1 = NT > 1 && P.stride[1][P.dims - 1] == 0, same2 = NT > 2 && P.stride[2][P.dims - 1] == 0;
      thcl_f4 o[U], a[U], b[U];
#pragma unroll
      for (int k = 0; k < U; k++) {  // all loads issued, no test between them
        o[k] = thcl_ld((const thcl_f4 *)(P.p[0] + off[k][0]));
        if (NT > 1) a[k] = thcl_ld_unit<thcl_f4>(P.p[1] + off[k][1], same1);
        if (NT > 2) b[k] = thcl_ld_unit<thcl_f4>(P.p[2] + off[k][2], same2);
      }
#pragma unroll
      for (int k = 0; k < U; k++) {
        if (base + k * THCL_APPLY_THREADS < P.nunits) {
#pragma unroll
          for (int c = 0; c < 4; c++) {
            float oo = o[k][c];
            thcl_apply_one<Op>(oo, NT > 1 ? a[k][c] : 0.f, NT > 2 ? b[k][c] : 0.f, v1, v2, p1, p2);
            o[k][c] = oo;
          }
          thcl_st(o[k], (thcl_f4 *)(P.p[0] + off[k][0]));
        }
      }
    } else {
      // The written operand streams (nontemporal) only when its rows are dense:
      // a wave then writes whole lines.  With a stride it writes parts of lines
      // it has just read, which must stay cached in between (measured: the
      // hint costs a stride-2 read-modify-write 17%).
      const bool stream0 = P.stride[0][P.dims - 1] == 1;
      float o[U], a[U], b[U];
#pragma unroll
      for (int k = 0; k < U; k++) {  // all loads issued, no test between them
        o[k] = stream0 ? thcl_ld(P.p[0] + off[k][0]) : P.p[0][off[k][0]];
        if (NT > 1) a[k] = thcl_ld(P.p[1] + off[k][1]);
        if (NT > 2) b[k] = thcl_ld(P.p[2] + off[k][2]);
      }
#pragma unroll
      for (int k = 0; k < U; k++) {
        if (base + k * THCL_APPLY_THREADS < P.nunits) {
          float oo = o[k];
          thcl_apply_one<Op>(oo, NT > 1 ? a[k] : 0.f, NT > 2 ? b[k] : 0.f, v1, v2, p1, p2);
          if (stream0)
            thcl_st(oo, P.p[0] + off[k][0]);
          else
            P.p[0][off[k][0]] = oo;
        }
      }
    }
  }
}

// ------------------------------------------------------------- generic ---
// Operands agree only in element count: each decomposes the linear index over
// its own collapsed dims (the reference's scheme, with cheaper division).
__device__ __forceinline__ thcl_u64 thcl_generic_offset(thcl_u32 i, const ThclGenericOperand &L) {
  thcl_u64 off = 0;
  for (int d = L.dims - 1; d > 0; d--) {
    const thcl_u32 q = thcl_div(i, L.size[d]);
    off += (thcl_u64)(i - q * L.size[d].d) * L.stride[d];
    i = q;
  }
  return off + (thcl_u64)i * L.stride[0];
}

template <class Op, int NT>
__device__ __forceinline__ void thcl_apply_generic(const ThclGenericParams &P) {
  const float p1 = P.pt[0] ? *P.pt[0] : 0.f;
  const float p2 = P.pt[1] ? *P.pt[1] : 0.f;
  const float v1 = P.val[0], v2 = P.val[1];
  for (thcl_u32 tile = blockIdx.x; tile < P.ntiles; tile += gridDim.x) {
    const thcl_u32 base = tile * (THCL_APPLY_THREADS * THCL_GENERIC_UNROLL) + threadIdx.x;
    // all of the tile's loads first (lanes past the end read the last element again and store nothing),
    // then the arithmetic, then the stores: a store between two loads would hold the second load back,
    // since the operands may share memory
    thcl_u64 o0[THCL_GENERIC_UNROLL];
    float oo[THCL_GENERIC_UNROLL], a[THCL_GENERIC_UNROLL], b[THCL_GENERIC_UNROLL];
#pragma unroll
    for (int k = 0; k < THCL_GENERIC_UNROLL; k++) {
      thcl_u32 i = base + k * THCL_APPLY_THREADS;
      if (i >= P.n) i = P.n - 1;
      o0[k] = thcl_generic_offset(i, P.op[0]);
      oo[k] = P.p[0][o0[k]];
      a[k] = b[k] = 0.f;
      if (NT > 1) a[k] = P.p[1][thcl_generic_offset(i, P.op[1])];
      if (NT > 2) b[k] = P.p[2][thcl_generic_offset(i, P.op[2])];
    }
#pragma unroll
    for (int k = 0; k < THCL_GENERIC_UNROLL; k++) {
      thcl_apply_one<Op>(oo[k], a[k], b[k], v1, v2, p1, p2);
      if (base + k * THCL_APPLY_THREADS < P.n) P.p[0][o0[k]] = oo[k];
    }
  }
}

// ---------------------------------------------------------------- tiled ---
// Same-shaped operands whose unit-stride dims differ (a transposed view meeting
// a dense tensor).  A block owns a TILE_A x TILE_B tile of the plane spanned by dim A
// (unit stride in the written operand) and dim B (unit stride in the
// transposed inputs): those inputs are read with lanes along B into LDS, then
// everything is processed with lanes along A, so every global access is a run
// of 256 contiguous bytes per wave.
// Three tile shapes (A x B) of 16384 elements share one kernel; the host picks
// per launch (field `shape`) the one that wastes least on the plane's edges.
#define THCL_TILE_SHAPES 3
#define THCL_TILE_SHAPE_A(s) ((s) == 0 ? 128 : (s) == 1 ? 64 : 256)
#define THCL_TILE_SHAPE_B(s) ((s) == 0 ? 128 : (s) == 1 ? 256 : 64)
#define THCL_TILE_LDS_FLOATS (256 * 65)  // the largest of rows x (columns + 1)
#ifndef THCL_TILE_UNROLL
#define THCL_TILE_UNROLL 8
#endif
#define THCL_TILE_THREADS 1024
#define THCL_TILE_MAX_OUTER 6
struct ThclTileParams {
  float *p[3];
  const float *pt[2];
  float val[2];
  thcl_u32 sizeA, sizeB;
  thcl_u32 strideA[3], strideB[3];
  thcl_u32 via_lds[3];                  // input t is staged through LDS (its strideB is 1)
  ThclDivisor tilesA, tilesB;
  int nouter;
  ThclDivisor osize[THCL_TILE_MAX_OUTER];
  thcl_u32 ostride[3][THCL_TILE_MAX_OUTER];
  thcl_u32 shape;     // index into THCL_TILE_SHAPE_A/B
  thcl_u32 diagonal;  // 1: shift the B tile coordinate by the A tile coordinate
  thcl_u32 vec4;      // 1: sizes, strides and bases allow 128-bit accesses on every operand
};

template <class Op, int NT, int TA, int TB>
__device__ __forceinline__ void thcl_apply_tiled_body(const ThclTileParams &P, float (*lds)[THCL_TILE_LDS_FLOATS]) {
  static_assert(TA * (TB + 1) <= THCL_TILE_LDS_FLOATS, "tile does not fit its LDS array");
  constexpr int PITCH = TB + 1;  // odd: the transposed read of phase 2 hits distinct banks
  const float p1 = P.pt[0] ? *P.pt[0] : 0.f;
  const float p2 = P.pt[1] ? *P.pt[1] : 0.f;
  const float v1 = P.val[0], v2 = P.val[1];
  // block -> (tile along A fastest, tile along B, outer indices)
  thcl_u32 bid = blockIdx.x;
  thcl_u32 q = thcl_div(bid, P.tilesA);
  const thcl_u32 ta = bid - q * P.tilesA.d;
  const thcl_u32 a0 = ta * TA;
  bid = q;
  q = thcl_div(bid, P.tilesB);
  // Diagonal order: blocks that run together differ in both tile coordinates,
  // so with a power-of-two row pitch neither their reads nor their writes pile
  // onto the same few memory channels.
  thcl_u32 tb = bid - q * P.tilesB.d;
  if (P.diagonal) {
    tb += ta;
    tb -= thcl_div(tb, P.tilesB) * P.tilesB.d;
  }
  const thcl_u32 b0 = tb * TB;
  bid = q;
  thcl_u64 base[3] = {0, 0, 0};
  for (int d = P.nouter - 1; d >= 0; d--) {
    q = thcl_div(bid, P.osize[d]);
    const thcl_u32 r = bid - q * P.osize[d].d;
    base[0] += (thcl_u64)r * P.ostride[0][d];
    if (NT > 1) base[1] += (thcl_u64)r * P.ostride[1][d];
    if (NT > 2) base[2] += (thcl_u64)r * P.ostride[2][d];
    bid = q;
  }
  // Addresses advance by a constant step per pass, so each access costs one
  // 64-bit add; full tiles skip the bounds tests.
  const bool full = (a0 + TA <= P.sizeA) && (b0 + TB <= P.sizeB);
  // phase 1: lanes along B
  {
    constexpr int ROWS = THCL_TILE_THREADS / TB;  // rows of the tile covered per pass
    const thcl_u32 lane = threadIdx.x % TB, row = threadIdx.x / TB;
#pragma unroll
    for (int t = 1; t < NT; t++) {
      if (P.via_lds[t]) {
        const float *src = P.p[t] + base[t] + (thcl_u64)(a0 + row) * P.strideA[t] + (thcl_u64)(b0 + lane) * P.strideB[t];
        const thcl_u64 step = (thcl_u64)ROWS * P.strideA[t];
        if (full) {
#pragma unroll
          for (int i = 0; i < TA / ROWS; i++) {
            lds[t - 1][(row + ROWS * i) * PITCH + lane] = thcl_ld(src);
            src += step;
          }
        } else {
          const bool bok = b0 + lane < P.sizeB;
#pragma unroll 4
          for (int i = 0; i < TA / ROWS; i++) {
            if (bok && a0 + row + ROWS * i < P.sizeA) lds[t - 1][(row + ROWS * i) * PITCH + lane] = thcl_ld(src);
            src += step;
          }
        }
      }
    }
  }
  __syncthreads();
  // phase 2: lanes along A
  {
    constexpr int ROWS = THCL_TILE_THREADS / TA;
    const thcl_u32 lane = threadIdx.x % TA, row = threadIdx.x / TA;
    float *op = P.p[0] + base[0] + (thcl_u64)(a0 + lane) * P.strideA[0] + (thcl_u64)(b0 + row) * P.strideB[0];
    const thcl_u64 ostep = (thcl_u64)ROWS * P.strideB[0];
    const float *q1 = nullptr, *q2 = nullptr;
    thcl_u64 step1 = 0, step2 = 0;
    if (NT > 1 && !P.via_lds[1]) {
      q1 = P.p[1] + base[1] + (thcl_u64)(a0 + lane) * P.strideA[1] + (thcl_u64)(b0 + row) * P.strideB[1];
      step1 = (thcl_u64)ROWS * P.strideB[1];
    }
    if (NT > 2 && !P.via_lds[2]) {
      q2 = P.p[2] + base[2] + (thcl_u64)(a0 + lane) * P.strideA[2] + (thcl_u64)(b0 + row) * P.strideB[2];
      step2 = (thcl_u64)ROWS * P.strideB[2];
    }
    const bool aok = a0 + lane < P.sizeA;
#pragma unroll THCL_TILE_UNROLL
    for (int i = 0; i < TB / ROWS; i++) {
      const thcl_u32 bl = row + ROWS * i;
      if (full || (aok && b0 + bl < P.sizeB)) {
        float oo = thcl_ld(op), x = 0.f, y = 0.f;
        if (NT > 1) x = P.via_lds[1] ? lds[0][lane * PITCH + bl] : thcl_ld(q1);
        if (NT > 2) y = P.via_lds[2] ? lds[NT > 2 ? 1 : 0][lane * PITCH + bl] : thcl_ld(q2);
        thcl_apply_one<Op>(oo, x, y, v1, v2, p1, p2);
        thcl_st(oo, op);
      }
      op += ostep;
      if (NT > 1) q1 += step1;
      if (NT > 2) q2 += step2;
    }
  }
}

// picks element e (0..3, differs per lane) of a 4-vector
__device__ __forceinline__ float thcl_pick4(const thcl_f4 &v, int e) {
  return e == 0 ? v[0] : e == 1 ? v[1] : e == 2 ? v[2] : v[3];
}

// The same tiling with 128-bit global accesses: phase 1 reads 4 values along B per
// lane, phase 2 reads, computes and writes 4 values along A per lane.  LDS is
// addressed one float at a time (the pitch is odd); each lane walks its 4 values
// starting at a different one (by its group of 8 lanes) so the 32 lanes of a pass
// fall on 32 different banks.  Needs sizeA, sizeB and every stride that is not 1
// to be multiples of 4, 16-byte aligned bases and no operand repeated along A.
template <class Op, int NT, int TA, int TB>
__device__ __forceinline__ void thcl_apply_tiled_body_v4(const ThclTileParams &P, float (*lds)[THCL_TILE_LDS_FLOATS]) {
  static_assert(TA * (TB + 1) <= THCL_TILE_LDS_FLOATS, "tile does not fit its LDS array");
  constexpr int PITCH = TB + 1;
  const float p1 = P.pt[0] ? *P.pt[0] : 0.f;
  const float p2 = P.pt[1] ? *P.pt[1] : 0.f;
  const float v1 = P.val[0], v2 = P.val[1];
  thcl_u32 bid = blockIdx.x;
  thcl_u32 q = thcl_div(bid, P.tilesA);
  const thcl_u32 ta = bid - q * P.tilesA.d;
  const thcl_u32 a0 = ta * TA;
  bid = q;
  q = thcl_div(bid, P.tilesB);
  thcl_u32 tb = bid - q * P.tilesB.d;
  if (P.diagonal) {
    tb += ta;
    tb -= thcl_div(tb, P.tilesB) * P.tilesB.d;
  }
  const thcl_u32 b0 = tb * TB;
  bid = q;
  thcl_u64 base[3] = {0, 0, 0};
  for (int d = P.nouter - 1; d >= 0; d--) {
    q = thcl_div(bid, P.osize[d]);
    const thcl_u32 r = bid - q * P.osize[d].d;
    base[0] += (thcl_u64)r * P.ostride[0][d];
    if (NT > 1) base[1] += (thcl_u64)r * P.ostride[1][d];
    if (NT > 2) base[2] += (thcl_u64)r * P.ostride[2][d];
    bid = q;
  }
  const bool full = (a0 + TA <= P.sizeA) && (b0 + TB <= P.sizeB);
  const int rot = (int)((threadIdx.x & 31u) >> 3);
  // phase 1: lanes along B, 4 values each
  {
    constexpr int BQ = TB / 4, ROWS = THCL_TILE_THREADS / BQ;
    const thcl_u32 l4 = threadIdx.x % BQ, row = threadIdx.x / BQ;
#pragma unroll
    for (int t = 1; t < NT; t++) {
      if (P.via_lds[t]) {
        const float *src = P.p[t] + base[t] + (thcl_u64)(a0 + row) * P.strideA[t] + (b0 + 4 * l4);
        const thcl_u64 step = (thcl_u64)ROWS * P.strideA[t];
        const bool bok = b0 + 4 * l4 < P.sizeB;
#pragma unroll
        for (int i = 0; i < TA / ROWS; i++) {
          if (full || (bok && a0 + row + ROWS * i < P.sizeA)) {
            const thcl_f4 v = thcl_ld((const thcl_f4 *)src);
            float *dst = &lds[t - 1][(row + ROWS * i) * PITCH + 4 * l4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
              const int e = (c + rot) & 3;
              dst[e] = thcl_pick4(v, e);
            }
          }
          src += step;
        }
      }
    }
  }
  __syncthreads();
  // phase 2: lanes along A, 4 values each
  {
    constexpr int AQ = TA / 4, ROWS = THCL_TILE_THREADS / AQ;
    const thcl_u32 l4 = threadIdx.x % AQ, row = threadIdx.x / AQ;
    float *op = P.p[0] + base[0] + (a0 + 4 * l4) + (thcl_u64)(b0 + row) * P.strideB[0];
    const thcl_u64 ostep = (thcl_u64)ROWS * P.strideB[0];
    const float *q1 = nullptr, *q2 = nullptr;
    thcl_u64 step1 = 0, step2 = 0;
    if (NT > 1 && !P.via_lds[1]) {
      q1 = P.p[1] + base[1] + (a0 + 4 * l4) + (thcl_u64)(b0 + row) * P.strideB[1];
      step1 = (thcl_u64)ROWS * P.strideB[1];
    }
    if (NT > 2 && !P.via_lds[2]) {
      q2 = P.p[2] + base[2] + (a0 + 4 * l4) + (thcl_u64)(b0 + row) * P.strideB[2];
      step2 = (thcl_u64)ROWS * P.strideB[2];
    }
    const bool aok = a0 + 4 * l4 < P.sizeA;
    auto gather = [&](const float *plane, thcl_u32 bl) {
      float t[4];
#pragma unroll
      for (int j = 0; j < 4; j++) t[j] = plane[(4 * l4 + ((j + rot) & 3)) * PITCH + bl];
      // t[j] holds element (j + rot) & 3
      thcl_f4 r;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int j = (c - rot) & 3;
        r[c] = j == 0 ? t[0] : j == 1 ? t[1] : j == 2 ? t[2] : t[3];
      }
      return r;
    };
#pragma unroll 4
    for (int i = 0; i < TB / ROWS; i++) {
      const thcl_u32 bl = row + ROWS * i;
      if (full || (aok && b0 + bl < P.sizeB)) {
        thcl_f4 oo = thcl_ld((const thcl_f4 *)op), x = {0.f, 0.f, 0.f, 0.f}, y = {0.f, 0.f, 0.f, 0.f};
        if (NT > 1) x = P.via_lds[1] ? gather(lds[0], bl) : thcl_ld((const thcl_f4 *)q1);
        if (NT > 2) y = P.via_lds[2] ? gather(lds[NT > 2 ? 1 : 0], bl) : thcl_ld((const thcl_f4 *)q2);
#pragma unroll
        for (int c = 0; c < 4; c++) {
          float o = oo[c];
          thcl_apply_one<Op>(o, x[c], y[c], v1, v2, p1, p2);
          oo[c] = o;
        }
        thcl_st(oo, (thcl_f4 *)op);
      }
      op += ostep;
      if (NT > 1) q1 += step1;
      if (NT > 2) q2 += step2;
    }
  }
}

template <class Op, int NT>
__device__ __forceinline__ void thcl_apply_tiled(const ThclTileParams &P) {
  __shared__ float lds[NT > 2 ? 2 : 1][THCL_TILE_LDS_FLOATS];
  if (P.vec4) {
    if (P.shape == 0)
      thcl_apply_tiled_body_v4<Op, NT, THCL_TILE_SHAPE_A(0), THCL_TILE_SHAPE_B(0)>(P, lds);
    else if (P.shape == 1)
      thcl_apply_tiled_body_v4<Op, NT, THCL_TILE_SHAPE_A(1), THCL_TILE_SHAPE_B(1)>(P, lds);
    else
      thcl_apply_tiled_body_v4<Op, NT, THCL_TILE_SHAPE_A(2), THCL_TILE_SHAPE_B(2)>(P, lds);
    return;
  }
  if (P.shape == 0)
    thcl_apply_tiled_body<Op, NT, THCL_TILE_SHAPE_A(0), THCL_TILE_SHAPE_B(0)>(P, lds);
  else if (P.shape == 1)
    thcl_apply_tiled_body<Op, NT, THCL_TILE_SHAPE_A(1), THCL_TILE_SHAPE_B(1)>(P, lds);
  else
    thcl_apply_tiled_body<Op, NT, THCL_TILE_SHAPE_A(2), THCL_TILE_SHAPE_B(2)>(P, lds);
}

// Entry points for one operator; K is a name prefix.  One macro per kernel family, so
// that a run-time compiled expression builds only the family a launch needs.
#define THCL_DEFINE_APPLY_CONTIG_V4(K, Op, NT)                                                                  \
  extern "C" __global__ __launch_bounds__(THCL_CONTIG_THREADS_FOR(NT)) void K##_contig_v4(ThclContigParams P) { \
    thcl_apply_contig_v4<Op, NT>(P);                                                                            \
  }
#define THCL_DEFINE_APPLY_CONTIG_S(K, Op, NT)                                                          \
  extern "C" __global__ __launch_bounds__(THCL_APPLY_THREADS) void K##_contig_s(ThclContigParams P) { \
    thcl_apply_contig_s<Op, NT>(P);                                                                    \
  }
#define THCL_DEFINE_APPLY_JOINT_V4(K, Op, NT)                                                         \
  extern "C" __global__ __launch_bounds__(THCL_APPLY_THREADS) void K##_joint_v4(ThclJointParams P) { \
    thcl_apply_joint<Op, NT, 4, THCL_JOINT_V4_UNROLL>(P);                                             \
  }
#define THCL_DEFINE_APPLY_JOINT_S(K, Op, NT)                                                         \
  extern "C" __global__ __launch_bounds__(THCL_APPLY_THREADS) void K##_joint_s(ThclJointParams P) { \
    thcl_apply_joint<Op, NT, 1, THCL_JOINT_S_UNROLL>(P);                                             \
  }
#define THCL_DEFINE_APPLY_GENERIC(K, Op, NT)                                                            \
  extern "C" __global__ __launch_bounds__(THCL_APPLY_THREADS) void K##_generic(ThclGenericParams P) { \
    thcl_apply_generic<Op, NT>(P);                                                                      \
  }
#define THCL_DEFINE_APPLY_TILED(K, Op, NT)                                                       \
  extern "C" __global__ __launch_bounds__(THCL_TILE_THREADS) void K##_tiled(ThclTileParams P) { \
    thcl_apply_tiled<Op, NT>(P);                                                                 \
  }
#define THCL_DEFINE_APPLY_KERNELS(K, Op, NT) \
  THCL_DEFINE_APPLY_CONTIG_V4(K, Op, NT)     \
  THCL_DEFINE_APPLY_CONTIG_S(K, Op, NT)      \
  THCL_DEFINE_APPLY_JOINT_V4(K, Op, NT)      \
  THCL_DEFINE_APPLY_JOINT_S(K, Op, NT)       \
  THCL_DEFINE_APPLY_GENERIC(K, Op, NT)       \
  THCL_DEFINE_APPLY_TILED(K, Op, NT)

#endif  // THCL_APPLY_DEVICE_H
