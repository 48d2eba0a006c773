// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32), column-major BLAS
// semantics: C[m x n] = alpha * op(A) * op(B) + beta * C.
//
// What it replaces: the clblasSgemm call of THClBlas_gemm (reference:
// src/lib/THClBlas.cpp:381-449), whose arithmetic lives in clBLAS.
//
// Shape of the kernel: 256 threads = 4 waves in a 2x2 arrangement over a
// BM x BN block tile (4x1 or 1x4 over the 128x32 and 32x128 tiles that serve
// products with one side of at most 32); K advances in slabs of 16 staged through double-buffered
// LDS (one barrier per slab), the next slab's global loads are issued before
// the current slab's MFMAs (two slabs ahead, through buffer descriptors whose
// base moves with scalar arithmetic, so the loop computes no address with vector
// instructions).  Operands that are contiguous along m/n in memory sit in LDS as
// [k][mn] with the wave's sub-tiles interleaved, and are read 64 bits per two
// MFMAs; operands contiguous along k sit as [mn][k+4] and are read 128 bits per
// four MFMAs.  Within a group of 8 k-values, MFMA step s consumes k = s (lanes
// 0-31) and k = 4+s (lanes 32-63) for both operands, which is what makes the
// 128-bit read usable.  Blocks are renumbered so the blocks an XCD receives form
// a compact patch of the tile grid and share its L2; tiles beyond a whole number
// per CU share their K among several blocks of the same launch (plan_tail).
// A product with a short side streams its long operand from memory straight into
// the matrix cores (sgemm_stream, further down).
#include <hip/hip_runtime.h>

#include <cstring>
#include <type_traits>

#include "internal.h"

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef f4 f4u __attribute__((aligned(4)));   // a 16-byte access that only needs the alignment of its elements

constexpr int BK = 16;
constexpr int KPITCH = BK + 4;  // [mn][k] rows: odd number of 16-byte chunks -> conflict-free 128-bit reads

struct GemmParams {
  const float *a, *b;
  float *c;
  int m, n, k;
  int lda, ldb, ldc;
  float alpha, beta;
  int tiles_m, tiles_n;
  int group_m;  // tiles along m per scheduling group
  int ksplit;   // blockIdx.y slices of K; > 1: raw partial products go to `work`
  int kchunk;   // K per slice (multiple of BK)
  float *work;  // [ksplit][n][m] dense partials
  // A launch of several tiles per CU whose tile count is no multiple of the CUs: the first `whole_tiles` logical
  // tiles (a multiple of the CUs) get a block each, and each of the `tail_tiles` after them gets `tail_split` blocks
  // that share its K (`tail_kchunk` each), numbered behind the others so that they fill the CUs as those run dry.
  // Their raw partial products go to `work` as [slice][tail tile][BN][BM] and tail_reduce adds them in slice order.
  int whole_tiles, tail_tiles, tail_split, tail_kchunk;
};

// logical tile id -> tile coordinates, grouped order: walk group_m tiles down m, then step along n
__device__ __forceinline__ void tile_of(const GemmParams &P, int bid, int &tm, int &tn) {
  const int gsz = P.group_m * P.tiles_n;
  const int g = bid / gsz, r = bid % gsz;
  const int m_first = g * P.group_m;
  const int m_count = (P.tiles_m - m_first < P.group_m) ? (P.tiles_m - m_first) : P.group_m;
  tm = m_first + r % m_count;
  tn = r / m_count;
}

// Buffer loads: the address is a descriptor's base + a per-lane 32-bit offset + a scalar 32-bit offset, so a loop
// that walks rows needs no vector arithmetic for its addresses, and what lies at or beyond the descriptor's extent
// reads as zero instead of being fetched (no clamping of addresses past the end of a range).
typedef unsigned st_u4 __attribute__((ext_vector_type(4)));
typedef unsigned st_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t st_buffer(const void *base, unsigned long long bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(bytes > 0xffffffffull ? 0xffffffffu : (unsigned)bytes), 0x00020000);
}
template <int N, bool STREAM>
__device__ __forceinline__ auto st_buffer_load(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned uniform_off) {
  typedef float T __attribute__((ext_vector_type(N)));
  constexpr int aux = STREAM ? 2 : 0;   // nontemporal: the long operand is read once
  if constexpr (N == 4) return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, uniform_off, aux));
  else if constexpr (N == 2) return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(r, lane_off, uniform_off, aux));
  else return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, uniform_off, aux));
}

// One operand tile in LDS.  KC: contiguous along k in global memory.
template <int BMN, bool KC>
struct TileLds {
  static constexpr int FLOATS = KC ? BMN * KPITCH : BK * BMN;
};

// Edge kernels 2 and 3 (pitches too long for a buffer descriptor's 32-bit offsets): what a lane's loads of one operand
// keep from slab to slab, worked out once per tile (with the extent tests and the 64-bit products redone at every slab
// a tile on the rim took 1.6 times as long as a whole one).
// EDGE 2: at[p] is the lane's 16-byte group in k row 0 (operands contiguous along m/n) or the start of its row
// (operands contiguous along k), moved to the operand's last group or row when it lies beyond the m/n extent; in[p]
// is 15 when it lies inside; a group that straddles the extent is read through a 16-byte window moved back to end at
// the extent and sh[p] tells by how many elements.  EDGE 3: per element: for operands contiguous along m/n at[p] is
// the operand's base, mo[p][c] the element's offset along m/n (the last one when it lies beyond), in[p] one bit per
// element.
template <int BMN, bool KC, int EDGE>
struct EdgeLanes {
  static constexpr int GROUPS = BMN * BK / 4;
  static constexpr int NV = GROUPS >= 256 ? GROUPS / 256 : 1;
  static constexpr bool PART = GROUPS < 256;
  const float *at[NV];
  unsigned in[NV];
  unsigned sh[NV];
  int mo[(EDGE == 3 && !KC) ? NV : 1][4];
  __device__ __forceinline__ void set(const float *g, int ld, int mn0, int lim_mn) {
#pragma unroll
    for (int p = 0; p < NV; p++) {
      const int f = PART ? (int)(threadIdx.x % GROUPS) : (int)(threadIdx.x + 256 * p);
      sh[p] = 0u;
      if (KC) {
        const int mn = mn0 + f / (BK / 4);
        in[p] = mn < lim_mn ? 15u : 0u;
        at[p] = g + (size_t)(mn < lim_mn ? mn : lim_mn - 1) * ld;
      } else if (EDGE == 2) {
        const int mq = mn0 + (f % (BMN / 4)) * 4;
        const int mw = mq + 4 <= lim_mn ? mq : lim_mn - 4;
        in[p] = mq < lim_mn ? 15u : 0u;
        sh[p] = mq < lim_mn ? (unsigned)(mq - mw) : 0u;
        at[p] = g + mw;
      } else {
        const int mq = mn0 + (f % (BMN / 4)) * 4;
        at[p] = g;
        in[p] = 0u;
#pragma unroll
        for (int c = 0; c < 4; c++) {
          in[p] |= (mq + c < lim_mn ? 1u : 0u) << c;
          mo[p][c] = mq + c < lim_mn ? mq + c : lim_mn - 1;
        }
      }
    }
  }
};

// global -> registers: each thread carries BMN*BK/256/4 float4 (a 32-wide tile has 128 of them: the upper half of the
// block loads the same groups again and does not store them).  EDGE 0: the tile is whole and aligned.
// EDGE 1: any extents and alignment, through the same buffer loads as EDGE 0 with the descriptor ending at the
// operand's last element.  Line i of op(A) only reaches row i of the result and line j of op(B) only column j, so
// what a tile on the rim reads for lines beyond m or n (the neighbouring row's elements, or zeros past the
// descriptor's end) lands in results that are never stored and needs no masking; only k beyond the extent has to
// read as zero, in both operands.  For an operand stored as [k][mn] every such row lies past the descriptor's end
// (the range check is per 4-byte element, so the last row's groups that straddle the end keep their elements
// inside); for one stored as [mn][k] the slabs that reach past k get a mask per group, applied on the way to LDS.
// EDGE 2: the same cases for pitches beyond the descriptor's 32-bit offsets, with 16-byte loads that need no
// alignment; every load is issued (from the operand's last row or group when the lane's own lies outside), a group
// that straddles the operand's extent is read through a window moved back to end there and shifted into place on the
// way to LDS.  Needs at least 4 elements along each operand's contiguous dimension.  EDGE 3: one element at a time,
// for what is left.
// The choice is made at compile time: a run-time branch between two edge forms made the compiler wait for all loads
// at every slab (aligned 4096^3 through such an edge kernel: 101 TFLOP/s with the branch against 138 without).
template <int BMN, bool KC, int EDGE>
struct TileLoader {
  using LoadT = typename std::conditional<EDGE == 2, f4u, f4>::type;
  static constexpr int GROUPS = BMN * BK / 4;
  static constexpr int NV = GROUPS >= 256 ? GROUPS / 256 : 1;
  static constexpr bool PART = GROUPS < 256;
  f4 r[NV];
  unsigned keep[NV];   // edge kernels: one bit per element that lies inside the operand (and, from bit 4, how far the
                       // window was moved back); looked at when the registers go to LDS, so that nothing has to
                       // wait for the load before then

  // edge kernels: every load is issued, from an address inside the operand; what lies outside becomes zeros in store()
  __device__ __forceinline__ void load_edge(const EdgeLanes<BMN, KC, EDGE> &e, int ld, int k0, int lim_k) {
#pragma unroll
    for (int p = 0; p < NV; p++) {
      const int f = PART ? (int)(threadIdx.x % GROUPS) : (int)(threadIdx.x + 256 * p);
      if (KC) {
        const int kc = k0 + (f % (BK / 4)) * 4;
        if (EDGE == 2) {
          const int kw = kc + 4 <= lim_k ? kc : lim_k - 4;
          r[p] = *(const LoadT *)(e.at[p] + kw);
          keep[p] = kc < lim_k ? (e.in[p] | (unsigned)(kc - kw) << 4) : 0u;
        } else {
          unsigned ok = 0u;
#pragma unroll
          for (int c = 0; c < 4; c++) {
            r[p][c] = e.at[p][kc + c < lim_k ? kc + c : lim_k - 1];
            ok |= (kc + c < lim_k ? 1u : 0u) << c;
          }
          keep[p] = e.in[p] & ok;
        }
      } else {
        const int kr = k0 + f / (BMN / 4);
        const float *row = e.at[p] + (size_t)(kr < lim_k ? kr : lim_k - 1) * ld;
        if (EDGE == 2) {
          r[p] = *(const LoadT *)row;
          keep[p] = kr < lim_k ? (e.in[p] | e.sh[p] << 4) : 0u;
        } else {
#pragma unroll
          for (int c = 0; c < 4; c++) r[p][c] = row[e.mo[p][c]];
          keep[p] = kr < lim_k ? e.in[p] : 0u;
        }
      }
    }
  }
  // EDGE 0 and 1: through a buffer descriptor whose base is the slab's first element (the same for the whole block,
  // moved from slab to slab with scalar arithmetic): a thread's groups keep constant 32-bit byte offsets, so the loop
  // spends no vector instruction on addresses.
  __device__ __forceinline__ void set_offsets(int ld, unsigned (&off)[NV]) const {
#pragma unroll
    for (int p = 0; p < NV; p++) {
      const int f = PART ? (int)(threadIdx.x % GROUPS) : (int)(threadIdx.x + 256 * p);
      if (KC) off[p] = ((unsigned)(f / (BK / 4)) * (unsigned)ld + (unsigned)(f % (BK / 4)) * 4u) * 4u;
      else off[p] = ((unsigned)(f / (BMN / 4)) * (unsigned)ld + (unsigned)(f % (BMN / 4)) * 4u) * 4u;
    }
  }
  __device__ __forceinline__ void load_buf(__amdgpu_buffer_rsrc_t slab, const unsigned (&off)[NV]) {
#pragma unroll
    for (int p = 0; p < NV; p++) {
      r[p] = st_buffer_load<4, false>(slab, off[p], 0u);
      keep[p] = 15u;
    }
  }
  // EDGE 1, operands contiguous along k: which of a group's elements lie below the k extent, for slabs that may reach past it
  __device__ __forceinline__ void mask_k(int k0, int lim_k) {
    if (!KC) return;
#pragma unroll
    for (int p = 0; p < NV; p++) {
      const int f = PART ? (int)(threadIdx.x % GROUPS) : (int)(threadIdx.x + 256 * p);
      const int left = lim_k - (k0 + (f % (BK / 4)) * 4);
      keep[p] = left >= 4 ? 15u : left <= 0 ? 0u : (1u << left) - 1u;
    }
  }
  // plain loads, for tiles and slabs that the caller knows to lie inside the operand
  __device__ __forceinline__ void load_whole(const float *g, int ld, int mn0, int k0) {
#pragma unroll
    for (int p = 0; p < NV; p++) {
      const int f = PART ? (int)(threadIdx.x % GROUPS) : (int)(threadIdx.x + 256 * p);
      if (KC) {
        const int mn = f / (BK / 4), kq = f % (BK / 4);
        r[p] = *(const LoadT *)(g + (size_t)(mn0 + mn) * ld + k0 + kq * 4);
      } else {
        const int kk = f / (BMN / 4), q = f % (BMN / 4);
        r[p] = *(const LoadT *)(g + (size_t)(k0 + kk) * ld + mn0 + q * 4);
      }
      keep[p] = 15u;
    }
  }
  template <bool MASKED = true>
  __device__ __forceinline__ void store(float *lds) const {
    if (PART && threadIdx.x >= GROUPS) return;
#pragma unroll
    for (int p = 0; p < NV; p++) {
      const int f = threadIdx.x + 256 * p;
      f4 v = r[p];
      if (EDGE == 1 && KC && MASKED) {
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = (keep[p] >> c & 1u) ? v[c] : 0.f;
      }
      if (EDGE == 2) {   // element c of the group sits at c + (how far the window was moved back)
        const unsigned back = keep[p] >> 4;
        const f4 w = r[p];
        v = back == 0u ? w : back == 1u ? f4{w[1], w[2], w[3], 0.f} : back == 2u ? f4{w[2], w[3], 0.f, 0.f} : f4{w[3], 0.f, 0.f, 0.f};
        v = (keep[p] & 15u) ? v : f4{0.f, 0.f, 0.f, 0.f};
      }
      if (EDGE == 3) {
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = (keep[p] >> c & 1u) ? v[c] : 0.f;
      }
      if (KC) {
        const int mn = f / (BK / 4), kq = f % (BK / 4);
        *(f4 *)(lds + mn * KPITCH + kq * 4) = v;
      } else {
        const int kk = f / (BMN / 4), q = f % (BMN / 4);
        *(f4 *)(lds + kk * BMN + q * 4) = v;
      }
    }
  }
};

// fragments of one 8-k group for the wave's sub-tiles: frag[t][s], t = 32-wide sub-tile, s = MFMA step.
// An operand stored as [k][mn] interleaves its sub-tiles: sub-tile t holds the lines mn_wave0 + NT * i + t (i = the
// MFMA's own row or column index), so a lane's NT fragments of one k are neighbours and arrive with one 8-byte read,
// two steps with one instruction (every LDS read beside the MFMAs costs the matrix pipe some cycles).  An operand
// stored as [mn][k] keeps sub-tile t at mn_wave0 + 32 t + i: its four steps are one 16-byte read already.
template <int BMN, bool KC, int NT>
__device__ __forceinline__ void read_frags(const float *lds, int mn_wave0, int kgroup, float (&frag)[NT][4]) {
  const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
  if (KC) {
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const int mn = mn_wave0 + t * 32 + l32;
      const f4 v = *(const f4 *)(lds + mn * KPITCH + kgroup * 8 + 4 * h);
#pragma unroll
      for (int s = 0; s < 4; s++) frag[t][s] = v[s];
    }
  } else {
    typedef float FT __attribute__((ext_vector_type(NT)));
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const FT v = *(const FT *)(lds + (kgroup * 8 + 4 * h + s) * BMN + mn_wave0 + NT * l32);
#pragma unroll
      for (int t = 0; t < NT; t++) frag[t][s] = v[t];
    }
  }
}
// where a lane's accumulators lie in the block tile, by the same rule: line of sub-tile t, index i
template <bool KC, int NT>
__device__ __forceinline__ int frag_line(int t, int i) {
  return KC ? 32 * t + i : NT * i + t;
}

// TA: op(A) = A^T (A stored k-contiguous); TB: op(B) = B^T (B stored n-contiguous)
template <int BM, int BN, bool TA, bool TB, int EDGE>
__global__ __launch_bounds__(256) void sgemm_mfma(GemmParams P) {
  constexpr bool AKC = TA;    // 'n': a[i + l*lda] (m-contiguous); 't': a[l + i*lda] (k-contiguous)
  constexpr bool BKC = !TB;   // 'n': b[l + j*ldb] (k-contiguous); 't': b[j + l*ldb] (n-contiguous)
  constexpr int WAVES_M = BN == 32 ? 4 : BM == 32 ? 1 : 2, WAVES_N = 4 / WAVES_M;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;   // wave tile
  constexpr int MT = WM / 32, NT = WN / 32; // 32x32 MFMA tiles per wave
  constexpr int AF = TileLds<BM, AKC>::FLOATS, BF = TileLds<BN, BKC>::FLOATS;
  __shared__ __attribute__((aligned(16))) float lds[2 * (AF + BF)];

  // XCD-aware renumbering: consecutive hardware block ids go to different
  // XCDs, so give XCD x the x-th contiguous chunk of logical ids.
  int bid = blockIdx.x;
  const bool tail = bid >= P.whole_tiles;   // one of several blocks that share a tile's K
  int tail_tile = 0, tail_slice = 0;
  if (tail) {
    tail_tile = (bid - P.whole_tiles) / P.tail_split;
    tail_slice = (bid - P.whole_tiles) % P.tail_split;
    bid = P.whole_tiles + tail_tile;
  } else {
    const int per = P.whole_tiles / 8;
    if (per > 0 && bid < per * 8) bid = (bid % 8) * per + bid / 8;
  }
  int tm, tn;
  tile_of(P, bid, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int wave = threadIdx.x >> 6;
  const int wm0 = (wave % WAVES_M) * WM, wn0 = (wave / WAVES_M) * WN;

  f16v acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  TileLoader<BM, AKC, EDGE> la;
  TileLoader<BN, BKC, EDGE> lb;
  const int k_begin = tail ? tail_slice * P.tail_kchunk : blockIdx.y * P.kchunk;
  const int k_len = tail ? P.tail_kchunk : P.kchunk;
  const int k_end = (k_begin + k_len < P.k) ? (k_begin + k_len) : P.k;
  const int KT = (k_end - k_begin + BK - 1) / BK;

  // Two register sets: while slab kt is multiplied out of LDS, slab kt+1 waits in one
  // set (it goes to the other LDS buffer at the end of the step) and the loads of
  // slab kt+2 are in flight into the other set, so a load has two steps to land.
  // Loads are issued unconditionally (past the end they re-read the last slab) so
  // that the wait counts the compiler derives stay exact.
  TileLoader<BM, AKC, EDGE> la1;
  TileLoader<BN, BKC, EDGE> lb1;
  const int last = KT > 0 ? KT - 1 : 0;
  auto slab_k = [&](int kt) { return k_begin + (kt < last ? kt : last) * BK; };
  EdgeLanes<BM, AKC, EDGE> ea;
  EdgeLanes<BN, BKC, EDGE> eb;
  constexpr bool DESCRIPTOR = EDGE == 0 || EDGE == 1;
  if (!DESCRIPTOR) {
    ea.set(P.a, P.lda, m0, P.m);
    eb.set(P.b, P.ldb, n0, P.n);
  }
  unsigned off_a[TileLoader<BM, AKC, EDGE>::NV], off_b[TileLoader<BN, BKC, EDGE>::NV];
  if (DESCRIPTOR) {
    la.set_offsets(P.lda, off_a);
    lb.set_offsets(P.ldb, off_b);
  }
  // one past each operand's last element (k > 0 here)
  const float *a_end = P.a + (AKC ? (size_t)(P.m - 1) * P.lda + P.k : (size_t)(P.k - 1) * P.lda + P.m);
  const float *b_end = P.b + (BKC ? (size_t)(P.n - 1) * P.ldb + P.k : (size_t)(P.k - 1) * P.ldb + P.n);
  constexpr std::true_type whole_slab{};
  constexpr std::false_type any_slab{};
  // `whole`: the caller knows that the slab ends at or below the k extent
  auto fetch = [&](auto whole, auto &to_a, auto &to_b, int k0) {
    if constexpr (DESCRIPTOR) {
      const float *sa = AKC ? P.a + (size_t)m0 * P.lda + k0 : P.a + (size_t)k0 * P.lda + m0;
      const float *sb = BKC ? P.b + (size_t)n0 * P.ldb + k0 : P.b + (size_t)k0 * P.ldb + n0;
      to_a.load_buf(st_buffer(sa, EDGE == 0 ? 0xffffffffull : (unsigned long long)(a_end - sa) * 4ull), off_a);
      to_b.load_buf(st_buffer(sb, EDGE == 0 ? 0xffffffffull : (unsigned long long)(b_end - sb) * 4ull), off_b);
      if constexpr (EDGE == 1 && !decltype(whole)::value) {
        to_a.mask_k(k0, k_end);
        to_b.mask_k(k0, k_end);
      }
    } else {
      to_a.load_edge(ea, P.lda, k0, k_end);
      to_b.load_edge(eb, P.ldb, k0, k_end);
    }
  };
  fetch(any_slab, la, lb, slab_k(0));
  fetch(any_slab, la1, lb1, slab_k(1));
  la.store(lds);
  lb.store(lds + AF);
  __syncthreads();

  auto step = [&](auto inside, int kt, int cur, auto &issue_a, auto &issue_b, auto &keep_a, auto &keep_b) {
    float *As = lds + cur * (AF + BF);
    float *Bs = As + AF;
    if constexpr (decltype(inside)::value && !DESCRIPTOR) {
      issue_a.load_whole(P.a, P.lda, m0, slab_k(kt + 2));
      issue_b.load_whole(P.b, P.ldb, n0, slab_k(kt + 2));
    } else {
      fetch(inside, issue_a, issue_b, slab_k(kt + 2));
    }
    __builtin_amdgcn_sched_barrier(0);   // keep the loads at the top of the step
    {
#pragma unroll
      for (int kg = 0; kg < BK / 8; kg++) {
        float fa[MT][4], fb[NT][4];
        read_frags<BM, AKC, MT>(As, wm0, kg, fa);
        read_frags<BN, BKC, NT>(Bs, wn0, kg, fb);
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
          for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < NT; j++)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
      }
    }
    float *An = lds + (cur ^ 1) * (AF + BF);
    keep_a.template store<!decltype(inside)::value>(An);
    keep_b.template store<!decltype(inside)::value>(An + AF);
    __syncthreads();
  };
  int kt = 0;
  if (EDGE == 1 || (EDGE == 2 && m0 + BM <= P.m && n0 + BN <= P.n)) {
    // slabs are whole except the last ones, so the steps that store and request whole slabs (kt + 1, and kt + 2 and
    // kt + 3 below KF) go without the k masks (EDGE 1) or, for a tile inside the matrix (the same for the whole
    // block), with plain loads (EDGE 2); the general form is left to the end of K and to EDGE 2's tiles on the rim
    const int KF = (k_end - k_begin) / BK;
    for (; kt + 3 < KF; kt += 2) {
      step(whole_slab, kt, 0, la, lb, la1, lb1);
      step(whole_slab, kt + 1, 1, la1, lb1, la, lb);
    }
  }
  for (; kt + 1 < KT; kt += 2) {
    step(any_slab, kt, 0, la, lb, la1, lb1);
    step(any_slab, kt + 1, 1, la1, lb1, la, lb);
  }
  if (kt < KT) step(any_slab, kt, 0, la, lb, la1, lb1);

  // epilogue: of sub-tile (i, j) a lane holds the tile's rows 8 (r / 4) + 4 (lane / 32) + r % 4, r = 0..15, of the tile's
  // column lane % 32; frag_line() tells where those lie in the wave's tile.  Per column sub-tile j and quarter rq the
  // lane's MT * 4 values form MT groups of four consecutive rows of the result: with interleaved row sub-tiles one run
  // of MT * 4 rows, else one group per sub-tile.  The edge kernels use 16-byte accesses that need no alignment wherever
  // a group's four rows lie inside the result, and single elements for the group that straddles its last row.
  using CT = typename std::conditional<EDGE == 0, f4, f4u>::type;
  const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
  auto group = [&](int j, int rq, int g, int &row, f4 &v) {   // group g of (j, rq): its first row and its raw sums
    if (AKC) {
      row = m0 + wm0 + 32 * g + rq * 8 + h * 4;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = acc[g][j][rq * 4 + e];
    } else {
      row = m0 + wm0 + MT * (rq * 8 + h * 4) + 4 * g;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = acc[(4 * g + e) % MT][j][rq * 4 + (4 * g + e) / MT];
    }
  };
  float *w = P.ksplit > 1 ? P.work + (size_t)blockIdx.y * P.m * P.n : nullptr;   // raw partial product of this K slice, dense [n][m]
#pragma unroll
  for (int j = 0; j < NT; j++) {
    const int col = n0 + wn0 + frag_line<BKC, NT>(j, l32);
#pragma unroll
    for (int rq = 0; rq < 4; rq++)
#pragma unroll
      for (int g = 0; g < MT; g++) {
        int row;
        f4 v;
        group(j, rq, g, row, v);
        if (tail) {   // scaled and summed by tail_reduce
          *(f4 *)(P.work + ((size_t)tail_slice * P.tail_tiles + tail_tile) * (BM * BN) + (col - n0) * BM + (row - m0)) = v;
          continue;
        }
        if (P.ksplit > 1) {   // scaled and summed by splitk_reduce
          float *wp = w + (size_t)col * P.m + row;
          if (!EDGE || (col < P.n && row + 3 < P.m)) {
            *(CT *)wp = v;
          } else if (col < P.n) {
#pragma unroll
            for (int c = 0; c < 4; c++)
              if (row + c < P.m) wp[c] = v[c];
          }
          continue;
        }
        float *cp = P.c + (size_t)col * P.ldc + row;
        if (!EDGE || (col < P.n && row + 3 < P.m)) {
#pragma unroll
          for (int c = 0; c < 4; c++) v[c] = P.alpha * v[c];
          if (P.beta != 0.f) {
            const f4 old = *(const CT *)cp;
#pragma unroll
            for (int c = 0; c < 4; c++) v[c] += P.beta * old[c];
          }
          *(CT *)cp = v;
        } else if (col < P.n) {
#pragma unroll
          for (int c = 0; c < 4; c++) {
            if (row + c < P.m) {
              float x = P.alpha * v[c];
              if (P.beta != 0.f) x += P.beta * cp[c];
              cp[c] = x;
            }
          }
        }
      }
  }
}

// The tiles whose K was shared by several blocks: C = alpha * (sum over their slices, in slice order) + beta * C.
// A thread takes four rows of a column of one tile; ALIGNED: the result's 16-byte groups are whole and aligned.
template <int BM, int BN, bool ALIGNED>
__global__ __launch_bounds__(256) void tail_reduce(GemmParams P) {
  constexpr int UNITS = BM * BN / 4;   // per tile
  const int u = (int)(((size_t)blockIdx.x * 256 + threadIdx.x) % UNITS), t = (int)(((size_t)blockIdx.x * 256 + threadIdx.x) / UNITS);
  if (t >= P.tail_tiles) return;
  const f4 *w = (const f4 *)P.work + (size_t)t * UNITS + u;
  const size_t step = (size_t)P.tail_tiles * UNITS;
  f4 s = w[0];
  for (int k = 1; k < P.tail_split; k++) s += w[(size_t)k * step];
  int tm, tn;
  tile_of(P, P.whole_tiles + t, tm, tn);
  const int col = tn * BN + u / (BM / 4), row = tm * BM + (u % (BM / 4)) * 4;
  if (col >= P.n || row >= P.m) return;
  float *cp = P.c + (size_t)col * P.ldc + row;
  if (ALIGNED || row + 3 < P.m) {
    f4 v = P.alpha * s;
    if (P.beta != 0.f) v += P.beta * *(const f4u *)cp;
    if (ALIGNED) *(f4 *)cp = v;
    else *(f4u *)cp = v;
  } else {
    for (int c = 0; c < 4; c++)
      if (row + c < P.m) cp[c] = P.beta != 0.f ? P.alpha * s[c] + P.beta * cp[c] : P.alpha * s[c];
  }
}

// C = alpha * (sum over K slices, in slice order) + beta * C.  VEC: four rows of a column per thread (m a multiple
// of 4, the result 16-byte aligned).  Four slices are requested before the first is added.
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce(GemmParams P) {
  typedef typename std::conditional<VEC, f4, float>::type T;
  constexpr int W = VEC ? 4 : 1;
  const size_t total = (size_t)P.m * P.n / W;   // in units of T
  const T *work = (const T *)P.work;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
    T s = work[e];
    int k = 1;
    for (; k + 3 < P.ksplit; k += 4) {
      const T a = work[(size_t)k * total + e], b = work[(size_t)(k + 1) * total + e], c = work[(size_t)(k + 2) * total + e],
              d = work[(size_t)(k + 3) * total + e];
      s += a;
      s += b;
      s += c;
      s += d;
    }
    for (; k < P.ksplit; k++) s += work[(size_t)k * total + e];
    const size_t col = e * W / P.m, row = e * W - col * P.m;
    T *cp = (T *)(P.c + col * P.ldc + row);
    T v = P.alpha * s;
    if (P.beta != 0.f) v += P.beta * *cp;
    *cp = v;
  }
}

// K = 0: the product is empty and the operands may not exist
__global__ __launch_bounds__(256) void scale_result(GemmParams P) {
  const size_t total = (size_t)P.m * P.n;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
    const size_t col = e / P.m, row = e - col * P.m;
    float *cp = P.c + col * P.ldc + row;
    *cp = P.beta != 0.f ? P.beta * *cp : 0.f;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Products with one short side (n <= 64 here, i.e. a row-major result of at most 64 rows) and a long operand that
// is contiguous along m.  The tiled kernel above spends a third of such a product between its multiply phases (LDS
// store, barrier, fragment reads of both operands every 16 k) and needs a second kernel to add its K slices.  Here
// the long operand never touches LDS: a lane loads four adjacent m-values of one k row straight into registers,
// lanes 0-31 from row k and lanes 32-63 from row k + 1, which is the layout the MFMA wants for its second operand
// when value c of the load is fed to the MFMA that computes result columns 4 j + c.  The MFMA computes the result
// transposed (rows = the short side), so a lane ends up with four adjacent m-values of one n: 16-byte stores.
//   A block of four waves (one per SIMD: the accumulators alone take 128 registers) owns 128 values of m; the
//   waves split the block's K range between them, each streaming its own rows, and meet once at the end, where
//   their accumulators are added through LDS in wave order.  The grid slices K as well (blockIdx.y) until about
//   every CU has a block.  Two slices are folded in the same launch: a block writes its sums through to device
//   scope, waits for the stores' acknowledgement and takes a ticket of its column block; the second arrival adds
//   the first one's sums to its own (the sum of two numbers does not depend on their order, so a product gives
//   the same bits every time) and writes the result.  More slices go to `work` and are added in slice order by
//   splitk_reduce.
//   The short operand is small and stays in L2.  Stored in rows of n, a lane's fragments of a k-pair are 4 or 8
//   adjacent bytes of memory and are loaded as such, through a second ring of registers beside the long
//   operand's: nothing passes through LDS and the K loop holds, per pair, eight MFMAs, two loads and scalar
//   address arithmetic.  Stored in rows of k, chunks of 32 k pass through LDS to be transposed, each wave staging
//   the rows of its own K range in a buffer of its own: there is no barrier inside the K loop either way.
//   A wave requests 16 k-pairs (one chunk) ahead through rings of registers whose slots are fixed at compile time.
//   All loads are buffer loads: descriptor base + the lane's constant 32-bit offset + a scalar offset per pair
//   (no vector instruction for addresses: beside an MFMA every vector instruction costs the matrix pipe several
//   cycles, scalar ones none), and what lies beyond a wave's rows reads as zero, so the rings run past the end
//   of a range without clamping.
// Needs: k even (a multiple of 4 when the short operand is contiguous along k), m a multiple of 4, the long
// operand, the result and the workspace 16-byte aligned with leading dimensions that are multiples of 4; the short
// operand in whole aligned 16-byte groups along its contiguous dim; a wave's rows of the long operand and the
// short operand within 4 GiB of their first byte.
constexpr int ST_CW = 128;      // values of m per block
constexpr int ST_WAVES = 4;
constexpr int ST_CK = 32;       // k per chunk
constexpr int ST_PAIRS = ST_CK / 2;   // k-pairs per chunk = pairs in flight per wave

struct StreamFold {
  unsigned *ticket;   // one arrival counter per column block, zero between launches; null: no fold in the launch
};

__device__ __forceinline__ void st_store_shared(float *p, f4 v) {   // through to device scope, 8 bytes at a time
  unsigned long long lo = (unsigned long long)__float_as_uint(v[0]) | ((unsigned long long)__float_as_uint(v[1]) << 32);
  unsigned long long hi = (unsigned long long)__float_as_uint(v[2]) | ((unsigned long long)__float_as_uint(v[3]) << 32);
  __hip_atomic_store((unsigned long long *)p, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store((unsigned long long *)p + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f4 st_load_fresh(const float *p) {       // past the caches
  const unsigned long long lo = __atomic_load_n((const unsigned long long *)p, __ATOMIC_RELAXED);
  const unsigned long long hi = __atomic_load_n((const unsigned long long *)p + 1, __ATOMIC_RELAXED);
  return f4{__uint_as_float((unsigned)lo), __uint_as_float((unsigned)(lo >> 32)), __uint_as_float((unsigned)hi),
            __uint_as_float((unsigned)(hi >> 32))};
}

template <int NT, bool SKC>
__global__ __launch_bounds__(64 * ST_WAVES) void sgemm_stream(GemmParams P, StreamFold F) {
  constexpr int VW = ST_CW / 32;          // m-values per lane and load
  constexpr int SP = 32 * NT;             // n-values per k row
  constexpr int PAIRS = ST_PAIRS;
  constexpr int SV = ST_CK * SP / 4 / 64; // rows of k: 16-byte groups of a chunk per lane
  constexpr int STAGE = SKC ? ST_WAVES * ST_CK * SP : 0, RED = ST_WAVES * SP * ST_CW;
  typedef float VT __attribute__((ext_vector_type(VW)));
  typedef float FT __attribute__((ext_vector_type(NT)));
  __shared__ __attribute__((aligned(16))) float lds[STAGE > RED ? STAGE : RED];
  __shared__ unsigned s_last;

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same for the whole wave: what follows from it stays in scalar registers
  const int kb = blockIdx.y * P.kchunk;
  const int ke = (kb + P.kchunk < P.k) ? (kb + P.kchunk) : P.k;
  // the wave's own K range: a multiple of the chunk, the last one takes what is left
  const int kw = ((ke - kb + ST_WAVES - 1) / ST_WAVES + ST_CK - 1) / ST_CK * ST_CK;
  const int k_begin = (kb + wave * kw < ke) ? kb + wave * kw : ke;
  const int k_end = (k_begin + kw < ke) ? k_begin + kw : ke;
  const int np = (k_end - k_begin) >> 1;           // k-pairs of this wave
  const int nchunks = (np + PAIRS - 1) / PAIRS;

  const int col = blockIdx.x * ST_CW + VW * l32;
  const int col_c = col + VW <= P.m ? col : P.m - VW;     // m is a multiple of VW: a lane's group is inside or outside
  // long operand: the wave's rows behind one descriptor; a lane's offset is its row parity and column, a pair's
  // the same for the whole wave
  const __amdgpu_buffer_rsrc_t a_rows = st_buffer(P.a + (size_t)k_begin * P.lda, (unsigned long long)(k_end - k_begin) * P.lda * 4ull);
  const unsigned a_lane = ((unsigned)h * (unsigned)P.lda + (unsigned)col_c) * 4u;
  const unsigned a_pair = 8u * (unsigned)P.lda;
  auto a_fetch = [&](int p) { return st_buffer_load<VW, true>(a_rows, a_lane, (unsigned)p * a_pair); };

  f16v acc[NT][VW];
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int c = 0; c < VW; c++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[t][c][r] = 0.f;

  // MFMA tile t takes the rows n = NT * i + t of the short side (i = the MFMA's own row index), so a lane's NT
  // fragments of one k are neighbours in memory and in LDS and arrive with one access.
  //
  // Short operand in rows of n (SKC false): a lane's fragments of a pair come straight from memory (the operand is
  // small and stays in L2), through a second ring that runs beside the long operand's.  Values of n at or beyond
  // P.n read the row's pitch or the next row: they only reach accumulator rows that are never stored.
  const __amdgpu_buffer_rsrc_t s_rows = st_buffer(SKC ? P.b : P.b + (size_t)k_begin * P.ldb,
                                                  SKC ? (unsigned long long)P.n * P.ldb * 4ull : (unsigned long long)(k_end - k_begin) * P.ldb * 4ull);
  const unsigned s_pair = 8u * (unsigned)P.ldb;
  const unsigned s_frag_lane = ((unsigned)h * (unsigned)P.ldb + (unsigned)(NT * l32)) * 4u;
  auto s_frag = [&](int p) { return st_buffer_load<NT, false>(s_rows, s_frag_lane, (unsigned)p * s_pair); };
  // Short operand in rows of k (SKC true): chunks of 32 k pass through LDS to be transposed, each wave staging the
  // rows of its own range in a buffer of its own (LDS serves a wave's accesses in order: no barrier, one buffer).
  // Group i of lane l: n = l % SP, k group l / SP + (64/SP) i.
  float *stage = lds + wave * (ST_CK * SP);
  f4 sreg[SKC ? SV : 1];
  const int s_row = lane / SP, s_col = lane % SP;
  const unsigned s_stage_lane = ((unsigned)s_col * (unsigned)P.ldb + 4u * s_row + (unsigned)k_begin) * 4u;
  auto s_fetch = [&](int ch) {
#pragma unroll
    for (int i = 0; i < (SKC ? SV : 0); i++)
      sreg[i] = st_buffer_load<4, false>(s_rows, s_stage_lane, (unsigned)(ch * ST_CK + 4 * (64 / SP) * i) * 4u);
  };
  auto s_store = [&]() {
#pragma unroll
    for (int i = 0; i < (SKC ? SV : 0); i++) {
      const int kq = s_row + (64 / SP) * i;
#pragma unroll
      for (int c = 0; c < 4; c++) stage[(4 * kq + c) * SP + s_col] = sreg[i][c];
    }
  };
  const float *S = stage + h * SP + NT * l32;

  // The rings fill in slot order: the wait counts the compiler derives for the loop below follow the later of the
  // positions a slot's load has here and in the loop, so a reordered fill would make the loop wait for loads it
  // does not need yet.
  VT ring[PAIRS];
  FT sring[SKC ? 1 : PAIRS];
  if constexpr (SKC) s_fetch(0);
#pragma unroll
  for (int i = 0; i < PAIRS; i++) {
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!SKC) sring[i] = s_frag(i);
    ring[i] = a_fetch(i);
  }
  __builtin_amdgcn_sched_barrier(0);
  FT fa[2], fn[2];
  if constexpr (SKC) {
    s_store();
    fa[0] = *(const FT *)S;
    fa[1] = *(const FT *)(S + 2 * SP);
  }

  // One chunk of 16 k-pairs.  Per pair: its MFMAs run, then the slots they emptied are refilled with the same pair
  // of the next chunk (beyond the wave's range the descriptors deliver zeros).  The scheduling barriers keep that
  // order: left alone the compiler gathers the refills into batches at the end of the chunk, where they no longer
  // run a chunk ahead.  Rows of k: the next chunk is requested at the top, and in front of the chunk's last two
  // pairs, whose fragments are already in registers, it replaces the staged chunk and its first fragments are
  // requested, all behind those pairs' MFMAs.
  auto chunk = [&](auto full, int ch) {
    const int p0 = ch * PAIRS;
    if constexpr (SKC) s_fetch(ch + 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pp = 0; pp < PAIRS; pp += 2) {
      if constexpr (SKC) {
        if (pp + 2 == PAIRS) s_store();
        fn[0] = *(const FT *)(S + (pp + 2 < PAIRS ? 2 * (pp + 2) * SP : 0));
        fn[1] = *(const FT *)(S + (pp + 2 < PAIRS ? 2 * (pp + 3) * SP : 2 * SP));
      }
#pragma unroll
      for (int q = 0; q < 2; q++) {
        // a range's last chunk may be short (the test is the same for the whole wave); the loads go on regardless
        if (decltype(full)::value || p0 + pp + q < np) {
          const VT v = ring[pp + q];
          FT f;
          if constexpr (SKC) f = fa[q];
          else f = sring[pp + q];
#pragma unroll
          for (int c = 0; c < VW; c++)
#pragma unroll
            for (int t = 0; t < NT; t++) acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(f[t], v[c], acc[t][c], 0, 0, 0);
        }
        if constexpr (!SKC) sring[pp + q] = s_frag(p0 + pp + q + PAIRS);
        ring[pp + q] = a_fetch(p0 + pp + q + PAIRS);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (SKC) {
        fa[0] = fn[0];
        fa[1] = fn[1];
      }
    }
  };
  const int nfull = np / PAIRS;
  int ch = 0;
  for (; ch < nfull; ch++) chunk(std::true_type{}, ch);
  if (ch < nchunks) chunk(std::false_type{}, ch);

  // acc[t][c][r] = C[m = col + c][n = NT (8 (r / 4) + 4 h + r % 4) + t]: the waves' parts meet in LDS as
  // [wave][n][m] and are added in wave order
  __syncthreads();
  float *red = lds + wave * (SP * ST_CW);
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int nn = NT * (8 * (r / 4) + 4 * h + r % 4) + t;
      VT v;
#pragma unroll
      for (int c = 0; c < VW; c++) v[c] = acc[t][c][r];
      *(VT *)(red + nn * ST_CW + VW * l32) = v;
    }
  __syncthreads();
  constexpr int GROUPS = SP * ST_CW / 4 / (64 * ST_WAVES);   // 16-byte groups of the block's result per thread
  f4 sum[GROUPS];
#pragma unroll
  for (int i = 0; i < GROUPS; i++) {
    const int g = tid + 64 * ST_WAVES * i;
    const int nn = g / (ST_CW / 4), c4 = g % (ST_CW / 4);
    sum[i] = *(const f4 *)(lds + nn * ST_CW + 4 * c4);
#pragma unroll
    for (int w = 1; w < ST_WAVES; w++) sum[i] += *(const f4 *)(lds + w * (SP * ST_CW) + nn * ST_CW + 4 * c4);
  }
  auto finish = [&](auto op) {   // op(i, nn, mcol) for the thread's groups inside the result
#pragma unroll
    for (int i = 0; i < GROUPS; i++) {
      const int g = tid + 64 * ST_WAVES * i;
      const int nn = g / (ST_CW / 4), mcol = blockIdx.x * ST_CW + 4 * (g % (ST_CW / 4));
      if (nn < P.n && mcol < P.m) op(i, nn, mcol);
    }
  };
  auto write_result = [&](int i, int nn, int mcol) {
    f4 *cp = (f4 *)(P.c + (size_t)nn * P.ldc + mcol);
    f4 v = P.alpha * sum[i];
    if (P.beta != 0.f) v += P.beta * *cp;
    *cp = v;
  };
  if (P.ksplit == 1) {
    finish(write_result);
    return;
  }
  if (F.ticket == nullptr) {   // more than two slices: splitk_reduce adds them in slice order
    finish([&](int i, int nn, int mcol) { *(f4 *)(P.work + ((size_t)blockIdx.y * P.n + nn) * P.m + mcol) = sum[i]; });
    return;
  }
  // Two slices.  The sums go through to where all XCDs meet (device-scope stores leave nothing dirty in this
  // XCD's L2); every wave waits for its stores' acknowledgement, the block meets, and one lane takes the column
  // block's ticket.  Whoever draws the second ticket knows that the other block's stores were acknowledged before
  // its ticket, reads them with loads that bypass the caches, and finishes the result.
  finish([&](int i, int nn, int mcol) { st_store_shared(P.work + ((size_t)blockIdx.y * P.n + nn) * P.m + mcol, sum[i]); });
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) s_last = atomicAdd(F.ticket + blockIdx.x, 1u) == 1u ? 1u : 0u;
  __syncthreads();
  if (!s_last) return;
  finish([&](int i, int nn, int mcol) {
    sum[i] += st_load_fresh(P.work + ((size_t)(1 - blockIdx.y) * P.n + nn) * P.m + mcol);
    write_result(i, nn, mcol);
  });
  if (tid == 0) F.ticket[blockIdx.x] = 0u;
}

template <int BM, int BN, int EDGE>
void launch_tt(bool ta, bool tb, dim3 grid, hipStream_t s, const GemmParams &P) {
  dim3 block(256);
  if (!ta && !tb) hipLaunchKernelGGL((sgemm_mfma<BM, BN, false, false, EDGE>), grid, block, 0, s, P);
  else if (ta && !tb) hipLaunchKernelGGL((sgemm_mfma<BM, BN, true, false, EDGE>), grid, block, 0, s, P);
  else if (!ta && tb) hipLaunchKernelGGL((sgemm_mfma<BM, BN, false, true, EDGE>), grid, block, 0, s, P);
  else hipLaunchKernelGGL((sgemm_mfma<BM, BN, true, true, EDGE>), grid, block, 0, s, P);
}

bool al16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
}  // namespace

// Few tiles and a long K: slice K over blockIdx.y so every CU has work; the slices'
// partial products are summed in slice order by a second kernel.  Below one tile per
// CU any K from 1024 up is sliced (from 512 up below half a tile per CU); between one and two tiles per CU only
// K >= 2048 (512x2048x4096: 96 -> 108 TFLOP/s, while 1024^3 loses 10 % when sliced).
static void choose_ksplit(long tiles, long k, int cus, int &ksplit, int &kchunk) {
  ksplit = 1;
  kchunk = (int)(k > 0 ? k : 0);
  if (!((tiles < cus && k >= 1024) || (tiles < 2L * cus && k >= 2048) || (2 * tiles <= cus && k >= 512))) return;
  long want = (2L * cus + tiles - 1) / tiles;
  long max_by_k = k / 256;  // at least 16 slabs per slice,
  if (tiles * max_by_k < cus) max_by_k = k / 128;  // 8 when that leaves CUs without a block (512^3: 13.2 -> 10.1 us)
  if (want > max_by_k) want = max_by_k;
  if (want > 512) want = 512;  // want * tiles stays near 2 * cus, so the partials stay near 2 * cus tiles
  if (want <= 1) return;
  const long chunk = ((k + want - 1) / want + BK - 1) / BK * BK;
  const long slices = (k + chunk - 1) / chunk;
  if (slices > 1) {
    ksplit = (int)slices;
    kchunk = (int)chunk;
  }
}
// Several tiles per CU, but not a whole number of them: the tiles beyond the last multiple of the CUs would occupy
// some CUs for a whole tile time while the others idle (3072^3 in 128 x 128 tiles: 576 tiles on 256 CUs, 2.25 tile
// times of work in a launch that takes close to 3).  When they are at most half the CUs, each of them is shared by
// `split` blocks along K, so that the tail takes 1 / split of a tile time on all CUs, at the price of a pass over
// those tiles' partial sums.
static bool plan_tail(long tiles, long k, int cus, int &whole, int &split, int &chunk) {
  const long q = tiles / cus, r = tiles % cus;
  if (q < 1 || r == 0 || 2 * r > cus) return false;
  long s = cus / r;
  if (s > k / 256) s = k / 256;   // at least 16 slabs a slice
  if (s > 16) s = 16;
  if (s < 2) return false;
  const long c = ((k + s - 1) / s + BK - 1) / BK * BK;
  whole = (int)(q * cus);
  split = (int)((k + c - 1) / c);
  chunk = (int)c;
  return split >= 2;
}
// Tile choice by a small model of the launch, fitted to measurements on 256 CUs (cubes of 1024 to 6144 and ragged
// shapes, predicted within a few percent):
//   rate     what the tile's kernel sustains on a large product, in TFLOP/s: whole tiles / tiles with edges
//   balance  a CU works through whole tiles, so the launch takes ceil(tiles / CUs) tile times, or, when the last
//            tiles share their K (plan_tail), the whole rounds plus that share of one
//   useful   the part of the tiles' area that lies inside the matrix
//   fill     one or two blocks on a CU do not keep its matrix pipes busy
//   start    a block's first loads and its epilogue cost about as much as 8 of its K slabs, 12 for the largest tile
//            (whose CU holds few other blocks to work meanwhile; 4096 x 4096 x 256: 92 TFLOP/s in 128 x 128 tiles,
//            109 in 128 x 64)
// Products with few tiles are sliced along K as well (choose_ksplit), which fills the chip at the price of a
// second pass over the result.
static void choose_tile(long m, long n, long k, int cus, bool aligned, int &bm, int &bn) {
  struct Cand {
    int bm, bn;
    double whole, edge;
    int resident;  // blocks a CU holds
    double start;  // what a block's first loads and its epilogue cost, in K slabs
  };
  // the two thin tiles only stand for products with a side of at most 32, where they halve the padding
  static const Cand cands[6] = {{128, 128, 147., 140., 3, 12.}, {128, 64, 131., 133., 5, 8.}, {64, 128, 139., 133., 5, 8.},
                                {64, 64, 127., 127., 8, 8.},    {128, 32, 115., 110., 8, 8.}, {32, 128, 115., 110., 8, 8.}};
  double best = -1.;
  bm = bn = 64;
  for (const Cand &c : cands) {
    if ((c.bm == 128 && m < 128) || (c.bn == 128 && n < 128)) continue;
    if ((c.bn == 32 && n > 32) || (c.bm == 32 && m > 32)) continue;
    if ((n <= 32 && m >= 1024 && c.bn != 32) || (m <= 32 && n >= 1024 && c.bm != 32)) continue;   // measured: the thin tile wins there
    const long tm = (m + c.bm - 1) / c.bm, tn = (n + c.bn - 1) / c.bn, tiles = tm * tn;
    const bool whole = aligned && m % c.bm == 0 && n % c.bn == 0;
    int ks, kc;
    choose_ksplit(tiles, k, cus, ks, kc);
    const long blocks = tiles * ks, rounds = (blocks + cus - 1) / cus;
    double balance = (double)blocks / (double)(rounds * cus);
    int tw, tsp, tch;
    if (ks == 1 && plan_tail(tiles, k, cus, tw, tsp, tch)) balance = ((double)tiles / cus) / ((double)(tiles / cus) + 1.0 / tsp + 0.05);
    const double useful = ((double)m * (double)n) / ((double)(tm * c.bm) * (double)(tn * c.bn));
    const long held = rounds < c.resident ? rounds : c.resident;
    const double fill = held >= 3 ? 1.0 : held == 2 ? 0.9 : 0.75;
    const double slabs = (double)((kc + BK - 1) / BK), start = slabs / (slabs + c.start);
    const double score = (whole ? c.whole : c.edge) * balance * useful * fill * start * (ks > 1 ? 0.93 : 1.0);
    if (score > best) {
      best = score;
      bm = c.bm;
      bn = c.bn;
    }
  }
}
// The streaming kernel's launch for a product with n <= 64: a block per 128 values of m, and K sliced over the grid
// as well while that leaves CUs without a block; a slice is a multiple of 128 k (32 k for each of a block's waves).
static void plan_stream(long m, long k, int cus, int &ksplit, int &kchunk) {
  const long bx = (m + ST_CW - 1) / ST_CW;
  long want = cus / bx;
  if (want > k / 256) want = k / 256;
  if (want < 1) want = 1;
  const long per = ST_WAVES * ST_CK;
  const long chunk = ((k + want - 1) / want + per - 1) / per * per;
  kchunk = (int)chunk;
  ksplit = (int)((k + chunk - 1) / chunk);
}

static void launch_stream(bool skc, int nt, dim3 grid, hipStream_t s, const GemmParams &P, const StreamFold &F) {
  dim3 block(64 * ST_WAVES);
  if (nt == 1 && skc) hipLaunchKernelGGL((sgemm_stream<1, true>), grid, block, 0, s, P, F);
  else if (nt == 1) hipLaunchKernelGGL((sgemm_stream<1, false>), grid, block, 0, s, P, F);
  else if (skc) hipLaunchKernelGGL((sgemm_stream<2, true>), grid, block, 0, s, P, F);
  else hipLaunchKernelGGL((sgemm_stream<2, false>), grid, block, 0, s, P, F);
}

// the block tile and the K slicing a product of this shape gets on a chip with `cus` compute units
void thcl_gemm_plan(long m, long n, long k, int cus, int *bm, int *bn, int *ksplit, int *kchunk, int *tail_tiles, int *tail_split) {
  choose_tile(m, n, k, cus, k % BK == 0, *bm, *bn);
  const long tiles = ((m + *bm - 1) / *bm) * ((n + *bn - 1) / *bn);
  choose_ksplit(tiles, k, cus, *ksplit, *kchunk);
  int whole = 0, chunk = 0;
  *tail_tiles = 0;
  *tail_split = 1;
  if (*ksplit == 1 && plan_tail(tiles, k, cus, whole, *tail_split, chunk)) *tail_tiles = (int)(tiles - whole);
  else *tail_split = 1;
}

void thcl_sgemm(THClState *state, thcl_rt *rt, char transa, char transb, long m, long n, long k, float alpha,
                const float *a, long lda, const float *b, long ldb, float beta, float *c, long ldc) {
  const bool ta = (transa == 't' || transa == 'T'), tb = (transb == 't' || transb == 'T');
  THCL_CHECK(ta || transa == 'n' || transa == 'N', "gemm: transa must be 'n' or 't'");
  THCL_CHECK(tb || transb == 'n' || transb == 'N', "gemm: transb must be 'n' or 't'");
  THCL_CHECK(m <= INT32_MAX && n <= INT32_MAX && k <= INT32_MAX && lda <= INT32_MAX && ldb <= INT32_MAX &&
                 ldc <= INT32_MAX,
             "gemm only supports m, n, k, lda, ldb, ldc with the bound [val] <= %d", INT32_MAX);
  if (m <= 0 || n <= 0) return;
  hipStream_t stream = (hipStream_t)thcl_rt_stream(rt);
  GemmParams P;
  memset(&P, 0, sizeof(P));
  P.a = a;
  P.b = b;
  P.c = c;
  P.m = (int)m;
  P.n = (int)n;
  P.k = (int)(k > 0 ? k : 0);
  P.lda = (int)lda;
  P.ldb = (int)ldb;
  P.ldc = (int)ldc;
  P.alpha = alpha;
  P.beta = beta;
  if (P.k == 0) {
    const size_t total = (size_t)m * n;
    hipLaunchKernelGGL(scale_result, dim3((unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256)), dim3(256), 0, stream, P);
    hipError_t e0 = hipGetLastError();
    THCL_CHECK(e0 == hipSuccess, "gemm launch failed: %s", hipGetErrorString(e0));
    thcl_after_launch(state, rt);
    return;
  }
  const int cus = thcl_rt_get_props(rt)->compute_units;
  // one short side and a long operand contiguous along m: the long operand streams from memory into the matrix cores
  const bool b_groups = tb ? (n % 4 == 0) : (k % 4 == 0);
  bool stream_fits = false;
  if (!ta && n <= 64 && m >= 2048 && k >= 512 && k % 2 == 0 && m % 4 == 0 && lda % 4 == 0 && ldc % 4 == 0 && al16(a) && al16(c) &&
      ldb % 4 == 0 && al16(b) && b_groups) {
    plan_stream(m, k, cus, P.ksplit, P.kchunk);
    // the kernel's buffer descriptors address a wave's rows of the long operand, and the short operand, with 32-bit
    // byte offsets (a wave's range is at most a slice long, and reads a chunk past it)
    stream_fits = ((long)P.kchunk + 2 * ST_CK) * lda < (1L << 30) && (tb ? (long)P.kchunk + 2 * ST_CK : n) * ldb < (1L << 30);
  }
  if (stream_fits) {
    if (P.ksplit > 1) {
      P.work = (float *)thcl_rt_workspace(rt, (size_t)P.ksplit * m * n * sizeof(float));
      THCL_CHECK(P.work != nullptr, "gemm workspace: %s", thcl_rt_error());
    }
    dim3 grid((unsigned)((m + ST_CW - 1) / ST_CW), (unsigned)P.ksplit);
    // two slices are folded inside the launch; the tickets are the column-tile counters of the context's scratch
    // block (uint32 [64, 4096), zero between launches; launches of one context run in order)
    StreamFold F{nullptr};
    if (P.ksplit == 2 && grid.x <= 4096 - 64) F.ticket = (unsigned *)thcl_rt_scratch(rt, nullptr) + 64;
    launch_stream(!tb, n <= 32 ? 1 : 2, grid, stream, P, F);
    if (P.ksplit > 1 && !F.ticket) {
      const size_t total = (size_t)m * n / 4;
      unsigned rg = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
      hipLaunchKernelGGL(splitk_reduce<true>, dim3(rg), dim3(256), 0, stream, P);
    }
    hipError_t e1 = hipGetLastError();
    THCL_CHECK(e1 == hipSuccess, "gemm launch failed: %s", hipGetErrorString(e1));
    thcl_after_launch(state, rt);
    return;
  }
  int bm, bn;
  const bool aligned = (k % BK == 0) && k > 0 && (lda % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0) && al16(a) && al16(b) && al16(c);
  choose_tile(m, n, k, thcl_rt_get_props(rt)->compute_units, aligned, bm, bn);
  // an operand's contiguous dim is m for a 'n', k for a 't'; n for b 't', k for b 'n'
  const long a_run = ta ? k : m, b_run = tb ? n : k;
  // the descriptor kernels address a slab of a tile with 32-bit byte offsets: 128 rows of either operand
  const bool short_pitch = lda < (1L << 22) && ldb < (1L << 22);
  // longer pitches with fewer than 4 elements along an operand's contiguous dim: one element at a time, one tile shape
  const bool by_element = !short_pitch && (a_run < 4 || b_run < 4);
  if (by_element) bm = bn = 64;
  const bool fast = aligned && (m % bm == 0) && (n % bn == 0) && short_pitch;
  P.tiles_m = (int)((m + bm - 1) / bm);
  P.tiles_n = (int)((n + bn - 1) / bn);
  P.group_m = P.tiles_m < 8 ? P.tiles_m : 8;
  choose_ksplit((long)P.tiles_m * P.tiles_n, k, thcl_rt_get_props(rt)->compute_units, P.ksplit, P.kchunk);
  if (P.ksplit > 1) {
    P.work = (float *)thcl_rt_workspace(rt, (size_t)P.ksplit * m * n * sizeof(float));
    THCL_CHECK(P.work != nullptr, "gemm workspace: %s", thcl_rt_error());
  }
  P.whole_tiles = P.tiles_m * P.tiles_n;
  P.tail_split = 1;
  if (P.ksplit == 1) {
    int whole, split, chunk;
    if (plan_tail((long)P.tiles_m * P.tiles_n, k, cus, whole, split, chunk)) {
      P.tail_tiles = P.whole_tiles - whole;
      P.whole_tiles = whole;
      P.tail_split = split;
      P.tail_kchunk = chunk;
      P.work = (float *)thcl_rt_workspace(rt, (size_t)split * P.tail_tiles * bm * bn * sizeof(float));
      THCL_CHECK(P.work != nullptr, "gemm workspace: %s", thcl_rt_error());
    }
  }
  dim3 grid((unsigned)(P.whole_tiles + P.tail_tiles * P.tail_split), (unsigned)P.ksplit);
#define GO(BM_, BN_)                                                   \
  if (fast) launch_tt<BM_, BN_, 0>(ta, tb, grid, stream, P);                        \
  else if (short_pitch) launch_tt<BM_, BN_, 1>(ta, tb, grid, stream, P);            \
  else launch_tt<BM_, BN_, 2>(ta, tb, grid, stream, P);
  if (by_element) launch_tt<64, 64, 3>(ta, tb, grid, stream, P);
  else if (bm == 128 && bn == 128) { GO(128, 128) }
  else if (bm == 128 && bn == 64) { GO(128, 64) }
  else if (bm == 64 && bn == 128) { GO(64, 128) }
  else if (bm == 128 && bn == 32) { GO(128, 32) }
  else if (bm == 32 && bn == 128) { GO(32, 128) }
  else { GO(64, 64) }
#undef GO
  if (P.tail_tiles > 0) {
    const bool vec = m % 4 == 0 && ldc % 4 == 0 && al16(c);
    const unsigned rg = (unsigned)(((size_t)P.tail_tiles * bm * bn / 4 + 255) / 256);
#define GO(BM_, BN_)                                                                                        \
  if (bm == BM_ && bn == BN_) {                                                                             \
    if (vec) hipLaunchKernelGGL((tail_reduce<BM_, BN_, true>), dim3(rg), dim3(256), 0, stream, P);          \
    else hipLaunchKernelGGL((tail_reduce<BM_, BN_, false>), dim3(rg), dim3(256), 0, stream, P);             \
  }
    GO(128, 128) GO(128, 64) GO(64, 128) GO(64, 64) GO(128, 32) GO(32, 128)
#undef GO
  }
  if (P.ksplit > 1) {
    const bool vec = m % 4 == 0 && ldc % 4 == 0 && al16(c);
    const size_t total = (size_t)m * n / (vec ? 4 : 1);
    unsigned rg = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
    if (vec) hipLaunchKernelGGL(splitk_reduce<true>, dim3(rg), dim3(256), 0, stream, P);
    else hipLaunchKernelGGL(splitk_reduce<false>, dim3(rg), dim3(256), 0, stream, P);
  }
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "gemm launch failed: %s", hipGetErrorString(e));
  thcl_after_launch(state, rt);
}
