/*
 * CPU restatement of the Torch7 `TH` FloatTensor semantics for the hot path
 * (pointwise apply, strided copy, reduce-all, reduce-along-dim, arg max/min,
 * addmm) plus the layout rules the reference applies before launching.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP library is
 * compared against; nothing in the shipped library links, loads or calls it.
 *
 * Compile with:  gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC
 * (contraction must stay off so that `a*b+c` rounds twice, exactly as the
 * device kernels do).
 *
 * Tensor views are passed as (base pointer, element offset, ndim, sizes[],
 * strides[]) with sizes/strides in elements, the layout of a THClTensor
 * (reference: src/lib/THClTensor.h:14-27).
 *
 * Reference lines each function follows are cited at the function.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define TH_MAXDIMS 25

typedef struct {
  float *base;
  long offset;
  int ndim;
  const long *size;
  const long *stride;
} thv;

static long thv_numel(const thv *v) {
  /* reference: src/lib/THClTensor.cpp:580-592 (0-dim tensors count 0 elements) */
  if (v->ndim == 0) return 0;
  long n = 1;
  for (int d = 0; d < v->ndim; d++) n *= v->size[d];
  return n;
}

/* element offset of the i-th element in logical (row-major) order */
static inline long thv_off(const thv *v, long i) {
  long off = v->offset;
  for (int d = v->ndim - 1; d >= 0; d--) {
    long q = i / v->size[d];
    off += (i - q * v->size[d]) * v->stride[d];
    i = q;
  }
  return off;
}

/* Odometer walk: calls BODY with `o0`,`o1`,`o2` element offsets of up to three
 * views that share the element count (not necessarily the shape), in logical
 * order, as TH_TENSOR_APPLY{1,2,3} do. */
typedef struct {
  long idx[TH_MAXDIMS];
  long off;
  const thv *v;
} walker;

static void walker_init(walker *w, const thv *v) {
  memset(w->idx, 0, sizeof(w->idx));
  w->off = v->offset;
  w->v = v;
}
static inline void walker_next(walker *w) {
  const thv *v = w->v;
  for (int d = v->ndim - 1; d >= 0; d--) {
    w->idx[d]++;
    w->off += v->stride[d];
    if (w->idx[d] < v->size[d]) return;
    w->off -= w->idx[d] * v->stride[d];
    w->idx[d] = 0;
  }
}

#define MKV(name, b, o, nd, sz, st) thv name = {b, o, nd, sz, st}

/* ------------------------------------------------------------------ */
/* pointwise                                                           */
/* ------------------------------------------------------------------ */

/* op codes for th_pointwise; arithmetic follows the op strings of
 * src/lib/THClTensorMathPointwise.h:84-140,
 * src/lib/THClTensorMathPairwise.cpp:18-135 and
 * src/lib/THClTensorMath.cpp:26-54 (operand order is kept). */
enum {
  OP_FILL = 0,      /* r = v                         */
  OP_COPY = 1,      /* r = a                         */
  OP_ADD_S = 2,     /* r = a + v                     */
  OP_MUL_S = 3,     /* r = a * v                     */
  OP_DIV_S = 4,     /* r = a / v   (TH divides; cltorch multiplies by 1/v) */
  OP_CADD = 5,      /* r = a + v*b (v==1: r = a + b) */
  OP_CMUL = 6,      /* r = a * b                     */
  OP_CDIV = 7,      /* r = a / b                     */
  OP_CSUB = 8,      /* r = a - v*b (v==1: r = a - b) */
  OP_SUB_S = 9,     /* r = a + (-v)                  */
  OP_MULRECIP_S = 10, /* r = a * (1.0f/v)  -- cltorch's own div(scalar) */
  OP_SQRT = 11,
  OP_NEG = 12,
  OP_ABS = 13,
  OP_CINV = 14,     /* r = 1.0f / a                  */
  OP_ADDCMUL = 15,  /* r = r + v*a*b                 */
  OP_MAP2_C1 = 16,  /* r = sqrt(1000*r*r + a*10 + b*b)   (config 1 expression) */
  OP_MAP_C2 = 17    /* r = 1000*r + a*10                 (config 2 expression) */
};

static inline float pw(int op, float r, float a, float b, float v) {
  switch (op) {
    case OP_FILL: return v;
    case OP_COPY: return a;
    case OP_ADD_S: return a + v;
    case OP_MUL_S: return a * v;
    case OP_DIV_S: return a / v;
    case OP_CADD: return (v == 1.0f) ? (a + b) : (a + v * b);
    case OP_CMUL: return a * b;
    case OP_CDIV: return a / b;
    case OP_CSUB: return (v == 1.0f) ? (a - b) : (a - v * b);
    case OP_SUB_S: return a + (-v);
    case OP_MULRECIP_S: return a * (1.0f / v);
    case OP_SQRT: return sqrtf(a);
    case OP_NEG: return -a;
    case OP_ABS: return fabsf(a);
    case OP_CINV: return 1.0f / a;
    case OP_ADDCMUL: return r + v * a * b;
    case OP_MAP2_C1: return sqrtf(1000 * r * r + a * 10 + b * b);
    case OP_MAP_C2: return 1000 * r + a * 10;
  }
  return NAN;
}

/* r[i] = op(r[i], a[i], b[i], v) over the logical element order of each view.
 * `a`/`b` may be absent (base NULL).  The walk is element-count based like the
 * reference (src/lib/THClApply.cpp:152-159: only nElement must agree). */
int th_pointwise(int op, float v,
                 float *rb, long ro, int rn, const long *rs, const long *rst,
                 float *ab, long ao, int an, const long *as, const long *ast,
                 float *bb, long bo, int bn, const long *bs, const long *bst) {
  MKV(R, rb, ro, rn, rs, rst);
  MKV(A, ab, ao, an, as, ast);
  MKV(B, bb, bo, bn, bs, bst);
  long n = thv_numel(&R);
  if (ab && thv_numel(&A) != n) return -1;
  if (bb && thv_numel(&B) != n) return -1;
  walker wr, wa, wb;
  walker_init(&wr, &R);
  if (ab) walker_init(&wa, &A);
  if (bb) walker_init(&wb, &B);
  for (long i = 0; i < n; i++) {
    float r = rb[wr.off];
    float a = ab ? ab[wa.off] : 0.0f;
    float b = bb ? bb[wb.off] : 0.0f;
    rb[wr.off] = pw(op, r, a, b, v);
    walker_next(&wr);
    if (ab) walker_next(&wa);
    if (bb) walker_next(&wb);
  }
  return 0;
}

/* Contiguous multi-threaded form used only for the timed CPU baseline; TH runs
 * contiguous cadd/cmul/div under `#pragma omp parallel for`. */
void th_pointwise_contig_omp(int op, float v, float *r, const float *a, const float *b, long n) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; i++)
    r[i] = pw(op, r[i], a ? a[i] : 0.0f, b ? b[i] : 0.0f, v);
}

/* ------------------------------------------------------------------ */
/* reduce all                                                          */
/* ------------------------------------------------------------------ */

/* TH sums a float tensor into a double accumulator in element order and the
 * caller narrows the result to float.  Wrapper semantics:
 * src/lib/THClTensorMath.cpp:346-382 (init 0). */
double th_sumall(float *b, long o, int nd, const long *sz, const long *st) {
  MKV(V, b, o, nd, sz, st);
  long n = thv_numel(&V);
  walker w;
  walker_init(&w, &V);
  double acc = 0.0;
  for (long i = 0; i < n; i++) {
    acc += (double)b[w.off];
    walker_next(&w);
  }
  return acc;
}

double th_prodall(float *b, long o, int nd, const long *sz, const long *st) {
  MKV(V, b, o, nd, sz, st);
  long n = thv_numel(&V);
  walker w;
  walker_init(&w, &V);
  double acc = 1.0;
  for (long i = 0; i < n; i++) {
    acc *= (double)b[w.off];
    walker_next(&w);
  }
  return acc;
}

/* TH max/min over all elements: start from element 0, replace when
 * !(value <= cur) (max) / !(value >= cur) (min), stop at the first NaN.
 * Wrapper: src/lib/THClTensorMath.cpp:257-328. */
float th_maxall(float *b, long o, int nd, const long *sz, const long *st) {
  MKV(V, b, o, nd, sz, st);
  long n = thv_numel(&V);
  if (n == 0) return -INFINITY;
  walker w;
  walker_init(&w, &V);
  float cur = b[w.off];
  for (long i = 0; i < n; i++) {
    float x = b[w.off];
    if (!(x <= cur)) {
      cur = x;
      if (isnan(x)) break;
    }
    walker_next(&w);
  }
  return cur;
}

float th_minall(float *b, long o, int nd, const long *sz, const long *st) {
  MKV(V, b, o, nd, sz, st);
  long n = thv_numel(&V);
  if (n == 0) return INFINITY;
  walker w;
  walker_init(&w, &V);
  float cur = b[w.off];
  for (long i = 0; i < n; i++) {
    float x = b[w.off];
    if (!(x >= cur)) {
      cur = x;
      if (isnan(x)) break;
    }
    walker_next(&w);
  }
  return cur;
}

/* ------------------------------------------------------------------ */
/* reduce along a dimension                                            */
/* ------------------------------------------------------------------ */

/* kind: 0 sum, 1 prod, 2 max, 3 min.  `out` has the source's shape with size 1
 * along `dim` (src/lib/THClReduce.cpp:258-262) and is written contiguously.
 * `idx` (may be NULL) receives 1-based positions for max/min, first
 * occurrence on ties, first NaN wins (TH rule); the 1-based convention is the
 * one the reference kernels write (src/lib/THClTensorMathTransformReduce.cl:32,74). */
int th_reduce_dim(int kind, int dim, float *b, long o, int nd, const long *sz, const long *st,
                  float *out, int64_t *idx) {
  if (dim < 0 || dim >= nd) return -1;
  long nslices = 1;
  for (int d = 0; d < nd; d++)
    if (d != dim) nslices *= sz[d];
  long R = sz[dim];
  long ssz[TH_MAXDIMS], sst[TH_MAXDIMS];
  for (int d = 0; d < nd; d++) {
    ssz[d] = (d == dim) ? 1 : sz[d];
    sst[d] = st[d];
  }
  thv S = {b, o, nd, ssz, sst};
  walker w;
  walker_init(&w, &S);
  for (long s = 0; s < nslices; s++) {
    const float *p = b + w.off;
    long rs = st[dim];
    if (kind == 0) {
      double acc = 0.0;
      for (long r = 0; r < R; r++) acc += (double)p[r * rs];
      out[s] = (float)acc;
    } else if (kind == 1) {
      double acc = 1.0;
      for (long r = 0; r < R; r++) acc *= (double)p[r * rs];
      out[s] = (float)acc;
    } else {
      float cur = p[0];
      long ci = 0;
      for (long r = 0; r < R; r++) {
        float x = p[r * rs];
        int take = (kind == 2) ? !(x <= cur) : !(x >= cur);
        if (take) {
          cur = x;
          ci = r;
          if (isnan(x)) break;
        }
      }
      out[s] = cur;
      if (idx) idx[s] = ci + 1;
    }
    walker_next(&w);
  }
  return 0;
}

/* ------------------------------------------------------------------ */
/* addmm                                                               */
/* ------------------------------------------------------------------ */

/* r = beta*t + alpha*(m1 @ m2) with an fp64 accumulator for the contraction
 * and fp64 for the epilogue; argument meaning follows
 * src/lib/THClTensorMathBlas.cpp:107-214.  All operands are 2-d strided views.
 * The result is returned in double so a caller can measure the device's
 * relative error against it. */
int th_addmm_f64(double *r, float beta, const float *t, long t0, long t1, float alpha,
                 const float *m1, long a0, long a1, const float *m2, long b0, long b1,
                 long M, long N, long K) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < M; i++) {
    double *acc = (double *)calloc((size_t)N, sizeof(double));
    for (long k = 0; k < K; k++) {
      double a = (double)m1[i * a0 + k * a1];
      const float *brow = m2 + k * b0;
      for (long j = 0; j < N; j++) acc[j] += a * (double)brow[j * b1];
    }
    for (long j = 0; j < N; j++)
      r[i * N + j] = (double)beta * (double)t[i * t0 + j * t1] + (double)alpha * acc[j];
    free(acc);
  }
  return 0;
}

/* fp64 value of selected entries only (for 8192^3, where the full product is
 * too slow on a CPU): entry e is (rows[e], cols[e]). */
int th_addmm_f64_sampled(double *r, long nsamp, const long *rows, const long *cols, float beta,
                         const float *t, long t0, long t1, float alpha, const float *m1, long a0,
                         long a1, const float *m2, long b0, long b1, long K) {
#pragma omp parallel for schedule(static)
  for (long e = 0; e < nsamp; e++) {
    long i = rows[e], j = cols[e];
    double acc = 0.0;
    for (long k = 0; k < K; k++) acc += (double)m1[i * a0 + k * a1] * (double)m2[k * b0 + j * b1];
    r[e] = (double)beta * (double)t[i * t0 + j * t1] + (double)alpha * acc;
  }
  return 0;
}

/* Plain fp32 blocked gemm, all host threads: the timed CPU baseline for addmm
 * (row-major contiguous operands only). */
void th_addmm_f32_omp(float *c, float beta, float alpha, const float *a, const float *b, long M,
                      long N, long K) {
  const long BK = 256, BJ = 1024;
#pragma omp parallel for schedule(static)
  for (long i = 0; i < M; i++) {
    float *crow = c + i * N;
    for (long j = 0; j < N; j++) crow[j] *= beta;
    for (long jj = 0; jj < N; jj += BJ) {
      long je = jj + BJ < N ? jj + BJ : N;
      for (long kk = 0; kk < K; kk += BK) {
        long ke = kk + BK < K ? kk + BK : K;
        for (long k = kk; k < ke; k++) {
          float av = alpha * a[i * K + k];
          const float *brow = b + k * N;
          for (long j = jj; j < je; j++) crow[j] += av * brow[j];
        }
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* layout rules                                                        */
/* ------------------------------------------------------------------ */

/* Dimension collapse, restated from src/lib/THClReduceApplyUtils.h:67-170:
 * walk inner -> outer, ignore size-1 dims (and `reduce_dim`, which counts as
 * size 1), merge an outer dim into the running inner one when
 * stride_outer == size_inner * stride_inner.  Returns the collapsed dim count;
 * writes collapsed sizes/strides outermost-first. */
int th_collapse(int nd, const long *sz, const long *st, int reduce_dim, long *csz, long *cst) {
  long tsz[TH_MAXDIMS], tst[TH_MAXDIMS];
  int k = 0; /* filled innermost-first */
  for (int d = nd - 1; d >= 0; d--) {
    long s = (d == reduce_dim) ? 1 : sz[d];
    if (s == 1) continue;
    if (k > 0 && st[d] == tsz[k - 1] * tst[k - 1]) {
      tsz[k - 1] *= s;
    } else {
      tsz[k] = s;
      tst[k] = st[d];
      k++;
    }
  }
  if (k == 0) { /* all sizes 1: a single point (reference :96-101) */
    csz[0] = 1;
    cst[0] = 1;
    return 1;
  }
  for (int i = 0; i < k; i++) {
    csz[i] = tsz[k - 1 - i];
    cst[i] = tst[k - 1 - i];
  }
  return k;
}

/* TH's contiguity test (src/lib/THClTensor.cpp:550-565). */
int th_is_contiguous(int nd, const long *sz, const long *st) {
  long z = 1;
  for (int d = nd - 1; d >= 0; d--) {
    if (sz[d] != 1) {
      if (st[d] == z)
        z *= sz[d];
      else
        return 0;
    }
  }
  return 1;
}

/* Overlap test restated from src/lib/THClReduceApplyUtils.cpp:69-121: order
 * the size>1 dims by stride; a view overlaps itself when the smallest stride
 * is < 1 or any stride is smaller than the extent of the next-smaller dim. */
int th_overlapping(int nd, const long *sz, const long *st) {
  long s[TH_MAXDIMS], t[TH_MAXDIMS];
  int k = 0;
  for (int d = 0; d < nd; d++)
    if (sz[d] > 1) {
      s[k] = sz[d];
      t[k] = st[d];
      k++;
    }
  if (k == 0) return 0;
  for (int i = 1; i < k; i++) { /* insertion sort, ascending stride */
    long cs = s[i], ct = t[i];
    int j = i - 1;
    while (j >= 0 && t[j] > ct) {
      s[j + 1] = s[j];
      t[j + 1] = t[j];
      j--;
    }
    s[j + 1] = cs;
    t[j + 1] = ct;
  }
  if (t[0] < 1) return 1;
  for (int i = 1; i < k; i++)
    if (t[i] < s[i - 1] * t[i - 1]) return 1;
  return 0;
}

/* ------------------------------------------------------------------ */
/* seeded inputs: MT19937 (Matsumoto & Nishimura 2002 reference algorithm,   */
/* init_genrand seeding) so "identical seeded inputs" needs no data files.   */
/* ------------------------------------------------------------------ */

typedef struct {
  uint32_t mt[624];
  int mti;
} mt_state;

static void mt_seed(mt_state *s, uint32_t seed) {
  s->mt[0] = seed;
  for (int i = 1; i < 624; i++)
    s->mt[i] = 1812433253u * (s->mt[i - 1] ^ (s->mt[i - 1] >> 30)) + (uint32_t)i;
  s->mti = 624;
}

static uint32_t mt_next(mt_state *s) {
  if (s->mti >= 624) {
    for (int k = 0; k < 624; k++) {
      uint32_t y = (s->mt[k] & 0x80000000u) | (s->mt[(k + 1) % 624] & 0x7fffffffu);
      s->mt[k] = s->mt[(k + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
    }
    s->mti = 0;
  }
  uint32_t y = s->mt[s->mti++];
  y ^= (y >> 11);
  y ^= (y << 7) & 0x9d2c5680u;
  y ^= (y << 15) & 0xefc60000u;
  y ^= (y >> 18);
  return y;
}

void th_mt_raw(uint32_t seed, long n, uint32_t *out) {
  mt_state s;
  mt_seed(&s, seed);
  for (long i = 0; i < n; i++) out[i] = mt_next(&s);
}

/* uniform [lo, hi): float(u32 * 2^-32 * (hi-lo) + lo), computed in double. */
void th_fill_uniform(uint32_t seed, long n, double lo, double hi, float *out) {
  mt_state s;
  mt_seed(&s, seed);
  for (long i = 0; i < n; i++) {
    double u = (double)mt_next(&s) * (1.0 / 4294967296.0);
    float f = (float)(u * (hi - lo) + lo);
    if (f >= (float)hi) f = nextafterf((float)hi, (float)lo); /* keep the interval half-open after rounding */
    out[i] = f;
  }
}

/* normal(mean, std) by Box-Muller on pairs of uniforms in (0,1]. */
void th_fill_normal(uint32_t seed, long n, double mean, double std, float *out) {
  mt_state s;
  mt_seed(&s, seed);
  for (long i = 0; i < n; i += 2) {
    double u1 = ((double)mt_next(&s) + 1.0) * (1.0 / 4294967296.0);
    double u2 = (double)mt_next(&s) * (1.0 / 4294967296.0);
    double r = sqrt(-2.0 * log(u1));
    out[i] = (float)(mean + std * r * cos(6.283185307179586 * u2));
    if (i + 1 < n) out[i + 1] = (float)(mean + std * r * sin(6.283185307179586 * u2));
  }
}

int th_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
