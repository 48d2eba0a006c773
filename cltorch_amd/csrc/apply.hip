// Pointwise apply engine, host side + the ahead-of-time kernels.
//
// Mirrors THClTensor_pointwiseApply (reference: src/lib/THClApply.cpp:145-240):
// element counts must agree, at most 25 dims, a written operand that overlaps
// itself is staged through a dense temporary.  What differs is the planning:
// instead of one kernel shape specialised per (dims...) tuple, a call is
// classified into one of five kernel families (dense 128-bit, dense scalar,
// joint-strided 128-bit, joint-strided scalar, per-operand generic).
#include <hip/hip_runtime.h>

#include <cstring>

#include "apply_kernels.h"
#include "internal.h"

namespace {

enum PlanKind { K_CONTIG_V4 = 0, K_CONTIG_S, K_JOINT_V4, K_JOINT_S, K_GENERIC, K_TILED, K_NONE };
const char *const kKindSuffix[] = {"_contig_v4", "_contig_s", "_joint_v4", "_joint_s", "_generic", "_tiled"};

struct ApplyPlan {
  PlanKind kind = K_NONE;
  unsigned grid = 0;
  thcl_rt *rt = nullptr;
  ThclContigParams c;
  ThclJointParams j;
  ThclGenericParams g;
  ThclTileParams t;
};

constexpr unsigned kMaxGrid = 1u << 23;  // x 256 threads stays below 2^32 work-items; larger inputs loop
long units_per_tile(PlanKind k, int nt) {
  switch (k) {
    case K_CONTIG_V4: return THCL_CONTIG_THREADS_FOR(nt) * THCL_CONTIG_UNROLL;
    case K_CONTIG_S: return THCL_APPLY_THREADS * THCL_CONTIG_S_UNROLL;
    case K_JOINT_V4: return THCL_APPLY_THREADS * THCL_JOINT_V4_UNROLL;
    case K_JOINT_S: return THCL_APPLY_THREADS * THCL_JOINT_S_UNROLL;
    default: return THCL_APPLY_THREADS * THCL_GENERIC_UNROLL;
  }
}


bool aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
bool aligned_vec(const void *p, int nt) { return (((uintptr_t)p) & (THCL_CONTIG_W_FOR(nt) * 4 - 1)) == 0; }

// Fills `plan`; returns false when there is nothing to launch.
// `dry`: classify only (no device context is opened) -- used by the host-side tests.
bool make_plan(THClState *state, const ApplyCall &call, ApplyPlan &plan, bool dry = false) {
  const int n = call.n;
  THClTensor *const *t = call.t;
  const long total = THClTensor_nElement(state, t[0]);
  for (int i = 1; i < n; i++)
    THCL_CHECK(THClTensor_nElement(state, t[i]) == total, "element size mismatch between tensors 1 and %d", i + 1);
  for (int i = 0; i < n; i++)
    THCL_CHECK(t[i]->nDimension <= THCL_MAX_DIMS, "Apply: too many dimensions in tensor %d", i + 1);
  if (total == 0) return false;
  for (int i = 0; i < n; i++)
    THCL_CHECK(t[i]->storage && t[i]->storage->wrapper, "tensor %d has no device storage", i + 1);
  thcl_check_same_device(state, 3, t[0], n > 1 ? t[1] : nullptr, n > 2 ? t[2] : nullptr);
  plan.rt = dry ? nullptr : thcl_ctx(state, t[0]->storage->device);

  float *p[3] = {nullptr, nullptr, nullptr};
  for (int i = 0; i < n; i++) p[i] = thcl_dptr(t[i]);

  bool all_contig = true;
  for (int i = 0; i < n; i++) all_contig = all_contig && THClTensor_isContiguous(state, t[i]);

  JointLayout J;
  if (!all_contig) {
    J = thcl_joint_collapse(n, t);
    if (J.valid && J.dims == 1) {
      bool unit = true;
      for (int i = 0; i < n; i++) unit = unit && J.strides[i][0] == 1;
      if (unit) all_contig = true;  // e.g. identically transposed views of dense tensors
    }
  }

  if (all_contig) {
    bool al = true;
    for (int i = 0; i < n; i++) al = al && aligned_vec(p[i], n);
    plan.kind = al ? K_CONTIG_V4 : K_CONTIG_S;
    ThclContigParams &c = plan.c;
    memset(&c, 0, sizeof(c));
    for (int i = 0; i < 3; i++) c.p[i] = p[i];
    c.pt[0] = call.pt[0];
    c.pt[1] = call.pt[1];
    c.val[0] = call.val[0];
    c.val[1] = call.val[1];
    c.n = (thcl_u64)total;
    const long units = al ? (total / THCL_CONTIG_W_FOR(n)) : total;
    const long upt = units_per_tile(plan.kind, n);
    const long tiles = (units + upt - 1) / upt;
    c.ntiles = (thcl_u64)tiles;
    plan.grid = (unsigned)(tiles < 1 ? 1 : (tiles > kMaxGrid ? kMaxGrid : tiles));
    return true;
  }

  // strided paths index with 32 bits
  THCL_CHECK(total < (1l << 31), THCL_DIM_WARNING);

  bool joint_ok = J.valid && J.dims <= THCL_JOINT_MAX_DIMS;
  if (joint_ok)
    for (int i = 0; i < n && joint_ok; i++)
      for (int d = 0; d < J.dims; d++)
        if (J.strides[i][d] < 0 || J.strides[i][d] >= (1l << 32)) joint_ok = false;

  // transposed inputs meeting a unit-stride destination: tile through LDS
  if (joint_ok && n >= 2 && J.dims >= 2 && J.dims - 2 <= THCL_TILE_MAX_OUTER) {
    const int A = J.dims - 1;
    int B = -1;
    if (J.strides[0][A] == 1 && J.sizes[A] >= 16) {
      for (int i = 1; i < n && B < 0; i++) {
        if (J.strides[i][A] == 1 || J.strides[i][A] == 0) continue;  // dense, or one value repeated along A
        for (int d = A - 1; d >= 0; d--)
          if (J.strides[i][d] == 1 && J.sizes[d] >= 16) {
            B = d;
            break;
          }
      }
    }
    if (B >= 0) {
      ThclTileParams &t = plan.t;
      memset(&t, 0, sizeof(t));
      for (int i = 0; i < 3; i++) t.p[i] = p[i];
      t.pt[0] = call.pt[0];
      t.pt[1] = call.pt[1];
      t.val[0] = call.val[0];
      t.val[1] = call.val[1];
      t.sizeA = (thcl_u32)J.sizes[A];
      t.sizeB = (thcl_u32)J.sizes[B];
      // Tile shape: the one whose edge tiles waste least of the plane; among
      // equals, 64 x 256 when outer dims exist and 128 x 128 for a plain 2-d
      // transpose (both preferences measured on MI355X, 5-20 %).
      const int prefer[THCL_TILE_SHAPES] = {J.dims > 2 ? 1 : 0, J.dims > 2 ? 0 : 1, 2};
      int shape = prefer[0];
      double best = -1.0;
      for (int k = 0; k < THCL_TILE_SHAPES; k++) {
        const int sh = prefer[k];
        const long ta = THCL_TILE_SHAPE_A(sh), tb = THCL_TILE_SHAPE_B(sh);
        const double used = (double)J.sizes[A] / (double)((J.sizes[A] + ta - 1) / ta * ta) * (double)J.sizes[B] /
                            (double)((J.sizes[B] + tb - 1) / tb * tb);
        if (used > best * 1.02) {
          best = used;
          shape = sh;
        }
      }
      t.shape = (thcl_u32)shape;
      const long tileA = THCL_TILE_SHAPE_A(shape), tileB = THCL_TILE_SHAPE_B(shape);
      // The diagonal order pays when rows of the plane start a multiple of
      // 4 KiB apart (power-of-two pitches) and costs a few percent otherwise.
      t.diagonal = 0;
      for (int i = 0; i < n; i++)
        if ((J.strides[i][A] > 1 && J.strides[i][A] % 1024 == 0) || (J.strides[i][B] > 1 && J.strides[i][B] % 1024 == 0))
          t.diagonal = 1;
      const long tilesA = (J.sizes[A] + tileA - 1) / tileA, tilesB = (J.sizes[B] + tileB - 1) / tileB;
      t.tilesA = thcl_make_divisor(tilesA);
      t.tilesB = thcl_make_divisor(tilesB);
      long blocks = tilesA * tilesB;
      for (int i = 0; i < n; i++) {
        t.strideA[i] = (thcl_u32)J.strides[i][A];
        t.strideB[i] = (thcl_u32)J.strides[i][B];
        t.via_lds[i] = (i > 0 && J.strides[i][B] == 1 && J.strides[i][A] != 1) ? 1u : 0u;
      }
      int no = 0;
      for (int d = 0; d < J.dims; d++) {
        if (d == A || d == B) continue;
        t.osize[no] = thcl_make_divisor(J.sizes[d]);
        for (int i = 0; i < n; i++) t.ostride[i][no] = (thcl_u32)J.strides[i][d];
        blocks *= J.sizes[d];
        no++;
      }
      t.nouter = no;
      // 128-bit accesses when every operand allows them.  Measured on MI355X: +50 % with
      // three operands, +15..70 % when edge tiles are partial, +3..7 % on plain 2-d
      // transposes, but -4 % on two-operand planes of full tiles under outer dims,
      // which therefore keep the 32-bit body.
      const bool ragged = (J.sizes[A] % tileA != 0) || (J.sizes[B] % tileB != 0);
      bool v4 = (J.sizes[A] % 4 == 0) && (J.sizes[B] % 4 == 0) && (n >= 3 || ragged || J.dims == 2);
      for (int i = 0; i < n && v4; i++) {
        if ((((uintptr_t)p[i]) & 15u) != 0) v4 = false;
        if (i > 0 && !t.via_lds[i] && J.strides[i][A] != 1) v4 = false;   // repeated along A: scalar kernel
        const int unit = (i > 0 && t.via_lds[i]) ? B : A;   // the one dim this operand walks with stride 1
        for (int d = 0; d < J.dims && v4; d++)
          if (d != unit && J.strides[i][d] % 4 != 0) v4 = false;
      }
      t.vec4 = v4 ? 1u : 0u;
      if (blocks < (1l << 31)) {
        plan.kind = K_TILED;
        plan.grid = (unsigned)blocks;
        return true;
      }
    }
  }

  if (joint_ok) {
    const int last = J.dims - 1;
    bool vec = (J.sizes[last] % 4 == 0);
    for (int i = 0; i < n && vec; i++) {
      // inputs may repeat one value along the innermost dim (stride 0: an expanded vector)
      if (i > 0 && J.strides[i][last] == 0) continue;
      vec = vec && J.strides[i][last] == 1 && aligned16(p[i]);
      for (int d = 0; d < last; d++) vec = vec && (J.strides[i][d] % 4 == 0);
    }
    plan.kind = vec ? K_JOINT_V4 : K_JOINT_S;
    ThclJointParams &j = plan.j;
    memset(&j, 0, sizeof(j));
    for (int i = 0; i < 3; i++) j.p[i] = p[i];
    j.pt[0] = call.pt[0];
    j.pt[1] = call.pt[1];
    j.val[0] = call.val[0];
    j.val[1] = call.val[1];
    j.dims = J.dims;
    const long units = vec ? total / 4 : total;
    j.nunits = (thcl_u32)units;
    for (int d = 0; d < J.dims; d++) {
      long s = J.sizes[d];
      if (vec && d == last) s /= 4;
      j.size[d] = thcl_make_divisor(s);
      for (int i = 0; i < n; i++) j.stride[i][d] = (thcl_u32)J.strides[i][d];
    }
    const long upt = units_per_tile(plan.kind, n);
    const long tiles = (units + upt - 1) / upt;
    j.ntiles = (thcl_u32)tiles;
    plan.grid = (unsigned)(tiles > kMaxGrid ? kMaxGrid : tiles);
    return true;
  }

  plan.kind = K_GENERIC;
  ThclGenericParams &g = plan.g;
  memset(&g, 0, sizeof(g));
  for (int i = 0; i < 3; i++) g.p[i] = p[i];
  g.pt[0] = call.pt[0];
  g.pt[1] = call.pt[1];
  g.val[0] = call.val[0];
  g.val[1] = call.val[1];
  g.n = (thcl_u32)total;
  for (int i = 0; i < n; i++) {
    Layout L = thcl_collapse(t[i]);
    g.op[i].dims = L.dims;
    for (int d = 0; d < L.dims; d++) {
      THCL_CHECK(L.strides[d] >= 0 && L.strides[d] < (1l << 32), THCL_DIM_WARNING);
      g.op[i].size[d] = thcl_make_divisor(L.sizes[d]);
      g.op[i].stride[d] = (thcl_u32)L.strides[d];
    }
  }
  const long upt = units_per_tile(plan.kind, n);
  const long tiles = (total + upt - 1) / upt;
  g.ntiles = (thcl_u32)tiles;
  plan.grid = (unsigned)(tiles > kMaxGrid ? kMaxGrid : tiles);
  return true;
}

// ---------------------------------------------------------- fixed kernels ---
THCL_FIXED_OPS(THCL_DEFINE_OP_STRUCT)
}  // namespace

#define X(name, nt, stmt) THCL_DEFINE_APPLY_KERNELS(thcl_k_##name, Op_##name, nt)
THCL_FIXED_OPS(X)
#undef X

namespace {
typedef ThclKernelSet KernelSet;
const KernelSet kFixed[OP_FIXED_COUNT] = {THCL_FIXED_OPS(THCL_KERNEL_SET_ENTRY)};
const KernelSet &kernel_set(ThclOp op) {
  return op < OP_FIXED_COUNT ? kFixed[op] : thcl_catalogue_kernel_sets()[op - OP_FIXED_COUNT];
}

void launch_fixed(const KernelSet &ks, ApplyPlan &plan) {
  hipStream_t stream = (hipStream_t)thcl_rt_stream(plan.rt);
  dim3 grid(plan.grid), block(THCL_APPLY_THREADS);
  switch (plan.kind) {
    case K_CONTIG_V4: hipLaunchKernelGGL(ks.contig_v4, grid, dim3(THCL_CONTIG_THREADS_FOR(ks.nt)), 0, stream, plan.c); break;
    case K_CONTIG_S: hipLaunchKernelGGL(ks.contig_s, grid, block, 0, stream, plan.c); break;
    case K_JOINT_V4: hipLaunchKernelGGL(ks.joint_v4, grid, block, 0, stream, plan.j); break;
    case K_JOINT_S: hipLaunchKernelGGL(ks.joint_s, grid, block, 0, stream, plan.j); break;
    case K_GENERIC: hipLaunchKernelGGL(ks.generic, grid, block, 0, stream, plan.g); break;
    case K_TILED: hipLaunchKernelGGL(ks.tiled, grid, dim3(THCL_TILE_THREADS), 0, stream, plan.t); break;
    default: return;
  }
  hipError_t e = hipGetLastError();
  THCL_CHECK(e == hipSuccess, "apply kernel launch failed: %s", hipGetErrorString(e));
}

void launch_expr(THClState *state, const std::string &expr, int nt, ApplyPlan &plan) {
  // one module per (expression, kernel family): a first use compiles only what it launches
  std::string key = std::to_string(nt) + "|" + std::to_string((int)plan.kind) + "|" + expr;
  std::string entry = thcl_expr_tag(expr, nt) + kKindSuffix[plan.kind];
  std::string source;
  if (!thcl_rt_kernel_cached(plan.rt, key.c_str())) source = thcl_expr_source(expr, nt, (int)plan.kind);
  thcl_rt_kernel *k = thcl_rt_kernel_get(plan.rt, key.c_str(), source.c_str(), entry.c_str());
  THCL_CHECK(k != nullptr, "%s", thcl_rt_error());
  void *params = nullptr;
  size_t bytes = 0;
  switch (plan.kind) {
    case K_CONTIG_V4:
    case K_CONTIG_S: params = &plan.c; bytes = sizeof(plan.c); break;
    case K_JOINT_V4:
    case K_JOINT_S: params = &plan.j; bytes = sizeof(plan.j); break;
    case K_TILED: params = &plan.t; bytes = sizeof(plan.t); break;
    default: params = &plan.g; bytes = sizeof(plan.g); break;
  }
  const unsigned threads = plan.kind == K_TILED ? THCL_TILE_THREADS
                           : plan.kind == K_CONTIG_V4 ? THCL_CONTIG_THREADS_FOR(nt) : THCL_APPLY_THREADS;
  THCL_CHECK(thcl_rt_launch(plan.rt, k, plan.grid, 1, 1, threads, 1, 1, 0, params, bytes) == 0, "%s",
             thcl_rt_error());
  (void)state;
}

// Runs `body(call)` with operand 0 replaced by a dense temporary when it
// aliases itself, then scatters the temporary back (any writer may win), as
// the reference does (src/lib/THClApply.cpp:183-190,231-237).
template <class F>
void with_overlap_fixup(THClState *state, ApplyCall &call, F body) {
  THClTensor *orig = nullptr;
  if (!call.ignore_overlap && call.t[0]->nDimension > 0 && thcl_overlapping(call.t[0])) {
    orig = call.t[0];
    call.t[0] = THClTensor_newContiguous(state, orig);
  }
  try {
    body(call);
  } catch (...) {
    if (orig) {
      THClTensor_free(state, call.t[0]);
      call.t[0] = orig;
    }
    throw;
  }
  if (orig) {
    ApplyCall back;
    back.n = 2;
    back.t[0] = orig;
    back.t[1] = call.t[0];
    back.ignore_overlap = true;
    thcl_apply_fixed(state, OP_COPY, back);
    THClTensor_free(state, call.t[0]);
    call.t[0] = orig;
  }
}
}  // namespace

// The tunable shape constants this build was compiled with, as #define lines:
// prepended to run-time compiled sources so both kinds of kernels agree with
// the host-side planning.
std::string thcl_apply_config_defines() {
#define THCL_STR2(x) #x
#define THCL_STR(x) THCL_STR2(x)
  return "#define THCL_TILE_UNROLL " THCL_STR(THCL_TILE_UNROLL) "\n"
         "#define THCL_CONTIG_S_UNROLL " THCL_STR(THCL_CONTIG_S_UNROLL) "\n";
#undef THCL_STR
#undef THCL_STR2
}

void thcl_apply_fixed(THClState *state, ThclOp op, ApplyCall &call) {
  THCL_CHECK(op >= 0 && op < OP_COUNT, "unknown operator %d", (int)op);
  const KernelSet &ks = kernel_set(op);
  THCL_CHECK(ks.nt == call.n, "operator %d takes %d tensors, got %d", (int)op, ks.nt, call.n);
  with_overlap_fixup(state, call, [&](ApplyCall &c) {
    ApplyPlan plan;
    if (!make_plan(state, c, plan)) return;
    launch_fixed(ks, plan);
    thcl_after_launch(state, plan.rt);
  });
}

void thcl_apply_expr(THClState *state, const std::string &expr, ApplyCall &call) {
  with_overlap_fixup(state, call, [&](ApplyCall &c) {
    ApplyPlan plan;
    if (!make_plan(state, c, plan)) return;
    launch_expr(state, expr, c.n, plan);
    thcl_after_launch(state, plan.rt);
  });
}

void thcl_fill_contig(thcl_rt *rt, float *dst, float value, long n) {
  if (n <= 0) return;
  ApplyPlan plan;
  plan.rt = rt;
  ThclContigParams &c = plan.c;
  memset(&c, 0, sizeof(c));
  c.p[0] = dst;
  c.val[0] = value;
  c.n = (thcl_u64)n;
  const bool al = aligned_vec(dst, 1);
  plan.kind = al ? K_CONTIG_V4 : K_CONTIG_S;
  const long units = al ? (n / THCL_CONTIG_W_FOR(1)) : n;
  const long upt = units_per_tile(plan.kind, 1);
  const long tiles = (units + upt - 1) / upt;
  c.ntiles = (thcl_u64)tiles;
  plan.grid = (unsigned)(tiles < 1 ? 1 : (tiles > kMaxGrid ? kMaxGrid : tiles));
  launch_fixed(kFixed[OP_FILL], plan);
}

// n / d by the multiply-and-shift the kernels use for their index arithmetic
unsigned thcl_host_divide(unsigned n, long d) {
  const ThclDivisor dv = thcl_make_divisor(d);
  return (unsigned)((((unsigned long long)n * dv.magic) >> 32) + n) >> dv.shift;
}

// Which kernel family a call would launch and with what grid, without opening a device or
// launching anything: 0 dense 128-bit, 1 dense scalar, 2 joint 128-bit, 3 joint scalar,
// 4 generic, 5 tiled, 6 nothing to do.
int thcl_apply_classify(const ApplyCall &call, unsigned *grid) {
  ApplyPlan plan;
  if (!make_plan(nullptr, call, plan, true)) return 6;
  if (grid) *grid = plan.grid;
  return (int)plan.kind;
}
