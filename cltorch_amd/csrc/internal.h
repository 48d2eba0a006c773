// Shared host-side declarations of the tensor library: error plumbing, the
// per-tensor and joint layout descriptions, and the launch entry points each
// kernel family exposes to the C-ABI functions.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "thcl_hip.h"
#include "thcl_rt.h"
#include "fixed_ops.h"

#define THCL_MAX_DIMS 25

// The kernels hand results from block to block with relaxed device-scope accesses ordered by `s_waitcnt vmcnt(0)`
// and by tickets, which is enough on this chip because its stores complete in the L2 that the reader's loads come
// from (reduce.hip, index.hip, gemm.hip say so where they do it); tile shapes, LDS sizes and the matrix instructions
// are this chip's too.  A device pass for any other target stops here instead of building code whose ordering would
// silently no longer hold; at run time thcl_rt_get refuses devices of another architecture.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "libthcl_hip's kernels are written for gfx950 only: build with --offload-arch=gfx950"
#endif

// ---------------------------------------------------------------- errors ---
// A failed check throws ThclError; every extern "C" entry point is wrapped in
// THCL_GUARD which converts it into the recorded message + handler call, so no
// exception crosses the ABI (the reference converts EasyCL exceptions into
// THError the same way: src/lib/THClKernels.cpp:23-29).
struct ThclError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
[[noreturn]] void thcl_throw(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void thcl_report(const char *msg);
void thcl_clear_error();

#define THCL_CHECK(cond, ...) \
  do {                        \
    if (!(cond)) thcl_throw(__VA_ARGS__); \
  } while (0)
#define THCL_ARGCHECK(cond, argn, msg) \
  do {                                 \
    if (!(cond)) thcl_throw("bad argument #%d: %s", (argn), (msg)); \
  } while (0)

// Entry points call one another; only the outermost one turns an exception
// into a recorded error, inner ones let it propagate.
void thcl_profile_enter(const char *entry);  // names the launches that follow (per-kernel profiling)
struct ThclGuardScope {
  static thread_local int depth;
  explicit ThclGuardScope(const char *entry) {
    if (++depth == 1) thcl_profile_enter(entry);
  }
  ~ThclGuardScope() { --depth; }
  bool outer() const { return depth == 1; }
};
#define THCL_GUARD_BEGIN                  \
  ThclGuardScope guard_scope_(__func__);  \
  if (guard_scope_.outer()) thcl_clear_error(); \
  try {
#define THCL_GUARD_END(...)              \
  }                                      \
  catch (const std::exception &e_) {     \
    if (!guard_scope_.outer()) throw;    \
    thcl_report(e_.what());              \
    return __VA_ARGS__;                  \
  }

#define THCL_DIM_WARNING "tensor too large or too many (>25) dimensions"

// ------------------------------------------------------------ runtime use ---
thcl_rt *thcl_ctx(THClState *state, int device);
inline float *thcl_dptr(const THClTensor *t) {
  return t->storage ? (float *)t->storage->wrapper + t->storageOffset : nullptr;
}
void thcl_after_launch(THClState *state, thcl_rt *rt);  // honours state->addFinish
void thcl_check_same_device(THClState *state, int n, ...);

// ---------------------------------------------------------------- layouts ---
// Collapsed description of one tensor: adjacent dims merged where there is no
// hole between them, size-1 dims dropped (rule of
// src/lib/THClReduceApplyUtils.h:67-170).  dims[0] is outermost.
struct Layout {
  int dims = 0;
  long sizes[THCL_MAX_DIMS];
  long strides[THCL_MAX_DIMS];
  long offset = 0;  // elements from the storage start
  bool contiguous() const { return dims == 1 && strides[0] == 1; }
};
Layout thcl_collapse(const THClTensor *t, int reduceDim = -1);
bool thcl_overlapping(const THClTensor *t);
bool thcl_fits_32bit(const THClTensor *t);

// Joint description of up to 3 same-shaped tensors: size-1 dims dropped, dims
// ordered so the first operand's strides descend (a pointwise op does not care
// about traversal order), then merged wherever every operand allows it.
struct JointLayout {
  int dims = 0;
  long sizes[THCL_MAX_DIMS];
  long strides[3][THCL_MAX_DIMS];
  bool valid = false;  // false: operands differ in shape
};
JointLayout thcl_joint_collapse(int n, THClTensor *const *t);

// ---------------------------------------------------------- apply engine ---
struct ApplyCall {
  int n = 0;                   // tensors: t[0] is written (and read if the op reads it)
  THClTensor *t[3] = {nullptr, nullptr, nullptr};
  float val[2] = {0.f, 0.f};
  const float *pt[2] = {nullptr, nullptr};  // device addresses of point-tensor scalars
  bool ignore_overlap = false;  // operand 0 may alias itself; any writer may win
};
// Fixed op, ahead-of-time compiled.
void thcl_apply_fixed(THClState *state, ThclOp op, ApplyCall &call);
// User expression (already rewritten to (*out)/(*in1)/(*in2) form), hipRTC.
void thcl_apply_expr(THClState *state, const std::string &expr, ApplyCall &call);
// The text transformation applied to user expressions (x/y/z -> pointers,
// float literals suffixed); exposed for host-side tests.
std::string thcl_rewrite_expr(const char *expr, int ntensors);
// family: index of the kernel family to build (the order of the plan kinds), -1 for all six
std::string thcl_expr_source(const std::string &rewritten, int ntensors, int family);
std::string thcl_expr_tag(const std::string &rewritten, int ntensors);
std::string thcl_apply_config_defines();
// Planning only (no device): the kernel family a call would launch (0 dense 128-bit, 1 dense scalar,
// 2 joint 128-bit, 3 joint scalar, 4 generic, 5 tiled, 6 nothing to do) and its grid.
int thcl_apply_classify(const ApplyCall &call, unsigned *grid);
unsigned thcl_host_divide(unsigned n, long d);  // n / d by the kernels' multiply-and-shift

// ------------------------------------------------------------- reductions ---
// The first four also run along a dimension with positions (max, min).  The
// rest are sums / extrema of a modified element: x != 0, |x|, x^2, |x|^p (p in
// the `exponent` argument), and the truth value (int)x != 0 the reference's
// all / any reductions use (src/lib/THClTensorMath.cpp:444-458).
enum ThclReduce : int {
  RED_SUM = 0, RED_PROD = 1, RED_MAX = 2, RED_MIN = 3,
  RED_SUM_NE0 = 4, RED_SUM_ABS = 5, RED_SUM_SQ = 6, RED_SUM_POW = 7, RED_ALL = 8, RED_ANY = 9
};
// whole tensor -> one float at device address `out`
void thcl_dot_dense(THClState *state, thcl_rt *rt, const float *a, const float *b, long n, float *out, unsigned host_tag = 0);
// queues a launch that hands the device scalar at `src` to the host through the tagged word pair
void thcl_scalar_to_host(THClState *state, thcl_rt *rt, const float *src, unsigned host_tag);
// n dense floats (at most the runtime's mailbox) to the mailbox, then the tagged pair
void thcl_small_to_host(THClState *state, thcl_rt *rt, const float *src, long n, unsigned host_tag);
void thcl_scan_dim(THClState *state, bool prod, THClTensor *self, THClTensor *src, long dim);
// host_tag != 0: `out` is the pinned word pair of thcl_rt_tagged_word_device, which receives {result, tag} in one store
void thcl_reduce_all(THClState *state, ThclReduce kind, THClTensor *src, float *out, float exponent = 0.f, unsigned host_tag = 0);
// The variant for callers that cannot allocate: tickets and partials in a static device array.
void thcl_reduce_all_noalloc(THClState *state, ThclReduce kind, THClTensor *src, float *out);
void thcl_reduce_static_setup(int device);  // once per device, with that device current
// along `dim`; `values` resized to size 1 along dim; idx outputs optional:
// idx_f32 = fp32 device buffer of 1-based positions laid out like `values`,
// idx_i64 = contiguous int64 device buffer.
void thcl_reduce_dim(THClState *state, ThclReduce kind, THClTensor *values, THClTensor *indices_f32,
                     int64_t *idx_i64_dev, THClTensor *src, long dim, float exponent = 0.f);

// ------------------------------------------------------------------ gemm ---
// column-major C[m x n] = alpha * op(A) * op(B) + beta * C on device pointers
void thcl_sgemm(THClState *state, thcl_rt *rt, char transa, char transb, long m, long n, long k, float alpha,
                const float *a, long lda, const float *b, long ldb, float beta, float *c, long ldc);

// the block tile and the K slicing a product of this shape gets on a chip with `cus` compute units
void thcl_gemm_plan(long m, long n, long k, int cus, int *bm, int *bn, int *ksplit, int *kchunk, int *tail_tiles, int *tail_split);

// ------------------------------------------------------------------ misc ---
// contiguous device fill / copy kernels used by storage-level calls
// A temporary tensor that is released when the scope ends, also by an exception.
// give_to() copies it into the tensor it stood in for and releases it.
struct ThclTemp {
  THClState *state;
  THClTensor *t;
  ThclTemp(THClState *s, THClTensor *x) : state(s), t(x) {}
  ThclTemp(const ThclTemp &) = delete;
  ThclTemp &operator=(const ThclTemp &) = delete;
  ~ThclTemp() {
    if (!t) return;
    try {
      THClTensor_free(state, t);
    } catch (...) {  // a destructor must not throw; the failed release is already recorded
    }
  }
  void give_to(THClTensor *dst) {
    THClTensor *x = t;
    t = nullptr;
    THClTensor_freeCopyTo(state, x, dst);
  }
};
void thcl_fill_contig(thcl_rt *rt, float *dst, float value, long n);
