// C-ABI pointwise, copy and reduction entry points: argument checks and
// overload selection only; the kernels live in apply.hip / reduce.hip.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "internal.h"

namespace {

// self == src: in-place with the 1-tensor operator; else resize self like src
// and use the 2-tensor operator (src/lib/THClTensorMathPairwise.cpp:60-75).
void unary_like(THClState *state, THClTensor *self, THClTensor *src, ThclOp op1, ThclOp op2, float v = 0.f,
                const float *pt = nullptr) {
  thcl_check_same_device(state, 2, self, src);
  ApplyCall c;
  c.val[0] = v;
  c.pt[0] = pt;
  if (self == src) {
    c.n = 1;
    c.t[0] = self;
    thcl_apply_fixed(state, op1, c);
  } else {
    THClTensor_resizeAs(state, self, src);
    c.n = 2;
    c.t[0] = self;
    c.t[1] = src;
    thcl_apply_fixed(state, op2, c);
  }
}

// same, for operators that go through the runtime compiler with their
// operator string (the reference compiles every operator this way)
void unary_like_expr(THClState *state, THClTensor *self, THClTensor *src, const char *fn) {
  thcl_check_same_device(state, 2, self, src);
  ApplyCall c;
  if (self == src) {
    c.n = 1;
    c.t[0] = self;
    thcl_apply_expr(state, std::string("*out = ") + fn + "(*out)", c);
  } else {
    THClTensor_resizeAs(state, self, src);
    c.n = 2;
    c.t[0] = self;
    c.t[1] = src;
    thcl_apply_expr(state, std::string("*out = ") + fn + "(*in1)", c);
  }
}

const float *point_value(THClState *state, THClTensor *value) {
  THCL_ARGCHECK(value->nDimension == 0, 3, "value must be a point tensor (zero dimensions)");
  THCL_ARGCHECK(value->storage && value->storage->wrapper, 3, "point tensor has no storage");
  (void)state;
  return thcl_dptr(value);
}

// self (op)= src2, or self = src1 (op) src2  (src/lib/THClTensorMathPointwise.cpp:148-189)
void binary_like(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2, ThclOp op2, ThclOp op3,
                 float v = 0.f) {
  thcl_check_same_device(state, 3, self, src1, src2);
  THCL_ARGCHECK(THClTensor_nElement(state, src1) == THClTensor_nElement(state, src2), 3, "sizes do not match");
  ApplyCall c;
  c.val[0] = v;
  if (self == src1) {
    c.n = 2;
    c.t[0] = self;
    c.t[1] = src2;
    thcl_apply_fixed(state, op2, c);
  } else {
    THClTensor_resizeAs(state, self, src1);
    c.n = 3;
    c.t[0] = self;
    c.t[1] = src1;
    c.t[2] = src2;
    thcl_apply_fixed(state, op3, c);
  }
}
}  // namespace

extern "C" {

// ------------------------------------------------------------------- fill ---
void THClTensor_fill(THClState *state, THClTensor *self, float value) {
  THCL_GUARD_BEGIN
  ApplyCall c;
  c.n = 1;
  c.t[0] = self;
  c.val[0] = value;
  thcl_apply_fixed(state, OP_FILL, c);
  THCL_GUARD_END()
}
void THClTensor_zero(THClState *state, THClTensor *self) { THClTensor_fill(state, self, 0.f); }
void THClTensor_fill_gpu(THClState *state, THClTensor *self, THClTensor *value) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, self, value);
  ApplyCall c;
  c.n = 1;
  c.t[0] = self;
  c.pt[0] = point_value(state, value);
  thcl_apply_fixed(state, OP_FILL_PT, c);
  THCL_GUARD_END()
}
void THClTensor_zeros(THClState *state, THClTensor *r_, THLongStorage *size) {
  THCL_GUARD_BEGIN
  THClTensor_resize(state, r_, size, nullptr);
  THClTensor_fill(state, r_, 0.f);
  THCL_GUARD_END()
}
void THClTensor_ones(THClState *state, THClTensor *r_, THLongStorage *size) {
  THCL_GUARD_BEGIN
  THClTensor_resize(state, r_, size, nullptr);
  THClTensor_fill(state, r_, 1.f);
  THCL_GUARD_END()
}
long THClTensor_numel(THClState *state, THClTensor *t) { return THClTensor_nElement(state, t); }
// r_ takes the given shape and t's elements in order (src/lib/THClTensorMath.cpp:97-104)
void THClTensor_reshape(THClState *state, THClTensor *r_, THClTensor *t, THLongStorage *size) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, r_, t);
  if (r_->nDimension < 0 && !r_->storage) r_->device = THClTensor_getDevice(state, t);
  THClTensor_resize(state, r_, size, nullptr);
  THClTensor_copy(state, r_, t);
  THCL_GUARD_END()
}

// ----------------------------------------------------------- scalar forms ---
void THClTensor_add(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  unary_like(state, self, src, OP_ADD_S1, OP_ADD_S2, value);
  THCL_GUARD_END()
}
void THClTensor_sub(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  unary_like(state, self, src, OP_ADD_S1, OP_ADD_S2, -value);  // src/lib/THClTensorMathPairwise.cpp:77-93
  THCL_GUARD_END()
}
void THClTensor_mul(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  unary_like(state, self, src, OP_MUL_S1, OP_MUL_S2, value);
  THCL_GUARD_END()
}
void THClTensor_div(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(value != 0.0f, 3, "divide by zero");
  unary_like(state, self, src, OP_DIV_S1, OP_DIV_S2, value);
  THCL_GUARD_END()
}

// ----------------------------------------------------- point-tensor forms ---
void THClTensor_add_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, src, value);
  unary_like(state, self, src, OP_ADD_PT1, OP_ADD_PT2, 0.f, point_value(state, value));
  THCL_GUARD_END()
}
void THClTensor_sub_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, src, value);
  unary_like(state, self, src, OP_SUB_PT1, OP_SUB_PT2, 0.f, point_value(state, value));
  THCL_GUARD_END()
}
void THClTensor_mul_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, src, value);
  unary_like(state, self, src, OP_MUL_PT1, OP_MUL_PT2, 0.f, point_value(state, value));
  THCL_GUARD_END()
}
void THClTensor_div_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, src, value);
  unary_like(state, self, src, OP_DIV_PT1, OP_DIV_PT2, 0.f, point_value(state, value));
  THCL_GUARD_END()
}

// ----------------------------------------------------------- tensor forms ---
void THClTensor_cadd(THClState *state, THClTensor *self, THClTensor *src1, float value, THClTensor *src2) {
  THCL_GUARD_BEGIN
  if (src2->nDimension == 0) {  // point tensor on the right: src/lib/THClTensorMathPointwise.cpp:151-154
    THClTensor_add_gpu(state, self, src1, src2);
    return;
  }
  if (value == 1.0f) binary_like(state, self, src1, src2, OP_ADD2, OP_ADD3);
  else binary_like(state, self, src1, src2, OP_CADD2, OP_CADD3, value);
  THCL_GUARD_END()
}
void THClTensor_csub(THClState *state, THClTensor *self, THClTensor *src1, float value, THClTensor *src2) {
  THCL_GUARD_BEGIN
  if (src2->nDimension == 0) {
    THClTensor_sub_gpu(state, self, src1, src2);
    return;
  }
  if (value == 1.0f) binary_like(state, self, src1, src2, OP_SUB2, OP_SUB3);
  else binary_like(state, self, src1, src2, OP_CSUB2, OP_CSUB3, value);
  THCL_GUARD_END()
}
void THClTensor_cmul(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  binary_like(state, self, src1, src2, OP_MUL2, OP_MUL3);
  THCL_GUARD_END()
}
void THClTensor_cdiv(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  binary_like(state, self, src1, src2, OP_DIV2, OP_DIV3);
  THCL_GUARD_END()
}

static void addc(THClState *state, THClTensor *self, THClTensor *t, float value, THClTensor *src1,
                 THClTensor *src2, ThclOp op) {
  // src/lib/THClTensorMath.cpp:177-257
  thcl_check_same_device(state, 4, self, t, src1, src2);
  if (self != t) {
    THClTensor_resizeAs(state, self, t);
    THClTensor_copy(state, self, t);
  } else {
    // element counts must agree, shapes need not: self keeps its own
    THCL_ARGCHECK(THClTensor_nElement(state, self) == THClTensor_nElement(state, src1), 1, "sizes do not match");
  }
  THCL_ARGCHECK(THClTensor_nElement(state, src1) == THClTensor_nElement(state, src2), 3, "sizes do not match");
  ApplyCall c;
  c.n = 3;
  c.t[0] = self;
  c.t[1] = src1;
  c.t[2] = src2;
  c.val[0] = value;
  thcl_apply_fixed(state, op, c);
}
void THClTensor_addcmul(THClState *state, THClTensor *self, THClTensor *t, float value, THClTensor *src1,
                        THClTensor *src2) {
  THCL_GUARD_BEGIN
  addc(state, self, t, value, src1, src2, OP_ADDCMUL);
  THCL_GUARD_END()
}
void THClTensor_addcdiv(THClState *state, THClTensor *self, THClTensor *t, float value, THClTensor *src1,
                        THClTensor *src2) {
  THCL_GUARD_BEGIN
  addc(state, self, t, value, src1, src2, OP_ADDCDIV);
  THCL_GUARD_END()
}

// ------------------------------------------------------------- unary math ---
#define THCL_UNARY_FIXED(NAME, OP)                                                 \
  void THClTensor_##NAME(THClState *state, THClTensor *self, THClTensor *src) {  \
    THCL_GUARD_BEGIN                                                               \
    unary_like(state, self, src, OP##1, OP##2);                                    \
    THCL_GUARD_END()                                                               \
  }
THCL_UNARY_FIXED(sqrt, OP_SQRT)
THCL_UNARY_FIXED(abs, OP_ABS)
THCL_UNARY_FIXED(neg, OP_NEG)
THCL_UNARY_FIXED(cinv, OP_CINV)
#undef THCL_UNARY_FIXED

#define THCL_UNARY_EXPR(NAME, FN)                                                  \
  void THClTensor_##NAME(THClState *state, THClTensor *self, THClTensor *src) {  \
    THCL_GUARD_BEGIN                                                               \
    unary_like_expr(state, self, src, FN);                                         \
    THCL_GUARD_END()                                                               \
  }
THCL_UNARY_EXPR(exp, "exp")
THCL_UNARY_EXPR(log, "log")
THCL_UNARY_EXPR(tanh, "tanh")
THCL_UNARY_EXPR(floor, "floor")
THCL_UNARY_EXPR(ceil, "ceil")
#undef THCL_UNARY_EXPR

void THClTensor_sigmoid(THClState *state, THClTensor *self, THClTensor *src) {
  // operator strings of src/lib/THClTensorMathPointwise.h:3-13
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, self, src);
  ApplyCall c;
  if (self == src) {
    c.n = 1;
    c.t[0] = self;
    thcl_apply_expr(state, "*out = 1.0f / (1 + exp(- (*out)))", c);
  } else {
    THClTensor_resizeAs(state, self, src);
    c.n = 2;
    c.t[0] = self;
    c.t[1] = src;
    thcl_apply_expr(state, "*out = 1.0f / (1 + exp(- (*in1)))", c);
  }
  THCL_GUARD_END()
}

// -------------------------------------------------------- user expressions ---
void THClTensor_apply(THClState *state, THClTensor *self, char const *operation1) {
  THCL_GUARD_BEGIN
  ApplyCall c;
  c.n = 1;
  c.t[0] = self;
  thcl_apply_expr(state, thcl_rewrite_expr(operation1, 1), c);
  THCL_GUARD_END()
}
void THClTensor_map(THClState *state, THClTensor *self, THClTensor *two, char const *operation2) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, self, two);
  ApplyCall c;
  c.n = 2;
  c.t[0] = self;
  c.t[1] = two;
  thcl_apply_expr(state, thcl_rewrite_expr(operation2, 2), c);
  THCL_GUARD_END()
}
void THClTensor_map2(THClState *state, THClTensor *self, THClTensor *in1, THClTensor *in2, char const *operation3) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, in1, in2);
  ApplyCall c;
  c.n = 3;
  c.t[0] = self;
  c.t[1] = in1;
  c.t[2] = in2;
  thcl_apply_expr(state, thcl_rewrite_expr(operation3, 3), c);
  THCL_GUARD_END()
}

// ------------------------------------------------------------------ copies ---
// Device to device (src/lib/THClTensorCopy.cpp:130-230).  The reference turns
// dense <-> dense between different storages into a buffer copy and sends the
// rest through its apply engine; here every case is the apply engine's copy
// operator.
void THClTensor_copy(THClState *state, THClTensor *dst, THClTensor *src) {
  THCL_GUARD_BEGIN
  const long total = THClTensor_nElement(state, dst);
  THCL_ARGCHECK(total == THClTensor_nElement(state, src), 2, "sizes do not match");
  if (dst->nDimension <= 0 || total == 0) return;
  THCL_CHECK(THClTensor_getDevice(state, dst) == THClTensor_getDevice(state, src),
             "copy between devices is not implemented");
  // Dense pairs go through the copy kernel as well: it moves 6.5 TB/s where the
  // runtime's device-to-device memcpy reaches 5.2 TB/s (3.1 TB/s when an
  // operand is only 4-byte aligned), and it stays on this library's stream.
  ApplyCall c;
  c.n = 2;
  c.t[0] = dst;
  c.t[1] = src;
  thcl_apply_fixed(state, OP_COPY, c);
  THCL_GUARD_END()
}
void THClTensor_copyCl(THClState *state, THClTensor *self, THClTensor *src) { THClTensor_copy(state, self, src); }

// Host -> device.  The reference stages through a dense device temporary and
// its whole-storage host mirror (src/lib/THClTensorCopy.cpp:18-36); here a
// dense host staging buffer holds exactly the elements, one transfer moves
// them, and a strided destination is filled by a device-side scatter.
void THClTensor_copyFloat(THClState *state, THClTensor *self, THFloatTensor *src) {
  THCL_GUARD_BEGIN
  const long n = THClTensor_nElement(state, self);
  THCL_ARGCHECK(n == THFloatTensor_nElement(src), 2, "sizes do not match");
  if (n == 0) return;
  THClTensor *selfc = THClTensor_isContiguous(state, self) ? self : nullptr;
  THClTensor *tmp = nullptr;
  if (!selfc) {
    tmp = THClTensor_newv2(state, THClTensor_getDevice(state, self));
    THClTensor_resizeAs(state, tmp, self);
    selfc = tmp;
  }
  // gather the host view in logical order
  const float *hsrc = src->storage->data + src->storageOffset;
  std::vector<float> stage;
  bool hdense = true;
  {
    long z = 1;
    for (int d = src->nDimension - 1; d >= 0; d--) {
      if (src->size[d] == 1) continue;
      if (src->stride[d] != z) hdense = false;
      z *= src->size[d];
    }
  }
  if (!hdense) {
    stage.resize((size_t)n);
    long idx[THCL_MAX_DIMS] = {0};
    long off = 0;
    for (long i = 0; i < n; i++) {
      stage[(size_t)i] = hsrc[off];
      for (int d = src->nDimension - 1; d >= 0; d--) {
        idx[d]++;
        off += src->stride[d];
        if (idx[d] < src->size[d]) break;
        off -= idx[d] * src->stride[d];
        idx[d] = 0;
      }
    }
    hsrc = stage.data();
  }
  thcl_rt *rt = thcl_ctx(state, selfc->storage->device);
  int rc = thcl_rt_memcpy_h2d(rt, thcl_dptr(selfc), hsrc, (size_t)n * sizeof(float));
  if (rc != 0) {
    if (tmp) THClTensor_free(state, tmp);
    thcl_throw("%s", thcl_rt_error());
  }
  if (tmp) THClTensor_freeCopyTo(state, tmp, self);
  THCL_GUARD_END()
}

// a host LongTensor whose elements lie dense in logical order
static constexpr long kLongConvertedFrom = 1l << 16;
static bool long_dense(const THLongTensor *t) {
  long z = 1;
  for (int d = t->nDimension - 1; d >= 0; d--) {
    if (t->size[d] != 1 && t->stride[d] != z) return false;
    z *= t->size[d];
  }
  return true;
}

void THClTensor_copyLong(THClState *state, THClTensor *self, THLongTensor *src) {
  // everything comes down to a copy from floats (src/lib/THClTensorCopy.cpp:38-66)
  THCL_GUARD_BEGIN
  const long n = THClTensor_nElement(state, self);
  THCL_ARGCHECK(n == THLongTensor_nElement(src), 2, "sizes do not match");
  if (n == 0) return;
  if (n >= kLongConvertedFrom && long_dense(src) && THClTensor_isContiguous(state, self)) {
    // large and dense on both sides: converted by the runtime's host threads on the way through its buffers
    thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, self));
    THCL_CHECK(thcl_rt_copy_converted(rt, thcl_dptr(self), src->storage->data + src->storageOffset, (size_t)n, THCL_RT_I64, 1) == 0, "%s",
               thcl_rt_error());
    return;
  }
  std::vector<float> f((size_t)n);
  long idx[THCL_MAX_DIMS] = {0};
  long off = src->storageOffset;
  for (long i = 0; i < n; i++) {
    f[(size_t)i] = (float)src->storage->data[off];
    for (int d = src->nDimension - 1; d >= 0; d--) {
      idx[d]++;
      off += src->stride[d];
      if (idx[d] < src->size[d]) break;
      off -= idx[d] * src->stride[d];
      idx[d] = 0;
    }
  }
  long sz[THCL_MAX_DIMS];
  for (int d = 0; d < src->nDimension; d++) sz[d] = src->size[d];
  THFloatTensor *ft = THFloatTensor_newWithData(f.data(), n, 0, src->nDimension, sz, nullptr);
  try {
    THClTensor_copyFloat(state, self, ft);
  } catch (...) {
    THFloatTensor_free(ft);
    throw;
  }
  THFloatTensor_free(ft);
  THCL_GUARD_END()
}

// Device -> host (src/lib/THClTensorCopy.cpp:70-91).
void THFloatTensor_copyCl(THClState *state, THFloatTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  const long n = THClTensor_nElement(state, src);
  THCL_ARGCHECK(THFloatTensor_nElement(self) == n, 2, "sizes do not match");
  if (n == 0) return;
  THClTensor *srcc = THClTensor_newContiguous(state, src);
  thcl_rt *rt = thcl_ctx(state, srcc->storage->device);
  bool hdense = true;
  {
    long z = 1;
    for (int d = self->nDimension - 1; d >= 0; d--) {
      if (self->size[d] == 1) continue;
      if (self->stride[d] != z) hdense = false;
      z *= self->size[d];
    }
  }
  float *hdst = self->storage->data + self->storageOffset;
  std::vector<float> stage;
  if (!hdense) stage.resize((size_t)n);
  int rc;
  size_t box_floats = 0;
  const float *box = thcl_rt_mailbox_host(rt, &box_floats);
  if ((size_t)n <= box_floats) {
    // small: a kernel leaves it in page-locked memory and the host waits for its tag, not for the stream
    const unsigned tag = thcl_rt_next_tag(rt);
    thcl_small_to_host(state, rt, thcl_dptr(srcc), n, tag);
    float unused;
    rc = thcl_rt_await_tagged(rt, tag, &unused);
    if (rc == 0) memcpy(hdense ? hdst : stage.data(), box, (size_t)n * sizeof(float));
  } else {
    rc = thcl_rt_memcpy_d2h(rt, hdense ? hdst : stage.data(), thcl_dptr(srcc), (size_t)n * sizeof(float));
  }
  THClTensor_free(state, srcc);
  THCL_CHECK(rc == 0, "%s", thcl_rt_error());
  if (!hdense) {
    long idx[THCL_MAX_DIMS] = {0};
    long off = 0;
    for (long i = 0; i < n; i++) {
      hdst[off] = stage[(size_t)i];
      for (int d = self->nDimension - 1; d >= 0; d--) {
        idx[d]++;
        off += self->stride[d];
        if (idx[d] < self->size[d]) break;
        off -= idx[d] * self->stride[d];
        idx[d] = 0;
      }
    }
  }
  THCL_GUARD_END()
}

void THLongTensor_copyCl(THClState *state, THLongTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  const long n = THClTensor_nElement(state, src);
  THCL_ARGCHECK(THLongTensor_nElement(self) == n, 2, "sizes do not match");
  if (n == 0) return;
  if (n >= kLongConvertedFrom && long_dense(self) && THClTensor_isContiguous(state, src)) {
    thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, src));
    THCL_CHECK(thcl_rt_copy_converted(rt, thcl_dptr(src), self->storage->data + self->storageOffset, (size_t)n, THCL_RT_I64, 0) == 0, "%s",
               thcl_rt_error());
    return;
  }
  std::vector<float> f((size_t)n);
  long sz[THCL_MAX_DIMS];
  for (int d = 0; d < src->nDimension; d++) sz[d] = src->size[d];
  THFloatTensor *ft = THFloatTensor_newWithData(f.data(), n, 0, src->nDimension, sz, nullptr);
  try {
    THFloatTensor_copyCl(state, ft, src);
  } catch (...) {
    THFloatTensor_free(ft);
    throw;
  }
  THFloatTensor_free(ft);
  long idx[THCL_MAX_DIMS] = {0};
  long off = self->storageOffset;
  for (long i = 0; i < n; i++) {
    self->storage->data[off] = (long)f[(size_t)i];
    for (int d = self->nDimension - 1; d >= 0; d--) {
      idx[d]++;
      off += self->stride[d];
      if (idx[d] < self->size[d]) break;
      off -= idx[d] * self->stride[d];
      idx[d] = 0;
    }
  }
  THCL_GUARD_END()
}

// -------------------------------------------------------------- reductions ---
static float reduce_all_to_host(THClState *state, ThclReduce kind, THClTensor *self, float exponent = 0.f) {
  THCL_CHECK(self->storage != nullptr || self->nDimension <= 0, "tensor has no storage");
  int device = THClTensor_getDevice(state, self);
  thcl_rt *rt = thcl_ctx(state, device);
  // the last block stores the scalar straight into pinned host memory; waiting
  // for the stream is the only synchronising step, no copy follows
  // (the reference: blocking read-back of the scratch buffer, src/lib/THClTensorMath.cpp:346-368)
  if (THClTensor_nElement(state, self) == 0) {
    thcl_reduce_all(state, kind, self, thcl_rt_host_word_device(rt), exponent);
    THCL_CHECK(thcl_rt_sync(rt) == 0, "%s", thcl_rt_error());
    return thcl_rt_host_word(rt)[0];
  }
  // the kernel stores {result, tag} in one piece; the host picks it up as soon as it lands
  const unsigned tag = thcl_rt_next_tag(rt);
  thcl_reduce_all(state, kind, self, thcl_rt_tagged_word_device(rt), exponent, tag);
  float value = 0.f;
  THCL_CHECK(thcl_rt_await_tagged(rt, tag, &value) == 0, "%s", thcl_rt_error());
  return value;
}
static void reduce_all_to_point(THClState *state, ThclReduce kind, THClTensor *self, THClTensor *src) {
  thcl_check_same_device(state, 2, self, src);
  THCL_CHECK(self != src, "result and source must be different tensors");
  if (self->nDimension < 0 && !self->storage) self->device = THClTensor_getDevice(state, src);
  THClTensor_resize0d(state, self);
  thcl_reduce_all(state, kind, src, thcl_dptr(self));
}

float THClTensor_sumall(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  return reduce_all_to_host(state, RED_SUM, self);
  THCL_GUARD_END(0.f)
}
float THClTensor_prodall(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  return reduce_all_to_host(state, RED_PROD, self);
  THCL_GUARD_END(0.f)
}
float THClTensor_maxall(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  return reduce_all_to_host(state, RED_MAX, self);
  THCL_GUARD_END(0.f)
}
float THClTensor_minall(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  return reduce_all_to_host(state, RED_MIN, self);
  THCL_GUARD_END(0.f)
}
void THClTensor_sumall_gpu(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  reduce_all_to_point(state, RED_SUM, self, src);
  THCL_GUARD_END()
}
// The variant that allocates nothing.  It stays clear of the guard macros and of thcl_ctx, both of
// which may create or destroy profiling events.
void THClTensor_sumall_gpu_noalloc(THClState *state, THClTensor *self, THClTensor *src) {
  thcl_clear_error();
  try {
    THCL_CHECK(state && self && src, "NULL argument");
    thcl_check_same_device(state, 2, self, src);
    THCL_CHECK(self != src, "result and source must be different tensors");
    THCL_CHECK(self->nDimension == 0 && self->storage != nullptr && self->storage->wrapper != nullptr,
               "the result must already be a point tensor that owns its storage: this entry point allocates nothing");
    thcl_reduce_all_noalloc(state, RED_SUM, src, thcl_dptr(self));
  } catch (const std::exception &e) {
    thcl_report(e.what());
  }
}
void THClTensor_prodall_gpu(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  reduce_all_to_point(state, RED_PROD, self, src);
  THCL_GUARD_END()
}
void THClTensor_maxall_gpu(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  reduce_all_to_point(state, RED_MAX, self, src);
  THCL_GUARD_END()
}
void THClTensor_minall_gpu(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  reduce_all_to_point(state, RED_MIN, self, src);
  THCL_GUARD_END()
}
float THClTensor_as_float(THClState *state, THClTensor *self) {
  // src/lib/THClTensorMath.cpp:331-344
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(self->nDimension == 0, 1, "tensor must be point tensor, zero dimensions");
  THCL_ARGCHECK(self->storage != nullptr && self->storage->wrapper != nullptr, 1, "tensor must have allocated storage");
  thcl_rt *rt = thcl_ctx(state, self->storage->device);
  // a one-thread launch hands the scalar over through the pinned {value, tag} pair: quicker than a copy
  // followed by a wait for the stream
  const unsigned tag = thcl_rt_next_tag(rt);
  thcl_scalar_to_host(state, rt, thcl_dptr(self), tag);
  float value = 0.f;
  THCL_CHECK(thcl_rt_await_tagged(rt, tag, &value) == 0, "%s", thcl_rt_error());
  return value;
  THCL_GUARD_END(0.f)
}

void THClTensor_sum(THClState *state, THClTensor *self, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  thcl_reduce_dim(state, RED_SUM, self, nullptr, nullptr, src, dim);
  THCL_GUARD_END()
}
void THClTensor_prod(THClState *state, THClTensor *self, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  thcl_reduce_dim(state, RED_PROD, self, nullptr, nullptr, src, dim);
  THCL_GUARD_END()
}
void THClTensor_max(THClState *state, THClTensor *values, THClTensor *indices, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  thcl_reduce_dim(state, RED_MAX, values, indices, nullptr, src, dim);
  THCL_GUARD_END()
}
void THClTensor_min(THClState *state, THClTensor *values, THClTensor *indices, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  thcl_reduce_dim(state, RED_MIN, values, indices, nullptr, src, dim);
  THCL_GUARD_END()
}

static void arg_reduce_long(THClState *state, ThclReduce kind, THClTensor *values, THLongTensor *indices,
                            THClTensor *src, long dim) {
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 3, "dimension out of range");
  long nslices = 1;
  for (int d = 0; d < src->nDimension; d++)
    if (d != dim) nslices *= src->size[d];
  THCL_ARGCHECK(THLongTensor_nElement(indices) == nslices, 2, "indices must hold one entry per slice");
  thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, src));
  int64_t *didx = (int64_t *)thcl_rt_malloc(rt, (size_t)nslices * sizeof(int64_t));
  THCL_CHECK(didx != nullptr, "%s", thcl_rt_error());
  std::vector<int64_t> h((size_t)nslices);
  int rc = 0;
  try {
    thcl_reduce_dim(state, kind, values, nullptr, didx, src, dim);
    rc = thcl_rt_memcpy_d2h(rt, h.data(), didx, (size_t)nslices * sizeof(int64_t));
  } catch (...) {
    thcl_rt_free(rt, didx);
    throw;
  }
  thcl_rt_free(rt, didx);
  THCL_CHECK(rc == 0, "%s", thcl_rt_error());
  long idx[THCL_MAX_DIMS] = {0};
  long off = indices->storageOffset;
  for (long i = 0; i < nslices; i++) {
    indices->storage->data[off] = (long)h[(size_t)i];
    for (int d = indices->nDimension - 1; d >= 0; d--) {
      idx[d]++;
      off += indices->stride[d];
      if (idx[d] < indices->size[d]) break;
      off -= idx[d] * indices->stride[d];
      idx[d] = 0;
    }
  }
}
void THClTensor_maxLong(THClState *state, THClTensor *values, THLongTensor *indices, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  arg_reduce_long(state, RED_MAX, values, indices, src, dim);
  THCL_GUARD_END()
}
void THClTensor_minLong(THClState *state, THClTensor *values, THLongTensor *indices, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  arg_reduce_long(state, RED_MIN, values, indices, src, dim);
  THCL_GUARD_END()
}

// ---- mean, norms, all / any (src/lib/THClTensorMath2.cpp:190-203,336-417,
//      src/lib/THClTensorMath.cpp:444-528)
float THClTensor_meanall(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(self->nDimension > 0, 1, "empty Tensor");
  return reduce_all_to_host(state, RED_SUM, self) / (float)THClTensor_nElement(state, self);
  THCL_GUARD_END(0.f)
}
void THClTensor_mean(THClState *state, THClTensor *self, THClTensor *src, long dim) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 3, "dimension out of range");
  const long len = src->size[dim];
  thcl_reduce_dim(state, RED_SUM, self, nullptr, nullptr, src, dim);
  THClTensor_div(state, self, self, (float)len);
  THCL_GUARD_END()
}
static ThclReduce norm_kind(float value) {
  if (value == 0.0f) return RED_SUM_NE0;   // number of non-zero elements
  if (value == 1.0f) return RED_SUM_ABS;
  if (value == 2.0f) return RED_SUM_SQ;
  return RED_SUM_POW;
}
float THClTensor_normall(THClState *state, THClTensor *self, float value) {
  THCL_GUARD_BEGIN
  const float sum = reduce_all_to_host(state, norm_kind(value), self, value);
  if (value == 0.0f) return sum;
  return (float)std::pow((double)sum, 1.0 / (double)value);
  THCL_GUARD_END(0.f)
}
void THClTensor_norm(THClState *state, THClTensor *self, THClTensor *src, float value, long dimension) {
  THCL_GUARD_BEGIN
  thcl_reduce_dim(state, norm_kind(value), self, nullptr, nullptr, src, dimension, value);
  if (value != 0.0f) THClTensor_pow(state, self, self, 1.0f / value);
  THCL_GUARD_END()
}
int THClTensor_logicalall(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  return (int)reduce_all_to_host(state, RED_ALL, self);
  THCL_GUARD_END(0)
}
int THClTensor_logicalany(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  return (int)reduce_all_to_host(state, RED_ANY, self);
  THCL_GUARD_END(0)
}
void THClTensor_logicalall_gpu(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  reduce_all_to_point(state, RED_ALL, self, src);
  THCL_GUARD_END()
}
void THClTensor_logicalany_gpu(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  reduce_all_to_point(state, RED_ANY, self, src);
  THCL_GUARD_END()
}

}  // extern "C"
