// The rest of the reference's pointwise operator catalogue: entry points that pick the
// 1-, 2- or 3-tensor form the reference picks and launch the ahead-of-time kernel of that
// operator (table THCL_CATALOGUE_OPS in fixed_ops.h) through the apply engine, so these ride
// the same layout families as add / cmul.  Run-time compilation is left to user expressions.
#include <cmath>

#include "internal.h"

namespace {

// self == src: 1-tensor form on `self`; else resize self like src, 2-tensor form
// (src/lib/THClTensorMathPointwise.cpp:18-35).
void one_or_two(THClState *state, THClTensor *self, THClTensor *src, ThclOp op1, ThclOp op2, float v1 = 0.f,
                float v2 = 0.f) {
  thcl_check_same_device(state, 2, self, src);
  ApplyCall c;
  c.val[0] = v1;
  c.val[1] = v2;
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

// self == src1: 2-tensor form; else resize self like src1, 3-tensor form
// (src/lib/THClTensorMathPointwise.cpp:201-218).
void two_or_three(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2, ThclOp op2, ThclOp op3) {
  thcl_check_same_device(state, 3, self, src1, src2);
  THCL_ARGCHECK(THClTensor_nElement(state, src1) == THClTensor_nElement(state, src2), 3, "sizes do not match");
  ApplyCall c;
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

// always the 2-tensor form after resizing self like src
// (src/lib/THClTensorMathCompare.cpp:17-24)
void resize_then_two(THClState *state, THClTensor *self, THClTensor *src, ThclOp op2, float v1, const float *pt) {
  thcl_check_same_device(state, 2, self, src);
  THClTensor_resizeAs(state, self, src);
  ApplyCall c;
  c.n = 2;
  c.t[0] = self;
  c.t[1] = src;
  c.val[0] = v1;
  c.pt[0] = pt;
  thcl_apply_fixed(state, op2, c);
}

const float *point_of(THClTensor *value) {
  THCL_ARGCHECK(value->nDimension == 0, 3, "value must be a point tensor (zero dimensions)");
  THCL_ARGCHECK(value->storage && value->storage->wrapper, 3, "point tensor has no storage");
  return thcl_dptr(value);
}
}  // namespace

extern "C" {

// ---- unary math: the reference's "*out = F( *out )" / "*out = F( *in1 )"
//      (src/lib/THClTensorMathPointwise.cpp:39-58, THClTensorMathPointwise.h:15-27)
#define THCL_UNARY(NAME, OP)                                                      \
  void THClTensor_##NAME(THClState *state, THClTensor *self, THClTensor *src) { \
    THCL_GUARD_BEGIN                                                              \
    one_or_two(state, self, src, OP_##OP##1, OP_##OP##2);                         \
    THCL_GUARD_END()                                                              \
  }
THCL_UNARY(log1p, LOG1P)
THCL_UNARY(cos, COS)
THCL_UNARY(acos, ACOS)
THCL_UNARY(cosh, COSH)
THCL_UNARY(sin, SIN)
THCL_UNARY(asin, ASIN)
THCL_UNARY(sinh, SINH)
THCL_UNARY(tan, TAN)
THCL_UNARY(atan, ATAN)
THCL_UNARY(round, ROUND)
#undef THCL_UNARY

// (src/lib/THClTensorMath2.cpp:165-188)
void THClTensor_sign(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, OP_SIGN1, OP_SIGN2);
  THCL_GUARD_END()
}

// integer-valued exponents use pown, others pow (src/lib/THClTensorMath2.cpp:22-61)
void THClTensor_pow(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  const bool integral = std::fabs(value) < 2147483648.f && (float)(int)value == value;
  if (integral) one_or_two(state, self, src, OP_POWN1, OP_POWN2, value);
  else one_or_two(state, self, src, OP_POW1, OP_POW2, value);
  THCL_GUARD_END()
}
// (src/lib/THClTensorMath2.cpp:63-94)
void THClTensor_tpow(THClState *state, THClTensor *self, float value, THClTensor *src) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, OP_TPOW1, OP_TPOW2, value);
  THCL_GUARD_END()
}
// (src/lib/THClTensorMath.cpp:111-142)
void THClTensor_cpow(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  two_or_three(state, self, src1, src2, OP_CPOW2, OP_CPOW3);
  THCL_GUARD_END()
}
// (src/lib/THClTensorMath2.cpp:120-163)
void THClTensor_clamp(THClState *state, THClTensor *self, THClTensor *src, float min_value, float max_value) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, OP_CLAMP1, OP_CLAMP2, min_value, max_value);
  THCL_GUARD_END()
}
// always the 3-tensor form (src/lib/THClTensorMath2.cpp:96-118)
void THClTensor_atan2(THClState *state, THClTensor *self, THClTensor *tx, THClTensor *ty) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, self, tx, ty);
  THCL_ARGCHECK(THClTensor_nElement(state, tx) == THClTensor_nElement(state, ty), 3, "sizes do not match");
  THClTensor_resizeAs(state, self, tx);
  ApplyCall c;
  c.n = 3;
  c.t[0] = self;
  c.t[1] = tx;
  c.t[2] = ty;
  thcl_apply_fixed(state, OP_ATAN2_3, c);
  THCL_GUARD_END()
}

// ---- element-wise max / min against a tensor or a number
//      (src/lib/THClTensorMathPointwise.cpp:191-319)
void THClTensor_cmax(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  two_or_three(state, self, src1, src2, OP_CMAX2, OP_CMAX3);
  THCL_GUARD_END()
}
void THClTensor_cmin(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  two_or_three(state, self, src1, src2, OP_CMIN2, OP_CMIN3);
  THCL_GUARD_END()
}
void THClTensor_cmaxValue(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, OP_CMAXV1, OP_CMAXV2, value);
  THCL_GUARD_END()
}
void THClTensor_cminValue(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, OP_CMINV1, OP_CMINV2, value);
  THCL_GUARD_END()
}

// ---- comparisons: 1.0f where the relation holds, else 0.0f
//      ("*out = (*in1 < val1)", "... *pointTensor1", "(float) (*in1 < *in2)" in the reference)
//      against a number and a point tensor (src/lib/THClTensorMathCompare.cpp:26-82),
//      against a tensor (src/lib/THClTensorMathCompareT.cpp:18-57)
#define THCL_COMPARE(NAME, OP)                                                                             \
  void THClTensor_##NAME##Value(THClState *state, THClTensor *self, THClTensor *src, float value) {      \
    THCL_GUARD_BEGIN                                                                                       \
    resize_then_two(state, self, src, OP_##OP##_V2, value, nullptr);                                       \
    THCL_GUARD_END()                                                                                       \
  }                                                                                                        \
  void THClTensor_##NAME##PointTensor(THClState *state, THClTensor *self, THClTensor *src,               \
                                      THClTensor *value) {                                                \
    THCL_GUARD_BEGIN                                                                                       \
    thcl_check_same_device(state, 2, self, value);                                                         \
    resize_then_two(state, self, src, OP_##OP##_PT2, 0.f, point_of(value));                                \
    THCL_GUARD_END()                                                                                       \
  }                                                                                                        \
  void THClTensor_##NAME##Tensor(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) { \
    THCL_GUARD_BEGIN                                                                                       \
    thcl_check_same_device(state, 3, self, src1, src2);                                                    \
    THClTensor_resizeAs(state, self, src1);                                                                \
    THCL_ARGCHECK(THClTensor_nElement(state, src1) == THClTensor_nElement(state, src2), 3,                 \
                  "sizes do not match");                                                                   \
    ApplyCall c;                                                                                           \
    c.n = 3;                                                                                               \
    c.t[0] = self;                                                                                         \
    c.t[1] = src1;                                                                                         \
    c.t[2] = src2;                                                                                         \
    thcl_apply_fixed(state, OP_##OP##_T3, c);                                                              \
    THCL_GUARD_END()                                                                                       \
  }
THCL_COMPARE(lt, LT)
THCL_COMPARE(gt, GT)
THCL_COMPARE(le, LE)
THCL_COMPARE(ge, GE)
THCL_COMPARE(eq, EQ)
THCL_COMPARE(ne, NE)
#undef THCL_COMPARE

// mask is a ClTensor holding 0 / non-0 (src/lib/THClTensorMasked.cpp:29-38,112-124)
void THClTensor_maskedFill(THClState *state, THClTensor *tensor, THClTensor *mask, float value) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 2, tensor, mask);
  THCL_ARGCHECK(THClTensor_nElement(state, tensor) == THClTensor_nElement(state, mask), 2, "sizes do not match");
  ApplyCall c;
  c.n = 2;
  c.t[0] = tensor;
  c.t[1] = mask;
  c.val[0] = value;
  thcl_apply_fixed(state, OP_MASKEDFILL2, c);
  THCL_GUARD_END()
}

}  // extern "C"
