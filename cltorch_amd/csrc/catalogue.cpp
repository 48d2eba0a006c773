// The rest of the reference's pointwise operator catalogue: every entry is an
// operator string (the reference's own, cited per group) handed to the apply
// engine's run-time compiler, so these ride the same kernels as
// THClTensor_apply / map / map2.
#include <cmath>
#include <string>

#include "internal.h"

namespace {

// self == src: 1-tensor form on `self`; else resize self like src, 2-tensor form
// (src/lib/THClTensorMathPointwise.cpp:18-35).
void one_or_two(THClState *state, THClTensor *self, THClTensor *src, const std::string &op1, const std::string &op2,
                float v1 = 0.f, float v2 = 0.f) {
  thcl_check_same_device(state, 2, self, src);
  ApplyCall c;
  c.val[0] = v1;
  c.val[1] = v2;
  if (self == src) {
    c.n = 1;
    c.t[0] = self;
    thcl_apply_expr(state, op1, c);
  } else {
    THClTensor_resizeAs(state, self, src);
    c.n = 2;
    c.t[0] = self;
    c.t[1] = src;
    thcl_apply_expr(state, op2, c);
  }
}

// self == src1: 2-tensor form; else resize self like src1, 3-tensor form
// (src/lib/THClTensorMathPointwise.cpp:201-218).
void two_or_three(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2, const std::string &op2,
                  const std::string &op3) {
  thcl_check_same_device(state, 3, self, src1, src2);
  THCL_ARGCHECK(THClTensor_nElement(state, src1) == THClTensor_nElement(state, src2), 3, "sizes do not match");
  ApplyCall c;
  if (self == src1) {
    c.n = 2;
    c.t[0] = self;
    c.t[1] = src2;
    thcl_apply_expr(state, op2, c);
  } else {
    THClTensor_resizeAs(state, self, src1);
    c.n = 3;
    c.t[0] = self;
    c.t[1] = src1;
    c.t[2] = src2;
    thcl_apply_expr(state, op3, c);
  }
}

// always the 2-tensor form after resizing self like src
// (src/lib/THClTensorMathCompare.cpp:17-24)
void resize_then_two(THClState *state, THClTensor *self, THClTensor *src, const std::string &op2, float v1,
                     const float *pt) {
  thcl_check_same_device(state, 2, self, src);
  THClTensor_resizeAs(state, self, src);
  ApplyCall c;
  c.n = 2;
  c.t[0] = self;
  c.t[1] = src;
  c.val[0] = v1;
  c.pt[0] = pt;
  thcl_apply_expr(state, op2, c);
}

const float *point_of(THClTensor *value) {
  THCL_ARGCHECK(value->nDimension == 0, 3, "value must be a point tensor (zero dimensions)");
  THCL_ARGCHECK(value->storage && value->storage->wrapper, 3, "point tensor has no storage");
  return thcl_dptr(value);
}
}  // namespace

extern "C" {

// ---- unary math: "*out = F( *out )" / "*out = F( *in1 )"
//      (src/lib/THClTensorMathPointwise.cpp:39-58, THClTensorMathPointwise.h:15-27)
#define THCL_UNARY(NAME, FN)                                                                      \
  void THClTensor_##NAME(THClState *state, THClTensor *self, THClTensor *src) {                 \
    THCL_GUARD_BEGIN                                                                              \
    one_or_two(state, self, src, "*out = " FN "( *out )", "*out = " FN "( *in1 )");               \
    THCL_GUARD_END()                                                                              \
  }
THCL_UNARY(log1p, "log1p")
THCL_UNARY(cos, "cos")
THCL_UNARY(acos, "acos")
THCL_UNARY(cosh, "cosh")
THCL_UNARY(sin, "sin")
THCL_UNARY(asin, "asin")
THCL_UNARY(sinh, "sinh")
THCL_UNARY(tan, "tan")
THCL_UNARY(atan, "atan")
THCL_UNARY(round, "round")
#undef THCL_UNARY

// (src/lib/THClTensorMath2.cpp:165-188)
void THClTensor_sign(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, "*out = (*out > 0) - (*out < 0)", "*out = (*in1 > 0) - (*in1 < 0)");
  THCL_GUARD_END()
}

// integer-valued exponents use pown, others pow (src/lib/THClTensorMath2.cpp:22-61)
void THClTensor_pow(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  const bool integral = std::fabs(value) < 2147483648.f && (float)(int)value == value;
  if (integral) one_or_two(state, self, src, "*out = pown(*out, val1)", "*out = pown(*in1, val1)", value);
  else one_or_two(state, self, src, "*out = pow(*out, val1)", "*out = pow(*in1, val1)", value);
  THCL_GUARD_END()
}
// (src/lib/THClTensorMath2.cpp:63-94)
void THClTensor_tpow(THClState *state, THClTensor *self, float value, THClTensor *src) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, "*out = pow(val1, *out)", "*out = pow(val1, *in1)", value);
  THCL_GUARD_END()
}
// (src/lib/THClTensorMath.cpp:111-142)
void THClTensor_cpow(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  two_or_three(state, self, src1, src2, "*out = pow(*out, *in1)", "*out = pow(*in1, *in2)");
  THCL_GUARD_END()
}
// (src/lib/THClTensorMath2.cpp:120-163)
void THClTensor_clamp(THClState *state, THClTensor *self, THClTensor *src, float min_value, float max_value) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, "*out = fmax(fmin(*out, val2), val1)", "*out = fmax(fmin(*in1, val2), val1)", min_value,
             max_value);
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
  thcl_apply_expr(state, "*out = atan2(*in1, *in2)", c);
  THCL_GUARD_END()
}

// ---- element-wise max / min against a tensor or a number
//      (src/lib/THClTensorMathPointwise.cpp:191-319)
void THClTensor_cmax(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  two_or_three(state, self, src1, src2, "*out = max(*out, *in1)", "*out = max(*in1, *in2)");
  THCL_GUARD_END()
}
void THClTensor_cmin(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2) {
  THCL_GUARD_BEGIN
  two_or_three(state, self, src1, src2, "*out = min(*out, *in1)", "*out = min(*in1, *in2)");
  THCL_GUARD_END()
}
void THClTensor_cmaxValue(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, "*out = max(*out, val1)", "*out = max(*in1, val1)", value);
  THCL_GUARD_END()
}
void THClTensor_cminValue(THClState *state, THClTensor *self, THClTensor *src, float value) {
  THCL_GUARD_BEGIN
  one_or_two(state, self, src, "*out = min(*out, val1)", "*out = min(*in1, val1)", value);
  THCL_GUARD_END()
}

// ---- comparisons: 1.0f where the relation holds, else 0.0f
//      against a number and a point tensor (src/lib/THClTensorMathCompare.cpp:26-82),
//      against a tensor (src/lib/THClTensorMathCompareT.cpp:18-57)
#define THCL_COMPARE(NAME, OP)                                                                             \
  void THClTensor_##NAME##Value(THClState *state, THClTensor *self, THClTensor *src, float value) {      \
    THCL_GUARD_BEGIN                                                                                       \
    resize_then_two(state, self, src, "*out = (*in1 " OP " val1)", value, nullptr);                        \
    THCL_GUARD_END()                                                                                       \
  }                                                                                                        \
  void THClTensor_##NAME##PointTensor(THClState *state, THClTensor *self, THClTensor *src,               \
                                      THClTensor *value) {                                                \
    THCL_GUARD_BEGIN                                                                                       \
    thcl_check_same_device(state, 2, self, value);                                                         \
    resize_then_two(state, self, src, "*out = (*in1 " OP " *pointTensor1)", 0.f, point_of(value));         \
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
    thcl_apply_expr(state, "*out = (float) (*in1 " OP " *in2)", c);                                        \
    THCL_GUARD_END()                                                                                       \
  }
THCL_COMPARE(lt, "<")
THCL_COMPARE(gt, ">")
THCL_COMPARE(le, "<=")
THCL_COMPARE(ge, ">=")
THCL_COMPARE(eq, "==")
THCL_COMPARE(ne, "!=")
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
  thcl_apply_expr(state, "if( *in1 != 0.0f ) { *out = val1; }", c);
  THCL_GUARD_END()
}

}  // extern "C"
