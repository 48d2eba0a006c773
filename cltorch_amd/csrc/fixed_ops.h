// The ahead-of-time compiled pointwise operators: X(name, tensors, statement).
// In a statement `o` is operand 0 (read-write), `a`/`b` operands 1 and 2,
// `v1`/`v2` host scalars, `p1` a scalar read from a point tensor on the
// device.  Each statement keeps the operand order of the reference's
// operator string it stands for, so rounding happens in the same places:
//   src/lib/THClTensorMathPointwise.h:84-140      (add/cadd/sub/csub/mul)
//   src/lib/THClTensorMathPairwise.cpp:18-135     (scalar and point-tensor forms)
//   src/lib/THClTensorMath.cpp:26-54,111-257      (fill, cdiv, addcmul, addcdiv)
//   src/lib/THClReduceApplyUtils.h:35-40          (copy)
// The scalar division divides (Torch7's CPU result) where the reference
// multiplies by a reciprocal.
#pragma once

#define THCL_FIXED_OPS(X)                    \
  X(FILL, 1, o = v1)                         \
  X(FILL_PT, 1, o = p1)                      \
  X(ADD_S1, 1, o += v1)                      \
  X(MUL_S1, 1, o *= v1)                      \
  X(DIV_S1, 1, o = o / v1)                   \
  X(ADD_PT1, 1, o += p1)                     \
  X(SUB_PT1, 1, o -= p1)                     \
  X(MUL_PT1, 1, o *= p1)                     \
  X(DIV_PT1, 1, o /= p1)                     \
  X(SQRT1, 1, o = sqrtf(o))                  \
  X(ABS1, 1, o = fabsf(o))                   \
  X(NEG1, 1, o = -(o))                       \
  X(CINV1, 1, o = 1.0f / (o))                \
  X(COPY, 2, o = a)                          \
  X(ADD_S2, 2, o = a + v1)                   \
  X(MUL_S2, 2, o = a * v1)                   \
  X(DIV_S2, 2, o = a / v1)                   \
  X(ADD_PT2, 2, o = a + p1)                  \
  X(SUB_PT2, 2, o = a - p1)                  \
  X(MUL_PT2, 2, o = a * p1)                  \
  X(DIV_PT2, 2, o = a / p1)                  \
  X(SQRT2, 2, o = sqrtf(a))                  \
  X(ABS2, 2, o = fabsf(a))                   \
  X(NEG2, 2, o = -(a))                       \
  X(CINV2, 2, o = 1.0f / (a))                \
  X(ADD2, 2, o += a)                         \
  X(CADD2, 2, o += v1 * a)                   \
  X(SUB2, 2, o -= a)                         \
  X(CSUB2, 2, o -= v1 * a)                   \
  X(MUL2, 2, o *= a)                         \
  X(DIV2, 2, o /= a)                         \
  X(ADD3, 3, o = a + b)                      \
  X(CADD3, 3, o = a + v1 * b)                \
  X(SUB3, 3, o = a - b)                      \
  X(CSUB3, 3, o = a - v1 * b)                \
  X(MUL3, 3, o = (a) * (b))                  \
  X(DIV3, 3, o = a / b)                      \
  X(ADDCMUL, 3, o += v1 * a * b)             \
  X(ADDCDIV, 3, o += v1 * a / b)

// The rest of the reference's pointwise catalogue, compiled ahead of time as
// well (a separate translation unit, so the two tables build side by side).
// Each statement is the reference's operator string with the float functions
// spelled out, in the 1-, 2- or 3-tensor form the entry point picks:
//   src/lib/THClTensorMathPointwise.cpp:39-58,191-319   (unary math, cmax/cmin)
//   src/lib/THClTensorMath2.cpp:22-188                  (pow, tpow, clamp, atan2, sign)
//   src/lib/THClTensorMath.cpp:111-142                  (cpow)
//   src/lib/THClTensorMathCompare.cpp:26-82, THClTensorMathCompareT.cpp:18-57
//   src/lib/THClTensorMasked.cpp:29-38                  (maskedFill)
// thcl_pown(x, n) is the OpenCL pown the reference's pow uses for integral
// exponents (repeated squaring; apply_device.h).
#define THCL_CAT_UNARY(X, NAME, FN) \
  X(NAME##1, 1, o = FN(o))          \
  X(NAME##2, 2, o = FN(a))
#define THCL_CAT_COMPARE(X, NAME, OP)              \
  X(NAME##_V2, 2, o = (float)(a OP v1))            \
  X(NAME##_PT2, 2, o = (float)(a OP p1))           \
  X(NAME##_T3, 3, o = (float)(a OP b))
#define THCL_CATALOGUE_OPS(X)                          \
  THCL_CAT_UNARY(X, LOG1P, log1pf)                     \
  THCL_CAT_UNARY(X, COS, cosf)                         \
  THCL_CAT_UNARY(X, ACOS, acosf)                       \
  THCL_CAT_UNARY(X, COSH, coshf)                       \
  THCL_CAT_UNARY(X, SIN, sinf)                         \
  THCL_CAT_UNARY(X, ASIN, asinf)                       \
  THCL_CAT_UNARY(X, SINH, sinhf)                       \
  THCL_CAT_UNARY(X, TAN, tanf)                         \
  THCL_CAT_UNARY(X, ATAN, atanf)                       \
  THCL_CAT_UNARY(X, ROUND, roundf)                     \
  X(SIGN1, 1, o = (float)((o > 0) - (o < 0)))          \
  X(SIGN2, 2, o = (float)((a > 0) - (a < 0)))          \
  X(POWN1, 1, o = thcl_pown(o, (int)v1))               \
  X(POWN2, 2, o = thcl_pown(a, (int)v1))               \
  X(POW1, 1, o = powf(o, v1))                          \
  X(POW2, 2, o = powf(a, v1))                          \
  X(TPOW1, 1, o = powf(v1, o))                         \
  X(TPOW2, 2, o = powf(v1, a))                         \
  X(CPOW2, 2, o = powf(o, a))                          \
  X(CPOW3, 3, o = powf(a, b))                          \
  X(CLAMP1, 1, o = fmaxf(fminf(o, v2), v1))            \
  X(CLAMP2, 2, o = fmaxf(fminf(a, v2), v1))            \
  X(ATAN2_3, 3, o = atan2f(a, b))                      \
  X(CMAX2, 2, o = fmaxf(o, a))                         \
  X(CMAX3, 3, o = fmaxf(a, b))                         \
  X(CMIN2, 2, o = fminf(o, a))                         \
  X(CMIN3, 3, o = fminf(a, b))                         \
  X(CMAXV1, 1, o = fmaxf(o, v1))                       \
  X(CMAXV2, 2, o = fmaxf(a, v1))                       \
  X(CMINV1, 1, o = fminf(o, v1))                       \
  X(CMINV2, 2, o = fminf(a, v1))                       \
  THCL_CAT_COMPARE(X, LT, <)                           \
  THCL_CAT_COMPARE(X, GT, >)                           \
  THCL_CAT_COMPARE(X, LE, <=)                          \
  THCL_CAT_COMPARE(X, GE, >=)                          \
  THCL_CAT_COMPARE(X, EQ, ==)                          \
  THCL_CAT_COMPARE(X, NE, !=)                          \
  X(MASKEDFILL2, 2, if (a != 0.0f) { o = v1; })

// one numbering over both tables: the catalogue's operators follow the fixed ones
enum ThclOp : int {
#define X(name, nt, stmt) OP_##name,
  THCL_FIXED_OPS(X)
  THCL_CATALOGUE_OPS(X)
#undef X
  OP_COUNT
};
#define X(name, nt, stmt) +1
enum : int { OP_FIXED_COUNT = 0 THCL_FIXED_OPS(X) };
#undef X
