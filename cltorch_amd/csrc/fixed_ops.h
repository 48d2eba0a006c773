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

enum ThclOp : int {
#define X(name, nt, stmt) OP_##name,
  THCL_FIXED_OPS(X)
#undef X
  OP_COUNT
};
