// addmm: layout derivation from strides + the column-major gemm entry point.
#include <utility>

#include "internal.h"

namespace {
struct GemmOperand {
  THClTensor *t = nullptr;
  char trans = 'n';
  long ld = 0;
  bool owned = false;
};

// How a 2-d operand enters a column-major gemm whose result is stored with
// unit stride along `fast` (0: result column-major, 1: result row-major and
// the product is computed transposed).  Follows the case analysis of
// src/lib/THClTensorMathBlas.cpp:152-184: unit stride along `fast` -> 'n',
// along the other dim -> 't', neither -> dense clone.
GemmOperand pick_operand(THClState *state, THClTensor *m, int fast) {
  const int slow = 1 - fast;
  GemmOperand o;
  if (m->stride[fast] == 1) {
    o.t = m;
    o.trans = 'n';
    o.ld = m->stride[slow];
  } else if (m->stride[slow] == 1) {
    o.t = m;
    o.trans = 't';
    o.ld = m->stride[fast];
  } else {
    o.t = THClTensor_newContiguous(state, m);  // dense row-major: unit stride along dim 1
    o.owned = true;
    o.trans = (fast == 0) ? 't' : 'n';
    o.ld = o.t->stride[0];
  }
  return o;
}
}  // namespace

extern "C" {

void THClBlas_gemm(THClState *state, char transa, char transb, long m, long n, long k, float alpha, THClTensor *a,
                   long lda, THClTensor *b, long ldb, float beta, THClTensor *c, long ldc) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 3, a, b, c);
  THCL_CHECK(a->storage && b->storage && c->storage, "gemm operands need device storage");
  thcl_rt *rt = thcl_ctx(state, c->storage->device);
  thcl_sgemm(state, rt, transa, transb, m, n, k, alpha, thcl_dptr(a), lda, thcl_dptr(b), ldb, beta, thcl_dptr(c), ldc);
  THCL_GUARD_END()
}

// r_ = beta * t + alpha * m1 * m2   (src/lib/THClTensorMathBlas.cpp:107-214)
void THClTensor_addmm(THClState *state, THClTensor *r_, float beta, THClTensor *t, float alpha, THClTensor *m1,
                      THClTensor *m2) {
  THCL_GUARD_BEGIN
  thcl_check_same_device(state, 4, r_, t, m1, m2);
  THCL_CHECK(m1->nDimension == 2 && m2->nDimension == 2, "matrix and matrix expected");
  THCL_CHECK(t->nDimension == 2, "size mismatch");
  THCL_CHECK(t->size[0] == m1->size[0] && t->size[1] == m2->size[1] && m1->size[1] == m2->size[0], "size mismatch");

  if (t != r_) {
    if (r_->nDimension < 0 && !r_->storage) r_->device = THClTensor_getDevice(state, t);
    THClTensor_resizeAs(state, r_, t);
    THClTensor_copy(state, r_, t);
  }

  // a result with one column or one row is a matrix-vector product: bound by reading the matrix once,
  // which the gemv kernels do at several times the rate of a 64-wide GEMM tile with one live line
  if ((r_->size[0] == 1 || r_->size[1] == 1) && m1->size[1] > 0) {
    const bool column = r_->size[1] == 1;
    ThclTemp out(state, THClTensor_newSelect(state, r_, column ? 1 : 0, 0));
    ThclTemp vec(state, column ? THClTensor_newSelect(state, m2, 1, 0) : THClTensor_newSelect(state, m1, 0, 0));
    ThclTemp mat(state, column ? THClTensor_newWithTensor(state, m1) : THClTensor_newTranspose(state, m2, 0, 1));
    THClTensor_addmv(state, out.t, beta, out.t, alpha, mat.t, vec.t);
    return;
  }

  // result layout decides whether the product is computed as is or transposed
  THClTensor *r = r_;
  int fast;
  if (r_->stride[0] == 1) {
    fast = 0;
  } else if (r_->stride[1] == 1) {
    fast = 1;
    std::swap(m1, m2);  // C^T = B^T A^T
  } else {
    // neither stride is 1: work on a column-major dense copy, copy back after
    fast = 0;
    THClTensor *rt_view = THClTensor_newTranspose(state, r_, 0, 1);
    r = THClTensor_newClone(state, rt_view);
    THClTensor_free(state, rt_view);
    THClTensor_transpose(state, r, nullptr, 0, 1);
  }
  GemmOperand a = pick_operand(state, m1, fast);
  GemmOperand b = pick_operand(state, m2, fast);
  const int slow = 1 - fast;
  try {
    THClBlas_gemm(state, a.trans, b.trans, r->size[fast], r->size[slow], a.t->size[slow], alpha, a.t, a.ld, b.t, b.ld,
                  beta, r, r->stride[slow]);
  } catch (...) {
    if (a.owned) THClTensor_free(state, a.t);
    if (b.owned) THClTensor_free(state, b.t);
    if (r != r_) THClTensor_free(state, r);
    throw;
  }
  if (a.owned) THClTensor_free(state, a.t);
  if (b.owned) THClTensor_free(state, b.t);
  if (r != r_) THClTensor_freeCopyTo(state, r, r_);
  THCL_GUARD_END()
}

}  // extern "C"
