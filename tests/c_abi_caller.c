/* A plain C caller of the library, as cltorch's own C layers are: state, tensors, host copies,
 * the config-1 operators, a point tensor, a reduction along a dim, addmm and the error path.
 * Built by tests/test_gpu_c_caller.py with gcc against include/ and libthcl_hip.so; prints
 * "ok" and returns 0 when every check holds. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "thcl_hip.h"

static int failures = 0;
#define EXPECT(cond)                                              \
  do {                                                            \
    if (!(cond)) {                                                \
      printf("line %d: %s failed\n", __LINE__, #cond);            \
      failures++;                                                 \
    }                                                             \
  } while (0)

static int error_calls = 0;
static void on_error(const char *msg, void *data) {
  (void)msg;
  (void)data;
  error_calls++;
}

static THClTensor *upload(THClState *S, float *data, int nd, const long *size) {
  long n = 1;
  for (int d = 0; d < nd; d++) n *= size[d];
  THFloatTensor *h = THFloatTensor_newWithData(data, n, 0, nd, size, NULL);
  THLongStorage *sz = THLongStorage_newWithSize(nd);
  for (int d = 0; d < nd; d++) THLongStorage_set(sz, d, size[d]);
  THClTensor *t = THClTensor_newWithSize(S, 0, sz, NULL);
  THLongStorage_free(sz);
  THClTensor_copyFloat(S, t, h);
  THFloatTensor_free(h);
  return t;
}

static void download(THClState *S, THClTensor *t, float *out, int nd, const long *size) {
  long n = 1;
  for (int d = 0; d < nd; d++) n *= size[d];
  THFloatTensor *h = THFloatTensor_newWithData(out, n, 0, nd, size, NULL);
  THFloatTensor_copyCl(S, h, t);
  THFloatTensor_free(h);
}

int main(void) {
  THClState state;
  memset(&state, 0, sizeof state);
  THClInit(&state);
  if (THClLastError()) {
    printf("init failed: %s\n", THClLastError());
    return 2;
  }
  THClState *S = &state;
  enum { N = 1000 };
  float x[N], y[N], z[N], want[N], got[N];
  for (int i = 0; i < N; i++) {
    x[i] = (float)(i % 17) * 0.25f - 2.0f;
    y[i] = (float)(i % 5) + 0.5f;
    z[i] = (float)(i % 3);
    float v = x[i] + y[i];
    v = v * y[i];
    want[i] = sqrtf(1000.0f * v * v + y[i] * 10.0f + z[i] * z[i]);
  }
  const long n1[1] = {N};
  THClTensor *X = upload(S, x, 1, n1), *Y = upload(S, y, 1, n1), *Z = upload(S, z, 1, n1);
  THClTensor_cadd(S, X, X, 1.0f, Y);
  THClTensor_cmul(S, X, X, Y);
  THClTensor_map2(S, X, Y, Z, "x = sqrt(1000*x*x + y*10 + z*z)");
  download(S, X, got, 1, n1);
  EXPECT(THClLastError() == NULL);
  int same = 1;
  double total = 0.0;
  float top = -INFINITY;
  for (int i = 0; i < N; i++) {
    same = same && (got[i] == want[i]);
    total += got[i];
    if (got[i] > top) top = got[i];
  }
  EXPECT(same);
  EXPECT(fabs(THClTensor_sumall(S, X) - total) <= 1e-5 * fabs(total));
  EXPECT(THClTensor_maxall(S, X) == top);
  /* a point tensor stays on the device between the reduction and its use */
  THClTensor *pt = THClTensor_newv2(S, 0);
  THClTensor_sumall_gpu(S, pt, X);
  THClTensor_div_gpu(S, X, X, pt);
  EXPECT(fabs(THClTensor_sumall(S, X) - 1.0) < 1e-5);
  /* sum along a dim of a transposed view */
  float m[6] = {1, 2, 3, 4, 5, 6};
  const long n2[2] = {2, 3};
  THClTensor *M = upload(S, m, 2, n2);
  THClTensor *Mt = THClTensor_newTranspose(S, M, 0, 1);
  THClTensor *R = THClTensor_newv2(S, 0);
  THClTensor_sum(S, R, Mt, 0);
  EXPECT(THClTensor_nDimension(S, R) == 2 && THClTensor_size(S, R, 0) == 1 && THClTensor_size(S, R, 1) == 2);
  EXPECT(THClTensor_get2d(S, R, 0, 0) == 6.0f && THClTensor_get2d(S, R, 0, 1) == 15.0f);
  /* addmm with the reference's integer matrices */
  float a[6] = {1, 2, -1, 3, 4, 0}, b[6] = {0, 1, 1, 2, 4, 5}, c[4] = {0, 0, 0, 0};
  const long na[2] = {2, 3}, nb[2] = {3, 2}, nc[2] = {2, 2};
  THClTensor *A = upload(S, a, 2, na), *B = upload(S, b, 2, nb), *C = upload(S, c, 2, nc);
  THClTensor_addmm(S, C, 0.0f, C, 1.0f, A, B);
  download(S, C, c, 2, nc);
  EXPECT(c[0] == -2 && c[1] == 0 && c[2] == 4 && c[3] == 11);
  /* errors come back as a message and a handler call, never as a crash */
  THClSetErrorHandler(on_error, NULL);
  THClTensor_cadd(S, X, X, 1.0f, M);
  EXPECT(error_calls == 1 && THClLastError() != NULL);
  THClClearError();
  EXPECT(THClLastError() == NULL);
  THClTensor *all[] = {X, Y, Z, pt, M, Mt, R, A, B, C};
  for (size_t i = 0; i < sizeof all / sizeof *all; i++) THClTensor_free(S, all[i]);
  THClShutdown(S);
  if (failures == 0) printf("ok\n");
  return failures ? 1 : 0;
}
