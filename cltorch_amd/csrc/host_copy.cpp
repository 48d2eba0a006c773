// Host tensors of the other element types to and from device tensors, and
// the byte-mask forms of the masked operators.
//
// What it replaces (reference): THClTensor_copy{Byte,Char,Short,Int,Double} and
// TH{Byte,...}Tensor_copyCl (src/lib/THClTensorCopy.cpp:38-66,93-128), which
// convert through a float host tensor, and THClTensor_masked{Fill,Select}Byte
// (src/lib/THClTensorMasked.cpp:248-281), which upload the mask as floats first.
// Same here: elements are converted on the host in logical order, one dense
// transfer moves them, strided device views go through the copy kernel.
#include <cstdlib>
#include <cstring>
#include <vector>

#include "internal.h"

namespace {

// every TH host tensor / storage shares this layout; only the element type differs
template <class T>
struct HostStorage {
  T *data;
  long size;
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  void *view;
};
template <class T>
struct HostTensor {
  long *size;
  long *stride;
  int nDimension;
  HostStorage<T> *storage;
  long storageOffset;
  int refcount;
  char flag;
};

template <class T>
long host_count(const HostTensor<T> *t) {
  if (t->nDimension <= 0) return 0;
  long n = 1;
  for (int d = 0; d < t->nDimension; d++) n *= t->size[d];
  return n;
}

template <class T> struct RtKind;
template <> struct RtKind<unsigned char> { static constexpr int value = THCL_RT_U8; };
template <> struct RtKind<char> { static constexpr int value = THCL_RT_I8; };
template <> struct RtKind<short> { static constexpr int value = THCL_RT_I16; };
template <> struct RtKind<int> { static constexpr int value = THCL_RT_I32; };
template <> struct RtKind<long> { static constexpr int value = THCL_RT_I64; };
template <> struct RtKind<double> { static constexpr int value = THCL_RT_F64; };

// dense in logical order: large tensors of this kind are converted by the runtime's host threads on their way
// through its page-locked buffers (2^26 doubles: 80 ms with the element-by-element walk below, one thread)
constexpr long kConvertedFrom = 1l << 16;
template <class T>
bool host_dense(const HostTensor<T> *t) {
  long z = 1;
  for (int d = t->nDimension - 1; d >= 0; d--) {
    if (t->size[d] != 1 && t->stride[d] != z) return false;
    z *= t->size[d];
  }
  return true;
}

// calls f(i, offset) for every element in logical order
template <class T, class F>
void host_walk(const HostTensor<T> *t, long n, F f) {
  long idx[THCL_MAX_DIMS] = {0};
  long off = t->storageOffset;
  for (long i = 0; i < n; i++) {
    f(i, off);
    for (int d = t->nDimension - 1; d >= 0; d--) {
      idx[d]++;
      off += t->stride[d];
      if (idx[d] < t->size[d]) break;
      off -= idx[d] * t->stride[d];
      idx[d] = 0;
    }
  }
}

template <class T>
void to_device(THClState *state, THClTensor *self, const void *src_) {
  const HostTensor<T> *src = (const HostTensor<T> *)src_;
  THCL_CHECK(src->nDimension <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  const long n = THClTensor_nElement(state, self);
  THCL_ARGCHECK(n == host_count(src), 2, "sizes do not match");
  if (n == 0) return;
  if (n >= kConvertedFrom && host_dense(src) && THClTensor_isContiguous(state, self)) {
    thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, self));
    THCL_CHECK(thcl_rt_copy_converted(rt, thcl_dptr(self), src->storage->data + src->storageOffset, (size_t)n, RtKind<T>::value, 1) == 0,
               "%s", thcl_rt_error());
    return;
  }
  std::vector<float> f((size_t)n);
  host_walk(src, n, [&](long i, long off) { f[(size_t)i] = (float)src->storage->data[off]; });
  long sz[1] = {n};
  THFloatTensor *ft = THFloatTensor_newWithData(f.data(), n, 0, 1, sz, nullptr);
  try {
    THClTensor_copyFloat(state, self, ft);  // counts match; shapes need not
  } catch (...) {
    THFloatTensor_free(ft);
    throw;
  }
  THFloatTensor_free(ft);
}

template <class T>
void to_host(THClState *state, void *self_, THClTensor *src) {
  HostTensor<T> *self = (HostTensor<T> *)self_;
  THCL_CHECK(self->nDimension <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  const long n = THClTensor_nElement(state, src);
  THCL_ARGCHECK(host_count(self) == n, 2, "sizes do not match");
  if (n == 0) return;
  if (n >= kConvertedFrom && host_dense(self) && THClTensor_isContiguous(state, src)) {
    thcl_rt *rt = thcl_ctx(state, THClTensor_getDevice(state, src));
    THCL_CHECK(thcl_rt_copy_converted(rt, thcl_dptr(src), self->storage->data + self->storageOffset, (size_t)n, RtKind<T>::value, 0) == 0,
               "%s", thcl_rt_error());
    return;
  }
  std::vector<float> f((size_t)n);
  long sz[1] = {n};
  THFloatTensor *ft = THFloatTensor_newWithData(f.data(), n, 0, 1, sz, nullptr);
  try {
    THFloatTensor_copyCl(state, ft, src);
  } catch (...) {
    THFloatTensor_free(ft);
    throw;
  }
  THFloatTensor_free(ft);
  host_walk(self, n, [&](long i, long off) { self->storage->data[off] = (T)f[(size_t)i]; });
}

template <class T>
void *host_new_with_data(T *data, long storageSize, long storageOffset, int nd, const long *size, const long *stride) {
  auto *t = (HostTensor<T> *)calloc(1, sizeof(HostTensor<T>));
  t->nDimension = nd;
  t->size = (long *)calloc((size_t)(nd > 0 ? nd : 1), sizeof(long));
  t->stride = (long *)calloc((size_t)(nd > 0 ? nd : 1), sizeof(long));
  long z = 1;
  for (int d = nd - 1; d >= 0; d--) {
    t->size[d] = size[d];
    t->stride[d] = stride ? stride[d] : z;
    z *= size[d];
  }
  t->storage = (HostStorage<T> *)calloc(1, sizeof(HostStorage<T>));
  t->storage->data = data;
  t->storage->size = storageSize;
  t->storage->refcount = 1;
  t->storage->flag = 1;  // borrowed memory
  t->storageOffset = storageOffset;
  t->refcount = 1;
  t->flag = 1;
  return t;
}
template <class T>
void host_free(void *t_) {
  auto *t = (HostTensor<T> *)t_;
  if (!t) return;
  if (--t->refcount > 0) return;
  if (t->storage && --t->storage->refcount <= 0) free(t->storage);
  free(t->size);
  free(t->stride);
  free(t);
}

// a device float tensor shaped like a host byte mask
THClTensor *upload_mask(THClState *state, int device, THByteTensor *mask) {
  const HostTensor<unsigned char> *m = (const HostTensor<unsigned char> *)mask;
  THCL_CHECK(m->nDimension > 0 && m->nDimension <= THCL_MAX_DIMS, "mask is empty or has too many dimensions");
  THLongStorage shape;
  memset(&shape, 0, sizeof(shape));
  shape.data = m->size;
  shape.size = m->nDimension;
  THClTensor *t = THClTensor_newWithSize(state, device, &shape, nullptr);
  try {
    THClTensor_copyByte(state, t, mask);
  } catch (...) {
    THClTensor_free(state, t);
    throw;
  }
  return t;
}
}  // namespace

extern "C" {

#define THCL_HOST_TYPE(Name, T)                                                                              \
  void THClTensor_copy##Name(THClState *state, THClTensor *self, TH##Name##Tensor *src) {                  \
    THCL_GUARD_BEGIN                                                                                         \
    to_device<T>(state, self, src);                                                                          \
    THCL_GUARD_END()                                                                                         \
  }                                                                                                          \
  void TH##Name##Tensor_copyCl(THClState *state, TH##Name##Tensor *self, THClTensor *src) {                \
    THCL_GUARD_BEGIN                                                                                         \
    to_host<T>(state, self, src);                                                                            \
    THCL_GUARD_END()                                                                                         \
  }
THCL_HOST_TYPE(Byte, unsigned char)
THCL_HOST_TYPE(Char, char)
THCL_HOST_TYPE(Short, short)
THCL_HOST_TYPE(Int, int)
THCL_HOST_TYPE(Double, double)
#undef THCL_HOST_TYPE

// whole storages, host element types other than float (src/lib/THClStorageCopy.cpp:45-60,75-94)
#define THCL_HOST_STORAGE(Name, T)                                                                           \
  void THClStorage_copy##Name(THClState *state, THClStorage *self, TH##Name##Storage *src) {               \
    THCL_GUARD_BEGIN                                                                                         \
    THCL_ARGCHECK(self->size == src->size, 2, "size does not match");                                        \
    if (src->size >= kConvertedFrom) {                                                                       \
      THCL_CHECK(thcl_rt_copy_converted(self->cl, self->wrapper, src->data, (size_t)src->size, RtKind<T>::value, 1) == 0, "%s", \
                 thcl_rt_error());                                                                           \
      return;                                                                                                \
    }                                                                                                        \
    std::vector<float> f((size_t)src->size);                                                                 \
    for (long i = 0; i < src->size; i++) f[(size_t)i] = (float)src->data[i];                                 \
    if (src->size > 0) THClStorage_rawCopy(state, self, f.data());                                           \
    THCL_GUARD_END()                                                                                         \
  }                                                                                                          \
  void TH##Name##Storage_copyCl(THClState *state, TH##Name##Storage *self, THClStorage *src) {             \
    THCL_GUARD_BEGIN                                                                                         \
    THCL_ARGCHECK(self->size == src->size, 2, "size does not match");                                        \
    if (src->size >= kConvertedFrom) {                                                                       \
      THCL_CHECK(thcl_rt_copy_converted(src->cl, src->wrapper, self->data, (size_t)src->size, RtKind<T>::value, 0) == 0, "%s", \
                 thcl_rt_error());                                                                           \
      return;                                                                                                \
    }                                                                                                        \
    std::vector<float> f((size_t)src->size);                                                                 \
    THFloatStorage fs;                                                                                       \
    memset(&fs, 0, sizeof(fs));                                                                              \
    fs.data = f.data();                                                                                      \
    fs.size = src->size;                                                                                     \
    if (src->size > 0) THFloatStorage_copyCl(state, &fs, src);                                               \
    for (long i = 0; i < src->size; i++) self->data[i] = (T)f[(size_t)i];                                    \
    THCL_GUARD_END()                                                                                         \
  }
THCL_HOST_STORAGE(Byte, unsigned char)
THCL_HOST_STORAGE(Char, char)
THCL_HOST_STORAGE(Short, short)
THCL_HOST_STORAGE(Int, int)
THCL_HOST_STORAGE(Long, long)
THCL_HOST_STORAGE(Double, double)
#undef THCL_HOST_STORAGE

#ifndef THCL_EXTERNAL_TH
#define THCL_HOST_STANDIN(Name, T)                                                                           \
  TH##Name##Tensor *TH##Name##Tensor_newWithData(T *data, long storageSize, long storageOffset, int nDimension, \
                                                 const long *size, const long *stride) {                   \
    return (TH##Name##Tensor *)host_new_with_data<T>(data, storageSize, storageOffset, nDimension, size, stride); \
  }                                                                                                          \
  void TH##Name##Tensor_free(TH##Name##Tensor *t) { host_free<T>(t); }
THCL_HOST_STANDIN(Byte, unsigned char)
THCL_HOST_STANDIN(Char, char)
THCL_HOST_STANDIN(Short, short)
THCL_HOST_STANDIN(Int, int)
THCL_HOST_STANDIN(Double, double)
#undef THCL_HOST_STANDIN
#endif

void THClTensor_maskedFillByte(THClState *state, THClTensor *tensor, THByteTensor *mask, float value) {
  THCL_GUARD_BEGIN
  THClTensor *m = upload_mask(state, THClTensor_getDevice(state, tensor), mask);
  try {
    THClTensor_maskedFill(state, tensor, m, value);
  } catch (...) {
    THClTensor_free(state, m);
    throw;
  }
  THClTensor_free(state, m);
  THCL_GUARD_END()
}
void THClTensor_maskedSelectByte(THClState *state, THClTensor *tensor, THClTensor *src, THByteTensor *mask) {
  THCL_GUARD_BEGIN
  THClTensor *m = upload_mask(state, THClTensor_getDevice(state, src), mask);
  try {
    THClTensor_maskedSelect(state, tensor, src, m);
  } catch (...) {
    THClTensor_free(state, m);
    throw;
  }
  THClTensor_free(state, m);
  THCL_GUARD_END()
}
void THClTensor_maskedCopyByte(THClState *state, THClTensor *tensor, THByteTensor *mask, THClTensor *src) {
  THCL_GUARD_BEGIN
  THClTensor *m = upload_mask(state, THClTensor_getDevice(state, tensor), mask);
  try {
    THClTensor_maskedCopy(state, tensor, m, src);
  } catch (...) {
    THClTensor_free(state, m);
    throw;
  }
  THClTensor_free(state, m);
  THCL_GUARD_END()
}

}  // extern "C"
