// Device storages, tensor headers and header-only views.
//
// A storage is a refcounted hipMalloc block (no mandatory host mirror, unlike
// the reference's CLWrapper pair: src/lib/THClStorage.cpp:112-140).  A tensor
// is a refcounted header (sizes, strides, offset) over a storage; narrow /
// select / transpose / unfold only rewrite the header
// (src/lib/THClTensor.cpp:389-520).
#include <cstdarg>
#include <cstdlib>
#include <cstdio>
#include <cstring>
#include <utility>

#include "internal.h"

namespace {
constexpr char kRefcounted = 1, kResizable = 2, kFreeMem = 4;

void storage_release_memory(THClStorage *s) {
  if (s->wrapper) {
    if (thcl_rt_free(s->cl, s->wrapper) != 0) thcl_throw("freeing device storage: %s", thcl_rt_error());
    s->wrapper = nullptr;
  }
  free(s->data);
  s->data = nullptr;
}

THClStorage *storage_new(THClState *state, int device, long size) {
  THCL_ARGCHECK(size >= 0, 2, "invalid size");
  thcl_rt *rt = thcl_ctx(state, device);
  auto *s = (THClStorage *)calloc(1, sizeof(THClStorage));
  s->device = device;
  s->cl = rt;
  s->refcount = 1;
  s->flag = kRefcounted | kResizable | kFreeMem;
  if (size > 0) {
    s->wrapper = thcl_rt_malloc(rt, (size_t)size * sizeof(float));
    if (!s->wrapper) {
      free(s);
      thcl_throw("cannot allocate %ld floats on device %d: %s", size, device, thcl_rt_error());
    }
    s->size = size;
    if (state->trace) fprintf(stderr, "[thcl] new storage, size %ld\n", size);
  }
  return s;
}

// Grows a storage keeping its contents (the reference drops them; keeping them
// is what Torch7's own THStorage_resize does and costs one device copy).
void storage_resize(THClState *state, THClStorage *s, long size) {
  if (size <= s->size) return;
  THCL_CHECK(s->flag & kResizable, "trying to resize a storage that is not resizable");
  thcl_rt *rt = s->cl ? s->cl : thcl_ctx(state, s->device);
  void *fresh = thcl_rt_malloc(rt, (size_t)size * sizeof(float));
  THCL_CHECK(fresh != nullptr, "cannot allocate %ld floats on device %d: %s", size, s->device, thcl_rt_error());
  if (s->wrapper && s->size > 0)
    THCL_CHECK(thcl_rt_memcpy_d2d(rt, fresh, s->wrapper, (size_t)s->size * sizeof(float)) == 0, "%s",
               thcl_rt_error());
  storage_release_memory(s);
  s->cl = rt;
  s->wrapper = fresh;
  s->size = size;
  if (state->trace) fprintf(stderr, "[thcl] storage resized to %ld\n", size);
}

// ----------------------------------------------------------------- headers ---
THClTensor *header_new(int device) {
  auto *t = (THClTensor *)calloc(1, sizeof(THClTensor));
  t->refcount = 1;
  t->nDimension = -1;  // empty header (src/lib/THClTensor.cpp:632-643)
  t->flag = kRefcounted;
  t->device = device;
  return t;
}

// Sets sizes/strides; a non-positive size ends the list (the reference's
// "-1 terminates" convention: src/lib/THClTensor.cpp:671-736).  Strides that
// are NULL or negative default to the contiguous ones.  Grows the storage to
// cover the addressed extent.
void header_resize(THClState *state, THClTensor *t, int nd_in, const long *size, const long *stride) {
  int nd = 0;
  while (nd < nd_in && size[nd] > 0) nd++;
  THCL_CHECK(nd <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  bool same = (nd == t->nDimension);
  for (int d = 0; same && d < nd; d++) {
    if (size[d] != t->size[d]) same = false;
    if (stride && stride[d] >= 0 && stride[d] != t->stride[d]) same = false;
  }
  if (same) return;
  if (nd != t->nDimension) {
    t->size = (long *)realloc(t->size, sizeof(long) * (nd > 0 ? nd : 1));
    t->stride = (long *)realloc(t->stride, sizeof(long) * (nd > 0 ? nd : 1));
    t->nDimension = nd;
  }
  long extent = 1;
  for (int d = nd - 1; d >= 0; d--) {
    t->size[d] = size[d];
    if (stride && stride[d] >= 0) t->stride[d] = stride[d];
    else t->stride[d] = (d == nd - 1) ? 1 : t->size[d + 1] * t->stride[d + 1];
    extent += (t->size[d] - 1) * t->stride[d];
  }
  // nd == 0 leaves extent == 1: a point tensor owns one element
  long need = extent + t->storageOffset;
  if (need > 0) {
    if (!t->storage) t->storage = storage_new(state, t->device, 0);
    if (need > t->storage->size) storage_resize(state, t->storage, need);
  }
}

void header_set(THClState *state, THClTensor *t, THClStorage *storage, long offset, int nd, const long *size,
                const long *stride) {
  if (t->storage != storage) {
    if (t->storage) THClStorage_free(state, t->storage);
    t->storage = storage;
    if (storage) THClStorage_retain(state, storage);
  }
  THCL_CHECK(offset >= 0, "Tensor: invalid storage offset");
  t->storageOffset = offset;
  if (storage) t->device = storage->device;
  if (nd < 0) {  // empty source header: stay empty
    t->nDimension = -1;
    return;
  }
  header_resize(state, t, nd, size, stride);
}
}  // namespace

extern "C" {

// ----------------------------------------------------------------- storage ---
float *THClStorage_data(THClState *, const THClStorage *s) { return s->data; }
long THClStorage_size(THClState *, const THClStorage *s) { return s->size; }

THClStorage *THClStorage_newv2(THClState *state, int device) {
  THCL_GUARD_BEGIN
  return storage_new(state, device, 0);
  THCL_GUARD_END(nullptr)
}
THClStorage *THClStorage_new(THClState *state) { return THClStorage_newv2(state, state->currentDevice); }
THClStorage *THClStorage_newWithSize(THClState *state, int device, long size) {
  THCL_GUARD_BEGIN
  return storage_new(state, device, size);
  THCL_GUARD_END(nullptr)
}
void THClStorage_retain(THClState *, THClStorage *s) {
  if (s && (s->flag & kRefcounted)) __atomic_add_fetch(&s->refcount, 1, __ATOMIC_SEQ_CST);
}
void THClStorage_free(THClState *state, THClStorage *s) {
  THCL_GUARD_BEGIN
  if (!s || !(s->flag & kRefcounted)) return;
  if (__atomic_sub_fetch(&s->refcount, 1, __ATOMIC_SEQ_CST) == 0) {
    if (s->flag & kFreeMem) {
      if (state && state->trace && s->size > 0) fprintf(stderr, "[thcl] delete storage, size %ld\n", s->size);
      storage_release_memory(s);
    }
    free(s);
  }
  THCL_GUARD_END()
}
void THClStorage_resize(THClState *state, THClStorage *s, long size) {
  THCL_GUARD_BEGIN
  storage_resize(state, s, size);
  THCL_GUARD_END()
}
void THClStorage_fill(THClState *state, THClStorage *s, float value) {
  THCL_GUARD_BEGIN
  if (s->size > 0) {
    thcl_fill_contig(s->cl, (float *)s->wrapper, value, s->size);
    thcl_after_launch(state, s->cl);
  }
  THCL_GUARD_END()
}
void THClStorage_set(THClState *state, THClStorage *s, long index, float value) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(index >= 0 && index < s->size, 2, "index out of bounds");
  THCL_ARGCHECK(s->wrapper != nullptr, 1, "storage argument not initialized, is empty");
  THCL_CHECK(thcl_rt_memcpy_h2d(s->cl, (float *)s->wrapper + index, &value, sizeof(float)) == 0, "%s",
             thcl_rt_error());
  THCL_GUARD_END()
}
float THClStorage_get(THClState *state, const THClStorage *s, long index) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(index >= 0 && index < s->size, 2, "index out of bounds");
  THCL_ARGCHECK(s->wrapper != nullptr, 1, "storage argument not initialized, is empty");
  float v = 0.f;
  THCL_CHECK(thcl_rt_memcpy_d2h(s->cl, &v, (const float *)s->wrapper + index, sizeof(float)) == 0, "%s",
             thcl_rt_error());
  return v;
  THCL_GUARD_END(0.f)
}
void THClStorage_rawCopy(THClState *state, THClStorage *s, float *src) {
  THCL_GUARD_BEGIN
  THCL_CHECK(thcl_rt_memcpy_h2d(s->cl, s->wrapper, src, (size_t)s->size * sizeof(float)) == 0, "%s",
             thcl_rt_error());
  THCL_GUARD_END()
}
void THClStorage_copyFloat(THClState *state, THClStorage *s, THFloatStorage *src) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(s->size == src->size, 2, "size mismatch");
  THCL_CHECK(thcl_rt_memcpy_h2d(s->cl, s->wrapper, src->data, (size_t)s->size * sizeof(float)) == 0, "%s",
             thcl_rt_error());
  THCL_GUARD_END()
}
void THFloatStorage_copyCl(THClState *state, THFloatStorage *self, THClStorage *src) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(self->size == src->size, 2, "size mismatch");
  THCL_CHECK(thcl_rt_memcpy_d2h(src->cl, self->data, src->wrapper, (size_t)src->size * sizeof(float)) == 0, "%s",
             thcl_rt_error());
  THCL_GUARD_END()
}

// ----------------------------------------------------------------- tensor ---
THClStorage *THClTensor_storage(THClState *, const THClTensor *self) { return self->storage; }
long THClTensor_storageOffset(THClState *, const THClTensor *self) { return self->storageOffset; }
int THClTensor_nDimension(THClState *, const THClTensor *self) { return self->nDimension; }
long THClTensor_size(THClState *, const THClTensor *self, int dim) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(dim >= 0 && dim < self->nDimension, 2, "out of range");
  return self->size[dim];
  THCL_GUARD_END(0)
}
long THClTensor_stride(THClState *, const THClTensor *self, int dim) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(dim >= 0 && dim < self->nDimension, 2, "out of range");
  return self->stride[dim];
  THCL_GUARD_END(0)
}
THLongStorage *THClTensor_newSizeOf(THClState *, THClTensor *self) {
  int nd = self->nDimension > 0 ? self->nDimension : 0;
  THLongStorage *s = THLongStorage_newWithSize(nd);
  for (int d = 0; d < nd; d++) s->data[d] = self->size[d];
  return s;
}
THLongStorage *THClTensor_newStrideOf(THClState *, THClTensor *self) {
  int nd = self->nDimension > 0 ? self->nDimension : 0;
  THLongStorage *s = THLongStorage_newWithSize(nd);
  for (int d = 0; d < nd; d++) s->data[d] = self->stride[d];
  return s;
}
float *THClTensor_data(THClState *, const THClTensor *self) { return thcl_dptr(self); }

THClTensor *THClTensor_newv2(THClState *state, int device) {
  THCL_GUARD_BEGIN
  THCL_CHECK(device >= 0 && device < state->allocatedDevices, "device %d out of range", device);
  return header_new(device);
  THCL_GUARD_END(nullptr)
}
THClTensor *THClTensor_new(THClState *state) { return THClTensor_newv2(state, state->currentDevice); }

int THClTensor_checkGPU(THClState *, unsigned int nTensors, ...) {
  va_list args;
  va_start(args, nTensors);
  int first = -1, same = 1;
  for (unsigned int i = 0; i < nTensors; i++) {
    const THClTensor *t = va_arg(args, const THClTensor *);
    if (!t) continue;
    if (first < 0) first = t->device;
    if (t->device != first) same = 0;
  }
  va_end(args);
  return same;
}

struct thcl_rt *THClTensor_getCl(THClState *, const THClTensor *tensor) {
  return tensor->storage ? tensor->storage->cl : nullptr;
}
void *THClTensor_wrapper(THClState *, const THClTensor *self) { return self->storage ? self->storage->wrapper : nullptr; }

THClTensor *THClTensor_newWithTensor(THClState *state, THClTensor *tensor) {
  THCL_GUARD_BEGIN
  THClTensor *t = header_new(tensor->device);
  header_set(state, t, tensor->storage, tensor->storageOffset, tensor->nDimension, tensor->size, tensor->stride);
  return t;
  THCL_GUARD_END(nullptr)
}
THClTensor *THClTensor_newWithStorage(THClState *state, int device, THClStorage *storage, long storageOffset,
                                      THLongStorage *size, THLongStorage *stride) {
  THCL_GUARD_BEGIN
  if (size && stride) THCL_ARGCHECK(size->size == stride->size, 4, "inconsistent size");
  THClTensor *t = header_new(device);
  int nd = size ? (int)size->size : (stride ? (int)stride->size : 0);
  header_set(state, t, storage, storageOffset, nd, size ? size->data : nullptr, stride ? stride->data : nullptr);
  return t;
  THCL_GUARD_END(nullptr)
}
// sizes and strides spelled out, -1 from the first dimension that is not there
// (src/lib/THClTensor.cpp:136-171)
THClTensor *THClTensor_newWithStorage4d(THClState *state, int device, THClStorage *storage, long storageOffset, long size0,
                                        long stride0, long size1, long stride1, long size2, long stride2, long size3,
                                        long stride3) {
  THCL_GUARD_BEGIN
  long size[4] = {size0, size1, size2, size3}, stride[4] = {stride0, stride1, stride2, stride3};
  THClTensor *t = header_new(device);
  header_set(state, t, storage, storageOffset, 4, size, stride);
  return t;
  THCL_GUARD_END(nullptr)
}
THClTensor *THClTensor_newWithStorage1d(THClState *state, int device, THClStorage *storage, long storageOffset, long size0,
                                        long stride0) {
  return THClTensor_newWithStorage4d(state, device, storage, storageOffset, size0, stride0, -1, -1, -1, -1, -1, -1);
}
THClTensor *THClTensor_newWithStorage2d(THClState *state, int device, THClStorage *storage, long storageOffset, long size0,
                                        long stride0, long size1, long stride1) {
  return THClTensor_newWithStorage4d(state, device, storage, storageOffset, size0, stride0, size1, stride1, -1, -1, -1, -1);
}
THClTensor *THClTensor_newWithStorage3d(THClState *state, int device, THClStorage *storage, long storageOffset, long size0,
                                        long stride0, long size1, long stride1, long size2, long stride2) {
  return THClTensor_newWithStorage4d(state, device, storage, storageOffset, size0, stride0, size1, stride1, size2, stride2, -1, -1);
}
THClTensor *THClTensor_newWithSize(THClState *state, int device, THLongStorage *size, THLongStorage *stride) {
  return THClTensor_newWithStorage(state, device, nullptr, 0, size, stride);
}
THClTensor *THClTensor_newWithSize4d(THClState *state, int device, long s0, long s1, long s2, long s3) {
  THCL_GUARD_BEGIN
  long size[4] = {s0, s1, s2, s3};
  THClTensor *t = header_new(device);
  header_resize(state, t, 4, size, nullptr);
  return t;
  THCL_GUARD_END(nullptr)
}
THClTensor *THClTensor_newWithSize1d(THClState *state, int device, long s0) {
  return THClTensor_newWithSize4d(state, device, s0, -1, -1, -1);
}
THClTensor *THClTensor_newWithSize2d(THClState *state, int device, long s0, long s1) {
  return THClTensor_newWithSize4d(state, device, s0, s1, -1, -1);
}
THClTensor *THClTensor_newWithSize3d(THClState *state, int device, long s0, long s1, long s2) {
  return THClTensor_newWithSize4d(state, device, s0, s1, s2, -1);
}

THClTensor *THClTensor_newClone(THClState *state, THClTensor *self) {
  THCL_GUARD_BEGIN
  THClTensor *t = header_new(self->storage ? self->storage->device : self->device);
  if (self->nDimension >= 0) header_resize(state, t, self->nDimension, self->size, nullptr);
  try {
    THClTensor_copy(state, t, self);
  } catch (...) {
    THClTensor_free(state, t);
    throw;
  }
  return t;
  THCL_GUARD_END(nullptr)
}
THClTensor *THClTensor_newContiguous(THClState *state, THClTensor *self) {
  if (!THClTensor_isContiguous(state, self)) return THClTensor_newClone(state, self);
  THClTensor_retain(state, self);
  return self;
}
THClTensor *THClTensor_newSelect(THClState *state, THClTensor *tensor, int dimension, long sliceIndex) {
  THClTensor *t = THClTensor_newWithTensor(state, tensor);
  if (t) THClTensor_select(state, t, nullptr, dimension, sliceIndex);
  return t;
}
THClTensor *THClTensor_newNarrow(THClState *state, THClTensor *tensor, int dimension, long firstIndex, long size) {
  THClTensor *t = THClTensor_newWithTensor(state, tensor);
  if (t) THClTensor_narrow(state, t, nullptr, dimension, firstIndex, size);
  return t;
}
THClTensor *THClTensor_newTranspose(THClState *state, THClTensor *tensor, int d1, int d2) {
  THClTensor *t = THClTensor_newWithTensor(state, tensor);
  if (t) THClTensor_transpose(state, t, nullptr, d1, d2);
  return t;
}
THClTensor *THClTensor_newUnfold(THClState *state, THClTensor *tensor, int dimension, long size, long step) {
  THClTensor *t = THClTensor_newWithTensor(state, tensor);
  if (t) THClTensor_unfold(state, t, nullptr, dimension, size, step);
  return t;
}

void THClTensor_resize(THClState *state, THClTensor *self, THLongStorage *size, THLongStorage *stride) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(size != nullptr, 2, "invalid size");
  if (stride) THCL_ARGCHECK(stride->size == size->size, 3, "invalid stride");
  header_resize(state, self, (int)size->size, size->data, stride ? stride->data : nullptr);
  THCL_GUARD_END()
}
void THClTensor_resizeAs(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  if (!THClTensor_isSameSizeAs(state, self, src))
    header_resize(state, self, src->nDimension > 0 ? src->nDimension : 0, src->size, nullptr);
  THCL_GUARD_END()
}
void THClTensor_resize4d(THClState *state, THClTensor *self, long s0, long s1, long s2, long s3) {
  THCL_GUARD_BEGIN
  long size[4] = {s0, s1, s2, s3};
  header_resize(state, self, 4, size, nullptr);
  THCL_GUARD_END()
}
void THClTensor_resize0d(THClState *state, THClTensor *self) { THClTensor_resize4d(state, self, -1, -1, -1, -1); }
void THClTensor_resize1d(THClState *state, THClTensor *self, long s0) { THClTensor_resize4d(state, self, s0, -1, -1, -1); }
void THClTensor_resize2d(THClState *state, THClTensor *self, long s0, long s1) {
  THClTensor_resize4d(state, self, s0, s1, -1, -1);
}
void THClTensor_resize3d(THClState *state, THClTensor *self, long s0, long s1, long s2) {
  THClTensor_resize4d(state, self, s0, s1, s2, -1);
}

void THClTensor_set(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  if (self != src) {
    header_set(state, self, src->storage, src->storageOffset, src->nDimension, src->size, src->stride);
  }
  THCL_GUARD_END()
}
void THClTensor_setStorage(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset,
                           THLongStorage *size, THLongStorage *stride) {
  THCL_GUARD_BEGIN
  if (size && stride) THCL_ARGCHECK(size->size == stride->size, 5, "inconsistent size/stride sizes");
  int nd = size ? (int)size->size : (stride ? (int)stride->size : 0);
  header_set(state, self, storage, storageOffset, nd, size ? size->data : nullptr, stride ? stride->data : nullptr);
  THCL_GUARD_END()
}

// (src/lib/THClTensor.cpp:342-386)
void THClTensor_setStorage4d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset, long size0,
                             long stride0, long size1, long stride1, long size2, long stride2, long size3, long stride3) {
  THCL_GUARD_BEGIN
  long size[4] = {size0, size1, size2, size3}, stride[4] = {stride0, stride1, stride2, stride3};
  header_set(state, self, storage, storageOffset, 4, size, stride);
  THCL_GUARD_END()
}
void THClTensor_setStorage1d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset, long size0,
                             long stride0) {
  THClTensor_setStorage4d(state, self, storage, storageOffset, size0, stride0, -1, -1, -1, -1, -1, -1);
}
void THClTensor_setStorage2d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset, long size0,
                             long stride0, long size1, long stride1) {
  THClTensor_setStorage4d(state, self, storage, storageOffset, size0, stride0, size1, stride1, -1, -1, -1, -1);
}
void THClTensor_setStorage3d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset, long size0,
                             long stride0, long size1, long stride1, long size2, long stride2) {
  THClTensor_setStorage4d(state, self, storage, storageOffset, size0, stride0, size1, stride1, size2, stride2, -1, -1);
}

void THClTensor_narrow(THClState *state, THClTensor *self, THClTensor *src, int dim, long first, long size) {
  THCL_GUARD_BEGIN
  if (!src) src = self;
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 3, "out of range");
  THCL_ARGCHECK(first >= 0 && first < src->size[dim], 4, "out of range");
  THCL_ARGCHECK(size > 0 && first + size <= src->size[dim], 5, "out of range");
  THClTensor_set(state, self, src);
  self->storageOffset += first * self->stride[dim];
  self->size[dim] = size;
  THCL_GUARD_END()
}
void THClTensor_select(THClState *state, THClTensor *self, THClTensor *src, int dim, long index) {
  THCL_GUARD_BEGIN
  if (!src) src = self;
  THCL_ARGCHECK(src->nDimension > 1, 1, "cannot select on a vector");
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 3, "out of range");
  THCL_ARGCHECK(index >= 0 && index < src->size[dim], 4, "out of range");
  THClTensor_set(state, self, src);
  self->storageOffset += index * self->stride[dim];
  for (int d = dim; d < self->nDimension - 1; d++) {
    self->size[d] = self->size[d + 1];
    self->stride[d] = self->stride[d + 1];
  }
  self->nDimension--;
  THCL_GUARD_END()
}
void THClTensor_transpose(THClState *state, THClTensor *self, THClTensor *src, int d1, int d2) {
  THCL_GUARD_BEGIN
  if (!src) src = self;
  THCL_ARGCHECK(d1 >= 0 && d1 < src->nDimension, 1, "out of range");
  THCL_ARGCHECK(d2 >= 0 && d2 < src->nDimension, 2, "out of range");
  THClTensor_set(state, self, src);
  if (d1 != d2) {
    std::swap(self->stride[d1], self->stride[d2]);
    std::swap(self->size[d1], self->size[d2]);
  }
  THCL_GUARD_END()
}
void THClTensor_unfold(THClState *state, THClTensor *self, THClTensor *src, int dim, long size, long step) {
  // windows of `size` every `step` along `dim`; the window becomes a new last
  // dimension (src/lib/THClTensor.cpp:465-512)
  THCL_GUARD_BEGIN
  if (!src) src = self;
  THCL_ARGCHECK(src->nDimension > 0, 1, "cannot unfold an empty tensor");
  THCL_ARGCHECK(dim >= 0 && dim < src->nDimension, 2, "out of range");
  THCL_ARGCHECK(size <= src->size[dim], 3, "out of range");
  THCL_ARGCHECK(step > 0, 4, "invalid step");
  THClTensor_set(state, self, src);
  int nd = self->nDimension;
  THCL_CHECK(nd + 1 <= THCL_MAX_DIMS, THCL_DIM_WARNING);
  long *nsz = (long *)malloc(sizeof(long) * (nd + 1));
  long *nst = (long *)malloc(sizeof(long) * (nd + 1));
  nsz[nd] = size;
  nst[nd] = self->stride[dim];
  for (int d = 0; d < nd; d++) {
    if (d == dim) {
      nsz[d] = (self->size[d] - size) / step + 1;
      nst[d] = step * self->stride[d];
    } else {
      nsz[d] = self->size[d];
      nst[d] = self->stride[d];
    }
  }
  free(self->size);
  free(self->stride);
  self->size = nsz;
  self->stride = nst;
  self->nDimension = nd + 1;
  THCL_GUARD_END()
}
void THClTensor_squeeze(THClState *state, THClTensor *self, THClTensor *src) {
  THCL_GUARD_BEGIN
  if (!src) src = self;
  THClTensor_set(state, self, src);
  int k = 0;
  for (int d = 0; d < src->nDimension; d++) {
    if (src->size[d] != 1) {
      if (d != k) {
        self->size[k] = src->size[d];
        self->stride[k] = src->stride[d];
      }
      k++;
    }
  }
  // a tensor of one element stays 1-d with that element
  if (k == 0 && src->nDimension > 0) {
    self->size[0] = 1;
    self->stride[0] = 1;
    k = 1;
  }
  self->nDimension = k;
  THCL_GUARD_END()
}

int THClTensor_isContiguous(THClState *, const THClTensor *self) {
  long z = 1;
  for (int d = self->nDimension - 1; d >= 0; d--) {
    if (self->size[d] == 1) continue;
    if (self->stride[d] != z) return 0;
    z *= self->size[d];
  }
  return 1;
}
int THClTensor_isSameSizeAs(THClState *, const THClTensor *self, const THClTensor *src) {
  if (self->nDimension != src->nDimension) return 0;
  for (int d = 0; d < self->nDimension; d++)
    if (self->size[d] != src->size[d]) return 0;
  return 1;
}
long THClTensor_nElement(THClState *, const THClTensor *self) {
  // a point tensor reports 0 elements (src/lib/THClTensor.cpp:580-592)
  if (self->nDimension <= 0) return 0;
  long n = 1;
  for (int d = 0; d < self->nDimension; d++) n *= self->size[d];
  return n;
}
void THClTensor_retain(THClState *, THClTensor *self) {
  if (self->flag & kRefcounted) __atomic_add_fetch(&self->refcount, 1, __ATOMIC_SEQ_CST);
}
void THClTensor_free(THClState *state, THClTensor *self) {
  if (!self || !(self->flag & kRefcounted)) return;
  if (__atomic_sub_fetch(&self->refcount, 1, __ATOMIC_SEQ_CST) == 0) {
    free(self->size);
    free(self->stride);
    if (self->storage) THClStorage_free(state, self->storage);
    free(self);
  }
}
void THClTensor_freeCopyTo(THClState *state, THClTensor *self, THClTensor *dst) {
  if (self != dst) THClTensor_copy(state, dst, self);
  THClTensor_free(state, self);
}
int THClTensor_getDevice(THClState *, const THClTensor *self) {
  return self->storage ? self->storage->device : self->device;
}

void THClTensor_set1d(THClState *state, THClTensor *t, long x0, float value) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 1, 1, "tensor must have one dimension");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0], 2, "out of range");
  THClStorage_set(state, t->storage, t->storageOffset + x0 * t->stride[0], value);
  THCL_GUARD_END()
}
void THClTensor_set2d(THClState *state, THClTensor *t, long x0, long x1, float value) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 2, 1, "tensor must have two dimensions");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0] && x1 >= 0 && x1 < t->size[1], 2, "out of range");
  THClStorage_set(state, t->storage, t->storageOffset + x0 * t->stride[0] + x1 * t->stride[1], value);
  THCL_GUARD_END()
}
float THClTensor_get1d(THClState *state, const THClTensor *t, long x0) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 1, 1, "tensor must have one dimension");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0], 2, "out of range");
  return THClStorage_get(state, t->storage, t->storageOffset + x0 * t->stride[0]);
  THCL_GUARD_END(0.f)
}
float THClTensor_get2d(THClState *state, const THClTensor *t, long x0, long x1) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 2, 1, "tensor must have two dimensions");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0] && x1 >= 0 && x1 < t->size[1], 2, "out of range");
  return THClStorage_get(state, t->storage, t->storageOffset + x0 * t->stride[0] + x1 * t->stride[1]);
  THCL_GUARD_END(0.f)
}

// ---- the rest of the header / storage interface (src/lib/THClTensor.h:31-145,
//      src/lib/THClStorage.h:28-59, src/lib/THClStorageCopy.h:9-30)
void THClTensor_setFlag(THClState *, THClTensor *self, const char flag) { self->flag |= flag; }
void THClTensor_clearFlag(THClState *, THClTensor *self, const char flag) { self->flag &= ~flag; }
void THClStorage_setFlag(THClState *, THClStorage *s, const char flag) { s->flag |= flag; }
void THClStorage_clearFlag(THClState *, THClStorage *s, const char flag) { s->flag &= ~flag; }

void THClTensor_resize5d(THClState *state, THClTensor *self, long s0, long s1, long s2, long s3, long s4) {
  THCL_GUARD_BEGIN
  long size[5] = {s0, s1, s2, s3, s4};
  header_resize(state, self, 5, size, nullptr);
  THCL_GUARD_END()
}
// drops `dimension` when its size is 1 (src/lib/THClTensor.cpp:528-548)
void THClTensor_squeeze1d(THClState *state, THClTensor *self, THClTensor *src, int dimension) {
  THCL_GUARD_BEGIN
  if (!src) src = self;
  THCL_ARGCHECK(dimension >= 0 && dimension < src->nDimension, 3, "dimension out of range");
  THClTensor_set(state, self, src);
  if (src->size[dimension] == 1 && src->nDimension > 1) {
    for (int d = dimension; d < self->nDimension - 1; d++) {
      self->size[d] = self->size[d + 1];
      self->stride[d] = self->stride[d + 1];
    }
    self->nDimension--;
  }
  THCL_GUARD_END()
}
void THClTensor_set3d(THClState *state, THClTensor *t, long x0, long x1, long x2, float value) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 3, 1, "tensor must have three dimensions");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0] && x1 >= 0 && x1 < t->size[1] && x2 >= 0 && x2 < t->size[2], 2, "out of range");
  THClStorage_set(state, t->storage, t->storageOffset + x0 * t->stride[0] + x1 * t->stride[1] + x2 * t->stride[2], value);
  THCL_GUARD_END()
}
float THClTensor_get3d(THClState *state, const THClTensor *t, long x0, long x1, long x2) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 3, 1, "tensor must have three dimensions");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0] && x1 >= 0 && x1 < t->size[1] && x2 >= 0 && x2 < t->size[2], 2, "out of range");
  return THClStorage_get(state, t->storage, t->storageOffset + x0 * t->stride[0] + x1 * t->stride[1] + x2 * t->stride[2]);
  THCL_GUARD_END(0.f)
}
void THClTensor_set4d(THClState *state, THClTensor *t, long x0, long x1, long x2, long x3, float value) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 4, 1, "tensor must have four dimensions");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0] && x1 >= 0 && x1 < t->size[1] && x2 >= 0 && x2 < t->size[2] && x3 >= 0 &&
                    x3 < t->size[3],
                2, "out of range");
  THClStorage_set(state, t->storage,
                  t->storageOffset + x0 * t->stride[0] + x1 * t->stride[1] + x2 * t->stride[2] + x3 * t->stride[3], value);
  THCL_GUARD_END()
}
float THClTensor_get4d(THClState *state, const THClTensor *t, long x0, long x1, long x2, long x3) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(t->nDimension == 4, 1, "tensor must have four dimensions");
  THCL_ARGCHECK(x0 >= 0 && x0 < t->size[0] && x1 >= 0 && x1 < t->size[1] && x2 >= 0 && x2 < t->size[2] && x3 >= 0 &&
                    x3 < t->size[3],
                2, "out of range");
  return THClStorage_get(state, t->storage,
                         t->storageOffset + x0 * t->stride[0] + x1 * t->stride[1] + x2 * t->stride[2] + x3 * t->stride[3]);
  THCL_GUARD_END(0.f)
}
// device to device, whole storages (src/lib/THClStorageCopy.cpp:17-25)
void THClStorage_copy(THClState *state, THClStorage *self, THClStorage *src) {
  THCL_GUARD_BEGIN
  THCL_ARGCHECK(self->size == src->size, 2, "size does not match");
  THCL_CHECK(self->device == src->device, "copy between devices is not implemented");
  if (self->size > 0 && self != src)
    THCL_CHECK(thcl_rt_memcpy_d2d(self->cl, self->wrapper, src->wrapper, (size_t)self->size * sizeof(float)) == 0, "%s",
               thcl_rt_error());
  THCL_GUARD_END()
}

}  // extern "C"
