/*
 * C ABI of the MI355X tensor backend: the entry points the Lua/C binding layer
 * of cltorch (cwrap-generated TensorMath.c, Tensor.cpp, Storage.cpp) binds for
 * the pointwise / copy / reduce / addmm path.  Names, argument order and
 * argument meaning are those of the reference's `THCL_API` functions; each
 * declaration cites the reference interface it replaces.  Dimensions are
 * 0-based here (the Lua layer subtracts 1), sizes/strides are `long` counts of
 * elements, the element type is fp32.
 *
 * Every function is `extern "C"`, takes plain pointers and sizes, and never
 * lets a C++ exception escape: a failed check calls the installed error
 * handler (THClSetErrorHandler) and records the message for THClLastError().
 */
#ifndef THCL_HIP_H
#define THCL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the library is built with hidden visibility: what is declared here is what it exports */
#pragma GCC visibility push(default)

/* ------------------------------------------------------------------------- */
/* Torch7 `TH` stand-ins.  Field order matches TH's own structs, so objects   */
/* made by a real libTH can be passed in; with a real Torch7 the definitions  */
/* come from <TH/TH.h> instead (build with -DTHCL_EXTERNAL_TH).               */
/* ------------------------------------------------------------------------- */
#ifndef THCL_EXTERNAL_TH
typedef struct THLongStorage {
  long *data;
  long size;
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct THLongStorage *view;
} THLongStorage;

typedef struct THFloatStorage {
  float *data;
  long size;
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct THFloatStorage *view;
} THFloatStorage;

typedef struct THFloatTensor {
  long *size;
  long *stride;
  int nDimension;
  THFloatStorage *storage;
  long storageOffset;
  int refcount;
  char flag;
} THFloatTensor;

typedef struct THLongTensor {
  long *size;
  long *stride;
  int nDimension;
  THLongStorage *storage;
  long storageOffset;
  int refcount;
  char flag;
} THLongTensor;

/* host tensors of the other element types: same layout, element type aside */
#define THCL_DECLARE_HOST_TENSOR(Name, T)                                        \
  typedef struct TH##Name##Storage {                                             \
    T *data;                                                                     \
    long size;                                                                   \
    int refcount;                                                                \
    char flag;                                                                   \
    void *allocator;                                                             \
    void *allocatorContext;                                                      \
    struct TH##Name##Storage *view;                                              \
  } TH##Name##Storage;                                                           \
  typedef struct TH##Name##Tensor {                                              \
    long *size;                                                                  \
    long *stride;                                                                \
    int nDimension;                                                              \
    TH##Name##Storage *storage;                                                  \
    long storageOffset;                                                          \
    int refcount;                                                                \
    char flag;                                                                   \
  } TH##Name##Tensor;
THCL_DECLARE_HOST_TENSOR(Byte, unsigned char)
THCL_DECLARE_HOST_TENSOR(Char, char)
THCL_DECLARE_HOST_TENSOR(Short, short)
THCL_DECLARE_HOST_TENSOR(Int, int)
THCL_DECLARE_HOST_TENSOR(Double, double)
#undef THCL_DECLARE_HOST_TENSOR
/* borrow `data` (not freed with the tensor): strided host views for the copies below */
THByteTensor *THByteTensor_newWithData(unsigned char *data, long storageSize, long storageOffset, int nDimension, const long *size, const long *stride);
THCharTensor *THCharTensor_newWithData(char *data, long storageSize, long storageOffset, int nDimension, const long *size, const long *stride);
THShortTensor *THShortTensor_newWithData(short *data, long storageSize, long storageOffset, int nDimension, const long *size, const long *stride);
THIntTensor *THIntTensor_newWithData(int *data, long storageSize, long storageOffset, int nDimension, const long *size, const long *stride);
THDoubleTensor *THDoubleTensor_newWithData(double *data, long storageSize, long storageOffset, int nDimension, const long *size, const long *stride);
void THByteTensor_free(THByteTensor *t);
void THCharTensor_free(THCharTensor *t);
void THShortTensor_free(THShortTensor *t);
void THIntTensor_free(THIntTensor *t);
void THDoubleTensor_free(THDoubleTensor *t);

THLongStorage *THLongStorage_newWithSize(long size);
void THLongStorage_free(THLongStorage *s);
void THLongStorage_set(THLongStorage *s, long i, long v);
long THLongStorage_get(const THLongStorage *s, long i);

THFloatTensor *THFloatTensor_newWithSize(THLongStorage *size, THLongStorage *stride);
/* borrows `data` (not freed with the tensor): a strided host view */
THFloatTensor *THFloatTensor_newWithData(float *data, long storageSize, long storageOffset, int nDimension,
                                         const long *size, const long *stride);
void THFloatTensor_free(THFloatTensor *t);
long THFloatTensor_nElement(const THFloatTensor *t);
THLongTensor *THLongTensor_newWithSize(THLongStorage *size, THLongStorage *stride);
void THLongTensor_free(THLongTensor *t);
long THLongTensor_nElement(const THLongTensor *t);
#endif

/* ------------------------------------------------------------------------- */
/* State (reference: src/lib/THClGeneral.h:70-131)                            */
/* ------------------------------------------------------------------------- */
struct thcl_rt; /* per-device HIP runtime context, see thcl_rt.h */

typedef struct THClScratchSpace {
  void *wrapper; /* device pointer of the per-device scratch block */
  float *data;   /* pinned host word used to hand scalars back     */
} THClScratchSpace;

typedef struct THClState {
  int initialized;
  int allowNonGpus;
  int allocatedDevices;
  int currentDevice;
  int trace;
  int addFinish; /* 1: synchronise after every launch (debugging) */
  int detailedTimings;
  struct THClScratchSpace **scratchSpaceByDevice;
  void **deviceInfoByDevice;
  struct thcl_rt **clByDevice;
} THClState;

/* src/lib/THClGeneral.h:95-98, src/lib/THClGeneral.cpp:29-96 */
void THCl_initializeState(THClState *state);
void THClSetAllowNonGpus(THClState *state, int allowNonGpus);
void THClInit(THClState *state);
void THClShutdown(THClState *state);
/* src/lib/THClGeneral.h:101-107 */
int THClState_getNumDevices(THClState *state);
void THClState_setDevice(THClState *state, int device);
int THClState_getDevice(THClState *state);
struct thcl_rt *THClState_getClv2(THClState *state, int device);
/* src/lib/THClGeneral.h:128-131 */
struct THClScratchSpace *THClState_getDeviceScratchSpace(THClState *state, int device, int stream);
size_t THClState_getDeviceScratchSpaceSize(THClState *state, int device);
/* Forms the reference keeps for old callers, all acting on the current device
 * (src/lib/THClGeneral.h:105-106,128,130; src/lib/THClGeneral.cpp:119-133,178-185). */
struct thcl_rt *THClState_getCl(THClState *state);
struct thcl_rt *THClState_getClAndDevice(THClState *state, int *p_device);
struct THClScratchSpace *THClState_getCurrentDeviceScratchSpace(THClState *state);
size_t THClState_getCurrentDeviceScratchSpaceSize(THClState *state);
/* `cltorch.setProfiling(on)` / `cltorch.dumpProfiling()` (src/init.cpp:149-178): while on,
 * every launch is timed with HIP events and booked under the entry point that
 * made it.  dumpProfiling waits for the device, writes "entry point, launches,
 * total ms, mean ms" lines into buf (NUL-terminated within cap), forgets the
 * records and returns the length of the full report. */
void THClState_setProfiling(THClState *state, int on);
long THClState_dumpProfiling(THClState *state, char *buf, long cap);
/* `cltorch.synchronize()` / `cltorch.finish()`: src/init.cpp:72-78 */
void THClState_synchronize(THClState *state);

/* Error reporting: the reference raises through Torch7's THError/THArgCheck
 * (src/lib/THClKernels.cpp:23-29, src/lib/THClTensorMath.cpp:19-24).  Here a
 * failed check records its message, calls the handler if one is installed and
 * returns from the entry point without touching its outputs further. */
typedef void (*THClErrorHandler)(const char *msg, void *data);
void THClSetErrorHandler(THClErrorHandler handler, void *data);
const char *THClLastError(void); /* NULL when the last call succeeded */
void THClClearError(void);

/* ------------------------------------------------------------------------- */
/* Storage (reference: src/lib/THClStorage.h:13-59)                           */
/* ------------------------------------------------------------------------- */
typedef struct THClStorage {
  int device;
  float *data;           /* host mirror; NULL unless a caller asked for one */
  struct thcl_rt *cl;    /* runtime context of `device`                     */
  void *wrapper;         /* device pointer (hipMalloc)                      */
  long size;             /* elements                                        */
  int refcount;
  char flag;
  void *allocator;
  void *allocatorContext;
  struct THClStorage *view;
} THClStorage;

float *THClStorage_data(THClState *state, const THClStorage *s);
long THClStorage_size(THClState *state, const THClStorage *s);
void THClStorage_set(THClState *state, THClStorage *s, long index, float value);
float THClStorage_get(THClState *state, const THClStorage *s, long index);
THClStorage *THClStorage_newv2(THClState *state, int device);
/* on the current device (src/lib/THClStorage.cpp:93-96) */
THClStorage *THClStorage_new(THClState *state);
THClStorage *THClStorage_newWithSize(THClState *state, int device, long size);
void THClStorage_retain(THClState *state, THClStorage *s);
void THClStorage_free(THClState *state, THClStorage *s);
void THClStorage_resize(THClState *state, THClStorage *s, long size);
void THClStorage_fill(THClState *state, THClStorage *s, float value);
void THClStorage_setFlag(THClState *state, THClStorage *s, const char flag);
void THClStorage_clearFlag(THClState *state, THClStorage *s, const char flag);
/* whole-storage copies: device to device, and host storages of every element
 * type both ways (src/lib/THClStorageCopy.h:9-30) */
void THClStorage_copy(THClState *state, THClStorage *self, THClStorage *src);
void THClStorage_copyByte(THClState *state, THClStorage *self, THByteStorage *src);
void THClStorage_copyChar(THClState *state, THClStorage *self, THCharStorage *src);
void THClStorage_copyShort(THClState *state, THClStorage *self, THShortStorage *src);
void THClStorage_copyInt(THClState *state, THClStorage *self, THIntStorage *src);
void THClStorage_copyLong(THClState *state, THClStorage *self, THLongStorage *src);
void THClStorage_copyDouble(THClState *state, THClStorage *self, THDoubleStorage *src);
void THByteStorage_copyCl(THClState *state, THByteStorage *self, THClStorage *src);
void THCharStorage_copyCl(THClState *state, THCharStorage *self, THClStorage *src);
void THShortStorage_copyCl(THClState *state, THShortStorage *self, THClStorage *src);
void THIntStorage_copyCl(THClState *state, THIntStorage *self, THClStorage *src);
void THLongStorage_copyCl(THClState *state, THLongStorage *self, THClStorage *src);
void THDoubleStorage_copyCl(THClState *state, THDoubleStorage *self, THClStorage *src);
/* src/lib/THClStorageCopy.h:9-10,27 */
void THClStorage_rawCopy(THClState *state, THClStorage *s, float *src);
void THClStorage_copyFloat(THClState *state, THClStorage *s, THFloatStorage *src);
void THFloatStorage_copyCl(THClState *state, THFloatStorage *self, THClStorage *src);

/* ------------------------------------------------------------------------- */
/* Tensor header and views (reference: src/lib/THClTensor.h:14-145)           */
/* ------------------------------------------------------------------------- */
typedef struct THClTensor {
  long *size;
  long *stride;
  int nDimension; /* -1: empty header, 0: point tensor (one element of storage) */
  THClStorage *storage;
  long storageOffset;
  int refcount;
  char flag;
  int device;
} THClTensor;

THClStorage *THClTensor_storage(THClState *state, const THClTensor *self);
long THClTensor_storageOffset(THClState *state, const THClTensor *self);
int THClTensor_nDimension(THClState *state, const THClTensor *self);
long THClTensor_size(THClState *state, const THClTensor *self, int dim);
long THClTensor_stride(THClState *state, const THClTensor *self, int dim);
THLongStorage *THClTensor_newSizeOf(THClState *state, THClTensor *self);
THLongStorage *THClTensor_newStrideOf(THClState *state, THClTensor *self);
/* device address of the first element (the reference returns its host mirror) */
float *THClTensor_data(THClState *state, const THClTensor *self);

THClTensor *THClTensor_newv2(THClState *state, int device);
/* on the current device (src/lib/THClTensor.cpp:92-95) */
THClTensor *THClTensor_new(THClState *state);
/* 1 when every non-NULL tensor of the nTensors that follow lives on one device
 * (src/lib/THClTensor.cpp:844-873) */
int THClTensor_checkGPU(THClState *state, unsigned int nTensors, ...);
/* the runtime context of the tensor's storage (src/lib/THClTensor.cpp:900-902) and the
 * device address of that storage's first element, NULL without a storage
 * (src/lib/THClTensor.cpp:66-72: the reference hands out its buffer wrapper) */
struct thcl_rt *THClTensor_getCl(THClState *state, const THClTensor *tensor);
void *THClTensor_wrapper(THClState *state, const THClTensor *self);
THClTensor *THClTensor_newWithTensor(THClState *state, THClTensor *tensor);
THClTensor *THClTensor_newWithStorage(THClState *state, int device, THClStorage *storage, long storageOffset,
                                      THLongStorage *size, THLongStorage *stride);
/* sizes and strides spelled out; -1 from the first dimension that is not there (src/lib/THClTensor.h:53-66) */
THClTensor *THClTensor_newWithStorage1d(THClState *state, int device, THClStorage *storage, long storageOffset,
                                        long size0, long stride0);
THClTensor *THClTensor_newWithStorage2d(THClState *state, int device, THClStorage *storage, long storageOffset,
                                        long size0, long stride0, long size1, long stride1);
THClTensor *THClTensor_newWithStorage3d(THClState *state, int device, THClStorage *storage, long storageOffset,
                                        long size0, long stride0, long size1, long stride1, long size2, long stride2);
THClTensor *THClTensor_newWithStorage4d(THClState *state, int device, THClStorage *storage, long storageOffset,
                                        long size0, long stride0, long size1, long stride1, long size2, long stride2,
                                        long size3, long stride3);
THClTensor *THClTensor_newWithSize(THClState *state, int device, THLongStorage *size, THLongStorage *stride);
THClTensor *THClTensor_newWithSize1d(THClState *state, int device, long size0);
THClTensor *THClTensor_newWithSize2d(THClState *state, int device, long size0, long size1);
THClTensor *THClTensor_newWithSize3d(THClState *state, int device, long size0, long size1, long size2);
THClTensor *THClTensor_newWithSize4d(THClState *state, int device, long size0, long size1, long size2, long size3);
THClTensor *THClTensor_newClone(THClState *state, THClTensor *self);
THClTensor *THClTensor_newContiguous(THClState *state, THClTensor *self);
THClTensor *THClTensor_newSelect(THClState *state, THClTensor *tensor, int dimension, long sliceIndex);
THClTensor *THClTensor_newNarrow(THClState *state, THClTensor *tensor, int dimension, long firstIndex, long size);
THClTensor *THClTensor_newTranspose(THClState *state, THClTensor *tensor, int dimension1, int dimension2);
THClTensor *THClTensor_newUnfold(THClState *state, THClTensor *tensor, int dimension, long size, long step);

void THClTensor_resize(THClState *state, THClTensor *self, THLongStorage *size, THLongStorage *stride);
void THClTensor_resizeAs(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_resize0d(THClState *state, THClTensor *self);
void THClTensor_setFlag(THClState *state, THClTensor *self, const char flag);
void THClTensor_clearFlag(THClState *state, THClTensor *self, const char flag);
void THClTensor_resize5d(THClState *state, THClTensor *self, long size0, long size1, long size2, long size3, long size4);
void THClTensor_squeeze1d(THClState *state, THClTensor *self, THClTensor *src, int dimension);
void THClTensor_set3d(THClState *state, THClTensor *tensor, long x0, long x1, long x2, float value);
float THClTensor_get3d(THClState *state, const THClTensor *tensor, long x0, long x1, long x2);
void THClTensor_set4d(THClState *state, THClTensor *tensor, long x0, long x1, long x2, long x3, float value);
float THClTensor_get4d(THClState *state, const THClTensor *tensor, long x0, long x1, long x2, long x3);
void THClTensor_resize1d(THClState *state, THClTensor *self, long size0);
void THClTensor_resize2d(THClState *state, THClTensor *self, long size0, long size1);
void THClTensor_resize3d(THClState *state, THClTensor *self, long size0, long size1, long size2);
void THClTensor_resize4d(THClState *state, THClTensor *self, long size0, long size1, long size2, long size3);

void THClTensor_set(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_setStorage(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset,
                           THLongStorage *size, THLongStorage *stride);
/* (src/lib/THClTensor.h:93-106) */
void THClTensor_setStorage1d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset,
                             long size0, long stride0);
void THClTensor_setStorage2d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset,
                             long size0, long stride0, long size1, long stride1);
void THClTensor_setStorage3d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset,
                             long size0, long stride0, long size1, long stride1, long size2, long stride2);
void THClTensor_setStorage4d(THClState *state, THClTensor *self, THClStorage *storage, long storageOffset,
                             long size0, long stride0, long size1, long stride1, long size2, long stride2,
                             long size3, long stride3);
void THClTensor_narrow(THClState *state, THClTensor *self, THClTensor *src, int dimension, long firstIndex, long size);
void THClTensor_select(THClState *state, THClTensor *self, THClTensor *src, int dimension, long sliceIndex);
void THClTensor_transpose(THClState *state, THClTensor *self, THClTensor *src, int dimension1, int dimension2);
void THClTensor_unfold(THClState *state, THClTensor *self, THClTensor *src, int dimension, long size, long step);
void THClTensor_squeeze(THClState *state, THClTensor *self, THClTensor *src);

int THClTensor_isContiguous(THClState *state, const THClTensor *self);
int THClTensor_isSameSizeAs(THClState *state, const THClTensor *self, const THClTensor *src);
long THClTensor_nElement(THClState *state, const THClTensor *self);
void THClTensor_retain(THClState *state, THClTensor *self);
void THClTensor_free(THClState *state, THClTensor *self);
void THClTensor_freeCopyTo(THClState *state, THClTensor *self, THClTensor *dst);
int THClTensor_getDevice(THClState *state, const THClTensor *self);

void THClTensor_set1d(THClState *state, THClTensor *t, long x0, float value);
void THClTensor_set2d(THClState *state, THClTensor *t, long x0, long x1, float value);
float THClTensor_get1d(THClState *state, const THClTensor *t, long x0);
float THClTensor_get2d(THClState *state, const THClTensor *t, long x0, long x1);

/* ------------------------------------------------------------------------- */
/* Copies (reference: src/lib/THClTensorCopy.h:7-23)                          */
/* ------------------------------------------------------------------------- */
void THClTensor_copy(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_copyCl(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_copyFloat(THClState *state, THClTensor *self, THFloatTensor *src);
void THClTensor_copyLong(THClState *state, THClTensor *self, THLongTensor *src);
void THFloatTensor_copyCl(THClState *state, THFloatTensor *self, THClTensor *src);
void THLongTensor_copyCl(THClState *state, THLongTensor *self, THClTensor *src);
/* the other host element types convert through float, as in the reference
 * (src/lib/THClTensorCopy.h:8-22, src/lib/THClTensorCopy.cpp:38-66,93-128) */
void THClTensor_copyByte(THClState *state, THClTensor *self, THByteTensor *src);
void THClTensor_copyChar(THClState *state, THClTensor *self, THCharTensor *src);
void THClTensor_copyShort(THClState *state, THClTensor *self, THShortTensor *src);
void THClTensor_copyInt(THClState *state, THClTensor *self, THIntTensor *src);
void THClTensor_copyDouble(THClState *state, THClTensor *self, THDoubleTensor *src);
void THByteTensor_copyCl(THClState *state, THByteTensor *self, THClTensor *src);
void THCharTensor_copyCl(THClState *state, THCharTensor *self, THClTensor *src);
void THShortTensor_copyCl(THClState *state, THShortTensor *self, THClTensor *src);
void THIntTensor_copyCl(THClState *state, THIntTensor *self, THClTensor *src);
void THDoubleTensor_copyCl(THClState *state, THDoubleTensor *self, THClTensor *src);

/* ------------------------------------------------------------------------- */
/* Pointwise (reference: src/lib/THClTensorMath.h:7-28,98-155)                */
/* `self == src` is the in-place form; otherwise `self` is resized to `src`.  */
/* ------------------------------------------------------------------------- */
void THClTensor_fill(THClState *state, THClTensor *self, float value);
void THClTensor_zero(THClState *state, THClTensor *self);
void THClTensor_fill_gpu(THClState *state, THClTensor *self, THClTensor *value);
void THClTensor_zeros(THClState *state, THClTensor *r_, THLongStorage *size);
void THClTensor_ones(THClState *state, THClTensor *r_, THLongStorage *size);
long THClTensor_numel(THClState *state, THClTensor *t);
void THClTensor_reshape(THClState *state, THClTensor *r_, THClTensor *t, THLongStorage *size);

void THClTensor_add(THClState *state, THClTensor *self, THClTensor *src, float value);
void THClTensor_sub(THClState *state, THClTensor *self, THClTensor *src, float value);
void THClTensor_mul(THClState *state, THClTensor *self, THClTensor *src, float value);
/* element-wise true division, as Torch7's CPU path computes it (the OpenCL
 * reference multiplies by 1.0f/value: src/lib/THClTensorMathPairwise.cpp:223-241) */
void THClTensor_div(THClState *state, THClTensor *self, THClTensor *src, float value);

void THClTensor_cadd(THClState *state, THClTensor *self, THClTensor *src1, float value, THClTensor *src2);
void THClTensor_csub(THClState *state, THClTensor *self, THClTensor *src1, float value, THClTensor *src2);
void THClTensor_cmul(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2);
void THClTensor_cdiv(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2);
void THClTensor_addcmul(THClState *state, THClTensor *self, THClTensor *t, float value, THClTensor *src1, THClTensor *src2);
void THClTensor_addcdiv(THClState *state, THClTensor *self, THClTensor *t, float value, THClTensor *src1, THClTensor *src2);

/* scalar operand held on the device as a point tensor (0-dim, 1 element) */
void THClTensor_add_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value);
void THClTensor_sub_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value);
void THClTensor_mul_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value);
void THClTensor_div_gpu(THClState *state, THClTensor *self, THClTensor *src, THClTensor *value);

void THClTensor_sqrt(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_abs(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_neg(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_cinv(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_exp(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_log(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_tanh(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_sigmoid(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_floor(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_ceil(THClState *state, THClTensor *self, THClTensor *src);
/* More of the operator catalogue; each is the reference's operator string run
 * through the same apply engine (src/lib/THClTensorMath.h:21,53-84,112,138-144). */
void THClTensor_log1p(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_cos(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_acos(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_cosh(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_sin(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_asin(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_sinh(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_tan(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_atan(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_round(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_sign(THClState *state, THClTensor *self, THClTensor *src);
/* src ^ value (integer-valued exponents by repeated multiplication: src/lib/THClTensorMath2.cpp:22-61) */
void THClTensor_pow(THClState *state, THClTensor *self, THClTensor *src, float value);
/* value ^ src */
void THClTensor_tpow(THClState *state, THClTensor *self, float value, THClTensor *src);
void THClTensor_cpow(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2);
void THClTensor_clamp(THClState *state, THClTensor *self, THClTensor *src, float min_value, float max_value);
void THClTensor_atan2(THClState *state, THClTensor *r_, THClTensor *tx, THClTensor *ty);
void THClTensor_cmax(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2);
void THClTensor_cmin(THClState *state, THClTensor *self, THClTensor *src1, THClTensor *src2);
void THClTensor_cmaxValue(THClState *state, THClTensor *self, THClTensor *src, float value);
void THClTensor_cminValue(THClState *state, THClTensor *self, THClTensor *src, float value);
/* comparisons write 1.0f / 0.0f; `self_` is resized to `src` */
void THClTensor_ltValue(THClState *state, THClTensor *self_, THClTensor *src, float value);
void THClTensor_gtValue(THClState *state, THClTensor *self_, THClTensor *src, float value);
void THClTensor_leValue(THClState *state, THClTensor *self_, THClTensor *src, float value);
void THClTensor_geValue(THClState *state, THClTensor *self_, THClTensor *src, float value);
void THClTensor_eqValue(THClState *state, THClTensor *self_, THClTensor *src, float value);
void THClTensor_neValue(THClState *state, THClTensor *self_, THClTensor *src, float value);
void THClTensor_ltTensor(THClState *state, THClTensor *self_, THClTensor *src1, THClTensor *src2);
void THClTensor_gtTensor(THClState *state, THClTensor *self_, THClTensor *src1, THClTensor *src2);
void THClTensor_leTensor(THClState *state, THClTensor *self_, THClTensor *src1, THClTensor *src2);
void THClTensor_geTensor(THClState *state, THClTensor *self_, THClTensor *src1, THClTensor *src2);
void THClTensor_eqTensor(THClState *state, THClTensor *self_, THClTensor *src1, THClTensor *src2);
void THClTensor_neTensor(THClState *state, THClTensor *self_, THClTensor *src1, THClTensor *src2);
void THClTensor_ltPointTensor(THClState *state, THClTensor *self_, THClTensor *src, THClTensor *value);
void THClTensor_gtPointTensor(THClState *state, THClTensor *self_, THClTensor *src, THClTensor *value);
void THClTensor_lePointTensor(THClState *state, THClTensor *self_, THClTensor *src, THClTensor *value);
void THClTensor_gePointTensor(THClState *state, THClTensor *self_, THClTensor *src, THClTensor *value);
void THClTensor_eqPointTensor(THClState *state, THClTensor *self_, THClTensor *src, THClTensor *value);
void THClTensor_nePointTensor(THClState *state, THClTensor *self_, THClTensor *src, THClTensor *value);
/* tensor[i] = value where mask[i] != 0; mask is a ClTensor of 0 / 1 */
void THClTensor_maskedFill(THClState *state, THClTensor *tensor, THClTensor *mask, float value);

/* User expressions over x (read-write), y, z -- or *out, *in1, *in2 -- compiled
 * at run time (reference: src/lib/THClTensorMathPointwise.cpp:79-146; Lua names
 * apply_on_gpu / map_on_gpu / map2_on_gpu, src/TensorMath.lua:591-620). */
void THClTensor_apply(THClState *state, THClTensor *self, char const *operation1);
void THClTensor_map(THClState *state, THClTensor *self, THClTensor *two, char const *operation2);
void THClTensor_map2(THClState *state, THClTensor *self, THClTensor *in1, THClTensor *in2, char const *operation3);

/* ------------------------------------------------------------------------- */
/* Reductions (reference: src/lib/THClTensorMath.h:30-39,133-155)             */
/* ------------------------------------------------------------------------- */
float THClTensor_sumall(THClState *state, THClTensor *self);
float THClTensor_prodall(THClState *state, THClTensor *self);
float THClTensor_maxall(THClState *state, THClTensor *self);
float THClTensor_minall(THClState *state, THClTensor *self);
/* result stays on the device in `self`, which becomes a point tensor */
void THClTensor_sumall_gpu(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_prodall_gpu(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_maxall_gpu(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_minall_gpu(THClState *state, THClTensor *self, THClTensor *src);
float THClTensor_as_float(THClState *state, THClTensor *self);
/* THClTensor_sumall_gpu for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference.
 * Requests and releases no device memory and creates no event: the kernel's arrival
 * ticket and per-block partials live in a static device array of 16.25 KiB that every
 * GPU the library runs on holds until the process ends, in place of the context's scratch
 * block.  `self` must already be a point tensor that owns its storage (it is not
 * resized), the device's context must already be open (any earlier call on that device
 * opens it), and `src` may have any layout with at most THCL_NOALLOC_MAX_ELEMENTS
 * elements; anything else is reported as an error and nothing is launched.  Same kernel,
 * same grid and same result as THClTensor_sumall_gpu.  All calls on one GPU share its
 * array: calls that overlap on one GPU (two host threads) race. */
#define THCL_NOALLOC_MAX_ELEMENTS 2147483647L
void THClTensor_sumall_gpu_noalloc(THClState *state, THClTensor *self, THClTensor *src);

void THClTensor_sum(THClState *state, THClTensor *self, THClTensor *src, long dim);
void THClTensor_prod(THClState *state, THClTensor *self, THClTensor *src, long dim);
/* `indices` receives 1-based positions as fp32, the reference's convention
 * (src/lib/THClTensorMathTransformReduce.cl:32,74) */
void THClTensor_max(THClState *state, THClTensor *values, THClTensor *indices, THClTensor *src, long dim);
void THClTensor_min(THClState *state, THClTensor *values, THClTensor *indices, THClTensor *src, long dim);
/* No counterpart in the reference: the same reductions with the positions
 * written as 1-based int64 into a host LongTensor (what `indices:long()` yields
 * in Lua), exact for reduction lengths beyond 2^24. */
void THClTensor_maxLong(THClState *state, THClTensor *values, THLongTensor *indices, THClTensor *src, long dim);
void THClTensor_minLong(THClState *state, THClTensor *values, THLongTensor *indices, THClTensor *src, long dim);

/* mean = sum / count; norms: value 0 counts non-zero elements, otherwise
 * (sum |x|^value)^(1/value), accumulated in fp64 like every sum here; all / any
 * take (int)x != 0 as an element's truth value
 * (reference: src/lib/THClTensorMath.h:86-96,125-126,138-139) */
float THClTensor_meanall(THClState *state, THClTensor *self);
void THClTensor_mean(THClState *state, THClTensor *self, THClTensor *src, long dim);
float THClTensor_normall(THClState *state, THClTensor *self, float value);
void THClTensor_norm(THClState *state, THClTensor *self, THClTensor *src, float value, long dimension);
int THClTensor_logicalall(THClState *state, THClTensor *self);
int THClTensor_logicalany(THClState *state, THClTensor *self);
void THClTensor_logicalall_gpu(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_logicalany_gpu(THClState *state, THClTensor *self, THClTensor *src);

/* inclusive running sum / product along `dim` (0-based); the running value is
 * fp64, each output its rounding to fp32
 * (reference: src/lib/THClTensorMath.h:36-37, src/lib/THClTensorMathScan.cpp:127-156) */
void THClTensor_cumsum(THClState *state, THClTensor *self, THClTensor *src, long dim);
void THClTensor_cumprod(THClState *state, THClTensor *self, THClTensor *src, long dim);

/* ------------------------------------------------------------------------- */
/* Dense contraction (reference: src/lib/THClTensorMath.h:47, THClBlas.h:42)  */
/* ------------------------------------------------------------------------- */
void THClTensor_addmm(THClState *state, THClTensor *self, float beta, THClTensor *t, float alpha,
                      THClTensor *mat1, THClTensor *mat2);
/* column-major sgemm on tensors' storages + offsets, BLAS argument meaning */
void THClBlas_gemm(THClState *state, char transa, char transb, long m, long n, long k, float alpha,
                   THClTensor *a, long lda, THClTensor *b, long ldb, float beta, THClTensor *c, long ldc);

/* Level 1 / level 2 (reference: src/lib/THClTensorMath.h:28,46,48, THClBlas.h:21-35).
 * Sums run in fp64 and round to fp32 once.  The THClBlas_* forms take the
 * tensors whose storage + offset mark each operand's first element. */
float THClTensor_dot(THClState *state, THClTensor *self, THClTensor *src);
void THClTensor_addmv(THClState *state, THClTensor *self, float beta, THClTensor *t, float alpha, THClTensor *mat,
                      THClTensor *vec);
void THClTensor_addr(THClState *state, THClTensor *self, float beta, THClTensor *t, float alpha, THClTensor *vec1,
                     THClTensor *vec2);
/* (src/lib/THClBlas.h:21-23) xwrapper / ywrapper: what storage->wrapper holds, the device address of the
 * storage's first element; offsets and increments in elements */
float THClBlas_dot(THClState *state, long n, void *xwrapper, long xoffset, long incx, void *ywrapper, long yoffset,
                   long incy);
void THClBlas_gemv(THClState *state, char trans, long m, long n, float alpha, THClTensor *a, long lda, THClTensor *x,
                   long incx, float beta, THClTensor *y, long incy);
void THClBlas_ger(THClState *state, long m, long n, float alpha, THClTensor *x, long incx, THClTensor *y, long incy,
                  THClTensor *a, long lda);

/* ------------------------------------------------------------------------- */
/* Indexed movement (reference: src/lib/THClTensorMath.h:101-116,130-132).     */
/* Index tensors hold 1-based positions as floats; `dim` is 0-based.  An       */
/* index outside the dimension moves nothing.                                  */
/* ------------------------------------------------------------------------- */
void THClTensor_indexSelect(THClState *state, THClTensor *tensor, THClTensor *src, int dim, THClTensor *index);
void THClTensor_indexCopy(THClState *state, THClTensor *res_, int dim, THClTensor *indices, THClTensor *src);
void THClTensor_indexFill(THClState *state, THClTensor *tensor, int dim, THClTensor *index, float val);
void THClTensor_indexSelect_long(THClState *state, THClTensor *tensor, THClTensor *src, int dim, THLongTensor *index);
void THClTensor_indexCopy_long(THClState *state, THClTensor *res_, int dim, THLongTensor *indices, THClTensor *src);
void THClTensor_indexFill_long(THClState *state, THClTensor *tensor, int dim, THLongTensor *index, float val);
void THClTensor_gather(THClState *state, THClTensor *self, THClTensor *src, long dim, THClTensor *index);
void THClTensor_scatter(THClState *state, THClTensor *self, long dim, THClTensor *index, THClTensor *src);
void THClTensor_scatterFill(THClState *state, THClTensor *self, long dim, THClTensor *index, float val);
/* mask: a ClTensor of 0 / non-0 with as many elements as the tensor it selects from */
void THClTensor_maskedSelect(THClState *state, THClTensor *tensor, THClTensor *src, THClTensor *mask);
void THClTensor_maskedCopy(THClState *state, THClTensor *tensor, THClTensor *mask, THClTensor *src);
/* host byte masks: uploaded as floats, then the forms above (src/lib/THClTensorMath.h:117-119) */
void THClTensor_maskedFillByte(THClState *state, THClTensor *tensor, THByteTensor *mask, float value);
void THClTensor_maskedCopyByte(THClState *state, THClTensor *tensor, THByteTensor *mask, THClTensor *src);
void THClTensor_maskedSelectByte(THClState *state, THClTensor *tensor, THClTensor *src, THByteTensor *mask);

/* ------------------------------------------------------------------------- */
/* User kernels compiled at run time: the C side of torch.ClKernel.  The      */
/* reference offers this to Lua only (src/UserKernel.cpp:217-383); these       */
/* entry points carry what its constructor and run() read from Lua tables.    */
/* ------------------------------------------------------------------------- */
typedef struct THClKernel THClKernel;
enum { THCL_KARG_INT = 0, THCL_KARG_FLOAT = 1, THCL_KARG_TENSOR = 2 };
enum { THCL_KDIR_INPUT = 0, THCL_KDIR_OUTPUT = 1, THCL_KDIR_INOUT = 2 };
/* `src` is the kernel body in OpenCL C as the reference's users write it
 * (get_global_id(0), NAME_data[..], NAME_info->offset, barrier(...)); `funcs`
 * optional helper functions placed ahead of the kernel; `name` NULL for
 * "user_kernel".  A tensor argument NAME appears in the body as
 * `struct THClTensorInfoCl *NAME_info` and `float *NAME_data` (first element of
 * the storage).  Returns NULL after reporting an error. */
THClKernel *THClKernel_new(THClState *state, const char *name, const char *src, const char *funcs, int nargs,
                           const char *const *arg_names, const int *arg_types, const int *arg_dirs);
void THClKernel_free(THClState *state, THClKernel *kernel);
const char *THClKernel_getRenderedKernel(THClKernel *kernel);
int THClKernel_numArgs(THClKernel *kernel);
/* Values by argument position (entries of the other two arrays are ignored
 * for that position).  numWorkgroups / workgroupSize <= 0 select the
 * reference's defaults: groups of 64 covering the first output or inout
 * tensor's elements.  Compilation happens on a kernel's first run per device. */
void THClKernel_run(THClState *state, THClKernel *kernel, const int *ints, const float *floats,
                    THClTensor *const *tensors, long numWorkgroups, long workgroupSize);
int THClKernel_compileCheck(THClKernel *kernel, const char *arch, size_t *code_bytes);

/* ------------------------------------------------------------------------- */
/* Defined by the reference only to raise an error; kept so that a binding     */
/* built from the reference's own sources resolves every name it mentions      */
/* (src/Storage.cpp:75 calls THClStorage_copyCl, src/TensorMath.lua:849 wraps  */
/* THClTensor_baddbmm).  Each reports the reference's message:                 */
/* "not available yet for THClStorage" (src/lib/THClStorage.cpp:142-200,       */
/* THClStorageCopy.cpp:27-32) or "Not implemented" (src/lib/THClBlas.cpp:      */
/* 67-147,451-470, THClTensorMathBlas.cpp:279-380).                            */
/* ------------------------------------------------------------------------- */
THClStorage *THClStorage_newWithSize1(THClState *state, int device, float data0);
THClStorage *THClStorage_newWithSize2(THClState *state, int device, float data0, float data1);
THClStorage *THClStorage_newWithSize3(THClState *state, int device, float data0, float data1, float data2);
THClStorage *THClStorage_newWithSize4(THClState *state, int device, float data0, float data1, float data2, float data3);
THClStorage *THClStorage_newWithMapping(THClState *state, int device, const char *filename, long size, int shared);
THClStorage *THClStorage_newWithData(THClState *state, int device, float *data, long size);
void THClStorage_copyCl(THClState *state, THClStorage *self, THClStorage *src);
void THClBlas_swap(THClState *state, long n, float *x, long incx, float *y, long incy);
void THClBlas_scal(THClState *state, long n, float a, float *x, long incx);
void THClBlas_copy(THClState *state, long n, float *x, long incx, float *y, long incy);
void THClBlas_axpy(THClState *state, long n, float a, float *x, long incx, float *y, long incy);
void THClBlas_gemmBatched(THClState *state, char transa, char transb, long m, long n, long k, float alpha,
                          const float **a, long lda, const float **b, long ldb, float beta, float **c, long ldc,
                          long batchCount);
void THClTensor_baddbmm(THClState *state, THClTensor *result, float beta, THClTensor *t, float alpha,
                        THClTensor *batch1, THClTensor *batch2);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif
