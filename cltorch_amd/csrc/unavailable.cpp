// Entry points that the reference's library defines only to raise an error.  A binding built from the reference's
// unchanged sources still names them (src/Storage.cpp:75 calls THClStorage_copyCl, the cwrap table at
// src/TensorMath.lua:849 wraps THClTensor_baddbmm), so a library that is to be loaded in its place must resolve
// them; calling one reports the reference's own message through the installed error handler.
#include "internal.h"

extern "C" {

// src/lib/THClStorage.cpp:142-200
THClStorage *THClStorage_newWithSize1(THClState *, int, float) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END(nullptr)
}
THClStorage *THClStorage_newWithSize2(THClState *, int, float, float) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END(nullptr)
}
THClStorage *THClStorage_newWithSize3(THClState *, int, float, float, float) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END(nullptr)
}
THClStorage *THClStorage_newWithSize4(THClState *, int, float, float, float, float) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END(nullptr)
}
THClStorage *THClStorage_newWithMapping(THClState *, int, const char *, long, int) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END(nullptr)
}
THClStorage *THClStorage_newWithData(THClState *, int, float *, long) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END(nullptr)
}
// src/lib/THClStorageCopy.cpp:27-32
void THClStorage_copyCl(THClState *, THClStorage *, THClStorage *) {
  THCL_GUARD_BEGIN
  thcl_throw("not available yet for THClStorage");
  THCL_GUARD_END()
}

// src/lib/THClBlas.cpp:67-147,451-470
void THClBlas_swap(THClState *, long, float *, long, float *, long) {
  THCL_GUARD_BEGIN
  thcl_throw("Not implemented");
  THCL_GUARD_END()
}
void THClBlas_scal(THClState *, long, float, float *, long) {
  THCL_GUARD_BEGIN
  thcl_throw("Not implemented");
  THCL_GUARD_END()
}
void THClBlas_copy(THClState *, long, float *, long, float *, long) {
  THCL_GUARD_BEGIN
  thcl_throw("Not implemented");
  THCL_GUARD_END()
}
void THClBlas_axpy(THClState *, long, float, float *, long, float *, long) {
  THCL_GUARD_BEGIN
  thcl_throw("Not implemented");
  THCL_GUARD_END()
}
void THClBlas_gemmBatched(THClState *, char, char, long, long, long, float, const float **, long, const float **, long,
                          float, float **, long, long) {
  THCL_GUARD_BEGIN
  thcl_throw("Not implemented");
  THCL_GUARD_END()
}

// src/lib/THClTensorMathBlas.cpp:279-380
void THClTensor_baddbmm(THClState *, THClTensor *, float, THClTensor *, float, THClTensor *, THClTensor *) {
  THCL_GUARD_BEGIN
  thcl_throw("Not implemented");
  THCL_GUARD_END()
}

}  // extern "C"
