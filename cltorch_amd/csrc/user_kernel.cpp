// User-written kernels compiled at run time: the C side of torch.ClKernel.
//
// What it replaces (reference): src/UserKernel.cpp:217-383, which renders an
// OpenCL kernel around the user's body -- one `global struct THClTensorInfoCl
// *NAME_info, global float *NAME_data` pair per tensor argument, `int NAME` /
// `float NAME` for scalars -- builds it with the OpenCL compiler and runs it
// over ceil(nElements / 64) work-groups of 64 (nElements of the first output
// or inout tensor), or the work-group count and size the caller gives.
//
// Here the body is compiled by hipRTC.  A short prelude gives it the OpenCL C
// names it is written in (get_global_id and friends, barrier, the address
// space qualifiers); the tensor descriptors travel in the kernel arguments and
// each NAME_info points at its copy, so no descriptor upload precedes a launch.
#include <cstring>
#include <string>
#include <vector>

#include "internal.h"

namespace {

constexpr int kMaxInfoDims = 25;  // MAX_CLTORCH_DIMS of the reference's descriptor

struct TensorInfoCl {  // layout of the reference's THClTensorInfoCl (README.md:176-181)
  unsigned sizes[kMaxInfoDims];
  unsigned strides[kMaxInfoDims];
  int offset;
  int dims;
};

const char kInfoStruct[] = R"PRELUDE(
typedef struct THClTensorInfoCl {
  unsigned int sizes[25];
  unsigned int strides[25];
  int offset;
  int dims;
} TensorInfoCl;
)PRELUDE";

const char kPrelude[] = R"PRELUDE(
#undef __kernel
#undef __global
#undef __constant
#undef __local
#define kernel
#define __kernel
#define global
#define __global
#define constant const
#define __constant const
#define local __shared__
#define __local __shared__
#define CLK_LOCAL_MEM_FENCE 1
#define CLK_GLOBAL_MEM_FENCE 2
#define barrier(flags) __syncthreads()
#define mem_fence(flags) __threadfence_block()
__device__ __forceinline__ int get_local_id(int d) { return (int)(d == 0 ? threadIdx.x : (d == 1 ? threadIdx.y : threadIdx.z)); }
__device__ __forceinline__ int get_group_id(int d) { return (int)(d == 0 ? blockIdx.x : (d == 1 ? blockIdx.y : blockIdx.z)); }
__device__ __forceinline__ int get_local_size(int d) { return (int)(d == 0 ? blockDim.x : (d == 1 ? blockDim.y : blockDim.z)); }
__device__ __forceinline__ int get_num_groups(int d) { return (int)(d == 0 ? gridDim.x : (d == 1 ? gridDim.y : gridDim.z)); }
__device__ __forceinline__ int get_global_id(int d) { return get_group_id(d) * get_local_size(d) + get_local_id(d); }
__device__ __forceinline__ int get_global_size(int d) { return get_num_groups(d) * get_local_size(d); }
#define native_exp(x) expf(x)
#define native_log(x) logf(x)
#define native_sqrt(x) sqrtf(x)
#define native_recip(x) (1.0f / (x))
#define mad(a, b, c) ((a) * (b) + (c))
)PRELUDE";

enum ArgType { ARG_INT = 0, ARG_FLOAT = 1, ARG_TENSOR = 2 };
enum ArgDir { DIR_IN = 0, DIR_OUT = 1, DIR_INOUT = 2 };

struct Arg {
  std::string name;
  int type, dir;
};

bool identifier(const std::string &s) {
  if (s.empty() || !(isalpha((unsigned char)s[0]) || s[0] == '_')) return false;
  for (char c : s)
    if (!(isalnum((unsigned char)c) || c == '_')) return false;
  return true;
}
}  // namespace

struct THClKernel {
  std::string name, key, rendered;
  std::vector<Arg> args;
};

extern "C" {

THClKernel *THClKernel_new(THClState *state, const char *name, const char *src, const char *funcs, int nargs,
                           const char *const *arg_names, const int *arg_types, const int *arg_dirs) {
  THCL_GUARD_BEGIN
  (void)state;
  THCL_CHECK(src != nullptr && src[0] != 0, "Missing parameter src, or was empty");
  THCL_CHECK(nargs >= 0 && (nargs == 0 || (arg_names && arg_types && arg_dirs)), "argument lists are missing");
  THClKernel *k = new THClKernel();
  try {
    k->name = (name && name[0]) ? name : "user_kernel";
    THCL_CHECK(identifier(k->name), "kernel name %s is not an identifier", k->name.c_str());
    std::string params, aliases, forward;
    for (int i = 0; i < nargs; i++) {
      Arg a;
      a.name = arg_names[i] ? arg_names[i] : "";
      a.type = arg_types[i];
      a.dir = arg_dirs[i];
      THCL_CHECK(identifier(a.name), "argument name '%s' is not an identifier", a.name.c_str());
      THCL_CHECK(a.type >= ARG_INT && a.type <= ARG_TENSOR, "Unrecognized type of argument %s", a.name.c_str());
      THCL_CHECK(a.dir >= DIR_IN && a.dir <= DIR_INOUT, "Unrecognized direction of argument %s", a.name.c_str());
      if (a.type == ARG_INT) THCL_CHECK(a.dir == DIR_IN, "ints can only be input parameters, not output, or inout");
      if (a.type == ARG_FLOAT) THCL_CHECK(a.dir == DIR_IN, "floats can only be input parameters, not output, or inout");
      if (i > 0) {
        params += ",\n";
        forward += ", ";
      }
      if (a.type == ARG_INT) {
        params += "    int " + a.name;
        forward += a.name;
      } else if (a.type == ARG_FLOAT) {
        params += "    float " + a.name;
        forward += a.name;
      } else {
        params += "    struct THClTensorInfoCl " + a.name + "_info_, ";
        params += std::string(a.dir == DIR_IN ? "const " : "") + "float *" + a.name + "_data";
        aliases += "  struct THClTensorInfoCl *" + a.name + "_info = &" + a.name + "_info_; (void)" + a.name + "_info;\n";
        forward += a.name + "_info_, " + a.name + "_data";
      }
      k->args.push_back(a);
    }
    // Layout of the rendered source.  The entry point comes first, ahead of the
    // prelude: the prelude defines `global`, `kernel`, `constant` away for the
    // user's OpenCL qualifiers, and HIP's __global__ spells one of those words.
    // The entry forwards to a device function that holds the user's body.
    // Helper functions are plain C in OpenCL; a pragma makes them callable
    // from device code.
    const std::string body_fn = k->name + "_body_";
    k->rendered = kInfoStruct;
    k->rendered += "static __device__ void " + body_fn + "(\n" + params + ");\n";
    k->rendered += "extern \"C\" __global__ void " + k->name + "(\n" + params + "\n) {\n  " + body_fn + "(" + forward + ");\n}\n";
    k->rendered += kPrelude;
    k->rendered += "\n";
    if (funcs) k->rendered += std::string("#pragma clang force_cuda_host_device begin\n") + funcs +
                              "\n#pragma clang force_cuda_host_device end\n";
    k->rendered += "static __device__ void " + body_fn + "(\n" + params + "\n) {\n" + aliases + src + "\n}\n";
    // compiled code is cached per device context under a key made of the whole text
    unsigned long long h = 1469598103934665603ull;
    for (unsigned char c : k->rendered) h = (h ^ c) * 1099511628211ull;
    char buf[64];
    snprintf(buf, sizeof(buf), "userkernel|%s|%016llx", k->name.c_str(), h);
    k->key = buf;
  } catch (...) {
    delete k;
    throw;
  }
  return k;
  THCL_GUARD_END(nullptr)
}

void THClKernel_free(THClState *state, THClKernel *kernel) {
  (void)state;
  delete kernel;
}

const char *THClKernel_getRenderedKernel(THClKernel *kernel) { return kernel ? kernel->rendered.c_str() : ""; }

int THClKernel_numArgs(THClKernel *kernel) { return kernel ? (int)kernel->args.size() : 0; }

void THClKernel_run(THClState *state, THClKernel *kernel, const int *ints, const float *floats,
                    THClTensor *const *tensors, long numWorkgroups, long workgroupSize) {
  THCL_GUARD_BEGIN
  THCL_CHECK(kernel != nullptr, "kernel is NULL");
  const size_t nargs = kernel->args.size();
  // kernel-argument block: each member at its natural alignment, as the compiler lays out the signature
  std::vector<unsigned char> block;
  auto put = [&](const void *p, size_t bytes, size_t align) {
    size_t at = (block.size() + align - 1) / align * align;
    block.resize(at + bytes);
    memcpy(block.data() + at, p, bytes);
  };
  long nelem = -1;
  int device = -1;
  for (size_t i = 0; i < nargs; i++) {
    const Arg &a = kernel->args[i];
    if (a.type == ARG_INT) {
      THCL_CHECK(ints != nullptr, "no value for int argument %s", a.name.c_str());
      put(&ints[i], sizeof(int), alignof(int));
    } else if (a.type == ARG_FLOAT) {
      THCL_CHECK(floats != nullptr, "no value for float argument %s", a.name.c_str());
      put(&floats[i], sizeof(float), alignof(float));
    } else {
      THClTensor *t = tensors ? tensors[i] : nullptr;
      THCL_CHECK(t != nullptr, "no value for tensor argument %s", a.name.c_str());
      THCL_CHECK(t->storage != nullptr && t->storage->wrapper != nullptr,
                 a.dir == DIR_IN ? "tensor %s has no data" : "tensor %s has no storage: size it before the launch",
                 a.name.c_str());
      THCL_CHECK(t->nDimension <= kMaxInfoDims, THCL_DIM_WARNING);
      if (device < 0) device = t->storage->device;
      THCL_CHECK(device == t->storage->device, "tensor arguments live on different devices");
      TensorInfoCl info;
      memset(&info, 0, sizeof(info));
      for (int d = 0; d < t->nDimension; d++) {
        THCL_CHECK(t->size[d] < (1l << 32) && t->stride[d] >= 0 && t->stride[d] < (1l << 32), THCL_DIM_WARNING);
        info.sizes[d] = (unsigned)t->size[d];
        info.strides[d] = (unsigned)t->stride[d];
      }
      THCL_CHECK(t->storageOffset < (1l << 31), THCL_DIM_WARNING);
      info.offset = (int)t->storageOffset;
      info.dims = t->nDimension;
      put(&info, sizeof(info), alignof(TensorInfoCl));
      float *base = (float *)t->storage->wrapper;  // NAME_data is the storage's first element; NAME_info->offset locates the view
      put(&base, sizeof(base), alignof(float *));
      if (nelem < 0 && a.dir != DIR_IN) nelem = THClTensor_nElement(state, t);
    }
  }
  THCL_CHECK(nelem >= 0, "Must provide at least one output, or inout, ClTensor");
  if (workgroupSize <= 0) workgroupSize = 64;
  if (numWorkgroups <= 0) numWorkgroups = (nelem + workgroupSize - 1) / workgroupSize;
  THCL_CHECK(workgroupSize <= 1024, "workgroupSize %ld is beyond the device's 1024", workgroupSize);
  THCL_CHECK(numWorkgroups < (1l << 31), "too many workgroups");
  if (numWorkgroups == 0) return;
  thcl_rt *rt = thcl_ctx(state, device);
  thcl_rt_kernel *fn = thcl_rt_kernel_get(rt, kernel->key.c_str(), kernel->rendered.c_str(), kernel->name.c_str());
  THCL_CHECK(fn != nullptr, "Failed to create kernel %s", thcl_rt_error());
  THCL_CHECK(thcl_rt_launch(rt, fn, (unsigned)numWorkgroups, 1, 1, (unsigned)workgroupSize, 1, 1, 0, block.data(),
                            block.size()) == 0,
             "%s", thcl_rt_error());
  thcl_after_launch(state, rt);
  THCL_GUARD_END()
}

// compile for an architecture without a device (build-time check of user kernels)
int THClKernel_compileCheck(THClKernel *kernel, const char *arch, size_t *code_bytes) {
  if (!kernel) return -1;
  return thcl_rt_compile_check(kernel->rendered.c_str(), arch, code_bytes);
}

}  // extern "C"
