// What the two translation units that hold ahead-of-time apply kernels share: the operator
// struct an X(name, tensors, statement) table entry expands to, and the set of entry points
// (one per kernel family) the launcher picks from.
#pragma once

#include "apply_device.h"
#include "fixed_ops.h"

#define THCL_DEFINE_OP_STRUCT(name, nt, stmt)                                                         \
  struct Op_##name {                                                                                  \
    static constexpr int NT = nt;                                                                     \
    static __device__ __forceinline__ void run(float &o, float a, float b, float v1, float v2, float p1, \
                                               float p2) {                                            \
      (void)a; (void)b; (void)v1; (void)v2; (void)p1; (void)p2;                                        \
      stmt;                                                                                           \
    }                                                                                                 \
  };

struct ThclKernelSet {
  int nt;
  void (*contig_v4)(ThclContigParams);
  void (*contig_s)(ThclContigParams);
  void (*joint_v4)(ThclJointParams);
  void (*joint_s)(ThclJointParams);
  void (*generic)(ThclGenericParams);
  void (*tiled)(ThclTileParams);
};
#define THCL_KERNEL_SET_ENTRY(name, nt, stmt) \
  {nt, thcl_k_##name##_contig_v4, thcl_k_##name##_contig_s, thcl_k_##name##_joint_v4, thcl_k_##name##_joint_s, thcl_k_##name##_generic, thcl_k_##name##_tiled},

// kernels of THCL_CATALOGUE_OPS, indexed by op - OP_FIXED_COUNT (apply_catalogue.hip)
const ThclKernelSet *thcl_catalogue_kernel_sets();
