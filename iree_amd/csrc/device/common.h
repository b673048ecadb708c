// Local definitions for the freestanding device microkernels: they are
// compiled as C23 for the amdgcn target without any header of the C library,
// of HIP or of the device libraries (-nogpulib), the way the reference's ROCm
// backend builds its own (build_tools/cmake/iree_bitcode_library.cmake:273-294;
// compiler/plugins/target/ROCM/builtins/ukernel/common.h has the same role
// there). Everything below is a Clang predefined macro or builtin.
#ifndef IREE_AMD_CSRC_DEVICE_COMMON_H_
#define IREE_AMD_CSRC_DEVICE_COMMON_H_

typedef __INT8_TYPE__ int8_t;
typedef __INT32_TYPE__ int32_t;
typedef __INT64_TYPE__ int64_t;
typedef __UINT32_TYPE__ uint32_t;
typedef __UINT64_TYPE__ uint64_t;

typedef __attribute__((__vector_size__(4 * 4))) int32_t int32x4_t;

// Workgroup barrier that also orders workgroup-memory accesses around it.
[[clang::convergent]] static inline void workgroup_barrier(void) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

#endif  // IREE_AMD_CSRC_DEVICE_COMMON_H_
