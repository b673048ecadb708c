// Internal declarations shared by the host shim (uk_api.hip) and the kernel
// translation units. Not installed; the public surface is
// include/iree_uk_mi355x.h.
#ifndef IREE_AMD_CSRC_UK_INTERNAL_H_
#define IREE_AMD_CSRC_UK_INTERNAL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/iree_uk_mi355x.h"

namespace uk {

// Resolved operand addresses: `buffer + offset` already applied, so kernels
// index from element 0.
struct Mmt4dArgs {
  const uint8_t* lhs;
  const uint8_t* rhs;
  uint8_t* out;
  int64_t lhs_stride0;  // elements of the lhs type
  int64_t rhs_stride0;  // elements of the rhs type
  int64_t out_stride0;  // elements of the out type
  int64_t M, N, K;
  int32_t M0, N0, K0;
  uint32_t flags;
};

struct PackArgs {
  const uint8_t* in;
  uint8_t* out;
  int64_t in_stride0, in_stride1;
  int64_t out_stride0;
  int64_t in_size0, in_size1;
  int64_t out_size0, out_size1, out_size2, out_size3;
  uint64_t padding_value;
  uint32_t flags;
  int elem_bytes;
};

struct UnpackArgs {
  const uint8_t* in;
  uint8_t* out;
  int64_t in_stride0;
  int64_t out_stride0, out_stride1;
  int64_t in_size0, in_size1, in_size2, in_size3;
  int64_t out_size0, out_size1;
  uint32_t flags;
  int elem_bytes;
};

// A launcher enqueues one operation on `stream` and returns the HIP status of
// the launch. `name` receives a static string naming the kernel variant.
typedef hipError_t (*Mmt4dLauncher)(const Mmt4dArgs& a, hipStream_t stream, const char** name);

// Specialised mmt4d kernels. Each returns nullptr when it does not cover the
// given problem (type, tile shape, alignment), else its launcher. `probe_only`
// problems carry only type flags and M0/N0/K0 (used by iree_uk_mmt4d_info).
Mmt4dLauncher select_mmt4d_mfma(const Mmt4dArgs& a, bool probe_only);
Mmt4dLauncher select_mmt4d_gemv(const Mmt4dArgs& a, bool probe_only);
Mmt4dLauncher select_mmt4d_skinny(const Mmt4dArgs& a, bool probe_only);
// Whether the skinny kernel beats a matrix kernel that also covers the problem.
bool mmt4d_skinny_preferred(const Mmt4dArgs& a);

// The in-dispatch int8 microkernel over a grid of data-tiled tiles (multi_mma.hip).
hipError_t launch_multi_mma_i8(const void* a, const void* b, void* c, int64_t outer_m, int64_t outer_n, int32_t k_size,
                               int intrinsics_m, int subgroups_m, int intrinsics_n, int subgroups_n, int intrinsics_k,
                               hipStream_t stream);

// One thread per output element; covers every type flag and tile shape.
hipError_t launch_mmt4d_generic(const Mmt4dArgs& a, hipStream_t stream, const char** name);

hipError_t launch_pack(const PackArgs& a, hipStream_t stream, const char** name);
hipError_t launch_unpack(const UnpackArgs& a, hipStream_t stream, const char** name);

// Bit widths of the (lhs, rhs, out) element types of an mmt4d type flag;
// returns false for an unknown flag.
inline bool mmt4d_type_bits(uint32_t flags, int* lhs, int* rhs, int* out) {
  switch (flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: *lhs = 32; *rhs = 32; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *lhs = 8; *rhs = 8; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *lhs = 16; *rhs = 16; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16: *lhs = 16; *rhs = 16; *out = 16; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *lhs = 16; *rhs = 16; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: *lhs = 16; *rhs = 16; *out = 16; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: *lhs = 16; *rhs = 16; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: *lhs = 16; *rhs = 4; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: *lhs = 16; *rhs = 8; *out = 32; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: *lhs = 8; *rhs = 4; *out = 32; return true;
    default: return false;
  }
}

}  // namespace uk

#endif  // IREE_AMD_CSRC_UK_INTERNAL_H_
