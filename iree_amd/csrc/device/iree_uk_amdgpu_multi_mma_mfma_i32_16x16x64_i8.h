// In-dispatch GPU microkernel for gfx950: the inner (K) loop of a data-tiled
// int8 matmul tile with the MFMA intrinsic v_mfma_i32_16x16x64_i8, in the
// calling convention of the reference's ROCm ukernels
// (compiler/plugins/target/ROCM/builtins/ukernel/
// iree_uk_amdgpu_multi_mma_mfma_i32_16x16x32_i8.c:82-181 is the gfx942
// counterpart with the 16x16x32 intrinsic). A compiler inlines this function
// into a dispatch; all the `intrinsics_*` / `subgroups_*` parameters are
// constants at that point, so the loops below unroll and the arrays become
// registers.
//
// Data layout (that of a DataTiledMMA operand with this intrinsic). One
// "vector" is the MFMA's per-lane operand: 16 int8 for A and B, 4 int32 for C.
//   A tile of one outer-K step: [subgroups_m][intrinsics_m][64 lanes][intrinsics_k] vectors;
//     lane l of (subgroup, intrinsic) (s, m) holds row 16*(intrinsics_m*s + m) + l % 16,
//     K bytes 64*k + 16*(l / 16) .. +15 of that step's 64*intrinsics_k.
//   B tile: the same with n for m (B is stored as its transpose: row = column of the product).
//   C: per thread [intrinsics_m][intrinsics_n] vectors, 64 vectors apart; lane l
//     holds product rows 4*(l / 16) + {0..3} of column l % 16 of its 16x16 block.
// The A/B/C pointers are "after thread distribution": they point at the calling
// thread's first vector.
//
// Differences from the gfx942 kernel, for the gfx950 memory system: 16-byte
// vectors; the shared-memory copy of a tile is double buffered and the next
// outer-K step's global loads are issued before the current step's MFMAs, so
// there is one workgroup barrier per step and the loads overlap the matrix
// pipe. The shared-memory size query accounts for the second buffer.
#ifndef IREE_AMD_CSRC_DEVICE_IREE_UK_AMDGPU_MULTI_MMA_MFMA_I32_16X16X64_I8_H_
#define IREE_AMD_CSRC_DEVICE_IREE_UK_AMDGPU_MULTI_MMA_MFMA_I32_16X16X64_I8_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace iree_uk_amdgpu {

typedef int int32x4_t __attribute__((ext_vector_type(4)));

// Largest intrinsics_m / intrinsics_n and largest per-thread share of a tile
// copy the register arrays are sized for (they shrink to what is used once the
// parameters are constants).
constexpr int kMaxIntrinsics = 8;
constexpr int kMaxCopyVecs = 16;

struct AbTile {
  int num_vecs;         // vectors in one outer-K step of the tile
  int num_shared_vecs;  // of which staged in shared memory (all or none)
};

__host__ __device__ inline AbTile ab_tile(int tile_intrinsics, int tile_subgroups, int opposite_subgroups) {
  AbTile t;
  t.num_vecs = 64 * tile_intrinsics * tile_subgroups;
  // Shared memory pays off when more than one subgroup reads the tile.
  t.num_shared_vecs = opposite_subgroups > 1 ? t.num_vecs : 0;
  return t;
}

}  // namespace iree_uk_amdgpu

// Bytes of workgroup memory the microkernel needs for these parameters (two
// buffers of every staged tile). A compiler evaluates this at compile time.
extern "C" __host__ __device__ inline int32_t
iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_query_shared_memory_bytes(int32_t intrinsics_m, int32_t subgroups_m,
                                                                        int32_t intrinsics_n, int32_t subgroups_n,
                                                                        int32_t intrinsics_k) {
  const iree_uk_amdgpu::AbTile a = iree_uk_amdgpu::ab_tile(intrinsics_m * intrinsics_k, subgroups_m, subgroups_n);
  const iree_uk_amdgpu::AbTile b = iree_uk_amdgpu::ab_tile(intrinsics_n * intrinsics_k, subgroups_n, subgroups_m);
  return 2 * 16 * (a.num_shared_vecs + b.num_shared_vecs);
}

extern "C" __device__ __attribute__((always_inline)) inline void iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8(
    const int8_t* a_base, int64_t a_offset, const int8_t* b_base, int64_t b_offset, int32_t* c_base,
    int64_t c_offset, int8_t* shared_memory_base, int64_t shared_memory_offset, int32_t shared_memory_bytes,
    int32_t k_size, int32_t intrinsics_m, int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n,
    int32_t intrinsics_k) {
  using namespace iree_uk_amdgpu;
  const AbTile a_tile = ab_tile(intrinsics_m * intrinsics_k, subgroups_m, subgroups_n);
  const AbTile b_tile = ab_tile(intrinsics_n * intrinsics_k, subgroups_n, subgroups_m);
  if (shared_memory_bytes != 2 * 16 * (a_tile.num_shared_vecs + b_tile.num_shared_vecs)) __builtin_trap();

  const int tid = __builtin_amdgcn_workitem_id_x();
  const int numthreads = 64 * subgroups_m * subgroups_n;
  __builtin_assume(tid < numthreads);
  const int lane_id = tid % 64, subgroup_id = tid / 64;
  const int subgroup_n_idx = subgroup_id % subgroups_n, subgroup_m_idx = subgroup_id / subgroups_n;
  const int a_thread_relative_offset = intrinsics_k * (lane_id + 64 * intrinsics_m * subgroup_m_idx);
  const int b_thread_relative_offset = intrinsics_k * (lane_id + 64 * intrinsics_n * subgroup_n_idx);

  // Shared memory: [2 buffers][A vectors, then B vectors].
  const int shared_vecs = a_tile.num_shared_vecs + b_tile.num_shared_vecs;
  int32x4_t* shared = (int32x4_t*)(shared_memory_base + shared_memory_offset);

  const int32x4_t* a_global = (const int32x4_t*)(a_base + a_offset);
  const int32x4_t* b_global = (const int32x4_t*)(b_base + b_offset);
  int32x4_t* c_global = (int32x4_t*)(c_base + c_offset);
  // The same tiles seen from the workgroup (for the cooperative copy).
  const int32x4_t* a_tile_global = a_global - a_thread_relative_offset;
  const int32x4_t* b_tile_global = b_global - b_thread_relative_offset;

  int32x4_t c_regs[kMaxIntrinsics][kMaxIntrinsics];
  for (int m = 0; m < intrinsics_m; ++m)
    for (int n = 0; n < intrinsics_n; ++n) c_regs[m][n] = c_global[64 * (m * intrinsics_n + n)];

  // This thread's share of the copy of one outer-K step: vectors tid,
  // tid + numthreads, ... of each staged tile.
  const int a_copies = a_tile.num_shared_vecs / numthreads, b_copies = b_tile.num_shared_vecs / numthreads;
  int32x4_t a_stage[kMaxCopyVecs], b_stage[kMaxCopyVecs];
  auto fetch = [&](int k_outer) {
    for (int i = 0; i < a_copies; ++i) a_stage[i] = a_tile_global[(int64_t)k_outer * a_tile.num_vecs + i * numthreads + tid];
    for (int i = 0; i < b_copies; ++i) b_stage[i] = b_tile_global[(int64_t)k_outer * b_tile.num_vecs + i * numthreads + tid];
  };
  auto stash = [&](int buffer) {
    int32x4_t* dst = shared + buffer * shared_vecs;
    for (int i = 0; i < a_copies; ++i) dst[i * numthreads + tid] = a_stage[i];
    for (int i = 0; i < b_copies; ++i) dst[a_tile.num_shared_vecs + i * numthreads + tid] = b_stage[i];
  };
  const bool staged = shared_vecs != 0;
  if (staged && k_size > 0) {
    fetch(0);
    stash(0);
    __syncthreads();
  }

  for (int k_outer = 0; k_outer < k_size; ++k_outer) {
    const int buffer = k_outer & 1;
    // Next step's tile on its way from global memory while this one is multiplied.
    if (staged && k_outer + 1 < k_size) fetch(k_outer + 1);
    const int32x4_t* a_vecs = a_tile.num_shared_vecs
                                  ? shared + buffer * shared_vecs + a_thread_relative_offset
                                  : a_global + (int64_t)k_outer * a_tile.num_vecs;
    const int32x4_t* b_vecs = b_tile.num_shared_vecs
                                  ? shared + buffer * shared_vecs + a_tile.num_shared_vecs + b_thread_relative_offset
                                  : b_global + (int64_t)k_outer * b_tile.num_vecs;
    for (int k = 0; k < intrinsics_k; ++k) {
      int32x4_t b_regs[kMaxIntrinsics];
      for (int n = 0; n < intrinsics_n; ++n) b_regs[n] = b_vecs[64 * intrinsics_k * n + k];
      for (int m = 0; m < intrinsics_m; ++m) {
        const int32x4_t a_reg = a_vecs[64 * intrinsics_k * m + k];
        for (int n = 0; n < intrinsics_n; ++n)
          c_regs[m][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_reg, b_regs[n], c_regs[m][n], 0, 0, 0);
      }
    }
    if (staged) {
      // The other buffer was last read in the previous step, which ended with
      // a barrier: it is free to be overwritten.
      if (k_outer + 1 < k_size) stash(buffer ^ 1);
      __syncthreads();
    }
  }

  for (int m = 0; m < intrinsics_m; ++m)
    for (int n = 0; n < intrinsics_n; ++n) c_global[64 * (m * intrinsics_n + n)] = c_regs[m][n];
}

#endif  // IREE_AMD_CSRC_DEVICE_IREE_UK_AMDGPU_MULTI_MMA_MFMA_I32_16X16X64_I8_H_
