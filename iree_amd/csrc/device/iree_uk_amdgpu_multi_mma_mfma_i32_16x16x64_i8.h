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
// vectors; a staged tile travels global memory -> workgroup memory without
// passing through registers (global_load_lds_dwordx4: lane l of a wavefront
// writes its 16 bytes at M0 + 16*l, and a wavefront's share of the copy is 64
// consecutive vectors in both places), into a ring of up to four buffers
// filled up to three outer-K steps ahead. One counter wait and one workgroup
// barrier per step. The shared-memory size query accounts for the ring.
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

__host__ __device__ constexpr AbTile ab_tile(int tile_intrinsics, int tile_subgroups, int opposite_subgroups) {
  // Shared memory pays off when more than one subgroup reads the tile.
  return AbTile{64 * tile_intrinsics * tile_subgroups, opposite_subgroups > 1 ? 64 * tile_intrinsics * tile_subgroups : 0};
}

// Buffers in the ring of staged tiles, two to four. A step of 32 KiB or more belongs to a tile that fills the
// register file with one workgroup per compute unit: as many buffers as fit 128 KiB. Smaller tiles run several
// workgroups per compute unit, which hide each other's waits: the ring stays within 32 KiB so that they still all
// fit (measured on 128x128 tiles: four buffers of 16 KiB 94 us per 4096^3, two 88 us).
__host__ __device__ constexpr int ring_buffers(int shared_vecs_per_step) {
  if (shared_vecs_per_step == 0) return 0;
  const int step_bytes = 16 * shared_vecs_per_step;
  const int fit = (step_bytes >= 32 * 1024 ? 128 * 1024 : 32 * 1024) / step_bytes;
  return fit >= 4 ? 4 : (fit >= 2 ? fit : 2);
}

__host__ __device__ constexpr int shared_memory_bytes_for(int intrinsics_m, int subgroups_m, int intrinsics_n,
                                                          int subgroups_n, int intrinsics_k) {
  const int vecs = ab_tile(intrinsics_m * intrinsics_k, subgroups_m, subgroups_n).num_shared_vecs +
                   ab_tile(intrinsics_n * intrinsics_k, subgroups_n, subgroups_m).num_shared_vecs;
  return ring_buffers(vecs) * 16 * vecs;
}

// 64 vectors from `base` (wavefront-uniform) + 16 * (first_vec + lane) to the LDS address lds_address + 16 * lane.
__device__ __forceinline__ void load_vectors_to_lds(uint32_t lds_address, const int32x4_t* base, uint32_t lane_byte_offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_address), "v"(lane_byte_offset), "s"(base)
               : "memory");
}

template <int N>
__device__ __forceinline__ void wait_for_all_loads_but() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// s_waitcnt takes an immediate; `n` is a constant once the microkernel's parameters are.
__device__ __forceinline__ void wait_for_all_loads_but(int n) {
#define IREE_UK_AMDGPU_WAIT_CASE(N) case N: wait_for_all_loads_but<N>(); break;
#define IREE_UK_AMDGPU_WAIT_CASES8(B)                                                             \
  IREE_UK_AMDGPU_WAIT_CASE(B) IREE_UK_AMDGPU_WAIT_CASE(B + 1) IREE_UK_AMDGPU_WAIT_CASE(B + 2)     \
  IREE_UK_AMDGPU_WAIT_CASE(B + 3) IREE_UK_AMDGPU_WAIT_CASE(B + 4) IREE_UK_AMDGPU_WAIT_CASE(B + 5) \
  IREE_UK_AMDGPU_WAIT_CASE(B + 6) IREE_UK_AMDGPU_WAIT_CASE(B + 7)
  switch (n) {
    IREE_UK_AMDGPU_WAIT_CASES8(0) IREE_UK_AMDGPU_WAIT_CASES8(8) IREE_UK_AMDGPU_WAIT_CASES8(16)
    IREE_UK_AMDGPU_WAIT_CASES8(24) IREE_UK_AMDGPU_WAIT_CASES8(32) IREE_UK_AMDGPU_WAIT_CASES8(40)
    IREE_UK_AMDGPU_WAIT_CASES8(48) IREE_UK_AMDGPU_WAIT_CASES8(56)
    default: wait_for_all_loads_but<0>(); break;  // more than the counter holds: wait for everything
  }
#undef IREE_UK_AMDGPU_WAIT_CASES8
#undef IREE_UK_AMDGPU_WAIT_CASE
}

}  // namespace iree_uk_amdgpu

// Bytes of workgroup memory the microkernel needs for these parameters (the
// ring of buffers of the staged tiles). A compiler evaluates this at compile time.
extern "C" __host__ __device__ inline int32_t
iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_query_shared_memory_bytes(int32_t intrinsics_m, int32_t subgroups_m,
                                                                        int32_t intrinsics_n, int32_t subgroups_n,
                                                                        int32_t intrinsics_k) {
  return iree_uk_amdgpu::shared_memory_bytes_for(intrinsics_m, subgroups_m, intrinsics_n, subgroups_n, intrinsics_k);
}

extern "C" __device__ __attribute__((always_inline)) inline void iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8(
    const int8_t* a_base, int64_t a_offset, const int8_t* b_base, int64_t b_offset, int32_t* c_base,
    int64_t c_offset, int8_t* shared_memory_base, int64_t shared_memory_offset, int32_t shared_memory_bytes,
    int32_t k_size, int32_t intrinsics_m, int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n,
    int32_t intrinsics_k) {
  using namespace iree_uk_amdgpu;
  const AbTile a_tile = ab_tile(intrinsics_m * intrinsics_k, subgroups_m, subgroups_n);
  const AbTile b_tile = ab_tile(intrinsics_n * intrinsics_k, subgroups_n, subgroups_m);
  const int shared_vecs = a_tile.num_shared_vecs + b_tile.num_shared_vecs;  // per buffer
  const int buffers = ring_buffers(shared_vecs);
  if (shared_memory_bytes != buffers * 16 * shared_vecs) __builtin_trap();

  const int tid = __builtin_amdgcn_workitem_id_x();
  const int numthreads = 64 * subgroups_m * subgroups_n;
  __builtin_assume(tid < numthreads);
  const int lane_id = tid % 64, subgroup_id = __builtin_amdgcn_readfirstlane(tid / 64);
  const int subgroup_n_idx = subgroup_id % subgroups_n, subgroup_m_idx = subgroup_id / subgroups_n;
  const int a_thread_relative_offset = intrinsics_k * (lane_id + 64 * intrinsics_m * subgroup_m_idx);
  const int b_thread_relative_offset = intrinsics_k * (lane_id + 64 * intrinsics_n * subgroup_n_idx);

  // Shared memory: [buffers][A vectors, then B vectors].
  int32x4_t* shared = (int32x4_t*)(shared_memory_base + shared_memory_offset);
  // Its address as the load instruction wants it: the offset inside the workgroup's memory, which is what the low
  // half of a generic pointer to it holds.
  const uint32_t shared_address = (uint32_t)(uintptr_t)shared;

  const int32x4_t* a_global = (const int32x4_t*)(a_base + a_offset);
  const int32x4_t* b_global = (const int32x4_t*)(b_base + b_offset);
  int32x4_t* c_global = (int32x4_t*)(c_base + c_offset);
  // The same tiles seen from the workgroup (for the cooperative copy): wavefront-uniform values, said so.
  auto uniform = [](const int32x4_t* p) -> const int32x4_t* {
    const uint64_t bits = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)bits), hi = __builtin_amdgcn_readfirstlane((uint32_t)(bits >> 32));
    return (const int32x4_t*)(uintptr_t)((uint64_t)hi << 32 | lo);
  };
  const int32x4_t* a_tile_global = uniform(a_global - a_thread_relative_offset);
  const int32x4_t* b_tile_global = uniform(b_global - b_thread_relative_offset);

  int32x4_t c_regs[kMaxIntrinsics][kMaxIntrinsics];
  for (int m = 0; m < intrinsics_m; ++m)
    for (int n = 0; n < intrinsics_n; ++n) c_regs[m][n] = c_global[64 * (m * intrinsics_n + n)];

  // This wavefront's share of the copy of one outer-K step: the 64 vectors from subgroup_id*64 + i*numthreads
  // of each staged tile, i < copies. Loads per wavefront and step:
  const int a_copies = a_tile.num_shared_vecs / numthreads, b_copies = b_tile.num_shared_vecs / numthreads;
  const int loads = a_copies + b_copies;
  const bool staged = shared_vecs != 0;
  // Steps in flight ahead of the one being multiplied; the counter of outstanding loads has 6 bits.
  int ahead = staged ? buffers - 1 : 0;
  while (ahead > 1 && (ahead - 1) * loads > 63) --ahead;
  const int last_step = k_size - 1;
  auto issue_step = [&](int k_outer, int buffer) {
    const int k = k_outer < last_step ? k_outer : last_step;  // beyond the end: redundant, keeps the counts uniform
    const uint32_t lane_bytes = 16 * (uint32_t)lane_id;
    for (int i = 0; i < a_copies; ++i) {
      const int first = i * numthreads + 64 * subgroup_id;
      load_vectors_to_lds(shared_address + 16 * (uint32_t)(buffer * shared_vecs + first),
                          a_tile_global + (int64_t)k * a_tile.num_vecs + first, lane_bytes);
    }
    for (int i = 0; i < b_copies; ++i) {
      const int first = i * numthreads + 64 * subgroup_id;
      load_vectors_to_lds(shared_address + 16 * (uint32_t)(buffer * shared_vecs + a_tile.num_shared_vecs + first),
                          b_tile_global + (int64_t)k * b_tile.num_vecs + first, lane_bytes);
    }
  };
  if (staged && k_size > 0) {
    for (int s = 0; s < ahead; ++s) issue_step(s, s);
    wait_for_all_loads_but((ahead - 1) * loads);
    __syncthreads();
  }

  int buffer = 0, fill = ahead % (buffers > 0 ? buffers : 1);  // the buffer being read, the buffer being filled
  for (int k_outer = 0; k_outer < k_size; ++k_outer) {
    // The buffer `fill` was last read in the previous step, which ended with a barrier.
    if (staged) issue_step(k_outer + ahead, fill);
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
      // The next step's tiles have landed (this wavefront's share; after the barrier everyone's), and everyone
      // is done reading this step's.
      wait_for_all_loads_but((ahead - 1) * loads);
      __syncthreads();
      buffer = buffer + 1 == buffers ? 0 : buffer + 1;
      fill = fill + 1 == buffers ? 0 : fill + 1;
    }
  }
  // No load may still be writing workgroup memory when the caller gets it back.
  if (staged) wait_for_all_loads_but<0>();

  for (int m = 0; m < intrinsics_m; ++m)
    for (int n = 0; n < intrinsics_n; ++n) c_global[64 * (m * intrinsics_n + n)] = c_regs[m][n];
}

#endif  // IREE_AMD_CSRC_DEVICE_IREE_UK_AMDGPU_MULTI_MMA_MFMA_I32_16X16X64_I8_H_
