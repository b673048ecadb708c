// In-dispatch GPU microkernel for gfx950: the inner (K) loop of a data-tiled
// int8 matmul tile with the MFMA intrinsic v_mfma_i32_16x16x64_i8, in the
// calling convention of the reference's ROCm ukernels
// (compiler/plugins/target/ROCM/builtins/ukernel/
// iree_uk_amdgpu_multi_mma_mfma_i32_16x16x32_i8.c:82-181 is the gfx942
// counterpart with the 16x16x32 intrinsic). Freestanding C23: it is compiled
// to AMDGPU bitcode (clang -std=c23 -nogpulib -target amdgcn-amd-amdhsa
// -march=gfx950 -emit-llvm) and a compiler links that bitcode into a dispatch
// and inlines this function; all the `intrinsics_*` / `subgroups_*`
// parameters are constants at that point, so the loops below unroll and the
// arrays become registers.
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
// writes its 16 bytes at M0 + 16*l), in groups of 64 consecutive vectors, one
// group per wavefront and load, into a ring of up to four buffers filled up to
// three outer-K steps ahead. One counter wait and one workgroup barrier per
// step. The shared-memory size query accounts for the ring.
//
// Any parameter combination is handled: a staged tile is 64 * intrinsics *
// intrinsics_k * subgroups vectors, which need not be a multiple of the 64 *
// subgroups_m * subgroups_n threads (e.g. subgroups_m = 1, subgroups_n = 4 with
// intrinsics_m narrowed to 1, 2 or 3, which is what the reference's heuristics
// pick for narrow M). Every wavefront issues the same number of loads per
// step, ceil(groups / wavefronts) per staged tile, so that one counter wait
// fits all; a wavefront whose turn falls past the last group repeats a group
// (the same bytes to the same place).
//
// The load instruction takes its workgroup-memory address from the M0
// register. The compiler accepts no clobber for M0, and this function is
// inlined into dispatches the compiler generates, which may keep a value of
// their own in M0 (LDS-DMA builtins, indirect register indexing, s_sendmsg,
// readlane-style moves): so the inline assembly below leaves M0 as it found
// it, at the price of two scalar moves per load. The loops here index their
// register arrays with constants only.
//
// Provenance: the signature, ab_tile_info_t / get_ab_tile_info (in the
// shared-memory header), the thread-relative offset arithmetic at the top of
// the microkernel, the loops that load and store the C registers and the
// parameter list in the comment above are the reference's, nearly as they
// stand in the gfx942 file named above: they are the calling convention a
// compiler generates calls against. The K loop (ring of buffers, loads straight
// to workgroup memory, one counter wait per step, repeated groups) is this
// library's.
#include "common.h"
#include "iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_shared_memory.h"

// The bitcode of this function is interpreted during compilation to determine
// the exact shared_memory_bytes to pass to the ukernel.
int32_t iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_query_shared_memory_bytes(
    int32_t intrinsics_m, int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n, int32_t intrinsics_k) {
  ab_tile_info_t a_tile = get_ab_tile_info(intrinsics_m * intrinsics_k, subgroups_m, subgroups_n);
  ab_tile_info_t b_tile = get_ab_tile_info(intrinsics_n * intrinsics_k, subgroups_n, subgroups_m);
  return get_shared_memory_bytes(a_tile, b_tile);
}

// 64 vectors from `base` (wavefront-uniform) + lane_byte_offset to the
// workgroup-memory address lds_address + 16 * lane.
static inline void load_vectors_to_lds(uint32_t lds_address, const int32x4_t *base, uint32_t lane_byte_offset) {
  uint32_t callers_m0;
  __asm__ volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                   : "=&s"(callers_m0)
                   : "s"(lds_address), "v"(lane_byte_offset), "s"(base)
                   : "memory");
}

// Waits until at most `n` of this wavefront's loads are outstanding. The
// instruction takes an immediate; `n` is a constant once the microkernel's
// parameters are, which leaves one case.
static inline void wait_for_all_loads_but(int n) {
#define WAIT_CASE(N) \
  case N:            \
    __asm__ volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); \
    break;
#define WAIT_CASES8(A, B, C, D, E, F, G, H) \
  WAIT_CASE(A) WAIT_CASE(B) WAIT_CASE(C) WAIT_CASE(D) WAIT_CASE(E) WAIT_CASE(F) WAIT_CASE(G) WAIT_CASE(H)
  switch (n) {
    WAIT_CASES8(0, 1, 2, 3, 4, 5, 6, 7)
    WAIT_CASES8(8, 9, 10, 11, 12, 13, 14, 15)
    WAIT_CASES8(16, 17, 18, 19, 20, 21, 22, 23)
    WAIT_CASES8(24, 25, 26, 27, 28, 29, 30, 31)
    WAIT_CASES8(32, 33, 34, 35, 36, 37, 38, 39)
    WAIT_CASES8(40, 41, 42, 43, 44, 45, 46, 47)
    WAIT_CASES8(48, 49, 50, 51, 52, 53, 54, 55)
    WAIT_CASES8(56, 57, 58, 59, 60, 61, 62, 63)
    default:  // more than the 6-bit counter holds: wait for everything
      __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
      break;
  }
#undef WAIT_CASES8
#undef WAIT_CASE
}

// The compiler keeps its own count of the loads it has issued and waits for
// a loaded register at its first use. It does not see the loads issued by the
// inline assembly above, and the counter completes in order: a first use of
// the loaded accumulators inside the K loop becomes a wait in every trip, which
// then also waits for the tile loads issued moments before and so undoes the
// ring. An empty statement that uses the accumulators puts that wait in front
// of the loop instead, once.
static inline void accumulators_have_arrived(int32x4_t *c) { __asm__ volatile("" : "+a"(*c)); }

// A pointer that is the same in every lane, said so to the compiler.
static inline const int32x4_t *wavefront_uniform(const int32x4_t *p) {
  const uint64_t bits = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)bits);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(bits >> 32));
  return (const int32x4_t *)((uint64_t)hi << 32 | lo);
}

// This wavefront's loads of one outer-K step of one staged tile: the groups of
// 64 vectors number wavefront, wavefront + wavefronts, ... of the tile's
// `groups`; `count` = ceil(groups / wavefronts) for every wavefront, a turn
// past the last group repeats group (turn % groups).
static inline void issue_tile_loads(uint32_t lds_address, const int32x4_t *tile_global, int groups, int count,
                                    int wavefront, int wavefronts, uint32_t lane_bytes) {
  for (int i = 0; i < count; ++i) {
    int group = i * wavefronts + wavefront;
    if (group >= groups) group %= groups;
    load_vectors_to_lds(lds_address + 16 * 64 * (uint32_t)group, tile_global + 64 * group, lane_bytes);
  }
}

// Microkernel for iree_gpu.multi_mma with DataTiledMMAAttr with
// intrinsic = MFMA_I32_16x16x64_I8 and a shape with outer M and N dimensions
// equal to 1 (the inner loop on the K dimension).
//
// Parameters                  | Constant?  | Description
// --------------------------- | ---------- | -----------
// a_base, a_offset            | No         | A-matrix pointer (thread-distrib.)
// b_base, b_offset            | No         | B-matrix pointer (thread-distrib.)
// c_base, c_offset            | No         | C-matrix pointer (thread-distrib.)
// shared_memory_{base,offset} | No         | Workgroup memory workspace pointer
// shared_memory_bytes         | Yes        | Its size, from the query function
// k_size                      | From shape | Size of outer K dimension
// intrinsics_m, subgroups_m   | Yes        | See DataTiledMMAAttr
// intrinsics_n, subgroups_n   | Yes        | See DataTiledMMAAttr
// intrinsics_k                | Yes        | See DataTiledMMAAttr
[[clang::always_inline]] void iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8(
    const int8_t *a_base, int64_t a_offset, const int8_t *b_base, int64_t b_offset, int32_t *c_base,
    int64_t c_offset, int8_t *shared_memory_base, int64_t shared_memory_offset, int32_t shared_memory_bytes,
    int32_t k_size, int32_t intrinsics_m, int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n,
    int32_t intrinsics_k) {
  const ab_tile_info_t a_tile = get_ab_tile_info(intrinsics_m * intrinsics_k, subgroups_m, subgroups_n);
  const ab_tile_info_t b_tile = get_ab_tile_info(intrinsics_n * intrinsics_k, subgroups_n, subgroups_m);
  const int shared_vecs = a_tile.num_shared_vecs + b_tile.num_shared_vecs;  // per buffer
  const int buffers = get_ring_buffers(shared_vecs);
  // shared_memory_bytes should match exactly, as the value ultimately comes
  // from the ..._query_shared_memory_bytes function defined just above.
  if (shared_memory_bytes != get_shared_memory_bytes(a_tile, b_tile)) {
    __builtin_trap();
  }

  const int tid = __builtin_amdgcn_workitem_id_x();
  const int wavefronts = subgroups_m * subgroups_n;
  __builtin_assume(tid < 64 * wavefronts);
  const int lane_id = tid % 64;
  const int subgroup_id = __builtin_amdgcn_readfirstlane(tid / 64);
  const int subgroup_n_idx = subgroup_id % subgroups_n;
  const int subgroup_m_idx = subgroup_id / subgroups_n;
  const int a_thread_relative_offset = intrinsics_k * (lane_id + 64 * intrinsics_m * subgroup_m_idx);
  const int b_thread_relative_offset = intrinsics_k * (lane_id + 64 * intrinsics_n * subgroup_n_idx);

  // Workgroup memory: [buffers][A vectors, then B vectors].
  int32x4_t *shared = (int32x4_t *)(shared_memory_base + shared_memory_offset);
  // Its address as the load instruction wants it: the offset inside the
  // workgroup's memory, which is what the low half of a generic pointer to it
  // holds.
  const uint32_t shared_address = (uint32_t)(uint64_t)shared;

  const int32x4_t *a_global = (const int32x4_t *)(a_base + a_offset);
  const int32x4_t *b_global = (const int32x4_t *)(b_base + b_offset);
  int32x4_t *c_global = (int32x4_t *)(c_base + c_offset);
  // The same tiles seen from the workgroup (for the cooperative copy).
  const int32x4_t *a_tile_global = wavefront_uniform(a_global - a_thread_relative_offset);
  const int32x4_t *b_tile_global = wavefront_uniform(b_global - b_thread_relative_offset);

  // Load existing accumulators from global memory into registers. The VLAs
  // become normal arrays after inlining.
  int32x4_t c_regs[intrinsics_m][intrinsics_n];
  // One K-step's B operands. (Declared here, not inside the loops: a variable
  // length array in a loop stays a stack allocation after inlining.)
  int32x4_t b_regs[intrinsics_n];
  for (int m = 0; m < intrinsics_m; ++m) {
    for (int n = 0; n < intrinsics_n; ++n) {
      c_regs[m][n] = c_global[64 * (m * intrinsics_n + n)];
    }
  }

  // Loads per wavefront and step.
  const int a_groups = a_tile.num_shared_vecs / 64, b_groups = b_tile.num_shared_vecs / 64;
  const int a_copies = (a_groups + wavefronts - 1) / wavefronts;
  const int b_copies = (b_groups + wavefronts - 1) / wavefronts;
  const int loads = a_copies + b_copies;
  const int staged = shared_vecs != 0;
  // Steps in flight ahead of the one being multiplied; the counter of
  // outstanding loads has 6 bits.
  int ahead = staged ? buffers - 1 : 0;
  while (ahead > 1 && (ahead - 1) * loads > 63) --ahead;
  const int last_step = k_size - 1;
  const uint32_t lane_bytes = 16 * (uint32_t)lane_id;

  if (staged && k_size > 0) {
    for (int s = 0; s < ahead; ++s) {
      const int k = s < last_step ? s : last_step;  // beyond the end: redundant, keeps the counts uniform
      issue_tile_loads(shared_address + 16 * (uint32_t)(s * shared_vecs), a_tile_global + (int64_t)k * a_tile.num_vecs,
                       a_groups, a_copies, subgroup_id, wavefronts, lane_bytes);
      issue_tile_loads(shared_address + 16 * (uint32_t)(s * shared_vecs + a_tile.num_shared_vecs),
                       b_tile_global + (int64_t)k * b_tile.num_vecs, b_groups, b_copies, subgroup_id, wavefronts,
                       lane_bytes);
    }
    wait_for_all_loads_but((ahead - 1) * loads);
    workgroup_barrier();
  }
  for (int m = 0; m < intrinsics_m; ++m) {
    for (int n = 0; n < intrinsics_n; ++n) accumulators_have_arrived(&c_regs[m][n]);
  }

  // The buffer being read and the buffer being filled.
  int buffer = 0, fill = ahead % (buffers > 0 ? buffers : 1);
  for (int k_outer = 0; k_outer < k_size; ++k_outer) {
    if (staged) {
      // The buffer `fill` was last read in the previous step, which ended with a barrier.
      const int k = k_outer + ahead < last_step ? k_outer + ahead : last_step;
      issue_tile_loads(shared_address + 16 * (uint32_t)(fill * shared_vecs),
                       a_tile_global + (int64_t)k * a_tile.num_vecs, a_groups, a_copies, subgroup_id, wavefronts,
                       lane_bytes);
      issue_tile_loads(shared_address + 16 * (uint32_t)(fill * shared_vecs + a_tile.num_shared_vecs),
                       b_tile_global + (int64_t)k * b_tile.num_vecs, b_groups, b_copies, subgroup_id, wavefronts,
                       lane_bytes);
    }
    const int32x4_t *a_vecs = a_tile.num_shared_vecs ? shared + buffer * shared_vecs + a_thread_relative_offset
                                                     : a_global + (int64_t)k_outer * a_tile.num_vecs;
    const int32x4_t *b_vecs = b_tile.num_shared_vecs
                                  ? shared + buffer * shared_vecs + a_tile.num_shared_vecs + b_thread_relative_offset
                                  : b_global + (int64_t)k_outer * b_tile.num_vecs;
    for (int k = 0; k < intrinsics_k; ++k) {
      for (int n = 0; n < intrinsics_n; ++n) {
        b_regs[n] = b_vecs[64 * intrinsics_k * n + k];
      }
      for (int m = 0; m < intrinsics_m; ++m) {
        const int32x4_t a_reg = a_vecs[64 * intrinsics_k * m + k];
        for (int n = 0; n < intrinsics_n; ++n) {
          c_regs[m][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_reg, b_regs[n], c_regs[m][n], 0, 0, 0);
        }
      }
    }
    if (staged) {
      // The next step's tiles have landed (this wavefront's share; after the
      // barrier everyone's), and everyone is done reading this step's.
      wait_for_all_loads_but((ahead - 1) * loads);
      workgroup_barrier();
      buffer = buffer + 1 == buffers ? 0 : buffer + 1;
      fill = fill + 1 == buffers ? 0 : fill + 1;
    }
  }
  // No load may still be writing workgroup memory when the caller gets it back.
  if (staged) wait_for_all_loads_but(0);

  // Store accumulators.
  for (int m = 0; m < intrinsics_m; ++m) {
    for (int n = 0; n < intrinsics_n; ++n) {
      c_global[64 * (m * intrinsics_n + n)] = c_regs[m][n];
    }
  }
}
