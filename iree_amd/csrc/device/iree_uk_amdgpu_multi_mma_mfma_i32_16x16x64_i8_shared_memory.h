// Workgroup-memory budget of the gfx950 multi_mma microkernel
// (iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8.c): which tiles are staged and
// how many buffers the ring has. Plain C without any include, so that the
// freestanding device source and host code that launches it (tests, the
// benchmark wrapper) compute the same number.
#ifndef IREE_AMD_CSRC_DEVICE_MULTI_MMA_MFMA_I32_16X16X64_I8_SHARED_MEMORY_H_
#define IREE_AMD_CSRC_DEVICE_MULTI_MMA_MFMA_I32_16X16X64_I8_SHARED_MEMORY_H_

// Encodes some information about an A/B tile, in vectors of 16 bytes.
typedef struct ab_tile_info_t {
  int num_vecs;         // vectors in one outer-K step of the tile
  int num_shared_vecs;  // of which staged in workgroup memory (all or none)
} ab_tile_info_t;

static inline ab_tile_info_t get_ab_tile_info(int tile_intrinsics, int tile_subgroups, int opposite_tile_subgroups) {
  ab_tile_info_t info;
  info.num_vecs = /*subgroup size*/ 64 * tile_intrinsics * tile_subgroups;
  // Workgroup memory pays off when more than one subgroup reads the tile.
  info.num_shared_vecs = opposite_tile_subgroups > 1 ? info.num_vecs : 0;
  return info;
}

// Buffers in the ring of staged tiles, two to four. A step of 32 KiB or more
// belongs to a tile that fills the register file with one workgroup per
// compute unit: as many buffers as fit 128 KiB. Smaller tiles run several
// workgroups per compute unit, which hide each other's waits: the ring stays
// within 32 KiB so that they still all fit.
static inline int get_ring_buffers(int shared_vecs_per_step) {
  if (shared_vecs_per_step == 0) return 0;
  const int step_bytes = 16 * shared_vecs_per_step;
  const int fit = (step_bytes >= 32 * 1024 ? 128 * 1024 : 32 * 1024) / step_bytes;
  return fit >= 4 ? 4 : (fit >= 2 ? fit : 2);
}

static inline int get_shared_memory_bytes(ab_tile_info_t a_tile, ab_tile_info_t b_tile) {
  const int vecs = a_tile.num_shared_vecs + b_tile.num_shared_vecs;
  return get_ring_buffers(vecs) * 16 * vecs;
}

#endif  // IREE_AMD_CSRC_DEVICE_MULTI_MMA_MFMA_I32_16X16X64_I8_SHARED_MEMORY_H_
