// Host-callable wrapper around the in-dispatch int8 microkernel
// (device/iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8.c): one workgroup per
// (outer m, outer n) tile of a data-tiled matmul, each running the
// microkernel's K loop. It exists to test and measure the microkernel the way
// a compiled dispatch uses it: the microkernel is not compiled as part of this
// file but linked in as the AMDGPU bitcode built from its freestanding C23
// source (iree_amd/build.py passes it to the device pass with
// -mlink-builtin-bitcode), and inlined, with the parameter combinations of the
// template instantiations below as its compile-time constants.
#include "device/iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_shared_memory.h"
#include "uk_internal.h"

// Defined by the bitcode.
extern "C" __device__ void iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8(
    const int8_t* a_base, int64_t a_offset, const int8_t* b_base, int64_t b_offset, int32_t* c_base,
    int64_t c_offset, int8_t* shared_memory_base, int64_t shared_memory_offset, int32_t shared_memory_bytes,
    int32_t k_size, int32_t intrinsics_m, int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n,
    int32_t intrinsics_k);
extern "C" __device__ int32_t iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_query_shared_memory_bytes(
    int32_t intrinsics_m, int32_t subgroups_m, int32_t intrinsics_n, int32_t subgroups_n, int32_t intrinsics_k);

namespace uk {
namespace {

struct MultiMmaArgs {
  const int8_t* a;
  const int8_t* b;
  int32_t* c;
  int64_t outer_n;
  int32_t k_size;
};

template <int IM, int SM, int IN, int SN, int IK>
__global__ __launch_bounds__(64 * SM * SN) void multi_mma_kernel(const MultiMmaArgs g) {
  extern __shared__ __attribute__((aligned(16))) int8_t workgroup_memory[];
  // What a compiler does at compile time by interpreting the bitcode; here the
  // call folds to a constant once the bitcode is inlined.
  const int32_t shared_bytes =
      iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8_query_shared_memory_bytes(IM, SM, IN, SN, IK);
  const int64_t outer_m = blockIdx.y, outer_n = blockIdx.x;
  const int tid = threadIdx.x, lane = tid % 64, subgroup = tid / 64;
  const int subgroup_n = subgroup % SN, subgroup_m = subgroup / SN;
  // Tiles: A [outer_m][k][SM][IM][64][IK], B [outer_n][k][SN][IN][64][IK],
  // C [outer_m][outer_n][SM][SN][IM][IN][64], in 16-byte vectors.
  const int64_t a_tile_vecs = 64 * IM * IK * SM, b_tile_vecs = 64 * IN * IK * SN;
  const int64_t c_tile_vecs = 64 * IM * IN * SM * SN;
  const int64_t a_vec = outer_m * g.k_size * a_tile_vecs + IK * (lane + 64 * IM * subgroup_m);
  const int64_t b_vec = outer_n * g.k_size * b_tile_vecs + IK * (lane + 64 * IN * subgroup_n);
  const int64_t c_vec = (outer_m * g.outer_n + outer_n) * c_tile_vecs + 64 * IM * IN * (subgroup_m * SN + subgroup_n) + lane;
  iree_uk_amdgpu_multi_mma_mfma_i32_16x16x64_i8(g.a, 16 * a_vec, g.b, 16 * b_vec, g.c, 4 * c_vec, workgroup_memory, 0,
                                                shared_bytes, g.k_size, IM, SM, IN, SN, IK);
}

template <int IM, int SM, int IN, int SN, int IK>
hipError_t launch(const MultiMmaArgs& g, int64_t outer_m, hipStream_t stream) {
  // The same arithmetic as the bitcode's query function, from the header both share.
  const int32_t shared_bytes =
      get_shared_memory_bytes(get_ab_tile_info(IM * IK, SM, SN), get_ab_tile_info(IN * IK, SN, SM));
  if (shared_bytes > 160 * 1024) return hipErrorInvalidValue;
  auto kernel = multi_mma_kernel<IM, SM, IN, SN, IK>;
  if (shared_bytes > 65536) {
    const hipError_t attr = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, shared_bytes);
    if (attr != hipSuccess) return attr;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)g.outer_n, (unsigned)outer_m), dim3(64 * SM * SN), shared_bytes, stream, g);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_multi_mma_i8(const void* a, const void* b, void* c, int64_t outer_m, int64_t outer_n, int32_t k_size,
                               int intrinsics_m, int subgroups_m, int intrinsics_n, int subgroups_n, int intrinsics_k,
                               hipStream_t stream) {
  if (outer_m <= 0 || outer_n <= 0 || outer_m > 65535 || outer_n > 0x7FFFFFFF || k_size < 0) return hipErrorInvalidValue;
  MultiMmaArgs g{(const int8_t*)a, (const int8_t*)b, (int32_t*)c, outer_n, k_size};
  const int key = intrinsics_m * 10000 + subgroups_m * 1000 + intrinsics_n * 100 + subgroups_n * 10 + intrinsics_k;
  switch (key) {
    case 82821: return launch<8, 2, 8, 2, 1>(g, outer_m, stream);  // 256x256 per workgroup, K 64 per step
    case 82822: return launch<8, 2, 8, 2, 2>(g, outer_m, stream);  // K 128 per step
    case 42421: return launch<4, 2, 4, 2, 1>(g, outer_m, stream);  // 128x128
    case 44411: return launch<4, 4, 4, 1, 1>(g, outer_m, stream);  // 256x64: only B staged
    case 21221: return launch<2, 1, 2, 2, 1>(g, outer_m, stream);  // only A staged
    case 21212: return launch<2, 1, 2, 1, 2>(g, outer_m, stream);  // one subgroup, nothing staged
    // What the reference's heuristics emit for wide N (subgroups 1 x 4), with M narrowed: the staged A tile is
    // smaller than, or not a multiple of, the 256 threads.
    case 81241: return launch<8, 1, 2, 4, 1>(g, outer_m, stream);
    case 11241: return launch<1, 1, 2, 4, 1>(g, outer_m, stream);
    case 21241: return launch<2, 1, 2, 4, 1>(g, outer_m, stream);
    case 31242: return launch<3, 1, 2, 4, 2>(g, outer_m, stream);
    case 32521: return launch<3, 2, 5, 2, 1>(g, outer_m, stream);  // odd counts on both sides
    default: return hipErrorInvalidValue;
  }
}

}  // namespace uk
