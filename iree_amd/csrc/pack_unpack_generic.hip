// pack / unpack for any tile shape, element size, stride and flag combination:
// one thread per element of the tiled buffer (pack) or of the 2-D buffer
// (unpack), walking the index map of the reference (tools/pack_test.c:13-71,
// tools/unpack_test.c:13-58). These are the fallbacks behind the LDS-staged
// kernels in pack_unpack_tiled.hip.
#include "uk_internal.h"

namespace uk {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void pack_generic_kernel(PackArgs a, int64_t total) {
  const bool tr_inner = a.flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER;
  const bool tr_outer = a.flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER;
  const int64_t S2 = a.out_size2, S3 = a.out_size3;
  const int64_t tile_elems = S2 * S3;
  const int64_t row_elems = a.out_size1 * tile_elems;
  const T* in = (const T*)a.in;
  T* out = (T*)a.out;
  const T pad = (T)a.padding_value;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    // Position in the tiled buffer, in its own dimension order.
    const int64_t q0 = idx / row_elems;
    const int64_t c = idx - q0 * row_elems;
    const int64_t q1 = c / tile_elems;
    const int64_t w = c - q1 * tile_elems;
    const int64_t u2 = w / S3;
    const int64_t u3 = w - u2 * S3;
    // The same position seen from the 2-D side.
    const int64_t o0 = tr_outer ? q1 : q0, o1 = tr_outer ? q0 : q1;
    const int64_t t0 = tr_inner ? u3 : u2, t1 = tr_inner ? u2 : u3;
    const int64_t T0 = tr_inner ? S3 : S2, T1 = tr_inner ? S2 : S3;
    const int64_t i0 = o0 * T0 + t0, i1 = o1 * T1 + t1;
    T v = pad;
    if (i0 < a.in_size0 && i1 < a.in_size1) v = in[i0 * a.in_stride0 + i1 * a.in_stride1];
    out[q0 * a.out_stride0 + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void unpack_generic_kernel(UnpackArgs a, int64_t total) {
  const bool tr_inner = a.flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER;
  const bool tr_outer = a.flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER;
  const int64_t S2 = a.in_size2, S3 = a.in_size3;
  const int64_t T0 = tr_inner ? S3 : S2, T1 = tr_inner ? S2 : S3;
  const int64_t tile_elems = S2 * S3;
  const T* in = (const T*)a.in;
  T* out = (T*)a.out;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t i0 = idx / a.out_size1;
    const int64_t i1 = idx - i0 * a.out_size1;
    const int64_t o0 = i0 / T0, t0 = i0 - o0 * T0;
    const int64_t o1 = i1 / T1, t1 = i1 - o1 * T1;
    const int64_t q0 = tr_outer ? o1 : o0, q1 = tr_outer ? o0 : o1;
    const int64_t u2 = tr_inner ? t1 : t0, u3 = tr_inner ? t0 : t1;
    out[i0 * a.out_stride0 + i1 * a.out_stride1] =
        in[q0 * a.in_stride0 + q1 * tile_elems + u2 * S3 + u3];
  }
}

unsigned grid_for(int64_t total) {
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  return (unsigned)blocks;
}

}  // namespace

hipError_t launch_pack_generic(const PackArgs& a, hipStream_t stream, const char** name) {
  const int64_t total = a.out_size0 * a.out_size1 * a.out_size2 * a.out_size3;
  if (total == 0) return hipSuccess;
  *name = "pack_generic";
  const dim3 grid(grid_for(total)), block(256);
  switch (a.elem_bytes) {
    case 1: hipLaunchKernelGGL(pack_generic_kernel<uint8_t>, grid, block, 0, stream, a, total); break;
    case 2: hipLaunchKernelGGL(pack_generic_kernel<uint16_t>, grid, block, 0, stream, a, total); break;
    case 4: hipLaunchKernelGGL(pack_generic_kernel<uint32_t>, grid, block, 0, stream, a, total); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_unpack_generic(const UnpackArgs& a, hipStream_t stream, const char** name) {
  const int64_t total = a.out_size0 * a.out_size1;
  if (total == 0) return hipSuccess;
  *name = "unpack_generic";
  const dim3 grid(grid_for(total)), block(256);
  switch (a.elem_bytes) {
    case 2: hipLaunchKernelGGL(unpack_generic_kernel<uint16_t>, grid, block, 0, stream, a, total); break;
    case 4: hipLaunchKernelGGL(unpack_generic_kernel<uint32_t>, grid, block, 0, stream, a, total); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace uk
