// mmt4d for any type flag and any (M0, N0, K0): one thread per output element,
// each running the sum over k (outer) and k0 (inner) sequentially in the order
// of the reference's generic tile functions (mmt4d_tile_generic.c:11-376), so
// integer results are bit-exact and float results repeat the reference's
// sequence of f32 operations. This is the fallback behind the MFMA kernels; it
// is correct everywhere and fast nowhere.
#include "uk_device.h"
#include "uk_internal.h"

namespace uk {
namespace {

struct ElemCoord {
  int64_t i, j;
  int32_t i0, j0;
};

__device__ __forceinline__ ElemCoord decode(int64_t idx, int64_t N, int32_t M0, int32_t N0) {
  const int64_t tile_elems = (int64_t)M0 * N0;
  const int64_t tile = idx / tile_elems;
  const int32_t e = (int32_t)(idx - tile * tile_elems);
  ElemCoord c;
  c.i = tile / N;
  c.j = tile - c.i * N;
  c.i0 = e / N0;
  c.j0 = e - c.i0 * N0;
  return c;
}

// TYPE is the IREE_UK_FLAG_MMT4D_TYPE_* value.
template <uint32_t TYPE>
__global__ __launch_bounds__(256) void mmt4d_generic_kernel(Mmt4dArgs a, int64_t total) {
  const bool accumulate = a.flags & IREE_UK_FLAG_MMT4D_ACCUMULATE;
  const bool skip_round = a.flags & IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS;
  const int64_t K = a.K;
  const int32_t M0 = a.M0, N0 = a.N0, K0 = a.K0;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const ElemCoord c = decode(idx, a.N, M0, N0);
    const int64_t out_index = c.i * a.out_stride0 + c.j * M0 * N0 + (int64_t)c.i0 * N0 + c.j0;
    // Element index of (k=0, i0, k0=0) in the lhs panel and (k=0, j0, k0=0) in
    // the rhs panel; consecutive k are M0*K0 resp. N0*K0 elements apart.
    const int64_t l0 = c.i * a.lhs_stride0 + (int64_t)c.i0 * K0;
    const int64_t r0 = c.j * a.rhs_stride0 + (int64_t)c.j0 * K0;
    const int64_t lstep = (int64_t)M0 * K0, rstep = (int64_t)N0 * K0;

    if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_S8S8S32) {
      const int8_t* l = (const int8_t*)a.lhs + l0;
      const int8_t* r = (const int8_t*)a.rhs + r0;
      int32_t* o = (int32_t*)a.out + out_index;
      uint32_t acc = accumulate ? (uint32_t)*o : 0u;
      for (int64_t k = 0; k < K; ++k)
        for (int k0 = 0; k0 < K0; ++k0)
          acc += (uint32_t)((int32_t)l[k * lstep + k0] * (int32_t)r[k * rstep + k0]);
      *o = (int32_t)acc;
    } else if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_S8S4S32 ||
                         TYPE == IREE_UK_FLAG_MMT4D_TYPE_S16U4S32) {
      // rhs rows are K0/2 bytes; element 2b sits in the low nibble of byte b.
      const uint8_t* r = a.rhs + r0 / 2;
      int32_t* o = (int32_t*)a.out + out_index;
      uint32_t acc = accumulate ? (uint32_t)*o : 0u;
      for (int64_t k = 0; k < K; ++k) {
        for (int k0 = 0; k0 < K0; ++k0) {
          const uint8_t byte = r[k * (rstep / 2) + (k0 >> 1)];
          int32_t rv = (k0 & 1) ? (byte >> 4) : (byte & 0xF);
          int32_t lv;
          if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_S8S4S32) {
            rv = (rv ^ 8) - 8;
            lv = ((const int8_t*)a.lhs)[l0 + k * lstep + k0];
          } else {
            lv = ((const int16_t*)a.lhs)[l0 + k * lstep + k0];
          }
          acc += (uint32_t)(lv * rv);
        }
      }
      *o = (int32_t)acc;
    } else if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32 ||
                         TYPE == IREE_UK_FLAG_MMT4D_TYPE_S16S8S32) {
      const int16_t* l = (const int16_t*)a.lhs + l0;
      int32_t* o = (int32_t*)a.out + out_index;
      uint32_t acc = accumulate ? (uint32_t)*o : 0u;
      for (int64_t k = 0; k < K; ++k)
        for (int k0 = 0; k0 < K0; ++k0) {
          int32_t rv;
          if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32)
            rv = ((const int16_t*)a.rhs)[r0 + k * rstep + k0];
          else
            rv = ((const int8_t*)a.rhs)[r0 + k * rstep + k0];
          acc += (uint32_t)((int32_t)l[k * lstep + k0] * rv);
        }
      *o = (int32_t)acc;
    } else if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_F32F32F32) {
      const float* l = (const float*)a.lhs + l0;
      const float* r = (const float*)a.rhs + r0;
      float* o = (float*)a.out + out_index;
      float acc = accumulate ? *o : 0.f;
      // Separate multiply and add, each rounded: no fused contraction.
      for (int64_t k = 0; k < K; ++k)
        for (int k0 = 0; k0 < K0; ++k0)
          acc = __fadd_rn(acc, __fmul_rn(l[k * lstep + k0], r[k * rstep + k0]));
      *o = acc;
    } else if constexpr (TYPE == IREE_UK_FLAG_MMT4D_TYPE_F16F16F32 ||
                         TYPE == IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32) {
      constexpr int EB = TYPE == IREE_UK_FLAG_MMT4D_TYPE_F16F16F32 ? 5 : 8;
      const uint16_t* l = (const uint16_t*)a.lhs + l0;
      const uint16_t* r = (const uint16_t*)a.rhs + r0;
      float* o = (float*)a.out + out_index;
      float acc = accumulate ? *o : 0.f;
      for (int64_t k = 0; k < K; ++k)
        for (int k0 = 0; k0 < K0; ++k0)
          acc = __fadd_rn(acc, __fmul_rn(widen16<EB>(l[k * lstep + k0]),
                                         widen16<EB>(r[k * rstep + k0])));
      *o = acc;
    } else {  // F16F16F16, BF16BF16BF16
      constexpr int EB = TYPE == IREE_UK_FLAG_MMT4D_TYPE_F16F16F16 ? 5 : 8;
      const uint16_t* l = (const uint16_t*)a.lhs + l0;
      const uint16_t* r = (const uint16_t*)a.rhs + r0;
      uint16_t* o = (uint16_t*)a.out + out_index;
      if (skip_round) {
        float acc = accumulate ? widen16<EB>(*o) : 0.f;
        for (int64_t k = 0; k < K; ++k)
          for (int k0 = 0; k0 < K0; ++k0)
            acc = __fadd_rn(acc, __fmul_rn(widen16<EB>(l[k * lstep + k0]),
                                           widen16<EB>(r[k * rstep + k0])));
        *o = narrow16<EB>(acc);
      } else {
        uint16_t acc = accumulate ? *o : (uint16_t)0;
        for (int64_t k = 0; k < K; ++k)
          for (int k0 = 0; k0 < K0; ++k0)
            acc = narrow16<EB>(__fadd_rn(widen16<EB>(acc),
                                         __fmul_rn(widen16<EB>(l[k * lstep + k0]),
                                                   widen16<EB>(r[k * rstep + k0]))));
        *o = acc;
      }
    }
  }
}

template <uint32_t TYPE>
hipError_t launch_typed(const Mmt4dArgs& a, int64_t total, hipStream_t stream) {
  const int block = 256;
  int64_t blocks = (total + block - 1) / block;
  if (blocks > 256 * 64) blocks = 256 * 64;  // grid-stride beyond that
  hipLaunchKernelGGL(mmt4d_generic_kernel<TYPE>, dim3((unsigned)blocks), dim3(block), 0, stream, a,
                     total);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_mmt4d_generic(const Mmt4dArgs& a, hipStream_t stream, const char** name) {
  const int64_t total = a.M * a.N * a.M0 * a.N0;
  if (total == 0) return hipSuccess;
  *name = "mmt4d_generic";
  switch (a.flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
#define UK_CASE(T) \
  case T:          \
    return launch_typed<T>(a, total, stream)
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_F32F32F32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_S8S8S32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_F16F16F32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_F16F16F16);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_S16S16S32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_S16U4S32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_S16S8S32);
    UK_CASE(IREE_UK_FLAG_MMT4D_TYPE_S8S4S32);
#undef UK_CASE
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace uk
