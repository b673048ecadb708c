// Kernel instantiations of the MFMA mmt4d for one operand type (see
// mmt4d_mfma_kernels.h).
#define UK_MFMA_KERNEL_BODIES
#include "mmt4d_mfma_kernels.h"

namespace uk {

hipError_t launch_mfma_i8(const MfmaArgs& m, int gather, bool rhs_i4, hipStream_t stream, const char** name) {
  if (rhs_i4) return launch_variant<kI8, true, 16, false>(m, stream, name);
  return gather == 16 ? launch_variant<kI8, false, 16, false>(m, stream, name)
                      : launch_variant<kI8, false, 4, false>(m, stream, name);
}

}  // namespace uk
