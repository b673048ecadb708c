// Kernel instantiations of the MFMA mmt4d for one operand type (see
// mmt4d_mfma_kernels.h).
#define UK_MFMA_KERNEL_BODIES
#include "mmt4d_mfma_kernels.h"

namespace uk {

hipError_t launch_mfma_bf16(const MfmaArgs& m, int gather, bool narrow, hipStream_t stream, const char** name) {
  if (narrow) return launch_mfma_bf16_narrow(m, gather, stream, name);
  switch (gather) {
    case 16: return launch_variant<kBF16, false, 16, false>(m, stream, name);
    case 8: return launch_variant<kBF16, false, 8, false>(m, stream, name);
    case 4: return launch_variant<kBF16, false, 4, false>(m, stream, name);
    default: return launch_variant<kBF16, false, 2, false>(m, stream, name);
  }
}

}  // namespace uk
