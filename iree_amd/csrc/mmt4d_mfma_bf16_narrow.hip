// Kernel instantiations of the MFMA mmt4d for one operand type with a 16-bit
// output (one rounding at the end; see mmt4d_mfma_kernels.h). A translation
// unit of their own so that they compile beside the f32-output ones.
#define UK_MFMA_KERNEL_BODIES
#include "mmt4d_mfma_kernels.h"

namespace uk {

hipError_t launch_mfma_bf16_narrow(const MfmaArgs& m, int gather, hipStream_t stream, const char** name) {
  switch (gather) {
    case 16: return launch_variant<kBF16, false, 16, true>(m, stream, name);
    case 8: return launch_variant<kBF16, false, 8, true>(m, stream, name);
    case 4: return launch_variant<kBF16, false, 4, true>(m, stream, name);
    default: return launch_variant<kBF16, false, 2, true>(m, stream, name);
  }
}

}  // namespace uk
