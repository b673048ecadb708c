// Kernel instantiations of the MFMA mmt4d for one operand type (see
// mmt4d_mfma_kernels.h).
#define UK_MFMA_KERNEL_BODIES
#include "mmt4d_mfma_kernels.h"

namespace uk {

hipError_t launch_mfma_i8(const MfmaArgs& m, int gather, bool rhs_i4, hipStream_t stream, const char** name) {
  if (rhs_i4) return launch_variant<kI8, true, 16, false>(m, stream, name);
  switch (gather) {
    case 16: return launch_variant<kI8, false, 16, false>(m, stream, name);
    case 8: return launch_variant<kI8, false, 8, false>(m, stream, name);
    case 4: return launch_variant<kI8, false, 4, false>(m, stream, name);
    case 1: return launch_variant<kI8, false, 1, false>(m, stream, name);
    default: return launch_variant<kI8, false, 2, false>(m, stream, name);
  }
}

bool mfma_direct_covers(const MfmaArgs& m, int gather, bool rhs_i4) {
  if (rhs_i4) return direct_covers<true, 16>(m);
  switch (gather) {
    case 16: return direct_covers<false, 16>(m);
    case 8: return direct_covers<false, 8>(m);
    case 4: return direct_covers<false, 4>(m);
    case 1: return direct_covers<false, 1>(m);
    default: return direct_covers<false, 2>(m);
  }
}

}  // namespace uk
