// Placeholder selectors until the specialised kernels land.
#include "uk_internal.h"
namespace uk {
Mmt4dLauncher select_mmt4d_i8_mfma(const Mmt4dArgs&, bool) { return nullptr; }
Mmt4dLauncher select_mmt4d_f16_mfma(const Mmt4dArgs&, bool) { return nullptr; }
Mmt4dLauncher select_mmt4d_gemv(const Mmt4dArgs&, bool) { return nullptr; }
Mmt4dLauncher select_mmt4d_s8s4_mfma(const Mmt4dArgs&, bool) { return nullptr; }
}  // namespace uk
