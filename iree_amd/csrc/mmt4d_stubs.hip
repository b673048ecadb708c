// Placeholder selector until the skinny-matrix kernel lands.
#include "uk_internal.h"
namespace uk {
Mmt4dLauncher select_mmt4d_gemv(const Mmt4dArgs&, bool) { return nullptr; }
}  // namespace uk
