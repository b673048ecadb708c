// Selection between the LDS-staged pack/unpack kernels and the generic ones.
#include "uk_internal.h"

namespace uk {

hipError_t launch_pack_generic(const PackArgs& a, hipStream_t stream, const char** name);
hipError_t launch_unpack_generic(const UnpackArgs& a, hipStream_t stream, const char** name);

hipError_t launch_pack(const PackArgs& a, hipStream_t stream, const char** name) {
  return launch_pack_generic(a, stream, name);
}

hipError_t launch_unpack(const UnpackArgs& a, hipStream_t stream, const char** name) {
  return launch_unpack_generic(a, stream, name);
}

}  // namespace uk
