/* libiree_uk_mi355x_plugin.so: the ukernels as a HAL executable plugin.
 *
 * One exported function, the one the reference runtime looks up by name when
 * it loads a plugin library
 * (runtime/src/iree/hal/local/executable_plugin.h:185-191, name :190-191). It
 * returns the version-0.1 interface (header, load, unload, resolve; :404-460)
 * or NULL when the caller's `max_version` is older than that. `resolve` knows
 * the imports iree_uk_mmt4d, iree_uk_pack, iree_uk_unpack and
 * iree_uk_query_tile_sizes.2d; each is a thunk
 * `int fn(void* params_ptr, void* context, void* reserved)` over the C ABI of
 * iree_uk_mi355x.h. */
#ifndef IREE_UK_MI355X_PLUGIN_H_
#define IREE_UK_MI355X_PLUGIN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct iree_hal_executable_plugin_header_t;

const struct iree_hal_executable_plugin_header_t** iree_hal_executable_plugin_query(uint32_t max_version,
                                                                                   void* reserved);

#ifdef __cplusplus
}
#endif

#endif /* IREE_UK_MI355X_PLUGIN_H_ */
