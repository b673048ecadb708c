/* The binary interface of a HAL executable plugin, version 0.1, restated from
 * runtime/src/iree/hal/local/executable_plugin.h of the reference (the line
 * numbers below are that file's) with private names, so that this library's
 * plugin builds without the reference tree. Only what a plugin that exports
 * plain functions needs. tests/test_plugin.py compiles a layout check of
 * every struct here against the reference's own header where that exists. */
#ifndef IREE_AMD_CSRC_PLUGIN_PLUGIN_ABI_H_
#define IREE_AMD_CSRC_PLUGIN_PLUGIN_ABI_H_

#include <stddef.h>
#include <stdint.h>

#define UKP_VERSION_0_1 0x00000001u /* :143 */
#define UKP_FEATURE_NONE 0u         /* :57-72: 1u << 0 would claim "standalone" */
#define UKP_SANITIZER_NONE 0        /* :80-100 */
#define UKP_EXPORT_NAME "iree_hal_executable_plugin_query" /* :190-191 */

/* :152-180 */
typedef struct ukp_header_t {
  uint32_t version;
  const char* name;
  const char* description;
  uint32_t features;
  int32_t sanitizer; /* an enum padded to INT32_MAX, i.e. int-sized */
  uint64_t reserved[8];
} ukp_header_t;

/* :221-243: a status is a pointer-sized value whose low 5 bits are the code;
 * 0 is OK. */
typedef void* ukp_status_t;
#define UKP_STATUS_OK ((ukp_status_t)(uintptr_t)0)
#define UKP_STATUS_NOT_FOUND ((ukp_status_t)(uintptr_t)5)
#define UKP_STATUS_UNAVAILABLE ((ukp_status_t)(uintptr_t)14)

/* :278-297 */
typedef ukp_status_t (*ukp_allocator_ctl_fn_t)(void* self, int command, const void* params, void** inout_ptr);
typedef struct ukp_allocator_t {
  void* self;
  ukp_allocator_ctl_fn_t ctl;
} ukp_allocator_t;

/* :324-340 */
typedef struct ukp_string_view_t {
  const char* data;
  size_t size;
} ukp_string_view_t;
typedef struct ukp_string_pair_t {
  ukp_string_view_t first;
  ukp_string_view_t second;
} ukp_string_pair_t;

#define UKP_RESOLUTION_MISSING_OPTIONAL (1u << 0) /* :347-351 */

/* :379-391 */
typedef struct ukp_environment_v0_t {
  ukp_allocator_t host_allocator;
} ukp_environment_v0_t;
typedef struct ukp_resolve_params_v0_t {
  size_t count;
  const char* const* symbol_names;
  void** out_fn_ptrs;
  void** out_fn_contexts;
} ukp_resolve_params_v0_t;

/* :404-460 */
typedef struct ukp_plugin_v0_t {
  const ukp_header_t* header;
  ukp_status_t (*load)(const ukp_environment_v0_t* environment, size_t param_count,
                       const ukp_string_pair_t* params, void** out_self);
  void (*unload)(void* self);
  ukp_status_t (*resolve)(void* self, const ukp_resolve_params_v0_t* params, uint32_t* out_resolution);
} ukp_plugin_v0_t;

/* An import as the runtime calls it (samples/custom_dispatch/cpu/plugin/
 * system_plugin.c:60-98): `params_ptr` points to the call's operands packed
 * as a C struct, nonzero return = failure. */
typedef int (*ukp_import_fn_t)(void* params_ptr, void* context, void* reserved);

#endif /* IREE_AMD_CSRC_PLUGIN_PLUGIN_ABI_H_ */
