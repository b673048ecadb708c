/* HAL executable plugin that resolves the ukernel imports of compiled
 * dispatches (iree_uk_mmt4d, iree_uk_pack, iree_uk_unpack,
 * iree_uk_query_tile_sizes_2d) to this library's MI355X implementation.
 *
 * The reference runtime loads such a plugin with
 *   --executable_plugin=libiree_uk_mi355x_plugin.so
 * (runtime/src/iree/hal/local/plugins/system_library_plugin.c), calls the one
 * exported function below, then `load` and `resolve`. A module compiled with
 * ukernels enabled and their bitcode not linked in
 * (--iree-llvmcpu-link-ukernel-bitcode=false) leaves the calls as imports whose
 * operands arrive packed in the order of the lowered call: per buffer (base
 * pointer, offset, strides of the outer dimensions), then the scalar operands,
 * then the `processor_data` field
 * (compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:93-114,
 * 240-260, 368-383, 455-471; memref expansion
 * compiler/src/iree/compiler/Codegen/Dialect/Codegen/IR/UKernelOps.cpp:113-145).
 *
 * The plugin is not "standalone" in the header's sense: it needs the HIP
 * runtime. */
#include <string.h>

#include "iree_uk_mi355x.h"
#include "plugin_abi.h"

#define UKP_PUBLIC __attribute__((visibility("default")))

typedef struct {
  const void* lhs; size_t lhs_offset; size_t lhs_stride0;
  const void* rhs; size_t rhs_offset; size_t rhs_stride0;
  void* out; size_t out_offset; size_t out_stride0;
  size_t M, N, K;
  int32_t M0, N0, K0;
  uint32_t flags;
  const uint64_t* processor_data;
} mmt4d_operands_t;

static int mmt4d_import(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  const mmt4d_operands_t* a = (const mmt4d_operands_t*)params_ptr;
  iree_uk_mmt4d(a->lhs, (iree_uk_index_t)a->lhs_offset, (iree_uk_index_t)a->lhs_stride0, a->rhs,
                (iree_uk_index_t)a->rhs_offset, (iree_uk_index_t)a->rhs_stride0, a->out,
                (iree_uk_index_t)a->out_offset, (iree_uk_index_t)a->out_stride0, (iree_uk_index_t)a->M,
                (iree_uk_index_t)a->N, (iree_uk_index_t)a->K, a->M0, a->N0, a->K0, a->flags,
                a->processor_data);
  return 0;
}

typedef struct {
  const void* in; size_t in_offset; size_t in_stride0; size_t in_stride1;
  void* out; size_t out_offset; size_t out_stride0; size_t out_stride1;
  size_t in_size0, in_size1;
  size_t out_size0, out_size1, out_size2, out_size3;
  uint64_t padding_value;
  uint32_t flags;
  const uint64_t* processor_data;
} pack_operands_t;

static int pack_import(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  const pack_operands_t* a = (const pack_operands_t*)params_ptr;
  iree_uk_pack(a->in, (iree_uk_index_t)a->in_offset, (iree_uk_index_t)a->in_stride0,
               (iree_uk_index_t)a->in_stride1, a->out, (iree_uk_index_t)a->out_offset,
               (iree_uk_index_t)a->out_stride0, (iree_uk_index_t)a->out_stride1,
               (iree_uk_index_t)a->in_size0, (iree_uk_index_t)a->in_size1, (iree_uk_index_t)a->out_size0,
               (iree_uk_index_t)a->out_size1, (iree_uk_index_t)a->out_size2, (iree_uk_index_t)a->out_size3,
               a->padding_value, a->flags, a->processor_data);
  return 0;
}

typedef struct {
  const void* in; size_t in_offset; size_t in_stride0; size_t in_stride1;
  void* out; size_t out_offset; size_t out_stride0; size_t out_stride1;
  size_t in_size0, in_size1, in_size2, in_size3;
  size_t out_size0, out_size1;
  uint32_t flags;
  const uint64_t* processor_data;
} unpack_operands_t;

static int unpack_import(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  const unpack_operands_t* a = (const unpack_operands_t*)params_ptr;
  iree_uk_unpack(a->in, (iree_uk_index_t)a->in_offset, (iree_uk_index_t)a->in_stride0,
                 (iree_uk_index_t)a->in_stride1, a->out, (iree_uk_index_t)a->out_offset,
                 (iree_uk_index_t)a->out_stride0, (iree_uk_index_t)a->out_stride1,
                 (iree_uk_index_t)a->in_size0, (iree_uk_index_t)a->in_size1, (iree_uk_index_t)a->in_size2,
                 (iree_uk_index_t)a->in_size3, (iree_uk_index_t)a->out_size0, (iree_uk_index_t)a->out_size1,
                 a->flags, a->processor_data);
  return 0;
}

/* Results come first in the packed struct (system_plugin.c:57-58). */
typedef struct {
  size_t tile_size0, tile_size1;
  size_t size0, size1;
  uint32_t flags;
  const uint64_t* processor_data;
} query_tile_sizes_operands_t;

static int query_tile_sizes_2d_import(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  query_tile_sizes_operands_t* a = (query_tile_sizes_operands_t*)params_ptr;
  iree_uk_query_tile_sizes_2d_params_t p;
  iree_uk_query_tile_sizes_2d_out_params_t out;
  memset(&p, 0, sizeof p);
  p.flags = a->flags;
  p.size0 = (iree_uk_index_t)a->size0;
  p.size1 = (iree_uk_index_t)a->size1;
  p.cpu_data = a->processor_data;
  iree_uk_query_tile_sizes_2d(&p, &out);
  a->tile_size0 = (size_t)out.tile_size0;
  a->tile_size1 = (size_t)out.tile_size1;
  return 0;
}

static const struct {
  const char* name;
  ukp_import_fn_t fn;
} kImports[] = {
    {"iree_uk_mmt4d", mmt4d_import},
    {"iree_uk_pack", pack_import},
    /* the name the compiler gives the call (CPULowerToUKernels.cpp:525, 93-114) and the C symbol's */
    {"iree_uk_query_tile_sizes.2d", query_tile_sizes_2d_import},
    {"iree_uk_query_tile_sizes_2d", query_tile_sizes_2d_import},
    {"iree_uk_unpack", unpack_import},
};

static ukp_status_t plugin_load(const ukp_environment_v0_t* environment, size_t param_count,
                                const ukp_string_pair_t* params, void** out_self) {
  (void)environment; (void)param_count; (void)params;
  *out_self = NULL; /* no per-instance state */
  /* Fail the load, not the first dispatch, when there is no usable GPU. */
  return iree_uk_mi355x_init(-1) == 0 ? UKP_STATUS_OK : UKP_STATUS_UNAVAILABLE;
}

static void plugin_unload(void* self) { (void)self; }

static ukp_status_t plugin_resolve(void* self, const ukp_resolve_params_v0_t* params, uint32_t* out_resolution) {
  (void)self;
  *out_resolution = 0;
  int required_missing = 0;
  for (size_t i = 0; i < params->count; ++i) {
    if (params->out_fn_ptrs[i]) continue; /* resolved by another provider */
    const char* name = params->symbol_names[i];
    const int optional = name && name[0] == '?';
    if (optional) ++name;
    ukp_import_fn_t fn = NULL;
    for (size_t k = 0; name && k < sizeof kImports / sizeof kImports[0]; ++k) {
      if (strcmp(name, kImports[k].name) == 0) fn = kImports[k].fn;
    }
    if (fn) {
      params->out_fn_ptrs[i] = (void*)fn;
      params->out_fn_contexts[i] = NULL;
    } else if (optional) {
      *out_resolution |= UKP_RESOLUTION_MISSING_OPTIONAL;
    } else {
      required_missing = 1;
    }
  }
  return required_missing ? UKP_STATUS_NOT_FOUND : UKP_STATUS_OK;
}

UKP_PUBLIC const ukp_header_t** iree_hal_executable_plugin_query(uint32_t max_version, void* reserved) {
  (void)reserved;
  static const ukp_header_t header = {
      UKP_VERSION_0_1,
      "iree_uk_mi355x",
      "mmt4d / pack / unpack ukernels on one MI355X (gfx950) through HIP",
      UKP_FEATURE_NONE,
      UKP_SANITIZER_NONE,
      {0},
  };
  static const ukp_plugin_v0_t plugin = {&header, plugin_load, plugin_unload, plugin_resolve};
  return max_version <= UKP_VERSION_0_1 - 1 ? NULL : (const ukp_header_t**)&plugin;
}
