// HAL executable plugin face of the library: lets an unmodified IREE runtime
// route the `iree_uk_mmt4d`, `iree_uk_pack`, `iree_uk_unpack` (and
// `iree_uk_conv_nchwc`) imports of
// compiled LLVMCPU programs to the GPU implementation
// (`--executable_plugin=libiree_uk_amd.so`).
//
// The plugin interface is a binary contract
// (runtime/src/iree/hal/local/executable_plugin.h in the reference): the
// declarations below restate the part of it this file needs, field for field,
// each with the line it mirrors. Nothing here depends on the IREE runtime.
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "iree_uk_amd.h"

// ---- the plugin ABI, version 0.1 -------------------------------------------

// executable_plugin.h:136-142
#define UK_PLUGIN_VERSION_0_1 0x00000001u

// executable_plugin.h:152-173 (iree_hal_executable_plugin_header_t)
typedef struct uk_plugin_header_t {
  uint32_t version;
  const char* name;
  const char* description;
  uint32_t features;   // executable_plugin.h:58-74: 0 = needs system facilities
  int32_t sanitizer;   // executable_plugin.h:80-100: 0 = none
  uint64_t reserved[8];
} uk_plugin_header_t;

// executable_plugin.h:211-233: status = a pointer-sized value whose low five
// bits are the code; 0 = OK, 5 = NOT_FOUND.
typedef struct uk_plugin_status_handle_t* uk_plugin_status_t;
#define UK_PLUGIN_STATUS(code) ((uk_plugin_status_t)(uintptr_t)((code) & 0x1Fu))
enum { UK_PLUGIN_OK = 0, UK_PLUGIN_NOT_FOUND = 5 };

// executable_plugin.h:294-297 (allocator), :335-348 (string pair), :381-387
// (environment): only passed through, never dereferenced here.
typedef struct uk_plugin_allocator_t {
  void* self;
  void* ctl;
} uk_plugin_allocator_t;
typedef struct uk_plugin_string_view_t {
  const char* data;
  size_t size;
} uk_plugin_string_view_t;
typedef struct uk_plugin_string_pair_t {
  uk_plugin_string_view_t key;
  uk_plugin_string_view_t value;
} uk_plugin_string_pair_t;
typedef struct uk_plugin_environment_v0_t {
  uk_plugin_allocator_t host_allocator;
} uk_plugin_environment_v0_t;

// executable_plugin.h:389-394
typedef struct uk_plugin_resolve_params_v0_t {
  size_t count;
  const char* const* symbol_names;
  void** out_fn_ptrs;
  void** out_fn_contexts;
} uk_plugin_resolve_params_v0_t;

// executable_plugin.h:350-356: bit 0 = one or more optional symbols missing.
#define UK_PLUGIN_RESOLUTION_MISSING_OPTIONAL 1u

// executable_plugin.h:404-461 (iree_hal_executable_plugin_v0_t)
typedef struct uk_plugin_v0_t {
  const uk_plugin_header_t* header;
  uk_plugin_status_t (*load)(const uk_plugin_environment_v0_t* environment,
                             size_t param_count,
                             const uk_plugin_string_pair_t* params,
                             void** out_self);
  void (*unload)(void* self);
  uk_plugin_status_t (*resolve)(void* self,
                                const uk_plugin_resolve_params_v0_t* params,
                                uint32_t* out_resolution);
} uk_plugin_v0_t;

// ---- import thunks -----------------------------------------------------------
//
// An import is called as `int fn(void* params_ptr, void* context, void*
// reserved)` (runtime/src/iree/hal/local/executable_library.h:150-158);
// `params_ptr` is a struct of results, then arguments, then extra fields in
// native alignment (compiler/src/iree/compiler/Codegen/LLVMCPU/DispatchABI.cpp:
// 1170-1186). For the ukernel calls the LLVMCPU lowering adds one dummy i32
// result (compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:
// 152-163), the arguments are the params struct field for field (memrefs
// become base pointer, offset and strides) and the one extra field is the
// processor-data pointer (`hal.import.fields = ["processor_data"]`, :113-116),
// which is the struct's `cpu_data`. Non-zero return = fatal.

typedef struct { int32_t unused_result; iree_uk_mmt4d_params_t p; } mmt4d_import_t;
typedef struct { int32_t unused_result; iree_uk_pack_params_t p; } pack_import_t;
typedef struct { int32_t unused_result; iree_uk_unpack_params_t p; } unpack_import_t;

static int mmt4d_thunk(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  iree_uk_mmt4d_p(&((const mmt4d_import_t*)params_ptr)->p);
  return iree_uk_amd_last_status() ? 1 : 0;
}
static int pack_thunk(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  iree_uk_pack_p(&((const pack_import_t*)params_ptr)->p);
  return iree_uk_amd_last_status() ? 1 : 0;
}
/* conv_nchwc: the arguments of the flat entry point in order (the params
 * struct has one more, internal, field, so it cannot be overlaid). */
typedef struct {
  int32_t unused_result;
  const void* input_buffer;
  iree_uk_index_t input_offset, input_stride_n, input_stride_ic_outer, input_stride_h;
  const void* filter_buffer;
  iree_uk_index_t filter_offset, filter_stride_oc_outer, filter_stride_ic_outer, filter_stride_fh;
  void* output_buffer;
  iree_uk_index_t output_offset, output_stride_n, output_stride_oc_outer, output_stride_oh;
  iree_uk_index_t N, OC_outer, OH, OW, IC_outer, FH, FW;
  int32_t k0, c0, stride_h, stride_w;
  uint32_t flags;
  const uint64_t* cpu_data;
} conv_import_t;

static int conv_thunk(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  const conv_import_t* a = (const conv_import_t*)params_ptr;
  iree_uk_conv_nchwc(a->input_buffer, a->input_offset, a->input_stride_n,
                     a->input_stride_ic_outer, a->input_stride_h, a->filter_buffer,
                     a->filter_offset, a->filter_stride_oc_outer, a->filter_stride_ic_outer,
                     a->filter_stride_fh, a->output_buffer, a->output_offset, a->output_stride_n,
                     a->output_stride_oc_outer, a->output_stride_oh, a->N, a->OC_outer, a->OH,
                     a->OW, a->IC_outer, a->FH, a->FW, a->k0, a->c0, a->stride_h, a->stride_w,
                     a->flags, a->cpu_data);
  return iree_uk_amd_last_status() ? 1 : 0;
}

static int unpack_thunk(void* params_ptr, void* context, void* reserved) {
  (void)context; (void)reserved;
  iree_uk_unpack_p(&((const unpack_import_t*)params_ptr)->p);
  return iree_uk_amd_last_status() ? 1 : 0;
}

// ---- plugin entry points ------------------------------------------------------

static uk_plugin_status_t plugin_load(const uk_plugin_environment_v0_t* environment,
                                      size_t param_count,
                                      const uk_plugin_string_pair_t* params,
                                      void** out_self) {
  (void)environment; (void)param_count; (void)params;
  // No per-instance state: everything the entry points keep is thread-local.
  *out_self = NULL;
  return UK_PLUGIN_STATUS(UK_PLUGIN_OK);
}

static void plugin_unload(void* self) { (void)self; }

// Resolution contract (executable_plugin.h:425-458): entries already resolved
// are left alone; a leading '?' marks an optional symbol, whose absence only
// sets the MISSING_OPTIONAL bit; a missing required symbol gives NOT_FOUND
// after everything available has been filled in.
static uk_plugin_status_t plugin_resolve(void* self,
                                         const uk_plugin_resolve_params_v0_t* params,
                                         uint32_t* out_resolution) {
  (void)self;
  static const struct { const char* name; void* fn; } table[] = {
      {"iree_uk_conv_nchwc", (void*)conv_thunk},
      {"iree_uk_mmt4d", (void*)mmt4d_thunk},
      {"iree_uk_pack", (void*)pack_thunk},
      {"iree_uk_unpack", (void*)unpack_thunk},
  };
  *out_resolution = 0;
  int missing_required = 0;
  for (size_t i = 0; i < params->count; ++i) {
    if (params->out_fn_ptrs[i]) continue;
    const char* name = params->symbol_names[i];
    if (!name) { missing_required = 1; continue; }
    const int optional = name[0] == '?';
    if (optional) ++name;
    void* fn = NULL;
    for (size_t j = 0; j < sizeof table / sizeof table[0]; ++j) {
      if (strcmp(name, table[j].name) == 0) fn = table[j].fn;
    }
    if (fn) {
      params->out_fn_ptrs[i] = fn;
      params->out_fn_contexts[i] = NULL;
    } else if (optional) {
      *out_resolution |= UK_PLUGIN_RESOLUTION_MISSING_OPTIONAL;
    } else {
      missing_required = 1;
    }
  }
  return UK_PLUGIN_STATUS(missing_required ? UK_PLUGIN_NOT_FOUND : UK_PLUGIN_OK);
}

// executable_plugin.h:175-191: returns NULL when the caller cannot take this
// version.
const void* iree_hal_executable_plugin_query(uint32_t max_version, void* reserved) {
  (void)reserved;
  static const uk_plugin_header_t header = {
      .version = UK_PLUGIN_VERSION_0_1,
      .name = "iree_uk_amd",
      .description = "iree_uk_mmt4d / iree_uk_pack / iree_uk_unpack on MI355X (gfx950)",
      .features = 0,
      .sanitizer = 0,
  };
  static const uk_plugin_v0_t plugin = {
      .header = &header,
      .load = plugin_load,
      .unload = plugin_unload,
      .resolve = plugin_resolve,
  };
  // The result is a `const iree_hal_executable_plugin_header_t**`: the address
  // of the interface struct, whose first field is the header pointer.
  return max_version >= UK_PLUGIN_VERSION_0_1 ? (const void*)&plugin : NULL;
}
