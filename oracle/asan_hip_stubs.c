/*
 * CPU stand-ins for the internal HIP C-ABI of the product's host layer
 * (iree_amd/csrc/uk_hip_abi.h), for the sanitizer build of `make asan` only.
 * "Device memory" is calloc'ed host memory, copies are row-wise memcpy, and a
 * "kernel launch" runs the CPU oracle on the parameters the host layer
 * prepared. With these, uk_host.c's validation, early returns, staging of
 * host operands (dense device copies, pitches, copy-back of only the rows an
 * op may touch) and uk_plugin.c's thunks run end to end under
 * AddressSanitizer + UBSan without a GPU. TEST INFRASTRUCTURE, NOT PRODUCT
 * CODE: nothing here is linked into libiree_uk_amd.so.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "uk_hip_abi.h"

int uk_oracle_mmt4d(const void*, int64_t, int64_t, const void*, int64_t, int64_t, void*, int64_t,
                    int64_t, int64_t, int64_t, int64_t, int32_t, int32_t, int32_t, uint32_t,
                    const uint64_t*);
int uk_oracle_pack(const void*, int64_t, int64_t, int64_t, void*, int64_t, int64_t, int64_t, int64_t,
                   int64_t, int64_t, int64_t, int64_t, int64_t, uint64_t, uint32_t, const uint64_t*);
int uk_oracle_unpack(const void*, int64_t, int64_t, int64_t, void*, int64_t, int64_t, int64_t,
                     int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, uint32_t,
                     const uint64_t*);
int uk_oracle_conv_nchwc(const void*, int64_t, int64_t, int64_t, int64_t, const void*, int64_t,
                         int64_t, int64_t, int64_t, void*, int64_t, int64_t, int64_t, int64_t,
                         int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int32_t,
                         int32_t, int32_t, int32_t, uint32_t, const uint64_t*);

enum { kNotSupported = 801 }; /* hipErrorNotSupported */

int iree_uk_amd_hip_launch_pack(const iree_uk_pack_params_t* p, void* stream, int kernel_mode,
                                const char** kernel_name) {
  (void)stream; (void)kernel_mode;
  *kernel_name = "oracle_pack";
  return uk_oracle_pack(p->in_buffer, p->in_offset, p->in_stride0, p->in_stride1, p->out_buffer,
                        p->out_offset, p->out_stride0, p->out_stride1, p->in_size0, p->in_size1,
                        p->out_size0, p->out_size1, p->out_size2, p->out_size3, p->padding_value,
                        p->flags, 0) ? kNotSupported : 0;
}

int iree_uk_amd_hip_launch_unpack(const iree_uk_unpack_params_t* p, void* stream, int kernel_mode,
                                  const char** kernel_name) {
  (void)stream; (void)kernel_mode;
  *kernel_name = "oracle_unpack";
  return uk_oracle_unpack(p->in_buffer, p->in_offset, p->in_stride0, p->in_stride1, p->out_buffer,
                          p->out_offset, p->out_stride0, p->out_stride1, p->in_size0, p->in_size1,
                          p->in_size2, p->in_size3, p->out_size0, p->out_size1, p->flags, 0)
             ? kNotSupported : 0;
}

int iree_uk_amd_hip_launch_mmt4d(const iree_uk_mmt4d_params_t* p,
                                 const iree_uk_amd_rowmajor_out_t* rowmajor, void* stream,
                                 int kernel_mode, const char** kernel_name) {
  (void)stream; (void)kernel_mode;
  *kernel_name = "oracle_mmt4d";
  if (rowmajor) return kNotSupported; /* the fused forms need a device */
  return uk_oracle_mmt4d(p->lhs_buffer, p->lhs_offset, p->lhs_stride0, p->rhs_buffer,
                         p->rhs_offset, p->rhs_stride0, p->out_buffer, p->out_offset,
                         p->out_stride0, p->M, p->N, p->K, p->M0, p->N0, p->K0, p->flags, 0)
             ? kNotSupported : 0;
}

int iree_uk_amd_hip_launch_conv_nchwc(const iree_uk_conv_nchwc_params_t* p, void* stream,
                                      int kernel_mode, const char** kernel_name) {
  (void)stream; (void)kernel_mode;
  *kernel_name = "oracle_conv_nchwc";
  return uk_oracle_conv_nchwc(p->input_buffer, p->input_offset, p->input_stride_n,
                              p->input_stride_ic_outer, p->input_stride_h, p->filter_buffer,
                              p->filter_offset, p->filter_stride_oc_outer,
                              p->filter_stride_ic_outer, p->filter_stride_fh, p->output_buffer,
                              p->output_offset, p->output_stride_n, p->output_stride_oc_outer,
                              p->output_stride_oh, p->N, p->OC_outer, p->OH, p->OW, p->IC_outer,
                              p->FH, p->FW, p->k0, p->c0, p->stride_h, p->stride_w, p->flags, 0)
             ? kNotSupported : 0;
}

/* No matrix cores here: every call needs the generic-fallback flag, which lets
 * the tests reach the "no tile function and fallback not enabled" report. */
int iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(int32_t k0, int32_t c0, uint32_t flags) {
  (void)k0; (void)c0; (void)flags;
  return 0;
}
int iree_uk_amd_hip_mmt4d_has_mfma_kernel(int32_t M0, int32_t N0, int32_t K0, uint32_t flags) {
  (void)M0; (void)N0; (void)K0; (void)flags;
  return 0;
}

void iree_uk_amd_hip_set_no_alloc(int on) { (void)on; }

int iree_uk_amd_hip_device_count(void) { return 1; }

int iree_uk_amd_hip_classify_pointer(const void* ptr, int* is_device) {
  (void)ptr;
  *is_device = 0; /* everything is a host operand and gets staged */
  return 0;
}

/* A fresh block of exactly the size asked for on every call, so that the
 * sanitizer sees an overrun of the arena as a whole. */
static void* g_arena;
int iree_uk_amd_hip_staging_reserve(void** base, int64_t bytes) {
  free(g_arena);
  g_arena = calloc(1, bytes > 0 ? (size_t)bytes : 1);
  *base = g_arena;
  return g_arena ? 0 : 2; /* hipErrorOutOfMemory */
}
void asan_stubs_release(void) {
  free(g_arena);
  g_arena = 0;
}

static int copy2d(void* dst, int64_t dst_pitch, const void* src, int64_t src_pitch, int64_t width,
                  int64_t height) {
  for (int64_t r = 0; r < height; ++r)
    memcpy((char*)dst + r * dst_pitch, (const char*)src + r * src_pitch, (size_t)width);
  return 0;
}
int iree_uk_amd_hip_copy2d_to_device(void* dst, int64_t dst_pitch, const void* src,
                                     int64_t src_pitch, int64_t width, int64_t height,
                                     void* stream) {
  (void)stream;
  return copy2d(dst, dst_pitch, src, src_pitch, width, height);
}
int iree_uk_amd_hip_copy2d_to_host(void* dst, int64_t dst_pitch, const void* src,
                                   int64_t src_pitch, int64_t width, int64_t height, void* stream) {
  (void)stream;
  return copy2d(dst, dst_pitch, src, src_pitch, width, height);
}
int iree_uk_amd_hip_stream_synchronize(void* stream) {
  (void)stream;
  return 0;
}
const char* iree_uk_amd_hip_error_string(int status) {
  return status == kNotSupported ? "not supported by the CPU stand-in" : "error (CPU stand-in)";
}
