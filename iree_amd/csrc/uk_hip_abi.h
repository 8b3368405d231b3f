/*
 * Internal C-ABI between the plain-C host layer (uk_host.c) and the HIP
 * translation units. Everything the host layer needs from HIP goes through
 * these functions: kernel launchers and a handful of runtime wrappers. No HIP
 * type appears here, so the host layer compiles with any C compiler.
 *
 * Every function returns 0 on success or a hipError_t value.
 */
#ifndef IREE_UK_AMD_HIP_ABI_H_
#define IREE_UK_AMD_HIP_ABI_H_

#include "iree_uk_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launchers. `params` has been validated and is not an early-return case; its
 * buffer pointers are device-accessible. `stream` is a hipStream_t.
 * `kernel_mode` is an IREE_UK_AMD_KERNEL_MODE_* value. `*kernel_name` receives
 * a static string naming the variant that was launched. */
int iree_uk_amd_hip_launch_pack(const iree_uk_pack_params_t* params,
                                void* stream, int kernel_mode,
                                const char** kernel_name);
int iree_uk_amd_hip_launch_unpack(const iree_uk_unpack_params_t* params,
                                  void* stream, int kernel_mode,
                                  const char** kernel_name);
/* Where an mmt4d result goes when it is not the tiled [M][N][M0][N0] buffer
 * that the params describe: a row-major matrix of size0 x size1 elements,
 * `stride0` elements between rows, starting at out_buffer + out_offset (the
 * fused mmt4d + unpack). Elements of tiles beyond size0 x size1 are dropped. */
typedef struct iree_uk_amd_rowmajor_out_t {
  int64_t stride0;
  int64_t size0, size1;
  /* Dequantizing store (iree_uk_amd_mmt4d_dequant_unpack); `dequant` 0: none
   * and the fields below are not read. The matrix is f32; element (i, j) is
   * (float)acc * row_scale[i] * col_scale[j], a NULL scale reading as 1. With
   * ACCUMULATE the initial accumulators come from the tiled [M][N][M0][N0]
   * buffer `acc` (first element, offset applied; `acc_stride0` elements
   * between rows of tiles), not from the matrix. */
  int dequant;
  const float* row_scale;
  const float* col_scale;
  const void* acc;
  int64_t acc_stride0;
} iree_uk_amd_rowmajor_out_t;

/* `rowmajor` NULL: the result is stored tiled, as iree_uk_mmt4d does. */
int iree_uk_amd_hip_launch_mmt4d(const iree_uk_mmt4d_params_t* params,
                                 const iree_uk_amd_rowmajor_out_t* rowmajor,
                                 void* stream, int kernel_mode,
                                 const char** kernel_name);

int iree_uk_amd_hip_launch_conv_nchwc(const iree_uk_conv_nchwc_params_t* params,
                                      void* stream, int kernel_mode,
                                      const char** kernel_name);
/* 1 when the MFMA kernel serves (k0, c0, type) for every problem size. */
int iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(int32_t k0, int32_t c0,
                                               uint32_t flags);

/* 1 when an MFMA kernel serves (M0,N0,K0,type) regardless of M,N,K. */
int iree_uk_amd_hip_mmt4d_has_mfma_kernel(int32_t M0, int32_t N0, int32_t K0,
                                          uint32_t flags);

/* 1: until switched off again, mmt4d launches of this thread take their K-split
 * workspace from the library's static device array and never allocate. */
void iree_uk_amd_hip_set_no_alloc(int on);

/* Runtime wrappers. */
int iree_uk_amd_hip_device_count(void);
/* *is_device = 1 if `ptr` is device-accessible memory known to HIP (device,
 * managed, or registered/pinned host memory), 0 for ordinary host memory. */
int iree_uk_amd_hip_classify_pointer(const void* ptr, int* is_device);
/* The calling thread's staging arena on the current device: one device
 * allocation that only grows. *base is valid until the thread's next call
 * that asks for more; whoever uses it synchronizes before reserving again. */
int iree_uk_amd_hip_staging_reserve(void** base, int64_t bytes);
/* 2-D copies of `height` rows of `width` bytes; pitches in bytes.
 * Asynchronous: ordered on `stream`; the host memory must stay untouched
 * until the stream has been synchronized. */
int iree_uk_amd_hip_copy2d_to_device(void* dst, int64_t dst_pitch,
                                     const void* src, int64_t src_pitch,
                                     int64_t width, int64_t height,
                                     void* stream);
int iree_uk_amd_hip_copy2d_to_host(void* dst, int64_t dst_pitch,
                                   const void* src, int64_t src_pitch,
                                   int64_t width, int64_t height, void* stream);
int iree_uk_amd_hip_stream_synchronize(void* stream);
const char* iree_uk_amd_hip_error_string(int status);
/* Counts one device allocation of the library (see
 * iree_uk_amd_device_alloc_count). */
void iree_uk_amd_hip_note_device_alloc(void);

#ifdef __cplusplus
}
#endif

#endif /* IREE_UK_AMD_HIP_ABI_H_ */
