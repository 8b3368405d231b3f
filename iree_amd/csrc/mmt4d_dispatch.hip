// mmt4d kernel selection: MFMA kernels where one covers (type, M0, N0, K0),
// otherwise the any-shape scalar kernel.
#include <hip/hip_runtime.h>

#include "uk_hip_abi.h"

extern "C" int iree_uk_amd_hip_launch_mmt4d_generic(
    const iree_uk_mmt4d_params_t* p, const iree_uk_amd_rowmajor_out_t* rowmajor,
    void* stream);
extern "C" int iree_uk_amd_hip_launch_mmt4d_mfma(
    const iree_uk_mmt4d_params_t* p, const iree_uk_amd_rowmajor_out_t* rowmajor,
    void* stream, int forced_variant, const char** kernel_name);
extern "C" int iree_uk_amd_hip_mmt4d_mfma_supported(int32_t M0, int32_t N0,
                                                    int32_t K0, uint32_t flags);
extern "C" int iree_uk_amd_hip_launch_mmt4d_s16_widened(
    const iree_uk_mmt4d_params_t* p, const iree_uk_amd_rowmajor_out_t* rowmajor,
    void* stream, const char** kernel_name);
extern "C" int iree_uk_amd_hip_launch_mmt4d_retiled(
    const iree_uk_mmt4d_params_t* p, const iree_uk_amd_rowmajor_out_t* rowmajor,
    void* stream, const char** kernel_name);
extern "C" int iree_uk_amd_hip_launch_mmt4d_dot2(
    const iree_uk_mmt4d_params_t* p, const iree_uk_amd_rowmajor_out_t* rowmajor,
    void* stream);

namespace uk_mfma {
void note_k_slices(int n);  // mmt4d_mfma.hip: records the slice count of the call
}

namespace {
// Calls on this thread that iree_uk_mmt4d_info advertises a matrix-core kernel
// for but that the scalar kernel served (see iree_uk_amd_mfma_decline_count).
thread_local uint64_t g_declined = 0;
}  // namespace

extern "C" IREE_UK_AMD_EXPORT uint64_t iree_uk_amd_mfma_decline_count(void) { return g_declined; }

extern "C" int iree_uk_amd_hip_mmt4d_has_mfma_kernel(int32_t M0, int32_t N0,
                                                     int32_t K0,
                                                     uint32_t flags) {
  return iree_uk_amd_hip_mmt4d_mfma_supported(M0, N0, K0, flags);
}

extern "C" int iree_uk_amd_hip_launch_mmt4d(const iree_uk_mmt4d_params_t* p,
                                            const iree_uk_amd_rowmajor_out_t* rowmajor,
                                            void* stream, int kernel_mode,
                                            const char** kernel_name) {
  // Every call starts from "one K slice": only the thin matrix-core kernel
  // ever reports more (iree_uk_amd_last_k_slices).
  uk_mfma::note_k_slices(1);
  // s8 x s4 -> s32 and s16 x s16 -> s32 have an MFMA kernel for some shapes
  // only; the launcher says "not served" (negative) for the rest.
  const uint32_t type = p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK;
  const bool maybe = type == IREE_UK_FLAG_MMT4D_TYPE_S8S4S32 || type == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32;
  if (kernel_mode != IREE_UK_AMD_KERNEL_MODE_GENERIC &&
      (maybe || iree_uk_amd_hip_mmt4d_mfma_supported(p->M0, p->N0, p->K0, p->flags))) {
    const int forced = kernel_mode >= IREE_UK_AMD_KERNEL_MODE_MFMA_VARIANT
                           ? kernel_mode - IREE_UK_AMD_KERNEL_MODE_MFMA_VARIANT
                           : 0;
    int st = iree_uk_amd_hip_launch_mmt4d_mfma(p, rowmajor, stream, forced, kernel_name);
    // A negative status means "not served after all" (a negative stride, an
    // operand spanning 2 GiB or more, a zero-fill): the scalar kernel, which
    // indexes with 64 bits, computes the same result. When the tile shape is
    // one the info query advertises, count the call so that the cliff shows.
    if (st >= 0) return st;
    if (!maybe && kernel_mode == IREE_UK_AMD_KERNEL_MODE_AUTO && p->K != 0) ++g_declined;
  }
  if (kernel_mode == IREE_UK_AMD_KERNEL_MODE_AUTO) {
    // Tile rows under 16 bytes in shapes the matrix-core kernels decline:
    // regrouped along K first (mmt4d_mfma.hip).
    const int st = iree_uk_amd_hip_launch_mmt4d_retiled(p, rowmajor, stream, kernel_name);
    if (st >= 0) return st;
  }
  if (kernel_mode == IREE_UK_AMD_KERNEL_MODE_AUTO) {
    // s16 x s8 and s16 x u4 with enough rows and columns: the matrix-core s16
    // kernel on a right-hand side widened to s16 (mmt4d_mfma_s16.hip).
    const int st = iree_uk_amd_hip_launch_mmt4d_s16_widened(p, rowmajor, stream, kernel_name);
    if (st >= 0) return st;
  }
  if (kernel_mode != IREE_UK_AMD_KERNEL_MODE_GENERIC) {
    // The 16-bit integer LHS types: vector dot products from LDS where the
    // tile shape allows (not a matrix-core kernel, so the info query does not
    // advertise it and callers pass the fallback flag as for the CPU library's
    // generic tiles).
    const int st = iree_uk_amd_hip_launch_mmt4d_dot2(p, rowmajor, stream);
    if (st >= 0) {
      *kernel_name = "mmt4d_dot2";
      return st;
    }
  }
  *kernel_name = "mmt4d_generic";
  return iree_uk_amd_hip_launch_mmt4d_generic(p, rowmajor, stream);
}
