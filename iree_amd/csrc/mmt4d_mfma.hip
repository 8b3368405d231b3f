// placeholder, replaced below
#include <hip/hip_runtime.h>
#include "uk_hip_abi.h"
extern "C" int iree_uk_amd_hip_mmt4d_mfma_supported(int32_t, int32_t, int32_t, uint32_t) { return 0; }
extern "C" int iree_uk_amd_hip_launch_mmt4d_mfma(const iree_uk_mmt4d_params_t*, void*, const char**) { return -1; }
