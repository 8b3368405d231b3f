// MFMA mmt4d kernels for one element type; see mmt4d_mfma_kernel.h.
#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
int launch_bf16bf16(const Problem& p, int forced, hipStream_t stream, const char** name) {
  return launch_elem<Elem::kBF16BF16>(p, forced, stream, name);
}
}  // namespace uk_mfma
