// MFMA mmt4d kernels for one element type; see mmt4d_mfma_kernel.h.
#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
int launch_f16f16(const Problem& p, int forced, hipStream_t stream, const char** name) {
  return launch_elem<Elem::kF16F16>(p, forced, stream, name);
}
}  // namespace uk_mfma
