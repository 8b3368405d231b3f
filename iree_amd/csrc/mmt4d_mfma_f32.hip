// MFMA mmt4d kernels for one element type; see mmt4d_mfma_kernel.h.
#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
int launch_f32(const Problem& p, int forced, hipStream_t stream, const char** name) {
  return launch_elem<Elem::kF32>(p, forced, stream, name);
}
}  // namespace uk_mfma
