// MFMA mmt4d kernels for one element type and one class of tile row widths
// (see mmt4d_mfma_kernel.h, mmt4d_mfma_launch.h). This file is compiled once
// per (type, row bytes) pair, with
//   -DUK_INST_ELEM=<enumerator of uk_mfma::Elem>  -DUK_INST_RBC=<2|4|8|16>
//   -DUK_INST_NAME=<name of the function it defines>
// so that the kernel instantiations build in parallel.
#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
int UK_INST_NAME(const Problem& p, int forced, hipStream_t stream, const char** name) {
  return launch_class<Elem::UK_INST_ELEM, UK_INST_RBC>(p, forced, stream, name);
}
}  // namespace uk_mfma
