// s8 x s4 -> s32 on the matrix cores: the barrier-free thin kernel only (any M;
// more than 64 rows run as several row blocks that each stream the RHS).
#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
int launch_s8s4(const Problem& p, hipStream_t stream, const char** name) {
  const int64_t rows_m = std::min<int64_t>((int64_t)p.M1 * p.M0, p.out_rows);  // rows that are stored
  int st;
  if (rows_m <= 16) {
    st = launch_thin<Elem::kS8S4, 16, 1, 2, 4, 4>(p, false, stream, true);
  } else if (rows_m <= 32) {
    st = launch_thin<Elem::kS8S4, 16, 2, 2, 4, 4>(p, false, stream, true);
  } else {
    st = launch_thin<Elem::kS8S4, 16, 4, 2, 4, 3>(p, false, stream, true);
  }
  if (st >= 0) *name = "mmt4d_mfma_thin_s8s4";
  return st;
}
}  // namespace uk_mfma
