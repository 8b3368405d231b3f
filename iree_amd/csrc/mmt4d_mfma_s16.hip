// s16 x s16 -> s32 on the matrix cores: four 8-bit integer products per
// element pair in the LDS-direct pipeline (mmt4d_mfma_kernel.h, PIPE 5), one
// 128x128 workgroup shape. Served: tile rows of 2 to 128 bytes (K0 = 1 .. 64),
// tiles of at most 64 rows, K in whole steps of 64 elements; everything else
// stays with the vector dot-product kernel (mmt4d_dot2.hip), as do problems too
// thin to fill 128x128 blocks.
#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
namespace {
template <int RBC>
int launch_s16_rows(const Problem& p, hipStream_t stream) {
  return launch_variant<Elem::kS16, RBC, 4, 2, 2, 4, 1, 5>(p, 0, p.K1, p.accumulate, stream);
}
}  // namespace

int launch_s16(const Problem& p, int forced, hipStream_t stream, const char** name) {
  const int64_t rows_m = std::min<int64_t>((int64_t)p.M1 * p.M0, p.out_rows);
  const int64_t cols_n = std::min<int64_t>((int64_t)p.N1 * p.N0, p.out_cols);
  if (forced == 0 && (rows_m <= 32 || cols_n <= 32)) return -1;
  int st;
  switch (p.rb) {
    case 2: st = launch_s16_rows<2>(p, stream); break;
    case 4: st = launch_s16_rows<4>(p, stream); break;
    case 8: st = launch_s16_rows<8>(p, stream); break;
    default: st = launch_s16_rows<16>(p, stream); break;
  }
  if (st >= 0) *name = "mmt4d_mfma_128x128_s16";
  return st;
}
}  // namespace uk_mfma
