// s8 x s4 -> s32 on the matrix cores. Few rows (a decode step): the
// barrier-free thin kernel, which unpacks the nibbles in registers (any M; more
// than 64 rows run as several row blocks that each stream the RHS). Many rows
// (a prefill against 4-bit weights): the weights are expanded to s8 once, into
// a buffer the library keeps, and the s8 kernels run on that.
#include "mmt4d_mfma_launch.h"
#include "uk_hip_abi.h"

namespace uk_mfma {

int launch_s8(const Problem& p, int forced, hipStream_t stream, const char** name);
}  // namespace uk_mfma

extern "C" int iree_uk_amd_hip_mmt4d_mfma_supported(int32_t M0, int32_t N0, int32_t K0, uint32_t flags);

namespace uk_mfma {

namespace {

typedef uint32_t v2u_g __attribute__((ext_vector_type(2), aligned(1)));
typedef uint32_t v4u_e __attribute__((ext_vector_type(4)));

// Eight nibbles of a word, low nibble first (element 2i of a tile row is the
// low nibble of byte i: mmt4d_tile_generic.c:31-47 of the reference), sign-extended to
// eight bytes.
__device__ __forceinline__ void expand_word(uint32_t w, uint32_t* lo, uint32_t* hi) {
  uint32_t b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) b[i] = (uint32_t)__builtin_amdgcn_sbfe((int)w, 4 * i, 4) & 0xFFu;
  *lo = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
  *hi = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
}

// Panel n of the RHS: `panel_in_bytes` bytes at src + n * src_stride become
// twice as many at dst + n * 2 * panel_in_bytes. A thread takes 8 bytes.
__global__ __launch_bounds__(256) void expand_s4_kernel(const char* src, int64_t src_stride, char* dst,
                                                         uint32_t panel_in_bytes) {
  const char* s = src + (int64_t)blockIdx.y * src_stride;
  char* d = dst + (int64_t)blockIdx.y * 2 * panel_in_bytes;
  for (uint32_t off = (blockIdx.x * 256 + threadIdx.x) * 8; off < panel_in_bytes; off += gridDim.x * 256 * 8) {
    const v2u_g in = *reinterpret_cast<const v2u_g*>(s + off);
    v4u_e out;
    uint32_t lo, hi;
    expand_word(in[0], &lo, &hi);
    out[0] = lo; out[1] = hi;
    expand_word(in[1], &lo, &hi);
    out[2] = lo; out[3] = hi;
    *reinterpret_cast<v4u_e*>(d + 2 * (int64_t)off) = out;
  }
}

// Rows from which the expansion pays: it costs a pass over the weights (1.5
// bytes moved per weight; 14336 x 4096: 20 us), the thin kernel costs a pass
// over them per 64 rows (s8 x s4, 14336 x 4096: 36.8 us at 256 rows, 143 at
// 1024, against 21 and 58 us for s8 x s8).
constexpr int64_t kExpandFromRows = 512;

}  // namespace

int launch_s8s4(const Problem& p, hipStream_t stream, const char** name) {
  const int64_t rows_m = std::min<int64_t>((int64_t)p.M1 * p.M0, p.out_rows);  // rows that are stored
  const int64_t panel_in_bytes = ((int64_t)p.K1 * p.N0 * p.rb) / 2;
  if (rows_m >= kExpandFromRows && p.N1 > 0 && p.N1 < 65536 && panel_in_bytes % 8 == 0 &&
      panel_in_bytes < (1ll << 31) &&
      iree_uk_amd_hip_mmt4d_mfma_supported(p.M0, p.N0, p.rb, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32)) {
    char* expanded = nullptr;
    if (acquire_expand_workspace((size_t)(2 * panel_in_bytes * p.N1), stream, &expanded) == 0) {
      const uint32_t per_panel = (uint32_t)std::min<int64_t>(uk::ceil_div(panel_in_bytes, (int64_t)(256 * 8)), 64);
      uk::launch(2, expand_s4_kernel, dim3(per_panel, (uint32_t)p.N1), dim3(256), 0, stream, p.rhs,
                 p.rhs_stride, expanded, (uint32_t)panel_in_bytes);
      Problem q = p;
      q.rhs = expanded;
      q.rhs_stride = 2 * panel_in_bytes;
      const char* s8_name = nullptr;
      const int st = launch_s8(q, 0, stream, &s8_name);
      if (st >= 0) {
        *name = "mmt4d_mfma_s8s4_expanded";
        return st;
      }
      // (not served as s8: the thin kernel below reads the packed weights)
    }
  }
  // Tile rows under 16 elements in a tile the s8 kernels do not take (arm64's
  // Mx16x2 with M = 1, 2, 4: arch/arm_64/mmt4d_arm_64_base.c:296): both operands
  // are regrouped along K into 16-byte rows, the weights widened on the way.
  if (rows_m >= kExpandFromRows && p.rb < 16 && p.rb >= 2 && p.M1 > 0 && p.M1 < 65536 && p.N1 > 0 &&
      p.N1 < 65536 && !iree_uk_amd_hip_mmt4d_mfma_supported(p.M0, p.N0, p.rb, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32) &&
      iree_uk_amd_hip_mmt4d_mfma_supported(p.M0, p.N0, 16, IREE_UK_FLAG_MMT4D_TYPE_S8S8S32)) {
    const int g = 16 / p.rb;
    const int64_t K1p = ((int64_t)p.K1 + g - 1) / g;
    const int64_t lhs_bytes = (int64_t)p.M1 * K1p * p.M0 * 16, rhs_bytes = (int64_t)p.N1 * K1p * p.N0 * 16;
    char* ws = nullptr;
    if (K1p * 64 * 16 < (1ll << 31) &&
        acquire_expand_workspace((size_t)(lhs_bytes + rhs_bytes), stream, &ws) == 0) {
      retile_rows(p.lhs, p.lhs_stride, p.M1, p.M0, p.rb, p.K1, 8, ws, stream);
      retile_rows(p.rhs, p.rhs_stride, p.N1, p.N0, p.rb, p.K1, 4, ws + lhs_bytes, stream);
      Problem q = p;
      q.lhs = ws;
      q.lhs_stride = K1p * p.M0 * 16;
      q.rhs = ws + lhs_bytes;
      q.rhs_stride = K1p * p.N0 * 16;
      q.K1 = (int32_t)K1p;
      q.rb = 16;
      q.lrb = 4;
      const char* s8_name = nullptr;
      const int st = launch_s8(q, 0, stream, &s8_name);
      if (st >= 0) {
        *name = "mmt4d_mfma_s8s4_expanded";
        return st;
      }
    }
  }
  if (p.rb < 16) return -1;  // the thin kernel unpacks 16 nibbles per lane: tile rows of 16 and more
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
