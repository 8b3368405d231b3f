// s16 x s16 -> s32 on the matrix cores: four 8-bit integer products per
// element pair in the LDS-direct pipeline (mmt4d_mfma_kernel.h, PIPE 5), one
// 128x128 workgroup shape. Served: tile rows of 2 to 128 bytes (K0 = 1 .. 64),
// tiles of at most 64 rows, K in whole steps of 64 elements; everything else
// stays with the vector dot-product kernel (mmt4d_dot2.hip), as do problems too
// thin to fill 128x128 blocks.
//
// s16 x s8 and s16 x u4 -> s32 reach the same kernel from 128 rows and columns
// on: their right-hand side is widened to s16 once per call, into a buffer the
// library keeps, and the call continues as s16 x s16 (the products are the same
// integers).
#include "mmt4d_mfma_launch.h"
#include "uk_hip_abi.h"

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

extern "C" int iree_uk_amd_hip_launch_mmt4d_mfma(const iree_uk_mmt4d_params_t* p,
                                                 const iree_uk_amd_rowmajor_out_t* rowmajor,
                                                 void* stream, int forced_variant,
                                                 const char** kernel_name);

namespace {

typedef uint32_t v2u_g __attribute__((ext_vector_type(2), aligned(1)));
typedef uint32_t v4u_w __attribute__((ext_vector_type(4)));

// Panel n of the RHS (`panel_in_bytes` bytes at src + n * src_stride) widened to
// 16-bit elements at dst + n * panel_out_bytes. BITS = 8: signed bytes, a thread
// takes 8 of them; BITS = 4: unsigned nibbles, low nibble first
// (mmt4d_tile_generic.c:128-133 of the reference), a thread takes 4 bytes.
template <int BITS>
__global__ __launch_bounds__(256) void widen_rhs_kernel(const char* src, int64_t src_stride, char* dst,
                                                         uint32_t panel_in_bytes) {
  constexpr uint32_t kIn = BITS == 8 ? 8 : 4;  // bytes a thread reads; it writes 16
  const char* s = src + (int64_t)blockIdx.y * src_stride;
  char* d = dst + (int64_t)blockIdx.y * (16 / kIn) * panel_in_bytes;
  for (uint32_t off = (blockIdx.x * 256 + threadIdx.x) * kIn; off < panel_in_bytes; off += gridDim.x * 256 * kIn) {
    v4u_w out;
    if constexpr (BITS == 8) {
      const v2u_g in = *reinterpret_cast<const v2u_g*>(s + off);
#pragma unroll
      for (int w = 0; w < 2; ++w) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t e0 = (uint32_t)__builtin_amdgcn_sbfe((int)in[w], 16 * h, 8) & 0xFFFFu;
          const uint32_t e1 = (uint32_t)__builtin_amdgcn_sbfe((int)in[w], 16 * h + 8, 8);
          out[2 * w + h] = e0 | (e1 << 16);
        }
      }
    } else {
      typedef uint32_t u32_g __attribute__((aligned(1)));
      const uint32_t in = *reinterpret_cast<const u32_g*>(s + off);
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = ((in >> (8 * j)) & 0xFu) | (((in >> (8 * j + 4)) & 0xFu) << 16);
    }
    *reinterpret_cast<v4u_w*>(d + (16 / kIn) * (int64_t)off) = out;
  }
}

}  // namespace

// s16 x s8 / s16 x u4 as s16 x s16 on a widened RHS. Returns a HIP status, or
// a negative value when the call is not served this way (other types, fewer
// than 128 rows or columns, K not in whole steps of 64 elements, no buffer to be
// had); nothing has been launched then.
extern "C" int iree_uk_amd_hip_launch_mmt4d_s16_widened(const iree_uk_mmt4d_params_t* p,
                                                        const iree_uk_amd_rowmajor_out_t* rowmajor,
                                                        void* stream_v, const char** kernel_name) {
  const uint32_t type = p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK;
  int bits;
  if (type == IREE_UK_FLAG_MMT4D_TYPE_S16S8S32) bits = 8;
  else if (type == IREE_UK_FLAG_MMT4D_TYPE_S16U4S32) bits = 4;
  else return -1;
  const int64_t rows = rowmajor ? rowmajor->size0 : (int64_t)p->M * p->M0;
  const int64_t cols = rowmajor ? rowmajor->size1 : (int64_t)p->N * p->N0;
  if (rows < 128 || cols < 128 || p->K <= 0 || p->N <= 0 || p->N >= 65536) return -1;
  const int64_t k_elems = (int64_t)p->K * p->K0;
  if (k_elems % 64 != 0 || (bits == 4 && p->K0 % 2 != 0)) return -1;
  if (p->rhs_stride0 < 0 || (bits == 4 && ((p->rhs_stride0 | p->rhs_offset) & 1))) return -1;
  // What the s16 kernel asks of the tile (checked here so that a call it would
  // decline is not widened first): tile rows of 2 to 128 bytes, a power of two;
  // tiles of at most 64 rows; whole rows per 16-byte piece.
  const int64_t rb = (int64_t)p->K0 * 2;
  if (rb < 2 || rb > 128 || (rb & (rb - 1)) != 0) return -1;
  if (p->M0 < 1 || p->N0 < 1 || p->M0 > 64 || p->N0 > 64) return -1;
  if (rb < 16 && (p->M0 % (16 / rb) || p->N0 % (16 / rb))) return -1;
  const int64_t panel_elems = (int64_t)p->K * p->N0 * p->K0;
  const int64_t panel_in_bytes = panel_elems * bits / 8;
  if (panel_in_bytes % 8 != 0 || panel_in_bytes >= (1ll << 30)) return -1;
  hipStream_t stream = (hipStream_t)stream_v;
  char* widened = nullptr;
  if (uk_mfma::acquire_expand_workspace((size_t)(2 * panel_elems * p->N), stream, &widened) != 0) return -1;
  const char* src = (const char*)p->rhs_buffer + p->rhs_offset * bits / 8;
  const int64_t src_stride = p->rhs_stride0 * bits / 8;
  const uint32_t per_thread = bits == 8 ? 8 : 4;
  const uint32_t per_panel =
      (uint32_t)std::min<int64_t>(uk::ceil_div(panel_in_bytes, (int64_t)(256 * per_thread)), 64);
  if (bits == 8) {
    uk::launch(2, widen_rhs_kernel<8>, dim3(per_panel, (uint32_t)p->N), dim3(256), 0, stream, src, src_stride,
               widened, (uint32_t)panel_in_bytes);
  } else {
    uk::launch(2, widen_rhs_kernel<4>, dim3(per_panel, (uint32_t)p->N), dim3(256), 0, stream, src, src_stride,
               widened, (uint32_t)panel_in_bytes);
  }
  iree_uk_mmt4d_params_t q = *p;
  q.flags = (p->flags & ~(uint32_t)IREE_UK_FLAG_MMT4D_TYPE_MASK) | IREE_UK_FLAG_MMT4D_TYPE_S16S16S32;
  q.rhs_buffer = widened;
  q.rhs_offset = 0;
  q.rhs_stride0 = panel_elems;
  // (A call the s16 launcher still declines - operands of 2 GiB, negative
  // strides - has cost one pass over the weights and goes on to the
  // dot-product kernel.)
  const char* inner = nullptr;
  const int st = iree_uk_amd_hip_launch_mmt4d_mfma(&q, rowmajor, stream_v, 0, &inner);
  if (st >= 0) *kernel_name = "mmt4d_mfma_128x128_s16_widened";
  return st;
}
