// mmt4d for the 16-bit integer LHS types (s16 x s16, s16 x s8, s16 x u4 -> s32;
// runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:80-169). gfx950 has
// no 16-bit integer matrix instruction; its widest exact one is the vector
// dot product v_dot2_i32_i16 (two s16 x s16 products added to a 32-bit
// accumulator, wrapping like the reference's int32 arithmetic). This kernel
// feeds it from LDS: a workgroup of 256 threads owns 64 x 64 output elements
// (rows and columns counted through the tiles, so any M0 / N0), walks K in
// steps of 32 elements, keeps each step's 64 x 32 LHS and RHS elements in LDS
// as s16 pairs (the RHS widened on the way in: s8 sign-extended, u4 low
// nibble first), and every thread accumulates a 4 x 4 block of outputs,
// sixteen dot products per four 16-byte LDS reads.
//
// Sums are exact modulo 2^32 in any order, so the result equals the
// reference's bit for bit. Needs K0 a power of two >= 2 (pairs of K elements
// then never straddle a tile row); other shapes stay on the scalar kernel.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace {

constexpr int kThreads = 256;
constexpr int kBlock = 64;   // rows and columns of outputs per workgroup
constexpr int kStepK = 32;   // K elements per step
constexpr int kPairs = kStepK / 2;
constexpr int kPitch = 20;   // dwords per LDS row: 16 pairs + 4, rows 16-byte aligned,
                             // 16 consecutive rows on 16 different bank groups

typedef short v2s __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

enum class Rhs { kS16, kS8, kU4 };

struct Dot2Args {
  const char* lhs;
  const char* rhs;
  char* out;
  int64_t lhs_stride_bytes, rhs_stride_bytes;
  // Output element (i, j, i0, j0) is out[i*out_s_i + i0*out_s_i0 + j*out_s_j + j0]
  // (elements): the tiled layout or a row-major matrix of out_rows x out_cols.
  int64_t out_s_i, out_s_i0, out_s_j;
  int64_t out_rows, out_cols;
  // Dequantizing store: f32 output scaled per row and column, ACCUMULATE input
  // from the tiled buffer `acc`.
  uint32_t dequant;
  const char* acc;
  int64_t acc_s_i;
  const float* row_scale;
  const float* col_scale;
  int64_t rows, cols;      // M * M0, N * N0
  int64_t k_total;         // K * K0
  int32_t M0, N0, K0, lk0; // lk0 = log2(K0)
  uint32_t accumulate;
};

// The pair of K elements (k, k + 1) of row `r0` of a tile of an operand whose
// tiles hold `T0` rows of K0 = 1 << lk0 elements: offset in elements from the
// start of the row panel. 32-bit arithmetic: the launcher checks that a panel
// spans fewer than 2^31 elements.
__device__ __forceinline__ uint32_t pair_offset(uint32_t k, uint32_t r0, uint32_t T0, uint32_t K0, uint32_t lk0) {
  return (((k >> lk0) * T0 + r0) << lk0) + (k & (K0 - 1));
}

template <Rhs RHS>
__global__ __launch_bounds__(kThreads) void mmt4d_dot2_kernel(Dot2Args a) {
  __shared__ __attribute__((aligned(16))) uint32_t lds_a[2][kBlock * kPitch];
  __shared__ __attribute__((aligned(16))) uint32_t lds_b[2][kBlock * kPitch];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int64_t row0 = (int64_t)blockIdx.y * kBlock, col0 = (int64_t)blockIdx.x * kBlock;

  // ---- loader items: 4 LHS pairs and 4 RHS pairs per thread and step --------
  // Item t = (K-tile of the step, row, pair in the tile row), pairs fastest,
  // so that consecutive lanes read consecutive memory for any K0.
  const int ppt = a.K0 / 2 < kPairs ? a.K0 / 2 : kPairs;  // pairs per tile row within a step
  const char* a_ptr[4];
  const char* b_ptr[4];
  int32_t a_r0[4], b_r0[4], pair_k[4], dst[4];
  bool a_ok[4], b_ok[4];
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    const int t = tid + n * kThreads;
    const int pp = t % ppt;
    const int rest = t / ppt;
    const int r = rest % kBlock;
    const int kt = rest / kBlock;
    pair_k[n] = (kt * ppt + pp) * 2;   // K element of the pair within the step
    dst[n] = r * kPitch + kt * ppt + pp;
    const int64_t R = row0 + r, C = col0 + r;
    a_ok[n] = R < a.rows;
    b_ok[n] = C < a.cols;
    const int64_t m1 = a_ok[n] ? R / a.M0 : 0, n1 = b_ok[n] ? C / a.N0 : 0;
    a_r0[n] = a_ok[n] ? (int32_t)(R - m1 * a.M0) : 0;
    b_r0[n] = b_ok[n] ? (int32_t)(C - n1 * a.N0) : 0;
    a_ptr[n] = a.lhs + m1 * a.lhs_stride_bytes;
    b_ptr[n] = a.rhs + n1 * a.rhs_stride_bytes;
  }
  const uint32_t k_total = (uint32_t)a.k_total;
  auto load_a = [&](int n, uint32_t kbase) -> uint32_t {
    const uint32_t k = kbase + (uint32_t)pair_k[n];
    if (!a_ok[n] || k >= k_total) return 0u;
    const uint32_t e = pair_offset(k, (uint32_t)a_r0[n], (uint32_t)a.M0, (uint32_t)a.K0, (uint32_t)a.lk0);
    typedef uint32_t u32_unaligned __attribute__((aligned(2)));
    return *reinterpret_cast<const u32_unaligned*>(a_ptr[n] + (uint64_t)e * 2);
  };
  auto load_b = [&](int n, uint32_t kbase) -> uint32_t {
    const uint32_t k = kbase + (uint32_t)pair_k[n];
    if (!b_ok[n] || k >= k_total) return 0u;
    const uint32_t e = pair_offset(k, (uint32_t)b_r0[n], (uint32_t)a.N0, (uint32_t)a.K0, (uint32_t)a.lk0);
    if constexpr (RHS == Rhs::kS16) {
      typedef uint32_t u32_unaligned __attribute__((aligned(2)));
      return *reinterpret_cast<const u32_unaligned*>(b_ptr[n] + (uint64_t)e * 2);
    } else if constexpr (RHS == Rhs::kS8) {
      typedef uint16_t u16_unaligned __attribute__((aligned(1)));
      const uint32_t w = *reinterpret_cast<const u16_unaligned*>(b_ptr[n] + e);
      const int32_t lo = (int8_t)(w & 0xFF), hi = (int8_t)(w >> 8);
      return ((uint32_t)lo & 0xFFFFu) | ((uint32_t)hi << 16);
    } else {
      // Two 4-bit values per byte, low nibble first; e is even.
      const uint8_t byte = *reinterpret_cast<const uint8_t*>(b_ptr[n] + (e >> 1));
      return (uint32_t)(byte & 0xF) | ((uint32_t)(byte >> 4) << 16);
    }
  };

  // ---- accumulators: rows ty + 16 i, columns tx + 16 j ----------------------------
  int32_t acc[4][4];
  int64_t out_index[4][4];   // may be negative: strides of any sign
  uint32_t exists = 0;       // bit 4 i + j: the element is part of the result
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t R = row0 + ty + 16 * i;
    const int64_t m1 = R / a.M0;
    const int64_t i0 = R - m1 * a.M0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t C = col0 + tx + 16 * j;
      const int64_t n1 = C / a.N0;
      const int64_t j0 = C - n1 * a.N0;
      const bool ok = R < a.rows && C < a.cols && R < a.out_rows && C < a.out_cols;
      out_index[i][j] = ok ? m1 * a.out_s_i + i0 * a.out_s_i0 + n1 * a.out_s_j + j0 : 0;
      if (ok) exists |= 1u << (4 * i + j);
      acc[i][j] = 0;
      if (ok && a.accumulate) {
        const int64_t ai = a.dequant ? m1 * a.acc_s_i + (n1 * a.M0 + i0) * a.N0 + j0 : out_index[i][j];
        acc[i][j] = reinterpret_cast<const int32_t*>(a.dequant ? a.acc : a.out)[ai];
      }
    }
  }

  // ---- K loop: LDS double-buffered, one barrier per step ---------------------------
  const uint32_t steps = (k_total + kStepK - 1) / kStepK;
  uint32_t ra[4], rb[4];
#pragma unroll
  for (int n = 0; n < 4; ++n) { ra[n] = load_a(n, 0); rb[n] = load_b(n, 0); }
#pragma unroll
  for (int n = 0; n < 4; ++n) { lds_a[0][dst[n]] = ra[n]; lds_b[0][dst[n]] = rb[n]; }
  __syncthreads();
  for (uint32_t s = 0; s < steps; ++s) {
    const int cur = (int)(s & 1);
    if (s + 1 < steps) {
#pragma unroll
      for (int n = 0; n < 4; ++n) { ra[n] = load_a(n, (s + 1) * kStepK); rb[n] = load_b(n, (s + 1) * kStepK); }
    }
#pragma unroll
    for (int q = 0; q < kPairs / 4; ++q) {
      v4u fa[4], fb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        fa[i] = *reinterpret_cast<const v4u*>(&lds_a[cur][(ty + 16 * i) * kPitch + 4 * q]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        fb[j] = *reinterpret_cast<const v4u*>(&lds_b[cur][(tx + 16 * j) * kPitch + 4 * q]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // (Through scalars: a bit cast applied directly to a vector
            // element reads element 0 whatever the index.)
            const uint32_t pa = fa[i][e], pb = fb[j][e];
            acc[i][j] = __builtin_amdgcn_sdot2(__builtin_bit_cast(v2s, pa), __builtin_bit_cast(v2s, pb),
                                               acc[i][j], false);
          }
    }
    if (s + 1 < steps) {
#pragma unroll
      for (int n = 0; n < 4; ++n) { lds_a[cur ^ 1][dst[n]] = ra[n]; lds_b[cur ^ 1][dst[n]] = rb[n]; }
    }
    __syncthreads();
  }

  // ---- store -------------------------------------------------------------------------
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!(exists & (1u << (4 * i + j)))) continue;
      if (a.dequant) {
        const int64_t R = row0 + ty + 16 * i, C = col0 + tx + 16 * j;
        const float rs = a.row_scale ? a.row_scale[R] : 1.0f;
        const float cs = a.col_scale ? a.col_scale[C] : 1.0f;
        reinterpret_cast<float*>(a.out)[out_index[i][j]] = (float)acc[i][j] * rs * cs;
      } else {
        reinterpret_cast<int32_t*>(a.out)[out_index[i][j]] = acc[i][j];
      }
    }
  }
}

}  // namespace

// Returns 0 when launched, a positive hipError_t value on a launch error, -1
// when this kernel does not serve the call (the scalar kernel then does).
extern "C" int iree_uk_amd_hip_launch_mmt4d_dot2(const iree_uk_mmt4d_params_t* p,
                                                 const iree_uk_amd_rowmajor_out_t* rowmajor,
                                                 void* stream_v) {
  hipStream_t stream = (hipStream_t)stream_v;
  Rhs rhs;
  int rhs_bits;
  switch (p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: rhs = Rhs::kS16; rhs_bits = 16; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: rhs = Rhs::kS8; rhs_bits = 8; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: rhs = Rhs::kU4; rhs_bits = 4; break;
    default: return -1;
  }
  const int32_t K0 = p->K0;
  if (K0 < 2 || (K0 & (K0 - 1)) != 0) return -1;
  if (p->M <= 0 || p->N <= 0 || p->K <= 0 || p->M0 <= 0 || p->N0 <= 0) return -1;
  Dot2Args a{};
  a.lhs = (const char*)p->lhs_buffer + p->lhs_offset * 2;
  a.rhs = (const char*)p->rhs_buffer + p->rhs_offset * rhs_bits / 8;
  a.out = (char*)p->out_buffer + p->out_offset * 4;
  a.lhs_stride_bytes = p->lhs_stride0 * 2;
  a.rhs_stride_bytes = p->rhs_stride0 * rhs_bits / 8;
  a.rows = p->M * (int64_t)p->M0;
  a.cols = p->N * (int64_t)p->N0;
  if (rowmajor) {
    a.out_s_i0 = rowmajor->stride0;
    a.out_s_i = rowmajor->stride0 * p->M0;
    a.out_s_j = p->N0;
    a.out_rows = rowmajor->size0;
    a.out_cols = rowmajor->size1;
  } else {
    a.out_s_i = p->out_stride0;
    a.out_s_i0 = p->N0;
    a.out_s_j = (int64_t)p->M0 * p->N0;
    a.out_rows = a.rows;
    a.out_cols = a.cols;
  }
  if (rowmajor && rowmajor->dequant) {
    a.dequant = 1;
    a.acc = (const char*)rowmajor->acc;
    a.acc_s_i = rowmajor->acc_stride0;
    a.row_scale = rowmajor->row_scale;
    a.col_scale = rowmajor->col_scale;
  }
  a.k_total = p->K * (int64_t)K0;
  // 32-bit offsets inside a row panel (in elements) and a 32-bit K counter.
  if (a.k_total >= (1ll << 31) - 64 || a.k_total * p->M0 >= (1ll << 31) || a.k_total * p->N0 >= (1ll << 31)) {
    return -1;
  }
  a.M0 = p->M0; a.N0 = p->N0; a.K0 = K0;
  while ((1 << a.lk0) < K0) ++a.lk0;
  a.accumulate = (p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  const int64_t grid_x = (a.cols + kBlock - 1) / kBlock, grid_y = (a.rows + kBlock - 1) / kBlock;
  if (grid_x >= (1ll << 31) || grid_y > 65535) return -1;
  const dim3 grid((uint32_t)grid_x, (uint32_t)grid_y);
  switch (rhs) {
    case Rhs::kS16: uk::launch(2, mmt4d_dot2_kernel<Rhs::kS16>, grid, dim3(kThreads), 0, stream, a); break;
    case Rhs::kS8: uk::launch(2, mmt4d_dot2_kernel<Rhs::kS8>, grid, dim3(kThreads), 0, stream, a); break;
    case Rhs::kU4: uk::launch(2, mmt4d_dot2_kernel<Rhs::kU4>, grid, dim3(kThreads), 0, stream, a); break;
  }
  return (int)hipGetLastError();
}
