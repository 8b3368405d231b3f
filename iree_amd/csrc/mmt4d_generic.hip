// mmt4d, any-shape scalar kernel: one thread per output element, sequential
// (k, k0) accumulation in the order and with the per-type conversions of the
// CPU generic tile functions
// (runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:11-376). It serves
// every type triple and every (M0, N0, K0); the MFMA kernels take over for the
// shapes they cover. Compiled with -ffp-contract=off so that the float paths
// round after the multiply and after the add, like the CPU build.
#include <hip/hip_runtime.h>

#include "uk_device_common.h"
#include "uk_float_convert.h"
#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace {

constexpr int kThreads = 256;

using uk::small16_to_f32;
using uk::f32_to_small16;

// f8E4M3FN -> f32 (runtime/src/iree/base/internal/math.h:324-362 with 4
// exponent bits, 3 mantissa bits, bias 7, no infinities): S.1111.111 is NaN,
// exponent field 0 is m * 2^-9, otherwise (8 + m) * 2^(e - 10).
__device__ __forceinline__ float f8e4m3fn_to_f32(uint8_t v) {
  const uint32_t e = (v >> 3) & 0xF;
  const uint32_t m = v & 0x7;
  if (e == 0xF && m == 0x7) return __uint_as_float(0x7FC00000u);
  const uint32_t sign = (uint32_t)(v >> 7) << 31;
  if (e == 0) {
    // m * 2^-9 is exact in f32; build it from the integer.
    const float mag = (float)m * 0.001953125f;
    return __uint_as_float(__float_as_uint(mag) | sign);
  }
  return __uint_as_float(sign | ((e + 120u) << 23) | (m << 20));
}

struct Mmt4dArgs {
  const char* lhs;
  const char* rhs;
  char* out;
  int64_t lhs_stride_bytes, rhs_stride_bytes;
  // Output element (i, j, i0, j0) is out[i*out_s_i + i0*out_s_i0 + j*out_s_j + j0]
  // (elements): the tiled layout, or a row-major matrix for the fused
  // mmt4d + unpack, of which only out_rows x out_cols elements exist.
  int64_t out_s_i, out_s_i0, out_s_j;
  int64_t out_rows, out_cols;
  // Dequantizing store (32-bit accumulator kinds only): the output is f32,
  // (float)acc * row_scale[row] * col_scale[col] with a null scale reading as
  // 1, and ACCUMULATE reads the tiled buffer `acc` (acc_s_i elements between
  // rows of tiles) instead of the output.
  uint32_t dequant;
  const char* acc;
  int64_t acc_s_i;
  const float* row_scale;
  const float* col_scale;
  int64_t M, N, K;
  int32_t M0, N0, K0;
  uint32_t accumulate, skip_round;
  int64_t total;
};

enum class Kind { kF32, kS8S8, kS16S16, kS16S8, kS8S4, kS16U4, kF16F32, kBF16F32, kF16F16, kBF16BF16, kF8F32 };

template <Kind KIND>
__global__ __launch_bounds__(kThreads) void mmt4d_generic_kernel(Mmt4dArgs a) {
  const int64_t tile = (int64_t)a.M0 * a.N0;
  const int64_t row = a.N * tile;
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < a.total;
       idx += (int64_t)gridDim.x * kThreads) {
    const int64_t i = idx / row;
    const int64_t rem = idx - i * row;
    const int64_t j = rem / tile;
    const int64_t t = rem - j * tile;
    const int32_t i0 = (int32_t)(t / a.N0);
    const int32_t j0 = (int32_t)(t - (int64_t)i0 * a.N0);
    const char* lp = a.lhs + i * a.lhs_stride_bytes;
    const char* rp = a.rhs + j * a.rhs_stride_bytes;
    if (i * a.M0 + i0 >= a.out_rows || j * a.N0 + j0 >= a.out_cols) continue;
    const int64_t o = i * a.out_s_i + i0 * a.out_s_i0 + j * a.out_s_j + j0;
    const int32_t M0 = a.M0, N0 = a.N0, K0 = a.K0;
    // Where the initial accumulator is read, and what the finished one becomes.
    const char* acc_base = a.dequant ? a.acc : a.out;
    const int64_t ai = a.dequant ? i * a.acc_s_i + j * tile + t : o;
    auto scaled = [&](float v) {
      const float rs = a.row_scale ? a.row_scale[i * M0 + i0] : 1.0f;
      const float cs = a.col_scale ? a.col_scale[j * N0 + j0] : 1.0f;
      return v * rs * cs;
    };

    if constexpr (KIND == Kind::kS8S8 || KIND == Kind::kS16S16 || KIND == Kind::kS16S8) {
      int32_t* out = reinterpret_cast<int32_t*>(a.out);
      uint32_t acc = a.accumulate ? (uint32_t) reinterpret_cast<const int32_t*>(acc_base)[ai] : 0u;
      for (int64_t k = 0; k < a.K; ++k) {
        for (int32_t k0 = 0; k0 < K0; ++k0) {
          const int64_t li = (k * M0 + i0) * K0 + k0;
          const int64_t ri = (k * N0 + j0) * K0 + k0;
          int32_t l, r;
          if constexpr (KIND == Kind::kS8S8) l = reinterpret_cast<const int8_t*>(lp)[li];
          else l = reinterpret_cast<const int16_t*>(lp)[li];
          if constexpr (KIND == Kind::kS16S16) r = reinterpret_cast<const int16_t*>(rp)[ri];
          else r = reinterpret_cast<const int8_t*>(rp)[ri];
          acc += (uint32_t)(l * r);
        }
      }
      if (a.dequant) reinterpret_cast<float*>(a.out)[o] = scaled((float)(int32_t)acc);
      else out[o] = (int32_t)acc;
    } else if constexpr (KIND == Kind::kS8S4 || KIND == Kind::kS16U4) {
      // Two 4-bit rhs values per byte, low nibble first.
      int32_t* out = reinterpret_cast<int32_t*>(a.out);
      uint32_t acc = a.accumulate ? (uint32_t) reinterpret_cast<const int32_t*>(acc_base)[ai] : 0u;
      const int32_t K0h = K0 / 2;
      const uint8_t* r8 = reinterpret_cast<const uint8_t*>(rp);
      for (int64_t k = 0; k < a.K; ++k) {
        for (int32_t h = 0; h < K0h; ++h) {
          const int64_t li = (k * M0 + i0) * K0 + 2 * h;
          int32_t l0, l1;
          if constexpr (KIND == Kind::kS8S4) {
            l0 = reinterpret_cast<const int8_t*>(lp)[li];
            l1 = reinterpret_cast<const int8_t*>(lp)[li + 1];
          } else {
            l0 = reinterpret_cast<const int16_t*>(lp)[li];
            l1 = reinterpret_cast<const int16_t*>(lp)[li + 1];
          }
          const uint8_t byte = r8[(k * N0 + j0) * K0h + h];
          int32_t r0 = byte & 0xF, r1 = byte >> 4;
          if constexpr (KIND == Kind::kS8S4) {
            if (r0 & 8) r0 -= 16;
            if (r1 & 8) r1 -= 16;
          }
          acc += (uint32_t)(l0 * r0 + l1 * r1);
        }
      }
      if (a.dequant) reinterpret_cast<float*>(a.out)[o] = scaled((float)(int32_t)acc);
      else out[o] = (int32_t)acc;
    } else if constexpr (KIND == Kind::kF32 || KIND == Kind::kF16F32 ||
                         KIND == Kind::kBF16F32 || KIND == Kind::kF8F32) {
      float* out = reinterpret_cast<float*>(a.out);
      float acc = a.accumulate ? reinterpret_cast<const float*>(acc_base)[ai] : 0.f;
      for (int64_t k = 0; k < a.K; ++k) {
        for (int32_t k0 = 0; k0 < K0; ++k0) {
          const int64_t li = (k * M0 + i0) * K0 + k0;
          const int64_t ri = (k * N0 + j0) * K0 + k0;
          float l, r;
          if constexpr (KIND == Kind::kF32) {
            l = reinterpret_cast<const float*>(lp)[li];
            r = reinterpret_cast<const float*>(rp)[ri];
          } else if constexpr (KIND == Kind::kF16F32) {
            l = small16_to_f32<5>(reinterpret_cast<const uint16_t*>(lp)[li]);
            r = small16_to_f32<5>(reinterpret_cast<const uint16_t*>(rp)[ri]);
          } else if constexpr (KIND == Kind::kBF16F32) {
            l = small16_to_f32<8>(reinterpret_cast<const uint16_t*>(lp)[li]);
            r = small16_to_f32<8>(reinterpret_cast<const uint16_t*>(rp)[ri]);
          } else {
            l = f8e4m3fn_to_f32(reinterpret_cast<const uint8_t*>(lp)[li]);
            r = f8e4m3fn_to_f32(reinterpret_cast<const uint8_t*>(rp)[ri]);
          }
          acc += l * r;
        }
      }
      out[o] = a.dequant ? scaled(acc) : acc;
    } else {
      // f16 / bf16 results, with or without rounding the running sum to the
      // 16-bit type after every multiply-add.
      constexpr int EB = (KIND == Kind::kF16F16) ? 5 : 8;
      uint16_t* out = reinterpret_cast<uint16_t*>(a.out);
      const uint16_t* l16 = reinterpret_cast<const uint16_t*>(lp);
      const uint16_t* r16 = reinterpret_cast<const uint16_t*>(rp);
      if (a.skip_round) {
        float acc = a.accumulate ? small16_to_f32<EB>(out[o]) : 0.f;
        for (int64_t k = 0; k < a.K; ++k)
          for (int32_t k0 = 0; k0 < K0; ++k0)
            acc += small16_to_f32<EB>(l16[(k * M0 + i0) * K0 + k0]) *
                   small16_to_f32<EB>(r16[(k * N0 + j0) * K0 + k0]);
        out[o] = f32_to_small16<EB>(acc);
      } else {
        uint16_t acc = a.accumulate ? out[o] : (uint16_t)0;
        for (int64_t k = 0; k < a.K; ++k)
          for (int32_t k0 = 0; k0 < K0; ++k0) {
            const float l = small16_to_f32<EB>(l16[(k * M0 + i0) * K0 + k0]);
            const float r = small16_to_f32<EB>(r16[(k * N0 + j0) * K0 + k0]);
            acc = f32_to_small16<EB>(small16_to_f32<EB>(acc) + l * r);
          }
        out[o] = acc;
      }
    }
  }
}

}  // namespace

extern "C" int iree_uk_amd_hip_launch_mmt4d_generic(
    const iree_uk_mmt4d_params_t* p, const iree_uk_amd_rowmajor_out_t* rowmajor,
    void* stream_v) {
  hipStream_t stream = (hipStream_t)stream_v;
  int lhs_bits, rhs_bits, out_bytes;
  Kind kind;
  switch (p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: kind = Kind::kF32; lhs_bits = 32; rhs_bits = 32; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: kind = Kind::kS8S8; lhs_bits = 8; rhs_bits = 8; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: kind = Kind::kF16F32; lhs_bits = 16; rhs_bits = 16; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16: kind = Kind::kF16F16; lhs_bits = 16; rhs_bits = 16; out_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: kind = Kind::kBF16F32; lhs_bits = 16; rhs_bits = 16; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: kind = Kind::kBF16BF16; lhs_bits = 16; rhs_bits = 16; out_bytes = 2; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S16S32: kind = Kind::kS16S16; lhs_bits = 16; rhs_bits = 16; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16U4S32: kind = Kind::kS16U4; lhs_bits = 16; rhs_bits = 4; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S16S8S32: kind = Kind::kS16S8; lhs_bits = 16; rhs_bits = 8; out_bytes = 4; break;
    case IREE_UK_FLAG_MMT4D_TYPE_S8S4S32: kind = Kind::kS8S4; lhs_bits = 8; rhs_bits = 4; out_bytes = 4; break;
    case IREE_UK_AMD_FLAG_MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: kind = Kind::kF8F32; lhs_bits = 8; rhs_bits = 8; out_bytes = 4; break;
    default: return (int)hipErrorInvalidValue;
  }
  Mmt4dArgs a;
  a.lhs = (const char*)p->lhs_buffer + p->lhs_offset * lhs_bits / 8;
  a.rhs = (const char*)p->rhs_buffer + p->rhs_offset * rhs_bits / 8;
  a.out = (char*)p->out_buffer + p->out_offset * out_bytes;
  a.lhs_stride_bytes = p->lhs_stride0 * lhs_bits / 8;
  a.rhs_stride_bytes = p->rhs_stride0 * rhs_bits / 8;
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
    a.out_rows = p->M * p->M0;
    a.out_cols = p->N * p->N0;
  }
  a.dequant = 0;
  a.acc = nullptr;
  a.acc_s_i = 0;
  a.row_scale = a.col_scale = nullptr;
  if (rowmajor && rowmajor->dequant) {
    if (out_bytes != 4) return (int)hipErrorInvalidValue;
    a.dequant = 1;
    a.acc = (const char*)rowmajor->acc;
    a.acc_s_i = rowmajor->acc_stride0;
    a.row_scale = rowmajor->row_scale;
    a.col_scale = rowmajor->col_scale;
  }
  a.M = p->M; a.N = p->N; a.K = p->K;
  a.M0 = p->M0; a.N0 = p->N0; a.K0 = p->K0;
  a.accumulate = (p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  a.skip_round = (p->flags & IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) != 0;
  a.total = p->M * p->N * (int64_t)p->M0 * p->N0;
  if (a.total == 0) return 0;
  int64_t blocks = uk::ceil_div(a.total, kThreads);
  const int64_t cap = 256 * 64;
  const int grid = (int)(blocks < cap ? blocks : cap);
#define UK_LAUNCH(K) \
  case K: uk::launch(2, mmt4d_generic_kernel<K>, dim3(grid), dim3(kThreads), 0, stream, a); break;
  switch (kind) {
    UK_LAUNCH(Kind::kF32) UK_LAUNCH(Kind::kS8S8) UK_LAUNCH(Kind::kS16S16)
    UK_LAUNCH(Kind::kS16S8) UK_LAUNCH(Kind::kS8S4) UK_LAUNCH(Kind::kS16U4)
    UK_LAUNCH(Kind::kF16F32) UK_LAUNCH(Kind::kBF16F32) UK_LAUNCH(Kind::kF16F16)
    UK_LAUNCH(Kind::kBF16BF16) UK_LAUNCH(Kind::kF8F32)
  }
#undef UK_LAUNCH
  return (int)hipGetLastError();
}
