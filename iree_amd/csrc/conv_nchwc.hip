// conv_nchwc, f32 only as in the reference. Two kernels:
//
//   * conv_nchwc_mfma, for k0 = 16 and c0 a multiple of 16 (the reference's own
//     tuned tile shape is 16 x 16 x 16,
//     runtime/src/iree/builtins/ukernel/arch/x86_64/conv_nchwc_x86_64_avx512_base.c:17-28):
//     an output panel of 16 pixels x 16 channels is a 16x16 MFMA block whose K
//     runs over (ic_outer, fh, fw, ci). A wave owns TW panels along OW times
//     TO along OC_outer and feeds v_mfma_f32_16x16x4_f32 straight from global
//     memory: a lane's 16-byte piece of one input pixel (four ci) is the
//     operand of four instructions, one per word, against four filter words
//     of the same four ci. Sums are in MFMA order, so results equal the
//     reference's to rounding, and exactly where every partial sum is exact
//     (the reference's own test data, tools/conv_nchwc_test.c:174-178).
//   * conv_nchwc_generic, for every other shape: one thread per output
//     element, accumulating in the order of the CPU generic tile function
//     (runtime/src/iree/builtins/ukernel/conv_nchwc_tile_generic.c:34-57) with
//     a separate multiply and add, so that results equal the reference's
//     generic path bit for bit.
#include <hip/hip_runtime.h>

#include "uk_device_common.h"
#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace {

constexpr int kThreads = 256;

struct ConvArgs {
  const float* in;
  const float* flt;
  float* out;
  int64_t in_sn, in_sic, in_sh;
  int64_t f_soc, f_sic, f_sfh;
  int64_t out_sn, out_soc, out_soh;
  int64_t OC, OH, OW, IC, FH, FW;
  int32_t k0, c0, stride_h, stride_w;
  uint32_t accumulate;
  int64_t total;
};

__global__ __launch_bounds__(kThreads) void conv_nchwc_generic_kernel(ConvArgs a) {
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < a.total;
       idx += (int64_t)gridDim.x * kThreads) {
    int64_t t = idx;
    const int32_t ko = (int32_t)(t % a.k0); t /= a.k0;
    const int64_t ow = t % a.OW; t /= a.OW;
    const int64_t oh = t % a.OH; t /= a.OH;
    const int64_t oc = t % a.OC;
    const int64_t n = t / a.OC;
    float* o = a.out + n * a.out_sn + oc * a.out_soc + oh * a.out_soh + ow * a.k0 + ko;
    float acc = a.accumulate ? *o : 0.f;
    const float* in_n = a.in + n * a.in_sn + (oh * a.stride_h) * a.in_sh + (ow * a.stride_w) * a.c0;
    const float* f_oc = a.flt + oc * a.f_soc + ko;
    for (int64_t ic = 0; ic < a.IC; ++ic) {
      for (int64_t fh = 0; fh < a.FH; ++fh) {
        const float* in_row = in_n + ic * a.in_sic + fh * a.in_sh;
        const float* f_row = f_oc + ic * a.f_sic + fh * a.f_sfh;
        for (int64_t fw = 0; fw < a.FW; ++fw) {
          for (int32_t ci = 0; ci < a.c0; ++ci) {
            acc += in_row[fw * a.c0 + ci] * f_row[(fw * a.c0 + ci) * (int64_t)a.k0];
          }
        }
      }
    }
    *o = acc;
  }
}

typedef float v4f __attribute__((ext_vector_type(4)));
typedef v4f v4f_a4 __attribute__((aligned(4)));  // dword-aligned wide accesses are legal here

// One wave per work item (n, group of TO output-channel blocks, oh, group of
// TW panels of 16 output pixels); no LDS, no barrier. Lane (q, r) = (lane / 16,
// lane % 16) supplies input pixel r, channels 4q..4q+3 of the current 16, and
// filter words [ci = 4q + w][ko = r]; with the filter as the first MFMA operand
// it ends up holding output pixel r, channels 4q..4q+3: one 16-byte store.
// Pixels and channel blocks past the end read the last valid one instead
// (their accumulators are not stored).
template <int TW, int TO>
__global__ __launch_bounds__(kThreads) void conv_nchwc_mfma_kernel(ConvArgs a, int64_t items,
                                                                   int64_t ow_chunks,
                                                                   int64_t oc_chunks) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t item = (int64_t)blockIdx.x * (kThreads / 64) + wave;
  if (item >= items) return;
  int64_t t = item;
  const int64_t owc = t % ow_chunks; t /= ow_chunks;
  const int64_t oh = t % a.OH; t /= a.OH;
  const int64_t occ = t % oc_chunks;
  const int64_t n = t / oc_chunks;
  const int r = lane & 15, q = lane >> 4;

  const float* pa[TW];
  const float* pb[TO];
  float* po[TW][TO];
  bool ok[TW][TO];
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    const int64_t ow = owc * (16 * TW) + tw * 16 + r;
    const int64_t ow_in = ow < a.OW ? ow : a.OW - 1;
    pa[tw] = a.in + n * a.in_sn + (oh * a.stride_h) * a.in_sh + (ow_in * a.stride_w) * a.c0 + 4 * q;
#pragma unroll
    for (int to = 0; to < TO; ++to) {
      const int64_t oc = occ * TO + to;
      const int64_t oc_in = oc < a.OC ? oc : a.OC - 1;
      ok[tw][to] = ow < a.OW && oc < a.OC;
      po[tw][to] = a.out + n * a.out_sn + oc_in * a.out_soc + oh * a.out_soh + ow_in * 16 + 4 * q;
    }
  }
#pragma unroll
  for (int to = 0; to < TO; ++to) {
    const int64_t oc = occ * TO + to;
    pb[to] = a.flt + (oc < a.OC ? oc : a.OC - 1) * a.f_soc + (4 * q) * 16 + r;
  }

  v4f acc[TW][TO];
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int to = 0; to < TO; ++to) {
      acc[tw][to] = v4f{0.f, 0.f, 0.f, 0.f};
      if (a.accumulate && ok[tw][to]) acc[tw][to] = *reinterpret_cast<const v4f_a4*>(po[tw][to]);
    }

  // Within one (ic_outer, fh) the taps (fw, 16 channels at a time) follow each
  // other at 16 input floats and 256 filter floats.
  const int64_t taps = a.FW * (a.c0 / 16);
  for (int64_t ic = 0; ic < a.IC; ++ic) {
    for (int64_t fh = 0; fh < a.FH; ++fh) {
      const int64_t ao = ic * a.in_sic + fh * a.in_sh;
      const int64_t bo = ic * a.f_sic + fh * a.f_sfh;
      for (int64_t tap = 0; tap < taps; ++tap) {
        v4f av[TW];
        float bv[TO][4];
#pragma unroll
        for (int tw = 0; tw < TW; ++tw)
          av[tw] = *reinterpret_cast<const v4f_a4*>(pa[tw] + ao + tap * 16);
#pragma unroll
        for (int to = 0; to < TO; ++to)
#pragma unroll
          for (int w = 0; w < 4; ++w) bv[to][w] = pb[to][bo + tap * 256 + w * 16];
#pragma unroll
        for (int w = 0; w < 4; ++w)
#pragma unroll
          for (int tw = 0; tw < TW; ++tw)
#pragma unroll
            for (int to = 0; to < TO; ++to)
              acc[tw][to] =
                  __builtin_amdgcn_mfma_f32_16x16x4f32(bv[to][w], av[tw][w], acc[tw][to], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int to = 0; to < TO; ++to)
      if (ok[tw][to]) *reinterpret_cast<v4f_a4*>(po[tw][to]) = acc[tw][to];
}

template <int TW, int TO>
int launch_mfma(const ConvArgs& a, int64_t N, hipStream_t stream) {
  const int64_t ow_chunks = uk::ceil_div(a.OW, (int64_t)16 * TW);
  const int64_t oc_chunks = uk::ceil_div(a.OC, (int64_t)TO);
  const int64_t items = N * oc_chunks * a.OH * ow_chunks;
  const int64_t blocks = uk::ceil_div(items, (int64_t)(kThreads / 64));
  if (blocks >= (1ll << 31)) return -1;
  uk::launch(3, conv_nchwc_mfma_kernel<TW, TO>, dim3((uint32_t)blocks), dim3(kThreads), 0, stream,
             a, items, ow_chunks, oc_chunks);
  return (int)hipGetLastError();
}

}  // namespace

extern "C" int iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(int32_t k0, int32_t c0,
                                                          uint32_t flags) {
  return (flags & IREE_UK_FLAG_CONV_NCHWC_TYPE_MASK) == IREE_UK_FLAG_CONV_NCHWC_TYPE_F32F32F32 &&
         k0 == 16 && c0 > 0 && c0 % 16 == 0;
}

extern "C" int iree_uk_amd_hip_launch_conv_nchwc(const iree_uk_conv_nchwc_params_t* p,
                                                 void* stream_v, int kernel_mode,
                                                 const char** kernel_name) {
  hipStream_t stream = (hipStream_t)stream_v;
  if ((p->flags & IREE_UK_FLAG_CONV_NCHWC_TYPE_MASK) != IREE_UK_FLAG_CONV_NCHWC_TYPE_F32F32F32) {
    return (int)hipErrorInvalidValue;
  }
  ConvArgs a;
  a.in = (const float*)p->input_buffer + p->input_offset;
  a.flt = (const float*)p->filter_buffer + p->filter_offset;
  a.out = (float*)p->output_buffer + p->output_offset;
  a.in_sn = p->input_stride_n; a.in_sic = p->input_stride_ic_outer; a.in_sh = p->input_stride_h;
  a.f_soc = p->filter_stride_oc_outer; a.f_sic = p->filter_stride_ic_outer;
  a.f_sfh = p->filter_stride_fh;
  a.out_sn = p->output_stride_n; a.out_soc = p->output_stride_oc_outer;
  a.out_soh = p->output_stride_oh;
  a.OC = p->OC_outer; a.OH = p->OH; a.OW = p->OW; a.IC = p->IC_outer; a.FH = p->FH; a.FW = p->FW;
  a.k0 = p->k0; a.c0 = p->c0; a.stride_h = p->stride_h; a.stride_w = p->stride_w;
  a.accumulate = (p->flags & IREE_UK_FLAG_CONV_NCHWC_ACCUMULATE) != 0;
  a.total = p->N * p->OC_outer * p->OH * p->OW * (int64_t)p->k0;
  if (a.total == 0) {
    *kernel_name = "";
    return 0;
  }
  if (kernel_mode != IREE_UK_AMD_KERNEL_MODE_GENERIC &&
      iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(p->k0, p->c0, p->flags)) {
    const bool wide = a.OW > 16, deep = a.OC > 1;
    int st = wide ? (deep ? launch_mfma<2, 2>(a, p->N, stream) : launch_mfma<2, 1>(a, p->N, stream))
                  : (deep ? launch_mfma<1, 2>(a, p->N, stream) : launch_mfma<1, 1>(a, p->N, stream));
    if (st >= 0) {
      *kernel_name = "conv_nchwc_mfma";
      return st;
    }
  }
  *kernel_name = "conv_nchwc_generic";
  const int64_t blocks = uk::ceil_div(a.total, kThreads);
  const int64_t cap = 256 * 64;
  uk::launch(3, conv_nchwc_generic_kernel, dim3((uint32_t)(blocks < cap ? blocks : cap)),
             dim3(kThreads), 0, stream, a);
  return (int)hipGetLastError();
}
