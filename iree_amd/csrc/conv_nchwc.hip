// conv_nchwc: one thread per output element, accumulating in the order of the
// CPU generic tile function
// (runtime/src/iree/builtins/ukernel/conv_nchwc_tile_generic.c:34-57) with a
// separate multiply and add (-ffp-contract=off), so that results equal the
// reference's generic path bit for bit. f32 only, as in the reference.
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

}  // namespace

extern "C" int iree_uk_amd_hip_launch_conv_nchwc(const iree_uk_conv_nchwc_params_t* p,
                                                 void* stream_v, const char** kernel_name) {
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
  *kernel_name = "conv_nchwc_generic";
  if (a.total == 0) return 0;
  const int64_t blocks = uk::ceil_div(a.total, kThreads);
  const int64_t cap = 256 * 64;
  uk::launch(3, conv_nchwc_generic_kernel, dim3((uint32_t)(blocks < cap ? blocks : cap)),
             dim3(kThreads), 0, stream, a);
  return (int)hipGetLastError();
}
