// conv_nchwc, f32 only as in the reference. Two kernels:
//
//   * conv_nchwc_mfma, for k0 = 16 and c0 a multiple of 16 (the reference's own
//     tuned tile shape is 16 x 16 x 16,
//     runtime/src/iree/builtins/ukernel/arch/x86_64/conv_nchwc_x86_64_avx512_base.c:17-28):
//     an output panel of 16 pixels x 16 channels is a 16x16 MFMA block whose K
//     runs over (ic_outer, fh, fw, ci). A wave owns TW panels of consecutive
//     output pixels times TO blocks of OC_outer and feeds
//     v_mfma_f32_16x16x4_f32: a lane's 16-byte piece of one input pixel (four
//     ci, straight from global memory) is the operand of four instructions,
//     one per word, against four filter words of the same four ci (staged
//     through LDS by the workgroup). Sums are in MFMA order, so results equal the
//     reference's to rounding, and exactly where every partial sum is exact
//     (the reference's own test data, tools/conv_nchwc_test.c:174-178).
//   * conv_nchwc_generic, for every other shape: one thread per output
//     element, accumulating in the order of the CPU generic tile function
//     (runtime/src/iree/builtins/ukernel/conv_nchwc_tile_generic.c:34-57) with
//     a separate multiply and add, so that results equal the reference's
//     generic path bit for bit.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "uk_device_common.h"
#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace uk_mfma {
// mmt4d_mfma.hip: a buffer the library keeps per host thread and stream (0 and
// the pointer, or 1 when there is none to be had).
int acquire_expand_workspace(size_t bytes, hipStream_t stream, char** base);
}  // namespace uk_mfma

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
  // conv_nchwc_mfma only: IC_outer split over `ic_slices` workgroups per output
  // block (1 = none). Slice s takes ic_per consecutive values of ic_outer and
  // stores its sums, as if it were the whole call without ACCUMULATE, at
  // `partial` + s * partial_stride with the output's own strides;
  // conv_reduce_slices_kernel adds the slices up in order.
  int64_t N;
  int32_t ic_slices;
  int64_t ic_per;
  float* partial;
  int64_t partial_stride;
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

// A workgroup of four waves owns (n, TO output-channel blocks, 4 x TW panels of
// 16 output pixels); each wave computes TW panels against all TO blocks.
// Pixels are counted through (oh, ow) together, so rows shorter than a panel
// waste nothing. A step is one (ic_outer, fh, fw, 16 channels): 16 input
// floats per pixel against a [16 ci][16 ko] filter tile per channel block.
//
// Lane (q, r) = (lane / 16, lane % 16) supplies input pixel r, channels
// 4q..4q+3 of the step's 16 (one 16-byte global load, a step ahead, two
// register buffers) and filter words [ci = 4q + w][ko = r], w = 0..3. Those
// four words are 64 bytes apart in memory, so the filter tiles go through LDS:
// the first TO waves copy a step's tiles with one 16-byte load per lane
// (global memory a step ahead, LDS double-buffered, rows padded to 20 floats so
// that the 64 lanes of a read hit 64 different banks), one barrier per step.
// With the filter as the first MFMA operand a lane ends up holding output
// pixel r, channels 4q..4q+3: one 16-byte store. Pixels, panels and channel
// blocks past the end read the last valid one instead and are not stored; a
// prefetch past the last step reloads the last step.
constexpr int kFilterRow = 20;                 // floats per padded ci row in LDS
constexpr int kFilterTile = 16 * kFilterRow;   // floats per [16][16] tile in LDS

template <int TW, int TO>
__global__ __launch_bounds__(kThreads) void conv_nchwc_mfma_kernel(ConvArgs a, int64_t px_chunks,
                                                                   int64_t px_groups,
                                                                   int64_t oc_chunks) {
  static_assert(TO * 64 <= kThreads, "one loader lane per 16 bytes of the step's filter tiles");
  __shared__ __attribute__((aligned(16))) float filt[2][TO * kFilterTile];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Consecutive workgroup ids go round-robin to the 8 XCDs, each with its own
  // L2. Give every XCD a contiguous range of the work instead, so that one L2
  // sees one image and one filter slice at a time, not a slice of all.
  const uint32_t nb = gridDim.x, xcd = blockIdx.x & 7u;
  int64_t t = (int64_t)(xcd * (nb / 8u) + min(xcd, nb % 8u) + (blockIdx.x >> 3));
  const int64_t pxg = t % px_groups; t /= px_groups;
  const int64_t occ = t % oc_chunks; t /= oc_chunks;
  const int64_t n = t % a.N;
  const int64_t slice = t / a.N;
  const int64_t ic0 = slice * a.ic_per;
  const int64_t ic_count = a.ic_slices > 1 ? min(a.ic_per, a.IC - ic0) : a.IC;
  float* const out_base = a.ic_slices > 1 ? a.partial + slice * a.partial_stride : a.out;
  const bool accumulate = a.ic_slices > 1 ? false : a.accumulate != 0;
  const int64_t pxc_raw = pxg * 4 + wave;
  const bool wave_ok = pxc_raw < px_chunks;
  const int64_t pxc = wave_ok ? pxc_raw : px_chunks - 1;
  const int r = lane & 15, q = lane >> 4;
  const int64_t pixels = a.OH * a.OW;

  const float* pa[TW];
  float* po[TW][TO];
  bool ok[TW][TO];
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    const int64_t px = pxc * (16 * TW) + tw * 16 + r;
    const int64_t px_in = px < pixels ? px : pixels - 1;
    const int64_t oh = px_in / a.OW, ow = px_in - oh * a.OW;
    pa[tw] = a.in + n * a.in_sn + ic0 * a.in_sic + (oh * a.stride_h) * a.in_sh + (ow * a.stride_w) * a.c0 + 4 * q;
#pragma unroll
    for (int to = 0; to < TO; ++to) {
      const int64_t oc = occ * TO + to;
      const int64_t oc_in = oc < a.OC ? oc : a.OC - 1;
      ok[tw][to] = wave_ok && px < pixels && oc < a.OC;
      po[tw][to] = out_base + n * a.out_sn + oc_in * a.out_soc + oh * a.out_soh + ow * 16 + 4 * q;
    }
  }
  // Loader lanes (waves 0..TO-1): wave `wave` copies channel block occ*TO+wave,
  // lane l the 16 bytes [ci = l / 4][ko = 4 * (l % 4) ..].
  const bool loader = wave < TO;
  const int64_t oc_ld = min(occ * TO + (loader ? wave : 0), a.OC - 1);
  const float* pf = a.flt + oc_ld * a.f_soc + ic0 * a.f_sic + lane * 4;
  const int f_dst = (loader ? wave : 0) * kFilterTile + (lane >> 2) * kFilterRow + (lane & 3) * 4;
  const int f_src = (4 * q) * kFilterRow + r;   // + to * kFilterTile + w * kFilterRow

  v4f acc[TW][TO];
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int to = 0; to < TO; ++to) {
      acc[tw][to] = v4f{0.f, 0.f, 0.f, 0.f};
      if (accumulate && ok[tw][to]) acc[tw][to] = *reinterpret_cast<const v4f_a4*>(po[tw][to]);
    }

  // Within one (ic_outer, fh) consecutive steps follow each other at 16 input
  // floats and 256 filter floats.
  const int64_t taps = a.FW * (a.c0 / 16);
  const int64_t steps = ic_count * a.FH * taps;
  if (steps > 0) {
    int64_t ic = 0, fh = 0, tap = 0;  // the step the next prefetch loads
    v4f av[2][TW];
    v4f fv = v4f{0.f, 0.f, 0.f, 0.f};
    auto prefetch = [&](auto buf) {
      constexpr int B = decltype(buf)::value;
      const int64_t ao = ic * a.in_sic + fh * a.in_sh + tap * 16;
      const int64_t bo = ic * a.f_sic + fh * a.f_sfh + tap * 256;
      // Every wave issues the filter load (the waves that do not stage it read
      // the first block's tile and drop it): one issue order on all paths
      // keeps the compiler's wait counts from covering the loads just issued.
      fv = *reinterpret_cast<const v4f_a4*>(pf + bo);
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) av[B][tw] = *reinterpret_cast<const v4f_a4*>(pa[tw] + ao);
      // Advance, staying on the last step once it is reached.
      if (!(ic == ic_count - 1 && fh == a.FH - 1 && tap == taps - 1)) {
        if (++tap == taps) {
          tap = 0;
          if (++fh == a.FH) {
            fh = 0;
            ++ic;
          }
        }
      }
    };
    auto stage_filter = [&](int b) {
      if (loader) *reinterpret_cast<v4f*>(&filt[b][f_dst]) = fv;
    };
    // Computes the step held in av[B] and filt[B]; meanwhile fetches the next
    // step into av[1 - B] and, through fv, filt[1 - B].
    auto iteration = [&](auto buf) {
      constexpr int B = decltype(buf)::value;
      prefetch(std::integral_constant<int, 1 - B>{});
      float bv[TO][4];
#pragma unroll
      for (int to = 0; to < TO; ++to)
#pragma unroll
        for (int w = 0; w < 4; ++w) bv[to][w] = filt[B][to * kFilterTile + w * kFilterRow + f_src];
#pragma unroll
      for (int w = 0; w < 4; ++w)
#pragma unroll
        for (int tw = 0; tw < TW; ++tw)
#pragma unroll
          for (int to = 0; to < TO; ++to)
            acc[tw][to] = __builtin_amdgcn_mfma_f32_16x16x4f32(bv[to][w], av[B][tw][w],
                                                               acc[tw][to], 0, 0, 0);
      stage_filter(1 - B);
      __syncthreads();
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    prefetch(B0{});
    stage_filter(0);
    __syncthreads();
    int64_t s = 0;
    for (; s + 1 < steps; s += 2) {
      iteration(B0{});
      iteration(B1{});
    }
    if (s < steps) iteration(B0{});
  }
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int to = 0; to < TO; ++to)
      if (ok[tw][to]) *reinterpret_cast<v4f_a4*>(po[tw][to]) = acc[tw][to];
}

// out = (ACCUMULATE ? out : 0) + slice 0 + slice 1 + ..., four channels per thread.
__global__ __launch_bounds__(kThreads) void conv_reduce_slices_kernel(ConvArgs a) {
  const int64_t quads = a.total / 4;   // k0 = 16: four quads per pixel
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < quads;
       idx += (int64_t)gridDim.x * kThreads) {
    int64_t t = idx;
    const int64_t q = t % 4; t /= 4;
    const int64_t ow = t % a.OW; t /= a.OW;
    const int64_t oh = t % a.OH; t /= a.OH;
    const int64_t oc = t % a.OC;
    const int64_t n = t / a.OC;
    const int64_t off = n * a.out_sn + oc * a.out_soc + oh * a.out_soh + ow * 16 + 4 * q;
    v4f sum = a.accumulate ? *reinterpret_cast<const v4f_a4*>(a.out + off) : v4f{0.f, 0.f, 0.f, 0.f};
    for (int32_t s = 0; s < a.ic_slices; ++s) {
      sum += *reinterpret_cast<const v4f_a4*>(a.partial + s * a.partial_stride + off);
    }
    *reinterpret_cast<v4f_a4*>(a.out + off) = sum;
  }
}

template <int TW, int TO>
int launch_mfma(const ConvArgs& a, int64_t N, hipStream_t stream) {
  const int64_t px_chunks = uk::ceil_div(a.OH * a.OW, (int64_t)16 * TW);
  const int64_t px_groups = uk::ceil_div(px_chunks, (int64_t)(kThreads / 64));
  const int64_t oc_chunks = uk::ceil_div(a.OC, (int64_t)TO);
  const int64_t blocks = N * oc_chunks * px_groups * a.ic_slices;
  if (blocks >= (1ll << 31)) return -1;
  uk::launch(3, conv_nchwc_mfma_kernel<TW, TO>, dim3((uint32_t)blocks), dim3(kThreads), 0, stream,
             a, px_chunks, px_groups, oc_chunks);
  if (a.ic_slices > 1) {
    const int64_t rblocks = uk::ceil_div(a.total / 4, (int64_t)kThreads);
    uk::launch(3, conv_reduce_slices_kernel, dim3((uint32_t)std::min<int64_t>(rblocks, 4096)), dim3(kThreads), 0,
               stream, a);
  }
  return (int)hipGetLastError();
}

// Workgroups a launch with TW panels and TO output-channel blocks per wave has.
int64_t mfma_blocks(const ConvArgs& a, int64_t N, int tw, int to) {
  const int64_t px_chunks = uk::ceil_div(a.OH * a.OW, (int64_t)16 * tw);
  return N * uk::ceil_div(a.OC, (int64_t)to) * uk::ceil_div(px_chunks, (int64_t)(kThreads / 64));
}

template <int TO>
int launch_mfma_for_pixels(const ConvArgs& a, int64_t N, hipStream_t stream, bool one_panel) {
  const int64_t pixels = a.OH * a.OW;
  // Two panels per wave: four measured no faster (608 against 583 us on a 3x3
  // 256 -> 256 channel layer at 56x56) and leave fewer, longer work items.
  if (pixels > 16 && !one_panel) return launch_mfma<2, TO>(a, N, stream);
  return launch_mfma<1, TO>(a, N, stream);
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
  a.N = p->N;
  a.ic_slices = 1;
  a.ic_per = p->IC_outer;
  a.partial = nullptr;
  a.partial_stride = 0;
  if (a.total == 0) {
    *kernel_name = "";
    return 0;
  }
  if (kernel_mode != IREE_UK_AMD_KERNEL_MODE_GENERIC &&
      iree_uk_amd_hip_conv_nchwc_has_mfma_kernel(p->k0, p->c0, p->flags)) {
    // Output-channel blocks per wave: four when that pads OC_outer no further
    // than two would (each input piece then meets four filter tiles: 583 -> 554
    // us on a 3x3 256 -> 256 channel layer at 56x56), else two, else one.
    const bool four = a.OC > 2 && uk::ceil_div(a.OC, (int64_t)4) * 4 == uk::ceil_div(a.OC, (int64_t)2) * 2;
    // A layer with few output pixels (the last stages of an image network at
    // batch 1: 512 -> 512 channels, 7x7 outputs) leaves most compute units
    // without a workgroup at those sizes: the wave's share shrinks, first in
    // output channels, then in pixels, until the workgroups outnumber the units
    // (8 -> 32 workgroups on that layer: 189 -> 72 us; 256 -> 256 channels at 56x56, batch 1: 97 -> 70 us).
    int to = four ? 4 : a.OC > 1 ? 2 : 1;
    int tw = a.OH * a.OW > 16 ? 2 : 1;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    }
    while (mfma_blocks(a, p->N, tw, to) < cus && (to > 1 || tw > 1)) {
      if (to > 1) to /= 2;
      else tw = 1;
    }
    // Still fewer workgroups than half the units: IC_outer is split over
    // several workgroups per output block, whose sums meet in a buffer the
    // library keeps and are added up in slice order by a second kernel (the
    // same result on every run; 512 -> 512 channels at 7x7, batch 1: 72 -> 17
    // us). While the stream is being captured into a graph there is no buffer
    // to be had, and the call runs unsplit.
    const int64_t blocks0 = mfma_blocks(a, p->N, tw, to);
    const int64_t steps_per_ic = a.FH * a.FW * (a.c0 / 16);
    if (blocks0 * 2 <= cus && a.IC >= 2 && a.out_sn >= 0 && a.out_soc >= 0 && a.out_soh >= 0) {
      int64_t slices = std::min<int64_t>(std::min<int64_t>(a.IC, cus / blocks0), 16);
      while (slices > 1 && uk::ceil_div(a.IC, slices) * steps_per_ic < 8) --slices;
      const int64_t ic_per = uk::ceil_div(a.IC, std::max<int64_t>(slices, 1));
      slices = uk::ceil_div(a.IC, ic_per);
      const int64_t span = (p->N - 1) * a.out_sn + (a.OC - 1) * a.out_soc + (a.OH - 1) * a.out_soh + a.OW * 16;
      char* ws = nullptr;
      if (slices > 1 && span * slices * 4 <= (64ll << 20) &&
          uk_mfma::acquire_expand_workspace((size_t)(span * slices * 4), stream, &ws) == 0) {
        a.ic_slices = (int32_t)slices;
        a.ic_per = ic_per;
        a.partial = (float*)ws;
        a.partial_stride = span;
      }
    }
    int st = to == 4   ? launch_mfma_for_pixels<4>(a, p->N, stream, tw == 1)
             : to == 2 ? launch_mfma_for_pixels<2>(a, p->N, stream, tw == 1)
                       : launch_mfma_for_pixels<1>(a, p->N, stream, tw == 1);
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
