// Host-side selection and launch of the MFMA mmt4d kernels for one element
// type. Included by one translation unit per element type so that the kernel
// instantiations compile in parallel.
#ifndef IREE_UK_AMD_MMT4D_MFMA_LAUNCH_H_
#define IREE_UK_AMD_MMT4D_MFMA_LAUNCH_H_

#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>

#include "mmt4d_mfma_kernel.h"
#include "mmt4d_mfma_narrow.h"
#include "mmt4d_mfma_persistent.h"
#include "mmt4d_mfma_thin.h"
#include "uk_device_common.h"
#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace uk_mfma {

// What the dispatcher hands to the per-type launcher: the problem in bytes.
struct Problem {
  const char* lhs;
  const char* rhs;
  char* out;
  int64_t lhs_stride, rhs_stride, out_stride;  // bytes between row panels
  // Output addressing beyond the panel stride (see Args in the kernel header):
  // bytes between rows inside a panel and between column panels, and how many
  // rows / columns exist counted from this problem's origin.
  int64_t out_sm0, out_spn;
  int64_t out_rows, out_cols;
  // Initial accumulators for ACCUMULATE, addressed like the output (the output
  // itself unless `dequant`), and the dequantizing store's scales, indexed
  // from this problem's origin (either may be null).
  const char* acc;
  int64_t acc_stride, acc_sm0, acc_spn;
  bool dequant;
  const float* row_scale;
  const float* col_scale;
  int32_t M1, N1, K1, M0, N0;
  int32_t rb, lrb;  // bytes per tile row and its log2
  bool accumulate;
};

// Launches one kernel variant over K-tiles [kt_begin, kt_begin + kt_count).
// Returns a HIP status, or -1 if the variant cannot serve the shape.
template <Elem E, int RBC, int TM, int TN, int WGM, int WGN, int NKK, int PIPE>
int launch_variant(const Problem& p, int kt_begin, int kt_count, bool accumulate,
                   hipStream_t stream) {
  using SH = Shape<E, TM, TN, WGM, WGN, NKK, PIPE>;
  constexpr int R = RBC >= 16 ? 1 : 16 / RBC;
  if (SH::kLdsBytes > 160 * 1024) return -1;          // more LDS than a compute unit has
  if (p.rb > SH::KS) return -1;                       // a tile row must fit one step
  if (p.M0 > SH::BM || p.N0 > SH::BN) return -1;      // at least one whole panel
  if (p.M0 % R || p.N0 % R) return -1;                // pieces hold whole rows
  if (p.out_rows <= 0 || p.out_cols <= 0) return 0;   // a strip beyond the matrix: nothing to store
  Args a{};
  const int64_t kt_bytes_m = (int64_t)p.M0 << p.lrb, kt_bytes_n = (int64_t)p.N0 << p.lrb;
  a.lhs = p.lhs + kt_begin * kt_bytes_m;
  a.rhs = p.rhs + kt_begin * kt_bytes_n;
  a.out = p.out;
  a.lhs_stride = p.lhs_stride;
  a.rhs_stride = p.rhs_stride;
  a.out_stride = p.out_stride;
  a.out_sm0 = (uint32_t)p.out_sm0;
  a.out_spn = (uint32_t)p.out_spn;
  a.out_rows = (int32_t)std::min<int64_t>(p.out_rows, INT32_MAX);
  a.out_cols = (int32_t)std::min<int64_t>(p.out_cols, INT32_MAX);
  a.M1 = p.M1; a.N1 = p.N1; a.K1 = kt_count;
  a.M0 = p.M0; a.N0 = p.N0; a.rb = p.rb; a.lrb = p.lrb;
  a.bpm = SH::BM / p.M0;
  a.bpn = SH::BN / p.N0;
  const int64_t grid_m = uk::ceil_div(p.M1, a.bpm), grid_n = uk::ceil_div(p.N1, a.bpn);
  if (grid_m * grid_n >= (1ll << 31)) return -1;
  a.grid_m = (int32_t)grid_m;
  a.grid_n = (int32_t)grid_n;
  const int64_t k_bytes = (int64_t)kt_count << p.lrb;
  a.steps = (int32_t)uk::ceil_div(k_bytes, SH::KS);
  if (a.steps < 1) a.steps = 1;
  a.tail = (k_bytes % SH::KS) != 0;
  if (PIPE != 0 && PIPE != 4 && (a.tail || kt_count == 0)) return -1;
  a.accumulate = accumulate;
  // A launch that starts K reads the caller's accumulators; a later one
  // continues from what the previous launch left in the output. Only the
  // launch that finishes K applies the dequantizing store.
  const bool first = kt_begin == 0;
  a.acc = first ? p.acc : p.out;
  a.acc_stride = first ? p.acc_stride : p.out_stride;
  a.acc_sm0 = (uint32_t)(first ? p.acc_sm0 : p.out_sm0);
  a.acc_spn = (uint32_t)(first ? p.acc_spn : p.out_spn);
  a.dequant = p.dequant && kt_begin + kt_count == p.K1;
  a.row_scale = p.row_scale;
  a.col_scale = p.col_scale;
  // Block rows per rasterization band: an XCD's 32 resident workgroups should
  // cover a near-square patch of the output (4 x 8 blocks of 256x256, 8 x 4 of
  // 128x512: 3072 operand rows either way).
  a.band = (WGM == 1 && WGN == 8) ? 8 : 4;
  // Four consecutive output columns of one row are contiguous when they lie in
  // one tile row (N0 % 4 == 0) or when column panels follow each other without
  // a gap (row-major output, or tiles that are single rows). 4-byte outputs
  // need no more alignment than their own; 2-byte outputs move as 8-byte
  // vectors and need that alignment.
  constexpr int OB = ElemTraits<E>::Out::kOutBytes;
  auto vector_ok = [&](const char* base, int64_t stride, int64_t sm0, int64_t spn) {
    const bool contiguous4 = p.N0 % 4 == 0 || spn == (int64_t)p.N0 * OB;
    const bool aligned4 = OB == 4 || (((uintptr_t)base | (uint64_t)stride | (uint64_t)sm0 |
                                       (uint64_t)spn) % 8) == 0;
    return contiguous4 && aligned4;
  };
  a.vec_out = vector_ok(p.out, p.out_stride, p.out_sm0, p.out_spn) &&
              (!accumulate || vector_ok(a.acc, a.acc_stride, a.acc_sm0, a.acc_spn));
  // The launch that finishes K stores non-temporally when the output is
  // larger than the memory-side cache can hand to its reader.
  a.nt_out = kt_begin + kt_count == p.K1 &&
             (int64_t)p.M1 * p.M0 * p.N1 * p.N0 * OB >= (192ll << 20);
  // 32-bit offsets inside a workgroup's share of each operand.
  const int64_t span_m = (int64_t)a.bpm * p.lhs_stride + (int64_t)p.K1 * kt_bytes_m;
  const int64_t span_n = (int64_t)a.bpn * p.rhs_stride + (int64_t)p.K1 * kt_bytes_n;
  const int64_t span_o = (int64_t)a.bpm * p.out_stride + (int64_t)p.M0 * p.out_sm0 +
                         (int64_t)p.N1 * p.out_spn;
  const int64_t span_a = (int64_t)a.bpm * a.acc_stride + (int64_t)p.M0 * a.acc_sm0 +
                         (int64_t)p.N1 * a.acc_spn;
  if (span_m >= (1ll << 31) || span_n >= (1ll << 31) || span_o >= (1ll << 31) ||
      span_a >= (1ll << 31)) {
    return -1;
  }
  auto kernel = mmt4d_mfma_kernel<E, RBC, TM, TN, WGM, WGN, NKK, PIPE>;
  if (SH::kLdsBytes > 64 * 1024) {
    // Raising the dynamic LDS limit is a per-function setting; do it once.
    static hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
        (int)SH::kLdsBytes);
    if (attr != hipSuccess) return (int)attr;
  }
  uk::launch(2, kernel, dim3((uint32_t)(grid_m * grid_n)), dim3(WGM * WGN * 64),
             SH::kLdsBytes, stream, a);
  return (int)hipGetLastError();
}

// Workspace of the thin kernel's K split over workgroups: `partial_bytes` of
// partial accumulators and `n_counters` arrival counters that are zero
// between launches. Defined in mmt4d_mfma.hip: ordinary calls get a buffer
// the library allocates per host thread and stream (grow-only; none while the
// stream is being captured into a graph and nothing fits yet), calls through
// iree_uk_amd_mmt4d_no_alloc get the library's static device array. Returns 0
// and the pointers, 1 when there is no workspace but the call can run without
// the split, or a status (> 1) that has to fail the call.
struct KSplitWorkspace {
  char* partials;
  uint32_t* counters;
};
int acquire_ksplit_workspace(size_t partial_bytes, uint32_t n_counters, hipStream_t stream,
                             KSplitWorkspace* ws);
// A buffer of `bytes` for s4 weights expanded to s8 (mmt4d_mfma_s8s4.hip), kept
// per host thread and stream like the K split's workspace and apart from it
// (the s8 launch that reads the expanded weights may itself split K). Returns
// 0 and the pointer, or 1 when there is none to be had: under
// iree_uk_amd_mmt4d_no_alloc, while the stream is being captured into a graph,
// or when the allocation fails.
int acquire_expand_workspace(size_t bytes, hipStream_t stream, char** base);
// Regroups the K tiles of an operand so that every tile row holds 16 bytes:
// `panels` panels of K1 tiles of R0 rows of `rb` bytes (rb = 1, 2, 4 or 8; panel
// n at src + n * src_stride) become ceil(K1 * rb / 16) tiles of R0 rows of 16
// bytes at dst + n * (that count * R0 * 16), the last one filled up with zero
// bytes. src_bits = 4: the source holds signed nibbles, low nibble first, half
// as many bytes, and `rb` counts the bytes they widen to. dst 16-byte aligned.
void retile_rows(const char* src, int64_t src_stride, int panels, int R0, int rb, int K1, int src_bits,
                 char* dst, hipStream_t stream);
// K slices set with iree_uk_amd_set_k_slices on this thread; 0 = choose.
int k_slices_override();
// 1: the calling thread has declared its weights streamed from HBM
// (iree_uk_amd_set_streamed_weights).
int streamed_weights();
// Records the slice count of the launch for iree_uk_amd_last_k_slices.
void note_k_slices(int n);

// Workgroup count set with iree_uk_amd_set_persistent_workgroups on this
// thread; 0 = one per compute unit (defined in mmt4d_mfma.hip).
int persistent_workgroups_override();

// Compute units of the current device (one persistent workgroup each).
inline int compute_units() {
  static thread_local int cached_device = -1, cached_cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_device) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached_device = dev;
    cached_cus = cus;
  }
  return cached_cus;
}

// Launches the persistent kernel (mmt4d_mfma_persistent.h) over K-tiles
// [0, kt_count): one workgroup per CU, each walking several output blocks
// without draining its pipeline in between. Returns a HIP status, or -1 if
// the kernel cannot serve the shape (or would not gain: fewer than two blocks
// per workgroup).
template <Elem E, int TM, int TN, int WGM, int WGN>
int launch_persistent(const Problem& p, int kt_count, bool force, hipStream_t stream) {
  constexpr int BM = WGM * TM * 16, BN = WGN * TN * 16, KS = 64;
  auto pow2 = [](int v) { return v > 0 && (v & (v - 1)) == 0; };
  if (p.rb < 16 || p.rb > KS) return -1;
  if (!pow2(p.M0) || !pow2(p.N0) || p.N0 < 4 || p.M0 > BM || p.N0 > BN) return -1;
  if (p.dequant) return -1;
  const int bpm = BM / p.M0, bpn = BN / p.N0;
  if (p.M1 % bpm || p.N1 % bpn) return -1;
  if (p.out_rows < (int64_t)p.M1 * p.M0 || p.out_cols < (int64_t)p.N1 * p.N0) return -1;
  const int64_t k_bytes = (int64_t)kt_count << p.lrb;
  if (k_bytes % (4 * KS) || k_bytes / KS < 8 || k_bytes / KS >= (1 << 24)) return -1;
  const int64_t grid_m = p.M1 / bpm, grid_n = p.N1 / bpn;
  const int64_t total = grid_m * grid_n;
  int cus = compute_units() & ~7;  // a multiple of the 8 XCDs keeps blocks on their XCD
  if (persistent_workgroups_override() > 0) cus = persistent_workgroups_override();
  if (cus < 1 || total >= (1ll << 30)) return -1;
  if (!force && total < 2 * (int64_t)cus) return -1;
  const int64_t grid = std::min<int64_t>(total, cus);
  Args a{};
  a.lhs = p.lhs; a.rhs = p.rhs; a.out = p.out;
  a.lhs_stride = p.lhs_stride; a.rhs_stride = p.rhs_stride; a.out_stride = p.out_stride;
  a.out_sm0 = (uint32_t)p.out_sm0; a.out_spn = (uint32_t)p.out_spn;
  a.out_rows = (int32_t)std::min<int64_t>(p.out_rows, INT32_MAX);
  a.out_cols = (int32_t)std::min<int64_t>(p.out_cols, INT32_MAX);
  a.M1 = p.M1; a.N1 = p.N1; a.K1 = kt_count;
  a.M0 = p.M0; a.N0 = p.N0; a.rb = p.rb; a.lrb = p.lrb;
  a.bpm = bpm; a.bpn = bpn;
  a.grid_m = (int32_t)grid_m; a.grid_n = (int32_t)grid_n;
  a.steps = (int32_t)(k_bytes / KS);
  a.accumulate = p.accumulate;
  a.band = (WGM == 1 && WGN == 8) ? 8 : 4;
  a.vec_out = 1;
  a.acc = p.acc; a.acc_stride = p.acc_stride;
  a.acc_sm0 = (uint32_t)p.acc_sm0; a.acc_spn = (uint32_t)p.acc_spn;
  while ((1 << a.lm0) < p.M0) ++a.lm0;
  while ((1 << a.ln0) < p.N0) ++a.ln0;
  const int64_t kt_bytes_m = (int64_t)p.M0 << p.lrb, kt_bytes_n = (int64_t)p.N0 << p.lrb;
  const int64_t span_m = (int64_t)bpm * p.lhs_stride + (int64_t)p.K1 * kt_bytes_m;
  const int64_t span_n = (int64_t)bpn * p.rhs_stride + (int64_t)p.K1 * kt_bytes_n;
  const int64_t span_o = (int64_t)bpm * p.out_stride + (int64_t)p.M0 * p.out_sm0 +
                         (int64_t)p.N1 * p.out_spn;
  const int64_t span_a = (int64_t)bpm * p.acc_stride + (int64_t)p.M0 * p.acc_sm0 +
                         (int64_t)p.N1 * p.acc_spn;
  if (span_m >= (1ll << 31) || span_n >= (1ll << 31) || span_o >= (1ll << 31) ||
      span_a >= (1ll << 31)) {
    return -1;
  }
  constexpr size_t kLds = 4 * (size_t)BM * KS;
  auto kernel = mmt4d_mfma_persistent_kernel<E, TM, TN, WGM, WGN>;
  uk::launch(2, kernel, dim3((uint32_t)grid), dim3(WGM * WGN * 64), kLds, stream, a);
  return (int)hipGetLastError();
}

// Launches the narrow-row kernel (mmt4d_mfma_narrow.h: tile rows of 2 or 4
// bytes, N0 = 16, RHS fragments loaded straight into registers) over K-tiles
// [0, kt_count). Returns a HIP status, or -1 if it cannot serve the shape.
template <Elem E, int RBC, int TM, int WGM, int WGN>
int launch_narrow(const Problem& p, int kt_count, hipStream_t stream) {
  constexpr int BM = WGM * TM * 16, BN = WGN * 64, KS = 64;
  if (p.rb != RBC || p.N0 != 16 || p.M0 % (16 / RBC) || p.M0 > BM || BM % p.M0) return -1;
  if (p.dequant) return -1;
  if (p.out_rows <= 0 || p.out_cols <= 0) return 0;
  if (p.out_cols < (int64_t)p.N1 * p.N0) return -1;   // a row-major matrix narrower than the tiles
  const int64_t k_bytes = (int64_t)kt_count << p.lrb;
  if (kt_count <= 0 || k_bytes % KS) return -1;
  Args a{};
  a.lhs = p.lhs; a.rhs = p.rhs; a.out = p.out;
  a.lhs_stride = p.lhs_stride; a.rhs_stride = p.rhs_stride; a.out_stride = p.out_stride;
  a.out_sm0 = (uint32_t)p.out_sm0; a.out_spn = (uint32_t)p.out_spn;
  a.out_rows = (int32_t)std::min<int64_t>(p.out_rows, INT32_MAX);
  a.out_cols = (int32_t)std::min<int64_t>(p.out_cols, INT32_MAX);
  a.M1 = p.M1; a.N1 = p.N1; a.K1 = kt_count;
  a.M0 = p.M0; a.N0 = p.N0; a.rb = p.rb; a.lrb = p.lrb;
  a.bpm = BM / p.M0; a.bpn = BN / p.N0;
  const int64_t grid_m = uk::ceil_div(p.M1, a.bpm), grid_n = uk::ceil_div(p.N1, a.bpn);
  if (grid_m * grid_n >= (1ll << 31)) return -1;
  a.grid_m = (int32_t)grid_m; a.grid_n = (int32_t)grid_n;
  a.steps = (int32_t)(k_bytes / KS);
  a.accumulate = p.accumulate;
  a.band = (WGM == 1 && WGN == 8) ? 8 : 4;
  a.vec_out = 1;
  a.acc = p.acc; a.acc_stride = p.acc_stride;
  a.acc_sm0 = (uint32_t)p.acc_sm0; a.acc_spn = (uint32_t)p.acc_spn;
  const int64_t kt_bytes_m = (int64_t)p.M0 << p.lrb, kt_bytes_n = (int64_t)p.N0 << p.lrb;
  const int64_t span_m = (int64_t)a.bpm * p.lhs_stride + (int64_t)p.K1 * kt_bytes_m;
  const int64_t span_n = (int64_t)a.bpn * p.rhs_stride + (int64_t)p.K1 * kt_bytes_n;
  const int64_t span_o = (int64_t)a.bpm * p.out_stride + (int64_t)p.M0 * p.out_sm0 +
                         (int64_t)p.N1 * p.out_spn;
  const int64_t span_a = (int64_t)a.bpm * p.acc_stride + (int64_t)p.M0 * p.acc_sm0 +
                         (int64_t)p.N1 * p.acc_spn;
  if (span_m >= (1ll << 31) || span_n >= (1ll << 31) || span_o >= (1ll << 31) ||
      span_a >= (1ll << 31)) {
    return -1;
  }
  constexpr size_t kLds = 3 * (size_t)BM * KS;
  uk::launch(2, mmt4d_mfma_narrow_kernel<E, RBC, TM, WGM, WGN>, dim3((uint32_t)(grid_m * grid_n)),
             dim3(WGM * WGN * 64), kLds, stream, a);
  return (int)hipGetLastError();
}

// Launches the M-thin kernel (mmt4d_mfma_thin.h) over all of K. Returns a HIP
// status, or -1 if it cannot serve the shape.
// `swapped`: the caller's problem is N-thin and is computed as its transpose
// (out^T = rhs * lhs^T): the kernel's rows are the caller's columns.
template <Elem E, int RBC, int TM, int TN, int KSPLIT, int D>
int launch_thin(const Problem& caller, bool swapped, hipStream_t stream, bool allow_k_slices = false,
                int max_k_slices = 8) {
  constexpr int OBYTES = ElemTraits<E>::Out::kOutBytes;
  Problem p = caller;
  if (swapped) {
    std::swap(p.lhs, p.rhs);
    std::swap(p.lhs_stride, p.rhs_stride);
    std::swap(p.M1, p.N1);
    std::swap(p.M0, p.N0);
    std::swap(p.out_rows, p.out_cols);
    std::swap(p.row_scale, p.col_scale);
    // Element (row i, col j) of the caller sits at
    //   (i / M0) * stride + (i % M0) * sm0 + (j / N0) * spn + (j % N0) * elem;
    // the kernel's row is j and its column is i.
    std::swap(p.out_stride, p.out_spn);
    std::swap(p.acc_stride, p.acc_spn);
  }
  constexpr int KS = 64 * ElemTraits<E>::kHalves;
  constexpr int OB = OBYTES;
  constexpr bool S4 = E == Elem::kS8S4;  // rb, lrb describe the LHS; RHS rows are half as wide
  if (p.rb > KS || p.rb < (S4 ? 16 : 8)) return -1;
  const int64_t k_bytes = (int64_t)p.K1 << p.lrb;
  if (k_bytes == 0 || k_bytes % KS) return -1;
  // 4-bit RHS: the accumulators hold 16 * sum; |sum| <= K * 128 * 8 must stay
  // below 2^27 for that to be exact.
  if (S4 && k_bytes >= 131072) return -1;
  if (p.out_rows <= 0 || p.out_cols <= 0) return 0;
  Args a{};
  a.lhs = p.lhs; a.rhs = p.rhs; a.out = p.out;
  a.lhs_stride = p.lhs_stride; a.rhs_stride = p.rhs_stride; a.out_stride = p.out_stride;
  a.out_sm0 = (uint32_t)(swapped ? OBYTES : p.out_sm0);
  a.out_sn0 = (uint32_t)(swapped ? p.out_sm0 : OBYTES);
  a.out_spn = (uint32_t)p.out_spn;
  a.out_rows = (int32_t)std::min<int64_t>(p.out_rows, INT32_MAX);
  a.out_cols = (int32_t)std::min<int64_t>(p.out_cols, INT32_MAX);
  a.M1 = p.M1; a.N1 = p.N1; a.K1 = p.K1; a.M0 = p.M0; a.N0 = p.N0; a.rb = p.rb; a.lrb = p.lrb;
  // Rows and columns that are stored: blocks wholly beyond them (tile padding of
  // a fused row-major result) are not computed at all.
  const int64_t grid_m = uk::ceil_div(std::min<int64_t>((int64_t)p.M1 * p.M0, p.out_rows), TM * 16);
  const int64_t grid_n = uk::ceil_div(std::min<int64_t>((int64_t)p.N1 * p.N0, p.out_cols), TN * 16);
  if (grid_m * grid_n >= (1ll << 31) || p.out_sm0 >= (1ll << 32) || p.out_spn >= (1ll << 32) ||
      p.acc_sm0 >= (1ll << 32) || p.acc_spn >= (1ll << 32)) {
    return -1;
  }
  a.grid_m = (int32_t)grid_m;
  a.grid_n = (int32_t)grid_n;
  a.steps = (int32_t)(k_bytes / KS);
  a.accumulate = p.accumulate;
  a.acc = p.acc; a.acc_stride = p.acc_stride;
  a.acc_sm0 = (uint32_t)(swapped ? OBYTES : p.acc_sm0);
  a.acc_sn0 = (uint32_t)(swapped ? p.acc_sm0 : OBYTES);
  a.acc_spn = (uint32_t)p.acc_spn;
  a.dequant = p.dequant; a.row_scale = p.row_scale; a.col_scale = p.col_scale;
  a.col_scale_first = swapped;
  auto vector_ok = [&](const char* base, int64_t stride, int64_t sm0, int64_t spn) {
    const bool contiguous4 = p.N0 % 4 == 0 || spn == (int64_t)p.N0 * OB;
    const bool aligned4 = OB == 4 || (((uintptr_t)base | (uint64_t)stride | (uint64_t)sm0 |
                                       (uint64_t)spn) % 8) == 0;
    return contiguous4 && aligned4;
  };
  a.vec_out = !swapped && vector_ok(p.out, p.out_stride, p.out_sm0, p.out_spn) &&
              (!p.accumulate || vector_ok(p.acc, p.acc_stride, p.acc_sm0, p.acc_spn));
  // 32-bit operand offsets inside a workgroup's panels.
  const int64_t span_m = (int64_t)(TM * 16 / p.M0 + 2) * p.lhs_stride + k_bytes * p.M0;
  const int64_t span_n =
      (int64_t)(TN * 16 / p.N0 + 2) * p.rhs_stride + k_bytes * p.N0 / (S4 ? 2 : 1);
  if (span_m >= (1ll << 31) || span_n >= (1ll << 31)) return -1;
  // Still too few output blocks for the chip, and a long K: split K over
  // workgroups as well, aiming at one workgroup per compute unit, each wave
  // keeping at least four steps. The split costs a few microseconds at the end
  // of the launch (the slices meet through device-scope accesses, three
  // dependent round trips to where the XCDs meet), so it has to at least halve
  // the streaming time to pay.
  int64_t kslices = 1;
  if (allow_k_slices) {
    const int64_t blocks = grid_m * grid_n;
    const int cus = compute_units();
    if (k_slices_override() > 0) {
      kslices = k_slices_override();
    } else if (cus > 0 && 2 * blocks <= cus) {
      kslices = std::min<int64_t>(max_k_slices, cus / blocks);
    }
    kslices = std::max<int64_t>(1, std::min<int64_t>(kslices, a.steps / (4 * KSPLIT)));
    if (blocks * kslices >= (1ll << 31)) kslices = 1;
  }
  if (kslices > 1) {
    KSplitWorkspace ws{};
    const int got = acquire_ksplit_workspace((size_t)(grid_m * grid_n * kslices) * TM * TN * 1024,
                                             (uint32_t)(grid_m * grid_n), stream, &ws);
    if (got > 1) return got;
    if (got == 0) {
      a.kslices = (uint32_t)kslices;
      a.ws_partials = ws.partials;
      a.ws_counters = ws.counters;
      note_k_slices((int)kslices);
    } else {
      kslices = 1;
    }
  }
  // Weights that the caller has declared streamed, when they are too large for
  // the L2s anyway: loaded non-temporally.
  if (streamed_weights() && (int64_t)p.N1 * p.N0 * k_bytes / (S4 ? 2 : 1) >= (16ll << 20)) {
    uk::launch(2, mmt4d_thin_kernel<E, RBC, TM, TN, KSPLIT, D, true>,
               dim3((uint32_t)(grid_m * grid_n * kslices)), dim3(KSPLIT * 64), 0, stream, a);
    return (int)hipGetLastError();
  }
  uk::launch(2, mmt4d_thin_kernel<E, RBC, TM, TN, KSPLIT, D>,
             dim3((uint32_t)(grid_m * grid_n * kslices)), dim3(KSPLIT * 64), 0, stream, a);
  return (int)hipGetLastError();
}

// Status of the second, accumulating launch over the remainder of K. The
// first launch has already written the output: "not served" (negative) must
// not reach the dispatcher, which would recompute the whole problem on the
// scalar kernel on top of it.
inline int finish_k(int st) { return st < 0 ? (int)hipErrorUnknown : st; }

// Number of workgroups a BM x BN blocking gives for the problem.
inline int64_t workgroups(const Problem& p, int BM, int BN) {
  const int bpm = BM / p.M0, bpn = BN / p.N0;
  if (bpm < 1 || bpn < 1) return 0;
  return uk::ceil_div(p.M1, bpm) * uk::ceil_div(p.N1, bpn);
}

// Variant choice for row-bytes class RBC:
//   big   256x256 workgroup tile, 8 waves of 128x64, software-pipelined
//         (register-direct RHS when RB >= 16): needs K in whole steps, the
//         remainder of K (if any) is a second, accumulating launch;
//   mid   128x128, 4 waves, any K;
//   small 64x64, 4 waves, any K: for problems with too few 128x128 blocks to
//         occupy the 256 CUs;
// `forced` (1 big, 2 mid, 3 small, 4 thin, 5 thin on the transposed problem,
// 6 the 64x64 K-split kernel, 7 the 256x128 shape, 8 the 128x512 shape,
// 9 / 10 the persistent kernel in the 128x512 / 256x256 shape, 11 the 64x64
// shape with 256-byte steps three steps ahead (tile rows under 16 bytes),
// 12 .. 15 the narrow-row kernel (tile rows of 2 or 4 bytes, N0 = 16) in the
// 256x256 / 128x512 / 128x128 / 64x64 shape, 16 / 17 / 18 / 19 the LDS-direct
// ping-pong pipeline in the 256x256 / 128x512 / 128x128 / 64x64 shape;
// 0 = choose) overrides the
// size heuristic for tests and tuning.
//   thin  M-thin (decode-shaped) problems, up to 64 rows, which are bound by
//         streaming the RHS: the barrier-free kernel of mmt4d_mfma_thin.h (16,
//         32 or 64 rows x 32 columns per workgroup, K split over its 4 waves)
//         when rows are at least 8 bytes wide and K is a whole number of
//         steps, else 32 rows x 64 columns through LDS with loads three steps
//         ahead.
template <Elem E, int RBC>
int launch_class(const Problem& p, int forced, hipStream_t stream, const char** name) {
  constexpr int H = ElemTraits<E>::kHalves;
  constexpr int NKK2 = 2 / H;             // 128 bytes of K per step
  // Three RHS fragment buffers fit the register file only with one fragment
  // register quad per block (all types but f8).
  constexpr int BIG_PIPE = RBC >= 16 ? (ElemTraits<E>::kHalves == 1 ? 3 : 2) : 1;
  constexpr int BIG_KS = 64 * H;
  // Rows / columns that exist in the result (fewer than the tiles hold when a
  // fused call drops tile padding: a decode step of 16 rows in 32-row tiles).
  const int64_t rows_m = std::min<int64_t>((int64_t)p.M1 * p.M0, p.out_rows);
  const int64_t cols_n = std::min<int64_t>((int64_t)p.N1 * p.N0, p.out_cols);
  int choice;
  if (forced == 11 || forced == 15) {
    choice = 3;  // 64x64: the deep pipeline (11) or the narrow-row kernel (15)
  } else if (forced == 12 || forced == 13) {
    choice = 1;  // the narrow-row kernel in the 256x256 (12) or 128x512 (13) shape
  } else if (forced == 14) {
    choice = 2;  // the narrow-row kernel in the 128x128 shape
  } else if (forced == 16 || forced == 17) {
    choice = 1;  // the LDS-direct ping-pong pipeline in the 256x256 (16) or 128x512 (17) shape
  } else if (forced == 20) {
    choice = 7;  // the same pipeline in the 256x128 shape
  } else if (forced == 18) {
    choice = 2;  // the same pipeline in the 128x128 shape
  } else if (forced == 19) {
    choice = 3;  // and in the 64x64 shape with 256-byte steps
  } else if (forced >= 8 && forced <= 10) {
    // The big variant in its 128x512 shape (8), the persistent kernel in that
    // shape (9) or in the square one (10); the plain square shape where the
    // requested one cannot serve.
    choice = 1;
  } else if (forced >= 1 && forced <= 7) {
    choice = forced;
  } else if (rows_m <= (RBC >= 8 ? 64 : 32) && workgroups(p, 32, 64) >= 1) {
    choice = 4;
  } else if (RBC >= 8 && cols_n <= 64) {
    choice = 5;
  } else if (workgroups(p, 256, 256) >= 192) {
    choice = 1;
  } else if (RBC >= 16 && workgroups(p, 256, 128) >= 192 && workgroups(p, 256, 128) <= 256) {
    // One round of 256x128 blocks (measured 5-7 % ahead of 128x128 there).
    choice = 7;
  } else if (workgroups(p, 128, 128) >= 192) {
    choice = 2;
  } else if (RBC >= 8 && ((int64_t)p.K1 << p.lrb) >= 8192) {
    // Measured: with 8 KiB of K per row and more, the 64x64 blocks' operands
    // outgrow the L2 and the K-split kernel's deeper queue of loads wins.
    choice = 6;
  } else {
    choice = 3;
  }
  if (choice == 1 && forced == 0) {
    // Tile quantization: a last row or column of 256x256 workgroups that is
    // mostly padding can cost a whole extra round on the 256 CUs. Compare, in
    // units of one round of big tiles, keeping it in the big launch against
    // splitting it off as a strip that the smaller variants compute (at
    // roughly 0.45 of the big variant's rate, and never faster than about a
    // quarter round: their K loop is as long).
    const int bpm = 256 / p.M0, bpn = 256 / p.N0;
    const int64_t gm_c = uk::ceil_div(p.M1, bpm), gn_c = uk::ceil_div(p.N1, bpn);
    const int64_t gm_f = p.M1 / bpm, gn_f = p.N1 / bpn;
    auto rounds = [](int64_t wgs) { return (double)uk::ceil_div(wgs, 256); };
    auto strip_cost = [&](int64_t panels_m, int64_t panels_n) {
      const double tiles = (double)(panels_m * p.M0) * (double)(panels_n * p.N0) / 65536.0;
      return std::max(0.25, tiles / 256.0 / 0.45);
    };
    double best = rounds(gm_c * gn_c);
    int split_m = 0, split_n = 0;
    for (int fm = 0; fm < 2; ++fm) {
      for (int fn = 0; fn < 2; ++fn) {
        if (!fm && !fn) continue;
        if (fm && (gm_f == 0 || gm_f == gm_c)) continue;
        if (fn && (gn_f == 0 || gn_f == gn_c)) continue;
        const int64_t gm = fm ? gm_f : gm_c, gn = fn ? gn_f : gn_c;
        double cost = rounds(gm * gn);
        const int64_t main_n = fn ? gn_f * bpn : p.N1;
        if (fn) cost += strip_cost(p.M1, p.N1 - main_n);
        if (fm) cost += strip_cost(p.M1 - gm_f * bpm, main_n);
        if (cost < best - 0.1) { best = cost; split_m = fm; split_n = fn; }
      }
    }
    int32_t main_m = split_m ? (int32_t)(gm_f * bpm) : p.M1;
    int32_t main_n = split_n ? (int32_t)(gn_f * bpn) : p.N1;
    if constexpr (RBC >= 16) {
      // Round quantization of the 128x512 shape: a problem it tiles exactly
      // whose last round of blocks fills at most half of the compute units
      // runs those block columns as a launch of their own, which then takes a
      // smaller shape that occupies every unit (f8 2048 x 28672 x 8192, 3.5
      // rounds: 392-399 us as one launch, 313 us for three rounds + 62 us for
      // the last 4096 columns in 256x128 blocks).
      const int bpm_w = 128 / p.M0, bpn_w = 512 / p.N0;
      if (!split_m && !split_n && bpm_w >= 1 && bpn_w >= 1 && p.M1 % bpm_w == 0 && p.N1 % bpn_w == 0) {
        const int64_t gm = p.M1 / bpm_w, gn = p.N1 / bpn_w, cus = compute_units();
        const int64_t rem = cus > 0 ? (gm * gn) % cus : 0;
        if (gm * gn > cus && rem > 0 && 2 * rem <= cus && rem % gm == 0) {
          split_n = 1;
          main_n = (int32_t)((gn - rem / gm) * bpn_w);
        }
      }
    }
    if (split_m || split_n) {
      Problem q = p;
      q.M1 = main_m;
      q.N1 = main_n;
      int st = launch_class<E, RBC>(q, 0, stream, name);
      if (st != 0) return st;
      const char* strip_name = nullptr;
      if (split_n) {  // columns [main_n, N1), all rows
        q = p;
        q.rhs = p.rhs + (int64_t)main_n * p.rhs_stride;
        q.out = p.out + (int64_t)main_n * p.out_spn;
        q.acc = p.acc + (int64_t)main_n * p.acc_spn;
        if (p.col_scale) q.col_scale = p.col_scale + (int64_t)main_n * p.N0;
        q.out_cols = p.out_cols - (int64_t)main_n * p.N0;
        q.N1 = p.N1 - main_n;
        st = launch_class<E, RBC>(q, 0, stream, &strip_name);
        // The main part has run: "not served" must not reach the caller, who
        // would recompute (and with ACCUMULATE, re-add) the whole problem.
        if (st != 0) return st < 0 ? (int)hipErrorUnknown : st;
      }
      if (split_m) {  // rows [main_m, M1), columns [0, main_n)
        q = p;
        q.lhs = p.lhs + (int64_t)main_m * p.lhs_stride;
        q.out = p.out + (int64_t)main_m * p.out_stride;
        q.acc = p.acc + (int64_t)main_m * p.acc_stride;
        if (p.row_scale) q.row_scale = p.row_scale + (int64_t)main_m * p.M0;
        q.out_rows = p.out_rows - (int64_t)main_m * p.M0;
        q.M1 = p.M1 - main_m;
        q.N1 = main_n;
        st = launch_class<E, RBC>(q, 0, stream, &strip_name);
        if (st != 0) return st < 0 ? (int)hipErrorUnknown : st;
      }
      return 0;
    }
  }
  // Whole pipeline steps of K go to a software-pipelined variant; what is left
  // of K (less than one step) to the two-stage variant of the same or a
  // smaller workgroup shape, as a second, accumulating launch.
  const int kts_per_step = BIG_KS >> p.lrb;
  // 16-bit outputs are rounded once, after all of K (the reference's
  // SKIP_INTERMEDIATE_ROUNDINGS semantics): a second launch would continue from
  // a rounded value. With a K remainder they take the variants that run any K
  // in one launch.
  constexpr bool kOneLaunchOnly = ElemTraits<E>::Out::kOutBytes == 2;
  int kt_main = kts_per_step > 0 ? (p.K1 / kts_per_step) * kts_per_step : 0;
  if (kOneLaunchOnly && kt_main != p.K1) kt_main = 0;
  constexpr bool NARROW = (RBC == 2 || RBC == 4) && H == 1 && ElemTraits<E>::Out::kOutBytes == 4;
  if (choice == 1) {
    if constexpr (RBC < 16 && H == 1) {
      // Tile rows of 2, 4 or 8 bytes through the LDS-direct ping-pong pipeline
      // (PIPE 5 of mmt4d_mfma_kernel.h: the loads copy the K-tiles as they lie
      // in memory, the fragment reads gather each row's pieces).
      // Measured against the register-regrouping kernels at 8192^3: s8 16x16x2
      // 496 -> 382 us, bf16 16x16x2 932 -> 726 us, s8 16x16x8 486 -> 383 us; at
      // 4096^3 s8 16x16x2 76 -> 57 us. (f32 keeps its kernels, as below.)
      if (kt_main > 0 && (forced == 16 || forced == 17 || (forced == 0 && E != Elem::kF32))) {
        int st = -1;
        if (forced == 17) {
          st = launch_variant<E, RBC, 8, 4, 1, 8, 1, 5>(p, 0, kt_main, p.accumulate, stream);
          if (st == 0) *name = "mmt4d_mfma_128x512_lds_direct";
        }
        if (st < 0) {
          st = launch_variant<E, RBC, 8, 4, 2, 4, 1, 5>(p, 0, kt_main, p.accumulate, stream);
          if (st == 0) *name = "mmt4d_mfma_256x256_lds_direct";
        }
        if (st == 0) {
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
    }
    if constexpr (NARROW) {
      // Tile rows of 2 or 4 bytes with N0 = 16 (the x86-style tiles): the RHS
      // goes straight to registers here too (mmt4d_mfma_narrow.h).
      // Measured: at 8192^3 (four rounds of blocks) it is ahead of the kernel
      // with both operands through LDS (s8 16x16x2: 540 us against 558 us,
      // bf16 16x16x2: 880 us against 955 us), at 4096^3 (one round) behind it
      // (76 us against 69 us, 122 us against 117 us), so it is chosen from two
      // rounds on. The square shape is the faster one for 2-byte rows (540 us
      // against 567 us) and equal to the wide one for 4-byte rows, so the wide
      // shape is taken only when asked for.
      if (kt_main > 0 && ((forced == 0 && workgroups(p, 256, 256) >= 512) || forced == 12 || forced == 13)) {
        int st = -1;
        const char* nm = "";
        if (forced == 13) {
          st = launch_narrow<E, RBC, 8, 1, 8>(p, kt_main, stream);
          nm = "mmt4d_mfma_128x512_narrow";
        }
        if (st < 0 && forced != 13) {
          st = launch_narrow<E, RBC, 8, 2, 4>(p, kt_main, stream);
          nm = "mmt4d_mfma_256x256_narrow";
        }
        if (st == 0) {
          *name = nm;
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
    }
    if (kt_main > 0) {
      int st = -1;
      bool wide = false;
      if constexpr (RBC >= 16 && H == 1 && ElemTraits<E>::Out::kOutBytes == 4) {
        // One persistent workgroup per CU whose pipeline runs across block
        // boundaries. Measured equal to the one-block-per-workgroup launches
        // below (s8 8192^3: 410-420 us either way: the time is not in the block
        // boundaries), so it is taken only when asked for.
        if (forced == 9) {
          st = launch_persistent<E, 8, 4, 1, 8>(p, kt_main, true, stream);
          if (st == 0) *name = "mmt4d_mfma_128x512_persistent";
        }
        if (st < 0 && forced == 10) {
          st = launch_persistent<E, 8, 4, 2, 4>(p, kt_main, true, stream);
          if (st == 0) *name = "mmt4d_mfma_256x256_persistent";
        }
        if (st == 0) {
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
      if constexpr (RBC >= 16) {
        // Both operands through LDS-direct loads, two wave groups alternating
        // between memory and compute phases (PIPE 5 of mmt4d_mfma_kernel.h): the
        // default for the big problems of the 8- and 16-bit types (s8 8192^3
        // 413 -> 388 us, bf16 8192^3 779 -> 718 us, f16 4096^3 102 -> 98 us, f8
        // 8192^3 415 -> 390 us against the register-direct-RHS pipeline in its
        // best shape). f32
        // keeps that pipeline (matrix-pipe bound there: 925 against 959 us).
        constexpr bool kDefault = E != Elem::kF32;
        if (forced == 17) {
          st = launch_variant<E, RBC, 8, 4, 1, 8, 1, 5>(p, 0, kt_main, p.accumulate, stream);
          if (st == 0) *name = "mmt4d_mfma_128x512_lds_direct";
        }
        if (st < 0 && (forced == 16 || forced == 17 || (forced == 0 && kDefault))) {
          st = launch_variant<E, RBC, 8, 4, 2, 4, 1, 5>(p, 0, kt_main, p.accumulate, stream);
          if (st == 0) *name = "mmt4d_mfma_256x256_lds_direct";
        }
        if (st == 0) {
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
      if constexpr (RBC >= 16) {
        // 128 rows x 512 columns, the 8 waves side by side (each 128x64): no two
        // waves load the same RHS fragments and the LDS holds half as much LHS,
        // i.e. fewer bytes moved per MFMA, which is what a power-bound kernel
        // is short of (8192^3 s8 418-423 -> 403-412 us, 4096^3 f16 101 -> 98 us,
        // 8192^3 f8 401-408 -> 389 us, 8192^3 bf16 unchanged). Taken where it tiles the problem exactly;
        // ragged problems keep the square shape and its strip logic.
        const int bpm_w = 128 / p.M0, bpn_w = 512 / p.N0;
        if (forced == 8 || (forced == 0 && bpm_w >= 1 && bpn_w >= 1 && p.M1 % bpm_w == 0 &&
                            p.N1 % bpn_w == 0 && workgroups(p, 128, 512) >= 192)) {
          st = launch_variant<E, RBC, 8, 4, 1, 8, 1, BIG_PIPE>(p, 0, kt_main, p.accumulate, stream);
          wide = st == 0;
        }
      }
      if (st < 0) {
        st = launch_variant<E, RBC, 8, 4, 2, 4, 1, BIG_PIPE>(p, 0, kt_main, p.accumulate, stream);
      }
      if (st == 0) {
        *name = wide ? "mmt4d_mfma_128x512_rhs_direct"
                     : (RBC >= 16 ? "mmt4d_mfma_256x256_rhs_direct" : "mmt4d_mfma_256x256_regroup");
        if (kt_main == p.K1) return 0;
        return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
      }
      if (st > 0) return st;
    }
    choice = 2;
  }
  if (choice == 7) {
    // 256 rows x 128 columns, 8 waves of 128x32: for problems with too few
    // 256x256 blocks to fill the CUs; moves fewer L1 bytes per MFMA than the
    // 128x128 shape.
    if constexpr (RBC >= 16) {
      if (kt_main > 0 && (forced == 20 || (forced == 0 && E != Elem::kF32))) {
        int st = launch_variant<E, RBC, 8, 2, 2, 4, 1, 5>(p, 0, kt_main, p.accumulate, stream);
        if (st == 0) {
          *name = "mmt4d_mfma_256x128_lds_direct";
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
      if (kt_main > 0) {
        int st = launch_variant<E, RBC, 8, 2, 2, 4, 1, 3>(p, 0, kt_main, p.accumulate, stream);
        if (st == 0) {
          *name = "mmt4d_mfma_256x128_rhs_direct";
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
    }
    choice = 2;
  }
  if (choice == 6) {
    // Few 64x64 blocks and a long K: the barrier-free kernel with a 64x64
    // block per workgroup, whose four waves split K.
    if constexpr (RBC >= 8) {
      // K over workgroups too where the 64x64 blocks are fewer than half the
      // compute units and K is long: the meeting of the slices costs about 15
      // us with blocks of this size, so only from 24 KB of K per row on (f16
      // 128 x 128 x 65536, four blocks: 177 -> 52 us; 256 x 256 x 32768: 80 ->
      // 35; 512 x 512 x 16384: 44 -> 27; with 8 KB of K per row, 384 x 384 x
      // 4096, it loses: 16 -> 20 us).
      const bool long_k = ((int64_t)p.K1 << p.lrb) >= 24576;
      int st = launch_thin<E, RBC, 4, 4, 4, 2>(p, false, stream, long_k, 32);
      if (st >= 0) { *name = "mmt4d_mfma_64x64_ksplit"; return st; }
    }
    choice = 3;
  }
  // The thin kernel for a problem with `thin_rows` rows on its thin side and
  // `wide_cols` columns on the other (M-thin as it is, N-thin transposed):
  // 32 columns per workgroup, or 16 when 32 would leave compute units without
  // a workgroup (a decode step against a weight matrix of few rows, e.g.
  // 16 x 4096 x 14336 s8: 16.1 -> 12.8 us); what K split over workgroups adds
  // on top is decided in launch_thin.
  // (A generic lambda: its body is only instantiated for the row widths that call it.)
  auto thin_launch = [&](auto swapped_c, int64_t thin_rows, int64_t wide_cols) {
    const bool swapped = swapped_c;
    const bool narrow = uk::ceil_div(wide_cols, (int64_t)32) < compute_units();
    if (thin_rows <= 16) {
      return narrow ? launch_thin<E, RBC, 1, 1, 4, 4>(p, swapped, stream, true)
                    : launch_thin<E, RBC, 1, 2, 4, 4>(p, swapped, stream, true);
    }
    if (thin_rows <= 32) {
      return narrow ? launch_thin<E, RBC, 2, 1, 4, 4>(p, swapped, stream, true)
                    : launch_thin<E, RBC, 2, 2, 4, 4>(p, swapped, stream, true);
    }
    return narrow ? launch_thin<E, RBC, 4, 1, 4, 4>(p, swapped, stream, true)
                  : launch_thin<E, RBC, 4, 2, 4, 3>(p, swapped, stream, true);
  };
  if (choice == 5) {
    // N-thin (a few columns against many rows, e.g. the last column strip of
    // a ragged problem): the thin kernel on the transposed problem.
    if constexpr (RBC >= 8) {
      int st = thin_launch(std::true_type{}, cols_n, rows_m);
      if (st >= 0) { *name = "mmt4d_mfma_thin_transposed"; return st; }
    }
    choice = 3;
  }
  if (choice == 4) {
    if constexpr (RBC >= 8) {
      int st = thin_launch(std::false_type{}, rows_m, cols_n);
      if (st >= 0) { *name = "mmt4d_mfma_thin"; return st; }
    }
    // With 2-byte rows a 16-byte piece spans 8 rows and 32 rows do not fill a
    // loader block; that combination takes the 64x64 variant.
    if constexpr (RBC != 2) {
      // 256 bytes of K per step: these problems are bound by memory latency,
      // and a longer step keeps more bytes in flight per workgroup, as do the
      // three steps of loads ahead of the MFMAs.
      int st = launch_variant<E, RBC, 2, 1, 1, 4, 4 / H, 4>(p, 0, p.K1, p.accumulate, stream);
      if (st >= 0) { *name = "mmt4d_mfma_32x64"; return st; }
    }
    choice = 3;
  }
  if (choice == 2) {
    if constexpr (H == 1) {
      // The LDS-direct ping-pong pipeline with 8 waves of 64x32 (measured against
      // the kernels below: s8 2048^3 16x16x2 20.6 -> 14.7 us, 16x16x16 14.8 ->
      // 14.5 us; 3072^3 40.5 -> 36.3 us; bf16 2048^3 23.4 -> 22.6 us).
      if (kt_main > 0 && (forced == 18 || (forced == 0 && E != Elem::kF32))) {
        int st = launch_variant<E, RBC, 4, 2, 2, 4, 1, 5>(p, 0, kt_main, p.accumulate, stream);
        if (st == 0) {
          *name = "mmt4d_mfma_128x128_lds_direct";
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
    }
    if constexpr (NARROW) {
      // (Not chosen by size: measured level with or behind the 128x128 kernel
      // that sends both operands through LDS.)
      if (kt_main > 0 && forced == 14) {
        int st = launch_narrow<E, RBC, 4, 2, 2>(p, kt_main, stream);
        if (st == 0) {
          *name = "mmt4d_mfma_128x128_narrow";
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
    }
    if constexpr (RBC >= 16) {
      if (kt_main > 0) {
        int st = launch_variant<E, RBC, 4, 2, 2, 4, 1, 3>(p, 0, kt_main, p.accumulate, stream);
        if (st == 0) {
          *name = "mmt4d_mfma_128x128_rhs_direct";
          if (kt_main == p.K1) return 0;
          return finish_k(launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
        }
        if (st > 0) return st;
      }
    }
    int st = launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, 0, p.K1, p.accumulate, stream);
    if (st >= 0) { *name = "mmt4d_mfma_128x128"; return st; }
  }
  if constexpr (H == 1) {
    // 64x64 blocks, 8 waves of 32x16, 256 bytes of K per step.
    const int kts256 = 256 >> p.lrb;
    int kt_main256 = kts256 > 0 ? (p.K1 / kts256) * kts256 : 0;
    if (kOneLaunchOnly && kt_main256 != p.K1) kt_main256 = 0;
    // Chosen for narrow tile rows when the 64x64 blocks fill the compute units
    // (s8 1024^3 16x16x2: 7.0 -> 6.4 us; with rows of 16 bytes and more the
    // register-direct kernel below is level or ahead: 5.7 against 5.9 us).
    const bool small_narrow = forced == 0 && RBC < 16 && E != Elem::kF32 && workgroups(p, 64, 64) >= 192;
    if (kt_main256 > 0 && (forced == 19 || small_narrow)) {
      int st = launch_variant<E, RBC, 2, 1, 2, 4, 4, 5>(p, 0, kt_main256, p.accumulate, stream);
      if (st == 0) {
        *name = "mmt4d_mfma_64x64_lds_direct";
        if (kt_main256 == p.K1) return 0;
        return finish_k(launch_variant<E, RBC, 2, 2, 2, 2, NKK2, 0>(p, kt_main256, p.K1 - kt_main256, true, stream));
      }
      if (st > 0) return st;
    }
  }
  if constexpr (RBC >= 16) {
    if (kt_main > 0) {
      int st = launch_variant<E, RBC, 2, 2, 2, 2, 1, 3>(p, 0, kt_main, p.accumulate, stream);
      if (st == 0) {
        *name = "mmt4d_mfma_64x64_rhs_direct";
        if (kt_main == p.K1) return 0;
        return finish_k(launch_variant<E, RBC, 2, 2, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
      }
      if (st > 0) return st;
    }
  }
  if constexpr (NARROW) {
    if (kt_main > 0 && forced == 15) {
      int st = launch_narrow<E, RBC, 2, 2, 1>(p, kt_main, stream);
      if (st == 0) {
        *name = "mmt4d_mfma_64x64_narrow";
        if (kt_main == p.K1) return 0;
        return finish_k(launch_variant<E, RBC, 2, 2, 2, 2, NKK2, 0>(p, kt_main, p.K1 - kt_main, true, stream));
      }
      if (st > 0) return st;
    }
  }
  if constexpr (RBC < 16) {
    // Narrow tile rows, small problem: latency-bound (a 64x64 block computes a
    // 64-byte step in 64 MFMA cycles against a global round trip of well over a
    // thousand). 256-byte steps with the loads three steps ahead put the whole K
    // of such a problem in flight at once.
    if (forced == 11 || (forced == 0 && ((int64_t)p.K1 << p.lrb) <= 8192)) {
      int st = launch_variant<E, RBC, 2, 2, 2, 2, 4 / H, 4>(p, 0, p.K1, p.accumulate, stream);
      if (st >= 0) { *name = "mmt4d_mfma_64x64_deep"; return st; }
    }
  }
  int st = launch_variant<E, RBC, 2, 2, 2, 2, NKK2, 0>(p, 0, p.K1, p.accumulate, stream);
  if (st >= 0) { *name = "mmt4d_mfma_64x64"; return st; }
  st = launch_variant<E, RBC, 4, 4, 2, 2, NKK2, 0>(p, 0, p.K1, p.accumulate, stream);
  if (st >= 0) *name = "mmt4d_mfma_128x128";
  return st;
}

}  // namespace uk_mfma

#endif  // IREE_UK_AMD_MMT4D_MFMA_LAUNCH_H_
