// Measured ceilings for the runner: what the matrix cores and the memory
// system of the device at hand sustain when nothing else is in the way. The
// benchmark reports its kernels against these next to the published peaks.
//
//   iree_uk_amd_probe_mfma_peak   a loop of nothing but MFMAs, 8 waves per CU
//                                 with the register blocking of the mmt4d
//                                 kernels (8 x 4 accumulator blocks per wave),
//                                 operands held in registers: no memory traffic
//   iree_uk_amd_probe_copy2d      a plain 2-D copy between two pitches (the
//                                 traffic of a pack / unpack without the
//                                 transposition)
//
// Counterpart in the reference: none; its benchmarks
// (runtime/src/iree/builtins/ukernel/tools/mmt4d_benchmark.c:82-84,
// tools/pack_benchmark.c:97-101) report rates without a ceiling beside them.
#include <hip/hip_runtime.h>

#include "mmt4d_mfma_kernel.h"
#include "uk_hip_abi.h"

namespace {

using uk_mfma::Elem;
using uk_mfma::ElemTraits;
using uk_mfma::v4i;

constexpr int kTM = 8, kTN = 4, kWaves = 8;

template <Elem E, int WAVES = kWaves>
__global__ __launch_bounds__(WAVES * 64) void mfma_peak_kernel(const v4i* operands, int n_operands,
                                                              int iters, int* sink, int sink_enable) {
  using TT = ElemTraits<E>;
  using Acc = typename TT::Acc;
  constexpr int H = TT::kHalves;
  v4i fa[kTM][H], fb[kTN][H];
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int h = 0; h < H; ++h) fa[i][h] = operands[(t * 31u + (uint32_t)(i * H + h) * 977u) % (uint32_t)n_operands];
#pragma unroll
  for (int i = 0; i < kTN; ++i)
#pragma unroll
    for (int h = 0; h < H; ++h)
      fb[i][h] = operands[(t * 17u + 7919u + (uint32_t)(i * H + h) * 613u) % (uint32_t)n_operands];
  Acc acc[kTM][kTN];
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int j = 0; j < kTN; ++j) acc[i][j] = Acc{0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < kTM; ++i)
#pragma unroll
      for (int j = 0; j < kTN; ++j) acc[i][j] = TT::mfma(fb[j], fa[i], acc[i][j]);
  }
  // Keep the accumulators alive without writing anything in practice: the
  // store depends on a kernel argument that the host always passes as zero,
  // which the compiler cannot know (nothing about `iters` or the data lets it
  // drop the loop).
  Acc s = acc[0][0];
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int j = 0; j < kTN; ++j)
      if (i || j) s = s + acc[i][j];
  const v4i bits = __builtin_bit_cast(v4i, s);
  if (sink_enable) sink[t] = bits[0] ^ bits[1] ^ bits[2] ^ bits[3];
}

// K elements per MFMA instruction group issued by ElemTraits<E>::mfma.
template <Elem E> constexpr int k_per_mfma() {
  return E == Elem::kS8 ? 64 : E == Elem::kF8 ? 128 : E == Elem::kF32 ? 16 : 32;
}

template <Elem E>
int run_mfma_peak(const v4i* operands, int n_operands, int iters, int workgroups, int* sink,
                  hipStream_t stream, double* ops) {
  hipLaunchKernelGGL(mfma_peak_kernel<E>, dim3(workgroups), dim3(kWaves * 64), 0, stream, operands,
                     n_operands, iters, sink, /*sink_enable=*/0);
  *ops = 2.0 * 16 * 16 * k_per_mfma<E>() * kTM * kTN * (double)iters * kWaves * workgroups;
  return (int)hipGetLastError();
}

// The s8 loop with its MFMAs written as assembly, in the order and on the
// registers given: what a wave can issue, not what the compiler makes of the
// loop. (With 256 threads the compiler moves the accumulators to the
// accumulator file and shuffles them around every MFMA; that loop reads 0.84
// of the rate below and says nothing about the hardware.)
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void mfma_asm_kernel(const v4i* operands, int n_operands,
                                                             int iters, int* sink, int sink_enable) {
  v4i fa[kTM], fb[kTN];
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
  for (int i = 0; i < kTM; ++i) fa[i] = operands[(t * 31u + (uint32_t)i * 977u) % (uint32_t)n_operands];
#pragma unroll
  for (int i = 0; i < kTN; ++i) fb[i] = operands[(t * 17u + 7919u + (uint32_t)i * 613u) % (uint32_t)n_operands];
  v4i acc[kTM][kTN];
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int j = 0; j < kTN; ++j) acc[i][j] = v4i{0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < kTM; ++i)
#pragma unroll
      for (int j = 0; j < kTN; ++j)
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[i][j]) : "v"(fb[j]), "v"(fa[i]));
  }
  // The last results leave the matrix pipe before anything reads them (the
  // compiler does not know that the assembly is MFMAs).
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  v4i s = acc[0][0];
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int j = 0; j < kTN; ++j)
      if (i || j) s = s + acc[i][j];
  if (sink_enable) sink[t] = s[0] ^ s[1] ^ s[2] ^ s[3];
}

// That loop with exactly `WAVES / 4` waves on every SIMD: one workgroup per
// CU (its LDS allocation leaves no room for a second one).
template <Elem E, int WAVES>
int run_mfma_peak_waves(const v4i* operands, int n_operands, int iters, int cus, int* sink,
                        hipStream_t stream, double* ops) {
  static_assert(E == Elem::kS8, "the assembly loop is the s8 instruction");
  constexpr size_t kLds = 84 * 1024;
  auto kernel = mfma_asm_kernel<WAVES>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds);
  if (attr != hipSuccess) return (int)attr;
  hipLaunchKernelGGL(kernel, dim3(cus), dim3(WAVES * 64), kLds, stream, operands, n_operands, iters, sink,
                     /*sink_enable=*/0);
  *ops = 2.0 * 16 * 16 * k_per_mfma<E>() * kTM * kTN * (double)iters * WAVES * cus;
  return (int)hipGetLastError();
}

// A workgroup copies 4 KiB pieces of rows (16 bytes per lane, 4-byte aligned
// like the pack kernels' 2-D side), walking pieces grid-stride, DEPTH pieces
// per turn: all loads of a turn are issued before its stores. NT: non-temporal
// stores (the destination is not read again). NTL: non-temporal loads too.
// LINES: the pieces of a row are shifted so that every store of a wave covers whole 128-byte lines of the
// destination whatever the pitch (one more, partial piece per row; the loads
// are then the unaligned side).
template <int DEPTH, bool NT, bool LINES = false, bool NTL = false>
__global__ __launch_bounds__(256) void copy2d_kernel(const char* src, int64_t src_pitch, char* dst,
                                                     int64_t dst_pitch, int64_t row_bytes,
                                                     int64_t rows) {
  typedef uk_mfma::v4i v4i_a4 __attribute__((aligned(4)));
  const int64_t pieces_per_row = (row_bytes + 4095) / 4096 + (LINES ? 1 : 0);
  const int64_t total = pieces_per_row * rows;
  // Byte offset of lane's vector of piece p inside its row (may start before the
  // row or end after it: such a vector moves word by word, or not at all).
  auto offset_of = [&](int64_t p, int64_t* row) {
    *row = p / pieces_per_row;
    int64_t off = (p - *row * pieces_per_row) * 4096 + (int64_t)threadIdx.x * 16;
    if (LINES) off -= (int64_t)(((uintptr_t)dst + (uint64_t)(*row * dst_pitch)) & 127);
    return off;
  };
  for (int64_t p0 = (int64_t)blockIdx.x * DEPTH; p0 < total; p0 += (int64_t)gridDim.x * DEPTH) {
    uk_mfma::v4i v[DEPTH];
    int64_t so[DEPTH], dof[DEPTH];
    bool whole[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      int64_t row;
      const int64_t off = offset_of(p0 + d, &row);
      so[d] = row * src_pitch + off;
      dof[d] = row * dst_pitch + off;
      whole[d] = p0 + d < total && off >= 0 && off + 16 <= row_bytes;
      if (whole[d]) {
        if (NTL) v[d] = __builtin_nontemporal_load(reinterpret_cast<const v4i_a4*>(src + so[d]));
        else v[d] = *reinterpret_cast<const v4i_a4*>(src + so[d]);
      }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (whole[d]) {
        if (NT) __builtin_nontemporal_store(v[d], reinterpret_cast<v4i_a4*>(dst + dof[d]));
        else *reinterpret_cast<v4i_a4*>(dst + dof[d]) = v[d];
      } else if (p0 + d < total) {
        // a vector that straddles an end of its row: word by word
        int64_t row;
        const int64_t off = offset_of(p0 + d, &row);
        for (int64_t b = off; b < off + 16; b += 4)
          if (b >= 0 && b < row_bytes)
            *reinterpret_cast<int*>(dst + row * dst_pitch + b) =
                *reinterpret_cast<const int*>(src + row * src_pitch + b);
      }
    }
  }
}

// One wave: LDS holds 16-bit values equal to their own index; lane l reads the
// eight bytes at 16-bit index lane_index[l] with ds_read_b64_tr_b16 and stores
// the four values it receives.
__global__ __launch_bounds__(64) void ds_read_tr16_kernel(const int* lane_index, short* out, int lds_values) {
  extern __shared__ __attribute__((aligned(16))) short tr16_lds[];
  for (int i = threadIdx.x; i < lds_values; i += 64) tr16_lds[i] = (short)i;
  __syncthreads();
  typedef int v2i __attribute__((ext_vector_type(2)));
  v2i v;
  const uint32_t addr = (uint32_t)(uintptr_t)(tr16_lds + lane_index[threadIdx.x]);   // LDS addresses are the low 32 bits
  asm volatile("ds_read_b64_tr_b16 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
  out[threadIdx.x * 4 + 0] = (short)(v[0] & 0xFFFF);
  out[threadIdx.x * 4 + 1] = (short)((uint32_t)v[0] >> 16);
  out[threadIdx.x * 4 + 2] = (short)(v[1] & 0xFFFF);
  out[threadIdx.x * 4 + 3] = (short)((uint32_t)v[1] >> 16);
}

}  // namespace

extern "C" {

// Runs ds_read_b64_tr_b16 in one wave for the lane addresses in `lane_index`
// (64 ints of device memory: the 16-bit index each lane addresses, a multiple
// of 4, below `lds_values` <= 16384) on an LDS image whose 16-bit values are
// their own indices; `out` (256 shorts of device memory) receives the four
// values of every lane. The mmt4d kernels' fragment reads for 2-byte tile rows
// rest on this instruction's lane mapping; tests/test_gpu_probe.py pins it.
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_ds_read_tr16(const int* lane_index, short* out,
                                                      int lds_values, void* stream_v) {
  hipStream_t stream = (hipStream_t)stream_v;
  if (!lane_index || !out || lds_values < 4 || lds_values > 16384) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(ds_read_tr16_kernel, dim3(1), dim3(64), (size_t)lds_values * 2, stream, lane_index,
                     out, lds_values);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return (int)err;
  return (int)hipStreamSynchronize(stream);
}


// Runs the MFMA-only loop of the element type in `type_flags` (an
// IREE_UK_FLAG_MMT4D_TYPE_* value: S8S8S32, F16F16F32, BF16BF16F32, F32F32F32
// or the f8 extension) on `stream`: `workgroups` workgroups of 8 waves (0 = two
// per compute unit), `iters` passes over the 32 accumulator blocks of a wave.
// `operands` points to `operand_bytes` (a multiple of 16, at least 16) of
// device memory from which the lanes take their register operands once;
// all-zero bytes and random bytes give different clocks on a power-limited
// part. `sink` is device memory for one int per thread that is never written
// in practice. Returns 0 and the operations per second in *ops_per_second.
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_mfma_peak(uint32_t type_flags, const void* operands,
                                                   int64_t operand_bytes, int iters,
                                                   int workgroups, void* sink, void* stream_v,
                                                   double* ops_per_second) {
  hipStream_t stream = (hipStream_t)stream_v;
  if (!operands || operand_bytes < 16 || iters < 1 || !sink || !ops_per_second) return (int)hipErrorInvalidValue;
  if (workgroups <= 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
      return (int)hipErrorUnknown;
    }
    workgroups = 2 * cus;
  }
  const v4i* ops_ptr = (const v4i*)operands;
  const int n = (int)(operand_bytes / 16);
  hipEvent_t start, stop;
  if (hipEventCreate(&start) != hipSuccess) return (int)hipErrorUnknown;
  if (hipEventCreate(&stop) != hipSuccess) {
    (void)hipEventDestroy(start);
    return (int)hipErrorUnknown;
  }
  double ops = 0;
  int st = 0;
  auto run = [&](int it) {
    switch (type_flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
      case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32:
        return run_mfma_peak<Elem::kS8>(ops_ptr, n, it, workgroups, (int*)sink, stream, &ops);
      case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32:
        return run_mfma_peak<Elem::kF16>(ops_ptr, n, it, workgroups, (int*)sink, stream, &ops);
      case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32:
        return run_mfma_peak<Elem::kBF16>(ops_ptr, n, it, workgroups, (int*)sink, stream, &ops);
      case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32:
        return run_mfma_peak<Elem::kF32>(ops_ptr, n, it, workgroups, (int*)sink, stream, &ops);
      case IREE_UK_AMD_FLAG_MMT4D_TYPE_F8E4M3FNF8E4M3FNF32:
        return run_mfma_peak<Elem::kF8>(ops_ptr, n, it, workgroups, (int*)sink, stream, &ops);
      default:
        return (int)hipErrorInvalidValue;
    }
  };
  st = run(iters / 8 + 1);  // warm-up
  if (st == 0) st = (int)hipEventRecord(start, stream);
  if (st == 0) st = run(iters);
  if (st == 0) st = (int)hipEventRecord(stop, stream);
  if (st == 0) st = (int)hipEventSynchronize(stop);
  float ms = 0.f;
  if (st == 0) st = (int)hipEventElapsedTime(&ms, start, stop);
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  if (st != 0) return st;
  *ops_per_second = ops / ((double)ms * 1e-3);
  return 0;
}

// The MFMA-only loop of the s8 instruction, written as assembly, with
// `waves_per_simd` (1 or 2) waves on every SIMD of every CU: a wave on its own
// keeps the matrix pipe as full as two do (0.98 on operands that draw no
// power), so the instruction itself does not ask for a second wave.
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_mfma_peak_waves(const void* operands, int64_t operand_bytes,
                                                         int iters, int waves_per_simd, void* sink,
                                                         void* stream_v, double* ops_per_second) {
  hipStream_t stream = (hipStream_t)stream_v;
  if (!operands || operand_bytes < 16 || iters < 1 || !sink || !ops_per_second ||
      (waves_per_simd != 1 && waves_per_simd != 2)) {
    return (int)hipErrorInvalidValue;
  }
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    return (int)hipErrorUnknown;
  }
  const v4i* ops_ptr = (const v4i*)operands;
  const int n = (int)(operand_bytes / 16);
  hipEvent_t start, stop;
  if (hipEventCreate(&start) != hipSuccess) return (int)hipErrorUnknown;
  if (hipEventCreate(&stop) != hipSuccess) {
    (void)hipEventDestroy(start);
    return (int)hipErrorUnknown;
  }
  double ops = 0;
  auto run = [&](int it) {
    return waves_per_simd == 1
               ? run_mfma_peak_waves<Elem::kS8, 4>(ops_ptr, n, it, cus, (int*)sink, stream, &ops)
               : run_mfma_peak_waves<Elem::kS8, 8>(ops_ptr, n, it, cus, (int*)sink, stream, &ops);
  };
  int st = run(iters / 8 + 1);  // warm-up
  if (st == 0) st = (int)hipEventRecord(start, stream);
  if (st == 0) st = run(iters);
  if (st == 0) st = (int)hipEventRecord(stop, stream);
  if (st == 0) st = (int)hipEventSynchronize(stop);
  float ms = 0.f;
  if (st == 0) st = (int)hipEventElapsedTime(&ms, start, stop);
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  if (st != 0) return st;
  *ops_per_second = ops / ((double)ms * 1e-3);
  return 0;
}

// Copies `rows` rows of `row_bytes` bytes (a multiple of 4) from `src` (rows
// `src_pitch` bytes apart) to `dst` (`dst_pitch`) `iters` times on `stream`,
// in five variants of the copy kernel (1, 4 or 8 vectors in flight per lane,
// ordinary or non-temporal stores, pieces shifted row by row so that only
// whole 128-byte lines of the destination are written), and returns the
// average seconds per copy of the fastest variant: the ceiling of a pack /
// unpack that moves the same matrix between the same two pitches. When
// `seconds_per_variant` is not null it receives the five averages (the last
// one is the whole-line variant). All pointers and pitches 4-byte aligned.
IREE_UK_AMD_EXPORT int iree_uk_amd_probe_copy2d(const void* src, int64_t src_pitch, void* dst,
                                                int64_t dst_pitch, int64_t row_bytes,
                                                int64_t rows, int iters, void* stream_v,
                                                double* seconds_per_copy) {
  return iree_uk_amd_probe_copy2d_variants(src, src_pitch, dst, dst_pitch, row_bytes, rows, iters,
                                           stream_v, seconds_per_copy, nullptr);
}

IREE_UK_AMD_EXPORT int iree_uk_amd_probe_copy2d_variants(const void* src, int64_t src_pitch, void* dst,
                                                         int64_t dst_pitch, int64_t row_bytes,
                                                         int64_t rows, int iters, void* stream_v,
                                                         double* seconds_per_copy,
                                                         double* seconds_per_variant) {
  hipStream_t stream = (hipStream_t)stream_v;
  if (!src || !dst || !seconds_per_copy || iters < 1 || row_bytes < 4 || (row_bytes & 3) || rows < 1 ||
      (((uintptr_t)src | (uintptr_t)dst | (uint64_t)src_pitch | (uint64_t)dst_pitch) & 3)) {
    return (int)hipErrorInvalidValue;
  }
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    return (int)hipErrorUnknown;
  }
  hipEvent_t start, stop;
  if (hipEventCreate(&start) != hipSuccess) return (int)hipErrorUnknown;
  if (hipEventCreate(&stop) != hipSuccess) {
    (void)hipEventDestroy(start);
    return (int)hipErrorUnknown;
  }
  // Five ways of writing the same copy; the fastest one is the ceiling.
  auto run = [&](int variant) {
    const char* s8 = (const char*)src;
    char* d8 = (char*)dst;
    switch (variant) {
      case 0: hipLaunchKernelGGL((copy2d_kernel<1, false>), dim3(cus * 8), dim3(256), 0, stream, s8, src_pitch, d8, dst_pitch, row_bytes, rows); break;
      case 1: hipLaunchKernelGGL((copy2d_kernel<4, false>), dim3(cus * 4), dim3(256), 0, stream, s8, src_pitch, d8, dst_pitch, row_bytes, rows); break;
      case 2: hipLaunchKernelGGL((copy2d_kernel<4, true>), dim3(cus * 4), dim3(256), 0, stream, s8, src_pitch, d8, dst_pitch, row_bytes, rows); break;
      case 3: hipLaunchKernelGGL((copy2d_kernel<8, true, false, true>), dim3(cus * 2), dim3(256), 0, stream, s8, src_pitch, d8, dst_pitch, row_bytes, rows); break;
      default: hipLaunchKernelGGL((copy2d_kernel<4, true, true>), dim3(cus * 4), dim3(256), 0, stream, s8, src_pitch, d8, dst_pitch, row_bytes, rows); break;
    }
  };
  int st = 0;
  double best = 0.0;
  for (int variant = 0; variant < 5 && st == 0; ++variant) {
    run(variant);
    run(variant);
    st = (int)hipEventRecord(start, stream);
    for (int i = 0; i < iters; ++i) run(variant);
    if (st == 0) st = (int)hipGetLastError();
    if (st == 0) st = (int)hipEventRecord(stop, stream);
    if (st == 0) st = (int)hipEventSynchronize(stop);
    float ms = 0.f;
    if (st == 0) st = (int)hipEventElapsedTime(&ms, start, stop);
    const double sec = (double)ms * 1e-3 / iters;
    if (st == 0 && (best == 0.0 || sec < best)) best = sec;
    if (st == 0 && seconds_per_variant) seconds_per_variant[variant] = sec;
  }
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  if (st != 0) return st;
  *seconds_per_copy = best;
  return 0;
}

}  // extern "C"
