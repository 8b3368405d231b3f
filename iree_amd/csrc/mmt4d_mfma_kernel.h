// mmt4d on the gfx950 matrix cores: the kernel template.
//
// Operands keep the ukernel ABI layout: LHS [M1][K1][M0][K0], RHS
// [N1][K1][N0][K0] (both K-major per tile row), OUT [M1][N1][M0][N0]
// (runtime/src/iree/builtins/ukernel/mmt4d.c:55-100 is the pointer arithmetic
// this replaces). A workgroup owns a block of whole LHS panels x whole RHS
// panels; each of its waves owns TM x TN accumulator blocks of 16x16.
//
// The MFMA instructions used take, per lane, 16 (2x16 for f8) consecutive
// bytes of K for ONE row: lane l feeds row l%16 with K-slice l/16. The sum
// over K is order-free as far as the instruction is concerned, so any
// assignment of K bytes to (instruction, slice, byte) works as long as LHS and
// RHS use the same one. That freedom is what lets every K0 be served:
//
//   row bytes RB = K0 * sizeof(elem)
//   RB >= 16 : a 16-byte piece of a tile row is already an MFMA operand;
//              global -> LDS is a 16-byte-granular copy in which each lane
//              fetches exactly the piece its LDS slot wants.
//   RB = 8/4/2: a 16-byte global piece holds R = 16/RB rows of one K-tile. A
//              lane loads the same R rows from R different K-tiles and
//              regroups them in registers into R one-row operands (register
//              selection for RB = 8 and 4, v_perm_b32 for RB = 2) before
//              storing them to LDS.
//
// LDS holds, per pipeline stage, the operands exactly as the waves consume
// them: [row block of 16][group of 4 K-slices][slice q][row r][16 bytes], so an
// operand fetch is one ds_read_b128 per lane over a contiguous KiB.
//
// Pipelines (template parameter PIPE), one barrier per K step in all of them:
//   0  two LDS stages, both operands through LDS, global loads one step
//      ahead, zero-filled K tail (any K);
//   1  three LDS stages, both operands through LDS, loads three steps ahead
//      through two register sets, fragments one step ahead;
//   2  LHS as in 1, RHS fragments loaded by each wave straight from global
//      memory into registers one step ahead (row bytes >= 16 only);
//   3  as 2 with every prefetch one step deeper (three register sets, three
//      RHS fragment buffers), unrolled by three;
//   4  as 0 with the global loads three steps ahead through three register
//      sets (any K): for M-thin problems, which are bound by memory latency
//      and want as many bytes in flight per workgroup as registers allow.
//   5  both operands brought into LDS by LDS-direct global loads
//      (global_load_lds, 16 bytes per lane: one instruction moves one 1 KiB
//      fragment and touches no register), kStages5 stages deep; the eight
//      waves form two groups of four (one wave of each group per SIMD) that
//      alternate, half a step apart, between a memory phase (fragment reads,
//      issue of the loads kStages5 - 1 steps ahead) and a compute phase (all MFMAs of
//      the step back to back), with a workgroup barrier between phases: while
//      one wave of a SIMD feeds the matrix pipe, the other one's memory
//      instructions issue beside it instead of in between its MFMAs (row
//      bytes >= 16, eight waves).
// Pipelines 1-3 and 5 need K in whole steps; the launcher gives a K remainder
// to a second, accumulating launch of a PIPE 0 variant.
#ifndef IREE_UK_AMD_MMT4D_MFMA_KERNEL_H_
#define IREE_UK_AMD_MMT4D_MFMA_KERNEL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "uk_float_convert.h"

namespace uk_mfma {

typedef int v4i __attribute__((ext_vector_type(4)));
// Operand pieces as they are read from global memory: no alignment beyond the
// element's is asked of the caller's buffers. The HSA ABI runs the memory
// pipeline in its unaligned mode, in which a 16-byte global load takes any
// address (the compiler itself emits one global_load_dwordx4 for this type).
typedef v4i v4i_g __attribute__((aligned(1)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

// kF16F16 / kBF16BF16: 16-bit float output, accumulated in f32 over all of K
// and rounded once at the end (IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS,
// runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:258-286,348-376).
// kS8S4: s8 x s4 -> s32 (two 4-bit RHS values per byte, low nibble first,
// runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:11-51); served by
// the thin kernel only (mmt4d_mfma_thin.h).
// kS16: s16 x s16 -> s32 as four 8-bit integer products per element pair (the
// hardware has no 16-bit integer matrix instruction); served by the LDS-direct
// pipeline only (PIPE 5 below, which describes the arithmetic).
enum class Elem { kS8, kF16, kBF16, kF8, kF32, kF16F16, kBF16BF16, kS8S4, kS16 };

typedef uint16_t v4u16 __attribute__((ext_vector_type(4)));

// Output access for 4-byte outputs: the accumulator quad as it is.
template <typename Acc, typename T>
struct Out32 {
  static constexpr int kOutBytes = 4;
  // 4-byte alignment is all these need (gfx950 under HSA takes dword-aligned
  // wide accesses); row-major outputs with odd row lengths rely on it.
  typedef Acc Acc4 __attribute__((aligned(4)));
  static __device__ __forceinline__ Acc load4(const char* p) { return *reinterpret_cast<const Acc4*>(p); }
  static __device__ __forceinline__ void store4(char* p, Acc v) { *reinterpret_cast<Acc4*>(p) = v; }
  // The non-temporal form, chosen at run time (Args::nt_out). As assembly:
  // beside the plain store of the same value in the other branch the compiler
  // would merge the two into one plain store.
  static __device__ __forceinline__ void store4_nt(char* p, Acc v) {
    asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(p), "v"(v) : "memory");
  }
  static __device__ __forceinline__ T load1(const char* p) { return *reinterpret_cast<const T*>(p); }
  static __device__ __forceinline__ void store1(char* p, T v) { *reinterpret_cast<T*>(p) = v; }
};
// 16-bit float outputs with EB exponent bits, converted like the CPU ukernel.
template <int EB>
struct Out16 {
  static constexpr int kOutBytes = 2;
  static __device__ __forceinline__ v4f load4(const char* p) {
    const v4u16 h = *reinterpret_cast<const v4u16*>(p);
    return v4f{uk::small16_to_f32<EB>(h[0]), uk::small16_to_f32<EB>(h[1]),
               uk::small16_to_f32<EB>(h[2]), uk::small16_to_f32<EB>(h[3])};
  }
  static __device__ __forceinline__ void store4(char* p, v4f v) {
    *reinterpret_cast<v4u16*>(p) = v4u16{uk::f32_to_small16<EB>(v[0]), uk::f32_to_small16<EB>(v[1]),
                                         uk::f32_to_small16<EB>(v[2]), uk::f32_to_small16<EB>(v[3])};
  }
  static __device__ __forceinline__ void store4_nt(char* p, v4f v) {
    const v4u16 h = v4u16{uk::f32_to_small16<EB>(v[0]), uk::f32_to_small16<EB>(v[1]),
                          uk::f32_to_small16<EB>(v[2]), uk::f32_to_small16<EB>(v[3])};
    typedef uint32_t v2u32 __attribute__((ext_vector_type(2)));
    asm volatile("global_store_dwordx2 %0, %1, off nt" : : "v"(p), "v"(__builtin_bit_cast(v2u32, h)) : "memory");
  }
  static __device__ __forceinline__ float load1(const char* p) {
    return uk::small16_to_f32<EB>(*reinterpret_cast<const uint16_t*>(p));
  }
  static __device__ __forceinline__ void store1(char* p, float v) {
    *reinterpret_cast<uint16_t*>(p) = uk::f32_to_small16<EB>(v);
  }
};

template <Elem E> struct ElemTraits;

template <> struct ElemTraits<Elem::kS8> {
  using Acc = v4i;
  using Out = Out32<v4i, int32_t>;
  static constexpr int kHalves = 1;  // 16-byte pieces per lane operand
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], b[0], c, 0, 0, 0);
  }
};
template <> struct ElemTraits<Elem::kS8S4> : ElemTraits<Elem::kS8> {};
template <> struct ElemTraits<Elem::kF16> {
  using Acc = v4f;
  using Out = Out32<v4f, float>;
  static constexpr int kHalves = 1;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(v8h, a[0]), __builtin_bit_cast(v8h, b[0]), c, 0, 0, 0);
  }
};
template <> struct ElemTraits<Elem::kBF16> {
  using Acc = v4f;
  using Out = Out32<v4f, float>;
  static constexpr int kHalves = 1;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(v8bf, a[0]), __builtin_bit_cast(v8bf, b[0]), c, 0, 0, 0);
  }
};
template <> struct ElemTraits<Elem::kF8> {
  using Acc = v4f;
  using Out = Out32<v4f, float>;
  static constexpr int kHalves = 2;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    v8i av = {a[0][0], a[0][1], a[0][2], a[0][3], a[1][0], a[1][1], a[1][2], a[1][3]};
    v8i bv = {b[0][0], b[0][1], b[0][2], b[0][3], b[1][0], b[1][1], b[1][2], b[1][3]};
    // Formats 0/0 = E4M3 x E4M3. Zero scale operands select the unscaled
    // instruction (v_mfma_f32_16x16x128_f8f6f4, plain products); the scaled
    // form with 2^0 block scales computes the same but is a two-part
    // instruction (scale load + MFMA) and issues more slowly.
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, 0, 0, 0, 0, 0, 0);
  }
};

// Sixteen 16-bit elements per lane operand (two 16-byte pieces, 128 bytes of K
// per step as for the 8-bit floats). The pipeline splits them into a register
// quad of high bytes and one of low bytes and issues the four byte products
// itself; `mfma` here is the low x low product, which accumulates unscaled.
template <> struct ElemTraits<Elem::kS16> {
  using Acc = v4i;
  using Out = Out32<v4i, int32_t>;
  static constexpr int kHalves = 2;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a[1], b[1], c, 0, 0, 0);
  }
};

template <> struct ElemTraits<Elem::kF32> {
  using Acc = v4f;
  using Out = Out32<v4f, float>;
  static constexpr int kHalves = 1;
  // v_mfma_f32_16x16x4_f32 takes one f32 of K per lane (row l%16, k = l/16):
  // the lane's 16-byte piece feeds four of them, one per word. Which four K
  // values meet in one instruction is the same for both operands, which is
  // all the sum needs.
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    const v4f af = __builtin_bit_cast(v4f, a[0]), bf = __builtin_bit_cast(v4f, b[0]);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[0], bf[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[1], bf[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[2], bf[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[3], bf[3], c, 0, 0, 0);
    return c;
  }
};

template <> struct ElemTraits<Elem::kF16F16> : ElemTraits<Elem::kF16> {
  using Out = Out16<5>;
};
template <> struct ElemTraits<Elem::kBF16BF16> : ElemTraits<Elem::kBF16> {
  using Out = Out16<8>;
};

// LDS-direct loads (PIPE 5): address-space-qualified pointers for the builtin,
// and the wait for "at most N vector memory operations still in flight" (the
// compiler does not track what these loads write, the kernel waits itself).
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;
template <int N>
__device__ __forceinline__ void wait_vmem_in_flight() {
  static_assert(N >= 0 && N < 64, "the counter has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));  // expcnt, lgkmcnt: no wait
}
// Waits for the wave's LDS reads (and scalar loads), not for vector memory.
__device__ __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(0xC07F); }
// LDS stages of PIPE 5.
constexpr int kStages5 = 4;
// Half-step slots of PIPE 5's ring for lane operands of two 16-byte pieces. The
// 16-bit integers finish a step in half the time of the 8-bit floats (same
// instruction count, instructions half as long), so the same distance in time
// between a load's issue and its use takes a ring twice as deep, where it fits.
template <Elem E, int BM, int BN>
constexpr int ring_slots() {
  return (E == Elem::kS16 && 9 * (BM + BN) * 64 <= 160 * 1024) ? 9 : 5;
}
// f(integral_constant<int, I>) for I = BEGIN .. END - 1.
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (BEGIN < END) {
    f(std::integral_constant<int, BEGIN>{});
    static_for<BEGIN + 1, END>(f);
  }
}

struct Args {
  const char* lhs;
  const char* rhs;
  char* out;
  int64_t lhs_stride;  // bytes between LHS panels
  int64_t rhs_stride;  // bytes between RHS panels
  int64_t out_stride;  // bytes between output row panels (tiled: rows of tiles; row-major: M0 rows)
  uint32_t out_sm0;    // bytes between rows inside a panel (tiled: N0 * elem; row-major: row pitch)
  uint32_t out_spn;    // bytes between column panels (tiled: M0 * N0 * elem; row-major: N0 * elem)
  int32_t out_rows, out_cols;  // rows / columns that exist, from this problem's origin
  int32_t M1, N1, K1;
  int32_t M0, N0;
  int32_t rb;          // bytes per tile row (K0 * element size), power of two
  int32_t lrb;         // log2(rb)
  int32_t bpm, bpn;    // whole panels per workgroup along M and N
  int32_t grid_m, grid_n;
  int32_t steps;       // K steps
  uint32_t accumulate;
  uint32_t tail;       // 1 when the last K step is partial
  uint32_t band;       // workgroup rows per rasterization band
  uint32_t vec_out;    // 1: 4 consecutive columns of a row are contiguous (and aligned enough)
  uint32_t nt_out;     // 1: the final store of the accumulators is non-temporal (mmt4d_mfma_kernel.h only)
  // Where ACCUMULATE reads the initial accumulators: the same four-stride
  // addressing as the output. It is the output itself except in the first
  // launch of a dequantizing call, which reads a tiled accumulator buffer and
  // writes a row-major matrix.
  const char* acc;
  int64_t acc_stride;
  uint32_t acc_sm0, acc_spn;
  // Dequantizing store (4-byte outputs only), applied by the launch that
  // finishes K: element (row, col) becomes
  //   (float)acc * row_scale[row] * col_scale[col]   (a NULL scale reads as 1)
  // with row / col counted from this problem's origin.
  uint32_t dequant;
  const float* row_scale;
  const float* col_scale;
  // mmt4d_mfma_thin.h only: bytes between consecutive columns inside a tile
  // row (the element size, unless the launcher has swapped the operands and
  // with them the meaning of rows and columns), and whether the column scale
  // is applied before the row scale (again the swapped case, which must keep
  // the caller's order of the two multiplications).
  uint32_t out_sn0, acc_sn0;
  uint32_t col_scale_first;
  // mmt4d_mfma_persistent.h only: log2 of M0 and N0 (powers of two there).
  int32_t lm0, ln0;
  // mmt4d_mfma_thin.h only: K split over `kslices` workgroups per output block
  // (1 = none). Workgroup b works on block b / kslices, K slice b % kslices;
  // the slices' partial accumulators meet in `ws_partials` (kslices x 16 bytes
  // per lane and accumulator block, per output block) and the workgroup that
  // finds `ws_counters[block]` at kslices - 1 adds them up and stores. The
  // counters are zero between launches (the last workgroup resets its own).
  uint32_t kslices;
  char* ws_partials;
  uint32_t* ws_counters;
};

// Row-slot swizzle for the regrouping loaders (RB < 16): the eight lanes that
// store together write rows of the same residue mod 8 for different K slices;
// XOR-ing the slot with (2*slice + top row bit) spreads them over the eight
// 16-byte bank groups. Readers apply the same mask.
__device__ __forceinline__ uint32_t swizzle_mask(uint32_t ch, uint32_t hi) {
  return (2 * (ch & 3) + hi) & 7;
}

// Regroups R pieces (each: R rows x RB bytes of one K-tile) into R pieces
// (each: one row x 16 bytes over R K-tiles). in[t] is K-tile t; out[j] row j.
template <int RBC>
__device__ __forceinline__ void regroup(const v4i* in, v4i* out) {
  if constexpr (RBC == 8) {
    out[0] = v4i{in[0][0], in[0][1], in[1][0], in[1][1]};
    out[1] = v4i{in[0][2], in[0][3], in[1][2], in[1][3]};
  } else if constexpr (RBC == 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = v4i{in[0][j], in[1][j], in[2][j], in[3][j]};
  } else if constexpr (RBC == 2) {
    // Dword d of K-tile t holds rows 2d (low half) and 2d+1 (high half).
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        out[j][w] = (int)__builtin_amdgcn_perm((uint32_t)in[2 * w + 1][j >> 1],
                                               (uint32_t)in[2 * w][j >> 1], sel);
      }
    }
  } else {
    out[0] = in[0];
  }
}

// Workgroup -> output block. Consecutive workgroup ids go round-robin to the
// 8 XCDs, each with its own L2; give every XCD a contiguous share of the
// blocks and walk that share in bands of `band` block rows so that the
// workgroups resident on one XCD at a time reuse each other's panels.
__device__ __forceinline__ void block_of_workgroup(uint32_t wg, const Args& a,
                                                   int* bm, int* bn) {
  const uint32_t total = (uint32_t)a.grid_m * (uint32_t)a.grid_n;
  const uint32_t per_xcd = (total + 7) / 8;
  uint32_t id = (wg & 7) * per_xcd + (wg >> 3);
  if (id >= total || (total & 7)) id = wg;  // uneven split: plain order
  const uint32_t band_blocks = a.band * (uint32_t)a.grid_n;
  const uint32_t b = id / band_blocks;
  const uint32_t in_band = id - b * band_blocks;
  const uint32_t rows = min(a.band, (uint32_t)a.grid_m - b * a.band);
  const uint32_t col = in_band / rows;
  *bm = (int)(b * a.band + (in_band - col * rows));
  *bn = (int)col;
}

// TM x TN accumulator blocks per wave, WGM x WGN waves per workgroup, NKK MFMA
// K-groups per pipeline step, PIPE as described at the top of this file.
// RBC: 16 = row bytes >= 16 (direct), 8/4/2 = regrouping loaders.
template <Elem E, int RBC, int TM, int TN, int WGM, int WGN, int NKK, int PIPE>
__global__ __launch_bounds__(WGM* WGN * 64)
void mmt4d_mfma_kernel(Args a) {
  using TT = ElemTraits<E>;
  using Acc = typename TT::Acc;
  using Out = typename TT::Out;
  constexpr int OB = Out::kOutBytes;  // bytes per output element
  constexpr int NW = WGM * WGN;
  constexpr int HALVES = TT::kHalves;
  constexpr int NCHB = NKK * HALVES;       // groups of 4 chunks per step
  constexpr int NCH = NCHB * 4;            // 16-byte chunks per row per step
  constexpr int KS = NCH * 16;             // bytes of K per row per step
  constexpr int BM = WGM * TM * 16;
  constexpr int BN = WGN * TN * 16;
  constexpr int R = RBC >= 16 ? 1 : 16 / RBC;
  // A loader block is 64 units (one per lane); a unit is R loads + R stores.
  constexpr int BLOCKS_A = BM * NCH / R / 64;
  // PIPE 2 and 3 keep only the LHS in LDS; RHS fragments come straight from global.
  constexpr bool RHS_DIRECT = PIPE == 2 || PIPE == 3;
  constexpr int BLOCKS = (RHS_DIRECT ? BM : BM + BN) * NCH / R / 64;
  constexpr int NU = (BLOCKS + NW - 1) / NW;
  constexpr int IMAGE_A = BM * KS;
  constexpr int STAGE = (RHS_DIRECT ? BM : BM + BN) * KS;
  static_assert((BM * NCH / R) % 64 == 0 && (BN * NCH / R) % 64 == 0, "block split");
  // When the blocks do not divide evenly over the waves, the surplus (wave, i)
  // slots are idle: they load from a valid address and skip the store.
  constexpr bool EVEN = BLOCKS % NW == 0;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN;
  const int wn = wave - wm * WGN;
  int wg_m, wg_n;
  block_of_workgroup(blockIdx.x, a, &wg_m, &wg_n);
  const int pm0 = wg_m * a.bpm;  // first LHS panel of this workgroup
  const int pn0 = wg_n * a.bpn;
  const int lrb = a.lrb;
  const int kts_per_step = KS >> lrb;
  const uint32_t q = lane >> 4, r = lane & 15;

  // ---- loader set-up: per-unit constants --------------------------------
  // Operand choice, base pointer and strides depend on (wave, i) only and live
  // in scalar registers; per lane there is one 32-bit offset per unit.
  const char* sbase[NU];
  uint32_t voff[NU];     // byte offset of the unit's first piece at step 0
  uint32_t sstep[NU];    // bytes to advance per K step
  uint32_t skt[NU];      // bytes between consecutive loads of a unit
  int32_t kt0[NU];       // K-tile index of the first load at step 0
  uint32_t loff[NU];     // LDS offset (within a stage) of the unit's first store
  // Regrouping loaders only: false for a unit whose rows lie beyond the
  // operand's LDS image. That happens when the tile height does not divide
  // the block (e.g. M0 = 24 in a 64-row block: the units of a third, partial
  // panel would land on rows 48..71); such a unit loads but must not store.
  bool lds_ok[NU];
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int blk = wave + i * NW;
    const bool is_b = blk >= BLOCKS_A;
    const int xblk = is_b ? blk - BLOCKS_A : blk;
    const int X0 = is_b ? a.N0 : a.M0;
    const int X1 = is_b ? a.N1 : a.M1;
    const int px0 = is_b ? pn0 : pm0;
    const int bpx = is_b ? a.bpn : a.bpm;
    const int64_t xstride = is_b ? a.rhs_stride : a.lhs_stride;
    const uint32_t image = is_b ? IMAGE_A : 0;
    const uint32_t kt_bytes = (uint32_t)X0 << lrb;  // one K-tile of the panel
    sbase[i] = (is_b ? a.rhs : a.lhs) + (int64_t)px0 * xstride;
    sstep[i] = (uint32_t)kts_per_step * kt_bytes;
    int pl;
    if constexpr (RBC >= 16) {
      // Block = (row block, chunk group); lane (q, r) owns LDS slot `lane` and
      // fetches the piece that belongs there: row r of the block, chunk 4*cb+q.
      const int rbk = xblk / NCHB, cb = xblk - rbk * NCHB;
      const uint32_t row = (uint32_t)rbk * 16 + r;
      pl = (int)(row / (uint32_t)X0);
      const uint32_t m0 = row - (uint32_t)pl * X0;
      const uint32_t kb = (uint32_t)(cb * 4 + q) * 16;  // K byte of the chunk
      const uint32_t ktl = kb >> lrb;
      kt0[i] = (int32_t)ktl;
      voff[i] = (uint32_t)pl * (uint32_t)xstride + ktl * kt_bytes + (m0 << lrb) +
                (kb & ((1u << lrb) - 1));
      skt[i] = 0;
      lds_ok[i] = true;
      loff[i] = image + (uint32_t)xblk * 1024 + lane * 16;
    } else {
      // Units in order [panel][chunk g][row group]; the unit's R loads read
      // K-tiles g, g + NCH, g + 2*NCH, ... so that one load instruction covers
      // NCH consecutive K-tiles of a panel.
      const uint32_t u = (uint32_t)xblk * 64 + lane;
      const uint32_t groups = (uint32_t)X0 / R;
      const uint32_t t1 = u / groups;
      const uint32_t mg = u - t1 * groups;
      pl = (int)(t1 / NCH);
      const uint32_t g = t1 - (uint32_t)pl * NCH;
      kt0[i] = (int32_t)g;
      voff[i] = (uint32_t)pl * (uint32_t)xstride + g * kt_bytes + mg * 16;
      skt[i] = NCH * kt_bytes;
      const uint32_t row = (uint32_t)pl * X0 + mg * R;  // first of R rows
      lds_ok[i] = row + R <= (uint32_t)(is_b ? BN : BM);
      const uint32_t rr = row & 15;  // R divides 16: the R rows share a block
      // Slot of row rr + j is (rr + j) ^ mask; R <= 8 and rr % R == 0, so j
      // only touches the low bits and the store applies j ^ ... itself.
      loff[i] = image + (((row >> 4) * NCHB + (g >> 2)) * 64 + (g & 3) * 16) * 16 +
                ((rr & 8) | ((rr & 7) ^ swizzle_mask(g, rr >> 3))) * 16;
    }
    // Units outside the problem read from the start of the first panel.
    if (!(pl < bpx && px0 + pl < X1)) voff[i] = 0;
    if (!EVEN && blk >= BLOCKS) {
      sbase[i] = a.lhs + (int64_t)pm0 * a.lhs_stride;
      voff[i] = 0;
      sstep[i] = 0;
      skt[i] = 0;
    }

  }

  // ---- reader set-up ------------------------------------------------------
  uint32_t rd_slot[NCHB];
#pragma unroll
  for (int cb = 0; cb < NCHB; ++cb) {
    const uint32_t mask = RBC >= 16 ? 0u : swizzle_mask(cb * 4 + q, r >> 3);
    rd_slot[cb] = (q * 16 + (r ^ mask)) * 16;
  }
  const uint32_t rd_a = (uint32_t)(wm * TM) * NCHB * 1024;
  const uint32_t rd_b = IMAGE_A + (uint32_t)(wn * TN) * NCHB * 1024;

  // ---- accumulators -------------------------------------------------------
  // The MFMA takes the RHS fragment as its first operand, so lane (q, r) of
  // block (tm, tn) holds output row r, columns 4q..4q+3: four consecutive
  // elements of one row of the [M0][N0] output tile when N0 is a multiple of
  // four, which one 16-byte access moves (a wave then covers whole tiles
  // contiguously). `vec_out` is 0 when that does not hold or the output is not
  // 16-byte aligned; elements then move one by one.
  Acc acc[TM][TN];
  // Output element (row, col) of the workgroup's block, with pl = row / M0,
  // m0 = row % M0, pc = col / N0, n0 = col % N0, lives at
  //   out + (pm0 + pl) * out_stride + m0 * out_sm0 + (pn0 + pc) * out_spn + n0 * elem,
  // which covers both the tiled [M1][N1][M0][N0] output and a plain row-major
  // matrix (the fused mmt4d + unpack). Rows and columns at or beyond
  // out_rows / out_cols do not exist (row-major output of a ragged problem).
  auto for_each_output = [&](const char* base, int64_t s_panel, uint32_t s_m0, uint32_t s_pn,
                             auto f4, auto f1) {
    // The lane coordinates pass through an empty asm so that the address
    // arithmetic of the prologue (ACCUMULATE loads) and of the epilogue
    // (stores) is not shared: shared, it would stay live across the K loop.
    uint32_t oq = q, orr = r;
    asm volatile("" : "+v"(oq), "+v"(orr));
    char* out_base = const_cast<char*>(base) + (int64_t)pm0 * s_panel + (int64_t)pn0 * s_pn;
    const int row_origin = pm0 * a.M0, col_origin = pn0 * a.N0;
    if (a.vec_out) {
      uint32_t col_off[TN];
      int col_n[TN];  // how many of the 4 columns exist
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const int col = (wn * TN + tn) * 16 + 4 * (int)oq;
        const int pl = col / a.N0, n0 = col - pl * a.N0;
        const bool ok = pl < a.bpn && pn0 + pl < a.N1;
        const int left = a.out_cols - (col_origin + col);
        col_n[tn] = ok ? (left >= 4 ? 4 : (left > 0 ? left : 0)) : 0;
        col_off[tn] = (uint32_t)pl * s_pn + (uint32_t)n0 * OB;
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const int row = (wm * TM + tm) * 16 + (int)orr;
        const int pl = row / a.M0, m0 = row - pl * a.M0;
        const bool row_ok = pl < a.bpm && pm0 + pl < a.M1 && row_origin + row < a.out_rows;
        const uint32_t row_off = (uint32_t)pl * (uint32_t)s_panel + (uint32_t)m0 * s_m0;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          if (row_ok && col_n[tn] == 4) {
            f4(tm, tn, out_base + (row_off + col_off[tn]));
          } else if (row_ok && col_n[tn] > 0) {
            // the matrix ends inside this group of four columns
#pragma unroll
            for (int e = 0; e < 3; ++e)
              if (e < col_n[tn]) f1(tm, tn, e, out_base + (row_off + col_off[tn] + e * OB));
          }
        }
        // Keep the unrolled rows from being hoisted together.
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const int row = (wm * TM + tm) * 16 + (int)orr;
        const int pl = row / a.M0, m0 = row - pl * a.M0;
        const bool row_ok = pl < a.bpm && pm0 + pl < a.M1 && row_origin + row < a.out_rows;
        const uint32_t row_off = (uint32_t)pl * (uint32_t)s_panel + (uint32_t)m0 * s_m0;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int col = (wn * TN + tn) * 16 + 4 * (int)oq + e;
            const int pc = col / a.N0, n0 = col - pc * a.N0;
            if (row_ok && pc < a.bpn && pn0 + pc < a.N1 && col_origin + col < a.out_cols)
              f1(tm, tn, e, out_base + (row_off + (uint32_t)pc * s_pn + (uint32_t)n0 * OB));
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = Acc{0, 0, 0, 0};
  if (a.accumulate) {
    for_each_output(a.acc, a.acc_stride, a.acc_sm0, a.acc_spn,
                    [&](int tm, int tn, char* p) { acc[tm][tn] = Out::load4(p); },
                    [&](int tm, int tn, int e, char* p) { acc[tm][tn][e] = Out::load1(p); });
  }

  // ---- pipeline -----------------------------------------------------------
  // Loads are unconditional in the steady state: units outside the problem
  // read (valid) bytes of the workgroup's first panel, and what they bring
  // only ever reaches accumulator rows or columns that are never stored.
  // `tail` marks the one step in which K-tiles past K1 must read as zero.
  auto load_piece = [&](int i, uint32_t off) {
    return *reinterpret_cast<const v4i_g*>(sbase[i] + off);
  };
  auto load_global = [&](v4i (&dst)[NU][R], int step, bool tail) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const uint32_t off = voff[i] + (uint32_t)step * sstep[i];
      const int kt = step * kts_per_step + kt0[i];
#pragma unroll
      for (int t = 0; t < R; ++t) {
        if (!tail) {
          dst[i][t] = load_piece(i, off + t * skt[i]);
        } else {
          const bool ok = (kt + t * NCH) < a.K1;
          const v4i v = load_piece(i, ok ? off + t * skt[i] : 0u);
          dst[i][t] = ok ? v : v4i{0, 0, 0, 0};
        }
      }
    }
  };
  auto store_lds = [&](const v4i (&src)[NU][R], uint32_t stage_off) {
    char* base = lds + stage_off;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      if (!EVEN && wave + i * NW >= BLOCKS) continue;
      if (RBC < 16 && !lds_ok[i]) continue;
      if constexpr (RBC >= 16) {
        *reinterpret_cast<v4i*>(base + loff[i]) = src[i][0];
      } else {
        v4i outp[R];
        regroup<RBC>(src[i], outp);
#pragma unroll
        for (int j = 0; j < R; ++j) {
          // Row rr + j sits at slot low bits (rr ^ mask) ^ j.
          *reinterpret_cast<v4i*>(base + (loff[i] ^ (uint32_t)(j * 16))) = outp[j];
        }
      }
    }
  };
  auto read_frags = [&](v4i (&fa)[TM][HALVES], v4i (&fb)[TN][HALVES], uint32_t stage_off,
                        int kk) {
    const char* base = lds + stage_off;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        fa[tm][h] = *reinterpret_cast<const v4i*>(
            base + rd_a + (tm * NCHB + kk * HALVES + h) * 1024 + rd_slot[kk * HALVES + h]);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        fb[tn][h] = *reinterpret_cast<const v4i*>(
            base + rd_b + (tn * NCHB + kk * HALVES + h) * 1024 + rd_slot[kk * HALVES + h]);
  };
  auto mfmas = [&](const v4i (&fa)[TM][HALVES], const v4i (&fb)[TN][HALVES]) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = TT::mfma(fb[tn], fa[tm], acc[tm][tn]);
  };
  // The same sweep column by column (consecutive instructions share the RHS
  // fragment): what the LDS-direct pipeline's compute phases issue. Measured
  // against the row-by-row sweep in alternating processes on one box, three
  // pairs: s8 8192^3 374.8 / 378.9 / 376.4 -> 371.7 / 371.7 / 375.2 us,
  // 16x16x2 382.0 / 382.5 / 384.5 -> 378.5 / 379.4 / 382.2, f16 4096^3 91.2 /
  // 91.3 / 91.3 -> 90.8 / 90.7 / 90.6, bf16 8192^3 unchanged.
  auto mfmas_by_columns = [&](const v4i (&fa)[TM][HALVES], const v4i (&fb)[TN][HALVES]) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tm][tn] = TT::mfma(fb[tn], fa[tm], acc[tm][tn]);
  };
  const int last = a.steps - 1;
  const bool has_tail = a.tail != 0;

  if constexpr (PIPE == 0) {
    // Two LDS stages; each step: issue next global loads, compute, store, barrier.
    v4i regs[NU][R];
    load_global(regs, 0, has_tail && last == 0);
    store_lds(regs, 0);
    __syncthreads();
    for (int s = 0; s < a.steps; ++s) {
      const uint32_t cur = (s & 1) * STAGE;
      if (s < last) {
        if (has_tail && s + 1 == last) load_global(regs, s + 1, true);
        else load_global(regs, s + 1, false);
      }
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        v4i fa[TM][HALVES], fb[TN][HALVES];
        read_frags(fa, fb, cur, kk);
        mfmas(fa, fb);
      }
      if (s < last) store_lds(regs, cur ^ STAGE);
      __syncthreads();
    }
  } else if constexpr (PIPE == 4) {
    // Two LDS stages as in PIPE 0, three register sets: iteration s issues the
    // global loads of step s+3 into the set that step s occupied, computes
    // step s from LDS and stores step s+1 (loaded two iterations ago) for the
    // next iteration. Unrolled by three so that the set index is static.
    constexpr int D = 3;
    v4i regs[D][NU][R];
    // Workgroups walk K from different starting steps (the sum over K is
    // order-free for the instruction): in lockstep from step 0 they would all
    // read the same offset of their panels at the same time, and panels are a
    // power-of-two distance apart, which concentrates the requests on a few
    // memory channels. Integer accumulators only: there the order cannot
    // show in the result, while float sums would differ between workgroups.
    const int rot = std::is_same<Acc, v4i>::value ? (int)(blockIdx.x % (uint32_t)a.steps) : 0;
    auto load_step = [&](v4i (&dst)[NU][R], int s) {
      int ks = s + rot;
      if (ks >= a.steps) ks -= a.steps;
      if (has_tail && ks == last) load_global(dst, ks, true);
      else load_global(dst, ks, false);
    };
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (d <= last) load_step(regs[d], d);
    }
    store_lds(regs[0], 0);
    __syncthreads();
    auto iteration = [&](int s, auto phase) {
      constexpr int P = decltype(phase)::value;
      const uint32_t cur = (s & 1) * STAGE;
      if (s + D <= last) load_step(regs[P], s + D);
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        v4i fa[TM][HALVES], fb[TN][HALVES];
        read_frags(fa, fb, cur, kk);
        mfmas(fa, fb);
      }
      if (s < last) store_lds(regs[(P + 1) % D], cur ^ STAGE);
      __syncthreads();
    };
    int s = 0;
    for (; s + 2 < a.steps; s += 3) {
      iteration(s, std::integral_constant<int, 0>{});
      iteration(s + 1, std::integral_constant<int, 1>{});
      iteration(s + 2, std::integral_constant<int, 2>{});
    }
    if (s < a.steps) iteration(s, std::integral_constant<int, 0>{});
    if (s + 1 < a.steps) iteration(s + 1, std::integral_constant<int, 1>{});
  } else if constexpr (PIPE == 1) {
    // Three LDS stages, two register sets. In iteration s a wave runs the
    // MFMAs of step s row by row (tm) and, between rows, issues everything
    // that does not depend on them: the global loads of step s+3, the LDS
    // stores of step s+2 (loaded during iteration s-1) into stage (s+2)%3,
    // the LHS fragments of the next row, and one RHS fragment of step s+1
    // from stage (s+1)%3. K must be a whole number of steps here (no tail).
    static_assert(NKK == 1, "pipelined variant steps one MFMA K-group at a time");
    static_assert(TM % 2 == 0, "LHS fragment slots alternate by row parity");
    constexpr int NP = NU * R;  // 16-byte pieces per thread per step
    v4i regs[2][NU][R];
    v4i fa[2][HALVES], fb[2][TN][HALVES];
    auto read_a = [&](v4i (&dst)[HALVES], uint32_t stage_off, int tm) {
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        dst[h] = *reinterpret_cast<const v4i*>(lds + stage_off + rd_a +
                                               (tm * NCHB + h) * 1024 + rd_slot[h]);
    };
    auto read_b = [&](v4i (&dst)[HALVES], uint32_t stage_off, int tn) {
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        dst[h] = *reinterpret_cast<const v4i*>(lds + stage_off + rd_b +
                                               (tn * NCHB + h) * 1024 + rd_slot[h]);
    };
    load_global(regs[0], 0, false);
    store_lds(regs[0], 0);
    load_global(regs[0], min(1, last), false);
    store_lds(regs[0], STAGE);
    load_global(regs[1], min(2, last), false);
    __syncthreads();
    read_a(fa[0], 0, 0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) read_b(fb[0][tn], 0, tn);
    uint32_t st_cur = 0, st_next = STAGE, st_write = 2 * STAGE;
    auto iteration = [&](int s, auto parity) {
      constexpr int P = decltype(parity)::value;
      const int ld_step = min(s + 3, last);
      v4i outp[NU][R];
      if constexpr (RBC < 16) {
#pragma unroll
        for (int i = 0; i < NU; ++i) regroup<RBC>(regs[P ^ 1][i], outp[i]);
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        // Stores of step s+2 and loads of step s+3, an even share per row.
#pragma unroll
        for (int k = tm * NP / TM; k < (tm + 1) * NP / TM; ++k) {
          const int i = k / R, j = k % R;
          if (!EVEN && wave + i * NW >= BLOCKS) continue;
          if (RBC < 16 && !lds_ok[i]) continue;
          char* dst = lds + st_write + (RBC >= 16 ? loff[i] : (loff[i] ^ (uint32_t)(j * 16)));
          *reinterpret_cast<v4i*>(dst) = RBC >= 16 ? regs[P ^ 1][i][0] : outp[i][j];
        }
#pragma unroll
        for (int k = tm * NP / TM; k < (tm + 1) * NP / TM; ++k) {
          const int i = k / R, t = k % R;
          regs[P][i][t] = load_piece(i, voff[i] + (uint32_t)ld_step * sstep[i] + t * skt[i]);
        }
        // Fragments: LHS of the next row (or of row 0 of step s+1), and this
        // row's share of the RHS fragments of step s+1.
        if (tm + 1 < TM) read_a(fa[(tm + 1) & 1], st_cur, tm + 1);
        else read_a(fa[0], st_next, 0);
#pragma unroll
        for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn)
          read_b(fb[P ^ 1][tn], st_next, tn);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = TT::mfma(fb[P][tn], fa[tm & 1], acc[tm][tn]);
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
      const uint32_t t = st_cur;
      st_cur = st_next;
      st_next = st_write;
      st_write = t;
    };
    int s = 0;
    for (; s + 1 < a.steps; s += 2) {
      iteration(s, std::integral_constant<int, 0>{});
      iteration(s + 1, std::integral_constant<int, 1>{});
    }
    if (s < a.steps) iteration(s, std::integral_constant<int, 0>{});
  }
  else if constexpr (PIPE == 2) {
    // LHS through three LDS stages as in PIPE 1; RHS fragments are loaded by
    // each wave straight from global memory into registers, one step ahead:
    // a 16-byte piece of a tile row IS the lane's MFMA operand when RB >= 16.
    // This halves the LDS traffic per MFMA, which is what bounds PIPE 1. The
    // waves that share a column block re-read the same lines from L1/L2.
    static_assert(RBC >= 16, "register-direct RHS needs row bytes >= 16");
    static_assert(NKK == 1 && TM % 2 == 0, "see PIPE 1");
    constexpr int NP = NU;  // 16-byte LHS pieces per thread per step
    v4i regs[2][NU][R];
    v4i fa[2][HALVES], fb[2][TN][HALVES];
    const char* sbase_b = a.rhs + (int64_t)pn0 * a.rhs_stride;
    const uint32_t kt_bytes_b = (uint32_t)a.N0 << lrb;
    const uint32_t sstep_b = (uint32_t)kts_per_step * kt_bytes_b;
    uint32_t voff_b[TN][HALVES];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint32_t row = (uint32_t)(wn * TN + tn) * 16 + r;
      const uint32_t pl = row / (uint32_t)a.N0;
      const uint32_t n0 = row - pl * a.N0;
      const bool ok = (int)pl < a.bpn && pn0 + (int)pl < a.N1;
#pragma unroll
      for (int h = 0; h < HALVES; ++h) {
        const uint32_t kb = (uint32_t)(h * 4 + q) * 16;
        voff_b[tn][h] = ok ? pl * (uint32_t)a.rhs_stride + (kb >> lrb) * kt_bytes_b +
                                 (n0 << lrb) + (kb & ((1u << lrb) - 1))
                           : 0u;
      }
    }
    auto load_b = [&](v4i (&dst)[HALVES], int tn, int step) {
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        dst[h] = *reinterpret_cast<const v4i_g*>(sbase_b + (voff_b[tn][h] + (uint32_t)step * sstep_b));
    };
    auto read_a = [&](v4i (&dst)[HALVES], uint32_t stage_off, int tm) {
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        dst[h] = *reinterpret_cast<const v4i*>(lds + stage_off + rd_a +
                                               (tm * NCHB + h) * 1024 + rd_slot[h]);
    };
    load_global(regs[0], 0, false);
    store_lds(regs[0], 0);
    load_global(regs[0], min(1, last), false);
    store_lds(regs[0], STAGE);
    // What iteration -1 would have left in flight, in the loop's own issue
    // order (see PIPE 3 below for why the order matters).
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn) load_b(fb[0][tn], tn, 0);
#pragma unroll
      for (int k = tm * NP / TM; k < (tm + 1) * NP / TM; ++k)
        regs[1][k][0] = load_piece(k, voff[k] + (uint32_t)min(2, last) * sstep[k]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    read_a(fa[0], 0, 0);
    uint32_t st_cur = 0, st_next = STAGE, st_write = 2 * STAGE;
    auto iteration = [&](int s, auto parity) {
      constexpr int P = decltype(parity)::value;
      const int ld_step = min(s + 3, last);
      const int b_step = min(s + 1, last);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
        for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn) {
          load_b(fb[P ^ 1][tn], tn, b_step);
        }
#pragma unroll
        for (int k = tm * NP / TM; k < (tm + 1) * NP / TM; ++k) {
          *reinterpret_cast<v4i*>(lds + st_write + loff[k]) = regs[P ^ 1][k][0];
          regs[P][k][0] = load_piece(k, voff[k] + (uint32_t)ld_step * sstep[k]);
        }
        if (tm + 1 < TM) read_a(fa[(tm + 1) & 1], st_cur, tm + 1);
        else read_a(fa[0], st_next, 0);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = TT::mfma(fb[P][tn], fa[tm & 1], acc[tm][tn]);
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
      const uint32_t t = st_cur;
      st_cur = st_next;
      st_next = st_write;
      st_write = t;
    };
    int s = 0;
    for (; s + 1 < a.steps; s += 2) {
      iteration(s, std::integral_constant<int, 0>{});
      iteration(s + 1, std::integral_constant<int, 1>{});
    }
    if (s < a.steps) iteration(s, std::integral_constant<int, 0>{});
  }

  else if constexpr (PIPE == 3) {
    // As PIPE 2 with every prefetch one step deeper, unrolled by three so that
    // LDS stage, register set and fragment buffer indices are all the
    // compile-time phase P = s % 3:
    //   iteration s computes step s from LDS stage P and RHS buffer P,
    //   issues the LHS global loads of step s+4 into register set (P+1)%3,
    //   stores register set (P+2)%3 (step s+2, loaded in iteration s-2) to
    //   LDS stage (P+2)%3, and loads the RHS fragments of step s+2 into
    //   buffer (P+2)%3. LHS fragments are fetched two rows ahead through a
    //   ring of three (an LDS read then has eight MFMAs to arrive in, not four).
    static_assert(RBC >= 16, "register-direct RHS needs row bytes >= 16");
    static_assert(NKK == 1 && TM % 2 == 0, "see PIPE 1");
    constexpr int NP = NU;
    constexpr int FR = 3;  // LHS fragment ring: row tm of phase P sits in slot (P * TM + tm) % 3
    v4i regs[3][NU][R];
    v4i fa[FR][HALVES], fb[3][TN][HALVES];
    const char* sbase_b = a.rhs + (int64_t)pn0 * a.rhs_stride;
    const uint32_t kt_bytes_b = (uint32_t)a.N0 << lrb;
    const uint32_t sstep_b = (uint32_t)kts_per_step * kt_bytes_b;
    uint32_t voff_b[TN][HALVES];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint32_t row = (uint32_t)(wn * TN + tn) * 16 + r;
      const uint32_t pl = row / (uint32_t)a.N0;
      const uint32_t n0 = row - pl * a.N0;
      const bool ok = (int)pl < a.bpn && pn0 + (int)pl < a.N1;
#pragma unroll
      for (int h = 0; h < HALVES; ++h) {
        const uint32_t kb = (uint32_t)(h * 4 + q) * 16;
        voff_b[tn][h] = ok ? pl * (uint32_t)a.rhs_stride + (kb >> lrb) * kt_bytes_b +
                                 (n0 << lrb) + (kb & ((1u << lrb) - 1))
                           : 0u;
      }
    }
    auto load_b = [&](v4i (&dst)[HALVES], int tn, int step) {
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        dst[h] = *reinterpret_cast<const v4i_g*>(sbase_b + (voff_b[tn][h] + (uint32_t)step * sstep_b));
    };
    auto read_a = [&](v4i (&dst)[HALVES], uint32_t stage_off, int tm) {
#pragma unroll
      for (int h = 0; h < HALVES; ++h)
        dst[h] = *reinterpret_cast<const v4i*>(lds + stage_off + rd_a +
                                               (tm * NCHB + h) * 1024 + rd_slot[h]);
    };
    load_global(regs[0], 0, false);
    load_global(regs[1], min(1, last), false);
    store_lds(regs[0], 0);
    store_lds(regs[1], STAGE);
    // What iterations -2 and -1 would have left in flight, issued in the order
    // in which the loop issues it (RHS fragments and LHS pieces interleaved
    // row by row). The order matters: the wait counters are in-order, and the
    // waits the compiler places in the loop must hold on entry from here as
    // well as around the back edge. Were the fragments of steps 0 and 1 the
    // newest loads here, the first phase of the loop would wait for nearly
    // everything in flight, every third step.
    auto issue_like_iteration = [&](auto bbuf, int b_step, auto aset, int a_step) {
      constexpr int BB = decltype(bbuf)::value, AS = decltype(aset)::value;
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
        for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn) load_b(fb[BB][tn], tn, b_step);
#pragma unroll
        for (int k = tm * NP / TM; k < (tm + 1) * NP / TM; ++k)
          regs[AS][k][0] = load_piece(k, voff[k] + (uint32_t)a_step * sstep[k]);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    issue_like_iteration(std::integral_constant<int, 0>{}, 0, std::integral_constant<int, 2>{},
                         min(2, last));
    issue_like_iteration(std::integral_constant<int, 1>{}, min(1, last),
                         std::integral_constant<int, 0>{}, min(3, last));
    __syncthreads();
    read_a(fa[0], 0, 0);
    read_a(fa[1], 0, 1);
    auto iteration = [&](int s, auto phase) {
      constexpr int P = decltype(phase)::value;
      constexpr uint32_t st_cur = P * STAGE, st_next = ((P + 1) % 3) * STAGE,
                         st_write = ((P + 2) % 3) * STAGE;
      const int ld_step = min(s + 4, last);
      const int b_step = min(s + 2, last);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
        for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn)
          load_b(fb[(P + 2) % 3][tn], tn, b_step);
#pragma unroll
        for (int k = tm * NP / TM; k < (tm + 1) * NP / TM; ++k) {
          *reinterpret_cast<v4i*>(lds + st_write + loff[k]) = regs[(P + 2) % 3][k][0];
          regs[(P + 1) % 3][k][0] = load_piece(k, voff[k] + (uint32_t)ld_step * sstep[k]);
        }
        if (tm + 2 < TM) read_a(fa[(P * TM + tm + 2) % FR], st_cur, tm + 2);
        else read_a(fa[(P * TM + tm + 2) % FR], st_next, tm + 2 - TM);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] = TT::mfma(fb[P][tn], fa[(P * TM + tm) % FR], acc[tm][tn]);
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
    };
    int s = 0;
    for (; s + 2 < a.steps; s += 3) {
      iteration(s, std::integral_constant<int, 0>{});
      iteration(s + 1, std::integral_constant<int, 1>{});
      iteration(s + 2, std::integral_constant<int, 2>{});
    }
    if (s < a.steps) iteration(s, std::integral_constant<int, 0>{});
    if (s + 1 < a.steps) iteration(s + 1, std::integral_constant<int, 1>{});
  }
  else if constexpr (PIPE == 5) {
    // Both operands through LDS by LDS-direct loads, two wave groups half a
    // step apart. A wave raises its priority (s_setprio) for its compute phase:
    // the SIMD then issues its MFMAs ahead of the address arithmetic, fragment
    // reads and loads of the wave that shares the SIMD and is in its memory
    // phase, which has the whole phase for them (measured in one process,
    // launches alternating: s8 8192^3 388 -> 380 us, bf16 8192^3 734 -> 707,
    // f16 4096^3 96.7 -> 94.3, f8 8192^3 362 -> 360, s16 4096^3 289 -> 288).
    // Phase k of the workgroup (a barrier ends each phase):
    //   group 0: memory phase of step k/2 when k is even, compute phase when odd;
    //   group 1: the same one phase later (it passes one extra barrier first,
    //            group 0 one extra at the end).
    // Memory phase of step s: read the step's fragments from stage s % NS,
    // issue the loads of step s + NS - 1 into stage (s - 1) % NS, wait until the
    // wave's own loads of step s + 1 have landed and its fragment reads have
    // returned. The barrier that follows makes that true of every wave before
    // anyone reads step s + 1 (its memory phase is at least one barrier away),
    // and every wave has finished reading stage (s - 1) % NS before the first
    // load into it is issued (their memory phases of step s - 1 ended at an
    // earlier barrier). Past the last step the loads repeat the last step into
    // a stage nobody reads any more, which keeps the in-flight count the waits
    // assume.
    //
    // Tile rows of 16 bytes and more: a 1 KiB block of the LDS image (16 rows x
    // 64 bytes of K) is the MFMA fragment as it is. Tile rows of 2 or 4 bytes
    // (the reference's x86 tiles 16x16x2 of s8 and bf16): the loads copy the
    // K-tiles as they lie in memory, 16 rows x RB bytes each, one after the
    // other ([K-tile][row][RB]: again 1 KiB per 16-row block and step, a
    // 16-byte piece holding 16 / RB rows of one K-tile), and the fragment reads
    // gather a row's pieces:
    //   RB = 8  lane (q, r) reads the 8 bytes of row r in K-tiles q and q + 4
    //           (one ds_read2_b64);
    //   RB = 4  lane (q, r) reads the dwords of row r in K-tiles q, q + 4,
    //           q + 8, q + 12 (two ds_read2st64_b32);
    //   RB = 2  two transposing reads (ds_read_b64_tr_b16). Within a block of 16
    //           lanes, lane i receives as element j the element i % 4 of what
    //           lane 4 j + i / 4 addressed: lane (q, s) addresses rows
    //           4 (s % 4) .. + 3 of K-tile 16 h + 4 q + s / 4 (eight contiguous
    //           bytes) and lane (q, r) receives row r of K-tiles 16 h + 4 q .. + 3.
    // Which K bytes of a step meet in which lane operand is the same for both
    // operands, which is all the sum over K needs.
    // A step of NKK x 64 bytes of K holds NKK such blocks per 16 rows, one
    // after the other ([row block][64-byte chunk of K]).
    static_assert(RBC >= 16 || RBC == 2 || RBC == 4 || RBC == 8,
                  "1 KiB blocks of 16 rows x 64 bytes of K");
    static_assert(NW == 8, "two groups of four waves");
    // Lane operands of two 16-byte pieces (the 8-bit floats: 128 bytes of K per
    // step, i.e. two 64-byte halves) do not leave room for four stages of whole
    // steps: their LDS is a ring of half-step slots instead (HALVES == 2
    // below).
    constexpr int NS = kStages5;
    constexpr int IW = HALVES == 2 ? 4 : NW;          // waves that share one issue of loads
    constexpr int DCH = HALVES == 2 ? 1 : NCHB;       // 64-byte chunks of K per issue
    constexpr int DB = (BM + BN) / 16 * DCH;          // 1 KiB blocks per issue
    static_assert(DB % IW == 0, "blocks split evenly over the issuing waves");
    constexpr int DU = DB / IW;
    const int group = wave >> 2;
    const char* d_base[DU];
    uint32_t d_voff[DU], d_step[DU], d_half[DU], d_lds[DU];
#pragma unroll
    for (int i = 0; i < DU; ++i) {
      const int blk = (wave & (IW - 1)) + i * IW;
      const bool is_b = blk >= BM / 16 * DCH;
      const int xblk = is_b ? blk - BM / 16 * DCH : blk;   // (row block, 64-byte chunk) of the operand's image
      const int rbk = xblk / DCH, chunk = xblk - rbk * DCH;
      const int X0 = is_b ? a.N0 : a.M0;
      const int X1 = is_b ? a.N1 : a.M1;
      const int px0 = is_b ? pn0 : pm0;
      const int bpx = is_b ? a.bpn : a.bpm;
      const int64_t xstride = is_b ? a.rhs_stride : a.lhs_stride;
      const uint32_t kt_bytes = (uint32_t)X0 << lrb;
      uint32_t pl;
      if constexpr (RBC >= 16) {
        // Lane (q, r): row r of the block, bytes 16 q .. 16 q + 15 of the chunk.
        const uint32_t row = (uint32_t)rbk * 16 + r;
        pl = row / (uint32_t)X0;
        const uint32_t x0 = row - pl * (uint32_t)X0;
        const uint32_t kb = (uint32_t)(chunk * 4 + q) * 16;
        d_voff[i] = pl * (uint32_t)xstride + (kb >> lrb) * kt_bytes + (x0 << lrb) + (kb & ((1u << lrb) - 1));
      } else {
        constexpr int RP = 16 / RBC;   // rows of a K-tile in one 16-byte piece
        constexpr int PPK = 16 / RP;   // pieces per K-tile of a 16-row block
        const uint32_t row0 = (uint32_t)rbk * 16 + ((uint32_t)lane % PPK) * RP;
        pl = row0 / (uint32_t)X0;
        const uint32_t x0 = row0 - pl * (uint32_t)X0;
        const uint32_t kt_l = (uint32_t)chunk * (64 / RBC) + (uint32_t)lane / PPK;  // K-tile within the step
        d_voff[i] = pl * (uint32_t)xstride + kt_l * kt_bytes + x0 * RBC;
      }
      if (!((int)pl < bpx && px0 + (int)pl < X1)) d_voff[i] = 0;  // rows beyond the problem: valid bytes, never stored
      d_base[i] = (is_b ? a.rhs : a.lhs) + (int64_t)px0 * xstride;
      d_step[i] = (uint32_t)kts_per_step * kt_bytes;
      // From the first to the second 64-byte half of a 128-byte step: further
      // along the tile row when it holds both, else on to later K-tiles.
      d_half[i] = a.rb >= 128 ? 64u : (uint32_t)(64 >> lrb) * kt_bytes;
      d_lds[i] = (is_b ? (uint32_t)BM * 64 * DCH : 0u) + (uint32_t)xblk * 1024;
    }
    // Loads of one issue: `step` and `half` (0 / 1, HALVES == 2 only) select the K bytes.
    auto issue_dma = [&](uint32_t lds_off, int step, int half) {
#pragma unroll
      for (int i = 0; i < DU; ++i) {
        uint32_t o = d_voff[i] + (uint32_t)step * d_step[i] + (half ? d_half[i] : 0u);
        // (kept as scalar base + 32-bit lane offset: see mmt4d_mfma_persistent.h)
        asm volatile("" : "+v"(o));
        __builtin_amdgcn_global_load_lds((glb_ptr_t)(d_base[i] + o),
                                         (lds_ptr_t)(lds + lds_off + d_lds[i]), 16, 0, 0);
      }
    };
    // Lane offset of a fragment read within its 1 KiB block.
    const uint32_t frag_lane = RBC >= 16 ? (uint32_t)lane * 16
                               : RBC == 8 ? q * 128 + r * 8
                               : RBC == 4 ? q * 64 + r * 4
                                          : (4 * q + (r >> 2)) * 32 + (r & 3) * 8;
    auto read_frag = [&](uint32_t block_off) -> v4i {
      const char* p = lds + block_off + frag_lane;
      if constexpr (RBC >= 16) {
        return *reinterpret_cast<const v4i*>(p);
      } else if constexpr (RBC == 8) {
        typedef int v2i __attribute__((ext_vector_type(2)));
        const v2i* w = reinterpret_cast<const v2i*>(p);
        const v2i lo = w[0], hi = w[64];
        return v4i{lo[0], lo[1], hi[0], hi[1]};
      } else if constexpr (RBC == 4) {
        const int* w = reinterpret_cast<const int*>(p);
        return v4i{w[0], w[64], w[128], w[192]};
      } else {
        // Written as assembly: the compiler does not track what the LDS-direct
        // loads write and would make the builtin form of this read wait for
        // every load in flight. The kernel waits for these reads itself
        // (wait_lds_reads before the phase's barrier; nothing uses the
        // registers before it).
        typedef int v2i __attribute__((ext_vector_type(2)));
        v2i lo, hi;
        const uint32_t addr = (uint32_t)(uintptr_t)p;  // LDS addresses are the low 32 bits
        asm volatile("ds_read_b64_tr_b16 %0, %2\n\tds_read_b64_tr_b16 %1, %2 offset:512"
                     : "=&v"(lo), "=&v"(hi) : "v"(addr) : "memory");
        return v4i{lo[0], lo[1], hi[0], hi[1]};
      }
    };
    if constexpr (HALVES == 2) {
      // A ring of RING = 2 D + 1 slots of half a step (64 bytes of K: (BM + BN) *
      // 64 bytes of LDS); half-step j (step j / 2, half j % 2) lives in slot
      // j % RING. In its memory phase of step s a wave reads both halves of the
      // step; group 0 then issues the whole half-step 2 s + RING - 2 (the slot of
      // half-step 2 s - 2, which group 1 finished reading a phase ago), group 1
      // the half-step 2 s + RING - 1 (the slot of 2 s - 1). Both groups thus bring
      // half of every step (group 0 the second halves, group 1 the first), each
      // in its own memory phase, D - 1 and D steps ahead; each waits, one barrier
      // before the first read of the half-step its group brought for step s + 1,
      // until only what it issued later is still in flight: group 0 at the end
      // of its compute phase (D - 2 issues), group 1 at the end of its memory
      // phase (D - 1 issues).
      static_assert(NKK == 1, "one MFMA K-group per step");
      constexpr int RING = ring_slots<E, BM, BN>();
      constexpr int D = (RING - 1) / 2;
      constexpr uint32_t SLOT = (BM + BN) * 64;
      constexpr uint32_t IMG_B = BM * 64;
      // Half-steps 0 .. RING - 3 before the first phase: group 1 brings the even
      // ones, group 0 the odd ones.
      if (group == 0) {
#pragma unroll
        for (int j = 1; j <= RING - 4; j += 2) issue_dma((uint32_t)j * SLOT, min(j / 2, last), 1);
      } else {
#pragma unroll
        for (int j = 0; j <= RING - 3; j += 2) issue_dma((uint32_t)j * SLOT, min(j / 2, last), 0);
      }
      wait_vmem_in_flight<0>();
      __builtin_amdgcn_s_barrier();
      v4i fa[TM][HALVES], fb[TN][HALVES];
      if constexpr (E == Elem::kS16) {
        // The 16-bit integers read the fragments of a step a phase ahead of its
        // memory phase (see their step below): those of step 0 here.
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          fa[tm][0] = read_frag((uint32_t)(wm * TM + tm) * 1024);
          fa[tm][1] = read_frag(SLOT + (uint32_t)(wm * TM + tm) * 1024);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          fb[tn][0] = read_frag(IMG_B + (uint32_t)(wn * TN + tn) * 1024);
          fb[tn][1] = read_frag(SLOT + IMG_B + (uint32_t)(wn * TN + tn) * 1024);
        }
      }
      if (group == 1) __builtin_amdgcn_s_barrier();
      // ---- 16-bit integers -------------------------------------------------
      // With a = 256 ah + al + 128 (ah the signed high byte, al the low byte
      // minus 128, both in [-128, 127]) and b likewise,
      //   sum a b = 65536 sum ah bh + 256 sum (ah bl + al bh) + sum al bl
      //             + 128 (sum a + sum b) - 16384 K,
      // all of it modulo 2^32: three accumulator sets fed by four 8-bit integer
      // MFMAs per block and step (the low x low products go to `acc`, on top of
      // the caller's accumulators), and the row sums of both operands, which
      // the vector ALUs add up with v_dot2_i32_i16 against (1, 1) in the memory
      // phase. A fragment is shared by the waves of a block row (column); each
      // of them sums one fragment in WGN (WGM) and the sums are exchanged
      // through LDS once the K loop is done.
      constexpr bool S16 = E == Elem::kS16;
      v4i hh[S16 ? TM : 1][S16 ? TN : 1], mid[S16 ? TM : 1][S16 ? TN : 1];
      int rsa[S16 ? TM : 1], rsb[S16 ? TN : 1];
      if constexpr (S16) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          rsa[tm] = 0;
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) hh[tm][tn] = mid[tm][tn] = v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) rsb[tn] = 0;
      }
      auto row_sum16 = [&](const v4i (&f)[HALVES], int sum) {
        typedef short v2s __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int h = 0; h < HALVES; ++h)
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            // (a copy first: a bit cast applied to the vector element itself
            // reads element 0 whatever the index)
            const int word = f[h][w];
            sum = __builtin_amdgcn_sdot2(__builtin_bit_cast(v2s, word), v2s{1, 1}, sum, false);
          }
        return sum;
      };
      // The sixteen elements of one row in f[0], f[1] -> their high bytes, or
      // their low bytes minus 128. The order of the sixteen is the same in both
      // and for both operands, which is all the sum over K needs.
      auto high_bytes = [&](const v4i (&f)[HALVES]) {
        v4i hi;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int w = 0; w < 2; ++w)
            hi[2 * h + w] = (int)__builtin_amdgcn_perm((uint32_t)f[h][2 * w + 1], (uint32_t)f[h][2 * w], 0x07050301u);
        return hi;
      };
      auto low_bytes = [&](const v4i (&f)[HALVES]) {
        v4i lo;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int w = 0; w < 2; ++w)
            lo[2 * h + w] = (int)(__builtin_amdgcn_perm((uint32_t)f[h][2 * w + 1], (uint32_t)f[h][2 * w], 0x06040200u) ^
                                  0x80808080u);
        return lo;
      };
      v4i ha[S16 ? TM : 1], hb[S16 ? TN : 1];
      // The fragment reads of a step, both halves of each fragment.
      auto read_frags16 = [&](uint32_t slot0, uint32_t slot1) __attribute__((always_inline)) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          fa[tm][0] = read_frag(slot0 + (uint32_t)(wm * TM + tm) * 1024);
          fa[tm][1] = read_frag(slot1 + (uint32_t)(wm * TM + tm) * 1024);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          fb[tn][0] = read_frag(slot0 + IMG_B + (uint32_t)(wn * TN + tn) * 1024);
          fb[tn][1] = read_frag(slot1 + IMG_B + (uint32_t)(wn * TN + tn) * 1024);
        }
      };
      // A step of the 16-bit integers. A wave issues one instruction per turn of
      // its SIMD (every fourth cycle), and this kernel has some 200 of them per
      // wave and step (32 MFMAs, 100 vector ALU instructions for the byte split
      // and the row sums, 24 LDS reads, the loads, scalar bookkeeping) against
      // 128 turns in the 512 cycles its MFMAs take: it is bound by instruction
      // issue, not by the matrix pipe. What helps is to spread the instructions
      // evenly over the two phases. A memory phase made of reads, then permutes,
      // is the longer one by far, so the reads move: a wave issues the reads of step s + 1
      // in the middle of its compute phase of step s, once the low bytes of
      // step s are out of the raw fragments (the same registers take the new
      // ones), and they return under the second half of its MFMAs. The memory
      // phase is then: issue of the loads, high bytes, row sums.
      //   compute phase: high x high and high x low products (need what the
      //   memory phase prepared, and the low bytes of the LHS) with the low
      //   bytes worked out beside them, three vector ALU instructions under each
      //   MFMA; then the fragment reads beside the low x low and low x high
      //   products. Products that share an accumulator are a whole sweep of the
      //   blocks apart.
      // Reading step s + 1 a phase early asks for its loads a phase early: every
      // wave waits at the end of both of its phases until at most D - 2 of its
      // issues are in flight, which covers group 0's half of step s + 1 at the end
      // of its memory phase of step s and group 1's half at the end of its
      // compute phase of step s - 1, both one barrier before group 0's reads.
      static_assert(!S16 || D >= 3, "the early fragment reads need a ring of seven slots or more");
      auto step_body16 = [&](int s, auto phase_c) __attribute__((always_inline)) {
        constexpr int P = decltype(phase_c)::value;  // s % RING
        // ---- memory phase ----
        // (no branch on the group: it would end the basic block and with it the
        // compiler's count of the fragment reads still in flight)
        const uint32_t dma_slot = group == 0 ? (uint32_t)((2 * P + RING - 2) % RING) * SLOT
                                             : (uint32_t)((2 * P + RING - 1) % RING) * SLOT;
        issue_dma(dma_slot, min(s + D - 1 + group, last), 1 - group);
        if constexpr (RBC == 2) wait_lds_reads();   // (the transposing reads: the compiler does not see them)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) ha[tm] = high_bytes(fa[tm]);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) hb[tn] = high_bytes(fb[tn]);
        __builtin_amdgcn_sched_barrier(0);
        // Row sums of the fragments this wave is responsible for.
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          if (tm % WGN == wn) rsa[tm] = row_sum16(fa[tm], rsa[tm]);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          if (tn % WGM == wm) rsb[tn] = row_sum16(fb[tn], rsb[tn]);
        wait_vmem_in_flight<DU*(D - 2)>();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- compute phase ----
        __builtin_amdgcn_s_setprio(3);
        v4i la[TM], lb[TN];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) la[tm] = low_bytes(fa[tm]);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) lb[tn] = low_bytes(fb[tn]);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            hh[tm][tn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hb[tn], ha[tm], hh[tm][tn], 0, 0, 0);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            mid[tm][tn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(hb[tn], la[tm], mid[tm][tn], 0, 0, 0);
        constexpr int kLowOps = 2 * 4 * (TM + TN);        // a permute and an exclusive-or per word
        constexpr int kBeside = 2 * TM * TN;              // the first two sweeps
        constexpr int kPer = (kLowOps + kBeside - 1) / kBeside;
        // (masks: 0x008 matrix instructions, 0x002 vector ALU, 0x100 LDS reads)
#pragma unroll
        for (int i = 0; i < kBeside; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, kPer, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        read_frags16((uint32_t)((2 * P + 2) % RING) * SLOT, (uint32_t)((2 * P + 3) % RING) * SLOT);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            acc[tm][tn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lb[tn], la[tm], acc[tm][tn], 0, 0, 0);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            mid[tm][tn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(lb[tn], ha[tm], mid[tm][tn], 0, 0, 0);
        if constexpr (RBC != 2) {
          // Two read instructions per 16-byte piece for tile rows under 16 bytes.
          constexpr int kReads = (RBC >= 16 ? 1 : 2) * 2 * (TM + TN);
          constexpr int kPerR = (kReads + kBeside - 1) / kBeside;
#pragma unroll
          for (int i = 0; i < kBeside; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
            __builtin_amdgcn_sched_group_barrier(0x100, kPerR, 1);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(0);
        wait_vmem_in_flight<DU*(D - 2)>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      };
      auto step_body = [&](int s, auto phase_c) __attribute__((always_inline)) {
        constexpr int P = decltype(phase_c)::value;  // s % RING
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t slot = (uint32_t)((2 * P + h) % RING) * SLOT;
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) fa[tm][h] = read_frag(slot + (uint32_t)(wm * TM + tm) * 1024);
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) fb[tn][h] = read_frag(slot + IMG_B + (uint32_t)(wn * TN + tn) * 1024);
        }
        if (group == 0) {
          issue_dma((uint32_t)((2 * P + RING - 2) % RING) * SLOT, min(s + D - 1, last), 1);
        } else {
          issue_dma((uint32_t)((2 * P + RING - 1) % RING) * SLOT, min(s + D, last), 0);
          wait_vmem_in_flight<DU*(D - 1)>();   // the first half of step s + 1 has landed
        }
        wait_lds_reads();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(3);
        mfmas_by_columns(fa, fb);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        if (group == 0) wait_vmem_in_flight<DU*(D - 2)>();   // the second half of step s + 1 has landed
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      };
      auto step = [&](int s, auto phase_c) __attribute__((always_inline)) {
        if constexpr (S16) step_body16(s, phase_c);
        else step_body(s, phase_c);
      };
      int s = 0;
      for (; s + RING <= a.steps; s += RING)
        static_for<0, RING>([&](auto p) __attribute__((always_inline)) { step(s + decltype(p)::value, p); });
      static_for<0, RING - 1>([&](auto p) __attribute__((always_inline)) {
        if (s + decltype(p)::value < a.steps) step(s + decltype(p)::value, p);
      });
      if constexpr (S16) {
        // Row sums through LDS (every load has landed and every fragment has
        // been read once all waves are past the barrier below): per row the
        // four K-slice partials of the wave that summed that fragment.
        static_assert(TM % WGN == 0 && TN % WGM == 0, "every fragment is summed by one wave");
        if (group == 0) __builtin_amdgcn_s_barrier();
        wait_vmem_in_flight<0>();
        __syncthreads();
        int* sums = reinterpret_cast<int*>(lds);   // [BM + BN rows][4 slices]
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          if (tm % WGN == wn) sums[((wm * TM + tm) * 16 + r) * 4 + q] = rsa[tm];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          if (tn % WGM == wm) sums[(BM + (wn * TN + tn) * 16 + r) * 4 + q] = rsb[tn];
        __syncthreads();
        const uint32_t k_term = 16384u * 64u * (uint32_t)a.steps;   // 64 elements of K per step
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          const v4i pa = *reinterpret_cast<const v4i*>(sums + ((wm * TM + tm) * 16 + r) * 4);
          const uint32_t sa = (uint32_t)pa[0] + (uint32_t)pa[1] + (uint32_t)pa[2] + (uint32_t)pa[3];
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const v4i pb = *reinterpret_cast<const v4i*>(sums + (BM + (wn * TN + tn) * 16 + 4 * q + e) * 4);
              const uint32_t sb = (uint32_t)pb[0] + (uint32_t)pb[1] + (uint32_t)pb[2] + (uint32_t)pb[3];
              acc[tm][tn][e] = (int)((uint32_t)acc[tm][tn][e] + ((uint32_t)hh[tm][tn][e] << 16) +
                                     ((uint32_t)mid[tm][tn][e] << 8) + 128u * (sa + sb) - k_term);
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < NS - 1; ++s) issue_dma(s * STAGE, min(s, last), 0);
      wait_vmem_in_flight<DU*(NS - 2)>();
      __builtin_amdgcn_s_barrier();
      if (group == 1) __builtin_amdgcn_s_barrier();
      // Fragment (row block b, MFMA K-group kk) sits in block b * NKK + kk of its
      // operand's image.
      v4i fa[NKK][TM][HALVES], fb[NKK][TN][HALVES];
      auto step_body = [&](int s, auto stage_c) {
        constexpr int ST = decltype(stage_c)::value;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
#pragma unroll
          for (int tm = 0; tm < TM; ++tm)
            fa[kk][tm][0] = read_frag(ST * STAGE + (uint32_t)((wm * TM + tm) * NKK + kk) * 1024);
#pragma unroll
          for (int tn = 0; tn < TN; ++tn)
            fb[kk][tn][0] = read_frag(ST * STAGE + IMAGE_A + (uint32_t)((wn * TN + tn) * NKK + kk) * 1024);
        }
        issue_dma(((ST + NS - 1) % NS) * STAGE, min(s + NS - 1, last), 0);
        wait_vmem_in_flight<DU*(NS - 2)>();
        wait_lds_reads();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(3);
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) mfmas_by_columns(fa[kk], fb[kk]);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      };
      static_assert(NS == 4, "the loop below is unrolled by the stage count");
      int s = 0;
      for (; s + 4 <= a.steps; s += 4) {
        step_body(s, std::integral_constant<int, 0>{});
        step_body(s + 1, std::integral_constant<int, 1>{});
        step_body(s + 2, std::integral_constant<int, 2>{});
        step_body(s + 3, std::integral_constant<int, 3>{});
      }
      if (s < a.steps) step_body(s, std::integral_constant<int, 0>{});
      if (s + 1 < a.steps) step_body(s + 1, std::integral_constant<int, 1>{});
      if (s + 2 < a.steps) step_body(s + 2, std::integral_constant<int, 2>{});
    }
    // (the 16-bit integers have done both already, before their exchange through LDS)
    if (group == 0 && E != Elem::kS16) __builtin_amdgcn_s_barrier();
    // No LDS-direct load may still be on its way when the workgroup ends (its
    // LDS goes to the next workgroup on the CU).
    wait_vmem_in_flight<0>();
  }
  // ---- epilogue -----------------------------------------------------------
  if constexpr (OB == 4) {
    if (a.dequant) {
      // Scales of this lane's rows and columns; indices beyond the matrix are
      // clamped (their elements are never stored).
      uint32_t oq = q, orr = r;
      asm volatile("" : "+v"(oq), "+v"(orr));
      const int row_origin = pm0 * a.M0, col_origin = pn0 * a.N0;
      float sm[TM];
      v4f sn[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const int row = max(min(row_origin + (wm * TM + tm) * 16 + (int)orr, a.out_rows - 1), 0);
        sm[tm] = a.row_scale ? a.row_scale[row] : 1.0f;
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int col =
              max(min(col_origin + (wn * TN + tn) * 16 + 4 * (int)oq + e, a.out_cols - 1), 0);
          sn[tn][e] = a.col_scale ? a.col_scale[col] : 1.0f;
        }
      }
      typedef v4f v4f_a4 __attribute__((aligned(4)));
      for_each_output(
          a.out, a.out_stride, a.out_sm0, a.out_spn,
          [&](int tm, int tn, char* p) {
            v4f v = __builtin_convertvector(acc[tm][tn], v4f);
            v = v * sm[tm];
            v = v * sn[tn];
            *reinterpret_cast<v4f_a4*>(p) = v;
          },
          [&](int tm, int tn, int e, char* p) {
            *reinterpret_cast<float*>(p) = (float)acc[tm][tn][e] * sm[tm] * sn[tn][e];
          });
      return;
    }
  }
  // Outputs larger than the memory-side cache are stored non-temporally (s8
  // 8192^3, 268 MB: 387-397 -> 377-385 us in the same process); smaller ones
  // are not: whoever reads them next finds them in that cache (the f16 chain's
  // step takes 3 us longer with non-temporal stores here, all of it in unpack).
  for_each_output(a.out, a.out_stride, a.out_sm0, a.out_spn,
                  [&](int tm, int tn, char* p) {
                    if (a.nt_out) Out::store4_nt(p, acc[tm][tn]);
                    else Out::store4(p, acc[tm][tn]);
                  },
                  [&](int tm, int tn, int e, char* p) { Out::store1(p, acc[tm][tn][e]); });
}

template <Elem E, int TM, int TN, int WGM, int WGN, int NKK, int PIPE>
struct Shape {
  static constexpr int NCH = NKK * ElemTraits<E>::kHalves * 4;
  static constexpr int KS = NCH * 16;
  static constexpr int BM = WGM * TM * 16;
  static constexpr int BN = WGN * TN * 16;
  static constexpr size_t kLdsBytes =
      (PIPE == 5 && ElemTraits<E>::kHalves == 2)
          ? ring_slots<E, BM, BN>() * (size_t)(BM + BN) * 64   // a ring of half-step slots
          : (PIPE == 5 ? kStages5 : PIPE == 0 || PIPE == 4 ? 2 : 3) *
                (size_t)(PIPE == 2 || PIPE == 3 ? BM : BM + BN) * KS;
};

}  // namespace uk_mfma

#endif  // IREE_UK_AMD_MMT4D_MFMA_KERNEL_H_
