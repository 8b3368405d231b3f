// mmt4d on the gfx950 matrix cores.
//
// Operands keep the ukernel ABI layout: LHS [M1][K1][M0][K0], RHS
// [N1][K1][N0][K0] (both K-major per tile row), OUT [M1][N1][M0][N0]
// (runtime/src/iree/builtins/ukernel/mmt4d.c:55-100 for the pointer
// arithmetic this replaces). A workgroup owns a block of whole LHS panels x
// whole RHS panels; its waves each own TM x TN accumulator blocks of 16x16.
//
// The MFMA instructions used take, per lane, 16 (or 2x16 for f8) consecutive
// bytes of K for ONE row: lane l feeds row l%16 with K-slice l/16. The sum
// over K is order-free as far as the instruction is concerned, so any
// assignment of K bytes to (instruction, K-slice, byte) works as long as LHS
// and RHS use the same one. That freedom is what lets every K0 be served:
//
//   row bytes RB = K0 * sizeof(elem)
//   RB >= 16 : a 16-byte piece of a tile row is already an MFMA operand;
//              global -> LDS is a 16-byte-granular copy.
//   RB = 8/4/2: a 16-byte global piece holds R = 16/RB rows of one K-tile. A
//              lane loads the same R rows from R different K-tiles and
//              regroups them in registers into R one-row operands (pure
//              register selection for RB = 8 and 4, v_perm_b32 for RB = 2)
//              before storing them to LDS.
//
// LDS holds, per pipeline stage, the operands exactly as the waves consume
// them: [row block of 16][group of 4 K-slices][slice q][row r][16 bytes], so an
// operand fetch is one ds_read_b128 per lane over a contiguous KiB. The row
// slot is XOR-swizzled so that the 16-byte stores of the loaders spread over
// the banks as well.
//
// Pipeline: double-buffered LDS, next step's global loads issued before the
// current step's MFMAs, one barrier per K step.
#include <hip/hip_runtime.h>

#include "uk_device_common.h"
#include "uk_hip_abi.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

enum class Elem { kS8, kF16, kBF16, kF8 };

template <Elem E> struct ElemTraits;

template <> struct ElemTraits<Elem::kS8> {
  using Acc = v4i;
  static constexpr int kHalves = 1;  // 16-byte pieces per lane operand
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], b[0], c, 0, 0, 0);
  }
};
template <> struct ElemTraits<Elem::kF16> {
  using Acc = v4f;
  static constexpr int kHalves = 1;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(v8h, a[0]), __builtin_bit_cast(v8h, b[0]), c, 0, 0, 0);
  }
};
template <> struct ElemTraits<Elem::kBF16> {
  using Acc = v4f;
  static constexpr int kHalves = 1;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(v8bf, a[0]), __builtin_bit_cast(v8bf, b[0]), c, 0, 0, 0);
  }
};
template <> struct ElemTraits<Elem::kF8> {
  using Acc = v4f;
  static constexpr int kHalves = 2;
  static __device__ __forceinline__ Acc mfma(const v4i* a, const v4i* b, Acc c) {
    v8i av = {a[0][0], a[0][1], a[0][2], a[0][3], a[1][0], a[1][1], a[1][2], a[1][3]};
    v8i bv = {b[0][0], b[0][1], b[0][2], b[0][3], b[1][0], b[1][1], b[1][2], b[1][3]};
    // Formats 0/0 = E4M3 x E4M3; block scales of 2^0 (E8M0 code 127).
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
        av, bv, c, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  }
};

struct MfmaArgs {
  const char* lhs;
  const char* rhs;
  char* out;
  int64_t lhs_stride;  // bytes between LHS panels
  int64_t rhs_stride;  // bytes between RHS panels
  int64_t out_stride;  // bytes between rows of output tiles
  int32_t M1, N1, K1;
  int32_t M0, N0;
  int32_t rb;          // bytes per tile row (K0 * element size), power of two
  int32_t lrb;         // log2(rb)
  int32_t bpm, bpn;    // whole panels per workgroup along M and N
  int32_t grid_n;      // workgroups along N
  int32_t steps;       // K steps
  uint32_t accumulate;
};

// Row-slot swizzle of the LDS operand image. `ch` is the 16-byte K chunk of
// the step, `hi` the top bit of the row index r (0..15). The low three bits of
// the slot decide which of the eight 16-byte bank groups a piece lands in;
// the mask is chosen per row-bytes class so that the eight lanes of one store
// wavefront quarter hit eight different groups. Readers apply the same mask.
__device__ __forceinline__ uint32_t swizzle_mask(uint32_t ch, uint32_t hi,
                                                 int lrb) {
  if (lrb <= 3) return (2 * (ch & 3) + hi) & 7;  // transposing loaders
  if (lrb == 4) return 0;
  if (lrb == 5) return 4 * (ch & 1);
  if (lrb == 6) return 2 * (ch & 3);
  return (2 * (ch & 3) + ((ch >> 2) & 1)) & 7;
}

template <int NCHB>
__device__ __forceinline__ uint32_t image_offset(uint32_t rowblock, uint32_t ch,
                                                 uint32_t r, int lrb) {
  const uint32_t q = ch & 3;
  const uint32_t slot = q * 16 + (r ^ swizzle_mask(ch, r >> 3, lrb));
  return ((rowblock * NCHB + (ch >> 2)) * 64 + slot) * 16;
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

// TM x TN accumulator blocks per wave, WGM x WGN waves per workgroup, NKK MFMA
// K-groups per pipeline step. RBC: 16 = row bytes >= 16 (direct), 8/4/2 =
// regrouping loaders.
template <Elem E, int RBC, int TM, int TN, int WGM, int WGN, int NKK>
__global__ __launch_bounds__(WGM* WGN * 64) void mmt4d_mfma_kernel(MfmaArgs a) {
  using TT = ElemTraits<E>;
  using Acc = typename TT::Acc;
  constexpr int NT = WGM * WGN * 64;
  constexpr int HALVES = TT::kHalves;
  constexpr int NCHB = NKK * HALVES;       // groups of 4 chunks per step
  constexpr int NCH = NCHB * 4;            // 16-byte chunks per row per step
  constexpr int KS = NCH * 16;             // bytes of K per row per step
  constexpr int BM = WGM * TM * 16;
  constexpr int BN = WGN * TN * 16;
  constexpr int R = RBC >= 16 ? 1 : 16 / RBC;
  constexpr int UNITS_A = BM * NCH / R;    // a unit = R loads + R stores
  constexpr int UNITS = (BM + BN) * NCH / R;
  constexpr int NU = (UNITS + NT - 1) / NT;
  constexpr int IMAGE_A = BM * KS;
  constexpr int STAGE = (BM + BN) * KS;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WGN;
  const int wn = wave - wm * WGN;
  const int wg_m = blockIdx.x / a.grid_n;
  const int wg_n = blockIdx.x - wg_m * a.grid_n;
  const int pm0 = wg_m * a.bpm;  // first LHS panel of this workgroup
  const int pn0 = wg_n * a.bpn;
  const int lrb = a.lrb;
  const int kts_per_step = KS >> lrb;

  // ---- loader set-up: per-unit constants --------------------------------
  const char* gbase[NU];     // address of the unit's first piece at step 0
  int64_t gstep[NU];         // bytes to advance per K step
  int64_t gkt[NU];           // bytes between consecutive loads of the unit
  int32_t kt0[NU];           // K-tile index of the first load at step 0
  uint32_t loff[NU][R];      // LDS offsets (within a stage) of the R stores
  bool active[NU];
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    int u = tid + i * NT;
    const bool in_range = u < UNITS;
    const bool is_b = u >= UNITS_A;
    if (is_b) u -= UNITS_A;
    const int X0 = is_b ? a.N0 : a.M0;
    const int X1 = is_b ? a.N1 : a.M1;
    const int px0 = is_b ? pn0 : pm0;
    const int bpx = is_b ? a.bpn : a.bpm;
    const int64_t xstride = is_b ? a.rhs_stride : a.lhs_stride;
    const char* xbase = is_b ? a.rhs : a.lhs;
    const uint32_t image = is_b ? IMAGE_A : 0;
    const int64_t kt_bytes = (int64_t)X0 << lrb;  // one K-tile of the panel
    int pl, row_in_panel, ch;
    int64_t in_tile;  // byte offset inside the first K-tile's rows
    if constexpr (RBC >= 16) {
      // Pieces in memory order [K-tile][row][16-byte column] of each panel.
      const int cr = 1 << (lrb - 4);  // chunks per tile row
      const int c = u & (cr - 1);
      const int t1 = u >> (lrb - 4);
      row_in_panel = t1 % X0;
      const int t2 = t1 / X0;
      const int ktl = t2 % kts_per_step;
      pl = t2 / kts_per_step;
      ch = ktl * cr + c;
      kt0[i] = ktl;
      in_tile = (int64_t)ktl * kt_bytes + ((int64_t)row_in_panel << lrb) + c * 16;
      gkt[i] = 0;
    } else {
      // Units in order [chunk g][row group] per panel; the unit's R loads read
      // K-tiles g, g + NCH, g + 2*NCH, ... so that one load instruction of the
      // workgroup covers NCH consecutive K-tiles.
      const int groups = X0 / R;
      const int mg = u % groups;
      const int t1 = u / groups;
      const int g = t1 % NCH;
      pl = t1 / NCH;
      row_in_panel = mg * R;
      ch = g;
      kt0[i] = g;
      in_tile = (int64_t)g * kt_bytes + mg * 16;
      gkt[i] = (int64_t)NCH * kt_bytes;
    }
    const int p = px0 + pl;
    active[i] = in_range && pl < bpx && p < X1;
    gbase[i] = xbase + (int64_t)(active[i] ? p : 0) * xstride + in_tile;
    gstep[i] = (int64_t)kts_per_step * kt_bytes;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const uint32_t row = (uint32_t)(pl * X0 + row_in_panel + j);
      loff[i][j] = image + image_offset<NCHB>(row >> 4, (uint32_t)ch, row & 15, lrb);
    }
  }

  // ---- reader set-up ------------------------------------------------------
  const uint32_t q = lane >> 4, r = lane & 15;
  uint32_t rd_slot[NCHB];
#pragma unroll
  for (int cb = 0; cb < NCHB; ++cb) {
    rd_slot[cb] = (q * 16 + (r ^ swizzle_mask(cb * 4 + q, r >> 3, lrb))) * 16;
  }
  const uint32_t rd_a = (uint32_t)(wm * TM) * NCHB * 1024;
  const uint32_t rd_b = IMAGE_A + (uint32_t)(wn * TN) * NCHB * 1024;

  // ---- accumulators -------------------------------------------------------
  // Lane (q, c = r) of block (tm, tn) holds rows 4q..4q+3, column c.
  Acc acc[TM][TN];
  int64_t out_row_off[TM][4];  // byte offset of (row, column 0 of the panel)
  int64_t out_col_off[TN];
  bool row_ok[TM][4], col_ok[TN];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int row = (wm * TM + tm) * 16 + 4 * q + e;
      const int pl = row / a.M0, m0 = row - pl * a.M0;
      row_ok[tm][e] = pl < a.bpm && pm0 + pl < a.M1;
      out_row_off[tm][e] = (int64_t)(pm0 + pl) * a.out_stride + (int64_t)m0 * a.N0 * 4;
    }
  }
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int col = (wn * TN + tn) * 16 + r;
    const int pl = col / a.N0, n0 = col - pl * a.N0;
    col_ok[tn] = pl < a.bpn && pn0 + pl < a.N1;
    out_col_off[tn] = (int64_t)(pn0 + pl) * a.M0 * a.N0 * 4 + (int64_t)n0 * 4;
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (a.accumulate && row_ok[tm][e] && col_ok[tn]) {
          acc[tm][tn][e] = *reinterpret_cast<const decltype(acc[0][0][0] + 0)*>(
              a.out + out_row_off[tm][e] + out_col_off[tn]);
        } else {
          acc[tm][tn][e] = 0;
        }
      }

  // ---- pipeline -----------------------------------------------------------
  v4i regs[NU][R];
  auto load_global = [&](int step) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const char* p = gbase[i] + (int64_t)step * gstep[i];
      const int kt = step * kts_per_step + kt0[i];
#pragma unroll
      for (int t = 0; t < R; ++t) {
        const bool ok = active[i] && (kt + t * NCH) < a.K1;
        regs[i][t] = ok ? *reinterpret_cast<const v4i*>(p + t * gkt[i]) : v4i{0, 0, 0, 0};
      }
    }
  };
  auto store_lds = [&](int stage) {
    char* base = lds + stage * STAGE;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      v4i outp[R];
      regroup<RBC>(regs[i], outp);
      if (tid + i * NT < UNITS) {
#pragma unroll
        for (int j = 0; j < R; ++j) *reinterpret_cast<v4i*>(base + loff[i][j]) = outp[j];
      }
    }
  };
  auto compute = [&](int stage) {
    const char* base = lds + stage * STAGE;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      v4i fa[TM][HALVES], fb[TN][HALVES];
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
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = TT::mfma(fa[tm], fb[tn], acc[tm][tn]);
    }
  };

  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int s = 0; s < a.steps; ++s) {
    const int stage = s & 1;
    const bool more = s + 1 < a.steps;
    if (more) load_global(s + 1);
    compute(stage);
    if (more) store_lds(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (row_ok[tm][e] && col_ok[tn]) {
          *reinterpret_cast<decltype(acc[0][0][0] + 0)*>(
              a.out + out_row_off[tm][e] + out_col_off[tn]) = acc[tm][tn][e];
        }
      }
}

struct Config {
  int TM, TN, WGM, WGN, NKK;
};

template <Elem E, int RBC, int TM, int TN, int WGM, int WGN, int NKK>
int launch_config(const MfmaArgs& base, const iree_uk_mmt4d_params_t* p,
                  hipStream_t stream) {
  using TT = ElemTraits<E>;
  constexpr int NCH = NKK * TT::kHalves * 4;
  constexpr int KS = NCH * 16;
  constexpr int BM = WGM * TM * 16;
  constexpr int BN = WGN * TN * 16;
  constexpr int R = RBC >= 16 ? 1 : 16 / RBC;
  MfmaArgs a = base;
  if (a.rb > KS) return -1;                    // a tile row must fit one step
  if (p->M0 > BM || p->N0 > BN) return -1;     // at least one whole panel
  if (p->M0 % R || p->N0 % R) return -1;       // 16-byte pieces hold whole rows
  a.bpm = BM / p->M0;
  a.bpn = BN / p->N0;
  const int64_t grid_m = uk::ceil_div(p->M, a.bpm);
  const int64_t grid_n = uk::ceil_div(p->N, a.bpn);
  if (grid_m * grid_n >= (1ll << 31)) return -1;
  a.grid_n = (int32_t)grid_n;
  const int64_t k_bytes = (int64_t)p->K << a.lrb;  // bytes of K per row
  a.steps = (int32_t)uk::ceil_div(k_bytes, KS);
  if (a.steps < 1) a.steps = 1;
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * KS;
  auto kernel = mmt4d_mfma_kernel<E, RBC, TM, TN, WGM, WGN, NKK>;
  if (lds_bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(kernel, dim3((uint32_t)(grid_m * grid_n)), dim3(WGM * WGN * 64),
                     lds_bytes, stream, a);
  return (int)hipGetLastError();
}

template <Elem E, int RBC>
int launch_rbc(const MfmaArgs& base, const iree_uk_mmt4d_params_t* p,
               hipStream_t stream, const char** name) {
  *name = "mmt4d_mfma_128x128";
  return launch_config<E, RBC, 4, 4, 2, 2, 2 / ElemTraits<E>::kHalves>(base, p, stream);
}

template <Elem E>
int launch_elem(const MfmaArgs& base, const iree_uk_mmt4d_params_t* p,
                hipStream_t stream, const char** name) {
  switch (base.rb) {
    case 2: if constexpr (E != Elem::kF8) return launch_rbc<E, 2>(base, p, stream, name); else return -1;
    case 4: if constexpr (E != Elem::kF8) return launch_rbc<E, 4>(base, p, stream, name); else return -1;
    case 8: if constexpr (E != Elem::kF8) return launch_rbc<E, 8>(base, p, stream, name); else return -1;
    default: return launch_rbc<E, 16>(base, p, stream, name);
  }
}

bool elem_of(uint32_t flags, Elem* e, int* elem_bytes) {
  switch (flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *e = Elem::kS8; *elem_bytes = 1; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *e = Elem::kF16; *elem_bytes = 2; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *e = Elem::kBF16; *elem_bytes = 2; return true;
    case IREE_UK_AMD_FLAG_MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: *e = Elem::kF8; *elem_bytes = 1; return true;
    default: return false;
  }
}

bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

}  // namespace

extern "C" int iree_uk_amd_hip_mmt4d_mfma_supported(int32_t M0, int32_t N0,
                                                    int32_t K0, uint32_t flags) {
  Elem e;
  int eb;
  if (!elem_of(flags, &e, &eb)) return 0;
  const int64_t rb = (int64_t)K0 * eb;
  if (!is_pow2(rb) || rb < 2 || rb > 128) return 0;
  if (e == Elem::kF8 && rb < 16) return 0;
  if (M0 < 1 || N0 < 1 || M0 > 128 || N0 > 128) return 0;
  if (rb < 16) {
    const int R = (int)(16 / rb);
    if (M0 % R || N0 % R) return 0;
  }
  return 1;
}

// Returns a HIP status (>= 0), or -1 when the case is not served after all.
extern "C" int iree_uk_amd_hip_launch_mmt4d_mfma(const iree_uk_mmt4d_params_t* p,
                                                 void* stream_v,
                                                 const char** kernel_name) {
  Elem e;
  int eb;
  if (!elem_of(p->flags, &e, &eb)) return -1;
  if (!iree_uk_amd_hip_mmt4d_mfma_supported(p->M0, p->N0, p->K0, p->flags)) return -1;
  hipStream_t stream = (hipStream_t)stream_v;
  MfmaArgs a;
  a.lhs = (const char*)p->lhs_buffer + p->lhs_offset * eb;
  a.rhs = (const char*)p->rhs_buffer + p->rhs_offset * eb;
  a.out = (char*)p->out_buffer + p->out_offset * 4;
  a.lhs_stride = p->lhs_stride0 * eb;
  a.rhs_stride = p->rhs_stride0 * eb;
  a.out_stride = p->out_stride0 * 4;
  // 16-byte vector loads need 16-byte aligned panels.
  if (((uintptr_t)a.lhs | (uintptr_t)a.rhs | (uint64_t)a.lhs_stride |
       (uint64_t)a.rhs_stride) & 15) {
    return -1;
  }
  if ((uintptr_t)a.out & 3) return -1;
  a.M1 = (int32_t)p->M;
  a.N1 = (int32_t)p->N;
  a.K1 = (int32_t)p->K;
  a.M0 = p->M0;
  a.N0 = p->N0;
  a.rb = p->K0 * eb;
  a.lrb = 0;
  while ((1 << a.lrb) < a.rb) ++a.lrb;
  a.accumulate = (p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  a.bpm = a.bpn = a.grid_n = a.steps = 0;
  switch (e) {
    case Elem::kS8: return launch_elem<Elem::kS8>(a, p, stream, kernel_name);
    case Elem::kF16: return launch_elem<Elem::kF16>(a, p, stream, kernel_name);
    case Elem::kBF16: return launch_elem<Elem::kBF16>(a, p, stream, kernel_name);
    case Elem::kF8: return launch_elem<Elem::kF8>(a, p, stream, kernel_name);
  }
  return -1;
}
