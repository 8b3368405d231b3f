// mmt4d on the gfx950 matrix cores for NARROW tile rows (2 or 4 bytes: the
// x86-style tiles 16x16x2 of s8 and bf16/f16, 16x16x1 of f32) with N0 = 16: the
// register-direct-RHS pipeline of mmt4d_mfma_kernel.h (PIPE 3) carried over to
// row widths where a 16-byte piece of memory holds several rows.
//
// A K-tile of an RHS panel is [16 rows][RB bytes]. With RB < 16 no 16-byte
// piece of it is a lane operand, and the general kernel therefore sends both
// operands through LDS, regrouping on the way. Here only the LHS does. For the
// RHS the freedom used is in the ROWS: the 16 rows that one MFMA block
// multiplies need not be neighbours, only known when the result is stored. A
// wave owns 64 columns = 4 panels of 16; lane (q, r) reads, of panel r / 4,
// the four rows 4 (r % 4) .. + 3 from its K-tiles q, q + 4, q + 8, ... of the
// step: R loads of 64 / R bytes each (16-byte loads for RB = 4, 8-byte loads
// for RB = 2) in which the four lanes r % 4 = 0..3 cover one K-tile of a
// panel contiguously and the four K-slices q cover four consecutive K-tiles.
// Regrouped in registers (register selection for RB = 4, v_perm_b32 for
// RB = 2), that is, for j = 0..3, the 16 K bytes of row 4 (r % 4) + j: the
// lane's operand in accumulator block j. Block j of the wave thus multiplies
// columns {panel i / 4, column 4 (i % 4) + j : i = 0..15}, and a lane that
// holds instruction rows 4q..4q+3 of the result holds columns j, 4 + j, 8 + j,
// 12 + j of panel q. Taking the same register of the four blocks gives four
// CONSECUTIVE columns again, so accumulators still move 16 bytes per lane.
// The LHS goes through LDS in the general kernel's image (chunk q of a step
// holds K-tiles q, q + 4, ...: the K assignment of the RHS lanes). Its loader
// lanes read whole 16-byte pieces (4 rows for RB = 4, 8 rows for RB = 2: the
// CU's address unit is the busiest part of this kernel, and a 16-byte load
// costs it what an 8-byte one does) and regroup them as the RHS lanes do. For
// RB = 2 a unit is a quarter of an operand's K (2 loads, 4 bytes per row, one
// v_perm_b32 and one 4-byte LDS store per row): three register sets of whole
// units would not fit beside the accumulators, and so all eight waves load,
// each a little.
//
// Restrictions (launcher): RB in {2, 4}, N0 == 16, M0 a multiple of the rows
// of an LHS piece (16 / RB) that divides the workgroup's rows,
// K in whole 64-byte steps, 4-byte accumulators, no dequantizing store, output
// columns complete (tiled output, or a row-major matrix as wide as the tiles).
#ifndef IREE_UK_AMD_MMT4D_MFMA_NARROW_H_
#define IREE_UK_AMD_MMT4D_MFMA_NARROW_H_

#include "mmt4d_mfma_kernel.h"

namespace uk_mfma {

typedef int v2i_n __attribute__((ext_vector_type(2)));
typedef v2i_n v2i_ng __attribute__((aligned(1)));

template <Elem E, int RBC, int TM, int WGM, int WGN>
__global__ __launch_bounds__(WGM* WGN * 64)
void mmt4d_mfma_narrow_kernel(Args a) {
  using TT = ElemTraits<E>;
  using Acc = typename TT::Acc;
  using Out = typename TT::Out;
  static_assert(RBC == 2 || RBC == 4, "narrow tile rows");
  static_assert(TT::kHalves == 1 && Out::kOutBytes == 4, "one piece per operand, 4-byte accumulators");
  static_assert(TM % 2 == 0, "LHS fragments are fetched two rows ahead");
  constexpr int TN = 4;                     // a wave's 64 columns: 4 panels of 16
  constexpr int NW = WGM * WGN;
  constexpr int NCH = 4, KS = 64;           // 16-byte chunks / bytes of K per row per step
  constexpr int BM = WGM * TM * 16;
  constexpr int R = 16 / RBC;               // loads per lane operand set: K-tiles per 16 bytes of K
  // The LHS loader moves 16-byte pieces: RU rows x RB bytes of one K-tile (the
  // address unit of the CU is what this kernel is short of, and a 16-byte load
  // costs it no more than an 8-byte one). RB = 2: 8 rows per piece, and a unit
  // covers a quarter of an operand's K (two K-tiles, 4 bytes per row).
  constexpr int RU = 16 / RBC;              // rows per LHS piece (8 or 4)
  constexpr int LH = RBC == 2 ? 4 : 1;      // LHS loader units per 16-byte operand (parts of its K)
  constexpr int RL = R / LH;                // loads per LHS unit (2 or 4)
  constexpr int UNITS = BM * NCH / RU * LH; // LHS loader units (RL loads, RU LDS stores each)
  constexpr int BLOCKS = (UNITS + 63) / 64; // in blocks of one unit per lane
  constexpr int NU = (BLOCKS + NW - 1) / NW;
  constexpr uint32_t STAGE = BM * KS;
  constexpr int FR = 3;
  constexpr int NLD = NU * RL;              // LHS loads per thread per step
  constexpr int NST = NU * RU;              // LHS LDS stores per thread per step
  using Raw = typename std::conditional<RBC == 4, v4i, v2i_n>::type;  // an RHS piece: 4 rows
  using RawL = v4i;                                                     // an LHS piece: RU rows

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN;
  const int wn = wave - wm * WGN;
  int wg_m, wg_n;
  block_of_workgroup(blockIdx.x, a, &wg_m, &wg_n);
  const int pm0 = wg_m * a.bpm;
  const int pn0 = wg_n * a.bpn;
  constexpr int lrb = RBC == 2 ? 1 : 2;  // the launcher checked a.lrb against it
  const uint32_t kts_per_step = KS >> lrb;
  const uint32_t q = lane >> 4, r = lane & 15;

  // Slot swizzle of the LDS image: row r of chunk (K-slice) g of 16-row block b
  // sits in slot r ^ piece_mask(g, b). A store instruction writes, for one j,
  // row RU mg + j of every (row group mg, chunk g) pair (and, for 2-byte rows,
  // of two neighbouring blocks and the four parts of K at their own offsets
  // inside the slot): the mask sends the lanes of such a store to different
  // bank groups. A fragment read (one chunk of one block, 16 rows) is a
  // permutation of the slots under any mask.
  auto piece_mask = [](uint32_t g, uint32_t blk) {
    return RBC == 2 ? ((g & 3u) | ((blk & 1u) << 2)) : (g & 3u);
  };

  // ---- LHS loader units ------------------------------------------------------------
  // Unit u (lane `lane` of loader block `blk`) = (panel, part h of K, chunk g,
  // row group mg): rows RU mg .. + RU - 1 of the panel, K-tiles g + 4 t of the
  // step for t = RL h .. RL h + RL - 1 (all R of them when there is one part).
  const char* sbase_a = a.lhs + (int64_t)pm0 * a.lhs_stride;
  const uint32_t kt_bytes_a = (uint32_t)a.M0 << lrb;
  const uint32_t sstep_a = kts_per_step * kt_bytes_a;
  const uint32_t skt_a = NCH * kt_bytes_a;  // between the R loads of a unit
  uint32_t voff[NU], loff[NU];
  static_assert(UNITS % 64 == 0, "whole loader blocks");
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int blk = wave + i * NW;  // blocks at or beyond BLOCKS do not exist: such a wave idles
    const uint32_t u = (uint32_t)blk * 64 + lane;
    const uint32_t groups = (uint32_t)a.M0 / RU;
    const uint32_t t1 = u / groups;
    const uint32_t mg = u - t1 * groups;
    const uint32_t t2 = t1 / NCH;
    const uint32_t g = t1 - t2 * NCH;
    const int pl = (int)(t2 / LH);
    const uint32_t h = t2 - (uint32_t)pl * LH;
    voff[i] = (uint32_t)pl * (uint32_t)a.lhs_stride + (g + h * RL * NCH) * kt_bytes_a + mg * (uint32_t)(RU * RBC);
    const uint32_t row = (uint32_t)pl * a.M0 + mg * RU;
    const uint32_t rr = row & 15;
    // Row rr + j (j < RU, rr % RU == 0) sits in slot (rr + j) ^ mask: the store
    // applies the j itself.
    loff[i] = (((row >> 4) * 64 + g * 16) * 16) + ((rr & 8) | ((rr & 7) ^ piece_mask(g, row >> 4))) * 16 +
              h * (16 / LH);
    if (!(pl < a.bpm && pm0 + pl < a.M1) || blk >= BLOCKS) voff[i] = 0;
  }
  // (wm * TM is even: the parity of a wave's block is the parity of tm.)
  const uint32_t rd_a0 = (uint32_t)(wm * TM) * 1024 + (q * 16 + (r ^ piece_mask(q, 0))) * 16;
  const uint32_t rd_a1 = (uint32_t)(wm * TM) * 1024 + (q * 16 + (r ^ piece_mask(q, 1))) * 16;

  // ---- RHS: lane (q, r) reads rows 4 (r % 4) .. + 3 of panel r / 4 ---------------
  // N0 = 16 and the row width is a template parameter: the distances are
  // compile-time, so a load is scalar base (advanced per step) + one vector
  // offset + an immediate.
  constexpr uint32_t kt_bytes_b = 16u * RBC;
  constexpr uint32_t sstep_b = (KS / RBC) * kt_bytes_b;
  constexpr uint32_t skt_b = NCH * kt_bytes_b;
  const int my_panel = wn * TN + (int)(r >> 2);          // within the workgroup's panels
  const bool panel_ok = my_panel < a.bpn && pn0 + my_panel < a.N1;
  const char* sbase_b = a.rhs + (int64_t)pn0 * a.rhs_stride;
  uint32_t voff_b =
      panel_ok ? (uint32_t)my_panel * (uint32_t)a.rhs_stride + q * kt_bytes_b + (r & 3) * (4u * RBC) : 0u;
  auto load_b = [&](int t, int step) -> Raw {
    const char* sb = sbase_b + (uint64_t)((uint32_t)step * sstep_b);
    return *reinterpret_cast<const typename std::conditional<RBC == 4, v4i_g, v2i_ng>::type*>(
        sb + voff_b + (uint32_t)t * skt_b);
  };
  // Row j (of the piece's four) as a 16-byte operand, from the R pieces of
  // K-tiles x, x + 4, ... that a lane has loaded: its 16 bytes of K. RB = 4:
  // dword j of every piece. RB = 2: dword d of a piece holds rows 2d (low
  // half) and 2d + 1 (high half).
  auto row_operand = [&](const Raw (&raw)[R], int j) {
    if constexpr (RBC == 4) {
      return v4i{raw[0][j], raw[1][j], raw[2][j], raw[3][j]};
    } else {
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      v4i o;
#pragma unroll
      for (int w = 0; w < 4; ++w)
        o[w] = (int)__builtin_amdgcn_perm((uint32_t)raw[2 * w + 1][j >> 1], (uint32_t)raw[2 * w][j >> 1], sel);
      return o;
    }
  };

  // ---- accumulators ---------------------------------------------------------------
  // acc[tm][j][e]: LHS row 16 (wm TM + tm) + r, column 4 e + j of panel wn TN + q.
  Acc acc[TM][TN];
  auto for_each_quad = [&](const char* base, int64_t s_panel, uint32_t s_m0, uint32_t s_pn, auto f) {
    uint32_t oq = q, orr = r;
    asm volatile("" : "+v"(oq), "+v"(orr));
    const int col_panel = wn * TN + (int)oq;
    const bool col_ok = col_panel < a.bpn && pn0 + col_panel < a.N1;
    char* out_base = const_cast<char*>(base) + (int64_t)pm0 * s_panel + (int64_t)pn0 * s_pn;
    const uint32_t col_off = (uint32_t)col_panel * s_pn;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int row = (wm * TM + tm) * 16 + (int)orr;
      const int pl = row / a.M0, m0 = row - pl * a.M0;
      const bool ok = col_ok && pl < a.bpm && pm0 + pl < a.M1 && pm0 * a.M0 + row < a.out_rows;
      const uint32_t row_off = (uint32_t)pl * (uint32_t)s_panel + (uint32_t)m0 * s_m0;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (ok) f(tm, e, out_base + (row_off + col_off + (uint32_t)e * 16));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[tm][j] = Acc{0, 0, 0, 0};
  if (a.accumulate) {
    for_each_quad(a.acc, a.acc_stride, a.acc_sm0, a.acc_spn, [&](int tm, int e, char* p) {
      const Acc v = Out::load4(p);
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[tm][j][e] = v[j];
    });
  }

  // ---- pipeline (PIPE 3 of mmt4d_mfma_kernel.h) ------------------------------------
  auto load_a = [&](int i, int t, int step) -> RawL {
    const char* sa = sbase_a + (uint64_t)((uint32_t)step * sstep_a + (uint32_t)t * skt_a);
    return *reinterpret_cast<const v4i_g*>(sa + voff[i]);
  };
  auto store_row = [&](uint32_t stage_off, int i, int j, const RawL (&in)[RL]) {
    if constexpr (BLOCKS % NW != 0) {
      if (wave + i * NW >= BLOCKS) return;  // wave-uniform
    }
    char* dst = lds + stage_off + (loff[i] ^ (uint32_t)(j * 16));
    if constexpr (LH == 1) {
      *reinterpret_cast<v4i*>(dst) = row_operand(in, j);
    } else {
      // A quarter of an operand: K-tiles x and x + 4 of row j, 2 bytes each.
      // Dword d of a piece holds rows 2d (low half) and 2d + 1 (high half).
      static_assert(RL == 2, "two K-tiles per unit");
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      *reinterpret_cast<uint32_t*>(dst) =
          __builtin_amdgcn_perm((uint32_t)in[1][j >> 1], (uint32_t)in[0][j >> 1], sel);
    }
  };
  auto read_a = [&](uint32_t stage_off, int tm) {
    return *reinterpret_cast<const v4i*>(lds + stage_off + ((tm & 1) ? rd_a1 : rd_a0) + tm * 1024);
  };
  const int last = a.steps - 1;
  RawL regs[3][NU][RL];
  Raw raw[3][R];
  v4i fa[FR];
  // Steps 0 and 1 go to LDS stages 0 and 1 right away.
#pragma unroll
  for (int st = 0; st < 2; ++st) {
#pragma unroll
    for (int i = 0; i < NU; ++i)
#pragma unroll
      for (int t = 0; t < RL; ++t) regs[st][i][t] = load_a(i, t, min(st, last));
  }
#pragma unroll
  for (int st = 0; st < 2; ++st) {
#pragma unroll
    for (int i = 0; i < NU; ++i)
#pragma unroll
      for (int j = 0; j < RU; ++j) store_row(st * STAGE, i, j, regs[st][i]);
  }
  // What iterations -2 and -1 would have left in flight, in the loop's own
  // issue order (the wait counters are in-order).
  auto issue_like_iteration = [&](auto bbuf, int b_step, auto aset, int a_step) {
    constexpr int BB = decltype(bbuf)::value, AS = decltype(aset)::value;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int l = tm * R / TM; l < (tm + 1) * R / TM; ++l) raw[BB][l] = load_b(l, b_step);
#pragma unroll
      for (int k = tm * NLD / TM; k < (tm + 1) * NLD / TM; ++k)
        regs[AS][k / RL][k % RL] = load_a(k / RL, k % RL, a_step);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  issue_like_iteration(std::integral_constant<int, 0>{}, 0, std::integral_constant<int, 2>{}, min(2, last));
  issue_like_iteration(std::integral_constant<int, 1>{}, min(1, last), std::integral_constant<int, 0>{},
                       min(3, last));
  __syncthreads();
  fa[0] = read_a(0, 0);
  fa[1] = read_a(0, 1);
  // Iteration s (phase P = s % 3) computes step s from LDS stage P and RHS
  // registers P, loads the RHS of step s + 2 into registers (P + 2) % 3 and the
  // LHS of step s + 4 into register set (P + 1) % 3, and stores register set
  // (P + 2) % 3 (the LHS of step s + 2), regrouped, to LDS stage (P + 2) % 3.
  // Loads past the end re-read the last step (valid addresses, unused data).
  auto iteration = [&](int s, auto phase) {
    constexpr int P = decltype(phase)::value;
    constexpr uint32_t st_cur = P * STAGE, st_next = ((P + 1) % 3) * STAGE,
                       st_write = ((P + 2) % 3) * STAGE;
    const int ld_step = min(s + 4, last);
    const int b_step = min(s + 2, last);
    // The vector offsets are made opaque once per iteration, so that they stay
    // 32-bit registers beside scalar bases instead of being folded into
    // hoisted 64-bit vector addresses that need a vector add per load.
    asm volatile("" : "+v"(voff_b));
#pragma unroll
    for (int i = 0; i < NU; ++i) asm volatile("" : "+v"(voff[i]));
    v4i fb[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = row_operand(raw[P], j);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int l = tm * R / TM; l < (tm + 1) * R / TM; ++l) raw[(P + 2) % 3][l] = load_b(l, b_step);
      // The stores read the whole register set (P + 2) % 3 and the loads fill
      // set (P + 1) % 3: different sets, so they can be spread independently.
#pragma unroll
      for (int k = tm * NST / TM; k < (tm + 1) * NST / TM; ++k)
        store_row(st_write, k / RU, k % RU, regs[(P + 2) % 3][k / RU]);
#pragma unroll
      for (int k = tm * NLD / TM; k < (tm + 1) * NLD / TM; ++k)
        regs[(P + 1) % 3][k / RL][k % RL] = load_a(k / RL, k % RL, ld_step);
      if (tm + 2 < TM) fa[(P * TM + tm + 2) % FR] = read_a(st_cur, tm + 2);
      else fa[(P * TM + tm + 2) % FR] = read_a(st_next, tm + 2 - TM);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[tm][j] = TT::mfma(&fb[j], &fa[(P * TM + tm) % FR], acc[tm][j]);
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

  // ---- epilogue -------------------------------------------------------------------
  for_each_quad(a.out, a.out_stride, a.out_sm0, a.out_spn, [&](int tm, int e, char* p) {
    Out::store4(p, Acc{acc[tm][0][e], acc[tm][1][e], acc[tm][2][e], acc[tm][3][e]});
  });
}

}  // namespace uk_mfma

#endif  // IREE_UK_AMD_MMT4D_MFMA_NARROW_H_
