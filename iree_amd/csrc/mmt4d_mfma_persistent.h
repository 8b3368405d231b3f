// mmt4d on the gfx950 matrix cores: persistent form of the register-direct-RHS
// pipeline (PIPE 3 of mmt4d_mfma_kernel.h) for problems of several rounds of
// workgroup blocks.
//
// One workgroup per CU walks a list of output blocks (block j of workgroup w
// is block w + j * gridDim.x of the XCD-aware order of block_of_workgroup, so
// every block stays on the XCD that the one-block-per-workgroup launch would
// give it). The software pipeline never drains between blocks: the LHS global
// loads (four steps ahead), the RHS fragment loads (two steps ahead) and the
// LDS stages simply run on into the next block's K range while the current
// block still computes, so a block boundary costs the accumulator stores and
// nothing else: no pipeline fill, no wait for a new workgroup to be placed.
// The stores of block j are issued in one go after its last step; the MFMAs
// of block j + 1 start as soon as the store instructions have read their
// registers.
//
// Restrictions (checked by the launcher): tile rows of 16..64 bytes, M0 and N0
// powers of two with N0 >= 4, the workgroup block tiles the problem exactly
// (no edge blocks), K a multiple of four 64-byte steps and at least eight of
// them (the load cursors are then at most one block ahead of the MFMAs), 4-byte
// accumulators (s8, f16, bf16 -> 32 bit), no dequantizing store.
#ifndef IREE_UK_AMD_MMT4D_MFMA_PERSISTENT_H_
#define IREE_UK_AMD_MMT4D_MFMA_PERSISTENT_H_

#include "mmt4d_mfma_kernel.h"

namespace uk_mfma {

template <Elem E, int TM, int TN, int WGM, int WGN>
__global__ __launch_bounds__(WGM* WGN * 64)
void mmt4d_mfma_persistent_kernel(Args a) {
  using TT = ElemTraits<E>;
  using Acc = typename TT::Acc;
  using Out = typename TT::Out;
  static_assert(TT::kHalves == 1, "one 16-byte piece per lane operand");
  static_assert(Out::kOutBytes == 4, "4-byte accumulators");
  static_assert(TM % 2 == 0, "LHS fragments are fetched two rows ahead");
  constexpr int NW = WGM * WGN;
  constexpr int KS = 64;                    // bytes of K per row per step
  constexpr int BM = WGM * TM * 16;
  constexpr int BLOCKS = BM * 4 / 64;       // 1 KiB loader blocks in the LHS image of a step
  constexpr int NU = (BLOCKS + NW - 1) / NW;
  constexpr bool EVEN = BLOCKS % NW == 0;
  constexpr uint32_t STAGE = BM * KS;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN;
  const int wn = wave - wm * WGN;
  const uint32_t q = lane >> 4, r = lane & 15;
  const int lrb = a.lrb;
  const uint32_t kt_bytes_a = (uint32_t)a.M0 << lrb, kt_bytes_b = (uint32_t)a.N0 << lrb;
  const uint32_t kts_per_step = KS >> lrb;
  const uint32_t sstep_a = kts_per_step * kt_bytes_a, sstep_b = kts_per_step * kt_bytes_b;
  const uint32_t total = (uint32_t)a.grid_m * (uint32_t)a.grid_n;
  const uint32_t G = gridDim.x;
  const uint32_t ntiles = (total - blockIdx.x + G - 1) / G;
  const uint32_t steps = (uint32_t)a.steps;

  // ---- per-lane constants: the same for every block (no edge blocks) -------
  // The lane's chunk of a 64-byte step: K bytes [16q, 16q + 16) of its row.
  const uint32_t kb = q * 16;
  const uint32_t k_in_panel = (kb >> lrb) * 1u;  // K-tile of the chunk within a step
  const uint32_t k_in_row = kb & ((1u << lrb) - 1);
  uint32_t voff[NU], loff[NU];
#pragma unroll
  for (int i = 0; i < NU; ++i) {
    const int blk = wave + i * NW;
    const uint32_t row = (uint32_t)blk * 16 + r;
    const uint32_t pl = row >> a.lm0, m0 = row & ((uint32_t)a.M0 - 1);
    voff[i] = pl * (uint32_t)a.lhs_stride + k_in_panel * kt_bytes_a + (m0 << lrb) + k_in_row;
    loff[i] = (uint32_t)blk * 1024 + lane * 16;
    if (!EVEN && blk >= BLOCKS) voff[i] = 0;
  }
  uint32_t voff_b[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const uint32_t row = (uint32_t)(wn * TN + tn) * 16 + r;
    const uint32_t pl = row >> a.ln0, n0 = row & ((uint32_t)a.N0 - 1);
    voff_b[tn] = pl * (uint32_t)a.rhs_stride + k_in_panel * kt_bytes_b + (n0 << lrb) + k_in_row;
  }
  const uint32_t rd_a = (uint32_t)(wm * TM) * 1024 + lane * 16;

  // ---- block bookkeeping (all uniform) --------------------------------------
  // First LHS / RHS panel of the j-th block of this workgroup.
  auto block_panels = [&](uint32_t j, int* pm0, int* pn0) {
    int bm, bn;
    block_of_workgroup(blockIdx.x + j * G, a, &bm, &bn);
    // Uniform, but computed with vector instructions (integer division):
    // bring the results back to scalar registers, so that everything derived
    // from them (panel base addresses) is scalar too.
    *pm0 = __builtin_amdgcn_readfirstlane(bm * a.bpm);
    *pn0 = __builtin_amdgcn_readfirstlane(bn * a.bpn);
  };
  int cur_pm0, cur_pn0, next_pm0, next_pn0;
  block_panels(0, &cur_pm0, &cur_pn0);
  block_panels(ntiles > 1 ? 1 : 0, &next_pm0, &next_pn0);

  Acc acc[TM][TN];
  // Element (row, col) of a block lives at
  //   base + (pm0 + row / M0) * stride + (row % M0) * sm0 + (pn0 + col / N0) * spn + (col % N0) * 4
  // (tiled output or row-major matrix alike); the lane holds, of accumulator
  // block (tm, tn), row 16 tm + r and the four columns from 16 tn + 4 q.
  auto for_each_quad = [&](const char* base, int64_t s_panel, uint32_t s_m0, uint32_t s_pn,
                           int pm0, int pn0, auto f) {
    // The lane coordinates pass through an empty asm so that this address
    // arithmetic is redone per block instead of staying live across the K loop.
    uint32_t oq = q, orr = r;
    asm volatile("" : "+v"(oq), "+v"(orr));
    char* blk_base = const_cast<char*>(base) + (int64_t)pm0 * s_panel + (int64_t)pn0 * s_pn;
    uint32_t col_off[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint32_t col = (uint32_t)(wn * TN + tn) * 16 + 4 * oq;
      col_off[tn] = (col >> a.ln0) * s_pn + (col & ((uint32_t)a.N0 - 1)) * 4;
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const uint32_t row = (uint32_t)(wm * TM + tm) * 16 + orr;
      const uint32_t row_off = (row >> a.lm0) * (uint32_t)s_panel + (row & ((uint32_t)a.M0 - 1)) * s_m0;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        // Scalar base + 32-bit lane offset, as for the operand loads below.
        uint32_t o = row_off + col_off[tn];
        asm volatile("" : "+v"(o));
        f(tm, tn, blk_base + o);
      }
      // Keep the unrolled rows from being hoisted together.
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto init_acc = [&](int pm0, int pn0) {
    if (a.accumulate) {
      for_each_quad(a.acc, a.acc_stride, a.acc_sm0, a.acc_spn, pm0, pn0,
                    [&](int tm, int tn, char* p) { acc[tm][tn] = Out::load4(p); });
    } else {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = Acc{0, 0, 0, 0};
    }
  };
  init_acc(cur_pm0, cur_pn0);

  // ---- load cursors -----------------------------------------------------------
  // pa / pb point at the K step the next LHS / RHS loads fetch, ra / rb count
  // the steps left in that cursor's block. Past the last block the cursors walk
  // the last block again: valid addresses, data nobody uses.
  const char* pa = a.lhs + (int64_t)cur_pm0 * a.lhs_stride;
  const char* pb = a.rhs + (int64_t)cur_pn0 * a.rhs_stride;
  uint32_t ra = steps, rb = steps;
  auto advance_a = [&]() {
    pa += sstep_a;
    if (--ra == 0) { pa = a.lhs + (int64_t)next_pm0 * a.lhs_stride; ra = steps; }
  };
  auto advance_b = [&]() {
    pb += sstep_b;
    if (--rb == 0) { pb = a.rhs + (int64_t)next_pn0 * a.rhs_stride; rb = steps; }
  };
  // The 32-bit lane offsets pass through an empty asm at every use: the loads
  // then take the scalar-base + 32-bit-offset addressing form, where otherwise
  // the offsets would be widened to 64 bits once, outside the loop, and held
  // (and spilled) as register pairs.
  auto load_a = [&](int k) {
    uint32_t o = voff[k];
    asm volatile("" : "+v"(o));
    return *reinterpret_cast<const v4i_g*>(pa + o);
  };
  auto load_b = [&](int tn) {
    uint32_t o = voff_b[tn];
    asm volatile("" : "+v"(o));
    return *reinterpret_cast<const v4i_g*>(pb + o);
  };
  auto read_a = [&](uint32_t stage_off, int tm) {
    return *reinterpret_cast<const v4i*>(lds + stage_off + rd_a + tm * 1024);
  };
  auto store_a = [&](uint32_t stage_off, int k, v4i v) {
    if (!EVEN && wave + k * NW >= BLOCKS) return;
    *reinterpret_cast<v4i*>(lds + stage_off + loff[k]) = v;
  };

  // ---- prologue: what iterations -4 .. -1 would have left behind ----------------
  // Everything that belongs to flattened step s lives in slot s % 4 of its
  // ring: LDS stage, LHS register set, RHS fragment buffer. Only three slots
  // of a ring are live at any time; four make the ring period divide the
  // number of steps of a block (a multiple of four), so that a block boundary
  // always falls between two whole passes of the unrolled loop below.
  v4i regs[4][NU];
  v4i fa[4], fb[4][TN];
#pragma unroll
  for (int k = 0; k < NU; ++k) regs[0][k] = load_a(k);
  advance_a();
#pragma unroll
  for (int k = 0; k < NU; ++k) regs[1][k] = load_a(k);
  advance_a();
#pragma unroll
  for (int k = 0; k < NU; ++k) store_a(0, k, regs[0][k]);
#pragma unroll
  for (int k = 0; k < NU; ++k) store_a(STAGE, k, regs[1][k]);
  // In the loop's own issue order (RHS fragments and LHS pieces interleaved row
  // by row): the in-order wait counters the compiler places in the loop must
  // hold on entry from here as well as around the back edge.
  auto issue_like_iteration = [&](auto slot_b, auto slot_a) {
    constexpr int SB = decltype(slot_b)::value, SA = decltype(slot_a)::value;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn) fb[SB][tn] = load_b(tn);
#pragma unroll
      for (int k = tm * NU / TM; k < (tm + 1) * NU / TM; ++k) regs[SA][k] = load_a(k);
      __builtin_amdgcn_sched_barrier(0);
    }
    advance_a();
    advance_b();
  };
  issue_like_iteration(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{});
  issue_like_iteration(std::integral_constant<int, 1>{}, std::integral_constant<int, 3>{});
  __syncthreads();
  fa[0] = read_a(0, 0);
  fa[1] = read_a(0, 1);

  // ---- the K loop, running on across blocks -------------------------------------
  // Iteration of phase P (flattened step s, P = s % 4) computes step s from
  // LDS stage P and RHS buffer P, issues the LHS global loads of step s + 4
  // into register set P (whose previous contents, step s, went to LDS two
  // iterations ago), stores register set (P+2)%4 (step s + 2) to LDS stage
  // (P+2)%4 and loads the RHS fragments of step s + 2 into buffer (P+2)%4.
  // LHS fragments are fetched two rows ahead; row tm sits in slot tm % 4.
  static_assert(TM % 4 == 0, "fragment slot of a row must not depend on the step");
  auto iteration = [&](auto phase) {
    constexpr int P = decltype(phase)::value;
    constexpr uint32_t st_cur = P * STAGE, st_next = ((P + 1) % 4) * STAGE,
                       st_write = ((P + 2) % 4) * STAGE;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int tn = tm * TN / TM; tn < (tm + 1) * TN / TM; ++tn) fb[(P + 2) % 4][tn] = load_b(tn);
#pragma unroll
      for (int k = tm * NU / TM; k < (tm + 1) * NU / TM; ++k) {
        store_a(st_write, k, regs[(P + 2) % 4][k]);
        regs[P][k] = load_a(k);
      }
      if (tm + 2 < TM) fa[(tm + 2) % 4] = read_a(st_cur, tm + 2);
      else fa[(tm + 2) % 4] = read_a(st_next, tm + 2 - TM);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        acc[tm][tn] = TT::mfma(&fb[P][tn], &fa[tm % 4], acc[tm][tn]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    advance_a();
    advance_b();
  };
  for (uint32_t j = 0; j < ntiles; ++j) {
    for (uint32_t n = steps >> 2; n; --n) {
      iteration(std::integral_constant<int, 0>{});
      iteration(std::integral_constant<int, 1>{});
      iteration(std::integral_constant<int, 2>{});
      iteration(std::integral_constant<int, 3>{});
    }
    // Block j is complete: store it and move on to the next one, whose first
    // steps are already in the pipeline.
    for_each_quad(a.out, a.out_stride, a.out_sm0, a.out_spn, cur_pm0, cur_pn0,
                  [&](int tm, int tn, char* p) { Out::store4(p, acc[tm][tn]); });
    cur_pm0 = next_pm0;
    cur_pn0 = next_pn0;
    if (j + 2 < ntiles) block_panels(j + 2, &next_pm0, &next_pn0);
    if (j + 1 < ntiles) init_acc(cur_pm0, cur_pn0);
  }
}

}  // namespace uk_mfma

#endif  // IREE_UK_AMD_MMT4D_MFMA_PERSISTENT_H_
