// mmt4d on the gfx950 matrix cores for M-thin (decode-shaped) problems: a few
// rows of LHS against a long RHS. Such a call streams the RHS once and is
// bound by memory, so the kernel is built around keeping loads in flight:
//
//   * no LDS staging and no barrier in the K loop. A workgroup owns TM x TN
//     output blocks of 16x16; its KSPLIT waves take the K steps (64 bytes of K
//     per row, 128 for f8) round robin (wave w: steps w, w + KSPLIT, ...), so
//     together they read the workgroup's RHS panels front to back;
//   * each lane loads its MFMA operands straight from global memory, the RHS
//     from HBM and the (small, shared) LHS from L2, D steps ahead of the MFMAs
//     through D register buffers;
//   * the KSPLIT partial accumulators meet in LDS once, at the end, and wave 0
//     adds them in wave order and stores;
//   * when the problem has too few output blocks to occupy the chip (a decode
//     step against a weight matrix with few rows and a long K), K is split
//     over several workgroups per block as well: each publishes its partial
//     block in a workspace, and the one that arrives last (an atomic counter
//     per block) adds the slices in slice order and stores.
//
// Operand layout, K-order freedom of the MFMA and the output addressing are
// those of mmt4d_mfma_kernel.h, whose Args this kernel takes. With TM = TN = 4
// the same kernel serves problems of few 64x64 blocks and a long K, where the
// split of K over the waves matters more than operand reuse. The launcher may
// hand the operands over swapped (RHS as LHS) to serve N-thin problems: rows
// and columns then trade places in Args, four consecutive columns of the
// kernel are four rows of the caller's matrix (so `vec_out` is 0), and the
// scales of a dequantizing store are applied column scale first. Row widths of 16
// bytes and more load one 16-byte piece per operand; 8-byte rows load the two
// 8-byte halves from two K-tiles (chunk g of a step holds K-tiles g and
// g + 4). K must be a whole number of steps.
//
// s8 x s4 -> s32 (Elem::kS8S4) runs here too. A lane loads 8 RHS bytes (16
// nibbles, the same 16 K elements as its 16 LHS bytes) and turns them into two
// groups of eight signed bytes without unpacking to true values: (x << 4) &
// 0xF0F0F0F0 holds 16 * (low nibble as s4) in every byte and x & 0xF0F0F0F0
// holds 16 * (high nibble as s4), i.e. the even and the odd K elements; the
// LHS bytes are split into even and odd positions to match (v_perm_b32). The
// MFMA then accumulates 16 times the true sum, exactly (the launcher bounds K
// so that this cannot wrap), and the store path shifts it back before it adds
// the ACCUMULATE input.
#ifndef IREE_UK_AMD_MMT4D_MFMA_THIN_H_
#define IREE_UK_AMD_MMT4D_MFMA_THIN_H_

#include "mmt4d_mfma_kernel.h"

namespace uk_mfma {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef v2i v2i_g __attribute__((aligned(1)));  // as v4i_g: read from global memory at any address

// STREAMED: the wide operand (the kernel's RHS: weights) is loaded
// non-temporally. For callers that say their weights come from HBM every time
// (iree_uk_amd_set_streamed_weights): a layer's weights then pass through the
// caches without displacing what is used again.
template <Elem E, int RBC, int TM, int TN, int KSPLIT, int D, bool STREAMED = false>
__global__ __launch_bounds__(KSPLIT * 64)
void mmt4d_thin_kernel(Args a) {
  using TT = ElemTraits<E>;
  using Acc = typename TT::Acc;
  using Out = typename TT::Out;
  constexpr int OB = Out::kOutBytes;
  constexpr int HALVES = TT::kHalves;
  constexpr int NCH = 4 * HALVES;             // 16-byte chunks per row per step
  constexpr int KS = NCH * 16;                // bytes of K per row per step
  constexpr int PIECES = RBC >= 16 ? 1 : 2;   // loads per 16-byte operand
  constexpr bool S4 = E == Elem::kS8S4;       // 4-bit RHS: half the bytes per row
  static_assert(RBC >= 8, "rows narrower than 8 bytes take the LDS kernels");
  static_assert(!S4 || RBC >= 16, "4-bit RHS: LHS rows of at least 16 bytes");

  __shared__ v4i partial[KSPLIT > 1 ? KSPLIT - 1 : 1][TM * TN][64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t q = lane >> 4, r = lane & 15;
  // With K split over workgroups, consecutive workgroups share an output block.
  const uint32_t kslices = a.kslices > 1 ? a.kslices : 1;
  const uint32_t block_id = kslices > 1 ? blockIdx.x / kslices : blockIdx.x;
  const uint32_t slice = kslices > 1 ? blockIdx.x - block_id * kslices : 0;
  const int bm = (int)(block_id / (uint32_t)a.grid_n);
  const int bn = (int)(block_id - (uint32_t)bm * a.grid_n);
  // K steps of this workgroup: [step_begin, step_begin + wg_steps).
  const uint32_t step_begin = (uint32_t)(((uint64_t)slice * (uint32_t)a.steps) / kslices);
  const int wg_steps = (int)((((uint64_t)(slice + 1) * (uint32_t)a.steps) / kslices) - step_begin);
  const int lrb = a.lrb;
  const int lrb_b = S4 ? lrb - 1 : lrb;       // log2 of the RHS row bytes
  const uint32_t kt_m = (uint32_t)a.M0 << lrb, kt_n = (uint32_t)a.N0 << lrb_b;
  const uint32_t kts_per_step = KS >> lrb;
  const uint32_t sstep_a = kts_per_step * kt_m, sstep_b = kts_per_step * kt_n;

  // Byte offset of the lane's piece(s) of block row `x` (a row of 16 rows of
  // the M or N dimension) at K step 0; 0 for rows outside the problem, whose
  // (valid) bytes only reach accumulators that are never stored.
  // Offsets are 32-bit and relative to the first panel the workgroup touches.
  const int pa0 = bm * TM * 16 / a.M0, pb0 = bn * TN * 16 / a.N0;
  const char* base_a = a.lhs + (int64_t)pa0 * a.lhs_stride;
  const char* base_b = a.rhs + (int64_t)pb0 * a.rhs_stride;
  auto operand_offsets = [&](uint32_t (&off)[HALVES][PIECES], int x, int X0, int X1, int p0,
                             int64_t stride, uint32_t kt_bytes, int lrb, uint32_t piece_bytes) {
    const uint32_t row = (uint32_t)x * 16 + r;
    const uint32_t pabs = row / (uint32_t)X0;
    const uint32_t x0 = row - pabs * X0;
    const bool ok = (int)pabs < X1;
    const uint32_t pl = pabs - (uint32_t)p0;
#pragma unroll
    for (int h = 0; h < HALVES; ++h) {
      const uint32_t g = (uint32_t)h * 4 + q;
#pragma unroll
      for (int t = 0; t < PIECES; ++t) {
        uint32_t o;
        if constexpr (RBC >= 16) {
          const uint32_t kb = g * piece_bytes;
          o = (kb >> lrb) * kt_bytes + (x0 << lrb) + (kb & ((1u << lrb) - 1));
        } else {
          o = (g + (uint32_t)t * NCH) * kt_bytes + x0 * 8;
        }
        off[h][t] = ok ? pl * (uint32_t)stride + o : 0u;
      }
    }
  };
  uint32_t offa[TM][HALVES][PIECES], offb[TN][HALVES][PIECES];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
    operand_offsets(offa[tm], bm * TM + tm, a.M0, a.M1, pa0, a.lhs_stride, kt_m, lrb, 16);
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
    operand_offsets(offb[tn], bn * TN + tn, a.N0, a.N1, pb0, a.rhs_stride, kt_n, lrb_b,
                    S4 ? 8 : 16);

  auto load_operand = [&](const char* base, const uint32_t (&off)[PIECES], uint32_t adv) {
    if constexpr (RBC >= 16) {
      return *reinterpret_cast<const v4i_g*>(base + (off[0] + adv));
    } else {
      const v2i lo = *reinterpret_cast<const v2i_g*>(base + (off[0] + adv));
      const v2i hi = *reinterpret_cast<const v2i_g*>(base + (off[1] + adv));
      return v4i{lo[0], lo[1], hi[0], hi[1]};
    }
  };
  auto load_wide_operand = [&](const char* base, const uint32_t (&off)[PIECES], uint32_t adv) {
    if constexpr (!STREAMED) {
      return load_operand(base, off, adv);
    } else if constexpr (RBC >= 16) {
      return __builtin_nontemporal_load(reinterpret_cast<const v4i_g*>(base + (off[0] + adv)));
    } else {
      const v2i lo = __builtin_nontemporal_load(reinterpret_cast<const v2i_g*>(base + (off[0] + adv)));
      const v2i hi = __builtin_nontemporal_load(reinterpret_cast<const v2i_g*>(base + (off[1] + adv)));
      return v4i{lo[0], lo[1], hi[0], hi[1]};
    }
  };
  using BFrag = typename std::conditional<S4, v2i, v4i>::type;
  v4i fa[D][TM][HALVES];
  BFrag fb[D][TN][HALVES];
  // Local step i of this wave is K step step_begin + wave + i * KSPLIT.
  auto load_step = [&](int d, int i) {
    const uint32_t s = step_begin + (uint32_t)(wave + i * KSPLIT);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int h = 0; h < HALVES; ++h) {
        if constexpr (S4) {
          const v2i_g* pb = reinterpret_cast<const v2i_g*>(base_b + (offb[tn][h][0] + s * sstep_b));
          if constexpr (STREAMED) fb[d][tn][h] = __builtin_nontemporal_load(pb);
          else fb[d][tn][h] = *pb;
        } else {
          fb[d][tn][h] = load_wide_operand(base_b, offb[tn][h], s * sstep_b);
        }
      }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int h = 0; h < HALVES; ++h) fa[d][tm][h] = load_operand(base_a, offa[tm][h], s * sstep_a);
  };

  // ---- output addressing (see for_each_output in mmt4d_mfma_kernel.h) ------
  // Lane (q, r) of block (tm, tn) holds output row r, columns 4q..4q+3.
  auto for_each_output = [&](const char* base, int64_t s_panel, uint32_t s_m0, uint32_t s_pn,
                             uint32_t s_n0, auto f4, auto f1) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int row = (bm * TM + tm) * 16 + (int)r;
      const int pl = row / a.M0, m0 = row - pl * a.M0;
      const bool row_ok = pl < a.M1 && row < a.out_rows;
      char* row_base = const_cast<char*>(base) + (int64_t)pl * s_panel + (int64_t)m0 * s_m0;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const int col = (bn * TN + tn) * 16 + 4 * (int)q;
        if (a.vec_out) {
          const int pc = col / a.N0, n0 = col - pc * a.N0;
          const int left = a.out_cols - col;
          char* p = row_base + (int64_t)pc * s_pn + (int64_t)n0 * s_n0;
          if (row_ok && pc < a.N1 && left >= 4) {
            f4(tm, tn, p);
          } else if (row_ok && pc < a.N1) {
#pragma unroll
            for (int e = 0; e < 3; ++e)
              if (e < left) f1(tm, tn, e, p + e * s_n0);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int c = col + e;
            const int pc = c / a.N0, n0 = c - pc * a.N0;
            if (row_ok && pc < a.N1 && c < a.out_cols)
              f1(tm, tn, e, row_base + (int64_t)pc * s_pn + (int64_t)n0 * s_n0);
          }
        }
      }
    }
  };

  Acc acc[TM][TN];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = Acc{0, 0, 0, 0};

  // ---- K loop ---------------------------------------------------------------
  const int my_steps = wg_steps > wave ? (wg_steps - wave + KSPLIT - 1) / KSPLIT : 0;
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < my_steps) load_step(d, d);
  // Wave 0, which stores, fetches what the store needs now, under the K loop:
  // the initial accumulators and the scales of the dequantizing store (indices
  // beyond the matrix are clamped; their elements are never stored).
  float sm[TM];
  v4f sn[TN];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) sm[tm] = 1.0f;
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) sn[tn] = v4f{1.0f, 1.0f, 1.0f, 1.0f};
  // With the 4-bit RHS the accumulators hold 16 times the sum, so the
  // ACCUMULATE input waits in registers of its own. With K split over
  // workgroups only the first slice starts from the ACCUMULATE input.
  Acc cin[S4 ? TM : 1][S4 ? TN : 1];
  if constexpr (S4) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) cin[tm][tn] = Acc{0, 0, 0, 0};
  }
  if (wave == 0) {
    if (a.accumulate && slice == 0) {
      for_each_output(a.acc, a.acc_stride, a.acc_sm0, a.acc_spn, a.acc_sn0,
                      [&](int tm, int tn, char* p) {
                        if constexpr (S4) cin[tm][tn] = Out::load4(p);
                        else acc[tm][tn] = Out::load4(p);
                      },
                      [&](int tm, int tn, int e, char* p) {
                        if constexpr (S4) cin[tm][tn][e] = Out::load1(p);
                        else acc[tm][tn][e] = Out::load1(p);
                      });
    }
    if (OB == 4 && a.dequant) {
      if (a.row_scale) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          sm[tm] = a.row_scale[max(min((bm * TM + tm) * 16 + (int)r, a.out_rows - 1), 0)];
      }
      if (a.col_scale) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            sn[tn][e] =
                a.col_scale[max(min((bn * TN + tn) * 16 + 4 * (int)q + e, a.out_cols - 1), 0)];
      }
    }
  }
  auto compute = [&](int d) {
    if constexpr (S4) {
      // LHS: even K bytes, then odd K bytes; RHS: low nibbles, then high ones.
      v4i ea[TM], eb[TN];
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const v4i x = fa[d][tm][0];
        ea[tm] = v4i{(int)__builtin_amdgcn_perm((uint32_t)x[1], (uint32_t)x[0], 0x06040200u),
                     (int)__builtin_amdgcn_perm((uint32_t)x[3], (uint32_t)x[2], 0x06040200u),
                     (int)__builtin_amdgcn_perm((uint32_t)x[1], (uint32_t)x[0], 0x07050301u),
                     (int)__builtin_amdgcn_perm((uint32_t)x[3], (uint32_t)x[2], 0x07050301u)};
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const uint32_t x0 = (uint32_t)fb[d][tn][0][0], x1 = (uint32_t)fb[d][tn][0][1];
        eb[tn] = v4i{(int)((x0 << 4) & 0xF0F0F0F0u), (int)((x1 << 4) & 0xF0F0F0F0u),
                     (int)(x0 & 0xF0F0F0F0u), (int)(x1 & 0xF0F0F0F0u)};
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = TT::mfma(&eb[tn], &ea[tm], acc[tm][tn]);
    } else {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = TT::mfma(fb[d][tn], fa[d][tm], acc[tm][tn]);
    }
  };
  int i = 0;
  // Steady state: every step computed is followed by the load of the step D
  // further on, which exists.
  for (; i + 2 * D <= my_steps; i += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      compute(d);
      load_step(d, i + d + D);
    }
  }
  // Fewer than 2 D steps left: the same with bounds.
#pragma unroll
  for (int d = 0; d < D; ++d) {
    if (i + d < my_steps) {
      compute(d);
      if (i + d + D < my_steps) load_step(d, i + d + D);
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (i + D + d < my_steps) compute(d);

  // ---- meet the partial sums ---------------------------------------------------
  if constexpr (KSPLIT > 1) {
    if (wave > 0) {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          partial[wave - 1][tm * TN + tn][lane] = __builtin_bit_cast(v4i, acc[tm][tn]);
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < KSPLIT - 1; ++w)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
          acc[tm][tn] += __builtin_bit_cast(Acc, partial[w][tm * TN + tn][lane]);
  }

  if constexpr (S4) {
    // Every slice holds 16 times its part of the sum (plus, in slice 0, nothing
    // else: the ACCUMULATE input waits in cin), so the shift is exact per slice.
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = (acc[tm][tn] >> 4) + cin[tm][tn];
  }

  // ---- meet the K slices of the other workgroups -----------------------------------
  // Only wave 0 is left. It publishes this workgroup's partial block, then
  // counts itself in; the workgroup that arrives last adds the slices up in
  // slice order (so a float result does not depend on who arrived when) and
  // goes on to store. The slices run on different XCDs, each with an L2 of
  // its own, so partials and counter are moved with device-scope atomic
  // accesses (relaxed 32-bit stores and loads: they go through to the point
  // where the XCDs meet and leave the caches alone). A device-scope FENCE
  // would be correct too and is far too expensive here: it writes back and
  // invalidates the whole L2, under the feet of every workgroup that streams
  // weights through it. What the counter increment has to wait for is only
  // that this wave's own partial stores are complete.
  if (kslices > 1) {
    uint32_t* mine = reinterpret_cast<uint32_t*>(a.ws_partials) +
                     (((size_t)block_id * kslices + slice) * (TM * TN * 64) + lane) * 4;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const v4i v = __builtin_bit_cast(v4i, acc[tm][tn]);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          __hip_atomic_store(mine + (tm * TN + tn) * 256 + e, (uint32_t)v[e], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      }
    // All of the wave's stores above have been acknowledged before the count.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    uint32_t arrived = 0;
    if (lane == 0) {
      arrived = __hip_atomic_fetch_add(a.ws_counters + block_id, 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    }
    arrived = (uint32_t)__builtin_amdgcn_readfirstlane((int)arrived);
    if (arrived != kslices - 1) return;
    // The reader side of the handoff. What the other slices stored is complete
    // at the point where the XCDs meet before their counter increments (their
    // agent-scope stores are acknowledged from there, and each waited for its
    // own before counting), and the agent-scope loads below go to that point
    // instead of a cache; this fence only keeps the compiler from moving those
    // loads above the test of the counter (workgroup scope: it costs no cache
    // write-back or invalidation).
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (lane == 0) {
      __hip_atomic_store(a.ws_counters + block_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const uint32_t* all = reinterpret_cast<const uint32_t*>(a.ws_partials) +
                          ((size_t)block_id * kslices * (TM * TN * 64) + lane) * 4;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) acc[tm][tn] = Acc{0, 0, 0, 0};
    for (uint32_t sl = 0; sl < kslices; ++sl) {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          v4i v;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[e] = (int)__hip_atomic_load(all + ((size_t)sl * (TM * TN) + tm * TN + tn) * 256 + e,
                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          acc[tm][tn] += __builtin_bit_cast(Acc, v);
        }
    }
  }

  // ---- store --------------------------------------------------------------------
  if constexpr (OB == 4) {
    if (a.dequant) {
      typedef v4f v4f_a4 __attribute__((aligned(4)));
      for_each_output(
          a.out, a.out_stride, a.out_sm0, a.out_spn, a.out_sn0,
          [&](int tm, int tn, char* p) {
            v4f v = __builtin_convertvector(acc[tm][tn], v4f);
            if (a.col_scale_first) {
              v = v * sn[tn];
              v = v * sm[tm];
            } else {
              v = v * sm[tm];
              v = v * sn[tn];
            }
            *reinterpret_cast<v4f_a4*>(p) = v;
          },
          [&](int tm, int tn, int e, char* p) {
            const float v = (float)acc[tm][tn][e];
            *reinterpret_cast<float*>(p) =
                a.col_scale_first ? v * sn[tn][e] * sm[tm] : v * sm[tm] * sn[tn][e];
          });
      return;
    }
  }
  for_each_output(a.out, a.out_stride, a.out_sm0, a.out_spn, a.out_sn0,
                  [&](int tm, int tn, char* p) { Out::store4(p, acc[tm][tn]); },
                  [&](int tm, int tn, int e, char* p) { Out::store1(p, acc[tm][tn][e]); });
}

}  // namespace uk_mfma

#endif  // IREE_UK_AMD_MMT4D_MFMA_THIN_H_
