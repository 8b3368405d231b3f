// pack / unpack for gfx950: HBM-bound byte movement between a 2-D matrix and
// its 4-D tiled form.
//
// Index algebra (runtime/src/iree/builtins/ukernel/tools/pack_test.c:13-71,
// unpack_test.c:13-58): with (outer0, outer1, tile0, tile1) the stored 4-D
// shape after undoing TRANSPOSE_OUTER / TRANSPOSE_INNER, matrix element
// (a0*tile0 + b0, a1*tile1 + b1) lives at tiled offset
//   a0*sl0 + a1*sl1 + b0*sl2 + b1*sl3.
//
// Two kernel families serve each op:
//   *_generic : one thread per destination element, any shape/stride/type.
//   *_tiled   : a workgroup stages a G0 x G1 block of tiles through LDS, held
//               in LDS as the row-major 2-D matrix block. Global reads and
//               writes are both contiguous runs of >= 256 bytes moved with up
//               to 16-byte vectors; the tile regrouping (and the transposes)
//               happens in the LDS addressing. Needs a unit inner stride on
//               the 2-D side and 4-byte alignment on the tiled side.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "uk_device_common.h"
#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace {

using uk::FastDiv;

constexpr int kThreads = 256;

//===----------------------------------------------------------------------===//
// Logical view shared by pack and unpack.
//===----------------------------------------------------------------------===//

struct TiledView {
  int64_t outer0, outer1, tile0, tile1;  // after undoing the transposes
  int64_t sl0, sl1, sl2, sl3;            // tiled-side strides, elements
  int64_t size0, size1;                  // stored 4-D outer shape
  int64_t size2, size3;                  // stored tile shape
  int64_t stride0;                       // stored outer stride, elements
};

TiledView make_view(int64_t size0, int64_t size1, int64_t size2, int64_t size3,
                    int64_t stride0, bool transpose_inner,
                    bool transpose_outer) {
  TiledView v;
  v.size0 = size0; v.size1 = size1; v.size2 = size2; v.size3 = size3;
  v.stride0 = stride0;
  v.outer0 = size0; v.outer1 = size1; v.tile0 = size2; v.tile1 = size3;
  v.sl0 = stride0; v.sl1 = size2 * size3; v.sl2 = size3; v.sl3 = 1;
  if (transpose_outer) { std::swap(v.outer0, v.outer1); std::swap(v.sl0, v.sl1); }
  if (transpose_inner) { std::swap(v.tile0, v.tile1); std::swap(v.sl2, v.sl3); }
  return v;
}

//===----------------------------------------------------------------------===//
// Generic kernels.
//===----------------------------------------------------------------------===//

struct GenericArgs {
  const char* src;
  char* dst;
  int64_t mat_stride0, mat_stride1;  // 2-D side strides, elements
  int64_t mat_size0, mat_size1;      // 2-D side sizes
  int64_t tile0, tile1;
  int64_t sl0, sl1, sl2, sl3;
  int64_t size1, size2, size3, stride0;  // stored 4-D shape (size0 implied)
  int64_t total;                         // number of destination elements
  uint64_t pad;
  int transpose_inner, transpose_outer;
};

// One thread per element of the tiled destination.
template <typename T>
__global__ __launch_bounds__(kThreads) void pack_generic_kernel(GenericArgs a) {
  const int64_t tile_elems = a.size2 * a.size3;
  const int64_t row_elems = a.size1 * tile_elems;
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < a.total;
       idx += (int64_t)gridDim.x * kThreads) {
    const int64_t o0 = idx / row_elems;
    const int64_t rem = idx - o0 * row_elems;
    const int64_t o1 = rem / tile_elems;
    const int64_t t = rem - o1 * tile_elems;
    const int64_t o2 = t / a.size3;
    const int64_t o3 = t - o2 * a.size3;
    const int64_t a0 = a.transpose_outer ? o1 : o0;
    const int64_t a1 = a.transpose_outer ? o0 : o1;
    const int64_t b0 = a.transpose_inner ? o3 : o2;
    const int64_t b1 = a.transpose_inner ? o2 : o3;
    const int64_t i0 = a0 * a.tile0 + b0;
    const int64_t i1 = a1 * a.tile1 + b1;
    T v;
    if (i0 < a.mat_size0 && i1 < a.mat_size1) {
      v = reinterpret_cast<const T*>(a.src)[i0 * a.mat_stride0 + i1 * a.mat_stride1];
    } else {
      v = (T)a.pad;
    }
    reinterpret_cast<T*>(a.dst)[o0 * a.stride0 + rem] = v;
  }
}

// One thread per element of the 2-D destination.
template <typename T>
__global__ __launch_bounds__(kThreads) void unpack_generic_kernel(GenericArgs a) {
  for (int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x; idx < a.total;
       idx += (int64_t)gridDim.x * kThreads) {
    const int64_t i0 = idx / a.mat_size1;
    const int64_t i1 = idx - i0 * a.mat_size1;
    const int64_t a0 = i0 / a.tile0, b0 = i0 - a0 * a.tile0;
    const int64_t a1 = i1 / a.tile1, b1 = i1 - a1 * a.tile1;
    const T v = reinterpret_cast<const T*>(
        a.src)[a0 * a.sl0 + a1 * a.sl1 + b0 * a.sl2 + b1 * a.sl3];
    reinterpret_cast<T*>(a.dst)[i0 * a.mat_stride0 + i1 * a.mat_stride1] = v;
  }
}

int grid_for(int64_t total) {
  int64_t blocks = uk::ceil_div(total, kThreads);
  const int64_t cap = 256 * 64;  // grid-stride beyond this
  return (int)(blocks < cap ? blocks : cap);
}

//===----------------------------------------------------------------------===//
// Tiled kernels.
//===----------------------------------------------------------------------===//

struct TiledArgs {
  const char* src;
  char* dst;
  int64_t mat_stride0_bytes;        // 2-D side row pitch
  int64_t sl0_bytes, sl1_bytes;     // tiled side: byte step of a0 / a1
  uint32_t mat_size0, mat_size1;    // 2-D side sizes, elements
  uint32_t outer0, outer1;          // tile counts (logical)
  uint32_t tile0, tile1;            // logical tile shape, elements
  uint32_t G0, G1;                  // tiles per block along each dim
  uint32_t nblk1;                   // blocks along dim 1
  uint32_t lds_pitch;               // bytes per LDS row
  uint32_t lds_piece;               // largest aligned LDS access on a row, bytes
  uint32_t elem_bytes;
  uint32_t block_rows;              // G0*tile0
  uint32_t block_row_bytes;         // G1*tile1*elem_bytes
  uint32_t mat_vec;                 // 2-D side global vector width, bytes
  uint32_t transpose_inner, transpose_outer;
  uint32_t pad32;                   // padding element replicated to 32 bits
  uint32_t tile_bytes;              // tile0*tile1*elem_bytes
  uint32_t run_tiles;               // tiles per contiguous tiled-side run
  uint32_t num_runs;                // runs per block
  uint32_t run_vecs;                // tiled-side vectors per run
  uint32_t tile_row_grans;          // granules per logical tile row (non-TI)
  FastDiv div_row_vecs;             // 2-D side vectors per block row
  FastDiv div_run_vecs;
  FastDiv div_tile_grans;           // granules per tile
  FastDiv div_tile_row_grans;
  FastDiv div_tile0;
  FastDiv div_tile_bytes;
  uint32_t nblk0;                   // blocks along dim 0
  uint32_t lds_buf_bytes;           // one LDS buffer of the streaming kernels
  uint32_t mat_stride0_bytes32;     // == mat_stride0_bytes when it fits
  uint32_t sl0_bytes32, sl1_bytes32;
  uint32_t streaming_stores;        // 16 KB-block streaming kernels: non-temporal stores
};

template <int N> struct Bytes;
template <> struct Bytes<1> { using type = uint8_t; };
template <> struct Bytes<2> { using type = uint16_t; };
template <> struct Bytes<4> { using type = uint32_t; };
template <> struct Bytes<8> { using type = uint2; };
template <> struct Bytes<16> { using type = uint4; };

template <int N>
__device__ __forceinline__ void copy_bytes(void* dst, const void* src) {
  using T = typename Bytes<N>::type;
  *reinterpret_cast<T*>(dst) = *reinterpret_cast<const T*>(src);
}

// Copies n = VEC bytes between a register buffer and memory using accesses of
// `piece` bytes (piece divides VEC, wave-uniform).
template <int VEC>
__device__ __forceinline__ void store_pieces(char* dst, const char* reg,
                                             uint32_t piece) {
  if (piece >= VEC) {
    copy_bytes<VEC>(dst, reg);
  } else if (VEC > 8 && piece == 8) {
#pragma unroll
    for (int i = 0; i < VEC; i += 8) copy_bytes<8>(dst + i, reg + i);
  } else if (VEC > 4 && piece == 4) {
#pragma unroll
    for (int i = 0; i < VEC; i += 4) copy_bytes<4>(dst + i, reg + i);
  } else if (VEC > 2 && piece == 2) {
#pragma unroll
    for (int i = 0; i < VEC; i += 2) copy_bytes<2>(dst + i, reg + i);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) dst[i] = reg[i];
  }
}

template <int VEC>
__device__ __forceinline__ void load_pieces(char* reg, const char* src,
                                            uint32_t piece) {
  if (piece >= VEC) {
    copy_bytes<VEC>(reg, src);
  } else if (VEC > 8 && piece == 8) {
#pragma unroll
    for (int i = 0; i < VEC; i += 8) copy_bytes<8>(reg + i, src + i);
  } else if (VEC > 4 && piece == 4) {
#pragma unroll
    for (int i = 0; i < VEC; i += 4) copy_bytes<4>(reg + i, src + i);
  } else if (VEC > 2 && piece == 2) {
#pragma unroll
    for (int i = 0; i < VEC; i += 2) copy_bytes<2>(reg + i, src + i);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) reg[i] = src[i];
  }
}

// LDS byte offset of the granule that starts at logical (tl0, tl1, b0, b1) of
// the block held row-major in LDS.
__device__ __forceinline__ uint32_t lds_offset(const TiledArgs& a, uint32_t tl0,
                                               uint32_t tl1, uint32_t b0,
                                               uint32_t b1) {
  return (tl0 * a.tile0 + b0) * a.lds_pitch +
         (tl1 * a.tile1 + b1) * a.elem_bytes;
}

// Walks the granules of one tiled-side vector. `pos` is the byte position of
// the vector inside its run. Calls f(i, lds_byte_offset) for granule i.
template <int G, int VEC, typename F>
__device__ __forceinline__ void for_each_granule(const TiledArgs& a, uint32_t run,
                                                 uint32_t t, uint32_t in_tile_byte,
                                                 F f) {
  const uint32_t tl0 = a.transpose_outer ? t : run;
  const uint32_t tl1 = a.transpose_outer ? run : t;
  uint32_t qg = in_tile_byte / G;  // granule index inside the tile
  uint32_t b0, b1;
  if (a.transpose_inner) {
    // Stored tile is [b1][b0]; a granule is one element.
    a.div_tile0.divmod(qg, b1, b0);
  } else {
    uint32_t b1g;
    a.div_tile_row_grans.divmod(qg, b0, b1g);
    b1 = b1g * (G / a.elem_bytes);
  }
#pragma unroll
  for (int i = 0; i < VEC / G; ++i) {
    f(i, lds_offset(a, tl0, tl1, b0, b1));
    if (a.transpose_inner) {
      if (++b0 == a.tile0) { b0 = 0; ++b1; }
    } else {
      b1 += G / a.elem_bytes;
      if (b1 == a.tile1) { b1 = 0; ++b0; }
    }
  }
}

// pack: 2-D rows -> LDS (phase 1, contiguous), LDS -> tiled runs (phase 2,
// gather by granules of G bytes into VEC-byte vectors).
template <int G, int VEC>
__global__ __launch_bounds__(kThreads) void pack_tiled_kernel(TiledArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const uint32_t blk0 = blockIdx.x / a.nblk1;
  const uint32_t blk1 = blockIdx.x - blk0 * a.nblk1;
  const uint32_t row_base = blk0 * a.block_rows;
  const uint32_t col_base_bytes = blk1 * a.block_row_bytes;
  const uint32_t es = a.elem_bytes;
  const uint32_t size1_bytes = a.mat_size1 * es;

  // Phase 1.
  {
    const uint32_t mv = a.mat_vec;
    const uint32_t row_vecs = a.div_row_vecs.d;
    const uint32_t total = a.block_rows * row_vecs;
    const uint32_t piece = a.lds_piece < mv ? a.lds_piece : mv;
    for (uint32_t idx = threadIdx.x; idx < total; idx += kThreads) {
      uint32_t r, v;
      a.div_row_vecs.divmod(idx, r, v);
      const uint32_t grow = row_base + r;
      const uint32_t cb = col_base_bytes + v * mv;  // byte column in the matrix
      __attribute__((aligned(16))) char reg[16];
      const bool row_ok = grow < a.mat_size0;
      const char* gp = a.src + (int64_t)grow * a.mat_stride0_bytes + cb;
      if (row_ok && cb + mv <= size1_bytes) {
        switch (mv) {
          case 16: copy_bytes<16>(reg, gp); break;
          case 8: copy_bytes<8>(reg, gp); break;
          case 4: copy_bytes<4>(reg, gp); break;
          case 2: copy_bytes<2>(reg, gp); break;
          default: reg[0] = gp[0]; break;
        }
      } else {
        // Edge: element-wise, padding outside the matrix.
        for (uint32_t b = 0; b < mv; b += es) {
          const bool ok = row_ok && (cb + b) < size1_bytes;
          if (es == 4) {
            uint32_t w = ok ? *reinterpret_cast<const uint32_t*>(gp + b) : a.pad32;
            *reinterpret_cast<uint32_t*>(reg + b) = w;
          } else if (es == 2) {
            uint16_t w = ok ? *reinterpret_cast<const uint16_t*>(gp + b)
                            : (uint16_t)a.pad32;
            *reinterpret_cast<uint16_t*>(reg + b) = w;
          } else {
            reg[b] = ok ? gp[b] : (char)a.pad32;
          }
        }
      }
      char* lp = lds + r * a.lds_pitch + v * mv;
      switch (mv) {
        case 16: store_pieces<16>(lp, reg, piece); break;
        case 8: store_pieces<8>(lp, reg, piece); break;
        case 4: store_pieces<4>(lp, reg, piece); break;
        case 2: store_pieces<2>(lp, reg, piece); break;
        default: lp[0] = reg[0]; break;
      }
    }
  }
  __syncthreads();

  // Phase 2.
  {
    const uint32_t total = a.num_runs * a.run_vecs;
    for (uint32_t idx = threadIdx.x; idx < total; idx += kThreads) {
      uint32_t run, v;
      a.div_run_vecs.divmod(idx, run, v);
      const uint32_t pos = v * VEC;
      const uint32_t t = pos / a.tile_bytes;  // tile inside the run
      const uint32_t in_tile = pos - t * a.tile_bytes;
      const uint32_t tl0 = a.transpose_outer ? t : run;
      const uint32_t tl1 = a.transpose_outer ? run : t;
      const uint32_t a0 = blk0 * a.G0 + tl0;
      const uint32_t a1 = blk1 * a.G1 + tl1;
      if (a0 >= a.outer0 || a1 >= a.outer1) continue;
      __attribute__((aligned(16))) char reg[VEC];
      for_each_granule<G, VEC>(a, run, t, in_tile, [&](int i, uint32_t off) {
        copy_bytes<G>(reg + i * G, lds + off);
      });
      char* gp = a.dst + (int64_t)a0 * a.sl0_bytes + (int64_t)a1 * a.sl1_bytes + in_tile;
      copy_bytes<VEC>(gp, reg);
    }
  }
}

// unpack: tiled runs -> LDS (phase 1, scatter by granules), LDS rows -> 2-D
// rows (phase 2, contiguous, clipped to the matrix bounds).
template <int G, int VEC>
__global__ __launch_bounds__(kThreads) void unpack_tiled_kernel(TiledArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const uint32_t blk0 = blockIdx.x / a.nblk1;
  const uint32_t blk1 = blockIdx.x - blk0 * a.nblk1;
  const uint32_t row_base = blk0 * a.block_rows;
  const uint32_t col_base_bytes = blk1 * a.block_row_bytes;
  const uint32_t es = a.elem_bytes;
  const uint32_t size1_bytes = a.mat_size1 * es;

  // Phase 1.
  {
    const uint32_t total = a.num_runs * a.run_vecs;
    for (uint32_t idx = threadIdx.x; idx < total; idx += kThreads) {
      uint32_t run, v;
      a.div_run_vecs.divmod(idx, run, v);
      const uint32_t pos = v * VEC;
      const uint32_t t = pos / a.tile_bytes;
      const uint32_t in_tile = pos - t * a.tile_bytes;
      const uint32_t tl0 = a.transpose_outer ? t : run;
      const uint32_t tl1 = a.transpose_outer ? run : t;
      const uint32_t a0 = blk0 * a.G0 + tl0;
      const uint32_t a1 = blk1 * a.G1 + tl1;
      if (a0 >= a.outer0 || a1 >= a.outer1) continue;
      __attribute__((aligned(16))) char reg[VEC];
      const char* gp =
          a.src + (int64_t)a0 * a.sl0_bytes + (int64_t)a1 * a.sl1_bytes + in_tile;
      copy_bytes<VEC>(reg, gp);
      for_each_granule<G, VEC>(a, run, t, in_tile, [&](int i, uint32_t off) {
        copy_bytes<G>(lds + off, reg + i * G);
      });
    }
  }
  __syncthreads();

  // Phase 2.
  {
    const uint32_t mv = a.mat_vec;
    const uint32_t row_vecs = a.div_row_vecs.d;
    const uint32_t total = a.block_rows * row_vecs;
    const uint32_t piece = a.lds_piece < mv ? a.lds_piece : mv;
    for (uint32_t idx = threadIdx.x; idx < total; idx += kThreads) {
      uint32_t r, v;
      a.div_row_vecs.divmod(idx, r, v);
      const uint32_t grow = row_base + r;
      const uint32_t cb = col_base_bytes + v * mv;
      if (grow >= a.mat_size0 || cb >= size1_bytes) continue;
      __attribute__((aligned(16))) char reg[16];
      const char* lp = lds + r * a.lds_pitch + v * mv;
      switch (mv) {
        case 16: load_pieces<16>(reg, lp, piece); break;
        case 8: load_pieces<8>(reg, lp, piece); break;
        case 4: load_pieces<4>(reg, lp, piece); break;
        case 2: load_pieces<2>(reg, lp, piece); break;
        default: reg[0] = lp[0]; break;
      }
      char* gp = a.dst + (int64_t)grow * a.mat_stride0_bytes + cb;
      if (cb + mv <= size1_bytes) {
        switch (mv) {
          case 16: copy_bytes<16>(gp, reg); break;
          case 8: copy_bytes<8>(gp, reg); break;
          case 4: copy_bytes<4>(gp, reg); break;
          case 2: copy_bytes<2>(gp, reg); break;
          default: gp[0] = reg[0]; break;
        }
      } else {
        for (uint32_t b = 0; b < mv && cb + b < size1_bytes; b += es) {
          if (es == 4) copy_bytes<4>(gp + b, reg + b);
          else if (es == 2) copy_bytes<2>(gp + b, reg + b);
          else gp[b] = reg[b];
        }
      }
    }
  }
}


//===----------------------------------------------------------------------===//
// Streaming (persistent) tiled kernels.
//
// Same two-phase LDS scheme as the kernels above, restructured so that the
// per-byte instruction count is small enough for HBM to be the bound:
//   * a workgroup walks many blocks; everything that depends only on the
//     thread and the block shape (global offsets inside a block, LDS offsets
//     of every granule) is computed once, before the walk;
//   * all loads of a phase are issued before any of their data is used, one
//     or two blocks ahead of their use;
//   * LDS is double-buffered, one barrier per block, so the stores of block b
//     and the loads of the following blocks are in flight together;
//   * interior blocks in which every thread has all of its items run without
//     per-item bounds checks.
// Blocks on the ragged edge of the matrix take a slower, bounds-checked path
// (their loads are issued ahead all the same, predicated).
//===----------------------------------------------------------------------===//

typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
template <int N> struct GBytes;
template <> struct GBytes<4> { using type = uint32_t; };
template <> struct GBytes<8> { using type = v2u; };
template <> struct GBytes<16> { using type = v4u; };

// Global accesses of the streaming kernels. Addresses are 4-byte aligned at
// least; wider vectors at such addresses are legal on gfx950 under HSA
// (unaligned access mode), and the types say so.
// Plain (cache-allocating) accesses on purpose: what pack writes is read by
// mmt4d next, and what unpack reads was just written by mmt4d, so for operands
// up to the size of the memory-side cache the hand-over never reaches HBM.
// STREAMING: a non-temporal load, for data that no later block and no later
// kernel reads again (see TiledPlan::streaming_loads).
template <int N, bool STREAMING = false>
__device__ __forceinline__ typename GBytes<N>::type gload(const char* gptr) {
  typedef typename GBytes<N>::type T4 __attribute__((aligned(4)));
  if constexpr (STREAMING) return __builtin_nontemporal_load(reinterpret_cast<const T4*>(gptr));
  else return *reinterpret_cast<const T4*>(gptr);
}
// STREAMING: a non-temporal store, for the 64 KB-block kernels, whose output is
// larger than the memory-side cache anyway (measured 3 % on a plain copy).
template <int N, bool STREAMING = false>
__device__ __forceinline__ void gstore(char* gptr, typename GBytes<N>::type v) {
  typedef typename GBytes<N>::type T4 __attribute__((aligned(4)));
  if constexpr (STREAMING) __builtin_nontemporal_store(v, reinterpret_cast<T4*>(gptr));
  else *reinterpret_cast<T4*>(gptr) = v;
}

// The non-temporal store chosen at run time, as assembly: beside a plain
// store of the same value to the same address in the other branch, the
// compiler merges the two into one plain store.
template <int N>
__device__ __forceinline__ void gstore_nt_asm(char* gptr, typename GBytes<N>::type v) {
  if constexpr (N == 16) asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(gptr), "v"(v) : "memory");
  else if constexpr (N == 8) asm volatile("global_store_dwordx2 %0, %1, off nt" : : "v"(gptr), "v"(v) : "memory");
  else asm volatile("global_store_dword %0, %1, off nt" : : "v"(gptr), "v"(v) : "memory");
}

constexpr uint32_t kStreamBlockBytes = 16384;     // matrix bytes per block, streaming kernels
constexpr uint32_t kStreamBigBlockBytes = 65536;  // same, large transposing problems

struct StreamTables1 {  // 2-D side items of one thread
  uint32_t goff;        // byte offset inside the block's 2-D window
  uint32_t loff;        // LDS byte offset
};

// Items of the 2-D side: vector idx of the block -> row r, vector v.
template <int MV>
__device__ __forceinline__ void mat_item(const TiledArgs& a, uint32_t idx,
                                         uint32_t* r, uint32_t* cb) {
  uint32_t v;
  a.div_row_vecs.divmod(idx, *r, v);
  *cb = v * MV;
}

// Items of the tiled side: vector idx of the block -> run, tile, byte in tile.
template <int VEC>
__device__ __forceinline__ void tiled_item(const TiledArgs& a, uint32_t idx,
                                           uint32_t* run, uint32_t* t,
                                           uint32_t* in_tile, uint32_t* tl0,
                                           uint32_t* tl1) {
  uint32_t v;
  a.div_run_vecs.divmod(idx, *run, v);
  const uint32_t pos = v * VEC;
  *t = a.div_tile_bytes.div(pos);
  *in_tile = pos - *t * a.tile_bytes;
  *tl0 = a.transpose_outer ? *t : *run;
  *tl1 = a.transpose_outer ? *run : *t;
}

template <int N>
__device__ __forceinline__ void lds_store_pieces(char* dst, typename GBytes<N>::type v,
                                                 uint32_t piece) {
  if (piece >= N) {
    *reinterpret_cast<typename GBytes<N>::type*>(dst) = v;
  } else {
    __attribute__((aligned(16))) char tmp[N];
    *reinterpret_cast<typename GBytes<N>::type*>(tmp) = v;
    store_pieces<N>(dst, tmp, piece);
  }
}
template <int N>
__device__ __forceinline__ typename GBytes<N>::type lds_load_pieces(const char* src,
                                                                     uint32_t piece) {
  if (piece >= N) return *reinterpret_cast<const typename GBytes<N>::type*>(src);
  __attribute__((aligned(16))) char tmp[N];
  load_pieces<N>(tmp, src, piece);
  return *reinterpret_cast<const typename GBytes<N>::type*>(tmp);
}

// The same with the piece size known at compile time (P divides N, P >= 4):
// the hot path of the streaming kernels picks P once per block.
template <int N> struct Words { uint32_t w[N / 4]; };
template <int N, int P>
__device__ __forceinline__ void lds_store_static(char* dst, typename GBytes<N>::type v) {
  if constexpr (P >= N) {
    *reinterpret_cast<typename GBytes<N>::type*>(dst) = v;
  } else {
    const Words<N> x = __builtin_bit_cast(Words<N>, v);
#pragma unroll
    for (int j = 0; j < N / P; ++j) {
      Words<P> y;
#pragma unroll
      for (int k = 0; k < P / 4; ++k) y.w[k] = x.w[j * (P / 4) + k];
      *reinterpret_cast<typename GBytes<P>::type*>(dst + j * P) =
          __builtin_bit_cast(typename GBytes<P>::type, y);
    }
  }
}
template <int N, int P>
__device__ __forceinline__ typename GBytes<N>::type lds_load_static(const char* src) {
  if constexpr (P >= N) {
    return *reinterpret_cast<const typename GBytes<N>::type*>(src);
  } else {
    Words<N> x;
#pragma unroll
    for (int j = 0; j < N / P; ++j) {
      const Words<P> y = __builtin_bit_cast(
          Words<P>, *reinterpret_cast<const typename GBytes<P>::type*>(src + j * P));
#pragma unroll
      for (int k = 0; k < P / 4; ++k) x.w[j * (P / 4) + k] = y.w[k];
    }
    return __builtin_bit_cast(typename GBytes<N>::type, x);
  }
}
// Four words rotated by a per-lane amount s in 0..3: y[g] = x[(g - s) & 3]
// (rotate_up) or y[g] = x[(g + s) & 3] (rotate_down), as selects.
__device__ __forceinline__ void rotate_up4(uint32_t (&x)[4], uint32_t s) {
  const bool b1 = s & 1, b2 = s & 2;
  const uint32_t a0 = b1 ? x[3] : x[0], a1 = b1 ? x[0] : x[1], a2 = b1 ? x[1] : x[2],
                 a3 = b1 ? x[2] : x[3];
  x[0] = b2 ? a2 : a0; x[1] = b2 ? a3 : a1; x[2] = b2 ? a0 : a2; x[3] = b2 ? a1 : a3;
}
__device__ __forceinline__ void rotate_down4(uint32_t (&x)[4], uint32_t s) {
  rotate_up4(x, (4 - s) & 3);
}

// A tiled-side vector of VEC bytes from / to its VEC / G granules in LDS.
// With four 4-byte granules per vector a lane may visit its granules in
// rotated order (`off` is then the rotated table, access k touching granule
// (k + rot) & 3) so that the lanes of one LDS instruction spread over the
// banks; the words are rotated back in registers.
template <int VEC, int G>
__device__ __forceinline__ typename GBytes<VEC>::type gather_granules(
    const char* lbuf, const uint32_t (&off)[VEC / G], uint32_t rot) {
  Words<VEC> x;
#pragma unroll
  for (int k = 0; k < VEC / G; ++k) {
    const Words<G> y = __builtin_bit_cast(
        Words<G>, *reinterpret_cast<const typename GBytes<G>::type*>(lbuf + off[k]));
#pragma unroll
    for (int j = 0; j < G / 4; ++j) x.w[k * (G / 4) + j] = y.w[j];
  }
  if constexpr (VEC == 16 && G == 4) rotate_up4(x.w, rot);
  return __builtin_bit_cast(typename GBytes<VEC>::type, x);
}
template <int VEC, int G>
__device__ __forceinline__ void scatter_granules(char* lbuf, const uint32_t (&off)[VEC / G],
                                                 typename GBytes<VEC>::type v, uint32_t rot) {
  Words<VEC> x = __builtin_bit_cast(Words<VEC>, v);
  if constexpr (VEC == 16 && G == 4) rotate_down4(x.w, rot);
#pragma unroll
  for (int k = 0; k < VEC / G; ++k) {
    Words<G> y;
#pragma unroll
    for (int j = 0; j < G / 4; ++j) y.w[j] = x.w[k * (G / 4) + j];
    *reinterpret_cast<typename GBytes<G>::type*>(lbuf + off[k]) =
        __builtin_bit_cast(typename GBytes<G>::type, y);
  }
}
// Calls f with the piece size as a compile-time constant (4, 8 or 16, capped
// at N); false when `piece` is none of them.
template <int N, typename F>
__device__ __forceinline__ bool with_static_piece(uint32_t piece, F f) {
  if (piece >= N) { f(std::integral_constant<int, N>{}); return true; }
  if (N > 8 && piece == 8) { f(std::integral_constant<int, (N > 8 ? 8 : N)>{}); return true; }
  if (N > 4 && piece == 4) { f(std::integral_constant<int, 4>{}); return true; }
  return false;
}

template <int G, int VEC, int MV, bool UNPACK, int BLK, int NT = kThreads, int DEPTH = 2, bool NTL = false>
__global__ __launch_bounds__(NT) void stream_tiled_kernel(TiledArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int N1 = BLK / MV / NT;   // 2-D side items per thread
  constexpr int N2 = BLK / VEC / NT;  // tiled side items per thread
  constexpr int NG = VEC / G;                             // granules per tiled vector
  constexpr bool kStreamingStores = BLK > (int)kStreamBlockBytes;
  using MatVec = typename GBytes<MV>::type;
  using TileVec = typename GBytes<VEC>::type;
  static_assert(G >= 4, "streaming kernels move granules of at least 4 bytes");

  // Non-temporal in the 64 KB-block kernels, and in the others when the host
  // asks for it (outputs beyond the memory-side cache).
  const bool nt_stores = kStreamingStores || a.streaming_stores;
  auto store_tiled = [&](char* p, TileVec v) {
    if constexpr (kStreamingStores) gstore<VEC, true>(p, v);
    else if (nt_stores) gstore_nt_asm<VEC>(p, v);
    else gstore<VEC, false>(p, v);
  };
  auto store_mat = [&](char* p, MatVec v) {
    if constexpr (kStreamingStores) gstore<MV, true>(p, v);
    else if (nt_stores) gstore_nt_asm<MV>(p, v);
    else gstore<MV, false>(p, v);
  };
  const uint32_t tid = threadIdx.x;
  const uint32_t total1 = a.block_rows * a.div_row_vecs.d;
  const uint32_t total2 = a.num_runs * a.run_vecs;
  const uint32_t piece = a.lds_piece < MV ? a.lds_piece : MV;
  const uint32_t size1_bytes = a.mat_size1 * a.elem_bytes;

  // ---- per-thread tables (block independent) ----------------------------
  uint32_t g1off[N1], l1off[N1];
#pragma unroll
  for (int i = 0; i < N1; ++i) {
    uint32_t r, cb;
    mat_item<MV>(a, tid + i * NT, &r, &cb);
    g1off[i] = r * a.mat_stride0_bytes32 + cb;
    l1off[i] = r * a.lds_pitch + cb;
  }
  uint32_t g2off[N2], l2off[N2][NG];
#pragma unroll
  for (int i = 0; i < N2; ++i) {
    uint32_t run, t, in_tile, tl0, tl1;
    tiled_item<VEC>(a, tid + i * NT, &run, &t, &in_tile, &tl0, &tl1);
    g2off[i] = tl0 * a.sl0_bytes32 + tl1 * a.sl1_bytes32 + in_tile;
    for_each_granule<G, VEC>(a, run, t, in_tile, [&](int k, uint32_t off) { l2off[i][k] = off; });
  }
  // Granule rotation (see gather_granules). With 4-byte granules, granule k of
  // a vector lies k LDS rows below granule 0 and the 32 lanes of a half wave
  // that walk one run sit 4 rows apart: unrotated, one LDS instruction would
  // reach only 8 of the 32 banks. Lane groups of 8 take rotations 0..3. The
  // position of a thread's vectors inside their run is the same for all of
  // its items when the run length divides the workgroup size.
  uint32_t rot = 0;
  if constexpr (NG == 4 && G == 4) {
    if ((a.run_vecs % 32 == 0 || a.run_vecs == 16) && NT % a.run_vecs == 0) {
      // Runs of 16 vectors put two runs (neighbouring LDS columns, one bank
      // apart) in a half wave: their lane groups take rotations 0 and 2.
      const uint32_t v = tid % a.run_vecs;
      rot = a.run_vecs == 16 ? ((v >> 3) & 1) * 2 : (v >> 3) & 3;
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        // table[k] = original[(k + rot) & 3]
        rotate_down4(l2off[i], rot);
      }
    }
  }

  const uint32_t nblocks = a.nblk0 * a.nblk1;
  // Every thread has all of its N1 and N2 items and the LDS piece size is one
  // of the compile-time cases: interior blocks then run without per-item
  // bounds checks and with the piece size resolved once per block.
  const bool full = total1 == (uint32_t)N1 * NT && total2 == (uint32_t)N2 * NT &&
                    (piece >= MV || piece == 8 || piece == 4);

  // Block coordinates, base pointers and whether the whole block lies inside
  // the matrix and the tile grid ("interior").
  struct Block {
    uint32_t blk0, blk1, row_base, col_base_bytes;
    const char* mat_c;
    const char* tiled_c;
    bool interior;
  };
  auto block_at = [&](uint32_t blk) {
    Block b;
    b.blk0 = blk / a.nblk1;
    b.blk1 = blk - b.blk0 * a.nblk1;
    b.row_base = b.blk0 * a.block_rows;
    b.col_base_bytes = b.blk1 * a.block_row_bytes;
    b.mat_c = (UNPACK ? a.dst : a.src) + (int64_t)b.row_base * a.mat_stride0_bytes + b.col_base_bytes;
    b.tiled_c = (UNPACK ? a.src : a.dst) + (int64_t)(b.blk0 * a.G0) * a.sl0_bytes +
                (int64_t)(b.blk1 * a.G1) * a.sl1_bytes;
    b.interior = b.row_base + a.block_rows <= a.mat_size0 &&
                 b.col_base_bytes + a.block_row_bytes <= size1_bytes &&
                 (b.blk0 + 1) * a.G0 <= a.outer0 && (b.blk1 + 1) * a.G1 <= a.outer1;
    return b;
  };

  // The global loads of an interior block are issued DEPTH (1 or 2) blocks
  // ahead, into one of DEPTH register sets (with two: the parity of the
  // block's turn), right after the set's previous contents have gone to LDS,
  // so that a workgroup keeps DEPTH blocks of loads and a block of stores in
  // flight.
  static_assert(DEPTH == 1 || DEPTH == 2, "one or two register sets");
  MatVec pre1[DEPTH][UNPACK ? 1 : N1];
  TileVec pre2[DEPTH][UNPACK ? N2 : 1];
  auto prefetch = [&](const Block& b, auto slot_c) {
    constexpr int S = decltype(slot_c)::value % DEPTH;
    if (!b.interior) {
      // Edge block: only what exists is loaded (2-D side: vectors that lie
      // wholly inside the matrix; tiled side: vectors of tiles that exist);
      // phase 1 applies the same predicate before it uses a register.
      if constexpr (!UNPACK) {
#pragma unroll
        for (int i = 0; i < N1; ++i) {
          const uint32_t idx = tid + i * NT;
          if (idx < total1) {
            uint32_t r, cb;
            mat_item<MV>(a, idx, &r, &cb);
            if (b.row_base + r < a.mat_size0 && b.col_base_bytes + cb + MV <= size1_bytes)
              pre1[S][i] = gload<MV>(b.mat_c + g1off[i]);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < N2; ++i) {
          const uint32_t idx = tid + i * NT;
          if (idx < total2) {
            uint32_t run, t, in_tile, tl0, tl1;
            tiled_item<VEC>(a, idx, &run, &t, &in_tile, &tl0, &tl1);
            if (b.blk0 * a.G0 + tl0 < a.outer0 && b.blk1 * a.G1 + tl1 < a.outer1)
              pre2[S][i] = gload<VEC>(b.tiled_c + g2off[i]);
          }
        }
      }
      return;
    }
    if (full) {
      if constexpr (!UNPACK) {
#pragma unroll
        for (int i = 0; i < N1; ++i) pre1[S][i] = gload<MV, NTL>(b.mat_c + g1off[i]);
      } else {
#pragma unroll
        for (int i = 0; i < N2; ++i) pre2[S][i] = gload<VEC, NTL>(b.tiled_c + g2off[i]);
      }
      return;
    }
    if constexpr (!UNPACK) {
#pragma unroll
      for (int i = 0; i < N1; ++i)
        if (tid + i * NT < total1) pre1[S][i] = gload<MV>(b.mat_c + g1off[i]);
    } else {
#pragma unroll
      for (int i = 0; i < N2; ++i)
        if (tid + i * NT < total2) pre2[S][i] = gload<VEC>(b.tiled_c + g2off[i]);
    }
  };

  // Workgroups are handed to the eight XCDs round-robin. Within one sweep of
  // the grid, the workgroups of one XCD take consecutive blocks (column blocks
  // of one block row first): neighbouring blocks share the cache lines that
  // their unaligned row segments straddle, and the L2 of the XCD then sees
  // both halves of such a line at about the same time.
  const uint32_t first_blk = (gridDim.x & 7) ? blockIdx.x
                                             : (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  bool have_pre[2] = {false, false};
  auto process = [&](uint32_t blk, auto slot_c) {
    constexpr int L = decltype(slot_c)::value;  // LDS buffer: parity of the turn
    constexpr int S = L % DEPTH;                // register set
    const Block b = block_at(blk);
    const uint32_t blk0 = b.blk0, blk1 = b.blk1, row_base = b.row_base,
                   col_base_bytes = b.col_base_bytes;
    const char* mat_c = b.mat_c;
    const char* tiled_c = b.tiled_c;
    const bool interior = b.interior;
    char* lbuf = lds + L * a.lds_buf_bytes;
    if (!have_pre[S]) prefetch(b, slot_c);

    if constexpr (!UNPACK) {
      // ---- pack phase 1: 2-D rows -> LDS ----
      if (interior && full) {
        with_static_piece<MV>(piece, [&](auto pc) {
          constexpr int P = decltype(pc)::value;
#pragma unroll
          for (int i = 0; i < N1; ++i) lds_store_static<MV, P>(lbuf + l1off[i], pre1[S][i]);
        });
      } else if (interior) {
#pragma unroll
        for (int i = 0; i < N1; ++i)
          if (tid + i * NT < total1) lds_store_pieces<MV>(lbuf + l1off[i], pre1[S][i], piece);
      } else {
#pragma unroll
        for (int i = 0; i < N1; ++i) {
          const uint32_t idx = tid + i * NT;
          if (idx >= total1) continue;
          uint32_t r, cb;
          mat_item<MV>(a, idx, &r, &cb);
          __attribute__((aligned(16))) char reg[MV];
          const bool row_ok = row_base + r < a.mat_size0;
          const char* gp = mat_c + (r * a.mat_stride0_bytes32 + cb);
          const uint32_t es = a.elem_bytes;
          // Whole vector inside the matrix (already loaded), or whole vector
          // padding: one access.
          if (row_ok && col_base_bytes + cb + MV <= size1_bytes) {
            lds_store_pieces<MV>(lbuf + l1off[i], pre1[S][i], piece);
            continue;
          }
          if (!row_ok || col_base_bytes + cb >= size1_bytes) {
            MatVec padv;
            uint32_t* pw = reinterpret_cast<uint32_t*>(&padv);
#pragma unroll
            for (int w = 0; w < MV / 4; ++w) pw[w] = a.pad32;
            lds_store_pieces<MV>(lbuf + r * a.lds_pitch + cb, padv, piece);
            continue;
          }
          for (uint32_t bb = 0; bb < MV; bb += es) {
            const bool ok = row_ok && (col_base_bytes + cb + bb) < size1_bytes;
            if (es == 4) {
              *reinterpret_cast<uint32_t*>(reg + bb) =
                  ok ? *reinterpret_cast<const uint32_t*>(gp + bb) : a.pad32;
            } else if (es == 2) {
              *reinterpret_cast<uint16_t*>(reg + bb) =
                  ok ? *reinterpret_cast<const uint16_t*>(gp + bb) : (uint16_t)a.pad32;
            } else {
              reg[bb] = ok ? gp[bb] : (char)a.pad32;
            }
          }
          store_pieces<MV>(lbuf + r * a.lds_pitch + cb, reg, piece);
        }
      }
    } else {
      // ---- unpack phase 1: tiled runs -> LDS (scatter by granules) ----
      if (interior && full) {
#pragma unroll
        for (int i = 0; i < N2; ++i) scatter_granules<VEC, G>(lbuf, l2off[i], pre2[S][i], rot);
      } else {
      bool ok[N2];
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        ok[i] = tid + i * NT < total2;
        if (!interior) {
          if (ok[i]) {
            uint32_t run, t, in_tile, tl0, tl1;
            tiled_item<VEC>(a, tid + i * NT, &run, &t, &in_tile, &tl0, &tl1);
            ok[i] = blk0 * a.G0 + tl0 < a.outer0 && blk1 * a.G1 + tl1 < a.outer1;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        if (ok[i]) scatter_granules<VEC, G>(lbuf, l2off[i], pre2[S][i], rot);
      }
      }
    }

    // This register set's next block, DEPTH turns on.
    have_pre[S] = false;
    if (blk + DEPTH * gridDim.x < nblocks) {
      prefetch(block_at(blk + DEPTH * gridDim.x), slot_c);
      have_pre[S] = true;
    }
    __syncthreads();

    if constexpr (!UNPACK) {
      // ---- pack phase 2: LDS -> tiled runs ----
      TileVec reg[N2];
      if (interior && full) {
#pragma unroll
        for (int i = 0; i < N2; ++i) reg[i] = gather_granules<VEC, G>(lbuf, l2off[i], rot);
#pragma unroll
        for (int i = 0; i < N2; ++i) store_tiled(const_cast<char*>(tiled_c) + g2off[i], reg[i]);
        return;
      }
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        if (tid + i * NT < total2) reg[i] = gather_granules<VEC, G>(lbuf, l2off[i], rot);
      }
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        if (tid + i * NT < total2) {
          bool ok = true;
          if (!interior) {
            uint32_t run, t, in_tile, tl0, tl1;
            tiled_item<VEC>(a, tid + i * NT, &run, &t, &in_tile, &tl0, &tl1);
            ok = blk0 * a.G0 + tl0 < a.outer0 && blk1 * a.G1 + tl1 < a.outer1;
          }
          if (ok) store_tiled(const_cast<char*>(tiled_c) + g2off[i], reg[i]);
        }
      }
    } else {
      // ---- unpack phase 2: LDS rows -> 2-D rows ----
      if (interior && full) {
        MatVec reg[N1];
        with_static_piece<MV>(piece, [&](auto pc) {
          constexpr int P = decltype(pc)::value;
#pragma unroll
          for (int i = 0; i < N1; ++i) reg[i] = lds_load_static<MV, P>(lbuf + l1off[i]);
        });
#pragma unroll
        for (int i = 0; i < N1; ++i) store_mat(const_cast<char*>(mat_c) + g1off[i], reg[i]);
      } else if (interior) {
        MatVec reg[N1];
#pragma unroll
        for (int i = 0; i < N1; ++i)
          if (tid + i * NT < total1) reg[i] = lds_load_pieces<MV>(lbuf + l1off[i], piece);
#pragma unroll
        for (int i = 0; i < N1; ++i)
          if (tid + i * NT < total1) store_mat(const_cast<char*>(mat_c) + g1off[i], reg[i]);
      } else {
        const uint32_t es = a.elem_bytes;
        for (uint32_t idx = tid; idx < total1; idx += NT) {
          uint32_t r, cb;
          mat_item<MV>(a, idx, &r, &cb);
          if (row_base + r >= a.mat_size0) continue;
          char* gp = const_cast<char*>(mat_c) + (r * a.mat_stride0_bytes32 + cb);
          if (col_base_bytes + cb + MV <= size1_bytes) {  // whole vector inside
            store_mat(gp, lds_load_pieces<MV>(lbuf + r * a.lds_pitch + cb, piece));
            continue;
          }
          __attribute__((aligned(16))) char reg[MV];
          load_pieces<MV>(reg, lbuf + r * a.lds_pitch + cb, piece);
          for (uint32_t bb = 0; bb < MV && col_base_bytes + cb + bb < size1_bytes; bb += es) {
            if (es == 4) copy_bytes<4>(gp + bb, reg + bb);
            else if (es == 2) copy_bytes<2>(gp + bb, reg + bb);
            else gp[bb] = reg[bb];
          }
        }
      }
    }
    // No second barrier: the next block uses the other LDS buffer, and its
    // barrier orders this block's LDS reads before the buffer is reused.
  };
  // Start the pipeline: the first two blocks of this workgroup.
  if (first_blk < nblocks) {
    prefetch(block_at(first_blk), std::integral_constant<int, 0>{});
    have_pre[0] = true;
    if (DEPTH == 2 && first_blk + gridDim.x < nblocks) {
      prefetch(block_at(first_blk + gridDim.x), std::integral_constant<int, 1>{});
      have_pre[1] = true;
    }
  }
  for (uint32_t blk = first_blk; blk < nblocks; blk += 2 * gridDim.x) {
    process(blk, std::integral_constant<int, 0>{});
    if (blk + gridDim.x < nblocks) process(blk + gridDim.x, std::integral_constant<int, 1>{});
  }
}

//===----------------------------------------------------------------------===//
// Host-side planning.
//===----------------------------------------------------------------------===//

struct TiledPlan {
  bool ok = false;
  TiledArgs args;
  int G = 0, VEC = 0, MV = 0;
  bool stream = false;
  bool big = false;  // 64 KB blocks (see plan_tiled)
  // 64 KB-block transposing kernels: interior blocks load non-temporally. The
  // data is read once, and more of it than the caches hold: a line that is not
  // kept leaves room for the lines that neighbouring blocks share. Right when
  // no later block needs a line again, or only the next one in the walk: pack's
  // row segments (their straddled lines are shared with the next block of the
  // same block row), unpack's runs of tiles when they are whole 128-byte lines
  // (f32 12289x12288: pack 248 -> 220 us; 12288x12289: unpack 255 -> 230 us;
  // runs that start in the middle of a line share it with a block far away in
  // the walk, and unpack lost 6 % there).
  bool streaming_loads = false;
  uint32_t grid = 0;
  uint32_t lds_bytes = 0;
};

// Chooses block shape, vector widths and LDS pitch. `mat` is the 2-D side
// (source of pack, destination of unpack), `tiled` the 4-D side.
TiledPlan plan_tiled(const TiledView& v, int es, const char* mat_ptr,
                     int64_t mat_stride0, int64_t mat_stride1, int64_t mat_size0,
                     int64_t mat_size1, const char* tiled_ptr, bool ti, bool to,
                     bool mat_is_dest, bool allow_big = true) {
  TiledPlan plan;
  if (mat_stride1 != 1) return plan;
  const int64_t tile_elems = v.tile0 * v.tile1;
  const int64_t tile_bytes = tile_elems * es;
  if (tile_bytes == 0 || tile_bytes > 16384) return plan;
  if (v.outer0 >= (1ll << 24) || v.outer1 >= (1ll << 24)) return plan;
  if (mat_size0 >= (1ll << 31) || mat_size1 * es >= (1ll << 31)) return plan;
  // Tiled-side vector width: alignment of base, outer stride and tile size.
  const int64_t tiled_align = std::min(
      {uk::pow2_divisor((int64_t)(uintptr_t)tiled_ptr, 16),
       uk::pow2_divisor(v.stride0 * es, 16), uk::pow2_divisor(tile_bytes, 16)});
  if (tiled_align < 4) return plan;
  const int VEC = tiled_align >= 16 ? 16 : 4;
  // Granule: bytes contiguous on both sides.
  int G = ti ? es : (int)uk::pow2_divisor(v.tile1 * es, 16);
  if (G > VEC) G = VEC;

  // Block shape. A run is the contiguous tiled-side span of one block.
  // Large element-granular transposes (4-byte granules: every 16-byte vector
  // of one side is four scattered words of the other) take 64 KB blocks with
  // 512-byte segments on both sides instead of 16 KB and 256: fewer, longer
  // segments mean fewer cache lines that a segment only partly covers, which
  // is what bounds them (f32 12288x12289 unpack: 3.3 -> 4.1 TB/s). Smaller
  // problems keep the small blocks: they need the parallelism.
  const int64_t total_bytes = v.outer0 * v.outer1 * tile_bytes;
  // Whole tile rows as granules (16 bytes contiguous on both sides, no
  // transposition) gain from the 64 KB blocks too, from smaller sizes on for
  // pack than for unpack (f8 28672x8192 pack: 85 -> 65 us; f16 4096x4096
  // pack: 10.6 -> 10.0 us, slower below that; f32 8192x8192 unpack: 98 -> 74
  // us, f32 4096x4096 unpack: 19.3 -> 20.0 us).
  const bool big_transposing = G == 4 && total_bytes >= (192ll << 20);
  const bool big_rows = G == 16 && !to && total_bytes >= ((mat_is_dest ? 192ll : 24ll) << 20);
  const bool big = allow_big && VEC == 16 && (big_transposing || big_rows);
  const int64_t kMinSpan = big ? 512 : 256;                      // bytes, both sides
  const int64_t kTarget = big ? kStreamBigBlockBytes : kStreamBlockBytes;  // bytes per block, about
  const int64_t stream_block = kTarget;
  int64_t G0 = 1, G1 = uk::ceil_div(kMinSpan, v.tile1 * es);
  const bool mat_rows_unaligned =
      uk::pow2_divisor(mat_stride0 * es, 16) < 16 || uk::pow2_divisor((int64_t)(uintptr_t)mat_ptr, 16) < 16;
  if (to && big && mat_is_dest) {
    // unpack writes matrix rows: 2 KB row segments (and 128-byte runs on the
    // tiled side, which is only read) leave fewer partly written cache lines
    // when the rows are not line-aligned (f32 12288x12289: 4.1 -> 4.7 TB/s;
    // no change for aligned rows).
    G0 = uk::ceil_div(128, tile_bytes);
    G1 = uk::ceil_div(2048, v.tile1 * es);
    while (G0 * G1 * tile_bytes * 2 <= kTarget) G1 *= 2;  // (larger tiles: fill the block)
  } else if (to && big && mat_rows_unaligned) {
    // pack reads matrix rows that start at odd 4-byte offsets: the side that
    // is written (the tiles) gets the long spans, 1 KB runs, and the rows are
    // read in 256-byte segments (f32 12288x12289: 248 -> 233 us; aligned rows
    // are better off with 512 bytes on both sides).
    G0 = uk::ceil_div(1024, tile_bytes);
    G1 = uk::ceil_div(256, v.tile1 * es);
    while (G0 * G1 * tile_bytes * 2 <= kTarget) G0 *= 2;  // (larger tiles: fill the block)
  } else if (to) {
    G0 = uk::ceil_div(kMinSpan, tile_bytes);
    // widen along dim 1 (more, longer 2-D row segments) up to the target
    while (G0 * G1 * tile_bytes * 2 <= kTarget) G1 *= 2;
  } else {
    // Tiles of one tile row are contiguous on the tiled side, so widening
    // along dim 1 lengthens the segments of both sides; do that up to 1 KB of
    // matrix row, then add tile rows.
    while (G0 * G1 * tile_bytes * 2 <= kTarget && G1 * v.tile1 * es < 1024 && G1 < v.outer1) G1 *= 2;
    while (G0 * G1 * tile_bytes * 2 <= kTarget) G0 *= 2;
  }
  G0 = std::min<int64_t>(G0, std::max<int64_t>(v.outer0, 1));
  G1 = std::min<int64_t>(G1, std::max<int64_t>(v.outer1, 1));
  const int64_t block_rows = G0 * v.tile0;
  const int64_t block_row_bytes = G1 * v.tile1 * es;

  // LDS pitch: rows that consecutive lanes touch in the granule phase should
  // start in different banks. Consecutive lanes sweep one tile row
  // (tile1*es bytes) and then move one LDS row down, or move one row down per
  // element when the inner transpose is on; so the pitch is made congruent to
  // that sweep width modulo the 256-byte bank span.
  int64_t sweep = ti ? es : v.tile1 * es;
  if (sweep < 4) sweep = 4;
  int64_t pitch = block_row_bytes;
  if (sweep < 256) {
    int64_t pad = ((sweep - block_row_bytes) % 256 + 256) % 256;
    pitch = block_row_bytes + pad;
  }
  pitch = uk::ceil_div(pitch, G) * G;
  const int64_t lds_bytes = block_rows * pitch;
  if (lds_bytes > (big ? 80 : 64) * 1024) {
    if (big) return plan_tiled(v, es, mat_ptr, mat_stride0, mat_stride1, mat_size0, mat_size1,
                               tiled_ptr, ti, to, mat_is_dest, false);
    return plan;
  }

  // 2-D side vector width.
  const int64_t mat_vec = std::min(
      {uk::pow2_divisor((int64_t)(uintptr_t)mat_ptr, 16),
       uk::pow2_divisor(mat_stride0 * es, 16),
       uk::pow2_divisor(block_row_bytes, 16)});
  if (mat_vec < es) return plan;

  const int64_t nblk0 = uk::ceil_div(v.outer0, G0);
  const int64_t nblk1 = uk::ceil_div(v.outer1, G1);
  if (nblk0 * nblk1 >= (1ll << 31)) return plan;

  TiledArgs& a = plan.args;
  a.mat_stride0_bytes = mat_stride0 * es;
  a.sl0_bytes = v.sl0 * es;
  a.sl1_bytes = v.sl1 * es;
  a.mat_size0 = (uint32_t)mat_size0;
  a.mat_size1 = (uint32_t)mat_size1;
  a.outer0 = (uint32_t)v.outer0;
  a.outer1 = (uint32_t)v.outer1;
  a.tile0 = (uint32_t)v.tile0;
  a.tile1 = (uint32_t)v.tile1;
  a.G0 = (uint32_t)G0;
  a.G1 = (uint32_t)G1;
  a.nblk1 = (uint32_t)nblk1;
  a.lds_pitch = (uint32_t)pitch;
  a.lds_piece = (uint32_t)uk::pow2_divisor(pitch, 16);
  a.elem_bytes = (uint32_t)es;
  a.block_rows = (uint32_t)block_rows;
  a.block_row_bytes = (uint32_t)block_row_bytes;
  a.mat_vec = (uint32_t)mat_vec;
  a.transpose_inner = ti;
  a.transpose_outer = to;
  a.tile_bytes = (uint32_t)tile_bytes;
  a.run_tiles = (uint32_t)(to ? G0 : G1);
  a.num_runs = (uint32_t)(to ? G1 : G0);
  a.run_vecs = (uint32_t)(a.run_tiles * tile_bytes / VEC);
  a.tile_row_grans = ti ? 1 : (uint32_t)(v.tile1 * es / G);
  a.div_row_vecs = FastDiv((uint32_t)(block_row_bytes / mat_vec));
  a.div_run_vecs = FastDiv(a.run_vecs);
  a.div_tile_grans = FastDiv((uint32_t)(tile_bytes / G));
  a.div_tile_row_grans = FastDiv(a.tile_row_grans);
  a.div_tile0 = FastDiv((uint32_t)v.tile0);
  a.div_tile_bytes = FastDiv((uint32_t)tile_bytes);
  a.nblk0 = (uint32_t)nblk0;
  a.lds_buf_bytes = (uint32_t)((lds_bytes + 255) / 256 * 256);
  // Streaming kernels: 32-bit offsets inside one block on both sides, granules
  // of at least 4 bytes, at most 4 granules per vector, block within budget.
  // (and non-negative strides: the 32-bit offsets are unsigned)
  plan.stream = mat_vec >= 4 && G >= 4 && VEC / G <= 4 && mat_stride0 >= 0 && v.sl0 >= 0 &&
                v.sl1 >= 0 &&
                block_rows * block_row_bytes <= stream_block &&
                lds_bytes <= (big ? 80 * 1024 : 2 * stream_block) &&
                block_rows * std::abs(mat_stride0) * es < (1ll << 31) &&
                (G0 * std::abs(v.sl0) + G1 * std::abs(v.sl1)) * es < (1ll << 31);
  plan.MV = mat_vec >= 16 ? 16 : 4;
  // The streaming kernels move 16 bytes per lane on the 2-D side from any
  // 4-byte aligned row start (LDS offsets stay 16-byte aligned: they are
  // relative to the block's window).
  if (plan.stream && block_row_bytes % 16 == 0) plan.MV = 16;
  if (big && !(plan.stream && plan.MV == 16)) {
    return plan_tiled(v, es, mat_ptr, mat_stride0, mat_stride1, mat_size0, mat_size1, tiled_ptr,
                      ti, to, mat_is_dest, false);
  }
  plan.big = big;
  if (big && G == 4) {
    // unpack: a run is (to ? G0 : G1) tiles, and runs lie (to ? sl1 : sl0) apart
    const uint64_t run_bytes = (uint64_t)((to ? G0 : G1) * tile_bytes);
    const uint64_t run_pitch = (uint64_t)((to ? v.sl1 : v.sl0) * es);
    plan.streaming_loads = !mat_is_dest || ((uintptr_t)tiled_ptr | run_bytes | run_pitch) % 128 == 0;
  }
  // Outputs beyond the memory-side cache are not worth allocating there: the
  // interior blocks of the 16 KB-block kernels store them non-temporally too
  // (f32 8192x8192 unpack under TRANSPOSE_OUTER: 106 -> 77 us). Below that
  // size the plain stores are as fast or faster.
  a.streaming_stores = total_bytes >= (192ll << 20) && uk::pow2_divisor(mat_stride0 * es, 16) >= 16;
  if (plan.stream) {
    a.mat_vec = (uint32_t)plan.MV;
    a.div_row_vecs = FastDiv((uint32_t)(block_row_bytes / plan.MV));
    a.mat_stride0_bytes32 = (uint32_t)(mat_stride0 * es);
    a.sl0_bytes32 = (uint32_t)(v.sl0 * es);
    a.sl1_bytes32 = (uint32_t)(v.sl1 * es);
  }
  plan.G = G;
  plan.VEC = VEC;
  plan.grid = (uint32_t)(nblk0 * nblk1);
  plan.lds_bytes = (uint32_t)lds_bytes;
  plan.ok = true;
  return plan;
}

template <template <int, int> class Launcher>
bool dispatch_gv(int G, int VEC, const TiledPlan& plan, hipStream_t stream) {
#define UK_CASE(g, vv)                              \
  if (G == g && VEC == vv) {                        \
    Launcher<g, vv>::launch(plan, stream);          \
    return true;                                    \
  }
  UK_CASE(16, 16) UK_CASE(8, 16) UK_CASE(4, 16) UK_CASE(2, 16) UK_CASE(1, 16)
  UK_CASE(4, 4) UK_CASE(2, 4) UK_CASE(1, 4)
#undef UK_CASE
  return false;
}

template <int G, int VEC>
struct PackLauncher {
  static void launch(const TiledPlan& plan, hipStream_t stream) {
    uk::launch(0, pack_tiled_kernel<G, VEC>, dim3(plan.grid), dim3(kThreads),
               plan.lds_bytes, stream, plan.args);
  }
};

template <int G, int VEC>
struct UnpackLauncher {
  static void launch(const TiledPlan& plan, hipStream_t stream) {
    uk::launch(1, unpack_tiled_kernel<G, VEC>, dim3(plan.grid), dim3(kThreads),
               plan.lds_bytes, stream, plan.args);
  }
};

template <bool UNPACK>
bool launch_stream(const TiledPlan& plan, hipStream_t stream) {
  // Persistent grid: up to 4 workgroups per CU, two LDS buffers each.
  const uint32_t nblocks = plan.grid;
  const uint32_t lds = 2 * plan.args.lds_buf_bytes;
  if (plan.big) {
    // One workgroup per CU: two 66 KB buffers fill its LDS.
    if (!((plan.G == 4 || plan.G == 16) && plan.VEC == 16 && plan.MV == 16)) return false;
    constexpr int kBigThreads = 1024;
    if (lds > 160 * 1024) return false;
    auto launch_big = [&](auto kernel, hipError_t attr) {
      if (attr != hipSuccess) return false;
      uk::launch(UNPACK ? 1 : 0, kernel, dim3(nblocks < 256 ? nblocks : 256), dim3(kBigThreads), lds,
                 stream, plan.args);
      return true;
    };
    if (plan.G == 4 && plan.streaming_loads) {
      auto kernel = stream_tiled_kernel<4, 16, 16, UNPACK, kStreamBigBlockBytes, kBigThreads, 1, true>;
      static hipError_t attr = hipFuncSetAttribute(
          reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      return launch_big(kernel, attr);
    }
    if (plan.G == 4) {
      auto kernel = stream_tiled_kernel<4, 16, 16, UNPACK, kStreamBigBlockBytes, kBigThreads, 1>;
      static hipError_t attr = hipFuncSetAttribute(
          reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      return launch_big(kernel, attr);
    }
    auto kernel = stream_tiled_kernel<16, 16, 16, UNPACK, kStreamBigBlockBytes, kBigThreads, 1>;
    static hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    return launch_big(kernel, attr);
  }
  const uint32_t grid = nblocks < 1024 ? nblocks : 1024;
#define UK_CASE(g, vv, mv)                                                          \
  if (plan.G == g && plan.VEC == vv && plan.MV == mv) {                              \
    uk::launch(UNPACK ? 1 : 0, stream_tiled_kernel<g, vv, mv, UNPACK, kStreamBlockBytes>, \
               dim3(grid), dim3(kThreads), lds, stream, plan.args);                  \
    return true;                                                                     \
  }
  UK_CASE(16, 16, 16) UK_CASE(8, 16, 16) UK_CASE(4, 16, 16) UK_CASE(4, 4, 16)
  UK_CASE(16, 16, 4) UK_CASE(8, 16, 4) UK_CASE(4, 16, 4) UK_CASE(4, 4, 4)
#undef UK_CASE
  return false;
}

//===----------------------------------------------------------------------===//
// Direct pack: untransposed tiles whose rows are whole 16-byte pieces, matrix
// tiled exactly (no padding). A 16-byte piece of a matrix row is a 16-byte
// piece of a tile row, so the data needs no regrouping in LDS: every thread
// moves kDirectPieces pieces from register to register. A workgroup takes 16
// matrix rows x 1 KiB: a wave reads 256 contiguous bytes of each of 4 rows and
// writes, per tile, 4 x (tile row bytes) contiguous bytes; the four waves
// together fill whole tiles when the tile height divides 16. No LDS round
// trip, no barrier: for problems of a few tens of megabytes, which are bound by
// the latency of one pass (launch, one load, one store) rather than by HBM.
//===----------------------------------------------------------------------===//
struct DirectArgs {
  const char* src;
  char* dst;
  int64_t src_pitch;     // bytes between matrix rows
  int64_t dst_stride0;   // bytes between rows of tiles
  uint32_t rows, row_bytes;
  uint32_t tile_rows, tile_row_bytes, log2_tile_row_bytes;
  uint32_t col_groups;   // 1 KiB column groups per matrix row
};
constexpr int kDirectPieces = 4;

__global__ __launch_bounds__(kThreads) void pack_direct_kernel(DirectArgs a) {
  const uint32_t rg = blockIdx.x / a.col_groups, cg = blockIdx.x - rg * a.col_groups;
  const uint32_t lane16 = threadIdx.x & 15;            // 16-byte piece within a 256-byte segment
  const uint32_t row = rg * 16 + (threadIdx.x >> 4);
  if (row >= a.rows) return;
  const uint32_t o0 = row / a.tile_rows, m0 = row - o0 * a.tile_rows;
  const char* srow = a.src + (int64_t)row * a.src_pitch;
  char* drow = a.dst + (int64_t)o0 * a.dst_stride0 + (int64_t)m0 * a.tile_row_bytes;
  const uint32_t tile_bytes = a.tile_rows * a.tile_row_bytes;
  v4u v[kDirectPieces];
  uint32_t col[kDirectPieces];
#pragma unroll
  for (int i = 0; i < kDirectPieces; ++i) {
    col[i] = cg * 1024 + (uint32_t)i * 256 + lane16 * 16;
    if (col[i] < a.row_bytes) v[i] = gload<16>(srow + col[i]);
  }
#pragma unroll
  for (int i = 0; i < kDirectPieces; ++i) {
    if (col[i] < a.row_bytes) {
      const uint32_t o1 = col[i] >> a.log2_tile_row_bytes;
      gstore<16>(drow + (int64_t)o1 * tile_bytes + (col[i] & (a.tile_row_bytes - 1)), v[i]);
    }
  }
}

// Launches the direct pack when the call is of that form (see above) and
// small enough to be latency-bound; false otherwise.
bool launch_pack_direct(const iree_uk_pack_params_t* p, int es, const char* src, char* dst,
                        bool transposed, hipStream_t stream) {
  if (transposed || p->in_stride1 != 1) return false;
  const int64_t trb = p->out_size3 * es;   // tile row bytes
  if (trb < 16 || trb > 4096 || (trb & (trb - 1))) return false;
  if (p->in_size0 != p->out_size0 * p->out_size2 || p->in_size1 != p->out_size1 * p->out_size3) return false;
  if (p->in_size0 <= 0 || p->in_size1 <= 0) return false;
  const int64_t row_bytes = p->in_size1 * es, pitch = p->in_stride0 * es;
  if (pitch < 0 || ((uintptr_t)src | (uintptr_t)dst | (uint64_t)pitch | (uint64_t)(p->out_stride0 * es)) & 15) return false;
  // Above a few tens of megabytes the streaming kernels (loads two blocks ahead,
  // larger blocks) are level or ahead (f16 4096 x 4096, 33.5 MB: 11.9 against
  // 11.6 us); below, one pass of latency is what counts (s8 2048 x 8192 in
  // 16x32 tiles, 16.8 MB: 8.4 -> 5.7 us).
  const int64_t total = p->in_size0 * row_bytes;
  if (total > (24ll << 20) || p->in_size0 >= (1ll << 31) || row_bytes >= (1ll << 31) ||
      p->out_size2 >= (1 << 20)) {
    return false;
  }
  DirectArgs a;
  a.src = src; a.dst = dst;
  a.src_pitch = pitch;
  a.dst_stride0 = p->out_stride0 * es;
  a.rows = (uint32_t)p->in_size0; a.row_bytes = (uint32_t)row_bytes;
  a.tile_rows = (uint32_t)p->out_size2; a.tile_row_bytes = (uint32_t)trb;
  a.log2_tile_row_bytes = 0;
  while ((1u << a.log2_tile_row_bytes) < a.tile_row_bytes) ++a.log2_tile_row_bytes;
  a.col_groups = (uint32_t)((row_bytes + 1023) / 1024);
  const int64_t grid = ((p->in_size0 + 15) / 16) * a.col_groups;
  if (grid >= (1ll << 31)) return false;
  uk::launch(0, pack_direct_kernel, dim3((uint32_t)grid), dim3(kThreads), 0, stream, a);
  return true;
}

uint32_t replicate_pad(uint64_t pad, int es) {
  if (es == 1) return (uint32_t)(pad & 0xFF) * 0x01010101u;
  if (es == 2) return (uint32_t)(pad & 0xFFFF) * 0x00010001u;
  return (uint32_t)pad;
}

int elem_bytes_of(uint32_t flags) {
  switch (flags & 0xFF) {
    case IREE_UK_FLAG_PACK_TYPE_F32F32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_I8I8: return 1;
    case IREE_UK_FLAG_PACK_TYPE_I32I32: return 4;
    case IREE_UK_FLAG_PACK_TYPE_F16F16: return 2;
    case IREE_UK_FLAG_PACK_TYPE_BF16BF16: return 2;
    default: return 0;
  }
}

}  // namespace

// pack_tr.hip: tiles transposed element by element (1-, 2- and 4-byte elements).
bool iree_uk_amd_launch_pack_tr(const iree_uk_pack_params_t* p, int es, const char* src, char* dst,
                                hipStream_t stream);

extern "C" int iree_uk_amd_hip_launch_pack(const iree_uk_pack_params_t* p_in,
                                           void* stream_v, int kernel_mode,
                                           const char** kernel_name) {
  hipStream_t stream = (hipStream_t)stream_v;
  // A tile that is a single row or a single column is the same bytes with and
  // without TRANSPOSE_INNER: take it as the untransposed tile of the swapped
  // shape, whose granules are whole tile rows instead of single elements (the
  // reference's f32 16x16x1 right-hand side from [K][N]: [N1][K1][16][1] under
  // both transposes is [N1][K1][1][16] under TRANSPOSE_OUTER alone).
  iree_uk_pack_params_t canonical = *p_in;
  if ((canonical.flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER) &&
      (canonical.out_size2 == 1 || canonical.out_size3 == 1)) {
    std::swap(canonical.out_size2, canonical.out_size3);
    canonical.flags &= ~(uint32_t)IREE_UK_FLAG_PACK_TRANSPOSE_INNER;
  }
  const iree_uk_pack_params_t* p = &canonical;
  const int es = elem_bytes_of(p->flags);
  if (!es) return (int)hipErrorInvalidValue;
  const bool ti = p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER;
  const bool to = p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER;
  const TiledView v = make_view(p->out_size0, p->out_size1, p->out_size2,
                                p->out_size3, p->out_stride0, ti, to);
  const char* src = (const char*)p->in_buffer + p->in_offset * es;
  char* dst = (char*)p->out_buffer + p->out_offset * es;

  // (Any forced mmt4d variant mode keeps pack on the LDS-staged kernels, so that
  // tests and timings can reach both.)
  if (kernel_mode == IREE_UK_AMD_KERNEL_MODE_AUTO &&
      launch_pack_direct(p, es, src, dst, ti || to, stream)) {
    *kernel_name = "pack_direct";
    return (int)hipGetLastError();
  }
  if (kernel_mode == IREE_UK_AMD_KERNEL_MODE_AUTO && iree_uk_amd_launch_pack_tr(p, es, src, dst, stream)) {
    *kernel_name = "pack_transposing";
    return (int)hipGetLastError();
  }
  if (kernel_mode != IREE_UK_AMD_KERNEL_MODE_GENERIC) {
    TiledPlan plan = plan_tiled(v, es, src, p->in_stride0, p->in_stride1,
                                p->in_size0, p->in_size1, dst, ti, to, false);
    if (plan.ok) {
      plan.args.src = src;
      plan.args.dst = dst;
      plan.args.pad32 = replicate_pad(p->padding_value, es);
      if (plan.stream && launch_stream<false>(plan, stream)) {
        *kernel_name = "pack_stream";
        return (int)hipGetLastError();
      }
      if (dispatch_gv<PackLauncher>(plan.G, plan.VEC, plan, stream)) {
        *kernel_name = "pack_tiled";
        return (int)hipGetLastError();
      }
    }
  }

  GenericArgs a;
  a.src = src;
  a.dst = dst;
  a.mat_stride0 = p->in_stride0;
  a.mat_stride1 = p->in_stride1;
  a.mat_size0 = p->in_size0;
  a.mat_size1 = p->in_size1;
  a.tile0 = v.tile0; a.tile1 = v.tile1;
  a.sl0 = v.sl0; a.sl1 = v.sl1; a.sl2 = v.sl2; a.sl3 = v.sl3;
  a.size1 = p->out_size1; a.size2 = p->out_size2; a.size3 = p->out_size3;
  a.stride0 = p->out_stride0;
  a.total = p->out_size0 * p->out_size1 * p->out_size2 * p->out_size3;
  a.pad = p->padding_value;
  a.transpose_inner = ti;
  a.transpose_outer = to;
  const int grid = grid_for(a.total);
  switch (es) {
    case 1: uk::launch(0, pack_generic_kernel<uint8_t>, dim3(grid), dim3(kThreads), 0, stream, a); break;
    case 2: uk::launch(0, pack_generic_kernel<uint16_t>, dim3(grid), dim3(kThreads), 0, stream, a); break;
    default: uk::launch(0, pack_generic_kernel<uint32_t>, dim3(grid), dim3(kThreads), 0, stream, a); break;
  }
  *kernel_name = "pack_generic";
  return (int)hipGetLastError();
}

extern "C" int iree_uk_amd_hip_launch_unpack(const iree_uk_unpack_params_t* p_in,
                                             void* stream_v, int kernel_mode,
                                             const char** kernel_name) {
  hipStream_t stream = (hipStream_t)stream_v;
  // (single-row and single-column tiles: see iree_uk_amd_hip_launch_pack)
  iree_uk_unpack_params_t canonical = *p_in;
  if ((canonical.flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER) &&
      (canonical.in_size2 == 1 || canonical.in_size3 == 1)) {
    std::swap(canonical.in_size2, canonical.in_size3);
    canonical.flags &= ~(uint32_t)IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER;
  }
  const iree_uk_unpack_params_t* p = &canonical;
  const int es = elem_bytes_of(p->flags);
  if (!es) return (int)hipErrorInvalidValue;
  const bool ti = p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_INNER;
  const bool to = p->flags & IREE_UK_FLAG_UNPACK_TRANSPOSE_OUTER;
  const TiledView v = make_view(p->in_size0, p->in_size1, p->in_size2,
                                p->in_size3, p->in_stride0, ti, to);
  const char* src = (const char*)p->in_buffer + p->in_offset * es;
  char* dst = (char*)p->out_buffer + p->out_offset * es;

  if (kernel_mode != IREE_UK_AMD_KERNEL_MODE_GENERIC) {
    TiledPlan plan = plan_tiled(v, es, dst, p->out_stride0, p->out_stride1,
                                p->out_size0, p->out_size1, src, ti, to, true);
    if (plan.ok) {
      plan.args.src = src;
      plan.args.dst = dst;
      plan.args.pad32 = 0;
      if (plan.stream && launch_stream<true>(plan, stream)) {
        *kernel_name = "unpack_stream";
        return (int)hipGetLastError();
      }
      if (dispatch_gv<UnpackLauncher>(plan.G, plan.VEC, plan, stream)) {
        *kernel_name = "unpack_tiled";
        return (int)hipGetLastError();
      }
    }
  }

  GenericArgs a;
  a.src = src;
  a.dst = dst;
  a.mat_stride0 = p->out_stride0;
  a.mat_stride1 = p->out_stride1;
  a.mat_size0 = p->out_size0;
  a.mat_size1 = p->out_size1;
  a.tile0 = v.tile0; a.tile1 = v.tile1;
  a.sl0 = v.sl0; a.sl1 = v.sl1; a.sl2 = v.sl2; a.sl3 = v.sl3;
  a.size1 = p->in_size1; a.size2 = p->in_size2; a.size3 = p->in_size3;
  a.stride0 = p->in_stride0;
  a.total = p->out_size0 * p->out_size1;
  a.pad = 0;
  a.transpose_inner = ti;
  a.transpose_outer = to;
  const int grid = grid_for(a.total);
  switch (es) {
    case 2: uk::launch(1, unpack_generic_kernel<uint16_t>, dim3(grid), dim3(kThreads), 0, stream, a); break;
    case 1: uk::launch(1, unpack_generic_kernel<uint8_t>, dim3(grid), dim3(kThreads), 0, stream, a); break;
    default: uk::launch(1, unpack_generic_kernel<uint32_t>, dim3(grid), dim3(kThreads), 0, stream, a); break;
  }
  *kernel_name = "unpack_generic";
  return (int)hipGetLastError();
}
