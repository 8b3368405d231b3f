// pack with an element-granular transposition inside the tile: 1- and 2-byte
// elements on the LDS transposing reads of gfx950, 4-byte elements on plain
// 32-bit LDS reads.
//
// TRANSPOSE_INNER stores a tile as [b1][b0] (b0 the position along the rows of
// the source matrix, b1 along its columns; index algebra of
// runtime/src/iree/builtins/ukernel/tools/pack_test.c:13-71): what is
// contiguous in the destination runs down a column of the source. That is the
// form a row-major [K][N] right-hand side takes on its way to [N1][K1][N0][K0]
// (tests/e2e/linalg/pack_i8.mlir:48-68). An untransposed tile whose rows hold
// one, two or four bytes is the same problem with the tile row as the element: the
// reference's x86 tiles for s8, 16x2 (arch/x86_64/mmt4d_x86_64_tiles.inl),
// are 16 two-byte elements that run down the source column.
//
// A workgroup stages a block of 32 rows x 512 bytes of the matrix in LDS, row
// major, and reads it back with ds_read_b64_tr_b16 / ds_read_b64_tr_b8. Within
// a block of 16 lanes these hand lane i, as element j of its eight bytes,
// element i % E of what lane (16 / E) j + i / E addressed (E = 4 two-byte or 8
// one-byte elements per lane): when lane l addresses row r0 + l / (16 / E),
// columns c0 + E (l % (16 / E)) ..., lane i receives column c0 + i of rows
// r0 .. r0 + E - 1, i.e. eight bytes that are contiguous in the destination.
// Two reads give a lane 16 such bytes where the tile is that tall. The walk over
// the blocks is the streaming pack kernels': persistent workgroups, the global
// loads of the next block issued before the barrier of the current one, two
// LDS buffers, one barrier per block.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "uk_device_common.h"
#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace {

// A block is 32 rows x 512 bytes of the matrix: 16 KB, 256 threads, four
// workgroups per CU. Measured on operands of 128 to 600 MB that no earlier
// launch had left in the memory-side cache: 64 x 256 is 3 to 8 % slower
// (row segments of 256 bytes), 64 x 512 with 512 threads in between, 64 x 1024
// with 1024 threads and 128 x 256 slower again. When the source is still in
// that cache all of them run alike.
constexpr int kBlockRows = 32, kBlockRowBytes = 512;

typedef uint32_t v2u __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

struct TrArgs {
  const char* src;
  char* dst;
  int64_t src_pitch;        // bytes between matrix rows
  int64_t s0, s1;           // tiled side: bytes from one row tile / column tile to the next
  uint32_t rows;            // matrix rows
  uint32_t row_bytes;       // matrix row length, bytes
  uint32_t outer0, outer1;  // tiles along rows / columns
  uint32_t lt0, lt1;        // log2 of the tile's extent along rows / columns, elements
  uint32_t nblk0, nblk1;    // blocks along rows / columns
  uint32_t strip;           // block columns per strip of the walk
  uint32_t down;            // TRANSPOSE_OUTER: tiles that follow each other down the rows are neighbours
  uint32_t lds_pitch;       // bytes per LDS row
  uint32_t lds_buf_bytes;
  uint32_t pad32;           // the padding element replicated over 32 bits
};

template <int EB>
__device__ __forceinline__ v2u read_tr(uint32_t lds_addr) {
  v2u v;
  if constexpr (EB == 2) {
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=&v"(v) : "v"(lds_addr) : "memory");
  } else {
    asm volatile("ds_read_b64_tr_b8 %0, %1" : "=&v"(v) : "v"(lds_addr) : "memory");
  }
  return v;
}

// EB: bytes per transposed element (4: no transposing read exists; a lane
// reads its column's word from four consecutive rows). V: bytes a lane stores
// at once (16 where the tile's extent along the rows is a multiple of 16 bytes,
// else 8). IL: 0,
// or the tile's extent along the rows where that is less than eight bytes (2
// or 4 elements: the K0 = 2 tiles of the reference's x86 kernels from a
// row-major [K][N] operand). A lane's 16 destination bytes are then 16 / IL
// bytes of each of IL neighbouring rows, read as they lie and interleaved in
// registers (v_perm_b32); neighbouring lanes take neighbouring columns, which
// are neighbours in the tile.
template <int EB, int V, int IL = 0>
__global__ __launch_bounds__(kBlockRows * kBlockRowBytes / 64) void pack_tr_kernel(TrArgs a) {
  static_assert(IL == 0 || (V == 16 && (IL * EB == 2 || IL * EB == 4)), "interleaved rows of 2 or 4 bytes");
  static_assert(EB != 4 || (V == 16 && IL == 0), "4-byte elements: four rows per 16-byte vector");
  constexpr int kThreads = kBlockRows * kBlockRowBytes / 64;  // 64 bytes of the block per thread
  constexpr int kBlockBytes = kBlockRows * kBlockRowBytes;
  constexpr int VPR = kBlockRowBytes / 16;     // 16-byte vectors per block row
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int E = EB == 4 ? 4 : 8 / EB;      // elements per lane and read (4-byte elements: per vector)
  constexpr int CH = EB == 4 ? 16 : 16 / E;    // 8-byte column chunks per 16 columns (4-byte elements: lanes)
  constexpr int BC = kBlockRowBytes / EB;      // block columns, elements
  constexpr int NCG = BC / 16;                 // groups of 16 columns
  constexpr int RPI = V / EB;                  // rows per item
  constexpr int N1 = kBlockBytes / 16 / kThreads;  // 16-byte source vectors per thread
  constexpr int N2 = kBlockBytes / V / kThreads;   // destination vectors per thread
  constexpr int R = V / 8;                     // reads per destination vector
  typedef v4u v4u_a4 __attribute__((aligned(4)));

  const uint32_t tid = threadIdx.x;
  // Row groups of one tile (its extent along the rows over what an item takes).
  const uint32_t lht = IL ? 0 : a.lt0 - (RPI == 16 ? 4 : RPI == 8 ? 3 : 2);  // log2

  // ---- per-thread tables (the same for every block) ----
  uint32_t g1off[N1], l1off[N1];
#pragma unroll
  for (int i = 0; i < N1; ++i) {
    const uint32_t idx = tid + i * kThreads;
    const uint32_t r = idx / VPR, v = idx % VPR;
    g1off[i] = r * (uint32_t)a.src_pitch + v * 16;
    l1off[i] = r * a.lds_pitch + v * 16;
  }
  uint32_t l2addr[N2], g2off[N2], tl0[N2], tl1[N2];
#pragma unroll
  for (int i = 0; i < N2; ++i) {
    const uint32_t idx = tid + i * kThreads;
    if constexpr (IL != 0) {
      // Vector idx of the block: 16 / (IL * EB) columns of one tile row
      // extent, columns first.
      constexpr uint32_t CPV = 16 / (IL * EB), VPT = BC / CPV;
      uint32_t rt = idx / VPT, c = (idx % VPT) * CPV;
      if (a.down) {
        // the vectors of a tile, then the tiles down the rows, then the next column of tiles
        const uint32_t vpt = (1u << a.lt1) / CPV, v = idx % vpt, t = idx / vpt;
        rt = t % (kBlockRows / IL);
        c = (t / (kBlockRows / IL) * vpt + v) * CPV;
      }
      l2addr[i] = rt * IL * a.lds_pitch + c * EB;
      tl0[i] = rt;
      tl1[i] = c >> a.lt1;
      g2off[i] = tl0[i] * (uint32_t)a.s0 + tl1[i] * (uint32_t)a.s1 + (c & ((1u << a.lt1) - 1)) * IL * EB;
      continue;
    }
    const uint32_t l = idx & 15, item = idx >> 4;
    // Items in the order (row group within the tile, column group, tile along
    // the rows): the four items of a wave's instruction then store bytes that
    // are neighbours in the destination wherever the tile shape allows.
    const uint32_t h = item & ((1u << lht) - 1);
    uint32_t cg = (item >> lht) & (NCG - 1);
    uint32_t rgt = (item >> lht) / NCG;
    if (a.down) {
      // (row group within the tile, tile down the rows, column group)
      const uint32_t tr = kBlockRows >> a.lt0;
      rgt = (item >> lht) % tr;
      cg = (item >> lht) / tr;
    }
    const uint32_t r0 = ((rgt << lht) + h) * RPI;
    // What this lane addresses for the item's reads.
    if constexpr (EB == 4) l2addr[i] = r0 * a.lds_pitch + (cg * 16 + l) * EB;  // its own column, four rows down
    else l2addr[i] = (r0 + l / CH) * a.lds_pitch + (cg * 16 + (l % CH) * E) * EB;
    // What it receives: column cg * 16 + l of rows r0 .. r0 + RPI - 1.
    const uint32_t c = cg * 16 + l;
    tl0[i] = r0 >> a.lt0;
    tl1[i] = c >> a.lt1;
    const uint32_t b0 = r0 & ((1u << a.lt0) - 1), b1 = c & ((1u << a.lt1) - 1);
    g2off[i] = tl0[i] * (uint32_t)a.s0 + tl1[i] * (uint32_t)a.s1 + ((b1 << a.lt0) + b0) * EB;
  }
  const uint32_t tiles0 = kBlockRows >> a.lt0, tiles1 = BC >> a.lt1;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;  // LDS addresses are the low 32 bits

  struct Block {
    uint32_t blk0, blk1, row_base, col_base_bytes;
    const char* src;
    char* dst;
    bool interior;
  };
  auto block_at = [&](uint32_t blk) {
    Block b;
    // Strips of `strip` block columns, each walked block row by block row.
    const uint32_t per_strip = a.strip * a.nblk0;
    const uint32_t st = blk / per_strip, rem = blk - st * per_strip;
    const uint32_t width = min(a.strip, a.nblk1 - st * a.strip);
    b.blk0 = rem / width;
    b.blk1 = st * a.strip + (rem - b.blk0 * width);
    b.row_base = b.blk0 * kBlockRows;
    b.col_base_bytes = b.blk1 * kBlockRowBytes;
    b.src = a.src + (int64_t)b.row_base * a.src_pitch + b.col_base_bytes;
    b.dst = a.dst + (int64_t)(b.blk0 * tiles0) * a.s0 + (int64_t)(b.blk1 * tiles1) * a.s1;
    b.interior = b.row_base + kBlockRows <= a.rows && b.col_base_bytes + kBlockRowBytes <= a.row_bytes &&
                 (b.blk0 + 1) * tiles0 <= a.outer0 && (b.blk1 + 1) * tiles1 <= a.outer1;
    return b;
  };
  v4u pre[N1];
  auto prefetch = [&](const Block& b) {
    if (b.interior) {
#pragma unroll
      for (int i = 0; i < N1; ++i) pre[i] = *reinterpret_cast<const v4u_a4*>(b.src + g1off[i]);
      return;
    }
    // Edge block: vectors that lie wholly inside the matrix; the rest is dealt
    // with when the block goes to LDS.
#pragma unroll
    for (int i = 0; i < N1; ++i) {
      const uint32_t idx = tid + i * kThreads;
      const uint32_t r = idx / VPR, cb = (idx % VPR) * 16;
      if (b.row_base + r < a.rows && b.col_base_bytes + cb + 16 <= a.row_bytes)
        pre[i] = *reinterpret_cast<const v4u_a4*>(b.src + g1off[i]);
    }
  };

  const uint32_t nblocks = a.nblk0 * a.nblk1;
  // Workgroups go to the eight XCDs round-robin; the workgroups of one XCD
  // take consecutive blocks.
  const uint32_t first_blk = (gridDim.x & 7) ? blockIdx.x
                                             : (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (first_blk < nblocks) prefetch(block_at(first_blk));
  uint32_t buf = 0;
  for (uint32_t blk = first_blk; blk < nblocks; blk += gridDim.x, buf ^= 1) {
    const Block b = block_at(blk);
    char* lbuf = lds + buf * a.lds_buf_bytes;
    // ---- matrix rows -> LDS ----
    if (b.interior) {
#pragma unroll
      for (int i = 0; i < N1; ++i) *reinterpret_cast<v4u*>(lbuf + l1off[i]) = pre[i];
    } else {
#pragma unroll
      for (int i = 0; i < N1; ++i) {
        const uint32_t idx = tid + i * kThreads;
        const uint32_t r = idx / VPR, cb = (idx % VPR) * 16;
        const bool row_ok = b.row_base + r < a.rows;
        v4u val;
        if (row_ok && b.col_base_bytes + cb + 16 <= a.row_bytes) {
          val = pre[i];
        } else {
          val = v4u{a.pad32, a.pad32, a.pad32, a.pad32};
          if (row_ok && b.col_base_bytes + cb < a.row_bytes) {
            // The row ends inside this vector: element by element.
            __attribute__((aligned(16))) char reg[16];
            *reinterpret_cast<v4u*>(reg) = val;
            const char* gp = b.src + g1off[i];
            const uint32_t left = a.row_bytes - (b.col_base_bytes + cb);
            for (uint32_t bb = 0; bb + EB <= left && bb < 16; bb += EB) {
              if constexpr (EB == 4) *reinterpret_cast<uint32_t*>(reg + bb) = *reinterpret_cast<const uint32_t*>(gp + bb);
              else if constexpr (EB == 2) *reinterpret_cast<uint16_t*>(reg + bb) = *reinterpret_cast<const uint16_t*>(gp + bb);
              else reg[bb] = gp[bb];
            }
            val = *reinterpret_cast<const v4u*>(reg);
          }
        }
        *reinterpret_cast<v4u*>(lbuf + l1off[i]) = val;
      }
    }
    if (blk + gridDim.x < nblocks) prefetch(block_at(blk + gridDim.x));
    __syncthreads();

    if constexpr (IL != 0) {
      // ---- LDS rows, interleaved -> tiles ----
      v4u out[N2];
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        const char* lp = lbuf + l2addr[i];
        if constexpr (IL == 2) {
          const v2u r0 = *reinterpret_cast<const v2u*>(lp);
          const v2u r1 = *reinterpret_cast<const v2u*>(lp + a.lds_pitch);
          constexpr uint32_t kLo = EB == 2 ? 0x05040100u : 0x05010400u;  // elements 0 (and 1) of both rows
          constexpr uint32_t kHi = EB == 2 ? 0x07060302u : 0x07030602u;
          out[i] = v4u{__builtin_amdgcn_perm(r1[0], r0[0], kLo), __builtin_amdgcn_perm(r1[0], r0[0], kHi),
                       __builtin_amdgcn_perm(r1[1], r0[1], kLo), __builtin_amdgcn_perm(r1[1], r0[1], kHi)};
        } else {
          uint32_t r[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) r[j] = *reinterpret_cast<const uint32_t*>(lp + j * a.lds_pitch);
          // bytes (c, row): pairs of rows first, then pairs of pairs
          const uint32_t a01 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);  // c0r0 c0r1 c1r0 c1r1
          const uint32_t b01 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);  // c2r0 c2r1 c3r0 c3r1
          const uint32_t a23 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
          const uint32_t b23 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
          out[i] = v4u{__builtin_amdgcn_perm(a23, a01, 0x05040100u), __builtin_amdgcn_perm(a23, a01, 0x07060302u),
                       __builtin_amdgcn_perm(b23, b01, 0x05040100u), __builtin_amdgcn_perm(b23, b01, 0x07060302u)};
        }
      }
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        if (!b.interior && !(b.blk0 * tiles0 + tl0[i] < a.outer0 && b.blk1 * tiles1 + tl1[i] < a.outer1)) continue;
        __builtin_nontemporal_store(out[i], reinterpret_cast<v4u*>(b.dst + g2off[i]));
      }
      continue;
    }
    if constexpr (EB == 4) {
      // ---- LDS columns, word by word -> tiles ----
      v4u out[N2];
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        const char* lp = lbuf + l2addr[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) out[i][j] = *reinterpret_cast<const uint32_t*>(lp + j * a.lds_pitch);
      }
#pragma unroll
      for (int i = 0; i < N2; ++i) {
        if (!b.interior && !(b.blk0 * tiles0 + tl0[i] < a.outer0 && b.blk1 * tiles1 + tl1[i] < a.outer1)) continue;
        __builtin_nontemporal_store(out[i], reinterpret_cast<v4u*>(b.dst + g2off[i]));
      }
      continue;
    }
    // ---- LDS, transposed -> tiles ----
    const uint32_t lb = lds_base + buf * a.lds_buf_bytes;
    v2u got[N2][R];
#pragma unroll
    for (int i = 0; i < N2; ++i)
#pragma unroll
      for (int h = 0; h < R; ++h) got[i][h] = read_tr<EB == 4 ? 2 : EB>(lb + l2addr[i] + (uint32_t)h * E * a.lds_pitch);
    // The compiler does not count these reads: wait for them here, and tie the
    // registers to the wait so that nothing uses them before it.
#define UK_GOT(k) "+v"(got[(k) % N2][(k) / N2 % R])
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : UK_GOT(0), UK_GOT(1), UK_GOT(2), UK_GOT(3), UK_GOT(4), UK_GOT(5), UK_GOT(6), UK_GOT(7)
                 :
                 : "memory");
#undef UK_GOT
    static_assert(N2 * R == 8, "eight reads per thread and block");
#pragma unroll
    for (int i = 0; i < N2; ++i) {
      if (!b.interior && !(b.blk0 * tiles0 + tl0[i] < a.outer0 && b.blk1 * tiles1 + tl1[i] < a.outer1)) continue;
      char* gp = b.dst + g2off[i];
      // Non-temporal stores: the tiles are written once, in whole lines over a
      // few instructions, and not read again by this kernel (f16 4096 x 4096:
      // 11.4 -> 9.4 us; s8 8192 x 28672: 97 -> 67 us).
      if constexpr (V == 16) {
        const v4u val = v4u{got[i][0][0], got[i][0][1], got[i][1][0], got[i][1][1]};
        __builtin_nontemporal_store(val, reinterpret_cast<v4u*>(gp));
      } else {
        __builtin_nontemporal_store(got[i][0], reinterpret_cast<v2u*>(gp));
      }
    }
    // No second barrier: the next block uses the other buffer, and its barrier
    // orders this block's reads before that buffer is written again.
  }
}

uint32_t log2_exact(int64_t x) {
  uint32_t l = 0;
  while ((1ll << l) < x) ++l;
  return l;
}
bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }


}  // namespace

// Launches the transposing pack when it serves the call (true), else launches
// nothing. `es`: bytes per element of the pack's type; src / dst with their
// offsets applied.
bool iree_uk_amd_launch_pack_tr(const iree_uk_pack_params_t* p, int es, const char* src, char* dst,
                                hipStream_t stream) {
  const bool ti = p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_INNER;
  const bool to = p->flags & IREE_UK_FLAG_PACK_TRANSPOSE_OUTER;
  if (p->in_stride1 != 1 || p->in_stride0 < 0) return false;
  // Element of the transposition and the tile's extents in such elements:
  // t0 along the matrix rows, t1 along its columns.
  int eb;
  int64_t t0, t1, size1;
  if (ti) {
    if (es > 4) return false;
    eb = es; t0 = p->out_size3; t1 = p->out_size2; size1 = p->in_size1;
  } else {
    // Tile rows of one, two or four bytes: the row is the element.
    if (p->out_size3 * es > 4) return false;
    eb = (int)(p->out_size3 * es);
    if (eb != 1 && eb != 2 && eb != 4) return false;
    if (p->in_size1 % p->out_size3 != 0) return false;  // (a last row of half padding)
    t0 = p->out_size2; t1 = 1; size1 = p->in_size1 / p->out_size3;
  }
  const int64_t tile_bytes = t0 * t1 * eb;
  const int64_t outer0 = to ? p->out_size1 : p->out_size0;  // tiles along the matrix rows
  const int64_t outer1 = to ? p->out_size0 : p->out_size1;
  // Four-byte elements are also what the streaming kernel's 4-byte granules
  // serve. Up to some hundreds of megabytes this kernel is the faster one
  // (f32 16x1 tiles of 2048 x 2048: 5.2 against 11.2 us; 4096 x 4096: 21
  // against 25; 6144 x 6144: 49 against 67), beyond that the other one, with
  // its 64 KB blocks (12288 x 12288: 241 against 194 us, 288 against 225 under
  // TRANSPOSE_OUTER).
  if (eb == 4 && p->in_size0 * size1 * eb + outer0 * outer1 * tile_bytes > (448ll << 20)) return false;
  const int64_t bc = kBlockRowBytes / eb;
  if (!is_pow2(t0) || !is_pow2(t1) || t0 > kBlockRows || t1 > bc) return false;
  // Tiles less than eight bytes tall: rows interleaved in registers, a vector
  // of 16 / (t0 * eb) columns inside one tile.
  const int il = (t0 * eb == 2 || t0 * eb == 4) && t0 > 1 ? (int)t0 : 0;
  if (il ? t1 * t0 * eb < 16 : (t0 * eb) % (eb == 4 ? 16 : 8) != 0) return false;
  const int V = il || (t0 * eb) % 16 == 0 ? 16 : 8;
  const int64_t s_outer = p->out_stride0 * es;
  const int64_t s0 = to ? tile_bytes : s_outer;
  const int64_t s1 = to ? s_outer : tile_bytes;
  const int64_t pitch = p->in_stride0 * es;
  if (s_outer < 0) return false;
  // Alignment: 4 bytes on the matrix side, the store width on the tiled side.
  if (((uintptr_t)src | (uint64_t)pitch) & 3) return false;
  if (((uintptr_t)dst | (uint64_t)s0 | (uint64_t)s1) & (uint64_t)(V - 1)) return false;
  const int64_t tiles0 = kBlockRows / t0, tiles1 = bc / t1;
  // 32-bit offsets inside a block, 32-bit sizes.
  if (pitch * kBlockRows >= (1ll << 31) || tiles0 * s0 + tiles1 * s1 >= (1ll << 31)) return false;
  if (p->in_size0 >= (1ll << 31) || size1 * eb >= (1ll << 31) || outer0 >= (1ll << 24) || outer1 >= (1ll << 24)) return false;
  const int64_t nblk0 = uk::ceil_div(outer0, tiles0), nblk1 = uk::ceil_div(outer1, tiles1);
  if (nblk0 * nblk1 >= (1ll << 31) || nblk0 * nblk1 == 0) return false;

  TrArgs a{};
  a.src = src;
  a.dst = dst;
  a.src_pitch = pitch;
  a.s0 = s0;
  a.s1 = s1;
  a.rows = (uint32_t)p->in_size0;
  a.row_bytes = (uint32_t)(size1 * eb);
  a.outer0 = (uint32_t)outer0;
  a.outer1 = (uint32_t)outer1;
  a.lt0 = log2_exact(t0);
  a.lt1 = log2_exact(t1);
  a.nblk0 = (uint32_t)nblk0;
  a.nblk1 = (uint32_t)nblk1;
  // Under TRANSPOSE_OUTER the tiles of one block column follow each other in
  // the destination: the walk goes down the block columns.
  a.strip = to ? 1u : (uint32_t)nblk1;
  a.down = to ? 1u : 0u;
  // Rows that the lanes of one read touch lie 16 (one-byte elements: 16 rows
  // of 16 bytes per half wave) or 32 bytes apart modulo the 256 bytes of the banks.
  // Four-byte elements: the four items of one read are row groups four rows
  // apart over the same 64 bytes of columns; 4 x 272 = 64 modulo 256.
  a.lds_pitch = kBlockRowBytes + (eb == 4 ? 16 : 16 * eb);
  a.lds_buf_bytes = kBlockRows * a.lds_pitch;
  uint64_t pad = p->padding_value & (es == 1 ? 0xFFull : es == 2 ? 0xFFFFull : 0xFFFFFFFFull);
  a.pad32 = es == 1 ? (uint32_t)(pad * 0x01010101ull) : es == 2 ? (uint32_t)(pad * 0x00010001ull) : (uint32_t)pad;
  const uint32_t nblocks = (uint32_t)(nblk0 * nblk1);
  const size_t lds = 2 * (size_t)a.lds_buf_bytes;
  const uint32_t grid = nblocks < 1024 ? nblocks : 1024;
  const dim3 block(kBlockRows * kBlockRowBytes / 64);
  if (il) {
    if (eb == 2) uk::launch(0, pack_tr_kernel<2, 16, 2>, dim3(grid), block, lds, stream, a);
    else if (il == 2) uk::launch(0, pack_tr_kernel<1, 16, 2>, dim3(grid), block, lds, stream, a);
    else uk::launch(0, pack_tr_kernel<1, 16, 4>, dim3(grid), block, lds, stream, a);
    return true;
  }
  if (eb == 4) uk::launch(0, pack_tr_kernel<4, 16>, dim3(grid), block, lds, stream, a);
  else if (eb == 2 && V == 16) uk::launch(0, pack_tr_kernel<2, 16>, dim3(grid), block, lds, stream, a);
  else if (eb == 2) uk::launch(0, pack_tr_kernel<2, 8>, dim3(grid), block, lds, stream, a);
  else if (V == 16) uk::launch(0, pack_tr_kernel<1, 16>, dim3(grid), block, lds, stream, a);
  else uk::launch(0, pack_tr_kernel<1, 8>, dim3(grid), block, lds, stream, a);
  return true;
}
