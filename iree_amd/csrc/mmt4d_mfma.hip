// mmt4d on the gfx950 matrix cores: shape checks and per-type dispatch. The
// kernel template lives in mmt4d_mfma_kernel.h, variant selection in
// mmt4d_mfma_launch.h; each element type and class of row widths is compiled on
// its own (mmt4d_mfma_inst.hip).
#include <hip/hip_runtime.h>

#include "mmt4d_mfma_launch.h"

namespace uk_mfma {
// One function per element type and class of tile row widths (2, 4, 8, and 16
// bytes and more), each defined by its own compilation of mmt4d_mfma_inst.hip.
#define UK_DECLARE_ROW_CLASSES(T)                                                         \
  int launch_##T##_rb2(const Problem& p, int forced, hipStream_t stream, const char** name); \
  int launch_##T##_rb4(const Problem& p, int forced, hipStream_t stream, const char** name); \
  int launch_##T##_rb8(const Problem& p, int forced, hipStream_t stream, const char** name); \
  int launch_##T##_rb16(const Problem& p, int forced, hipStream_t stream, const char** name);
UK_DECLARE_ROW_CLASSES(s8)
UK_DECLARE_ROW_CLASSES(f16)
UK_DECLARE_ROW_CLASSES(bf16)
UK_DECLARE_ROW_CLASSES(f16f16)
UK_DECLARE_ROW_CLASSES(bf16bf16)
int launch_f32_rb4(const Problem& p, int forced, hipStream_t stream, const char** name);
int launch_f32_rb8(const Problem& p, int forced, hipStream_t stream, const char** name);
int launch_f32_rb16(const Problem& p, int forced, hipStream_t stream, const char** name);
int launch_f8_rb16(const Problem& p, int forced, hipStream_t stream, const char** name);
#undef UK_DECLARE_ROW_CLASSES
#define UK_DEFINE_BY_ROW_BYTES(T)                                                            \
  inline int launch_##T(const Problem& p, int forced, hipStream_t stream, const char** name) { \
    switch (p.rb) {                                                                          \
      case 2: return launch_##T##_rb2(p, forced, stream, name);                              \
      case 4: return launch_##T##_rb4(p, forced, stream, name);                              \
      case 8: return launch_##T##_rb8(p, forced, stream, name);                              \
      default: return launch_##T##_rb16(p, forced, stream, name);                            \
    }                                                                                        \
  }
UK_DEFINE_BY_ROW_BYTES(s8)
UK_DEFINE_BY_ROW_BYTES(f16)
UK_DEFINE_BY_ROW_BYTES(bf16)
UK_DEFINE_BY_ROW_BYTES(f16f16)
UK_DEFINE_BY_ROW_BYTES(bf16bf16)
#undef UK_DEFINE_BY_ROW_BYTES
inline int launch_f32(const Problem& p, int forced, hipStream_t stream, const char** name) {
  switch (p.rb) {
    case 2: return -1;
    case 4: return launch_f32_rb4(p, forced, stream, name);
    case 8: return launch_f32_rb8(p, forced, stream, name);
    default: return launch_f32_rb16(p, forced, stream, name);
  }
}
inline int launch_f8(const Problem& p, int forced, hipStream_t stream, const char** name) {
  return p.rb >= 16 ? launch_f8_rb16(p, forced, stream, name) : -1;
}
int launch_s8s4(const Problem& p, hipStream_t stream, const char** name);
int launch_s16(const Problem& p, int forced, hipStream_t stream, const char** name);
}  // namespace uk_mfma

#include <mutex>
#include <vector>

// ---- workspace of the K split over workgroups (mmt4d_mfma_thin.h) -----------
//
// Ordinary calls: a buffer the library allocates, per host thread and stream
// (two streams of one thread may run their kernels side by side), grown when a
// call needs more. Calls through iree_uk_amd_mmt4d_no_alloc: the static device
// array below, one copy per GPU, shared by every such call on that GPU.
namespace {

constexpr size_t kScratchPartialBytes = 8u << 20;   // partial accumulator blocks
constexpr uint32_t kScratchCounters = 16384;        // one arrival counter per output block
constexpr size_t kScratchBytes = kScratchPartialBytes + kScratchCounters * sizeof(uint32_t);

// Zero when the code object is loaded; the kernels leave the counters at zero
// (the workgroup that arrives last at a block resets that block's counter), and
// partial blocks are written before they are read, so nothing needs clearing
// between calls. Calls that overlap on one GPU would race on it.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, looked up once

// The array's name is a host-side stand-in, not a device address: ask the
// runtime for the address on the current device, once per device.
int scratch_address(void** ptr) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (!p) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

struct OwnedWorkspace {
  int device;
  hipStream_t stream;
  char* base;
  size_t partial_bytes;
  uint32_t n_counters;
  uint64_t last_use;   // value of the thread's use counter when last handed out
};
// Freed when the thread ends; hipFree waits for the device, so no kernel in
// flight can still use a workspace then.
struct OwnedWorkspaces : std::vector<OwnedWorkspace> {
  uint64_t uses = 0;
  ~OwnedWorkspaces() {
    for (OwnedWorkspace& w : *this) {
      if (w.base) (void)hipFree(w.base);
    }
  }
};
// Workspaces a thread keeps at most: beyond that the one used longest ago is
// freed (a thread that runs through many short-lived streams would otherwise
// hold a megabyte and more per stream handle it ever saw).
constexpr size_t kMaxOwnedWorkspaces = 8;
thread_local OwnedWorkspaces g_workspaces;
thread_local OwnedWorkspaces g_expand_workspaces;   // s4 weights expanded to s8 (n_counters unused)
thread_local bool g_no_alloc = false;
thread_local int g_k_slices = 0;
thread_local int g_last_k_slices = 1;
thread_local int g_persistent_workgroups = 0;
thread_local bool g_streamed_weights = false;

}  // namespace

namespace uk_mfma {

int persistent_workgroups_override() { return g_persistent_workgroups; }
int k_slices_override() { return g_k_slices; }
int streamed_weights() { return g_streamed_weights ? 1 : 0; }
void note_k_slices(int n) { g_last_k_slices = n; }

int acquire_ksplit_workspace(size_t partial_bytes, uint32_t n_counters, hipStream_t stream,
                             KSplitWorkspace* ws) {
  if (g_no_alloc) {
    // A split that does not fit the static array: the call runs without the
    // split, which needs no scratch memory at all.
    if (partial_bytes > kScratchPartialBytes || n_counters > kScratchCounters) return 1;
    void* base = nullptr;
    const int st = scratch_address(&base);
    if (st != 0) return st;
    ws->partials = (char*)base;
    ws->counters = (uint32_t*)((char*)base + kScratchPartialBytes);
    return 0;
  }
  // A stream that is being captured into a graph gets no library-owned
  // workspace at all: the graph would keep the pointer beyond the life of the
  // thread that owns the block, and its replays would share the block with
  // this thread's eager calls. Such a call runs without the split (callers that
  // want the split inside a graph use iree_uk_amd_mmt4d_no_alloc and its
  // serialization rule).
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) { (void)hipGetLastError(); return 1; }
  if (capture != hipStreamCaptureStatusNone) return 1;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 1;
  const uint64_t now = ++g_workspaces.uses;
  for (OwnedWorkspace& w : g_workspaces) {
    if (w.device == dev && w.stream == stream && w.partial_bytes >= partial_bytes &&
        w.n_counters >= n_counters) {
      w.last_use = now;
      ws->partials = w.base;
      ws->counters = (uint32_t*)(w.base + w.partial_bytes);
      return 0;
    }
  }
  // Nothing fits: allocate (sizes rounded up so that similar calls share it).
  // First make room: a smaller workspace of the same stream is replaced, and
  // beyond kMaxOwnedWorkspaces the one used longest ago goes. hipFree waits for
  // the device, so no kernel in flight can still be using what is freed.
  for (size_t i = 0; i < g_workspaces.size();) {
    OwnedWorkspace& w = g_workspaces[i];
    if (w.device == dev && w.stream == stream) {
      (void)hipFree(w.base);
      g_workspaces.erase(g_workspaces.begin() + (ptrdiff_t)i);
    } else {
      ++i;
    }
  }
  while (g_workspaces.size() >= kMaxOwnedWorkspaces) {
    size_t oldest = 0;
    for (size_t i = 1; i < g_workspaces.size(); ++i) {
      if (g_workspaces[i].last_use < g_workspaces[oldest].last_use) oldest = i;
    }
    (void)hipFree(g_workspaces[oldest].base);
    g_workspaces.erase(g_workspaces.begin() + (ptrdiff_t)oldest);
  }
  size_t want_partials = 1u << 20;
  while (want_partials < partial_bytes) want_partials <<= 1;
  uint32_t want_counters = 4096;
  while (want_counters < n_counters) want_counters <<= 1;
  char* base = nullptr;
  const size_t bytes = want_partials + (size_t)want_counters * sizeof(uint32_t);
  if (hipMalloc((void**)&base, bytes) != hipSuccess) { (void)hipGetLastError(); return 1; }
  iree_uk_amd_hip_note_device_alloc();
  // The counters start at zero; the kernels keep them there. The fill is
  // ordered before the launch that follows on the same stream.
  if (hipMemsetAsync(base + want_partials, 0, (size_t)want_counters * sizeof(uint32_t), stream) !=
      hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(base);
    return 1;
  }
  g_workspaces.push_back(OwnedWorkspace{dev, stream, base, want_partials, want_counters, now});
  ws->partials = base;
  ws->counters = (uint32_t*)(base + want_partials);
  return 0;
}

namespace {
typedef uint32_t v4u_rt __attribute__((ext_vector_type(4)));

// An unsigned integer of BYTES bytes, and the same read from any address.
template <int BYTES> struct PieceOf;
template <> struct PieceOf<1> { typedef uint8_t type; typedef uint8_t loaded; };
template <> struct PieceOf<2> { typedef uint16_t type; typedef uint16_t loaded __attribute__((aligned(1))); };
template <> struct PieceOf<4> { typedef uint32_t type; typedef uint32_t loaded __attribute__((aligned(1))); };
template <> struct PieceOf<8> { typedef uint64_t type; typedef uint64_t loaded __attribute__((aligned(1))); };

// Signed nibbles of the low BYTES bytes of v, low nibble first, as 2 * BYTES bytes.
template <int BYTES>
__device__ __forceinline__ uint64_t widen_nibbles(uint32_t v) {
  uint64_t out = 0;
#pragma unroll
  for (int i = 0; i < 2 * BYTES; ++i) {
    out |= (uint64_t)((uint32_t)__builtin_amdgcn_sbfe((int)v, 4 * i, 4) & 0xFFu) << (8 * i);
  }
  return out;
}

// One thread per 16-byte destination row: 16 / RB source tile rows of RB bytes
// (SRC_BITS = 4: of RB / 2 bytes holding RB nibbles), one load each.
template <int SRC_BITS, int RB>
__global__ __launch_bounds__(256) void retile_rows_kernel(const char* src, int64_t src_stride, char* dst,
                                                           int64_t dst_stride, uint32_t R0, uint32_t K1,
                                                           uint32_t K1p) {
  constexpr uint32_t G = 16 / RB;         // source tiles per destination tile
  constexpr int SB = RB * SRC_BITS / 8;   // bytes of a source tile row
  typedef typename PieceOf<RB>::type out_piece_t;
  typedef typename PieceOf<SB>::loaded src_piece_t;
  const char* s = src + (int64_t)blockIdx.y * src_stride;
  char* d = dst + (int64_t)blockIdx.y * dst_stride;
  const uint32_t pieces = K1p * R0;
  for (uint32_t idx = blockIdx.x * 256 + threadIdx.x; idx < pieces; idx += gridDim.x * 256) {
    const uint32_t ktp = idx / R0, r = idx - ktp * R0;
    union {
      v4u_rt v;
      out_piece_t p[G];
    } out;
    out.v = v4u_rt{0u, 0u, 0u, 0u};
#pragma unroll
    for (uint32_t j = 0; j < G; ++j) {
      const uint32_t kt = ktp * G + j;
      if (kt >= K1) break;
      const char* sp = s + ((int64_t)kt * R0 + r) * SB;
      if constexpr (SRC_BITS == 8) {
        out.p[j] = *reinterpret_cast<const src_piece_t*>(sp);
      } else {
        const uint32_t packed = *reinterpret_cast<const src_piece_t*>(sp);
        out.p[j] = (out_piece_t)widen_nibbles<SB>(packed);
      }
    }
    *reinterpret_cast<v4u_rt*>(d + (int64_t)idx * 16) = out.v;
  }
}

// One-byte tile rows in tiles whose height is a multiple of four: a thread
// takes four rows of one destination tile, loads them as sixteen words (four
// rows of one K position each) and transposes bytes in registers.
__global__ __launch_bounds__(256) void retile_bytes_by_four_rows_kernel(const char* src, int64_t src_stride,
                                                                         char* dst, int64_t dst_stride,
                                                                         uint32_t R0, uint32_t K1, uint32_t K1p) {
  typedef uint32_t u32_g __attribute__((aligned(1)));
  const char* s = src + (int64_t)blockIdx.y * src_stride;
  char* d = dst + (int64_t)blockIdx.y * dst_stride;
  const uint32_t r4s = R0 / 4, items = K1p * r4s;
  for (uint32_t idx = blockIdx.x * 256 + threadIdx.x; idx < items; idx += gridDim.x * 256) {
    const uint32_t ktp = idx / r4s, r = (idx - ktp * r4s) * 4;
    uint32_t w[16];
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) {
      const uint32_t kt = ktp * 16 + j;
      w[j] = kt < K1 ? *reinterpret_cast<const u32_g*>(s + (int64_t)kt * R0 + r) : 0u;
    }
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      const uint32_t pick = i | ((4 + i) << 8);   // byte i of the first word, byte i of the second
      v4u_rt row;
#pragma unroll
      for (uint32_t q = 0; q < 4; ++q) {
        const uint32_t lo = __builtin_amdgcn_perm(w[4 * q + 1], w[4 * q], pick);
        const uint32_t hi = __builtin_amdgcn_perm(w[4 * q + 3], w[4 * q + 2], pick);
        row[q] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
      }
      *reinterpret_cast<v4u_rt*>(d + ((int64_t)ktp * R0 + r + i) * 16) = row;
    }
  }
}
}  // namespace

void retile_rows(const char* src, int64_t src_stride, int panels, int R0, int rb, int K1, int src_bits,
                 char* dst, hipStream_t stream) {
  const int g = 16 / rb;
  const uint32_t K1p = (uint32_t)((K1 + g - 1) / g);
  const int64_t dst_stride = (int64_t)K1p * R0 * 16;
  if (src_bits == 8 && rb == 1 && R0 % 4 == 0) {
    const uint32_t per_panel = (uint32_t)std::min<int64_t>(((int64_t)K1p * (R0 / 4) + 255) / 256, 64);
    uk::launch(2, retile_bytes_by_four_rows_kernel, dim3(per_panel, (uint32_t)panels), dim3(256), 0, stream, src,
               src_stride, dst, dst_stride, (uint32_t)R0, (uint32_t)K1, K1p);
    return;
  }
  const uint32_t per_panel = (uint32_t)std::min<int64_t>(((int64_t)K1p * R0 + 255) / 256, 64);
  const dim3 grid(per_panel, (uint32_t)panels), block(256);
#define UK_RETILE(BITS, RB)                                                                              \
  uk::launch(2, retile_rows_kernel<BITS, RB>, grid, block, 0, stream, src, src_stride, dst, dst_stride, \
             (uint32_t)R0, (uint32_t)K1, K1p)
  if (src_bits == 4) {
    if (rb == 2) UK_RETILE(4, 2);
    else if (rb == 4) UK_RETILE(4, 4);
    else UK_RETILE(4, 8);
  } else {
    if (rb == 1) UK_RETILE(8, 1);
    else if (rb == 2) UK_RETILE(8, 2);
    else if (rb == 4) UK_RETILE(8, 4);
    else UK_RETILE(8, 8);
  }
#undef UK_RETILE
}

int acquire_expand_workspace(size_t bytes, hipStream_t stream, char** base_out) {
  if (g_no_alloc || bytes == 0 || bytes > ((size_t)2 << 30)) return 1;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) { (void)hipGetLastError(); return 1; }
  if (capture != hipStreamCaptureStatusNone) return 1;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 1;
  OwnedWorkspaces& pool = g_expand_workspaces;
  const uint64_t now = ++pool.uses;
  for (OwnedWorkspace& w : pool) {
    if (w.device == dev && w.stream == stream && w.partial_bytes >= bytes) {
      w.last_use = now;
      *base_out = w.base;
      return 0;
    }
  }
  // Nothing fits: the stream's smaller buffer goes, and beyond two buffers per
  // thread the one used longest ago (hipFree waits for the device first).
  for (size_t i = 0; i < pool.size();) {
    if (pool[i].device == dev && pool[i].stream == stream) {
      (void)hipFree(pool[i].base);
      pool.erase(pool.begin() + (ptrdiff_t)i);
    } else {
      ++i;
    }
  }
  while (pool.size() >= 2) {
    size_t oldest = 0;
    for (size_t i = 1; i < pool.size(); ++i) {
      if (pool[i].last_use < pool[oldest].last_use) oldest = i;
    }
    (void)hipFree(pool[oldest].base);
    pool.erase(pool.begin() + (ptrdiff_t)oldest);
  }
  size_t want = (size_t)16 << 20;
  while (want < bytes) want <<= 1;
  char* base = nullptr;
  if (hipMalloc((void**)&base, want) != hipSuccess) { (void)hipGetLastError(); return 1; }
  iree_uk_amd_hip_note_device_alloc();
  pool.push_back(OwnedWorkspace{dev, stream, base, want, 0, now});
  *base_out = base;
  return 0;
}

}  // namespace uk_mfma

extern "C" IREE_UK_AMD_EXPORT int64_t iree_uk_amd_workspace_bytes(void) {
  int64_t total = 0;
  for (const OwnedWorkspace& w : g_workspaces) total += (int64_t)w.partial_bytes + (int64_t)w.n_counters * 4;
  for (const OwnedWorkspace& w : g_expand_workspaces) total += (int64_t)w.partial_bytes;
  return total;
}

extern "C" IREE_UK_AMD_EXPORT int iree_uk_amd_release_workspaces(void) {
  int status = 0, current = 0;
  (void)hipGetDevice(&current);
  for (OwnedWorkspaces* pool : {&g_workspaces, &g_expand_workspaces}) {
    for (OwnedWorkspace& w : *pool) {
      if (!w.base) continue;
      (void)hipSetDevice(w.device);
      const hipError_t err = hipFree(w.base);   // waits for the device: nothing in flight still uses it
      if (err != hipSuccess && !status) status = (int)err;
    }
    pool->clear();
  }
  (void)hipSetDevice(current);
  return status;
}

extern "C" void iree_uk_amd_hip_set_no_alloc(int on) { g_no_alloc = on != 0; }

extern "C" IREE_UK_AMD_EXPORT void iree_uk_amd_set_k_slices(int n) { g_k_slices = n > 0 ? n : 0; }
extern "C" IREE_UK_AMD_EXPORT void iree_uk_amd_set_streamed_weights(int on) { g_streamed_weights = on != 0; }

extern "C" IREE_UK_AMD_EXPORT int iree_uk_amd_last_k_slices(void) { return g_last_k_slices; }

extern "C" IREE_UK_AMD_EXPORT int64_t iree_uk_amd_no_alloc_scratch_bytes(void) {
  return (int64_t)kScratchBytes;
}

extern "C" IREE_UK_AMD_EXPORT void iree_uk_amd_set_persistent_workgroups(int n) {
  g_persistent_workgroups = n > 0 ? n : 0;
}

namespace {

using uk_mfma::Elem;

// Element type of the MFMA kernel that serves the type triple in `flags`, the
// operand element size and the output element size; false when there is none.
// The 16-bit float outputs are served only with
// IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS (one rounding at the end is
// what an f32 accumulator gives; rounding after every K element is not).
bool elem_of(uint32_t flags, Elem* e, int* elem_bytes, int* out_bytes) {
  const bool skip = (flags & IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) != 0;
  *out_bytes = 4;
  switch (flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_UK_FLAG_MMT4D_TYPE_S8S8S32: *e = Elem::kS8; *elem_bytes = 1; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F32: *e = Elem::kF16; *elem_bytes = 2; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *e = Elem::kBF16; *elem_bytes = 2; return true;
    case IREE_UK_AMD_FLAG_MMT4D_TYPE_F8E4M3FNF8E4M3FNF32: *e = Elem::kF8; *elem_bytes = 1; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_F32F32F32: *e = Elem::kF32; *elem_bytes = 4; return true;
    case IREE_UK_FLAG_MMT4D_TYPE_F16F16F16:
      *e = Elem::kF16F16; *elem_bytes = 2; *out_bytes = 2; return skip;
    case IREE_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      *e = Elem::kBF16BF16; *elem_bytes = 2; *out_bytes = 2; return skip;
    default: return false;
  }
}

bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

}  // namespace

// 1 when an MFMA kernel serves (type, M0, N0, K0) for every M, N, K: the row
// width K0*sizeof(elem) is a power of two in [2, 128] bytes (f8: [16, 128]),
// tiles are at most 64 rows, and for rows narrower than 16 bytes the tile
// height is a multiple of the 16/RB rows that share a 16-byte piece.
extern "C" int iree_uk_amd_hip_mmt4d_mfma_supported(int32_t M0, int32_t N0,
                                                    int32_t K0, uint32_t flags) {
  Elem e;
  int eb, ob;
  if (!elem_of(flags, &e, &eb, &ob)) return 0;
  const int64_t rb = (int64_t)K0 * eb;
  if (!is_pow2(rb) || rb < 2 || rb > 128) return 0;
  if (e == Elem::kF8 && rb < 16) return 0;
  if (M0 < 1 || N0 < 1 || M0 > 64 || N0 > 64) return 0;
  if (rb < 16) {
    const int R = (int)(16 / rb);
    if (M0 % R || N0 % R) return 0;
  }
  return 1;
}

// Returns a HIP status (>= 0), or -1 when the call is not served after all
// (negative strides, spans beyond 2 GiB, ...).
extern "C" int iree_uk_amd_hip_launch_mmt4d_mfma(const iree_uk_mmt4d_params_t* p,
                                                 const iree_uk_amd_rowmajor_out_t* rowmajor,
                                                 void* stream_v, int forced_variant,
                                                 const char** kernel_name) {
  Elem e;
  int eb, ob;
  // s8 x s4 -> s32 has a kernel for some shapes only (K0 a power of two in
  // [16, 64], K in whole 64-element steps; from 512 rows on, what the s8
  // kernels take): it does not count as "supported"
  // for iree_uk_mmt4d_info, but is tried before the generic kernel.
  const bool s8s4 = (p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) == IREE_UK_FLAG_MMT4D_TYPE_S8S4S32;
  // s16 x s16 -> s32 likewise: four 8-bit products per element pair in the
  // LDS-direct pipeline, for K in whole steps of 64 elements (forced variant 18
  // is that kernel's 128x128 shape).
  const bool s16 = (p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK) == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32;
  if (s8s4) {
    e = Elem::kS8S4;
    eb = 1;
    ob = 4;
    // (K0 below 16 - the reference's arm64 tiles Mx16x2 and Mx8x8 - only on
    // expanded weights, i.e. from 512 rows on: launch_s8s4)
    if (p->K0 != 2 && p->K0 != 4 && p->K0 != 8 && p->K0 != 16 && p->K0 != 32 && p->K0 != 64) return -1;
    if (p->M0 < 1 || p->N0 < 1 || p->M0 > 64 || p->N0 > 64) return -1;
    if (forced_variant != 0 && forced_variant != 4) return -1;
  } else if (s16) {
    e = Elem::kS16;
    eb = 2;
    ob = 4;
    const int64_t rb = (int64_t)p->K0 * eb;
    if (!is_pow2(rb) || rb < 2 || rb > 128) return -1;
    if (p->M0 < 1 || p->N0 < 1 || p->M0 > 64 || p->N0 > 64) return -1;
    if (rb < 16 && (p->M0 % (16 / rb) || p->N0 % (16 / rb))) return -1;
    if (forced_variant != 0 && forced_variant != 18) return -1;
  } else {
    if (!elem_of(p->flags, &e, &eb, &ob)) return -1;
    if (!iree_uk_amd_hip_mmt4d_mfma_supported(p->M0, p->N0, p->K0, p->flags)) return -1;
  }
  if (p->K == 0) return -1;  // zero fill only: the generic kernel does it
  uk_mfma::note_k_slices(1);
  hipStream_t stream = (hipStream_t)stream_v;
  uk_mfma::Problem pr;
  pr.lhs = (const char*)p->lhs_buffer + p->lhs_offset * eb;
  // 4-bit elements: offsets and strides land on byte boundaries (validated).
  pr.rhs = (const char*)p->rhs_buffer + (s8s4 ? p->rhs_offset / 2 : p->rhs_offset * eb);
  pr.out = (char*)p->out_buffer + p->out_offset * ob;
  pr.lhs_stride = p->lhs_stride0 * eb;
  pr.rhs_stride = s8s4 ? p->rhs_stride0 / 2 : p->rhs_stride0 * eb;
  if (rowmajor) {
    // Row m of panel pl is matrix row pl * M0 + m; column panels follow each
    // other inside a row.
    pr.out_sm0 = rowmajor->stride0 * ob;
    pr.out_stride = pr.out_sm0 * p->M0;
    pr.out_spn = (int64_t)p->N0 * ob;
    pr.out_rows = rowmajor->size0;
    pr.out_cols = rowmajor->size1;
  } else {
    pr.out_stride = p->out_stride0 * ob;
    pr.out_sm0 = (int64_t)p->N0 * ob;
    pr.out_spn = (int64_t)p->M0 * p->N0 * ob;
    pr.out_rows = p->M * p->M0;
    pr.out_cols = p->N * p->N0;
  }
  pr.acc = pr.out;
  pr.acc_stride = pr.out_stride;
  pr.acc_sm0 = pr.out_sm0;
  pr.acc_spn = pr.out_spn;
  pr.dequant = false;
  pr.row_scale = pr.col_scale = nullptr;
  if (rowmajor && rowmajor->dequant) {
    if (ob != 4) return -1;
    pr.dequant = true;
    pr.row_scale = rowmajor->row_scale;
    pr.col_scale = rowmajor->col_scale;
    if (p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) {
      pr.acc = (const char*)rowmajor->acc;
      pr.acc_stride = rowmajor->acc_stride0 * ob;
      pr.acc_sm0 = (int64_t)p->N0 * ob;
      pr.acc_spn = (int64_t)p->M0 * p->N0 * ob;
      if ((uintptr_t)pr.acc & 3) return -1;
    }
  }
  // The kernels add unsigned 32-bit offsets to panel bases: no negative strides.
  if (pr.lhs_stride < 0 || pr.rhs_stride < 0 || pr.out_stride < 0 || pr.out_sm0 < 0 ||
      pr.acc_stride < 0) {
    return -1;
  }
  // Operands need no alignment beyond their element's: the kernels read them
  // with vector loads that take any address (v4i_g in the kernel header).
  if (((uintptr_t)pr.lhs | (uintptr_t)pr.rhs) & (uintptr_t)(s8s4 ? 0 : eb - 1)) return -1;
  if ((uintptr_t)pr.out & (uintptr_t)(ob - 1)) return -1;
  pr.M1 = (int32_t)p->M;
  pr.N1 = (int32_t)p->N;
  pr.K1 = (int32_t)p->K;
  pr.M0 = p->M0;
  pr.N0 = p->N0;
  pr.rb = p->K0 * eb;
  pr.lrb = 0;
  while ((1 << pr.lrb) < pr.rb) ++pr.lrb;
  pr.accumulate = (p->flags & IREE_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  switch (e) {
    case Elem::kS8S4: return uk_mfma::launch_s8s4(pr, stream, kernel_name);
    case Elem::kS16: return uk_mfma::launch_s16(pr, forced_variant, stream, kernel_name);
    case Elem::kS8: return uk_mfma::launch_s8(pr, forced_variant, stream, kernel_name);
    case Elem::kF16: return uk_mfma::launch_f16(pr, forced_variant, stream, kernel_name);
    case Elem::kBF16: return uk_mfma::launch_bf16(pr, forced_variant, stream, kernel_name);
    case Elem::kF8: return uk_mfma::launch_f8(pr, forced_variant, stream, kernel_name);
    case Elem::kF32: return uk_mfma::launch_f32(pr, forced_variant, stream, kernel_name);
    case Elem::kF16F16: return uk_mfma::launch_f16f16(pr, forced_variant, stream, kernel_name);
    case Elem::kBF16BF16: return uk_mfma::launch_bf16bf16(pr, forced_variant, stream, kernel_name);
  }
  return -1;
}

// Tile rows under 16 bytes that the matrix-core kernels do not take as they
// are (one-byte rows; rows of 2, 4 or 8 bytes in tiles whose height is not a
// multiple of the 16 / rb rows a 16-byte piece spans; f8 rows under 16 bytes):
// both operands are regrouped along K into tiles of the same height with
// 16-byte rows, in the buffer the library keeps for expanded weights, and the
// call goes on with K0 = 16 bytes. The K order of the products is unchanged and
// the zero bytes that fill up the last tile pair zero with zero, so integers
// come out the same and floats as the matrix-core kernels give them for the
// wider tile. Returns a HIP status, or a negative value when the call is not
// served this way (nothing launched then).
extern "C" int iree_uk_amd_hip_launch_mmt4d_retiled(const iree_uk_mmt4d_params_t* p,
                                                    const iree_uk_amd_rowmajor_out_t* rowmajor,
                                                    void* stream_v, const char** kernel_name) {
  const uint32_t type = p->flags & IREE_UK_FLAG_MMT4D_TYPE_MASK;
  Elem e = Elem::kS16;
  int eb, ob;
  if (type == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32) {
    eb = 2;
  } else if (!elem_of(p->flags, &e, &eb, &ob)) {
    return -1;
  }
  const int64_t rb = (int64_t)p->K0 * eb;
  if (rb != 1 && rb != 2 && rb != 4 && rb != 8) return -1;
  if (p->M0 < 1 || p->N0 < 1 || p->M0 > 64 || p->N0 > 64) return -1;
  // A shape the kernels take as it is has been declined for another reason
  // (strides, spans), which the regrouping does not change.
  const bool whole_rows = rb >= 2 && p->M0 % (16 / rb) == 0 && p->N0 % (16 / rb) == 0;
  if (whole_rows && (type == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32 || e != Elem::kF8)) return -1;
  if (type == IREE_UK_FLAG_MMT4D_TYPE_S16S16S32) {
    // (what the s16 kernel asks for: K in whole steps of 64 elements, more than 32 rows and columns)
    const int64_t k_tiles = ((int64_t)p->K + 16 / rb - 1) / (16 / rb);
    if ((k_tiles * 8) % 64 != 0 || (int64_t)p->M * p->M0 <= 32 || (int64_t)p->N * p->N0 <= 32) return -1;
  }
  if (p->M <= 0 || p->N <= 0 || p->K <= 0 || p->M >= 65536 || p->N >= 65536) return -1;
  // The two passes over the operands cost a few microseconds: from about 256^3
  // multiply-adds on that is less than the scalar kernel loses.
  if ((double)p->M * p->M0 * (double)p->N * p->N0 * (double)p->K * p->K0 < 16777216.0) return -1;
  const int g = (int)(16 / rb);
  const int64_t K1p = ((int64_t)p->K + g - 1) / g;
  const int64_t lhs_bytes = (int64_t)p->M * K1p * p->M0 * 16, rhs_bytes = (int64_t)p->N * K1p * p->N0 * 16;
  if (K1p * p->M0 * 16 >= (1ll << 31) || K1p * p->N0 * 16 >= (1ll << 31) || K1p >= (1ll << 31)) return -1;
  hipStream_t stream = (hipStream_t)stream_v;
  char* ws = nullptr;
  if (uk_mfma::acquire_expand_workspace((size_t)(lhs_bytes + rhs_bytes), stream, &ws) != 0) return -1;
  uk_mfma::retile_rows((const char*)p->lhs_buffer + p->lhs_offset * eb, p->lhs_stride0 * eb, (int)p->M, p->M0,
                       (int)rb, (int)p->K, 8, ws, stream);
  uk_mfma::retile_rows((const char*)p->rhs_buffer + p->rhs_offset * eb, p->rhs_stride0 * eb, (int)p->N, p->N0,
                       (int)rb, (int)p->K, 8, ws + lhs_bytes, stream);
  iree_uk_mmt4d_params_t q = *p;
  q.K0 = 16 / eb;
  q.K = (iree_uk_index_t)K1p;
  q.lhs_buffer = ws;
  q.lhs_offset = 0;
  q.lhs_stride0 = K1p * p->M0 * q.K0;
  q.rhs_buffer = ws + lhs_bytes;
  q.rhs_offset = 0;
  q.rhs_stride0 = K1p * p->N0 * q.K0;
  const char* inner = nullptr;
  const int st = iree_uk_amd_hip_launch_mmt4d_mfma(&q, rowmajor, stream_v, 0, &inner);
  if (st >= 0) *kernel_name = "mmt4d_mfma_retiled";
  return st;
}
