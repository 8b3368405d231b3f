// Thin C-ABI wrappers over the HIP runtime for the plain-C host layer.
#include <hip/hip_runtime.h>

#include <atomic>
#include <vector>

#include "uk_hip_abi.h"
#include "uk_launch.h"

namespace {

// Per-thread ring of event pairs for kernel timing.
struct TimingState {
  bool on = false;
  std::vector<hipEvent_t> start, stop;
  std::vector<int> kind;
  size_t used = 0;
};
thread_local TimingState g_timing;

}  // namespace

namespace uk {

bool timing_next_events(int kind, hipEvent_t* start, hipEvent_t* stop) {
  TimingState& t = g_timing;
  if (!t.on) return false;
  if (t.used == t.start.size()) {
    hipEvent_t a, b;
    if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return false;
    t.start.push_back(a);
    t.stop.push_back(b);
    t.kind.push_back(0);
  }
  t.kind[t.used] = kind;
  *start = t.start[t.used];
  *stop = t.stop[t.used];
  ++t.used;
  return true;
}

}  // namespace uk

extern "C" {

int iree_uk_amd_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

int iree_uk_amd_hip_classify_pointer(const void* ptr, int* is_device) {
  hipPointerAttribute_t attr;
  hipError_t err = hipPointerGetAttributes(&attr, ptr);
  if (err != hipSuccess) {
    // Memory HIP has never seen is ordinary host memory; the runtime reports
    // it as an invalid value. Clear the sticky error.
    (void)hipGetLastError();
    *is_device = 0;
    return 0;
  }
  switch (attr.type) {
    case hipMemoryTypeDevice:
    case hipMemoryTypeManaged:
    case hipMemoryTypeArray:
      *is_device = 1;
      break;
    case hipMemoryTypeHost:
      // Pinned host memory is device-accessible through its device alias.
      *is_device = attr.devicePointer != nullptr;
      break;
    default:  // hipMemoryTypeUnregistered
      *is_device = 0;
      break;
  }
  return 0;
}

namespace {
// Staging arenas of the calling thread, one per device it has staged on.
// Grow-only and kept until iree_uk_amd_release_staging or the thread's end: a
// thread that keeps passing host operands allocates a handful of times in
// its life instead of several times per call.
struct StagingArena {
  int device;
  void* base;
  size_t bytes;
};
// Freed when the thread ends (a pool of short-lived threads must not leak
// device memory); hipFree waits for the device, so nothing in flight can still
// read the block.
struct StagingArenas : std::vector<StagingArena> {
  ~StagingArenas() {
    for (StagingArena& a : *this) {
      if (a.base) (void)hipFree(a.base);
    }
  }
};
thread_local StagingArenas g_staging;
}  // namespace

int iree_uk_amd_hip_staging_reserve(void** base, int64_t bytes) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  StagingArena* arena = nullptr;
  for (StagingArena& a : g_staging) {
    if (a.device == dev) arena = &a;
  }
  if (!arena) {
    g_staging.push_back(StagingArena{dev, nullptr, 0});
    arena = &g_staging.back();
  }
  if (arena->bytes < (size_t)bytes) {
    // The previous user synchronized before returning: nothing in flight
    // reads the old block.
    if (arena->base) (void)hipFree(arena->base);
    arena->base = nullptr;
    arena->bytes = 0;
    size_t want = 1u << 20;
    while (want < (size_t)bytes) want <<= 1;
    // Above 256 MiB grow by what is asked, rounded to 64 MiB, not by doubling.
    if (want > (256u << 20)) want = ((size_t)bytes + (64u << 20) - 1) / (64u << 20) * (64u << 20);
    err = hipMalloc(&arena->base, want);
    if (err != hipSuccess) {
      arena->base = nullptr;
      return (int)err;
    }
    iree_uk_amd_hip_note_device_alloc();
    arena->bytes = want;
  }
  *base = arena->base;
  return 0;
}

// Device allocations (hipMalloc calls) the library has made in this process:
// the staging arenas here and the K-split workspaces of mmt4d_mfma.hip.
static std::atomic<int64_t> g_device_allocs{0};
extern "C" void iree_uk_amd_hip_note_device_alloc(void) { g_device_allocs.fetch_add(1, std::memory_order_relaxed); }
extern "C" IREE_UK_AMD_EXPORT int64_t iree_uk_amd_device_alloc_count(void) {
  return g_device_allocs.load(std::memory_order_relaxed);
}

extern "C" IREE_UK_AMD_EXPORT int64_t iree_uk_amd_staging_bytes(void) {
  int64_t total = 0;
  for (const StagingArena& a : g_staging) total += (int64_t)a.bytes;
  return total;
}

extern "C" IREE_UK_AMD_EXPORT int iree_uk_amd_release_staging(void) {
  int status = 0;
  int current = 0;
  (void)hipGetDevice(&current);
  for (StagingArena& a : g_staging) {
    if (!a.base) continue;
    (void)hipSetDevice(a.device);
    const hipError_t err = hipFree(a.base);
    if (err != hipSuccess && !status) status = (int)err;
  }
  (void)hipSetDevice(current);
  g_staging.clear();
  return status;
}

int iree_uk_amd_hip_copy2d_to_device(void* dst, int64_t dst_pitch,
                                     const void* src, int64_t src_pitch,
                                     int64_t width, int64_t height,
                                     void* stream) {
  return (int)hipMemcpy2DAsync(dst, (size_t)dst_pitch, src, (size_t)src_pitch,
                               (size_t)width, (size_t)height,
                               hipMemcpyHostToDevice, (hipStream_t)stream);
}

int iree_uk_amd_hip_copy2d_to_host(void* dst, int64_t dst_pitch,
                                   const void* src, int64_t src_pitch,
                                   int64_t width, int64_t height,
                                   void* stream) {
  return (int)hipMemcpy2DAsync(dst, (size_t)dst_pitch, src, (size_t)src_pitch,
                               (size_t)width, (size_t)height,
                               hipMemcpyDeviceToHost, (hipStream_t)stream);
}

int iree_uk_amd_hip_stream_synchronize(void* stream) {
  return (int)hipStreamSynchronize((hipStream_t)stream);
}

void iree_uk_amd_timing_begin(void) {
  g_timing.on = true;
  g_timing.used = 0;
}

int iree_uk_amd_timing_end(double* elapsed_us, int* kinds, int capacity) {
  TimingState& t = g_timing;
  t.on = false;
  int n = 0;
  for (size_t i = 0; i < t.used; ++i) {
    if (hipEventSynchronize(t.stop[i]) != hipSuccess) break;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, t.start[i], t.stop[i]) != hipSuccess) break;
    if (n < capacity) {
      if (elapsed_us) elapsed_us[n] = (double)ms * 1e3;
      if (kinds) kinds[n] = t.kind[i];
    }
    ++n;
  }
  t.used = 0;
  return n;
}

const char* iree_uk_amd_hip_error_string(int status) {
  if (status == IREE_UK_AMD_STATUS_SCRATCH_TOO_SMALL) {
    return "the call's K-split workspace exceeds the static scratch array of "
           "iree_uk_amd_mmt4d_no_alloc (iree_uk_amd_no_alloc_scratch_bytes); use iree_uk_mmt4d";
  }
  if (status == IREE_UK_AMD_STATUS_NEEDS_ALLOCATION) {
    return "iree_uk_amd_mmt4d_no_alloc takes device-accessible operands only: a host operand "
           "would have to be staged through a device allocation; use iree_uk_mmt4d";
  }
  return hipGetErrorString((hipError_t)status);
}

}  // extern "C"
