// Thin C-ABI wrappers over the HIP runtime for the plain-C host layer.
#include <hip/hip_runtime.h>

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

int iree_uk_amd_hip_malloc(void** ptr, int64_t bytes) {
  return (int)hipMalloc(ptr, (size_t)bytes);
}

int iree_uk_amd_hip_free(void* ptr) { return (int)hipFree(ptr); }

int iree_uk_amd_hip_copy2d_to_device(void* dst, int64_t dst_pitch,
                                     const void* src, int64_t src_pitch,
                                     int64_t width, int64_t height,
                                     void* stream) {
  hipError_t err =
      hipMemcpy2DAsync(dst, (size_t)dst_pitch, src, (size_t)src_pitch,
                       (size_t)width, (size_t)height, hipMemcpyHostToDevice,
                       (hipStream_t)stream);
  if (err != hipSuccess) return (int)err;
  // Pageable host memory: the caller may reuse or free `src` right after the
  // entry point returns, so wait for the copy.
  return (int)hipStreamSynchronize((hipStream_t)stream);
}

int iree_uk_amd_hip_copy2d_to_host(void* dst, int64_t dst_pitch,
                                   const void* src, int64_t src_pitch,
                                   int64_t width, int64_t height,
                                   void* stream) {
  hipError_t err =
      hipMemcpy2DAsync(dst, (size_t)dst_pitch, src, (size_t)src_pitch,
                       (size_t)width, (size_t)height, hipMemcpyDeviceToHost,
                       (hipStream_t)stream);
  if (err != hipSuccess) return (int)err;
  return (int)hipStreamSynchronize((hipStream_t)stream);
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
