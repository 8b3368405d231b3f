// Kernel launch helper shared by the HIP translation units.
//
// Normally a plain launch. When the calling thread has switched kernel timing
// on (iree_uk_amd_timing_begin), each launch carries its own start/stop event
// pair through hipExtLaunchKernelGGL, which timestamps the kernel itself: the
// elapsed time is the kernel's device duration, without the marker and
// dispatch gaps that events recorded around a launch include.
#ifndef IREE_UK_AMD_LAUNCH_H_
#define IREE_UK_AMD_LAUNCH_H_

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

namespace uk {

// Returns false when timing is off for this thread. Otherwise hands out the
// next event pair of the thread's ring and tags it with `kind`
// (0 pack, 1 unpack, 2 mmt4d).
bool timing_next_events(int kind, hipEvent_t* start, hipEvent_t* stop);

template <typename Kernel, typename... Args>
inline void launch(int kind, Kernel kernel, dim3 grid, dim3 block, size_t lds_bytes,
                   hipStream_t stream, Args... args) {
  hipEvent_t start, stop;
  if (timing_next_events(kind, &start, &stop)) {
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, start, stop, 0, args...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, args...);
  }
}

}  // namespace uk

#endif  // IREE_UK_AMD_LAUNCH_H_
