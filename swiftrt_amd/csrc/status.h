// hipError_t -> srtStatus mapping shared by the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/srt_hip.h"

namespace srt {
srtStatus from_hip(hipError_t e);

// Status of the launch just queued on `stream`.  A build with -DSRT_DEBUG_LAUNCH (make DEBUG=1) also
// waits for the stream and reports what the kernel itself raised, as the reference's DEBUG builds do
// after every launch (Modules/SwiftRTCuda/cuda_macros.cuh:34-47); a release build observes
// asynchronous errors at the caller's next synchronisation.
inline hipError_t launch_status(hipStream_t stream) {
  hipError_t e = hipGetLastError();
#ifdef SRT_DEBUG_LAUNCH
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e == hipSuccess) e = hipGetLastError();
#else
  (void)stream;
#endif
  return e;
}
}  // namespace srt
