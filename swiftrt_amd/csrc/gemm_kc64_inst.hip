// One instantiation unit of the k-contiguous 64-deep kernel: compiled once per element type with
// -DSRT_KC_TYPE=BF16|F16.
#include "gemm_mfma_kc64.h"

namespace srt {

#define SRT_CAT2(a, b) a##_##b
#define SRT_CAT(a, b) SRT_CAT2(a, b)

// launch_kc64_<type>
hipError_t SRT_CAT(launch_kc64, SRT_KC_TYPE)(const GemmProblem& p, hipStream_t stream) {
  return kc64::launch<SRT_KC_TYPE>(p, stream);
}

}  // namespace srt
