// One instantiation unit of the 128 x 256 half tile of the 64-deep 16x16x32 kernel (k-contiguous A): compiled once per
// (element type, B layout) with -DSRT_M16_TYPE=BF16|F16 -DSRT_M16_BKC=0|1.
#include "gemm_mfma_m16d.h"

namespace srt {

#define SRT_CAT2(a, b, c) a##_##b##_1##c
#define SRT_CAT(a, b, c) SRT_CAT2(a, b, c)

// launch_m16dh_<type>_1<bkc>
hipError_t SRT_CAT(launch_m16dh, SRT_M16_TYPE, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch_half<SRT_M16_TYPE, SRT_M16_BKC != 0>(p, stream);
}

// launch_m16dh_partial_<type>_11: the split-K pass (used for a k-contiguous B only)
#if SRT_M16_BKC
hipError_t SRT_CAT(launch_m16dh_partial, SRT_M16_TYPE, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch_half_partial<SRT_M16_TYPE, true>(p, stream);
}
#endif

}  // namespace srt
