// One instantiation unit of the 16x16x32 form of the 256 x 256 ring kernel: compiled once per
// (element type, A layout, B layout) with -DSRT_M16_TYPE=BF16|F16 -DSRT_M16_AKC=0|1
// -DSRT_M16_BKC=0|1, so the eight combinations build in parallel.
#include "gemm_mfma_m16.h"

namespace srt {

#define SRT_CAT2(a, b, c, d) a##_##b##_##c##d
#define SRT_CAT(a, b, c, d) SRT_CAT2(a, b, c, d)

// launch_m16_<type>_<akc><bkc>
hipError_t SRT_CAT(launch_m16, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16::launch<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

// launch_m16_partial_<type>_<akc><bkc>: the split-K pass (fp32 accumulators to a workspace)
hipError_t SRT_CAT(launch_m16_partial, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16::launch_partial<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

#if SRT_M16_AKC
// launch_m16h_<type>_1<bkc>: the 128 x 256 tile (k-contiguous A only), and its split-K pass
hipError_t SRT_CAT(launch_m16h, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16::launch<SRT_M16_TYPE, true, SRT_M16_BKC != 0, 5, 4>(p, stream);
}
hipError_t SRT_CAT(launch_m16h_partial, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16::launch_partial<SRT_M16_TYPE, true, SRT_M16_BKC != 0, 5, 4>(p, stream);
}
#endif

}  // namespace srt
