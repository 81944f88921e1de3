// One instantiation unit of the 64-deep form of the 16x16x32 256 x 256 kernel: compiled once per
// (element type, A layout, B layout) with -DSRT_M16_TYPE=BF16|F16 -DSRT_M16_AKC=0|1 -DSRT_M16_BKC=0|1.
#include "gemm_mfma_m16d.h"

namespace srt {

#define SRT_CAT2(a, b, c, d) a##_##b##_##c##d
#define SRT_CAT(a, b, c, d) SRT_CAT2(a, b, c, d)

// launch_m16d_<type>_<akc><bkc>
hipError_t SRT_CAT(launch_m16d, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

// launch_m16d_tail_<type>_<akc><bkc>: the tail-sharing form
hipError_t SRT_CAT(launch_m16d_tail, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch_tail<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

// launch_m16d_partial_<type>_<akc><bkc>: the split-K pass (fp32 accumulators to a workspace)
hipError_t SRT_CAT(launch_m16d_partial, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch_partial<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

// whether the tail-sharing form applies to `p` (defined once)
#if SRT_M16_AKC == 0 && SRT_M16_BKC == 0
bool SRT_CAT(m16d_tail_fits, SRT_M16_TYPE, x, x)(const GemmProblem& p) { return m16d::tail_fits(p); }
#endif

}  // namespace srt
