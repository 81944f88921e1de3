// One instantiation unit of the 128 x 128 quarter tile of the 16x16x32 kernel (128-deep staging units): compiled once per
// (element type, A layout, B layout) with -DSRT_M16_TYPE=BF16|F16 -DSRT_M16_AKC=0|1 -DSRT_M16_BKC=0|1.
#include "gemm_mfma_m16q.h"

namespace srt {

#define SRT_CAT2(a, b, c, d) a##_##b##_##c##d
#define SRT_CAT(a, b, c, d) SRT_CAT2(a, b, c, d)

// launch_m16q_<type>_<akc><bkc>
hipError_t SRT_CAT(launch_m16q, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16q::launch<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

}  // namespace srt
