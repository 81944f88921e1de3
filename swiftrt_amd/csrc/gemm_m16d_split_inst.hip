// One instantiation unit of the split form of the 64-deep 16x16x32 kernel (whole rounds of 256 x 256 tiles, then one round
// of 256 x 192 tiles): compiled once per (element type, A layout, B layout) with -DSRT_M16_TYPE=BF16|F16
// -DSRT_M16_AKC=0|1 -DSRT_M16_BKC=0|1.
#include "gemm_mfma_m16d.h"

namespace srt {

#define SRT_CAT2(a, b, c, d) a##_##b##_##c##d
#define SRT_CAT(a, b, c, d) SRT_CAT2(a, b, c, d)

// launch_m16d_split_<type>_<akc><bkc>
hipError_t SRT_CAT(launch_m16d_split, SRT_M16_TYPE, SRT_M16_AKC, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch_split<SRT_M16_TYPE, SRT_M16_AKC != 0, SRT_M16_BKC != 0>(p, stream);
}

// whether the split form applies to `p` (defined once)
#if SRT_M16_AKC == 0 && SRT_M16_BKC == 0
bool SRT_CAT(m16d_split_fits, SRT_M16_TYPE, x, x)(const GemmProblem& p) { return m16d::split_fits(p); }
#endif

}  // namespace srt
