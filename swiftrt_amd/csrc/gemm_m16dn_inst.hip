// One instantiation unit of the 256 x 128 half tile of the 64-deep 16x16x32 kernel (A not k-contiguous): compiled once per
// (element type, B layout) with -DSRT_M16_TYPE=BF16|F16 -DSRT_M16_BKC=0|1.
#include "gemm_mfma_m16d.h"

namespace srt {

#define SRT_CAT2(a, b, c) a##_##b##_0##c
#define SRT_CAT(a, b, c) SRT_CAT2(a, b, c)

// launch_m16dn_<type>_0<bkc>
hipError_t SRT_CAT(launch_m16dn, SRT_M16_TYPE, SRT_M16_BKC)(const GemmProblem& p, hipStream_t stream) {
  return m16d::launch_narrow<SRT_M16_TYPE, SRT_M16_BKC != 0>(p, stream);
}

}  // namespace srt
