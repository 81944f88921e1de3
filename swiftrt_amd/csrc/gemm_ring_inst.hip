// One instantiation unit of the ring kernel: compiled once per (element type, A layout,
// B layout) with -DSRT_RING_TYPE=BF16|F16 -DSRT_RING_AKC=0|1 -DSRT_RING_BKC=0|1, so the eight
// combinations build in parallel.
#include "gemm_mfma_ring.h"

namespace srt {

#define SRT_CAT2(a, b, c, d) a##_##b##_##c##d
#define SRT_CAT(a, b, c, d) SRT_CAT2(a, b, c, d)

// launch_ring_<type>_<akc><bkc>
hipError_t SRT_CAT(launch_ring, SRT_RING_TYPE, SRT_RING_AKC, SRT_RING_BKC)(const GemmProblem& p, hipStream_t stream) {
  return ring::launch<SRT_RING_TYPE, SRT_RING_AKC != 0, SRT_RING_BKC != 0>(p, stream);
}

}  // namespace srt
