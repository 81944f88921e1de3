// Host-side admission test of the ring kernel (kept out of the per-layout instantiation units).
#include "gemm_mfma_ring.h"

namespace srt {
bool ring_fits_problem(const GemmProblem& p, bool a_kc, bool b_kc) { return ring::ring_fits(p, a_kc, b_kc); }
}  // namespace srt
