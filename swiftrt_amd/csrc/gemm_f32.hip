// fp32 matmul on the matrix cores (v_mfma_f32_32x32x2_f32): true fp32 products and sums.
#include "gemm_common.h"

namespace srt {

bool f32_mfma_supported(const GemmProblem&) { return false; }

hipError_t launch_f32_mfma(const GemmProblem&, hipStream_t) { return hipErrorNotSupported; }

}  // namespace srt
