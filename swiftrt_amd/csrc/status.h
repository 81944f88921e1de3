// hipError_t -> srtStatus mapping shared by the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/srt_hip.h"

namespace srt {
srtStatus from_hip(hipError_t e);
}
