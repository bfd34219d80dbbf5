// Launch entry points of the kernel translation units (one per .hip file).
#pragma once
#include <hip/hip_runtime.h>
#include "../problem.h"

namespace fk {

// Any shape, one factor per launch.
hipError_t launchGenericStep(const StepArgs& a, DType dt, hipStream_t stream);

}  // namespace fk
