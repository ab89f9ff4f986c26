// Launch of the fused prolog operator (internal to the library).
#pragma once
#include "lip_kernels.h"
#include "mlap_kernels.h"

namespace pto {

// the kernels of both prologs on one stream, the last launches of the two merged into one
hipError_t prolog_fused_launch(const MlapParams &pm, const LipParams &pl, hipStream_t stream);

}  // namespace pto
