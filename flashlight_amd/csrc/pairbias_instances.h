// Launchers of the shared-bias streaming forward (pairbias_kernel.h): 32-key blocks per row in {8, 10, 12}
// (256, 320 or 384 keys), with or without the sigmoid gate, bf16 or fp16 elements.
#pragma once
#include <hip/hip_runtime.h>

#include "pairbias_kernel.h"

namespace fl {
hipError_t launch_pairbias_bf16(int nkb, bool gate, const PParams& p, int grid, hipStream_t stream);
hipError_t launch_pairbias_f16(int nkb, bool gate, const PParams& p, int grid, hipStream_t stream);
inline bool pairbias_has_shape(int nkb) { return nkb == 8 || nkb == 10 || nkb == 12; }
}  // namespace fl
