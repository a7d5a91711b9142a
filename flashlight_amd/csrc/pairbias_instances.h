// Launchers of the shared-bias streaming forward (pairbias_kernel.h).  Head dim 32: 32-key blocks per row in
// {4, 6, 8, 10, 12} (128 .. 384 keys), with or without the sigmoid gate.  Head dim 64: 4, 6 or 8 blocks (128, 192 or
// 256 keys), no gate (its
// 16 registers of logits in flight do not fit beside 64 of bias and 32 of results).  Both with or without a second bias
// that is one row per batch entry.  bf16 or fp16 elements.
#pragma once
#include <hip/hip_runtime.h>

#include "pairbias_kernel.h"

namespace fl {
hipError_t launch_pairbias_bf16(int d, int nkb, bool gate, bool rowb, const PParams& p, int grid, hipStream_t stream);
hipError_t launch_pairbias_f16(int d, int nkb, bool gate, bool rowb, const PParams& p, int grid, hipStream_t stream);
inline bool pairbias_has_shape(int d, int nkb, bool gate, bool rowb) {
  (void)rowb;
  if (d == 32) return nkb == 4 || nkb == 6 || nkb == 8 || nkb == 10 || nkb == 12;
  if (d == 64) return !gate && (nkb == 4 || nkb == 6 || nkb == 8);
  return false;
}
}  // namespace fl
