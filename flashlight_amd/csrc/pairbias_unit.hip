// The shared-bias streaming forward (pairbias_kernel.h), every compiled shape for one element type.
// -DFL_INST_F16=1 compiles the fp16 set instead of the bf16 one.
#include "pairbias_instances.h"

namespace fl {
namespace {
template <int NKB, bool GATE, class E>
hipError_t launch_one(const PParams& p, int grid, hipStream_t stream) {
  hipLaunchKernelGGL((pairbias_kernel<PairBiasTraits<NKB, GATE, E>>), dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}
template <class E>
hipError_t launch_any(int nkb, bool gate, const PParams& p, int grid, hipStream_t stream) {
  switch (nkb * 2 + (gate ? 1 : 0)) {
    case 8 * 2: return launch_one<8, false, E>(p, grid, stream);
    case 8 * 2 + 1: return launch_one<8, true, E>(p, grid, stream);
    case 10 * 2: return launch_one<10, false, E>(p, grid, stream);
    case 10 * 2 + 1: return launch_one<10, true, E>(p, grid, stream);
    case 12 * 2: return launch_one<12, false, E>(p, grid, stream);
    case 12 * 2 + 1: return launch_one<12, true, E>(p, grid, stream);
    default: return hipErrorInvalidValue;
  }
}
}  // namespace

#if defined(FL_INST_F16) && FL_INST_F16
hipError_t launch_pairbias_f16(int nkb, bool gate, const PParams& p, int grid, hipStream_t stream) {
  return launch_any<f16_t>(nkb, gate, p, grid, stream);
}
#else
hipError_t launch_pairbias_bf16(int nkb, bool gate, const PParams& p, int grid, hipStream_t stream) {
  return launch_any<bf16_t>(nkb, gate, p, grid, stream);
}
#endif
}  // namespace fl
