// The shared-bias streaming forward (pairbias_kernel.h), every compiled shape for one element type.
// -DFL_INST_F16=1 compiles the fp16 set instead of the bf16 one.
#include "pairbias_instances.h"

namespace fl {
namespace {
template <int NKB, bool GATE, class E, int D = 32, bool ROWB = false, bool EXACT = false>
hipError_t launch_one(const PParams& p, int grid, hipStream_t stream) {
  using T = PairBiasTraits<NKB, GATE, E, D, ROWB, EXACT>;
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&pairbias_kernel<T>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL((pairbias_kernel<T>), dim3(grid), dim3(256), T::LDS_BYTES, stream, p);
  return hipGetLastError();
}
template <class E>
hipError_t launch_any(int d, int nkb, bool gate, bool rowb, const PParams& p, int grid, hipStream_t stream) {
  if (d == 64) {
    if (gate) return hipErrorInvalidValue;
    // (1 / scale exact in the element type: the default scale of head dim 64 is 1 / 8)
    const float w = 1.0f / p.scale;
    const bool exact = (float)(E)w == w;
    auto pick = [&](auto nkb_tag) {
      constexpr int N = decltype(nkb_tag)::value;
      if (exact) return rowb ? launch_one<N, false, E, 64, true, true>(p, grid, stream) : launch_one<N, false, E, 64, false, true>(p, grid, stream);
      return rowb ? launch_one<N, false, E, 64, true>(p, grid, stream) : launch_one<N, false, E, 64, false>(p, grid, stream);
    };
    if (nkb == 4) return pick(std::integral_constant<int, 4>{});
    if (nkb == 6) return pick(std::integral_constant<int, 6>{});
    if (nkb == 8) return pick(std::integral_constant<int, 8>{});
    return hipErrorInvalidValue;
  }
  if (d != 32) return hipErrorInvalidValue;
  switch (nkb * 4 + (gate ? 1 : 0) + (rowb ? 2 : 0)) {
    case 4 * 4: return launch_one<4, false, E>(p, grid, stream);
    case 4 * 4 + 1: return launch_one<4, true, E>(p, grid, stream);
    case 4 * 4 + 2: return launch_one<4, false, E, 32, true>(p, grid, stream);
    case 4 * 4 + 3: return launch_one<4, true, E, 32, true>(p, grid, stream);
    case 6 * 4: return launch_one<6, false, E>(p, grid, stream);
    case 6 * 4 + 1: return launch_one<6, true, E>(p, grid, stream);
    case 6 * 4 + 2: return launch_one<6, false, E, 32, true>(p, grid, stream);
    case 6 * 4 + 3: return launch_one<6, true, E, 32, true>(p, grid, stream);
    case 8 * 4: return launch_one<8, false, E>(p, grid, stream);
    case 8 * 4 + 1: return launch_one<8, true, E>(p, grid, stream);
    case 8 * 4 + 2: return launch_one<8, false, E, 32, true>(p, grid, stream);
    case 8 * 4 + 3: return launch_one<8, true, E, 32, true>(p, grid, stream);
    case 10 * 4: return launch_one<10, false, E>(p, grid, stream);
    case 10 * 4 + 1: return launch_one<10, true, E>(p, grid, stream);
    case 10 * 4 + 2: return launch_one<10, false, E, 32, true>(p, grid, stream);
    case 10 * 4 + 3: return launch_one<10, true, E, 32, true>(p, grid, stream);
    case 12 * 4: return launch_one<12, false, E>(p, grid, stream);
    case 12 * 4 + 1: return launch_one<12, true, E>(p, grid, stream);
    case 12 * 4 + 2: return launch_one<12, false, E, 32, true>(p, grid, stream);
    case 12 * 4 + 3: return launch_one<12, true, E, 32, true>(p, grid, stream);
    default: return hipErrorInvalidValue;
  }
}
}  // namespace

#if defined(FL_INST_F16) && FL_INST_F16
hipError_t launch_pairbias_f16(int d, int nkb, bool gate, bool rowb, const PParams& p, int grid, hipStream_t stream) {
  return launch_any<f16_t>(d, nkb, gate, rowb, p, grid, stream);
}
#else
hipError_t launch_pairbias_bf16(int d, int nkb, bool gate, bool rowb, const PParams& p, int grid, hipStream_t stream) {
  return launch_any<bf16_t>(d, nkb, gate, rowb, p, grid, stream);
}
#endif
}  // namespace fl
