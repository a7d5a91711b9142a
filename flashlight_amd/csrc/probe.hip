// Matrix-pipe rate probe behind fl_probe_mfma_rate: a measurement aid, not part of the forward.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flashlight_amd.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Nothing but MFMAs: 8 A and 4 B fragments per lane stay in registers; 4 independent accumulators, so consecutive
// MFMAs never wait for each other.  With data-dependent power limits the rate depends on the operand values.
__global__ void __launch_bounds__(512) mfma_rate_kernel(const bf16x8* in, int64_t n, float* out, int iters) {
  bf16x8 a[8], b[4];
  const int64_t t = (int64_t)blockIdx.x * 512 + threadIdx.x;
  for (int j = 0; j < 8; ++j) a[j] = in[(t * 12 + j) % n];
  for (int j = 0; j < 4; ++j) b[j] = in[(t * 12 + 8 + j) % n];
  f32x16 c[4] = {{0}, {0}, {0}, {0}};
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) c[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], b[q], c[q], 0, 0, 0);
  }
  float s = 0.f;
  for (int q = 0; q < 4; ++q)
    for (int j = 0; j < 16; ++j) s += c[q][j];
  out[t] = s;
}

}  // namespace

extern "C" int fl_probe_mfma_rate(const void* operands, int64_t n_fragments, int iters, int n_workgroups, float* sink,
                                  void* stream) {
  if (!operands || !sink || n_fragments <= 0 || iters <= 0 || n_workgroups <= 0) return FL_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(operands) % 16 != 0) return FL_ERR_ALIGN;
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(n_workgroups), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const bf16x8*>(operands), n_fragments, sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}
