// Merge of partial attention results over key chunks, behind fl_attn_merge_chunks.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flashlight_amd.h"

namespace {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

// One wave per result row.  part [outer][chunks][inner][dv] holds normalised partial results (each the attention of
// the row over one chunk of the keys), lse [outer][chunks][inner] their row statistics (base-2 logarithm of the chunk's
// sum of weights; +inf marks a chunk in which the row attends nothing).  out [outer][inner][dv] = sum_c w_c part_c /
// sum_c w_c with w_c = 2^(lse_c - max_c lse_c): the softmax over all keys.  A row without keys in any chunk is zeros.
template <class E>
__global__ void __launch_bounds__(64) merge_chunks_kernel(const E* __restrict__ part, const float* __restrict__ lse,
                                                          E* __restrict__ out, int chunks, int64_t inner, int dv) {
  const int64_t row = blockIdx.x, o = row / inner, i = row % inner;
  const int lane = threadIdx.x;
  const float* l = lse + (o * chunks) * inner + i;
  float top = -INFINITY;
  for (int c = 0; c < chunks; ++c) {
    const float x = l[(int64_t)c * inner];
    if (x != INFINITY) top = fmaxf(top, x);
  }
  float total = 0.f;
  for (int c = 0; c < chunks; ++c) {
    const float x = l[(int64_t)c * inner];
    if (x != INFINITY && top != -INFINITY) total += exp2f(x - top);
  }
  const float inv = total > 0.f ? 1.0f / total : 0.f;
  for (int d = 2 * lane; d < dv; d += 128) {   // dv is even: two elements per lane and step
    float a0 = 0.f, a1 = 0.f;
    for (int c = 0; c < chunks; ++c) {
      const float x = l[(int64_t)c * inner];
      if (x == INFINITY || top == -INFINITY) continue;
      const float w = exp2f(x - top);
      const E* p = part + (((o * chunks + c) * inner + i) * dv + d);
      a0 += w * (float)p[0];
      a1 += w * (float)p[1];
    }
    E* q = out + (row * dv + d);
    q[0] = (E)(a0 * inv);
    q[1] = (E)(a1 * inv);
  }
}

}  // namespace

extern "C" int fl_attn_merge_chunks(const void* part, const float* lse, void* out, int64_t outer, int32_t chunks,
                                    int64_t inner, int32_t dv, int32_t dtype, void* stream) {
  if (!part || !lse || !out) return FL_ERR_NULL;
  if (outer <= 0 || inner <= 0 || chunks <= 0 || dv <= 0 || (dv & 1) || outer * inner > ((int64_t)1 << 31) - 1)
    return FL_ERR_SHAPE;
  if (dtype != FL_BF16 && dtype != FL_F16) return FL_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)(outer * inner)), block(64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FL_BF16)
    hipLaunchKernelGGL(merge_chunks_kernel<bf16_t>, grid, block, 0, s, static_cast<const bf16_t*>(part), lse,
                       static_cast<bf16_t*>(out), chunks, inner, dv);
  else
    hipLaunchKernelGGL(merge_chunks_kernel<f16_t>, grid, block, 0, s, static_cast<const f16_t*>(part), lse,
                       static_cast<f16_t*>(out), chunks, inner, dv);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}
