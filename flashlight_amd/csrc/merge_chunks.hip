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
  // maximum and sum over the chunks: the lanes take a chunk each, then the wave reduces
  float top = -INFINITY;
  for (int c = lane; c < chunks; c += 64) {
    const float x = l[(int64_t)c * inner];
    top = fmaxf(top, x == INFINITY ? -INFINITY : x);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) top = fmaxf(top, __shfl_xor(top, d, 64));
  const float ref = top == -INFINITY ? 0.f : top;   // (no keys anywhere: every weight below is 0)
  float total = 0.f;
  for (int c = lane; c < chunks; c += 64) {
    const float x = l[(int64_t)c * inner];
    total += x == INFINITY ? 0.f : exp2f(x - ref);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) total += __shfl_xor(total, d, 64);
  const float inv = total > 0.f ? 1.0f / total : 0.f;
  // the weighted sum: two elements per lane and step (dv is even); the loads of the chunks do not depend on one another
  const int64_t chunk_stride = inner * dv;
  for (int d = 2 * lane; d < dv; d += 128) {
    const E* p = part + ((o * chunks * inner + i) * dv + d);
    float a0 = 0.f, a1 = 0.f;
#pragma unroll 8
    for (int c = 0; c < chunks; ++c) {
      const float x = l[(int64_t)c * inner];
      const float w = x == INFINITY ? 0.f : exp2f(x - ref);
      const float v0 = (float)p[c * chunk_stride], v1 = (float)p[c * chunk_stride + 1];
      a0 += w * v0;
      a1 += w * v1;
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
