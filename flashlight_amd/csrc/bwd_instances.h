// Launchers of the backward kernels: one translation unit per (head dim, feature set), both roles in it.
#pragma once
#include <hip/hip_runtime.h>

#include "bwd_kernel.h"
#include "instances.h"

namespace fl {

struct BwdInstance {
  int d;
  uint32_t feat;
  int dtype;  // element type of q, k, v, o, dout and the gradients: FL_BF16 (0) or FL_F16 (2)
  hipError_t (*launch_dq)(const BParams&, hipStream_t);
  hipError_t (*launch_dkv)(const BParams&, hipStream_t);
  hipError_t (*launch_delta)(const BParams&, hipStream_t);
};

extern const BwdInstance kBwdInstances[];
extern const int kNumBwdInstances;

template <class T>
hipError_t launch_bwd(const BParams& bp, hipStream_t stream) {
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_kernel<T>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
  if (attr != hipSuccess) return attr;
  const int len = T::ROLE == ROLE_DQ ? bp.Lq : bp.Lk, heads = T::ROLE == ROLE_DQ ? bp.Hq : bp.Hkv;
  const int64_t grid = (int64_t)bp.B * heads * ((len + T::OWN - 1) / T::OWN);
  hipLaunchKernelGGL(bwd_kernel<T>, dim3((unsigned)grid), dim3(T::NT), T::LDS_BYTES, stream, bp);
  return hipGetLastError();
}

template <int DV, class E>
hipError_t launch_delta(const BParams& bp, hipStream_t stream) {
  const int64_t rows = (int64_t)bp.B * bp.Hq * bp.Lq;
  const int rows_per_block = 256 / (DV / 8);
  hipLaunchKernelGGL((bwd_delta_kernel<DV, E>), dim3((unsigned)((rows + rows_per_block - 1) / rows_per_block)), dim3(256), 0,
                     stream, bp);
  return hipGetLastError();
}

}  // namespace fl

// (D, FEAT) pairs with compiled backward kernels.  FEAT 3 = ALiBi and/or soft-cap (either may be off at run time),
// 4 = bias operands, 8 = document ids in the element predicate, 11 = document ids with ALiBi and/or a soft-cap,
// 7, 12, 15 = bias operands with ALiBi / soft-cap, with document ids, with both,
// 128 + any of these = the same with dropout (head dims 64 and 128).
#define FL_BWD_LIST(X) X(32, 0) X(32, 3) X(32, 4) X(32, 7) X(32, 8) X(32, 11) X(32, 12) X(32, 15) X(64, 0) X(64, 3) X(64, 4) X(64, 7) X(64, 8) X(64, 11) X(64, 12) X(64, 15) X(64, 128) X(64, 131) X(64, 132) X(64, 135) X(64, 136) X(64, 139) X(64, 140) X(64, 143) X(128, 0) X(128, 3) X(128, 4) X(128, 7) X(128, 8) X(128, 11) X(128, 12) X(128, 15) X(128, 128) X(128, 131) X(128, 132) X(128, 135) X(128, 136) X(128, 139) X(128, 140) X(128, 143)

// Every (D, FEAT) pair is compiled for bf16 and for fp16 elements (suffix _bf16 / _f16).
#define FL_BWD_DECL_(D, FEAT, SFX)                                            \
  namespace fl {                                                              \
  hipError_t launch_bwd_dq_##D##_##FEAT##SFX(const BParams&, hipStream_t);    \
  hipError_t launch_bwd_dkv_##D##_##FEAT##SFX(const BParams&, hipStream_t);   \
  hipError_t launch_bwd_delta_##D##_##FEAT##SFX(const BParams&, hipStream_t); \
  }
#define FL_BWD_DECL(D, FEAT) FL_BWD_DECL_(D, FEAT, _bf16) FL_BWD_DECL_(D, FEAT, _f16)
#define FL_BWD_DEF(D, FEAT, SFX, ELEM)                                                                              \
  namespace fl {                                                                                                    \
  hipError_t launch_bwd_dq_##D##_##FEAT##SFX(const BParams& bp, hipStream_t s) {                                    \
    return launch_bwd<BwdTraits<D, ROLE_DQ, FEAT, ELEM>>(bp, s);                                                    \
  }                                                                                                                 \
  hipError_t launch_bwd_dkv_##D##_##FEAT##SFX(const BParams& bp, hipStream_t s) {                                   \
    return launch_bwd<BwdTraits<D, ROLE_DKV, FEAT, ELEM>>(bp, s);                                                   \
  }                                                                                                                 \
  hipError_t launch_bwd_delta_##D##_##FEAT##SFX(const BParams& bp, hipStream_t s) { return launch_delta<D, ELEM>(bp, s); } \
  }
#define FL_BWD_ROW_(D, FEAT, SFX, DT) \
  {D, FEAT, DT, &fl::launch_bwd_dq_##D##_##FEAT##SFX, &fl::launch_bwd_dkv_##D##_##FEAT##SFX, &fl::launch_bwd_delta_##D##_##FEAT##SFX},
#define FL_BWD_ROW(D, FEAT) FL_BWD_ROW_(D, FEAT, _bf16, 0) FL_BWD_ROW_(D, FEAT, _f16, 2)
