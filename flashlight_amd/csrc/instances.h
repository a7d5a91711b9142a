// Kernel instance registry: one launcher per compiled (head dims, tile shape, feature set).
#pragma once
#include <hip/hip_runtime.h>

#include "fwd_kernel.h"

namespace fl {

struct Instance {
  const char* name;
  int dtype;  // element type of q, k, v, o: FL_BF16 (0) or FL_F16 (2)
  int dqk, dv;
  int rw, bn, nw, ns;  // rows per wave, keys per tile, waves per workgroup, K/V tiles resident in LDS
  uint32_t feat;
  int lds_fixed_bytes;  // LDS without the tile list (4 more bytes per key tile)
  hipError_t (*launch)(const KParams&, int grid, int lds_bytes, hipStream_t);
};

// Defined by instances_table.cpp from the per-file launchers.
extern const Instance kInstances[];
extern const int kNumInstances;

constexpr int kMaxLdsBytes = 160 * 1024;  // per workgroup on gfx950

template <class T>
hipError_t launch_fwd(const KParams& kp, int grid, int lds_bytes, hipStream_t stream) {
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_kernel<T>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(fwd_kernel<T>, dim3(grid), dim3(T::NT), lds_bytes, stream, kp);
  return hipGetLastError();
}

}  // namespace fl

// Declares (FL_INSTANCE_DECL) or defines (FL_INSTANCE_DEF) the launcher of one instance for one element type
// (SFX = _bf16 / _f16, ELEM = fl::bf16_t / fl::f16_t), and its row of the table (DT = FL_BF16 / FL_F16).
#define FL_INSTANCE_DECL_(NAME, SFX) \
  namespace fl { hipError_t launch_##NAME##SFX(const KParams&, int, int, hipStream_t); }
#define FL_INSTANCE_DECL(NAME, DQK, DV, RW, BN, NW, NS, FEAT) \
  FL_INSTANCE_DECL_(NAME, _bf16) FL_INSTANCE_DECL_(NAME, _f16)
#define FL_INSTANCE_DEF_(NAME, SFX, ELEM, DQK, DV, RW, BN, NW, NS, FEAT)                          \
  namespace fl {                                                                                  \
  hipError_t launch_##NAME##SFX(const KParams& kp, int grid, int lds, hipStream_t s) {            \
    return launch_fwd<FwdTraits<DQK, DV, RW, BN, NW, (FEAT), NS, ELEM>>(kp, grid, lds, s);        \
  }                                                                                               \
  }
#define FL_INSTANCE_DEF(NAME, SFX, ELEM, ...) FL_INSTANCE_DEF_(NAME, SFX, ELEM, __VA_ARGS__)
#define FL_INSTANCE_ROW_(NAME, SFX, DT, DQK, DV, RW, BN, NW, NS, FEAT) \
  {#NAME, DT, DQK, DV, RW, BN, NW, NS, (FEAT), fl::FwdTraits<DQK, DV, RW, BN, NW, (FEAT), NS>::LDS_FIXED_BYTES, &fl::launch_##NAME##SFX},
#define FL_INSTANCE_ROW(NAME, ...) \
  FL_INSTANCE_ROW_(NAME, _bf16, 0, __VA_ARGS__) FL_INSTANCE_ROW_(NAME, _f16, 2, __VA_ARGS__)
