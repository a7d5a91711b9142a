// Kernel instance registry: one launcher per compiled (head dims, tile shape, feature set).
#pragma once
#include <hip/hip_runtime.h>

#include "fwd_kernel.h"

namespace fl {

struct Instance {
  const char* name;
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

// Declares (FL_INSTANCE_DECL) or defines (FL_INSTANCE_DEF) the launcher of one instance.
#define FL_INSTANCE_DECL(NAME, DQK, DV, RW, BN, NW, NS, FEAT) \
  namespace fl { hipError_t launch_##NAME(const KParams&, int, int, hipStream_t); }
#define FL_INSTANCE_DEF(NAME, DQK, DV, RW, BN, NW, NS, FEAT)                               \
  namespace fl {                                                                           \
  hipError_t launch_##NAME(const KParams& kp, int grid, int lds, hipStream_t s) {          \
    return launch_fwd<FwdTraits<DQK, DV, RW, BN, NW, (FEAT), NS>>(kp, grid, lds, s);       \
  }                                                                                        \
  }
#define FL_INSTANCE_ROW(NAME, DQK, DV, RW, BN, NW, NS, FEAT) \
  {#NAME, DQK, DV, RW, BN, NW, NS, (FEAT), fl::FwdTraits<DQK, DV, RW, BN, NW, (FEAT), NS>::LDS_FIXED_BYTES, &fl::launch_##NAME},
