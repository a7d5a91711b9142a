// Measurement aids beside the forward, built into a library of their own (libflashlight_amd_probe.so) that only the
// benchmark loads: the matrix-pipe rate probe behind fl_probe_mfma_rate and the key-tile step probe behind fl_probe_step.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flashlight_amd_probe.h"

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
  if (!operands || !sink || n_fragments <= 0 || iters <= 0 || n_workgroups <= 0) return FLP_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(operands) % 16 != 0) return FLP_ERR_ALIGN;
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(n_workgroups), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const bf16x8*>(operands), n_fragments, sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

namespace {

typedef __bf16 bf16x4p __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2p __attribute__((ext_vector_type(2)));
typedef short s16x4p __attribute__((ext_vector_type(4)));
enum : int { PSG_VALU = 0x2, PSG_MFMA = 0x8, PSG_TRANS = 0x400 };

// The forward's key-tile step reduced to its instruction mix and data dependences, per 32-key block and wave:
// D / 16 MFMAs S(next) = K . Q^T chained on one accumulator, 16 x (multiply-add, exponential), 8 packs and 8 row-sum
// dot products on S(current), D / 16 MFMAs O += V . P from the packed weights.  No global memory, no transfers, no
// barriers, no masks.  LEVEL 0: the MFMAs alone; 1: MFMAs and vector work without dependences between them (the
// vector work runs on constants); 2: the step as the forward has it, operands in registers; 3: the same with the K
// and V fragments read from LDS like the forward's (ds_read_b128, transposing ds_read_b64).
template <int D, int LEVEL>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) step_probe_kernel(float* out, int iters, float c2, float seed) {
  constexpr int KS = D / 16, DVB = D / 32, CPR = D / 8;
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * 32 * D * 2];
  const int lane = threadIdx.x % 64, r = lane % 32, h = lane / 32;
  for (int i = threadIdx.x; i < 2 * 32 * D * 2 / 4; i += 256) reinterpret_cast<float*>(smem)[i] = seed;
  __syncthreads();
  bf16x8 kf[KS], qf[KS], vf[2][DVB];
  for (int i = 0; i < KS; ++i)
    for (int e = 0; e < 8; ++e) {
      kf[i][e] = (__bf16)(seed * (i + e));
      qf[i][e] = (__bf16)(seed * (i - e));
    }
  for (int c = 0; c < 2; ++c)
    for (int i = 0; i < DVB; ++i)
      for (int e = 0; e < 8; ++e) vf[c][i][e] = (__bf16)(seed * (c + i + e));
  f32x16 oacc[DVB], sa, sb, fixed;
  for (int i = 0; i < DVB; ++i)
    for (int e = 0; e < 16; ++e) oacc[i][e] = 0.f;
  for (int e = 0; e < 16; ++e) {
    sa[e] = seed * e;
    sb[e] = seed;
    fixed[e] = seed + e;
  }
  float l = 0.f, mc = seed;
  auto qk = [&](f32x16& s) __attribute__((always_inline)) {
    for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      bf16x8 a = kf[ks];
      if (LEVEL == 3) a = *reinterpret_cast<const bf16x8*>(smem + r * (D * 2) + (((2 * ks + h) ^ (r % (CPR < 16 ? CPR : 16))) * 16));
      else asm volatile("" : "+v"(kf[ks]));  // opaque, like a fresh LDS read
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s, 0, 0, 0);
    }
  };
  auto weights = [&](const f32x16& s, bf16x8 (&pf)[2]) __attribute__((always_inline)) {
    const bf16x2p ones = {(__bf16)1.0f, (__bf16)1.0f};
    float rs = 0.f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int e = 0; e < 8; ++e) pf[j][e] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(s[8 * j + e], c2, -mc));
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const bf16x2p pr = {pf[j][e], pf[j][e + 1]};
        rs = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, rs, false);
      }
    }
    l += rs;
  };
  auto pv = [&](const bf16x8 (&pf)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb) {
        bf16x8 a = vf[c][dvb];
        if (LEVEL == 3) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int i16 = lane % 16, g = (lane / 16) % 2;
            const int row = 16 * c + 8 * j + 4 * h + i16 / 4, col = dvb * 32 + g * 16 + 4 * (i16 % 4);
            const unsigned char* ap = smem + 32 * D * 2 + row * (D * 2) + (col / 8) * 16 + (col % 8) * 2;
            typedef s16x4p __attribute__((address_space(3))) * lds_ptr;
            const bf16x4p b4 = __builtin_bit_cast(bf16x4p, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(ap)));
            for (int e = 0; e < 4; ++e) a[4 * j + e] = b4[e];
          }
        } else {
          asm volatile("" : "+v"(vf[c][dvb]));
        }
        oacc[dvb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[c], oacc[dvb], 0, 0, 0);
      }
  };
  bf16x8 pconst[2];
  for (int c = 0; c < 2; ++c)
    for (int e = 0; e < 8; ++e) pconst[c][e] = (__bf16)seed;
  auto step = [&](f32x16& sc, f32x16& sn) __attribute__((always_inline)) {
    bf16x8 pf[2];
    qk(sn);
    if (LEVEL == 0) {
      pv(pconst);
    } else if (LEVEL == 1) {
      asm volatile("" : "+v"(fixed));
      weights(fixed, pf);  // vector work on values no MFMA produces; its results feed nothing
      asm volatile("" ::"v"(pf[0]), "v"(pf[1]));
      pv(pconst);
    } else {
      weights(sc, pf);
#pragma unroll
      for (int i = 0; i < KS; ++i) {  // the forward's interleave: each S MFMA followed by its share of the vector work
        __builtin_amdgcn_sched_group_barrier(PSG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(PSG_VALU | PSG_TRANS, (48 + KS - 1) / KS, 0);
      }
      pv(pf);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  for (int it = 0; it < iters; ++it) {
    step(sa, sb);
    step(sb, sa);
  }
  float s = l;
  for (int i = 0; i < DVB; ++i)
    for (int e = 0; e < 16; ++e) s += oacc[i][e];
  for (int e = 0; e < 16; ++e) s += sa[e] + sb[e];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

template <int D>
hipError_t launch_step_probe(int level, int iters, int n_workgroups, float* sink, hipStream_t stream) {
  switch (level) {
    case 0: hipLaunchKernelGGL((step_probe_kernel<D, 0>), dim3(n_workgroups), dim3(256), 0, stream, sink, iters, 0.f, 0.f); break;
    case 1: hipLaunchKernelGGL((step_probe_kernel<D, 1>), dim3(n_workgroups), dim3(256), 0, stream, sink, iters, 0.f, 0.f); break;
    case 2: hipLaunchKernelGGL((step_probe_kernel<D, 2>), dim3(n_workgroups), dim3(256), 0, stream, sink, iters, 0.f, 0.f); break;
    default: hipLaunchKernelGGL((step_probe_kernel<D, 3>), dim3(n_workgroups), dim3(256), 0, stream, sink, iters, 0.f, 0.f); break;
  }
  return hipGetLastError();
}

}  // namespace

extern "C" int fl_probe_step(int head_dim, int level, int iters, int n_workgroups, float* sink, void* stream) {
  if (!sink || iters <= 0 || n_workgroups <= 0 || level < 0 || level > 3) return FLP_ERR_ARG;
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e;
  if (head_dim == 64) e = launch_step_probe<64>(level, iters, n_workgroups, sink, st);
  else if (head_dim == 128) e = launch_step_probe<128>(level, iters, n_workgroups, sink, st);
  else return FLP_ERR_UNSUPPORTED;
  return e == hipSuccess ? 0 : 1;
}

