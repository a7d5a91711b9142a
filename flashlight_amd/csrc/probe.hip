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
// and V fragments read from LDS like the forward's (ds_read_b128, transposing ds_read_b64); 4: level 2 in a
// three-stage order: the second product takes the PREVIOUS block's weights, so that both groups of MFMAs are issued
// under this block's vector work (a rung the forward was built and measured on, and does not use).
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
  bf16x8 pa[2], pb[2];  // level 4: the weights of one block live until the next block's second product
  for (int c = 0; c < 2; ++c)
    for (int e = 0; e < 8; ++e) pa[c][e] = pb[c][e] = (__bf16)seed;
  auto step = [&](f32x16& sc, f32x16& sn, bf16x8 (&pnew)[2], const bf16x8 (&pold)[2]) __attribute__((always_inline)) {
    bf16x8 pf[2];
    qk(sn);
    if (LEVEL == 4) {
      weights(sc, pnew);
      pv(pold);
      constexpr int NM = KS + 2 * DVB;
#pragma unroll
      for (int i = 0; i < NM; ++i) {
        __builtin_amdgcn_sched_group_barrier(PSG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(PSG_VALU | PSG_TRANS, (48 + NM - 1) / NM, 0);
      }
    } else if (LEVEL == 0) {
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
    step(sa, sb, pa, pb);
    step(sb, sa, pb, pa);
  }
  float s = l;
  for (int c = 0; c < 2; ++c) s += (float)pa[c][0] + (float)pb[c][0];
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
    case 4: hipLaunchKernelGGL((step_probe_kernel<D, 4>), dim3(n_workgroups), dim3(256), 0, stream, sink, iters, 0.f, 0.f); break;
    default: hipLaunchKernelGGL((step_probe_kernel<D, 3>), dim3(n_workgroups), dim3(256), 0, stream, sink, iters, 0.f, 0.f); break;
  }
  return hipGetLastError();
}

}  // namespace

extern "C" int fl_probe_step(int head_dim, int level, int iters, int n_workgroups, float* sink, void* stream) {
  if (!sink || iters <= 0 || n_workgroups <= 0 || level < 0 || level > 4) return FLP_ERR_ARG;
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e;
  if (head_dim == 64) e = launch_step_probe<64>(level, iters, n_workgroups, sink, st);
  else if (head_dim == 128) e = launch_step_probe<128>(level, iters, n_workgroups, sink, st);
  else return FLP_ERR_UNSUPPORTED;
  return e == hipSuccess ? 0 : 1;
}


// ---- co-issue probe: how much vector work fits under matrix instructions -------------------------------------------------
// A loop of 8 matrix instructions on independent accumulators (32x32x16 bf16, or twice as many 16x16x32 bf16), each
// followed by K vector instructions of one kind on registers no matrix instruction touches; zero operands, nothing
// else.  Written with fixed registers so that the compiler neither reorders nor merges anything.  The time per matrix
// instruction against the bare loop's says how many cycles of an MFMA the vector ALU can use, whether the shorter
// matrix instruction leaves more room, and which vector instructions do not overlap with the matrix pipe at all.
namespace {

#define FLP_CLOBBER                                                                                                      \
  "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", "v10", "v11", "v12", "v13", "v14", "v15", "v16", "v17",    \
      "v18", "v19", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v30", "v31", "v32", "v33",    \
      "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47", "v48", "v49",    \
      "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62", "v63", "v64", "v65",    \
      "v66", "v67", "v68", "v69", "v70", "v71", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108",  \
      "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v118", "v121", "s4"

// one 32 x 32 x 16 matrix instruction on accumulator j (of four), or the same work as two 16 x 16 x 32 instructions on
// accumulators 2j, 2j + 1 (of sixteen)
#define FLP_M32(j) "v_mfma_f32_32x32x16_bf16 v[" #j "*16:" #j "*16+15], v[64:67], v[68:71], v[" #j "*16:" #j "*16+15]\n"
#define FLP_M16(j)                                                                                       \
  "v_mfma_f32_16x16x32_bf16 v[" #j "*8:" #j "*8+3], v[64:67], v[68:71], v[" #j "*8:" #j "*8+3]\n"            \
  "v_mfma_f32_16x16x32_bf16 v[" #j "*8+4:" #j "*8+7], v[64:67], v[68:71], v[" #j "*8+4:" #j "*8+7]\n"
// K vector instructions of kind KIND (0 multiply-add, 1 exponential, 2 pack to bf16, 3 dot product of two bf16 pairs with
// accumulation, 4 addition): destinations v100.., sources v108.., v118, v121.  %0 = K, %1 = KIND (assembler constants).
#define FLP_VALU                                                                                         \
  ".set flp_k, 0\n .rept %0\n"                                                                           \
  " .if %1 == 0\n v_fma_f32 v[100+flp_k], v[108+flp_k], v121, v118\n .endif\n"                           \
  " .if %1 == 1\n v_exp_f32 v[100+flp_k], v[108+flp_k]\n .endif\n"                                       \
  " .if %1 == 2\n v_cvt_pk_bf16_f32 v[100+flp_k], v[108+flp_k], v[108+((flp_k+1)&7)]\n .endif\n"         \
  " .if %1 == 3\n v_dot2c_f32_bf16 v[100+flp_k], 0x3f803f80, v[108+flp_k]\n .endif\n"                    \
  " .if %1 == 4\n v_add_f32 v[100+flp_k], v[100+flp_k], v[108+flp_k]\n .endif\n"                         \
  " .set flp_k, flp_k+1\n .endr\n"

template <int MF, int KIND, int K>
__global__ void __launch_bounds__(512) coissue_kernel(float* out, int iters, long long* cycles) {
  const long long c0 = clock64();
  asm volatile("s_mov_b32 s4, 0\n .set flp_i, 0\n .rept 72\n v_mov_b32 v[flp_i], 0\n .set flp_i, flp_i+1\n .endr\n"
               " .set flp_i, 100\n .rept 22\n v_mov_b32 v[flp_i], 0\n .set flp_i, flp_i+1\n .endr" ::: FLP_CLOBBER);
  for (int it = 0; it < iters; ++it) {
    if (MF == 32)
      asm volatile(FLP_M32(0) FLP_VALU FLP_M32(1) FLP_VALU FLP_M32(2) FLP_VALU FLP_M32(3) FLP_VALU
                   FLP_M32(0) FLP_VALU FLP_M32(1) FLP_VALU FLP_M32(2) FLP_VALU FLP_M32(3) FLP_VALU ::"n"(K), "n"(KIND) : FLP_CLOBBER);
    else
      asm volatile(FLP_M16(0) FLP_VALU FLP_M16(1) FLP_VALU FLP_M16(2) FLP_VALU FLP_M16(3) FLP_VALU
                   FLP_M16(4) FLP_VALU FLP_M16(5) FLP_VALU FLP_M16(6) FLP_VALU FLP_M16(7) FLP_VALU ::"n"(K), "n"(KIND) : FLP_CLOBBER);
  }
  float r;
  asm volatile("v_add_f32 %0, v0, v100" : "=v"(r)::FLP_CLOBBER);
  const long long c1 = clock64();
  out[blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (threadIdx.x % 64 == 0) cycles[blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64] = c1 - c0;
}

template <int MF, int KIND>
hipError_t launch_coissue(int k, int waves_per_simd, int iters, int n_workgroups, float* sink, long long* cycles, hipStream_t st) {
  const dim3 g(n_workgroups), b(256 * waves_per_simd);
  switch (k) {
    case 0: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 0>), g, b, 0, st, sink, iters, cycles); break;
    case 1: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 1>), g, b, 0, st, sink, iters, cycles); break;
    case 2: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 2>), g, b, 0, st, sink, iters, cycles); break;
    case 3: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 3>), g, b, 0, st, sink, iters, cycles); break;
    case 4: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 4>), g, b, 0, st, sink, iters, cycles); break;
    case 6: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 6>), g, b, 0, st, sink, iters, cycles); break;
    case 8: hipLaunchKernelGGL((coissue_kernel<MF, KIND, 8>), g, b, 0, st, sink, iters, cycles); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

template <int MF>
hipError_t launch_coissue_kind(int kind, int k, int w, int iters, int n, float* sink, long long* cycles, hipStream_t st) {
  switch (kind) {
    case 0: return launch_coissue<MF, 0>(k, w, iters, n, sink, cycles, st);
    case 1: return launch_coissue<MF, 1>(k, w, iters, n, sink, cycles, st);
    case 2: return launch_coissue<MF, 2>(k, w, iters, n, sink, cycles, st);
    case 3: return launch_coissue<MF, 3>(k, w, iters, n, sink, cycles, st);
    case 4: return launch_coissue<MF, 4>(k, w, iters, n, sink, cycles, st);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

extern "C" int fl_probe_coissue(int mfma_rows, int valu_kind, int valu_per_mfma, int waves_per_simd, int iters,
                                int n_workgroups, float* sink, long long* wave_cycles, void* stream) {
  if (!sink || !wave_cycles || iters <= 0 || n_workgroups <= 0 || (waves_per_simd != 1 && waves_per_simd != 2))
    return FLP_ERR_ARG;
  if ((mfma_rows != 32 && mfma_rows != 16) || valu_kind < 0 || valu_kind > 4) return FLP_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const hipError_t e = mfma_rows == 32
                           ? launch_coissue_kind<32>(valu_kind, valu_per_mfma, waves_per_simd, iters, n_workgroups, sink, wave_cycles, st)
                           : launch_coissue_kind<16>(valu_kind, valu_per_mfma, waves_per_simd, iters, n_workgroups, sink, wave_cycles, st);
  if (e == hipErrorInvalidValue) return FLP_ERR_UNSUPPORTED;
  return e == hipSuccess ? 0 : 1;
}
