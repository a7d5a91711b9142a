// Operand packing of invariant point attention behind fl_ipa_pack.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flashlight_amd.h"

namespace {

typedef __bf16 bf16_t;

// One thread per (batch, head, residue) row: [scalar channels | point coordinates | zeros] for q, k and v, and the
// per-key term w * sum(k_points^2) in fp32.
__global__ void __launch_bounds__(256) ipa_pack_kernel(const fl_ipa_pack_params p) {
  const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (row >= p.rows) return;
  const bf16_t* qs = static_cast<const bf16_t*>(p.q_scalar) + row * p.c_qk;
  const bf16_t* ks = static_cast<const bf16_t*>(p.k_scalar) + row * p.c_qk;
  const bf16_t* vs = static_cast<const bf16_t*>(p.v_scalar) + row * p.c_v;
  const bf16_t* qp = static_cast<const bf16_t*>(p.q_points) + row * p.n_qk_coords;
  const bf16_t* kp = static_cast<const bf16_t*>(p.k_points) + row * p.n_qk_coords;
  const bf16_t* vp = static_cast<const bf16_t*>(p.v_points) + row * p.n_v_coords;
  bf16_t* qc = static_cast<bf16_t*>(p.q_cat) + row * p.dqk;
  bf16_t* kc = static_cast<bf16_t*>(p.k_cat) + row * p.dqk;
  bf16_t* vc = static_cast<bf16_t*>(p.v_cat) + row * p.dv;
  for (int i = 0; i < p.c_qk; ++i) {
    qc[i] = (bf16_t)((float)qs[i] * p.q_scale);
    kc[i] = ks[i];
  }
  float sq = 0.f;
  for (int i = 0; i < p.n_qk_coords; ++i) {
    qc[p.c_qk + i] = qp[i];
    const bf16_t x = kp[i];
    kc[p.c_qk + i] = x;
    sq += (float)x * (float)x;
  }
  for (int i = p.c_qk + p.n_qk_coords; i < p.dqk; ++i) {
    qc[i] = (bf16_t)0.f;
    kc[i] = (bf16_t)0.f;
  }
  for (int i = 0; i < p.c_v; ++i) vc[i] = vs[i];
  for (int i = 0; i < p.n_v_coords; ++i) vc[p.c_v + i] = vp[i];
  for (int i = p.c_v + p.n_v_coords; i < p.dv; ++i) vc[i] = (bf16_t)0.f;
  p.key_term[row] = p.point_weight * sq;
}

}  // namespace

extern "C" int fl_ipa_pack(const fl_ipa_pack_params* p, void* stream) {
  if (!p) return FL_ERR_NULL;
  if (!p->q_scalar || !p->k_scalar || !p->v_scalar || !p->q_points || !p->k_points || !p->v_points || !p->q_cat ||
      !p->k_cat || !p->v_cat || !p->key_term)
    return FL_ERR_NULL;
  if (p->rows <= 0 || p->c_qk < 0 || p->c_v < 0 || p->n_qk_coords < 0 || p->n_v_coords < 0 ||
      p->dqk < p->c_qk + p->n_qk_coords || p->dv < p->c_v + p->n_v_coords || p->rows > ((int64_t)1 << 38))
    return FL_ERR_SHAPE;
  hipLaunchKernelGGL(ipa_pack_kernel, dim3((unsigned)((p->rows + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), *p);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}
