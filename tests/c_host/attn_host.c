/* A host program in plain C: the boundary of this library is its C ABI (include/flashlight_amd.h), with device pointers
 * from hipMalloc and a stream of the caller's own -- no Python, no torch.  It runs one causal grouped-query forward
 * (the reference's attention_variants/causal.py:4-36 with enable_gqa) and the backward of the same call on a
 * non-default stream, and checks both against loops in double precision written out below.
 * Exit status 0 = every check passed.  Built by `python -m flashlight_amd.build` into tests/c_host/attn_host. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "flashlight_amd.h"

#define CHECK_HIP(x)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      return 2;                                                                           \
    }                                                                                     \
  } while (0)
#define CHECK_FL(x)                                                                  \
  do {                                                                               \
    int rc_ = (x);                                                                   \
    if (rc_ != 0) {                                                                  \
      fprintf(stderr, "%s:%d: %s = %d: %s\n", __FILE__, __LINE__, #x, rc_, fl_last_error()); \
      return 3;                                                                      \
    }                                                                                \
  } while (0)

enum { B = 2, HQ = 4, HKV = 2, L = 200, D = 64 };

static uint16_t to_bf16(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t rng_state = 12345u;
static float next_uniform(void) { /* xorshift, in [-1, 1) */
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 17;
  rng_state ^= rng_state << 5;
  return (float)(rng_state >> 8) / 8388608.0f - 1.0f;
}
static void fill(uint16_t* p, size_t n, float amp) {
  for (size_t i = 0; i < n; ++i) p[i] = to_bf16(amp * next_uniform());
}

int main(void) {
  const size_t nq = (size_t)B * HQ * L * D, nk = (size_t)B * HKV * L * D;
  uint16_t *q = malloc(2 * nq), *k = malloc(2 * nk), *v = malloc(2 * nk), *dout = malloc(2 * nq);
  uint16_t *o = malloc(2 * nq), *dq = malloc(2 * nq), *dk = malloc(2 * nk), *dv = malloc(2 * nk);
  if (!q || !k || !v || !dout || !o || !dq || !dk || !dv) return 2;
  fill(q, nq, 2.0f);
  fill(k, nk, 2.0f);
  fill(v, nk, 1.0f);
  fill(dout, nq, 1.0f);

  printf("flashlight_amd C ABI version %d, sizeof(fl_attn_params) %zu / library %llu\n", fl_version(), sizeof(fl_attn_params),
         (unsigned long long)fl_params_sizeof());
  if (fl_params_sizeof() != sizeof(fl_attn_params) || fl_bwd_params_sizeof() != sizeof(fl_attn_bwd_params)) {
    fprintf(stderr, "header and library disagree on the struct sizes\n");
    return 3;
  }

  void *d_q, *d_k, *d_v, *d_o, *d_dout, *d_dq, *d_dk, *d_dv;
  float *d_lse, *d_delta;
  CHECK_HIP(hipMalloc(&d_q, 2 * nq));
  CHECK_HIP(hipMalloc(&d_k, 2 * nk));
  CHECK_HIP(hipMalloc(&d_v, 2 * nk));
  CHECK_HIP(hipMalloc(&d_o, 2 * nq));
  CHECK_HIP(hipMalloc(&d_dout, 2 * nq));
  CHECK_HIP(hipMalloc(&d_dq, 2 * nq));
  CHECK_HIP(hipMalloc(&d_dk, 2 * nk));
  CHECK_HIP(hipMalloc(&d_dv, 2 * nk));
  CHECK_HIP(hipMalloc((void**)&d_lse, sizeof(float) * B * HQ * L));
  CHECK_HIP(hipMalloc((void**)&d_delta, sizeof(float) * B * HQ * L));
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  CHECK_HIP(hipMemcpyAsync(d_q, q, 2 * nq, hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemcpyAsync(d_k, k, 2 * nk, hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemcpyAsync(d_v, v, 2 * nk, hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemcpyAsync(d_dout, dout, 2 * nq, hipMemcpyHostToDevice, stream));

  fl_attn_params p;
  memset(&p, 0, sizeof(p));
  p.q = d_q, p.k = d_k, p.v = d_v, p.o = d_o;
  const int64_t sq[4] = {(int64_t)HQ * L * D, (int64_t)L * D, D, 1}, sk[4] = {(int64_t)HKV * L * D, (int64_t)L * D, D, 1};
  memcpy(p.q_strides, sq, sizeof(sq));
  memcpy(p.o_strides, sq, sizeof(sq));
  memcpy(p.k_strides, sk, sizeof(sk));
  memcpy(p.v_strides, sk, sizeof(sk));
  p.B = B, p.Hq = HQ, p.Hkv = HKV, p.Lq = L, p.Lk = L, p.Dqk = D, p.Dv = D;
  p.scale = 1.0f / sqrtf((float)D);
  p.mask_kind = FL_MASK_CAUSAL;
  p.dtype = FL_BF16;
  p.lse = d_lse;
  CHECK_FL(fl_attn_validate(&p));
  CHECK_FL(fl_attn_fwd(&p, stream));

  fl_attn_bwd_params bw;
  memset(&bw, 0, sizeof(bw));
  bw.fwd = p;
  bw.dout = d_dout, bw.dq = d_dq, bw.dk = d_dk, bw.dv = d_dv, bw.delta = d_delta;
  memcpy(bw.dout_strides, sq, sizeof(sq));
  memcpy(bw.dq_strides, sq, sizeof(sq));
  memcpy(bw.dk_strides, sk, sizeof(sk));
  memcpy(bw.dv_strides, sk, sizeof(sk));
  CHECK_FL(fl_attn_bwd_validate(&bw));
  CHECK_FL(fl_attn_bwd(&bw, stream));

  CHECK_HIP(hipMemcpyAsync(o, d_o, 2 * nq, hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipMemcpyAsync(dq, d_dq, 2 * nq, hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipMemcpyAsync(dk, d_dk, 2 * nk, hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipMemcpyAsync(dv, d_dv, 2 * nk, hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipStreamSynchronize(stream));

  /* an argument error is reported, not launched */
  fl_attn_params bad = p;
  bad.Dqk = 48;
  if (fl_attn_fwd(&bad, stream) != FL_ERR_UNSUPPORTED || strstr(fl_last_error(), "no kernel instance") == NULL) {
    fprintf(stderr, "head dim 48 was not refused as expected: %s\n", fl_last_error());
    return 3;
  }

  /* the same computation in double: out, and the textbook gradients dV = P^T dO, dP = dO V^T,
   * dS = P (dP - rowsum(dO o O)), dQ = dS K scale, dK = dS^T Q scale */
  double *ro = calloc(nq, 8), *rdq = calloc(nq, 8), *rdk = calloc(nk, 8), *rdv = calloc(nk, 8), *w = malloc(8 * L), *dp = malloc(8 * L);
  if (!ro || !rdq || !rdk || !rdv || !w || !dp) return 2;
  const double scale = 1.0 / sqrt((double)D);
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < HQ; ++h) {
      const int hk = h / (HQ / HKV);
      const uint16_t *qh = q + ((size_t)b * HQ + h) * L * D, *kh = k + ((size_t)b * HKV + hk) * L * D, *vh = v + ((size_t)b * HKV + hk) * L * D;
      const uint16_t* gh = dout + ((size_t)b * HQ + h) * L * D;
      double *oh = ro + ((size_t)b * HQ + h) * L * D, *dqh = rdq + ((size_t)b * HQ + h) * L * D;
      double *dkh = rdk + ((size_t)b * HKV + hk) * L * D, *dvh = rdv + ((size_t)b * HKV + hk) * L * D;
      for (int i = 0; i < L; ++i) {
        double m = -INFINITY, sum = 0.0, delta = 0.0;
        for (int j = 0; j <= i; ++j) {
          double s = 0.0;
          for (int d = 0; d < D; ++d) s += (double)from_bf16(qh[i * D + d]) * from_bf16(kh[j * D + d]);
          w[j] = s * scale;
          if (w[j] > m) m = w[j];
        }
        for (int j = 0; j <= i; ++j) sum += (w[j] = exp(w[j] - m));
        for (int j = 0; j <= i; ++j) {
          w[j] /= sum;
          for (int d = 0; d < D; ++d) oh[i * D + d] += w[j] * from_bf16(vh[j * D + d]);
        }
        for (int d = 0; d < D; ++d) delta += (double)from_bf16(gh[i * D + d]) * oh[i * D + d];
        for (int j = 0; j <= i; ++j) {
          dp[j] = 0.0;
          for (int d = 0; d < D; ++d) {
            dp[j] += (double)from_bf16(gh[i * D + d]) * from_bf16(vh[j * D + d]);
            dvh[j * D + d] += w[j] * from_bf16(gh[i * D + d]);
          }
          const double ds = w[j] * (dp[j] - delta) * scale;
          for (int d = 0; d < D; ++d) {
            dqh[i * D + d] += ds * from_bf16(kh[j * D + d]);
            dkh[j * D + d] += ds * from_bf16(qh[i * D + d]);
          }
        }
      }
    }
  /* the suite's bound for a 16-bit kernel against a full-precision reference: max-abs 2e-2, mean-abs 2e-3, gradients
   * scaled by their largest reference entry */
  struct {
    const char* name;
    const uint16_t* got;
    const double* want;
    size_t n;
  } checks[4] = {{"out", o, ro, nq}, {"dq", dq, rdq, nq}, {"dk", dk, rdk, nk}, {"dv", dv, rdv, nk}};
  int failed = 0;
  for (int c = 0; c < 4; ++c) {
    double biggest = 1.0, worst = 0.0, mean = 0.0;
    for (size_t i = 0; i < checks[c].n; ++i)
      if (fabs(checks[c].want[i]) > biggest) biggest = fabs(checks[c].want[i]);
    for (size_t i = 0; i < checks[c].n; ++i) {
      const double d = fabs((double)from_bf16(checks[c].got[i]) - checks[c].want[i]) / biggest;
      if (!(d <= worst)) worst = d; /* (a NaN ends up here too) */
      mean += d / (double)checks[c].n;
    }
    const int ok = worst <= 2e-2 && mean <= 2e-3;
    printf("%-3s max-abs %.3e mean-abs %.3e (scaled by %.3g)  %s\n", checks[c].name, worst, mean, biggest, ok ? "ok" : "FAILED");
    failed |= !ok;
  }
  hipStreamDestroy(stream);
  return failed;
}
