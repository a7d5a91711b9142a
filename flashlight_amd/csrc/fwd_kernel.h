// Fused attention forward for gfx950 (CDNA4): one workgroup = one (batch, head, block of query rows).
//
// Replaces the Triton kernel that the reference's TorchInductor patches generate for
// attention_variants/*.py (hot loop restated in monkeypatch/fusion/_reduction.py:420-433 and
// monkeypatch/fusion/block_reduction.py:86-134).  Differences that matter: the matmuls are issued as
// v_mfma_f32_32x32x16_bf16 on transposed tiles, and key tiles whose mask is empty are never visited.
//
// Data flow per key tile (BN keys), per wave (RW query rows):
//   S^T[key, q]  = K[key, :] . Q[q, :]              MFMA, A = K fragment from LDS, B = Q fragment (registers)
//   score mods / mask on S^T in registers           lane (r, h) owns query r and 16 keys per 32-key block
//   online softmax over keys                        in-lane max/sum + one cross-half exchange per tile
//   O^T[dv, q]  += V^T[dv, key] . P^T[key, q]       MFMA, A = V fragment via transposing LDS read, B = P (registers)
// Computing the transposed products makes the fp32 accumulator layout of S^T exactly the bf16 B-operand
// layout of the second MFMA, so P never leaves registers, and the softmax statistics are per lane.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fl {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Feature bits selected at compile time; everything else is a runtime field.
enum : uint32_t {
  F_ALIBI = 1u,    // add slope_h * (k - q)
  F_SOFTCAP = 2u,  // cap * tanh(x / cap)
  F_BIAS = 4u,     // dense additive bias tensors (up to two)
  F_DOC = 8u,      // document ids take part in the element predicate
  F_DIFF = 16u,    // two softmax branches, out = A0 - lambda * A1
  F_GATE = 32u,    // out *= sigmoid(gate)
  F_DUMP = 64u,    // write the attended-pair bitmap (test hook), skip nothing else
};

enum : int { MASK_NONE = 0, MASK_CAUSAL = 1, MASK_SLIDING = 2, MASK_PREFIX = 3, MASK_DOC = 4, MASK_DOC_CAUSAL = 5 };
enum : int { TILE_EMPTY = 0, TILE_PARTIAL = 1, TILE_FULL = 2 };

// Maximum number of key tiles whose class fits the LDS table.
constexpr int kMaxKeyTiles = 4096;
// Granularity (positions) of the document-id min/max table built by doc_table_kernel.
constexpr int kDocBlock = 32;

struct KParams {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  bf16_t* o;
  int64_t qs[3], ks[3], vs[3], os[3];  // element strides: batch, head, seq
  int32_t B, Hq, Hkv, Lq, Lk;
  int32_t group;        // Hq / Hkv
  float scale;          // multiplies qk
  float scale_log2;     // scale * log2(e)
  int32_t mask_kind, window, prefix;
  const int64_t* doc_ids;
  int64_t doc_stride;
  const int64_t* doc_table;  // [B][ceil(L/kDocBlock)][2] = (min, max)
  int32_t doc_blocks;
  int32_t alibi_heads;
  float softcap;
  const bf16_t* bias[2];
  int64_t bs[2][4];
  int32_t bdiv[2];
  int32_t bias_vec[2];  // rows of this bias may be read 4 keys (8 bytes) at a time
  const bf16_t* gate;
  int64_t gs[3];
  float lambda;
  int64_t q_branch_stride, k_branch_stride;  // element offset of the second softmax branch (diff)
  uint8_t* dump;
  int32_t n_qtiles;  // ceil(Lq / BM)
  int32_t n_ktiles;  // ceil(Lk / BN)
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Exchange between the two half-waves: returns (x[l % 32], x[l % 32 + 32]) in every lane.
// The second operand goes through an empty asm so the compiler cannot assume both results are equal
// (it folds the pair to one value when it sees the same register twice).
__device__ __forceinline__ void xhalf_pair(float x, float& lo, float& hi) {
  unsigned u = __builtin_bit_cast(unsigned, x);
  unsigned w = u;
  asm volatile("" : "+v"(w));
  auto r = __builtin_amdgcn_permlane32_swap(u, w, false, false);
  // copy the elements out first: bit-casting r[1] directly is compiled as if it were r[0]
  const unsigned r0 = r[0], r1 = r[1];
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
// max / sum over the two half-waves: lanes l and l^32 both end up with the combined value.
__device__ __forceinline__ float xhalf_max(float x) {
  float a, b;
  xhalf_pair(x, a, b);
  return __builtin_fmaxf(a, b);
}
__device__ __forceinline__ float xhalf_sum(float x) {
  float a, b;
  xhalf_pair(x, a, b);
  return a + b;
}

// ---- mask logic (integer, shared by the tile classifier and the element predicate) -------------------------------

// Does query position q attend key position k?  Document ids are compared by the caller.
__device__ __forceinline__ bool attend_positional(int kind, int q, int k, int window, int prefix) {
  switch (kind) {
    case MASK_CAUSAL:
    case MASK_DOC_CAUSAL: return k <= q;
    case MASK_SLIDING: return k <= q && q - k <= window;
    case MASK_PREFIX: return k < prefix || k <= q;
    default: return true;
  }
}

// Class of the key tile [k0, k1) against query rows [q0, q1) for the positional part of the mask.
// k1 and q1 are exclusive and already clipped to the sequence lengths.
__device__ __forceinline__ int classify_positional(int kind, int q0, int q1, int k0, int k1, int window, int prefix) {
  switch (kind) {
    case MASK_CAUSAL:
    case MASK_DOC_CAUSAL:
      if (k0 > q1 - 1) return TILE_EMPTY;
      return (k1 - 1 <= q0) ? TILE_FULL : TILE_PARTIAL;
    case MASK_SLIDING:
      if (k0 > q1 - 1 || q0 - (k1 - 1) > window) return TILE_EMPTY;
      return (k1 - 1 <= q0 && (q1 - 1) - k0 <= window) ? TILE_FULL : TILE_PARTIAL;
    case MASK_PREFIX:
      if (k0 >= prefix && k0 > q1 - 1) return TILE_EMPTY;
      return (k1 <= prefix || k1 - 1 <= q0) ? TILE_FULL : TILE_PARTIAL;
    default: return TILE_FULL;
  }
}

// (min, max) document id over positions [p0, p1) from the per-kDocBlock table.
__device__ __forceinline__ void doc_range(const int64_t* table, int p0, int p1, int64_t& mn, int64_t& mx) {
  int b0 = p0 / kDocBlock, b1 = (p1 - 1) / kDocBlock;
  mn = table[2 * b0];
  mx = table[2 * b0 + 1];
  for (int b = b0 + 1; b <= b1; ++b) {
    int64_t a = table[2 * b], c = table[2 * b + 1];
    mn = a < mn ? a : mn;
    mx = c > mx ? c : mx;
  }
}

// ---- LDS tile layout ------------------------------------------------------------------------------------------------
// A tile is [rows][D] bf16, row-major, addressed in 16-byte chunks; the chunk index is XOR-swizzled with a
// function of the row so that the MFMA operand reads below spread over the banks.

template <int D>
struct TileLayout {
  static constexpr int CPR = D / 8;                          // 16-byte chunks per row
  static constexpr int RPW = (CPR >= 16) ? 1 : (16 / CPR);   // rows per 256-byte bank window
  // K operand reads: 16 consecutive rows at one logical chunk.
  __device__ static __forceinline__ int swz_k(int row, int chunk) {
    constexpr int M = (CPR >= 16 ? 16 : CPR) - 1;
    return chunk ^ ((row / RPW) & M);
  }
  // V operand reads (transposing): 4 consecutive rows x 64 contiguous bytes.
  __device__ static __forceinline__ int swz_v(int row, int chunk) {
    constexpr int G = (CPR >= 16 ? 16 : CPR) / 4;  // 64-byte groups per window row
    if constexpr (G <= 1) return chunk;
    return chunk ^ (((row / RPW) & (G - 1)) << 2);
  }
};

template <int DQK_, int DV_, int RW_, int BN_, int NW_, uint32_t FEAT_>
struct FwdTraits {
  static constexpr int DQK = DQK_, DV = DV_, RW = RW_, BN = BN_, NW = NW_;
  static constexpr uint32_t FEAT = FEAT_;
  static constexpr int NT = NW * 64;
  static constexpr int BM = NW * RW;
  static constexpr int QB = RW / 32;   // 32-row query blocks per wave
  static constexpr int KB = BN / 32;   // 32-key blocks per tile
  static constexpr int KS = DQK / 16;  // MFMA k-steps of the first product
  static constexpr int DVB = DV / 32;  // 32-wide blocks of the value dimension
  static constexpr int KBYTES = BN * DQK * 2, VBYTES = BN * DV * 2;
  static constexpr int STAGE = KBYTES + VBYTES;
  static constexpr int K_CHUNKS = BN * DQK / 8, V_CHUNKS = BN * DV / 8;
  static constexpr int K_PER_T = K_CHUNKS / NT, V_PER_T = V_CHUNKS / NT;
  static_assert(K_CHUNKS % NT == 0 && V_CHUNKS % NT == 0, "tile must divide evenly over the threads");
  static_assert(RW % 32 == 0 && BN % 32 == 0 && DQK % 16 == 0 && DV % 32 == 0, "MFMA 32x32x16 blocking");
  static constexpr int CLS_BYTES = kMaxKeyTiles * 2;
  static constexpr int LDS_BYTES = 2 * STAGE + CLS_BYTES + 16;
};

template <class T>
__global__ __launch_bounds__(T::NT) void fwd_kernel(const KParams p) {
  constexpr int DQK = T::DQK, DV = T::DV, RW = T::RW, BN = T::BN, NW = T::NW, NT = T::NT, BM = T::BM;
  constexpr int QB = T::QB, KB = T::KB, KS = T::KS, DVB = T::DVB;
  constexpr uint32_t FEAT = T::FEAT;
  constexpr bool kAlibi = FEAT & F_ALIBI, kSoftcap = FEAT & F_SOFTCAP, kBias = FEAT & F_BIAS, kDoc = FEAT & F_DOC;
  constexpr bool kDiff = FEAT & F_DIFF, kGate = FEAT & F_GATE, kDump = FEAT & F_DUMP;
  constexpr bool kMod = kAlibi || kSoftcap || kBias;  // scores are transformed before the softmax
  using LK = TileLayout<DQK>;
  using LV = TileLayout<DV>;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* cls = reinterpret_cast<uint16_t*>(smem + 2 * T::STAGE);
  int* range = reinterpret_cast<int*>(smem + 2 * T::STAGE + T::CLS_BYTES);  // [0]=first, [1]=last+1 non-empty tile

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int r = lane % 32, h = lane / 32;

  // ---- workgroup -> (batch, head, query tile).  Consecutive workgroup ids land on different XCDs, so ids are
  // regrouped to give every XCD a contiguous run of (batch, head) pairs: their K/V stay in that XCD's L2.
  // Within a run the query tiles are visited from the last (longest under a causal mask) to the first.
  int wg = blockIdx.x;
  {
    const int total = gridDim.x;
    if (total % 8 == 0) wg = (wg % 8) * (total / 8) + wg / 8;
  }
  const int qt = p.n_qtiles - 1 - (wg % p.n_qtiles);
  const int bh = wg / p.n_qtiles;
  const int head = bh % p.Hq, batch = bh / p.Hq;
  const int kvh = head / p.group;

  const int q0 = qt * BM;             // first query row of the workgroup
  const int qw0 = q0 + wave * RW;     // first query row of this wave
  const int nk = p.n_ktiles;

  // ---- classify every key tile for every wave -----------------------------------------------------------------
  if (tid == 0) {
    range[0] = nk;
    range[1] = 0;
  }
  __syncthreads();
  {
    const int64_t* dtab = kDoc ? p.doc_table + (int64_t)batch * p.doc_blocks * 2 : nullptr;
    int64_t qmn[NW], qmx[NW];
    if constexpr (kDoc) {
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        int a = q0 + w * RW, b = min(a + RW, p.Lq);
        qmn[w] = 0;
        qmx[w] = 0;
        if (a < b) doc_range(dtab, a, b, qmn[w], qmx[w]);
      }
    }
    for (int t = tid; t < nk; t += NT) {
      const int k0 = t * BN, k1 = min(k0 + BN, p.Lk);
      int64_t kmn = 0, kmx = 0;
      if constexpr (kDoc) doc_range(dtab, k0, k1, kmn, kmx);
      unsigned c = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        int a = q0 + w * RW, b = min(a + RW, p.Lq);
        int cw = TILE_EMPTY;
        if (a < b) {
          cw = classify_positional(p.mask_kind, a, b, k0, k1, p.window, p.prefix);
          if constexpr (kDoc) {
            if (kmx < qmn[w] || kmn > qmx[w]) cw = TILE_EMPTY;
            else if (!(kmn == kmx && qmn[w] == qmx[w] && kmn == qmn[w]) && cw == TILE_FULL) cw = TILE_PARTIAL;
          }
          if (cw == TILE_FULL && k0 + BN > p.Lk) cw = TILE_PARTIAL;  // ragged tail: keys >= Lk are masked
        }
        c |= (unsigned)cw << (2 * w);
      }
      cls[t] = (uint16_t)c;
      if (c) {
        atomicMin(&range[0], t);
        atomicMax(&range[1], t + 1);
      }
    }
  }
  __syncthreads();
  const int t_first = __builtin_amdgcn_readfirstlane(range[0]), t_end = __builtin_amdgcn_readfirstlane(range[1]);

  // ---- per-lane constants ----------------------------------------------------------------------------------------
  int qrow[QB];  // query position owned by this lane in each query block
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) qrow[qb] = qw0 + qb * 32 + r;

  float slope_l2 = 0.f;  // ALiBi slope in log2 units
  if constexpr (kAlibi)
    slope_l2 = p.alibi_heads > 0 ? exp2f(-8.0f * (float)(head + 1) / (float)p.alibi_heads) * 1.4426950408889634f : 0.f;
  float cap_k1 = 0.f, cap_c = 0.f;
  if constexpr (kSoftcap) {
    cap_k1 = p.scale / p.softcap * 2.0f * 1.4426950408889634f;  // exp2 argument of e^{2x/cap}
    cap_c = p.softcap * 1.4426950408889634f;                    // cap in log2 units
  }
  int64_t qdoc[QB];
  if constexpr (kDoc) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
      qdoc[qb] = qrow[qb] < p.Lq ? p.doc_ids[(int64_t)batch * p.doc_stride + qrow[qb]] : 0;
  }

  f32x16 ofin[kDiff ? DVB : 1][kDiff ? QB : 1];  // branch-0 result kept while branch 1 runs (diff only)

  f32x16 oacc[DVB][QB];
  float m_run[QB], l_run[QB];

#pragma unroll
  for (int br = 0; br < (kDiff ? 2 : 1); ++br) {
    const bf16_t* qptr = p.q + (int64_t)batch * p.qs[0] + (int64_t)head * p.qs[1] + (int64_t)br * p.q_branch_stride;
    const bf16_t* kptr = p.k + (int64_t)batch * p.ks[0] + (int64_t)kvh * p.ks[1] + (int64_t)br * p.k_branch_stride;
    const bf16_t* vptr = p.v + (int64_t)batch * p.vs[0] + (int64_t)kvh * p.vs[1];

    // Q fragments: B operand of S^T = K.Q^T; lane (r, h) holds Q[q = r][16*ks + 8h .. +8].
    bf16x8 qf[QB][KS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        qf[qb][ks] = qrow[qb] < p.Lq
                         ? *reinterpret_cast<const bf16x8*>(qptr + (int64_t)qrow[qb] * p.qs[2] + ks * 16 + 8 * h)
                         : z;
      }

#pragma unroll
    for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dvb][qb][i] = 0.f;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      m_run[qb] = -INFINITY;
      l_run[qb] = 0.f;
    }

    // ---- global -> register -> LDS staging of one K/V tile ---------------------------------------------------
    u32x4 kst[T::K_PER_T], vst[T::V_PER_T];
    auto load_tile = [&](int t) {
      const int k0 = t * BN;
#pragma unroll
      for (int it = 0; it < T::K_PER_T; ++it) {
        int id = it * NT + tid, row = id / LK::CPR, c = id % LK::CPR;
        u32x4 z = {0, 0, 0, 0};
        kst[it] = (k0 + row < p.Lk)
                      ? *reinterpret_cast<const u32x4*>(kptr + (int64_t)(k0 + row) * p.ks[2] + c * 8)
                      : z;
      }
#pragma unroll
      for (int it = 0; it < T::V_PER_T; ++it) {
        int id = it * NT + tid, row = id / LV::CPR, c = id % LV::CPR;
        u32x4 z = {0, 0, 0, 0};
        vst[it] = (k0 + row < p.Lk)
                      ? *reinterpret_cast<const u32x4*>(vptr + (int64_t)(k0 + row) * p.vs[2] + c * 8)
                      : z;
      }
    };
    auto store_tile = [&](int buf) {
      unsigned char* kb_ = smem + buf * T::STAGE;
      unsigned char* vb_ = kb_ + T::KBYTES;
#pragma unroll
      for (int it = 0; it < T::K_PER_T; ++it) {
        int id = it * NT + tid, row = id / LK::CPR, c = id % LK::CPR;
        *reinterpret_cast<u32x4*>(kb_ + row * (DQK * 2) + LK::swz_k(row, c) * 16) = kst[it];
      }
#pragma unroll
      for (int it = 0; it < T::V_PER_T; ++it) {
        int id = it * NT + tid, row = id / LV::CPR, c = id % LV::CPR;
        *reinterpret_cast<u32x4*>(vb_ + row * (DV * 2) + LV::swz_v(row, c) * 16) = vst[it];
      }
    };
    // next tile >= t that is non-empty for at least one wave, or t_end
    auto next_tile = [&](int t) {
      while (t < t_end && __builtin_amdgcn_readfirstlane((int)cls[t]) == 0) ++t;
      return t;
    };

    __syncthreads();  // previous branch (if any) is done with the LDS buffers
    int t = t_first;
    int buf = 0;
    if (t < t_end) {
      load_tile(t);
      store_tile(0);
    }
    __syncthreads();

    while (t < t_end) {
      const int tn = next_tile(t + 1);
      if (tn < t_end) load_tile(tn);

      const int tclass = (__builtin_amdgcn_readfirstlane((int)cls[t]) >> (2 * wave)) & 3;
      if (tclass != TILE_EMPTY) {
        const unsigned char* kb_ = smem + buf * T::STAGE;
        const unsigned char* vb_ = kb_ + T::KBYTES;
        const int k0 = t * BN;

        // ---- S^T = K . Q^T --------------------------------------------------------------------------------------
        f32x16 s[KB][QB];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kb][qb][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            const int row = kb * 32 + r;
            bf16x8 kf = *reinterpret_cast<const bf16x8*>(kb_ + row * (DQK * 2) + LK::swz_k(row, 2 * ks + h) * 16);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
              s[kb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qb][ks], s[kb][qb], 0, 0, 0);
          }

        // ---- score modifications; afterwards s is in log2 units when kMod -----------------------------------------
        // Register i of block (kb, qb) is key k0 + 32*kb + 8*(i/4) + 4*h + i%4 against query qrow[qb].
        if constexpr (kMod) {
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
              const int kbase = k0 + 32 * kb + 4 * h;
              const float rel0 = (float)(kbase - qrow[qb]);
              float bv[16];
              if constexpr (kBias) {
#pragma unroll
                for (int i = 0; i < 16; ++i) bv[i] = 0.f;
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                  if (p.bias[nb] == nullptr) continue;
                  const bf16_t* bp = p.bias[nb] + (int64_t)(batch / p.bdiv[nb]) * p.bs[nb][0] +
                                     (int64_t)head * p.bs[nb][1] +
                                     (int64_t)min(qrow[qb], p.Lq - 1) * p.bs[nb][2];
#pragma unroll
                  for (int g = 0; g < 4; ++g) {
                    const int key = kbase + 8 * g;
                    if (p.bias_vec[nb] && key + 3 < p.Lk) {
                      bf16x4 b4 = *reinterpret_cast<const bf16x4*>(bp + key);
#pragma unroll
                      for (int e = 0; e < 4; ++e) bv[4 * g + e] += (float)b4[e];
                    } else {
#pragma unroll
                      for (int e = 0; e < 4; ++e)
                        if (key + e < p.Lk) bv[4 * g + e] += (float)bp[(int64_t)(key + e) * p.bs[nb][3]];
                    }
                  }
                }
              }
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                float x = s[kb][qb][i];
                float tl2;
                if constexpr (kSoftcap) {
                  float e = fast_exp2(x * cap_k1);
                  float rc = fast_rcp(e + 1.0f);
                  tl2 = __builtin_fmaf(rc, -2.0f * cap_c, cap_c);
                } else {
                  tl2 = x * p.scale_log2;
                }
                if constexpr (kAlibi) tl2 = __builtin_fmaf(slope_l2, rel0 + (float)(8 * (i / 4) + (i % 4)), tl2);
                if constexpr (kBias) tl2 = __builtin_fmaf(bv[i], 1.4426950408889634f, tl2);
                s[kb][qb][i] = tl2;
              }
            }
        }

        // ---- element mask on partial tiles ------------------------------------------------------------------------
        if (tclass == TILE_PARTIAL) {
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            int64_t kdoc[16];
            if constexpr (kDoc) {
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                int key = k0 + 32 * kb + 8 * (i / 4) + 4 * h + (i % 4);
                kdoc[i] = key < p.Lk ? p.doc_ids[(int64_t)batch * p.doc_stride + key] : 0;
              }
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const int key = k0 + 32 * kb + 8 * (i / 4) + 4 * h + (i % 4);
                bool ok = key < p.Lk && attend_positional(p.mask_kind, qrow[qb], key, p.window, p.prefix);
                if constexpr (kDoc) ok = ok && (kdoc[i] == qdoc[qb]);
                s[kb][qb][i] = ok ? s[kb][qb][i] : -INFINITY;
              }
          }
        }

        if constexpr (kDump) {
          if (br == 0) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
              for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                  const int key = k0 + 32 * kb + 8 * (i / 4) + 4 * h + (i % 4);
                  if (qrow[qb] < p.Lq && key < p.Lk && s[kb][qb][i] != -INFINITY)
                    p.dump[(((int64_t)batch * p.Hq + head) * p.Lq + qrow[qb]) * p.Lk + key] = 1;
                }
          }
        }

        // ---- online softmax ---------------------------------------------------------------------------------------
        const float c2 = kMod ? 1.0f : p.scale_log2;  // s * c2 is the logit in log2 units
        bf16x8 pf[QB][2 * KB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          float mx = -INFINITY;
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = __builtin_fmaxf(mx, s[kb][qb][i]);
          mx = xhalf_max(mx);
          const float m_new = __builtin_fmaxf(m_run[qb], mx);
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // row fully masked so far
          const float alpha = fast_exp2((m_run[qb] - m_use) * c2);
          const float mc = m_use * c2;
          m_run[qb] = m_new;
          float rs = 0.f;
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            float pv[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              pv[i] = fast_exp2(__builtin_fmaf(s[kb][qb][i], c2, -mc));
              rs += pv[i];
            }
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int e = 0; e < 8; ++e) pf[qb][2 * kb + j][e] = (bf16_t)pv[8 * j + e];
          }
          l_run[qb] = l_run[qb] * alpha + rs;
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[dvb][qb][i] *= alpha;
        }

        // ---- O^T += V^T . P^T ----------------------------------------------------------------------------------------
        // A operand slot j of lane (r, h) for 16-key chunk c is key 16c + 8*(j/4) + 4h + j%4, matching pf above.
#pragma unroll
        for (int c = 0; c < 2 * KB; ++c)
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb) {
            bf16x8 vf;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              // transposing read: within each 16-lane group, lane i supplies row (key) i/4, 4 columns at 4*(i%4),
              // and receives column i of the 4 rows.
              const int i16 = lane % 16, g = (lane / 16) % 2;
              const int row = 16 * c + 8 * j + 4 * h + i16 / 4;
              const int col = dvb * 32 + g * 16 + 4 * (i16 % 4);
              const unsigned char* ap = vb_ + row * (DV * 2) + LV::swz_v(row, col / 8) * 16 + (col % 8) * 2;
              typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
              s16x4 t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ap));
              bf16x4 b4 = __builtin_bit_cast(bf16x4, t4);
#pragma unroll
              for (int e = 0; e < 4; ++e) vf[4 * j + e] = b4[e];
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
              oacc[dvb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qb][c], oacc[dvb][qb], 0, 0, 0);
          }
      }

      if (tn < t_end) store_tile(buf ^ 1);
      __syncthreads();
      t = tn;
      buf ^= 1;
    }

    // ---- normalise this branch ---------------------------------------------------------------------------------
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float l = xhalf_sum(l_run[qb]);
      const float inv = l > 0.f ? 1.0f / l : 0.f;  // a row that attends nothing yields zeros
      if constexpr (kDiff) {
        if (br == 0) {
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
            for (int i = 0; i < 16; ++i) ofin[dvb][qb][i] = oacc[dvb][qb][i] * inv;
        } else {
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[dvb][qb][i] = ofin[dvb][qb][i] - p.lambda * (oacc[dvb][qb][i] * inv);
        }
      } else {
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[dvb][qb][i] *= inv;
      }
    }
  }

  // ---- epilogue: O^T register i of block (dvb, qb) is out[q = qrow[qb]][dv = 32*dvb + 8*(i/4) + 4h + i%4] ----------
  bf16_t* optr = p.o + (int64_t)batch * p.os[0] + (int64_t)head * p.os[1];
  const bf16_t* gptr = (kGate && p.gate) ? p.gate + (int64_t)batch * p.gs[0] + (int64_t)head * p.gs[1] : nullptr;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    if (qrow[qb] >= p.Lq) continue;
#pragma unroll
    for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int dv = 32 * dvb + 8 * g + 4 * h;
        bf16x4 o4;
        if (kGate && gptr) {
          bf16x4 g4 = *reinterpret_cast<const bf16x4*>(gptr + (int64_t)qrow[qb] * p.gs[2] + dv);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float sg = fast_rcp(1.0f + fast_exp2(-1.4426950408889634f * (float)g4[e]));
            o4[e] = (bf16_t)(oacc[dvb][qb][4 * g + e] * sg);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = (bf16_t)oacc[dvb][qb][4 * g + e];
        }
        *reinterpret_cast<bf16x4*>(optr + (int64_t)qrow[qb] * p.os[2] + dv) = o4;
      }
  }
}

}  // namespace fl
