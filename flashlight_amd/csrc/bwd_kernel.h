// Backward of the fused attention forward for gfx950: dQ, dK, dV from dO, the forward's inputs and its row statistics.
//
// The reference is forward-only (its FLOP helper models a backward, benchmarks/_utils.py:16-21, but no kernel exists);
// the arithmetic is the textbook one for softmax attention with recomputation:
//   P = exp2(S2 - LSE2),  dP = dO V^T,  dS = P o (dP - Delta) * d(score)/d(qk),  dQ = dS K,  dK = dS^T Q,  dV = P^T dO
// with S2 the modified logits in log2 units, LSE2 the forward's log2-sum-exp2 per row and Delta = rowsum(dO o O).
//
// One kernel template, two roles, no atomics:
//   ROLE_DQ   a workgroup owns 128 query rows of one head and streams the key tiles they attend;
//   ROLE_DKV  a workgroup owns 128 keys of one key/value head and streams the query tiles (of every query head of the
//             group) that attend them.
// In both roles a lane owns one *owner* position (the column of every accumulator it holds) and its registers run over
// the streamed positions, because every product is issued with the streamed tile as the A operand:
//   X1 = T1 . O1^T   (ROLE_DQ: K.Q^T = S^T;   ROLE_DKV: Q.K^T = S)       v_mfma_f32_32x32x16_bf16
//   X2 = T2 . O2^T   (ROLE_DQ: V.dO^T = dP^T; ROLE_DKV: dO.V^T = dP)
//   acc1 += T1^T . dS  (ROLE_DQ: dQ^T;  ROLE_DKV: dK^T),  ROLE_DKV also acc2 += T2^T . P  (dV^T)
// so the fp32 layout of X1/X2 is the bf16 B-operand layout of the accumulating products (as in the forward kernel) and
// P, dS never leave registers.  T1/T2 are staged in LDS by global_load_lds transfers, two slots, one barrier per tile;
// T^T operands come from the same tiles through the transposing LDS read.
#pragma once
#include "fwd_kernel.h"

namespace fl {

enum : int { ROLE_DQ = 0, ROLE_DKV = 1 };

struct BParams {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  const bf16_t* o;
  const bf16_t* dout;
  const float* lse;    // [B, Hq, Lq], log2 units; +inf for a row that attends nothing
  float* delta;        // [B, Hq, Lq] scratch: minus rowsum(dO o O)
  bf16_t* dq;
  bf16_t* dk;
  bf16_t* dv;
  int64_t qs[3], ks[3], vs[3], os[3], dos[3], dqs[3], dks[3], dvs[3];  // element strides: batch, head, seq
  int32_t B, Hq, Hkv, Lq, Lk, group;
  float scale, scale_log2;
  int32_t mask_kind, window, prefix;
  int32_t dmin, dmax, pfx;  // attend iff key < Lk && ((dmin <= key - q <= dmax) || key < pfx)
  const int64_t* doc_ids;
  int64_t doc_stride;
  const int64_t* doc_table;  // [B][ceil(L / kDocBlock)][2] = (min, max), as in the forward
  int32_t doc_blocks;
  int32_t alibi_heads;
  float softcap;
  uint32_t drop_thr;      // as in KParams: 0 = no dropout
  uint32_t drop_seed[2];
  float drop_rescale;
  // Bias operands (F_BIAS), addressed as in the forward: element (batch / bdiv, head, query, key) through bbs, 16-bit
  // elements of the call's type or fp32.  They are read from global memory where they are used.
  const void* bias[2];
  int64_t bbs[2][4];
  int32_t bdiv[2];
  int32_t bias_f32[2];
  float* dscores;  // optional [B, Hq, Lq, Lk]: d(loss) / d(score), written by the dQ kernel for the tiles it visits
};

// delta[b, h, q] = -sum_d dO[b, h, q, d] * O[b, h, q, d]; one row per group of DV / 8 lanes.
template <int DV, class E>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const BParams p) {
  typedef E ex8 __attribute__((ext_vector_type(8)));
  constexpr int LPR = DV / 8;  // lanes per row, 16 bytes each
  const int64_t rows = (int64_t)p.B * p.Hq * p.Lq;
  const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
  const int c = threadIdx.x % LPR;
  float s = 0.f;
  if (row < rows) {
    const int q = (int)(row % p.Lq), h = (int)((row / p.Lq) % p.Hq), b = (int)(row / ((int64_t)p.Lq * p.Hq));
    const ex8 a = *reinterpret_cast<const ex8*>(p.dout + b * p.dos[0] + h * p.dos[1] + q * p.dos[2] + 8 * c);
    const ex8 o = *reinterpret_cast<const ex8*>(p.o + b * p.os[0] + h * p.os[1] + q * p.os[2] + 8 * c);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)o[e];
  }
#pragma unroll
  for (int d = 1; d < LPR; d *= 2) s += __shfl_xor(s, d);
  if (row < rows && c == 0) p.delta[row] = -s;  // stored negated: the consumers add it (or start dP's accumulators from it)
}

template <int D_, int ROLE_, uint32_t FEAT_, class Elem_ = bf16_t>
struct BwdTraits {
  using Elem = Elem_;  // element type of q, k, v, o, dout and the gradients: bf16_t or f16_t
  static constexpr int D = D_, ROLE = ROLE_;
  static constexpr uint32_t FEAT = FEAT_;
  static constexpr int OWN = 128;                          // owner positions per workgroup: 4 waves x 32
  // ROLE_DKV at D = 128 holds 128 accumulator registers per lane; to still run two waves per SIMD its workgroup has
  // 8 waves, two per owner block, which take the two halves of every streamed tile and add up their partial sums
  // through LDS at the end (one workgroup per CU, 128 KB of LDS).
  static constexpr int QH = (ROLE == ROLE_DKV && D_ > 64) ? 2 : 1;   // waves per owner block
  static constexpr int NW = 4 * QH, NT = 64 * NW;
  static constexpr int TB = (D_ <= 64) ? 2 : 1;  // 32-position blocks per wave and step (register budget)
  static constexpr int BT = 32 * TB * QH;                  // streamed positions per step
  static constexpr int KS = D / 16, DB = D / 32;
  static constexpr int TBYTES = BT * D * 2;                // one streamed tile
  static constexpr int T_PER_T = TBYTES / (NT * 16);       // 16-byte transfers per thread per tile
  static_assert(TBYTES % (NT * 16) == 0, "streamed tile must divide evenly over the threads");
  static constexpr int OBYTES = (ROLE == ROLE_DKV) ? OWN * D * 2 : 0;  // owner tile kept in LDS (ROLE_DKV: K and V)
  static constexpr int O_PER_T = OBYTES / (NT * 16);
  static_assert(OBYTES % (NT * 16) == 0, "owner tile must divide evenly over the threads");
  // ROLE_DKV also stages the streamed rows' statistics (LSE and Delta, fp32) with every tile: 1 KiB each per slot
  static constexpr int SBYTES = (ROLE == ROLE_DKV) ? 1024 : 0;
  static constexpr int T1_OFF = 0, T2_OFF = 2 * TBYTES, O1_OFF = 4 * TBYTES, O2_OFF = O1_OFF + OBYTES,
                       S1_OFF = O2_OFF + OBYTES, S2_OFF = S1_OFF + 2 * SBYTES;
  static constexpr int LDS_BYTES = S2_OFF + 2 * SBYTES;
  static_assert(QH == 1 || LDS_BYTES >= 4 * 64 * 64 * 4, "the partial sums of one accumulator set must fit in LDS");
  static constexpr int WAVES_PER_EU = 2;
  static constexpr bool WIDE_X2 = D_ > 64;                      // dP's fp32 tile declared next to S's
  static constexpr bool EARLY_X2 = ROLE == ROLE_DQ && WIDE_X2;  // and its MFMAs issued right after those of S
};

template <bool FIRST, class A>
__device__ __forceinline__ A& pick(A& a, A& b) {
  if constexpr (FIRST) return a; else return b;
}

template <class T>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::WAVES_PER_EU, T::WAVES_PER_EU)))
void bwd_kernel(const BParams p) {
  constexpr int D = T::D, ROLE = T::ROLE, TB = T::TB, BT = T::BT, KS = T::KS, DB = T::DB, NT = T::NT;
  constexpr uint32_t FEAT = T::FEAT;
  constexpr bool kAlibi = FEAT & F_ALIBI, kSoftcap = FEAT & F_SOFTCAP, kDoc = FEAT & F_DOC, kBias = FEAT & F_BIAS;
  constexpr bool kDQ = ROLE == ROLE_DQ;
  using E = typename T::Elem;  // pointers in BParams are typed bf16_t whatever E is: 16 opaque bits
  typedef E ex8 __attribute__((ext_vector_type(8)));
  typedef E ex4 __attribute__((ext_vector_type(4)));
  constexpr bool kDrop = FEAT & F_DROPOUT;
  constexpr float kLog2e = 1.4426950408889634f;
  using L = TileLayout<D>;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int r = lane % 32, h = lane / 32;
  const int ow = wave % 4;       // owner block of this wave
  const int qh = wave / 4;       // which part of every streamed tile this wave takes (0 unless QH == 2)

  // workgroup -> (batch, owner head, owner tile).  All owner tiles of one head stream the same tensors, so they should
  // run at the same time on one XCD (its L2 then serves all but the first read): consecutive workgroup ids land on
  // different XCDs, hence ids are regrouped to give every XCD a contiguous run of (batch, head) pairs, head by head.
  // Under causal-like masks the work of a tile grows with the query position (ROLE_DQ) or shrinks with the key position
  // (ROLE_DKV): heads are taken four at a time and their tiles dealt longest first, so the grid drains on short ones.
  const int n_own = kDQ ? (p.Lq + T::OWN - 1) / T::OWN : (p.Lk + T::OWN - 1) / T::OWN;
  const int oh = kDQ ? p.Hq : p.Hkv;
  int ot, bh;
  {
    const int nbh = p.B * oh;
    int i = blockIdx.x, run = nbh, base = 0;
    if (nbh % 8 == 0) {
      run = nbh / 8;
      base = (i % 8) * run;
      i /= 8;
    }
    const int G = (p.mask_kind == MASK_CAUSAL || p.mask_kind == MASK_PREFIX || p.mask_kind == MASK_DOC_CAUSAL) ? 4 : 1;
    const int g = i / (G * n_own), rem = i % (G * n_own);
    const int gg = min(G, run - G * g);
    const int rank = rem / gg;  // 0 = longest under a causal-like mask
    bh = base + G * g + rem % gg;
    ot = kDQ ? n_own - 1 - rank : rank;
  }
  const int ohead = bh % oh, batch = bh / oh;
  const int o0 = ot * T::OWN;               // first owner position of the workgroup
  const int o1 = min(o0 + T::OWN, kDQ ? p.Lq : p.Lk);
  const int opos = o0 + ow * 32 + r;        // this lane's owner position (a query row or a key)
  const int olen = kDQ ? p.Lq : p.Lk;
  const int slen = kDQ ? p.Lk : p.Lq;       // streamed sequence length
  const int kvh = kDQ ? ohead / p.group : ohead;

  // ---- streamed tile range [t_lo, t_hi] for the workgroup's owner range [o0, o1) under the positional mask ----------
  int t_lo = 0, t_hi = (slen + BT - 1) / BT - 1;
  {
    const bool causal_like = p.mask_kind == MASK_CAUSAL || p.mask_kind == MASK_SLIDING || p.mask_kind == MASK_DOC_CAUSAL;
    if (kDQ) {  // keys attended by queries [o0, o1)
      if (causal_like) t_hi = min(t_hi, (o1 - 1) / BT);
      if (p.mask_kind == MASK_PREFIX) t_hi = min(t_hi, (max(o1, p.prefix) - 1) / BT);
      if (p.mask_kind == MASK_SLIDING) t_lo = max(0, o0 - p.window) / BT;
    } else {    // queries that attend keys [o0, o1)
      if (causal_like) t_lo = o0 / BT;
      if (p.mask_kind == MASK_PREFIX && o0 >= p.prefix) t_lo = o0 / BT;
      if (p.mask_kind == MASK_SLIDING) t_hi = min(t_hi, (int)min((int64_t)o1 - 1 + p.window, (int64_t)slen - 1) / BT);
    }
  }
  const int n_tiles = t_hi >= t_lo ? t_hi - t_lo + 1 : 0;
  const int n_heads = kDQ ? 1 : p.group;   // ROLE_DKV walks the query heads of its group
  const int n_steps = n_tiles * n_heads;

  // ---- per-lane constants ---------------------------------------------------------------------------------------------
  float cap_k1 = 0.f, cap_c = 0.f;
  bool cap_on = false;  // kernels compiled with the soft-cap also serve calls without one
  if constexpr (kSoftcap) {
    cap_on = p.softcap > 0.f;
    cap_k1 = cap_on ? p.scale / p.softcap * 2.0f * kLog2e : 0.f;
    cap_c = p.softcap * kLog2e;
  }
  int64_t odoc = 0;
  if constexpr (kDoc) odoc = p.doc_ids[(int64_t)batch * p.doc_stride + min(opos, olen - 1)];
  int64_t own_mn = 0, own_mx = 0;
  if constexpr (kDoc) doc_range(p.doc_table + (int64_t)batch * p.doc_blocks * 2, o0, o1, own_mn, own_mx);

  // ---- owner operands ---------------------------------------------------------------------------------------------------
  // ROLE_DQ: Q and dO fragments of this lane's query row live in registers (B operands), with its LSE and Delta.
  // ROLE_DKV: the workgroup's K and V rows are staged in LDS once and read as B operands where they are used.
  ex8 o1f[kDQ ? KS : 1], o2f[kDQ ? KS : 1];
  float lse_o = 0.f, delta_o = 0.f;  // delta_o: minus this row's rowsum(dO o O)
  const bf16_t* kptr = p.k + (int64_t)batch * p.ks[0] + (int64_t)kvh * p.ks[1];
  const bf16_t* vptr = p.v + (int64_t)batch * p.vs[0] + (int64_t)kvh * p.vs[1];
  if constexpr (kDQ) {
    const int qr = min(opos, p.Lq - 1);
    const bf16_t* qp = p.q + (int64_t)batch * p.qs[0] + (int64_t)ohead * p.qs[1] + (int64_t)qr * p.qs[2];
    const bf16_t* dp = p.dout + (int64_t)batch * p.dos[0] + (int64_t)ohead * p.dos[1] + (int64_t)qr * p.dos[2];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      o1f[ks] = *reinterpret_cast<const ex8*>(qp + ks * 16 + 8 * h);
      o2f[ks] = *reinterpret_cast<const ex8*>(dp + ks * 16 + 8 * h);
    }
    const int64_t row = ((int64_t)batch * p.Hq + ohead) * p.Lq + qr;
    lse_o = p.lse[row];
    delta_o = p.delta[row];
  }

  // ---- global -> LDS transfers of a [rows][D] tile into its swizzled image ---------------------------------------------------
  // lane l of a 1 KiB transfer writes LDS bytes [16 l, 16 l + 16); it fetches the logical chunk that the swizzle maps
  // there.  Rows past `valid` repeat the last valid row (their contributions are masked).
  auto load_tile = [&](const bf16_t* row0, int64_t stride, int valid, unsigned lds_off, int n_per_t) FL_INLINE {
    const uint64_t base = uniform_ptr(row0);
    const unsigned lds0 = (unsigned)(uintptr_t)smem + lds_off + wave * 1024;
    for (int it = 0; it < n_per_t; ++it) {
      const int id = it * NT + tid, row = id / L::CPR, pc = id % L::CPR;
      const unsigned off = (unsigned)(min(row, valid - 1) * (int)stride + L::swz_kv(row, pc) * 8) * 2u;
      dma16(base, off, lds0 + it * NT * 16);
    }
  };
  // streamed step s -> (query head of the group, tile).  ROLE_DKV: the statistics of the streamed rows (LSE, Delta) ride
  // the tile transfers into LDS, 4 bytes per lane, so that the loop holds no ordinary global load: the wait such a load
  // needs would also wait for the tile transfers that are in flight for the next step.
  auto step_head = [&](int s) FL_INLINE { return kDQ ? ohead : kvh * p.group + s / n_tiles; };
  auto step_tile = [&](int s) FL_INLINE { return t_lo + (kDQ ? s : s % n_tiles); };
  auto load_step = [&](int s, int slot) FL_INLINE {
    const int t0 = step_tile(s) * BT, valid = min(BT, slen - t0);
    if constexpr (kDQ) {
      load_tile(kptr + (int64_t)t0 * p.ks[2], p.ks[2], valid, T::T1_OFF + slot * T::TBYTES, T::T_PER_T);
      load_tile(vptr + (int64_t)t0 * p.vs[2], p.vs[2], valid, T::T2_OFF + slot * T::TBYTES, T::T_PER_T);
    } else {
      const int hd = step_head(s);
      load_tile(p.q + (int64_t)batch * p.qs[0] + (int64_t)hd * p.qs[1] + (int64_t)t0 * p.qs[2], p.qs[2], valid,
                T::T1_OFF + slot * T::TBYTES, T::T_PER_T);
      load_tile(p.dout + (int64_t)batch * p.dos[0] + (int64_t)hd * p.dos[1] + (int64_t)t0 * p.dos[2], p.dos[2], valid,
                T::T2_OFF + slot * T::TBYTES, T::T_PER_T);
      if (wave == 0) {
        // one wave brings both arrays (every wave waits for all of its own transfers before the barrier, so the counts
        // need not match).  Lane l fetches row t0 + l; lanes past the end of the tile or of the sequence repeat the last
        // valid row (those rows are masked).
        static_assert(BT <= 64, "one lane per streamed row");
        const int64_t row0 = ((int64_t)batch * p.Hq + hd) * p.Lq + t0;
        const unsigned off = (unsigned)min(lane, valid - 1) * 4u;
        dma4(uniform_ptr(p.lse + row0), off, (unsigned)(uintptr_t)smem + T::S1_OFF + slot * T::SBYTES);
        dma4(uniform_ptr(p.delta + row0), off, (unsigned)(uintptr_t)smem + T::S2_OFF + slot * T::SBYTES);
      }
    }
  };

  // ---- LDS operand reads --------------------------------------------------------------------------------------------------
  // row-wise: 8 consecutive elements [row][16 ks + 8 h, +8) (A operand of X1/X2 from a streamed tile, or B operand from
  // an owner tile)
  auto frag_row = [&](unsigned tile_off, int row, int ks) FL_INLINE -> ex8 {
    return *reinterpret_cast<const ex8*>(smem + tile_off + row * (D * 2) + L::swz_kv(row, 2 * ks + h) * 16);
  };
  // transposing: A operand of the accumulating products for 16-position chunk c and column block db; slot j of lane
  // (r, h) is streamed position 16 c + 8 (j / 4) + 4 h + j % 4, the order in which the weights are packed
  auto frag_tr = [&](unsigned tile_off, int c, int db) FL_INLINE -> ex8 {
    ex8 f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i16 = lane % 16, g = (lane / 16) % 2;
      const int row = 16 * c + 8 * j + 4 * h + i16 / 4;
      const int col = db * 32 + g * 16 + 4 * (i16 % 4);
      const unsigned char* ap = smem + tile_off + row * (D * 2) + L::swz_kv(row, col / 8) * 16 + (col % 8) * 2;
      typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
      const s16x4 t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ap));
      const ex4 b4 = __builtin_bit_cast(ex4, t4);
#pragma unroll
      for (int e = 0; e < 4; ++e) f[4 * j + e] = b4[e];
    }
    return f;
  };

  f32x16 acc1[DB], acc2[kDQ ? 1 : DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc1[db][i] = 0.f;
  if constexpr (!kDQ) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc2[db][i] = 0.f;
  }

  if (n_steps > 0) {
    if constexpr (!kDQ) {
      const int valid = o1 - o0;
      load_tile(kptr + (int64_t)o0 * p.ks[2], p.ks[2], valid, T::O1_OFF, T::O_PER_T);
      load_tile(vptr + (int64_t)o0 * p.vs[2], p.vs[2], valid, T::O2_OFF, T::O_PER_T);
    }
  }

  // Workgroup-level class of a step: nothing of its tile is attended by the workgroup's owner range (`skip`: document
  // ranges apart; positional emptiness inside [t_lo, t_hi] only occurs for a prefix-LM mask), everything is (`full`),
  // or every position of the tile and of the owner range carries one and the same document id (`doc_uniform`).
  // Steps that are skipped are never transferred: the loop goes from one live step to the next (under a document mask
  // most steps of the range are dead).
  auto classify_step = [&](int s, bool& full, bool& doc_uniform) FL_INLINE -> bool {
    const int t0 = step_tile(s) * BT;
    const int s1 = min(t0 + BT, slen);
    const int qa = kDQ ? o0 : t0, qb_ = kDQ ? o1 : s1, ka = kDQ ? t0 : o0, kb_ = kDQ ? s1 : o1;
    const int cls = classify_positional(p.mask_kind, qa, qb_, ka, kb_, p.window, p.prefix);
    bool skip = cls == TILE_EMPTY;
    // every pair of the step attended: the positional mask holds everywhere and both ranges lie inside the sequences
    full = cls == TILE_FULL && t0 + BT <= slen && o0 + T::OWN <= olen;
    doc_uniform = false;
    if constexpr (kDoc) {
      int64_t mn, mx;
      doc_range(p.doc_table + (int64_t)batch * p.doc_blocks * 2, t0, s1, mn, mx);
      skip = skip || mx < own_mn || mn > own_mx;
      doc_uniform = mn == mx && own_mn == own_mx && mn == own_mn;
      full = full && doc_uniform;
    }
    return skip;
  };
  // Sum of the bias operands at (query, key) of head `hd` (positions inside the sequences)
  auto bias_at = [&](int qpos, int kpos, int hd) FL_INLINE -> float {
    float b = 0.f;
    if constexpr (kBias) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        if (p.bias[nb] == nullptr) continue;
        const int64_t off = (int64_t)(batch / p.bdiv[nb]) * p.bbs[nb][0] + (int64_t)hd * p.bbs[nb][1] +
                            (int64_t)qpos * p.bbs[nb][2] + (int64_t)kpos * p.bbs[nb][3];
        b += p.bias_f32[nb] ? static_cast<const float*>(p.bias[nb])[off] : (float)static_cast<const E*>(p.bias[nb])[off];
      }
    }
    return b;
  };
  // One step: the tile in ring slot `slot` against the owner operands.
  auto run_step = [&](int s, int slot, bool full, bool doc_uniform) FL_INLINE {
    const int t0 = step_tile(s) * BT;
    const int shead = step_head(s);  // the query head of this step
    {
      const unsigned t1 = T::T1_OFF + slot * T::TBYTES, t2 = T::T2_OFF + slot * T::TBYTES;
      // ---- X1 = T1 . O1^T, then the weights; X2 = T2 . O2^T, then dS (one after the other: the two fp32 tiles are
      // never live together, which is what lets 128 accumulator registers fit) ----------------------------------------------
      // register i of block sb is streamed position t0 + 32 (qh TB + sb) + 8 (i / 4) + 4 h + i % 4
      float slope_l2 = 0.f;
      if constexpr (kAlibi)
        slope_l2 = p.alibi_heads > 0 ? exp2f(-8.0f * (float)(shead + 1) / (float)p.alibi_heads) * kLog2e : 0.f;
      // 4 consecutive streamed rows of a staged per-row fp32 array
      auto rows4 = [&](unsigned staged_off, int q4) FL_INLINE -> f32x4 {
        return *reinterpret_cast<const f32x4*>(smem + staged_off + slot * T::SBYTES + (q4 - t0) * 4);
      };
      // X2 = T2 . O2^T (dP).  At D = 128 its fp32 tile is declared out here, next to X1's, and (ROLE_DQ) its MFMAs are issued
      // right after X1's, before the weights' vector work; at D = 64 it lives in the block that consumes it.  Both choices
      // are measured: the first is 15 % faster at D = 128 and 1-2 % slower at D = 64.
      f32x16 x2_wide[TB];
      // dP's accumulators start from zero, or (ROLE_DKV without dropout) from the staged -Delta of their rows, which saves
      // the subtraction per score later
      constexpr bool kDeltaInit = !kDQ && !kDrop;
      auto init_x2 = [&](f32x16 (&x2)[TB]) FL_INLINE {
#pragma unroll
        for (int sb = 0; sb < TB; ++sb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 nd = {0.f, 0.f, 0.f, 0.f};
            if constexpr (kDeltaInit) nd = rows4(T::S2_OFF, t0 + 32 * (qh * TB + sb) + 4 * h + 8 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) x2[sb][4 * g + e] = nd[e];
          }
      };
      auto second_product = [&](f32x16 (&x2)[TB]) FL_INLINE {
        init_x2(x2);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          ex8 b2;
          if constexpr (kDQ) b2 = o2f[ks]; else b2 = frag_row(T::O2_OFF, ow * 32 + r, ks);
#pragma unroll
          for (int sb = 0; sb < TB; ++sb)
            x2[sb] = mfma32(frag_row(t2, (qh * TB + sb) * 32 + r, ks), b2, x2[sb]);
        }
      };
      ex8 pf[2 * TB], dsf[2 * TB];
      float pd[TB][16];  // weight times d(score) / d(qk * scale); with dropout its sign bit marks a dropped weight
      // dropout: the owner position's share of the hash argument (see drop_pair_hash); the streamed head changes from step
      // to step in ROLE_DKV
      uint32_t drop_o = 0;
      if constexpr (kDrop) {
        const uint32_t s0 = drop_head_seed(p.drop_seed[0], p.drop_seed[1], (uint32_t)(batch * p.Hq + shead));
        drop_o = s0 + (kDQ ? (uint32_t)opos * kDropQ : (uint32_t)(opos >> 1) * kDropK);
      }
      {
        f32x16 x1[TB];
#pragma unroll
        for (int sb = 0; sb < TB; ++sb)
#pragma unroll
          for (int i = 0; i < 16; ++i) x1[sb][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          ex8 b1;
          if constexpr (kDQ) b1 = o1f[ks]; else b1 = frag_row(T::O1_OFF, ow * 32 + r, ks);
#pragma unroll
          for (int sb = 0; sb < TB; ++sb)
            x1[sb] = mfma32(frag_row(t1, (qh * TB + sb) * 32 + r, ks), b1, x1[sb]);
        }
        // where the registers allow and it pays (measured), dP's MFMAs are issued before the weights' vector work
        if constexpr (T::EARLY_X2) second_product(x2_wide);
#pragma unroll
        for (int sb = 0; sb < TB; ++sb) {
          const int sbase = t0 + 32 * (qh * TB + sb) + 4 * h;  // streamed position of register 0
          // element predicate as an interval of the register offset `off` (8 (i / 4) + i % 4): lo <= off <= hi
          int lo, hi;
          if constexpr (kDQ) {
            // streamed = key, owner = query: key < Lk && (dmin <= key - q <= dmax || key < pfx)
            const int rel = sbase - opos;
            hi = min(p.Lk - sbase - 1, max(p.dmax - rel, p.pfx - sbase - 1));
            lo = p.dmin - rel;
          } else {
            // streamed = query, owner = key: q < Lq && (dmin <= key - q <= dmax || key < pfx), key = opos
            const int rel = opos - sbase;  // key - q at off = 0; key - q = rel - off
            hi = min(p.Lq - sbase - 1, opos < p.pfx ? (1 << 29) : rel - p.dmin);
            lo = opos < p.pfx ? -(1 << 29) : rel - p.dmax;
            if (opos >= p.Lk) hi = -(1 << 29);
          }
          float pv[16];
          // what does not depend on the register goes into one addend: minus the row's LSE, and the ALiBi term at
          // off = 0 (key - q = rel0 + off in ROLE_DQ, rel0 - off in ROLE_DKV), which leaves slope * off as one
          // multiply-add with a literal per score
          const float alibi0 = kAlibi ? slope_l2 * (float)(kDQ ? sbase - opos : opos - sbase) : 0.f;
          const float slope_off = kDQ ? slope_l2 : -slope_l2;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 lse4;
            if constexpr (!kDQ) lse4 = rows4(T::S1_OFF, sbase + 8 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int i = 4 * g + e, off = 8 * g + e;
              const float x = x1[sb][i];
              const float c0 = alibi0 - (kDQ ? lse_o : lse4[e]);
              float s2, dfac = 1.0f;  // logit in log2 units minus the LSE; d(score) / d(qk * scale)
              if constexpr (kSoftcap) {
                const float ex = fast_exp2(x * cap_k1);
                const float rc = fast_rcp(ex + 1.0f);
                const float th = __builtin_fmaf(rc, -2.0f, 1.0f);  // tanh(x * scale / cap)
                s2 = cap_on ? __builtin_fmaf(th, cap_c, c0) : __builtin_fmaf(x, p.scale_log2, c0);
                dfac = cap_on ? __builtin_fmaf(-th, th, 1.0f) : 1.0f;
              } else {
                s2 = __builtin_fmaf(x, p.scale_log2, c0);
              }
              if constexpr (kAlibi) s2 = __builtin_fmaf(slope_off, (float)off, s2);
              if constexpr (kBias) {
                const int sp = min(sbase + off, slen - 1), op = min(opos, olen - 1);
                s2 = __builtin_fmaf(bias_at(kDQ ? op : sp, kDQ ? sp : op, shead), kLog2e, s2);
              }
              float pw = fast_exp2(s2);
              if (!full) {  // workgroup-uniform
                bool ok = (off <= hi) & (off >= lo);
                if constexpr (kDoc) {
                  if (!doc_uniform) ok = ok & (p.doc_ids[(int64_t)batch * p.doc_stride + min(sbase + off, slen - 1)] == odoc);
                }
                pw = ok ? pw : 0.f;
              }
              pv[i] = pw;
              pd[sb][i] = kSoftcap ? pw * dfac : pw;
            }
          }
          if constexpr (kDrop) {
            // ROLE_DQ: registers (i, i + 1), i even, are the key pair (sbase + off) / 2 of this lane's query: one hash.
            // ROLE_DKV: register i is query sbase + off against this lane's key: its own hash, the key's half of it.
#pragma unroll
            for (int i = 0; i < 16; i += kDQ ? 2 : 1) {
              const int off = 8 * (i / 4) + i % 4;
              if constexpr (kDQ) {
                const uint32_t x = drop_pair_hash(drop_o + (uint32_t)((sbase + off) >> 1) * kDropK);
                const bool keep0 = (x & 0xFFFFu) >= p.drop_thr, keep1 = (x >> 16) >= p.drop_thr;
                pv[i] = keep0 ? pv[i] : 0.f;
                pv[i + 1] = keep1 ? pv[i + 1] : 0.f;
                pd[sb][i] = keep0 ? pd[sb][i] : -pd[sb][i];
                pd[sb][i + 1] = keep1 ? pd[sb][i + 1] : -pd[sb][i + 1];
              } else {
                const uint32_t x = drop_pair_hash(drop_o + (uint32_t)(sbase + off) * kDropQ);
                const bool keep = ((x >> (16 * (opos & 1))) & 0xFFFFu) >= p.drop_thr;
                pv[i] = keep ? pv[i] : 0.f;
                pd[sb][i] = keep ? pd[sb][i] : -pd[sb][i];
              }
            }
          }
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[2 * sb + j][e] = (E)pv[8 * j + e];
        }
      }
      {
        f32x16 x2_here[TB];
        f32x16 (&x2)[TB] = pick<T::WIDE_X2>(x2_wide, x2_here);
        if constexpr (!T::WIDE_X2) {
          init_x2(x2);
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            ex8 b2;
            if constexpr (kDQ) b2 = o2f[ks]; else b2 = frag_row(T::O2_OFF, ow * 32 + r, ks);
#pragma unroll
            for (int sb = 0; sb < TB; ++sb)
              x2[sb] = mfma32(frag_row(t2, (qh * TB + sb) * 32 + r, ks), b2, x2[sb]);
          }
        } else if constexpr (!T::EARLY_X2) {
          second_product(x2);
        }
#pragma unroll
        for (int sb = 0; sb < TB; ++sb) {
          const int sbase = t0 + 32 * (qh * TB + sb) + 4 * h;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 dl4 = {0.f, 0.f, 0.f, 0.f};  // minus Delta of the four rows, unless dP already started from it
            if constexpr (!kDQ && !kDeltaInit) dl4 = rows4(T::S2_OFF, sbase + 8 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int i = 4 * g + e;
              float ds;
              if constexpr (kDrop) {
                // d(loss) / d(weight) is dP / (1 - p) where the weight was kept and 0 where it was dropped
                const bool kept = __builtin_bit_cast(int, pd[sb][i]) >= 0;
                ds = __builtin_fabsf(pd[sb][i]) * ((kept ? x2[sb][i] * p.drop_rescale : 0.f) + (kDQ ? delta_o : dl4[e]));
              } else {
                ds = kDeltaInit ? pd[sb][i] * x2[sb][i] : pd[sb][i] * (x2[sb][i] + (kDQ ? delta_o : dl4[e]));
              }
              dsf[2 * sb + i / 8][i % 8] = (E)ds;
              if constexpr (kBias && kDQ) {
                // the gradient with respect to the score; with the soft-cap switched on ds carries d(cap) / d(qk * scale)
                // besides, which is not part of it: the host refuses dscores then
                const int key = sbase + 8 * g + e;
                if (p.dscores != nullptr && opos < p.Lq && key < p.Lk)
                  p.dscores[(((int64_t)batch * p.Hq + ohead) * p.Lq + opos) * p.Lk + key] = ds;
              }
            }
          }
        }
      }
      // ---- acc1 += T1^T . dS,  acc2 += T2^T . P -------------------------------------------------------------------------------
#pragma unroll
      for (int c = 0; c < 2 * TB; ++c)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          acc1[db] = mfma32(frag_tr(t1, 2 * TB * qh + c, db), dsf[c], acc1[db]);
          if constexpr (!kDQ)
            acc2[db] = mfma32(frag_tr(t2, 2 * TB * qh + c, db), pf[c], acc2[db]);
        }
    }
  };
  if constexpr (kDoc) {
    // (the class of a step is worked out before its transfers are issued: the table reads must not wait on them)
    auto next_live = [&](int s, bool& full, bool& doc_uniform) FL_INLINE -> int {
      while (s < n_steps && classify_step(s, full, doc_uniform)) ++s;
      return s;
    };
    bool full = false, doc_uniform = false;
    int s = next_live(0, full, doc_uniform);
    if (s < n_steps) load_step(s, 0);
    dma_wait<0>();
    for (int slot = 0; s < n_steps; slot ^= 1) {
      __syncthreads();  // publishes slot `slot` (every wave waited for its own transfers) and frees the other slot
      bool full_next = false, doc_uniform_next = false;
      const int s_next = next_live(s + 1, full_next, doc_uniform_next);
      if (s_next < n_steps) load_step(s_next, slot ^ 1);
      run_step(s, slot, full, doc_uniform);
      dma_wait<0>();
      s = s_next;
      full = full_next;
      doc_uniform = doc_uniform_next;
    }
  } else {
    // positional masks: every step of [t_lo, t_hi] is visited (a dead one only occurs under a prefix-LM mask)
    if (n_steps > 0) load_step(0, 0);
    dma_wait<0>();
    for (int s = 0; s < n_steps; ++s) {
      const int slot = s & 1;
      __syncthreads();  // publishes slot `slot` (every wave waited for its own transfers) and frees the other slot
      if (s + 1 < n_steps) load_step(s + 1, slot ^ 1);
      bool full, doc_uniform;
      if (!classify_step(s, full, doc_uniform)) run_step(s, slot, full, doc_uniform);
      dma_wait<0>();
    }
  }

  // ---- the waves of one owner block add up their partial sums: the second wave parks its accumulators in LDS (element
  // (register, lane) of owner block ow at float ((ow * 64 + register) * 64 + lane): consecutive lanes, no conflicts) ----
  if constexpr (T::QH == 2) {
    float* park = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int set = 0; set < 2; ++set) {
      __syncthreads();  // the tiles (set 0) or the previous set's sums (set 1) have been read
      if (qh == 1) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) park[((ow * 64 + db * 16 + i) * 64) + lane] = set == 0 ? acc1[db][i] : acc2[db][i];
      }
      __syncthreads();
      if (qh == 0) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float x = park[((ow * 64 + db * 16 + i) * 64) + lane];
            if (set == 0) acc1[db][i] += x; else acc2[db][i] += x;
          }
      }
    }
  }

  // ---- epilogue: register i of block db is column 32 db + 8 (i / 4) + 4 h + i % 4 of this lane's owner row ---------------
  if (opos < olen && qh == 0) {
    bf16_t* out1 = kDQ ? p.dq + (int64_t)batch * p.dqs[0] + (int64_t)ohead * p.dqs[1] + (int64_t)opos * p.dqs[2]
                       : p.dk + (int64_t)batch * p.dks[0] + (int64_t)ohead * p.dks[1] + (int64_t)opos * p.dks[2];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        ex4 o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) o4[e] = (E)(acc1[db][4 * g + e] * p.scale);
        *reinterpret_cast<ex4*>(out1 + 32 * db + 8 * g + 4 * h) = o4;
      }
    if constexpr (!kDQ) {
      bf16_t* out2 = p.dv + (int64_t)batch * p.dvs[0] + (int64_t)ohead * p.dvs[1] + (int64_t)opos * p.dvs[2];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          ex4 o4;
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = (E)(kDrop ? acc2[db][4 * g + e] * p.drop_rescale : acc2[db][4 * g + e]);
          *reinterpret_cast<ex4*>(out2 + 32 * db + 8 * g + 4 * h) = o4;
        }
    }
  }
}

}  // namespace fl
