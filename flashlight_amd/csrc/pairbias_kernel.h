// Attention with one dense bias that many batch entries share (the Evoformer's row attention: N_seq rows of an MSA
// attend over N_res residues, and every row adds the same pair bias [H, N_res, N_res]; reference
// attention_variants/evoformer.py:8-36), head dim 32 or 64, a few hundred keys; optionally a second bias that is one
// row of keys per batch entry, the same for every head and query (the mask bias [B, N_seq, 1, 1, N_res] of the
// reference's benchmark inputs, evoformer.py:45).
//
// The general forward (fwd_kernel.h) gives such a call one short-lived workgroup per (row, head, 128 queries): six key
// tiles, a bias tile staged next to every K/V tile, and eight or nine vector instructions per score against eight
// MFMAs per tile.  This kernel turns the loops inside out:
//   * a workgroup owns (head, 128 queries) and streams over the batch entries (MSA rows) of its chunk; the K/V tile
//     ring runs on across entries, the next entry's queries are fetched while this one is computed, so the latencies
//     that bound a six-tile workgroup are paid once per chunk;
//   * the bias of the workgroup's queries against ALL keys stays in registers for the whole chunk, already laid out as
//     MFMA B operands (8 consecutive keys of one query per lane and 16-key group);
//   * the matrix pipe, which idles at head dim 32, adds it: S^T += Sel . Bias^T with Sel the 32 x 16 selector that puts
//     key 16m + j on row j of the group, weighted 1/scale (in fp16 unless the element type holds it exactly: relative
//     error of the bias term at most 2^-12), so the accumulators hold qk + bias/scale and the weights are
//     exp2(scale * log2(e) * acc - ref): per score one multiply-add, one exponential, one addition for the row sum and
//     half a pack.
//   * the row bias takes the same road as a rank-one product: A = the row's values down the keys (two copies side by
//     side), B = the two terms of 1/scale across the queries; the row of the next entry rides into LDS with the
//     transfers of the current one.
// Infinite bias entries are clamped to the largest finite value when the fragments are loaded (0 * inf inside the
// selector product would poison the 15 other keys of the group); as an additive term that is the same mask.
#pragma once
#include "fwd_kernel.h"

namespace fl {

struct PParams {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  bf16_t* o;
  int64_t qs[3], ks[3], vs[3], os[3];  // element strides: batch, head, seq
  int32_t B, H, Lq, Lk;
  float scale;
  const bf16_t* bias;  // [B / bdiv][H][Lq][Lk], unit key stride
  int64_t bs[3];       // element strides: group, head, query
  int32_t bdiv;        // batch entries that share one bias slice
  const bf16_t* gate;  // optional, addressed like o
  int64_t gs[3];
  int32_t n_qtiles;   // ceil(Lq / 128)
  int32_t chunks;     // chunks per bias group
  int32_t chunk_len;  // batch entries per chunk (the last chunk of a group may be shorter)
  int32_t hgroup;     // heads whose workgroups are kept on one XCD (they share cache lines when heads are adjacent)
  int32_t n_units;    // (bias groups * chunks) * (H / hgroup)
  const bf16_t* rowb;  // optional second bias: one row of Lk values per batch entry, unit key stride
  int64_t rbs;         // its element stride between batch entries
};

// 16 bytes per lane from global memory into registers, and 16 bytes back, as asm: inside the streaming loop every
// vector-memory operation is issued by hand in a fixed order, because the waits there count operations
// (s_waitcnt vmcnt(N): at most N still outstanding, completion in issue order) and a compiler-issued access would not
// be in the count.  The loaded registers may be read only after the wait that covers them and a pin_loaded() on them.
__device__ __forceinline__ u32x4 load16_counted(uint64_t sbase, unsigned voff) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase));
  return v;
}
// (a store of more than 8 bytes still reads its data registers for two cycles after it has issued, and the compiler,
// which inserts that distance for its own stores, does not look into an asm: the idle cycles are part of it)
__device__ __forceinline__ void store16_counted(uint64_t sbase, unsigned voff, u32x4 data) {
  asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" ::"v"(voff), "v"(data), "s"(sbase));
}

template <class V>
__device__ __forceinline__ void pin_loaded(V& v) {
  asm volatile("" : "+v"(v));
}

template <int NKB_, bool GATE_, class Elem_, int D_ = 32, bool ROWB_ = false, bool EXACT_ = false>
struct PairBiasTraits {
  using Elem = Elem_;
  static constexpr int NKB = NKB_;       // 32-key blocks per row: Lk = 32 * NKB
  static constexpr bool GATE = GATE_;
  static constexpr bool ROWB = ROWB_;    // a row bias per batch entry besides the shared one
  // 1 / scale is exact in the element type (a power of two, say): the selector product runs in that type as it is
  static constexpr bool EXACT = EXACT_;
  static constexpr int D = D_, BN = 64, NW = 4, NT = 256, BM = 128;
  static constexpr int KS = D / 16;      // k-steps of the first product
  static constexpr int DVB = D / 32;     // 32-column blocks of the result
  static constexpr int NTI = NKB / 2;    // key tiles per batch entry
#ifdef FL_PB_NS64
  static constexpr int NS = D == 32 ? 6 : FL_PB_NS64;
#else
  static constexpr int NS = D == 32 ? 6 : 4;  // K/V tiles resident in LDS
#endif
  static constexpr int AHEAD = NS - 1;   // transfers run this many tiles ahead of their use
  // K fragments read from LDS one block ahead of the scores that use them (head dim 64 has no registers for that)
#ifdef FL_PB_KAHEAD
  static constexpr bool KAHEAD = FL_PB_KAHEAD;
#else
  static constexpr bool KAHEAD = D == 32;
#endif
  static_assert(D == 32 || D == 64, "head dim");
  static_assert(NKB % 2 == 0 && NTI >= 2, "whole tiles");
  static constexpr int TILE_BYTES = BN * D * 2;
  static constexpr int XPW = TILE_BYTES / (NW * 1024);  // 1 KiB wave transfers per wave and operand tile
  static constexpr int ROW_SLOT = 1024;                 // LDS bytes of one staged bias row (a whole wave transfer)
  static_assert(32 * NKB * 2 <= ROW_SLOT, "a bias row fits one wave transfer");
  // per wave two row slots: the current entry's row and the next one's
  static constexpr int K_OFF = 0, V_OFF = NS * TILE_BYTES, R_OFF = 2 * NS * TILE_BYTES;
  static constexpr int LDS_BYTES = R_OFF + (ROWB ? NW * 2 * ROW_SLOT : 0);
};

template <class T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void pairbias_kernel(const PParams p) {
  using E = typename T::Elem;
  typedef E ex8 __attribute__((ext_vector_type(8)));
  typedef E ex4 __attribute__((ext_vector_type(4)));
  typedef E ex2 __attribute__((ext_vector_type(2)));
  constexpr int NKB = T::NKB, NTI = T::NTI, NS = T::NS, D = T::D, BN = T::BN, KS = T::KS, DVB = T::DVB, XPW = T::XPW;
  constexpr bool kGate = T::GATE, kRowB = T::ROWB, kAheadK = T::KAHEAD;
  constexpr float kLog2e = 1.4426950408889634f;
  using LK = TileLayout<D>;
  using LV = TileLayout<D>;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // T::LDS_BYTES

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int r = lane % 32, h = lane / 32;

  // ---- workgroup -> (bias group, chunk of batch entries, head, query tile).  Consecutive workgroup ids land on
  // different XCDs; a unit = (chunk, group of adjacent heads) is kept on one XCD, all its query tiles together: they read
  // the same K/V, and adjacent heads share cache lines when the head axis is the second-fastest in memory.
  int fb0, n_items, head, qt, grp;
  {
    const int per_unit = p.hgroup * p.n_qtiles;
    const int x = blockIdx.x % 8, rest = blockIdx.x / 8;
    const int local = rest % per_unit, u = (rest / per_unit) * 8 + x;
    if (u >= p.n_units) return;  // (before any barrier)
    const int hg_count = p.H / p.hgroup;
    const int ct = u / hg_count, hg = u % hg_count;  // chunk over all groups, head group
    grp = ct / p.chunks;
    const int c = ct % p.chunks;
    head = hg * p.hgroup + local / p.n_qtiles;
    qt = local % p.n_qtiles;
    fb0 = grp * p.bdiv + c * p.chunk_len;
    n_items = min(p.chunk_len, p.bdiv - c * p.chunk_len);
  }
  const int qrow = min(qt * T::BM + wave * 32 + r, p.Lq - 1);  // rows past Lq repeat the last row (same values stored)

  // ---- the resident bias: B operands of the selector products, lane (r, h) holds bias[qrow][32 kb + 16 m + 8 h .. + 8].
  // The selector product has one term, 1 / scale times the bias, and runs in the type that holds 1 / scale best: the
  // element type when the value is exact in it (EXACT), fp16 otherwise (11 bits: the bias enters the logits with a
  // relative error of at most 2^-12; bf16's 8 bits would need a second product for the remainder).  bf16 bias values
  // are fp16 values as they stand up to 65504; larger ones (masks like -1e9) saturate there, which times 1 / scale is
  // still tens of thousands below any score.
  using SE = std::conditional_t<T::EXACT, E, f16_t>;
  typedef SE sx8 __attribute__((ext_vector_type(8)));
  sx8 bfrag[NKB][2];
  {
    const bf16_t* brow = p.bias + (int64_t)grp * p.bs[0] + (int64_t)head * p.bs[1] + (int64_t)qrow * p.bs[2];
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int m = 0; m < 2; ++m) {
        u32x4 raw = *reinterpret_cast<const u32x4*>(brow + 32 * kb + 16 * m + 8 * h);
        // +-inf -> +-largest finite, two elements per register: an element is infinite when its low 15 bits are
        // exactly the exponent mask (bf16 0x7F80, fp16 0x7C00)
        constexpr uint32_t kInf = std::is_same<E, f16_t>::value ? 0x7C00u : 0x7F80u;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t x = raw[w];
          const uint32_t lo_inf = ((x & 0x7FFFu) == kInf) ? 1u : 0u;
          const uint32_t hi_inf = (((x >> 16) & 0x7FFFu) == kInf) ? 0x10000u : 0u;
          raw[w] = x - lo_inf - hi_inf;
        }
        if constexpr (!std::is_same<SE, E>::value) {
          // bf16 pair -> fp16 pair (rounding toward zero: exact in range, the largest finite value beyond it)
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            const float lo = __builtin_bit_cast(float, raw[w] << 16), hi = __builtin_bit_cast(float, raw[w] & 0xFFFF0000u);
            raw[w] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
          }
        }
        bfrag[kb][m] = __builtin_bit_cast(sx8, raw);
      }
  }
  // selectors: A operand of group m puts key 16 m + j on row j; lane (r, h) holds Sel[key = r][j = 8 h .. 8 h + 7]
  sx8 sel[2];
  {
    const SE w = (SE)(1.0f / p.scale);
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int j = 0; j < 8; ++j) sel[m][j] = (r == 16 * m + 8 * h + j) ? w : (SE)0.0f;
  }
  // row bias: B operand of the rank-one product, lane (query r, h) holds rows 8 h .. 8 h + 7 of the 16: rows 0 and 1
  // carry the two terms of 1 / scale, the A operand has the row's value in columns 0 and 1
  ex8 rsel;
  uint32_t rkeep = 0;  // all ones in the lanes that hold columns 0 .. 7 of the A operand
  if constexpr (kRowB) {
    const float w = 1.0f / p.scale;
    const E w_hi = (E)w;
    const E w_lo = (E)(w - (float)w_hi);
#pragma unroll
    for (int j = 0; j < 8; ++j) rsel[j] = (E)0.0f;
    if (h == 0) {
      rsel[0] = w_hi;
      rsel[1] = w_lo;
      rkeep = 0xFFFFFFFFu;
    }
  }
  const float c2 = p.scale * kLog2e;  // acc * c2 = (qk * scale + bias) in log2 units

  // ---- addresses.  Per-lane byte offsets are constant; scalar bases move with the batch entry and the tile.
  // K/V tile = 64 rows x 2 D bytes = 4 XPW wave transfers of 1 KiB: wave w brings transfers w, w + 4, ...; lane l ->
  // (row, physical chunk); transfer j of a wave lies 64 / XPW rows (whole swizzle periods) below its transfer j - 1
  unsigned koff, voff;
  {
    const int id = wave * 64 + lane, row = id / LK::CPR, pc = id % LK::CPR;
    koff = (unsigned)(row * (int)p.ks[2] + LK::swz_k(row, pc) * 8) * 2u;
    voff = (unsigned)(row * (int)p.vs[2] + LV::swz_v(row, pc) * 8) * 2u;
  }
  const unsigned lds_k = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::K_OFF + wave * 1024);
  const unsigned lds_v = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::V_OFF + wave * 1024);
  const uint64_t kbase = uniform_ptr(p.k + (int64_t)head * p.ks[1]), vbase = uniform_ptr(p.v + (int64_t)head * p.vs[1]);
  const uint64_t qbase = uniform_ptr(p.q + (int64_t)head * p.qs[1]);
  const uint64_t obase = uniform_ptr(p.o + (int64_t)head * p.os[1]);
  const uint64_t gbase = kGate ? uniform_ptr(p.gate + (int64_t)head * p.gs[1]) : 0;
  const unsigned qoff = (unsigned)(qrow * (int)p.qs[2] + 8 * h) * 2u;  // + 32 bytes per k-step
  const unsigned ooff = (unsigned)(qrow * (int)p.os[2] + 8 * h) * 2u;  // + 32 bytes per group of 16 value columns
  const unsigned goff = kGate ? (unsigned)(qrow * (int)p.gs[2] + 8 * h) * 2u : 0u;  // 16-byte loads, see the epilogue
  // the row bias: every wave stages its own copy of the row (lane l brings 16 bytes; lanes past the row's end repeat
  // its start), slot (entry % 2) of the wave's two
  const uint64_t rbase = kRowB ? uniform_ptr(p.rowb) : 0;
  const unsigned roff = (unsigned)(lane % (NKB * 4)) * 16u;
  const unsigned lds_r = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::R_OFF + wave * 2 * T::ROW_SLOT);
  const unsigned k_step_bytes = __builtin_amdgcn_readfirstlane((unsigned)((64 / XPW) * (int)p.ks[2] * 2));
  const unsigned v_step_bytes = __builtin_amdgcn_readfirstlane((unsigned)((64 / XPW) * (int)p.vs[2] * 2));

  // tile j of the stream (entry j / NTI of the chunk, tile j % NTI of its keys; past the end the last entry again, so
  // that every step issues the same operations) -> ring slot j % NS
  auto issue_tile = [&](int item, int t, int slot) FL_INLINE {
    const int64_t fb = fb0 + min(item, n_items - 1);
    const uint64_t kb_ = kbase + (uint64_t)((fb * p.ks[0] + (int64_t)t * BN * p.ks[2]) * 2);
    const uint64_t vb_ = vbase + (uint64_t)((fb * p.vs[0] + (int64_t)t * BN * p.vs[2]) * 2);
#pragma unroll
    for (int j = 0; j < XPW; ++j) dma16(kb_ + (uint64_t)(j * k_step_bytes), koff, lds_k + slot * T::TILE_BYTES + j * 4096);
#pragma unroll
    for (int j = 0; j < XPW; ++j) dma16(vb_ + (uint64_t)(j * v_step_bytes), voff, lds_v + slot * T::TILE_BYTES + j * 4096);
  };
  auto issue_row = [&](int item) FL_INLINE {
    const int64_t fb = fb0 + min(item, n_items - 1);
    dma16(rbase + (uint64_t)(fb * p.rbs * 2), roff, lds_r + (item % 2) * T::ROW_SLOT);
  };
  // A operand of the row-bias product for block kb of entry `item`: the value of key 32 kb + r, twice, in the lanes
  // of the first half; infinite values clamped like the shared bias
  auto row_frag = [&](int item, int kb) FL_INLINE -> ex8 {
    const unsigned char* rp = smem + T::R_OFF + (wave * 2 + item % 2) * T::ROW_SLOT;
    uint32_t x = *reinterpret_cast<const uint16_t*>(rp + (32 * kb + r) * 2);
    constexpr uint32_t kInf = std::is_same<E, f16_t>::value ? 0x7C00u : 0x7F80u;
    x -= ((x & 0x7FFFu) == kInf) ? 1u : 0u;
    u32x4 raw = {(x | (x << 16)) & rkeep, 0u, 0u, 0u};
    return __builtin_bit_cast(ex8, raw);
  };

  // ---- K fragments (A operands of S^T = K . Q^T) of block b of the tile in ring slot `slot`
  auto k_frags = [&](ex8 (&kf)[KS], int slot, int b) FL_INLINE {
    const unsigned char* kt = smem + T::K_OFF + slot * T::TILE_BYTES;
    const int row = 32 * b + r;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      kf[ks] = *reinterpret_cast<const ex8*>(kt + row * (D * 2) + LK::swz_k(row, 2 * ks + h) * 16);
  };
  // ---- S^T block: K fragments as A operand, Q fragments as B; then the bias through the selectors
  auto scores = [&](f32x16& s, const ex8 (&kf)[KS], const ex8 (&qf)[KS], int kb, const ex8& rowf) FL_INLINE {
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s = mfma32(kf[ks], qf[ks], s);
#pragma unroll
    for (int m = 0; m < 2; ++m) s = mfma32(sel[m], bfrag[kb][m], s);
    if constexpr (kRowB) s = mfma32(rowf, rsel, s);
  };
  // A operand of O^T += V^T . P^T for 16-key chunk c of the tile (the transposing LDS read of the general kernel)
  auto v_frag = [&](int slot, int c, int dvb) FL_INLINE -> ex8 {
    const unsigned char* vt = smem + T::V_OFF + slot * T::TILE_BYTES;
    ex8 vf;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i16 = lane % 16, g = (lane / 16) % 2;
      const int row = 16 * c + 8 * j + 4 * h + i16 / 4;
      const int col = dvb * 32 + g * 16 + 4 * (i16 % 4);
      const unsigned char* ap = vt + row * (D * 2) + LV::swz_v(row, col / 8) * 16 + (col % 8) * 2;
      typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
      const s16x4 t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ap));
      const ex4 b4 = __builtin_bit_cast(ex4, t4);
#pragma unroll
      for (int e = 0; e < 4; ++e) vf[4 * j + e] = b4[e];
    }
    return vf;
  };

  // ---- softmax state of the current entry.  ref is the reference the weights are formed against, in log2 units; it
  // starts at 0 and moves only when a row sum says it must (a weight overflowed, or a whole block underflowed with
  // nothing accumulated yet): any reference gives the same O / l.
  f32x16 oacc[DVB];
  float ref = 0.f, l_run = 0.f;
  // (the row sum adds the weights before they are rounded: an fp16 weight overflows at 65504 where its fp32 original is
  // still an ordinary number, so the bound on the sum stays below that)
  constexpr float kBig = std::is_same<E, f16_t>::value ? 0x1p15f : 0x1p24f, kTiny = std::is_same<E, f16_t>::value ? 0x1p-4f : 0x1p-24f;
  auto weights = [&](const f32x16& s, ex8 (&pf)[2]) FL_INLINE {
    auto form = [&]() FL_INLINE -> float {
      float rs = 0.f;
      // (the row sum takes the weights before they are rounded, with plain additions: v_dot2c_f32_bf16, which would add
      // two rounded weights at once, does not overlap with matrix instructions on this part)
      float rs1 = 0.f;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float p0 = fast_exp2(__builtin_fmaf(s[8 * j + e], c2, -ref)), p1 = fast_exp2(__builtin_fmaf(s[8 * j + e + 1], c2, -ref));
          pf[j][e] = (E)p0;
          pf[j][e + 1] = (E)p1;
          rs += p0;
          rs1 += p1;
        }
      rs += rs1;
      return rs;
    };
    float rs = form();
    const bool bad = !(rs <= kBig) | ((rs < kTiny) & (l_run < kTiny));
    if (__builtin_amdgcn_ballot_w64(bad) != 0) {
      float m = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) m = __builtin_fmaxf(m, s[i]);
      m = xhalf_max(m) * c2;
      // (a block whose every key carries a finite mask value such as -1e9 must not become the reference: subtracted
      // from itself it leaves the rounding of its own magnitude in the exponent; against this floor its weights are 0)
      m = (m == -INFINITY) ? m : __builtin_fmaxf(m, -32768.0f);
      const float ref_new = (m == -INFINITY) ? ref : __builtin_fmaxf(ref, m);
      // (when nothing has been accumulated yet the old reference carries no weight: take the block's own maximum.  The
      // two lanes of a query hold different keys and so different partial sums; the decision takes their total, so
      // that both form their weights against the same reference and scale the shared accumulators alike)
      const float use = (xhalf_sum(l_run) == 0.f && m != -INFINITY) ? m : ref_new;
      const float alpha = __builtin_fminf(fast_exp2(ref - use), 0x1p126f);
      ref = use;
      l_run *= alpha;
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dvb][i] *= alpha;
      rs = form();
    }
    l_run += rs;
  };

  // ---- prologue: queries (and bias row) of the first entry, the first AHEAD tiles, scores of the first block
  ex8 qf[KS];
  {
    const uint64_t qb0 = qbase + (uint64_t)((int64_t)fb0 * p.qs[0] * 2);
    u32x4 qraw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[ks] = load16_counted(qb0, qoff + 32u * ks);
    if constexpr (kRowB) issue_row(0);
#pragma unroll
    for (int j = 0; j < T::AHEAD; ++j) issue_tile(j / NTI, j % NTI, j);
    dma_wait<0>();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      pin_loaded(qraw[ks]);
      qf[ks] = __builtin_bit_cast(ex8, qraw[ks]);
    }
  }
  __syncthreads();
  f32x16 s_a, s_b;
  ex8 kf[KS];  // K fragments of the block whose scores are formed next (with KAHEAD: read one block ahead of their use)
  ex8 rowf;    // row-bias fragment of that block
  k_frags(kf, 0, 0);
  if constexpr (kRowB) rowf = row_frag(0, 0);
  scores(s_a, kf, qf, 0, rowf);
  if constexpr (kAheadK) k_frags(kf, 0, 1);
#pragma unroll
  for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dvb][i] = 0.f;

  // Operations a wave issues, in order, per entry:  at the barrier point of tile t: the PT transfers of the tile AHEAD
  // tiles on, and at t == 0 also the gate loads of this entry (if there is a gate), the query loads of the next and
  // the transfer of its bias row (NI in all); after the entry's last block: ST stores.  The barrier point of tile t
  // waits for the transfers of tile t + 1, issued AHEAD - 1 barrier points earlier; allowed(t) counts what was issued
  // after them: the extras of that point, and everything of the points since.  Running far ahead keeps the stores out
  // of the way: a wait completes in issue order, so a transfer issued after the stores is only known to have landed
  // once the stores are acknowledged.
  constexpr int PT = 2 * XPW, ST = 2 * DVB;
  constexpr int NI = KS + (kGate ? 2 * DVB : 0) + (kRowB ? 1 : 0);
  constexpr int AHEAD = T::AHEAD;
  auto extras = [](int j) constexpr { const int t = ((j % NTI) + NTI) % NTI; return (t == 0 ? NI : 0) + (t == NTI - 1 ? ST : 0); };
  auto allowed = [extras](int t) constexpr {
    int n = extras(t + 1 - AHEAD);
    for (int j = t + 2 - AHEAD; j < t; ++j) n += PT + extras(j);
    return n;
  };
  for (int item = 0; item < n_items; ++item) {
    const int slot0 = (item * NTI) % NS;
    u32x4 qn[KS];            // next entry's query fragments, in flight from tile 0 on
    u32x4 gl[2 * DVB];       // this entry's gate logits, likewise (8 consecutive columns per load)
    const int64_t fbn = fb0 + min(item + 1, n_items - 1);
    const int64_t fbc = fb0 + item;
    ex8 qnext[KS];
    static_while<0, NTI>([&](auto tt) FL_INLINE {
      constexpr int t = decltype(tt)::value;
      const int slot = (slot0 + t) % NS;
      static_while<0, 2>([&](auto bb) FL_INLINE {
        constexpr int b = decltype(bb)::value;
        constexpr int kb = 2 * t + b;
        constexpr bool last_block = kb == NKB - 1;
        if constexpr (b == 0) {
          // barrier point of tile t, before anything of the tile after it is touched
          // (the last point of an entry also takes the loads of point 0 into use: only the transfers issued since may stay out)
          constexpr int kAllowed = t == NTI - 1 && PT * (NTI - 2) < allowed(t) ? PT * (NTI - 2) : allowed(t);
          static_assert(kAllowed < 64, "vmcnt is a 6-bit counter");
          dma_wait<kAllowed>();
          __syncthreads();  // tile t + 1 is visible; everyone is done with tile t - 1, whose slot the new tile takes
          issue_tile(item + (t + AHEAD) / NTI, (t + AHEAD) % NTI, (slot + AHEAD) % NS);
          if constexpr (t == 0) {
            if constexpr (kGate) {
              const uint64_t gb = gbase + (uint64_t)(fbc * p.gs[0] * 2);
#pragma unroll
              for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
                for (int j = 0; j < 2; ++j) gl[2 * dvb + j] = load16_counted(gb, goff + 64u * dvb + 32u * j);
            }
            const uint64_t qb = qbase + (uint64_t)(fbn * p.qs[0] * 2);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) qn[ks] = load16_counted(qb, qoff + 32u * ks);
            // (the slot it goes to held the previous entry's row, last read a whole entry ago)
            if constexpr (kRowB) issue_row(item + 1);
          }
          if constexpr (t == NTI - 1) {
            // everything issued at tile 0 has landed (the wait above covers later transfers): next entry's queries
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
              pin_loaded(qn[ks]);
              qnext[ks] = __builtin_bit_cast(ex8, qn[ks]);
            }
            if constexpr (kGate) {
#pragma unroll
              for (int g = 0; g < 2 * DVB; ++g) pin_loaded(gl[g]);
            }
          }
        }
        // Scores of the next block (the first block of the next entry after the last one of this) go to the matrix pipe
        // under this block's exponentials.  With KAHEAD their K fragments were read from LDS during the previous block
        // and the reads issued now are for the block after next; without, they are read now, first thing.  The V
        // fragments for this block's second product have the exponentials to land under.
        f32x16& cur = (kb % 2 == 0) ? s_a : s_b;
        f32x16& nxt = (kb % 2 == 0) ? s_b : s_a;
        ex8 kf_ahead[KS], vf[2][DVB];
        if constexpr (kAheadK) k_frags(kf_ahead, (slot + 1) % NS, b);  // block kb + 2: same half of the next tile in the ring
        else k_frags(kf, (slot + (b == 1 ? 1 : 0)) % NS, 1 - b);          // block kb + 1
        if constexpr (kRowB) rowf = last_block ? row_frag(item + 1, 0) : row_frag(item, kb + 1);
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb) vf[c][dvb] = v_frag(slot, 2 * b + c, dvb);
        if constexpr (last_block) scores(nxt, kf, qnext, 0, rowf);
        else scores(nxt, kf, qf, kb + 1, rowf);
        if constexpr (kAheadK) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) kf[ks] = kf_ahead[ks];
        }
        ex8 pf[2];
        weights(cur, pf);
        // the LDS reads first, then the score MFMAs spread over the exponentials (64 vector instructions per block)
        constexpr int kReads = KS + 4 * DVB + (kRowB ? 1 : 0), kScoreMfmas = KS + 2 + (kRowB ? 1 : 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, kReads, 0);
        // (without KAHEAD the first MFMA waits for the K fragments just asked for: some exponentials go first)
        if constexpr (!kAheadK) __builtin_amdgcn_sched_group_barrier(SG_VALU | SG_TRANS, 8, 0);
#pragma unroll
        for (int i = 0; i < kScoreMfmas; ++i) {
          __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
          __builtin_amdgcn_sched_group_barrier(SG_VALU | SG_TRANS, (60 + kScoreMfmas - 1) / kScoreMfmas, 0);
        }
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb) oacc[dvb] = mfma32(vf[c][dvb], pf[c], oacc[dvb]);
        return true;
      });
      return true;
    });
    // ---- this entry is complete: normalise, gate, store; then start the next one
    {
      const float l = xhalf_sum(l_run);
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      const uint64_t ob = obase + (uint64_t)(fbc * p.os[0] * 2);
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb) {
        u32x2 quad[4];  // group g: columns 32 dvb + 8 g + 4 h .. + 4 of this lane's query
        u32x2 gq[4];    // their gate logits: loaded as 8 consecutive columns per lane, the trade below in reverse
        if constexpr (kGate) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            uint32_t a0 = gl[2 * dvb + j][0], a1 = gl[2 * dvb + j][1], b0 = gl[2 * dvb + j][2], b1 = gl[2 * dvb + j][3];
            swap_halves(a0, b0);
            swap_halves(a1, b1);
            gq[2 * j] = u32x2{a0, a1};
            gq[2 * j + 1] = u32x2{b0, b1};
          }
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          ex4 o4;
          if constexpr (kGate) {
            const ex4 g4 = __builtin_bit_cast(ex4, gq[g]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float sg = fast_rcp(1.0f + fast_exp2(-kLog2e * (float)g4[e]));
              o4[e] = (E)(oacc[dvb][4 * g + e] * inv * sg);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) o4[e] = (E)(oacc[dvb][4 * g + e] * inv);
          }
          quad[g] = __builtin_bit_cast(u32x2, o4);
        }
        // the two lanes of a query trade halves of two groups, after which the first holds columns 16 j .. + 8 and the
        // second the next 8: one 16-byte store each instead of two of 8 bytes, and half as many partial lines
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          uint32_t a0 = quad[2 * j][0], a1 = quad[2 * j][1], b0 = quad[2 * j + 1][0], b1 = quad[2 * j + 1][1];
          swap_halves(a0, b0);
          swap_halves(a1, b1);
          const u32x4 w = {a0, a1, b0, b1};
          store16_counted(ob, ooff + 64u * dvb + 32u * j, w);
        }
      }
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dvb][i] = 0.f;
      ref = 0.f;
      l_run = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[ks] = qnext[ks];
    }
  }
  dma_wait<0>();  // nothing of this wave may still be on its way into LDS when the workgroup's allocation is released
}

}  // namespace fl
