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

#include <type_traits>

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
  F_DROPOUT = 128u,  // softmax weights are dropped by a counter-based hash of (seed, batch, head, query, key)
  F_SCOREFN = 256u,  // a function of the scaled score from a small compiled-in set (KParams::score_fn), in the soft-cap's place
};

enum : int { MASK_NONE = 0, MASK_CAUSAL = 1, MASK_SLIDING = 2, MASK_PREFIX = 3, MASK_DOC = 4, MASK_DOC_CAUSAL = 5 };
enum : int { TILE_EMPTY = 0, TILE_PARTIAL = 1, TILE_FULL = 2 };

// Key tiles are numbered in 16 bits inside the LDS tile list.
constexpr int kMaxKeyTiles = 65535;
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
  // element predicate of every positional mask: key < Lk && ((dmin <= key - q <= dmax) || key < pfx)
  int32_t dmin, dmax, pfx;
  const int64_t* doc_ids;
  int64_t doc_stride;
  // Document masks: the key tiles each query tile visits, listed by doc_lists_kernel before the launch (the lists are
  // the same for every head): per (batch, query tile) doc_list_stride words, word 0 = number of entries, then the
  // entries in key order (bits 0-15 tile index, two class bits per wave from bit 16 on).
  const uint32_t* doc_lists;
  int32_t doc_list_stride;  // words per (batch, query tile): a multiple of 4, at least n_ktiles + 1
  // per batch row the query tiles ordered by falling list length (doc_order_kernel): workgroups are dealt in that order,
  // so that the ones still running when the grid drains are the short ones whatever the document layout
  const int32_t* doc_order;
  int32_t alibi_heads;
  float softcap;
  const bf16_t* bias[2];
  int64_t bs[2][4];
  int32_t bdiv[2];
  int32_t bias_vec[2];  // rows of this bias may be read 4 keys at a time (8-byte pieces of bf16, 16-byte of fp32)
  int32_t bias_f32[2];  // elements are fp32 instead of bf16 (such an operand is never staged through LDS)
  int32_t bias_lds;     // index of the bias operand staged through LDS (16-byte aligned rows, Lk % 8 == 0), or -1
  int32_t bias_row;     // index of a row-broadcast bias operand staged through LDS as single rows, or -1
  const bf16_t* gate;
  int64_t gs[3];
  float lambda;
  int64_t q_branch_stride, k_branch_stride;  // element offset of the second softmax branch (diff)
  uint8_t* dump;
  float* lse;        // optional [B, Hq, Lq]: log2 of the row's sum of 2^(logit in log2 units); +inf if nothing attended
  uint32_t drop_thr;      // a weight is dropped when its 16 hash bits are < drop_thr (1 .. 65535; 0: no dropout)
  uint32_t drop_seed[2];  // low and high half of the 64-bit seed
  float drop_rescale;     // 65536 / (65536 - drop_thr), applied to the kept weights
  int32_t head_group;  // (batch, head) pairs whose query tiles are dealt together, longest first (1: head by head)
  int32_t o_wide;      // o is 16-byte aligned with strides that are multiples of 8 elements: 16-byte stores
  // F_SCOREFN: 1 sigmoid, 2 clamp, 3 cubic polynomial, with four constants the host has folded scale and log2(e) into
  // (x = the raw q.k; results in log2 units):  1: k2 / (1 + 2^(k0 x + k1)) + k3;  2: med3(k0 x + k1, k2, k3);
  // 3: ((k3 x + k2) x + k1) x + k0
  int32_t score_fn;
  float score_k[4];
  int32_t n_qtiles;  // ceil(Lq / BM)
  int32_t n_ktiles;  // ceil(Lk / BN)
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- dropout decisions ------------------------------------------------------------------------------------------------
// Whether the weight of (batch, head, query q, key k) survives is a pure function of those and the seed, so that the
// forward, both backward kernels and a CPU restatement agree without exchanging a mask.  One 32-bit hash serves the
// key pair (2j, 2j + 1): the even key takes the low 16 bits, the odd key the high 16, and a weight is dropped when its
// 16 bits are below the threshold.  The hash of x = head_seed + q * kDropQ + (k / 2) * kDropK is two rounds of a
// 24-bit multiply-add between xor-shifts: full-rate vector instructions only (a 32-bit multiply is quarter rate).
constexpr uint32_t kDropQ = 0x9E3779B1u, kDropK = 0x85EBCA77u;
__device__ __forceinline__ uint32_t drop_fmix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x85EBCA6Bu;
  x ^= x >> 13;
  x *= 0xC2B2AE35u;
  x ^= x >> 16;
  return x;
}
// start value of head bh = batch * Hq + head (once per workgroup: the 32-bit multiplies do not matter here)
__device__ __forceinline__ uint32_t drop_head_seed(uint32_t seed_lo, uint32_t seed_hi, uint32_t bh) {
  return drop_fmix32(seed_lo ^ drop_fmix32(seed_hi + 0x9E3779B9u * (bh + 1u)));
}
__device__ __forceinline__ uint32_t drop_pair_hash(uint32_t x) {
  x ^= x >> 16;
  x = (x & 0xFFFFFFu) * 0xCA6B35u + (x >> 8);
  x ^= x >> 13;
  x = ((x >> 8) & 0xFFFFFFu) * 0xB2AE3Du + x;
  x ^= x >> 16;
  return x;
}
// 0xFFFF in each half of the result whose 16 hash bits are > c (c = threshold - 1 in both halves of c2): three packed
// 16-bit instructions
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t drop_pair_mask(uint32_t hash, uint32_t c2) {
  const u16x2 d = __builtin_elementwise_sub_sat(__builtin_bit_cast(u16x2, hash), __builtin_bit_cast(u16x2, c2));
  const u16x2 one = {1, 1}, all = {0xFFFF, 0xFFFF};
  return __builtin_bit_cast(uint32_t, (u16x2)(__builtin_elementwise_min(d, one) * all));
}
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

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// a <-> b across the two halves of the wave: lanes 32..63 of `a` change places with lanes 0..31 of `b`
__device__ __forceinline__ void swap_halves(uint32_t& a, uint32_t& b) {
  auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  const uint32_t r0 = r[0], r1 = r[1];  // (copied out element by element: see xhalf_pair)
  a = r0;
  b = r1;
}

// 16 bytes per lane from global memory straight into LDS (global_load_lds_dwordx4): lane l of the wave reads
// gbase + voff[l] and writes LDS bytes [lds_base + 16 l, +16).  gbase and lds_base are wave-uniform.  Written as asm
// so that the compiler does not order later LDS reads of *other* buffers behind it with a vmcnt(0) wait; completion
// is awaited explicitly (dma_wait) before the barrier that publishes the data.
// Pins an (already wave-uniform) pointer to scalar registers whatever the compiler's divergence analysis concluded.
// readfirstlane returns int: each half goes through uint32_t so the low half is not sign-extended over the high one.
__device__ __forceinline__ uint64_t uniform_ptr(const void* ptr) {
  const uint64_t b = reinterpret_cast<uint64_t>(ptr);
  return (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b) |
         ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32);
}
__device__ __forceinline__ int64_t uniform_i64(int64_t x) {
  return (int64_t)((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)x) |
                   ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)x >> 32)) << 32));
}
__device__ __forceinline__ void dma16(uint64_t gbase_uniform, unsigned voff, unsigned lds_base) {
  const unsigned lds_base_uniform = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_base);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" ::"s"(gbase_uniform), "v"(voff),
               "s"(lds_base_uniform)
               : "m0");
}

// The same with 4 bytes per lane (lane l writes LDS bytes [4 l, 4 l + 4)): for fp32 rows whose start is only 4-byte aligned.
__device__ __forceinline__ void dma4(uint64_t gbase_uniform, unsigned voff, unsigned lds_base) {
  const unsigned lds_base_uniform = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_base);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %1, %0" ::"s"(gbase_uniform), "v"(voff),
               "s"(lds_base_uniform)
               : "m0");
}

// Waits until at most N of this wave's vector-memory operations (the transfers above included) are outstanding;
// they complete in issue order.  Leaves the LDS/scalar and export counters alone.
template <int N>
__device__ __forceinline__ void dma_wait() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 0xf) | ((N >> 4) << 14));
}

// f(integral_constant<int, I>) for I = I0, I0+1, ... < N while f returns true; false if some call returned false.
template <int I, int N, class F>
__device__ __forceinline__ bool static_while(F&& f) {
  if constexpr (I < N) {
    if (!f(std::integral_constant<int, I>{})) return false;
    return static_while<I + 1, N>(f);
  } else {
    return true;
  }
}

// ---- mask logic (integer, shared by the tile classifier and the element predicate) -------------------------------

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
  // Tiles that are read both ways (the backward's streamed operands): the row's window index rotated left by two
  // bits.  Still a permutation of the chunk index over 16 consecutive rows (row-wise reads), and 4 consecutive rows
  // land in 4 different 64-byte groups (transposing reads).
  __device__ static __forceinline__ int swz_kv(int row, int chunk) {
    constexpr int NB = CPR >= 16 ? 4 : (CPR >= 8 ? 3 : 2);
    const int m = (row / RPW) & ((1 << NB) - 1);
    return chunk ^ (((m << 2) | (m >> (NB - 2))) & ((1 << NB) - 1));
  }
  // V operand reads (transposing): 4 consecutive rows x 64 contiguous bytes.
  __device__ static __forceinline__ int swz_v(int row, int chunk) {
    constexpr int G = (CPR >= 16 ? 16 : CPR) / 4;  // 64-byte groups per window row
    if constexpr (G <= 1) return chunk;
    return chunk ^ (((row / RPW) & (G - 1)) << 2);
  }
};

// Staged bias tile of one wave: [RW rows][BN keys] bf16, 16-byte chunks XOR-swizzled with the row so that the 8-byte
// reads of 32 consecutive rows at one key offset spread over the banks.
template <int BN>
struct BiasLayout {
  static constexpr int CPR = BN / 8;                         // chunks per row
  static constexpr int RPW = (CPR >= 16) ? 1 : (16 / CPR);   // rows per 256-byte bank window
  __device__ static __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row / RPW) & (CPR - 1)); }
};

// Scheduling pipeline for the straight-line tile step (see fwd_kernel): instruction classes of
// __builtin_amdgcn_sched_group_barrier.
enum : int { SG_VALU = 0x2, SG_MFMA = 0x8, SG_DS_READ = 0x100, SG_TRANS = 0x400 };
// Every lambda of the kernel must be inlined: an outlined one would take its captures (the accumulators) by address
// through scratch memory.
#define FL_INLINE __attribute__((always_inline))

#ifndef FL_SCHED
#define FL_SCHED 1
#endif

// Orders the step's instructions as: each first-product MFMA preceded by its K fragment read and followed by a
// share of the exponential work; each second-product MFMA preceded by its two transposing V reads and followed
// by a share of the next tile's row maximum.  NA / NB = MFMAs in the two products, VA / VB = vector ops to spread.
template <int NA, int VA>
__device__ __forceinline__ void sched_first_product() {
#if FL_SCHED == 1
  __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 2, 0);
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
    if (i + 2 < NA) __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
    __builtin_amdgcn_sched_group_barrier(SG_VALU | SG_TRANS, VA, 0);
  }
#endif
}
template <int NB, int VB>
__device__ __forceinline__ void sched_second_product() {
#if FL_SCHED == 1
  __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 4, 0);
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
    if (i + 2 < NB) __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 2, 0);
    if (VB > 0) __builtin_amdgcn_sched_group_barrier(SG_VALU | SG_TRANS, VB, 0);
  }
#endif
}

// Element types of q, k, v, biases (unless fp32), gate and the output: bf16 or fp16.  The two differ in the MFMA and dot
// instructions and in the conversions from and to fp32; everything else treats the elements as 16 opaque bits.
typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ float dot2acc(bf16x2 a, bf16x2 b, float c) { return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false); }
__device__ __forceinline__ float dot2acc(f16x2 a, f16x2 b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }

template <int DQK_, int DV_, int RW_, int BN_, int NW_, uint32_t FEAT_, int NS_ = 4, class Elem_ = bf16_t>
struct FwdTraits {
  using Elem = Elem_;
  static constexpr int DQK = DQK_, DV = DV_, RW = RW_, BN = BN_, NW = NW_;
  static constexpr int NS = NS_;  // K/V tiles resident in LDS (ring); transfers run NS - 1 tiles ahead of their use
  static_assert(NS >= 2 && NS <= 8 && NS % 2 == 0, "ring depth (even: the two score buffers alternate with the slots)");
  static constexpr uint32_t FEAT = FEAT_;
  static constexpr int NT = NW * 64;
  static constexpr int BM = NW * RW;
  static constexpr int QB = RW / 32;   // 32-row query blocks per wave
  static constexpr int KB = BN / 32;   // 32-key blocks per tile
  static constexpr int KS = DQK / 16;  // MFMA k-steps of the first product
  static constexpr int DVB = DV / 32;  // 32-wide blocks of the value dimension
  static constexpr int KBYTES = BN * DQK * 2, VBYTES = BN * DV * 2;
  static constexpr int K_CHUNKS = BN * DQK / 8, V_CHUNKS = BN * DV / 8;
  static constexpr int K_PER_T = K_CHUNKS / NT, V_PER_T = V_CHUNKS / NT;
  static_assert(K_CHUNKS % NT == 0 && V_CHUNKS % NT == 0, "tile must divide evenly over the threads");
  static_assert(RW % 32 == 0 && BN % 32 == 0 && DQK % 16 == 0 && DV % 32 == 0, "MFMA 32x32x16 blocking");
  static_assert(NW <= 8, "tile classes are packed two bits per wave into 16 bits");
  // waves per SIMD the register budget is sized for
#ifdef FL_WPE
  static constexpr int WAVES_PER_EU = FL_WPE;
#else
  static constexpr int WAVES_PER_EU = (RW == 32 && DQK <= 256 && !(DQK == 256 && (FEAT_ & F_BIAS))) ? 2 : 1;
#endif
  // One dense bias operand is staged through LDS like K and V: per ring slot a [BM][BN] bf16 tile, every wave
  // transferring (and later reading) only its own RW rows.
  static constexpr int BBYTES = (FEAT & F_BIAS) ? BM * BN * 2 : 0;
  static constexpr int B_PER_T = (FEAT & F_BIAS) ? RW * BN / 8 / 64 : 0;  // 16-byte transfers per lane per tile
  static_assert(!(FEAT & F_BIAS) || ((RW * BN / 8) % 64 == 0 && NS == 2), "staged bias: whole transfers, ring of two");
  // LDS: K tiles [NS], V tiles [NS], bias tiles [NS], row-bias images [NS], document-id images [NS], then (document
  // masks only) the tile list, sized at launch: 4 bytes per entry plus the count, rounded up to whole wave transfers
  // A second, row-broadcast operand (query stride 0, e.g. a key-padding bias) is staged as one row of BN keys per wave
  // and slot; the transfer is a whole 1 KiB wave transfer whose lanes repeat the row.
  static constexpr int RBYTES = (FEAT & F_BIAS) ? NW * 1024 : 0;
  static constexpr int R_PER_T = (FEAT & F_BIAS) ? 1 : 0;
  // Document ids of a tile's keys ride with its V tile: per ring slot and wave a private image of the BN int64 ids,
  // brought by transfers of 4 bytes per lane (any alignment, exact clamping at the ragged end).
  static constexpr int I_PER_T = (FEAT & F_DOC) ? BN * 8 / 256 : 0;  // transfers per tile
  static constexpr int IBYTES = (FEAT & F_DOC) ? NW * BN * 8 : 0;
  static_assert(!(FEAT & F_DOC) || (BN * 8) % 256 == 0, "whole transfers of 64 dwords");
  static constexpr int K_OFF = 0, V_OFF = NS * KBYTES, B_OFF = NS * (KBYTES + VBYTES), R_OFF = B_OFF + NS * BBYTES,
                       I_OFF = R_OFF + NS * RBYTES, LIST_OFF = I_OFF + NS * IBYTES;
  static constexpr int LDS_FIXED_BYTES = LIST_OFF;
};

// The main loop is software-pipelined over key tiles so that one wave keeps both the matrix pipe and the vector
// ALU busy.  With ta, tb, tc three consecutive non-empty tiles, iteration i does
//     region A   S(tb) = K(tb).Q^T on MFMA          ||   P(ta) = exp2(S(ta) - m), row sums, bf16 pack   (VALU)
//     region B   O^T  += V(ta)^T.P(ta)^T on MFMA     ||   running max of S(tb)                            (VALU)
//     rare       element mask of S(tb) on partial tiles; rescale of O, l when the maximum grew
// while the global -> LDS transfers of K(tc) and V(tb), issued at the top of the iteration into the buffers that
// iteration i-1 freed, are in flight; the barrier that ends the iteration publishes them.
template <class T>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::WAVES_PER_EU, T::WAVES_PER_EU)))
void fwd_kernel(const KParams p) {
  constexpr int DQK = T::DQK, DV = T::DV, RW = T::RW, BN = T::BN, NW = T::NW, NT = T::NT, BM = T::BM;
  constexpr int QB = T::QB, KB = T::KB, KS = T::KS, DVB = T::DVB;
  constexpr uint32_t FEAT = T::FEAT;
  constexpr bool kAlibi = FEAT & F_ALIBI, kSoftcap = FEAT & F_SOFTCAP, kBias = FEAT & F_BIAS, kDoc = FEAT & F_DOC;
  constexpr bool kDiff = FEAT & F_DIFF, kGate = FEAT & F_GATE, kDump = FEAT & F_DUMP;
  constexpr bool kDrop = FEAT & F_DROPOUT;
  constexpr bool kScoreFn = FEAT & F_SCOREFN;
  static_assert(!(kScoreFn && (kSoftcap || kAlibi)), "one function of the score per kernel");
  constexpr bool kMod = kAlibi || kSoftcap || kBias || kScoreFn;  // scores are transformed before the softmax
  constexpr float kLog2e = 1.4426950408889634f;
  using E = typename T::Elem;  // pointers in KParams are typed bf16_t whatever E is: 16 opaque bits
  typedef E ex8 __attribute__((ext_vector_type(8)));
  typedef E ex4 __attribute__((ext_vector_type(4)));
  typedef E ex2 __attribute__((ext_vector_type(2)));
  using LK = TileLayout<DQK>;
  using LV = TileLayout<DV>;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // tile list (document masks): word 0 = number of entries, then one entry per key tile that is not empty for the
  // whole workgroup, in key order: bits 0-15 tile index, bits 16.. two class bits per wave
  const uint32_t* tlist = reinterpret_cast<const uint32_t*>(smem + T::LIST_OFF) + 1;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int r = lane % 32, h = lane / 32;

  // ---- workgroup -> (batch, head, query tile).  Consecutive workgroup ids land on different XCDs, so ids are
  // regrouped to give every XCD a contiguous run of (batch, head) pairs: their K/V stay in that XCD's L2.
  // Under masks whose work grows with the query position (causal, prefix-LM, causal documents) heads are taken
  // p.head_group at a time (enough of them to fill the XCD's workgroup slots about twice over) and their query tiles
  // dealt from the last (longest) to the first, round-robin over those heads: the workgroups still running when the grid
  // drains are the short ones.  Under the other masks every query tile costs the same, and heads are taken one at a
  // time (HBM then sees each K/V tile once).
  int bh, qt;
  {
    const int nbh = p.B * p.Hq, nq = p.n_qtiles;
    int i = blockIdx.x, run = nbh, base = 0;
    if (nbh % 8 == 0) {
      run = nbh / 8;
      base = (i % 8) * run;
      i /= 8;
    }
    const int G = p.head_group;
    const int g = i / (G * nq), rem = i % (G * nq);
    const int gg = min(G, run - G * g);
    qt = nq - 1 - rem / gg;
    bh = base + G * g + rem % gg;
    // document masks: the work of a query tile is the length of its tile list, known from the pre-pass
    if constexpr (kDoc) qt = p.doc_order[(bh / p.Hq) * nq + rem / gg];
  }
  const int head = bh % p.Hq, batch = bh / p.Hq;
  const int kvh = head / p.group;

  const int q0 = qt * BM;             // first query row of the workgroup
  const int qw0 = q0 + wave * RW;     // first query row of this wave
  const int nk = p.n_ktiles;

  // ---- which key tiles this workgroup visits ------------------------------------------------------------------------
  // Positional masks attend one contiguous range of key tiles, [t_lo, t_lo + n_list): list position i is tile t_lo + i
  // and its class for this wave is computed where it is needed.  Document masks can attend scattered tiles: every key
  // tile is classified for every wave and the non-empty ones are compacted into the LDS tile list.
  int n_list = 0, t_lo = 0;
  if constexpr (kDoc) {
    // the list of this (batch, query tile) goes global -> LDS in whole wave transfers (64 chunks of 16 bytes each; chunks
    // past the end repeat the last one); it is awaited, together with the first K/V transfers' predecessors, right
    // before the key loop, so that the query loads below run under its latency
    const int n_chunks = p.doc_list_stride / 4;
    const uint64_t lbase = uniform_ptr(p.doc_lists + ((int64_t)batch * p.n_qtiles + qt) * p.doc_list_stride);
    const unsigned lds_l = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::LIST_OFF);
    for (int c0 = wave * 64; c0 < n_chunks; c0 += NW * 64)
      dma16(lbase, (unsigned)min(c0 + lane, n_chunks - 1) * 16u, lds_l + c0 * 16);
  } else {
    const int q1 = min(q0 + BM, p.Lq);
    int hi_key = p.Lk - 1, lo_key = 0;  // first / last key position some row of the workgroup may attend
    if (p.mask_kind == MASK_CAUSAL || p.mask_kind == MASK_SLIDING) hi_key = min(hi_key, q1 - 1);
    if (p.mask_kind == MASK_PREFIX) hi_key = min(hi_key, max(q1, p.prefix) - 1);
    if (p.mask_kind == MASK_SLIDING) lo_key = max(0, q0 - p.window);
    t_lo = lo_key / BN;
    n_list = hi_key >= lo_key ? hi_key / BN - t_lo + 1 : 0;
  }
  // This wave's tile classes for a positional mask, as index ranges: tiles outside [e_lo, e_hi] are EMPTY for its
  // rows [a, b), tiles inside [f_lo, f_hi] FULL, the rest PARTIAL (the same closed forms as classify_positional,
  // solved for the tile index; the ragged last tile is never FULL because keys >= Lk are masked; a tile may be
  // called PARTIAL where it is in fact EMPTY or FULL, never the other way round).
  int e_lo = 0, e_hi = -1, f_lo = 0, f_hi = -1;
  if constexpr (!kDoc) {
    const int a = qw0, b = min(qw0 + RW, p.Lq);
    if (a < b) {
      const int last = nk - 1, whole = p.Lk / BN - 1;  // last tile; last tile that lies entirely below Lk
      e_hi = last;
      f_hi = whole;
      if (p.mask_kind == MASK_CAUSAL || p.mask_kind == MASK_SLIDING) {
        e_hi = min(last, (b - 1) / BN);
        f_hi = min(whole, (a + 1) / BN - 1);
      }
      if (p.mask_kind == MASK_SLIDING) {
        e_lo = max(0, a - p.window) / BN;
        f_lo = b - 1 - p.window > 0 ? (b - 1 - p.window + BN - 1) / BN : 0;
      }
      if (p.mask_kind == MASK_PREFIX) {
        e_hi = min(last, (max(p.prefix, b) + BN - 1) / BN - 1);
        f_hi = min(whole, max(p.prefix / BN, (a + 1) / BN) - 1);
      }
    }
  }
  // tile-list entry of list position i (the last entry again past the end): bits 0-15 tile index, two class bits per
  // wave from bit 16 on (only this wave's are filled in when the entry is computed rather than read)
  auto list_entry = [&](int i) FL_INLINE -> uint32_t {
    if constexpr (kDoc) {
      return tlist[min(i, n_list - 1)];
    } else {
      // ALiBi adds a term that grows with the key position: visiting the tiles from the last one down makes every
      // later tile's scores fall away from the running reference instead of climbing above it, so the reference set by
      // the first tile visited holds and the accumulators are never rescaled
      const int t = (FEAT & F_ALIBI) ? t_lo + n_list - 1 - min(i, n_list - 1) : t_lo + min(i, n_list - 1);
      const int cw = (t < e_lo || t > e_hi) ? TILE_EMPTY : ((t >= f_lo && t <= f_hi) ? TILE_FULL : TILE_PARTIAL);
      return ((uint32_t)cw << (16 + 2 * wave)) | (uint32_t)t;
    }
  };

  // ---- per-lane constants ----------------------------------------------------------------------------------------
  int qrow[QB];  // query position owned by this lane in each query block
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) qrow[qb] = qw0 + qb * 32 + r;

  float slope_l2 = 0.f;  // ALiBi slope in log2 units
  if constexpr (kAlibi)
    slope_l2 = p.alibi_heads > 0 ? exp2f(-8.0f * (float)(head + 1) / (float)p.alibi_heads) * kLog2e : 0.f;
  float cap_k1 = 0.f, cap_c = 0.f;
  if constexpr (kSoftcap) {
    cap_k1 = p.scale / p.softcap * 2.0f * kLog2e;  // exp2 argument of e^{2x/cap}
    cap_c = p.softcap * kLog2e;                    // cap in log2 units
  }
  int fn_kind = 0;
  float fn_k[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (kScoreFn) {
    fn_kind = __builtin_amdgcn_readfirstlane(p.score_fn);
#pragma unroll
    for (int i = 0; i < 4; ++i) fn_k[i] = p.score_k[i];
  }
  int64_t qdoc[QB];
  if constexpr (kDoc) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
      qdoc[qb] = p.doc_ids[(int64_t)batch * p.doc_stride + min(qrow[qb], p.Lq - 1)];
  }
  // dropout: this lane's rows' share of the hash argument, and the threshold (minus one) in both 16-bit halves
  uint32_t drop_q[QB];
  uint32_t drop_c2 = 0;
  if constexpr (kDrop) {
    const uint32_t s0 = drop_head_seed(p.drop_seed[0], p.drop_seed[1], (uint32_t)(batch * p.Hq + head));
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) drop_q[qb] = s0 + (uint32_t)qrow[qb] * kDropQ;
    drop_c2 = (p.drop_thr - 1u) * 0x10001u;
  }
  // With dense biases as the only score modification the modified scores stay in natural units (s = qk * scale + bias)
  // and the factor log2(e) rides in the exponential's multiply-add; other modifications produce log2 units directly.
  constexpr bool kNatural = kBias && !kSoftcap && !kAlibi && !kScoreFn;
  const float c2 = kNatural ? kLog2e : (kMod ? 1.0f : p.scale_log2);  // s * c2 is the logit in log2 units
  // The running maximum only moves when some row of the wave sees a score more than kTau (log2 units) above it,
  // so exp2 arguments stay <= kTau and the accumulators are rescaled on few tiles.  Any m gives the same O / l.
  constexpr float kTau = 8.0f;
  // Soft-capped scores are bounded, so every tile of such a kernel forms its weights against the running reference as it
  // stands (see weights_checked): the reference is then known when the tile's scores are modified, one step earlier,
  // and is subtracted there, in the addend of a multiply-add that is issued anyway.  The modified scores of these
  // kernels are relative to the reference of the moment; it can move only on the path that recomputes a tile's
  // weights, which accounts for the difference.
  constexpr bool kFoldRef = kSoftcap && !kDrop;  // (the dropout instances have no registers to spare for it)

  // Gate logits of this lane's output elements, fetched before the key loop when they fit the register budget so that
  // their latency is not paid in the epilogue.
  constexpr bool kGateEarly = kGate && DV <= 32;
  ex4 gpre[kGateEarly ? DVB : 1][kGateEarly ? QB : 1][4];
  if constexpr (kGateEarly) {
    if (p.gate) {
      const bf16_t* gp = p.gate + (int64_t)batch * p.gs[0] + (int64_t)head * p.gs[1];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            gpre[dvb][qb][g] = *reinterpret_cast<const ex4*>(gp + (int64_t)min(qrow[qb], p.Lq - 1) * p.gs[2] +
                                                                32 * dvb + 8 * g + 4 * h);
    }
  }

  f32x16 ofin[kDiff ? DVB : 1][kDiff ? QB : 1];  // branch-0 result kept while branch 1 runs (diff only)
  f32x16 oacc[DVB][QB];
  float m_run[QB], l_run[QB];
  auto ref_now = [&](int qb) FL_INLINE { return (m_run[qb] == -INFINITY) ? 0.f : m_run[qb]; };

#pragma unroll
  for (int br = 0; br < (kDiff ? 2 : 1); ++br) {
    const bf16_t* qptr = p.q + (int64_t)batch * p.qs[0] + (int64_t)head * p.qs[1] + (int64_t)br * p.q_branch_stride;
    const bf16_t* kptr = p.k + (int64_t)batch * p.ks[0] + (int64_t)kvh * p.ks[1] + (int64_t)br * p.k_branch_stride;
    const bf16_t* vptr = p.v + (int64_t)batch * p.vs[0] + (int64_t)kvh * p.vs[1];

    // Q fragments: B operand of S^T = K.Q^T; lane (r, h) holds Q[q = r][16*ks + 8h .. +8].
    ex8 qf[QB][KS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[qb][ks] = *reinterpret_cast<const ex8*>(qptr + (int64_t)min(qrow[qb], p.Lq - 1) * p.qs[2] + ks * 16 + 8 * h);

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

    // ---- global -> LDS, without passing through registers: each wave fills 1 KiB of the tile per transfer, lane l
    // writing bytes [16 l, 16 l + 16) of that KiB from its own global address.  The LDS image is the swizzled tile, so
    // lane (row, physical chunk) fetches the logical chunk that maps there (the swizzles are XORs, hence their own
    // inverses).  The global address is a per-tile scalar base plus a per-lane byte offset that does not change from
    // tile to tile; only the ragged last tile recomputes it, repeating the last key for rows past the end (those
    // keys are masked, p = 0).
    // LDS byte addresses this wave's transfers of slot 0, first transfer, land at
    const unsigned lds_k = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::K_OFF + wave * 1024);
    const unsigned lds_v = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::V_OFF + wave * 1024);
    const unsigned lds_i = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::I_OFF + wave * (BN * 8));
    // The rows of a thread's transfer `it` lie it * (NT / CPR) below those of its transfer 0.  When that step is a multiple
    // of the swizzle's period in rows, the chunk a lane fetches is the same for every transfer, and one per-lane offset
    // serves them all: the row step goes into the scalar base address instead of into a register per transfer.
    constexpr int K_ROWS_PER_T = NT / LK::CPR, V_ROWS_PER_T = NT / LV::CPR;
    constexpr bool kOneKoff = NT % LK::CPR == 0 && K_ROWS_PER_T % (LK::RPW * (LK::CPR >= 16 ? 16 : LK::CPR)) == 0;
    constexpr bool kOneVoff = NT % LV::CPR == 0 && V_ROWS_PER_T % (LV::RPW * (LV::CPR >= 16 ? 16 : LV::CPR)) == 0;
    unsigned koff[kOneKoff ? 1 : T::K_PER_T], voff[kOneVoff ? 1 : T::V_PER_T];
#pragma unroll
    for (int it = 0; it < (kOneKoff ? 1 : T::K_PER_T); ++it) {
      const int id = it * NT + tid, row = id / LK::CPR, pc = id % LK::CPR;
      koff[it] = (unsigned)(row * (int)p.ks[2] + LK::swz_k(row, pc) * 8) * 2u;
    }
#pragma unroll
    for (int it = 0; it < (kOneVoff ? 1 : T::V_PER_T); ++it) {
      const int id = it * NT + tid, row = id / LV::CPR, pc = id % LV::CPR;
      voff[it] = (unsigned)(row * (int)p.vs[2] + LV::swz_v(row, pc) * 8) * 2u;
    }
    const uint32_t k_step_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(K_ROWS_PER_T * (uint32_t)p.ks[2] * 2u));
    const uint32_t v_step_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(V_ROWS_PER_T * (uint32_t)p.vs[2] * 2u));
    // scalar base addresses; one key tile is less than 2^31 bytes from start to end (checked on the host)
    const uint64_t kbase = uniform_ptr(kptr), vbase = uniform_ptr(vptr);
    const uint32_t k_tile_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(BN * (uint32_t)p.ks[2] * 2u));
    const uint32_t v_tile_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(BN * (uint32_t)p.vs[2] * 2u));
    auto load_k = [&](int t, int slot) FL_INLINE  {
      const uint64_t base = kbase + (uint64_t)(uint32_t)t * k_tile_bytes;
      if (t * BN + BN <= p.Lk) {
#pragma unroll
        for (int it = 0; it < T::K_PER_T; ++it) {
          if constexpr (kOneKoff) dma16(base + (uint64_t)((uint32_t)it * k_step_bytes), koff[0], lds_k + slot * T::KBYTES + it * NT * 16);
          else dma16(base, koff[it], lds_k + slot * T::KBYTES + it * NT * 16);
        }
      } else {
#pragma unroll
        for (int it = 0; it < T::K_PER_T; ++it) {
          const int id = it * NT + tid, row = id / LK::CPR, pc = id % LK::CPR;
          const unsigned off = (unsigned)(min(row, p.Lk - 1 - t * BN) * (int)p.ks[2] + LK::swz_k(row, pc) * 8) * 2u;
          dma16(base, off, lds_k + slot * T::KBYTES + it * NT * 16);
        }
      }
    };
    // this wave's copy of a tile's key ids (document masks), one dword per lane and transfer; keys past Lk repeat the last id
    auto load_ids = [&](int t, int slot) FL_INLINE {
      if constexpr (kDoc) {
        const uint64_t ibase = uniform_ptr(p.doc_ids + (int64_t)batch * p.doc_stride + (int64_t)t * BN);
        const int last = p.Lk - 1 - t * BN;
#pragma unroll
        for (int it = 0; it < T::I_PER_T; ++it) {
          const int d = 64 * it + lane;
          dma4(ibase, (unsigned)(min(d / 2, last) * 8 + (d % 2) * 4), lds_i + slot * T::IBYTES + it * 256);
        }
      }
    };
    // (with_ids: some wave of the workgroup may apply the element mask to the tile, which compares document ids)
    auto load_v = [&](int t, int slot, bool with_ids) FL_INLINE  {
      if (with_ids) load_ids(t, slot);
      const uint64_t base = vbase + (uint64_t)(uint32_t)t * v_tile_bytes;
      if (t * BN + BN <= p.Lk) {
#pragma unroll
        for (int it = 0; it < T::V_PER_T; ++it) {
          if constexpr (kOneVoff) dma16(base + (uint64_t)((uint32_t)it * v_step_bytes), voff[0], lds_v + slot * T::VBYTES + it * NT * 16);
          else dma16(base, voff[it], lds_v + slot * T::VBYTES + it * NT * 16);
        }
      } else {
#pragma unroll
        for (int it = 0; it < T::V_PER_T; ++it) {
          const int id = it * NT + tid, row = id / LV::CPR, pc = id % LV::CPR;
          const unsigned off = (unsigned)(min(row, p.Lk - 1 - t * BN) * (int)p.vs[2] + LV::swz_v(row, pc) * 8) * 2u;
          dma16(base, off, lds_v + slot * T::VBYTES + it * NT * 16);
        }
      }
    };
    // Staged bias operand: this wave's rows [qw0, qw0 + RW) x the tile's BN keys, lane -> (row, physical chunk) of the
    // wave's LDS image; rows past Lq repeat the last row (their results are never stored).
    using LB = BiasLayout<BN>;
    const int nbl = kBias ? p.bias_lds : -1;
    const bool stage_bias = kBias && nbl >= 0;
    const bf16_t* bptr = nullptr;
    const unsigned lds_b = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::B_OFF + wave * (RW * BN * 2));
    unsigned boff[T::B_PER_T > 0 ? T::B_PER_T : 1];
    if constexpr (kBias) {
      if (stage_bias) {
        bptr = p.bias[nbl] + (int64_t)(batch / p.bdiv[nbl]) * p.bs[nbl][0] + (int64_t)head * p.bs[nbl][1];
#pragma unroll
        for (int it = 0; it < T::B_PER_T; ++it) {
          const int id = it * 64 + lane, row = id / LB::CPR, pc = id % LB::CPR;
          boff[it] = (unsigned)(min(qw0 + row, p.Lq - 1) * (int)p.bs[nbl][2] + LB::swz(row, pc) * 8) * 2u;
        }
      }
    }
    const int nbr = kBias ? p.bias_row : -1;
    const bf16_t* rptr = nullptr;
    bool row_f32 = false;  // the staged row operand holds fp32 elements (4 keys per 16-byte chunk instead of 8)
    const unsigned lds_r = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)smem + T::R_OFF + wave * 1024);
    if constexpr (kBias) {
      if (nbr >= 0) {
        row_f32 = p.bias_f32[nbr] != 0;
        // (element offsets; the pointer is typed bf16_t, so an fp32 operand's offset counts twice)
        rptr = p.bias[nbr] + ((int64_t)(batch / p.bdiv[nbr]) * p.bs[nbr][0] + (int64_t)head * p.bs[nbr][1]) * (row_f32 ? 2 : 1);
      }
    }
    bool any_direct = false;
    if constexpr (kBias) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) any_direct = any_direct || (p.bias[nb] != nullptr && nb != nbr && nb != nbl);
    }
    auto load_b = [&](int t, int slot) FL_INLINE {
      if constexpr (kBias) {
        if (nbr >= 0) {
          // lanes repeat the row's BN / 8 chunks; chunks past Lk repeat the last one
          const int last_chunk = (min(p.Lk - t * BN, BN)) / 8 - 1;
          if (row_f32) {
            const int last4 = (min(p.Lk - t * BN, BN)) / 4 - 1;
            dma16(uniform_ptr(rptr + (int64_t)t * BN * 2), (unsigned)min(lane % (BN / 4), last4) * 16u, lds_r + slot * T::RBYTES);
          } else {
            dma16(uniform_ptr(rptr + (int64_t)t * BN), (unsigned)min(lane % LB::CPR, last_chunk) * 16u, lds_r + slot * T::RBYTES);
          }
        }
        if (!stage_bias) return;
        const uint64_t base = uniform_ptr(bptr + (int64_t)t * BN);
        if (t * BN + BN <= p.Lk) {
#pragma unroll
          for (int it = 0; it < T::B_PER_T; ++it) dma16(base, boff[it], lds_b + slot * T::BBYTES + it * 1024);
        } else {
          const int last_chunk = (p.Lk - t * BN) / 8 - 1;  // Lk % 8 == 0 whenever a bias is staged
#pragma unroll
          for (int it = 0; it < T::B_PER_T; ++it) {
            const int id = it * 64 + lane, row = id / LB::CPR, pc = id % LB::CPR;
            const unsigned off =
                (unsigned)(min(qw0 + row, p.Lq - 1) * (int)p.bs[nbl][2] + min(LB::swz(row, pc), last_chunk) * 8) * 2u;
            dma16(base, off, lds_b + slot * T::BBYTES + it * 1024);
          }
        }
      }
    };
    // tile index / this wave's class of a tile-list entry
    auto entry_tile = [&](uint32_t e) FL_INLINE  { return (int)(__builtin_amdgcn_readfirstlane(e) & 0xffffu); };
    auto entry_class = [&](uint32_t e) FL_INLINE  { return (int)((__builtin_amdgcn_readfirstlane(e) >> (16 + 2 * wave)) & 3u); };

    // whether some wave may apply the element mask to the entry's tile: not when it is FULL (class bits 10) for every
    // wave.  (A tile that is EMPTY for a wave can still lie inside that wave's run, where it is computed and masked.)
    auto entry_masked = [&](uint32_t e) FL_INLINE {
      constexpr uint32_t kAll = (1u << (2 * NW)) - 1u;
      return ((__builtin_amdgcn_readfirstlane(e) >> 16) & kAll) != (0xAAAAu & kAll);
    };

    // ---- S^T = K . Q^T for one tile: A = K fragment from LDS, B = Q fragment ---------------------------------------
    auto qk = [&](f32x16 (&s)[KB][QB], int buf) FL_INLINE {
      const unsigned char* kb_ = smem + T::K_OFF + buf * T::KBYTES;
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
          const ex8 kf = *reinterpret_cast<const ex8*>(kb_ + row * (DQK * 2) + LK::swz_k(row, 2 * ks + h) * 16);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            s[kb][qb] = mfma32(kf, qf[qb][ks], s[kb][qb]);
        }
    };

    // ---- score modifications of one tile; afterwards s * c2 is the logit in log2 units ---------------------------------
    // Register i of block (kb, qb) is key k0 + 32*kb + 8*(i/4) + 4*h + i%4 against query qrow[qb].
    auto score_mods = [&](f32x16 (&s)[KB][QB], int t, int bslot) FL_INLINE {
      const int k0 = t * BN;
      if constexpr (kMod) {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            const int kbase = k0 + 32 * kb + 4 * h;
            const float rel0 = (float)(kbase - qrow[qb]);
            float bv[16];
            // (called once on every path below, so that the path without global loads does not meet the other one
            // before the scores are final: a wait for those loads after the join would run on every tile, and would
            // also wait for the K/V transfers in flight)
            // ALiBi: slope * (rel0 + off) with off a per-register constant; slope * rel0 rides in the addend of the
            // multiply-add that precedes it, leaving one multiply-add with a literal per score
            const float alibi0 = kAlibi ? slope_l2 * rel0 : 0.f;
            const float cap_shift = cap_c + alibi0 - (kFoldRef ? ref_now(qb) : 0.f);
            auto combine_as = [&](auto fn_tag) FL_INLINE {
              constexpr int kFn = decltype(fn_tag)::value;
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const float x = s[kb][qb][i];
                float tl2;
                if constexpr (kNatural) {
                  tl2 = __builtin_fmaf(x, p.scale, bv[i]);  // natural units: one operation per score
                } else {
                  if constexpr (kSoftcap) {
                    const float e = fast_exp2(x * cap_k1);
                    const float rc = fast_rcp(e + 1.0f);
                    tl2 = __builtin_fmaf(rc, -2.0f * cap_c, cap_shift);
                  } else if constexpr (kFn == 1) {
                    tl2 = __builtin_fmaf(fast_rcp(1.0f + fast_exp2(__builtin_fmaf(x, fn_k[0], fn_k[1]))), fn_k[2], fn_k[3]);
                  } else if constexpr (kFn == 2) {
                    tl2 = __builtin_amdgcn_fmed3f(__builtin_fmaf(x, fn_k[0], fn_k[1]), fn_k[2], fn_k[3]);
                  } else if constexpr (kFn == 3) {
                    tl2 = __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(x, fn_k[3], fn_k[2]), x, fn_k[1]), x, fn_k[0]);
                  } else {
                    tl2 = kAlibi ? __builtin_fmaf(x, p.scale_log2, alibi0) : x * p.scale_log2;
                  }
                  if constexpr (kAlibi) tl2 = __builtin_fmaf(slope_l2, (float)(8 * (i / 4) + (i % 4)), tl2);
                  if constexpr (kBias) tl2 = __builtin_fmaf(bv[i], kLog2e, tl2);
                }
                s[kb][qb][i] = tl2;
              }
            };
            // (the kind of score function is uniform: one branch per block, outside the loop over the scores)
            auto combine = [&]() FL_INLINE {
              if constexpr (kScoreFn) {
                if (fn_kind == 1) combine_as(std::integral_constant<int, 1>{});
                else if (fn_kind == 2) combine_as(std::integral_constant<int, 2>{});
                else combine_as(std::integral_constant<int, 3>{});
              } else {
                combine_as(std::integral_constant<int, 0>{});
              }
            };
            if constexpr (kBias) {
#pragma unroll
              for (int i = 0; i < 16; ++i) bv[i] = 0.f;
              if (nbr >= 0) {
                // row-broadcast operand: keys 32 kb + 8 g + 4 h .. + 4 of this wave's staged row
                const unsigned char* bl = smem + T::R_OFF + bslot * T::RBYTES + wave * 1024;
                if (row_f32) {
#pragma unroll
                  for (int g = 0; g < 4; ++g) {
                    const f32x4 b4 = *reinterpret_cast<const f32x4*>(bl + (32 * kb + 8 * g + 4 * h) * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) bv[4 * g + e] += b4[e];
                  }
                } else {
#pragma unroll
                  for (int g = 0; g < 4; ++g) {
                    const ex4 b4 = *reinterpret_cast<const ex4*>(bl + 8 * h + (4 * kb + g) * 16);
#pragma unroll
                    for (int e = 0; e < 4; ++e) bv[4 * g + e] += (float)b4[e];
                  }
                }
              }
              if (nbl >= 0) {
                // staged tile: the same keys of row 32 qb + r from this wave's LDS image
                const int row = 32 * qb + r;
                const unsigned char* bl = smem + T::B_OFF + bslot * T::BBYTES + wave * (RW * BN * 2) + row * (BN * 2) + 8 * h;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                  const ex4 b4 = *reinterpret_cast<const ex4*>(bl + LB::swz(row, 4 * kb + g) * 16);
#pragma unroll
                  for (int e = 0; e < 4; ++e) bv[4 * g + e] += (float)b4[e];
                }
              }
              if (any_direct) {
                // operands that cannot be staged (unaligned rows, ragged key count, a third dense operand): read from
                // global memory where they are used
                for (int nb = 0; nb < 2; ++nb) {
                  if (p.bias[nb] == nullptr || nb == nbr || nb == nbl) continue;
                  const int64_t boff = (int64_t)(batch / p.bdiv[nb]) * p.bs[nb][0] + (int64_t)head * p.bs[nb][1] +
                                       (int64_t)min(qrow[qb], p.Lq - 1) * p.bs[nb][2];
                  if (p.bias_f32[nb]) {
                    const float* fp = reinterpret_cast<const float*>(p.bias[nb]) + boff;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                      const int key = kbase + 8 * g;
                      if (p.bias_vec[nb] && key + 3 < p.Lk) {
                        const f32x4 b4 = *reinterpret_cast<const f32x4*>(fp + key);
#pragma unroll
                        for (int e = 0; e < 4; ++e) bv[4 * g + e] += b4[e];
                      } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                          if (key + e < p.Lk) bv[4 * g + e] += fp[(int64_t)(key + e) * p.bs[nb][3]];
                      }
                    }
                    continue;
                  }
                  const bf16_t* bp = p.bias[nb] + boff;
#pragma unroll
                  for (int g = 0; g < 4; ++g) {
                    const int key = kbase + 8 * g;
                    if (p.bias_vec[nb] && key + 3 < p.Lk) {
                      ex4 b4 = *reinterpret_cast<const ex4*>(bp + key);
#pragma unroll
                      for (int e = 0; e < 4; ++e) bv[4 * g + e] += (float)b4[e];
                    } else {
#pragma unroll
                      for (int e = 0; e < 4; ++e)
                        if (key + e < p.Lk) bv[4 * g + e] += (float)reinterpret_cast<const E*>(bp)[(int64_t)(key + e) * p.bs[nb][3]];
                    }
                  }
                }
                combine();
              } else {
                combine();
              }
            } else {
              combine();
            }
          }
      }
    };
    // Element mask of a tile that is not FULL for this wave: attend iff
    // key < Lk && ((dmin <= key - q <= dmax) || key < pfx) [&& same document]; with key = kbase + off and off a
    // compile-time constant per register, every test compares off with a per-lane bound (branch-free).
    // A tile that is empty for this wave (but not for the workgroup) takes the same path and loses every score.
    // With off = key - kbase a compile-time constant per register, the positional predicate is lo <= off <= hi for
    // per-lane bounds: every mask is one interval of key - q cut at Lk; the prefix-LM mask is the union of two
    // intervals that both start at -inf, i.e. again one (dmin is far below any offset unless a window is set).
    auto apply_mask = [&](f32x16 (&s)[KB][QB], int t, int vslot) FL_INLINE {
      const int k0 = t * BN;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int kbase = k0 + 32 * kb + 4 * h;
        const int t_len = p.Lk - kbase;   // off < t_len   <=> key < Lk
        const int t_pfx = p.pfx - kbase;  // off < t_pfx   <=> key < pfx
        // Under a document mask the ids of this lane's 16 keys come from the wave's LDS image of the tile's ids (it
        // arrived with the V tile in ring slot `vslot`): four runs of four consecutive keys.
        int64_t kdoc[16];
        if constexpr (kDoc) {
          typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
          const unsigned char* il = smem + T::I_OFF + vslot * T::IBYTES + wave * (BN * 8) + (32 * kb + 4 * h) * 8;
#pragma unroll
          for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int e2 = 0; e2 < 2; ++e2) {
              const i64x2 two = *reinterpret_cast<const i64x2*>(il + (8 * g + 2 * e2) * 8);
              kdoc[4 * g + 2 * e2] = two[0];
              kdoc[4 * g + 2 * e2 + 1] = two[1];
            }
        }
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          const int rel = kbase - qrow[qb];
          // off <= hi <=> key < Lk && (key - q <= dmax || key < pfx);  off >= lo <=> key - q >= dmin
          const int hi = min(t_len - 1, max(p.dmax - rel, t_pfx - 1));
          const int lo = p.dmin - rel;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int off = 8 * (i / 4) + (i % 4);
            bool ok = (off <= hi) & (off >= lo);
            if constexpr (kDoc) ok = ok & (kdoc[i] == qdoc[qb]);
            s[kb][qb][i] = ok ? s[kb][qb][i] : -INFINITY;
          }
        }
      }
    };
    auto dump_attended = [&](const f32x16 (&s)[KB][QB], int t) FL_INLINE {
      const int k0 = t * BN;
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
    };

    // ---- A operand of O^T += V^T . P^T for 16-key chunk c and value block dvb, through the transposing LDS read.
    // Slot j of lane (r, h) is key 16c + 8*(j/4) + 4h + j%4, the key order of the packed weights.
    auto v_frag = [&](int buf, int c, int dvb) FL_INLINE -> ex8 {
      const unsigned char* vb_ = smem + T::V_OFF + buf * T::VBYTES;
      ex8 vf;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // within each 16-lane group, lane i supplies row (key) i/4, 4 columns at 4*(i%4), and receives column i
        // of the 4 rows
        const int i16 = lane % 16, g = (lane / 16) % 2;
        const int row = 16 * c + 8 * j + 4 * h + i16 / 4;
        const int col = dvb * 32 + g * 16 + 4 * (i16 % 4);
        const unsigned char* ap = vb_ + row * (DV * 2) + LV::swz_v(row, col / 8) * 16 + (col % 8) * 2;
        typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
        const s16x4 t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(ap));
        const ex4 b4 = __builtin_bit_cast(ex4, t4);
#pragma unroll
        for (int e = 0; e < 4; ++e) vf[4 * j + e] = b4[e];
      }
      return vf;
    };
    // ---- running maximum: row maxima of one tile; the accumulators are rescaled when a maximum grew by more than kTau
    auto row_max = [&](const f32x16 (&s)[KB][QB], float (&mx)[QB]) FL_INLINE {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        float m = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) m = __builtin_fmaxf(m, s[kb][qb][i]);
        mx[qb] = xhalf_max(m);
      }
    };
    auto rescale_if_grown = [&](const float (&mx)[QB], bool force) FL_INLINE {
      bool grow = force;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
        grow = grow | ((mx[qb] - m_run[qb]) * c2 > kTau);  // m_run = -inf before the first tile: always true
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        // (in the units of the scores: s * c2 is in log2 units; worked out here, on the rare path, so that it does not
        // hold a register through the loop)
        const float ref_floor = kBias ? -32768.0f * fast_rcp(c2) : 0.f;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          // Before the first update the reference is 0 (see softmax_p), and tiles may already have been accumulated
          // against it without this function being called (the reference-free path).  The reference then never moves
          // below 0: a tile whose every key carries a huge finite negative term (an additive padding mask such as
          // -1e9 over a ragged last tile) would otherwise pull it down there and scale the accumulated weights up
          // past the largest float.  With nothing accumulated yet the tile's own maximum is taken, whatever it is.
          const bool fresh = m_run[qb] == -INFINITY;
          const float floor_ = (fresh && xhalf_sum(l_run[qb]) > 0.f) ? 0.f : m_run[qb];
          // Nor does it go below -2^15 log2 units: scores further down are additive masks written as finite numbers
          // (-1e9, the element type's most negative value), all of whose weights are zero against any real score.
          // Taken as the reference they would be subtracted from themselves with the rounding of their own magnitude
          // (2^+-64 instead of 1 at -1e9, inf - inf at -3e38); held against this floor their weights are plain zeros.
          // (a row that is fully masked so far takes the floor as its reference too: whatever comes next is above it).
          // Only bias operands bring such numbers: the other kernels keep the plain maximum.
          float m_new = __builtin_fmaxf(floor_, mx[qb]);
          if constexpr (kBias) m_new = __builtin_fmaxf(m_new, ref_floor);
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // row fully masked so far
          // (the clamp keeps 0 * inf out of accumulators whose contents have underflowed to nothing)
          const float m_old = fresh ? 0.f : m_run[qb];
          const float alpha = __builtin_fminf(fast_exp2((m_old - m_use) * c2), 0x1p126f);
          m_run[qb] = m_new;
          l_run[qb] *= alpha;
#pragma unroll
          for (int dvb = 0; dvb < DVB; ++dvb)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[dvb][qb][i] *= alpha;
        }
      }
    };

    // ---- P = exp2(s - m) (bf16 B operand of the second product) and row sums ----------------------------------------------
    // (the row sums take every weight; with dropout the weights that go on to the second product are then thinned:
    // t is the tile, whose keys enter the hash)
    // (kernels whose scores already are relative to a reference pass what the reference has moved by since, or the
    // tag `relative` when it has not moved)
    auto softmax_p = [&](const f32x16 (&s)[KB][QB], ex8 (&pf)[QB][2 * KB], float (&rsum)[QB], int t, auto relative,
                         const float (&moved)[QB]) FL_INLINE {
      const ex2 ones = {(E)1.0f, (E)1.0f};
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float mc = kFoldRef ? moved[qb] : ((m_run[qb] == -INFINITY) ? 0.f : m_run[qb] * c2);
        float rs = 0.f;
        uint32_t drop_x0 = 0;
        if constexpr (kDrop) drop_x0 = drop_q[qb] + (uint32_t)(t * (BN / 2) + 2 * h) * kDropK;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          float pv[16];
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            if constexpr (kFoldRef && decltype(relative)::value) pv[i] = fast_exp2(s[kb][qb][i]);
            else pv[i] = fast_exp2(__builtin_fmaf(s[kb][qb][i], c2, -mc));
          }
#pragma unroll
          for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[qb][2 * kb + j][e] = (E)pv[8 * j + e];
            // the row sum adds up the rounded weights, the very numbers the second product uses (v_dot2 with ones:
            // two weights per instruction)
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              const ex2 pr = {pf[qb][2 * kb + j][e], pf[qb][2 * kb + j][e + 1]};
              rs = dot2acc(pr, ones, rs);
              if constexpr (kDrop) {
                // registers 8j + e, 8j + e + 1 are keys t BN + 32 kb + 8 (2j + e / 4) + 4h + e % 4 and the next one
                // (pair index = (t BN) / 2 + 2h + a constant: one multiply per tile, one add per pair)
                const uint32_t x = drop_x0 + (uint32_t)((32 * kb + 8 * (2 * j + e / 4) + e % 4) / 2) * kDropK;
                const uint32_t m = drop_pair_mask(drop_pair_hash(x), drop_c2);
                const ex2 kept = __builtin_bit_cast(ex2, __builtin_bit_cast(uint32_t, pr) & m);
                pf[qb][2 * kb + j][e] = kept[0];
                pf[qb][2 * kb + j][e + 1] = kept[1];
              }
            }
          }
        }
        rsum[qb] = rs;
      }
    };
    // Tiles that need no element mask skip the row maximum altogether: their weights are formed against the running
    // reference m_run as it stands, and the row sums (needed anyway) tell whether that was safe.  A lane whose sum
    // is not <= kBig (a weight overflowed, or NaN), or whose sum and running sum are both < kTiny (the tile may have
    // underflowed with nothing to be negligible against), sends the wave through the exact path: row maxima, new
    // reference, weights again.  Any reference gives the same O / l; fp32 sums keep their relative precision.
    // ALiBi moves the scores by a large, steady amount from tile to tile; its kernels visit the tiles in descending key
    // order (see list_entry), so that the amount is downwards and the first reference holds.
    // The underflow bound follows the element type: a bf16 weight keeps its 8 bits down to 2^-126, an fp16 weight is
    // subnormal below 2^-14 (absolute error up to 2^-25) and zero below 2^-25.  With a row sum of at least 2^-4 the
    // rounding of one tile's 64 subnormal weights stays below 2^-15 of the sum.
    constexpr float kBig = 0x1p24f, kTiny = std::is_same<typename T::Elem, f16_t>::value ? 0x1p-4f : 0x1p-24f;
    constexpr bool kFastRef = true;
    // Soft-capped scores are bounded, so tiles with an element mask skip the row maximum as well and leave it to the
    // same row-sum test (measured: 2 % on the soft-cap configurations, nothing or a loss on the others).
    constexpr bool kLazyMasked = kFastRef && kSoftcap;
    auto weights_checked = [&](const f32x16 (&s)[KB][QB], ex8 (&pf)[QB][2 * KB], bool check, auto in_loop,
                               ex8 (&vfirst)[DVB], int vslot, int t, auto prefetch_v) FL_INLINE {
      float rs[QB];
      float moved[QB] = {};
      softmax_p(s, pf, rs, t, std::true_type{}, moved);
      if constexpr (decltype(in_loop)::value) {
        // inside the pipelined step the exponentials share a block with the first product's MFMAs (issued by the
        // caller just before): interleave them
        constexpr int NA = KS * KB * QB;
        constexpr int n_exp = 16 * KB * QB;  // per lane: fma + exp per score, one pack and one dot2 per two
        sched_first_product<NA, (n_exp * (kDrop ? 9 : 3) + NA - 1) / NA>();
      }
      if constexpr (decltype(in_loop)::value && decltype(prefetch_v)::value) {
        // the second product's first V fragments are fetched here, ahead of the branch below, so that their LDS
        // latency runs under the exponentials
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb) {
          vfirst[dvb] = v_frag(vslot, 0, dvb);
        }
      }
      if (check) {
        bool bad = false;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) bad = bad | !(rs[qb] <= kBig) | ((rs[qb] < kTiny) & (l_run[qb] < kTiny));
        if (__builtin_amdgcn_ballot_w64(bad) != 0) {
          float mx[QB];
          row_max(s, mx);
          if constexpr (kFoldRef) {
            // the maxima are relative to the reference the scores were formed against, which is still the current one
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
              moved[qb] = ref_now(qb);
              mx[qb] += moved[qb];
            }
          }
          rescale_if_grown(mx, true);
          if constexpr (kFoldRef) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) moved[qb] = ref_now(qb) - moved[qb];
          }
          softmax_p(s, pf, rs, t, std::false_type{}, moved);
        }
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) l_run[qb] += rs[qb];
    };

    // ---- O^T += V^T . P^T: A = V fragment through the transposing LDS read, B = P ---------------------------------------
    // A operand slot j of lane (r, h) for 16-key chunk c is key 16c + 8*(j/4) + 4h + j%4, the key order of pf.
    // `first` holds the fragments of key chunk 0 when the caller has fetched them ahead (HAVE_FIRST)
    auto pv_mma = [&](const ex8 (&pf)[QB][2 * KB], int buf, const ex8 (&first)[DVB], auto have_first) FL_INLINE {
#pragma unroll
      for (int c = 0; c < 2 * KB; ++c)
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb) {
          ex8 vf;
          if (decltype(have_first)::value && c == 0) vf = first[dvb];
          else vf = v_frag(buf, c, dvb);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            oacc[dvb][qb] = mfma32(vf, pf[qb][c], oacc[dvb][qb]);
        }
    };

    if constexpr (kDoc) dma_wait<0>();  // the tile list (issued first thing) has landed
    // (the previous branch is done with the LDS buffers; every wave's share of the tile list is visible to all)
    if (br > 0 || kDoc) __syncthreads();
    if constexpr (kDoc) n_list = __builtin_amdgcn_readfirstlane((int)tlist[-1]);
    // whether the weights of a tile-list entry's tile are formed without looking at its row maxima first
    auto reference_free = [&](uint32_t e) FL_INLINE { return kFastRef && (kLazyMasked || entry_class(e) == TILE_FULL); };
    // Head of a step, vector work only: element mask of the current tile if it is not FULL for this wave, its row
    // maxima, and the (rare) rescale.
    auto settle = [&](f32x16 (&sc)[KB][QB], uint32_t e, int vslot) FL_INLINE {
      const int t = entry_tile(e);
      const bool full = entry_class(e) == TILE_FULL;
      if constexpr (kLazyMasked) {
        if (!full) apply_mask(sc, t, vslot);
      } else if (!full || !kFastRef) {
        if (!full) apply_mask(sc, t, vslot);
        float mx[QB];
        row_max(sc, mx);
        rescale_if_grown(mx, false);
      }
      dump_attended(sc, t);
    };
    // This wave's run [a_live, b_live) of list positions: those whose tiles are not EMPTY for its rows (an EMPTY tile
    // between two others, possible under unsorted document ids, counts as live: it is computed and masked).  Before
    // and after its run the wave takes part in the transfers and barriers of the steps and computes nothing: the far
    // side of the diagonal, the keys outside a window, other documents.  A run starts at an even position (the loops
    // below are unrolled over the two ring slots and entered at slot 0): an EMPTY tile ahead of it is taken into the run
    // and computed and masked like any other.
    auto live_run = [&](int& a_live, int& b_live) FL_INLINE {
      a_live = 0;
      b_live = n_list;
      if constexpr (kDoc) {
        int a = n_list, b = 0;
        for (int base = 0; base < n_list; base += 64) {
          const int i = base + lane;
          const bool live = i < n_list && ((tlist[min(i, n_list - 1)] >> (16 + 2 * wave)) & 3u) != (unsigned)TILE_EMPTY;
          const uint64_t m = __builtin_amdgcn_ballot_w64(live);
          if (m != 0) {
            a = min(a, base + (int)__builtin_ctzll(m));
            b = max(b, base + 64 - (int)__builtin_clzll(m));
          }
        }
        a_live = __builtin_amdgcn_readfirstlane(a);
        b_live = __builtin_amdgcn_readfirstlane(b);
      } else if constexpr (FEAT & F_ALIBI) {  // positions run from the last tile down
        a_live = max(0, t_lo + n_list - 1 - e_hi);
        b_live = min(n_list, t_lo + n_list - e_lo);
      } else {
        a_live = max(0, e_lo - t_lo);
        b_live = min(n_list, e_hi - t_lo + 1);
      }
      if (a_live >= b_live) a_live = b_live = n_list;  // nothing for this wave
      else a_live -= a_live % T::NS;
    };

    if (n_list > 0) {
      constexpr int NS = T::NS;
      constexpr int LPS = T::K_PER_T + T::V_PER_T + T::B_PER_T + T::R_PER_T + T::I_PER_T;  // transfers per thread per step
      // ent[j] = tile-list entry of list position pos + j (the last entry again past the end of the list).  Entries are
      // read from LDS NS steps before they are needed, so the read latency never shows.
      int pos = 0;
      uint32_t ent[NS + 1];
#pragma unroll
      for (int j = 0; j <= NS; ++j) ent[j] = list_entry(j);
      // prologue: K of the first NS tiles and V of the first NS - 1 go to their ring slots; raw S of the first tile
#pragma unroll
      for (int j = 0; j < NS; ++j)
        if (j < n_list) {
          load_k(entry_tile(ent[j]), j);
          load_b(entry_tile(ent[j]), j);
        }
#pragma unroll
      for (int j = 0; j + 1 < NS; ++j)
        if (j < n_list) load_v(entry_tile(ent[j]), j, entry_masked(ent[j]));
      dma_wait<0>();
      __syncthreads();
      int a_live, b_live;
      live_run(a_live, b_live);
      f32x16 s_a[KB][QB], s_b[KB][QB];
      if (a_live == 0 && b_live > 0) {
        qk(s_a, 0);
        score_mods(s_a, entry_tile(ent[0]), 0);
      }
      __syncthreads();  // K slot 0 may be overwritten from here on

      // What every wave does in every step but the workgroup's last, whatever it computes: at the top, the transfers of K
      // NS tiles on into the slot whose tile was consumed in the previous step, and of V NS - 1 tiles on; at the end,
      // the wait for the transfers the next step reads (later ones may stay in flight) and the barrier.
      auto issue_loads = [&](int slot) FL_INLINE -> bool {
        const bool steady = pos + NS < n_list;
        if (steady) {
          load_k(entry_tile(ent[NS]), slot);
          load_b(entry_tile(ent[NS]), slot);  // the bias of this step's tile was consumed at the end of the previous step
        }
        if (pos + NS - 1 < n_list) load_v(entry_tile(ent[NS - 1]), (slot + NS - 1) % NS, entry_masked(ent[NS - 1]));
        return steady;
      };
      auto end_step = [&](bool steady) FL_INLINE {
        if (steady) dma_wait<(NS - 2) * LPS>(); else dma_wait<0>();
        __syncthreads();
        ++pos;
#pragma unroll
        for (int j = 0; j < NS; ++j) ent[j] = ent[j + 1];
        ent[NS] = list_entry(pos + NS);
      };
      // One pipeline step for list position pos with pos % NS == slot: `sc` holds the (score-modified, unmasked)
      // scores of the current tile on entry and `sn` receives those of the next one.  K of list position j lives in K
      // slot j % NS, V likewise.  The body after `settle` is one straight-line block in which the scheduler
      // interleaves both MFMA groups with the exponentials.  The loop unrolls NS steps so that every slot index is a
      // constant and the two score buffers swap roles without copies.
      auto step = [&](f32x16 (&sc)[KB][QB], f32x16 (&sn)[KB][QB], auto slot_tag) FL_INLINE {
        constexpr int slot = decltype(slot_tag)::value;
        // K slot `slot` held this tile's K and V slot `slot - 1` the previous tile's V: both were last read before the
        // barrier that ended the previous step
        const bool steady = issue_loads(slot);
        settle(sc, ent[0], slot);
        ex8 pf[QB][2 * KB];
        // Raised issue priority while this wave has matrix work: of the two waves sharing a SIMD, the one that is in
        // its MFMA phase wins the issue port, which drives the pair into opposite phases (one on the matrix pipe while
        // the other does vector work) instead of both stalling on each other.
        __builtin_amdgcn_s_setprio(3);
        qk(sn, (slot + 1) % NS);
        ex8 vfirst[DVB];
        weights_checked(sc, pf, reference_free(ent[0]), std::true_type{}, vfirst, slot, entry_tile(ent[0]), std::true_type{});
        pv_mma(pf, slot, vfirst, std::true_type{});
        score_mods(sn, entry_tile(ent[1]), (slot + 1) % NS);
        {
          // the next tile's score modifications (if any) go under the second product's MFMAs
          constexpr int NB = 2 * KB * DVB * QB;
          constexpr int mod_ops = (kSoftcap ? 4 : (kMod ? 1 : 0)) + (kAlibi ? 2 : 0) + (kBias ? 3 : 0);
          sched_second_product<NB, (16 * KB * QB * mod_ops + NB - 1) / NB>();
        }
        __builtin_amdgcn_s_setprio(0);
        end_step(steady);
      };
      // steps before this wave's run: transfers and barriers only, except that the step before the run forms the scores
      // of the run's first tile, as every step does for the tile after it
      while (pos < a_live && pos + 1 < n_list) {
        const bool steady = issue_loads(pos % NS);
        if (pos + 1 == a_live) {
          qk(s_a, 0);
          score_mods(s_a, entry_tile(ent[1]), 0);
        }
        end_step(steady);
      }
      if (pos >= a_live && pos < b_live) {
      int last_slot = 0;  // ring slot of the run's final tile; its scores are in s_a when the slot is even
      bool more = true;
      while (more) {
        more = static_while<0, NS>([&](auto idx) FL_INLINE  {
          constexpr int slot = decltype(idx)::value;
          if (!(pos + 1 < b_live)) {
            last_slot = slot;
            return false;
          }
          if constexpr (slot % 2 == 0) step(s_a, s_b, idx); else step(s_b, s_a, idx);
          return true;
        });
      }
      // the run's last tile: no scores of a next tile to form; the step's transfers and barrier only if the workgroup
      // has further steps
      const bool more_steps = pos + 1 < n_list;
      bool steady_tail = false;
      if (more_steps) steady_tail = issue_loads(last_slot);
      static_while<0, NS>([&](auto idx) FL_INLINE  {
        constexpr int slot = decltype(idx)::value;
        if (last_slot != slot) return true;
        ex8 pf[QB][2 * KB];
        ex8 vfirst[DVB];
        if constexpr (slot % 2 == 0) {
          settle(s_a, ent[0], slot);
          weights_checked(s_a, pf, reference_free(ent[0]), std::false_type{}, vfirst, slot, entry_tile(ent[0]), std::false_type{});
        } else {
          settle(s_b, ent[0], slot);
          weights_checked(s_b, pf, reference_free(ent[0]), std::false_type{}, vfirst, slot, entry_tile(ent[0]), std::false_type{});
        }
        pv_mma(pf, slot, vfirst, std::false_type{});
        return false;
      });
      if (more_steps) end_step(steady_tail);
      }
      // steps after the run
      while (pos + 1 < n_list) {
        const bool steady = issue_loads(pos % NS);
        end_step(steady);
      }
    }

    // ---- normalise this branch ---------------------------------------------------------------------------------
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float l = xhalf_sum(l_run[qb]);
      float inv = l > 0.f ? 1.0f / l : 0.f;  // a row that attends nothing yields zeros
      if constexpr (kDrop) inv *= p.drop_rescale;  // the row sum counted every weight; the kept ones are scaled up
      if constexpr (!kDiff) {
        // row statistic for a backward pass: weights were exp2(s * c2 - m_run * c2), so the row's log2-sum-exp2 is
        if (p.lse != nullptr && h == 0 && qrow[qb] < p.Lq) {
          const float mc = (m_run[qb] == -INFINITY) ? 0.f : m_run[qb] * c2;
          p.lse[((int64_t)batch * p.Hq + head) * p.Lq + qrow[qb]] = l > 0.f ? mc + __builtin_log2f(l) : INFINITY;
        }
      }
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
  const bool wide = __builtin_amdgcn_readfirstlane(p.o_wide) != 0;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    // (the wide path trades register halves between the two lanes of a query: rows past Lq go along and store nothing)
    if (!wide && qrow[qb] >= p.Lq) continue;
#pragma unroll
    for (int dvb = 0; dvb < DVB; ++dvb) {
      ex4 quad[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int dv = 32 * dvb + 8 * g + 4 * h;
        ex4 o4;
        if (kGate && gptr) {
          ex4 g4;
          if constexpr (kGateEarly) g4 = gpre[dvb][qb][g];
          else g4 = *reinterpret_cast<const ex4*>(gptr + (int64_t)min(qrow[qb], p.Lq - 1) * p.gs[2] + dv);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float sg = fast_rcp(1.0f + fast_exp2(-kLog2e * (float)g4[e]));
            o4[e] = (E)(oacc[dvb][qb][4 * g + e] * sg);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = (E)oacc[dvb][qb][4 * g + e];
        }
        quad[g] = o4;
      }
      if (wide) {
        // the two lanes of a query trade halves of two groups of 4 columns, after which the first holds columns
        // 16 j .. + 8 of the block and the second the next 8: 16-byte stores, half as many partial lines per store
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const u32x2 qa = __builtin_bit_cast(u32x2, quad[2 * j]), qb_ = __builtin_bit_cast(u32x2, quad[2 * j + 1]);
          uint32_t a0 = qa[0], a1 = qa[1], b0 = qb_[0], b1 = qb_[1];
          swap_halves(a0, b0);
          swap_halves(a1, b1);
          const u32x4 w = {a0, a1, b0, b1};
          if (qrow[qb] < p.Lq) *reinterpret_cast<u32x4*>(optr + (int64_t)qrow[qb] * p.os[2] + 32 * dvb + 16 * j + 8 * h) = w;
        }
      } else {
#pragma unroll
        for (int g = 0; g < 4; ++g)
          *reinterpret_cast<ex4*>(optr + (int64_t)qrow[qb] * p.os[2] + 32 * dvb + 8 * g + 4 * h) = quad[g];
      }
    }
  }
}

}  // namespace fl
