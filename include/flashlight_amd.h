/*
 * flashlight_amd.h -- C ABI of libflashlight_amd.so
 *
 * Fused FlashAttention-style forward kernels for gfx950 (MI355X), one launch per call:
 * QK^T on bf16 MFMA -> score modification / masking in registers -> online softmax ->
 * P.V on MFMA -> normalise -> bf16 store.  Tiles whose mask is empty are never visited.
 *
 * The reference (bozhiyou/flashlight) has no FFI: its boundary for this path is the set
 * of eager PyTorch functions under attention_variants/ that callers wrap in
 * torch.compile (tests/test_causal.py:14-17,33; benchmarks/run_flex_variants.py:118-147).
 * What torch.compile + monkeypatch/fusion generate for those functions (one fused Triton
 * kernel, monkeypatch/fusion/block_reduction.py:1302-1522) is what fl_attn_fwd replaces.
 * Each field below cites the reference argument it carries.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; the library never allocates,
 *     frees or retains device memory and never synchronises: work is queued on `stream`.
 *   - strides are in ELEMENTS, order [batch, head, seq, dim]; the dim stride must be 1.
 *   - return value: 0 ok; <0 invalid argument (nothing was launched, see fl_last_error());
 *     >0 a hipError_t from the launch.
 *   - re-entrant; the only mutable state is the thread-local error string.
 */
#ifndef FLASHLIGHT_AMD_H
#define FLASHLIGHT_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FL_ABI_VERSION 1

/* Which (q, k) pairs are attended.  q, k are 0-based positions, top-left aligned. */
enum fl_mask_kind {
  FL_MASK_NONE = 0,       /* vanilla.py:20-35, alibi.py:13-33, softcap.py:4-53, diff_attn.py:6-30, evoformer.py:8-36 */
  FL_MASK_CAUSAL = 1,     /* k <= q                      causal.py:32-33 */
  FL_MASK_SLIDING = 2,    /* 0 <= q - k <= window        sliding_window.py:4-12 (window+1 keys) */
  FL_MASK_PREFIX_LM = 3,  /* k < prefix || k <= q        prefix_lm.py:33-42 */
  FL_MASK_DOCUMENT = 4,   /* doc[q] == doc[k]            document_mask.py:25-27 */
  FL_MASK_DOCUMENT_CAUSAL = 5 /* doc[q] == doc[k] && k <= q  (what the reference's Flex baseline computes,
                                 benchmarks/run_flex_variants.py:86) */
};

enum fl_dtype { FL_BF16 = 0, FL_F32 = 1, FL_F16 = 2 };

/* error codes (negative) */
#define FL_ERR_NULL (-1)
#define FL_ERR_SHAPE (-2)
#define FL_ERR_STRIDE (-3)
#define FL_ERR_UNSUPPORTED (-4)
#define FL_ERR_ARG (-5)
#define FL_ERR_WORKSPACE (-6)
#define FL_ERR_ALIGN (-7)

typedef struct fl_attn_params {
  /* query [B, Hq, Lq, Dqk], key [B, Hkv, Lk, Dqk], value [B, Hkv, Lk, Dv], out [B, Hq, Lq, Dv]
   * (causal.py:8-10).  With diff != 0, query/key hold 2*Hq / 2*Hkv heads: heads [0, H) feed softmax 0
   * and heads [H, 2H) feed softmax 1 (diff_attn.py:14-17). */
  const void* q;
  const void* k;
  const void* v;
  void* o;
  int64_t q_strides[4], k_strides[4], v_strides[4], o_strides[4];
  int32_t B, Hq, Hkv, Lq, Lk, Dqk, Dv;
  /* multiplies QK^T before anything else (`scale` / `sm_scale` of every reference function); must be > 0 */
  float scale;

  int32_t mask_kind; /* enum fl_mask_kind */
  int32_t window;    /* FL_MASK_SLIDING: `window_size` of sliding_window.py:14 */
  int32_t prefix;    /* FL_MASK_PREFIX_LM: `prefix_lengths` of prefix_lm.py:5 */
  /* FL_MASK_DOCUMENT*: `document_id`, int64 [B, L] with Lq == Lk (document_mask.py:10,25-27); any integers */
  const int64_t* doc_ids;
  int64_t doc_stride; /* elements between batches */

  /* score = softcap_or_identity(qk * scale) + alibi + bias[0] + bias[1], then the mask.
   * alibi_heads > 0 adds 2^(-8 (h+1) / alibi_heads) * (k - q) for query head h (alibi.py:5-9).
   * softcap > 0 applies softcap * tanh(x / softcap) (softcap.py:48). */
  int32_t alibi_heads;
  float softcap;

  /* Optional additive biases (evoformer.py:26-27; the dense fp32 tensor `score_mod(L, S)` of alibi.py:26),
   * logical shape [B, Hq, Lq, Lk] with strides in elements over (batch / bias_batch_div, head, q, k); a
   * stride of 0 broadcasts; the k stride must be 1 (or 0 when Lk == 1).  bias_dtype (below) says per operand
   * whether its elements are fp32 or of the same 16-bit type as q. */
  const void* bias[2];
  int64_t bias_strides[2][4];
  int32_t bias_batch_div[2];

  /* Optional sigmoid gate: out *= sigmoid(gate); bf16 gate logits addressed like `o` with gate_strides.
   * No counterpart in the reference (Evoformer gating is applied outside evoformer.py:8-36). */
  const void* gate;
  int64_t gate_strides[4];

  /* diff != 0: out = softmax(q0 k0^T) v - lambda * softmax(q1 k1^T) v  (diff_attn.py:29) */
  int32_t diff;
  float lambda;

  int32_t dtype; /* element type of q, k, v, o and gate: FL_BF16 or FL_F16 (the reference's typing admits both,
                  * monkeypatch/fusion/_reduction.py:55-57) */

  /* Scratch of document-mask calls (the forward's lists of key tiles per query tile, the backward's table of id
   * ranges); size from fl_workspace_bytes(), 16-byte aligned; may be NULL otherwise. */
  void* workspace;
  uint64_t workspace_bytes;

  /* Test hook: when non-NULL, a uint8 [B, Hq, Lq, Lk] buffer, zeroed by the caller; the kernel writes 1
   * for every (q, k) pair it attends (after tile skipping and the element predicate). */
  uint8_t* attended_dump;

  int32_t bias_dtype[2]; /* element type of bias[0], bias[1]: FL_F32, or the same as `dtype` */

  /* Optional output for a later fl_attn_bwd: fp32 [B, Hq, Lq], contiguous; per query row the base-2 logarithm of
   * the sum over attended keys of 2^(score * log2(e)) (+inf for a row that attends nothing).  Not with diff. */
  float* lse;

  /* Dropout on the softmax weights (torch.nn.functional.dropout semantics: the row normalisation counts every weight,
   * kept weights are scaled by 65536 / (65536 - dropout_threshold)).  The reference's functions accept `dropout_p` and
   * ignore it (attention_variants/causal.py:4-36, alibi.py:13-33, softcap.py:4-53); 0 here does the same.
   * dropout_threshold = round(p * 65536), 1 .. 65535: a weight is dropped when the 16 bits a counter-based hash of
   * (dropout_seed, batch * Hq + head, query, key) gives it are below the threshold.  fl_attn_bwd regenerates the same
   * decisions from the same fields.  With every mask kind, GQA, ALiBi, the soft-cap, bias operands and the gate, in any
   * combination; not with differential attention, score_fn or the dump hook; Dqk = Dv in {64, 128}. */
  uint32_t dropout_threshold;
  uint32_t dropout_seed[2]; /* low, high half of a 64-bit seed */

  /* Bit set of FL_FLAG_*; unknown bits are rejected.  No counterpart in the reference. */
  uint32_t flags;

  /* A function of the scaled score other than the tanh soft-cap, applied where `softcap` would be: the reference's
   * softcap.py:49 calls an arbitrary score_mod(score, b, h, q_idx, kv_idx) on the score matrix inside its fused kernel;
   * this is the part of that freedom the kernel has compiled in.  With z = qk * scale:
   *   FL_SCORE_SIGMOID  y = p[2] * sigmoid(p[0] * z + p[1]) + p[3]
   *   FL_SCORE_CLAMP    y = min(max(p[0] * z + p[1], p[2]), p[3])      (p[2] <= p[3], either may be infinite: a ReLU
   *                                                                     is (1, 0, 0, +inf))
   *   FL_SCORE_POLY     y = p[0] + p[1] z + p[2] z^2 + p[3] z^3
   * y takes the place of the scaled score (biases and the mask follow).  Positional masks, grouped heads and bias
   * operands go with it; soft-cap, ALiBi, document masks, gate, differential attention, dropout and fl_attn_bwd do
   * not.  Head dims 64 and 128. */
  int32_t score_fn; /* FL_SCORE_NONE (0, what a zeroed struct says) or one of the above */
  float score_fn_params[4];
} fl_attn_params;

#define FL_SCORE_NONE 0
#define FL_SCORE_SIGMOID 1
#define FL_SCORE_CLAMP 2
#define FL_SCORE_POLY 3

/* fl_attn_fwd, document masks only: `workspace` still holds what an earlier fl_attn_fwd call (without this flag) wrote
 * there for the same doc_ids contents, doc_stride, B, Lq = Lk, mask_kind, head dims, dtype and features, and the
 * pre-pass that derives the key-tile lists from the ids is skipped.  For callers that run many layers over one packed
 * batch, as the reference's Flex baseline builds its block mask once (benchmarks/run_flex_variants.py:66-90).  The ids
 * are still read by the kernel itself; passing other ids than the workspace was prepared for gives wrong results. */
#define FL_FLAG_DOC_PREPARED 1u

/* ABI version of the loaded library (FL_ABI_VERSION it was built with). */
int fl_version(void);

/* sizeof(fl_attn_params) in the loaded library, for bindings to check their own mirror of the struct. */
uint64_t fl_params_sizeof(void);

/* Message for the last negative/positive return on this thread ("" if none). */
const char* fl_last_error(void);

/* Host-only argument check: the same validation fl_attn_fwd runs before it launches.  Touches no GPU. */
int fl_attn_validate(const fl_attn_params* p);

/* Bytes of device scratch fl_attn_fwd needs in `workspace` for *p (0 unless a document mask is used): the key tiles
 * every query tile visits, so the figure grows with Lq * Lk / (rows per workgroup * keys per tile).  Enough for
 * fl_attn_bwd as well. */
uint64_t fl_workspace_bytes(const fl_attn_params* p);

/* Bytes of device scratch fl_attn_bwd alone needs in fwd.workspace (0 unless a document mask is used): 16 bytes per 32
 * positions of every batch row.  No counterpart in the reference. */
uint64_t fl_bwd_workspace_bytes(const fl_attn_params* p);

/* Runs the fused forward on hipStream_t `stream` (NULL = default stream).
 * Replaces torch.compile(fn)(q, k, v, ...) for the functions of attention_variants/. */
int fl_attn_fwd(const fl_attn_params* p, void* stream);

/* Describes the kernel instance fl_attn_fwd would pick for *p: tile sizes and launch shape.
 * out[0]=rows per workgroup, out[1]=keys per tile, out[2]=threads, out[3]=workgroups, out[4]=LDS bytes,
 * out[5]=feature bits of the instance, out[6]=1 when the call goes to the shared-bias streaming kernel instead (head
 * dim 32, one dense bias shared by several batch entries, 256 / 320 / 384 keys: the Evoformer shape). */
int fl_attn_plan(const fl_attn_params* p, int64_t out[8]);

/* Backward of fl_attn_fwd.  No counterpart in the reference, which is forward-only (its FLOP helper models a
 * backward pass, benchmarks/_utils.py:16-21, but no kernel or autograd rule exists): the textbook gradients of
 * softmax attention, recomputing the weights from the forward's row statistics.
 * `fwd` describes the forward call whose gradients are wanted: same q, k, v, sizes, scale, mask and score
 * modification; fwd.o is the forward's output and fwd.lse the row statistics that call wrote.  Supported: every mask
 * kind, grouped-query heads, ALiBi, the tanh soft-cap and bias operands (fwd.bias, as in the forward) in any
 * combination, with or without dropout (dropout: head dims 64 and 128); Dqk == Dv in {32, 64, 128}.
 * Not supported (FL_ERR_UNSUPPORTED): gate, differential attention
 * (both are compositions of calls that are supported: out * sigmoid(gate); one call per branch and half of the value
 * columns), the attended_dump hook.
 * dout [B, Hq, Lq, Dv] is the gradient of the output; dq [B, Hq, Lq, Dqk], dk [B, Hkv, Lk, Dqk], dv [B, Hkv, Lk, Dv]
 * receive the gradients (element type fwd.dtype like dout; strides in elements, last stride 1, others multiples of 8).
 * delta: caller-provided scratch of B * Hq * Lq floats; delta and fwd.lse must be 16-byte aligned.
 * fwd.workspace: fl_bwd_workspace_bytes(&fwd) bytes of scratch under a document mask. */
typedef struct fl_attn_bwd_params {
  fl_attn_params fwd;
  const void* dout;
  int64_t dout_strides[4];
  void* dq;
  void* dk;
  void* dv;
  int64_t dq_strides[4], dk_strides[4], dv_strides[4];
  float* delta;
  /* Optional, with bias operands: fp32 [B, Hq, Lq, Lk], contiguous, 16-byte aligned.  Receives the gradient of the
   * loss with respect to the score of every (query, key) pair, i.e. with respect to whatever was added to q k^T * scale:
   * the gradient of a bias operand is this array summed over the axes (and batch entries) the operand broadcasts
   * over.  Only key tiles that some query of the workgroup attends are written (zeros where a pair is masked inside
   * them): clear the array before the call.  Not under a soft-cap (the bias is added after the cap, and the kernels
   * keep only the gradient with respect to the capped product there). */
  float* dscores;
  int32_t reserved[6]; /* must be 0 */
} fl_attn_bwd_params;

/* sizeof(fl_attn_bwd_params) in the loaded library. */
uint64_t fl_bwd_params_sizeof(void);

/* Host-only argument check of a backward call. */
int fl_attn_bwd_validate(const fl_attn_bwd_params* p);

/* Launches the three backward kernels (row sums of dO o O, then dQ, then dK and dV) on `stream`. */
int fl_attn_bwd(const fl_attn_bwd_params* p, void* stream);

/* fl_attn_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight training loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as fl_attn_bwd,
 * except that p->delta and p->fwd.workspace / workspace_bytes are ignored: the row sums and the document table live in
 * a static device array inside the library (FL_STATIC_SCRATCH_BYTES per GPU, held until the process ends), whose
 * address is looked up once per device on the first call made with that device current.  A call that needs more
 * (4 bytes per query row of every head, rounded up to 256, plus fl_bwd_workspace_bytes()) returns FL_ERR_WORKSPACE and
 * launches nothing.  Calls no hipMalloc / hipFree and no allocating library routine (one event per GPU is created on the
 * first call there).  All calls on one GPU share the array, so two such calls that overlap on that GPU would race:
 * calls queued on one stream are ordered and safe; a call on another stream while the previous call's kernels are
 * still running returns FL_ERR_WORKSPACE and launches nothing (queue them on one stream, or wait for the first).  Calls
 * made under stream capture are outside this check, and so are the replays of the graphs they build: ordering those
 * against other users of the array is the caller's.  Nothing in the array needs clearing between calls: each call
 * rewrites what it reads. */
#define FL_STATIC_SCRATCH_BYTES (8u << 20)
int fl_attn_bwd_static(const fl_attn_bwd_params* p, void* stream);
/* FL_STATIC_SCRATCH_BYTES of the loaded library. */
uint64_t fl_static_scratch_bytes(void);

/* Operand packing for invariant point attention (tests/test_ipa.py:57-125, a test-only function of the reference):
 * builds the concatenated operands with which the function becomes one fl_attn_fwd call.  All tensors are bf16,
 * contiguous, `rows` = batch * heads * residues rows each:
 *   q_cat[row] = [q_scalar[row] * q_scale | q_points[row] | 0...]   (dqk columns)
 *   k_cat[row] = [k_scalar[row]           | k_points[row] | 0...]
 *   v_cat[row] = [v_scalar[row]           | v_points[row] | 0...]   (dv columns)
 *   key_term[row] = point_weight * sum(k_points[row]^2)              (fp32)
 * The squared-distance term of test_ipa.py:102-108 then equals -2 * point_weight * (q_points . k_points) + key_term[k]
 * plus a term that is constant along a softmax row. */
typedef struct fl_ipa_pack_params {
  const void *q_scalar, *k_scalar, *v_scalar; /* [rows, c_qk], [rows, c_qk], [rows, c_v] */
  const void *q_points, *k_points, *v_points; /* [rows, n_qk_coords], [rows, n_qk_coords], [rows, n_v_coords] */
  void *q_cat, *k_cat, *v_cat;                /* [rows, dqk], [rows, dqk], [rows, dv] */
  float* key_term;                            /* [rows] */
  int64_t rows;
  int32_t c_qk, c_v, n_qk_coords, n_v_coords, dqk, dv;
  float q_scale, point_weight;
} fl_ipa_pack_params;
int fl_ipa_pack(const fl_ipa_pack_params* p, void* stream);

/* Merges partial results of one attention over `chunks` disjoint chunks of its keys (no counterpart in the reference,
 * whose kernel walks all keys of a row in one program, monkeypatch/fusion/reduction_kernel_fusion.py:1102; used by the
 * front end for decoding steps, where a few query rows meet a long key sequence and the chunks run as extra heads of
 * one fl_attn_fwd launch).  part [outer, chunks, inner, dv] (element type `dtype`, contiguous) holds the chunks' results
 * as fl_attn_fwd wrote them, lse [outer, chunks, inner] the row statistics of the same launch (fl_attn_params.lse: +inf
 * for a row that attends nothing in a chunk); out [outer, inner, dv] receives sum_c w_c part_c / sum_c w_c with
 * w_c = 2^(lse_c - max_c lse_c), zeros for a row that attends nothing at all.  dv even. */
int fl_attn_merge_chunks(const void* part, const float* lse, void* out, int64_t outer, int32_t chunks, int64_t inner,
                         int32_t dv, int32_t dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHLIGHT_AMD_H */
