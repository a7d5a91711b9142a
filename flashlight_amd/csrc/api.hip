// C ABI of libflashlight_amd.so: argument validation (host only), instance selection, launch.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "flashlight_amd.h"
#include "bwd_instances.h"
#include "instances.h"
#include "pairbias_instances.h"

namespace fl {
// Builds (min, max) of the document ids of every block of kDocBlock positions.
static __global__ void doc_table_kernel(const int64_t* ids, int64_t ids_stride, int L, int nblocks, int total, int64_t* table) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  int b = i / nblocks, blk = i % nblocks;
  const int64_t* p = ids + (int64_t)b * ids_stride;
  int p0 = blk * kDocBlock, p1 = min(L, p0 + kDocBlock);
  // (the loads are independent of one another: unrolled, they are all in flight together instead of one round trip
  // to memory each; positions past the end repeat the last one)
  int64_t x[kDocBlock];
#pragma unroll
  for (int j = 0; j < kDocBlock; ++j) x[j] = p[min(p0 + j, p1 - 1)];
  int64_t mn = x[0], mx = x[0];
#pragma unroll
  for (int j = 1; j < kDocBlock; ++j) {
    mn = x[j] < mn ? x[j] : mn;
    mx = x[j] > mx ? x[j] : mx;
  }
  table[2 * (int64_t)i] = mn;
  table[2 * (int64_t)i + 1] = mx;
}

// (min, max) over a wave of one int64 per lane, wave-uniform.  Nearly every 32- or 64-position run lies inside one
// document, so "all equal to the first lane's" is tested with one ballot before the reduction.
static __device__ __forceinline__ void wave_id_range(int64_t x, int64_t& mn, int64_t& mx) {
  const int64_t first = uniform_i64(x);
  mn = mx = first;
  if (__builtin_amdgcn_ballot_w64(x != first) != 0) {
    int64_t a = x, b = x;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const int64_t a2 = __shfl_xor(a, d, 64), b2 = __shfl_xor(b, d, 64);
      a = a2 < a ? a2 : a;
      b = b2 > b ? b2 : b;
    }
    mn = uniform_i64(a);
    mx = uniform_i64(b);
  }
}

// Forward pre-pass for document masks, one workgroup of 1024 threads per (batch, query tile of `bm` rows), straight from
// the ids: lists the key tiles (of `bn` keys) that some row of the query tile attends, with the class of each for every
// wave of the forward (`rw` rows per wave): EMPTY when the id ranges of the tile's keys and the wave's rows do not meet,
// FULL when both are the same single id and the positional part of the mask agrees, PARTIAL otherwise.  Valid for
// arbitrary (unsorted, negative) ids.  The lists are the same for every head.  Output per workgroup: word 0 = number of
// entries, then the entries in key order (bits 0-15 tile index, two class bits per wave from bit 16 on).
// Three phases: a wave per key tile reads its ids with one coalesced load and leaves their (min, max) in LDS (every
// load of a wave is in flight before the first is looked at: the kernel is a chain of round trips to memory with little
// to do in between); a thread per key tile classifies it for every wave; one wave compacts the non-empty entries.
static __global__ __launch_bounds__(1024) void doc_lists_kernel(const int64_t* ids, int64_t ids_stride, int L, int mask_kind,
                                                                int bm, int rw, int bn, int n_qtiles, int nk, int list_stride,
                                                                uint32_t* lists) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  int64_t* krange = reinterpret_cast<int64_t*>(lds_raw);                // [nk][2] = (min, max) id of a key tile
  uint32_t* tl = reinterpret_cast<uint32_t*>(lds_raw + (size_t)nk * 16);  // [nk] uncompacted entries
  __shared__ int64_t qrange[16];  // (min, max) id of the rows of each of up to 8 waves of the forward
  constexpr int kWaves = 16, kBatch = 16;
  const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int b = blockIdx.x / n_qtiles, qt = blockIdx.x % n_qtiles;
  const int nw = bm / rw, q0 = qt * bm;
  const int64_t* idb = ids + (int64_t)b * ids_stride;
  // rows past L repeat the last row (a wave without valid rows is EMPTY for every tile whatever its range)
  const int64_t qid = idb[min(q0 + min(wave, nw - 1) * rw + lane % rw, L - 1)];
  // key tiles some row may attend under the positional part of the mask: all of them, or those up to the diagonal
  const int t_end = mask_kind == MASK_DOC_CAUSAL ? min(nk, (min(q0 + bm, L) - 1) / bn + 1) : nk;
  const int nj = (bn + 63) / 64;  // loads per lane that cover one tile's ids
  for (int t0 = wave; t0 < t_end || t0 == wave; t0 += kWaves * kBatch) {
    int64_t lo[kBatch], hi[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int k0 = min(t0 + kWaves * u, t_end - 1) * bn;
      lo[u] = hi[u] = idb[min(k0 + lane % bn, L - 1)];
      for (int j = 1; j < nj; ++j) {
        const int64_t x = idb[min(k0 + j * 64 + lane, L - 1)];
        lo[u] = x < lo[u] ? x : lo[u];
        hi[u] = x > hi[u] ? x : hi[u];
      }
    }
    if (t0 == wave) {  // (every wave passes here exactly once)
      int64_t mn, mx;
      wave_id_range(qid, mn, mx);
      if (lane == 0 && wave < nw) {
        qrange[2 * wave] = mn;
        qrange[2 * wave + 1] = mx;
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int t = t0 + kWaves * u;
      if (t >= t_end) break;
      int64_t kmn, kmx, unused;
      wave_id_range(lo[u], kmn, unused);
      if (nj > 1) wave_id_range(hi[u], unused, kmx); else kmx = unused;
      if (lane == 0) {
        krange[2 * t] = kmn;
        krange[2 * t + 1] = kmx;
      }
    }
  }
  __syncthreads();
  for (int t = tid; t < t_end; t += 1024) {
    const int k0 = t * bn, k1 = min(k0 + bn, L);
    const int64_t kmn = krange[2 * t], kmx = krange[2 * t + 1];
    unsigned c = 0;
    for (int w = 0; w < nw; ++w) {
      const int a = q0 + w * rw, e = min(a + rw, L);
      const int64_t qmn = qrange[2 * w], qmx = qrange[2 * w + 1];
      int cw = TILE_EMPTY;
      if (a < e) {
        cw = classify_positional(mask_kind, a, e, k0, k1, 0, 0);
        if (kmx < qmn || kmn > qmx) cw = TILE_EMPTY;
        else if (!(kmn == kmx && qmn == qmx && kmn == qmn) && cw == TILE_FULL) cw = TILE_PARTIAL;
        if (cw == TILE_FULL && k0 + bn > L) cw = TILE_PARTIAL;  // ragged tail: keys >= L are masked
      }
      c |= (unsigned)cw << (2 * w);
    }
    tl[t] = (c << 16) | (unsigned)t;
  }
  __syncthreads();
  if (wave == 0) {
    uint32_t* out = lists + (int64_t)blockIdx.x * list_stride;
    int count = 0;
    for (int base = 0; base < t_end; base += 64) {
      const int t = base + lane;
      const uint32_t e = t < t_end ? tl[t] : 0u;
      const bool keep = (e >> 16) != 0;
      const uint64_t m = __builtin_amdgcn_ballot_w64(keep);
      const int pos = count + __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0));
      if (keep) out[1 + pos] = e;
      count += __builtin_popcountll(m);
    }
    if (lane == 0) out[0] = (uint32_t)count;
  }
}

// Second step of the forward pre-pass for document masks, one workgroup per batch row: the query tiles ordered by
// falling length of their tile lists (ties by falling index), by counting for every tile how many come before it.
static __global__ __launch_bounds__(1024) void doc_order_kernel(const uint32_t* lists, int list_stride, int n_qtiles,
                                                               int32_t* order) {
  extern __shared__ uint32_t cnt[];  // n_qtiles words
  const int b = blockIdx.x;
  const uint32_t* lb = lists + (int64_t)b * n_qtiles * list_stride;
  for (int i = threadIdx.x; i < n_qtiles; i += 1024) cnt[i] = lb[(int64_t)i * list_stride];
  __syncthreads();
  for (int i = threadIdx.x; i < n_qtiles; i += 1024) {
    const uint32_t mine = cnt[i];
    int rank = 0;
    for (int j = 0; j < n_qtiles; ++j) rank += (cnt[j] > mine) || (cnt[j] == mine && j > i);
    order[(int64_t)b * n_qtiles + rank] = i;
  }
}

}  // namespace fl

// Scratch of the entry point that allocates nothing (fl_attn_bwd_static): one copy per GPU the library runs on, held
// until the process ends.  In host code this name is only a handle for hipGetSymbolAddress; kernels and memory calls
// take the device address that call returns (static_scratch_ptr below).
constexpr size_t kStaticScratchBytes = (size_t)FL_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

extern "C" uint64_t fl_bwd_workspace_bytes(const fl_attn_params* p);

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};
int static_scratch_ptr(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(FL_ERR_UNSUPPORTED, "device ordinal %d is beyond the %d this library tracks", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail((int)(e != hipSuccess ? e : hipErrorInvalidSymbol), "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// Guard of the static scratch: one event per device, recorded behind every eager fl_attn_bwd_static call.  A call on
// another stream while that event has not completed would share the array with kernels still running: it is refused
// instead.  Calls on the stream of the previous call are ordered behind it and pass; calls under stream capture are
// neither checked nor recorded (a graph's replays are the caller's to order).
struct ScratchGuard {
  hipEvent_t done = nullptr;
  hipStream_t last = nullptr;
  bool armed = false;
};
ScratchGuard g_scratch_guard[kMaxDevices];

bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st == hipStreamCaptureStatusActive;
}

// 0 when the scratch of the current device may be used by a call on `s`.
int static_scratch_acquire(hipStream_t s, int* dev_out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(FL_ERR_UNSUPPORTED, "no current device the library tracks");
  *dev_out = dev;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ScratchGuard& g = g_scratch_guard[dev];
  if (!g.done) {
    e = hipEventCreateWithFlags(&g.done, hipEventDisableTiming);
    if (e != hipSuccess) return fail((int)e, "hipEventCreateWithFlags failed: %s", hipGetErrorString(e));
  }
  if (g.armed && g.last != s) {
    e = hipEventQuery(g.done);
    if (e == hipErrorNotReady) {
      (void)hipGetLastError();
      return fail(FL_ERR_WORKSPACE,
                  "fl_attn_bwd_static: the static scratch of this GPU is still in use by a call on another stream; queue "
                  "such calls on one stream, wait for the earlier one, or use fl_attn_bwd with buffers of your own");
    }
    if (e != hipSuccess) return fail((int)e, "hipEventQuery failed: %s", hipGetErrorString(e));
  }
  return 0;
}

void static_scratch_release(hipStream_t s, int dev) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ScratchGuard& g = g_scratch_guard[dev];
  if (g.done && hipEventRecord(g.done, s) == hipSuccess) {
    g.last = s;
    g.armed = true;
  } else {
    (void)hipGetLastError();
  }
}

bool is_doc(int kind) { return kind == FL_MASK_DOCUMENT || kind == FL_MASK_DOCUMENT_CAUSAL; }

uint32_t wanted_features(const fl_attn_params* p) {
  uint32_t f = 0;
  if (p->alibi_heads > 0) f |= fl::F_ALIBI;
  if (p->softcap > 0.f) f |= fl::F_SOFTCAP;
  if (p->score_fn != FL_SCORE_NONE) f |= fl::F_SCOREFN;
  if (p->bias[0] || p->bias[1]) f |= fl::F_BIAS;
  if (is_doc(p->mask_kind)) f |= fl::F_DOC;
  if (p->diff) f |= fl::F_DIFF;
  if (p->gate) f |= fl::F_GATE;
  if (p->attended_dump) f |= fl::F_DUMP;
  if (p->dropout_threshold) f |= fl::F_DROPOUT;
  return f;
}

// Features a kernel may be compiled with yet leave unused at run time (null pointer / zero slope).
constexpr uint32_t kOptionalFeatures = fl::F_ALIBI | fl::F_BIAS | fl::F_GATE;

const fl::Instance* select_instance(const fl_attn_params* p) {
  const uint32_t want = wanted_features(p);
  const fl::Instance* best = nullptr;
  int best_extra = 1 << 30;
  // Tuning knob: FL_TILE=<rows per wave>x<keys per tile>x<waves>x<ring depth>, e.g. 32x32x4x4, restricts the choice
  // to instances of that shape (the default is the first listed instance that fits).
  // The environment is read once, when the first launch is planned.
  struct TileKnob {
    int rw = 0, bn = 0, nw = 0, ns = 0;
    TileKnob() {
      if (const char* e = std::getenv("FL_TILE")) std::sscanf(e, "%dx%dx%dx%d", &rw, &bn, &nw, &ns);
    }
  };
  static const TileKnob knob;
  const int want_rw = knob.rw, want_bn = knob.bn, want_nw = knob.nw, want_ns = knob.ns;
  // keys one workgroup of 128 query rows visits: the window plus its own rows for a sliding window, else up to Lk
  const int64_t visited = p->mask_kind == FL_MASK_SLIDING ? std::min<int64_t>(p->Lk, (int64_t)p->window + 128) : p->Lk;
  // (measured: from a window of 256 on the 4-wave tile ties or wins on warm operands and wins by 4 % on cold ones)
  const bool short_loop = p->mask_kind == FL_MASK_SLIDING && visited < 384;
  // Unmasked calls at head dim 128 whose grid still fills the part twice over with 256-row workgroups take the
  // 8-wave tile: one workgroup per compute unit brings every K/V tile in once for 256 rows instead of twice, which on
  // ordinary data is worth more than the second workgroup's independence (2.4 % on N(0,1) operands; at head dim 64,
  // under masks and on all-zero operands it is not).
  const bool wide_group = p->mask_kind == FL_MASK_NONE && want == 0 && p->Dqk == 128 && p->Dv == 128 &&
                          (int64_t)p->B * p->Hq * ((p->Lq + 255) / 256) >= 512;
  const int preferred_nw = short_loop ? 2 : (wide_group ? 8 : 4);
  for (int i = 0; i < fl::kNumInstances; ++i) {
    const fl::Instance& in = fl::kInstances[i];
    if (in.dqk != p->Dqk || in.dv != p->Dv || in.dtype != p->dtype) continue;
    if ((in.feat & want) != want) continue;
    const uint32_t extra = in.feat & ~want;
    if (extra & ~kOptionalFeatures) continue;
    if (want_rw && (in.rw != want_rw || in.bn != want_bn || in.nw != want_nw || (want_ns && in.ns != want_ns))) continue;
    // fewer unused features first; among equals the preferred workgroup size, then the listed order
    const int n = 2 * __builtin_popcount(extra) + (in.nw == preferred_nw ? 0 : 1);
    if (n < best_extra) {
      best = &in;
      best_extra = n;
    }
  }
  return best;
}

// Device scratch of a document-mask call, in this order (every part a multiple of 16 bytes):
//   table   [B][ceil(L / 32)][2] int64   (min, max) id per 32 positions (backward)
//   lists   [B][query tiles][stride] u32 the key tiles each query tile visits (forward; bm / bn = query rows per
//                                        workgroup and keys per tile of the forward instance)
//   order   [B][query tiles] i32          the query tiles by falling list length (forward), rounded up to 16 bytes
struct DocScratch {
  int64_t blocks, n_qtiles, nk, list_stride;
  uint64_t table_bytes, lists_bytes, order_bytes;
};
DocScratch doc_scratch(int64_t B, int64_t L, int64_t bm, int64_t bn) {
  DocScratch d;
  d.blocks = (L + fl::kDocBlock - 1) / fl::kDocBlock;
  d.n_qtiles = (L + bm - 1) / bm;
  d.nk = (L + bn - 1) / bn;
  d.list_stride = (d.nk + 1 + 3) / 4 * 4;
  d.table_bytes = (uint64_t)B * d.blocks * 2 * sizeof(int64_t);
  d.lists_bytes = (uint64_t)B * d.n_qtiles * d.list_stride * sizeof(uint32_t);
  d.order_bytes = ((uint64_t)B * d.n_qtiles * sizeof(int32_t) + 15) / 16 * 16;
  return d;
}

// LDS bytes of a launch: the instance's fixed part plus, under a document mask, the tile list in whole 1 KiB wave
// transfers.
int64_t lds_bytes_for(const fl::Instance* in, const fl_attn_params* p) {
  if (!(in->feat & fl::F_DOC)) return in->lds_fixed_bytes;
  const DocScratch d = doc_scratch(p->B, p->Lk, (int64_t)in->rw * in->nw, in->bn);
  return in->lds_fixed_bytes + (d.list_stride * 4 + 1023) / 1024 * 1024;
}
// Dynamic LDS bytes of the document-mask pre-pass (doc_lists_kernel): 20 per key tile; it has 128 static bytes besides
int64_t prepass_lds_bytes(int64_t n_ktiles) { return n_ktiles * 20; }
int64_t max_keys_for(const fl::Instance* in) {
  int64_t tiles = fl::kMaxKeyTiles;
  if (in->feat & fl::F_DOC) {
    tiles = std::min<int64_t>(tiles, (fl::kMaxLdsBytes - in->lds_fixed_bytes) / 1024 * 256 - 4);
    tiles = std::min<int64_t>(tiles, (fl::kMaxLdsBytes - 128) / 20);  // the pre-pass: 20 bytes of LDS per key tile
  }
  return tiles * in->bn;
}

int check_strides(const char* what, const int64_t* s, int align) {
  if (s[3] != 1) return fail(FL_ERR_STRIDE, "%s: the last (dim) stride must be 1, got %lld", what, (long long)s[3]);
  for (int i = 0; i < 3; ++i) {
    if (s[i] < 0) return fail(FL_ERR_STRIDE, "%s: negative stride %lld", what, (long long)s[i]);
    if (s[i] % align != 0)
      return fail(FL_ERR_ALIGN, "%s: stride[%d]=%lld must be a multiple of %d elements", what, i, (long long)s[i], align);
  }
  return 0;
}

int check_ptr(const char* what, const void* ptr, int align) {
  if (!ptr) return fail(FL_ERR_NULL, "%s pointer is null", what);
  if (reinterpret_cast<uintptr_t>(ptr) % align != 0)
    return fail(FL_ERR_ALIGN, "%s pointer must be %d-byte aligned", what, align);
  return 0;
}

int validate(const fl_attn_params* p, const fl::Instance** out, bool for_bwd = false) {
  if (!p) return fail(FL_ERR_NULL, "params is null");
  int rc;
  if ((rc = check_ptr("q", p->q, 16)) || (rc = check_ptr("k", p->k, 16)) || (rc = check_ptr("v", p->v, 16)) ||
      (rc = check_ptr("o", p->o, 8)))
    return rc;
  if (p->dtype != FL_BF16 && p->dtype != FL_F16)
    return fail(FL_ERR_UNSUPPORTED, "dtype %d is not supported (FL_BF16 or FL_F16)", p->dtype);
  if (p->B <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->Lq <= 0 || p->Lk <= 0 || p->Dqk <= 0 || p->Dv <= 0)
    return fail(FL_ERR_SHAPE, "sizes must be positive: B=%d Hq=%d Hkv=%d Lq=%d Lk=%d Dqk=%d Dv=%d", p->B, p->Hq, p->Hkv,
                p->Lq, p->Lk, p->Dqk, p->Dv);
  if (p->Hq % p->Hkv != 0)
    return fail(FL_ERR_SHAPE, "query heads (%d) must be a multiple of key/value heads (%d)", p->Hq, p->Hkv);
  if ((int64_t)p->B * p->Hq > (int64_t)1 << 30) return fail(FL_ERR_SHAPE, "B*Hq too large");
  if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return fail(FL_ERR_ARG, "scale must be finite and > 0, got %g", p->scale);
  if ((rc = check_strides("q", p->q_strides, 8)) || (rc = check_strides("k", p->k_strides, 8)) ||
      (rc = check_strides("v", p->v_strides, 8)) || (rc = check_strides("o", p->o_strides, 4)))
    return rc;
  if (p->flags & ~(uint32_t)FL_FLAG_DOC_PREPARED) return fail(FL_ERR_ARG, "unknown bits in flags: 0x%x", p->flags);
  if ((p->flags & FL_FLAG_DOC_PREPARED) && !is_doc(p->mask_kind))
    return fail(FL_ERR_ARG, "FL_FLAG_DOC_PREPARED goes with a document mask only");
  if (p->dropout_threshold) {
    if (p->dropout_threshold > 65535u)
      return fail(FL_ERR_ARG, "dropout_threshold must be at most 65535 (rate 65535/65536), got %u", p->dropout_threshold);
    if (p->diff || p->attended_dump)
      return fail(FL_ERR_UNSUPPORTED, "dropout is not built for differential attention and the dump hook");
  }
  if (p->lse) {
    if (reinterpret_cast<uintptr_t>(p->lse) % 4) return fail(FL_ERR_ALIGN, "lse must be 4-byte aligned");
    if (p->diff) return fail(FL_ERR_UNSUPPORTED, "lse is not produced for differential attention");
  }

  switch (p->mask_kind) {
    case FL_MASK_NONE:
    case FL_MASK_CAUSAL: break;
    case FL_MASK_SLIDING:
      if (p->window < 0) return fail(FL_ERR_ARG, "window must be >= 0, got %d", p->window);
      if (p->Lq != p->Lk) return fail(FL_ERR_SHAPE, "sliding window needs Lq == Lk (got %d, %d)", p->Lq, p->Lk);
      break;
    case FL_MASK_PREFIX_LM:
      if (p->Lq != p->Lk) return fail(FL_ERR_SHAPE, "prefix-LM needs Lq == Lk (got %d, %d)", p->Lq, p->Lk);
      break;
    case FL_MASK_DOCUMENT:
    case FL_MASK_DOCUMENT_CAUSAL:
      if (!p->doc_ids) return fail(FL_ERR_NULL, "doc_ids pointer is null");
      if (reinterpret_cast<uintptr_t>(p->doc_ids) % 8) return fail(FL_ERR_ALIGN, "doc_ids must be 8-byte aligned");
      if (p->Lq != p->Lk) return fail(FL_ERR_SHAPE, "document mask needs Lq == Lk (got %d, %d)", p->Lq, p->Lk);
      if (p->doc_stride < 0) return fail(FL_ERR_STRIDE, "doc_stride must be >= 0");
      break;
    default: return fail(FL_ERR_ARG, "unknown mask_kind %d", p->mask_kind);
  }
  if (p->alibi_heads < 0) return fail(FL_ERR_ARG, "alibi_heads must be >= 0");
  if (!(p->softcap >= 0.f) || !std::isfinite(p->softcap)) return fail(FL_ERR_ARG, "softcap must be finite and >= 0");
  if (p->score_fn != FL_SCORE_NONE) {
    if (p->score_fn < FL_SCORE_SIGMOID || p->score_fn > FL_SCORE_POLY) return fail(FL_ERR_ARG, "unknown score_fn %d", p->score_fn);
    const float* c = p->score_fn_params;
    // clamp bounds may be infinite (a one-sided clamp); every other constant is an ordinary number
    const int n_finite = p->score_fn == FL_SCORE_CLAMP ? 2 : 4;
    for (int i = 0; i < n_finite; ++i)
      if (!std::isfinite(c[i])) return fail(FL_ERR_ARG, "score_fn_params[%d] must be finite", i);
    if (p->score_fn == FL_SCORE_CLAMP && !(c[2] <= c[3])) return fail(FL_ERR_ARG, "score_fn clamp: lower bound above upper bound");
    if (p->softcap > 0.f || p->alibi_heads > 0 || is_doc(p->mask_kind) || p->gate || p->diff || p->dropout_threshold)
      return fail(FL_ERR_UNSUPPORTED, "score_fn goes with positional masks and bias operands only (no soft-cap, ALiBi, "
                                      "document mask, gate, differential attention or dropout)");
  }
  for (int nb = 0; nb < 2; ++nb) {
    if (!p->bias[nb]) continue;
    if (p->bias_dtype[nb] != p->dtype && p->bias_dtype[nb] != FL_F32)
      return fail(FL_ERR_UNSUPPORTED, "bias_dtype[%d]=%d is not supported (fp32, or the element type of q)", nb, p->bias_dtype[nb]);
    const int esz = p->bias_dtype[nb] == FL_F32 ? 4 : 2;
    if (reinterpret_cast<uintptr_t>(p->bias[nb]) % esz)
      return fail(FL_ERR_ALIGN, "bias[%d] must be %d-byte aligned", nb, esz);
    if (p->bias_batch_div[nb] <= 0) return fail(FL_ERR_ARG, "bias_batch_div[%d] must be >= 1", nb);
    for (int i = 0; i < 4; ++i)
      if (p->bias_strides[nb][i] < 0) return fail(FL_ERR_STRIDE, "bias[%d]: negative stride", nb);
    if (p->bias_strides[nb][3] > 1) return fail(FL_ERR_STRIDE, "bias[%d]: the key stride must be 0 or 1", nb);
  }
  if (p->gate) {
    if ((rc = check_ptr("gate", p->gate, 8)) || (rc = check_strides("gate", p->gate_strides, 4))) return rc;
  }
  if (p->diff) {
    if (!std::isfinite(p->lambda)) return fail(FL_ERR_ARG, "lambda must be finite");
  }
  const fl::Instance* in = select_instance(p);
  if (!in)
    return fail(FL_ERR_UNSUPPORTED,
                "no kernel instance for Dqk=%d Dv=%d features=0x%x (alibi=1 softcap=2 bias=4 doc=8 diff=16 gate=32 dump=64 "
                "dropout=128 score_fn=256)",
                p->Dqk, p->Dv, wanted_features(p));
  const int64_t nkt = ((int64_t)p->Lk + in->bn - 1) / in->bn;
  if (nkt > fl::kMaxKeyTiles || lds_bytes_for(in, p) > fl::kMaxLdsBytes)
    return fail(FL_ERR_SHAPE, "Lk=%d exceeds the supported maximum of %lld keys for this kernel", p->Lk,
                (long long)max_keys_for(in));
  // per-lane byte offsets inside one key tile are 32-bit
  if (((int64_t)in->bn * p->k_strides[2] + p->Dqk) * 2 >= ((int64_t)1 << 31) ||
      ((int64_t)in->bn * p->v_strides[2] + p->Dv) * 2 >= ((int64_t)1 << 31))
    return fail(FL_ERR_STRIDE, "key/value sequence stride too large (%lld, %lld elements)", (long long)p->k_strides[2],
                (long long)p->v_strides[2]);
  const int64_t bm = (int64_t)in->rw * in->nw;
  const int64_t grid = (int64_t)p->B * p->Hq * (((int64_t)p->Lq + bm - 1) / bm);
  if (grid > 0x7fffffff) return fail(FL_ERR_SHAPE, "too many workgroups (%lld)", (long long)grid);
  if (is_doc(p->mask_kind)) {
    // the forward's pre-pass keeps 20 bytes per key tile (and 128 more) in LDS
    if (!for_bwd && prepass_lds_bytes(nkt) + 128 > fl::kMaxLdsBytes)
      return fail(FL_ERR_SHAPE, "Lk=%d exceeds the supported maximum of %lld keys for a document mask with this kernel", p->Lk,
                  (long long)max_keys_for(in));
    // (a backward call needs the table of id ranges only, not the forward's lists)
    const uint64_t need = for_bwd ? fl_bwd_workspace_bytes(p) : fl_workspace_bytes(p);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(FL_ERR_WORKSPACE, "document mask needs a %llu-byte workspace (got %llu)", (unsigned long long)need,
                  (unsigned long long)(p->workspace ? p->workspace_bytes : 0));
    if (reinterpret_cast<uintptr_t>(p->workspace) % 16) return fail(FL_ERR_ALIGN, "workspace must be 16-byte aligned");
  }
  if (out) *out = in;
  g_err[0] = 0;
  return 0;
}

// Whether *p (already validated) is a call the shared-bias streaming forward covers: head dim 32, no mask or other
// score modification, one dense 16-bit bias operand that several consecutive batch entries share (and optionally one
// row of keys per batch entry), a key count the kernel is compiled for (pairbias_has_shape).  Fills the kernel's
// parameters and launch shape.
bool plan_pairbias(const fl_attn_params* p, fl::PParams* out, int* grid) {
  static const bool disabled = std::getenv("FL_NO_PAIRBIAS") != nullptr;  // A/B knob: the general kernel instead
  if (disabled) return false;
  if (p->Dqk != p->Dv || p->mask_kind != FL_MASK_NONE || p->alibi_heads > 0 || p->softcap > 0.f ||
      p->diff || p->attended_dump || p->dropout_threshold || p->lse || p->score_fn != FL_SCORE_NONE)
    return false;
  // one operand that several consecutive batch entries share (dense over heads, queries and keys), and optionally one
  // that is a row of keys per batch entry, the same for every head and query; in either order
  int pi = -1, ri = -1;
  for (int i = 0; i < 2; ++i) {
    if (!p->bias[i]) continue;
    const int64_t* st = p->bias_strides[i];
    if (p->bias_dtype[i] != p->dtype || st[3] != 1) return false;
    if (p->bias_batch_div[i] >= 2 && (st[1] != 0 || p->Hq == 1) && st[2] != 0 && pi < 0) pi = i;  // (one head: no head stride)
    else if (p->bias_batch_div[i] == 1 && st[1] == 0 && st[2] == 0 && ri < 0) ri = i;
    else return false;
  }
  if (pi < 0) return false;
  const int64_t* bst = p->bias_strides[pi];
  const int div = p->bias_batch_div[pi];
  if (p->B % div != 0) return false;
  if (p->Lk % 32 != 0 || !fl::pairbias_has_shape(p->Dqk, p->Lk / 32, p->gate != nullptr, ri >= 0)) return false;
  if (reinterpret_cast<uintptr_t>(p->bias[pi]) % 16 != 0 || bst[0] % 8 || bst[1] % 8 || bst[2] % 8) return false;
  if (ri >= 0 && (reinterpret_cast<uintptr_t>(p->bias[ri]) % 16 != 0 || p->bias_strides[ri][0] % 8)) return false;
  // (results leave in 16-byte stores, gate logits arrive in 16-byte loads)
  if (reinterpret_cast<uintptr_t>(p->o) % 16 != 0 || p->o_strides[0] % 8 || p->o_strides[1] % 8 || p->o_strides[2] % 8) return false;
  if (p->gate && (reinterpret_cast<uintptr_t>(p->gate) % 16 != 0 || p->gate_strides[0] % 8 || p->gate_strides[1] % 8 ||
                  p->gate_strides[2] % 8))
    return false;
  // per-lane byte offsets inside one (batch entry, head) slice are 32-bit
  const int64_t worst = std::max(std::max(p->q_strides[2], p->o_strides[2]), p->gate ? p->gate_strides[2] : 0);
  if (((int64_t)p->Lq * worst + 64) * 2 >= ((int64_t)1 << 31)) return false;
  // ... and so are those inside one key tile of 64 rows
  if ((64 * std::max(p->k_strides[2], p->v_strides[2]) + p->Dqk) * 2 >= ((int64_t)1 << 31)) return false;
  // the selector weight 1 / scale must be an ordinary number in the element type (bf16 shares fp32's range; fp16 ends at
  // 65504 and loses precision below 2^-14)
  {
    const float w = 1.0f / p->scale;
    const float w_max = p->dtype == FL_F16 ? 32768.0f : 0x1p100f, w_min = p->dtype == FL_F16 ? 0x1p-10f : 0x1p-100f;
    if (!(w <= w_max) || !(w >= w_min)) return false;
  }
  fl::PParams k;
  std::memset(&k, 0, sizeof(k));
  k.q = static_cast<const fl::bf16_t*>(p->q);
  k.k = static_cast<const fl::bf16_t*>(p->k);
  k.v = static_cast<const fl::bf16_t*>(p->v);
  k.o = static_cast<fl::bf16_t*>(p->o);
  for (int i = 0; i < 3; ++i) {
    k.qs[i] = p->q_strides[i];
    k.ks[i] = p->k_strides[i];
    k.vs[i] = p->v_strides[i];
    k.os[i] = p->o_strides[i];
    k.gs[i] = p->gate_strides[i];
    k.bs[i] = bst[i];
  }
  k.B = p->B;
  k.H = p->Hq;
  if (p->Hq != p->Hkv) return false;
  k.Lq = p->Lq;
  k.Lk = p->Lk;
  k.scale = p->scale;
  k.bias = static_cast<const fl::bf16_t*>(p->bias[pi]);
  k.bdiv = div;
  if (ri >= 0) {
    k.rowb = static_cast<const fl::bf16_t*>(p->bias[ri]);
    k.rbs = p->bias_strides[ri][0];
  }
  k.gate = static_cast<const fl::bf16_t*>(p->gate);
  k.n_qtiles = (p->Lq + 127) / 128;
  // Launch shape: every workgroup should be resident at once (two per compute unit, 32 compute units per XCD), and a
  // unit = (chunk of batch entries, pair of heads) with all its query tiles stays on one XCD.  The batch entries of a
  // bias group are cut into as many chunks as that allows; more chunks than entries make no sense, fewer than one
  // means several rounds of workgroups.
  const int64_t groups = p->B / div;
  k.hgroup = p->Hq % 2 == 0 ? 2 : 1;
  const int64_t per_unit = (int64_t)k.hgroup * k.n_qtiles;
  const int64_t units_per_xcd = std::max<int64_t>(1, 64 / per_unit);
  const int64_t head_groups = p->Hq / k.hgroup;
  int64_t chunks = (8 * units_per_xcd) / (groups * head_groups);
  chunks = std::max<int64_t>(1, std::min<int64_t>(chunks, div));
  k.chunk_len = (int)((div + chunks - 1) / chunks);
  k.chunks = (div + k.chunk_len - 1) / k.chunk_len;
  const int64_t n_units = groups * k.chunks * head_groups;
  const int64_t g = (n_units + 7) / 8 * 8 * per_unit;
  if (n_units > 0x7fffffff || g > 0x7fffffff) return false;
  k.n_units = (int)n_units;
  *grid = (int)g;
  *out = k;
  return true;
}

}  // namespace

extern "C" {

int fl_version(void) { return FL_ABI_VERSION; }

const char* fl_last_error(void) { return g_err; }

uint64_t fl_params_sizeof(void) { return sizeof(fl_attn_params); }

uint64_t fl_workspace_bytes(const fl_attn_params* p) {
  if (!p || !is_doc(p->mask_kind) || p->B <= 0 || p->Lk <= 0) return 0;
  // tile shape of the instance the forward would run (the largest lists any compiled shape needs, if the call names no
  // valid one)
  const fl::Instance* in = select_instance(p);
  const DocScratch d = doc_scratch(p->B, p->Lk, in ? (int64_t)in->rw * in->nw : 64, in ? in->bn : 32);
  return d.table_bytes + d.lists_bytes + d.order_bytes;
}

uint64_t fl_bwd_workspace_bytes(const fl_attn_params* p) {
  if (!p || !is_doc(p->mask_kind) || p->B <= 0 || p->Lk <= 0) return 0;
  return doc_scratch(p->B, p->Lk, 128, 64).table_bytes;
}

int fl_attn_validate(const fl_attn_params* p) { return validate(p, nullptr); }

int fl_attn_plan(const fl_attn_params* p, int64_t out[8]) {
  const fl::Instance* in = nullptr;
  int rc = validate(p, &in);
  if (rc) return rc;
  if (!out) return fail(FL_ERR_NULL, "out is null");
  const int64_t bm = (int64_t)in->rw * in->nw;
  out[0] = bm;
  out[1] = in->bn;
  out[2] = in->nw * 64;
  out[3] = (int64_t)p->B * p->Hq * ((p->Lq + bm - 1) / bm);
  out[4] = lds_bytes_for(in, p);
  out[5] = in->feat;
  out[6] = 0;
  {
    // calls the shared-bias streaming forward takes: its fixed shape, and out[6] = 1
    fl::PParams pb;
    int pb_grid = 0;
    if (plan_pairbias(p, &pb, &pb_grid)) {
      out[0] = 128;
      out[1] = 64;
      out[2] = 256;
      out[3] = pb_grid;
      out[4] = 2 * (p->Dqk == 32 ? 6 : 4) * 64 * p->Dqk * 2 + (pb.rowb ? 4 * 2 * 1024 : 0);
      out[6] = 1;
    }
  }
  out[7] = 0;
  return 0;
}

int fl_attn_fwd(const fl_attn_params* p, void* stream_) {
  const fl::Instance* in = nullptr;
  int rc = validate(p, &in);
  if (rc) return rc;
  hipStream_t stream = static_cast<hipStream_t>(stream_);

  {
    fl::PParams pb;
    int pb_grid = 0;
    if (plan_pairbias(p, &pb, &pb_grid)) {
      const hipError_t e = (p->dtype == FL_F16 ? fl::launch_pairbias_f16 : fl::launch_pairbias_bf16)(
          p->Dqk, p->Lk / 32, p->gate != nullptr, pb.rowb != nullptr, pb, pb_grid, stream);
      if (e != hipSuccess) return fail((int)e, "launch of the shared-bias forward failed: %s", hipGetErrorString(e));
      return 0;
    }
  }

  fl::KParams kp;
  std::memset(&kp, 0, sizeof(kp));
  kp.q = static_cast<const fl::bf16_t*>(p->q);
  kp.k = static_cast<const fl::bf16_t*>(p->k);
  kp.v = static_cast<const fl::bf16_t*>(p->v);
  kp.o = static_cast<fl::bf16_t*>(p->o);
  for (int i = 0; i < 3; ++i) {
    kp.qs[i] = p->q_strides[i];
    kp.ks[i] = p->k_strides[i];
    kp.vs[i] = p->v_strides[i];
    kp.os[i] = p->o_strides[i];
    kp.gs[i] = p->gate_strides[i];
  }
  kp.B = p->B;
  kp.Hq = p->Hq;
  kp.Hkv = p->Hkv;
  kp.Lq = p->Lq;
  kp.Lk = p->Lk;
  kp.group = p->Hq / p->Hkv;
  kp.scale = p->scale;
  kp.scale_log2 = p->scale * 1.4426950408889634f;
  kp.mask_kind = p->mask_kind;
  kp.window = p->window;
  kp.prefix = p->prefix;
  {
    const int kFar = 1 << 29;
    const bool causal_like = p->mask_kind == FL_MASK_CAUSAL || p->mask_kind == FL_MASK_SLIDING ||
                             p->mask_kind == FL_MASK_PREFIX_LM || p->mask_kind == FL_MASK_DOCUMENT_CAUSAL;
    kp.dmax = causal_like ? 0 : kFar;
    kp.dmin = p->mask_kind == FL_MASK_SLIDING ? -(p->window < kFar ? p->window : kFar) : -kFar;
    kp.pfx = p->mask_kind == FL_MASK_PREFIX_LM ? (p->prefix < 0 ? 0 : p->prefix) : 0;
  }
  kp.doc_ids = p->doc_ids;
  kp.doc_stride = p->doc_stride;
  kp.alibi_heads = p->alibi_heads;
  kp.softcap = p->softcap;
  if (p->score_fn != FL_SCORE_NONE) {
    // scale and log2(e) folded into the constants (in double): the kernel works on the raw q.k and in log2 units
    const double l2e = 1.4426950408889634, sc = p->scale;
    const float* c = p->score_fn_params;
    kp.score_fn = p->score_fn;
    if (p->score_fn == FL_SCORE_SIGMOID) {
      kp.score_k[0] = (float)(-(double)c[0] * sc * l2e);
      kp.score_k[1] = (float)(-(double)c[1] * l2e);
      kp.score_k[2] = (float)((double)c[2] * l2e);
      kp.score_k[3] = (float)((double)c[3] * l2e);
    } else if (p->score_fn == FL_SCORE_CLAMP) {
      kp.score_k[0] = (float)((double)c[0] * sc * l2e);
      kp.score_k[1] = (float)((double)c[1] * l2e);
      kp.score_k[2] = (float)((double)c[2] * l2e);
      kp.score_k[3] = (float)((double)c[3] * l2e);
    } else {
      kp.score_k[0] = (float)((double)c[0] * l2e);
      kp.score_k[1] = (float)((double)c[1] * sc * l2e);
      kp.score_k[2] = (float)((double)c[2] * sc * sc * l2e);
      kp.score_k[3] = (float)((double)c[3] * sc * sc * sc * l2e);
    }
  }
  for (int nb = 0; nb < 2; ++nb) {
    kp.bias[nb] = static_cast<const fl::bf16_t*>(p->bias[nb]);
    kp.bdiv[nb] = p->bias[nb] ? p->bias_batch_div[nb] : 1;
    kp.bias_f32[nb] = p->bias[nb] && p->bias_dtype[nb] == FL_F32;
    // four consecutive keys of a row in one load: 8 bytes of bf16 or 16 bytes of fp32
    bool vec = p->bias[nb] && p->bias_strides[nb][3] == 1 &&
               reinterpret_cast<uintptr_t>(p->bias[nb]) % (kp.bias_f32[nb] ? 16 : 8) == 0;
    for (int i = 0; i < 4; ++i) {
      kp.bs[nb][i] = p->bias_strides[nb][i];
      if (i < 3 && p->bias_strides[nb][i] % 4 != 0) vec = false;
    }
    kp.bias_vec[nb] = vec ? 1 : 0;
  }
  // Bias operands travel through LDS with the K/V tiles when their rows are addressable in 16-byte pieces: one
  // row-broadcast operand (query stride 0) as single rows, one more as [rows][keys] tiles; any other takes the direct
  // path.
  kp.bias_lds = -1;
  kp.bias_row = -1;
  for (int nb = 0; nb < 2; ++nb) {
    if (!p->bias[nb] || p->bias_strides[nb][3] != 1 || reinterpret_cast<uintptr_t>(p->bias[nb]) % 16 != 0) continue;
    if (p->Lk % 8 != 0) continue;
    // fp32: staged only as the row-broadcast operand (the [rows][keys] tiles hold 16-bit elements, so a second fp32 row
    // operand takes the direct path)
    if (kp.bias_f32[nb] && (p->bias_strides[nb][2] != 0 || kp.bias_row >= 0)) continue;
    bool ok = true;
    for (int i = 0; i < 3; ++i) ok = ok && p->bias_strides[nb][i] % 8 == 0;
    // per-lane byte offsets inside one (batch, head) slice are 32-bit
    ok = ok && ((int64_t)p->Lq * p->bias_strides[nb][2] + p->Lk) * 4 < ((int64_t)1 << 31);
    if (!ok) continue;
    if (p->bias_strides[nb][2] == 0 && kp.bias_row < 0) kp.bias_row = nb;
    else if (kp.bias_lds < 0) kp.bias_lds = nb;
  }
  kp.gate = static_cast<const fl::bf16_t*>(p->gate);
  kp.lambda = p->lambda;
  if (p->diff) {
    // heads [0, H) are branch 0, heads [H, 2H) branch 1 (query: H = Hq, key: H = Hkv)
    kp.q_branch_stride = (int64_t)p->Hq * p->q_strides[1];
    kp.k_branch_stride = (int64_t)p->Hkv * p->k_strides[1];
  }
  kp.dump = p->attended_dump;
  kp.lse = p->lse;
  kp.drop_thr = p->dropout_threshold;
  kp.drop_seed[0] = p->dropout_seed[0];
  kp.drop_seed[1] = p->dropout_seed[1];
  kp.drop_rescale = 65536.0f / (65536.0f - (float)p->dropout_threshold);
  const int bm = in->rw * in->nw;
  kp.n_qtiles = (p->Lq + bm - 1) / bm;
  kp.n_ktiles = (p->Lk + in->bn - 1) / in->bn;
  {
    // Masks whose work grows with the query position: (batch, head) pairs are taken four at a time (measured: one at a
    // time costs the document-mask configuration 20 %, whose two heads per XCD then drain one after the other; two, eight
    // or sixteen instead of four change the causal launch by 1-4 %)
    const bool growing = p->mask_kind == FL_MASK_CAUSAL || p->mask_kind == FL_MASK_PREFIX_LM || is_doc(p->mask_kind);
    static const int knob = std::getenv("FL_HEAD_GROUP") ? std::atoi(std::getenv("FL_HEAD_GROUP")) : 0;  // tuning knob
    kp.head_group = !growing ? 1 : (knob > 0 ? knob : 4);
  }
  kp.o_wide = reinterpret_cast<uintptr_t>(p->o) % 16 == 0 && p->o_strides[0] % 8 == 0 && p->o_strides[1] % 8 == 0 &&
              p->o_strides[2] % 8 == 0;
  const int grid = p->B * p->Hq * kp.n_qtiles;

  if (is_doc(p->mask_kind)) {
    const DocScratch d = doc_scratch(p->B, p->Lk, bm, in->bn);
    uint32_t* lists = reinterpret_cast<uint32_t*>(static_cast<unsigned char*>(p->workspace) + d.table_bytes);
    int32_t* order = reinterpret_cast<int32_t*>(static_cast<unsigned char*>(p->workspace) + d.table_bytes + d.lists_bytes);
    if (!(p->flags & FL_FLAG_DOC_PREPARED)) {
      static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&fl::doc_lists_kernel),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, fl::kMaxLdsBytes - 128);
      if (attr != hipSuccess) return fail((int)attr, "doc_lists_kernel: %s", hipGetErrorString(attr));
      hipLaunchKernelGGL(fl::doc_lists_kernel, dim3(p->B * kp.n_qtiles), dim3(1024), (size_t)prepass_lds_bytes(kp.n_ktiles), stream,
                         p->doc_ids, p->doc_stride, p->Lk, p->mask_kind, bm, in->rw, in->bn, kp.n_qtiles, kp.n_ktiles,
                         (int)d.list_stride, lists);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail((int)e, "doc_lists_kernel launch failed: %s", hipGetErrorString(e));
      hipLaunchKernelGGL(fl::doc_order_kernel, dim3(p->B), dim3(1024), (size_t)kp.n_qtiles * 4, stream, lists,
                         (int)d.list_stride, kp.n_qtiles, order);
      e = hipGetLastError();
      if (e != hipSuccess) return fail((int)e, "doc_order_kernel launch failed: %s", hipGetErrorString(e));
    }
    kp.doc_lists = lists;
    kp.doc_list_stride = (int)d.list_stride;
    kp.doc_order = order;
  }
  hipError_t e = in->launch(kp, grid, (int)lds_bytes_for(in, p), stream);
  if (e != hipSuccess) return fail((int)e, "launch of %s failed: %s", in->name, hipGetErrorString(e));
  return 0;
}

uint64_t fl_static_scratch_bytes(void) { return kStaticScratchBytes; }

uint64_t fl_bwd_params_sizeof(void) { return sizeof(fl_attn_bwd_params); }

static int validate_bwd(const fl_attn_bwd_params* b, const fl::BwdInstance** out) {
  if (!b) return fail(FL_ERR_NULL, "params is null");
  const fl_attn_params* p = &b->fwd;
  int rc = validate(p, nullptr, true);
  if (rc) return rc;
  if (p->gate || p->diff || p->attended_dump)
    return fail(FL_ERR_UNSUPPORTED, "backward: gate, differential attention and the dump hook are not supported");
  if (p->score_fn != FL_SCORE_NONE) return fail(FL_ERR_UNSUPPORTED, "backward: score_fn is forward-only");
  const bool has_bias = p->bias[0] || p->bias[1];
  if (b->dscores && p->softcap > 0.f)
    return fail(FL_ERR_UNSUPPORTED, "backward: dscores is not produced under a soft-cap (gradients of bias operands added after the cap)");
  if (b->dscores && !has_bias) return fail(FL_ERR_ARG, "backward: dscores is only written for calls with bias operands");
  if (b->dscores && reinterpret_cast<uintptr_t>(b->dscores) % 16) return fail(FL_ERR_ALIGN, "backward: dscores must be 16-byte aligned");
  if (p->Dqk != p->Dv) return fail(FL_ERR_UNSUPPORTED, "backward needs Dqk == Dv (got %d, %d)", p->Dqk, p->Dv);
  if ((rc = check_ptr("dout", b->dout, 16)) || (rc = check_ptr("dq", b->dq, 8)) || (rc = check_ptr("dk", b->dk, 8)) ||
      (rc = check_ptr("dv", b->dv, 8)) || (rc = check_ptr("delta", b->delta, 16)) ||
      (rc = check_ptr("fwd.lse", p->lse, 16)))
    return rc;
  if ((rc = check_strides("dout", b->dout_strides, 8)) || (rc = check_strides("dq", b->dq_strides, 4)) ||
      (rc = check_strides("dk", b->dk_strides, 4)) || (rc = check_strides("dv", b->dv_strides, 4)) ||
      (rc = check_strides("o", p->o_strides, 8)))
    return rc;
  if (reinterpret_cast<uintptr_t>(p->o) % 16) return fail(FL_ERR_ALIGN, "backward: o must be 16-byte aligned");
  for (int i = 0; i < 6; ++i)
    if (b->reserved[i] != 0) return fail(FL_ERR_ARG, "reserved[%d] must be 0", i);
  // per-lane byte offsets inside one staged tile (up to 128 rows) are 32-bit
  const int64_t worst = std::max(std::max(p->q_strides[2], p->k_strides[2]), std::max(p->v_strides[2], b->dout_strides[2]));
  if ((128 * worst + p->Dqk) * 2 >= ((int64_t)1 << 31))
    return fail(FL_ERR_STRIDE, "backward: sequence stride too large (%lld elements)", (long long)worst);
  if ((int64_t)p->B * p->Hq * ((p->Lq + 127) / 128) > 0x7fffffff || (int64_t)p->B * p->Hkv * ((p->Lk + 127) / 128) > 0x7fffffff)
    return fail(FL_ERR_SHAPE, "backward: too many workgroups");
  uint32_t want = 0;
  if (p->alibi_heads > 0 || p->softcap > 0.f) want = fl::F_ALIBI | fl::F_SOFTCAP;
  if (is_doc(p->mask_kind)) want |= fl::F_DOC;
  if (has_bias) want |= fl::F_BIAS;
  if (p->dropout_threshold) want |= fl::F_DROPOUT;  // (head dims 64 and 128)
  const fl::BwdInstance* in = nullptr;
  for (int i = 0; i < fl::kNumBwdInstances; ++i)
    if (fl::kBwdInstances[i].d == p->Dqk && fl::kBwdInstances[i].feat == want && fl::kBwdInstances[i].dtype == p->dtype)
      in = &fl::kBwdInstances[i];
  if (!in)
    return fail(FL_ERR_UNSUPPORTED, "backward: no kernel for head dim %d with features 0x%x (compiled: 32, 64 and 128; dropout at 64 "
                "and 128)", p->Dqk, want);
  if (out) *out = in;
  g_err[0] = 0;
  return 0;
}

int fl_attn_bwd_validate(const fl_attn_bwd_params* b) { return validate_bwd(b, nullptr); }

int fl_attn_bwd(const fl_attn_bwd_params* b, void* stream_) {
  const fl::BwdInstance* in = nullptr;
  int rc = validate_bwd(b, &in);
  if (rc) return rc;
  const fl_attn_params* p = &b->fwd;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  fl::BParams bp;
  std::memset(&bp, 0, sizeof(bp));
  bp.q = static_cast<const fl::bf16_t*>(p->q);
  bp.k = static_cast<const fl::bf16_t*>(p->k);
  bp.v = static_cast<const fl::bf16_t*>(p->v);
  bp.o = static_cast<const fl::bf16_t*>(p->o);
  bp.dout = static_cast<const fl::bf16_t*>(b->dout);
  bp.lse = p->lse;
  bp.delta = b->delta;
  bp.dq = static_cast<fl::bf16_t*>(b->dq);
  bp.dk = static_cast<fl::bf16_t*>(b->dk);
  bp.dv = static_cast<fl::bf16_t*>(b->dv);
  for (int i = 0; i < 3; ++i) {
    bp.qs[i] = p->q_strides[i];
    bp.ks[i] = p->k_strides[i];
    bp.vs[i] = p->v_strides[i];
    bp.os[i] = p->o_strides[i];
    bp.dos[i] = b->dout_strides[i];
    bp.dqs[i] = b->dq_strides[i];
    bp.dks[i] = b->dk_strides[i];
    bp.dvs[i] = b->dv_strides[i];
  }
  bp.B = p->B;
  bp.Hq = p->Hq;
  bp.Hkv = p->Hkv;
  bp.Lq = p->Lq;
  bp.Lk = p->Lk;
  bp.group = p->Hq / p->Hkv;
  bp.scale = p->scale;
  bp.scale_log2 = p->scale * 1.4426950408889634f;
  bp.mask_kind = p->mask_kind;
  bp.window = p->window;
  bp.prefix = p->prefix;
  {
    const int kFar = 1 << 29;
    const bool causal_like = p->mask_kind == FL_MASK_CAUSAL || p->mask_kind == FL_MASK_SLIDING ||
                             p->mask_kind == FL_MASK_PREFIX_LM || p->mask_kind == FL_MASK_DOCUMENT_CAUSAL;
    bp.dmax = causal_like ? 0 : kFar;
    bp.dmin = p->mask_kind == FL_MASK_SLIDING ? -(p->window < kFar ? p->window : kFar) : -kFar;
    bp.pfx = p->mask_kind == FL_MASK_PREFIX_LM ? (p->prefix < 0 ? 0 : p->prefix) : 0;
  }
  bp.doc_ids = p->doc_ids;
  bp.doc_stride = p->doc_stride;
  bp.alibi_heads = p->alibi_heads;
  bp.softcap = p->softcap;
  bp.drop_thr = p->dropout_threshold;
  bp.drop_seed[0] = p->dropout_seed[0];
  bp.drop_seed[1] = p->dropout_seed[1];
  bp.drop_rescale = 65536.0f / (65536.0f - (float)p->dropout_threshold);
  for (int nb = 0; nb < 2; ++nb) {
    bp.bias[nb] = p->bias[nb];
    for (int i = 0; i < 4; ++i) bp.bbs[nb][i] = p->bias_strides[nb][i];
    bp.bdiv[nb] = p->bias_batch_div[nb] > 0 ? p->bias_batch_div[nb] : 1;
    bp.bias_f32[nb] = p->bias_dtype[nb] == FL_F32;
  }
  bp.dscores = b->dscores;
  if (is_doc(p->mask_kind)) {
    const int blocks = (p->Lk + fl::kDocBlock - 1) / fl::kDocBlock;
    const int total = p->B * blocks;
    int64_t* table = static_cast<int64_t*>(p->workspace);
    hipLaunchKernelGGL(fl::doc_table_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, p->doc_ids, p->doc_stride,
                       p->Lk, blocks, total, table);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "doc_table_kernel launch failed: %s", hipGetErrorString(e));
    bp.doc_table = table;
    bp.doc_blocks = blocks;
  }
  hipError_t e = in->launch_delta(bp, stream);
  if (e != hipSuccess) return fail((int)e, "backward: launch of the row-sum kernel failed: %s", hipGetErrorString(e));
  e = in->launch_dq(bp, stream);
  if (e != hipSuccess) return fail((int)e, "backward: launch of the dQ kernel failed: %s", hipGetErrorString(e));
  e = in->launch_dkv(bp, stream);
  if (e != hipSuccess) return fail((int)e, "backward: launch of the dK/dV kernel failed: %s", hipGetErrorString(e));
  return 0;
}

int fl_attn_bwd_static(const fl_attn_bwd_params* b, void* stream) {
  if (!b) return fail(FL_ERR_NULL, "params is null");
  fl_attn_bwd_params c = *b;
  const fl_attn_params* p = &b->fwd;
  if (p->B <= 0 || p->Hq <= 0 || p->Lq <= 0) return fail(FL_ERR_SHAPE, "sizes must be positive");
  // layout of the static scratch: the row sums (B * Hq * Lq floats, rounded up to 256 bytes), then the document table
  const uint64_t delta_bytes = ((uint64_t)p->B * p->Hq * p->Lq * sizeof(float) + 255) / 256 * 256;
  const uint64_t table_bytes = fl_bwd_workspace_bytes(p);
  if (delta_bytes + table_bytes > kStaticScratchBytes)
    return fail(FL_ERR_WORKSPACE,
                "fl_attn_bwd_static: this call needs %llu bytes of scratch (4 per query row of every head, plus 16 per 32 "
                "positions of every batch row under a document mask), the library's static scratch holds %llu; use "
                "fl_attn_bwd with caller-provided delta and workspace",
                (unsigned long long)(delta_bytes + table_bytes), (unsigned long long)kStaticScratchBytes);
  void* ptr = nullptr;
  int rc = static_scratch_ptr(&ptr);
  if (rc) return rc;
  c.delta = static_cast<float*>(ptr);
  c.fwd.workspace = table_bytes ? static_cast<unsigned char*>(ptr) + delta_bytes : nullptr;
  c.fwd.workspace_bytes = table_bytes;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool capturing = stream_is_capturing(s);
  int dev = -1;
  if (!capturing) {
    rc = static_scratch_acquire(s, &dev);
    if (rc) return rc;
  }
  rc = fl_attn_bwd(&c, stream);
  if (!capturing && dev >= 0) static_scratch_release(s, dev);
  return rc;
}

}  // extern "C"
