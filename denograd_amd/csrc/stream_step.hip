// One decode step of the whole Llama decoder as a single persistent kernel with role-specialised wavefronts (gfx950).
//
// At batch 1 every weight byte is used once, so a step is as fast as the weight stream from HBM is continuous.  One launch
// per fused op leaves the memory system idle at every launch boundary (dispatch ramp, the read of the input row, its
// RMSNorm, the first load round trip, the tail), which at five boundaries per layer costs as much as the stream itself.
// Here one block of 12 wavefronts per CU stays resident for the whole step (Transformer.forward,
// /root/reference/jsgrad/models/llama.ts:201-213) and its wavefronts have fixed roles:
//
//   * weight wavefronts do nothing but stream: each walks its own static list of weight items (2 rows x 4 KiB of a
//     matrix, or 2 rows x 2 KiB of the w1/w3 pair) through ALL phases of the step with two register buffers, so the
//     loads of the next phase are in flight while the current phase is handed over.  They never issue any other global
//     load or store (vector memory operations of a wavefront complete in order, so anything else would wait behind the
//     stream): the input row comes from LDS, the raw row sums go to LDS.
//   * the control wavefront of the block owns every hand-off: it waits for the other blocks, stages the input row of a
//     phase in LDS (RMSNorm included), and when the block's weight wavefronts have delivered their sums it applies the
//     epilogue (row scale, fp16 rounding, residual / rotary + KV-cache write / SwiGLU / logits + arg-max partial), stores
//     the results for the other blocks and raises the block's flag.
//   * attention wavefronts run grouped-query attention over the KV cache (llama.ts:89-95) between the QKV and the wo
//     phase, one (kv head, chunk of positions) item per wavefront, the last item of a kv head merging the chunks.
//
// Blocks synchronise through one flag per block (its own 128-byte line) that every control wavefront polls; data that
// crosses blocks is written with agent-scope stores and read with agent-scope loads.  Every wait is bounded: when a spin
// runs out the error word is raised, all later waits fall through and the grid drains.
//
// The arithmetic is that of the stand-alone kernels (gemv_core.h): an output row is summed by one wavefront in the same
// order, scaled, rounded and combined by the same expressions.
#include <algorithm>

#include "gemv_core.h"

namespace jsg {

constexpr int SS_NWW = 7;                        // weight wavefronts per block; the eighth wavefront is the control wavefront
#ifndef SS_NBUF
#define SS_NBUF 4
#endif                                           // register buffers (8 x 16 bytes per lane each) of a weight wavefront
constexpr int SS_THREADS = (SS_NWW + 1) * 64;    // 8 wavefronts per CU = 2 per SIMD: 256 registers per lane
constexpr int SS_YMAX = 1024;                    // raw row sums a block can hold per phase
constexpr int SS_CHUNK = 128;                    // most positions per attention item
constexpr int SS_MAXCH = 64;                     // most attention items per kv head
constexpr int SS_ATT_LOADS = 12;                 // 128-bit loads of K (and of V) an attention item keeps in flight per lane
constexpr int SS_FLAG_STRIDE = 32;               // ints between block flags: one 128-byte line each
constexpr int SS_MAX_BLOCKS = 1024;
constexpr int SS_SPIN_GLOBAL = 1 << 18;          // polls of ~0.5 us
constexpr int SS_SPIN_LDS = 1 << 21;             // polls of ~0.1 us
constexpr int SS_NORM_CHUNKS = 8;                // 16-byte chunks of the input row a lane keeps for the fused RMSNorm

// workspace layout (bytes)
constexpr size_t SS_WS_EPOCH = 0, SS_WS_ERR = 128, SS_WS_COUNTERS = 256, SS_WS_AMAX_VAL = 512, SS_WS_AMAX_IDX = 512 + 4096,
                 SS_WS_FLAGS = 16384, SS_WS_PARTIAL = SS_WS_FLAGS + (size_t)SS_MAX_BLOCKS * SS_FLAG_STRIDE * 4;
constexpr int SS_TAG_DIM = SS_NORM_CHUNKS * 512, SS_TAG_HIDDEN = 65536;   // entries reserved for the tagged h / h2 rows and the g row

struct SsLayer {   // = jsgrad_hip_layer_t
  const void *wq, *wk, *wv, *wo, *w1, *w2, *w3;
  const void *sq, *sk, *sv, *so, *s1, *s2, *s3;
  const void *attention_norm, *ffn_norm;
  void *cache_k, *cache_v;
};
struct SsArgs {
  const SsLayer *layers;
  int n_layers, dim, hidden, n_heads, n_kv_heads, head_dim, vocab, max_context;
  float eps;
  int embed_kind;
  const void *tok_emb, *tok_scale, *out_w, *out_s, *final_norm, *rope_table;
  int32_t *state, *tokens_out;
  int tokens_cap;
  void *h, *h2, *q, *attn, *g, *logits;
  // activation rows as they pass between blocks: one 32-bit word per element, fp16 value | version tag << 16
  uint32_t *th, *th2, *tg, *tattn, *tq, *tkv;   // dim, dim, hidden, n_heads*hd, n_heads*hd, 2 * n_kv_heads*hd (k | v of this position)
  int *epoch, *err, *flags, *attn_counters;
  float *attn_partial;   // [n_kv_heads][SS_MAXCH][n_rep][HD + 2]
  float *amax_val;
  int *amax_idx;
  long long *trace;
  int x_bytes;           // LDS bytes reserved for the staged input row
  int grid;              // blocks of the launch (gridDim.x costs a trip to the dispatch packet wherever it is used)
};

// LDS control words of a block
struct SsCtl {
  int x_ready;            // weight phases whose input row is staged
  int go;                 // unused
  int abort;              // a bounded wait ran out somewhere: nobody waits any more
  int pad;
  // One progress word per wavefront, not a shared count: a wavefront without work in a phase passes it at once and
  // may be several phases ahead, so a count of completions would say nothing about the slowest wavefront.
  int wdone[8];           // weight phases wavefront w has delivered (SS_NWW <= 8)
  int pad2[4];
};
static_assert(SS_NWW <= 8 && sizeof(SsCtl) % 8 == 0, "the table of layer tensors follows the control words, 8-byte aligned");

enum { PH_QKV = 0, PH_ATTN = 1, PH_WO = 2, PH_FFN = 3, PH_W2 = 4, PH_LM = 5 };

// Two tables are built in LDS when the kernel starts, because a weight wavefront must not fetch a pointer from global
// memory (that load would sit behind its weight stream; an LDS read does not touch that queue):
//   * the layer tensors (a copy of the jsgrad_hip_layer_t array), and
//   * one record per phase with everything that depends on the phase kind (matrices, scales, shapes, input row,
//     norm weight, residual, output).  Each record is filled by ONE THREAD with ordinary per-lane code, and the
//     wavefronts later read whole records by index: selecting among pointers with wavefront-uniform branches on the
//     phase kind was compiled wrongly (the pointer of another branch survived), a table lookup has nothing to select.
typedef const __attribute__((address_space(3))) uint64_t *LtPtr;
struct SsTabs { LtPtr layers, phases; };
constexpr int SS_LAYER_WORDS = sizeof(SsLayer) / 8;
constexpr int SS_PHASE_WORDS = 16;   // w0 w1 w2 s0 s1 s2 src norm_w residual y (rows0,rows1) (rows2,in_f) (nm,kind) + three words of the item walk
// a value that is the same in every lane, moved to scalar registers
__device__ __forceinline__ uint64_t uni64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ SsLayer ss_layer(const SsTabs &lt, int l) {
  LtPtr w = lt.layers + (size_t)l * SS_LAYER_WORDS;
  auto P = [&](int i) { return (const void *)uni64(w[i]); };
  SsLayer L;
  L.wq = P(0); L.wk = P(1); L.wv = P(2); L.wo = P(3); L.w1 = P(4); L.w2 = P(5); L.w3 = P(6);
  L.sq = P(7); L.sk = P(8); L.sv = P(9); L.so = P(10); L.s1 = P(11); L.s2 = P(12); L.s3 = P(13);
  L.attention_norm = P(14); L.ffn_norm = P(15);
  L.cache_k = (void *)P(16); L.cache_v = (void *)P(17);
  return L;
}

// ---- small helpers -------------------------------------------------------------------------------------------------
__device__ __forceinline__ int lds_ld(const int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
__device__ __forceinline__ void lds_st(int *p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
// the compiler must not move LDS accesses across a hand-off; the LDS pipeline itself runs a wavefront's accesses in order
__device__ __forceinline__ void lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void vm_drain() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// 16 bytes at the device-wide coherence point, as two 64-bit accesses
__device__ __forceinline__ u4_t ld16_coherent(const void *p) {
  const JSG_GLOBAL uint64_t *q = as_global<uint64_t>(p);
  const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return u4_t{(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
}
__device__ __forceinline__ void st16_coherent(void *p, u4_t v) {
  JSG_GLOBAL uint64_t *q = as_global_mut<uint64_t>(p);
  __hip_atomic_store(q, (uint64_t)v[0] | ((uint64_t)v[1] << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(q + 1, (uint64_t)v[2] | ((uint64_t)v[3] << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- tagged rows: how activations pass from block to block ------------------------------------------------------------
// An element of a row that other blocks read is one 32-bit word: the fp16 value below, the version of the phase that wrote
// it above.  A reader asks for the words and takes them when every tag is the version it expects, else it asks again: the
// data is its own flag, so a writer neither waits for its stores to be acknowledged nor raises a flag, and a reader needs
// no round trip for a flag before the round trip for the data.  Nothing is overwritten too early: a block writes the
// outputs of phase p + 1 only after it has seen every output of phase p, and whoever wrote those had finished reading
// whatever it read in phases up to p.
__device__ __forceinline__ uint32_t ss_tag(int version) { return (uint32_t)version % 65535u + 1u; }   // never 0: fresh memory matches nothing
__device__ __forceinline__ uint32_t ss_tagged(uint32_t tag, float v) {
  const _Float16 h = (_Float16)v;
  return (tag << 16) | (uint32_t)__builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ void st_tagged(uint32_t *p, uint32_t tag, float v) { st_coherent((int *)p, (int)ss_tagged(tag, v)); }
__device__ __forceinline__ float ld_tagged_value(const uint32_t *p) {   // a word known to be there: its value
  const uint32_t w = (uint32_t)ld_coherent((const int *)p);
  return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
}
// A tagged row as a buffer resource: 16-byte loads that are coherent across the device (sc1, like the agent-scope atomic
// loads, which exist up to 64 bits only); a word is the unit that has to arrive whole, and every word carries its own tag.
typedef __amdgpu_buffer_rsrc_t TagRow;
__device__ __forceinline__ TagRow tag_row(const uint32_t *p, int n) {
  return __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)uni64((uint64_t)(uintptr_t)p), 0, n * 4, 0x00020000);
}
// eight tagged words -> eight packed halves; ok: all eight carry `tag`
__device__ __forceinline__ u4_t ss_untag8(u4_t a, u4_t b, uint32_t tag, bool &ok);
// (words i .. i + 7 of a row given as a buffer resource: the few loads of an attention item)
__device__ __forceinline__ u4_t ld8_tagged(TagRow row, int i, uint32_t tag, bool &ok) {
  return ss_untag8(__builtin_amdgcn_raw_buffer_load_b128(row, i * 4, 0, 16), __builtin_amdgcn_raw_buffer_load_b128(row, i * 4 + 16, 0, 16), tag, ok);
}
// (32 bytes at p, as four 64-bit agent-scope loads: staging a whole row this way measured faster than with 16-byte loads)
__device__ __forceinline__ u4_t ld8_tagged(const uint32_t *p, uint32_t tag, bool &ok) { return ss_untag8(ld16_coherent(p), ld16_coherent(p + 4), tag, ok); }
__device__ __forceinline__ u4_t ss_untag8(u4_t a, u4_t b, uint32_t tag, bool &ok) {
  const uint32_t e = tag << 16;
  const uint32_t bad = ((a[0] ^ e) | (a[1] ^ e) | (a[2] ^ e) | (a[3] ^ e) | (b[0] ^ e) | (b[1] ^ e) | (b[2] ^ e) | (b[3] ^ e)) >> 16;
  ok = ok && bad == 0;
  return u4_t{(a[0] & 0xffffu) | (a[1] << 16), (a[2] & 0xffffu) | (a[3] << 16), (b[0] & 0xffffu) | (b[1] << 16), (b[2] & 0xffffu) | (b[3] << 16)};
}

// One more round of a wait on tagged rows; false: give up (the error word is set and nobody waits any more).
__device__ __forceinline__ bool ss_poll_again(const SsArgs &s, SsCtl &ctl, int &it) {
  if ((++it & 15) == 0) {
    if (lds_ld(&ctl.abort) != 0) return false;
    if (it > SS_SPIN_GLOBAL || ld_coherent(s.err) != 0) {
      st_coherent(s.err, 1);
      lds_st(&ctl.abort, 1);
      return false;
    }
  }
  return true;
}

// Wait until an LDS word reaches `target`.  Returns false when the wait was abandoned.
__device__ __forceinline__ bool lds_wait(const SsArgs &s, SsCtl &ctl, const int *word, int target) {
  int it = 0;
  while (__builtin_amdgcn_readfirstlane(lds_ld(word)) - target < 0) {
    __builtin_amdgcn_s_sleep(1);
    if ((++it & 255) == 0) {
      if (lds_ld(&ctl.abort) != 0) return false;
      if (it > SS_SPIN_LDS) {
        st_coherent(s.err, 1);
        lds_st(&ctl.abort, 1);
        return false;
      }
    }
  }
  return true;
}

// Wait until every one of n (<= 64) LDS words has reached `target`.
__device__ __forceinline__ bool lds_wait_all(const SsArgs &s, SsCtl &ctl, const int *words, int n, int target) {
  const int lane = threadIdx.x & 63;
  int it = 0;
  while (true) {
    const int v = lds_ld(words + (lane < n ? lane : 0));
    if (__all(v - target >= 0)) return true;
    __builtin_amdgcn_s_sleep(1);
    if ((++it & 255) == 0) {
      if (lds_ld(&ctl.abort) != 0) return false;
      if (it > SS_SPIN_LDS) {
        st_coherent(s.err, 1);
        lds_st(&ctl.abort, 1);
        return false;
      }
    }
  }
}

// ---- weight phases -------------------------------------------------------------------------------------------------
struct WDesc {
  const char *w0, *w1, *w2;   // QKV: wq, wk, wv stacked; FFN: w1 and w3 on the same rows (nm == 2); otherwise w0 alone
  const void *s0, *s1, *s2;   // int8 row scales
  const void *src, *norm_w, *residual;   // input row (activation dtype), RMSNorm weight or null, residual row or null
  void *y;                    // output row (null for QKV: queries and cache rows have their own places)
  int rows0, rows1, rows2;
  int in_f, nm, kind;
};
__device__ __forceinline__ int ss_phases(const SsArgs &s) { return 5 * s.n_layers + 1; }
__device__ __forceinline__ int ss_kind(const SsArgs &s, int p) { return p == 5 * s.n_layers ? PH_LM : p % 5; }
// weight phases before phase p (p itself a weight phase)
__device__ __forceinline__ int ss_wordinal(const SsArgs &s, int p) {
  const int l = p / 5, k = p % 5;
  return p == 5 * s.n_layers ? 4 * s.n_layers : 4 * l + (k == 0 ? 0 : k - 1);
}
__device__ __forceinline__ int ss_next_weight(const SsArgs &s, int p) {
  p++;
  if (p < 5 * s.n_layers && p % 5 == PH_ATTN) p++;
  return p;
}
// record of phase p, written by one thread (per-lane code: the selects below are plain conditional moves)
// vec: weight elements per 16-byte load (the walk over the items depends on the weight format)
__device__ __forceinline__ void ss_build_phase(const SsArgs &s, uint64_t *rec, int p, int vec) {
  const int k = ss_kind(s, p);
  const int l = k == PH_LM ? s.n_layers - 1 : p / 5;
  const uint64_t *L = (const uint64_t *)s.layers + (size_t)l * SS_LAYER_WORDS;
  // word indices of jsgrad_hip_layer_t: wq wk wv wo w1 w2 w3 | sq sk sv so s1 s2 s3 | attention_norm ffn_norm | cache_k cache_v
  uint64_t w0 = 0, w1 = 0, w2 = 0, s0 = 0, s1 = 0, s2 = 0, src = 0, norm_w = 0, residual = 0, y = 0;
  int rows0 = 0, rows1 = 0, rows2 = 0, in_f = 0, nm = 1;
  const int qdim = s.n_heads * s.head_dim, kvdim = s.n_kv_heads * s.head_dim;
  if (k == PH_QKV) {
    w0 = ldg(L + 0); w1 = ldg(L + 1); w2 = ldg(L + 2); s0 = ldg(L + 7); s1 = ldg(L + 8); s2 = ldg(L + 9);
    rows0 = qdim; rows1 = kvdim; rows2 = kvdim; in_f = s.dim; src = (uint64_t)(uintptr_t)s.th; norm_w = ldg(L + 14);
  } else if (k == PH_WO) {
    w0 = ldg(L + 3); s0 = ldg(L + 10); rows0 = s.dim; in_f = qdim;
    src = (uint64_t)(uintptr_t)s.tattn; residual = (uint64_t)(uintptr_t)s.th; y = (uint64_t)(uintptr_t)s.th2;
  } else if (k == PH_FFN) {
    w0 = ldg(L + 4); w1 = ldg(L + 6); s0 = ldg(L + 11); s1 = ldg(L + 13); rows0 = s.hidden; in_f = s.dim; nm = 2;
    src = (uint64_t)(uintptr_t)s.th2; norm_w = ldg(L + 15); y = (uint64_t)(uintptr_t)s.tg;
  } else if (k == PH_W2) {
    w0 = ldg(L + 5); s0 = ldg(L + 12); rows0 = s.dim; in_f = s.hidden;
    src = (uint64_t)(uintptr_t)s.tg; residual = (uint64_t)(uintptr_t)s.th2; y = (uint64_t)(uintptr_t)s.th;
  } else if (k == PH_LM) {
    w0 = (uint64_t)(uintptr_t)s.out_w; s0 = (uint64_t)(uintptr_t)s.out_s; rows0 = s.vocab; in_f = s.dim;
    src = (uint64_t)(uintptr_t)s.th; norm_w = (uint64_t)(uintptr_t)s.final_norm; y = (uint64_t)(uintptr_t)s.logits;
  }
  rec[0] = w0; rec[1] = w1; rec[2] = w2; rec[3] = s0; rec[4] = s1; rec[5] = s2; rec[6] = src; rec[7] = norm_w; rec[8] = residual; rec[9] = y;
  rec[10] = (uint32_t)rows0 | ((uint64_t)(uint32_t)rows1 << 32);
  rec[11] = (uint32_t)rows2 | ((uint64_t)(uint32_t)in_f << 32);
  rec[12] = (uint32_t)nm | ((uint64_t)(uint32_t)k << 32);
  // the walk of this block's weight wavefronts over the items of the phase
  uint64_t cnt = 0, str = 0, first = 0;
  if (in_f > 0) {
    const int step = 64 * vec, un = nm == 2 ? 2 : 4;
    const int nb = ((in_f + step - 1) / step + un - 1) / un;
    const int rows = rows0 + (nm == 1 ? rows1 + rows2 : 0), ngroups = (rows + 1) >> 1;
    const int G = gridDim.x, blk = blockIdx.x;
    const int mine = ngroups > blk ? (ngroups - blk + G - 1) / G : 0;
    cnt = (uint32_t)nb | ((uint64_t)(uint32_t)(mine * nb) << 32);
    str = (uint32_t)(in_f * 16 / vec) | ((uint64_t)(uint32_t)(SS_NWW / nb) << 32) | ((uint64_t)(uint32_t)(SS_NWW % nb) << 48);
    for (int w = 0; w < SS_NWW; w++) first |= ((uint64_t)(uint32_t)(w / nb) << (4 * w)) | ((uint64_t)(uint32_t)(w % nb) << (32 + 4 * w));
  }
  rec[13] = cnt; rec[14] = str; rec[15] = first;
}
// the record of phase p, in scalar registers
__device__ __forceinline__ WDesc ss_wdesc(const SsArgs &s, const SsTabs &lt, int p) {
  LtPtr r = lt.phases + (size_t)p * SS_PHASE_WORDS;
  WDesc d;
  d.w0 = (const char *)uni64(r[0]); d.w1 = (const char *)uni64(r[1]); d.w2 = (const char *)uni64(r[2]);
  d.s0 = (const void *)uni64(r[3]); d.s1 = (const void *)uni64(r[4]); d.s2 = (const void *)uni64(r[5]);
  d.src = (const void *)uni64(r[6]); d.norm_w = (const void *)uni64(r[7]); d.residual = (const void *)uni64(r[8]); d.y = (void *)uni64(r[9]);
  const uint64_t a = uni64(r[10]), b = uni64(r[11]), c = uni64(r[12]);
  d.rows0 = (int)(uint32_t)a; d.rows1 = (int)(a >> 32); d.rows2 = (int)(uint32_t)b; d.in_f = (int)(b >> 32);
  d.nm = (int)(uint32_t)c; d.kind = (int)(c >> 32);
  return d;
}
__device__ __forceinline__ int wd_rows(const WDesc &d) { return d.rows0 + (d.nm == 1 ? d.rows1 + d.rows2 : 0); }
__device__ __forceinline__ int wd_groups(const WDesc &d) { return (wd_rows(d) + 1) >> 1; }

// The weight format of the step: VEC elements per 16-byte load, STEP elements per wavefront k-step; an item is 8 loads:
// 2 rows x 4 k-steps of one matrix, or 2 rows x 2 k-steps of two.
template <int KIND> struct SsFmt {
  static constexpr int VEC = WFmt<KIND>::VEC;
  static constexpr int BITS = KIND == JSGRAD_W_F16 ? 16 : 8;
  static constexpr int STEP = 64 * VEC;
  __device__ static __forceinline__ int unroll(int nm) { return nm == 2 ? 2 : 4; }
  __device__ static __forceinline__ int nbatch(const WDesc &d) { const int u = unroll(d.nm); return ((d.in_f + STEP - 1) / STEP + u - 1) / u; }
};
// LDS elements the staged input row of a phase occupies (whole batches; the tail is zero)
static int ss_x_elems(int kind, int in_f, int nm) {
  const int step = 64 * (kind == JSGRAD_W_F16 ? 8 : 16), u = nm == 2 ? 2 : 4;
  return (((in_f + step - 1) / step + u - 1) / u) * u * step;
}

struct WBuf { u4_t w[8]; };

// Work split of a weight phase.  Row groups (2 consecutive rows) are dealt to the blocks round-robin: block b owns groups
// b, b + G, b + 2G, ...  An item is one k-batch of one group; the items of a block, in (group, batch) order, are dealt to
// its weight wavefronts round-robin, so the wavefronts of a block differ by at most one item whatever the shapes are.  The
// partial sum of every item goes to LDS and the control wavefront adds the batches of a row in batch order.
__device__ __forceinline__ int ss_block_groups(int ngroups) {   // groups of this block
  const int G = gridDim.x, b = blockIdx.x;
  return ngroups > b ? (ngroups - b + G - 1) / G : 0;
}

// Everything a weight wavefront does per item is on its critical path (two of them share a SIMD and an item is only 8 KiB),
// so whatever depends on the phase alone is worked out once per block when the phase table is built (words 13-15 of a
// record) and the walk over the items is a handful of scalar adds:
//   word 13: k-batches per group | items of this block
//   word 14: bytes per weight row | (SS_NWW / nb) | (SS_NWW % nb) << 16
//   word 15: for wavefront w, 4 bits each: w / nb at bit 4w, w % nb at bit 32 + 4w
struct WIter {
  int p, w;             // phase and its ordinal among the weight phases
  int t, gl, b;         // item index in the block's list, local group index, k-batch
  bool live;
  // of the phase
  int nitems, nb, step_gl, step_b, rows0, rows1, grid;
  uint32_t row_bytes;
  bool nm2;
  // of the item: first row inside its matrix, and the matrix pointer(s) as read from the LDS record (per lane, not yet
  // moved to scalar registers: the read is issued when the iterator moves and waited for when the loads are issued)
  int row;
  uint64_t raw0, raw1;
};
// what the consumer of a register buffer needs to know about the item in it
struct WRec {
  int t, b, w;
  bool nm2, live;
};

// v[i] + v[i ^ 16] + v[i ^ 32] + v[i ^ 48] in every lane i, through the two row-swap instructions of the vector ALU (no
// trip through LDS): with both operands holding v, one swap leaves "v of my half" in one and "v of the other half" in the other
__device__ __forceinline__ float ss_rows_sum(float v) {
  const uint32_t a = __float_as_uint(v);
  const auto h = __builtin_amdgcn_permlane16_swap(a, a, false, false);   // rows 1 and 3 of the first <-> rows 0 and 2 of the second
  const uint32_t b = __float_as_uint(__uint_as_float(h[0]) + __uint_as_float(h[1]));
  const auto w = __builtin_amdgcn_permlane32_swap(b, b, false, false);   // upper half of the first <-> lower half of the second
  return __uint_as_float(w[0]) + __uint_as_float(w[1]);
}

// Totals of four per-lane values over the wavefront: every lane gets the total of value (lane & 3).  Two exchange steps
// halve the number of values a lane carries, the rest adds lanes that carry the same value.
__device__ __forceinline__ float ss_reduce4(float v0, float v1, float v2, float v3) {
  const int lane = threadIdx.x & 63;
  const bool o1 = (lane & 1) != 0, o2 = (lane & 2) != 0;
  float k0 = o1 ? v1 : v0, s0 = o1 ? v0 : v1;
  float k1 = o1 ? v3 : v2, s1 = o1 ? v2 : v3;
  k0 += dpp_f<0xB1>(s0);   // quad_perm [1,0,3,2]: value (lane & 1) of the pair
  k1 += dpp_f<0xB1>(s1);   //                      value 2 + (lane & 1)
  float k = o2 ? k1 : k0;
  const float sd = o2 ? k0 : k1;
  k += dpp_f<0x4E>(sd);    // quad_perm [2,3,0,1]: value (lane & 3) of the quad
  k += dpp_f<0x124>(k);    // row_ror:4
  k += dpp_f<0x128>(k);    // row_ror:8: value (lane & 3) of the 16-lane row
  return ss_rows_sum(k);
}
// the same for two values: every lane gets the total of value (lane & 1)
__device__ __forceinline__ float ss_reduce2(float v0, float v1) {
  const int lane = threadIdx.x & 63;
  const bool o1 = (lane & 1) != 0;
  float k = o1 ? v1 : v0;
  const float sd = o1 ? v0 : v1;
  k += dpp_f<0xB1>(sd);
  k += dpp_f<0x4E>(k);
  k += dpp_f<0x124>(k);
  k += dpp_f<0x128>(k);
  return ss_rows_sum(k);
}

template <int KIND> struct SsWeights {
  typedef SsFmt<KIND> F;
  static constexpr uint32_t STEP_BYTES = 64 * 16;   // bytes one k-step of the wavefront covers in a weight row

  // items of this block in phase p
  __device__ static __forceinline__ int phase_items(const SsTabs &lt, int p) {
    return (int)(uint32_t)(uni64(lt.phases[(size_t)p * SS_PHASE_WORDS + 13]) >> 32);
  }
  __device__ static __forceinline__ void enter(const SsTabs &lt, WIter &it, int p, int w, int wave) {
    LtPtr r = lt.phases + (size_t)p * SS_PHASE_WORDS;
    const uint64_t rows = uni64(r[10]), kind = uni64(r[12]), cnt = uni64(r[13]), str = uni64(r[14]), first = uni64(r[15]);
    it.p = p;
    it.w = w;
    it.rows0 = (int)(uint32_t)rows;
    it.rows1 = (int)(rows >> 32);
    it.nm2 = (uint32_t)kind == 2u;
    it.nb = (int)(uint32_t)cnt;
    it.nitems = (int)(cnt >> 32);
    it.row_bytes = (uint32_t)str;
    it.step_gl = (int)((str >> 32) & 0xffff);
    it.step_b = (int)(str >> 48);
    it.t = wave;
    it.gl = (int)((first >> (4 * wave)) & 15);
    it.b = (int)((first >> (32 + 4 * wave)) & 15);
    locate(lt, it);
  }
  // Matrix and row of the item the iterator stands on.  The matrix pointers come out of the LDS record by index (the stacked
  // wq | wk | wv have one each); every row count is even, so both rows of a group are in one matrix.
  __device__ static __forceinline__ void locate(const SsTabs &lt, WIter &it) {
    LtPtr r = lt.phases + (size_t)it.p * SS_PHASE_WORDS;
    int row = (blockIdx.x + it.gl * it.grid) * 2;
    const int in1 = row >= it.rows0 ? 1 : 0;                  // rows1 is 0 unless the phase stacks three matrices,
    const int in2 = row >= it.rows0 + it.rows1 ? in1 : 0;     // and then no row reaches past rows0
    const int m = it.rows1 > 0 ? in1 + in2 : 0;
    it.row = row - (it.rows1 > 0 ? in1 * it.rows0 + in2 * it.rows1 : 0);
    it.raw0 = r[m];
    it.raw1 = r[m + (it.nm2 ? 1 : 0)];
  }
  // first phase at or after p (ordinal w) in which this wavefront has an item; when there is none the iterator parks on
  // an item that exists (the block's first lm_head item), so that the loads it keeps issuing stay inside a matrix
  __device__ static __forceinline__ void seek(const SsArgs &s, const SsTabs &lt, WIter &it, int p, int w, int wave) {
    const int nph = ss_phases(s);
    while (p < nph) {
      if (wave < phase_items(lt, p)) {
        enter(lt, it, p, w, wave);
        it.live = true;
        return;
      }
      p = ss_next_weight(s, p);
      w++;
    }
    enter(lt, it, nph - 1, 4 * s.n_layers, 0);
    it.live = false;
  }
  __device__ static __forceinline__ void advance(const SsArgs &s, const SsTabs &lt, WIter &it, int wave) {
    if (!it.live) return;
    it.t += SS_NWW;
    it.gl += it.step_gl;
    it.b += it.step_b;
    if (it.b >= it.nb) { it.b -= it.nb; it.gl++; }
    if (it.t < it.nitems) { locate(lt, it); return; }
    seek(s, lt, it, ss_next_weight(s, it.p), it.w + 1, wave);
  }
  __device__ static __forceinline__ WRec record(const WIter &it) { return WRec{it.t, it.b, it.w, it.nm2, it.live}; }

  // Issue the 8 loads of the item the iterator stands on.  Load v = a*4 + c*2 + r is row r of the group; with one matrix
  // it is k-step a*2 + c of the batch, with two it is k-step a of matrix c.
  __device__ static __forceinline__ void load(WBuf &buf, const WIter &it) {
    const uint32_t lane16 = (threadIdx.x & 63) * 16;
    const uint64_t rowoff = (uint64_t)(uint32_t)it.row * it.row_bytes;
    const char *base[4];
    base[0] = (const char *)(uintptr_t)(uni64(it.raw0) + rowoff);
    base[1] = base[0] + it.row_bytes;
    base[2] = (const char *)(uintptr_t)(uni64(it.raw1) + rowoff);
    base[3] = base[2] + it.row_bytes;
    const uint32_t un = it.nm2 ? 2u : 4u;
    const uint32_t k0 = (uint32_t)it.b * un * STEP_BYTES;
    const uint32_t last = it.row_bytes - 16;   // lanes past the end of the row reload its last vector; their x is zero
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int c = 0; c < 2; c++) {
        const uint32_t ks = it.nm2 ? (uint32_t)a : (uint32_t)(a * 2 + c);
        uint32_t koff = k0 + ks * STEP_BYTES + lane16;
        koff = koff < last ? koff : last;
#pragma unroll
        for (int rr = 0; rr < 2; rr++) buf.w[a * 4 + c * 2 + rr] = ldg_stream16(base[c * 2 + rr] + koff);
      }
  }

  // consume item t (k-batch b) of a phase with NM matrices: its partial row sums go to LDS
  template <int NM>
  __device__ static __forceinline__ void consume(const WBuf &buf, int t, int b, const _Float16 *xs, float *y_local) {
    constexpr int UN = NM == 2 ? 2 : 4;
    const int lane = threadIdx.x & 63;
    float acc[NM][2];
#pragma unroll
    for (int j = 0; j < NM; j++)
#pragma unroll
      for (int r = 0; r < 2; r++) acc[j][r] = 0.0f;
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int k = (b * UN + u) * F::STEP + lane * F::VEC;   // may lie in the zero padding of xs
      XFrag<_Float16, F::VEC> xf;
      xf.load(xs + k);
#pragma unroll
      for (int j = 0; j < NM; j++)
#pragma unroll
        for (int r = 0; r < 2; r++) acc[j][r] += Dot<KIND, _Float16>::run(buf.w[(u * NM + j) * 2 + r], xf, 0.0f, 1.0f, nullptr);
    }
    float *dst = y_local + (size_t)t * NM * 2;
    if constexpr (NM == 2) {
      const float tot = ss_reduce4(acc[0][0], acc[0][1], acc[1][0], acc[1][1]);
      if (lane < 4) dst[lane] = tot;
    } else {
      const float tot = ss_reduce2(acc[0][0], acc[0][1]);
      if (lane < 2) dst[lane] = tot;
    }
  }

  // The whole life of a weight wavefront: ONE flat loop over its items of all phases, unrolled over the register buffers,
  // so that buffer i is always filled and consumed by the same instructions.  (With the buffer chosen by a run-time
  // index the compiler can no longer tell the loads of one buffer from those of another and waits for every load in
  // flight before each item, which is the end of all prefetching.)  One iterator walks the item list, SS_NBUF items ahead
  // of the arithmetic; a small record per buffer tells the consumer what the buffer holds.  The loads are unconditional
  // (a parked iterator re-reads an existing item) so that the number of loads in flight is the same on every path.
  __device__ static __forceinline__ void run(const SsArgs &s, const SsTabs &lt, SsCtl &ctl, const _Float16 *xs, float *y_local, int wave) {
    const int n_weight_phases = 4 * s.n_layers + 1;
    WIter li;
    li.grid = s.grid;
    WRec rec[SS_NBUF];
    WBuf buf[SS_NBUF];   // indexed with compile-time constants only: they live in registers
    seek(s, lt, li, 0, 0, wave);
#pragma unroll
    for (int i = 0; i < SS_NBUF; i++) {
      rec[i] = record(li);
      load(buf[i], li);
      advance(s, lt, li, wave);
    }
    int wtr = 0;
    auto wstamp = [&](int tag) {   // optional trace of block 0's first weight wavefront: (100 MHz clock, tag) pairs
      if (s.trace && blockIdx.x == 0 && wave == 0 && (threadIdx.x & 63) == 0 && wtr < 3000) {
        s.trace[4096 + 2 * wtr] = (long long)__builtin_amdgcn_s_memrealtime();
        s.trace[4096 + 2 * wtr + 1] = tag;
        wtr++;
      }
    };
    // phases before the first item need nothing from this wavefront
    if ((threadIdx.x & 63) == 0) lds_st(&ctl.wdone[wave], rec[0].live ? rec[0].w : n_weight_phases);
    int cur_w = -1;
    while (rec[0].live) {
#pragma unroll
      for (int i = 0; i < SS_NBUF; i++) {
        if (rec[i].live) {
          if (rec[i].w != cur_w) {   // first item of a phase: its input row must be staged
            cur_w = rec[i].w;
            lds_wait(s, ctl, &ctl.x_ready, cur_w + 1);
            lds_fence();
            wstamp(1000 + cur_w);
          }
          if (rec[i].nm2) consume<2>(buf[i], rec[i].t, rec[i].b, xs, y_local);
          else consume<1>(buf[i], rec[i].t, rec[i].b, xs, y_local);
        }
        rec[i] = record(li);
        load(buf[i], li);
        advance(s, lt, li, wave);
        const WRec &nxt = rec[(i + 1) % SS_NBUF];
        if (cur_w >= 0 && (!nxt.live || nxt.w != cur_w)) {   // last item of the phase: everything before the next item's phase is delivered
          lds_fence();
          if ((threadIdx.x & 63) == 0) lds_st(&ctl.wdone[wave], nxt.live ? nxt.w : n_weight_phases);
        }
        wstamp(i);
      }
    }
  }
};

// ---- attention wavefronts ------------------------------------------------------------------------------------------
template <int G> __device__ __forceinline__ float ss_group_sum(float v) {
  static_assert(G == 8 || G == 16, "lane group");
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  if (G == 16) v += dpp_f<0x140>(v);
  return v;
}

template <int HD, int NREP> struct SsAttn {
  static constexpr int GL = HD / 8;     // lanes per cache row (8 halves = one 128-bit load per lane)
  static constexpr int RPI = 64 / GL;   // rows per wavefront load

  // rows per item for T visible positions when `waves` wavefronts are available per kv head
  // Rows per item for T visible positions.  The wavefront that merges a kv head fetches the partials of 16 chunks per
  // round trip and an item fetches up to SS_ATT_LOADS x RPI rows of K and of V per round trip, so up to ~750 positions
  // (head_dim 128) everything is one round trip each; longer contexts get longer items, at most SS_MAXCH per kv head.
  __device__ static __forceinline__ int chunk_rows(int T, int waves) {
    int per = waves < 16 ? waves : 16;
    per = per < 1 ? 1 : per;
    int chunk = ((T + per - 1) / per + RPI - 1) / RPI * RPI;
    chunk = chunk < 32 ? 32 : chunk;
    if (chunk > SS_CHUNK) chunk = SS_CHUNK;   // the host keeps max_context <= SS_MAXCH * SS_CHUNK
    return chunk;
  }

  // item (kv head g, chunk c): scores, softmax numerators and P.V of rows [c * chunk, ...) for the NREP query heads of
  // the kv head; the wavefront that completes the kv head merges all chunks.  sc: this wavefront's LDS float[NREP][SS_CHUNK].
  // optional trace of block 0's first attention wavefront
  __device__ static __forceinline__ void astamp(const SsArgs &s, int tag) {
    if (s.trace && blockIdx.x == 0 && (threadIdx.x & 63) == 0) {
      const int i = (int)s.trace[12288];
      if (i < 1500) {
        s.trace[12290 + 2 * i] = (long long)__builtin_amdgcn_s_memrealtime();
        s.trace[12291 + 2 * i] = tag;
        s.trace[12288] = i + 1;
      }
    }
  }
  // tin: version of the queries and of this position's k / v rows; tout: version the output row gets
  __device__ static void item(const SsArgs &s, SsCtl &ctl, const SsLayer &L, float *sc, int g, int c, int T, int chunk, int n_active, uint32_t tin, uint32_t tout) {
    typedef _Float16 AT;
    const int lane = threadIdx.x & 63, sub = lane % GL, grp = lane / GL;
    const int t0 = c * chunk, t1 = min(T, t0 + chunk), CH = t1 - t0;
    const size_t row_stride = (size_t)s.n_kv_heads * HD;
    const AT *kbase = (const AT *)L.cache_k + (size_t)g * HD + (size_t)sub * 8;
    const AT *vbase = (const AT *)L.cache_v + (size_t)g * HD + (size_t)sub * 8;
    const float scale = (float)(1.0 / sqrt((double)HD));

    // A batch is NLD loads of RPI rows each; the first batch of K and of V goes out at once (most chunks are one batch)
    constexpr int NLD = SS_ATT_LOADS, BR = NLD * RPI;
    u4_t kraw[NLD], vraw[NLD];
    auto load_batch = [&](u4_t (&raw)[NLD], const AT *base, int tb) {
#pragma unroll
      for (int u = 0; u < NLD; u++) {
        const int t = tb + u * RPI + grp;
        raw[u] = ldg((const u4_t *)(base + (size_t)(t < t1 ? t : t1 - 1) * row_stride));
      }
    };
    load_batch(kraw, kbase, t0);
    load_batch(vraw, vbase, t0);
    // The queries, and for the chunk that ends at this position its k and v rows (their cache rows are being written by
    // other blocks right now, for later tokens to read), come as tagged rows.
    const bool has_cur = t1 == T;
    const int kvdim = s.n_kv_heads * HD;
    h2_t qh[NREP][4];
    u4_t kcur = {0, 0, 0, 0}, vcur = {0, 0, 0, 0};
    const TagRow rq = tag_row(s.tq, s.n_heads * HD), rkv = tag_row(s.tkv, 2 * kvdim);
    for (int it = 0;;) {
      bool ok = true;
#pragma unroll
      for (int j = 0; j < NREP; j++) {
        const u4_t raw = ld8_tagged(rq, (g * NREP + j) * HD + sub * 8, tin, ok);
#pragma unroll
        for (int e = 0; e < 4; e++) qh[j][e] = as_h2(raw[e]);
      }
      if (has_cur) {
        kcur = ld8_tagged(rkv, g * HD + sub * 8, tin, ok);
        vcur = ld8_tagged(rkv, kvdim + g * HD + sub * 8, tin, ok);
      }
      if (__all(ok) || !ss_poll_again(s, ctl, it)) break;
    }
    if (has_cur && T - 1 - t0 < BR) {   // the row sits in the first batch: replace what came from the cache
#pragma unroll
      for (int u = 0; u < NLD; u++)
        if (t0 + u * RPI + grp == T - 1) { kraw[u] = kcur; vraw[u] = vcur; }
    }
    // scores of the chunk and their maximum
    float mx[NREP];
#pragma unroll
    for (int j = 0; j < NREP; j++) mx[j] = -INFINITY;
    for (int tb = t0; tb < t1; tb += BR) {
      if (tb != t0) {
        load_batch(kraw, kbase, tb);
        if (has_cur) {
#pragma unroll
          for (int u = 0; u < NLD; u++)
            if (tb + u * RPI + grp == T - 1) kraw[u] = kcur;
        }
      }
#pragma unroll
      for (int u = 0; u < NLD; u++) {
        const int t = tb + u * RPI + grp;
#pragma unroll
        for (int j = 0; j < NREP; j++) {
          float p = 0.0f;
#pragma unroll
          for (int e = 0; e < 4; e++) p = __builtin_amdgcn_fdot2(qh[j][e], as_h2(kraw[u][e]), p, false);
          p = ss_group_sum<GL>(p) * scale;
          if (t < t1) {
            if (sub == 0) sc[j * SS_CHUNK + (t - t0)] = p;
            mx[j] = fmaxf(mx[j], p);
          }
        }
      }
    }
    float ls[NREP];
#pragma unroll
    for (int j = 0; j < NREP; j++) { mx[j] = wave_max(mx[j]); ls[j] = 0.0f; }
    lds_fence();
    astamp(s, 2);
    for (int i = lane; i < CH; i += 64)
#pragma unroll
      for (int j = 0; j < NREP; j++) {
        const float e = exp_f32(sc[j * SS_CHUNK + i] - mx[j]);
        sc[j * SS_CHUNK + i] = e;
        ls[j] += e;
      }
#pragma unroll
    for (int j = 0; j < NREP; j++) ls[j] = wave_sum(ls[j]);
    lds_fence();
    // o[j][d] = sum_t p[j][t] * V[t][d]
    float of[NREP][8];
#pragma unroll
    for (int j = 0; j < NREP; j++)
#pragma unroll
      for (int e = 0; e < 8; e++) of[j][e] = 0.0f;
    for (int tb = t0; tb < t1; tb += BR) {
      if (tb != t0) {
        load_batch(vraw, vbase, tb);
        if (has_cur) {
#pragma unroll
          for (int u = 0; u < NLD; u++)
            if (tb + u * RPI + grp == T - 1) vraw[u] = vcur;
        }
      }
#pragma unroll
      for (int u = 0; u < NLD; u++) {
        const int t = tb + u * RPI + grp;
        float vf[8];
#pragma unroll
        for (int e = 0; e < 4; e++) { h2_t h = as_h2(vraw[u][e]); vf[2 * e] = (float)h[0]; vf[2 * e + 1] = (float)h[1]; }
#pragma unroll
        for (int j = 0; j < NREP; j++) {
          const float p = t < t1 ? sc[j * SS_CHUNK + (t - t0)] : 0.0f;
#pragma unroll
          for (int e = 0; e < 8; e++) of[j][e] = fmaf(p, vf[e], of[j][e]);
        }
      }
    }
    // lanes with the same `sub` hold different rows: fold the row groups of the wavefront together
#pragma unroll
    for (int j = 0; j < NREP; j++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float v = of[j][e];
#pragma unroll
        for (int off = GL; off < 64; off <<= 1) v += __shfl_xor(v, off);
        of[j][e] = v;
      }
    astamp(s, 3);
    float *mine = s.attn_partial + ((size_t)g * SS_MAXCH + c) * NREP * (HD + 2);
    if (grp == 0) {
#pragma unroll
      for (int j = 0; j < NREP; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) st_coherent(&mine[j * (HD + 2) + sub * 8 + e], of[j][e]);
    }
#pragma unroll
    for (int j = 0; j < NREP; j++)
      if (lane == j) {
        st_coherent(&mine[j * (HD + 2) + HD], mx[j]);
        st_coherent(&mine[j * (HD + 2) + HD + 1], ls[j]);
      }
    vm_drain();   // the partial is at the coherence point before the item is counted
    astamp(s, 4);
    int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(&s.attn_counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    old = __builtin_amdgcn_readfirstlane(old);
    astamp(s, 5);
    if (old != n_active - 1) return;
    // the counter is zero again long before the next layer counts on it (four hand-offs away)
    if (lane == 0) __hip_atomic_store(&s.attn_counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- merge the chunks of kv head g: weights exp(m_s - M), normalisation 1 / sum(l_s * w_s)
    const float *base = s.attn_partial + (size_t)g * SS_MAXCH * NREP * (HD + 2);
    float inv[NREP], ms[NREP], lsum[NREP];
    const bool on = lane < n_active;   // n_active <= SS_MAXCH = 64: one chunk per lane
#pragma unroll
    for (int j = 0; j < NREP; j++) {   // all (m, l) pairs in one round trip; lanes past the end re-read the last chunk
      const float *ps = base + ((size_t)(on ? lane : n_active - 1) * NREP + j) * (HD + 2);
      ms[j] = ld_coherent(ps + HD);
      lsum[j] = ld_coherent(ps + HD + 1);
    }
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      ms[j] = on ? ms[j] : -INFINITY;
      lsum[j] = on ? lsum[j] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      const float M = wave_max(ms[j]);
      const float w = on ? exp_f32(ms[j] - M) : 0.0f;
      if (on) sc[j * SS_CHUNK + lane] = w;
      const float Ls = wave_sum(lsum[j] * w);
      inv[j] = 1.0f / Ls;   // softmax normalisation is e * (1/sum) (tensor.ts:2211-2214)
    }
    lds_fence();
    // Every lane owns NOUT of the NREP x HD outputs; the partials of 8 chunks x NOUT outputs are requested at once
    // (one round trip per 16 chunks), and summed in chunk order.
    constexpr int NOUT = NREP * HD / 64;
    float O[NOUT];
    int off[NOUT], jj[NOUT];
#pragma unroll
    for (int i = 0; i < NOUT; i++) {
      const int e = i * 64 + lane;
      jj[i] = e / HD;
      off[i] = jj[i] * (HD + 2) + e % HD;
      O[i] = 0.0f;
    }
    for (int c2 = 0; c2 < n_active; c2 += 16) {
      float t16[NOUT][16];
#pragma unroll
      for (int u = 0; u < 16; u++) {
        const size_t cb = (size_t)(c2 + u < n_active ? c2 + u : n_active - 1) * NREP * (HD + 2);
#pragma unroll
        for (int i = 0; i < NOUT; i++) t16[i][u] = ld_coherent(base + cb + off[i]);
      }
#pragma unroll
      for (int u = 0; u < 16; u++)
        if (c2 + u < n_active) {
#pragma unroll
          for (int i = 0; i < NOUT; i++) O[i] = fmaf(t16[i][u], sc[jj[i] * SS_CHUNK + c2 + u], O[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < NOUT; i++) {
      float iv = inv[0];
#pragma unroll
      for (int j = 1; j < NREP; j++) iv = jj[i] == j ? inv[j] : iv;
      st_tagged(s.tattn + (size_t)g * NREP * HD + i * 64 + lane, tout, rn16(O[i] * iv));
    }
    astamp(s, 6);
  }

  // the attention phase of layer l as the control wavefront of this block runs it: items block, block + G, ...
  __device__ static __forceinline__ void phase(const SsArgs &s, const SsTabs &lt, SsCtl &ctl, float *sc, int l, int pos, uint32_t tin, uint32_t tout) {
    const int G = gridDim.x;
    const bool pos_ok = pos >= 0 && pos < s.max_context;
    astamp(s, 1);
    if (pos_ok && lds_ld(&ctl.abort) == 0) {
      const int T = pos + 1;
      const int chunk = chunk_rows(T, G / s.n_kv_heads);
      const int n_active = (T + chunk - 1) / chunk;
      const SsLayer L = ss_layer(lt, l);
      for (int item_id = blockIdx.x; item_id < s.n_kv_heads * n_active; item_id += G)
        item(s, ctl, L, sc, item_id / n_active, item_id % n_active, T, chunk, n_active, tin, tout);
    }
    astamp(s, 7);
  }
};

// ---- the control wavefront -----------------------------------------------------------------------------------------
template <int KIND, int HD, int NREP> struct SsControl {
  typedef _Float16 AT;
  typedef SsFmt<KIND> F;

  // wait until every block's flag has reached `target`
  __device__ static __forceinline__ void wait_flags(const SsArgs &s, SsCtl &ctl, int target) {
    const int lane = threadIdx.x & 63, G = gridDim.x;
    int it = 0;
    while (true) {
      int worst = 0;
      for (int b0 = 0; b0 < G; b0 += 256) {
        int v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const int b = b0 + k * 64 + lane;
          v[k] = b < G ? ld_coherent(&s.flags[b * SS_FLAG_STRIDE]) - target : 0;
        }
        worst = min(worst, min(min(v[0], v[1]), min(v[2], v[3])));
      }
      if (__all(worst >= 0)) return;
      if ((++it & 15) == 0) {
        if (lds_ld(&ctl.abort) != 0) return;
        if (it > SS_SPIN_GLOBAL || ld_coherent(s.err) != 0) {
          st_coherent(s.err, 1);
          lds_st(&ctl.abort, 1);
          return;
        }
      }
    }
  }

  // where the input row of a phase comes from: a tagged row written by other blocks, or a row of the embedding table
  enum { SRC_TAGGED = 0, SRC_EMB_F16 = 1, SRC_EMB_I8 = 2 };
  // N chunks of 8 halves of the input row for this lane: chunks c_first + i * 64 + lane (lanes past the end re-read the last
  // chunk: a load under a lane mask costs a full wait).  Tagged rows are asked for until every word carries `tag`.  An int8
  // embedding row becomes RN16(code * scale) per element (llama3.ts:71-77).
  template <int MODE, int N>
  __device__ static __forceinline__ void fetch_chunks(const SsArgs &s, SsCtl &ctl, const void *src, int c_first, int nchunks, uint32_t tag, float emb_scale, u4_t (&out)[N]) {
    const int lane = threadIdx.x & 63;
    if constexpr (MODE == SRC_TAGGED) {
      for (int it = 0;;) {
        bool ok = true;
#pragma unroll
        for (int i = 0; i < N; i++) {
          const int c = c_first + i * 64 + lane;
          out[i] = ld8_tagged((const uint32_t *)src + (size_t)(c < nchunks ? c : nchunks - 1) * 8, tag, ok);
        }
        if (__all(ok) || !ss_poll_again(s, ctl, it)) return;
      }
    } else {
#pragma unroll
      for (int i = 0; i < N; i++) {
        const int c = c_first + i * 64 + lane, cc = c < nchunks ? c : nchunks - 1;
        if constexpr (MODE == SRC_EMB_F16) {
          out[i] = ldg((const u4_t *)src + cc);
        } else {
          const uint64_t raw = ldg((const uint64_t *)src + cc);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            h2_t y;
            y[0] = mul_rn16((float)(int8_t)(raw >> (16 * e)), emb_scale);
            y[1] = mul_rn16((float)(int8_t)(raw >> (16 * e + 8)), emb_scale);
            out[i][e] = __builtin_bit_cast(uint32_t, y);
          }
        }
      }
    }
  }
  // RMSNorm'ed row -> LDS (nn/index.ts:586-588); a lane keeps NR chunks between the sum of squares and the scaling.
  template <int MODE, int NR>
  __device__ static __forceinline__ void stage_norm(const SsArgs &s, SsCtl &ctl, u4_t *xl, const void *src, const void *norm_w, int nchunks, float inv_d, uint32_t tag, float emb_scale) {
    const int lane = threadIdx.x & 63;
    u4_t xr[NR];
    fetch_chunks<MODE, NR>(s, ctl, src, 0, nchunks, tag, emb_scale, xr);
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < NR; i++) {
      const int c = i * 64 + lane;
      float part = ss;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        h2_t h = as_h2(xr[i][e]);
        part = fmaf((float)h[0], (float)h[0], part);
        part = fmaf((float)h[1], (float)h[1], part);
      }
      ss = c < nchunks ? part : ss;
    }
    const float tot = wave_sum(ss);
    // sqrt(1 / (mean + eps)), mean = sum * float(1/d)  (nn/index.ts:586, tensor.ts:2944-2946)
    const float r = __fsqrt_rn(__fdiv_rn(1.0f, __fadd_rn(__fmul_rn(tot, inv_d), s.eps)));
    constexpr int WB = NR < 8 ? NR : 8;   // norm weights are fetched WB chunks at a time
#pragma unroll
    for (int i0 = 0; i0 < NR; i0 += WB) {
      u4_t wr[WB];
#pragma unroll
      for (int i = 0; i < WB; i++) {
        const int c = (i0 + i) * 64 + lane;
        wr[i] = ldg((const u4_t *)norm_w + (c < nchunks ? c : nchunks - 1));
      }
#pragma unroll
      for (int i = 0; i < WB; i++) {
        const int c = (i0 + i) * 64 + lane;
        u4_t o;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          h2_t h = as_h2(xr[i0 + i][e]), w = as_h2(wr[i][e]), y;
          // .cast(x.dtype) before the weight multiply (nn/index.ts:588)
          y[0] = (_Float16)((float)(_Float16)((float)h[0] * r) * (float)w[0]);
          y[1] = (_Float16)((float)(_Float16)((float)h[1] * r) * (float)w[1]);
          o[e] = __builtin_bit_cast(uint32_t, y);
        }
        if (c < nchunks) xl[c] = o;
      }
    }
  }
  // Stage the input row of a weight phase in LDS.  src: in_f elements (tagged words written by other blocks, or the embedding
  // row); norm_w != nullptr applies RMSNorm.  The tail up to `padded` is zeroed.
  template <int MODE>
  __device__ static __forceinline__ void stage_x(const SsArgs &s, SsCtl &ctl, AT *xs, const void *src, const void *norm_w, int in_f, int padded, float inv_d, uint32_t tag, float emb_scale) {
    const int lane = threadIdx.x & 63;
    const int nchunks = in_f / 8;
    u4_t *xl = (u4_t *)xs;
    for (int c = nchunks + lane; c < padded / 8; c += 64) xl[c] = u4_t{0, 0, 0, 0};
    if (norm_w == nullptr) {
      constexpr int NB = 8;    // 32 loads of 8 bytes per lane and round trip
      for (int c0 = 0; c0 < nchunks; c0 += 64 * NB) {
        u4_t t[NB];
        fetch_chunks<MODE, NB>(s, ctl, src, c0, nchunks, tag, emb_scale, t);
#pragma unroll
        for (int i = 0; i < NB; i++) {
          const int c = c0 + i * 64 + lane;
          if (c < nchunks) xl[c] = t[i];
        }
      }
      return;
    }
    const int nr = (nchunks + 63) / 64;   // <= SS_NORM_CHUNKS (host)
    if (nr <= 1) stage_norm<MODE, 1>(s, ctl, xl, src, norm_w, nchunks, inv_d, tag, emb_scale);
    else if (nr <= 2) stage_norm<MODE, 2>(s, ctl, xl, src, norm_w, nchunks, inv_d, tag, emb_scale);
    else if (nr <= 4) stage_norm<MODE, 4>(s, ctl, xl, src, norm_w, nchunks, inv_d, tag, emb_scale);
    else stage_norm<MODE, 8>(s, ctl, xl, src, norm_w, nchunks, inv_d, tag, emb_scale);
  }

  // what the epilogue of one 64-slot pass needs besides the sums
  struct EpiOps {
    float sc0, sc1;   // row scale(s)
    float e0, e1;     // residual | (cos, sin)
  };
  struct EpiCtx {
    int kind;          // PH_*
    WDesc d;
    int ngroups, nb;
    const void *residual;
    void *y;
    SsLayer L;
    int pos;
    bool pos_ok;
    uint32_t tout;          // version tag of the rows this phase writes
    // layer 0: the residual of wo is the embedding row itself (every block reads it from the table)
    const void *emb_row;    // null: the residual is a tagged row
    bool emb_i8;
    float emb_scale;
  };
  // slot -> stacked row of the phase (or -1): slot = 2 * (local group of this block) + row of the pair
  __device__ static __forceinline__ int slot_row(const EpiCtx &e, int slot) {
    const int g = blockIdx.x + (slot >> 1) * gridDim.x;
    return g < e.ngroups ? 2 * g + (slot & 1) : -1;
  }
  __device__ static __forceinline__ void locate(const WDesc &d, int row, int &m, int &rr) {
    m = 0; rr = row;
    if (d.nm == 1 && d.rows1 > 0) {
      if (rr >= d.rows0) { rr -= d.rows0; m = 1; }
      if (m == 1 && rr >= d.rows1) { rr -= d.rows1; m = 2; }
    }
  }
  __device__ static __forceinline__ EpiOps epi_load(const SsArgs &s, const EpiCtx &e, int slot) {
    EpiOps o = {1.0f, 1.0f, 0.0f, 0.0f};
    const int row = slot_row(e, slot);
    if (row < 0) return o;
    int m, rr;
    locate(e.d, row, m, rr);
    if constexpr (KIND == JSGRAD_W_I8) {
      const _Float16 *sp = (const _Float16 *)((uintptr_t)e.d.s0 * (uintptr_t)(m == 0) + (uintptr_t)e.d.s1 * (uintptr_t)(m == 1) + (uintptr_t)e.d.s2 * (uintptr_t)(m == 2));
      o.sc0 = (float)ldg(sp + rr);
      if (e.d.nm == 2) o.sc1 = (float)ldg((const _Float16 *)e.d.s1 + rr);
    }
    if (e.kind == PH_QKV) {
      if (e.pos_ok && m < 2) {
        const int i = (rr % s.head_dim) >> 1;
        const AT *tp = (const AT *)s.rope_table + (size_t)e.pos * s.head_dim + 2 * i;
        o.e0 = (float)ldg(tp);
        o.e1 = (float)ldg(tp + 1);
      }
    } else if (e.residual != nullptr) {
      // a tagged row this block has already seen complete (it staged all of it one or two phases ago)
      if (e.emb_row == nullptr) o.e0 = ld_tagged_value((const uint32_t *)e.residual + row);
      else if (e.emb_i8) o.e0 = mul_rn16((float)ldg((const int8_t *)e.emb_row + row), e.emb_scale);
      else o.e0 = (float)ldg((const AT *)e.emb_row + row);
    }
    return o;
  }
  // best: running arg-max of the logits this lane has stored (PH_LM)
  __device__ static __forceinline__ void epi_apply(const SsArgs &s, const EpiCtx &e, int slot, const EpiOps &o, const float *y_local, float &best, int &best_i) {
    const int row = slot_row(e, slot);
    float v0 = 0.0f, v1 = 0.0f;
    if (row >= 0) {   // the k-batches of the row, added in batch order
      const float *part = y_local + ((size_t)(slot >> 1) * e.nb * e.d.nm) * 2 + (slot & 1);
      for (int bb = 0; bb < e.nb; bb++) {
        v0 += part[(bb * e.d.nm) * 2];
        if (e.d.nm == 2) v1 += part[(bb * e.d.nm + 1) * 2];
      }
    }
    if constexpr (KIND == JSGRAD_W_I8) { v0 = v0 * o.sc0; v1 = v1 * o.sc1; }
    v0 = rn16(v0);
    v1 = rn16(v1);
    // the other row of the pair sits in the neighbouring lane
    const float partner = dpp_f<0xB1>(v0);
    if (row < 0) return;
    if (e.kind == PH_QKV) {
      if (!e.pos_ok) return;
      int m, rr;
      locate(e.d, row, m, rr);
      if (m == 2) {
        st_coherent((AT *)e.L.cache_v + (size_t)e.pos * e.d.rows2 + rr, (AT)v0);   // for later tokens
        st_tagged(s.tkv + e.d.rows1 + rr, e.tout, v0);                              // for this token's attention
      } else {
        // interleaved pairs (llama.ts:17-32): (a, b) -> (a cos - b sin, a sin + b cos), unfused as in plain C
        const float c = o.e0, d = o.e1;
        const float out = (row & 1) ? rn16(partner * d + v0 * c) : rn16(v0 * c - partner * d);
        if (m == 0) st_tagged(s.tq + rr, e.tout, out);
        else {
          st_coherent((AT *)e.L.cache_k + (size_t)e.pos * e.d.rows1 + rr, (AT)out);
          st_tagged(s.tkv + rr, e.tout, out);
        }
      }
    } else if (e.kind == PH_FFN) {
      st_tagged((uint32_t *)e.y + row, e.tout, rn16(silu_act<AT>(v0) * v1));
    } else if (e.kind == PH_LM) {
      st_coherent((AT *)e.y + row, (AT)v0);
      if (v0 > best || (v0 == best && row < best_i)) { best = v0; best_i = row; }
    } else {
      float v = v0;
      if (e.residual != nullptr) v = rn16(o.e0 + v);
      st_tagged((uint32_t *)e.y + row, e.tout, v);
    }
  }

  __device__ static __forceinline__ void run(const SsArgs &s, const SsTabs &lt, SsCtl &ctl, AT *xs, const float *y_local, float *att_sc, int pos, int tok) {
    const int lane = threadIdx.x & 63, G = gridDim.x, nph = ss_phases(s);
    const bool pos_ok = pos >= 0 && pos < s.max_context;
    const int base = ld_coherent(s.epoch);
    int tr = 0;
    auto stamp = [&]() {
      if (s.trace && blockIdx.x == 0 && lane == 0 && tr < 2040) s.trace[tr++] = (long long)__builtin_amdgcn_s_memrealtime();
    };
    stamp();
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    if (!pos_ok && lane == 0) lds_st(&ctl.abort, 1);   // nothing will be written for such a position: nobody waits
    for (int p = 0; p < nph; p++) {
      const int kind = ss_kind(s, p);
      const uint32_t tin = ss_tag(base + p), tout = ss_tag(base + p + 1);   // versions of what the phase reads and writes
      stamp();
      if (kind == PH_ATTN) {
        stamp();
        SsAttn<HD, NREP>::phase(s, lt, ctl, att_sc, p / 5, pos, tin, tout);
        stamp();
      } else {
        EpiCtx e;
        e.kind = kind;
        e.d = ss_wdesc(s, lt, p);
        e.ngroups = wd_groups(e.d);
        e.nb = F::nbatch(e.d);
        e.pos = pos;
        e.pos_ok = pos_ok;
        e.tout = tout;
        e.L = ss_layer(lt, kind == PH_LM ? 0 : p / 5);
        e.residual = e.d.residual;
        e.y = e.d.y;
        // the embedding row (Embedding.call: a row gather) is the input of the first phase and the residual of the first wo
        const bool emb_i8 = s.embed_kind == JSGRAD_W_I8;
        const void *emb_row = (const char *)s.tok_emb + (size_t)tok * s.dim * (emb_i8 ? 1 : 2);
        float emb_scale = 1.0f;
        if (emb_i8 && p < 5) emb_scale = (float)ldg((const _Float16 *)s.tok_scale + tok);
        e.emb_row = p == PH_WO ? emb_row : nullptr;
        e.emb_i8 = emb_i8;
        e.emb_scale = emb_scale;
        const void *src = e.d.src, *norm_w = e.d.norm_w;
        const int padded = F::nbatch(e.d) * F::unroll(e.d.nm) * F::STEP;
        const float inv_d = (float)(1.0 / (double)e.d.in_f);
        if (p != 0) stage_x<SRC_TAGGED>(s, ctl, xs, src, norm_w, e.d.in_f, padded, inv_d, tin, 1.0f);
        else if (emb_i8) stage_x<SRC_EMB_I8>(s, ctl, xs, emb_row, norm_w, e.d.in_f, padded, inv_d, tin, emb_scale);
        else stage_x<SRC_EMB_F16>(s, ctl, xs, emb_row, norm_w, e.d.in_f, padded, inv_d, tin, emb_scale);
        lds_fence();
        lds_st(&ctl.x_ready, ss_wordinal(s, p) + 1);
        stamp();
        const int nslots = ss_block_groups(e.ngroups) * 2;
        EpiOps cur = epi_load(s, e, lane);
        lds_wait_all(s, ctl, ctl.wdone, SS_NWW, ss_wordinal(s, p) + 1);
        lds_fence();
        stamp();
        for (int s0 = 0; s0 < nslots; s0 += 64) {
          EpiOps nxt = cur;
          if (s0 + 64 < nslots) nxt = epi_load(s, e, s0 + 64 + lane);
          epi_apply(s, e, s0 + lane, cur, y_local, best, best_i);
          cur = nxt;
        }
        if (kind == PH_LM) {
          for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(best, off);
            const int oi = __shfl_xor(best_i, off);
            if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
          }
          if (lane == 0) { st_coherent(&s.amax_val[blockIdx.x], best); st_coherent(&s.amax_idx[blockIdx.x], best_i); }
          // the one flag of the step: this block's logits and arg-max partial are at the coherence point
          vm_drain();
          if (lane == 0) st_coherent(&s.flags[blockIdx.x * SS_FLAG_STRIDE], base + nph);
        }
        stamp();
      }
    }
    if (blockIdx.x != 0) return;
    // ---- greedy arg-max over the blocks' partials (Tensor.argmax: lowest index among the maxima), state update
    wait_flags(s, ctl, base + nph);
    best = -INFINITY;
    best_i = 0x7fffffff;
    for (int b = lane; b < G; b += 64) {
      const float ov = ld_coherent(&s.amax_val[b]);
      const int oi = ld_coherent(&s.amax_idx[b]);
      if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off);
      const int oi = __shfl_xor(best_i, off);
      if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (lane == 0) {
      if (best_i == 0x7fffffff) best_i = s.vocab;
      if (s.tokens_out && pos >= 0 && pos < s.tokens_cap) s.tokens_out[pos] = best_i;
      s.state[0] = best_i;
      s.state[1] = pos + 1;
      st_coherent(s.epoch, base + nph + 1);
    }
    stamp();
  }
};

template <int KIND, int HD, int NREP>
__global__ __launch_bounds__(SS_THREADS) void stream_step_kernel(SsArgs s) {
  extern __shared__ __align__(16) unsigned char smem[];
  _Float16 *xs = (_Float16 *)smem;
  float *y_local = (float *)(smem + s.x_bytes);
  float *att_sc = y_local + SS_YMAX;
  SsCtl &ctl = *(SsCtl *)(att_sc + NREP * SS_CHUNK);
  uint64_t *lt_w = (uint64_t *)(&ctl + 1);   // 8-byte aligned: everything before it is a multiple of 8 bytes
  uint64_t *pt_w = lt_w + (size_t)s.n_layers * SS_LAYER_WORDS;
  SsTabs lt;
  lt.layers = (LtPtr)lt_w;
  lt.phases = (LtPtr)pt_w;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pos = s.state[1];
  int tok = s.state[0];
  tok = tok < 0 ? 0 : (tok >= s.vocab ? s.vocab - 1 : tok);
  if (threadIdx.x < (int)(sizeof(SsCtl) / sizeof(int))) ((int *)&ctl)[threadIdx.x] = 0;
  for (int i = threadIdx.x; i < s.n_layers * SS_LAYER_WORDS; i += SS_THREADS) lt_w[i] = ldg((const uint64_t *)s.layers + i);
  for (int p = threadIdx.x; p < ss_phases(s); p += SS_THREADS) ss_build_phase(s, pt_w + (size_t)p * SS_PHASE_WORDS, p, SsFmt<KIND>::VEC);
  __syncthreads();   // the only block-wide barrier: from here on the wavefronts go their own ways

  if (wave < SS_NWW) SsWeights<KIND>::run(s, lt, ctl, xs, y_local, wave);
  else SsControl<KIND, HD, NREP>::run(s, lt, ctl, xs, y_local, att_sc, pos, tok);
}

template <int KIND, int HD> static int launch_stream(const SsArgs &s, int n_rep, int grid, size_t lds) {
#define JSG_REP(N)                                                                                                              \
  case N: {                                                                                                                     \
    static size_t configured = 0;                                                                                               \
    if (lds > 48 * 1024 && lds > configured) {                                                                                  \
      JSG_HIP(hipFuncSetAttribute((const void *)stream_step_kernel<KIND, HD, N>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
      configured = lds;                                                                                                         \
    }                                                                                                                           \
    JSG_LAUNCH(PROF_STEP, (stream_step_kernel<KIND, HD, N>), dim3(grid), dim3(SS_THREADS), lds, s);                            \
  } break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(4)
    default: return fail("jsgrad_hip_stream_step: n_heads/n_kv_heads = %d is not one of 1,2,4", n_rep);
  }
#undef JSG_REP
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_stream_workspace_bytes(int n_heads, int n_kv_heads, int head_dim) {
  // flags and counters | attention partials | tagged rows: h, h2 (SS_TAG_DIM each), g (SS_TAG_HIDDEN), attn, q, k | v of the position
  const size_t partial = (size_t)n_heads * SS_MAXCH * (head_dim + 2) * sizeof(float);
  const size_t tagged = ((size_t)2 * SS_TAG_DIM + SS_TAG_HIDDEN + (size_t)2 * n_heads * head_dim + (size_t)2 * n_kv_heads * head_dim) * sizeof(uint32_t);
  return SS_WS_PARTIAL + partial + tagged;
}

int jsgrad_hip_stream_step(const jsgrad_hip_step_t *d) {
  const char *who = "jsgrad_hip_stream_step";
  JSG_READY();
  JSG_REQUIRE(d && d->layers && d->workspace && d->state && d->h && d->h2 && d->q && d->attn && d->g && d->logits && d->tok_emb && d->out_w && d->final_norm && d->rope_table,
              "%s: null pointer in the descriptor", who);
  JSG_REQUIRE(d->act == JSGRAD_F16, "%s: built for fp16 activations", who);
  JSG_REQUIRE(d->kind == JSGRAD_W_F16 || d->kind == JSGRAD_W_I8, "%s: weight kind %d (fp16 and int8 are built)", who, d->kind);
  JSG_REQUIRE(d->out_kind == d->kind, "%s: the lm_head must be stored like the layers (kind %d vs %d)", who, d->out_kind, d->kind);
  JSG_REQUIRE(d->embed_kind == JSGRAD_W_F16 || (d->embed_kind == JSGRAD_W_I8 && d->tok_scale), "%s: embedding kind %d", who, d->embed_kind);
  JSG_REQUIRE(d->n_layers >= 1 && d->dim > 0 && d->hidden > 0 && d->vocab > 0 && d->max_context > 0, "%s: bad shape", who);
  JSG_REQUIRE(d->n_kv_heads > 0 && d->n_kv_heads <= 64 && d->n_heads % d->n_kv_heads == 0, "%s: n_heads %d / n_kv_heads %d", who, d->n_heads, d->n_kv_heads);
  JSG_REQUIRE(d->head_dim == 64 || d->head_dim == 128, "%s: head_dim %d (64 and 128 are built)", who, d->head_dim);
  const int vec = d->kind == JSGRAD_W_F16 ? 8 : 16;
  const int qdim = d->n_heads * d->head_dim;
  JSG_REQUIRE(d->dim % vec == 0 && d->hidden % vec == 0 && qdim % vec == 0, "%s: feature sizes must be multiples of %d", who, vec);
  JSG_REQUIRE(d->dim % 2 == 0 && d->hidden % 2 == 0 && d->vocab % 2 == 0, "%s: row counts must be even", who);
  JSG_REQUIRE(d->dim <= SS_NORM_CHUNKS * 64 * 8, "%s: dim %d exceeds the fused RMSNorm limit of %d", who, d->dim, SS_NORM_CHUNKS * 64 * 8);
  JSG_REQUIRE(d->dim <= SS_TAG_DIM && d->hidden <= SS_TAG_HIDDEN, "%s: dim %d / hidden %d exceed the workspace rows of %d / %d", who, d->dim, d->hidden, SS_TAG_DIM, SS_TAG_HIDDEN);
  JSG_REQUIRE(d->dim % 8 == 0 && d->hidden % 8 == 0 && qdim % 8 == 0, "%s: feature sizes must be multiples of 8", who);
  JSG_REQUIRE(d->kind == JSGRAD_W_F16 || d->out_s, "%s: quantised lm_head needs a scale", who);
  JSG_REQUIRE(d->max_context <= SS_MAXCH * SS_CHUNK, "%s: max_context %d exceeds %d", who, d->max_context, SS_MAXCH * SS_CHUNK);
  const int grid = state().cu_count;   // one block per CU: every block is resident, which the flags need
  JSG_REQUIRE(grid <= SS_MAX_BLOCKS, "%s: %d CUs exceed the flag array", who, grid);
  // partial sums a block holds in LDS per phase: groups per block x k-batches x matrices x 2 rows
  const int step_k = 64 * (d->kind == JSGRAD_W_F16 ? 8 : 16);
  auto sums = [&](int rows, int in_f, int nm) {
    const int u = nm == 2 ? 2 : 4, nb = ((in_f + step_k - 1) / step_k + u - 1) / u;
    return ((rows / 2 + grid - 1) / grid) * nb * nm * 2;
  };
  const int most = std::max(std::max(sums(qdim + 2 * d->n_kv_heads * d->head_dim, d->dim, 1), sums(d->hidden, d->dim, 2)),
                            std::max(std::max(sums(d->dim, qdim, 1), sums(d->dim, d->hidden, 1)), sums(d->vocab, d->dim, 1)));
  JSG_REQUIRE(most <= SS_YMAX, "%s: %d partial sums per block exceed %d", who, most, SS_YMAX);
  JSG_REQUIRE(d->vocab >= 2 * grid, "%s: vocab %d is smaller than two rows per block", who, d->vocab);
  const int n_rep = d->n_heads / d->n_kv_heads;
  int xe = std::max(ss_x_elems(d->kind, d->dim, 1), ss_x_elems(d->kind, d->dim, 2));
  xe = std::max(xe, std::max(ss_x_elems(d->kind, qdim, 1), ss_x_elems(d->kind, d->hidden, 1)));
  const size_t x_bytes = ((size_t)xe * sizeof(_Float16) + 255) & ~(size_t)255;
  const size_t lds = x_bytes + SS_YMAX * sizeof(float) + (size_t)n_rep * SS_CHUNK * sizeof(float) + sizeof(SsCtl) + (size_t)d->n_layers * sizeof(SsLayer) +
                     (size_t)(5 * d->n_layers + 1) * SS_PHASE_WORDS * 8;
  JSG_REQUIRE(d->n_layers <= 128, "%s: %d layers exceed the LDS table of layer tensors", who, d->n_layers);
  JSG_REQUIRE(lds <= 160 * 1024, "%s: %zu bytes of LDS needed", who, lds);

  SsArgs s = {};
  s.layers = (const SsLayer *)d->layers;
  s.n_layers = d->n_layers; s.dim = d->dim; s.hidden = d->hidden; s.n_heads = d->n_heads; s.n_kv_heads = d->n_kv_heads; s.head_dim = d->head_dim;
  s.vocab = d->vocab; s.max_context = d->max_context; s.eps = d->eps; s.embed_kind = d->embed_kind;
  s.tok_emb = d->tok_emb; s.tok_scale = d->tok_scale; s.out_w = d->out_w; s.out_s = d->out_s; s.final_norm = d->final_norm; s.rope_table = d->rope_table;
  s.state = d->state; s.tokens_out = d->tokens_out; s.tokens_cap = d->tokens_cap;
  s.h = d->h; s.h2 = d->h2; s.q = d->q; s.attn = d->attn; s.g = d->g; s.logits = d->logits;
  char *ws = (char *)d->workspace;
  s.epoch = (int *)(ws + SS_WS_EPOCH);
  s.err = (int *)(ws + SS_WS_ERR);
  s.attn_counters = (int *)(ws + SS_WS_COUNTERS);
  s.amax_val = (float *)(ws + SS_WS_AMAX_VAL);
  s.amax_idx = (int *)(ws + SS_WS_AMAX_IDX);
  s.flags = (int *)(ws + SS_WS_FLAGS);
  s.attn_partial = (float *)(ws + SS_WS_PARTIAL);
  s.th = (uint32_t *)(ws + SS_WS_PARTIAL + (size_t)d->n_heads * SS_MAXCH * (d->head_dim + 2) * sizeof(float));
  s.th2 = s.th + SS_TAG_DIM;
  s.tg = s.th2 + SS_TAG_DIM;
  s.tattn = s.tg + SS_TAG_HIDDEN;
  s.tq = s.tattn + (size_t)d->n_heads * d->head_dim;
  s.tkv = s.tq + (size_t)d->n_heads * d->head_dim;
  s.trace = d->trace;
  s.x_bytes = (int)x_bytes;
  s.grid = grid;
#define JSG_KIND(K)                                                                                  \
  case K:                                                                                            \
    return d->head_dim == 64 ? launch_stream<K, 64>(s, n_rep, grid, lds) : launch_stream<K, 128>(s, n_rep, grid, lds);
  switch (d->kind) {
    JSG_KIND(JSGRAD_W_F16)
    JSG_KIND(JSGRAD_W_I8)
  }
#undef JSG_KIND
  return fail("%s: weight kind %d", who, d->kind);
}

int jsgrad_hip_stream_status(const void *workspace, int *host_out_error) {
  JSG_READY();
  JSG_REQUIRE(workspace && host_out_error, "jsgrad_hip_stream_status: null pointer");
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_stream_status during graph capture");
  JSG_HIP(hipMemcpyAsync(host_out_error, (const char *)workspace + SS_WS_ERR, sizeof(int), hipMemcpyDeviceToHost, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));
  return 0;
}

}  // extern "C"
