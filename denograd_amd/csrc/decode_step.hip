// One decode step of the whole Llama decoder as a single persistent kernel for gfx950.
//
// The stand-alone kernels spend 4-5 us per launch on dispatch ramp, first-load latency and tail, and a decode step has
// 5 launches per layer: at batch 1 that fixed cost is as large as the time the weights need at full HBM rate.  Here one
// block of 16 wavefronts per CU stays resident for the whole step (Transformer.forward, models/llama.ts:201-213) and walks
// the same phases - attention_norm + wq/wk/wv + rotary + cache write | GQA attention | wo + residual | ffn_norm + w1/w3 +
// SwiGLU | w2 + residual - separated by grid barriers.  Every wavefront requests the first weight batch of the NEXT
// phase before it waits at a barrier, so the HBM stream does not stop while the barrier and the x hand-off complete.
// The arithmetic is the stand-alone kernels' (gemv_core.h, attention_core.h): every output row is summed by one wavefront
// in the same order, so the results are identical.
//
// Cross-block data (activation rows, the new KV row, attention partials) is written with agent-scope stores and read
// with agent-scope loads; the barrier is two levels of agent-scope counters (8 groups, then one word everybody polls).
// Every wait is bounded: when a spin runs out the block raises the error word and goes on, so the grid always drains.
#include "attention_core.h"
#include "gemv_core.h"

namespace jsg {

constexpr int STEP_THREADS = 512;
constexpr int STEP_NW = STEP_THREADS / 64;
constexpr int BAR_GROUPS = 8;
constexpr int BAR_STRIDE = 32;   // ints between counters: one 128-byte line each
constexpr int SPIN_LIMIT = 1 << 19;  // polls of ~0.2 us: about 0.1 s, then the error word is raised and no later wait spins

// device copy of one TransformerBlock's tensors (layout shared with the host, see jsgrad_hip_layer_t)
struct StepLayer {
  const void *wq, *wk, *wv, *wo, *w1, *w2, *w3;
  const void *sq, *sk, *sv, *so, *s1, *s2, *s3;
  const void *attention_norm, *ffn_norm;
  void *cache_k, *cache_v;
};
struct StepArgs {
  const StepLayer *layers;
  int n_layers, dim, hidden, n_heads, n_kv_heads, head_dim, vocab, max_context;
  float eps;
  int embed_kind;
  const void *tok_emb, *tok_scale, *out_w, *out_s, *final_norm, *rope_table;
  int32_t *state, *tokens_out;
  int tokens_cap;
  void *h, *h2, *q, *attn, *g, *logits;
  float *attn_partial;   // [n_kv_heads][nsplit][n_rep][HD + 2]
  int *attn_counters;    // [n_kv_heads]
  int nsplit;
  int *bar;              // BAR_WORDS ints, zero between launches
  int *err;              // set to 1 when a bounded wait ran out
  float *amax_val;       // [gridDim] per-block argmax partials
  int *amax_idx;
  long long *trace;      // optional: block 0 stamps the 100 MHz clock at every phase boundary (debugging aid)
};

// ---- grid barrier in two halves: arrive (after this block's outputs are acknowledged), then - after the caller has
// put the next phase's first weight loads in flight - wait.  Arrival is on a group counter; the last of a group arrives
// on the top counter, which everybody polls.  The arrival must go out BEFORE the bulk loads: a CU's memory pipeline is
// in order, so an atomic queued behind 64 KiB of weight loads reaches the counter microseconds late.
__device__ __forceinline__ void barrier_arrive(const StepArgs &s, int epoch) {
  __syncthreads();  // all coherent stores of this block are acknowledged
  if (threadIdx.x == 0) {
    const int G = gridDim.x, grp = blockIdx.x % BAR_GROUPS, gsize = (G - grp + BAR_GROUPS - 1) / BAR_GROUPS;
    const int old = __hip_atomic_fetch_add(&s.bar[BAR_STRIDE * (1 + grp)], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old == gsize * (epoch + 1) - 1) __hip_atomic_fetch_add(&s.bar[0], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
__device__ __forceinline__ void barrier_wait(const StepArgs &s, int &epoch) {
  if (threadIdx.x == 0) {
    const int G = gridDim.x, ngrp = G < BAR_GROUPS ? G : BAR_GROUPS;
    const int target = ngrp * (epoch + 1);
    int it = 0;
    while (ld_coherent(&s.bar[0]) < target) {
      __builtin_amdgcn_s_sleep(1);
      if ((++it & 1023) == 0 && ld_coherent(s.err) != 0) break;      // somebody already gave up: drain
      if (it > SPIN_LIMIT) { st_coherent(s.err, 1); break; }
    }
  }
  epoch++;
  __syncthreads();
}
__device__ __forceinline__ void grid_barrier(const StepArgs &s, int &epoch) {
  barrier_arrive(s, epoch);
  barrier_wait(s, epoch);
}

#ifndef JSG_STEP_TOUCH
#define JSG_STEP_TOUCH 0
#endif

template <int KIND, int HD, int NREP>
__global__ __launch_bounds__(STEP_THREADS) void decode_step_kernel(StepArgs s) {
  typedef _Float16 AT;
  typedef Gemv<KIND, AT, EPI_ROPE_KV, 2, 4, true> GQ;
  typedef Gemv<KIND, AT, EPI_STORE, 2, 4, true> GL;
  typedef Gemv<KIND, AT, EPI_SWIGLU, 2, 2, true> GF;
  typedef Attn<AT, HD, NREP, STEP_NW, true> AttnT;
  extern __shared__ __align__(16) unsigned char smem[];  // x row of the current GEMV phase, or the attention scratch
  __shared__ float red[STEP_NW];
  __shared__ float lut[16];
  __shared__ float vmax[STEP_NW];
  __shared__ int imax[STEP_NW];
  AT *xs = (AT *)smem;
  typename AttnT::Smem &asm_ = *(typename AttnT::Smem *)smem;

  const int tid = threadIdx.x;
  const int pos = s.state[1];
  int tok = s.state[0];
  tok = tok < 0 ? 0 : (tok >= s.vocab ? s.vocab - 1 : tok);
  const bool pos_ok = pos >= 0 && pos < s.max_context;
  int epoch = 0;
  int tr = 0;
  auto stamp = [&]() {
    if (s.trace && blockIdx.x == 0 && tid == 0 && tr < 2040) s.trace[tr++] = (long long)__builtin_amdgcn_s_memrealtime();
  };
  stamp();
  const float inv_dim = (float)(1.0 / (double)s.dim);

  auto qkv_args = [&](const StepLayer &L) {
    GemvArgs a = {};
    a.w0 = L.wq; a.w1 = L.wk; a.w2 = L.wv; a.s0 = L.sq; a.s1 = L.sk; a.s2 = L.sv;
    a.rows0 = s.n_heads * HD; a.rows1 = s.n_kv_heads * HD; a.rows2 = s.n_kv_heads * HD;
    a.in_f = s.dim; a.x = s.h; a.norm_w = L.attention_norm; a.eps = s.eps; a.inv_d = inv_dim; a.y = s.q;
    a.rope_table = s.rope_table; a.st = s.state; a.cache_k = L.cache_k; a.cache_v = L.cache_v; a.head_dim = HD; a.max_context = s.max_context;
    return a;
  };
  auto lin_args = [&](const void *w, const void *sc, int out_f, int in_f, const void *x, void *y, const void *norm, const void *res, float inv_d) {
    GemvArgs a = {};
    a.w0 = w; a.s0 = sc; a.rows0 = out_f; a.in_f = in_f; a.x = x; a.norm_w = norm; a.eps = s.eps; a.inv_d = inv_d; a.y = y; a.residual = res;
    return a;
  };
  auto ffn_args = [&](const StepLayer &L) {
    GemvArgs a = {};
    a.w0 = L.w1; a.s0 = L.s1; a.w1 = L.w3; a.s1 = L.s3; a.rows0 = s.hidden; a.rows1 = s.hidden; a.in_f = s.dim; a.x = s.h2;
    a.norm_w = L.ffn_norm; a.eps = s.eps; a.inv_d = inv_dim; a.y = s.g;
    return a;
  };

  // Lines of the next phase's weights beyond the one prefetched item are pulled into L2 while the block waits at a
  // barrier or works through attention (TOUCH items per wavefront; 0 switches it off).
  constexpr int TOUCH = JSG_STEP_TOUCH;
  uint32_t tw[TOUCH > 0 ? TOUCH : 1], sink = 0;

  // first weights of layer 0 go out before anything else
  GemvBuf pre;   // the one buffer that carries the next phase's first item across a barrier
  if (s.n_layers > 0) GQ::prefetch(qkv_args(s.layers[0]), pre, pos);

  // ---- embedding row -> h (Embedding.call / Int8Embedding.call: a row gather)
  if (blockIdx.x == 0) {
    for (int i = tid; i < s.dim; i += STEP_THREADS) {
      float v;
      if (s.embed_kind == JSGRAD_W_F16) v = (float)((const _Float16 *)s.tok_emb)[(size_t)tok * s.dim + i];
      else v = (float)mul_rn16((float)((const int8_t *)s.tok_emb)[(size_t)tok * s.dim + i], (float)((const _Float16 *)s.tok_scale)[tok]);
      st_coherent((AT *)s.h + i, (AT)v);
    }
  }
  grid_barrier(s, epoch);

  for (int l = 0; l < s.n_layers; l++) {
    const StepLayer &L = s.layers[l];
    // attention_norm + wq/wk/wv + rotary + cache write
    GQ::run(qkv_args(L), xs, red, lut, pre, true, pos);
    stamp();
    const GemvArgs awo = lin_args(L.wo, L.so, s.dim, s.n_heads * HD, s.attn, s.h2, nullptr, s.h, 0.0f);
    barrier_arrive(s, epoch);
    GL::prefetch(awo, pre, pos);
    if constexpr (TOUCH > 0) GL::template touch<TOUCH>(awo, 1, tw);
    barrier_wait(s, epoch);
    if constexpr (TOUCH > 0) GL::template touch_wait<TOUCH>(tw, sink);
    stamp();

    // attention over cache rows [0, pos]: items (kv head, chunk) spread over the blocks
    if (pos_ok) {
      const int T = pos + 1;
      int per_head = gridDim.x / s.n_kv_heads;                     // blocks available per kv head
      per_head = per_head < 1 ? 1 : (per_head > s.nsplit ? s.nsplit : per_head);
      int chunk = (T + per_head - 1) / per_head;
      chunk = chunk < 64 ? 64 : chunk;                               // one pass of the 16 wavefronts covers 64-128 rows
      chunk = chunk > ATT_CHUNK_MAX ? ATT_CHUNK_MAX : chunk;         // (host guarantees max_context <= nsplit * ATT_CHUNK_MAX)
      const int n_active = (T + chunk - 1) / chunk;
      AttnArgs aa;
      aa.q = s.q; aa.cache_k = L.cache_k; aa.cache_v = L.cache_v; aa.st = s.state; aa.out = s.attn;
      aa.counters = s.attn_counters; aa.partial = s.attn_partial; aa.n_kv_heads = s.n_kv_heads; aa.nsplit = s.nsplit; aa.max_context = s.max_context;
      aa.scale = (float)(1.0 / sqrt((double)HD));
      for (int item = blockIdx.x; item < s.n_kv_heads * n_active; item += gridDim.x) {
        AttnT::item(aa, asm_, item / n_active, item % n_active, T, chunk, n_active);
        __syncthreads();
      }
    }
    stamp();
    grid_barrier(s, epoch);
    stamp();

    // wo + residual -> h2
    GL::run(awo, xs, red, lut, pre, true, pos);
    stamp();
    barrier_arrive(s, epoch);
    GF::prefetch(ffn_args(L), pre, pos);
    if constexpr (TOUCH > 0) GF::template touch<TOUCH>(ffn_args(L), 1, tw);
    barrier_wait(s, epoch);
    if constexpr (TOUCH > 0) GF::template touch_wait<TOUCH>(tw, sink);
    stamp();

    // ffn_norm + w1/w3 + SwiGLU -> g
    GF::run(ffn_args(L), xs, red, lut, pre, true, pos);
    stamp();
    const GemvArgs aw2 = lin_args(L.w2, L.s2, s.dim, s.hidden, s.g, s.h, nullptr, s.h2, 0.0f);
    barrier_arrive(s, epoch);
    GL::prefetch(aw2, pre, pos);
    if constexpr (TOUCH > 0) GL::template touch<TOUCH>(aw2, 1, tw);
    barrier_wait(s, epoch);
    if constexpr (TOUCH > 0) GL::template touch_wait<TOUCH>(tw, sink);
    stamp();

    // w2 + residual -> h
    GL::run(aw2, xs, red, lut, pre, true, pos);
    stamp();
    barrier_arrive(s, epoch);
    if (l + 1 < s.n_layers) {
      GQ::prefetch(qkv_args(s.layers[l + 1]), pre, pos);
      if constexpr (TOUCH > 0) GQ::template touch<TOUCH>(qkv_args(s.layers[l + 1]), 1, tw);
    } else {
      const GemvArgs alm = lin_args(s.out_w, s.out_s, s.vocab, s.dim, s.h, s.logits, s.final_norm, nullptr, inv_dim);
      GL::prefetch(alm, pre, pos);
      if constexpr (TOUCH > 0) GL::template touch<TOUCH>(alm, 1, tw);
    }
    barrier_wait(s, epoch);
    if constexpr (TOUCH > 0) GL::template touch_wait<TOUCH>(tw, sink);
    stamp();
  }

  // ---- final norm + lm_head -> logits
  GL::run(lin_args(s.out_w, s.out_s, s.vocab, s.dim, s.h, s.logits, s.final_norm, nullptr, inv_dim), xs, red, lut, pre, s.n_layers > 0, pos);
  stamp();
  grid_barrier(s, epoch);
  stamp();

  // ---- greedy argmax (Tensor.argmax: lowest index among the maxima), two levels
  {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    auto merge = [&](float ov, int oi) { if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; } };
    auto block_reduce = [&]() {
      for (int off = 32; off > 0; off >>= 1) merge(__shfl_xor(best, off), __shfl_xor(bi, off));
      if ((tid & 63) == 0) { vmax[tid >> 6] = best; imax[tid >> 6] = bi; }
      __syncthreads();
      if (tid == 0)
        for (int w = 1; w < STEP_NW; w++) merge(vmax[w], imax[w]);
    };
    for (int i = blockIdx.x * STEP_THREADS + tid; i < s.vocab; i += gridDim.x * STEP_THREADS) merge((float)ld_coherent((const AT *)s.logits + i), i);
    block_reduce();
    if (tid == 0) { st_coherent(&s.amax_val[blockIdx.x], best); st_coherent(&s.amax_idx[blockIdx.x], bi); }
    grid_barrier(s, epoch);
    if (blockIdx.x == 0) {
      best = -INFINITY;
      bi = 0x7fffffff;
      for (int i = tid; i < (int)gridDim.x; i += STEP_THREADS) merge(ld_coherent(&s.amax_val[i]), ld_coherent(&s.amax_idx[i]));
      block_reduce();
      if (tid == 0) {
        if (bi == 0x7fffffff) bi = s.vocab;
        if (s.tokens_out && pos >= 0 && pos < s.tokens_cap) s.tokens_out[pos] = bi;
        s.state[0] = bi;
        s.state[1] = pos + 1;
      }
    }
  }

  if (s.n_layers < 0) st_coherent(s.err, (int)sink);   // never taken (the host checks n_layers): keeps the touched words alive

  // ---- leave the barrier words at zero for the next launch: the last block out clears them
  if (tid == 0) {
    const int done = __hip_atomic_fetch_add(&s.bar[BAR_STRIDE * (BAR_GROUPS + 1)], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (done == (int)gridDim.x - 1)
      for (int i = 0; i <= BAR_GROUPS + 1; i++) st_coherent(&s.bar[BAR_STRIDE * i], 0);
  }
}

template <int KIND, int HD> static int launch_step(const StepArgs &s, int n_rep, int grid, size_t lds) {
#define JSG_REP(N)                                                                                                   \
  case N:                                                                                                            \
    JSG_LAUNCH(PROF_STEP, (decode_step_kernel<KIND, HD, N>), dim3(grid), dim3(STEP_THREADS), lds, s);                \
    break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(3) JSG_REP(4)
    default: return fail("jsgrad_hip_decode_step: n_heads/n_kv_heads = %d is not one of 1,2,3,4", n_rep);
  }
#undef JSG_REP
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_step_workspace_bytes(int n_heads, int n_kv_heads, int head_dim) {
  (void)n_kv_heads;
  // barrier words | error word | attention counters | argmax partials | attention partials (64 chunks per kv head)
  return 4096 + 256 + 256 + 8192 + (size_t)n_heads * 64 * (head_dim + 2) * sizeof(float);
}

int jsgrad_hip_decode_step(const jsgrad_hip_step_t *d) {
  JSG_READY();
  JSG_REQUIRE(d && d->layers && d->workspace && d->state && d->h && d->h2 && d->q && d->attn && d->g && d->logits && d->tok_emb && d->out_w && d->final_norm && d->rope_table,
              "jsgrad_hip_decode_step: null pointer in the descriptor");
  JSG_REQUIRE(d->act == JSGRAD_F16, "jsgrad_hip_decode_step: built for fp16 activations");
  JSG_REQUIRE(d->kind == JSGRAD_W_F16 || d->kind == JSGRAD_W_I8, "jsgrad_hip_decode_step: weight kind %d (fp16 and int8 are built)", d->kind);
  JSG_REQUIRE(d->out_kind == d->kind, "jsgrad_hip_decode_step: the lm_head must be stored like the layers (kind %d vs %d)", d->out_kind, d->kind);
  JSG_REQUIRE(d->embed_kind == JSGRAD_W_F16 || (d->embed_kind == JSGRAD_W_I8 && d->tok_scale), "jsgrad_hip_decode_step: embedding kind %d", d->embed_kind);
  JSG_REQUIRE(d->n_layers >= 0 && d->dim > 0 && d->hidden > 0 && d->vocab > 0 && d->max_context > 0, "jsgrad_hip_decode_step: bad shape");
  JSG_REQUIRE(d->n_kv_heads > 0 && d->n_kv_heads <= 64 && d->n_heads % d->n_kv_heads == 0, "jsgrad_hip_decode_step: n_heads %d / n_kv_heads %d", d->n_heads, d->n_kv_heads);
  JSG_REQUIRE(d->head_dim == 64 || d->head_dim == 128, "jsgrad_hip_decode_step: head_dim %d (64 and 128 are built)", d->head_dim);
  const int vec = d->kind == JSGRAD_W_F16 ? 8 : 16;
  JSG_REQUIRE(d->dim % vec == 0 && d->hidden % vec == 0 && (d->n_heads * d->head_dim) % vec == 0, "jsgrad_hip_decode_step: feature sizes must be multiples of %d", vec);
  JSG_REQUIRE(d->dim <= 4 * STEP_THREADS * 8, "jsgrad_hip_decode_step: dim %d exceeds the fused RMSNorm limit", d->dim);
  JSG_REQUIRE(d->kind == JSGRAD_W_F16 || d->out_s, "jsgrad_hip_decode_step: quantised lm_head needs a scale");
  JSG_REQUIRE(fits_buffer_offsets((size_t)d->vocab, (size_t)d->dim, 16) && fits_buffer_offsets((size_t)d->hidden, (size_t)d->dim, 16),
              "jsgrad_hip_decode_step: a weight matrix reaches 4 GiB (32-bit byte offsets)");
  const int nsplit = 64;
  JSG_REQUIRE(d->max_context <= nsplit * ATT_CHUNK_MAX, "jsgrad_hip_decode_step: max_context %d exceeds %d", d->max_context, nsplit * ATT_CHUNK_MAX);
  const int feat = d->hidden > d->dim ? d->hidden : d->dim;
  size_t lds = (size_t)(feat > d->n_heads * d->head_dim ? feat : d->n_heads * d->head_dim) * sizeof(_Float16);
  const size_t attn_lds = 40 * 1024;   // >= sizeof(Attn<half, 128, 4, 16>::Smem)
  static_assert(sizeof(Attn<_Float16, 128, 4, 16, true>::Smem) <= 40 * 1024, "attention LDS of the step kernel");
  if (lds < attn_lds) lds = attn_lds;
  JSG_REQUIRE(lds <= 60 * 1024, "jsgrad_hip_decode_step: %zu bytes of LDS needed", lds);

  StepArgs s = {};
  s.layers = (const StepLayer *)d->layers;
  s.n_layers = d->n_layers; s.dim = d->dim; s.hidden = d->hidden; s.n_heads = d->n_heads; s.n_kv_heads = d->n_kv_heads; s.head_dim = d->head_dim;
  s.vocab = d->vocab; s.max_context = d->max_context; s.eps = d->eps; s.embed_kind = d->embed_kind;
  s.tok_emb = d->tok_emb; s.tok_scale = d->tok_scale; s.out_w = d->out_w; s.out_s = d->out_s; s.final_norm = d->final_norm; s.rope_table = d->rope_table;
  s.state = d->state; s.tokens_out = d->tokens_out; s.tokens_cap = d->tokens_cap;
  s.h = d->h; s.h2 = d->h2; s.q = d->q; s.attn = d->attn; s.g = d->g; s.logits = d->logits;
  char *ws = (char *)d->workspace;
  s.bar = (int *)ws;
  s.err = (int *)(ws + 4096);
  s.attn_counters = (int *)(ws + 4096 + 256);
  s.amax_val = (float *)(ws + 4096 + 512);
  s.amax_idx = (int *)(ws + 4096 + 512 + 4096);
  s.attn_partial = (float *)(ws + 4096 + 512 + 8192);
  s.nsplit = nsplit;
  s.trace = d->trace;
  const int grid = state().cu_count;   // one block of 16 wavefronts per CU: every block is resident, which the barriers need
  JSG_REQUIRE(grid <= 1024, "jsgrad_hip_decode_step: %d CUs exceed the argmax partial buffer", grid);
  // Attention items (kv head, chunk) are dealt to the blocks round-robin, and the item of a head's chunk 0 waits for that
  // head's other chunks.  With at least as many blocks as a head has chunks, two waiting items can never each sit in
  // front of a chunk the other waits for (that takes a head of more chunks than there are blocks), so the waits end.
  JSG_REQUIRE(nsplit <= grid, "jsgrad_hip_decode_step: %d compute units are fewer than the %d chunks a kv head can have", grid, nsplit);
  const int n_rep = d->n_heads / d->n_kv_heads;
#define JSG_KIND(K)                                                                                  \
  case K:                                                                                            \
    return d->head_dim == 64 ? launch_step<K, 64>(s, n_rep, grid, lds) : launch_step<K, 128>(s, n_rep, grid, lds);
  switch (d->kind) {
    JSG_KIND(JSGRAD_W_F16)
    JSG_KIND(JSGRAD_W_I8)
  }
#undef JSG_KIND
  return fail("jsgrad_hip_decode_step: weight kind %d", d->kind);
}

int jsgrad_hip_step_status(const void *workspace, int *host_out_error) {
  JSG_READY();
  JSG_REQUIRE(workspace && host_out_error, "jsgrad_hip_step_status: null pointer");
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_step_status during graph capture");
  JSG_HIP(hipMemcpyAsync(host_out_error, (const char *)workspace + 4096, sizeof(int), hipMemcpyDeviceToHost, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));
  return 0;
}

}  // extern "C"
