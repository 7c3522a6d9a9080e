// Decode attention and the wo projection of one layer in ONE launch.
//
// As two launches the pair costs a chain of latencies: the attention kernel ends (its last block merges the chunks of a kv
// head), the wo kernel starts, requests its weights, stages x, and only then computes; wo of a small model is little more
// than that ramp.  Here every wavefront requests its first wo item (8 KiB of weights) before the attention items run, the
// blocks that have an attention item run it, and the merged attention row travels to all blocks as tagged words (value |
// version tag, common.h): the wo part of a block asks for the row until every word carries the tag of this launch, then
// multiplies with weights that are already in registers.
//
// Deadlock freedom.  Two kinds of block wait on the device for blocks of the same launch: blocks [0, n_kv_heads) run chunk 0
// of a kv head and then wait for that head's other chunks (attention_core.h), and the wo part of every block waits for the
// merged attention row.  Nobody waits for a block that waits: an item block publishes its partial result before it waits
// for anything.  So the launch finishes if every block that runs an item gets onto the device while the others wait
// there, i.e. if the items fit the device at once: the host asks the occupancy calculator (blocks per CU x CUs, which
// assumes this process has the device to itself) and refuses a launch with more items than that.  Every wait is bounded
// all the same, reports through the error word of the workspace, and the host raises when it reads the word.
//
// Reference: models/llama.ts:89-96 (repeat_kv + scaled_dot_product_attention + wo) and :125 (the residual add).
#include "attention_core.h"
#include "gemv_core.h"

namespace jsg {

// Two blocks of 8 wavefronts per CU: an attention item is worked on by 8 wavefronts, as in jsgrad_hip_attn_decode for
// contexts of up to 16384 positions (the two agree bit for bit), and the attention row is fetched by 512 blocks.  Measured
// against blocks of 16 wavefronts: 1B 1394 -> 1448 tok/s, 3B int8 813 -> 831, 8B int8 515 -> 524 (at 4100 positions
// 448 -> 446); blocks of 4 wavefronts are slower than both.
#ifndef JSG_AW_THREADS
#define JSG_AW_THREADS 512
#endif
constexpr int AW_THREADS = JSG_AW_THREADS;
constexpr int AW_WAVES = AW_THREADS / 64;
constexpr int AW_CHUNK_CAP = AW_WAVES * 16 < ATT_CHUNK_MAX ? AW_WAVES * 16 : ATT_CHUNK_MAX;   // attention_core.h: 16 rows per wavefront

template <int KIND, int HD, int NREP, bool SLICED>
__global__ __launch_bounds__(AW_THREADS, AW_WAVES <= 8 ? 2 * AW_WAVES / 4 : AW_WAVES / 4) void attn_wo_kernel(AttnArgs at, GemvArgs a, int layer) {   // 16 wavefronts per CU (128 registers): two blocks of eight
  typedef _Float16 AT;
  typedef Attn<AT, HD, NREP, AW_THREADS / 64, false, SLICED> A;   // SLICED: as jsgrad_hip_attn_decode picks it, so that the two agree bit for bit
  typedef Gemv<KIND, AT, EPI_STORE, 2, 4, false> G;
  extern __shared__ __align__(16) unsigned char smem[];   // the staged input row of wo
  __shared__ typename A::Smem sm;
  __shared__ float red[AW_WAVES];
  __shared__ float lut[KIND == JSGRAD_W_NF4 ? NF4_LUT_WORDS : 16];   // NF4: the code book and the table of code pairs (Gemv::fill_lut)

  // The position first, and nothing else until it is here: a small request issued into an idle memory system is back in a
  // fraction of a microsecond, behind the bursts of weight requests of all blocks it takes several times as long, and every
  // later step of the attention items hangs on it.
  JSG_LCLEAR();
  const int pos = at.st[1];
  JSG_LSTAMP(0);
  const uint32_t tag = tw_tag(pos * 128 + layer);   // the version of this launch: no other launch that writes the same tagged
  at.out_tag = tag;                                 // row has it (another layer, or another position of the same layer)
  a.x_tag = tag;

  // Blocks [0, n_kv_heads) run chunk 0 of a kv head and merge that head's chunks; they take no part in wo (the merged row is
  // what everybody else waits for, and their weights would arrive last).  The wo rows are shared by the other blocks.
  GemvBuf buf;
  const int wo_blk = (int)blockIdx.x - at.n_kv_heads, wo_nblk = (int)gridDim.x - at.n_kv_heads;
  const int grp = G::first_group(wo_blk, wo_nblk);
  const bool preloaded = wo_blk >= 0 && grp < G::ngroups(a);
  // A block either runs an attention item or, without one, asks for its first wo item right away.  The two are the
  // branches of one if / else on purpose: written as two tests in a row, the compiler's wait-count pass saw the requests of
  // the second reach the first, and made every K and V request of the item wait for the one before it.
  int T = 1, chunk = ATT_CHUNK_MIN, n_active = 0;
  if (pos >= 0 && pos < at.max_context) {
    T = pos + 1;
    chunk = att_policy_rows(T, AW_CHUNK_CAP);                        // the host sized nsplit for max_context and this cap
    n_active = att_chunk_count(T, chunk);
  } else if (blockIdx.x == 0 && threadIdx.x == 0) {
    st_coherent(a.err, 1);   // no attention row will come for such a position
  }
  const int id = blockIdx.x;
  if (id < at.n_kv_heads * n_active) {
    // This wavefront's first wo item is requested as soon as the attention item lets it (attention_core.h: loads return in
    // order and the item's barriers wait for every outstanding one, so weights requested earlier would sit in front of the
    // rows and partial results the item waits for): when the block has published its chunk, or, in the block that merges,
    // behind the merge's requests, so that the weights travel while the merge computes.
    // (kv head, chunk) of block id without an integer division: the host passes ceil(65536 / n_kv_heads)
    const int split = (int)(((uint32_t)id * (uint32_t)at.kv_magic) >> 16), g = id - split * at.n_kv_heads;
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    A::item(at, sm, g, split, T, chunk, n_active, [&]() { G::load_item(a, buf, grp, 0, 0, preloaded); });
  } else {
    // The other blocks give the items' small requests a head start before they flood the memory system with theirs; either
    // way the weights are there before the attention row is.
    __builtin_amdgcn_s_sleep(64);
    G::load_item(a, buf, grp, 0, 0, preloaded);
  }
  JSG_LSTAMP(1);
  if (wo_blk >= 0) {
    __syncthreads();   // the LDS of the attention item is done with
    G::run(a, (AT *)smem, red, lut, buf, preloaded, 0, wo_blk, wo_nblk);
    JSG_LSTAMP(21);
  }
  JSG_LFLUSH(blockIdx.x == 0 ? 0 : (blockIdx.x == (unsigned)at.n_kv_heads ? 1 : (blockIdx.x == gridDim.x - 1 ? 2 : -1)));
}
JSG_TRACE_ENTRY(jsgrad_hip_attn_wo_trace)

static int aw_nsplit(int max_context) { return att_max_chunks(max_context, AW_CHUNK_CAP); }

// Blocks of attn_wo_kernel<KIND, HD, n_rep> the device can hold at once (occupancy x CUs).  The blocks that run attention
// items are the first `items` of the grid; the rest, and the attention blocks themselves once their item is done, wait in
// the wo part for the attention row.  If more items existed than blocks fit the device, the waiting blocks could keep
// item blocks from ever starting, so such a launch is refused.
template <int KIND, int HD> static int aw_capacity(int n_rep, size_t lds, int *out) {
  int per_cu = 0;
#define JSG_REP(N)                                                                                                                      \
  case N:                                                                                                                               \
    JSG_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)attn_wo_kernel<KIND, HD, N, true>, AW_THREADS, lds));          \
    break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(3) JSG_REP(4)
    default: return fail("jsgrad_hip_attn_wo: n_heads/n_kv_heads = %d is not one of 1,2,3,4", n_rep);
  }
#undef JSG_REP
  *out = per_cu * state().cu_count;
  return 0;
}

template <int KIND, int HD> static int launch_attn_wo(const AttnArgs &at, const GemvArgs &a, int n_rep, int layer, int out_f, int *query_capacity) {
  const int ngroups = (out_f + 1) / 2, need = (ngroups + AW_WAVES - 1) / AW_WAVES + at.n_kv_heads;   // the merging blocks do no wo rows
  const int cap = state().cu_count * (16 / AW_WAVES);
  int blocks = need < cap ? need : cap;
  const int items = at.n_kv_heads * at.nsplit;
  if (blocks < items) blocks = items;
  const size_t lds = (size_t)Gemv<KIND, _Float16, EPI_STORE, 2, 4, false>::x_elems(a.in_f) * sizeof(_Float16);
  // capacity per (kernel instance, staging size): asked for once, the answer does not change
  static int cached_capacity[5] = {0, 0, 0, 0, 0};
  static size_t cached_lds[5] = {0, 0, 0, 0, 0};
  if (n_rep < 1 || n_rep > 4) return fail("jsgrad_hip_attn_wo: n_heads/n_kv_heads = %d is not one of 1,2,3,4", n_rep);
  if (cached_capacity[n_rep] == 0 || cached_lds[n_rep] != lds) {
    if (int e = aw_capacity<KIND, HD>(n_rep, lds, &cached_capacity[n_rep])) return e;
    cached_lds[n_rep] = lds;
  }
  if (query_capacity) { *query_capacity = cached_capacity[n_rep]; return 0; }
  JSG_REQUIRE(items <= cached_capacity[n_rep],
              "jsgrad_hip_attn_wo: %d attention items (%d kv heads x %d chunks of the context) but the device holds %d blocks of this kernel at once; "
              "use jsgrad_hip_attn_decode + jsgrad_hip_linear for this shape", items, at.n_kv_heads, at.nsplit, cached_capacity[n_rep]);
  const bool sliced = att_sliced_merge(at.max_context, AW_CHUNK_CAP);
#define JSG_REP(N)                                                                                                   \
  case N:                                                                                                            \
    if (sliced) JSG_LAUNCH(PROF_ATTN_WO, (attn_wo_kernel<KIND, HD, N, true>), dim3(blocks), dim3(AW_THREADS), lds, at, a, layer);   \
    else JSG_LAUNCH(PROF_ATTN_WO, (attn_wo_kernel<KIND, HD, N, false>), dim3(blocks), dim3(AW_THREADS), lds, at, a, layer);         \
    break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(3) JSG_REP(4)
  }
#undef JSG_REP
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_attn_wo_workspace_bytes(int n_heads, int n_kv_heads, int head_dim) {
  // [0, 256): chunk counters per kv head; [256, 512): error word; attention partials; the tagged attention row
  (void)n_kv_heads;
  return 512 + (size_t)n_heads * 256 * (head_dim + 2) * sizeof(float) + (size_t)n_heads * head_dim * sizeof(uint32_t);
}

int jsgrad_hip_attn_wo_items(int n_kv_heads, int max_context) { return n_kv_heads * aw_nsplit(max_context); }

static int attn_wo_impl(const void *q, const void *cache_k, const void *cache_v, const int32_t *st, void *workspace, int n_heads, int n_kv_heads,
                        int head_dim, int max_context, int kind, const void *wo, const void *so, int dim, const void *residual, void *y, int layer,
                        int *query_capacity) {
  JSG_READY();
  if (!query_capacity) JSG_REQUIRE(q && cache_k && cache_v && st && workspace && wo && y, "jsgrad_hip_attn_wo: null pointer argument");
  JSG_REQUIRE(kind == JSGRAD_W_F16 || kind == JSGRAD_W_I8 || kind == JSGRAD_W_NF4, "jsgrad_hip_attn_wo: weight kind %d (fp16, int8 and nf4 are built)", kind);
  JSG_REQUIRE(kind == JSGRAD_W_F16 || so || query_capacity, "jsgrad_hip_attn_wo: quantised weight needs a scale");
  JSG_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_kv_heads <= 64 && n_heads % n_kv_heads == 0, "jsgrad_hip_attn_wo: n_heads %d / n_kv_heads %d", n_heads, n_kv_heads);
  JSG_REQUIRE(head_dim == 64 || head_dim == 128, "jsgrad_hip_attn_wo: head_dim %d (64 and 128 are built)", head_dim);
  JSG_REQUIRE(max_context > 0 && max_context <= 64 * AW_CHUNK_CAP, "jsgrad_hip_attn_wo: max_context %d exceeds %d", max_context, 64 * AW_CHUNK_CAP);
  JSG_REQUIRE(layer >= 0 && layer < 128, "jsgrad_hip_attn_wo: layer index %d", layer);
  const int qdim = n_heads * head_dim;
  JSG_REQUIRE(dim > 0 && dim % 2 == 0 && qdim % 16 == 0 && (size_t)qdim * 2 <= 64 * 1024, "jsgrad_hip_attn_wo: dim %d / n_heads*head_dim %d", dim, qdim);
  JSG_REQUIRE(fits_buffer_offsets((size_t)dim, (size_t)qdim, 16), "jsgrad_hip_attn_wo: wo of %d x %d elements reaches 4 GiB (32-bit byte offsets)", dim, qdim);
  JSG_REQUIRE(kind != JSGRAD_W_NF4 || qdim % 64 == 0, "jsgrad_hip_attn_wo: nf4 rows of %d elements (blocks of 64)", qdim);
  char *ws = (char *)workspace;
  AttnArgs at;
  at.q = q; at.cache_k = cache_k; at.cache_v = cache_v; at.st = st; at.out = nullptr;
  at.counters = (int *)ws;
  at.partial = (float *)(ws + 512);
  at.n_kv_heads = n_kv_heads; at.nsplit = aw_nsplit(max_context); at.max_context = max_context;
  at.kv_magic = (65536 + n_kv_heads - 1) / n_kv_heads;   // exact for block ids below 65536 / n_kv_heads >= 1024 (the grid has at most two blocks per CU)
  at.scale = (float)(1.0 / sqrt((double)head_dim));
  at.out_tagged = (uint32_t *)(ws + 512 + (size_t)n_heads * 256 * (head_dim + 2) * sizeof(float));
  at.err = (int *)(ws + 256);
  GemvArgs a = {};
  a.w0 = wo; a.s0 = so; a.rows0 = dim; a.in_f = qdim; a.norm_w = nullptr; a.eps = 0.0f;
  a.inv_d = (float)(1.0 / (double)qdim); a.y = y; a.residual = residual;
  a.x_tagged = at.out_tagged;
  a.x = at.out_tagged;   // never read as the input; a readable address for the load that stands in for a missing residual
  a.err = (int *)(ws + 256);
  const int n_rep = n_heads / n_kv_heads;
#define JSG_KIND(K) \
  case K: return head_dim == 64 ? launch_attn_wo<K, 64>(at, a, n_rep, layer, dim, query_capacity) : launch_attn_wo<K, 128>(at, a, n_rep, layer, dim, query_capacity);
  switch (kind) {
    JSG_KIND(JSGRAD_W_F16)
    JSG_KIND(JSGRAD_W_I8)
    JSG_KIND(JSGRAD_W_NF4)
  }
#undef JSG_KIND
  return fail("jsgrad_hip_attn_wo: weight kind %d", kind);
}

int jsgrad_hip_attn_wo(const void *q, const void *cache_k, const void *cache_v, const int32_t *st, void *workspace, int n_heads, int n_kv_heads,
                       int head_dim, int max_context, int kind, const void *wo, const void *so, int dim, const void *residual, void *y, int layer) {
  return attn_wo_impl(q, cache_k, cache_v, st, workspace, n_heads, n_kv_heads, head_dim, max_context, kind, wo, so, dim, residual, y, layer, nullptr);
}

int jsgrad_hip_attn_wo_fits(int n_heads, int n_kv_heads, int head_dim, int max_context, int kind, int dim, int *host_out_items, int *host_out_capacity) {
  JSG_REQUIRE(host_out_items && host_out_capacity, "jsgrad_hip_attn_wo_fits: null pointer");
  int cap = 0;
  if (int e = attn_wo_impl(nullptr, nullptr, nullptr, nullptr, nullptr, n_heads, n_kv_heads, head_dim, max_context, kind, nullptr, nullptr, dim, nullptr, nullptr, 0, &cap))
    return e;
  *host_out_items = jsgrad_hip_attn_wo_items(n_kv_heads, max_context);
  *host_out_capacity = cap;
  return 0;
}

int jsgrad_hip_attn_wo_status(const void *workspace, int *host_out_error) {
  JSG_READY();
  JSG_REQUIRE(workspace && host_out_error, "jsgrad_hip_attn_wo_status: null pointer");
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_attn_wo_status during graph capture");
  JSG_HIP(hipMemcpyAsync(host_out_error, (const char *)workspace + 256, sizeof(int), hipMemcpyDeviceToHost, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));
  return 0;
}

}  // extern "C"
