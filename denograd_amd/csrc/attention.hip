// Stand-alone decode attention kernel: grid (n_kv_heads, NSPLIT), one work item per block (see attention_core.h).
// NSPLIT is fixed from max_context, so the grid does not depend on T and a captured graph replays unchanged while T grows.
#include "attention_core.h"
#include "attention_stream.h"

namespace jsg {

// One sequence (or few): an item's rows are requested up front by a block of NW wavefronts (attention_core.h), 16 rows per
// wavefront at most.  Blocks of 8 wavefronts measured faster than 16 at every context tried (8B shape at 4100 positions:
// 12.4 us against 15.8); their chunks hold 128 rows, and the merge can index 128 chunks, so contexts beyond 16384 positions
// take the 16-wavefront shape (256-row chunks, 256 chunks).  jsgrad_hip_attn_wo runs the same item with 8 wavefronts, so
// the two agree bit for bit wherever both apply.
constexpr int ATT_NW = 8, ATT_NW_LONG = 16;
constexpr int ATT_SHORT_CONTEXT = (ATT_NW * 16) * (ATT_NW * 16);
template <typename AT, int HD, int NREP, int NW, bool SLICED>
__global__ __launch_bounds__(NW * 64) void attn_decode_kernel(AttnArgs a) {
  typedef Attn<AT, HD, NREP, NW, false, SLICED> A;
  __shared__ typename A::Smem sm;
  const int g = blockIdx.x, split = blockIdx.y;
  JSG_LCLEAR();
  const int pos = a.st[1];
  JSG_LSTAMP(0);
  if (pos < 0 || pos >= a.max_context) return;
  const int T = pos + 1;
  const int chunk = att_policy_rows(T, A::CHUNK_CAP);            // the host sized nsplit for max_context and this cap
  const int n_active = att_chunk_count(T, chunk);
  if (split >= n_active) return;
  A::item(a, sm, g, split, T, chunk, n_active);
  JSG_LSTAMP(1);
  // traced builds: the block that merges kv head 0, the block of that head's chunk 1, the block of the last kv head's last chunk
  JSG_LFLUSH(g == 0 && split == 0 ? 0 : (g == 0 && split == 1 ? 1 : (g == (int)gridDim.x - 1 && split == n_active - 1 ? 2 : -1)));
}
JSG_TRACE_ENTRY(jsgrad_hip_attn_decode_trace)

// Many sequences at the same position (grid z): blocks of 4 wavefronts that stream their rows (attention_stream.h).
constexpr int ATT_STREAM_NW = 4;
template <int HD, int NREP>
__global__ __launch_bounds__(ATT_STREAM_NW * 64) void attn_decode_stream_kernel(AttnArgs a) {
  typedef AttnStream<_Float16, HD, NREP, ATT_STREAM_NW, false> A;
  __shared__ typename A::Smem sm;
  const int g = blockIdx.x, split = blockIdx.y;
  if (const int z = blockIdx.z) {   // sequence z: its own rows of q / out / cache / workspace
    a.q = (const char *)a.q + z * a.q_bstride;
    a.out = (char *)a.out + z * a.q_bstride;
    a.cache_k = (const char *)a.cache_k + z * a.cache_bstride;
    a.cache_v = (const char *)a.cache_v + z * a.cache_bstride;
    a.counters += z * a.n_kv_heads;
    a.partial += z * a.partial_bstride;
  }
  const int pos = a.st[1];
  if (pos < 0 || pos >= a.max_context) return;
  const int T = pos + 1;
  const int chunk = att_stream_chunk_rows(T, a.nsplit);  // <= ATT_CHUNK_MAX, checked on the host against max_context
  const int n_active = (T + chunk - 1) / chunk;
  if (split >= n_active) return;
  A::item(a, sm, g, split, T, chunk, n_active);
}

// splits of the streaming launch: enough that a chunk fits the LDS score buffer, no more than the merge can index there, and
// as many blocks as the device holds at once (5 per CU at this kernel's registers): the sequences fill the chip by
// themselves, every extra split only adds its fixed cost (query load, partial store, counter, merge), and a launch of one
// full round of blocks has no thinly filled second round (16 sequences x 8 kv heads at 2100 positions: 34.5 us with 5 blocks
// per CU, 35.7 us with 4 or 8, 37.8 us with 10)
static int stream_nsplit(int max_context, int heads_x_batch) {
  int by_lds = (max_context + ATT_CHUNK_MAX - 1) / ATT_CHUNK_MAX;
  int wanted = (max_context + 31) / 32;
  if (wanted > 64) wanted = 64;
  const int fill = (5 * state().cu_count + heads_x_batch - 1) / heads_x_batch;
  if (wanted > fill) wanted = fill;
  return by_lds > wanted ? by_lds : wanted;
}

template <typename AT, int HD, int NW> static int launch_attn(const AttnArgs &a, int n_rep) {
  dim3 grid(a.n_kv_heads, a.nsplit, 1), block(NW * 64);
  // the merge shared by several threads per output element for contexts that would cost the plain one three round trips
  const bool sliced = att_sliced_merge(a.max_context, NW * 16 < ATT_CHUNK_MAX ? NW * 16 : ATT_CHUNK_MAX);
#define JSG_REP(N)                                                                                   \
  case N:                                                                                            \
    if (sliced) JSG_LAUNCH(PROF_ATTN, (attn_decode_kernel<AT, HD, N, NW, true>), grid, block, 0, a);   \
    else JSG_LAUNCH(PROF_ATTN, (attn_decode_kernel<AT, HD, N, NW, false>), grid, block, 0, a);         \
    break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(3) JSG_REP(4) JSG_REP(8)
    default: return fail("jsgrad_hip_attn_decode: n_heads/n_kv_heads = %d is not one of 1,2,3,4,8", n_rep);
  }
#undef JSG_REP
  return 0;
}
template <int HD> static int launch_attn_stream(const AttnArgs &a, int n_rep, int batch) {
  dim3 grid(a.n_kv_heads, a.nsplit, batch), block(ATT_STREAM_NW * 64);
#define JSG_REP(N)                                                                                   \
  case N:                                                                                            \
    JSG_LAUNCH(PROF_ATTN, (attn_decode_stream_kernel<HD, N>), grid, block, 0, a);                      \
    break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(3) JSG_REP(4) JSG_REP(8)
    default: return fail("jsgrad_hip_attn_decode_batch: n_heads/n_kv_heads = %d is not one of 1,2,3,4,8", n_rep);
  }
#undef JSG_REP
  return 0;
}

// ---- the variant that allocates nothing: its workspace is a file-scope device array
// Each GPU the library runs on holds its own copy of the array (at its own address) until the process ends.  In host code
// the array's name is only a stand-in: the device address comes from hipGetSymbolAddress, once per device, and that
// pointer is what kernels and fills are given.
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
constexpr int NOALLOC_MAX_DEVICES = 64;
static void *g_scratch_ptr[NOALLOC_MAX_DEVICES];   // per device, set by jsgrad_hip_init there (attn_static_init)

// The device address of the built-in workspace on the current device; called by jsgrad_hip_init with that device current, so
// that no later call (one under graph capture, say) has to resolve a symbol.
int attn_static_init(int dev) {
  JSG_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES, "jsgrad_hip_init: device %d beyond the %d the built-in attention workspace is kept for", dev, NOALLOC_MAX_DEVICES);
  if (g_scratch_ptr[dev] != nullptr) return 0;
  void *p = nullptr;
  JSG_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  JSG_REQUIRE(p != nullptr, "jsgrad_hip_init: no device address for the built-in attention workspace");
  g_scratch_ptr[dev] = p;
  return 0;
}

// the partial results a call uses must start at zero (a zero word means `partial result not written yet`) whatever an
// earlier call left behind, one that gave up waiting included (a fill kernel, not a memset node: callers may be capturing a
// graph).  The first 256 bytes are not touched: the error word there stays set until it is read.
__global__ void zero_words_kernel(int *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_attn_workspace_bytes(int n_heads, int n_kv_heads, int head_dim) {
  // counters + partials for the largest split count any max_context can ask for (256)
  (void)n_kv_heads;
  return 256 + (size_t)n_heads * 256 * (head_dim + 2) * sizeof(float);
}

size_t jsgrad_hip_attn_batch_workspace_bytes(int batch, int n_heads, int n_kv_heads, int head_dim) {
  // per sequence: n_kv_heads counters, then the partials as above
  return (size_t)batch * (((size_t)n_kv_heads * sizeof(int) + 255) / 256 * 256 + (size_t)n_heads * 256 * (head_dim + 2) * sizeof(float));
}

int jsgrad_hip_attn_decode_batch(const void *q, const void *cache_k, const void *cache_v, const int32_t *st, void *out, void *workspace, int batch,
                                 int n_heads, int n_kv_heads, int head_dim, int max_context) {
  JSG_READY();
  JSG_REQUIRE(q && cache_k && cache_v && st && out && workspace, "jsgrad_hip_attn_decode_batch: null pointer argument");
  JSG_REQUIRE(batch > 0 && batch <= 65535, "jsgrad_hip_attn_decode_batch: batch %d", batch);
  JSG_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_kv_heads <= 64 && n_heads % n_kv_heads == 0, "jsgrad_hip_attn_decode_batch: n_heads %d / n_kv_heads %d", n_heads, n_kv_heads);
  JSG_REQUIRE(head_dim == 64 || head_dim == 128, "jsgrad_hip_attn_decode_batch: head_dim %d (64 and 128 are built)", head_dim);
  JSG_REQUIRE(max_context > 0 && max_context <= 256 * ATT_CHUNK_MAX, "jsgrad_hip_attn_decode_batch: max_context %d exceeds %d", max_context, 256 * ATT_CHUNK_MAX);
  const size_t counter_bytes = ((size_t)n_kv_heads * sizeof(int) + 255) / 256 * 256;
  AttnArgs a;
  a.q = q; a.cache_k = cache_k; a.cache_v = cache_v; a.st = st; a.out = out;
  a.counters = (int *)workspace;                                   // [batch][n_kv_heads], densely packed
  a.partial = (float *)((char *)workspace + (size_t)batch * counter_bytes);
  a.n_kv_heads = n_kv_heads; a.nsplit = stream_nsplit(max_context, n_kv_heads * batch); a.max_context = max_context;
  a.scale = (float)(1.0 / sqrt((double)head_dim));
  a.q_bstride = (size_t)n_heads * head_dim * sizeof(_Float16);
  a.cache_bstride = (size_t)max_context * n_kv_heads * head_dim * sizeof(_Float16);
  a.partial_bstride = (size_t)n_heads * 256 * (head_dim + 2);
  const int n_rep = n_heads / n_kv_heads;
  return head_dim == 64 ? launch_attn_stream<64>(a, n_rep, batch) : launch_attn_stream<128>(a, n_rep, batch);
}

size_t jsgrad_hip_attn_decode_static_max_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

static int attn_decode_check(const char *who, int n_heads, int n_kv_heads, int head_dim, int max_context, int act) {
  JSG_REQUIRE(act == JSGRAD_F16 || act == JSGRAD_F32, "%s: unknown activation dtype %d", who, act);
  JSG_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_kv_heads <= 64 && n_heads % n_kv_heads == 0, "%s: n_heads %d / n_kv_heads %d", who, n_heads, n_kv_heads);
  JSG_REQUIRE(head_dim == 64 || head_dim == 128, "%s: head_dim %d (64 and 128 are built)", who, head_dim);
  JSG_REQUIRE(max_context > 0 && max_context <= 256 * ATT_CHUNK_MAX, "%s: max_context %d exceeds %d", who, max_context, 256 * ATT_CHUNK_MAX);
  const int n_rep = n_heads / n_kv_heads;
  JSG_REQUIRE(n_rep <= 4 || n_rep == 8, "%s: n_heads/n_kv_heads = %d is not one of 1,2,3,4,8", who, n_rep);
  // The blocks of chunk 0 (the first n_kv_heads of the grid) wait on the device for the other chunks' partial results.
  // Those other blocks wait for nobody, so the launch finishes as long as the waiting blocks leave room on the device for
  // at least one of them; the device is required to have more compute units than there are waiting blocks.
  JSG_REQUIRE(n_kv_heads < state().cu_count, "%s: %d kv heads but only %d compute units", who, n_kv_heads, state().cu_count);
  return 0;
}

static int read_error_word(const char *who, void *word, int *host_out_error) {
  JSG_READY();
  JSG_REQUIRE(word && host_out_error, "%s: null pointer", who);
  JSG_REQUIRE(!state().capturing, "%s during graph capture", who);
  JSG_HIP(hipMemcpyAsync(host_out_error, word, sizeof(int), hipMemcpyDeviceToHost, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));
  return 0;
}

int jsgrad_hip_attn_decode_status(void *workspace, int n_heads, int n_kv_heads, int head_dim, int *host_out_error) {
  if (int e = read_error_word("jsgrad_hip_attn_decode_status", workspace, host_out_error)) return e;
  if (*host_out_error != 0) {
    // the merging block had cleared the words it saw and the late chunks stored afterwards: the workspace is not zero any
    // more.  Clear all of it (the error word included), so that it can be used again.
    JSG_REQUIRE(n_heads > 0 && n_kv_heads > 0 && head_dim > 0, "jsgrad_hip_attn_decode_status: n_heads %d / n_kv_heads %d / head_dim %d", n_heads, n_kv_heads, head_dim);
    JSG_HIP(hipMemsetAsync(workspace, 0, jsgrad_hip_attn_workspace_bytes(n_heads, n_kv_heads, head_dim), state().stream));
    JSG_HIP(hipStreamSynchronize(state().stream));
    *host_out_error = 1;
  }
  return 0;
}

int jsgrad_hip_attn_decode_static_status(int *host_out_error) {
  JSG_READY();
  const int dev = state().device;
  JSG_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES && g_scratch_ptr[dev] != nullptr, "jsgrad_hip_attn_decode_static_status: no built-in workspace on device %d", dev);
  if (int e = read_error_word("jsgrad_hip_attn_decode_static_status", g_scratch_ptr[dev], host_out_error)) return e;
  if (*host_out_error != 0) {      // the partial results are cleared by every call; only the error word is sticky
    JSG_HIP(hipMemsetAsync(g_scratch_ptr[dev], 0, 256, state().stream));
    JSG_HIP(hipStreamSynchronize(state().stream));
    *host_out_error = 1;
  }
  return 0;
}

int jsgrad_hip_attn_decode_static(const void *q, const void *cache_k, const void *cache_v, const int32_t *st, void *out, int n_heads, int n_kv_heads,
                                  int head_dim, int max_context, int act) {
  JSG_READY();
  JSG_REQUIRE(q && cache_k && cache_v && st && out, "jsgrad_hip_attn_decode_static: null pointer argument");
  if (int e = attn_decode_check("jsgrad_hip_attn_decode_static", n_heads, n_kv_heads, head_dim, max_context, act)) return e;
  // 256 bytes of header (the error word), then one partial result per (head, chunk): only the chunks this max_context can
  // produce are needed
  const int cap = max_context <= ATT_SHORT_CONTEXT ? ATT_NW * 16 : ATT_CHUNK_MAX;
  const size_t need = 256 + (size_t)n_heads * att_max_chunks(max_context, cap) * ((size_t)head_dim + 2) * sizeof(float);
  JSG_REQUIRE(need <= NOALLOC_SCRATCH_BYTES,
              "jsgrad_hip_attn_decode_static: %d heads of %d at max_context %d need %zu bytes of workspace, the built-in one holds %zu; use jsgrad_hip_attn_decode "
              "with a workspace of its own", n_heads, head_dim, max_context, need, (size_t)NOALLOC_SCRATCH_BYTES);
  const int dev = state().device;
  JSG_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES && g_scratch_ptr[dev] != nullptr, "jsgrad_hip_attn_decode_static: no built-in workspace on device %d", dev);
  void *ws = g_scratch_ptr[dev];
  const int words = (int)((need - 256 + 3) / 4);
  hipLaunchKernelGGL(zero_words_kernel, dim3((words + 255) / 256), dim3(256), 0, state().stream, (int *)((char *)ws + 256), words);
  JSG_LAUNCHED();
  return jsgrad_hip_attn_decode(q, cache_k, cache_v, st, out, ws, n_heads, n_kv_heads, head_dim, max_context, act);
}

int jsgrad_hip_attn_decode(const void *q, const void *cache_k, const void *cache_v, const int32_t *st, void *out, void *workspace, int n_heads,
                           int n_kv_heads, int head_dim, int max_context, int act) {
  JSG_READY();
  JSG_REQUIRE(q && cache_k && cache_v && st && out && workspace, "jsgrad_hip_attn_decode: null pointer argument");
  if (int e = attn_decode_check("jsgrad_hip_attn_decode", n_heads, n_kv_heads, head_dim, max_context, act)) return e;
  AttnArgs a;
  a.q = q; a.cache_k = cache_k; a.cache_v = cache_v; a.st = st; a.out = out;
  a.counters = nullptr;              // this kernel's partial results say by themselves whether they are there
  a.err = (int *)workspace;          // set when the merging block's bounded wait runs out (jsgrad_hip_attn_decode_status)
  a.partial = (float *)((char *)workspace + 256);
  const bool short_ctx = max_context <= ATT_SHORT_CONTEXT;
  a.n_kv_heads = n_kv_heads; a.nsplit = att_max_chunks(max_context, short_ctx ? ATT_NW * 16 : ATT_CHUNK_MAX); a.max_context = max_context;
  a.scale = (float)(1.0 / sqrt((double)head_dim));
  const int n_rep = n_heads / n_kv_heads;
  if (short_ctx) {
    if (act == JSGRAD_F16) return head_dim == 64 ? launch_attn<_Float16, 64, ATT_NW>(a, n_rep) : launch_attn<_Float16, 128, ATT_NW>(a, n_rep);
    return head_dim == 64 ? launch_attn<float, 64, ATT_NW>(a, n_rep) : launch_attn<float, 128, ATT_NW>(a, n_rep);
  }
  if (act == JSGRAD_F16) return head_dim == 64 ? launch_attn<_Float16, 64, ATT_NW_LONG>(a, n_rep) : launch_attn<_Float16, 128, ATT_NW_LONG>(a, n_rep);
  return head_dim == 64 ? launch_attn<float, 64, ATT_NW_LONG>(a, n_rep) : launch_attn<float, 128, ATT_NW_LONG>(a, n_rep);
}

}  // extern "C"
