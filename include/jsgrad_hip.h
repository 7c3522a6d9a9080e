/*
 * jsgrad_hip.h -- C ABI of libjsgrad_hip.so, the MI355X (gfx950) backend for jsgrad's
 * Llama-3 inference path.
 *
 * Plain C: `int` status returns (0 = ok, non-zero = error; text via jsgrad_hip_last_error),
 * no C++ types and no exceptions across the boundary.  Every pointer is a DEVICE pointer
 * unless its name starts with `host_`.  All work is queued on one library-owned HIP stream
 * (default priority); calls are asynchronous unless stated otherwise.  The caller is a
 * single thread (a JS event loop through Deno.dlopen, or Python ctypes); the library takes
 * no locks.
 *
 * Each entry point cites the reference interface it stands behind
 * (/root/reference/<file>:<line>).
 */
#ifndef JSGRAD_HIP_H
#define JSGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype of activations / tables: jsgrad dtypes.float32 and dtypes.float16 (jsgrad/dtype.ts) */
enum { JSGRAD_F32 = 0, JSGRAD_F16 = 1 };
/* storage of a Linear weight: nn.Linear float32 / float16 (jsgrad/nn/index.ts:403-412),
 * Int8Linear int8 + per-output-row fp16 scale (jsgrad/models/llama3.ts:27-36),
 * NF4Linear(64) two 4-bit codes per byte + one fp16 scale per 64 elements (llama3.ts:79-97) */
enum { JSGRAD_W_F32 = 0, JSGRAD_W_F16 = 1, JSGRAD_W_I8 = 2, JSGRAD_W_NF4 = 3 };

/* ---------------------------------------------------------------------------------
 * Device, memory, programs: what a `Compiled` device needs (jsgrad/runtime/allocator.ts:166-191)
 * --------------------------------------------------------------------------------- */

/* Compiled.init (allocator.ts:179; awaited lazily from engine/realize.ts:133,157): select the
 * device, create the stream.  Idempotent. */
int jsgrad_hip_init(int device);
/* Text of the last error on this thread's library state; never NULL. */
const char *jsgrad_hip_last_error(void);
/* Device name and gcnArchName ("gfx950...") for the `Device` registry entry (jsgrad/device.ts:26-35). */
int jsgrad_hip_device_name(char *host_out, size_t cap);
/* Number of compute units (used to size grids host-side). */
int jsgrad_hip_cu_count(int *host_out);

/* Allocator._alloc / _free (allocator.ts:40-41) with LRUAllocator's reuse behind them (allocator.ts:53-77).  size 0 is an
 * error as in Allocator.alloc (:30-33).  A request is rounded up to a size class; a freed block waits for the next
 * request of its class and changes hands without a wait (one in-order stream serves every launch and copy).  free may
 * be called at any time (Buffer finalisers, jsgrad/device.ts:72-74) and never waits for the stream; memory returns to
 * the driver at the next jsgrad_hip_sync once more than JSGRAD_HIP_CACHE_MB (default: an eighth of the device) lies
 * idle, when hipMalloc runs out, or through jsgrad_hip_free_cache.  LRU=0 in the environment turns reuse off
 * (allocator.ts:73): free then waits for the stream and calls hipFree.  A pointer that jsgrad_hip_malloc did not hand
 * out, or a second free of one that it did, is an error. */
int jsgrad_hip_malloc(size_t nbytes, void **host_out_ptr);
int jsgrad_hip_free(void *ptr);
/* LRUAllocator.free_cache (allocator.ts:65-70): wait for the stream and give every idle block back to the driver. */
int jsgrad_hip_free_cache(void);
/* Bytes handed out and bytes lying idle, in size classes (the library's view of GlobalCounters.mem_used, device.ts:128,135). */
int jsgrad_hip_mem_info(size_t *host_out_live_bytes, size_t *host_out_idle_bytes);
/* Allocator._copyin / _copyout (allocator.ts:42-43).  copyout returns after the data is in host memory. */
int jsgrad_hip_copyin(void *dst, const void *host_src, size_t nbytes);
int jsgrad_hip_copyout(void *host_dst, const void *src, size_t nbytes);
/* BufferCopy between two device buffers (engine/realize.ts:92-122, Allocator._transfer allocator.ts:46). */
int jsgrad_hip_copy(void *dst, const void *src, size_t nbytes);
/* Tensor.zeros(...).contiguous().realize() for the KV cache (models/llama.ts:79): byte fill. */
int jsgrad_hip_memset(void *dst, int byte, size_t nbytes);
/* Compiled.synchronize (allocator.ts:185-186). */
int jsgrad_hip_sync(void);

/* Program.init(name, lib) (allocator.ts:101-103; ops_clang.ts:30-38 is the CPU counterpart): load a
 * gfx950 code object and look a kernel up by name. */
int jsgrad_hip_module_load(const void *host_image, size_t nbytes, void **host_out_module);
int jsgrad_hip_module_unload(void *module);
int jsgrad_hip_module_get(void *module, const char *name, void **host_out_function);
/* Program.call(bufs, {global_size, local_size, vals}, wait) (allocator.ts:104-106, called from
 * engine/realize.ts:62-80): grid is in BLOCKS, `vals` are int32 kernel arguments appended after the
 * buffer pointers (ops_clang.ts:46).  With wait != 0 the call blocks and *host_seconds gets the
 * kernel time measured with HIP events on the library stream. */
int jsgrad_hip_launch(void *function, const uint32_t host_grid[3], const uint32_t host_block[3], void *const *host_bufs, int nbufs,
                      const int32_t *host_vals, int nvals, int wait, double *host_seconds);

/* Timing on the library stream (the `wait` contract of Program.call and DEBUG>=2 per-kernel
 * statistics, engine/realize.ts:168-178). */
int jsgrad_hip_event_create(void **host_out_event);
int jsgrad_hip_event_record(void *event);
int jsgrad_hip_event_elapsed_ms(void *start, void *stop, float *host_out_ms); /* waits for `stop` */
int jsgrad_hip_event_destroy(void *event);

/* Per-kernel statistics (DEBUG>=2 of engine/realize.ts:168-178; ProfileRangeEvent, runtime/allocator.ts:147-151):
 * while enabled, every Llama kernel launched outside a graph capture is bracketed by an event pair.  `read` waits
 * for the stream and returns launch count and summed milliseconds of one kind since profiling was enabled. */
enum { JSGRAD_PROF_EMBED = 0, JSGRAD_PROF_RMSNORM, JSGRAD_PROF_LINEAR, JSGRAD_PROF_QKV_ROPE, JSGRAD_PROF_ATTN, JSGRAD_PROF_FFN_GATE, JSGRAD_PROF_ARGMAX, JSGRAD_PROF_STEP, JSGRAD_PROF_GEMM, JSGRAD_PROF_ATTN_PREFILL, JSGRAD_PROF_ATTN_WO, JSGRAD_PROF_READ, JSGRAD_PROF_SAMPLE };
int jsgrad_hip_profile(int enable);
int jsgrad_hip_profile_read(int kind, int *host_out_count, double *host_out_total_ms);

/* A measuring stick, with no counterpart in the reference: one launch that reads nbytes (a multiple of 16) of device memory
 * at src through registers and keeps nothing (two blocks per CU, eight 16-byte streaming loads in flight per thread).  Its
 * duration (kind JSGRAD_PROF_READ of the statistics above) is what a launch that only had to read that many bytes takes
 * on this device: the ceiling for a one-launch linear layer of that size.  sink: 4 writable bytes of device memory. */
int jsgrad_hip_read_probe(const void *src, size_t nbytes, void *sink);

/* TinyJit capture / replay as a device graph (engine/jit.ts:14-69 apply_graph_to_jit, :71 GraphRunner,
 * `Compiled.graph` allocator.ts:176): everything queued between begin and end becomes one HIP graph. */
int jsgrad_hip_graph_begin(void);
int jsgrad_hip_graph_end(void **host_out_graph);
int jsgrad_hip_graph_launch(void *graph);
int jsgrad_hip_graph_destroy(void *graph);

/* ---------------------------------------------------------------------------------
 * Llama-3 decode kernels (one sequence, one new position).
 *
 * `state` is a device int32[2] = { token, start_pos } that the kernels read, so that a captured
 * graph replays unchanged while start_pos advances (the role of the bound `start_pos` Variable,
 * models/llama.ts:217).  Activations, norm weights, the RoPE table and the KV cache are in the
 * activation dtype `act` (JSGRAD_F32 / JSGRAD_F16).
 * --------------------------------------------------------------------------------- */

/* precompute_freqs_cis(dim=head_dim, end, theta) (models/llama.ts:10-14) followed by the cast to the
 * activation dtype (llama.ts:205): table [end][head_dim/2][2] = (cos, sin). */
int jsgrad_hip_rope_table(void *table, int head_dim, int end, float theta, int act);

/* Embedding.call (nn/index.ts:607-619) / Int8Embedding.call (llama3.ts:71-77) for the token in
 * state[0]: out[dim] = row of the table (int8: RN16(code * scale[row])).  kind: F32 / F16 / I8. */
int jsgrad_hip_embed(int kind, const void *table, const void *scale, const int32_t *state, void *out, int dim, int vocab, int act);

/* RMSNorm.call (nn/index.ts:586-588) on one row. */
int jsgrad_hip_rmsnorm(const void *x, const void *weight, void *y, int dim, float eps, int act);

/* Linear.call / Int8Linear.call / NF4Linear.call on one row (nn/index.ts:411, llama3.ts:35,91-97):
 * y[out_f] = x[in_f] . W^T, float accumulation, result in the activation dtype.
 * norm_weight != NULL fuses RMSNorm(x) in front (TransformerBlock.call, models/llama.ts:125-126);
 * residual != NULL adds it after the cast: y = residual + linear (the `x.add(...)` of llama.ts:125-126).
 * The one-row launches (this one, _qkv_rope, _ffn_gate, _attn_wo, _decode_step) address a weight matrix with 32-bit byte
 * offsets: a matrix of 4 GiB or more is refused. */
int jsgrad_hip_linear(int kind, const void *w, const void *scale, int out_f, int in_f, const void *x, void *y,
                      const void *norm_weight, float eps, const void *residual, int act);

/* attention_norm + wq/wk/wv + apply_rotary_emb + KV-cache assign (models/llama.ts:61-87) for the
 * position state[1]: q_out[n_heads*head_dim] gets the rotated query; the rotated key and the value are
 * written into row state[1] of cache_k / cache_v ([max_context][n_kv_heads][head_dim], one layer). */
int jsgrad_hip_qkv_rope(int kind, const void *wq, const void *sq, const void *wk, const void *sk, const void *wv, const void *sv,
                        const void *x, const void *norm_weight, float eps, const void *rope_table, const int32_t *state,
                        void *q_out, void *cache_k, void *cache_v, int dim, int n_heads, int n_kv_heads, int head_dim, int max_context, int act);

/* repeat_kv + scaled_dot_product_attention over cache rows [0, state[1]] (models/llama.ts:89-95,
 * tensor.ts:3920-3934), grouped-query: query head h reads kv head h / (n_heads/n_kv_heads).
 * workspace: jsgrad_hip_attn_workspace_bytes() bytes, zero-filled once before first use: a zero word means `partial result not
 * written yet`, and every launch leaves the workspace zero again.  Inside the launch the block of a kv head's first chunk waits
 * for the other chunks' results; the wait is bounded, and if it ever runs out (the blocks of the launch were kept off the
 * device, by another process for instance) the output row is NaN, the first word of the workspace is set, and the workspace
 * is NOT zero any more: results of later launches on it are invalid until jsgrad_hip_attn_decode_status has been called, which
 * reports the word (*host_out_error = 1) and, when it was set, clears the whole workspace for further use.  _status waits
 * for the stream; callers check it where they wait for the device anyway. */
size_t jsgrad_hip_attn_workspace_bytes(int n_heads, int n_kv_heads, int head_dim);
int jsgrad_hip_attn_decode(const void *q, const void *cache_k, const void *cache_v, const int32_t *state, void *out, void *workspace,
                           int n_heads, int n_kv_heads, int head_dim, int max_context, int act);
int jsgrad_hip_attn_decode_status(void *workspace, int n_heads, int n_kv_heads, int head_dim, int *host_out_error);

/* jsgrad_hip_attn_decode without the workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The partial
 * results live in an array built into the library: jsgrad_hip_attn_decode_static_max_bytes() bytes
 * (8 MiB) on every GPU the library runs on, held until the process ends.  The call allocates and frees nothing; shapes whose
 * workspace (256 + n_heads * chunks(max_context) * (head_dim + 2) * 4 bytes, chunks <= 256) does not fit are refused with an
 * error.  All calls on one GPU share the array: they are ordered by the library's stream; calls that overlap on one GPU
 * (other streams, other threads) race.  Same results as jsgrad_hip_attn_decode, bit for bit.  The array's device address is
 * resolved by jsgrad_hip_init, so the call itself only launches kernels (a fill of the partial results it will use, then
 * the attention) and may be captured into a graph.  jsgrad_hip_attn_decode_static_status reports, and clears, the error word
 * of a bounded wait that ran out (see jsgrad_hip_attn_decode); the partial results are cleared by every call anyway. */
size_t jsgrad_hip_attn_decode_static_max_bytes(void);
int jsgrad_hip_attn_decode_static(const void *q, const void *cache_k, const void *cache_v, const int32_t *state, void *out,
                                  int n_heads, int n_kv_heads, int head_dim, int max_context, int act);
int jsgrad_hip_attn_decode_static_status(int *host_out_error);

/* ffn_norm + w1, w3 + SwiGLU (FeedForward.call, models/llama.ts:108-110): g[hidden] = silu(w1 x) * (w3 x). */
int jsgrad_hip_ffn_gate(int kind, const void *w1, const void *s1, const void *w3, const void *s3, const void *x,
                        const void *norm_weight, float eps, void *g, int dim, int hidden, int act);

/* sample() at temperature 0 (models/llama.ts:137 -> Tensor.argmax tensor.ts:2314-2320): lowest index among
 * the maxima of logits[n] (activation dtype).  Writes the token to state[0] and, when advance != 0,
 * increments state[1]; tokens_out != NULL (an int32[tokens_cap] history) also receives the token at
 * tokens_out[old start_pos] when that index is inside it. */
int jsgrad_hip_argmax(const void *logits, int n, int32_t *state, int32_t *tokens_out, int tokens_cap, int advance, int act);

/* ---------------------------------------------------------------------------------
 * Several rows at once: batched prefill (S > 1 new positions) and batched decode (B > 1 sequences).
 *
 * Transformer.forward with tokens of shape [B, S] (models/llama.ts:201-213): the rows are the B*S positions, row
 * m = b*S + s sits at position start_pos + s of sequence b.  fp16 activations; fp16, int8 or NF4 weights.  With more
 * than one row the reference expands the weight over the rows, which realises a quantised weight in fp16 first
 * (W = RN16(code * scale)); the kernels below reproduce that.  Linear layers run on the matrix cores (MFMA) with
 * float accumulation.  Output widths must be multiples of 128, in_features multiples of 64; weights, activations,
 * outputs, the rope table and the caches 16-byte aligned.
 * The KV cache of a layer is [B][max_context][n_kv_heads][head_dim] (models/llama.ts:78-80).
 * --------------------------------------------------------------------------------- */

/* Embedding.call / Int8Embedding.call (nn/index.ts:607-619, llama3.ts:71-77) for `rows` device token ids. */
int jsgrad_hip_embed_rows(int kind, const void *table, const void *scale, const int32_t *tokens, int rows, void *out, int dim, int vocab);

/* RMSNorm.call (nn/index.ts:586-588) on every row of x[rows][dim]. */
int jsgrad_hip_rmsnorm_rows(const void *x, const void *weight, void *y, int rows, int dim, float eps);

/* Linear.call / Int8Linear.call / NF4Linear.call (nn/index.ts:411, llama3.ts:35,91-97) on x[rows][in_f]:
 * y[rows][out_f] = x . W^T (+ residual[rows][out_f] added after the cast, models/llama.ts:125-126). */
int jsgrad_hip_gemm(int kind, const void *w, const void *scale, int out_f, int in_f, const void *x, int rows, void *y, const void *residual);

/* wq/wk/wv + apply_rotary_emb + KV-cache assign (models/llama.ts:61-87) for rows = B * seq_len positions starting
 * at start_pos: q_out[rows][n_heads*head_dim] gets the rotated queries, cache rows [start_pos, start_pos+seq_len) of
 * every sequence get the rotated keys and the values.  x is the already normed input. */
int jsgrad_hip_gemm_qkv_rope(int kind, const void *wq, const void *sq, const void *wk, const void *sk, const void *wv, const void *sv, const void *x,
                             int rows, int seq_len, int start_pos, const void *rope_table, void *q_out, void *cache_k, void *cache_v, int dim,
                             int n_heads, int n_kv_heads, int head_dim, int max_context);

/* w1, w3 + SwiGLU (FeedForward.call, models/llama.ts:108-110) on the already normed x[rows][dim]:
 * g[rows][hidden] = silu(w1 x) * (w3 x). */
int jsgrad_hip_gemm_ffn_gate(int kind, const void *w1, const void *s1, const void *w3, const void *s3, const void *x, int rows, void *g, int dim,
                             int hidden);

/* repeat_kv + scaled_dot_product_attention with the causal mask triu(start_pos + 1) (models/llama.ts:89-95,208;
 * tensor.ts:3920-3934): query row s of sequence b sees cache rows [0, start_pos + s].  q / out: [B*seq_len][n_heads*head_dim]. */
int jsgrad_hip_attn_prefill(const void *q, const void *cache_k, const void *cache_v, void *out, int batch, int seq_len, int start_pos, int n_heads,
                            int n_kv_heads, int head_dim, int max_context);

/* jsgrad_hip_attn_decode for B sequences that sit at the same position state[1]: q / out are [B][n_heads*head_dim].
 * workspace: jsgrad_hip_attn_batch_workspace_bytes() bytes, zero-filled once before first use. */
size_t jsgrad_hip_attn_batch_workspace_bytes(int batch, int n_heads, int n_kv_heads, int head_dim);
int jsgrad_hip_attn_decode_batch(const void *q, const void *cache_k, const void *cache_v, const int32_t *state, void *out, void *workspace, int batch,
                                 int n_heads, int n_kv_heads, int head_dim, int max_context);

/* Tensor.argmax (tensor.ts:2314-2320) of every row of logits[rows][n]: tokens_out[rows]. */
int jsgrad_hip_argmax_rows(const void *logits, int rows, int n, int32_t *tokens_out);

/* ---------------------------------------------------------------------------------
 * The whole decode step as ONE kernel.
 *
 * What TinyJit + a device graph do in the reference - replay every kernel of Transformer.forward for one token as a
 * single device-side program (engine/jit.ts:71 GraphRunner, :190-217 CapturedJit.call, models/llama.ts:201-220) - done
 * here by a persistent kernel: one resident block per CU walks embedding, the five phases of every TransformerBlock,
 * final norm + lm_head and the greedy argmax, with grid barriers in between and the next phase's weights already in
 * flight.  Same arithmetic and results as the per-kernel entry points above.  fp16 activations; fp16 or int8 layers with
 * an lm_head stored the same way.
 * --------------------------------------------------------------------------------- */

/* tensors of one TransformerBlock (models/llama.ts:112-128); scales are NULL for fp16 weights */
typedef struct {
  const void *wq, *wk, *wv, *wo, *w1, *w2, *w3;
  const void *sq, *sk, *sv, *so, *s1, *s2, *s3;
  const void *attention_norm, *ffn_norm;
  void *cache_k, *cache_v; /* [max_context][n_kv_heads][head_dim] each */
} jsgrad_hip_layer_t;

/* host-side descriptor; `layers` is a DEVICE array of n_layers jsgrad_hip_layer_t */
typedef struct {
  const jsgrad_hip_layer_t *layers;
  int n_layers, dim, hidden, n_heads, n_kv_heads, head_dim, vocab, max_context;
  float eps;
  int kind, out_kind, embed_kind, act; /* JSGRAD_W_* of the layers / lm_head / embedding table, JSGRAD_F16 */
  const void *tok_emb, *tok_scale, *out_w, *out_s, *final_norm, *rope_table;
  int32_t *state;      /* device {token, start_pos}: read at the start, advanced at the end */
  int32_t *tokens_out; /* optional int32[tokens_cap] history, receives the token at [start_pos] */
  int tokens_cap;
  void *h, *h2, *q, *attn, *g, *logits; /* activation rows: dim, dim, n_heads*head_dim, n_heads*head_dim, hidden, vocab */
  void *workspace;     /* jsgrad_hip_step_workspace_bytes(), zero-filled once before first use */
  long long *trace;    /* optional device int64[2048]: block 0 stamps the 100 MHz device clock at every phase boundary */
} jsgrad_hip_step_t;

size_t jsgrad_hip_step_workspace_bytes(int n_heads, int n_kv_heads, int head_dim);
int jsgrad_hip_decode_step(const jsgrad_hip_step_t *host_desc);
/* Every wait inside the step kernel is bounded; *host_out_error becomes 1 if one ever ran out (the blocks were not all
 * resident, e.g. another process held CUs) - the tokens of that step are then not to be trusted.  Waits for the stream. */
int jsgrad_hip_step_status(const void *workspace, int *host_out_error);

/* The same step (same descriptor, same results) with role-specialised wavefronts instead of phase-by-phase blocks: in
 * every resident block seven wavefronts only stream weights through all phases of the step, each with four register
 * buffers, so the loads of the next phase are in flight while the current one is handed over; the eighth wavefront owns
 * the hand-offs (input row -> LDS with the RMSNorm, row epilogues, block flags) and the attention items.  fp16
 * activations with fp16 or int8 weights (lm_head in the same format).  Stands for the same reference interfaces as
 * jsgrad_hip_decode_step (engine/jit.ts:71,190-217; models/llama.ts:201-220).  The workspace has its own layout:
 * jsgrad_hip_stream_workspace_bytes() bytes, zero-filled once before first use.  head_dim 64 or 128, 1, 2 or 4 query
 * heads per kv head, dim <= 4096, max_context <= 8192. */
size_t jsgrad_hip_stream_workspace_bytes(int n_heads, int n_kv_heads, int head_dim);
int jsgrad_hip_stream_step(const jsgrad_hip_step_t *host_desc);
int jsgrad_hip_stream_status(const void *workspace, int *host_out_error);

/* jsgrad_hip_attn_decode followed by jsgrad_hip_linear(wo, residual) of one layer as ONE launch (models/llama.ts:89-96 and the
 * residual add of :125): y[dim] = residual + wo . attention(q, cache).  The first wo weights of every wavefront are requested
 * before the attention items run, and the attention row reaches the wo part inside the launch.  fp16 activations; fp16, int8
 * or nf4 wo.  layer: index of the layer in the model (0..127; launches that share a workspace must differ in layer or position, so
 * a model needs at least two layers).  workspace: jsgrad_hip_attn_wo_workspace_bytes() bytes, zero-filled once before first
 * use, one per model.  The wait inside the launch is bounded; jsgrad_hip_attn_wo_status reads whether one ever ran out. */
size_t jsgrad_hip_attn_wo_workspace_bytes(int n_heads, int n_kv_heads, int head_dim);
int jsgrad_hip_attn_wo(const void *q, const void *cache_k, const void *cache_v, const int32_t *state, void *workspace, int n_heads, int n_kv_heads,
                       int head_dim, int max_context, int kind, const void *wo, const void *wo_scale, int dim, const void *residual, void *y, int layer);
int jsgrad_hip_attn_wo_status(const void *workspace, int *host_out_error);
/* Launch geometry of jsgrad_hip_attn_wo.  _items: blocks that run an attention item (kv heads x chunks of max_context; plain
 * arithmetic, needs no device).  _fits: that number and the number of blocks of the kernel the device holds at once; a launch
 * with more items than that is refused by jsgrad_hip_attn_wo (blocks that are done wait on the device for the attention row,
 * so every item block must be resident), and the caller runs jsgrad_hip_attn_decode + jsgrad_hip_linear instead. */
int jsgrad_hip_attn_wo_items(int n_kv_heads, int max_context);
int jsgrad_hip_attn_wo_fits(int n_heads, int n_kv_heads, int head_dim, int max_context, int kind, int dim, int *host_out_items, int *host_out_capacity);

/* ---------------------------------------------------------------------------------
 * Load-time kernels
 * --------------------------------------------------------------------------------- */

/* Int8Linear.quantize for one [out_f][in_f] matrix given in the activation dtype (llama3.ts:37-60). */
int jsgrad_hip_int8_quantize(const void *w, int out_f, int in_f, int8_t *codes, void *scale_f16, int act);
/* weight.cast(half) * scale materialised (llama3.ts:35,75): w16[out_f][in_f] = RN16(code * scale[row]). */
int jsgrad_hip_int8_dequant(const int8_t *codes, const void *scale_f16, int out_f, int in_f, void *w16);
/* NF4Linear(64).quantize / the dequantisation of NF4Linear.call for n elements (llama3.ts:91-96,98-114). */
int jsgrad_hip_nf4_quantize(const void *w, size_t n, uint8_t *packed, void *scale_f16, int act);
int jsgrad_hip_nf4_dequant(const uint8_t *packed, const void *scale_f16, size_t n, void *w16);
/* `sample` (models/llama.ts:131-185) on the logits of one position: alpha penalties with their counter, NaN -> -inf,
 * softmax(logits / temp), then Tensor.multinomial (tensor.ts:1164-1172) over the whole vocabulary (k == 0) or over the k
 * largest after the top-p mask; temp < 1e-6 is the greedy jsgrad_hip_argmax.  The uniform number is the float32 that
 * Tensor.rand([1,1,1]) draws (tensor.ts:798-843): Threefry-2x32-20 under the key rng[0] (sha256 of the device count, see
 * Tensor._device_seeds), rng[1] (the seed of Tensor.manual_seed) at the counter rng[2], which the call advances by one.
 * The token goes to state[0] (and tokens_out[state[1]]), state[1] advances when `advance` is set, alpha_counter[token]
 * grows by one when af or ap is set (may be NULL otherwise).  Everything is device memory and the call only queues
 * kernels, so it can sit inside a captured graph.  workspace: jsgrad_hip_sample_workspace_bytes(n) bytes, zero-filled once
 * before first use.  n: more than 512 and at most 1048576 logits; k <= 256. */
size_t jsgrad_hip_sample_workspace_bytes(int n);
int jsgrad_hip_sample(const void *logits, int n, int act, double temp, int k, double p, double af, double ap, int32_t *alpha_counter, uint32_t *rng,
                      int32_t *state, int32_t *tokens_out, int tokens_cap, int advance, void *workspace);

/* Checkpoint formats on the way into the model.
 * ggml_dequant: ggml_data_to_tensor (nn/state.ts:192-223) for the quantised GGML types Q4_0 (2), Q4_1 (3), Q8_0 (8) and
 *   Q6_K (14): n elements (whole blocks) from the block bytes at `blocks` (2-byte aligned) to float32.
 *   ggml_nbytes: bytes that n elements of a type occupy (0 for a type that is not one of the four).
 * cast: n elements between JSGRAD_F32 / JSGRAD_F16, and from JSGRAD_BF16 (fix_bf16, models/llama.ts:272-279: bfloat16 ->
 *   float32 -> float16; `v.cast(float16)`, models/llama3.ts:234).
 * hf_permute: the q_proj / k_proj row permutation of convert_from_huggingface (models/llama.ts:225-227),
 *   dst = src.reshape(n_heads, 2, rows/n_heads/2, row).transpose(1, 2), rows of row_bytes bytes (a multiple of 16). */
enum { JSGRAD_BF16 = 2 };
size_t jsgrad_hip_ggml_nbytes(int ggml_type, size_t n);
int jsgrad_hip_ggml_dequant(int ggml_type, const void *blocks, size_t n, void *out_f32);
int jsgrad_hip_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n);
int jsgrad_hip_hf_permute(const void *src, void *dst, int rows, int row_bytes, int n_heads);

/* Random-init weights ~ N(0, std) in the given dtype (the role of Tensor.randn / Linear's random
 * initialisation, nn/index.ts:406-409, for synthetic models); counter-based, reproducible from seed. */
int jsgrad_hip_randn(void *out, size_t n, int dtype, uint64_t seed, float std);
/* Fill n elements of the given dtype with a constant (Tensor.ones for RMSNorm weights, nn/index.ts:583). */
int jsgrad_hip_fill(void *out, size_t n, int dtype, float value);

#ifdef __cplusplus
}
#endif
#endif /* JSGRAD_HIP_H */
