// FFI table of libjsgrad_hip.so for jsgrad: drop into jsgrad/runtime/ beside ops_dawn.ts.
// Pattern: dawn/bindings.ts:5-8 (env.dlopen with a symbol table) and jsgrad/env/deno.ts:17-22 (pointer helpers).
//
// The table between the two markers is written by integration/jsgrad/gen_hip_bindings.py from include/jsgrad_hip.h:
// one entry per declaration, parameters in the header's order.  `pointer` is a device address (or an opaque handle:
// module, function, event, graph), `buffer` is host memory the call reads or fills before it returns (the header
// names those parameters host_*), `usize` is size_t.
import { env } from '../env/index.ts'

const P = 'pointer', B = 'buffer', I = 'i32', U32 = 'u32', F = 'f32', D = 'f64', U = 'usize', U64 = 'u64'

// <symbols>
const SYMBOLS = {
  jsgrad_hip_init: { parameters: [I], result: I }, // device
  jsgrad_hip_last_error: { parameters: [], result: P },
  jsgrad_hip_device_name: { parameters: [B, U], result: I }, // host_out, cap
  jsgrad_hip_cu_count: { parameters: [B], result: I }, // host_out
  jsgrad_hip_malloc: { parameters: [U, B], result: I }, // nbytes, host_out_ptr
  jsgrad_hip_free: { parameters: [P], result: I }, // ptr
  jsgrad_hip_free_cache: { parameters: [], result: I },
  jsgrad_hip_mem_info: { parameters: [B, B], result: I }, // host_out_live_bytes, host_out_idle_bytes
  jsgrad_hip_copyin: { parameters: [P, B, U], result: I }, // dst, host_src, nbytes
  jsgrad_hip_copyout: { parameters: [B, P, U], result: I }, // host_dst, src, nbytes
  jsgrad_hip_copy: { parameters: [P, P, U], result: I }, // dst, src, nbytes
  jsgrad_hip_memset: { parameters: [P, I, U], result: I }, // dst, byte, nbytes
  jsgrad_hip_sync: { parameters: [], result: I },
  jsgrad_hip_module_load: { parameters: [B, U, B], result: I }, // host_image, nbytes, host_out_module
  jsgrad_hip_module_unload: { parameters: [P], result: I }, // module
  jsgrad_hip_module_get: { parameters: [P, B, B], result: I }, // module, name, host_out_function
  jsgrad_hip_launch: { parameters: [P, B, B, B, I, B, I, I, B], result: I }, // function, host_grid, host_block, host_bufs, nbufs, host_vals, nvals, wait, host_seconds
  jsgrad_hip_event_create: { parameters: [B], result: I }, // host_out_event
  jsgrad_hip_event_record: { parameters: [P], result: I }, // event
  jsgrad_hip_event_elapsed_ms: { parameters: [P, P, B], result: I }, // start, stop, host_out_ms
  jsgrad_hip_event_destroy: { parameters: [P], result: I }, // event
  jsgrad_hip_profile: { parameters: [I], result: I }, // enable
  jsgrad_hip_profile_read: { parameters: [I, B, B], result: I }, // kind, host_out_count, host_out_total_ms
  jsgrad_hip_read_probe: { parameters: [P, U, P], result: I }, // src, nbytes, sink
  jsgrad_hip_graph_begin: { parameters: [], result: I },
  jsgrad_hip_graph_end: { parameters: [B], result: I }, // host_out_graph
  jsgrad_hip_graph_launch: { parameters: [P], result: I }, // graph
  jsgrad_hip_graph_destroy: { parameters: [P], result: I }, // graph
  jsgrad_hip_rope_table: { parameters: [P, I, I, F, I], result: I }, // table, head_dim, end, theta, act
  jsgrad_hip_embed: { parameters: [I, P, P, P, P, I, I, I], result: I }, // kind, table, scale, state, out, dim, vocab, act
  jsgrad_hip_rmsnorm: { parameters: [P, P, P, I, F, I], result: I }, // x, weight, y, dim, eps, act
  jsgrad_hip_linear: { parameters: [I, P, P, I, I, P, P, P, F, P, I], result: I }, // kind, w, scale, out_f, in_f, x, y, norm_weight, eps, residual, act
  jsgrad_hip_qkv_rope: { parameters: [I, P, P, P, P, P, P, P, P, F, P, P, P, P, P, I, I, I, I, I, I], result: I }, // kind, wq, sq, wk, sk, wv, sv, x, norm_weight, eps, rope_table, state, q_out, cache_k, cache_v, dim, n_heads, n_kv_heads, head_dim, max_context, act
  jsgrad_hip_attn_workspace_bytes: { parameters: [I, I, I], result: U }, // n_heads, n_kv_heads, head_dim
  jsgrad_hip_attn_decode: { parameters: [P, P, P, P, P, P, I, I, I, I, I], result: I }, // q, cache_k, cache_v, state, out, workspace, n_heads, n_kv_heads, head_dim, max_context, act
  jsgrad_hip_attn_decode_status: { parameters: [P, I, I, I, B], result: I }, // workspace, n_heads, n_kv_heads, head_dim, host_out_error
  jsgrad_hip_attn_decode_static_max_bytes: { parameters: [], result: U },
  jsgrad_hip_attn_decode_static: { parameters: [P, P, P, P, P, I, I, I, I, I], result: I }, // q, cache_k, cache_v, state, out, n_heads, n_kv_heads, head_dim, max_context, act
  jsgrad_hip_attn_decode_static_status: { parameters: [B], result: I }, // host_out_error
  jsgrad_hip_ffn_gate: { parameters: [I, P, P, P, P, P, P, F, P, I, I, I], result: I }, // kind, w1, s1, w3, s3, x, norm_weight, eps, g, dim, hidden, act
  jsgrad_hip_argmax: { parameters: [P, I, P, P, I, I, I], result: I }, // logits, n, state, tokens_out, tokens_cap, advance, act
  jsgrad_hip_embed_rows: { parameters: [I, P, P, P, I, P, I, I], result: I }, // kind, table, scale, tokens, rows, out, dim, vocab
  jsgrad_hip_rmsnorm_rows: { parameters: [P, P, P, I, I, F], result: I }, // x, weight, y, rows, dim, eps
  jsgrad_hip_gemm: { parameters: [I, P, P, I, I, P, I, P, P], result: I }, // kind, w, scale, out_f, in_f, x, rows, y, residual
  jsgrad_hip_gemm_qkv_rope: { parameters: [I, P, P, P, P, P, P, P, I, I, I, P, P, P, P, I, I, I, I, I], result: I }, // kind, wq, sq, wk, sk, wv, sv, x, rows, seq_len, start_pos, rope_table, q_out, cache_k, cache_v, dim, n_heads, n_kv_heads, head_dim, max_context
  jsgrad_hip_gemm_ffn_gate: { parameters: [I, P, P, P, P, P, I, P, I, I], result: I }, // kind, w1, s1, w3, s3, x, rows, g, dim, hidden
  jsgrad_hip_attn_prefill: { parameters: [P, P, P, P, I, I, I, I, I, I, I], result: I }, // q, cache_k, cache_v, out, batch, seq_len, start_pos, n_heads, n_kv_heads, head_dim, max_context
  jsgrad_hip_attn_batch_workspace_bytes: { parameters: [I, I, I, I], result: U }, // batch, n_heads, n_kv_heads, head_dim
  jsgrad_hip_attn_decode_batch: { parameters: [P, P, P, P, P, P, I, I, I, I, I], result: I }, // q, cache_k, cache_v, state, out, workspace, batch, n_heads, n_kv_heads, head_dim, max_context
  jsgrad_hip_argmax_rows: { parameters: [P, I, I, P], result: I }, // logits, rows, n, tokens_out
  jsgrad_hip_step_workspace_bytes: { parameters: [I, I, I], result: U }, // n_heads, n_kv_heads, head_dim
  jsgrad_hip_decode_step: { parameters: [B], result: I }, // host_desc
  jsgrad_hip_step_status: { parameters: [P, B], result: I }, // workspace, host_out_error
  jsgrad_hip_stream_workspace_bytes: { parameters: [I, I, I], result: U }, // n_heads, n_kv_heads, head_dim
  jsgrad_hip_stream_step: { parameters: [B], result: I }, // host_desc
  jsgrad_hip_stream_status: { parameters: [P, B], result: I }, // workspace, host_out_error
  jsgrad_hip_attn_wo_workspace_bytes: { parameters: [I, I, I], result: U }, // n_heads, n_kv_heads, head_dim
  jsgrad_hip_attn_wo: { parameters: [P, P, P, P, P, I, I, I, I, I, P, P, I, P, P, I], result: I }, // q, cache_k, cache_v, state, workspace, n_heads, n_kv_heads, head_dim, max_context, kind, wo, wo_scale, dim, residual, y, layer
  jsgrad_hip_attn_wo_status: { parameters: [P, B], result: I }, // workspace, host_out_error
  jsgrad_hip_attn_wo_items: { parameters: [I, I], result: I }, // n_kv_heads, max_context
  jsgrad_hip_attn_wo_fits: { parameters: [I, I, I, I, I, I, B, B], result: I }, // n_heads, n_kv_heads, head_dim, max_context, kind, dim, host_out_items, host_out_capacity
  jsgrad_hip_int8_quantize: { parameters: [P, I, I, P, P, I], result: I }, // w, out_f, in_f, codes, scale_f16, act
  jsgrad_hip_int8_dequant: { parameters: [P, P, I, I, P], result: I }, // codes, scale_f16, out_f, in_f, w16
  jsgrad_hip_nf4_quantize: { parameters: [P, U, P, P, I], result: I }, // w, n, packed, scale_f16, act
  jsgrad_hip_nf4_dequant: { parameters: [P, P, U, P], result: I }, // packed, scale_f16, n, w16
  jsgrad_hip_sample_workspace_bytes: { parameters: [I], result: U }, // n
  jsgrad_hip_sample: { parameters: [P, I, I, D, I, D, D, D, P, P, P, P, I, I, P], result: I }, // logits, n, act, temp, k, p, af, ap, alpha_counter, rng, state, tokens_out, tokens_cap, advance, workspace
  jsgrad_hip_ggml_nbytes: { parameters: [I, U], result: U }, // ggml_type, n
  jsgrad_hip_ggml_dequant: { parameters: [I, P, U, P], result: I }, // ggml_type, blocks, n, out_f32
  jsgrad_hip_cast: { parameters: [P, I, P, I, U], result: I }, // src, src_dtype, dst, dst_dtype, n
  jsgrad_hip_hf_permute: { parameters: [P, P, I, I, I], result: I }, // src, dst, rows, row_bytes, n_heads
  jsgrad_hip_randn: { parameters: [P, U, I, U64, F], result: I }, // out, n, dtype, seed, std
  jsgrad_hip_fill: { parameters: [P, U, I, F], result: I }, // out, n, dtype, value
} as const
// </symbols>

export type HipLib = { symbols: { [K in keyof typeof SYMBOLS]: (...args: any[]) => any }; close: () => void }
export let hip: HipLib
/** Opens the library once; later calls return the same handle. */
export const init = async (path: string): Promise<HipLib> => {
  if (!hip) hip = (await env.dlopen(path, SYMBOLS)) as unknown as HipLib
  return hip
}
/** Every int entry point returns 0 or an error code whose text jsgrad_hip_last_error holds. */
export const check = (rc: number): void => {
  if (rc !== 0) throw new Error(`HIP: ${env.getCString(hip.symbols.jsgrad_hip_last_error())} (${rc})`)
}

// include/jsgrad_hip.h: activation dtypes, weight formats, cast sources, profile kinds
export const JSGRAD_F32 = 0, JSGRAD_F16 = 1, JSGRAD_BF16 = 2
export const JSGRAD_W_F32 = 0, JSGRAD_W_F16 = 1, JSGRAD_W_I8 = 2, JSGRAD_W_NF4 = 3
export const PROF = ['EMBED', 'RMSNORM', 'LINEAR', 'QKV_ROPE', 'ATTN', 'FFN_GATE', 'ARGMAX', 'STEP', 'GEMM', 'ATTN_PREFILL', 'ATTN_WO', 'READ', 'SAMPLE'] as const

/** A device address as the number Deno's FFI passes for `pointer` parameters. */
export type DevPtr = bigint
export const dev = (p: DevPtr) => p === 0n ? null : env.u64ToPtr(p)
export const NULL = null

/** jsgrad_hip_malloc's out parameter and friends: one 8-byte slot read back as a bigint. */
export const out_ptr = () => new BigUint64Array(1)
export const out_i32 = () => new Int32Array(1)
export const cstr = (s: string) => new TextEncoder().encode(s + '\0')

// ---- jsgrad_hip_layer_t / jsgrad_hip_step_t (include/jsgrad_hip.h): natural C layout on x86-64, 8-byte pointers
export const LAYER_FIELDS = ['wq', 'wk', 'wv', 'wo', 'w1', 'w2', 'w3', 'sq', 'sk', 'sv', 'so', 's1', 's2', 's3', 'attention_norm', 'ffn_norm', 'cache_k', 'cache_v'] as const
export const LAYER_BYTES = LAYER_FIELDS.length * 8
export type LayerPtrs = { [K in (typeof LAYER_FIELDS)[number]]: DevPtr }
/** The device array `layers` points to: n_layers records of 18 pointers, to be copied in with jsgrad_hip_copyin. */
export const pack_layers = (layers: LayerPtrs[]): Uint8Array => {
  const out = new BigUint64Array(layers.length * LAYER_FIELDS.length)
  layers.forEach((l, i) => LAYER_FIELDS.forEach((f, j) => out[i * LAYER_FIELDS.length + j] = l[f] ?? 0n))
  return new Uint8Array(out.buffer)
}
export type StepDesc = {
  layers: DevPtr
  n_layers: number, dim: number, hidden: number, n_heads: number, n_kv_heads: number, head_dim: number, vocab: number, max_context: number
  eps: number
  kind: number, out_kind: number, embed_kind: number, act: number
  tok_emb: DevPtr, tok_scale: DevPtr, out_w: DevPtr, out_s: DevPtr, final_norm: DevPtr, rope_table: DevPtr
  state: DevPtr, tokens_out: DevPtr
  tokens_cap: number
  h: DevPtr, h2: DevPtr, q: DevPtr, attn: DevPtr, g: DevPtr, logits: DevPtr
  workspace: DevPtr, trace?: DevPtr
}
export const STEP_BYTES = 200
/** The host descriptor handed to jsgrad_hip_decode_step / jsgrad_hip_stream_step. */
export const pack_step = (d: StepDesc): Uint8Array => {
  const buf = new ArrayBuffer(STEP_BYTES), v = new DataView(buf)
  let o = 0
  const ptr = (p?: DevPtr) => { v.setBigUint64(o, p ?? 0n, true); o += 8 }
  const i32 = (x: number) => { v.setInt32(o, x, true); o += 4 }
  ptr(d.layers)                                                                                                                    // 0
  for (const x of [d.n_layers, d.dim, d.hidden, d.n_heads, d.n_kv_heads, d.head_dim, d.vocab, d.max_context]) i32(x)             // 8..40
  v.setFloat32(o, d.eps, true); o += 4                                                                                             // 40
  for (const x of [d.kind, d.out_kind, d.embed_kind, d.act]) i32(x)                                                               // 44..60
  o += 4                                                                                                                           // pad to 64
  for (const p of [d.tok_emb, d.tok_scale, d.out_w, d.out_s, d.final_norm, d.rope_table, d.state, d.tokens_out]) ptr(p)           // 64..128
  i32(d.tokens_cap); o += 4                                                                                                        // 128, pad to 136
  for (const p of [d.h, d.h2, d.q, d.attn, d.g, d.logits, d.workspace, d.trace]) ptr(p)                                           // 136..200
  if (o !== STEP_BYTES) throw new Error(`jsgrad_hip_step_t layout: ${o} bytes`)
  return new Uint8Array(buf)
}
