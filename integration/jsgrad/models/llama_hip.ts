// Decode step of models/llama.ts on the fused kernels of libjsgrad_hip.so: drop into jsgrad/models/ beside llama.ts.
//
// `HipDecoder.from(model)` takes a loaded Transformer (models/llama.ts:186-222) whose tensors live on a HIP device and
// replaces what `model.call(tokens [1,1], start_pos, ...)` does for start_pos > 0 - the TinyJit replay of forward
// (llama.ts:215-218) - by the launch sequence below.  Weights stay where load_state_dict put them; nothing is copied.
//   per layer: attention_norm + wq/wk/wv + rotary + cache write   jsgrad_hip_qkv_rope      (llama.ts:61-90, nn/index.ts:586-588)
//              attention + wo + residual                           jsgrad_hip_attn_wo       (llama.ts:92-100,124)
//              ffn_norm + w1/w3 + SwiGLU                           jsgrad_hip_ffn_gate      (llama.ts:108-110)
//              w2 + residual                                       jsgrad_hip_linear        (llama.ts:109,125)
//   then:      norm + output                                       jsgrad_hip_linear        (llama.ts:209)
//              sample / argmax, token and position advanced        jsgrad_hip_sample/argmax (llama.ts:131-185)
// The sequence is captured once as a HIP graph and replayed per token; token and position live in two device words.
import { type Buffer, uop_realized } from '../device.ts'
import { dtypes } from '../dtype.ts'
import type { UOp } from '../ops.ts'
import { Tensor } from '../tensor.ts'
import type { Transformer } from './llama.ts'
import * as c from '../runtime/hip_bindings.ts'

const buf = (t: Tensor): Buffer => {
  const b = uop_realized((t.lazydata as UOp).base)
  if (b === undefined) throw new Error('tensor is not realized')
  return b.ensure_allocated()
}
const addr = (t?: Tensor): bigint => t === undefined ? 0n : buf(t)._buf as bigint
const ptr = (t?: Tensor) => c.dev(addr(t))

type Lin = { weight: Tensor; scale?: Tensor }
const kind_of = (l: Lin): number => {
  if (l.weight.dtype === dtypes.int8) return c.JSGRAD_W_I8
  if (l.weight.dtype === dtypes.uint8) return c.JSGRAD_W_NF4
  return l.weight.dtype === dtypes.half ? c.JSGRAD_W_F16 : c.JSGRAD_W_F32
}

export class HipDecoder {
  state!: Tensor // int32 {token, start_pos}
  tokens_out!: Tensor // int32[max_context]: the token produced at each position
  private h!: Tensor
  private h2!: Tensor
  private q!: Tensor
  private attn!: Tensor
  private g!: Tensor
  private logits!: Tensor
  private attn_ws!: Tensor
  private attn_wo_ws?: Tensor
  private sample_ws!: Tensor
  private alpha_counter!: Tensor
  private rng!: Tensor
  private rope!: Tensor
  private graph = 0n
  private graph_key = ''
  private constructor(public model: Transformer, public device: string, public act: number) {}

  static from = async (model: Transformer): Promise<HipDecoder> => {
    const l0 = model.layers[0].attention
    const x = model.norm.weight
    if (Array.isArray(x.device) || !x.device.startsWith('HIP')) throw new Error(`HipDecoder needs the model on a HIP device, got ${x.device}`)
    const act = x.dtype === dtypes.half ? c.JSGRAD_F16 : c.JSGRAD_F32
    const d = new HipDecoder(model, x.device, act)
    const dim = x.shape_num[0], hidden = model.layers[0].feed_forward.w1.weight.shape_num[0], vocab = model.output.weight.shape_num[0]
    const opt = { dtype: x.dtype, device: x.device }
    const mk = async (n: number) => await Tensor.zeros([n], opt).contiguous().realize()
    ;[d.h, d.h2, d.q, d.attn, d.g, d.logits] = await Promise.all([dim, dim, l0.n_heads * l0.head_dim, l0.n_heads * l0.head_dim, hidden, vocab].map(mk))
    const bytes = async (n: number) => await Tensor.zeros([Math.max(n, 16)], { dtype: dtypes.uint8, device: x.device }).contiguous().realize()
    const S = c.hip.symbols
    d.attn_ws = await bytes(Number(S.jsgrad_hip_attn_workspace_bytes(l0.n_heads, l0.n_kv_heads, l0.head_dim)))
    d.sample_ws = await bytes(Number(S.jsgrad_hip_sample_workspace_bytes(vocab)))
    d.alpha_counter = await Tensor.zeros([vocab], { dtype: dtypes.int32, device: x.device }).contiguous().realize()
    d.state = await Tensor.zeros([2], { dtype: dtypes.int32, device: x.device }).contiguous().realize()
    d.tokens_out = await Tensor.zeros([model.max_context], { dtype: dtypes.int32, device: x.device }).contiguous().realize()
    // {device seed, Tensor._seed, counter}: the three words Tensor.rand would combine (tensor.ts:813-819)
    d.rng = await new Tensor([0, Tensor._seed, 0], { dtype: dtypes.uint32, device: x.device }).contiguous().realize()
    d.rope = await model.freqs_cis.cast(x.dtype).contiguous().realize()
    for (const layer of model.layers) {
      const a = layer.attention
      if (a.cache_kv === undefined) a.cache_kv = await Tensor.zeros([2, 1, model.max_context, a.n_kv_heads, a.head_dim], opt).contiguous().realize()
    }
    // attention and wo share a launch when every attention block fits the device at once and the format allows it
    const wo = l0.wo as Lin, items = c.out_i32(), cap = c.out_i32()
    c.check(S.jsgrad_hip_attn_wo_fits(l0.n_heads, l0.n_kv_heads, l0.head_dim, model.max_context, kind_of(wo), dim, items, cap))
    if (act === c.JSGRAD_F16 && model.layers.length >= 2 && model.layers.length <= 128 && [c.JSGRAD_W_F16, c.JSGRAD_W_I8, c.JSGRAD_W_NF4].includes(kind_of(wo)) && items[0] <= cap[0]) {
      d.attn_wo_ws = await bytes(Number(S.jsgrad_hip_attn_wo_workspace_bytes(l0.n_heads, l0.n_kv_heads, l0.head_dim)))
    }
    return d
  }

  /** The launches of one token, queued on the library's stream (directly, or into a graph under capture). */
  private step = (temperature: number, top_k: number, top_p: number, alpha_f: number, alpha_p: number) => {
    const S = c.hip.symbols, m = this.model, act = this.act
    const dim = this.h.shape_num[0], hidden = this.g.shape_num[0], vocab = this.logits.shape_num[0]
    const emb = m.tok_embeddings as unknown as Lin
    c.check(S.jsgrad_hip_embed(kind_of(emb), ptr(emb.weight), ptr(emb.scale), ptr(this.state), ptr(this.h), dim, vocab, act))
    let x = this.h, y = this.h2
    m.layers.forEach((layer, li) => {
      const a = layer.attention, f = layer.feed_forward, eps = layer.attention_norm.eps
      const [wq, wk, wv, wo, w1, w2, w3] = [a.wq, a.wk, a.wv, a.wo, f.w1, f.w2, f.w3] as Lin[]
      const cache_bytes = BigInt(this.model.max_context * a.n_kv_heads * a.head_dim * (act === c.JSGRAD_F16 ? 2 : 4))
      const ck = c.dev(addr(a.cache_kv)), cv = c.dev(addr(a.cache_kv) + cache_bytes)
      c.check(S.jsgrad_hip_qkv_rope(kind_of(wq), ptr(wq.weight), ptr(wq.scale), ptr(wk.weight), ptr(wk.scale), ptr(wv.weight), ptr(wv.scale), ptr(x), ptr(layer.attention_norm.weight), eps,
        ptr(this.rope), ptr(this.state), ptr(this.q), ck, cv, dim, a.n_heads, a.n_kv_heads, a.head_dim, m.max_context, act))
      if (this.attn_wo_ws) {
        c.check(S.jsgrad_hip_attn_wo(ptr(this.q), ck, cv, ptr(this.state), ptr(this.attn_wo_ws), a.n_heads, a.n_kv_heads, a.head_dim, m.max_context, kind_of(wo), ptr(wo.weight), ptr(wo.scale), dim, ptr(x), ptr(y), li))
      } else {
        c.check(S.jsgrad_hip_attn_decode(ptr(this.q), ck, cv, ptr(this.state), ptr(this.attn), ptr(this.attn_ws), a.n_heads, a.n_kv_heads, a.head_dim, m.max_context, act))
        c.check(S.jsgrad_hip_linear(kind_of(wo), ptr(wo.weight), ptr(wo.scale), dim, a.n_heads * a.head_dim, ptr(this.attn), ptr(y), null, 0, ptr(x), act))
      }
      c.check(S.jsgrad_hip_ffn_gate(kind_of(w1), ptr(w1.weight), ptr(w1.scale), ptr(w3.weight), ptr(w3.scale), ptr(y), ptr(layer.ffn_norm.weight), layer.ffn_norm.eps, ptr(this.g), dim, hidden, act))
      c.check(S.jsgrad_hip_linear(kind_of(w2), ptr(w2.weight), ptr(w2.scale), dim, hidden, ptr(this.g), ptr(x), null, 0, ptr(y), act))
    })
    const out = m.output as Lin
    c.check(S.jsgrad_hip_linear(kind_of(out), ptr(out.weight), ptr(out.scale), vocab, dim, ptr(x), ptr(this.logits), ptr(m.norm.weight), m.norm.eps, null, act))
    if (temperature < 1e-6) c.check(S.jsgrad_hip_argmax(ptr(this.logits), vocab, ptr(this.state), ptr(this.tokens_out), m.max_context, 1, act))
    else c.check(S.jsgrad_hip_sample(ptr(this.logits), vocab, act, temperature, top_k, top_p, alpha_f, alpha_p, ptr(this.alpha_counter), ptr(this.rng), ptr(this.state), ptr(this.tokens_out), m.max_context, 1, ptr(this.sample_ws)))
  }

  /** Same arguments and result as Transformer.call for tokens of shape [1,1] (llama.ts:214-220): the sampled token, on the device. */
  call = async (tokens: Tensor, start_pos: number, temperature = 0.0, top_k = 0, top_p = 0.8, alpha_f = 0.0, alpha_p = 0.0): Promise<Tensor> => {
    if (tokens.shape_num[0] !== 1 || tokens.shape_num[1] !== 1) return await this.model.call(tokens, start_pos, temperature, top_k, top_p, alpha_f, alpha_p)
    if (start_pos + 1 > this.model.max_context) throw new Error(`position ${start_pos} is outside max_context ${this.model.max_context}`)
    const S = c.hip.symbols
    // the fed token: copied device to device when it is the previous result, otherwise written from the host
    c.check(S.jsgrad_hip_copy(ptr(this.state), ptr(await tokens.cast(dtypes.int32).contiguous().realize()), 4n))
    c.check(S.jsgrad_hip_copyin(c.dev(addr(this.state) + 4n), new Int32Array([start_pos]), 4n))
    const key = [temperature, top_k, top_p, alpha_f, alpha_p].join()
    if (this.graph && key !== this.graph_key) {
      c.check(S.jsgrad_hip_graph_destroy(c.dev(this.graph)))
      this.graph = 0n
    }
    if (!this.graph) {
      // This position runs outside a graph (it produces the token and moves the position on); the same launches are
      // then recorded, without running, for the positions that follow.
      this.step(temperature, top_k, top_p, alpha_f, alpha_p)
      c.check(S.jsgrad_hip_graph_begin())
      let g: BigUint64Array
      try {
        this.step(temperature, top_k, top_p, alpha_f, alpha_p)
      } finally {
        g = c.out_ptr()
        c.check(S.jsgrad_hip_graph_end(g))
      }
      this.graph = g[0], this.graph_key = key
    } else c.check(S.jsgrad_hip_graph_launch(c.dev(this.graph)))
    if (this.attn_wo_ws) {
      const err = c.out_i32()
      c.check(S.jsgrad_hip_attn_wo_status(ptr(this.attn_wo_ws), err)) // waits for the stream, like the caller's .item()
      if (err[0]) throw new Error('jsgrad_hip_attn_wo: a bounded wait ran out; the tokens of this step are not to be trusted')
    } else {
      const a = this.model.layers[0].attention, err = c.out_i32()
      c.check(S.jsgrad_hip_attn_decode_status(ptr(this.attn_ws), a.n_heads, a.n_kv_heads, a.head_dim, err)) // reports and clears
      if (err[0]) throw new Error('jsgrad_hip_attn_decode: a bounded wait ran out; the tokens of this step are not to be trusted')
    }
    return this.state.shrink([[0, 1]])
  }
}
