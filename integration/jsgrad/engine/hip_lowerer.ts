// Routing of Llama's matrix-vector kernels to libjsgrad_hip.so at the schedule level: drop into jsgrad/engine/ and
// put `hip_linear_rule` in front of the generic SINK rule of si_lowerer (jsgrad/engine/realize.ts:185-193):
//
//   export const si_lowerer = new PatternMatcher<Buffer[], ...>([
//     hip_linear_rule,                                   // <- added; returns undefined for every other kernel
//     new UPat(Ops.SINK).named('sink').fn(({ ctx, sink }) => get_runner(ctx[0].device, sink).then(...)),
//     ...
//
// A rule sees ONE ScheduleItem: its AST (`SINK(STORE(DEFINE_GLOBAL#0, VIEW, value))`, schedule.ts:201-252) and its buffers
// in DEFINE_GLOBAL order, output first.  The kernels that span several ScheduleItems of the reference's schedule
// (rmsnorm + q/k/v + rotary + cache write, the attention chain, w1/w3 + SwiGLU) are reached from the model instead:
// see models/llama_hip.ts.
import type { Buffer } from '../device.ts'
import { dtypes } from '../dtype.ts'
import { Ops, type UOp, UPat, type Variable } from '../ops.ts'
import { Estimates } from '../renderer/index.ts'
import { Runner } from './realize.ts'
import * as c from '../runtime/hip_bindings.ts'

type Match = { kind: number; act: number; out_f: number; in_f: number; x: number; w: number; scale?: number; residual?: number }

const global_index = (load: UOp): number | undefined => load.op === Ops.LOAD && load.src[0].op === Ops.DEFINE_GLOBAL ? load.src[0].arg as number : undefined
const view_of = (load: UOp) => load.src[1].arg.views.at(-1)! // ShapeTracker of the LOAD; one view for these kernels
const through_cast = (u: UOp) => u.op === Ops.CAST ? u.src[0] : u

// [.., out, in] with strides (.., in, 1): the weight matrix, read once, row by row
const is_weight_view = (load: UOp, out_f: number, in_f: number) => {
  const v = view_of(load), n = v.shape.length
  return load.src[1].arg.views.length === 1 && v.mask === undefined && v.offset === 0 && v.shape[n - 1] === in_f && v.shape[n - 2] === out_f && v.strides[n - 1] === 1 && v.strides[n - 2] === in_f &&
    v.shape.slice(0, n - 2).every((s: number) => s === 1)
}
// the input row, broadcast over the output axis (stride 0 there)
const is_row_view = (load: UOp, out_f: number, in_f: number) => {
  const v = view_of(load), n = v.shape.length
  return load.src[1].arg.views.length === 1 && v.mask === undefined && v.offset === 0 && v.shape[n - 1] === in_f && v.strides[n - 1] === 1 && v.strides[n - 2] === 0 && v.shape.slice(0, n - 2).every((s: number) => s === 1)
}
// one number per output row, broadcast over the input axis
const is_scale_view = (load: UOp, out_f: number) => {
  const v = view_of(load), n = v.shape.length
  return v.mask === undefined && v.offset === 0 && v.shape[n - 2] === out_f && v.strides[n - 2] === 1 && v.strides[n - 1] === 0
}
// the output row itself (residual operand of the epilogue)
const is_out_view = (load: UOp, out_f: number) => {
  const v = view_of(load), n = v.shape.length
  return v.mask === undefined && v.offset === 0 && v.shape[n - 2] === out_f && v.strides[n - 2] === 1 && v.shape[n - 1] === 1
}

/**
 * Recognises `x.linear(W.T)` for a [1,1,in] row as Tensor.dot leaves it (tensor.ts:2602-2604):
 *   STORE( CAST:act( REDUCE_AXIS ADD last( CAST:float( MUL( LOAD x, W ) ) ) ) [ + LOAD residual ] )
 * with W = LOAD w (fp16 / fp32 weights) or MUL( CAST:half( LOAD w:int8 ), LOAD scale ) (Int8Linear.call, llama3.ts:31-35).
 * Anything else - other shapes, masks, more than one view, several rows - is left to the generic rule.
 */
export const match_linear = (sink: UOp): Match | undefined => {
  if (sink.src.length !== 1 || sink.src[0].op !== Ops.STORE) return undefined
  const [out, out_view, value0] = sink.src[0].src
  if (out.op !== Ops.DEFINE_GLOBAL || out.arg !== 0) return undefined
  const act = out.dtype.base === dtypes.half ? c.JSGRAD_F16 : out.dtype.base === dtypes.float ? c.JSGRAD_F32 : undefined
  if (act === undefined) return undefined
  const oshape = out_view.arg.shape as number[]
  const out_f = oshape[oshape.length - 2]
  if (oshape[oshape.length - 1] !== 1 || oshape.slice(0, -2).some((s) => s !== 1)) return undefined

  // epilogue: value = dot + residual, operands in either order
  let value = value0, residual: number | undefined
  if (value.op === Ops.ADD) {
    const side = value.src.findIndex((s) => s.op === Ops.LOAD && is_out_view(s, out_f))
    if (side < 0) return undefined
    residual = global_index(value.src[side])
    value = value.src[1 - side]
  }
  const red = through_cast(value)
  if (red.op !== Ops.REDUCE_AXIS || red.arg[0] !== Ops.ADD || red.arg[1].length !== 1 || red.arg[1][0] !== oshape.length - 1) return undefined
  const mul = through_cast(red.src[0])
  if (mul.op !== Ops.MUL) return undefined

  for (const [xi, wi] of [[0, 1], [1, 0]]) {
    const x = mul.src[xi], w = mul.src[wi]
    if (x.op !== Ops.LOAD) continue
    const in_f = view_of(x).shape.at(-1) as number
    if (!is_row_view(x, out_f, in_f) || x.dtype !== out.dtype.base) continue
    if (w.op === Ops.LOAD && is_weight_view(w, out_f, in_f) && w.dtype === out.dtype.base) {
      return { kind: act === c.JSGRAD_F16 ? c.JSGRAD_W_F16 : c.JSGRAD_W_F32, act, out_f, in_f, x: global_index(x)!, w: global_index(w)!, residual }
    }
    if (w.op === Ops.MUL) { // int8 codes widened to half, times the row's scale
      for (const [qi, si] of [[0, 1], [1, 0]]) {
        const q = through_cast(w.src[qi]), s = w.src[si]
        if (q.op === Ops.LOAD && q.dtype === dtypes.int8 && is_weight_view(q, out_f, in_f) && s.op === Ops.LOAD && s.dtype === dtypes.half && is_scale_view(s, out_f)) {
          return { kind: c.JSGRAD_W_I8, act, out_f, in_f, x: global_index(x)!, w: global_index(q)!, scale: global_index(s), residual }
        }
      }
    }
  }
  return undefined
}

/** One jsgrad_hip_linear call in place of the rendered kernel; captured by TinyJit like any Runner (jit.ts:253-255). */
export class HipLinearRunner extends Runner {
  constructor(public m: Match, device: string) {
    const weight_bytes = m.out_f * m.in_f * (m.kind === c.JSGRAD_W_I8 ? 1 : m.kind === c.JSGRAD_W_F16 ? 2 : 4)
    super(`hip_linear_${['f32', 'f16', 'i8'][m.kind]}_${m.out_f}_${m.in_f}${m.residual !== undefined ? '_res' : ''}`, device, new Estimates(2 * m.out_f * m.in_f, weight_bytes, weight_bytes))
  }
  override call = (rawbufs: Buffer[], var_vals: Map<Variable, number>, wait = false): number | undefined => {
    const m = this.m, p = (i?: number) => i === undefined ? null : c.dev(rawbufs[i]._buf as bigint)
    const st = performance.now()
    c.check(c.hip.symbols.jsgrad_hip_linear(m.kind, p(m.w), p(m.scale), m.out_f, m.in_f, p(m.x), p(0), null, 0, p(m.residual), m.act))
    if (wait) {
      c.check(c.hip.symbols.jsgrad_hip_sync())
      return (performance.now() - st) / 1e3
    }
  }
}

// The rule itself.  ctx = the ScheduleItem's buffers; only kernels on a HIP device are looked at.
export const hip_linear_rule = new UPat(Ops.SINK).named('sink').fn<Buffer[], [Runner, Buffer[]] | undefined>(({ ctx, sink }) => {
  if (ctx[0].device.split(':')[0] !== 'HIP') return undefined
  const m = match_linear(sink)
  if (m === undefined || m.in_f % 8 !== 0) return undefined // rows are read in 16-byte pieces
  return [new HipLinearRunner(m, ctx[0].device), [...ctx]]
})
