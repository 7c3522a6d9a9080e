// The `HIP` device of jsgrad on libjsgrad_hip.so (gfx950): drop into jsgrad/runtime/ beside ops_dawn.ts.
// Pattern: jsgrad/runtime/ops_dawn.ts:234-307 (an FFI-backed Compiled), jsgrad/runtime/ops_clang.ts:7-60 (a compiler
// that shells out, a Program that calls native code), jsgrad/runtime/allocator.ts:28-47,99-139,166-191 (the contracts).
import { Allocator, type BufferSpec, Compiled, CompileError, Compiler, Program, type ProgramCallArgs } from './allocator.ts'
import { HIPRenderer } from '../renderer/cstyle.ts'
import type { MemoryView } from '../helpers/memoryview.ts'
import { vars } from '../helpers/helpers.ts'
import { env } from '../env/index.ts'
import type { Buffer } from '../device.ts'
import type { Variable } from '../ops.ts'
import { GraphException, GraphRunner } from '../engine/jit.ts'
import type { ExecItem } from '../engine/realize.ts'
import * as c from './hip_bindings.ts'

const LIB = () => vars.get('JSGRAD_HIP_LIB') || `${env.CACHE_DIR}/libjsgrad_hip.so`

// Buffers are device addresses kept as bigint: `_offset` is an addition, a view needs no second handle, and the value
// goes through Deno's FFI as a pointer object made on the spot (c.dev).
class HIPAllocator extends Allocator<bigint> {
  _alloc = (size: number, options?: BufferSpec): bigint => {
    const out = c.out_ptr()
    c.check(c.hip.symbols.jsgrad_hip_malloc(BigInt(size), out))
    return out[0]
  }
  // Callable from a FinalizationRegistry: the library parks the block for the next request of its size class and
  // never waits for the stream here (LRUAllocator's job, allocator.ts:53-77, done behind the C ABI).
  _free = (opaque: bigint, options?: BufferSpec) => c.check(c.hip.symbols.jsgrad_hip_free(c.dev(opaque)))
  free_cache = () => c.check(c.hip.symbols.jsgrad_hip_free_cache())
  _copyin = (dest: bigint, src: MemoryView) => c.check(c.hip.symbols.jsgrad_hip_copyin(c.dev(dest), src.bytes, BigInt(src.byteLength)))
  _copyout = (dest: MemoryView, src: bigint) => c.check(c.hip.symbols.jsgrad_hip_copyout(dest.bytes, c.dev(src), BigInt(dest.byteLength)))
  override _offset = (buf: bigint, size: number, offset: number): bigint => buf + BigInt(offset)
  override _transfer = (dest: bigint, src: bigint, sz: number, src_dev: unknown, dest_dev: unknown) => c.check(c.hip.symbols.jsgrad_hip_copy(c.dev(dest), c.dev(src), BigInt(sz)))
}

export class HIPProgram extends Program {
  module = 0n
  fn = 0n
  static override init = async (name: string, lib: Uint8Array) => {
    if (!lib?.length) throw new Error('Lib is empty')
    if (!name) throw new Error("Name can't be undefined")
    const res = new HIPProgram(name, lib)
    const mod = c.out_ptr(), fn = c.out_ptr()
    c.check(c.hip.symbols.jsgrad_hip_module_load(lib, BigInt(lib.length), mod))
    res.module = mod[0]
    c.check(c.hip.symbols.jsgrad_hip_module_get(c.dev(res.module), c.cstr(name), fn))
    res.fn = fn[0]
    return res
  }
  // Kernels take their buffers first and their int32 values after them, as the C-style renderers declare them.
  // Returns seconds when `wait` is set (engine/realize.ts:62-80 adds them to GlobalCounters.time_sum_s).
  override call = (bufs: bigint[], args: ProgramCallArgs, wait = false) => {
    const { global_size = [1, 1, 1], local_size = [1, 1, 1], vals = [] } = args
    if (vals.some((x) => x === undefined)) throw new Error(`${vals}`)
    const secs = new Float64Array(1)
    // the renderer's global_size counts blocks, like hipModuleLaunchKernel's grid
    c.check(c.hip.symbols.jsgrad_hip_launch(c.dev(this.fn), new Uint32Array(global_size), new Uint32Array(local_size), new BigUint64Array(bufs), bufs.length, new Int32Array(vals), vals.length, wait ? 1 : 0, secs))
    if (wait) return secs[0]
  }
  unload = () => {
    if (this.module) c.check(c.hip.symbols.jsgrad_hip_module_unload(c.dev(this.module)))
    this.module = 0n
  }
}

// packed fp32 instructions stay off on this hardware generation
const HIPCC_FLAGS = ['-O3', '-x', 'hip', '-include', 'hip/hip_runtime.h', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']
// A short stable number over the flags, so that a change of flags starts a new table of the disk cache.  (The Python twin
// also folds in `hipcc --version`; here a new compiler is told apart by ROCM_VERSION in the environment, when set.)
const flags_id = () => {
  let h = 2166136261
  for (const ch of HIPCC_FLAGS.join(' ') + '\n' + (vars.get('ROCM_VERSION') || '')) h = Math.imul(h ^ ch.charCodeAt(0), 16777619) >>> 0
  return h.toString(16).padStart(8, '0')
}

export class HIPCompiler extends Compiler {
  constructor(public arch = 'gfx950', cachekey = `compile_hip_${arch}_${flags_id()}`) {
    super(cachekey) // compile_cached keeps code objects in env's disk cache under this key (allocator.ts:129-137)
  }
  override compile = async (src: string): Promise<Uint8Array> => {
    const code = await env.tempFile(), bin = await env.tempFile()
    await env.writeTextFile(code, src)
    const args = ['hipcc', '--genco', `--offload-arch=${this.arch}`, ...HIPCC_FLAGS, code, '-o', bin]
    try {
      await env.exec(args.join(' '))
    } catch (e) {
      throw new CompileError(`${e}`)
    } finally {
      await env.remove(code)
    }
    const data = await env.readFile(bin)
    await env.remove(bin)
    return data
  }
}

// One HIP graph for a batch of captured ExecItems (the class apply_graph_to_jit instantiates, engine/jit.ts:14-69).
// The graph holds addresses and values as they were at capture: a batch whose kernels take symbolic values, or whose
// buffers are jit inputs, is refused and runs item by item.  The fused Llama runners qualify: position and token live
// in device words that the kernels read and advance, so nothing in their arguments changes from token to token.
export class HIPGraph extends GraphRunner {
  graph = 0n
  constructor(jit_cache: ExecItem[], input_rawbuffers: Buffer[], var_vals: Map<Variable, number>) {
    super(jit_cache, input_rawbuffers, var_vals)
    if (this.input_replace.size || this.var_vals_replace.size || this.launch_dims_replace.size) throw new GraphException('HIP graphs replay fixed arguments')
  }
  private capture = async (var_vals: Map<Variable, number>) => {
    c.check(c.hip.symbols.jsgrad_hip_graph_begin())
    try {
      for (const ji of this.jit_cache) await ji.prg.call(ji.bufs.map((b) => b!), var_vals, false)
    } finally {
      const out = c.out_ptr()
      c.check(c.hip.symbols.jsgrad_hip_graph_end(out))
      this.graph = out[0]
    }
  }
  override call = async (rawbufs: Buffer[], var_vals: Map<Variable, number>, wait = false) => {
    if (!this.graph) await this.capture(var_vals)
    const st = performance.now()
    c.check(c.hip.symbols.jsgrad_hip_graph_launch(c.dev(this.graph)))
    if (wait) {
      c.check(c.hip.symbols.jsgrad_hip_sync())
      return (performance.now() - st) / 1e3
    }
  }
  destroy = () => {
    if (this.graph) c.check(c.hip.symbols.jsgrad_hip_graph_destroy(c.dev(this.graph)))
    this.graph = 0n
  }
}

export class HIP extends Compiled {
  static ready = false
  static cu_count = 0
  constructor(device: string) {
    // HIPRenderer (renderer/cstyle.ts:496-498) serves every kernel the Llama rules do not claim; its tensor_cores
    // list (RDNA3 wave32 WMMA, inherited from AMDRenderer) must be emptied for gfx950's 64-wide wavefronts.
    super(device, new HIPAllocator(), Object.assign(new HIPRenderer(), { tensor_cores: [] }), new HIPCompiler(), HIPProgram, HIPGraph)
  }
  // Awaited before every use (engine/realize.ts:133,157): must be cheap the second time.
  override init = async () => {
    if (HIP.ready) return
    await c.init(LIB())
    const index = this.device.includes(':') ? Number(this.device.split(':')[1]) : 0
    c.check(c.hip.symbols.jsgrad_hip_init(index))
    const n = c.out_i32()
    c.check(c.hip.symbols.jsgrad_hip_cu_count(n))
    HIP.cu_count = n[0]
    HIP.ready = true
  }
  override synchronize = () => c.check(c.hip.symbols.jsgrad_hip_sync())
}
