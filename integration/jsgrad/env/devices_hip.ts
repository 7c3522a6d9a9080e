// Registry entry for the HIP device.  jsgrad keeps one table of device classes per JS runtime
// (jsgrad/env/deno.ts:16, jsgrad/env/bun.ts:22, jsgrad/env/node.ts:22; default in jsgrad/env/web.ts:27) and
// `Device.get('HIP')` / `Device.get('HIP:0')` look the prefix up there (jsgrad/device.ts:20-35).  The change in each
// of those files is one import and one key:
//
//   import { HIP } from '../runtime/ops_hip.ts'
//   override DEVICES = { HIP, CLANG, WEBGPU: DAWN, WGPU: WEBGPU, WASM, JS, DISK, CLOUD }
//
// Putting HIP first makes it the default device when DEVICE / D is not set (jsgrad/device.ts:12-19).  Node's ffi-rs
// shim passes only `pointer` and `i32` (jsgrad/env/node.ts:49-53), so the table of hip_bindings.ts needs Deno or Bun.
//
// For code that cannot edit the env files, the same at run time:
import { env } from './index.ts'
import { HIP } from '../runtime/ops_hip.ts'

export const register_hip = (first = true) => {
  const rest = Object.fromEntries(Object.entries(env.DEVICES).filter(([k]) => k !== 'HIP'))
  env.DEVICES = first ? { HIP, ...rest } : { ...rest, HIP }
}
