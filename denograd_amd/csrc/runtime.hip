// Device, memory, program loading, launch, timing and graph capture for libjsgrad_hip.so.
// Stands behind jsgrad's Compiled / Allocator / Program contracts
// (/root/reference/jsgrad/runtime/allocator.ts:28-47,99-107,166-191).
#include <stdarg.h>
#include <string.h>

#include <stdlib.h>

#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace jsg {

static thread_local char g_err[1024] = "";

State &state() {
  static State s;
  return s;
}
int fail(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}
int fail_hip(hipError_t e, const char *what) {
  snprintf(g_err, sizeof(g_err), "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
  return (int)e ? (int)e : 1;
}


// ---- profiling: one event pair per launch, summed per kernel kind when read back
struct ProfState {
  bool on = false;
  std::vector<hipEvent_t> ev;  // 2 per slot
  std::vector<int> kind;
  size_t used = 0;
};
static ProfState g_prof;
static constexpr size_t PROF_SLOTS = 16384;

bool prof_events(int kind, hipEvent_t *start, hipEvent_t *stop) {
  if (!g_prof.on || state().capturing || g_prof.used >= PROF_SLOTS) return false;
  const size_t slot = g_prof.used++;
  g_prof.kind[slot] = kind;
  *start = g_prof.ev[2 * slot];
  *stop = g_prof.ev[2 * slot + 1];
  return true;
}


// ---- device memory: blocks that were freed wait, by size class, for the next request of that class
// (LRUAllocator, /root/reference/jsgrad/runtime/allocator.ts:53-77).  Every launch and copy of this library is queued on one
// in-order stream, so a block can change hands without waiting for the stream: whatever still reads the old contents
// was queued before anything the new owner queues.  Memory goes back to the driver only where the stream is waited for
// anyway (jsgrad_hip_sync, a failed hipMalloc, jsgrad_hip_free_cache), never from jsgrad_hip_free.
struct MemCache {
  std::unordered_map<void *, size_t> live;                // every block handed out -> bytes of its class
  std::unordered_map<size_t, std::vector<void *>> idle;   // freed blocks by class, last freed on top
  size_t live_bytes = 0, idle_bytes = 0;
  size_t limit = 0;                                       // idle bytes beyond which the next stream wait gives them back
  bool enabled = true;                                    // LRU=0 switches the cache off (allocator.ts:73)
  // Frees arrive from finalisers on whatever thread runs them (ctypes releases the interpreter lock during a call), so the
  // books are kept under a lock; the stream waits and driver calls made while it is held are short and rare.
  std::mutex lock;
};
static MemCache g_mem;

// Classes are fine enough to waste under 2 % and coarse enough that tensors of nearly one size share blocks.
// n <= MEM_MAX_REQUEST (checked by the caller): rounding up cannot wrap.
constexpr size_t MEM_MAX_REQUEST = (size_t)1 << 48;
static size_t mem_class(size_t n) {
  const size_t step = n <= (64u << 10) ? 256 : n <= (4u << 20) ? (4u << 10) : n <= (256u << 20) ? (256u << 10) : (4u << 20);
  return (n + step - 1) / step * step;
}
// The stream must have been waited for.
static int mem_release_idle() {
  hipError_t first = hipSuccess;
  for (auto &kv : g_mem.idle)
    for (void *p : kv.second) {
      const hipError_t e = hipFree(p);
      if (e != hipSuccess && first == hipSuccess) first = e;
    }
  g_mem.idle.clear();
  g_mem.idle_bytes = 0;
  return first == hipSuccess ? 0 : fail_hip(first, "hipFree");
}

}  // namespace jsg

using jsg::state;

extern "C" {

const char *jsgrad_hip_last_error(void) { return jsg::g_err; }

int jsgrad_hip_init(int device) {
  jsg::State &s = state();
  if (s.ready && s.device == device) return 0;
  JSG_REQUIRE(!s.ready, "jsgrad_hip_init: already initialised on device %d", s.device);
  int n = 0;
  JSG_HIP(hipGetDeviceCount(&n));
  JSG_REQUIRE(device >= 0 && device < n, "jsgrad_hip_init: device %d out of range (%d devices)", device, n);
  JSG_HIP(hipSetDevice(device));
  hipDeviceProp_t p;
  JSG_HIP(hipGetDeviceProperties(&p, device));
  JSG_REQUIRE(strncmp(p.gcnArchName, "gfx950", 6) == 0, "jsgrad_hip_init: this library holds gfx950 code only, device is %s", p.gcnArchName);
  s.cu_count = p.multiProcessorCount;
  JSG_HIP(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking));
  {
    const char *lru = getenv("LRU"), *mb = getenv("JSGRAD_HIP_CACHE_MB");
    jsg::g_mem.enabled = !(lru && atoi(lru) == 0);
    jsg::g_mem.limit = mb ? (size_t)strtoull(mb, nullptr, 10) << 20 : p.totalGlobalMem / 8;
  }
  s.device = device;
  if (int e = jsg::attn_static_init(device)) return e;
  s.ready = true;
  return 0;
}

int jsgrad_hip_device_name(char *host_out, size_t cap) {
  JSG_READY();
  hipDeviceProp_t p;
  JSG_HIP(hipGetDeviceProperties(&p, state().device));
  snprintf(host_out, cap, "%s (%s)", p.name, p.gcnArchName);
  return 0;
}
int jsgrad_hip_cu_count(int *host_out) {
  JSG_READY();
  *host_out = state().cu_count;
  return 0;
}

int jsgrad_hip_malloc(size_t nbytes, void **host_out_ptr) {
  JSG_READY();
  JSG_REQUIRE(nbytes > 0, "alloc size must be positive, getting %zu", nbytes);
  JSG_REQUIRE(nbytes <= jsg::MEM_MAX_REQUEST, "alloc size %zu is beyond any device", nbytes);
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_malloc during graph capture");
  jsg::MemCache &m = jsg::g_mem;
  std::lock_guard<std::mutex> guard(m.lock);
  const size_t cls = jsg::mem_class(nbytes);
  auto it = m.idle.find(cls);
  void *p = nullptr;
  if (it != m.idle.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    m.idle_bytes -= cls;
  } else {
    if (m.idle_bytes > m.limit) {
      JSG_HIP(hipStreamSynchronize(state().stream));
      if (int r = jsg::mem_release_idle()) return r;
    }
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess && m.idle_bytes > 0) {
      // out of memory with blocks lying idle: give them back and ask again (allocator.ts:60-66)
      (void)hipGetLastError();
      JSG_HIP(hipStreamSynchronize(state().stream));
      if (int r = jsg::mem_release_idle()) return r;
      e = hipMalloc(&p, cls);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return jsg::fail_hip(e, "hipMalloc");
    }
  }
  m.live[p] = cls;
  m.live_bytes += cls;
  *host_out_ptr = p;
  return 0;
}
int jsgrad_hip_free(void *ptr) {
  JSG_READY();
  if (!ptr) return 0;
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_free during graph capture");
  jsg::MemCache &m = jsg::g_mem;
  std::lock_guard<std::mutex> guard(m.lock);
  auto it = m.live.find(ptr);
  JSG_REQUIRE(it != m.live.end(), "jsgrad_hip_free: %p was not handed out by jsgrad_hip_malloc (or was freed already)", ptr);
  const size_t cls = it->second;
  m.live.erase(it);
  m.live_bytes -= cls;
  if (!m.enabled) {
    JSG_HIP(hipStreamSynchronize(state().stream));
    JSG_HIP(hipFree(ptr));
    return 0;
  }
  m.idle[cls].push_back(ptr);
  m.idle_bytes += cls;
  return 0;
}
int jsgrad_hip_free_cache(void) {
  JSG_READY();
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_free_cache during graph capture");
  JSG_HIP(hipStreamSynchronize(state().stream));
  std::lock_guard<std::mutex> guard(jsg::g_mem.lock);
  return jsg::mem_release_idle();
}
int jsgrad_hip_mem_info(size_t *host_out_live_bytes, size_t *host_out_idle_bytes) {
  JSG_READY();
  std::lock_guard<std::mutex> guard(jsg::g_mem.lock);
  if (host_out_live_bytes) *host_out_live_bytes = jsg::g_mem.live_bytes;
  if (host_out_idle_bytes) *host_out_idle_bytes = jsg::g_mem.idle_bytes;
  return 0;
}
int jsgrad_hip_copyin(void *dst, const void *host_src, size_t nbytes) {
  JSG_READY();
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_copyin during graph capture");
  if (nbytes == 0) return 0;
  JSG_HIP(hipMemcpyAsync(dst, host_src, nbytes, hipMemcpyHostToDevice, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));  // the caller may reuse host_src as soon as this returns
  return 0;
}
int jsgrad_hip_copyout(void *host_dst, const void *src, size_t nbytes) {
  JSG_READY();
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_copyout during graph capture");
  if (nbytes == 0) return 0;
  JSG_HIP(hipMemcpyAsync(host_dst, src, nbytes, hipMemcpyDeviceToHost, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));
  return 0;
}
int jsgrad_hip_copy(void *dst, const void *src, size_t nbytes) {
  JSG_READY();
  if (nbytes == 0) return 0;
  JSG_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, state().stream));
  return 0;
}
int jsgrad_hip_sync(void) {
  JSG_READY();
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_sync during graph capture");
  JSG_HIP(hipStreamSynchronize(state().stream));
  {
    std::lock_guard<std::mutex> guard(jsg::g_mem.lock);
    if (jsg::g_mem.idle_bytes > jsg::g_mem.limit) return jsg::mem_release_idle();
  }
  return 0;
}

int jsgrad_hip_module_load(const void *host_image, size_t nbytes, void **host_out_module) {
  JSG_READY();
  JSG_REQUIRE(host_image && nbytes > 0, "jsgrad_hip_module_load: empty image");
  hipModule_t m;
  JSG_HIP(hipModuleLoadData(&m, host_image));
  *host_out_module = (void *)m;
  return 0;
}
int jsgrad_hip_module_unload(void *module) {
  JSG_READY();
  JSG_HIP(hipStreamSynchronize(state().stream));
  JSG_HIP(hipModuleUnload((hipModule_t)module));
  return 0;
}
int jsgrad_hip_module_get(void *module, const char *name, void **host_out_function) {
  JSG_READY();
  hipFunction_t f;
  JSG_HIP(hipModuleGetFunction(&f, (hipModule_t)module, name));
  *host_out_function = (void *)f;
  return 0;
}

int jsgrad_hip_launch(void *function, const uint32_t host_grid[3], const uint32_t host_block[3], void *const *host_bufs, int nbufs,
                      const int32_t *host_vals, int nvals, int wait, double *host_seconds) {
  JSG_READY();
  JSG_REQUIRE(function, "jsgrad_hip_launch: null function");
  JSG_REQUIRE(nbufs >= 0 && nvals >= 0 && nbufs + nvals <= 64, "jsgrad_hip_launch: %d buffers + %d vals exceeds 64 arguments", nbufs, nvals);
  for (int i = 0; i < 3; i++) JSG_REQUIRE(host_grid[i] > 0 && host_block[i] > 0, "jsgrad_hip_launch: zero grid/block dimension");
  JSG_REQUIRE((uint64_t)host_block[0] * host_block[1] * host_block[2] <= 1024, "jsgrad_hip_launch: block of %u x %u x %u exceeds 1024 threads", host_block[0], host_block[1], host_block[2]);
  // argument block laid out as the generated kernel declares it: pointers first, then int32 values
  struct {
    void *p[64];
  } packed;
  size_t off = 0;
  char *base = (char *)&packed;
  for (int i = 0; i < nbufs; i++) { memcpy(base + off, &host_bufs[i], sizeof(void *)); off += sizeof(void *); }
  for (int i = 0; i < nvals; i++) { memcpy(base + off, &host_vals[i], sizeof(int32_t)); off += sizeof(int32_t); }
  size_t size = off;
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, base, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (wait) {
    JSG_REQUIRE(!state().capturing, "jsgrad_hip_launch: wait during graph capture");
    JSG_HIP(hipEventCreate(&e0));
    JSG_HIP(hipEventCreate(&e1));
    JSG_HIP(hipEventRecord(e0, state().stream));
  }
  JSG_HIP(hipModuleLaunchKernel((hipFunction_t)function, host_grid[0], host_grid[1], host_grid[2], host_block[0], host_block[1], host_block[2], 0, state().stream, nullptr, config));
  if (wait) {
    JSG_HIP(hipEventRecord(e1, state().stream));
    JSG_HIP(hipEventSynchronize(e1));
    float ms = 0;
    JSG_HIP(hipEventElapsedTime(&ms, e0, e1));
    if (host_seconds) *host_seconds = (double)ms * 1e-3;
    JSG_HIP(hipEventDestroy(e0));
    JSG_HIP(hipEventDestroy(e1));
  }
  return 0;
}

int jsgrad_hip_event_create(void **host_out_event) {
  JSG_READY();
  hipEvent_t e;
  JSG_HIP(hipEventCreate(&e));
  *host_out_event = (void *)e;
  return 0;
}
int jsgrad_hip_event_record(void *event) {
  JSG_READY();
  JSG_HIP(hipEventRecord((hipEvent_t)event, state().stream));
  return 0;
}
int jsgrad_hip_event_elapsed_ms(void *start, void *stop, float *host_out_ms) {
  JSG_READY();
  JSG_HIP(hipEventSynchronize((hipEvent_t)stop));
  JSG_HIP(hipEventElapsedTime(host_out_ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}
int jsgrad_hip_event_destroy(void *event) {
  JSG_READY();
  JSG_HIP(hipEventDestroy((hipEvent_t)event));
  return 0;
}

int jsgrad_hip_profile(int enable) {
  JSG_READY();
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_profile during graph capture");
  jsg::ProfState &p = jsg::g_prof;
  if (enable && p.ev.empty()) {
    p.ev.resize(2 * jsg::PROF_SLOTS);
    p.kind.resize(jsg::PROF_SLOTS);
    for (auto &e : p.ev) JSG_HIP(hipEventCreate(&e));
  }
  JSG_HIP(hipStreamSynchronize(state().stream));
  p.on = enable != 0;
  p.used = 0;
  return 0;
}
int jsgrad_hip_profile_read(int kind, int *host_out_count, double *host_out_total_ms) {
  JSG_READY();
  JSG_REQUIRE(kind >= 0 && kind < jsg::PROF_KINDS, "jsgrad_hip_profile_read: kind %d out of range", kind);
  JSG_HIP(hipStreamSynchronize(state().stream));
  jsg::ProfState &p = jsg::g_prof;
  int n = 0;
  double tot = 0.0;
  for (size_t i = 0; i < p.used; i++) {
    if (p.kind[i] != kind) continue;
    float ms = 0.0f;
    JSG_HIP(hipEventElapsedTime(&ms, p.ev[2 * i], p.ev[2 * i + 1]));
    tot += ms;
    n++;
  }
  *host_out_count = n;
  *host_out_total_ms = tot;
  return 0;
}

int jsgrad_hip_graph_begin(void) {
  JSG_READY();
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_graph_begin: capture already in progress");
  JSG_HIP(hipStreamSynchronize(state().stream));
  JSG_HIP(hipStreamBeginCapture(state().stream, hipStreamCaptureModeThreadLocal));
  state().capturing = true;
  return 0;
}
int jsgrad_hip_graph_end(void **host_out_graph) {
  JSG_READY();
  JSG_REQUIRE(state().capturing, "jsgrad_hip_graph_end: no capture in progress");
  state().capturing = false;
  hipGraph_t g = nullptr;
  JSG_HIP(hipStreamEndCapture(state().stream, &g));
  hipGraphExec_t ge = nullptr;
  hipError_t e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (e != hipSuccess) return jsg::fail_hip(e, "hipGraphInstantiate");
  *host_out_graph = (void *)ge;
  return 0;
}
int jsgrad_hip_graph_launch(void *graph) {
  JSG_READY();
  JSG_REQUIRE(graph, "jsgrad_hip_graph_launch: null graph");
  JSG_HIP(hipGraphLaunch((hipGraphExec_t)graph, state().stream));
  return 0;
}
int jsgrad_hip_graph_destroy(void *graph) {
  JSG_READY();
  if (!graph) return 0;
  JSG_HIP(hipStreamSynchronize(state().stream));
  JSG_HIP(hipGraphExecDestroy((hipGraphExec_t)graph));
  return 0;
}

}  // extern "C"
