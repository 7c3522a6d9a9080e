// Shared device/host helpers for libjsgrad_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/jsgrad_hip.h"

namespace jsg {

// ---------------------------------------------------------------- host side state / errors
struct State {
  bool ready = false;
  int device = -1;
  int cu_count = 0;
  hipStream_t stream = nullptr;
  bool capturing = false;
};
State &state();
int attn_static_init(int dev);   // attention.hip: resolves the built-in attention workspace's device address (jsgrad_hip_init)
int fail(const char *fmt, ...);
int fail_hip(hipError_t e, const char *what);

// per-kernel timing with HIP events on the library stream (off unless jsgrad_hip_profile(1))
enum { PROF_EMBED = 0, PROF_RMSNORM, PROF_LINEAR, PROF_QKV_ROPE, PROF_ATTN, PROF_FFN_GATE, PROF_ARGMAX, PROF_STEP, PROF_GEMM, PROF_ATTN_PREFILL, PROF_ATTN_WO, PROF_READ, PROF_SAMPLE, PROF_KINDS };
// Event pair for the next launch of `kind`, or false when profiling is off (or capturing, or out of slots).  The pair
// is handed to hipExtLaunchKernelGGL, which stamps it with the dispatch's own begin/end times, so the elapsed time is
// the kernel alone: no marker packets, no launch latency.
bool prof_events(int kind, hipEvent_t *start, hipEvent_t *stop);

// Launch on the library stream, timed when profiling is on.
#define JSG_LAUNCH(kind, kernel, grid, block, lds, ...)                                                                  \
  do {                                                                                                                   \
    hipEvent_t ps_, pe_;                                                                                                 \
    if (jsg::prof_events(kind, &ps_, &pe_)) hipExtLaunchKernelGGL(kernel, grid, block, lds, jsg::state().stream, ps_, pe_, 0, __VA_ARGS__); \
    else hipLaunchKernelGGL(kernel, grid, block, lds, jsg::state().stream, __VA_ARGS__);                                 \
    JSG_LAUNCHED();                                                                                                      \
  } while (0)

#define JSG_HIP(call)                                   \
  do {                                                  \
    hipError_t e_ = (call);                             \
    if (e_ != hipSuccess) return jsg::fail_hip(e_, #call); \
  } while (0)
#define JSG_REQUIRE(cond, ...)               \
  do {                                       \
    if (!(cond)) return jsg::fail(__VA_ARGS__); \
  } while (0)
#define JSG_READY() JSG_REQUIRE(jsg::state().ready, "jsgrad_hip_init has not been called")
// after a kernel launch
#define JSG_LAUNCHED() JSG_HIP(hipGetLastError())

// ---------------------------------------------------------------- device helpers
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u4_t __attribute__((ext_vector_type(4)));

// Reinterpret a 32-bit word as two halves.  Always go through this by-value helper: __builtin_bit_cast applied
// directly to an element of an ext_vector (e.g. bit_cast(h2_t, vec[i])) reads element 0 whatever i is.
__device__ __forceinline__ h2_t as_h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
__device__ __forceinline__ float h2f(_Float16 h) { return (float)h; }
__device__ __forceinline__ _Float16 f2h(float f) { return (_Float16)f; }  // round-to-nearest-even
__device__ __forceinline__ float rn16(float f) { return (float)(_Float16)f; }
// RN16(a * b) with the sign of zero intact.  Written the plain way, the compiler fuses the multiply and the
// conversion into v_fma_mixlo_f16 a, b, +0, and (-0) + (+0) is +0; the empty asm keeps the product a separate value.
__device__ __forceinline__ _Float16 mul_rn16(float a, float b) {
  float p = a * b;
  asm volatile("" : "+v"(p));
  return (_Float16)p;
}

// activation dtype traits: float tensors keep float, half tensors round to fp16 at every store
template <typename AT> struct Act;
template <> struct Act<float> {
  static constexpr bool is16 = false;
  __device__ static __forceinline__ float rn(float f) { return f; }
  __device__ static __forceinline__ float ld(const float *p) { return *p; }
  __device__ static __forceinline__ void st(float *p, float f) { *p = f; }
};
template <> struct Act<_Float16> {
  static constexpr bool is16 = true;
  __device__ static __forceinline__ float rn(float f) { return rn16(f); }
  __device__ static __forceinline__ float ld(const _Float16 *p) { return (float)*p; }
  __device__ static __forceinline__ void st(_Float16 *p, float f) { *p = (_Float16)f; }
};

// Cross-block hand-off without cache-wide fences.  Data that another block will read in the same launch is written
// with agent-scope (write-through) stores and read with agent-scope loads, which are served at the device-wide
// coherence point rather than from a per-XCD L2 copy.  A block publishes by: coherent stores -> __syncthreads (which
// waits for the stores to be acknowledged) -> one relaxed agent-scope atomic on a counter.  A full release/acquire
// fence would write back and invalidate the whole L2 of the XCD once per block, which costs far more than the kernel.
// Pointers that were loaded from memory (a table of layer tensors) or built with integer arithmetic are generic to the
// compiler, which then emits flat_* instructions: those count against the LDS counter as well as the vector-memory one,
// so every LDS wait also waits for them.  Everything below the C ABI is device memory: say so.
#define JSG_GLOBAL __attribute__((address_space(1)))
template <typename T> __device__ __forceinline__ const JSG_GLOBAL T *as_global(const void *p) { return (const JSG_GLOBAL T *)(uintptr_t)p; }
template <typename T> __device__ __forceinline__ JSG_GLOBAL T *as_global_mut(void *p) { return (JSG_GLOBAL T *)(uintptr_t)p; }
// 16 bytes that are read once: streamed past the caches
__device__ __forceinline__ u4_t ldg_stream16(const void *p) { return __builtin_nontemporal_load(as_global<u4_t>(p)); }
// Streaming 16-byte loads through a buffer descriptor: base + 32-bit byte offset, and an offset of BUF_END asks for
// nothing (the load returns zeros without a memory request, and still takes its place among the outstanding loads).  A caller
// can thus issue "the load of an item that may not exist" as straight-line code instead of a branch around it.
constexpr uint32_t BUF_END = 0xFFFFFF00u;
// host side: a matrix read this way must end below BUF_END
inline bool fits_buffer_offsets(size_t rows, size_t row_elems, int bits) { return rows * row_elems * (size_t)bits / 8 < (size_t)BUF_END; }
// p, nbytes: the same for every lane of the wavefront.  nbytes is the size of what p points to: a load that reaches past it
// returns zeros without touching memory, whatever the offset arithmetic of the caller did (BUF_END is past every size).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_buffer(const void *p, uint32_t nbytes) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)hi << 32) | lo), 0, (int)__builtin_amdgcn_readfirstlane(nbytes), 0x00020000);
}
__device__ __forceinline__ u4_t buf_stream16(__amdgpu_buffer_rsrc_t rs, uint32_t off) {
  return __builtin_bit_cast(u4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, 2));   // 2: nontemporal
}
template <typename T> __device__ __forceinline__ T ldg(const T *p) { return *as_global<T>(p); }

__device__ __forceinline__ void st_coherent(float *p, float v) { __hip_atomic_store(as_global_mut<float>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_coherent(int *p, int v) { __hip_atomic_store(as_global_mut<int>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_coherent(_Float16 *p, _Float16 v) {
  __hip_atomic_store(as_global_mut<uint16_t>(p), __builtin_bit_cast(uint16_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ _Float16 ld_coherent(const _Float16 *p) {
  return __builtin_bit_cast(_Float16, __hip_atomic_load(as_global<uint16_t>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ float ld_coherent(const float *p) { return __hip_atomic_load(as_global<float>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int ld_coherent(const int *p) { return __hip_atomic_load(as_global<int>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// A block barrier that waits for the wavefront's LDS traffic only.  __syncthreads() also waits for every global load the
// wavefront has in flight (the counter that tracks loads tracks stores too, and a barrier publishes stores), which ends
// any prefetch at the barrier.  Use where only LDS contents must be agreed on.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// DPP cross-lane moves inside a 64-lane wavefront
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float readlane_f(float v, int lane) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane)); }

// sum over the 64 lanes; every lane gets the total
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror
  v += dpp_f<0x140>(v);  // row_mirror: every lane of a 16-lane row now holds the row total
  return (readlane_f(v, 0) + readlane_f(v, 16)) + (readlane_f(v, 32) + readlane_f(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));
  return fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)), fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
}
// v[l] + v[l ^ 16] and v[l] + v[l ^ 32] for every lane, in the vector ALU (v_permlane16_swap / v_permlane32_swap exchange
// the odd 16-lane rows, or the upper half, of one operand with the even rows, or the lower half, of the other; given the
// same value twice, the two results added hold the pair sum in both places).  A shuffle through the LDS crossbar does the
// same and queues behind every other LDS access of the CU.
__device__ __forceinline__ float add_xor16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float add_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// sum over aligned groups of 16 lanes (one DPP row); every lane of the group gets the group total
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  v += dpp_f<0x140>(v);
  return v;
}
// sum over aligned groups of 8 lanes
__device__ __forceinline__ float row8_sum(float v) {
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  return v;
}

// ---------------------------------------------------------------- time stamps inside kernels (diagnostic builds only)
// `make TRACE=1` compiles the stamps in: thread 0 of a traced block stores the 100 MHz device clock into a per-translation-unit
// table, which the unit's *_trace entry point copies to the host.  Row 0: block JSG_TRACE_BLOCK (default 0), row 1: whatever
// code path names it explicitly, row 2: the last block of the grid.  Normal builds contain none of this.
#ifdef JSG_TRACE
#ifndef JSG_TRACE_BLOCK
#define JSG_TRACE_BLOCK 0
#endif
static __device__ unsigned long long g_trace[4][32];   // row 3: over all blocks of the launch (JSG_LALL)
__device__ __forceinline__ int trace_row() { return blockIdx.x == JSG_TRACE_BLOCK ? 0 : (blockIdx.x == gridDim.x - 1 ? 2 : -1); }
__device__ __forceinline__ void trace_stamp(int row, int slot) {
  if (row >= 0 && threadIdx.x == 0) g_trace[row][slot] = __builtin_amdgcn_s_memrealtime();
}
#define JSG_STAMP(slot) jsg::trace_stamp(jsg::trace_row(), slot)
#define JSG_STAMP_ROW(row, slot) jsg::trace_stamp(row, slot)
// The same stamps kept in LDS and copied out when the block ends: a stamp written to memory is a store, and the next wait for
// a load waits for it too, which stretches whatever follows it.  JSG_LCLEAR() first, JSG_LFLUSH(row) last (both block-wide).
static __shared__ unsigned long long jsg_tl[32];
#ifndef JSG_TRACE_THREAD
#define JSG_TRACE_THREAD 0      // the thread whose time is kept: 0, or the first lane of another wavefront of the block
#endif
#define JSG_LSTAMP(slot) do { if (threadIdx.x == JSG_TRACE_THREAD) jsg::jsg_tl[slot] = __builtin_amdgcn_s_memrealtime(); } while (0)
#define JSG_LMAX(slot) do { if ((threadIdx.x & 63) == 0) atomicMax(&jsg::jsg_tl[slot], (unsigned long long)__builtin_amdgcn_s_memrealtime()); } while (0)   /* the last wavefront to get here */
#define JSG_LALL(slot, late) do { if (threadIdx.x == 0) { const unsigned long long t_ = __builtin_amdgcn_s_memrealtime(); atomicMax(&jsg::g_trace[3][slot], (late) ? t_ : ~t_); } } while (0)   /* latest (or, complemented, earliest) block */
#define JSG_LCLEAR() do { if (threadIdx.x < 32) jsg::jsg_tl[threadIdx.x] = 0; __syncthreads(); } while (0)
#define JSG_LFLUSH(row) do { __syncthreads(); const int row_ = (row); if (row_ >= 0 && threadIdx.x < 32) jsg::g_trace[row_][threadIdx.x] = jsg::jsg_tl[threadIdx.x]; } while (0)
#define JSG_TRACE_ENTRY(name)                                                                              \
  extern "C" int name(unsigned long long *host_out) {                                                      \
    JSG_HIP(hipStreamSynchronize(jsg::state().stream));                                                    \
    JSG_HIP(hipMemcpyFromSymbol(host_out, HIP_SYMBOL(jsg::g_trace), sizeof(jsg::g_trace)));                  \
    unsigned long long z[4][32] = {};                                                                      \
    JSG_HIP(hipMemcpyToSymbol(HIP_SYMBOL(jsg::g_trace), z, sizeof(z)));                                     \
    return 0;                                                                                              \
  }
#else
#define JSG_STAMP(slot) ((void)0)
#define JSG_STAMP_ROW(row, slot) ((void)0)
#define JSG_LSTAMP(slot) ((void)0)
#define JSG_LMAX(slot) ((void)0)
#define JSG_LALL(slot, late) ((void)0)
#define JSG_LCLEAR() ((void)0)
#define JSG_LFLUSH(row) ((void)0)
#define JSG_TRACE_ENTRY(name)
#endif

// ---------------------------------------------------------------- tagged words: data that is its own flag
// A row that blocks of one launch hand to each other: one 32-bit word per element, the fp16 value below, a version tag
// above.  A reader asks for the words and takes them once every tag is the one it expects: no flag, and the writer does
// not have to wait for its stores to be acknowledged before anything.
// The tag is the version modulo 65535, plus one (never 0: fresh or cleared memory matches nothing).  Two versions that differ
// by a multiple of 65535 share a tag, so a tag tells launches apart only among versions close to each other: rows are
// rewritten in full by every launch, and whoever makes the version jump (the host moving the decode position) clears the row.
__device__ __forceinline__ uint32_t tw_tag(int version) { return (uint32_t)version % 65535u + 1u; }
__device__ __forceinline__ void tw_store(uint32_t *p, uint32_t tag, float v) {
  const _Float16 h = (_Float16)v;
  st_coherent((int *)p, (int)((tag << 16) | (uint32_t)__builtin_bit_cast(uint16_t, h)));
}
// eight tagged words at p -> eight packed halves; ok: all eight carry `tag`
__device__ __forceinline__ u4_t tw_load8(const uint32_t *p, uint32_t tag, bool &ok) {
  const JSG_GLOBAL uint64_t *q = as_global<uint64_t>(p);
  uint64_t w[4];
#pragma unroll
  for (int i = 0; i < 4; i++) w[i] = __hip_atomic_load(q + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint64_t e = ((uint64_t)tag << 16) | ((uint64_t)tag << 48);
  const uint64_t bad = ((w[0] ^ e) | (w[1] ^ e) | (w[2] ^ e) | (w[3] ^ e)) & 0xffff0000ffff0000ull;
  ok = ok && bad == 0;
  u4_t o;
#pragma unroll
  for (int i = 0; i < 4; i++) o[i] = (uint32_t)(w[i] & 0xffffu) | ((uint32_t)(w[i] >> 32) << 16);
  return o;
}

// ---------------------------------------------------------------- jsgrad's polynomial exp2 / sin
// The reference's CPU backend has no native exp2/sin and lowers them to polynomials
// (/root/reference/jsgrad/ops.ts:1625-1676, renderer/cstyle.ts:215).  These follow the same
// operation order without FMA contraction so that results agree to the bit with a C evaluation.

__device__ __forceinline__ float pow2i(int q) { return __int_as_float((uint32_t)(q + 127) << 23); }
__device__ __forceinline__ int rintk(float d) {
  float t = __fadd_rn(d, d < 0.0f ? -0.5f : 0.5f);
  if (!(t > -2147483000.0f) || !(t < 2147483000.0f)) return (int)0x80000000;
  return (int)t;
}
__device__ __forceinline__ float mask_nonfinite(float d) { return (d != INFINITY) ? ((d != d) ? 0.0f : ((d != -INFINITY) ? d : 0.0f)) : 0.0f; }

// xexp2 for float32 (ops.ts:1650-1673)
__device__ __forceinline__ float xexp2f(float d) {
  const float c[7] = {0.1535920892e-3f, 0.1339262701e-2f, 0.9618384764e-2f, 0.5550347269e-1f, 0.2402264476e+0f, 0.6931471825e+0f, 1.0f};
  float x = mask_nonfinite(d);
  int q = rintk(x);
  float s = __fsub_rn(x, (float)q);
  float u = c[0];
#pragma unroll
  for (int i = 1; i < 7; i++) u = __fadd_rn(__fmul_rn(u, s), c[i]);
  u = __fmul_rn(__fmul_rn(u, pow2i(q >> 1)), pow2i(q - (q >> 1)));
  if (d >= 128.0f) u = INFINITY;
  if (d < -150.0f) u = 0.0f;
  if (d != d) u = NAN;
  return u;
}
// xexp2 for half tensors: fp16-rounded coefficients, float Horner chain, bounds [23, -22].
// The same values as the float version's sequence with fewer instructions: whatever d lies outside [-22, 23) or is not a
// number gets its result from the three tests at the end, so the non-finite mask and the range test of the rounding are
// not needed in front (the conversion to int saturates, nothing traps, q is clamped before it is used); inside the bounds
// u * 2^q is a normal number, so one exact scaling by 2^q equals the two exact multiplications by 2^(q>>1) and 2^(q-(q>>1)).
__device__ __forceinline__ float xexp2h(float d) {
  const float c[7] = {0.1535920892e-3f, 0.1339262701e-2f, 0.9618384764e-2f, 0.5550347269e-1f, 0.2402264476e+0f, 0.6931471825e+0f, 1.0f};
  int q = (int)__fadd_rn(d, d < 0.0f ? -0.5f : 0.5f);
  float s = __fsub_rn(d, (float)q);
  float u = rn16(c[0]);
#pragma unroll
  for (int i = 1; i < 7; i++) u = __fadd_rn(__fmul_rn(u, s), rn16(c[i]));
  q = q > 60 ? 60 : (q < -60 ? -60 : q);
  u = __builtin_amdgcn_ldexpf(u, q);
  if (d >= 23.0f) u = INFINITY;
  if (d < -22.0f) u = 0.0f;
  if (d != d) u = NAN;
  return u;
}
// Tensor.exp on float tensors (tensor.ts:147-154)
__device__ __forceinline__ float exp_f32(float x) { return xexp2f(__fmul_rn(x, 1.4426950408889634f)); }

// NF4 code book (llama3.ts:80-81); the CODE tensor is float16, so every literal is rounded to fp16 first.
// NF4 code n as fp16 bits, selected from literals by the four bits of n: a table in memory would cost its readers a memory
// round trip per entry, and the look-up tables are built at the head of a launch, in front of everything else.
#define JSG_H16(x) ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)(x)))
__device__ __forceinline__ uint32_t nf4_code_bits(int n) {
  const bool b0 = n & 1, b1 = n & 2, b2 = n & 4, b3 = n & 8;
  const uint32_t q0 = b0 ? JSG_H16(-0.6961928009986877f) : JSG_H16(-1.0f), q1 = b0 ? JSG_H16(-0.39491748809814453f) : JSG_H16(-0.5250730514526367f);
  const uint32_t q2 = b0 ? JSG_H16(-0.18477343022823334f) : JSG_H16(-0.28444138169288635f), q3 = b0 ? JSG_H16(0.0f) : JSG_H16(-0.09105003625154495f);
  const uint32_t q4 = b0 ? JSG_H16(0.16093020141124725f) : JSG_H16(0.07958029955625534f), q5 = b0 ? JSG_H16(0.33791524171829224f) : JSG_H16(0.24611230194568634f);
  const uint32_t q6 = b0 ? JSG_H16(0.5626170039176941f) : JSG_H16(0.44070982933044434f), q7 = b0 ? JSG_H16(1.0f) : JSG_H16(0.7229568362236023f);
  const uint32_t p0 = b1 ? q1 : q0, p1 = b1 ? q3 : q2, p2 = b1 ? q5 : q4, p3 = b1 ? q7 : q6;
  const uint32_t o0 = b2 ? p1 : p0, o1 = b2 ? p3 : p2;
  return b3 ? o1 : o0;
}

// silu(a) = a * 1/(1 + exp2(a * -1/ln2)) (tensor.ts:2909-2911, 3210-3226) in the activation dtype's arithmetic
template <typename AT> __device__ __forceinline__ float silu_act(float a);
template <> __device__ __forceinline__ float silu_act<float>(float a) {
  float u = xexp2f(__fmul_rn(a, -1.4426950408889634f));
  return __fmul_rn(a, __fdiv_rn(1.0f, __fadd_rn(1.0f, u)));
}
// 1 / d for d = 1 + exp2(...) >= 1 (or +inf, or NaN): no scaling for tiny or huge operands is needed, so the division is the
// hardware reciprocal refined the way the full IEEE sequence does it (two residual steps), without that sequence's range
// handling.  Same bits as __fdiv_rn(1, d) for every input the fp16 silu can produce (checked exhaustively in the tests).
__device__ __forceinline__ float recip_ge1(float d) {
  float r = __builtin_amdgcn_rcpf(d);
  float e = __builtin_fmaf(-d, r, 1.0f);
  r = __builtin_fmaf(e, r, r);
  e = __builtin_fmaf(-d, r, 1.0f);
  r = __builtin_fmaf(e, r, r);
  return d == INFINITY ? 0.0f : r;
}
template <> __device__ __forceinline__ float silu_act<_Float16>(float a) {
  float u = xexp2h(rn16(__fmul_rn(a, rn16(-1.4426950408889634f))));
  return __fmul_rn(a, recip_ge1(__fadd_rn(1.0f, u)));
}

}  // namespace jsg
