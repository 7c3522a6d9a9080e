// Small kernels around the GEMV / attention hot loops: embedding gather, stand-alone RMSNorm, greedy
// argmax, the rotary table, the int8 / NF4 quantisers and dequantisers, fills and random init.
#include "common.h"

namespace jsg {

// ---------------------------------------------------------------- fills
template <typename T> __global__ void fill_kernel(T *p, size_t n, T v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
static unsigned grid_for(size_t n, int block) {
  size_t g = (n + block - 1) / block;
  size_t cap = (size_t)state().cu_count * 16;
  return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

// ---------------------------------------------------------------- embedding gather
// Embedding.call / Int8Embedding.call (nn/index.ts:607-619, llama3.ts:71-77): the one-hot product summed
// over the vocabulary has a single non-zero term, so it is the row of the token.
template <typename AT> __global__ void embed_kernel(int kind, const void *table, const _Float16 *scale, const int32_t *st, AT *out, int dim, int vocab) {
  int tok = st[0];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < dim; i += gridDim.x * blockDim.x) {
    float v;
    if (kind == JSGRAD_W_F32) v = ((const float *)table)[(size_t)tok * dim + i];
    else if (kind == JSGRAD_W_F16) v = (float)((const _Float16 *)table)[(size_t)tok * dim + i];
    else v = (float)mul_rn16((float)((const int8_t *)table)[(size_t)tok * dim + i], (float)scale[tok]);
    out[i] = (AT)v;
  }
}

// ---------------------------------------------------------------- stand-alone RMSNorm (one row, one block)
template <typename AT> __global__ __launch_bounds__(1024) void rmsnorm_kernel(const AT *x, const AT *w, AT *y, int d, float eps, float inv_d) {
  __shared__ float red[16];
  float ss = 0.0f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) { float f = (float)x[i]; ss = fmaf(f, f, ss); }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.0f;
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) tot += red[i];
  const float r = __fsqrt_rn(__fdiv_rn(1.0f, __fadd_rn(__fmul_rn(tot, inv_d), eps)));
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = Act<AT>::rn(__fmul_rn((float)x[i], r));
    y[i] = (AT)Act<AT>::rn(__fmul_rn(v, (float)w[i]));
  }
}

// ---------------------------------------------------------------- greedy argmax
// Tensor.argmax (tensor.ts:2314-2320): the lowest index among the maxima.  ARGMAX_BLOCKS blocks each reduce a
// slice; the last one to finish (agent-scope counter) reduces the per-block winners and updates the state words.
constexpr int ARGMAX_BLOCKS = 128, ARGMAX_THREADS = 256;
__device__ float g_argmax_val[ARGMAX_BLOCKS];
__device__ int g_argmax_idx[ARGMAX_BLOCKS];
__device__ int g_argmax_count;  // zero between launches: the finishing block resets it

__device__ __forceinline__ void argmax_merge(float &best, int &bi, float ov, int oi) {
  if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
}
template <typename AT> __global__ __launch_bounds__(ARGMAX_THREADS) void argmax_kernel(const AT *x, int n, int32_t *st, int32_t *tokens_out, int tokens_cap, int advance) {
  __shared__ float vmax[ARGMAX_THREADS / 64];
  __shared__ int imax[ARGMAX_THREADS / 64];
  __shared__ int is_last;
  const int tid = threadIdx.x;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = blockIdx.x * ARGMAX_THREADS + tid; i < n; i += gridDim.x * ARGMAX_THREADS) argmax_merge(best, bi, (float)x[i], i);
  auto block_reduce = [&]() {
    for (int off = 32; off > 0; off >>= 1) argmax_merge(best, bi, __shfl_xor(best, off), __shfl_xor(bi, off));
    if ((tid & 63) == 0) { vmax[tid >> 6] = best; imax[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0)
      for (int w = 1; w < ARGMAX_THREADS / 64; w++) argmax_merge(best, bi, vmax[w], imax[w]);
  };
  block_reduce();
  if (tid == 0) {
    st_coherent(&g_argmax_val[blockIdx.x], best);
    st_coherent(&g_argmax_idx[blockIdx.x], bi);
    __builtin_amdgcn_s_waitcnt(0);  // both stores acknowledged before the counter moves
    is_last = __hip_atomic_fetch_add(&g_argmax_count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (int)gridDim.x - 1;
  }
  __syncthreads();
  if (!is_last) return;
  best = -INFINITY;
  bi = 0x7fffffff;
  if (tid < (int)gridDim.x) {
    best = ld_coherent(&g_argmax_val[tid]);
    bi = ld_coherent(&g_argmax_idx[tid]);
  }
  __syncthreads();  // vmax / imax are reused
  block_reduce();
  if (tid == 0) {
    if (bi == 0x7fffffff) bi = n;  // all-NaN input: the reference's formula yields n
    const int pos = st[1];
    if (tokens_out && pos >= 0 && pos < tokens_cap) tokens_out[pos] = bi;
    st[0] = bi;
    if (advance) st[1] = pos + 1;
    __hip_atomic_store(&g_argmax_count, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ---------------------------------------------------------------- rotary table
// precompute_freqs_cis (models/llama.ts:10-14) in float32 with the reference's polynomial sin
// (ops.ts:1577-1644), then the cast to the activation dtype (llama.ts:205).
__device__ __forceinline__ float sin_poly(float d) {
  const float c[5] = {2.6083159809786593541503e-06f, -0.0001981069071916863322258f, 0.00833307858556509017944336f, -0.166666597127914428710938f, 1.0f};
  float d2 = __fmul_rn(d, d), u = c[0];
#pragma unroll
  for (int i = 1; i < 5; i++) u = __fadd_rn(__fmul_rn(u, d2), c[i]);
  return __fmul_rn(d, u);
}
__device__ __forceinline__ float xsinf(float d) {
  float x = mask_nonfinite(d);
  float x_sign = (x != 0.0f) ? (x < 0.0f ? -1.0f : 1.0f) : 0.0f;
  float x_abs = __fmul_rn(x, x_sign);
  float result;
  if (x_abs < 30.0f) {  // Cody-Waite reduction, float32 branch
    int quad = rintk(__fmul_rn(x_abs, 0.318309886183790671537767526745028724f));
    float qf = (float)quad, r = x_abs;
    r = __fadd_rn(__fmul_rn(qf, -3.1414794921875f), r);
    r = __fadd_rn(__fmul_rn(qf, -0.00011315941810607910156f), r);
    r = __fadd_rn(__fmul_rn(qf, -1.9841872589410058936e-09f), r);
    r = __fadd_rn(__fmul_rn(qf, -1.2154201256553420762e-10f), r);
    result = __fmul_rn(sin_poly(r), (quad & 1) ? -1.0f : 1.0f);
  } else {              // Payne-Hanek reduction with 190 bits of 2/pi
    const uint32_t two_over_pi_f[7] = {0x00000000u, 0x28be60dbu, 0x9391054au, 0x7f09d5f4u, 0x7d4d3770u, 0x36d8a566u, 0x4f10e410u};
    uint32_t bits = __float_as_uint(x_abs);
    uint32_t expo = (bits >> 23) & 255u;
    float f = __uint_as_float((bits & 0x807FFFFFu) | 0x3F000000u);
    int e = (int)expo - 127 + 1;
    uint64_t ia = (uint64_t)__fmul_rn(f, 4.294967296e9f);
    uint64_t idx = ((uint64_t)(int64_t)e) >> 5;
    int es = e & 31, offset = 32 - es;
    uint32_t av[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      av[k] = 0;
      for (int count = 0; count + k < 6; count++)
        if (idx == (uint64_t)count) { av[k] = two_over_pi_f[count + k]; break; }
    }
    // shifts written as the reference does them: multiply / divide by 2^y taken through float
    auto shl = [](uint32_t v, int y) { return (uint32_t)((uint64_t)v * (uint64_t)pow2i(y)); };
    auto shr = [](uint32_t v, int y) { return (uint32_t)((uint64_t)v / (uint64_t)pow2i(y)); };
    uint32_t hi = shl(av[0], es) | shr(av[1], offset);
    uint32_t mi = shl(av[1], es) | shr(av[2], offset);
    uint32_t lo = shl(av[2], es) | shr(av[3], offset);
    uint64_t p = ((ia * (uint64_t)hi) << 32) + ia * (uint64_t)mi + ((ia * (uint64_t)lo) >> 32);
    int q = (int)(p >> 62);
    p &= 0x3fffffffffffffffull;
    float r = __fmul_rn((float)p, 3.4061215800865545e-19f);
    if (!(f < 0.5f)) { r = __fsub_rn(r, 1.5707963267948966f); q = q + 1; }
    result = __fmul_rn(sin_poly(__fadd_rn(r, (q & 1) ? 1.5707963267948966f : 0.0f)), (q & 2) ? -1.0f : 1.0f);
  }
  result = __fmul_rn(result, x_sign);
  if (!(d == d) || d == INFINITY || d == -INFINITY) result = NAN;
  return result;
}
template <typename AT> __global__ void rope_table_kernel(AT *out, int hd, int end, float inv_dim, float ln_theta) {
  const int half = hd / 2;
  const size_t n = (size_t)end * half;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
    const int pos = (int)(idx / half), i = (int)(idx % half);
    float t = __fmul_rn((float)(2 * i), inv_dim);
    float p = exp_f32(__fmul_rn(t, ln_theta));
    float fr = __fmul_rn(1.0f, __fdiv_rn(1.0f, p));
    float ang = __fmul_rn((float)pos, fr);
    out[idx * 2 + 0] = (AT)xsinf(__fsub_rn(1.5707963267948966f, ang));
    out[idx * 2 + 1] = (AT)xsinf(ang);
  }
}

// ---------------------------------------------------------------- Int8Linear.quantize (llama3.ts:37-60)
// Tensor.round (tensor.ts:3054-3057): half-to-even assembled from trunc / ceil / floor
__device__ __forceinline__ float round_half_even(float x) {
  int ti = (int)x;
  float b = __fmul_rn((float)ti, 0.5f);
  bool even = ((float)(int)b == b);
  if ((x > 0.0f) == even) { float v = __fsub_rn(x, 0.5f), t = (float)(int)v; return (v > t) ? __fadd_rn(t, 1.0f) : t; }
  float v = __fadd_rn(x, 0.5f), t = (float)(int)v;
  return (v < t) ? __fsub_rn(t, 1.0f) : t;
}
// one block per output row: scale = RN16(absmax * RN16(1/127)); code = round(RN16(w * (1/scale)))
template <typename AT> __global__ __launch_bounds__(256) void int8_quantize_kernel(const AT *w, int in_f, int8_t *codes, _Float16 *scale) {
  __shared__ float red[4];
  const size_t row = blockIdx.x;
  const AT *wr = w + row * in_f;
  float amax = 0.0f;
  for (int k = threadIdx.x; k < in_f; k += blockDim.x) amax = fmaxf(amax, fabsf(rn16((float)wr[k])));
  amax = wave_max(amax);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const _Float16 sh = (_Float16)__fmul_rn(amax, rn16((float)(1.0 / 127.0)));
  const float s = (float)sh;
  if (threadIdx.x == 0) scale[row] = sh;
  const float inv = __fdiv_rn(1.0f, s);
  for (int k = threadIdx.x; k < in_f; k += blockDim.x) {
    float t = rn16(__fmul_rn(rn16((float)wr[k]), inv));
    float r = (s == 0.0f) ? 0.0f : round_half_even(t);
    codes[row * in_f + k] = (int8_t)(int)r;
  }
}
__global__ void int8_dequant_kernel(const int8_t *codes, const _Float16 *scale, int in_f, size_t n, _Float16 *w16) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    w16[i] = mul_rn16((float)codes[i], (float)scale[i / in_f]);
}

// ---------------------------------------------------------------- NF4Linear(64) quantize / dequant (llama3.ts:91-114)
__device__ __constant__ float NF4_CODE_Q[16] = {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f, -0.28444138169288635f, -0.18477343022823334f,
                                                -0.09105003625154495f, 0.0f, 0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
                                                0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};
// one wavefront per 64-element block: lane = element
template <typename AT> __global__ __launch_bounds__(256) void nf4_quantize_kernel(const AT *w, size_t nblk, uint8_t *packed, _Float16 *scale) {
  const int lane = threadIdx.x & 63;
  const size_t blk = blockIdx.x * (size_t)(blockDim.x >> 6) + (threadIdx.x >> 6);
  if (blk >= nblk) return;
  const float x = (float)w[blk * 64 + lane];
  const float amax = wave_max(fabsf(x));
  if (lane == 0) scale[blk] = (_Float16)amax;
  const float r = __fmul_rn(x, __fdiv_rn(1.0f, amax));
  float best = INFINITY;
  int bi = 0;
#pragma unroll
  for (int j = 0; j < 16; j++) {
    float d = fabsf(__fsub_rn(r, rn16(NF4_CODE_Q[j])));
    if (d < best) { best = d; bi = j; }  // strict '<': ties keep the lowest index (argmin first-index rule)
  }
  const int other = __shfl_xor(bi, 1);
  if ((lane & 1) == 0) packed[blk * 32 + (lane >> 1)] = (uint8_t)(bi * 16 + other);  // even element in the high nibble
}
__global__ void nf4_dequant_kernel(const uint8_t *packed, const _Float16 *scale, size_t nbytes, _Float16 *w16) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < nbytes; i += (size_t)gridDim.x * blockDim.x) {
    const float s = (float)scale[i / 32];
    const uint8_t b = packed[i];
    w16[2 * i] = mul_rn16(rn16(NF4_CODE_Q[b >> 4]), s);
    w16[2 * i + 1] = mul_rn16(rn16(NF4_CODE_Q[b & 15]), s);
  }
}

// ---------------------------------------------------------------- random init
// counter-based: element i of stream `seed` is a fixed function of (seed, i); Box-Muller on two hashed uniforms
__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <typename T> __global__ void randn_kernel(T *out, size_t n, uint64_t seed, float std) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint64_t h = splitmix64(seed * 0xD1342543DE82EF95ull + i);
    float u1 = ((float)(uint32_t)(h >> 40) + 1.0f) * (1.0f / 16777217.0f);  // (0, 1]
    float u2 = (float)(uint32_t)((h >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
    float z = sqrtf(-2.0f * logf(u1)) * cospif(2.0f * u2);
    out[i] = (T)(z * std);
  }
}

}  // namespace jsg

using namespace jsg;

// ---------------------------------------------------------------- read probe
// Reads n 16-byte vectors and keeps nothing: every thread has eight streaming loads in flight, grid-stride.  The compare
// at the end keeps the loads alive (a match only writes a word nobody reads).
__global__ __launch_bounds__(256) void read_probe_kernel(const u4_t *p, size_t n, uint32_t *sink) {
  u4_t acc = {0, 0, 0, 0};
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += 8 * stride) {
    u4_t v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const size_t k = i + u * stride;
      v[u] = ldg_stream16(p + (k < n ? k : i));
    }
#pragma unroll
    for (int u = 0; u < 8; u++) acc ^= v[u];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) *sink = 1;
}

extern "C" {

int jsgrad_hip_read_probe(const void *src, size_t nbytes, void *sink) {
  JSG_READY();
  JSG_REQUIRE(src && sink && nbytes >= 16 && nbytes % 16 == 0 && (uintptr_t)src % 16 == 0, "jsgrad_hip_read_probe: bad argument");
  JSG_LAUNCH(PROF_READ, read_probe_kernel, dim3(state().cu_count * 2), dim3(256), 0, (const u4_t *)src, nbytes / 16, (uint32_t *)sink);
  return 0;
}

int jsgrad_hip_memset(void *dst, int byte, size_t nbytes) {
  JSG_READY();
  if (nbytes == 0) return 0;
  JSG_REQUIRE(dst, "jsgrad_hip_memset: null pointer");
  // a fill kernel rather than hipMemsetAsync, so that the call may sit inside a captured graph
  const uint8_t b = (uint8_t)byte;
  if (((uintptr_t)dst | nbytes) % 4 == 0) {
    uint32_t v = b * 0x01010101u;
    hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(grid_for(nbytes / 4, 256)), dim3(256), 0, state().stream, (uint32_t *)dst, nbytes / 4, v);
  } else {
    hipLaunchKernelGGL(fill_kernel<uint8_t>, dim3(grid_for(nbytes, 256)), dim3(256), 0, state().stream, (uint8_t *)dst, nbytes, b);
  }
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_fill(void *out, size_t n, int dtype, float value) {
  JSG_READY();
  if (n == 0) return 0;
  JSG_REQUIRE(out, "jsgrad_hip_fill: null pointer");
  if (dtype == JSGRAD_F16) hipLaunchKernelGGL(fill_kernel<_Float16>, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, (_Float16 *)out, n, (_Float16)value);
  else if (dtype == JSGRAD_F32) hipLaunchKernelGGL(fill_kernel<float>, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, (float *)out, n, value);
  else return fail("jsgrad_hip_fill: unknown dtype %d", dtype);
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_randn(void *out, size_t n, int dtype, uint64_t seed, float std) {
  JSG_READY();
  if (n == 0) return 0;
  JSG_REQUIRE(out, "jsgrad_hip_randn: null pointer");
  if (dtype == JSGRAD_F16) hipLaunchKernelGGL(randn_kernel<_Float16>, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, (_Float16 *)out, n, seed, std);
  else if (dtype == JSGRAD_F32) hipLaunchKernelGGL(randn_kernel<float>, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, (float *)out, n, seed, std);
  else return fail("jsgrad_hip_randn: unknown dtype %d", dtype);
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_embed(int kind, const void *table, const void *scale, const int32_t *st, void *out, int dim, int vocab, int act) {
  JSG_READY();
  JSG_REQUIRE(table && st && out && dim > 0 && vocab > 0, "jsgrad_hip_embed: bad argument");
  JSG_REQUIRE(kind == JSGRAD_W_F32 || kind == JSGRAD_W_F16 || kind == JSGRAD_W_I8, "jsgrad_hip_embed: table kind %d", kind);
  JSG_REQUIRE(kind != JSGRAD_W_I8 || scale, "jsgrad_hip_embed: int8 table needs row scales");
  dim3 grid((dim + 255) / 256), block(256);
  if (act == JSGRAD_F16) JSG_LAUNCH(PROF_EMBED, (embed_kernel<_Float16>), grid, block, 0, kind, table, (const _Float16 *)scale, st, (_Float16 *)out, dim, vocab);
  else if (act == JSGRAD_F32) JSG_LAUNCH(PROF_EMBED, (embed_kernel<float>), grid, block, 0, kind, table, (const _Float16 *)scale, st, (float *)out, dim, vocab);
  else return fail("jsgrad_hip_embed: unknown activation dtype %d", act);
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_rmsnorm(const void *x, const void *weight, void *y, int dim, float eps, int act) {
  JSG_READY();
  JSG_REQUIRE(x && weight && y && dim > 0, "jsgrad_hip_rmsnorm: bad argument");
  const float inv_d = (float)(1.0 / (double)dim);
  if (act == JSGRAD_F16) JSG_LAUNCH(PROF_RMSNORM, (rmsnorm_kernel<_Float16>), dim3(1), dim3(1024), 0, (const _Float16 *)x, (const _Float16 *)weight, (_Float16 *)y, dim, eps, inv_d);
  else if (act == JSGRAD_F32) JSG_LAUNCH(PROF_RMSNORM, (rmsnorm_kernel<float>), dim3(1), dim3(1024), 0, (const float *)x, (const float *)weight, (float *)y, dim, eps, inv_d);
  else return fail("jsgrad_hip_rmsnorm: unknown activation dtype %d", act);
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_argmax(const void *logits, int n, int32_t *st, int32_t *tokens_out, int tokens_cap, int advance, int act) {
  JSG_READY();
  JSG_REQUIRE(logits && st && n > 0, "jsgrad_hip_argmax: bad argument");
  const int nb = n >= ARGMAX_BLOCKS * ARGMAX_THREADS ? ARGMAX_BLOCKS : (n + ARGMAX_THREADS - 1) / ARGMAX_THREADS;
  if (act == JSGRAD_F16) JSG_LAUNCH(PROF_ARGMAX, (argmax_kernel<_Float16>), dim3(nb), dim3(ARGMAX_THREADS), 0, (const _Float16 *)logits, n, st, tokens_out, tokens_cap, advance);
  else if (act == JSGRAD_F32) JSG_LAUNCH(PROF_ARGMAX, (argmax_kernel<float>), dim3(nb), dim3(ARGMAX_THREADS), 0, (const float *)logits, n, st, tokens_out, tokens_cap, advance);
  else return fail("jsgrad_hip_argmax: unknown activation dtype %d", act);
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_rope_table(void *table, int head_dim, int end, float theta, int act) {
  JSG_READY();
  JSG_REQUIRE(table && head_dim > 0 && head_dim % 2 == 0 && end > 0 && theta > 0.0f, "jsgrad_hip_rope_table: bad argument");
  const float inv_dim = (float)(1.0 / (double)head_dim), ln_theta = (float)log((double)theta);
  const size_t n = (size_t)end * (head_dim / 2);
  if (act == JSGRAD_F16) hipLaunchKernelGGL(rope_table_kernel<_Float16>, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, (_Float16 *)table, head_dim, end, inv_dim, ln_theta);
  else if (act == JSGRAD_F32) hipLaunchKernelGGL(rope_table_kernel<float>, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, (float *)table, head_dim, end, inv_dim, ln_theta);
  else return fail("jsgrad_hip_rope_table: unknown activation dtype %d", act);
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_int8_quantize(const void *w, int out_f, int in_f, int8_t *codes, void *scale_f16, int act) {
  JSG_READY();
  JSG_REQUIRE(w && codes && scale_f16 && out_f > 0 && in_f > 0, "jsgrad_hip_int8_quantize: bad argument");
  if (act == JSGRAD_F16) hipLaunchKernelGGL(int8_quantize_kernel<_Float16>, dim3(out_f), dim3(256), 0, state().stream, (const _Float16 *)w, in_f, codes, (_Float16 *)scale_f16);
  else if (act == JSGRAD_F32) hipLaunchKernelGGL(int8_quantize_kernel<float>, dim3(out_f), dim3(256), 0, state().stream, (const float *)w, in_f, codes, (_Float16 *)scale_f16);
  else return fail("jsgrad_hip_int8_quantize: unknown dtype %d", act);
  JSG_LAUNCHED();
  return 0;
}
int jsgrad_hip_int8_dequant(const int8_t *codes, const void *scale_f16, int out_f, int in_f, void *w16) {
  JSG_READY();
  JSG_REQUIRE(codes && scale_f16 && w16 && out_f > 0 && in_f > 0, "jsgrad_hip_int8_dequant: bad argument");
  const size_t n = (size_t)out_f * in_f;
  hipLaunchKernelGGL(int8_dequant_kernel, dim3(grid_for(n, 256)), dim3(256), 0, state().stream, codes, (const _Float16 *)scale_f16, in_f, n, (_Float16 *)w16);
  JSG_LAUNCHED();
  return 0;
}
int jsgrad_hip_nf4_quantize(const void *w, size_t n, uint8_t *packed, void *scale_f16, int act) {
  JSG_READY();
  JSG_REQUIRE(w && packed && scale_f16 && n > 0 && n % 64 == 0, "jsgrad_hip_nf4_quantize: n must be a positive multiple of 64");
  const size_t nblk = n / 64;
  dim3 grid((unsigned)((nblk + 3) / 4)), block(256);
  if (act == JSGRAD_F16) hipLaunchKernelGGL(nf4_quantize_kernel<_Float16>, grid, block, 0, state().stream, (const _Float16 *)w, nblk, packed, (_Float16 *)scale_f16);
  else if (act == JSGRAD_F32) hipLaunchKernelGGL(nf4_quantize_kernel<float>, grid, block, 0, state().stream, (const float *)w, nblk, packed, (_Float16 *)scale_f16);
  else return fail("jsgrad_hip_nf4_quantize: unknown dtype %d", act);
  JSG_LAUNCHED();
  return 0;
}
int jsgrad_hip_nf4_dequant(const uint8_t *packed, const void *scale_f16, size_t n, void *w16) {
  JSG_READY();
  JSG_REQUIRE(packed && scale_f16 && w16 && n > 0 && n % 64 == 0, "jsgrad_hip_nf4_dequant: n must be a positive multiple of 64");
  hipLaunchKernelGGL(nf4_dequant_kernel, dim3(grid_for(n / 2, 256)), dim3(256), 0, state().stream, packed, (const _Float16 *)scale_f16, n / 2, (_Float16 *)w16);
  JSG_LAUNCHED();
  return 0;
}

}  // extern "C"
