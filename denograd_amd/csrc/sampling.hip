// The sampler of the reference on the device: `sample` (/root/reference/jsgrad/models/llama.ts:131-185) with
// `Tensor.multinomial` (/root/reference/jsgrad/tensor.ts:1164-1172) and the one float32 of `Tensor.rand` it draws
// (tensor.ts:798-843, Threefry-2x32-20 of ops.ts:1874-1890).
//
// float32 throughout; a / b is a * (1 / b) (tensor.ts:3576-3579); exp is the polynomial exp2 (common.h).  The running sum
// is the reference's two-level scheme (tensor.ts:2629-2641): the vector padded on the LEFT to a multiple of 256,
// sequential sums inside chunks of 256, plus the sequential sum of the totals of the chunks before.  "Sequential" is meant
// literally - ((x0 + x1) + x2) + ... - so a chunk is one block whose thread j adds up elements 0..j of the chunk out of
// LDS, and the sums over chunk totals are loops of one thread.  The plain sums (softmax denominator, the mass left after
// top-k) use the same chunks: sequential inside, then sequential over the chunk sums.  With that the token is a function
// of (logits, parameters, random word) alone: any evaluation that adds in this order gets the same bits.
//
// Four launches for the whole-vocabulary draw (chunk c of the padded vector = block c):
//   prep  y = (logit - penalty, NaN -> -inf) * (1/temp); chunk maxima
//   exp   e = exp(y - max); chunk sums
//   cdf   t = e * (1 / sum); running sums inside the chunk; chunk totals
//   pick  (one block) cdf = (running sum + totals before) * (1 / grand total); count of cdf entries <= u, found in the one
//         chunk where the cdf passes u; writes the token, advances the position, the alpha counter and the random counter
// With top_k > 0 the last launch is one block instead: k times (largest value, lowest index among equals, zero it), the
// top-p mask over those k, and the draw among them.
#include "common.h"

namespace jsg {

constexpr int SM_CHUNK = 256;     // the reference's SPLIT
constexpr int SM_MAXK = 256;      // top_k values the one-block kernel holds in LDS (one-level running sum: k <= 512)
constexpr int SM_TOPK_THREADS = 1024;
constexpr int SM_MAXCH = 4096;    // chunks a block stages in LDS to add them up: vocabularies up to 1 Mi entries

struct SampleArgs {
  const void *logits;
  int n, pad, nch;                // elements, zeros in front of them, chunks of 256
  float inv_temp, af, ap, one_minus_p;
  int use_alpha, k;
  int32_t *alpha;                 // [n] or null
  uint32_t *rng;                  // {key0, key1, counter}
  int32_t *st, *tokens_out;
  int tokens_cap, advance;
  float *y, *prefix, *cmax, *csum, *ctot;   // workspace: [nch*256] x 2, [nch] x 3
};

__device__ __forceinline__ void threefry2x32(uint32_t &x0, uint32_t &x1, uint32_t k0, uint32_t k1) {
  const uint32_t ks[3] = {k1, k0 ^ k1 ^ 0x1BD11BDAu, k0};
  const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
  x0 += ks[2];
  x1 += ks[0];
#pragma unroll
  for (int i = 0; i < 5; i++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      x0 += x1;
      x1 = x0 ^ ((x1 << rot[i % 2][r]) | (x1 >> (32 - rot[i % 2][r])));
    }
    x0 += ks[i % 3];
    x1 += ks[(i + 1) % 3] + (uint32_t)(i + 1);
  }
}
// Tensor.rand([1, 1, 1]) with the device counter at rng[2]
__device__ __forceinline__ float sample_uniform(const uint32_t *rng) {
  uint32_t x0 = rng[2], x1 = rng[2] + 1u;
  threefry2x32(x0, x1, rng[0], rng[1]);
  return __uint_as_float((x0 >> 9) | 0x3F800000u) - 1.0f;
}

template <typename AT> __global__ __launch_bounds__(SM_CHUNK) void sample_prep_kernel(SampleArgs a) {
  __shared__ float red[SM_CHUNK / 64];
  const int slot = blockIdx.x * SM_CHUNK + threadIdx.x, i = slot - a.pad;
  float y = -INFINITY;                       // the padding: exp gives 0, as the reference's zero padding of the weights
  if (i >= 0 && i < a.n) {
    float v = (float)((const AT *)a.logits)[i];
    if (a.use_alpha) {
      const int c = a.alpha[i];
      const float pen = (float)c * a.af + (c >= 0 ? 1.0f : 0.0f) * a.ap;     // llama.ts:147
      v = v - pen;
    }
    if (v != v) v = -INFINITY;               // llama.ts:151
    y = v * a.inv_temp;
  }
  a.y[slot] = y;
  const float m = wave_max(y);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) a.cmax[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// max over the chunk maxima (exact, any order), by every block for itself
__device__ __forceinline__ float sample_global_max(const SampleArgs &a, float *red) {
  float m = -INFINITY;
  for (int c = threadIdx.x; c < a.nch; c += blockDim.x) m = fmaxf(m, a.cmax[c]);
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  float r = red[0];
  for (int w = 1; w < (int)(blockDim.x >> 6); w++) r = fmaxf(r, red[w]);
  __syncthreads();
  return r;
}
// ((v[0] + v[1]) + v[2]) + ... over the n chunk values at v: every thread of the block copies its share to LDS (one round
// trip instead of n dependent ones), thread 0 adds them up in order.  Returns the sum to thread 0 (others get garbage);
// `mark`: also the sum of the first `mark` values.  Contains a barrier.
__device__ __forceinline__ float sample_seq_sum(const float *v, int n, int mark, float &before, float *stage) {
  for (int c = threadIdx.x; c < n; c += blockDim.x) stage[c] = v[c];
  __syncthreads();
  float s = 0.0f;
  before = 0.0f;
  if (threadIdx.x == 0) {
    int c = 0;
    for (; c + 4 <= n; c += 4) {           // four values per LDS read; only the additions depend on each other
      const f4_t t = *(const f4_t *)&stage[c];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (c + e == mark) before = s;
        s = s + t[e];
      }
    }
    for (; c < n; c++) {
      if (c == mark) before = s;
      s = s + stage[c];
    }
    if (mark >= n) before = s;
  }
  return s;
}

__global__ __launch_bounds__(SM_CHUNK) void sample_exp_kernel(SampleArgs a) {
  __shared__ float red[SM_CHUNK / 64];
  __shared__ __align__(16) float e_sh[SM_CHUNK];
  const int slot = blockIdx.x * SM_CHUNK + threadIdx.x;
  const float M = sample_global_max(a, red);
  const float e = exp_f32(a.y[slot] - M);
  a.y[slot] = e;
  e_sh[threadIdx.x] = e;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (int l = 0; l < SM_CHUNK; l += 4) {
      const f4_t t = *(const f4_t *)&e_sh[l];
      s = s + t[0]; s = s + t[1]; s = s + t[2]; s = s + t[3];
    }
    a.csum[blockIdx.x] = s;
  }
}

// WITH_PREFIX: also the running sums inside the chunk and the chunk total (the whole-vocabulary draw); without, only t
template <bool WITH_PREFIX> __global__ __launch_bounds__(SM_CHUNK) void sample_cdf_kernel(SampleArgs a) {
  __shared__ float t_sh[SM_CHUNK];
  __shared__ __align__(16) float stage[SM_MAXCH];
  __shared__ float rs_sh;
  const int slot = blockIdx.x * SM_CHUNK + threadIdx.x;
  float unused;
  const float total_e = sample_seq_sum(a.csum, a.nch, -1, unused, stage);
  if (threadIdx.x == 0) rs_sh = 1.0f / total_e;
  __syncthreads();
  const float t = a.y[slot] * rs_sh;
  a.y[slot] = t;
  if constexpr (WITH_PREFIX) {
    t_sh[threadIdx.x] = t;
    __syncthreads();
    float s = 0.0f;
    for (int l = 0; l <= (int)threadIdx.x; l++) s = s + t_sh[l];
    a.prefix[slot] = s;
    if (threadIdx.x == SM_CHUNK - 1) a.ctot[blockIdx.x] = s;
  }
}

// what the block that ends a draw writes
__device__ __forceinline__ void sample_finish(const SampleArgs &a, int token) {
  const int pos = a.st[1];
  if (a.tokens_out && pos >= 0 && pos < a.tokens_cap) a.tokens_out[pos] = token;
  a.st[0] = token;
  if (a.advance) a.st[1] = pos + 1;
  if (a.use_alpha && token >= 0 && token < a.n) a.alpha[token] += 1;     // llama.ts:183
  a.rng[2] = a.rng[2] + 1u;                                              // the next Tensor.rand of one number (tensor.ts:819)
}

// One block.  The cdf never decreases (running sums of non-negative weights, float addition and the multiplication by a
// positive number are monotone), and the last cdf entry of a chunk is (chunk total + totals before) * inv, which the chunk
// totals alone give.  So: thread 0 turns the totals into the totals BEFORE each chunk and the grand total; the threads
// look for the first chunk whose last entry is above u; only that chunk's running sums are read and compared.  Every
// chunk before it counts whole, every chunk after it not at all - the same count as comparing all entries.
__global__ __launch_bounds__(SM_CHUNK) void sample_pick_kernel(SampleArgs a) {
  __shared__ __align__(16) float tot_sh[SM_MAXCH], base_sh[SM_MAXCH];
  __shared__ float inv_sh, u_sh;
  __shared__ int red_sh[SM_CHUNK / 64];
  const int tid = threadIdx.x;
  for (int c = tid; c < a.nch; c += SM_CHUNK) tot_sh[c] = a.ctot[c];
  __syncthreads();
  if (tid == 0) {
    // reads of one array, writes to another: only the additions depend on each other
    float s = 0.0f;
    int c = 0;
    for (; c + 4 <= a.nch; c += 4) {
      const f4_t t = *(const f4_t *)&tot_sh[c];
      f4_t b;
      b[0] = s; s = s + t[0];
      b[1] = s; s = s + t[1];
      b[2] = s; s = s + t[2];
      b[3] = s; s = s + t[3];
      *(f4_t *)&base_sh[c] = b;
    }
    for (; c < a.nch; c++) { base_sh[c] = s; s = s + tot_sh[c]; }
    inv_sh = 1.0f / s;
    u_sh = sample_uniform(a.rng);
  }
  __syncthreads();
  const float inv = inv_sh, u = u_sh;
  int first = a.nch;                                    // first chunk that is not counted whole
  for (int c = tid; c < a.nch; c += SM_CHUNK)
    if (!(u >= (tot_sh[c] + base_sh[c]) * inv)) { first = c; break; }
  for (int off = 32; off > 0; off >>= 1) first = min(first, __shfl_xor(first, off));
  if ((tid & 63) == 0) red_sh[tid >> 6] = first;
  __syncthreads();
  first = min(min(red_sh[0], red_sh[1]), min(red_sh[2], red_sh[3]));
  __syncthreads();
  int token = a.n;                                      // u >= every entry (possible when the last entry rounds below 1)
  if (first < a.nch) {
    const int slot = first * SM_CHUNK + tid, i = slot - a.pad;
    const bool hit = i >= 0 && i < a.n && u >= (a.prefix[slot] + base_sh[first]) * inv;
    const int c = __popcll(__ballot(hit));
    if ((tid & 63) == 0) red_sh[tid >> 6] = c;
    __syncthreads();
    token = (first > 0 ? first * SM_CHUNK - a.pad : 0) + red_sh[0] + red_sh[1] + red_sh[2] + red_sh[3];
  }
  if (tid == 0) sample_finish(a, token);
}

// top_k > 0: one block over t (in a.y, the padding holds zeros)
__global__ __launch_bounds__(SM_TOPK_THREADS) void sample_topk_kernel(SampleArgs a) {
  __shared__ float out[SM_MAXK];
  __shared__ int idx[SM_MAXK];
  __shared__ float wv[SM_TOPK_THREADS / 64];
  __shared__ int wi[SM_TOPK_THREADS / 64];
  const int tid = threadIdx.x, total = a.nch * SM_CHUNK;
  for (int it = 0; it < a.k; it++) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int s = a.pad + tid; s < total; s += SM_TOPK_THREADS) {
      const float v = __hip_atomic_load(a.y + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // the element zeroed a round ago must be seen
      if (v > best || (v == best && s < bi)) { best = v; bi = s; }
    }
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off);
      const int oi = __shfl_xor(bi, off);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((tid & 63) == 0) { wv[tid >> 6] = best; wi[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < SM_TOPK_THREADS / 64; w++)
        if (wv[w] > best || (wv[w] == best && wi[w] < bi)) { best = wv[w]; bi = wi[w]; }
      out[it] = best;
      idx[it] = bi - a.pad;
      __hip_atomic_store(a.y + bi, 0.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);           // llama.ts:169
      __builtin_amdgcn_s_waitcnt(0);
    }
    __syncthreads();
  }
  // the mass that is left: sequential inside chunks (one thread per chunk), then sequential over the chunk sums
  for (int c = tid; c < a.nch; c += SM_TOPK_THREADS) {
    float s = 0.0f;
    for (int l = 0; l < SM_CHUNK; l++) s = s + __hip_atomic_load(a.y + c * SM_CHUNK + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    a.csum[c] = s;
  }
  __threadfence();
  __syncthreads();
  if (tid != 0) return;
  float rest = 0.0f;
  for (int c = 0; c < a.nch; c++) rest = rest + __hip_atomic_load(a.csum + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // approximate top p (llama.ts:172-176): an entry stays when the mass from it downwards, plus the rest, reaches 1 - p
  float run = 0.0f;
  for (int j = a.k - 1; j >= 0; j--) {
    run = run + out[j];
    const bool keep = (run + rest) >= a.one_minus_p;
    if (!keep) { out[j] = 0.0f; idx[j] = 0; }
  }
  // the draw among the k (one-level running sum, k <= 512)
  float kept = 0.0f;
  for (int j = 0; j < a.k; j++) kept = kept + out[j];
  const float inv = 1.0f / kept, u = sample_uniform(a.rng);
  float cw = 0.0f;
  int count = 0;
  for (int j = 0; j < a.k; j++) {
    cw = cw + out[j];
    if (u >= cw * inv) count++;
  }
  sample_finish(a, count < a.k ? idx[count] : 0);   // an index past the end gathers nothing (tensor.ts:1495-1519)
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_sample_workspace_bytes(int n) {
  if (n <= 0) return 0;
  const size_t nch = ((size_t)n + SM_CHUNK - 1) / SM_CHUNK;
  return 256 + (2 * nch * SM_CHUNK + 3 * ((nch + 63) / 64 * 64)) * sizeof(float);
}

int jsgrad_hip_sample(const void *logits, int n, int act, double temp, int k, double p, double af, double ap, int32_t *alpha_counter, uint32_t *rng,
                      int32_t *st, int32_t *tokens_out, int tokens_cap, int advance, void *workspace) {
  JSG_READY();
  JSG_REQUIRE(logits && st && n > 0, "jsgrad_hip_sample: bad argument");
  JSG_REQUIRE(act == JSGRAD_F16 || act == JSGRAD_F32, "jsgrad_hip_sample: unknown activation dtype %d", act);
  JSG_REQUIRE(p >= 0.0 && p <= 1.0, "p must be between 0 and 1");
  JSG_REQUIRE(k >= 0 && k <= n, "k must be between 0 and numel");
  if (temp < 1e-6) return jsgrad_hip_argmax(logits, n, st, tokens_out, tokens_cap, advance, act);   // llama.ts:138
  JSG_REQUIRE(k <= SM_MAXK, "jsgrad_hip_sample: top_k %d exceeds the %d this build holds", k, SM_MAXK);
  JSG_REQUIRE(n > 2 * SM_CHUNK && n <= SM_MAXCH * SM_CHUNK, "jsgrad_hip_sample: %d logits (more than %d and at most %d are built: the two-level running sum)", n, 2 * SM_CHUNK, SM_MAXCH * SM_CHUNK);
  JSG_REQUIRE(rng && workspace, "jsgrad_hip_sample: sampling needs the random state and a workspace");
  const bool alpha = af != 0.0 || ap != 0.0;
  JSG_REQUIRE(!alpha || alpha_counter, "jsgrad_hip_sample: alpha penalties need the counter");
  SampleArgs a = {};
  a.logits = logits; a.n = n;
  a.nch = (n + SM_CHUNK - 1) / SM_CHUNK;
  a.pad = a.nch * SM_CHUNK - n;
  a.inv_temp = (float)(1.0 / temp);          // the constant 1/temp folded in double, then a float (ops.ts:1322)
  a.af = (float)af; a.ap = (float)ap; a.one_minus_p = (float)(1.0 - p);
  a.use_alpha = alpha; a.k = k; a.alpha = alpha_counter; a.rng = rng;
  a.st = st; a.tokens_out = tokens_out; a.tokens_cap = tokens_cap; a.advance = advance;
  char *ws = (char *)workspace;
  a.y = (float *)(ws + 256);
  a.prefix = a.y + (size_t)a.nch * SM_CHUNK;
  const size_t nchp = ((size_t)a.nch + 63) / 64 * 64;
  a.cmax = a.prefix + (size_t)a.nch * SM_CHUNK;
  a.csum = a.cmax + nchp;
  a.ctot = a.csum + nchp;
  const dim3 grid(a.nch), block(SM_CHUNK);
  if (act == JSGRAD_F16) JSG_LAUNCH(PROF_SAMPLE, sample_prep_kernel<_Float16>, grid, block, 0, a);
  else JSG_LAUNCH(PROF_SAMPLE, sample_prep_kernel<float>, grid, block, 0, a);
  JSG_LAUNCH(PROF_SAMPLE, sample_exp_kernel, grid, block, 0, a);
  if (k == 0) {
    JSG_LAUNCH(PROF_SAMPLE, sample_cdf_kernel<true>, grid, block, 0, a);
    JSG_LAUNCH(PROF_SAMPLE, sample_pick_kernel, dim3(1), dim3(SM_CHUNK), 0, a);
  } else {
    JSG_LAUNCH(PROF_SAMPLE, sample_cdf_kernel<false>, grid, block, 0, a);
    JSG_LAUNCH(PROF_SAMPLE, sample_topk_kernel, dim3(1), dim3(SM_TOPK_THREADS), 0, a);
  }
  return 0;
}

}  // extern "C"
