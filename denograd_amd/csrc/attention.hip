// Decode-time grouped-query attention over the HBM-resident KV cache for gfx950.
//
// One new query position against cache rows [0, T), T = start_pos + 1: repeat_kv +
// scaled_dot_product_attention of the reference (/root/reference/jsgrad/models/llama.ts:89-95,
// /root/reference/jsgrad/tensor.ts:3920-3934).  Scores, the softmax and the P.V sum are float32; the
// exponential is the reference's polynomial exp2 (ops.ts:1650-1673).
//
// Mapping: grid (n_kv_heads, NSPLIT).  A block owns one kv head and one contiguous chunk of
// positions, and serves all n_rep query heads of that kv head from a single read of K and V
// (the GQA saving).  Inside the block a group of HD/EPL lanes covers one cache row with one 128-bit
// load per lane.  Phase 1 writes the chunk's scores to LDS and finds the chunk maximum, phase 2
// accumulates exp(s - m) and exp(s - m) * V.  Each block leaves (m, l, o) in the workspace; the last
// block of a kv head to finish (agent-scope counter) merges the chunks and writes the output row.
// The grid does not depend on T, so a captured graph replays unchanged while T grows.
#include "common.h"

namespace jsg {

constexpr int ATT_THREADS = 256;
constexpr int ATT_CHUNK_MAX = 256;  // positions per block held in LDS

struct AttnArgs {
  const void *q, *cache_k, *cache_v;
  const int32_t *st;
  void *out;
  int *counters;   // [n_kv_heads], zero before the first launch; the merging block leaves them zero
  float *partial;  // [n_kv_heads][nsplit][n_rep][HD + 2]
  int n_kv_heads, nsplit, max_context;
  float scale;     // float(1 / sqrt(head_dim)) (tensor.ts:3923 `.div(Math.sqrt(d))` = mul by the folded reciprocal)
};

template <int G> __device__ __forceinline__ float group_sum(float v) {
  static_assert(G == 8 || G == 16 || G == 32, "lane group");
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  v += dpp_f<0x141>(v);
  if (G >= 16) v += dpp_f<0x140>(v);
  if (G == 32) v += __shfl_xor(v, 16);
  return v;
}

template <typename AT, int HD, int NREP>
__global__ __launch_bounds__(ATT_THREADS) void attn_decode_kernel(AttnArgs a) {
  constexpr int EPL = 16 / sizeof(AT);  // elements per lane per 128-bit load
  constexpr int G = HD / EPL;           // lanes per cache row
  constexpr int RPI = 64 / G;           // rows per wavefront iteration
  constexpr int NW = ATT_THREADS / 64;
  const int g = blockIdx.x, split = blockIdx.y;
  const int pos = a.st[1];
  if (pos < 0 || pos >= a.max_context) return;
  const int T = pos + 1;
  const int chunk = (T + a.nsplit - 1) / a.nsplit;  // <= ATT_CHUNK_MAX, checked on the host against max_context
  const int n_active = (T + chunk - 1) / chunk;
  if (split >= n_active) return;
  const int t0 = split * chunk, t1 = min(T, t0 + chunk), CH = t1 - t0;

  __shared__ float sc[NREP][ATT_CHUNK_MAX];
  __shared__ float red[NREP][NW];
  __shared__ float o_part[NW][NREP][HD];
  __shared__ float m_sh[NREP], l_sh[NREP];
  __shared__ int is_last;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % G, grp = lane / G;
  const size_t row_stride = (size_t)a.n_kv_heads * HD;
  const AT *kbase = (const AT *)a.cache_k + (size_t)g * HD + (size_t)sub * EPL;
  const AT *vbase = (const AT *)a.cache_v + (size_t)g * HD + (size_t)sub * EPL;

  // this lane's slice of the n_rep query rows
  float qf[NREP][EPL];
#pragma unroll
  for (int j = 0; j < NREP; j++) {
    const AT *qp = (const AT *)a.q + (size_t)(g * NREP + j) * HD + sub * EPL;
#pragma unroll
    for (int e = 0; e < EPL; e++) qf[j][e] = (float)qp[e];
  }

  // ---- phase 1: scores of the chunk
  for (int t = t0 + wave * RPI + grp; t < t1; t += NW * RPI) {
    u4_t raw = *(const u4_t *)(kbase + (size_t)t * row_stride);
    float kf[EPL];
    if constexpr (sizeof(AT) == 2) {
#pragma unroll
      for (int e = 0; e < 4; e++) { h2_t h = as_h2(raw[e]); kf[2 * e] = (float)h[0]; kf[2 * e + 1] = (float)h[1]; }
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) kf[e] = __uint_as_float(raw[e]);
    }
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      float p = 0.0f;
#pragma unroll
      for (int e = 0; e < EPL; e++) p = fmaf(qf[j][e], kf[e], p);
      p = group_sum<G>(p);
      if (sub == 0) sc[j][t - t0] = __fmul_rn(p, a.scale);
    }
  }
  __syncthreads();
  // chunk maximum per head
  {
    float mx[NREP];
#pragma unroll
    for (int j = 0; j < NREP; j++) mx[j] = -INFINITY;
    for (int i = tid; i < CH; i += ATT_THREADS)
#pragma unroll
      for (int j = 0; j < NREP; j++) mx[j] = fmaxf(mx[j], sc[j][i]);
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      float w = wave_max(mx[j]);
      if (lane == 0) red[j][wave] = w;
    }
    __syncthreads();
    if (tid < NREP) {
      float w = red[tid][0];
      for (int i = 1; i < NW; i++) w = fmaxf(w, red[tid][i]);
      m_sh[tid] = w;
    }
    __syncthreads();
  }
  // scores -> exp(s - m) in place, and their sum
  {
    float ls[NREP];
#pragma unroll
    for (int j = 0; j < NREP; j++) ls[j] = 0.0f;
    for (int i = tid; i < CH; i += ATT_THREADS)
#pragma unroll
      for (int j = 0; j < NREP; j++) {
        float e = exp_f32(__fsub_rn(sc[j][i], m_sh[j]));
        sc[j][i] = e;
        ls[j] += e;
      }
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      float w = wave_sum(ls[j]);
      if (lane == 0) red[j][wave] = w;
    }
    __syncthreads();
    if (tid < NREP) {
      float w = 0.0f;
      for (int i = 0; i < NW; i++) w += red[tid][i];
      l_sh[tid] = w;
    }
    // the barrier below also orders the in-place exp writes before phase 2 reads them
  }
  __syncthreads();

  // ---- phase 2: o[j][d] = sum_t p[j][t] * V[t][d]
  float of[NREP][EPL];
#pragma unroll
  for (int j = 0; j < NREP; j++)
#pragma unroll
    for (int e = 0; e < EPL; e++) of[j][e] = 0.0f;
  for (int t = t0 + wave * RPI + grp; t < t1; t += NW * RPI) {
    u4_t raw = *(const u4_t *)(vbase + (size_t)t * row_stride);
    float vf[EPL];
    if constexpr (sizeof(AT) == 2) {
#pragma unroll
      for (int e = 0; e < 4; e++) { h2_t h = as_h2(raw[e]); vf[2 * e] = (float)h[0]; vf[2 * e + 1] = (float)h[1]; }
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) vf[e] = __uint_as_float(raw[e]);
    }
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      const float p = sc[j][t - t0];
#pragma unroll
      for (int e = 0; e < EPL; e++) of[j][e] = fmaf(p, vf[e], of[j][e]);
    }
  }
  // lanes with the same `sub` hold different rows: fold the RPI groups of the wavefront together
#pragma unroll
  for (int j = 0; j < NREP; j++)
#pragma unroll
    for (int e = 0; e < EPL; e++) {
      float v = of[j][e];
#pragma unroll
      for (int off = G; off < 64; off <<= 1) v += __shfl_xor(v, off);
      of[j][e] = v;
    }
  if (grp == 0) {
#pragma unroll
    for (int j = 0; j < NREP; j++)
#pragma unroll
      for (int e = 0; e < EPL; e++) o_part[wave][j][sub * EPL + e] = of[j][e];
  }
  __syncthreads();
  float *mine = a.partial + ((size_t)g * a.nsplit + split) * NREP * (HD + 2);
  for (int i = tid; i < NREP * HD; i += ATT_THREADS) {
    const int j = i / HD, d = i % HD;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; w++) v += o_part[w][j][d];
    st_coherent(&mine[j * (HD + 2) + d], v);
  }
  if (tid < NREP) {
    st_coherent(&mine[tid * (HD + 2) + HD], m_sh[tid]);
    st_coherent(&mine[tid * (HD + 2) + HD + 1], l_sh[tid]);
  }

  // ---- publish, and let the last chunk of this kv head merge
  __syncthreads();  // every coherent store of the block has been acknowledged
  if (tid == 0) {
    int old = __hip_atomic_fetch_add(&a.counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    is_last = (old == n_active - 1);
  }
  __syncthreads();
  if (!is_last) return;
  // merge: one wavefront per query head turns the per-chunk (m, l) into weights exp(m_s - M) and 1/L ...
  const float *base = a.partial + (size_t)g * a.nsplit * NREP * (HD + 2);
  for (int j = wave; j < NREP; j += NW) {
    float M = -INFINITY;
    for (int s = lane; s < n_active; s += 64) M = fmaxf(M, ld_coherent(base + ((size_t)s * NREP + j) * (HD + 2) + HD));
    M = wave_max(M);
    float L = 0.0f;
    for (int s = lane; s < n_active; s += 64) {
      const float *ps = base + ((size_t)s * NREP + j) * (HD + 2);
      const float w = exp_f32(ld_coherent(ps + HD) - M);
      sc[j][s] = w;  // n_active <= nsplit <= ATT_CHUNK_MAX
      L = fmaf(ld_coherent(ps + HD + 1), w, L);
    }
    L = wave_sum(L);
    if (lane == 0) l_sh[j] = 1.0f / L;  // softmax normalisation is e * (1/sum) (tensor.ts:2211-2214)
  }
  __syncthreads();
  // ... then every thread sums its output elements over the chunks; the loads are independent, so they pipeline
  for (int i = tid; i < NREP * HD; i += ATT_THREADS) {
    const int j = i / HD, d = i % HD;
    const float *po = base + (size_t)j * (HD + 2) + d;
    float O = 0.0f;
#pragma unroll 8
    for (int s = 0; s < n_active; s++) O = fmaf(ld_coherent(po + (size_t)s * NREP * (HD + 2)), sc[j][s], O);
    ((AT *)a.out)[(size_t)(g * NREP + j) * HD + d] = (AT)Act<AT>::rn(O * l_sh[j]);  // the cast of the P.V result
  }
  if (tid == 0) __hip_atomic_store(&a.counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// splits: enough that a chunk fits the LDS score buffer, and no more than the merge can index there
static int nsplit_for(int max_context) {
  int by_lds = (max_context + ATT_CHUNK_MAX - 1) / ATT_CHUNK_MAX;
  int wanted = (max_context + 31) / 32;
  if (wanted > 64) wanted = 64;
  return by_lds > wanted ? by_lds : wanted;
}

template <typename AT, int HD> static int launch_attn(const AttnArgs &a, int n_rep) {
  dim3 grid(a.n_kv_heads, a.nsplit), block(ATT_THREADS);
#define JSG_REP(N)                                                                                   \
  case N:                                                                                            \
    JSG_LAUNCH(PROF_ATTN, (attn_decode_kernel<AT, HD, N>), grid, block, 0, a);                         \
    break;
  switch (n_rep) {
    JSG_REP(1) JSG_REP(2) JSG_REP(3) JSG_REP(4) JSG_REP(8)
    default: return fail("jsgrad_hip_attn_decode: n_heads/n_kv_heads = %d is not one of 1,2,3,4,8", n_rep);
  }
#undef JSG_REP
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_attn_workspace_bytes(int n_heads, int n_kv_heads, int head_dim) {
  // counters + partials for the largest split count any max_context can ask for (256)
  (void)n_kv_heads;
  return 256 + (size_t)n_heads * 256 * (head_dim + 2) * sizeof(float);
}

int jsgrad_hip_attn_decode(const void *q, const void *cache_k, const void *cache_v, const int32_t *st, void *out, void *workspace, int n_heads,
                           int n_kv_heads, int head_dim, int max_context, int act) {
  JSG_READY();
  JSG_REQUIRE(q && cache_k && cache_v && st && out && workspace, "jsgrad_hip_attn_decode: null pointer argument");
  JSG_REQUIRE(act == JSGRAD_F16 || act == JSGRAD_F32, "jsgrad_hip_attn_decode: unknown activation dtype %d", act);
  JSG_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_kv_heads <= 64 && n_heads % n_kv_heads == 0, "jsgrad_hip_attn_decode: n_heads %d / n_kv_heads %d", n_heads, n_kv_heads);
  JSG_REQUIRE(head_dim == 64 || head_dim == 128, "jsgrad_hip_attn_decode: head_dim %d (64 and 128 are built)", head_dim);
  JSG_REQUIRE(max_context > 0 && max_context <= 256 * ATT_CHUNK_MAX, "jsgrad_hip_attn_decode: max_context %d exceeds %d", max_context, 256 * ATT_CHUNK_MAX);
  AttnArgs a;
  a.q = q; a.cache_k = cache_k; a.cache_v = cache_v; a.st = st; a.out = out;
  a.counters = (int *)workspace;
  a.partial = (float *)((char *)workspace + 256);
  a.n_kv_heads = n_kv_heads; a.nsplit = nsplit_for(max_context); a.max_context = max_context;
  a.scale = (float)(1.0 / sqrt((double)head_dim));
  const int n_rep = n_heads / n_kv_heads;
  if (act == JSGRAD_F16) return head_dim == 64 ? launch_attn<_Float16, 64>(a, n_rep) : launch_attn<_Float16, 128>(a, n_rep);
  return head_dim == 64 ? launch_attn<float, 64>(a, n_rep) : launch_attn<float, 128>(a, n_rep);
}

}  // extern "C"
