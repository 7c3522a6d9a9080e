// Several-position kernels for fp16 activations: causal grouped-query attention on the matrix cores for S > 1 new
// positions per sequence (batched prefill), and the row-wise companions of the one-row kernels (embedding gather,
// RMSNorm, greedy argmax) for [rows][...] inputs.
//
// Reference semantics: Attention.call with a mask (/root/reference/jsgrad/models/llama.ts:61-97, mask :208 =
// triu(start_pos + 1) of -inf), repeat_kv :34-39, scaled_dot_product_attention /root/reference/jsgrad/tensor.ts:3920-3934
// (float32 scores and softmax, probabilities cast to fp16, float32 P.V sum, fp16 out).
#include "common.h"

namespace jsg {

typedef float f16_t __attribute__((ext_vector_type(16)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- causal attention, S new positions
//
// Block = 4 wavefronts = 128 query rows of one head of one sequence; a wavefront owns 32 rows.  Keys are walked in tiles
// of 64.  Scores are computed TRANSPOSED, S^T = K . Q^T (A operand = K rows from LDS, B operand = the lane's query row
// held in registers), so that a lane holds 32 scores of ONE query row per tile: the online-softmax statistics are
// lane-local (plus one exchange between the two lane halves), and the fp16 probabilities are already laid out as the
// B operand of O^T = V^T . P^T.  The k-slot order of an MFMA operand is free as long as both operands agree; V^T
// fragments are read from a transposed LDS tile in the order the score accumulators come out.
// Two blocks per CU: at head_dim 128 the kernel wants a few registers more than half of a SIMD's file, and a second block
// that computes while this one waits at its barriers is worth more than those registers.
constexpr int PF_THREADS = 256, PF_QROWS = 128, PF_KEYS = 64;

struct PrefillAttnArgs {
  const _Float16 *q;                 // [B*S][H*HD]
  const _Float16 *cache_k, *cache_v; // [B][max_context][KV][HD]
  _Float16 *out;                     // [B*S][H*HD]
  int S, start_pos, n_heads, n_kv_heads, max_context;
  float scale_log2;                  // float(1/sqrt(HD)) * log2(e)
};

template <int HD> __global__ __launch_bounds__(PF_THREADS, 2) void attn_prefill_kernel(PrefillAttnArgs a) {
  constexpr int KS = HD + 8;          // K tile row stride in halves
  constexpr int VS = PF_KEYS + 8;     // V^T tile row stride in halves
  constexpr int KC = HD / 8;          // 16-byte chunks per cache row
  constexpr int K_LOADS = PF_KEYS * KC / PF_THREADS;
  constexpr int V_PASSES = KC / 8;    // a pass covers 8 chunks x 32 key pairs
  __shared__ __align__(16) _Float16 Ks[PF_KEYS * KS];
  __shared__ __align__(16) _Float16 Vt[HD * VS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, lg = lane >> 5;
  // the block with the most keys (the last query tile) is scheduled first
  const int qt = gridDim.x - 1 - blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int g = h / (a.n_heads / a.n_kv_heads);
  const int q0 = qt * PF_QROWS, qw0 = q0 + wave * 32;
  const int row_hi = min(q0 + PF_QROWS, a.S) - 1;            // last valid query row of the block
  const int n_tiles = (a.start_pos + row_hi) / PF_KEYS + 1;
  int qrow = qw0 + l32;
  const bool q_valid = qrow < a.S;
  if (!q_valid) qrow = a.S - 1;
  const int qpos = a.start_pos + qrow;                       // keys <= qpos are visible

  // query row fragments: chunk c covers features [16c, 16c+16), the lane half picks 8 of them
  h8_t qf[HD / 16];
  {
    const _Float16 *qp = a.q + ((size_t)b * a.S + qrow) * a.n_heads * HD + (size_t)h * HD + lg * 8;
#pragma unroll
    for (int c = 0; c < HD / 16; c++) qf[c] = *(const h8_t *)(qp + c * 16);
  }

  const size_t row_stride = (size_t)a.n_kv_heads * HD;
  const _Float16 *kbase = a.cache_k + (size_t)b * a.max_context * row_stride + (size_t)g * HD;
  const _Float16 *vbase = a.cache_v + (size_t)b * a.max_context * row_stride + (size_t)g * HD;
  const int last_row = a.max_context - 1;

  u4_t gk[K_LOADS], gv[V_PASSES][2];
  auto issue = [&](int t) {
    const int k0 = t * PF_KEYS;
#pragma unroll
    for (int i = 0; i < K_LOADS; i++) {
      const int idx = tid + i * PF_THREADS, key = min(k0 + idx / KC, last_row), c = idx % KC;
      gk[i] = *(const u4_t *)(kbase + (size_t)key * row_stride + c * 8);
    }
    const int kp = tid & 31;
#pragma unroll
    for (int p = 0; p < V_PASSES; p++) {
      const int c = (tid >> 5) + p * 8;
      gv[p][0] = *(const u4_t *)(vbase + (size_t)min(k0 + 2 * kp, last_row) * row_stride + c * 8);
      gv[p][1] = *(const u4_t *)(vbase + (size_t)min(k0 + 2 * kp + 1, last_row) * row_stride + c * 8);
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < K_LOADS; i++) {
      const int idx = tid + i * PF_THREADS;
      *(u4_t *)&Ks[(idx / KC) * KS + (idx % KC) * 8] = gk[i];
    }
    const int kp = tid & 31;
#pragma unroll
    for (int p = 0; p < V_PASSES; p++) {
      const int c = (tid >> 5) + p * 8;
      const uint32_t e[4] = {gv[p][0].x, gv[p][0].y, gv[p][0].z, gv[p][0].w}, o[4] = {gv[p][1].x, gv[p][1].y, gv[p][1].z, gv[p][1].w};
#pragma unroll
      for (int w = 0; w < 4; w++) {
        // features 2w, 2w+1 of the chunk for the even key (e) and the odd key (o): pack (even key, odd key) per feature
        const uint32_t f0 = __builtin_amdgcn_perm(o[w], e[w], 0x05040100u);   // {e.lo16, o.lo16}
        const uint32_t f1 = __builtin_amdgcn_perm(o[w], e[w], 0x07060302u);   // {e.hi16, o.hi16}
        *(uint32_t *)&Vt[(c * 8 + 2 * w) * VS + 2 * kp] = f0;
        *(uint32_t *)&Vt[(c * 8 + 2 * w + 1) * VS + 2 * kp] = f1;
      }
    }
  };

  f16_t o_acc[HD / 32];
#pragma unroll
  for (int t = 0; t < HD / 32; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) o_acc[t][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  issue(0);
  for (int t = 0; t < n_tiles; t++) {
    __syncthreads();           // everyone is done with the previous tile
    commit();
    __syncthreads();
    if (t + 1 < n_tiles) issue(t + 1);
    const int k0 = t * PF_KEYS;
    if (k0 > a.start_pos + min(qw0 + 31, a.S - 1)) continue;   // every key of the tile is masked for this wavefront (uniform)

    // S^T tile: 64 keys x 32 query rows
    f16_t s[2];
#pragma unroll
    for (int tk = 0; tk < 2; tk++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[tk][r] = 0.0f;
#pragma unroll
      for (int c = 0; c < HD / 16; c++) {
        const h8_t kf = *(const h8_t *)&Ks[(tk * 32 + l32) * KS + c * 16 + lg * 8];
        s[tk] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[c], s[tk], 0, 0, 0);
      }
    }
    // accumulator r of s[tk] is key k0 + tk*32 + 8*(r/4) + 4*lg + r%4 for query row l32.  Only a tile that reaches past
    // the first query row of the wavefront has masked keys (uniform test); the scale is positive, so the maximum is
    // taken over the raw scores and the scale folded into the exponent: exp2(s * scale - max * scale).
    if (k0 + PF_KEYS - 1 > a.start_pos + qw0) {
#pragma unroll
      for (int tk = 0; tk < 2; tk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int key = k0 + tk * 32 + 8 * (r / 4) + 4 * lg + (r % 4);
          if (key > qpos) s[tk][r] = -INFINITY;
        }
    }
    float mx = m_run;
#pragma unroll
    for (int tk = 0; tk < 2; tk++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[tk][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float alpha = __builtin_amdgcn_exp2f((m_run - mx) * a.scale_log2);   // first visible tile: exp2(-inf) = 0
    m_run = mx;
    const float mxs = mx * a.scale_log2;
    float psum = 0.0f;
    h8_t pf[2][2];
#pragma unroll
    for (int tk = 0; tk < 2; tk++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[tk][r], a.scale_log2, -mxs));
        psum += p;
        pf[tk][r / 8][r % 8] = (_Float16)p;
      }
    l_run = l_run * alpha + psum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {   // the running maximum of some row moved (uniform branch)
#pragma unroll
      for (int td = 0; td < HD / 32; td++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[td][r] *= alpha;
    }

    // O^T += V^T . P^T : k-slot s' of lane half lg in step (tk, hs) is key tk*32 + hs*16 + 8*(s'/4) + 4*lg + s'%4
#pragma unroll
    for (int tk = 0; tk < 2; tk++)
#pragma unroll
      for (int hs = 0; hs < 2; hs++) {
        const int kb = tk * 32 + hs * 16 + 4 * lg;
#pragma unroll
        for (int td = 0; td < HD / 32; td++) {
          const _Float16 *vp = &Vt[(td * 32 + l32) * VS + kb];
          const h4_t v0 = *(const h4_t *)vp, v1 = *(const h4_t *)(vp + 8);
          const h8_t vf = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
          o_acc[td] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[tk][hs], o_acc[td], 0, 0, 0);
        }
      }
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  if (q_valid) {
    _Float16 *op = a.out + ((size_t)b * a.S + qrow) * a.n_heads * HD + (size_t)h * HD;
#pragma unroll
    for (int td = 0; td < HD / 32; td++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        h4_t v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = (_Float16)(o_acc[td][r4 * 4 + e] * inv);
        *(h4_t *)(op + td * 32 + 8 * r4 + 4 * lg) = v;
      }
  }
}

// ---------------------------------------------------------------- row-wise companions

// Embedding.call / Int8Embedding.call (nn/index.ts:607-619, llama3.ts:71-77) for `rows` token ids
__global__ void embed_rows_kernel(int kind, const void *table, const _Float16 *scale, const int32_t *tokens, _Float16 *out, int dim, int vocab) {
  int tok = tokens[blockIdx.x];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  _Float16 *o = out + (size_t)blockIdx.x * dim;
  if (kind == JSGRAD_W_F16) {
    const _Float16 *src = (const _Float16 *)table + (size_t)tok * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = src[i];
  } else {
    const int8_t *src = (const int8_t *)table + (size_t)tok * dim;
    const float s = (float)scale[tok];
    for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = mul_rn16((float)src[i], s);
  }
}

// RMSNorm.call (nn/index.ts:586-588), one block per row.  A thread keeps its 16-byte chunks of the row (and of the weight)
// in registers between the sum of squares and the scaling: one round of loads.  MAXCH chunks per thread (d <= 2048 * MAXCH);
// longer rows take the two-pass loop.
template <int MAXCH>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const _Float16 *x, const _Float16 *w, _Float16 *y, int d, float eps, float inv_d) {
  __shared__ float red[4];
  const _Float16 *xr = x + (size_t)blockIdx.x * d;
  _Float16 *yr = y + (size_t)blockIdx.x * d;
  float ss = 0.0f;
  if constexpr (MAXCH > 0) {
    const int nch = d / 8;
    h8_t xv[MAXCH], wv[MAXCH];
#pragma unroll
    for (int c = 0; c < MAXCH; c++) {
      const int i = threadIdx.x + c * 256;
      if (i < nch) { xv[c] = *(const h8_t *)(xr + i * 8); wv[c] = *(const h8_t *)(w + i * 8); }
    }
#pragma unroll
    for (int c = 0; c < MAXCH; c++)
      if (threadIdx.x + c * 256 < nch)
#pragma unroll
        for (int e = 0; e < 8; e++) { const float f = (float)xv[c][e]; ss = fmaf(f, f, ss); }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float r = __fsqrt_rn(__fdiv_rn(1.0f, __fadd_rn(__fmul_rn(tot, inv_d), eps)));
#pragma unroll
    for (int c = 0; c < MAXCH; c++) {
      const int i = threadIdx.x + c * 256;
      if (i < nch) {
        h8_t o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = (_Float16)__fmul_rn(rn16(__fmul_rn((float)xv[c][e], r)), (float)wv[c][e]);
        *(h8_t *)(yr + i * 8) = o;
      }
    }
  } else {
    for (int i = threadIdx.x; i < d; i += 256) { const float f = (float)xr[i]; ss = fmaf(f, f, ss); }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float r = __fsqrt_rn(__fdiv_rn(1.0f, __fadd_rn(__fmul_rn(tot, inv_d), eps)));
    for (int i = threadIdx.x; i < d; i += 256) {
      const float v = rn16(__fmul_rn((float)xr[i], r));
      yr[i] = (_Float16)__fmul_rn(v, (float)w[i]);
    }
  }
}

// Tensor.argmax (tensor.ts:2314-2320) of every row: lowest index among the maxima.  One block per row.
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const _Float16 *x, int n, int32_t *out) {
  __shared__ float vmax[16];
  __shared__ int imax[16];
  const _Float16 *xr = x + (size_t)blockIdx.x * n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  auto merge = [&](float ov, int oi) { if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; } };
  for (int i = threadIdx.x; i < n; i += 1024) merge((float)xr[i], i);
  for (int off = 32; off > 0; off >>= 1) merge(__shfl_xor(best, off), __shfl_xor(bi, off));
  if ((threadIdx.x & 63) == 0) { vmax[threadIdx.x >> 6] = best; imax[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; w++) merge(vmax[w], imax[w]);
    out[blockIdx.x] = bi == 0x7fffffff ? n : bi;
  }
}

}  // namespace jsg

using namespace jsg;

extern "C" {

int jsgrad_hip_attn_prefill(const void *q, const void *cache_k, const void *cache_v, void *out, int batch, int seq_len, int start_pos, int n_heads,
                            int n_kv_heads, int head_dim, int max_context) {
  JSG_READY();
  JSG_REQUIRE(q && cache_k && cache_v && out, "jsgrad_hip_attn_prefill: null pointer argument");
  JSG_REQUIRE(batch > 0 && batch <= 65535 && seq_len > 0, "jsgrad_hip_attn_prefill: batch %d, seq_len %d", batch, seq_len);
  JSG_REQUIRE(n_heads > 0 && n_heads <= 65535 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "jsgrad_hip_attn_prefill: n_heads %d / n_kv_heads %d", n_heads, n_kv_heads);
  JSG_REQUIRE(head_dim == 64 || head_dim == 128, "jsgrad_hip_attn_prefill: head_dim %d (64 and 128 are built)", head_dim);
  JSG_REQUIRE(start_pos >= 0 && start_pos + seq_len <= max_context, "jsgrad_hip_attn_prefill: positions [%d, %d) outside the cache of %d", start_pos,
              start_pos + seq_len, max_context);
  PrefillAttnArgs a;
  a.q = (const _Float16 *)q; a.cache_k = (const _Float16 *)cache_k; a.cache_v = (const _Float16 *)cache_v; a.out = (_Float16 *)out;
  a.S = seq_len; a.start_pos = start_pos; a.n_heads = n_heads; a.n_kv_heads = n_kv_heads; a.max_context = max_context;
  a.scale_log2 = (float)(1.0 / sqrt((double)head_dim)) * 1.4426950408889634f;
  dim3 grid((seq_len + PF_QROWS - 1) / PF_QROWS, n_heads, batch), block(PF_THREADS);
  if (head_dim == 64) JSG_LAUNCH(PROF_ATTN_PREFILL, attn_prefill_kernel<64>, grid, block, 0, a);
  else JSG_LAUNCH(PROF_ATTN_PREFILL, attn_prefill_kernel<128>, grid, block, 0, a);
  return 0;
}

int jsgrad_hip_embed_rows(int kind, const void *table, const void *scale, const int32_t *tokens, int rows, void *out, int dim, int vocab) {
  JSG_READY();
  JSG_REQUIRE(table && tokens && out, "jsgrad_hip_embed_rows: null pointer argument");
  JSG_REQUIRE(kind == JSGRAD_W_F16 || (kind == JSGRAD_W_I8 && scale), "jsgrad_hip_embed_rows: table kind %d (fp16, or int8 with row scales)", kind);
  JSG_REQUIRE(rows > 0 && dim > 0 && vocab > 0, "jsgrad_hip_embed_rows: rows %d, dim %d, vocab %d", rows, dim, vocab);
  JSG_LAUNCH(PROF_EMBED, embed_rows_kernel, dim3(rows), dim3(256), 0, kind, table, (const _Float16 *)scale, tokens, (_Float16 *)out, dim, vocab);
  return 0;
}

int jsgrad_hip_rmsnorm_rows(const void *x, const void *w, void *y, int rows, int d, float eps) {
  JSG_READY();
  JSG_REQUIRE(x && w && y && rows > 0 && d > 0, "jsgrad_hip_rmsnorm_rows: bad argument");
  const float inv_d = (float)(1.0 / (double)d);
  if (d % 8 == 0 && d <= 2048) JSG_LAUNCH(PROF_RMSNORM, rmsnorm_rows_kernel<1>, dim3(rows), dim3(256), 0, (const _Float16 *)x, (const _Float16 *)w, (_Float16 *)y, d, eps, inv_d);
  else if (d % 8 == 0 && d <= 8192) JSG_LAUNCH(PROF_RMSNORM, rmsnorm_rows_kernel<4>, dim3(rows), dim3(256), 0, (const _Float16 *)x, (const _Float16 *)w, (_Float16 *)y, d, eps, inv_d);
  else JSG_LAUNCH(PROF_RMSNORM, rmsnorm_rows_kernel<0>, dim3(rows), dim3(256), 0, (const _Float16 *)x, (const _Float16 *)w, (_Float16 *)y, d, eps, inv_d);
  return 0;
}

int jsgrad_hip_argmax_rows(const void *logits, int rows, int n, int32_t *tokens_out) {
  JSG_READY();
  JSG_REQUIRE(logits && tokens_out && rows > 0 && n > 0, "jsgrad_hip_argmax_rows: bad argument");
  JSG_LAUNCH(PROF_ARGMAX, argmax_rows_kernel, dim3(rows), dim3(1024), 0, (const _Float16 *)logits, n, tokens_out);
  return 0;
}

}  // extern "C"
