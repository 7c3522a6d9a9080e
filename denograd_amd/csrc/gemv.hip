// One-row linear layers (GEMV) with in-register dequantisation for gfx950.
//
// y[out] = x[in] . W^T for W stored as float32, float16, int8 (+ fp16 scale per output row) or NF4
// (+ fp16 scale per 64 elements): Linear.call / Int8Linear.call / NF4Linear.call of the reference
// (/root/reference/jsgrad/nn/index.ts:411, /root/reference/jsgrad/models/llama3.ts:35,91-97) at batch 1,
// where the whole cost is streaming W once from HBM.
//
// Mapping: a block first stages the input row in LDS (optionally applying RMSNorm,
// nn/index.ts:586-588), then each 64-lane wavefront owns ROWS consecutive output rows and walks the
// reduce axis in steps of 64 lanes x 16 bytes: one 128-bit coalesced weight load per lane per row,
// dequantised in registers, accumulated in float.  A wavefront needs no barrier after staging; the
// final cross-lane sum is DPP.  Fused epilogues: plain store (+ residual), rotary embedding with the
// KV-cache write (models/llama.ts:61-87), SwiGLU (llama.ts:108-110).
#include "common.h"

namespace jsg {

enum { EPI_STORE = 0, EPI_ROPE_KV = 1, EPI_SWIGLU = 2 };

struct GemvArgs {
  const void *w[3];       // up to three matrices sharing the input row: (wq, wk, wv) or (w1, w3)
  const void *s[3];       // their scales (int8: per row, nf4: per 64 elements)
  int rows[3];            // rows of each matrix (0 = unused)
  int in_f;
  const void *x;          // input row, activation dtype
  const void *norm_w;     // RMSNorm weight or nullptr
  float eps;
  float inv_d;            // float(1/in_f), the constant the mean is multiplied with (tensor.ts:2113-2117)
  void *y;                // EPI_STORE: y[rows0]; EPI_SWIGLU: g[rows0]; EPI_ROPE_KV: q_out[rows0]
  const void *residual;   // EPI_STORE only, may be nullptr
  const void *rope_table; // [2*max_context][hd/2][2], activation dtype
  const int32_t *st;      // device {token, start_pos}
  void *cache_k, *cache_v;
  int head_dim, max_context;
};

// ---- weight formats: VEC elements per 16-byte load --------------------------------------------
template <int KIND> struct WFmt;
template <> struct WFmt<JSGRAD_W_F32> { static constexpr int VEC = 4; };
template <> struct WFmt<JSGRAD_W_F16> { static constexpr int VEC = 8; };
template <> struct WFmt<JSGRAD_W_I8> { static constexpr int VEC = 16; };
template <> struct WFmt<JSGRAD_W_NF4> { static constexpr int VEC = 32; };

// NF4 code book (llama3.ts:80-81); the CODE tensor is float16, so every literal is rounded to fp16 first
#define JSG_C16(x) ((float)(_Float16)(x))
__device__ __constant__ float NF4_CODE[16] = {JSG_C16(-1.0f), JSG_C16(-0.6961928009986877f), JSG_C16(-0.5250730514526367f), JSG_C16(-0.39491748809814453f),
                                              JSG_C16(-0.28444138169288635f), JSG_C16(-0.18477343022823334f), JSG_C16(-0.09105003625154495f), JSG_C16(0.0f),
                                              JSG_C16(0.07958029955625534f), JSG_C16(0.16093020141124725f), JSG_C16(0.24611230194568634f), JSG_C16(0.33791524171829224f),
                                              JSG_C16(0.44070982933044434f), JSG_C16(0.5626170039176941f), JSG_C16(0.7229568362236023f), JSG_C16(1.0f)};

// x fragment of one lane for one step: VEC activations
template <typename AT, int VEC> struct XFrag;
template <int VEC> struct XFrag<_Float16, VEC> {
  h2_t v[VEC / 2];
  __device__ __forceinline__ void load(const _Float16 *xs) {
    const u4_t *p = (const u4_t *)xs;
#pragma unroll
    for (int i = 0; i < VEC / 8; i++) {
      u4_t t = p[i];
#pragma unroll
      for (int j = 0; j < 4; j++) v[i * 4 + j] = as_h2(t[j]);
    }
  }
  __device__ __forceinline__ float get(int i) const { return (float)v[i >> 1][i & 1]; }
};
template <int VEC> struct XFrag<float, VEC> {
  float v[VEC];
  __device__ __forceinline__ void load(const float *xs) {
    const f4_t *p = (const f4_t *)xs;
#pragma unroll
    for (int i = 0; i < VEC / 4; i++) {
      f4_t t = p[i];
#pragma unroll
      for (int j = 0; j < 4; j++) v[i * 4 + j] = t[j];
    }
  }
  __device__ __forceinline__ float get(int i) const { return v[i]; }
};

// dot of one 16-byte weight vector with the lane's x fragment, accumulated into acc
template <int KIND, typename AT> struct Dot {
  static constexpr int VEC = WFmt<KIND>::VEC;
  // generic float path
  __device__ static __forceinline__ float run(u4_t wv, const XFrag<AT, VEC> &xf, float acc, float blk_scale, const float *lut) {
    if constexpr (KIND == JSGRAD_W_F32) {
#pragma unroll
      for (int i = 0; i < 4; i++) acc = fmaf(xf.get(i), __uint_as_float(wv[i]), acc);
    } else if constexpr (KIND == JSGRAD_W_F16) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        h2_t w2 = as_h2(wv[i]);
        acc = fmaf(xf.get(2 * i), (float)w2[0], acc);
        acc = fmaf(xf.get(2 * i + 1), (float)w2[1], acc);
      }
    } else if constexpr (KIND == JSGRAD_W_I8) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        int d = (int)wv[i];
        acc = fmaf(xf.get(4 * i + 0), (float)((d << 24) >> 24), acc);
        acc = fmaf(xf.get(4 * i + 1), (float)((d << 16) >> 24), acc);
        acc = fmaf(xf.get(4 * i + 2), (float)((d << 8) >> 24), acc);
        acc = fmaf(xf.get(4 * i + 3), (float)(d >> 24), acc);
      }
    } else {
      // 32 codes; element 2j is the high nibble of byte j (llama3.ts:92-94,105). One scale per lane-step
      // because 32 | 64 and k is a multiple of 32.  Each term is x * (code * scale) as the reference forms it:
      // the inner product is exact in float (11 x 11 significant bits).
#pragma unroll
      for (int i = 0; i < 4; i++) {
        uint32_t d = wv[i];
#pragma unroll
        for (int b = 0; b < 4; b++) {
          uint32_t byte = (d >> (8 * b)) & 0xffu;
          acc = fmaf(xf.get(8 * i + 2 * b), lut[byte >> 4] * blk_scale, acc);
          acc = fmaf(xf.get(8 * i + 2 * b + 1), lut[byte & 15u] * blk_scale, acc);
        }
      }
    }
    return acc;
  }
};
// fp16 activations x fp16 weights: packed dot with float accumulation
template <> struct Dot<JSGRAD_W_F16, _Float16> {
  static constexpr int VEC = 8;
  __device__ static __forceinline__ float run(u4_t wv, const XFrag<_Float16, 8> &xf, float acc, float, const float *) {
#pragma unroll
    for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_fdot2(as_h2(wv[i]), xf.v[i], acc, false);
    return acc;
  }
};
// fp16 activations x int8 weights: bytes -> exact fp16 integers through the 0x6400 exponent trick
// (0x6400 | u is the half 1024 + u for u in 0..255), then the packed dot
template <> struct Dot<JSGRAD_W_I8, _Float16> {
  static constexpr int VEC = 16;
  __device__ static __forceinline__ float run(u4_t wv, const XFrag<_Float16, 16> &xf, float acc, float, const float *) {
    const h2_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};  // 1024 + 128
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t u = wv[i] ^ 0x80808080u;  // signed byte w -> unsigned w + 128
      h2_t lo = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
      h2_t hi = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
      acc = __builtin_amdgcn_fdot2(lo, xf.v[2 * i], acc, false);
      acc = __builtin_amdgcn_fdot2(hi, xf.v[2 * i + 1], acc, false);
    }
    return acc;
  }
};

template <int KIND> __device__ __forceinline__ u4_t load_w(const void *w, size_t row, int in_f, int k) {
  // element (row, k) sits at bit offset (row*in_f + k) * bits
  constexpr int BITS = KIND == JSGRAD_W_F32 ? 32 : KIND == JSGRAD_W_F16 ? 16 : KIND == JSGRAD_W_I8 ? 8 : 4;
  const char *p = (const char *)w + ((row * (size_t)in_f + (size_t)k) * BITS) / 8;
  return __builtin_nontemporal_load((const u4_t *)p);
}

// Stage x (optionally RMSNorm'ed) into LDS in the activation dtype.  Every thread moves 16-byte chunks; with a
// norm the chunks stay in registers between the sum of squares and the scaling, so x is read from memory once and
// the whole prologue costs one round of global loads and two barriers.
template <typename AT> __device__ __forceinline__ void stage_x(const GemvArgs &a, AT *xs, float *red) {
  constexpr int EPC = 16 / sizeof(AT);  // elements per 16-byte chunk
  constexpr int MAXCH = 4;              // chunks a thread keeps in registers on the norm path
  const int n = a.in_f, tid = threadIdx.x, nt = blockDim.x;
  const int nchunks = n / EPC;          // in_f is a multiple of EPC (checked on the host)
  const u4_t *xg = (const u4_t *)a.x;
  u4_t *xl = (u4_t *)xs;
  if (a.norm_w == nullptr) {
    for (int c = tid; c < nchunks; c += nt) xl[c] = xg[c];
    __syncthreads();
    return;
  }
  const u4_t *wg = (const u4_t *)a.norm_w;
  u4_t xr[MAXCH], wr[MAXCH];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < MAXCH; i++) {
    const int c = tid + i * nt;
    if (c < nchunks) { xr[i] = xg[c]; wr[i] = wg[c]; }
  }
#pragma unroll
  for (int i = 0; i < MAXCH; i++) {
    const int c = tid + i * nt;
    if (c < nchunks) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if constexpr (sizeof(AT) == 2) {
          h2_t h = as_h2(xr[i][e]);
          ss = fmaf((float)h[0], (float)h[0], ss);
          ss = fmaf((float)h[1], (float)h[1], ss);
        } else {
          float f = __uint_as_float(xr[i][e]);
          ss = fmaf(f, f, ss);
        }
      }
    }
  }
  ss = wave_sum(ss);
  const int wave = tid >> 6, nw = nt >> 6;
  if ((tid & 63) == 0) red[wave] = ss;
  __syncthreads();
  float tot = 0.0f;
  for (int i = 0; i < nw; i++) tot += red[i];
  // sqrt(1 / (mean + eps)), mean = sum * float(1/d)  (nn/index.ts:586, tensor.ts:2944-2946)
  const float r = __fsqrt_rn(__fdiv_rn(1.0f, __fadd_rn(__fmul_rn(tot, a.inv_d), a.eps)));
#pragma unroll
  for (int i = 0; i < MAXCH; i++) {
    const int c = tid + i * nt;
    if (c < nchunks) {
      u4_t o;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if constexpr (sizeof(AT) == 2) {
          h2_t h = as_h2(xr[i][e]), w = as_h2(wr[i][e]), y;
          // .cast(x.dtype) before the weight multiply (nn/index.ts:588)
          y[0] = (_Float16)((float)(_Float16)((float)h[0] * r) * (float)w[0]);
          y[1] = (_Float16)((float)(_Float16)((float)h[1] * r) * (float)w[1]);
          o[e] = __builtin_bit_cast(uint32_t, y);
        } else {
          o[e] = __float_as_uint((__uint_as_float(xr[i][e]) * r) * __uint_as_float(wr[i][e]));
        }
      }
      xl[c] = o;
    }
  }
  __syncthreads();
}

// A block stages x once and then its wavefronts walk row groups (ROWS consecutive output rows of the NM matrices
// that share x) grid-stride.  A wavefront's work is the flat sequence of (row group, k-batch) items; the weight
// loads of item i+1 are issued into a second register buffer before item i is consumed, and the first item is
// requested before x is staged, so a wavefront always has a batch of 128-bit loads in flight.
template <int KIND, typename AT, int EPI, int ROWS, int UNROLL>
__global__ __launch_bounds__(256) void gemv_kernel(GemvArgs a) {
  constexpr int VEC = WFmt<KIND>::VEC;
  constexpr int BITS = KIND == JSGRAD_W_F32 ? 32 : KIND == JSGRAD_W_F16 ? 16 : KIND == JSGRAD_W_I8 ? 8 : 4;
  constexpr int STEP = 64 * VEC;                 // elements one wavefront covers per k-step
  constexpr int NM = EPI == EPI_SWIGLU ? 2 : 1;  // matrices a wavefront evaluates on the same rows
  static_assert(ROWS % 2 == 0 || EPI != EPI_ROPE_KV, "rotary pairs need an even row group");
  extern __shared__ __align__(16) unsigned char smem[];
  AT *xs = (AT *)smem;
  __shared__ float red[8];
  __shared__ float lut[16];
  if (KIND == JSGRAD_W_NF4 && threadIdx.x < 16) lut[threadIdx.x] = NF4_CODE[threadIdx.x];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int in_f = a.in_f;
  const int total = EPI == EPI_SWIGLU ? a.rows[0] : a.rows[0] + a.rows[1] + a.rows[2];
  const int ngroups = (total + ROWS - 1) / ROWS;
  const int gstride = gridDim.x * nw;
  const int nsteps = (in_f + STEP - 1) / STEP;
  const int nbatch = (nsteps + UNROLL - 1) / UNROLL;
  // One item's registers: the weight vectors plus, on the item that finishes a row group, the operands its epilogue
  // will need (row scales, residual, rotary pair), fetched now so that no load latency is left at the end.
  struct Buf {
    u4_t w[UNROLL][NM][ROWS];
    float scale[NM][ROWS];
    float extra[ROWS];   // EPI_STORE: residual[row]; EPI_ROPE_KV: (cos, sin) of the pair in extra[r], extra[r+1]
  };
  // read the position now, not in the epilogue: the load then overlaps the weight stream instead of ending the kernel
  const int pos = EPI == EPI_ROPE_KV ? a.st[1] : 0;

  // rows of a group: matrix m (EPI_ROPE_KV stacks wq, wk, wv; boundaries are multiples of ROWS), first row r0
  struct Where { int m, r0, mrows; };
  auto locate = [&](int grp) {
    Where w = {0, grp * ROWS, 0};
    if (EPI == EPI_ROPE_KV) {
      if (w.r0 >= a.rows[0]) { w.r0 -= a.rows[0]; w.m = 1; }
      if (w.m == 1 && w.r0 >= a.rows[1]) { w.r0 -= a.rows[1]; w.m = 2; }
    }
    // selects, not a.rows[m]: indexing the argument struct with a run-time m would copy it to scratch memory
    w.mrows = w.m == 0 ? a.rows[0] : (w.m == 1 ? a.rows[1] : a.rows[2]);
    return w;
  };
  auto wbase = [&](int m, int j) -> const void * { return NM == 2 ? (j == 0 ? a.w[0] : a.w[1]) : (m == 0 ? a.w[0] : (m == 1 ? a.w[1] : a.w[2])); };
  auto sbase = [&](int m, int j) -> const void * { return NM == 2 ? (j == 0 ? a.s[0] : a.s[1]) : (m == 0 ? a.s[0] : (m == 1 ? a.s[1] : a.s[2])); };

  auto load_item = [&](Buf &buf, int grp, int b) {
    const Where w = locate(grp);
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const int k = (b * UNROLL + u) * STEP + lane * VEC;
      if (k < in_f) {
#pragma unroll
        for (int j = 0; j < NM; j++)
#pragma unroll
          for (int r = 0; r < ROWS; r++) {
            const int row = w.r0 + r < w.mrows ? w.r0 + r : w.mrows - 1;  // tail rows reload the last row, never stored
            const char *p = (const char *)wbase(w.m, j) + (((size_t)row * in_f + (size_t)k) * BITS) / 8;
            buf.w[u][j][r] = __builtin_nontemporal_load((const u4_t *)p);
          }
      }
    }
    if (b != nbatch - 1) return;
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      const int row = w.r0 + r < w.mrows ? w.r0 + r : w.mrows - 1;
      if constexpr (KIND == JSGRAD_W_I8) {
#pragma unroll
        for (int j = 0; j < NM; j++) buf.scale[j][r] = (float)((const _Float16 *)sbase(w.m, j))[row];
      }
      if constexpr (EPI == EPI_STORE) {
        buf.extra[r] = a.residual ? (float)((const AT *)a.residual)[row] : 0.0f;
      } else if constexpr (EPI == EPI_ROPE_KV) {
        // table row `pos`, entry (cos, sin) of pair i = (row % head_dim) / 2: even r gets cos, odd r gets sin
        const bool ok = pos >= 0 && pos < a.max_context;
        const int i = (row % a.head_dim) >> 1;
        buf.extra[r] = ok ? (float)((const AT *)a.rope_table)[(size_t)pos * a.head_dim + 2 * i + (r & 1)] : 0.0f;
      }
    }
  };

  float acc[NM][ROWS];
  auto use_item = [&](const Buf &buf, int grp, int b) {
    const Where w = locate(grp);
    if (b == 0) {
#pragma unroll
      for (int j = 0; j < NM; j++)
#pragma unroll
        for (int r = 0; r < ROWS; r++) acc[j][r] = 0.0f;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const int k = (b * UNROLL + u) * STEP + lane * VEC;
      if (k < in_f) {
        XFrag<AT, VEC> xf;
        xf.load(xs + k);
#pragma unroll
        for (int j = 0; j < NM; j++)
#pragma unroll
          for (int r = 0; r < ROWS; r++) {
            float bs = 1.0f;
            if constexpr (KIND == JSGRAD_W_NF4) {
              const int row = w.r0 + r < w.mrows ? w.r0 + r : w.mrows - 1;
              bs = (float)((const _Float16 *)sbase(w.m, j))[((size_t)row * in_f + k) >> 6];
            }
            acc[j][r] = Dot<KIND, AT>::run(buf.w[u][j][r], xf, acc[j][r], bs, lut);
          }
      }
    }
    if (b != nbatch - 1) return;

    // ---- the group is complete: cross-lane sum, scale, cast, epilogue
    float val[NM][ROWS];
#pragma unroll
    for (int j = 0; j < NM; j++)
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        float v = wave_sum(acc[j][r]);
        if constexpr (KIND == JSGRAD_W_I8) v = v * buf.scale[j][r];
        val[j][r] = Act<AT>::rn(v);
      }
    const int r0 = w.r0, mrows = w.mrows;
    if constexpr (EPI == EPI_STORE) {
      AT *y = (AT *)a.y;
      const bool has_res = a.residual != nullptr;
#pragma unroll
      for (int r = 0; r < ROWS; r++)
        if (lane == r && r0 + r < mrows) {
          float v = val[0][r];
          if (has_res) v = Act<AT>::rn(buf.extra[r] + v);
          y[r0 + r] = (AT)v;
        }
    } else if constexpr (EPI == EPI_SWIGLU) {
      AT *g = (AT *)a.y;
#pragma unroll
      for (int r = 0; r < ROWS; r++)
        if (lane == r && r0 + r < mrows) g[r0 + r] = (AT)Act<AT>::rn(silu_act<AT>(val[0][r]) * val[1][r]);
    } else {
      if (pos < 0 || pos >= a.max_context) return;  // never write outside the cache
      if (w.m == 2) {  // value rows: plain copy into the cache row
        AT *cv = (AT *)a.cache_v + (size_t)pos * a.rows[2];
#pragma unroll
        for (int r = 0; r < ROWS; r++)
          if (lane == r && r0 + r < mrows) cv[r0 + r] = (AT)val[0][r];
      } else {         // query / key rows: rotate interleaved pairs (llama.ts:17-32)
        AT *dst = w.m == 0 ? (AT *)a.y : (AT *)a.cache_k + (size_t)pos * a.rows[1];
#pragma unroll
        for (int r = 0; r < ROWS; r += 2)
          if (lane == r && r0 + r + 1 < mrows) {
            const float c = buf.extra[r], d = buf.extra[r + 1];
            const float av = val[0][r], bv = val[0][r + 1];
            dst[r0 + r] = (AT)Act<AT>::rn(av * c - bv * d);  // the build keeps a*b+c unfused: two roundings as in plain C
            dst[r0 + r + 1] = (AT)Act<AT>::rn(av * d + bv * c);
          }
      }
    }
  };

  // flat item sequence of this wavefront: (grp, b) -> next
  int grp = blockIdx.x * nw + wave, b = 0;
  auto advance = [&](int &g, int &bb) {
    if (++bb == nbatch) { bb = 0; g += gstride; }
  };
  Buf bufA, bufB;
  if (grp < ngroups) load_item(bufA, grp, 0);

  stage_x<AT>(a, xs, red);  // block-wide, ends with a barrier (which also publishes lut)

  while (grp < ngroups) {
    int g1 = grp, b1 = b;
    advance(g1, b1);
    if (g1 < ngroups) load_item(bufB, g1, b1);
    use_item(bufA, grp, b);
    if (g1 >= ngroups) break;
    grp = g1; b = b1;
    advance(g1, b1);
    if (g1 < ngroups) load_item(bufA, g1, b1);
    use_item(bufB, grp, b);
    grp = g1; b = b1;
  }
}

// ---- host-side dispatch ------------------------------------------------------------------------

template <int KIND, typename AT, int EPI, int ROWS, int UNROLL> static int launch_cfg(const GemvArgs &a, int total_rows) {
  constexpr int kind = EPI == EPI_STORE ? PROF_LINEAR : (EPI == EPI_SWIGLU ? PROF_FFN_GATE : PROF_QKV_ROPE);
  constexpr int NW = 4;
  const int ngroups = (total_rows + ROWS - 1) / ROWS;
  const int need = (ngroups + NW - 1) / NW;      // one group per wavefront
  const int cap = state().cu_count * 4;          // 16 resident wavefronts per CU; more rows than that are walked grid-stride
  dim3 grid(need < cap ? need : cap), block(NW * 64);
  size_t lds = (size_t)a.in_f * sizeof(AT);
  JSG_LAUNCH(kind, (gemv_kernel<KIND, AT, EPI, ROWS, UNROLL>), grid, block, lds, a);
  return 0;
}
// Two register buffers of UNROLL x NM x ROWS 16-byte loads each: (2 rows, 4 steps) for one matrix, (2 rows, 2 steps)
// for the SwiGLU pair, i.e. 8 loads = 8 KiB per wavefront per buffer either way.
template <int KIND, typename AT, int EPI> static int launch_rows(const GemvArgs &a, int total_rows) {
  if constexpr (EPI == EPI_SWIGLU) return launch_cfg<KIND, AT, EPI, 2, 2>(a, total_rows);
  else
  return launch_cfg<KIND, AT, EPI, 2, 4>(a, total_rows);
}
template <int EPI> static int dispatch(int kind, int act, const GemvArgs &a, int total_rows) {
#define JSG_CASE(K)                                                          \
  case K:                                                                    \
    return act == JSGRAD_F16 ? launch_rows<K, _Float16, EPI>(a, total_rows) : launch_rows<K, float, EPI>(a, total_rows);
  switch (kind) {
    JSG_CASE(JSGRAD_W_F32)
    JSG_CASE(JSGRAD_W_F16)
    JSG_CASE(JSGRAD_W_I8)
    JSG_CASE(JSGRAD_W_NF4)
  }
#undef JSG_CASE
  return fail("unknown weight kind %d", kind);
}

static int check_common(const char *who, int kind, int act, int in_f, const void *x) {
  JSG_REQUIRE(act == JSGRAD_F16 || act == JSGRAD_F32, "%s: unknown activation dtype %d", who, act);
  JSG_REQUIRE(kind >= JSGRAD_W_F32 && kind <= JSGRAD_W_NF4, "%s: unknown weight kind %d", who, kind);
  JSG_REQUIRE(x, "%s: null input", who);
  const int vec = kind == JSGRAD_W_F32 ? 4 : kind == JSGRAD_W_F16 ? 8 : kind == JSGRAD_W_I8 ? 16 : 64;
  JSG_REQUIRE(in_f > 0 && in_f % vec == 0, "%s: in_features %d must be a positive multiple of %d for this weight format", who, in_f, vec);
  JSG_REQUIRE((size_t)in_f * (act == JSGRAD_F16 ? 2 : 4) <= 64 * 1024, "%s: in_features %d does not fit the 64 KiB LDS staging buffer", who, in_f);
  return 0;
}
// the fused RMSNorm keeps 4 x 16 bytes of x per thread in registers (256 threads)
static int check_norm(const char *who, const void *norm_weight, int act, int in_f) {
  const int cap = 4 * 256 * (act == JSGRAD_F16 ? 8 : 4);
  JSG_REQUIRE(norm_weight == nullptr || in_f <= cap, "%s: a fused RMSNorm handles at most %d features in this activation dtype, got %d", who, cap, in_f);
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

int jsgrad_hip_linear(int kind, const void *w, const void *scale, int out_f, int in_f, const void *x, void *y, const void *norm_weight, float eps,
                      const void *residual, int act) {
  JSG_READY();
  if (int e = check_common("jsgrad_hip_linear", kind, act, in_f, x)) return e;
  JSG_REQUIRE(w && y && out_f > 0, "jsgrad_hip_linear: null weight/output or out_features %d", out_f);
  JSG_REQUIRE(kind < JSGRAD_W_I8 || scale, "jsgrad_hip_linear: quantised weight needs a scale");
  JSG_REQUIRE(y != x, "jsgrad_hip_linear: output must not alias the input");
  if (int e = check_norm("jsgrad_hip_linear", norm_weight, act, in_f)) return e;
  GemvArgs a = {};
  a.w[0] = w; a.s[0] = scale; a.rows[0] = out_f; a.in_f = in_f; a.x = x; a.norm_w = norm_weight; a.eps = eps;
  a.inv_d = (float)(1.0 / (double)in_f); a.y = y; a.residual = residual;
  return dispatch<EPI_STORE>(kind, act, a, out_f);
}

int jsgrad_hip_ffn_gate(int kind, const void *w1, const void *s1, const void *w3, const void *s3, const void *x, const void *norm_weight, float eps,
                        void *g, int dim, int hidden, int act) {
  JSG_READY();
  if (int e = check_common("jsgrad_hip_ffn_gate", kind, act, dim, x)) return e;
  JSG_REQUIRE(w1 && w3 && g && hidden > 0, "jsgrad_hip_ffn_gate: null weight/output or hidden %d", hidden);
  JSG_REQUIRE(kind < JSGRAD_W_I8 || (s1 && s3), "jsgrad_hip_ffn_gate: quantised weights need scales");
  JSG_REQUIRE(norm_weight, "jsgrad_hip_ffn_gate: null norm weight");
  if (int e = check_norm("jsgrad_hip_ffn_gate", norm_weight, act, dim)) return e;
  GemvArgs a = {};
  a.w[0] = w1; a.s[0] = s1; a.w[1] = w3; a.s[1] = s3; a.rows[0] = hidden; a.rows[1] = hidden; a.in_f = dim; a.x = x;
  a.norm_w = norm_weight; a.eps = eps; a.inv_d = (float)(1.0 / (double)dim); a.y = g;
  return dispatch<EPI_SWIGLU>(kind, act, a, hidden);
}

int jsgrad_hip_qkv_rope(int kind, const void *wq, const void *sq, const void *wk, const void *sk, const void *wv, const void *sv, const void *x,
                        const void *norm_weight, float eps, const void *rope_table, const int32_t *st, void *q_out, void *cache_k, void *cache_v, int dim,
                        int n_heads, int n_kv_heads, int head_dim, int max_context, int act) {
  JSG_READY();
  if (int e = check_common("jsgrad_hip_qkv_rope", kind, act, dim, x)) return e;
  JSG_REQUIRE(wq && wk && wv && rope_table && st && q_out && cache_k && cache_v, "jsgrad_hip_qkv_rope: null pointer argument");
  JSG_REQUIRE(kind < JSGRAD_W_I8 || (sq && sk && sv), "jsgrad_hip_qkv_rope: quantised weights need scales");
  JSG_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "jsgrad_hip_qkv_rope: n_heads %d must be a multiple of n_kv_heads %d", n_heads, n_kv_heads);
  JSG_REQUIRE(head_dim > 0 && head_dim % 4 == 0, "jsgrad_hip_qkv_rope: head_dim %d must be a multiple of 4", head_dim);
  JSG_REQUIRE(max_context > 0, "jsgrad_hip_qkv_rope: max_context %d", max_context);
  JSG_REQUIRE(norm_weight, "jsgrad_hip_qkv_rope: null norm weight");
  if (int e = check_norm("jsgrad_hip_qkv_rope", norm_weight, act, dim)) return e;
  GemvArgs a = {};
  a.w[0] = wq; a.s[0] = sq; a.w[1] = wk; a.s[1] = sk; a.w[2] = wv; a.s[2] = sv;
  a.rows[0] = n_heads * head_dim; a.rows[1] = n_kv_heads * head_dim; a.rows[2] = n_kv_heads * head_dim;
  a.in_f = dim; a.x = x; a.norm_w = norm_weight; a.eps = eps; a.inv_d = (float)(1.0 / (double)dim); a.y = q_out;
  a.rope_table = rope_table; a.st = st; a.cache_k = cache_k; a.cache_v = cache_v; a.head_dim = head_dim; a.max_context = max_context;
  return dispatch<EPI_ROPE_KV>(kind, act, a, a.rows[0] + a.rows[1] + a.rows[2]);
}

}  // extern "C"
