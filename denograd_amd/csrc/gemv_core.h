// Device code of the one-row linear layers (GEMV) with in-register dequantisation for gfx950, shared by the
// stand-alone kernels (gemv.hip) and the whole-step kernel (decode_step.hip).
//
// y[out] = x[in] . W^T for W stored as float32, float16, int8 (+ fp16 scale per output row) or NF4 (+ fp16 scale per
// 64 elements): Linear.call / Int8Linear.call / NF4Linear.call of the reference
// (/root/reference/jsgrad/nn/index.ts:411, /root/reference/jsgrad/models/llama3.ts:35,91-97) at batch 1, where the whole
// cost is streaming W once from HBM.  Fused around it: RMSNorm of the input (nn/index.ts:586-588), and as epilogues a
// plain store (+ residual), the rotary embedding with the KV-cache write (models/llama.ts:61-87), SwiGLU (llama.ts:108-110).
#pragma once
#include "common.h"

namespace jsg {

enum { EPI_STORE = 0, EPI_ROPE_KV = 1, EPI_SWIGLU = 2 };

struct GemvArgs {
  const void *w0, *w1, *w2;  // up to three matrices sharing the input row: (wq, wk, wv) or (w1, w3).  Separate fields,
                             // not arrays: a run-time index into the argument struct would force it into scratch memory
  const void *s0, *s1, *s2;  // their scales (int8: per row, nf4: per 64 elements)
  int rows0, rows1, rows2;   // rows of each matrix (0 = unused)
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
  // when set, the input row is read from here instead of x: tagged words (fp16 value | x_tag << 16) that other blocks of
  // the same launch are writing; err: set when the wait for them ran out
  const uint32_t *x_tagged = nullptr;
  uint32_t x_tag = 0;
  int *err = nullptr;
};

// ---- weight formats: VEC elements per 16-byte load --------------------------------------------
template <int KIND> struct WFmt;
template <> struct WFmt<JSGRAD_W_F32> { static constexpr int VEC = 4; };
template <> struct WFmt<JSGRAD_W_F16> { static constexpr int VEC = 8; };
template <> struct WFmt<JSGRAD_W_I8> { static constexpr int VEC = 16; };
template <> struct WFmt<JSGRAD_W_NF4> { static constexpr int VEC = 32; };

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
      // The empty asm pins the unpacking of this word here.  Left alone, the scheduler unpacks a whole item as its loads
      // arrive, which doubles the registers the item occupies.
      uint32_t word = wv[i];
      asm volatile("" : "+v"(word));
      uint32_t u = word ^ 0x80808080u;  // signed byte w -> unsigned w + 128
      h2_t lo = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
      h2_t hi = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
      acc = __builtin_amdgcn_fdot2(lo, xf.v[2 * i], acc, false);
      acc = __builtin_amdgcn_fdot2(hi, xf.v[2 * i + 1], acc, false);
    }
    return acc;
  }
};

// fp16 activations x NF4 weights.  One byte holds two codes (element 2j in the high nibble, llama3.ts:92-94,105), and the
// lane's x fragment holds the two activations they meet as one packed pair: a 256-entry LDS table indexed by the byte gives
// both code values as a packed fp16 pair, ready for the packed dot.  The block scale (one per 64 elements, so one per
// 16-byte vector) multiplies the sum of the 32 products once: code * scale is exact in float either way, the sums differ
// from the generic path's in the last float bits only.  lut: 16 floats (the generic table), then the 256 pairs.
constexpr int NF4_LUT_WORDS = 16 + 256;
template <> struct Dot<JSGRAD_W_NF4, _Float16> {
  static constexpr int VEC = 32;
  __device__ static __forceinline__ float run(u4_t wv, const XFrag<_Float16, 32> &xf, float acc, float blk_scale, const float *lut) {
    const uint32_t *pairs = (const uint32_t *)lut + 16;
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t d = wv[i];
#pragma unroll
      for (int b = 0; b < 4; b++) s = __builtin_amdgcn_fdot2(as_h2(pairs[(d >> (8 * b)) & 0xffu]), xf.v[4 * i + b], s, false);
    }
    return acc + s * blk_scale;
  }
};

// The same table kept once PER LANE, for launches with enough rows to give every CU one block of sixteen wavefronts
// (Gemv<..., WIDE>): entry e of lane l is the word at byte e * 256 + l * 4 behind NF4_TAB_OFFSET, 64 KiB in all.  The weight
// bytes are as good as random, and 64 lanes asking one shared table for 64 random entries keep the 32 LDS banks busy for
// ~7 cycles instead of 2 (counted: 4.8 conflict cycles per look-up).  With a copy per lane, lane l only ever touches bank
// l % 32, and the address is one byte permute: byte 1 = the weight byte, byte 0 = 4 l, no shift, no add.
constexpr int NF4_TAB_OFFSET = 256, NF4_TAB_BYTES = 256 * 256;
constexpr int NF4_WIDE_LUT_WORDS = (NF4_TAB_OFFSET + NF4_TAB_BYTES) / 4;

// Stage x (optionally RMSNorm'ed) into LDS in the activation dtype.  Every thread moves 16-byte chunks; with a
// norm the chunks stay in registers between the sum of squares and the scaling, so x is read from memory once and
// the whole prologue costs one round of loads and two barriers.  Ends with a barrier.
// COHERENT: x was written by other blocks of the same launch, so it is read at the device-wide coherence point.
// `padded` >= in_f (a multiple of the 16-byte chunk): LDS elements [in_f, padded) are set to zero, so that a k-step
// that reaches past in_f multiplies whatever weights it loaded by zero.
template <typename AT, bool COHERENT> __device__ __forceinline__ void stage_x(const GemvArgs &a, AT *xs, float *red, int padded) {
  constexpr int EPC = 16 / sizeof(AT);  // elements per 16-byte chunk
  for (int c = a.in_f / EPC + threadIdx.x; c < padded / EPC; c += blockDim.x) ((u4_t *)xs)[c] = u4_t{0, 0, 0, 0};
  constexpr int MAXCH = 4;              // chunks a thread keeps in registers on the norm path (host checks the size)
  const int n = a.in_f, tid = threadIdx.x, nt = blockDim.x;
  const int nchunks = n / EPC;          // in_f is a multiple of EPC (checked on the host)
  const u4_t *xg = (const u4_t *)a.x;
  u4_t *xl = (u4_t *)xs;
  auto ldx = [&](int c) -> u4_t {
    if constexpr (sizeof(AT) == 2) {
      if (a.x_tagged != nullptr) {   // ask until the eight words of the chunk carry the tag of this launch
        u4_t v;
        for (int it = 0;; it++) {
          bool ok = true;
          v = tw_load8(a.x_tagged + (size_t)c * 8, a.x_tag, ok);
          if (ok) break;
          if (it > (1 << 18)) { st_coherent(a.err, 1); break; }
        }
        return v;
      }
    }
    if constexpr (COHERENT) {
      const uint32_t *p = (const uint32_t *)(xg + c);
      u4_t v;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = __hip_atomic_load(p + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return v;
    } else {
      return xg[c];
    }
  };
  if (a.norm_w == nullptr) {
    if (sizeof(AT) == 2 && a.x_tagged != nullptr) {
      // Waiting cheaply first: a block that asked for the whole row over and over would take memory bandwidth from the
      // blocks that are still producing it.  Eight words spread over the row are watched by one wavefront until they carry
      // the tag (a hint that the row is about there); what decides is the check of every word below.
      if (tid < 64) {
        // eight elements spread over the row (a row made of parts that different blocks finish, such as the heads of an
        // attention row) and the last eight (a row dealt in order to its producers' wavefronts: what is written last)
        const int probe = (tid & 8) ? n - 8 + (tid & 7) : (tid & 7) * (n / 8);
        for (int it = 0; it < (1 << 18); it++) {
          const uint32_t w = (uint32_t)ld_coherent((const int *)a.x_tagged + probe);
          if (__all((w >> 16) == a.x_tag)) break;
          __builtin_amdgcn_s_sleep(8);
        }
      }
      JSG_LSTAMP(2);
      lds_barrier();   // only "the probe is through": requests of this wavefront that are in flight stay in flight
      JSG_LSTAMP(3);
      // all chunks of a thread are asked for together, again and again until every one carries the tag: one round trip
      // when the row is there, instead of one per chunk
      constexpr int NCH = 2;
      if (nchunks <= nt) {
        // one chunk per thread at most (every block of the launch fetches the whole row at the same moment: nothing is
        // requested twice)
        if (tid < nchunks) {
          u4_t v;
          for (int it = 0;; it++) {
            bool ok = true;
            v = tw_load8(a.x_tagged + (size_t)tid * 8, a.x_tag, ok);
            if (ok) break;
            if (it > (1 << 18)) { st_coherent(a.err, 1); break; }
            __builtin_amdgcn_s_sleep(4);   // not there yet: leave the memory system to those who are producing it
          }
          xl[tid] = v;
        }
      } else {
        for (int c0 = tid; c0 < nchunks; c0 += NCH * nt) {
          u4_t v[NCH];
          for (int it = 0;; it++) {
            bool ok = true;
#pragma unroll
            for (int i = 0; i < NCH; i++) {
              const int c = c0 + i * nt;
              v[i] = tw_load8(a.x_tagged + (size_t)(c < nchunks ? c : c0) * 8, a.x_tag, ok);   // past the end: its own first chunk again
            }
            if (ok) break;
            if (it > (1 << 18)) { st_coherent(a.err, 1); break; }
            __builtin_amdgcn_s_sleep(4);   // not there yet: leave the memory system to those who are producing it
          }
#pragma unroll
          for (int i = 0; i < NCH; i++) {
            const int c = c0 + i * nt;
            if (c < nchunks) xl[c] = v[i];
          }
        }
      }
    } else {
      for (int c = tid; c < nchunks; c += nt) xl[c] = ldx(c);
    }
    __syncthreads();
    JSG_LSTAMP(4);
    return;
  }
  const u4_t *wg = (const u4_t *)a.norm_w;
  u4_t xr[MAXCH], wr[MAXCH];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < MAXCH; i++) {
    const int c = tid + i * nt;
    if (c < nchunks) { xr[i] = ldx(c); wr[i] = wg[c]; }
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

// The same staging in two halves, for an input row that is ready when the kernel starts: issue() requests x (and the norm
// weight) into registers BEFORE the first weight items are requested, finish() turns them into the LDS row afterwards.
// Loads return in the order they were issued, so a row requested behind 16 KiB of weights per wavefront arrives only when
// that whole window has landed (tens of megabytes over the chip) and nothing can be multiplied until then; requested first,
// it is there after one round trip and the arithmetic runs along with the weight stream.  The barriers wait for LDS traffic
// only, so the weight requests stay in flight.
constexpr int XSTAGE_CHUNKS = 8;   // 16-byte chunks of x a thread holds (plain rows; a normed row has at most 4, host-checked)
struct XStage {
  u4_t xr[XSTAGE_CHUNKS];   // a normed row: chunks in xr[0..3], the norm weight's in xr[4..7]
};
template <typename AT> __device__ __forceinline__ void stage_x_issue(const GemvArgs &a, XStage &st) {
  constexpr int EPC = 16 / sizeof(AT);
  const int tid = threadIdx.x, nt = blockDim.x, nchunks = a.in_f / EPC;
  const u4_t *xg = (const u4_t *)a.x;
  // Lanes (and whole wavefronts) without a chunk in round i load a valid chunk all the same: leaving those loads out under a
  // test the wavefront agrees on measured 1.2 % slower on the 8B int8 step (the branches and the merged wait counts cost
  // more than the address path's time for loads whose lines are in the cache anyway).
  if (a.norm_w != nullptr) {
    const u4_t *wg = (const u4_t *)a.norm_w;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int c = tid + i * nt;
      const int cc = c < nchunks ? c : nchunks - 1;   // past the end: a valid chunk again, not used
      st.xr[i] = ldg(xg + cc);
      st.xr[4 + i] = ldg(wg + cc);
    }
  } else {
#pragma unroll
    for (int i = 0; i < XSTAGE_CHUNKS; i++) {
      const int c = tid + i * nt;
      st.xr[i] = ldg(xg + (c < nchunks ? c : nchunks - 1));
    }
  }
}
template <typename AT> __device__ __forceinline__ void stage_x_finish(const GemvArgs &a, const XStage &st, AT *xs, float *red, int padded) {
  constexpr int EPC = 16 / sizeof(AT);
  const int n = a.in_f, tid = threadIdx.x, nt = blockDim.x, nchunks = n / EPC;
  u4_t *xl = (u4_t *)xs;
  for (int c = nchunks + tid; c < padded / EPC; c += nt) xl[c] = u4_t{0, 0, 0, 0};
  if (a.norm_w == nullptr) {
#pragma unroll
    for (int i = 0; i < XSTAGE_CHUNKS; i++) {
      const int c = tid + i * nt;
      if (c < nchunks) xl[c] = st.xr[i];
    }
    for (int c = tid + XSTAGE_CHUNKS * nt; c < nchunks; c += nt) xl[c] = ldg((const u4_t *)a.x + c);   // rows longer than the registers hold
    lds_barrier();
    return;
  }
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (tid + i * nt < nchunks) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if constexpr (sizeof(AT) == 2) {
          h2_t h = as_h2(st.xr[i][e]);
          ss = fmaf((float)h[0], (float)h[0], ss);
          ss = fmaf((float)h[1], (float)h[1], ss);
        } else {
          float f = __uint_as_float(st.xr[i][e]);
          ss = fmaf(f, f, ss);
        }
      }
    }
  }
  ss = wave_sum(ss);
  JSG_LSTAMP(7);
  JSG_LMAX(28);
  const int wave = tid >> 6, nw = nt >> 6;
  if ((tid & 63) == 0) red[wave] = ss;
  lds_barrier();
  JSG_LSTAMP(9);
  float tot = 0.0f;
  for (int i = 0; i < nw; i++) tot += red[i];
  const float r = __fsqrt_rn(__fdiv_rn(1.0f, __fadd_rn(__fmul_rn(tot, a.inv_d), a.eps)));
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int c = tid + i * nt;
    if (c < nchunks) {
      u4_t o;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if constexpr (sizeof(AT) == 2) {
          h2_t h = as_h2(st.xr[i][e]), w = as_h2(st.xr[4 + i][e]), y;
          y[0] = (_Float16)((float)(_Float16)((float)h[0] * r) * (float)w[0]);
          y[1] = (_Float16)((float)(_Float16)((float)h[1] * r) * (float)w[1]);
          o[e] = __builtin_bit_cast(uint32_t, y);
        } else {
          o[e] = __float_as_uint((__uint_as_float(st.xr[i][e]) * r) * __uint_as_float(st.xr[4 + i][e]));
        }
      }
      xl[c] = o;
    }
  }
  lds_barrier();
}

// One item's registers: the weight vectors plus, on the item that finishes a row group, the operands its epilogue will
// need (row scales, residual, rotary pair), fetched with the weights so that no load latency is left at the end.
// Every configuration in use moves 8 x 16 bytes per lane and item (UNROLL x NM x ROWS = 8) and has ROWS = 2, so one
// plain struct serves all of them; the whole-step kernel can then carry ONE prefetched buffer from phase to phase.
struct GemvBuf {
  u4_t w[8];            // [u][j][r] flattened
  // Small per-row operands, kept exactly as the loads returned them (16-bit loads stay 16-bit values) and converted
  // where they are used: any arithmetic at load time, even a zero-extension, waits for the load, and loads complete in
  // order, so it would wait for the weight vectors issued before it as well.
  _Float16 scale[4];    // [j][r] flattened: the int8 row scale
  _Float16 nscale[8];   // NF4: the block scale of each of the 8 vectors (one per 64 elements), fetched with them
  _Float16 extra_h[2];  // fp16 activations - EPI_STORE: residual[row]; EPI_ROPE_KV: cos or sin of the rotary pair
  float extra_f[2];     // the same for float32 activations
};
template <typename AT> __device__ __forceinline__ float extra_of(const GemvBuf &b, int r);
template <> __device__ __forceinline__ float extra_of<float>(const GemvBuf &b, int r) { return b.extra_f[r]; }
template <> __device__ __forceinline__ float extra_of<_Float16>(const GemvBuf &b, int r) { return (float)b.extra_h[r]; }
__device__ __forceinline__ void set_extra(GemvBuf &b, int r, float v) { b.extra_f[r] = v; }
__device__ __forceinline__ void set_extra(GemvBuf &b, int r, _Float16 v) { b.extra_h[r] = v; }

// The GEMV of one launch (or of one phase of the whole-step kernel).  A block stages x once, then its wavefronts walk
// row groups (ROWS consecutive output rows of the NM matrices that share x) grid-stride.  A wavefront's work is the flat
// sequence of (row group, k-batch) items; the loads of item i+1 go into a second register buffer before item i is
// consumed, and the first item is requested before x is staged (or, with `preloaded`, before the caller even waited
// for the previous phase), so a wavefront always has a batch of 128-bit loads in flight.
// COHERENT: x, residual and outputs cross between blocks of the same launch.
// WIDE (NF4 weights, fp16 activations): the look-up table is kept per lane (NF4_TAB_OFFSET); lut then has NF4_WIDE_LUT_WORDS words.
template <int KIND, typename AT, int EPI, int ROWS, int UNROLL, bool COHERENT, int EXACT = 0, bool WIDE = false> struct Gemv {
  static constexpr int VEC = WFmt<KIND>::VEC;
  static constexpr int BITS = KIND == JSGRAD_W_F32 ? 32 : KIND == JSGRAD_W_F16 ? 16 : KIND == JSGRAD_W_I8 ? 8 : 4;
  static constexpr int STEP = 64 * VEC;                 // elements one wavefront covers per k-step
  static constexpr int NM = EPI == EPI_SWIGLU ? 2 : 1;  // matrices a wavefront evaluates on the same rows
  typedef GemvBuf Buf;
  static_assert(ROWS == 2 && UNROLL * NM * ROWS == 8, "GemvBuf holds 8 vectors for 2 rows");
  __device__ static __forceinline__ constexpr int wi(int u, int j, int r) { return (u * NM + j) * ROWS + r; }
  __device__ static __forceinline__ constexpr int si(int j, int r) { return j * ROWS + r; }

  struct Where { int m, r0, mrows; };
  // rows of a group: matrix m (EPI_ROPE_KV stacks wq, wk, wv; boundaries are multiples of ROWS), first row r0
  __device__ static __forceinline__ Where locate(const GemvArgs &a, int grp) {
    Where w = {0, grp * ROWS, 0};
    if (EPI == EPI_ROPE_KV) {
      if (w.r0 >= a.rows0) { w.r0 -= a.rows0; w.m = 1; }
      if (w.m == 1 && w.r0 >= a.rows1) { w.r0 -= a.rows1; w.m = 2; }
    }
    w.mrows = a.rows0 * (w.m == 0) + a.rows1 * (w.m == 1) + a.rows2 * (w.m == 2);
    return w;
  }
  // Pick one of three pointers by a run-time index with arithmetic, not `?:` or an array: the optimiser turns a
  // select of loads from the argument struct into a load from a selected address, which forces the whole struct
  // into scratch memory.
  __device__ static __forceinline__ const void *pick(const void *p0, const void *p1, const void *p2, int m) {
    return (const void *)((uintptr_t)p0 * (uintptr_t)(m == 0) + (uintptr_t)p1 * (uintptr_t)(m == 1) + (uintptr_t)p2 * (uintptr_t)(m == 2));
  }
  __device__ static __forceinline__ const void *wbase(const GemvArgs &a, int m, int j) { return NM == 2 ? pick(a.w0, a.w1, a.w2, j) : pick(a.w0, a.w1, a.w2, m); }
  __device__ static __forceinline__ const void *sbase(const GemvArgs &a, int m, int j) { return NM == 2 ? pick(a.s0, a.s1, a.s2, j) : pick(a.s0, a.s1, a.s2, m); }
  __device__ static __forceinline__ int ngroups(const GemvArgs &a) {
    return ((EPI == EPI_SWIGLU ? a.rows0 : a.rows0 + a.rows1 + a.rows2) + ROWS - 1) / ROWS;
  }
  __device__ static __forceinline__ int nbatch(const GemvArgs &a) { return ((a.in_f + STEP - 1) / STEP + UNROLL - 1) / UNROLL; }
  // LDS elements the staged x needs: in_f rounded up to whole batches (host side)
  static int x_elems(int in_f) { return (((in_f + STEP - 1) / STEP + UNROLL - 1) / UNROLL) * UNROLL * STEP; }

  // Row groups are dealt to the wavefronts of the grid in order: wavefront w of block blk (of nblk) takes groups
  // (blk * nw + w) + nblk * nw * i, i = 0, 1, ...  The wavefronts of a block then stream neighbouring rows (one contiguous
  // piece of the matrix at a time, which the memory system rewards: dealt block by block, rows nblk apart, the SwiGLU launch
  // measured 6 % slower).
  __device__ static __forceinline__ int first_group(int blk, int nblk) { (void)nblk; return blk * (int)(blockDim.x >> 6) + (int)(threadIdx.x >> 6); }

  // Issue the loads of item (grp, b), if it exists.
  // Not STRAIGHT: an item that does not exist is a branch around this function.  Where a path with requests and a path
  // without them meet, the compiler's wait counts have to hold for both, i.e. they are those of the path WITHOUT the
  // requests: a buffer is then waited for as if nothing had been requested after it, a wait that takes in most of the
  // requests that were (the other buffer, just sent).
  // STRAIGHT: straight-line code.  An item that does not exist asks for nothing through the buffer descriptor (no memory
  // request, but its place among the outstanding loads) and reads its few scalars from a clamped, valid row; the row's
  // scale, residual element or rotary pair are asked for with every item, not only with the last batch of a row.  Every
  // wait after it is then the exact count; the price is the address arithmetic of an item that does not exist.
  // Which requests are straight-line (EXACT, chosen by the host from the items a wavefront of the launch walks): the first
  // item always; the second when every wavefront has two (EXACT >= 1); those inside the loop when it has three or more
  // (EXACT >= 2).
  __device__ static __forceinline__ void load_item(const GemvArgs &a, Buf &buf, int grp, int b, int pos, bool exists = true) { load_item_as<(EXACT >= 2)>(a, buf, grp, b, pos, exists); }
  template <bool STRAIGHT> __device__ static __forceinline__ void load_item_as(const GemvArgs &a, Buf &buf, int grp, int b, int pos, bool exists) {
    if constexpr (!STRAIGHT) {
      if (!exists) return;
    }
    const int lane = threadIdx.x & 63, in_f = a.in_f;
    const Where w = locate(a, grp);
    __amdgpu_buffer_rsrc_t rs[NM];
#pragma unroll
    for (int j = 0; j < NM; j++) rs[j] = wave_buffer(wbase(a, w.m, j), (uint32_t)(((size_t)w.mrows * (size_t)in_f * BITS) / 8));   // below 4 GiB: host-checked
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      // Lanes past the end of the row reload its last vector instead of branching around the load (their x is zero,
      // see stage_x): a load under a lane mask makes the compiler wait for every outstanding load at the join.
      int k = (b * UNROLL + u) * STEP + lane * VEC;
      k = k < in_f ? k : in_f - VEC;
#pragma unroll
      for (int j = 0; j < NM; j++)
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
          const int row = w.r0 + r < w.mrows ? w.r0 + r : w.mrows - 1;  // tail rows reload the last row, never stored
          const size_t el = (size_t)row * in_f + (size_t)k;
          buf.w[wi(u, j, r)] = buf_stream16(rs[j], (STRAIGHT && !exists) ? BUF_END : (uint32_t)((el * BITS) / 8));
          if constexpr (KIND == JSGRAD_W_NF4) buf.nscale[wi(u, j, r)] = ldg((const _Float16 *)sbase(a, w.m, j) + (el >> 6));
        }
    }
    if constexpr (!STRAIGHT) {
      if (b != nbatch(a) - 1) return;
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      const int row = w.r0 + r < w.mrows ? w.r0 + r : w.mrows - 1;
      if constexpr (KIND == JSGRAD_W_I8) {
#pragma unroll
        for (int j = 0; j < NM; j++) buf.scale[si(j, r)] = ldg((const _Float16 *)sbase(a, w.m, j) + row);
      }
      if constexpr (EPI == EPI_STORE) {
        // no residual: read element 0 of x instead (always readable; the value is not used), so that there is one
        // straight-line load here and no branch for the register allocator to merge
        const uintptr_t has = a.residual != nullptr;
        const AT *res = (const AT *)((uintptr_t)a.residual * has + (uintptr_t)a.x * (1 - has)) + (size_t)row * has;
        if constexpr (COHERENT) set_extra(buf, r, ld_coherent(res));
        else set_extra(buf, r, ldg(res));
      } else if constexpr (EPI == EPI_ROPE_KV) {
        // table row `pos`, entry (cos, sin) of pair i = (row % head_dim) / 2: even r gets cos, odd r gets sin
        const bool ok = pos >= 0 && pos < a.max_context;
        const int i = (row % a.head_dim) >> 1;
        set_extra(buf, r, ((const AT *)a.rope_table)[ok ? (size_t)pos * a.head_dim + 2 * i + (r & 1) : 0]);
      }
    }
  }

  // the first item of this wavefront, requested ahead of run()
  __device__ static __forceinline__ void prefetch(const GemvArgs &a, Buf &buf, int pos) {
    const int grp = first_group(blockIdx.x, gridDim.x);
    load_item(a, buf, grp, 0, pos, grp < ngroups(a));
  }

  // Ask for one dword of every 128-byte line of items [first, first + DEPTH) of this wavefront's sequence without
  // waiting for it, so that the lines sit in this XCD's L2 when load_item() wants them (item 0 is what prefetch()
  // loads).  One load instruction covers one item: 8 vectors x 8 lines = 64 lanes.  The loads are issued from inline
  // assembly, so the compiler does not know they are in flight: the caller must run touch_wait() before it reads t[].
  template <int DEPTH> __device__ static __forceinline__ void touch(const GemvArgs &a, int first, uint32_t (&t)[DEPTH]) {
    const int lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    const int ng = ngroups(a), nb = nbatch(a), gstride = gridDim.x * nw;
    int grp = first_group(blockIdx.x, gridDim.x), b = 0;
    const int v = lane >> 3, line = lane & 7;
    const int u = v / (NM * ROWS), j = (v / ROWS) % NM, r = v % ROWS;
    for (int i = 0; i < first; i++)
      if (++b == nb) { b = 0; grp += gstride; }
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      t[d] = 0;
      if (grp < ng) {
        const Where w = locate(a, grp);
        const int k = (b * UNROLL + u) * STEP + line * (1024 / BITS);   // first element of this lane's 128-byte line
        if (k < a.in_f) {
          const int row = w.r0 + r < w.mrows ? w.r0 + r : w.mrows - 1;
          const char *p = (const char *)wbase(a, w.m, j) + (((size_t)row * a.in_f + (size_t)k) * BITS) / 8;
          asm volatile("global_load_dword %0, %1, off" : "=v"(t[d]) : "v"(p) : "memory");
        }
      }
      if (++b == nb) { b = 0; grp += gstride; }
    }
  }
  // wait for every outstanding load of this wavefront (touch() loads included) and fold the touched words into `sink`
  template <int DEPTH> __device__ static __forceinline__ void touch_wait(uint32_t (&t)[DEPTH], uint32_t &sink) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int d = 0; d < DEPTH; d++) sink ^= t[d];
  }

  __device__ static __forceinline__ void store_out(AT *p, float v) {
    if constexpr (COHERENT) st_coherent(p, (AT)v);
    else *p = (AT)v;
  }

  // consume item (grp, b) from buf; on the last batch of the group: cross-lane sum, scale, cast, epilogue
  __device__ static __forceinline__ void use_item(const GemvArgs &a, const Buf &buf, int grp, int b, float (&acc)[NM][ROWS], const AT *xs, const float *lut, int pos) {
    const int lane = threadIdx.x & 63;
    const Where w = locate(a, grp);
    if (b == 0) {
#pragma unroll
      for (int j = 0; j < NM; j++)
#pragma unroll
        for (int r = 0; r < ROWS; r++) acc[j][r] = 0.0f;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      // a k-step that lies wholly behind the end of the row (the last batch of a row whose length is not a multiple of the
      // batch) has only reloaded vectors against zero padding: nothing to add.  The same for every lane: a scalar branch.
      if ((b * UNROLL + u) * STEP >= a.in_f) continue;
      const int k = (b * UNROLL + u) * STEP + lane * VEC;   // may lie in the zero padding of xs
      XFrag<AT, VEC> xf;
      xf.load(xs + k);
      if constexpr (WIDE && KIND == JSGRAD_W_NF4 && sizeof(AT) == 2) {
        // The NM x ROWS vectors of this k-step in stages of eight weight bytes: the table look-ups of stage s + 1 are sent
        // before the products of stage s are formed.  Written vector by vector, every wavefront asks the table for eight
        // entries and then waits for them with nothing else to do, and the wavefronts of a CU do so in step: the vector
        // ALUs and the LDS pipe took turns (counted: each busy 44 % of the launch, and the launch as long as both together).
        constexpr int NVU = NM * ROWS, NST = NVU * 2;
        const char *tab = (const char *)lut + NF4_TAB_OFFSET;
        const uint32_t lane4 = (uint32_t)lane << 2;
        uint32_t ent[2][8];
        float sv[NVU];
#pragma unroll
        for (int v = 0; v < NVU; v++) sv[v] = 0.0f;
        auto issue = [&](int st, uint32_t (&e)[8]) {
          const u4_t wv = buf.w[wi(u, 0, 0) + (st >> 1)];      // wi(u, j, r) = wi(u, 0, 0) + j * ROWS + r
#pragma unroll
          for (int q = 0; q < 2; q++) {
            const uint32_t d = wv[(st & 1) * 2 + q];
#pragma unroll
            for (int bb = 0; bb < 4; bb++) e[q * 4 + bb] = *(const uint32_t *)(tab + __builtin_amdgcn_perm(lane4, d, 0x0c0c0004u | ((uint32_t)bb << 8)));
          }
        };
        issue(0, ent[0]);
#pragma unroll
        for (int st = 0; st < NST; st++) {
          if (st + 1 < NST) issue(st + 1, ent[(st + 1) & 1]);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int q = 0; q < 2; q++)
#pragma unroll
            for (int bb = 0; bb < 4; bb++)
              sv[st >> 1] = __builtin_amdgcn_fdot2(as_h2(ent[st & 1][q * 4 + bb]), xf.v[((st & 1) * 2 + q) * 4 + bb], sv[st >> 1], false);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NM; j++)
#pragma unroll
          for (int r = 0; r < ROWS; r++) acc[j][r] += sv[j * ROWS + r] * (float)buf.nscale[wi(u, j, r)];
      } else {
#pragma unroll
        for (int j = 0; j < NM; j++)
#pragma unroll
          for (int r = 0; r < ROWS; r++) {
            float bs = 1.0f;
            if constexpr (KIND == JSGRAD_W_NF4) bs = (float)buf.nscale[wi(u, j, r)];
            // every 16-byte vector is summed on its own and then added: eight short dependent chains per item
            // instead of two long ones
            acc[j][r] += Dot<KIND, AT>::run(buf.w[wi(u, j, r)], xf, 0.0f, bs, lut);
          }
      }
    }
    if (b != nbatch(a) - 1) return;

    float val[NM][ROWS];
#pragma unroll
    for (int j = 0; j < NM; j++)
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        float v = wave_sum(acc[j][r]);
        if constexpr (KIND == JSGRAD_W_I8) v = v * (float)buf.scale[si(j, r)];
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
          if (has_res) v = Act<AT>::rn(extra_of<AT>(buf, r) + v);
          store_out(y + r0 + r, v);
        }
    } else if constexpr (EPI == EPI_SWIGLU) {
      AT *g = (AT *)a.y;
#pragma unroll
      for (int r = 0; r < ROWS; r++)
        if (lane == r && r0 + r < mrows) store_out(g + r0 + r, Act<AT>::rn(silu_act<AT>(val[0][r]) * val[1][r]));
    } else {
      if (pos < 0 || pos >= a.max_context) return;  // never write outside the cache
      if (w.m == 2) {  // value rows: plain copy into the cache row
        AT *cv = (AT *)a.cache_v + (size_t)pos * a.rows2;
#pragma unroll
        for (int r = 0; r < ROWS; r++)
          if (lane == r && r0 + r < mrows) store_out(cv + r0 + r, val[0][r]);
      } else {         // query / key rows: rotate interleaved pairs (llama.ts:17-32)
        AT *dst = w.m == 0 ? (AT *)a.y : (AT *)a.cache_k + (size_t)pos * a.rows1;
#pragma unroll
        for (int r = 0; r < ROWS; r += 2)
          if (lane == r && r0 + r + 1 < mrows) {
            const float c = extra_of<AT>(buf, r), d = extra_of<AT>(buf, r + 1);
            const float av = val[0][r], bv = val[0][r + 1];
            store_out(dst + r0 + r, Act<AT>::rn(av * c - bv * d));  // the build keeps a*b+c unfused: two roundings as in plain C
            store_out(dst + r0 + r + 1, Act<AT>::rn(av * d + bv * c));
          }
      }
    }
  }

  // the NF4 tables in LDS (published by the barrier at the end of stage_x).  The code values come from literals
  // (nf4_code_bits): read from a table in memory they cost a round trip at the head of every launch.
  __device__ static __forceinline__ void fill_lut(float *lut) {
    if constexpr (KIND == JSGRAD_W_NF4) {
      if (threadIdx.x < 16) lut[threadIdx.x] = (float)__builtin_bit_cast(_Float16, (uint16_t)nf4_code_bits(threadIdx.x));
      if constexpr (sizeof(AT) == 2) {   // the table of code pairs, one entry per byte value: element 2j (the high nibble) in the low half
        if constexpr (WIDE) {            // ... and per lane: entry e is a 256-byte row of 64 copies; neighbouring lanes write
          u4_t *tab = (u4_t *)((char *)lut + NF4_TAB_OFFSET);   // neighbouring 16 bytes
          for (int i = threadIdx.x; i < 256 * 16; i += blockDim.x) {
            const int e = i >> 4;
            const uint32_t w = nf4_code_bits(e >> 4) | (nf4_code_bits(e & 15) << 16);
            tab[i] = u4_t{w, w, w, w};
          }
        } else {
          for (int e = threadIdx.x; e < 256; e += blockDim.x) ((uint32_t *)lut)[16 + e] = nf4_code_bits(e >> 4) | (nf4_code_bits(e & 15) << 16);
        }
      }
    }
  }

  // xs: LDS for in_f activations; red: LDS float[blockDim/64]; lut: LDS float[16] (NF4 code book, written here), and for
  // NF4 weights with fp16 activations NF4_LUT_WORDS words (the table of code pairs behind it)
  // EARLY_X: the input row exists when the kernel starts (it is not produced inside this launch): request it first.
  // blk / nblk: this block's index among the nblk blocks that share the rows (the whole grid unless the caller says otherwise).
  template <bool EARLY_X = false>
  __device__ static __forceinline__ void run(const GemvArgs &a, AT *xs, float *red, float *lut, Buf &bufA, bool preloaded, int pos, int blk = blockIdx.x,
                                             int nblk = gridDim.x) {
    const int nw = blockDim.x >> 6;
    const int ng = ngroups(a), nb = nbatch(a);
    // Which row groups this wavefront walks: group first_group + i * (all wavefronts of the launch).  WIDE (one block of
    // sixteen wavefronts per CU): every block takes one contiguous stretch of ceil(ng / nblk) groups and deals it to its
    // wavefronts in turn, so that all blocks carry the same load and the wavefronts that come last in their CU's request queue
    // are the ones with one item fewer (dealt launch-wide, 7168 groups over 256 blocks gave three quarters of the CUs 32
    // items and the rest 16).
    int gstride = nblk * nw, lim = ng, g0 = first_group(blk, nblk);
    if constexpr (WIDE) {
      const int per = (ng + nblk - 1) / nblk;
      g0 = blk * per + (int)(threadIdx.x >> 6);
      lim = (blk + 1) * per < ng ? (blk + 1) * per : ng;
      gstride = nw;
    }
    XStage xst;
    if constexpr (EARLY_X) stage_x_issue<AT>(a, xst);
    fill_lut(lut);
    JSG_LSTAMP(5);
    JSG_LMAX(26);
    int grp = g0, b = 0;
    auto advance = [&](int &g, int &bb) {
      if (++bb == nb) { bb = 0; g += gstride; }
    };
    Buf bufB;
    int gB = grp, bB = b;
    advance(gB, bB);
    // the first item is straight-line code in every launch (the staging of x below then waits for x and not for it)
    if (!preloaded) load_item_as<true>(a, bufA, grp, 0, pos, grp < lim);
    JSG_LSTAMP(6);
    JSG_LMAX(27);
    // block-wide, ends with a barrier (which also publishes lut)
    if constexpr (EARLY_X) {
      // x is back after one round trip; its registers are free again before the second item's are needed
      stage_x_finish<AT>(a, xst, xs, red, nb * UNROLL * STEP);
      load_item_as<(EXACT >= 1)>(a, bufB, gB, bB, pos, gB < lim);
    } else {
      // the second item goes out before x is staged too: staging (a read of x, the RMSNorm reduction, a block barrier)
      // would otherwise be a stretch with nothing new in flight
      load_item_as<(EXACT >= 1)>(a, bufB, gB, bB, pos, gB < lim);
      stage_x<AT, COHERENT>(a, xs, red, nb * UNROLL * STEP);
    }

    float acc[NM][ROWS];
    JSG_LSTAMP(23);
    while (grp < lim) {
      use_item(a, bufA, grp, b, acc, xs, lut, pos);
      JSG_LSTAMP(24);
      if (gB >= lim) break;
      grp = gB; b = bB;
      advance(grp, b);                                   // the item after B goes into A
      load_item(a, bufA, grp, b, pos, grp < lim);
      use_item(a, bufB, gB, bB, acc, xs, lut, pos);
      JSG_LSTAMP(25);
      gB = grp; bB = b;
      advance(gB, bB);                                   // and the one after that into B
      load_item(a, bufB, gB, bB, pos, grp < lim && gB < lim);
    }
  }
};

}  // namespace jsg
