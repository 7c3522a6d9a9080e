// Stand-alone one-row linear kernels: one launch per Linear / fused group of Linears (see gemv_core.h).
#include <stdlib.h>

#include "gemv_core.h"

namespace jsg {

// fp16 activations: 16 wavefronts per CU (128 registers per lane), which the grid is sized for: four blocks of four (NW = 4), or,
// for NF4 launches with rows enough for that on every CU, one block of sixteen around a per-lane look-up table of 64 KiB
// (NW = 16, Gemv<..., WIDE>).
// EXACT: see Gemv::load_item; the host picks it from the items a wavefront of the launch walks
// traced builds: the three blocks whose stamps are kept (first, middle, last unless the build says otherwise)
#ifndef JSG_TRACE_ROWS
#define JSG_TRACE_ROWS(b, n) ((b) == 0 ? 0 : ((b) == (n) / 2 ? 1 : ((b) == (n) - 1 ? 2 : -1)))
#endif
template <int KIND, typename AT> constexpr bool gemv_may_be_wide() { return KIND == JSGRAD_W_NF4 && sizeof(AT) == 2; }
template <int KIND, typename AT, int EPI, int ROWS, int UNROLL, int EXACT, int NW = 4>
__global__ __launch_bounds__(64 * NW, sizeof(AT) == 2 ? 4 : 1) void gemv_kernel(GemvArgs a) {
  constexpr bool WIDE = NW == 16;
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ float red[16];
  __shared__ float lut[KIND == JSGRAD_W_NF4 ? (WIDE ? NF4_WIDE_LUT_WORDS : NF4_LUT_WORDS) : 16];
  typedef Gemv<KIND, AT, EPI, ROWS, UNROLL, false, EXACT, WIDE> G;
  // read the position now, not in the epilogue: the load then overlaps the weight stream instead of ending the kernel
  JSG_LCLEAR();
  const int pos = EPI == EPI_ROPE_KV ? a.st[1] : 0;
  JSG_LSTAMP(0);
  GemvBuf buf;
  G::template run<true>(a, (AT *)smem, red, lut, buf, false, pos);
  JSG_LSTAMP(8);
  JSG_LALL(2, true);
  JSG_LFLUSH(JSG_TRACE_ROWS((int)blockIdx.x, (int)gridDim.x));
}
JSG_TRACE_ENTRY(jsgrad_hip_gemv_trace)

// ---- host-side dispatch ------------------------------------------------------------------------

template <int KIND, typename AT, int EPI, int ROWS, int UNROLL, int NW = 4> static int launch_cfg(const GemvArgs &a, int total_rows) {
  constexpr int kind = EPI == EPI_STORE ? PROF_LINEAR : (EPI == EPI_SWIGLU ? PROF_FFN_GATE : PROF_QKV_ROPE);
  const int ngroups = (total_rows + ROWS - 1) / ROWS;
  if constexpr (gemv_may_be_wide<KIND, AT>() && NW == 4) {
    // rows enough to give every CU a block of sixteen wavefronts: the per-lane table (measured on the 8B shapes: w1 | w3
    // 20.0 -> 17.2 us; with fewer rows the launch is a few microseconds either way and the larger block's staging costs more)
    static const int force = getenv("JSG_NF4_WAVES") ? atoi(getenv("JSG_NF4_WAVES")) : 0;
    if (force ? force == 16 : ngroups >= 16 * state().cu_count) return launch_cfg<KIND, AT, EPI, ROWS, UNROLL, 16>(a, total_rows);
  }
  const int need = (ngroups + NW - 1) / NW;      // one group per wavefront
  static const int waves_per_cu = getenv("JSG_GEMV_BLOCKS_PER_CU") ? 4 * atoi(getenv("JSG_GEMV_BLOCKS_PER_CU")) : 16;
  // 16 resident wavefronts per CU; more rows than that are walked grid-stride
  const int cap = state().cu_count * (waves_per_cu / NW > 0 ? waves_per_cu / NW : 1);
  dim3 grid(need < cap ? need : cap), block(NW * 64);
  typedef Gemv<KIND, AT, EPI, ROWS, UNROLL, false> G;
  const int most_rows = a.rows0 > a.rows1 ? (a.rows0 > a.rows2 ? a.rows0 : a.rows2) : (a.rows1 > a.rows2 ? a.rows1 : a.rows2);
  JSG_REQUIRE(fits_buffer_offsets((size_t)most_rows, (size_t)a.in_f, G::BITS), "one-row Linear: a weight matrix of %d x %d elements reaches 4 GiB (32-bit byte offsets)", most_rows, a.in_f);
  size_t lds = (size_t)G::x_elems(a.in_f) * sizeof(AT);
  // items a wavefront walks: its row groups (dealt grid-stride) x the batches of a row
  const int waves = (int)grid.x * NW;
  const int nbatch = G::x_elems(a.in_f) / (UNROLL * G::STEP);
  const int items = ((ngroups + waves - 1) / waves) * nbatch;
  if constexpr (NW == 16) {
    // the look-up table is static LDS of more than 64 KiB: the staged row on top of it is dynamic LDS the runtime must be told about
    static bool told = false;
    if (!told) {
      const int most = 64 * 1024;
      JSG_HIP(hipFuncSetAttribute((const void *)gemv_kernel<KIND, AT, EPI, ROWS, UNROLL, 0, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
      JSG_HIP(hipFuncSetAttribute((const void *)gemv_kernel<KIND, AT, EPI, ROWS, UNROLL, 1, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
      JSG_HIP(hipFuncSetAttribute((const void *)gemv_kernel<KIND, AT, EPI, ROWS, UNROLL, 2, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
      told = true;
    }
  }
  // the second request is straight-line code where every wavefront has a second item, and also where only some have (rows
  // of one batch, more row groups than wavefronts): a wavefront whose second request sits behind a test waits for both
  // items before it starts on the first, which costs the launch more than the others' address arithmetic for nothing
  if (items >= 3) JSG_LAUNCH(kind, (gemv_kernel<KIND, AT, EPI, ROWS, UNROLL, 2, NW>), grid, block, lds, a);
  else if (nbatch >= 2 || ngroups > waves) JSG_LAUNCH(kind, (gemv_kernel<KIND, AT, EPI, ROWS, UNROLL, 1, NW>), grid, block, lds, a);
  else JSG_LAUNCH(kind, (gemv_kernel<KIND, AT, EPI, ROWS, UNROLL, 0, NW>), grid, block, lds, a);
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
  a.w0 = w; a.s0 = scale; a.rows0 = out_f; a.in_f = in_f; a.x = x; a.norm_w = norm_weight; a.eps = eps;
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
  a.w0 = w1; a.s0 = s1; a.w1 = w3; a.s1 = s3; a.rows0 = hidden; a.rows1 = hidden; a.in_f = dim; a.x = x;
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
  a.w0 = wq; a.s0 = sq; a.w1 = wk; a.s1 = sk; a.w2 = wv; a.s2 = sv;
  a.rows0 = n_heads * head_dim; a.rows1 = n_kv_heads * head_dim; a.rows2 = n_kv_heads * head_dim;
  a.in_f = dim; a.x = x; a.norm_w = norm_weight; a.eps = eps; a.inv_d = (float)(1.0 / (double)dim); a.y = q_out;
  a.rope_table = rope_table; a.st = st; a.cache_k = cache_k; a.cache_v = cache_v; a.head_dim = head_dim; a.max_context = max_context;
  return dispatch<EPI_ROPE_KV>(kind, act, a, a.rows0 + a.rows1 + a.rows2);
}

}  // extern "C"
