// The feed-forward block of one layer in ONE launch: ffn_norm + w1, w3 + SwiGLU, then w2 + residual
// (FeedForward.call, models/llama.ts:108-110, with the residual add of :126).
//
// As two launches the pair pays a kernel boundary between the two matrices: the first one drains, the second is dispatched,
// requests its first weights and waits a memory round trip for them, and w2 has so few rows that its launch is little more
// than that ramp.  Here every wavefront that has finished its rows of w1 / w3 requests its first two items of w2 at once, so
// the weight stream goes on while the slowest block still works on the gate; the gate row g travels to all blocks as tagged
// words (value | version tag, common.h): a block asks for the row until every word carries the tag of this launch.
//
// One block of 16 wavefronts per CU, so that the row is fetched by as many blocks as there are CUs and not four times as
// many.  Every block both produces a part of g and waits for all of it, so all blocks must be on the device together: the
// grid is at most what the device holds at once (checked against the occupancy calculator on the host).  The wait is
// bounded all the same and reports through an error word.
#include "gemv_core.h"

namespace jsg {

constexpr int FFN_THREADS = 1024;
constexpr int FFN_WAVES = FFN_THREADS / 64;

template <int KIND>
__global__ __launch_bounds__(FFN_THREADS) void ffn_kernel(GemvArgs a1, GemvArgs a2, int layer) {
  typedef _Float16 AT;
  typedef Gemv<KIND, AT, EPI_SWIGLU, 2, 2, false> G1;
  typedef Gemv<KIND, AT, EPI_STORE, 2, 4, false> G2;
  extern __shared__ __align__(16) unsigned char smem[];   // the staged input row: x for w1 / w3, then g for w2
  __shared__ float red[FFN_WAVES];
  __shared__ float lut[16];

  // the version of this launch's g row: no other launch that writes the row has it (another layer, or another position)
  const int pos = a1.st[1];
  const uint32_t tag = tw_tag(pos * 128 + layer);
  a1.y_tag = tag;
  a2.x_tag = tag;

  GemvBuf buf;
  G1::template run<true>(a1, (AT *)smem, red, lut, buf, false, 0);
  // This wavefront is done with the gate rows; its first w2 items go out inside run(), before it waits for g.  The staged x is
  // not touched before every wavefront of the block has arrived at the barrier inside the staging of g (the zero padding
  // written before that barrier lies behind the end of g, far behind the end of x).
  G2::template run<false>(a2, (AT *)smem, red, lut, buf, false, 0);
}

template <int KIND> static int ffn_capacity(size_t lds, int *out) {
  int per_cu = 0;
  JSG_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)ffn_kernel<KIND>, FFN_THREADS, lds));
  *out = per_cu * state().cu_count;
  return 0;
}

template <int KIND> static int launch_ffn(const GemvArgs &a1, const GemvArgs &a2, int layer) {
  typedef Gemv<KIND, _Float16, EPI_SWIGLU, 2, 2, false> G1;
  typedef Gemv<KIND, _Float16, EPI_STORE, 2, 4, false> G2;
  const size_t e1 = G1::x_elems(a1.in_f), e2 = G2::x_elems(a2.in_f);
  const size_t lds = (e1 > e2 ? e1 : e2) * sizeof(_Float16);
  static int capacity = 0;
  static size_t capacity_lds = 0;
  if (capacity == 0 || capacity_lds != lds) {
    if (int e = ffn_capacity<KIND>(lds, &capacity)) return e;
    capacity_lds = lds;
  }
  const int ngroups = (a1.rows0 + 1) / 2, need = (ngroups + FFN_WAVES - 1) / FFN_WAVES;
  int blocks = need < state().cu_count ? need : state().cu_count;
  JSG_REQUIRE(capacity >= 1, "jsgrad_hip_ffn: the kernel does not fit a CU with %zu bytes of LDS", lds);
  if (blocks > capacity) blocks = capacity;      // every block waits for all the others: all must be resident
  JSG_LAUNCH(PROF_FFN, (ffn_kernel<KIND>), dim3(blocks), dim3(FFN_THREADS), lds, a1, a2, layer);
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_ffn_workspace_bytes(int hidden) {
  // [0, 256): error word; then the gate row as tagged words
  return 256 + (size_t)hidden * sizeof(uint32_t);
}

int jsgrad_hip_ffn(int kind, const void *w1, const void *s1, const void *w3, const void *s3, const void *w2, const void *s2, const void *x,
                   const void *norm_weight, float eps, void *y, int dim, int hidden, const int32_t *st, void *workspace, int layer) {
  JSG_READY();
  JSG_REQUIRE(w1 && w3 && w2 && x && norm_weight && y && st && workspace, "jsgrad_hip_ffn: null pointer argument");
  JSG_REQUIRE(kind == JSGRAD_W_F16 || kind == JSGRAD_W_I8, "jsgrad_hip_ffn: weight kind %d (fp16 and int8 are built)", kind);
  JSG_REQUIRE(kind == JSGRAD_W_F16 || (s1 && s3 && s2), "jsgrad_hip_ffn: quantised weights need scales");
  JSG_REQUIRE(y != x, "jsgrad_hip_ffn: output must not alias the input");
  JSG_REQUIRE(layer >= 0 && layer < 128, "jsgrad_hip_ffn: layer index %d", layer);
  JSG_REQUIRE(dim > 0 && dim % 16 == 0 && dim <= 4 * 1024 * 8, "jsgrad_hip_ffn: dim %d (a multiple of 16, at most %d for the fused RMSNorm)", dim, 4 * 1024 * 8);
  JSG_REQUIRE(hidden > 0 && hidden % 16 == 0 && (size_t)hidden * 2 <= 64 * 1024, "jsgrad_hip_ffn: hidden %d (a multiple of 16 that fits the 64 KiB staging buffer)", hidden);
  char *ws = (char *)workspace;
  GemvArgs a1 = {};
  a1.w0 = w1; a1.s0 = s1; a1.w1 = w3; a1.s1 = s3; a1.rows0 = hidden; a1.rows1 = hidden; a1.in_f = dim; a1.x = x;
  a1.norm_w = norm_weight; a1.eps = eps; a1.inv_d = (float)(1.0 / (double)dim); a1.y = nullptr; a1.st = st;
  a1.y_tagged = (uint32_t *)(ws + 256);
  GemvArgs a2 = {};
  a2.w0 = w2; a2.s0 = s2; a2.rows0 = dim; a2.in_f = hidden; a2.norm_w = nullptr; a2.eps = 0.0f; a2.inv_d = (float)(1.0 / (double)hidden);
  a2.y = y; a2.residual = x;
  a2.x_tagged = (const uint32_t *)(ws + 256);
  a2.x = x;   // never read as the input; a readable address
  a2.err = (int *)ws;
  switch (kind) {
    case JSGRAD_W_F16: return launch_ffn<JSGRAD_W_F16>(a1, a2, layer);
    case JSGRAD_W_I8: return launch_ffn<JSGRAD_W_I8>(a1, a2, layer);
  }
  return fail("jsgrad_hip_ffn: weight kind %d", kind);
}

int jsgrad_hip_ffn_status(const void *workspace, int *host_out_error) {
  JSG_READY();
  JSG_REQUIRE(workspace && host_out_error, "jsgrad_hip_ffn_status: null pointer");
  JSG_REQUIRE(!state().capturing, "jsgrad_hip_ffn_status during graph capture");
  JSG_HIP(hipMemcpyAsync(host_out_error, workspace, sizeof(int), hipMemcpyDeviceToHost, state().stream));
  JSG_HIP(hipStreamSynchronize(state().stream));
  return 0;
}

}  // extern "C"
