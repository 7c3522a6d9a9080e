// Device code of decode-time grouped-query attention over the HBM-resident KV cache for gfx950, shared by the
// stand-alone kernel (attention.hip) and the whole-step kernel (decode_step.hip).
//
// One new query position against cache rows [0, T), T = start_pos + 1: repeat_kv + scaled_dot_product_attention of the
// reference (/root/reference/jsgrad/models/llama.ts:89-95, /root/reference/jsgrad/tensor.ts:3920-3934).  Scores, the
// softmax and the P.V sum are float32; the exponential is the reference's polynomial exp2 (ops.ts:1650-1673).
//
// A work item is (kv head g, chunk `split` of the positions).  The block that runs it serves all n_rep query heads of
// the kv head from a single read of K and V (the GQA saving): a group of HD/EPL lanes covers one cache row with one
// 128-bit load per lane.  Phase 1 writes the chunk's scores to LDS and finds the chunk maximum, phase 2 accumulates
// exp(s - m) and exp(s - m) * V.  The item leaves (m, l, o) in the workspace; the last item of a kv head to finish
// (agent-scope counter) merges the chunks and writes the output rows.
#pragma once
#include "common.h"

namespace jsg {

constexpr int ATT_CHUNK_MAX = 256;  // positions per item held in LDS; also the most chunks the merge can index

// A partial result as a workspace word that says by itself whether it has been written: the complement of the float's bits,
// so that zero means `not yet`.  Only the NaN with all bits set would come out as zero; it is stored as another NaN.
__device__ __forceinline__ uint32_t att_word(float v) {
  const uint32_t b = __float_as_uint(v);
  return ~(b == 0xFFFFFFFFu ? 0x7FC00000u : b);
}

// Rows per chunk for T visible positions.  A launch is a chain of round trips (rows, partial results, merge): the rows of a
// chunk are fetched by one block, which takes time in proportion to the rows, and the merge fetches one partial result per
// chunk, which takes time in proportion to T / rows; the sum is least where rows grows like the square root of T.
// Measured with blocks of 8 wavefronts (tok/s of the whole decode step, chunks of 48 / 64 / 80 / 96 / 128 rows): 1B at 600
// positions 1452 / 1455 / 1438 / 1440 / -; 8B int8 at 584 positions 526 / 526 / 516 / 504 / -; 3B int8 at 1064 positions
// 820 / 815 / 841 / 835 / -; 8B int8 at 2100 positions 467 / 471 / 483 / 481 / 474 (112 rows); at 4100 positions
// 423 / 434 / 437 / 443 / 449.  rows = 2 sqrt(T) in whole 16s, at least ATT_CHUNK_MIN, at most what the block shape takes.
// `cap`: the longest chunk the block shape can take (16 rows per wavefront, at most ATT_CHUNK_MAX; never below 64).
constexpr int ATT_ROWS_SQ_PER_T = 4, ATT_CHUNK_MIN = 48;   // rows^2 = 4 T; ATT_CHUNK_MIN is a multiple of 16
// ceil(T / chunk) without an integer division (dozens of dependent instructions on the device, at the head of a launch
// that is a chain of latencies): an estimate from a reciprocal, made exact by the two loops
__host__ __device__ __forceinline__ int att_chunk_count(int T, int chunk) {
  int n = (int)((float)T * (1.0f / (float)chunk)) + 1;
  while ((n - 1) * chunk >= T) n--;
  while (n * chunk < T) n++;
  return n;
}
// floor(sqrt(K T)) rounded up to a whole 16 is the smallest r = 16 i with K T < (r + 1)^2: a few compares, no square root
__host__ __device__ __forceinline__ int att_policy_rows(int T, int cap) {
  int r = ATT_CHUNK_MIN;
  while (r < cap && ATT_ROWS_SQ_PER_T * T >= (r + 1) * (r + 1)) r += 16;
  return r < cap ? r : cap;
}
// (A launch provides att_max_chunks(max_context, cap) chunks, the most this rule asks for at any T <= max_context, so the
// kernels take the rule as it is.)
// chunks a launch must provide for every T up to max_context.  The rows per chunk never shrink as T grows, so for each
// chunk length r the most chunks are asked for at the largest T that still gets r rows: sqrt(K T) <= r, i.e.
// T <= ((r + 1)^2 - 1) / K (any T for the shortest and up to max_context for the longest).
constexpr int ATT_MERGE_BATCH = 16;    // chunks whose partial sums the merge requests in one round trip
__host__ __device__ __forceinline__ int att_max_chunks(int max_context, int cap);   // below
// Whether a launch for this max_context takes the sliced merge: from three round trips of the plain one on (see Attn::item).
__host__ __device__ __forceinline__ bool att_sliced_merge(int max_context, int cap) { return att_max_chunks(max_context, cap) > 2 * ATT_MERGE_BATCH; }
__host__ __device__ __forceinline__ int att_max_chunks(int max_context, int cap = ATT_CHUNK_MAX) {
  int most = 1;
  for (int r = ATT_CHUNK_MIN; ; r += 16) {
    if (r > cap) r = cap;
    int t_last = ((r + 1) * (r + 1) - 1) / ATT_ROWS_SQ_PER_T;
    if (r == cap || t_last > max_context) t_last = max_context;
    const int n = (t_last + r - 1) / r;
    most = n > most ? n : most;
    if (r == cap || t_last == max_context) break;
  }
  return most;
}

struct AttnArgs {
  const void *q, *cache_k, *cache_v;
  const int32_t *st;
  void *out;
  int *counters;   // [n_kv_heads], zero before the first launch; the merging block leaves them zero
  int *err = nullptr;   // optional: set to 1 when the merging block's bounded wait for the other chunks ran out
  float *partial;  // [n_kv_heads][nsplit][n_rep][HD + 2]
  int n_kv_heads, nsplit, max_context;
  int kv_magic = 0;   // ceil(65536 / n_kv_heads): block id / n_kv_heads = (id * kv_magic) >> 16 for id * n_kv_heads < 65536 (attn_wo.hip)
  float scale;     // float(1 / sqrt(head_dim)) (tensor.ts:3923 `.div(Math.sqrt(d))` = mul by the folded reciprocal)
  // several sequences at the same position (grid z): distance between consecutive sequences, in bytes (q, out, caches)
  // and in elements (counters, partial); zero for a single sequence
  size_t q_bstride = 0, cache_bstride = 0, partial_bstride = 0;
  // when set, the merged output goes here as tagged words (value | out_tag << 16) for other blocks of the same launch
  uint32_t *out_tagged = nullptr;
  uint32_t out_tag = 0;
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

// NW wavefronts per block.  COHERENT: q and the output cross between blocks of the same launch.
//
// Lane mappings.  Scores: a group of G = HD/EPL lanes covers one K row with one 128-bit load per lane (RPI = 64/G rows per
// wavefront load); the dot products are reduced inside the group with DPP.  P.V: a lane takes ONE dword of a V row, so the 64
// lanes cover a whole row (or two rows of 32 dwords) and every lane accumulates its own output elements over the rows of
// its wavefront: no reduction across lanes at the end (with 16 wavefronts a CU that alone would cost as much as the item).
// SLICED: the merge of a kv head's chunks is shared by several threads per output element (below); chosen by the host for
// contexts long enough to need it (att_sliced_merge), because the larger code costs the short ones a little.
template <typename AT, int HD, int NREP, int NW, bool COHERENT, bool SLICED = false> struct Attn {
  static constexpr int EPL = 16 / sizeof(AT);  // K: elements per lane per 128-bit load
  static constexpr int G = HD / EPL;           // K: lanes per cache row
  static constexpr int RPI = 64 / G;           // K: rows per wavefront load
  // Every row of a chunk is requested up front, 16 rows per wavefront at most: the longest chunk this block shape takes.
  // Sixteen wavefronts (one sequence: few items, each a chain of dependent steps that the launch waits for) take 256 rows;
  // smaller blocks (many sequences: many items, several blocks per CU overlapping their chains) take shorter chunks.
  static constexpr int CHUNK_CAP = NW * 16 < ATT_CHUNK_MAX ? NW * 16 : ATT_CHUNK_MAX;
  static constexpr int KIT = (CHUNK_CAP + NW * RPI - 1) / (NW * RPI);   // K loads per lane for the longest chunk
  static constexpr int EP = 4 / sizeof(AT);    // V: elements per dword
  static constexpr int PIECES = HD / EP;       // V: dwords per row
  static constexpr int LPR = PIECES < 64 ? PIECES : 64;   // V: lanes per row
  static constexpr int RPV = 64 / LPR;         // V: rows per wavefront load (1 or 2)
  static constexpr int IPR = PIECES / LPR;     // V: loads per row (1 or 2)
  static constexpr int VROWS = (CHUNK_CAP + NW - 1) / NW;          // rows of the longest chunk per wavefront
  static constexpr int VIT = (VROWS + RPV - 1) / RPV * IPR;        // V loads per lane for the longest chunk
  static_assert(G == 8 || G == 16 || G == 32, "scores are reduced over 8, 16 or 32 lanes per row");
  static_assert(RPV == 1 || RPV == 2, "a V row is 32, 64 or 128 dwords");
  static_assert(KIT <= 8 && VIT <= 32, "all rows of a chunk are requested up front: the block needs enough wavefronts");
  struct Smem {
    float sc[NREP][CHUNK_CAP];   // scores / probabilities of the chunk; in the merge, the weights of up to CHUNK_CAP chunks
    __attribute__((aligned(16))) float o_part[NW][NREP][HD];   // every wavefront's partial output; summed in wavefront order
    float m_sh[NREP], l_sh[NREP];
    __attribute__((aligned(16))) AT qs[NREP][HD];   // the query rows of the kv head
  };

  // T visible positions cut into chunks of `chunk` rows (n_active of them); this call handles chunk `split` of kv head g.
  // Must be called by every thread of the block (it contains barriers).
  // Loads return in the order they were issued, and the block's barriers in front of the partial results wait for every
  // outstanding one: a caller with other loads to issue (weights of a following stage) passes them as `then`, which is
  // called exactly once, when nothing the item still waits for can end up behind them: after the block has published its
  // partial results (and, in the block of chunk 0, merged the kv head).
  struct Nothing { __device__ __forceinline__ void operator()() const {} };
  __device__ static void item(const AttnArgs &a, Smem &sm, int g, int split, int T, int chunk, int n_active) { item(a, sm, g, split, T, chunk, n_active, Nothing()); }
  template <typename Then> __device__ static __forceinline__ void item(const AttnArgs &a, Smem &sm, int g, int split, int T, int chunk, int n_active, Then then) {
    const int t0 = split * chunk, t1 = min(T, t0 + chunk), CH = t1 - t0;   // t1 > t0: the item exists
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = NW * 64;
    const int sub = lane % G, grp = lane / G;
    const size_t row_stride = (size_t)a.n_kv_heads * HD;
    const AT *kbase = (const AT *)a.cache_k + (size_t)g * HD + (size_t)sub * EPL;
    const AT *vbase = (const AT *)a.cache_v + (size_t)g * HD;
    JSG_LSTAMP(10);

    // ---- every request of the item goes out now: the query rows (once per block, 16-byte pieces), then this lane's K rows,
    // then its V dwords.  They come back in that order.
    constexpr int QCH = NREP * HD / EPL;      // 16-byte pieces of the query rows
    u4_t qpiece = u4_t{0, 0, 0, 0};
    if (tid < QCH) {
      const AT *qp = (const AT *)a.q + (size_t)g * NREP * HD + (size_t)tid * EPL;
      if constexpr (COHERENT) {
#pragma unroll
        for (int e = 0; e < 4; e++) qpiece[e] = __hip_atomic_load(as_global<uint32_t>(qp) + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        qpiece = *(const u4_t *)qp;
      }
    }
    u4_t kreg[KIT];
#pragma unroll
    for (int i = 0; i < KIT; i++) {
      if (i * NW * RPI < CH) {                // the same for the whole block
        const int t = t0 + (wave + i * NW) * RPI + grp;
        kreg[i] = *(const u4_t *)(kbase + (size_t)(t < t1 ? t : t1 - 1) * row_stride);
      }
    }
    const int VR = (CH + NW - 1) / NW;        // rows of this chunk per wavefront: wavefront w has rows [w * VR, (w + 1) * VR)
    const int vsel = lane / LPR, vcol = lane % LPR;
    uint32_t vreg[VIT];
#pragma unroll
    for (int i = 0; i < VIT; i++) {
      const int ri = i / IPR, part = i % IPR;
      if (ri * RPV < VR) {                    // the same for the whole block
        const int r = ri * RPV + vsel;
        const int t = t0 + wave * VR + r;
        const bool ok = r < VR && t < t1;
        vreg[i] = *(const uint32_t *)(vbase + (size_t)(ok ? t : t1 - 1) * row_stride + (size_t)(vcol + LPR * part) * EP);
      }
    }

    // ---- phase 1: scores of the chunk.  The query rows are here first: publish them, take this lane's slice.
    if (tid < QCH) ((u4_t *)sm.qs)[tid] = qpiece;
    lds_barrier();
    JSG_LSTAMP(11);
    u4_t qv[NREP];
#pragma unroll
    for (int j = 0; j < NREP; j++) qv[j] = ((const u4_t *)sm.qs)[j * G + sub];
#pragma unroll
    for (int i = 0; i < KIT; i++) {
      if (i * NW * RPI < CH) {
        const int t = t0 + (wave + i * NW) * RPI + grp;
        // all heads' dot products, then their sums over the lane group step by step for all heads together, then one test
        // for the lanes that store: head by head with a test in each, every head waits out its own chain of instructions
        float p[NREP];
#pragma unroll
        for (int j = 0; j < NREP; j++) {
          p[j] = 0.0f;
          if constexpr (sizeof(AT) == 2) {     // packed dot products with float accumulation (the products are exact in float)
#pragma unroll
            for (int e = 0; e < 4; e++) p[j] = __builtin_amdgcn_fdot2(as_h2(qv[j][e]), as_h2(kreg[i][e]), p[j], false);
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++) p[j] = fmaf(__uint_as_float(qv[j][e]), __uint_as_float(kreg[i][e]), p[j]);
          }
        }
#pragma unroll
        for (int j = 0; j < NREP; j++) p[j] = group_sum<G>(p[j]);
        if (sub == 0 && t < t1) {
#pragma unroll
          for (int j = 0; j < NREP; j++) sm.sc[j][t - t0] = p[j] * a.scale;
        }
      }
    }
    lds_barrier();
    JSG_LSTAMP(12);
    // Wavefront j does the whole softmax of head j by itself - maximum, exp, sum - with no barrier in between: lane i holds
    // rows i, i + 64, ... of the chunk.
    for (int j = wave; j < NREP; j += NW) {
      constexpr int PL = (CHUNK_CAP + 63) / 64;
      float sv[PL];
      float m = -INFINITY;
#pragma unroll
      for (int q = 0; q < PL; q++) {
        const int i = lane + 64 * q;
        sv[q] = (q * 64 < CH && i < CH) ? sm.sc[j][i] : -INFINITY;
        m = fmaxf(m, sv[q]);
      }
      m = wave_max(m);
      float l = 0.0f;
#pragma unroll
      for (int q = 0; q < PL; q++) {
        const int i = lane + 64 * q;
        if (q * 64 < CH) {      // the same for the whole wavefront
          const float e = i < CH ? exp_f32(sv[q] - m) : 0.0f;
          if (i < CH) sm.sc[j][i] = e;
          l += e;
        }
      }
      l = wave_sum(l);
      if (lane == 0) { sm.m_sh[j] = m; sm.l_sh[j] = l; }
    }
    lds_barrier();
    JSG_LSTAMP(13);

    // ---- phase 2: o[j][d] = sum_t p[j][t] * V[t][d] over the rows of this wavefront; this lane's elements are
    // d = (vcol + LPR * part) * EP + e
    float of[NREP][IPR][EP];
#pragma unroll
    for (int j = 0; j < NREP; j++)
#pragma unroll
      for (int c = 0; c < IPR; c++)
#pragma unroll
        for (int e = 0; e < EP; e++) of[j][c][e] = 0.0f;
    // The probabilities of PB row steps are read from LDS together, then multiplied: read one step at a time behind the
    // test that skips the steps a short chunk does not have, every step would wait out an LDS round trip of its own.
    constexpr int PB = (NREP * HD >= 512 ? 2 : 4) * IPR;   // loads per batch: 4 row steps, 2 where the sums already fill the registers
#pragma unroll
    for (int i0 = 0; i0 < VIT; i0 += PB) {
      if ((i0 / IPR) * RPV < VR) {             // the same for the whole block
        float pr[PB / IPR][NREP];
        bool okr[PB / IPR];
#pragma unroll
        for (int q = 0; q < PB / IPR; q++) {
          const int r = (i0 / IPR + q) * RPV + vsel;
          const int t = t0 + wave * VR + r;
          okr[q] = r < VR && t < t1;
#pragma unroll
          for (int j = 0; j < NREP; j++) pr[q][j] = sm.sc[j][okr[q] ? t - t0 : 0];
        }
#pragma unroll
        for (int ii = 0; ii < PB; ii++) {
          const int i = i0 + ii;
          if (i < VIT && (i / IPR) * RPV < VR) {   // a step past the wavefront's rows has no value loaded
            const int q = ii / IPR, part = i % IPR;
            float vf[EP];
            if constexpr (sizeof(AT) == 2) { const h2_t h = as_h2(vreg[i]); vf[0] = (float)h[0]; vf[1] = (float)h[1]; }
            else vf[0] = __uint_as_float(vreg[i]);
#pragma unroll
            for (int j = 0; j < NREP; j++) {
              const float p = okr[q] ? pr[q][j] : 0.0f;   // rows past the chunk: an existing row times zero
#pragma unroll
              for (int e = 0; e < EP; e++) of[j][part][e] = fmaf(p, vf[e], of[j][part][e]);
            }
          }
        }
      }
    }
    // two rows per load: the halves of the wavefront hold different rows of the same elements
    if constexpr (RPV == 2) {
#pragma unroll
      for (int j = 0; j < NREP; j++)
#pragma unroll
        for (int c = 0; c < IPR; c++)
#pragma unroll
          for (int e = 0; e < EP; e++) of[j][c][e] = add_xor32(of[j][c][e]);
    }
    // every wavefront leaves its partial output in a slot of its own, one barrier, then each element is the sum over the
    // slots in wavefront order: independent reads, one LDS round trip
    if (vsel == 0) {
#pragma unroll
      for (int j = 0; j < NREP; j++)
#pragma unroll
        for (int c = 0; c < IPR; c++)
#pragma unroll
          for (int e = 0; e < EP; e++) sm.o_part[wave][j][(vcol + LPR * c) * EP + e] = of[j][c][e];
    }
    lds_barrier();
    JSG_LSTAMP(14);
    constexpr int SLOTS = NW;
    // ---- hand-over of the chunk's partial result.
    // WORDS (kernels whose launch is the whole life of the workspace contents, COHERENT false): every 32-bit word says by
    // itself whether it has been written.  The workspace holds zeros; a value is stored as the complement of its bits
    // (att_word), so no block waits for its stores or counts itself in: the block of chunk 0 asks for the words of all chunks
    // until none is zero, and puts the zeros back for the next launch.  The chain store - acknowledge - count - see the count
    // - fetch becomes store - fetch.
    // Otherwise (kernels that run many layers in one launch, where a cleared word could meet the next layer's store) the
    // blocks count themselves in after their stores were acknowledged, and the block of chunk 0 waits for the count.
    constexpr bool WORDS = !COHERENT;
    auto enc = [](float v) { return WORDS ? __uint_as_float(att_word(v)) : v; };
    auto dec = [](uint32_t w) { return __uint_as_float(WORDS ? ~w : w); };
    float *mine = a.partial + ((size_t)g * a.nsplit + split) * NREP * (HD + 2);
    for (int i = tid; i < NREP * HD; i += nthreads) {
      const int j = i / HD, d = i % HD;
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < SLOTS; w++) v += sm.o_part[w][j][d];
      st_coherent(&mine[j * (HD + 2) + d], enc(v));
    }
    if (tid < NREP) {
      st_coherent(&mine[tid * (HD + 2) + HD], enc(sm.m_sh[tid]));
      st_coherent(&mine[tid * (HD + 2) + HD + 1], enc(sm.l_sh[tid]));
    }
    JSG_LSTAMP(15);
    // One way through for every block: the block of chunk 0 merges, then every block calls `then`.  (With an early exit
    // for the others, the compiler placed their `then` in front of the merge and made the merging block wait for its own
    // stores, as if they were `then`'s requests, before it could ask for anybody's results.)
    const bool merges = split == 0;
    if constexpr (WORDS) {
      if (merges) lds_barrier();   // m_sh / l_sh / sc are written again below
    } else {
      __syncthreads();  // every coherent store of the block has been acknowledged
      if (!merges) {
        if (tid == 0) __hip_atomic_fetch_add(&a.counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // nobody waits for the answer
      } else if (n_active > 1) {
        if (tid == 0) {
          // The other chunks' blocks never wait for anything before they count themselves in, and the launch keeps them all on the
          // device, so this wait ends; it is bounded all the same and reports through the error word where one is given.
          int it = 0;
          while (ld_coherent(&a.counters[g]) != n_active - 1) {
            if (++it > (1 << 20)) { if (a.err != nullptr) st_coherent(a.err, 1); break; }
            __builtin_amdgcn_s_sleep(2);
          }
          __hip_atomic_store(&a.counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // zero again for the next launch
        }
        __syncthreads();
      }
    }
    if (merges) {
      // merge.  Every thread owns two neighbouring output elements and requests their partial sums of the first MB chunks
      // right away; while those travel, one wavefront per query head fetches the per-chunk (m, l), turns them into weights
      // exp(m_s - M) and 1/L in LDS; then the sums are folded in chunk order.  One round trip for up to MB chunks.
      // WORDS: a request is repeated while one of its words is still zero.  The other chunks' blocks never wait for anything
      // before they store, and the launch keeps them all on the device, so this ends; it is bounded all the same, reports
      // through the error word where one is given, and the result is then NaN.
      const float *base = a.partial + (size_t)g * a.nsplit * NREP * (HD + 2);
      constexpr int MB = SLICED ? ATT_MERGE_BATCH + 2 : ATT_MERGE_BATCH;   // chunks per batch of requests (sliced: 36 chunks in one batch per slice)
      constexpr int NPAIR = NREP * HD / 2;         // element pairs of this kv head's query heads
      constexpr int POLL_LIMIT = 1 << 18;
      // Folding the chunks is a chain of round trips, one per batch of MB chunks, and a thread folds one pair of output
      // elements.  SLICED: with more threads than pairs, the chunks are cut into slices, thread (slice, pair) folds its
      // slice, and the slices' sums are added in order through LDS.  (4100 positions in chunks of 128 rows: 33 chunks, three
      // round trips for one thread, one for two threads with 17 chunks each.)
      static_assert(NPAIR <= NW * 64, "a thread folds at most one pair");
      constexpr int SL_FIT = (NW * 64) / NPAIR < NW ? (NW * 64) / NPAIR : NW;   // the slices' sums fit the wavefronts' output slots
      constexpr int SL = !SLICED ? 1 : (SL_FIT < 4 ? SL_FIT : 4);
      const int nsl = (SL > 1 && n_active > MB) ? SL : 1;
      const int per = (n_active + nsl - 1) / nsl;
      const int sl = SLICED ? tid / NPAIR : 0, pr = SLICED ? tid - sl * NPAIR : tid;     // this thread's slice and pair
      const int sb = sl * per;
      const bool folds = SLICED ? (sl < nsl && sb < n_active) : tid < NPAIR;
      const int send = (SLICED && folds) ? min(n_active, sb + per) : n_active;   // chunks [sb, send) are this thread's
      // a chunk index past the end stands for the last chunk (of the head for the (m, l) words, of the slice for the sums),
      // whose words are checked and cleared again and enter the sum with weight zero
      auto pair_at = [&](const float *po, int s_) { return po + (size_t)(s_ < send ? s_ : send - 1) * NREP * (HD + 2); };
      auto ml_at = [&](const float *po, int s_) { return po + (size_t)(s_ < n_active ? s_ : n_active - 1) * NREP * (HD + 2); };
      auto ld_pair = [&](const float *po, int s_) -> uint64_t {   // two floats of chunk s_ (8-byte aligned: HD + 2 is even)
        return __hip_atomic_load(as_global<uint64_t>(pair_at(po, s_)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      auto ld_ml = [&](const float *po, int s_) -> uint64_t {
        return __hip_atomic_load(as_global<uint64_t>(ml_at(po, s_)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      auto clear_pair = [&](const float *po, int s_) {
        __hip_atomic_store(as_global_mut<uint64_t>(const_cast<float *>(pair_at(po, s_))), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      auto written = [](uint64_t w) { return (uint32_t)w != 0u && (uint32_t)(w >> 32) != 0u; };
      auto gave_up = [&]() { if (a.err != nullptr) st_coherent(a.err, 1); };
      const int p0 = folds ? pr : 0;               // threads with nothing to fold request nothing
      const int j0 = (2 * p0) / HD, d0 = (2 * p0) % HD;
      const float *po0 = base + (size_t)j0 * (HD + 2) + d0;
      constexpr int MSL = (CHUNK_CAP + 63) / 64;   // chunks per lane (the host keeps n_active <= CHUNK_CAP)
      uint64_t mls[MSL];                         // wavefront j: (m, l) of this lane's chunks of head j, requested in one go
      if (wave < NREP) {
  #pragma unroll
        for (int i = 0; i < MSL; i++)
          if (i * 64 < n_active) mls[i] = ld_ml(base + (size_t)wave * (HD + 2) + HD, lane + i * 64);   // same test for the whole wavefront
      }
      // The partial sums of this thread's first pair are asked for as soon as its wavefront has seen every chunk's (m, l)
      // (the owners of pairs are threads of those wavefronts: NREP * HD / 128 <= NREP of them): asked for before that, the
      // words of a chunk that is still computing come back empty and the request has to be repeated a round trip later.
      uint64_t part[MB];
      bool asked = false;
      for (int j = wave; j < NREP; j += NW) {
        const float *pml = base + (size_t)j * (HD + 2) + HD;
        bool lost = false;
        // the first head of this wavefront was requested above; further heads (more query heads than wavefronts) and repeated
        // requests cost a round trip each
        for (int it = 0;; it++) {
          if (j != wave || it > 0) {
  #pragma unroll
            for (int i = 0; i < MSL; i++)
              if (i * 64 < n_active) mls[i] = ld_ml(pml, lane + i * 64);
          }
          if constexpr (!WORDS) break;
          bool ok = true;
  #pragma unroll
          for (int i = 0; i < MSL; i++)
            if (lane + i * 64 < n_active && !written(mls[i])) ok = false;
          if (ok) break;
          if (it >= POLL_LIMIT) { lost = true; gave_up(); break; }
          __builtin_amdgcn_s_sleep(1);
        }
        if (!asked && folds) {
  #pragma unroll
          for (int u = 0; u < MB; u++) part[u] = ld_pair(po0, sb + u);
        }
        asked = true;
        JSG_LSTAMP(16);
        if constexpr (WORDS) {
  #pragma unroll
          for (int i = 0; i < MSL; i++)
            if (lane + i * 64 < n_active) __hip_atomic_store(as_global_mut<uint64_t>(const_cast<float *>(ml_at(pml, lane + i * 64))), 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        float M = -INFINITY;
  #pragma unroll
        for (int i = 0; i < MSL; i++)
          if (lane + i * 64 < n_active) M = fmaxf(M, dec((uint32_t)mls[i]));
        M = wave_max(M);
        float L = 0.0f;
  #pragma unroll
        for (int i = 0; i < MSL; i++) {
          const int s_ = lane + i * 64;
          if (s_ < n_active) {
            const float w = exp_f32(dec((uint32_t)mls[i]) - M);
            sm.sc[j][s_] = w;  // n_active <= nsplit <= CHUNK_CAP
            L = fmaf(dec((uint32_t)(mls[i] >> 32)), w, L);
          }
        }
        L = wave_sum(L);
        if (__builtin_amdgcn_ballot_w64(lost) != 0) L = __builtin_nanf("");
        if (lane == 0) sm.l_sh[j] = 1.0f / L;  // softmax normalisation is e * (1/sum) (tensor.ts:2211-2214)
      }
      if constexpr (!SLICED) {
        if (!asked && folds) {        // a wavefront without a query head of its own (no built shape has one that owns pairs)
  #pragma unroll
          for (int u = 0; u < MB; u++) part[u] = ld_pair(po0, sb + u);
        }
      }
      lds_barrier();
      if constexpr (SLICED) {
        if (!asked && folds) {        // a wavefront without a query head of its own asks now that every chunk's (m, l) has been seen
  #pragma unroll
          for (int u = 0; u < MB; u++) part[u] = ld_pair(po0, sb + u);
        }
      }
      JSG_LSTAMP(17);
      auto finish = [&](int i, float O) {
        const int j = i / HD, d = i % HD;
        AT *dst = (AT *)a.out + (size_t)(g * NREP + j) * HD + d;
        const float r = Act<AT>::rn(O * sm.l_sh[j]);  // the cast of the P.V result
        if (a.out_tagged != nullptr) tw_store(a.out_tagged + (size_t)(g * NREP + j) * HD + d, a.out_tag, r);
        else if constexpr (COHERENT) st_coherent(dst, (AT)r);
        else *dst = (AT)r;
      };
      if constexpr (SLICED) {
        float Oa = 0.0f, Ob = 0.0f;
        if (folds) {
          const float *po = po0;
          for (int s0 = sb; s0 < send; s0 += MB) {
            for (int it = 0;; it++) {
              if (s0 > sb || it > 0) {     // the first batch is already here
  #pragma unroll
                for (int u = 0; u < MB; u++) part[u] = ld_pair(po, s0 + u);
              }
              if constexpr (!WORDS) break;
              bool ok = true;              // no branches from here to the sums (see pair_at)
  #pragma unroll
              for (int u = 0; u < MB; u++) ok = ok & written(part[u]);
              if (ok) break;
              if (it >= POLL_LIMIT) { Oa = Ob = __builtin_nanf(""); gave_up(); break; }
              __builtin_amdgcn_s_sleep(1);
            }
            if constexpr (WORDS) {
  #pragma unroll
              for (int u = 0; u < MB; u++) clear_pair(po, s0 + u);
            }
            float wgt[MB];
  #pragma unroll
            for (int u = 0; u < MB; u++) wgt[u] = sm.sc[j0][s0 + u < send ? s0 + u : send - 1];
  #pragma unroll
            for (int u = 0; u < MB; u++) {
              const bool in = s0 + u < send;
              const float w = in ? wgt[u] : 0.0f;
              Oa = fmaf(in ? dec((uint32_t)part[u]) : 0.0f, w, Oa);
              Ob = fmaf(in ? dec((uint32_t)(part[u] >> 32)) : 0.0f, w, Ob);
            }
          }
        }
        if (nsl > 1) {      // the same for the whole block: the slices' sums meet in LDS (the wavefronts' output slots are free by now)
          float *ps = &sm.o_part[0][0][0];
          if (sl < nsl) { ps[tid * 2] = Oa; ps[tid * 2 + 1] = Ob; }      // tid = sl * NPAIR + pr; a slice without chunks adds zeros
          lds_barrier();
          if (sl == 0)
            for (int q = 1; q < nsl; q++) { Oa += ps[(q * NPAIR + pr) * 2]; Ob += ps[(q * NPAIR + pr) * 2 + 1]; }
        }
        if (sl == 0) {
          finish(2 * pr, Oa);
          finish(2 * pr + 1, Ob);
        }
      } else {
        for (int p = tid; p < NPAIR; p += nthreads) {
          const int j = (2 * p) / HD, d = (2 * p) % HD;
          const float *po = base + (size_t)j * (HD + 2) + d;
          float Oa = 0.0f, Ob = 0.0f;
          for (int s0 = 0; s0 < n_active; s0 += MB) {
            for (int it = 0;; it++) {
              if (s0 > 0 || p != tid || it > 0) {     // the first batch of the first pair is already here
    #pragma unroll
                for (int u = 0; u < MB; u++) part[u] = ld_pair(po, s0 + u);
              }
              if constexpr (!WORDS) break;
              // no branches from here to the sums: a chunk index past the end stands for the last chunk (ld_pair, clear_pair),
              // whose words are checked and cleared again and enter the sum with weight zero
              bool ok = true;
    #pragma unroll
              for (int u = 0; u < MB; u++) ok = ok & written(part[u]);
              if (ok) break;
              if (it >= POLL_LIMIT) { Oa = Ob = __builtin_nanf(""); gave_up(); break; }
              __builtin_amdgcn_s_sleep(1);
            }
            if constexpr (WORDS) {
    #pragma unroll
              for (int u = 0; u < MB; u++) clear_pair(po, s0 + u);
            }
            float wgt[MB];
    #pragma unroll
            for (int u = 0; u < MB; u++) wgt[u] = sm.sc[j][s0 + u < n_active ? s0 + u : n_active - 1];
    #pragma unroll
            for (int u = 0; u < MB; u++) {
              const bool in = s0 + u < n_active;
              const float w = in ? wgt[u] : 0.0f;
              Oa = fmaf(in ? dec((uint32_t)part[u]) : 0.0f, w, Oa);
              Ob = fmaf(in ? dec((uint32_t)(part[u] >> 32)) : 0.0f, w, Ob);
            }
          }
          finish(2 * p, Oa);
          finish(2 * p + 1, Ob);
        }
      }
      JSG_LSTAMP(18);
    }
    then();
  }
};

}  // namespace jsg
