// Decode-time grouped-query attention for MANY sequences at once (jsgrad_hip_attn_decode_batch): the streaming form of the
// work item of attention_core.h.
//
// With one sequence a launch has a few dozen items and waits for the chain of dependent steps inside each, so an item there
// is worked on by 16 wavefronts that request all their rows up front (attention_core.h).  With 16 sequences a launch has
// thousands of items and moves over a hundred megabytes: what counts is that every CU keeps requests in flight all the time.
// Here an item is run by a block of 4 wavefronts that walk their rows in batches of eight requests, five or more blocks to
// a CU, so the loads of one block travel while another computes; the last block of a kv head to finish (an agent-scope
// counter) merges the chunks.  Same arithmetic as attention_core.h (float scores, the reference's polynomial exp2, float
// P.V), different chunk boundaries, so the float sums differ in their last bits.
#pragma once
#include "attention_core.h"

namespace jsg {

constexpr int ATT_STREAM_CHUNK_MIN = 32;   // shorter chunks finish no sooner and only add partial results for the merge to fetch
__host__ __device__ __forceinline__ int att_stream_chunk_rows(int T, int nsplit) {
  const int c = (T + nsplit - 1) / nsplit;
  return c < ATT_STREAM_CHUNK_MIN ? ATT_STREAM_CHUNK_MIN : c;
}

// NW wavefronts per block.  COHERENT: q and the output cross between blocks of the same launch.
template <typename AT, int HD, int NREP, int NW, bool COHERENT> struct AttnStream {
  static constexpr int EPL = 16 / sizeof(AT);  // elements per lane per 128-bit load
  static constexpr int G = HD / EPL;           // lanes per cache row
  static constexpr int RPI = 64 / G;           // rows per wavefront iteration
  static_assert(G == 8 || G == 16 || G == 32, "the fold over row groups is written for 8, 16 or 32 lanes per row");
  struct Smem {
    float sc[NREP][ATT_CHUNK_MAX];
    float red[NREP][NW];
    float o_part[NW < 4 ? NW : 4][NREP][HD];   // wavefronts fold into four slots, then the slots are summed
    float m_sh[NREP], l_sh[NREP];
    int is_last;
  };

  // T visible positions cut into chunks of `chunk` rows (n_active of them); this call handles chunk `split` of kv head g.
  // Must be called by every thread of the block (it contains barriers).
  __device__ static void item(const AttnArgs &a, Smem &sm, int g, int split, int T, int chunk, int n_active) {
    const int t0 = split * chunk, t1 = min(T, t0 + chunk), CH = t1 - t0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthreads = NW * 64;
    const int sub = lane % G, grp = lane / G;
    const size_t row_stride = (size_t)a.n_kv_heads * HD;
    const AT *kbase = (const AT *)a.cache_k + (size_t)g * HD + (size_t)sub * EPL;
    const AT *vbase = (const AT *)a.cache_v + (size_t)g * HD + (size_t)sub * EPL;

    // this lane's slice of the n_rep query rows (fp16: kept packed, two elements to a register, for the packed dot product)
    constexpr int QW = sizeof(AT) == 2 ? 4 : EPL;
    uint32_t qv[NREP][QW];
#pragma unroll
    for (int j = 0; j < NREP; j++) {
      const AT *qp = (const AT *)a.q + (size_t)(g * NREP + j) * HD + sub * EPL;
#pragma unroll
      for (int e = 0; e < QW; e++) {
        if constexpr (COHERENT) qv[j][e] = __hip_atomic_load(as_global<uint32_t>(qp) + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else qv[j][e] = ((const uint32_t *)qp)[e];
      }
    }

    // The K and V rows of this thread's first NPRE iterations are requested together, before anything is computed: a chunk is
    // usually that short, and the launch is a chain of round trips, so V must not wait for the softmax.
    constexpr int NPRE = 2;
    u4_t kpre[NPRE], vpre[NPRE];
#pragma unroll
    for (int i = 0; i < NPRE; i++) {
      const int t = t0 + (wave + i * NW) * RPI + grp;
      const size_t off = (size_t)(t < t1 ? t : t1 - 1) * row_stride;   // t1 > t0: the item exists
      kpre[i] = *(const u4_t *)(kbase + off);
      vpre[i] = *(const u4_t *)(vbase + off);
    }

    // ---- phase 1: scores of the chunk
    auto score_row = [&](u4_t raw, int t) {
#pragma unroll
      for (int j = 0; j < NREP; j++) {
        float p = 0.0f;
        if constexpr (sizeof(AT) == 2) {     // packed dot products with float accumulation (the products are exact in float)
#pragma unroll
          for (int e = 0; e < 4; e++) p = __builtin_amdgcn_fdot2(as_h2(qv[j][e]), as_h2(raw[e]), p, false);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) p = fmaf(__uint_as_float(qv[j][e]), __uint_as_float(raw[e]), p);
        }
        p = group_sum<G>(p);
        if (sub == 0) sm.sc[j][t - t0] = p * a.scale;
      }
    };
    // a chunk with more rows than the up-front requests cover: its first batch of K rows is asked for before the first
    // scores are computed
    const int tb_v = t0 + (wave + NPRE * NW) * RPI + grp;
    const bool more_v = CH > NPRE * NW * RPI;              // the same for the whole block
    constexpr int NBATCH = 8;
    u4_t kbat[NBATCH];
    if (more_v) {
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb_v + i * NW * RPI;
        kbat[i] = *(const u4_t *)(kbase + (size_t)(t < t1 ? t : t1 - 1) * row_stride);
      }
    }
#pragma unroll
    for (int i = 0; i < NPRE; i++) {
      const int t = t0 + (wave + i * NW) * RPI + grp;
      if (t < t1) score_row(kpre[i], t);
    }
    if (more_v) {
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb_v + i * NW * RPI;
        if (t < t1) score_row(kbat[i], t);
      }
    }
    // still longer chunks: the remaining rows in batches of NBATCH requests, so that an iteration does not wait a round trip
    // of its own
    for (int tb = tb_v + NBATCH * NW * RPI; tb < t1; tb += NBATCH * NW * RPI) {
      u4_t raw[NBATCH];
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb + i * NW * RPI;
        raw[i] = *(const u4_t *)(kbase + (size_t)(t < t1 ? t : t1 - 1) * row_stride);
      }
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb + i * NW * RPI;
        if (t < t1) score_row(raw[i], t);
      }
    }
    // A chunk with more rows than the requests sent up front cover (several sequences, long contexts): the first batch of V
    // rows is requested now, so that it travels while the softmax is computed.  The two barriers around the softmax wait
    // for LDS traffic only; __syncthreads() would also wait for these requests.
    u4_t vbat[NBATCH];
    if (more_v) {
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb_v + i * NW * RPI;
        vbat[i] = *(const u4_t *)(vbase + (size_t)(t < t1 ? t : t1 - 1) * row_stride);
      }
    }
    lds_barrier();
    if (NREP <= NW) {
      // Wavefront j does the whole softmax of head j by itself - maximum, exp, sum - with no barrier in between: lane i holds
      // rows i, i + 64, ... of the chunk (one row per lane for the short chunks of a single sequence).
      if (wave < NREP) {
        const int j = wave;
        constexpr int PL = ATT_CHUNK_MAX / 64;
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
    } else {
    // chunk maximum per head
    {
      float mx[NREP];
#pragma unroll
      for (int j = 0; j < NREP; j++) mx[j] = -INFINITY;
      for (int i = tid; i < CH; i += nthreads)
#pragma unroll
        for (int j = 0; j < NREP; j++) mx[j] = fmaxf(mx[j], sm.sc[j][i]);
#pragma unroll
      for (int j = 0; j < NREP; j++) {
        float w = wave_max(mx[j]);
        if (lane == 0) sm.red[j][wave] = w;
      }
      __syncthreads();
      if (tid < NREP) {
        float w = sm.red[tid][0];
        for (int i = 1; i < NW; i++) w = fmaxf(w, sm.red[tid][i]);
        sm.m_sh[tid] = w;
      }
      __syncthreads();
    }
    // scores -> exp(s - m) in place, and their sum
    {
      float ls[NREP];
#pragma unroll
      for (int j = 0; j < NREP; j++) ls[j] = 0.0f;
      for (int i = tid; i < CH; i += nthreads)
#pragma unroll
        for (int j = 0; j < NREP; j++) {
          float e = exp_f32(sm.sc[j][i] - sm.m_sh[j]);
          sm.sc[j][i] = e;
          ls[j] += e;
        }
#pragma unroll
      for (int j = 0; j < NREP; j++) {
        float w = wave_sum(ls[j]);
        if (lane == 0) sm.red[j][wave] = w;
      }
      __syncthreads();
      if (tid < NREP) {
        float w = 0.0f;
        for (int i = 0; i < NW; i++) w += sm.red[tid][i];
        sm.l_sh[tid] = w;
      }
      // the barrier below also orders the in-place exp writes before phase 2 reads them
    }
    }
    lds_barrier();

    // ---- phase 2: o[j][d] = sum_t p[j][t] * V[t][d]
    float of[NREP][EPL];
#pragma unroll
    for (int j = 0; j < NREP; j++)
#pragma unroll
      for (int e = 0; e < EPL; e++) of[j][e] = 0.0f;
    auto pv_row = [&](u4_t raw, int t) {
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
        const float p = sm.sc[j][t - t0];
#pragma unroll
        for (int e = 0; e < EPL; e++) of[j][e] = fmaf(p, vf[e], of[j][e]);
      }
    };
#pragma unroll
    for (int i = 0; i < NPRE; i++) {
      const int t = t0 + (wave + i * NW) * RPI + grp;
      if (t < t1) pv_row(vpre[i], t);
    }
    if (more_v) {
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb_v + i * NW * RPI;
        if (t < t1) pv_row(vbat[i], t);
      }
    }
    for (int tb = tb_v + NBATCH * NW * RPI; tb < t1; tb += NBATCH * NW * RPI) {
      u4_t raw[NBATCH];
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb + i * NW * RPI;
        raw[i] = *(const u4_t *)(vbase + (size_t)(t < t1 ? t : t1 - 1) * row_stride);
      }
#pragma unroll
      for (int i = 0; i < NBATCH; i++) {
        const int t = tb + i * NW * RPI;
        if (t < t1) pv_row(raw[i], t);
      }
    }
    // lanes with the same `sub` hold different rows: fold the RPI groups of the wavefront together
#pragma unroll
    for (int j = 0; j < NREP; j++)
#pragma unroll
      for (int e = 0; e < EPL; e++) {
        float v = of[j][e];
        if constexpr (G <= 8) v += dpp_f<0x128>(v);    // row_ror:8: lane l ^ 8 of the same 16-lane row
        if constexpr (G <= 16) v = add_xor16(v);
        v = add_xor32(v);
        of[j][e] = v;
      }
    // wavefronts fold into (at most) four LDS slots, four at a time
    constexpr int SLOTS = NW < 4 ? NW : 4;
    for (int round = 0; round < NW / SLOTS; round++) {
      if (grp == 0 && wave / SLOTS == round) {
#pragma unroll
        for (int j = 0; j < NREP; j++)
#pragma unroll
          for (int e = 0; e < EPL; e++) {
            float *slot = &sm.o_part[wave % SLOTS][j][sub * EPL + e];
            *slot = round == 0 ? of[j][e] : *slot + of[j][e];
          }
      }
      __syncthreads();
    }
    float *mine = a.partial + ((size_t)g * a.nsplit + split) * NREP * (HD + 2);
    for (int i = tid; i < NREP * HD; i += nthreads) {
      const int j = i / HD, d = i % HD;
      float v = 0.0f;
#pragma unroll
      for (int w = 0; w < SLOTS; w++) v += sm.o_part[w][j][d];
      st_coherent(&mine[j * (HD + 2) + d], v);
    }
    if (tid < NREP) {
      st_coherent(&mine[tid * (HD + 2) + HD], sm.m_sh[tid]);
      st_coherent(&mine[tid * (HD + 2) + HD + 1], sm.l_sh[tid]);
    }

    // ---- publish, and let the last chunk of this kv head merge
    __syncthreads();  // every coherent store of the block has been acknowledged
    if (tid == 0) {
      int old = __hip_atomic_fetch_add(&a.counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sm.is_last = (old == n_active - 1);
    }
    __syncthreads();
    if (!sm.is_last) return;
    // merge: one wavefront per query head turns the per-chunk (m, l) into weights exp(m_s - M) and 1/L ...
    const float *base = a.partial + (size_t)g * a.nsplit * NREP * (HD + 2);
    constexpr int MSL = ATT_CHUNK_MAX / 64;   // chunks per lane
    for (int j = wave; j < NREP; j += NW) {
      float ms[MSL], ls[MSL];                  // (m, l) of this lane's chunks, all requested in one go
#pragma unroll
      for (int i = 0; i < MSL; i++) {
        const int s_ = lane + i * 64;
        if (i * 64 < n_active) {               // same for the whole wavefront
          const float *ps = base + ((size_t)(s_ < n_active ? s_ : n_active - 1) * NREP + j) * (HD + 2);
          ms[i] = ld_coherent(ps + HD);
          ls[i] = ld_coherent(ps + HD + 1);
        }
      }
      float M = -INFINITY;
#pragma unroll
      for (int i = 0; i < MSL; i++)
        if (lane + i * 64 < n_active) M = fmaxf(M, ms[i]);
      M = wave_max(M);
      float L = 0.0f;
#pragma unroll
      for (int i = 0; i < MSL; i++) {
        const int s_ = lane + i * 64;
        if (s_ < n_active) {
          const float w = exp_f32(ms[i] - M);
          sm.sc[j][s_] = w;  // n_active <= nsplit <= ATT_CHUNK_MAX
          L = fmaf(ls[i], w, L);
        }
      }
      L = wave_sum(L);
      if (lane == 0) sm.l_sh[j] = 1.0f / L;  // softmax normalisation is e * (1/sum) (tensor.ts:2211-2214)
    }
    __syncthreads();
    // ... then every thread sums its output elements over the chunks in chunk order, two elements at a time
    auto finish = [&](int i, float O) {
      const int j = i / HD, d = i % HD;
      AT *dst = (AT *)a.out + (size_t)(g * NREP + j) * HD + d;
      const float r = Act<AT>::rn(O * sm.l_sh[j]);  // the cast of the P.V result
      if (a.out_tagged != nullptr) tw_store(a.out_tagged + (size_t)(g * NREP + j) * HD + d, a.out_tag, r);
      else if constexpr (COHERENT) st_coherent(dst, (AT)r);
      else *dst = (AT)r;
    };
    auto ld_part = [&](const float *po, int s) { return ld_coherent(po + (size_t)(s < n_active ? s : n_active - 1) * NREP * (HD + 2)); };
    constexpr bool PAIRS = NREP * HD > NW * 64;              // more elements than threads: a thread has at least two
    for (int i0 = tid; i0 < NREP * HD; i0 += (PAIRS ? 2 : 1) * nthreads) {
      const int i1 = i0 + nthreads;
      const bool two = PAIRS && i1 < NREP * HD;
      const int ja = i0 / HD, jb = (two ? i1 : i0) / HD;
      const float *pa = base + (size_t)ja * (HD + 2) + i0 % HD, *pb = base + (size_t)jb * (HD + 2) + (two ? i1 : i0) % HD;
      // 16 chunks of both elements per round of requests (the usual number of chunks fits one round), summed in chunk order
      // without a branch per chunk (a branch each would make every weight an LDS read with a wait of its own): the weights
      // of 8 chunks are read together; an index past the last chunk stands for the last chunk (ld_part) with weight zero.
      constexpr int MBS = 16;
      float Oa = 0.0f, Ob = 0.0f;
      auto add = [&](const float (&part)[MBS], int j, int s0, float O) {
#pragma unroll
        for (int u0 = 0; u0 < MBS; u0 += 8) {
          float w[8];
#pragma unroll
          for (int u = 0; u < 8; u++) w[u] = sm.sc[j][s0 + u0 + u < n_active ? s0 + u0 + u : n_active - 1];
#pragma unroll
          for (int u = 0; u < 8; u++) {
            const bool in = s0 + u0 + u < n_active;
            O = fmaf(in ? part[u0 + u] : 0.0f, in ? w[u] : 0.0f, O);
          }
        }
        return O;
      };
      for (int s0 = 0; s0 < n_active; s0 += MBS) {
        float parta[MBS], partb[MBS];
#pragma unroll
        for (int u = 0; u < MBS; u++) parta[u] = ld_part(pa, s0 + u);
        if constexpr (PAIRS) {
#pragma unroll
          for (int u = 0; u < MBS; u++) partb[u] = ld_part(pb, s0 + u);
        }
        Oa = add(parta, ja, s0, Oa);
        if constexpr (PAIRS) Ob = add(partb, jb, s0, Ob);
      }
      finish(i0, Oa);
      if (two) finish(i1, Ob);
    }
    if (tid == 0) __hip_atomic_store(&a.counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
};

}  // namespace jsg
