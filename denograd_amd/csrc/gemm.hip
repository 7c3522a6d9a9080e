// Several-row linear layers on the gfx950 matrix cores: y[M][N] = x[M][K] . W[N][K]^T for M > 1 rows of fp16
// activations (batched prefill and batched decode), fp32 accumulate, fp16 out.
//
// What the reference computes (/root/reference/jsgrad/tensor.ts:2593-2605 `dot`, :3800 `linear`; Int8Linear.call
// /root/reference/jsgrad/models/llama3.ts:35; NF4Linear.call :91-97): with more than one input row the weight operand is
// expanded over the rows, so a quantised weight is first realised in fp16, W = RN16(code * scale), and the products of
// two fp16 values are then summed in float.  The dequantised fp16 tile written to LDS here is exactly that realised
// matrix; v_pk_mul_f16 of the exact fp16 code by the fp16 scale is the single rounding RN16(code * scale).
//
// Tiling: 256 threads = 4 wavefronts laid out WGM x WGN; a wavefront owns TM x TN tiles of 32x32 outputs and walks K in
// steps of 16 with v_mfma_f32_32x32x16_f16.  Both operands are K-contiguous in memory (x rows, W rows), so a lane's
// 8-element operand fragment is one 128-bit LDS read.  LDS rows are padded by 8 halves (144-byte stride), which
// spreads the 32 rows of a fragment read over all banks.  The weight fragment is the first MFMA operand, so a lane ends up
// with four neighbouring output columns of one output row per accumulator quad: 8-byte stores in the epilogue.
//
// Two loop shapes.  One LDS buffer (two barriers per K tile, the next tile prefetched into registers) with two or three
// blocks per CU, whose wavefronts cover each other's barriers and conversions.  Two LDS buffers with one 256x256 block
// per CU (one wavefront per SIMD): one barrier per K tile, and the instruction order of a K tile is spelled out so that
// fragment reads, conversion, LDS writes and the requests of the tile after next sit between the matrix instructions.
// Tile ids are remapped so that the blocks resident on one XCD (round-robin by block id) share operand tiles in that
// XCD's L2.
#include <stdlib.h>
#include <string.h>

#include <type_traits>

#include "common.h"

namespace jsg {

typedef float f16_t __attribute__((ext_vector_type(16)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));

enum { GEPI_STORE = 0, GEPI_ROPE_KV = 1, GEPI_SWIGLU = 2 };

constexpr int GEMM_BK = 64;           // K elements per LDS tile
constexpr int GEMM_LDS_STRIDE = 72;   // halves per LDS row (64 + 8 padding)
constexpr int GEMM_THREADS = 256;

struct GemmArgs {
  const void *w0, *w1, *w2;           // up to three weight matrices stacked along N (wq|wk|wv, or w1|w3)
  const _Float16 *s0, *s1, *s2;       // their scales (int8: per row; nf4: per 64 elements)
  int n0, n1, n2;                     // their row counts
  int M, N, K;                        // N = columns of the output this launch produces
  const _Float16 *x;                  // [M][K]
  _Float16 *y;                        // [M][N]  (ROPE_KV: q rows [M][n0])
  const _Float16 *residual;           // [M][N] or null
  // ROPE_KV
  const _Float16 *rope_table;         // [2*max_context][hd/2][2]
  _Float16 *cache_k, *cache_v;        // [B][max_context][n1]
  int seq_len, start_pos, head_dim, max_context;
};

__device__ __forceinline__ uint32_t pk_mul_h2(uint32_t a, h2_t s) {
  h2_t r = as_h2(a) * s;
  return __builtin_bit_cast(uint32_t, r);
}

// 4 int8 codes (one dword) -> 4 exact fp16 values: byte | 0x6400 is 1024 + (code ^ 0x80), minus 1152 leaves the code
__device__ __forceinline__ void i8x4_to_h2x2(uint32_t q, uint32_t &lo, uint32_t &hi) {
  const uint32_t u = q ^ 0x80808080u;
  const h2_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};
  h2_t a = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;   // bytes 0,1
  h2_t b = as_h2(__builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;   // bytes 2,3
  lo = __builtin_bit_cast(uint32_t, a);
  hi = __builtin_bit_cast(uint32_t, b);
}

template <int KIND, int EPI, int WGM, int WGN, int TM, int TN, bool DB = false>
__global__ __launch_bounds__(GEMM_THREADS, (TM * TN > 8 ? 1 : (TM * TN > 4 ? 2 : 3))) void gemm_kernel(GemmArgs a) {
  static_assert(WGM * WGN == 4, "four wavefronts");
  static_assert(EPI != GEPI_SWIGLU || TN % 2 == 0, "a wavefront holds the w1 and the w3 tile of the same columns");
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32, LS = GEMM_LDS_STRIDE;
  constexpr int A_LOADS = BM / 32;                                                    // 16-byte loads per thread per K tile
  constexpr int B_ROWS_PER_PASS = KIND == JSGRAD_W_F16 ? 32 : KIND == JSGRAD_W_I8 ? 64 : 128;
  constexpr int B_CHUNKS = GEMM_THREADS / B_ROWS_PER_PASS;                             // 16-byte chunks per row of the K tile
  constexpr int B_LOADS = BN / B_ROWS_PER_PASS;
  static_assert(B_LOADS >= 1, "tile too narrow for this weight format");
  constexpr int BUF = (BM + BN) * LS;                     // halves per LDS buffer
  extern __shared__ __align__(16) _Float16 gemm_lds[];   // one or two buffers of [BM + BN rows][LS], then 32 spare bytes and the 256-entry NF4 table
  _Float16 *As = gemm_lds, *Bs = gemm_lds + BM * LS, *lut = gemm_lds + (DB ? 2 : 1) * BUF;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int l32 = lane & 31, lg = lane >> 5;

  // NF4: one table entry per BYTE, the two code values of its nibbles as a packed pair (element 2j is the high nibble,
  // llama3.ts:92-94), so a byte costs one LDS read and one packed multiplication by the block scale
  uint32_t *pairs = (uint32_t *)(lut + 16);
  if constexpr (KIND == JSGRAD_W_NF4) {
    pairs[tid] = nf4_code_bits(tid >> 4) | (nf4_code_bits(tid & 15) << 16);   // from literals: no memory round trip at the head of the launch
  }

  // ---- tile id: XCD-contiguous, then grouped so that neighbouring ids share an x tile column-block
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = a.N / (EPI == GEPI_SWIGLU ? BN / 2 : BN);
  const int nblocks = tiles_m * tiles_n;
  int bid = blockIdx.x;
  {
    const int per = nblocks / 8;
    if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  }
  constexpr int GROUP = KIND == JSGRAD_W_F16 ? 8 : 4;   // quantised weight tiles are half or a quarter of the bytes of an x tile: fewer x tiles, more weight tiles per XCD
  const int in_group = GROUP * tiles_n;
  const int first_m = (bid / in_group) * GROUP;
  const int gsz = min(tiles_m - first_m, GROUP);
  const int tm_ = first_m + (bid % in_group) % gsz, tn_ = (bid % in_group) / gsz;
  const int m0 = tm_ * BM;
  const int n0_out = tn_ * (EPI == GEPI_SWIGLU ? BN / 2 : BN);   // first output column of this tile

  // ---- B source of every row this thread loads: (matrix, row) is fixed over the K loop
  const unsigned char *bsrc[B_LOADS];
  h2_t bscale[B_LOADS];
  const _Float16 *bscale_ptr[B_LOADS];
  const int brow_t = tid / B_CHUNKS, bchunk = tid % B_CHUNKS;
#pragma unroll
  for (int i = 0; i < B_LOADS; i++) {
    const int r = brow_t + i * B_ROWS_PER_PASS;      // row inside the B tile
    const void *w; const _Float16 *s; int row;
    if constexpr (EPI == GEPI_SWIGLU) {
      const bool up = r >= BN / 2;
      w = up ? a.w1 : a.w0; s = up ? a.s1 : a.s0; row = n0_out + (up ? r - BN / 2 : r);
    } else if constexpr (EPI == GEPI_ROPE_KV) {
      const int n = n0_out + r;
      if (n < a.n0) { w = a.w0; s = a.s0; row = n; }
      else if (n < a.n0 + a.n1) { w = a.w1; s = a.s1; row = n - a.n0; }
      else { w = a.w2; s = a.s2; row = n - a.n0 - a.n1; }
    } else { w = a.w0; s = a.s0; row = n0_out + r; }
    const size_t e = (size_t)row * a.K;              // element offset of the row
    if constexpr (KIND == JSGRAD_W_F16) bsrc[i] = (const unsigned char *)w + e * 2 + bchunk * 16;
    else if constexpr (KIND == JSGRAD_W_I8) { bsrc[i] = (const unsigned char *)w + e + bchunk * 16; const _Float16 sv = s[row]; bscale[i] = h2_t{sv, sv}; }
    else { bsrc[i] = (const unsigned char *)w + e / 2 + bchunk * 16; bscale_ptr[i] = s + e / 64; }
  }
  const unsigned char *asrc[A_LOADS];
  const int arow_t = tid / 8, achunk = tid % 8;
#pragma unroll
  for (int i = 0; i < A_LOADS; i++) {
    int m = m0 + arow_t + i * 32;
    if (m >= a.M) m = a.M - 1;                        // rows past the end are computed and never stored
    asrc[i] = (const unsigned char *)(a.x + (size_t)m * a.K) + achunk * 16;
  }

  f16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  u4_t ga[A_LOADS], gb[B_LOADS];
  _Float16 gs[B_LOADS];
  auto issue_a = [&](int kt) {
    const size_t ko = (size_t)kt * GEMM_BK;
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) ga[i] = *(const u4_t *)(asrc[i] + ko * 2);
  };
  auto issue_b = [&](int kt, int lo = 0, int hi = 1 << 30) {
    const size_t ko = (size_t)kt * GEMM_BK;
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
      if (i < lo || i >= hi) continue;
      if constexpr (KIND == JSGRAD_W_F16) gb[i] = *(const u4_t *)(bsrc[i] + ko * 2);
      else if constexpr (KIND == JSGRAD_W_I8) gb[i] = *(const u4_t *)(bsrc[i] + ko);
      else { gb[i] = *(const u4_t *)(bsrc[i] + ko / 2); gs[i] = bscale_ptr[i][kt]; }
    }
  };
  auto issue = [&](int kt) { issue_a(kt); issue_b(kt); };
  auto commit_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) *(u4_t *)&As[buf * BUF + (arow_t + i * 32) * LS + achunk * 8] = ga[i];
  };
  auto commit_b = [&](int buf, int lo = 0, int hi = 1 << 30) {
#pragma unroll
    for (int i = 0; i < B_LOADS; i++) {
      if (i < lo || i >= hi) continue;
      _Float16 *dst = &Bs[buf * BUF + (brow_t + i * B_ROWS_PER_PASS) * LS];
      if constexpr (KIND == JSGRAD_W_F16) *(u4_t *)(dst + bchunk * 8) = gb[i];
      else if constexpr (KIND == JSGRAD_W_I8) {
        u4_t o0, o1;
        uint32_t lo, hi;
        i8x4_to_h2x2(gb[i].x, lo, hi); o0.x = pk_mul_h2(lo, bscale[i]); o0.y = pk_mul_h2(hi, bscale[i]);
        i8x4_to_h2x2(gb[i].y, lo, hi); o0.z = pk_mul_h2(lo, bscale[i]); o0.w = pk_mul_h2(hi, bscale[i]);
        i8x4_to_h2x2(gb[i].z, lo, hi); o1.x = pk_mul_h2(lo, bscale[i]); o1.y = pk_mul_h2(hi, bscale[i]);
        i8x4_to_h2x2(gb[i].w, lo, hi); o1.z = pk_mul_h2(lo, bscale[i]); o1.w = pk_mul_h2(hi, bscale[i]);
        *(u4_t *)(dst + bchunk * 16) = o0;
        *(u4_t *)(dst + bchunk * 16 + 8) = o1;
      } else {
        // 16 bytes = 32 elements; the high nibble of a byte is the even element (llama3.ts:92-94)
        const h2_t sv = {gs[i], gs[i]};
        uint32_t wds[4] = {gb[i].x, gb[i].y, gb[i].z, gb[i].w};
#pragma unroll
        for (int d = 0; d < 4; d++) {
          u4_t o;
          uint32_t outw[4];
#pragma unroll
          for (int b = 0; b < 4; b++) {
            const uint32_t byte = (wds[d] >> (8 * b)) & 0xffu;
            outw[b] = pk_mul_h2(pairs[byte], sv);
          }
          o.x = outw[0]; o.y = outw[1]; o.z = outw[2]; o.w = outw[3];
          *(u4_t *)(dst + bchunk * 32 + d * 8) = o;
        }
      }
    }
  };
  auto commit = [&](int buf = 0) { commit_a(buf); commit_b(buf); };

  auto frags = [&](int buf, int kk, h8_t *af, h8_t *bf) {
#pragma unroll
    for (int i = 0; i < TM; i++) af[i] = *(const h8_t *)&As[buf * BUF + ((wm * TM + i) * 32 + l32) * LS + kk * 16 + lg * 8];
#pragma unroll
    for (int j = 0; j < TN; j++) {
      int rbase;
      if constexpr (EPI == GEPI_SWIGLU) rbase = j < TN / 2 ? (wn * (TN / 2) + j) * 32 : BN / 2 + (wn * (TN / 2) + j - TN / 2) * 32;
      else rbase = (wn * TN + j) * 32;
      bf[j] = *(const h8_t *)&Bs[buf * BUF + (rbase + l32) * LS + kk * 16 + lg * 8];
    }
  };
  auto mfmas = [&](const h8_t *af, const h8_t *bf) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);   // D = W tile . x tile^T
  };

  const int nk = a.K / GEMM_BK;
  issue(0);
  if constexpr (KIND == JSGRAD_W_NF4) __syncthreads();   // the code table is in LDS
  if constexpr (DB) {
    // Two LDS buffers, one barrier per K tile: while the matrix cores work on tile kt out of one buffer, the same
    // wavefront turns the registers of tile kt+1 into the other buffer and requests tile kt+2 into the registers just
    // freed: the x half in K step 0, the weight half in K steps 1 and 2 (half of its loads each, which also spreads the
    // conversion of quantised weights), so every request has a whole tile's time to arrive and the requests of a CU
    // (64 KiB per tile through a 64 B/clock L1) are spread over the tile.
    // The barrier sits between K steps 2 and 3.  By then every wavefront has written its share of tile kt+1 and has
    // read all fragments of tile kt (those of step 3 are read during step 2), so during step 3 the fragments of the
    // first step of tile kt+1 are read and the matrix instructions run on across the end of the tile.  The buffer
    // written during tile kt is the one read during tile kt-1, whose last reads precede the barrier of kt-1.  The
    // barrier waits for LDS traffic only, so the requests stay in flight across it.
    commit(0);
    if (nk > 1) issue(1);
    lds_barrier();
    h8_t af[2][TM], bf[2][TN];
    frags(0, 0, af[0], bf[0]);
    for (int kt = 0; kt < nk; kt++) {
      const int cur = kt & 1;
      const int after_next = min(kt + 2, nk - 1);   // past the last tile the same steps run on the last tile again, into
                                                    // the buffer nobody computes from any more: a straight-line loop body
      __builtin_amdgcn_sched_barrier(0);
      auto k_step = [&](auto KK) {
        constexpr int kk = decltype(KK)::value;
        constexpr int LAST = GEMM_BK / 16 - 1;
        if (kk == LAST) lds_barrier();
        if (kk < LAST) frags(cur, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
        else frags(cur ^ 1, 0, af[0], bf[0]);
        if (kk == 0) { commit_a(cur ^ 1); issue_a(after_next); }
        constexpr int HB = B_LOADS > 1 ? B_LOADS / 2 : 1;   // weight loads of K step 1; the rest in step 2
        if (kk == 1) { commit_b(cur ^ 1, 0, HB); issue_b(after_next, 0, HB); }
        if (kk == 2) { commit_b(cur ^ 1, HB, B_LOADS); issue_b(after_next, HB, B_LOADS); }
        mfmas(af[kk & 1], bf[kk & 1]);
        // The order inside this K step, spelled out for the instruction scheduler: every matrix instruction is followed by
        // a share of the other work of the step (fragment reads of the next step, conversion and LDS writes of the next
        // tile, then the requests of the tile after it), so that work runs while the matrix core is busy.  Left alone the
        // scheduler puts each fragment read directly before its first use and waits out the LDS latency every time.
        constexpr int NMF = TM * TN;
        constexpr int BL = kk == 1 ? HB : B_LOADS - HB;
        constexpr int LOADS = kk == 0 ? A_LOADS : BL;
        constexpr int WRITES = kk == 0 ? A_LOADS : (KIND == JSGRAD_W_F16 ? BL : (KIND == JSGRAD_W_I8 ? 2 * BL : 4 * BL));
        constexpr int WSTEPS = NMF - (LOADS < NMF / 2 ? LOADS : NMF / 2);     // matrix instructions that carry the writes
#pragma unroll
        for (int i = 0; i < NMF; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                          // one MFMA
          if (i < TM + TN) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);          // one LDS read
          if (kk < LAST && LOADS > 0) {
            if (i < WSTEPS) {
              if (kk > 0 && KIND != JSGRAD_W_F16) __builtin_amdgcn_sched_group_barrier(0x002, KIND == JSGRAD_W_I8 ? 6 : 10, 0);
              if constexpr (kk > 0 && KIND == JSGRAD_W_NF4) __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);   // table look-ups
              __builtin_amdgcn_sched_group_barrier(0x200, (WRITES + WSTEPS - 1) / WSTEPS, 0);
            } else {
              __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
              __builtin_amdgcn_sched_group_barrier(0x020, (LOADS + NMF - WSTEPS - 1) / (NMF - WSTEPS), 0);
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      static_assert(GEMM_BK / 16 == 4, "four K steps per tile");
      k_step(std::integral_constant<int, 0>{});
      k_step(std::integral_constant<int, 1>{});
      k_step(std::integral_constant<int, 2>{});
      k_step(std::integral_constant<int, 3>{});
    }
  } else {
    for (int kt = 0; kt < nk; kt++) {
      commit();
      __syncthreads();
      if (kt + 1 < nk) issue(kt + 1);
#pragma unroll
      for (int kk = 0; kk < GEMM_BK / 16; kk++) {
        h8_t af[TM], bf[TN];
        frags(0, kk, af, bf);
        mfmas(af, bf);
      }
      __syncthreads();
    }
  }

  // ---- epilogue.  The weight fragment is the first MFMA operand, so the 32x32 result tile is held transposed: a lane has
  // output row m = lane % 32 and, in accumulators 4g .. 4g+3, the four neighbouring output columns 8g + 4 * (lane / 32) + 0..3.
  // Stored from there, one instruction would touch 32 output rows with 8 bytes each.  Instead every wavefront turns 32 rows
  // x its CW columns at a time through its own piece of LDS (free after the K loop; rows padded by 8 bytes, which spreads
  // the 8-byte writes of 16 rows over all banks) and reads them back as 16-byte pieces along the rows: a store instruction
  // then covers whole cache lines, and so do the loads of the residual and of the rope table.
  constexpr int TNE = EPI == GEPI_SWIGLU ? TN / 2 : TN;   // 32-column tiles of output per wavefront and row tile
  constexpr int CW = TNE * 32, RS = CW + 4;               // columns per wavefront; halves per LDS row
  constexpr int CPR = CW / 8;                             // 16-byte pieces per row
  static_assert((size_t)4 * 32 * RS <= (size_t)(BM + BN) * LS, "the transposing pieces fit the K-loop buffer");
  _Float16 *ep = gemm_lds + wave * 32 * RS;
  const int ncol0 = n0_out + wn * CW;                     // first output column of this wavefront
  // the residual of the whole wavefront tile is requested at once (the registers of the K loop are free): one trip to
  // memory instead of one per 32 rows
  h8_t res[EPI == GEPI_STORE ? TM : 1][EPI == GEPI_STORE ? 2 * TNE : 1];
  if constexpr (EPI == GEPI_STORE) {
    if (a.residual) {
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int p = 0; p < 2 * TNE; p++) {
          const int q = p * 64 + lane, row = q / CPR, piece = q % CPR;
          int m = m0 + (wm * TM + i) * 32 + row;
          if (m >= a.M) m = a.M - 1;
          res[i][p] = *(const h8_t *)&a.residual[(size_t)m * a.N + ncol0 + piece * 8];
        }
    }
  }
  __syncthreads();                                        // every wavefront is done with the K-loop buffers
#pragma unroll
  for (int i = 0; i < TM; i++) {
#pragma unroll
    for (int j = 0; j < TNE; j++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        h4_t o;
#pragma unroll
        for (int c = 0; c < 4; c++) {
          if constexpr (EPI == GEPI_SWIGLU) {
            // silu(w1 x) * (w3 x), each GEMM output and the product stored as fp16 (llama.ts:108-110)
            const float gt = rn16(acc[i][j][4 * g + c]), up = rn16(acc[i][j + TN / 2][4 * g + c]);
            o[c] = (_Float16)(silu_act<_Float16>(gt) * up);
          } else {
            o[c] = (_Float16)acc[i][j][4 * g + c];
          }
        }
        *(h4_t *)&ep[l32 * RS + j * 32 + 8 * g + 4 * lg] = o;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wavefront's own writes, before its own reads
    const int mrow0 = m0 + (wm * TM + i) * 32;
#pragma unroll
    for (int p = 0; p < 2 * TNE; p++) {
      const int q = p * 64 + lane, row = q / CPR, piece = q % CPR;
      const int m = mrow0 + row, n = ncol0 + piece * 8;
      const h8_t v = *(const h8_t *)&ep[row * RS + piece * 8];
      if (m >= a.M) continue;
      if constexpr (EPI == GEPI_SWIGLU) {
        *(h8_t *)&a.y[(size_t)m * a.N + n] = v;
      } else if constexpr (EPI == GEPI_STORE) {
        h8_t o = v;
        if (a.residual) {
#pragma unroll
          for (int c = 0; c < 8; c++) o[c] = (_Float16)((float)res[i][p][c] + (float)v[c]);
        }
        *(h8_t *)&a.y[(size_t)m * a.N + n] = o;
      } else {
        // wq | wk | wv columns; q and k get the interleaved-pair rotation (llama.ts:17-32), k and v go to the cache rows.
        // Eight neighbouring columns are four pairs of one head of one matrix (every boundary is a multiple of 8).
        const int b = m / a.seq_len, pos = a.start_pos + m % a.seq_len;
        const int which = n < a.n0 ? 0 : (n < a.n0 + a.n1 ? 1 : 2);
        const int nl = which == 0 ? n : (which == 1 ? n - a.n0 : n - a.n0 - a.n1);
        h8_t o = v;
        if (which < 2) {
          const int pair = (nl % a.head_dim) >> 1;
          const h8_t cs = *(const h8_t *)(a.rope_table + ((size_t)pos * (a.head_dim / 2) + pair) * 2);   // cos, sin of four pairs
#pragma unroll
          for (int h = 0; h < 4; h++) {
            const float ev = (float)v[2 * h], od = (float)v[2 * h + 1];
            const float c = (float)cs[2 * h], d = (float)cs[2 * h + 1];
            o[2 * h] = (_Float16)(ev * c - od * d);
            o[2 * h + 1] = (_Float16)(ev * d + od * c);
          }
        }
        if (which == 0) *(h8_t *)&a.y[(size_t)m * a.n0 + nl] = o;
        else {
          _Float16 *cache = which == 1 ? a.cache_k : a.cache_v;
          *(h8_t *)&cache[((size_t)b * a.max_context + pos) * a.n1 + nl] = o;
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the reads, before the next row tile overwrites the piece
  }
}

// ---- at most 32 rows (batched decode): the weights are streamed once, straight from memory into the B operand ------------
//
// With a handful of rows the launch is bound by reading W once, so it is laid out like the one-row GEMV, not like a tiled
// GEMM.  v_mfma_f32_16x16x32_f16 takes, per lane, 8 consecutive K elements of one weight row as B and of one x row as
// A; a lane's 16-byte load is 8 fp16, 16 int8 codes or 32 nf4 codes of weight row n0 + lane % 16, i.e. one, two or four
// MFMAs, and goes from memory to registers with nothing in between (int8 and nf4 codes become RN16(code * scale) in
// registers: the realised fp16 matrix the reference multiplies by; nf4 through a 256-entry table of code pairs in LDS, one
// look-up per byte, with the scale of the lane's 64-element block loaded beside the codes).  The loads run through a register ring of 12 to 16 loads per wavefront.
// Only x goes through LDS, in K chunks of 512, four buffers.  The fifth wavefront of a block does nothing but move
// x chunks from memory to LDS (direct loads, no registers), up to three chunks ahead: a wavefront's loads return in order, so x loads issued by
// the arithmetic wavefronts would have to be waited for together with every weight load issued before them, which
// empties the ring once per chunk.
//
// A block owns 16 weight rows and its four arithmetic wavefronts split K: each takes a quarter of the k-blocks of every
// chunk, and the partial accumulators are added in wavefront order through LDS.  N/16 blocks fill the chip even for
// N = 4096.  (A block shape with 128 weight rows, which reads x once for all of them instead of once per 16, was tried for
// the wide layers: faster for the lm_head only, and its register ring did not survive the register allocator.)
template <int KIND> struct SkFmt {
  static constexpr int VEC = KIND == JSGRAD_W_F16 ? 8 : (KIND == JSGRAD_W_I8 ? 16 : 32);   // K elements per 16-byte load of a lane
  static constexpr int KB = 4 * VEC;                          // K elements per wavefront load (a k-block)
  static constexpr int KC = 512;                              // K elements per x chunk: 1 KiB per x row, one direct load
  static constexpr int KBC = KC / KB;                         // k-blocks per chunk
};
constexpr int SK_THREADS = 320;
constexpr int SK_KS = 4;                                      // wavefronts that split K
constexpr int SK_XBUF = 4;                                    // x chunks in LDS: one being read, up to three on their way
template <int KIND, int EPI, int RTW> struct SkShape {
  static constexpr int NMAT = EPI == GEPI_SWIGLU ? 2 : 1;
  static constexpr int SPC = SkFmt<KIND>::KBC / SK_KS;        // k-blocks of a chunk one wavefront walks
  static constexpr int RS = 8;                                // k-blocks in the ring
  static constexpr int BR = 16 * RTW;                         // weight rows per block: RTW tiles of 16
  static_assert(RS % SPC == 0, "chunk ends fall on fixed ring slots");
};

// Block barriers of the weight-streaming kernel.  __syncthreads() also waits for every global load of the wavefront (the
// counter that tracks loads tracks stores too, and a barrier publishes stores), which would empty the ring of weight loads
// at every x chunk; what has to be finished at these barriers is only LDS traffic, or, for the wavefront that moves x,
// its direct loads into LDS.
__device__ __forceinline__ void sk_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int KIND, int EPI, int MB, int RTW>
__global__ __launch_bounds__(SK_THREADS, 2) void skinny_gemm_kernel(GemmArgs a) {
  static_assert(KIND == JSGRAD_W_F16 || KIND == JSGRAD_W_I8 || KIND == JSGRAD_W_NF4, "fp16, int8 and nf4 weights");
  typedef SkFmt<KIND> F;
  typedef SkShape<KIND, EPI, RTW> S;
  constexpr int NMAT = S::NMAT, SPC = S::SPC, RS = S::RS;
  constexpr int NMF = F::VEC / 8;                        // MFMAs per load
  constexpr int LS = F::KC + 8;                          // halves per LDS row of x (padded: rows start in different banks)
  constexpr int XROWS = MB * 16;
  constexpr int PPR = F::KC / 8;                         // 16-byte pieces per x row of a chunk
  static_assert(PPR % 64 == 0, "a direct load of the wavefront fills 1 KiB of one LDS row");
  constexpr int XLOADS = XROWS * PPR / 64;               // direct loads per chunk
  extern __shared__ __align__(16) _Float16 sk_lds[];     // SK_XBUF x [XROWS][LS]; afterwards the partial accumulators

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, lq = lane >> 4;
  const int nchunks = a.K / F::KC;
  // NF4: one table entry per BYTE, the code values of its two nibbles as a packed pair (element 2j, the high nibble, in the
  // low half: llama3.ts:92-94); written here, read after the first barrier of either path below
  __shared__ uint32_t pairs[KIND == JSGRAD_W_NF4 ? 256 : 1];
  if constexpr (KIND == JSGRAD_W_NF4) {
    if (tid < 256) pairs[tid] = nf4_code_bits(tid >> 4) | (nf4_code_bits(tid & 15) << 16);
  }

  if (wave == 4) {
    // ---- the x mover: up to three chunks ahead of the one being read (a chunk takes a trip to L2 to arrive, longer than
    // the others need for a chunk), into the buffer whose readers passed the barrier of the chunk before
    auto move = [&](int c) {
      _Float16 *dst = sk_lds + (c % SK_XBUF) * XROWS * LS;
#pragma unroll
      for (int i = 0; i < XLOADS; i++) {
        const int r = (i * 64) / PPR, c8 = (i * 64) % PPR + lane;
        const int m = r < a.M ? r : a.M - 1;             // rows past the end are computed and never stored
        const _Float16 *src = a.x + (size_t)m * a.K + (size_t)c * F::KC + c8 * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                         (__attribute__((address_space(3))) void *)(dst + r * LS + ((i * 64) % PPR) * 8), 16, 0, 0);
      }
    };
    // wait until chunk `target` has landed: the direct loads complete in order, so whatever was issued after it may stay
    // in flight (the counter holds 63 loads at most)
    constexpr int MAX_BEHIND = 63 / XLOADS < 2 ? 63 / XLOADS : 2;
    int issued = 0;
    auto landed = [&](int target) {
      const int behind = issued - target - 1;
      if (MAX_BEHIND >= 2 && behind >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * XLOADS <= 63 ? 2 * XLOADS : 0) : "memory");
      else if (MAX_BEHIND >= 1 && behind >= 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(XLOADS <= 63 ? XLOADS : 0) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    while (issued < SK_XBUF - 1 && issued < nchunks) move(issued++);
    landed(0);
    sk_barrier();
    for (int c = 0; c < nchunks; c++) {
      if (issued < nchunks) move(issued++);              // into the buffer of chunk c - 1
      if (c + 1 < nchunks) landed(c + 1);
      sk_barrier();
    }
    sk_barrier();
    return;
  }

  const int ks = wave;
  const int n_first = blockIdx.x * S::BR;               // first weight row of the block
  // ---- the weight rows of this lane: row n_first + rt * 16 + lane % 16 of matrix q
  const unsigned char *wrow[RTW][NMAT];
  h2_t wscale[RTW][NMAT];
  const _Float16 *srow[RTW][NMAT];
#pragma unroll
  for (int rt = 0; rt < RTW; rt++)
#pragma unroll
    for (int q = 0; q < NMAT; q++) {
      const int n = n_first + rt * 16 + l16;
      const void *w; const _Float16 *sc; int row;
      if constexpr (EPI == GEPI_SWIGLU) { w = q ? a.w1 : a.w0; sc = q ? a.s1 : a.s0; row = n; }
      else if constexpr (EPI == GEPI_ROPE_KV) {
        if (n < a.n0) { w = a.w0; sc = a.s0; row = n; }
        else if (n < a.n0 + a.n1) { w = a.w1; sc = a.s1; row = n - a.n0; }
        else { w = a.w2; sc = a.s2; row = n - a.n0 - a.n1; }
      } else { w = a.w0; sc = a.s0; row = n; }
      const size_t e = (size_t)row * a.K;
      wrow[rt][q] = (const unsigned char *)w + (KIND == JSGRAD_W_F16 ? e * 2 : (KIND == JSGRAD_W_I8 ? e : e / 2)) + lq * 16;
      if constexpr (KIND == JSGRAD_W_I8) { const _Float16 sv = sc[row]; wscale[rt][q] = h2_t{sv, sv}; }
      // nf4: a scale per 64 elements of the flattened matrix; a lane's 32 elements of a k-block share one (two per k-block)
      if constexpr (KIND == JSGRAD_W_NF4) srow[rt][q] = sc + (e >> 6) + (lq >> 1);
    }
  // Step s of this wavefront is k-block ks * SPC + s % SPC of chunk s / SPC: its SPC k-blocks of a chunk are neighbours, so
  // that the halves of a 128-byte line of a weight row are asked for by one wavefront, back to back.  Byte offset of the
  // step inside a weight row.  Past the end the last k-block is asked for again: the refills of the last RS steps keep the
  // number of loads in flight the same on every path, and a line that was fetched a moment ago costs no HBM traffic (the
  // first k-block of the row, read at the start, has long left the caches by then: that was 1.2-1.5x the bytes).
  const int nsteps = nchunks * SPC;
  auto woff = [&](int s) -> uint32_t {
    const int sc = s < nsteps ? s : nsteps - 1;
    const int kb = (sc / SPC) * F::KBC + ks * SPC + sc % SPC;
    return (uint32_t)(kb * 4) * 16u;
  };

  u4_t ring[RS][RTW][NMAT];
  _Float16 rsc[KIND == JSGRAD_W_NF4 ? RS : 1][RTW][NMAT];   // nf4: the block scale travels with its load
  f4_t acc[NMAT][RTW][MB];
#pragma unroll
  for (int q = 0; q < NMAT; q++)
#pragma unroll
    for (int rt = 0; rt < RTW; rt++)
#pragma unroll
      for (int mb = 0; mb < MB; mb++) acc[q][rt][mb] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < RS; i++)
#pragma unroll
    for (int rt = 0; rt < RTW; rt++)
#pragma unroll
      for (int q = 0; q < NMAT; q++) {
        ring[i][rt][q] = ldg_stream16(wrow[rt][q] + woff(i));
        if constexpr (KIND == JSGRAD_W_NF4) rsc[i][rt][q] = ldg(srow[rt][q] + (woff(i) >> 5));   // 64 bytes of codes per k-block = two scales
        __builtin_amdgcn_sched_barrier(0);               // issued in the order the loop consumes them: the waits count on it
      }
  sk_barrier();                                          // x chunk 0 is in LDS

  // The ring slots are refilled on every path, also by the steps past the end (the number of loads in flight then is the
  // same wherever the wait counters are set, so they can let RS - 1 steps stay in flight instead of none).
  for (int s0 = 0; s0 < nsteps; s0 += RS) {
#pragma unroll
    for (int i = 0; i < RS; i++) {
      const int s = s0 + i;
      const bool on = s < nsteps;                        // same for every thread of the block
      const int c = s / SPC, kb = ks * SPC + s % SPC;
      const _Float16 *xs = sk_lds + (c % SK_XBUF) * XROWS * LS;
      if (on) {
        h8_t af[NMF][MB];
#pragma unroll
        for (int f = 0; f < NMF; f++)
#pragma unroll
          for (int mb = 0; mb < MB; mb++) af[f][mb] = *(const h8_t *)&xs[(mb * 16 + l16) * LS + kb * F::KB + lq * F::VEC + f * 8];
#pragma unroll
        for (int rt = 0; rt < RTW; rt++)
#pragma unroll
          for (int q = 0; q < NMAT; q++) {
            const u4_t raw = ring[i][rt][q];
            h8_t bf[NMF];
            if constexpr (KIND == JSGRAD_W_F16) bf[0] = __builtin_bit_cast(h8_t, raw);
            else if constexpr (KIND == JSGRAD_W_NF4) {
              const _Float16 s1 = rsc[i][rt][q];
              const h2_t sv = {s1, s1};
              const uint32_t wds[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
              for (int d = 0; d < 4; d++) {                // a dword = 8 elements = one matrix instruction
                u4_t o;
                o.x = pk_mul_h2(pairs[wds[d] & 0xffu], sv);
                o.y = pk_mul_h2(pairs[(wds[d] >> 8) & 0xffu], sv);
                o.z = pk_mul_h2(pairs[(wds[d] >> 16) & 0xffu], sv);
                o.w = pk_mul_h2(pairs[wds[d] >> 24], sv);
                bf[d] = __builtin_bit_cast(h8_t, o);
              }
            } else {
              const h2_t sc = wscale[rt][q];
              u4_t o0, o1;
              uint32_t lo, hi;
              i8x4_to_h2x2(raw.x, lo, hi); o0.x = pk_mul_h2(lo, sc); o0.y = pk_mul_h2(hi, sc);
              i8x4_to_h2x2(raw.y, lo, hi); o0.z = pk_mul_h2(lo, sc); o0.w = pk_mul_h2(hi, sc);
              i8x4_to_h2x2(raw.z, lo, hi); o1.x = pk_mul_h2(lo, sc); o1.y = pk_mul_h2(hi, sc);
              i8x4_to_h2x2(raw.w, lo, hi); o1.z = pk_mul_h2(lo, sc); o1.w = pk_mul_h2(hi, sc);
              bf[0] = __builtin_bit_cast(h8_t, o0);
              bf[NMF - 1] = __builtin_bit_cast(h8_t, o1);
            }
#pragma unroll
            for (int f = 0; f < NMF; f++)
#pragma unroll
              for (int mb = 0; mb < MB; mb++) acc[q][rt][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[f][mb], bf[f], acc[q][rt][mb], 0, 0, 0);
          }
      }
      // The slots are refilled only now that their old contents are used up (and the scheduler may not move the loads up):
      // issued earlier, a load gets registers of its own and a copy into the slot afterwards, and the copy waits for the
      // load on the spot.
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int rt = 0; rt < RTW; rt++)
#pragma unroll
        for (int q = 0; q < NMAT; q++) {
          ring[i][rt][q] = ldg_stream16(wrow[rt][q] + woff(s + RS));
          if constexpr (KIND == JSGRAD_W_NF4) rsc[i][rt][q] = ldg(srow[rt][q] + (woff(s + RS) >> 5));
        }
      if (on && (s + 1) % SPC == 0) sk_barrier();        // chunk c is consumed, chunk c + 1 is in the other buffer
    }
  }

  // ---- epilogue of one 16x16 tile.  Accumulator r of a lane is output row 4 * (lane / 16) + r, column lane % 16.
  auto epilogue = [&](const f4_t (&tot)[NMAT], int n_tile, int mb) {
    const int n = n_tile + l16;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = mb * 16 + lq * 4 + r;
      if constexpr (EPI == GEPI_SWIGLU) {
        const float g = rn16(tot[0][r]), u = rn16(tot[NMAT - 1][r]);
        if (m < a.M) a.y[(size_t)m * a.N + n] = (_Float16)(silu_act<_Float16>(g) * u);
      } else if constexpr (EPI == GEPI_STORE) {
        if (m < a.M) {
          float v = rn16(tot[0][r]);
          if (a.residual) v = (float)a.residual[(size_t)m * a.N + n] + v;
          a.y[(size_t)m * a.N + n] = (_Float16)v;
        }
      } else {
        const int which = n < a.n0 ? 0 : (n < a.n0 + a.n1 ? 1 : 2);
        const int nl = which == 0 ? n : (which == 1 ? n - a.n0 : n - a.n0 - a.n1);
        const int pair = (nl % a.head_dim) >> 1;
        const bool odd = nl & 1;
        const float own = rn16(tot[0][r]);
        const float other = dpp_f<0xB1>(own);            // the neighbouring column: the other half of the pair
        if (m < a.M) {
          const int b = m / a.seq_len, pos = a.start_pos + m % a.seq_len;
          float v = own;
          if (which < 2) {
            const h2_t cs = *(const h2_t *)(a.rope_table + ((size_t)pos * (a.head_dim / 2) + pair) * 2);
            const float cc = (float)cs.x, dd = (float)cs.y;
            v = odd ? other * dd + own * cc : own * cc - other * dd;
          }
          if (which == 0) a.y[(size_t)m * a.n0 + nl] = (_Float16)v;
          else {
            _Float16 *cache = which == 1 ? a.cache_k : a.cache_v;
            cache[((size_t)b * a.max_context + pos) * a.n1 + nl] = (_Float16)v;
          }
        }
      }
    }
  };

  // the four K parts, added in wavefront order; the (tile, row block) pairs are dealt to the wavefronts
  constexpr int NACC = NMAT * RTW * MB;
  float *red = (float *)sk_lds;                          // [4][NACC][64 lanes] x 4 floats
#pragma unroll
  for (int q = 0; q < NMAT; q++)
#pragma unroll
    for (int rt = 0; rt < RTW; rt++)
#pragma unroll
      for (int mb = 0; mb < MB; mb++) *(f4_t *)&red[((wave * NACC + (q * RTW + rt) * MB + mb) * 64 + lane) * 4] = acc[q][rt][mb];
  sk_barrier();
  for (int item = wave; item < RTW * MB; item += 4) {
    const int rt = item / MB, mb = item % MB;
    f4_t tot[NMAT];
#pragma unroll
    for (int q = 0; q < NMAT; q++) {
      tot[q] = *(const f4_t *)&red[((0 * NACC + (q * RTW + rt) * MB + mb) * 64 + lane) * 4];
#pragma unroll
      for (int w = 1; w < 4; w++) tot[q] += *(const f4_t *)&red[((w * NACC + (q * RTW + rt) * MB + mb) * 64 + lane) * 4];
    }
    epilogue(tot, n_first + rt * 16, mb);
  }
}

// ---- at most 16 rows, int8 weights: whole stretches of weight rows, turned into operand layout through LDS -----------------
//
// The kernel above asks for 64 bytes of each of 16 rows per load and lives for 16 rows.  Measured with loads alone, that
// map reaches 4.0 TB/s where 512 contiguous bytes per row and wavefronts that keep streaming reach 5.0, and the kernel
// itself stays far below its own map: a block is over before its pipeline has filled, and every block reads all of x.
// Here a block stays on its compute unit and walks a list of units of work; a unit is COLS output columns times a K range.
// A step of a wavefront is a tile of 16 weight rows times 512 bytes (one x chunk): eight loads of 1 KiB = two rows, held
// in a ring of NS steps of registers (what is in flight is bounded by registers, and eight wavefronts per compute unit
// with two to three steps each keep ~150 KiB on their way; the same ring in LDS would hold less than half).  A step that
// has arrived is written to a 16 x 528-byte patch of LDS that belongs to the wavefront and read back in the matrix
// instruction's operand layout (lane = row, 8 K elements = 64 bits), rows 16 bytes apart modulo the bank cycle, so the
// 32 lanes of a read pass hit 64 different banks.  x goes through LDS as above (the fifth wavefront moves it), but one
// chunk now serves 64 or 128 weight rows instead of 16.
//
// Matrices with few rows are split along K as well (wo, w2: 4096 rows): the partial accumulators go to a workspace that
// belongs to the library, a counter per (column group, wavefront) tells the last arriver, and that wavefront adds the
// parts in K order - the result does not depend on which block finishes last.
constexpr int SG_THREADS = 320;
constexpr int SG_KC = 512;                                    // K elements per x chunk = bytes of a weight row per step
constexpr int SG_XB = 3;                                      // x chunks in LDS
constexpr int SG_XLS = SG_KC + 8;                             // halves per LDS row of x
#ifndef JSG_SG_NS
#define JSG_SG_NS 3
#endif
constexpr int SG_NS = JSG_SG_NS;                                      // steps in a wavefront's ring
constexpr int SG_WLS = SG_KC + 16;                            // bytes per LDS row of a weight tile
constexpr size_t SG_LDS = (size_t)SG_XB * 16 * SG_XLS * 2 + (size_t)4 * 16 * SG_WLS;
constexpr size_t SG_WS_BYTES = 8u << 20;
constexpr int SG_MAX_GROUPS = 4096;
static __device__ __align__(256) unsigned char sg_scratch[SG_WS_BYTES];
static __device__ int sg_counters[4 * SG_MAX_GROUPS];

template <int EPI, int TPW> struct SgShape {
  static constexpr int NMAT = EPI == GEPI_SWIGLU ? 2 : 1;
  static_assert(TPW % NMAT == 0, "w1 and w3 tiles of one column tile sit in one wavefront");
  static constexpr int CT = TPW / NMAT;                       // column tiles per wavefront
  static constexpr int COLS = 4 * CT * 16;                    // output columns per unit
};

struct SgArgs {
  GemmArgs g;
  int groups, splitk, nck;                                    // column groups, K parts, x chunks per part
  float *ws;
  int *counters;
};

template <int EPI, int TPW>
__global__ __launch_bounds__(SG_THREADS, 1) void stream_gemm_kernel(SgArgs sa) {
  typedef SgShape<EPI, TPW> S;
  constexpr int NMAT = S::NMAT, NS = SG_NS;
  const GemmArgs &a = sa.g;
  extern __shared__ __align__(16) unsigned char sg_lds[];
  _Float16 *xl = (_Float16 *)sg_lds;                          // SG_XB x [16][SG_XLS]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l16 = lane & 15, lq = lane >> 4;
  const int units = sa.groups * sa.splitk, nck = sa.nck;
  const int my_units = (units - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
  const int CS = my_units * nck;                              // x chunks this block walks

  if (wave == 4) {
    // ---- the x mover: chunk cs of the block is chunk part * nck + cs % nck of x; one chunk ahead of the readers
    auto move = [&](int cs) {
      const int unit = blockIdx.x + (cs / nck) * gridDim.x;
      const int kc = (unit % sa.splitk) * nck + (cs % nck + unit / sa.splitk) % nck;
      _Float16 *dst = xl + (cs % SG_XB) * 16 * SG_XLS;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = r < a.M ? r : a.M - 1;                  // rows past the end are computed and never stored
        const _Float16 *src = a.x + (size_t)m * a.K + (size_t)kc * SG_KC + lane * 8;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src, (__attribute__((address_space(3))) void *)(dst + r * SG_XLS), 16, 0, 0);
      }
    };
    int issued = 0;
    auto landed = [&](int target) {                           // the direct loads complete in order, 16 per chunk
      const int behind = issued - target - 1;
      if (behind >= 2) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
      else if (behind == 1) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    while (issued < SG_XB - 1 && issued < CS) move(issued++);
    landed(0);
    sk_barrier();
    for (int cs = 0; cs < CS; cs++) {
      if (issued < CS) move(issued++);                        // into the buffer of chunk cs - 1, whose readers are past their barrier
      if (cs + 1 < CS) landed(cs + 1);
      sk_barrier();
    }
    return;
  }

  unsigned char *stg = sg_lds + (size_t)SG_XB * 16 * SG_XLS * 2 + (size_t)wave * 16 * SG_WLS;   // this wavefront's tile
  // load side: a load is 1 KiB = two rows of the tile; lane -> (row of the pair, 16-byte piece)
  const int sub = lane >> 5;
  const uint32_t wr_off = (uint32_t)(sub * SG_WLS + (lane & 31) * 16);
  // read side: lane (l16, lq) takes 8 bytes of row l16 per matrix instruction
  const uint32_t rd_off = (uint32_t)(l16 * SG_WLS + lq * 8);
  const int xoff = l16 * SG_XLS + lq * 8;

  // first weight row of tile tt of this wavefront in column group grp, and the matrix it belongs to
  auto tile_of = [&](int grp, int tt, const unsigned char *&w, const _Float16 *&sc, int &row) {
    const int n = grp * S::COLS + (wave * S::CT + tt / NMAT) * 16;
    if constexpr (EPI == GEPI_SWIGLU) { w = (const unsigned char *)(tt % NMAT ? a.w1 : a.w0); sc = tt % NMAT ? a.s1 : a.s0; row = n; }
    else if constexpr (EPI == GEPI_ROPE_KV) {
      if (n < a.n0) { w = (const unsigned char *)a.w0; sc = a.s0; row = n; }
      else if (n < a.n0 + a.n1) { w = (const unsigned char *)a.w1; sc = a.s1; row = n - a.n0; }
      else { w = (const unsigned char *)a.w2; sc = a.s2; row = n - a.n0 - a.n1; }
    } else { w = (const unsigned char *)a.w0; sc = a.s0; row = n; }
  };

  // Step gs of this wavefront: tile gs % TPW of x chunk gs / TPW.  The scale of the tile's row l16 travels with the step.
  const int GS = CS * TPW;
  u4_t ring[NS][8];
  _Float16 rscale[NS];
  auto issue = [&](int gs, u4_t (&dst)[8], _Float16 &scale) {
    const int cs = gs / TPW, tt = gs % TPW;
    const int unit = blockIdx.x + (cs / nck) * gridDim.x;
    const int grp = unit / sa.splitk, part = unit % sa.splitk, c = cs % nck;
    const unsigned char *w; const _Float16 *sc; int row;
    tile_of(grp, tt, w, sc, row);
    // the scale stays as loaded until its step is consumed: packed into two halves here, the pack would wait for the load on
    // the spot, and with it for every load issued before it (w1 | w3 of the 8B shape at 16 rows 29.4 -> 26.8 us)
    scale = sc[row + l16];
    // Column group grp starts its walk through K at chunk grp % nck and wraps around: at any moment the blocks of the
    // launch read at different offsets inside the weight rows, which are a power of two apart in memory
    const unsigned char *src = w + (size_t)(row + sub) * a.K + (size_t)(part * nck + (c + grp) % nck) * SG_KC + (lane & 31) * 16;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      dst[i] = ldg_stream16(src + (size_t)(2 * i) * a.K);
      __builtin_amdgcn_sched_barrier(0);                      // issued in the order they are used: the waits count on it
    }
  };

  // ---- epilogue of one 16x16 tile.  Accumulator r of a lane is output row 4 * (lane / 16) + r, column lane % 16.
  auto epilogue = [&](const f4_t (&tot)[NMAT], int n_tile) {
    const int n = n_tile + l16;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = lq * 4 + r;
      if constexpr (EPI == GEPI_SWIGLU) {
        const float g = rn16(tot[0][r]), u = rn16(tot[NMAT - 1][r]);
        if (m < a.M) a.y[(size_t)m * a.N + n] = (_Float16)(silu_act<_Float16>(g) * u);
      } else if constexpr (EPI == GEPI_STORE) {
        if (m < a.M) {
          float v = rn16(tot[0][r]);
          if (a.residual) v = (float)a.residual[(size_t)m * a.N + n] + v;
          a.y[(size_t)m * a.N + n] = (_Float16)v;
        }
      } else {
        const int which = n < a.n0 ? 0 : (n < a.n0 + a.n1 ? 1 : 2);
        const int nl = which == 0 ? n : (which == 1 ? n - a.n0 : n - a.n0 - a.n1);
        const int pair = (nl % a.head_dim) >> 1;
        const bool odd = nl & 1;
        const float own = rn16(tot[0][r]);
        const float other = dpp_f<0xB1>(own);                // the neighbouring column: the other half of the pair
        if (m < a.M) {
          const int b = m / a.seq_len, pos = a.start_pos + m % a.seq_len;
          float v = own;
          if (which < 2) {
            const h2_t cs = *(const h2_t *)(a.rope_table + ((size_t)pos * (a.head_dim / 2) + pair) * 2);
            const float cc = (float)cs.x, dd = (float)cs.y;
            v = odd ? other * dd + own * cc : own * cc - other * dd;
          }
          if (which == 0) a.y[(size_t)m * a.n0 + nl] = (_Float16)v;
          else {
            _Float16 *cache = which == 1 ? a.cache_k : a.cache_v;
            cache[((size_t)b * a.max_context + pos) * a.n1 + nl] = (_Float16)v;
          }
        }
      }
    }
  };

  f4_t acc[TPW];
#pragma unroll
  for (int tt = 0; tt < TPW; tt++) acc[tt] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < NS; j++)
    if (j < GS) issue(j, ring[j], rscale[j]);
  sk_barrier();                                               // x chunk 0 is in LDS

  for (int gs0 = 0; gs0 < GS; gs0 += NS) {
#pragma unroll
    for (int j = 0; j < NS; j++) {
      const int gs = gs0 + j;
      if (gs < GS) {                                          // the same for every thread of the block
        const int cs = gs / TPW, tt = gs % TPW, c = cs % nck;
        // ---- the step's tile: registers -> LDS patch (the reads of the step before were waited for), then the slot is free
        const h2_t sc = {rscale[j], rscale[j]};
#pragma unroll
        for (int i = 0; i < 8; i++) *(u4_t *)(stg + wr_off + i * 2 * SG_WLS) = ring[j][i];
        __builtin_amdgcn_sched_barrier(0);
        if (gs + NS < GS) issue(gs + NS, ring[j], rscale[j]);
        __builtin_amdgcn_sched_barrier(0);
        const _Float16 *xs = xl + (cs % SG_XB) * 16 * SG_XLS + xoff;
        f4_t r = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int f = 0; f < SG_KC / 32; f++) {
          const h8_t af = *(const h8_t *)&xs[f * 32];
          const uint2 raw = *(const uint2 *)(stg + rd_off + f * 32);
          u4_t o;
          uint32_t lo, hi;
          i8x4_to_h2x2(raw.x, lo, hi); o.x = pk_mul_h2(lo, sc); o.y = pk_mul_h2(hi, sc);
          i8x4_to_h2x2(raw.y, lo, hi); o.z = pk_mul_h2(lo, sc); o.w = pk_mul_h2(hi, sc);
          r = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, __builtin_bit_cast(h8_t, o), r, 0, 0, 0);
        }
#pragma unroll
        for (int t2 = 0; t2 < TPW; t2++)
          if (t2 == tt) acc[t2] += r;
        if (tt == TPW - 1) {
          if (c == nck - 1) {
            // ---- the unit is done
            const int unit = blockIdx.x + (cs / nck) * gridDim.x;
            const int grp = unit / sa.splitk;
            bool mine = true;
            if (sa.splitk > 1) {
              // Partial sums travel between compute units (other XCDs have their own L2): stores and loads that go to the
              // point all of them share, and the count goes up once this wavefront's stores are acknowledged.  No fences: a
              // fence at that scope empties the caches the other blocks are streaming x through.
              uint64_t *part = (uint64_t *)(sa.ws + ((size_t)unit * 4 + wave) * TPW * 256) + lane * 2;
#pragma unroll
              for (int t2 = 0; t2 < TPW; t2++) {
                const uint64_t lo = ((uint64_t)__float_as_uint(acc[t2][1]) << 32) | __float_as_uint(acc[t2][0]);
                const uint64_t hi = ((uint64_t)__float_as_uint(acc[t2][3]) << 32) | __float_as_uint(acc[t2][2]);
                __hip_atomic_store(as_global_mut<uint64_t>(part + t2 * 128), lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(as_global_mut<uint64_t>(part + t2 * 128 + 1), hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              }
              asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
              int old = 0;
              if (lane == 0) old = __hip_atomic_fetch_add(&sa.counters[grp * 4 + wave], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              old = __builtin_amdgcn_readfirstlane(old);
              mine = old == sa.splitk - 1;
              if (mine) {
#pragma unroll
                for (int t2 = 0; t2 < TPW; t2++) acc[t2] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
                for (int p = 0; p < sa.splitk; p++) {
                  const uint64_t *src = (const uint64_t *)(sa.ws + ((size_t)(grp * sa.splitk + p) * 4 + wave) * TPW * 256) + lane * 2;
#pragma unroll
                  for (int t2 = 0; t2 < TPW; t2++) {
                    const uint64_t lo = __hip_atomic_load(as_global<uint64_t>(src + t2 * 128), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const uint64_t hi = __hip_atomic_load(as_global<uint64_t>(src + t2 * 128 + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    acc[t2][0] += __uint_as_float((uint32_t)lo); acc[t2][1] += __uint_as_float((uint32_t)(lo >> 32));
                    acc[t2][2] += __uint_as_float((uint32_t)hi); acc[t2][3] += __uint_as_float((uint32_t)(hi >> 32));
                  }
                }
                if (lane == 0) __hip_atomic_store(&sa.counters[grp * 4 + wave], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
              }
            }
            if (mine) {
#pragma unroll
              for (int ct = 0; ct < S::CT; ct++) {
                f4_t tot[NMAT];
#pragma unroll
                for (int q = 0; q < NMAT; q++) tot[q] = acc[ct * NMAT + q];
                epilogue(tot, grp * S::COLS + (wave * S::CT + ct) * 16);
              }
            }
#pragma unroll
            for (int t2 = 0; t2 < TPW; t2++) acc[t2] = f4_t{0.0f, 0.0f, 0.0f, 0.0f};
          }
          sk_barrier();                                       // chunk cs is consumed, chunk cs + 1 is in its buffer
        }
      }
    }
  }
}

// ---- host side ---------------------------------------------------------------------------------------------------

template <int KIND, int EPI, int MB, int RTW> static int launch_skinny(const GemmArgs &a, int prof_kind) {
  typedef SkFmt<KIND> F;
  typedef SkShape<KIND, EPI, RTW> S;
  constexpr size_t x_bytes = (size_t)SK_XBUF * MB * 16 * (F::KC + 8) * sizeof(_Float16);
  constexpr size_t red_bytes = (size_t)4 * S::NMAT * RTW * MB * 64 * 4 * sizeof(float);
  constexpr size_t lds = x_bytes > red_bytes ? x_bytes : red_bytes;
  if constexpr (lds > 64 * 1024) {
    static bool raised = false;   // one process, one device, one thread: set once per instantiation
    if (!raised) {
      JSG_HIP(hipFuncSetAttribute((const void *)skinny_gemm_kernel<KIND, EPI, MB, RTW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      raised = true;
    }
  }
  JSG_LAUNCH(prof_kind, (skinny_gemm_kernel<KIND, EPI, MB, RTW>), dim3(a.N / S::BR), dim3(SK_THREADS), lds, a);
  return 0;
}
// The LDS-streamed kernel: how many K parts.  Every block should get the same number of units; more parts than needed
// only add partial sums.
template <int EPI, int TPW> static int launch_stream(const GemmArgs &a, int prof_kind, bool *taken) {
  typedef SgShape<EPI, TPW> S;
  *taken = false;
  if (a.M > 16 || a.K % SG_KC || a.N % S::COLS) return 0;
  const int groups = a.N / S::COLS, nchunks = a.K / SG_KC, cus = state().cu_count;
  if (groups > SG_MAX_GROUPS) return 0;
  int best = 0;
  double best_score = 0.0;
  const char *pin = getenv("JSG_SG_SPLITK");
  for (int d = 1; d <= nchunks && d <= 16; d++) {
    if (nchunks % d) continue;
    const int units = groups * d;
    if ((size_t)units * 4 * TPW * 1024 > SG_WS_BYTES) continue;
    if (pin && atoi(pin) != d) continue;
    const int slots = cus;                                 // one block per compute unit (LDS)
    const int rounds = (units + slots - 1) / slots;
    // busy share of the chip, less what the parts cost (their sums travel through memory, and the last one waits for them:
    // on the 8B shapes 2 parts for wq|wk|wv, 4 for wo and w2 and none for w1|w3 measured best)
    const double score = (double)units / ((double)rounds * slots) - (d > 1 ? 0.05 * d : 0.0);
    if (score > best_score + 1e-9) { best_score = score; best = d; }
  }
  if (!best) return 0;
  static float *ws = nullptr;
  static int *counters = nullptr;
  if (!ws) {
    JSG_HIP(hipGetSymbolAddress((void **)&ws, HIP_SYMBOL(sg_scratch)));
    JSG_HIP(hipGetSymbolAddress((void **)&counters, HIP_SYMBOL(sg_counters)));
    JSG_HIP(hipFuncSetAttribute((const void *)stream_gemm_kernel<GEPI_STORE, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SG_LDS));
    JSG_HIP(hipFuncSetAttribute((const void *)stream_gemm_kernel<GEPI_STORE, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SG_LDS));
    JSG_HIP(hipFuncSetAttribute((const void *)stream_gemm_kernel<GEPI_ROPE_KV, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SG_LDS));
    JSG_HIP(hipFuncSetAttribute((const void *)stream_gemm_kernel<GEPI_ROPE_KV, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SG_LDS));
    JSG_HIP(hipFuncSetAttribute((const void *)stream_gemm_kernel<GEPI_SWIGLU, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)SG_LDS));
  }
  SgArgs sa;
  sa.g = a;
  sa.groups = groups; sa.splitk = best; sa.nck = nchunks / best;
  sa.ws = ws; sa.counters = counters;
  const int units = groups * best;
  *taken = true;
  JSG_LAUNCH(prof_kind, (stream_gemm_kernel<EPI, TPW>), dim3(units < cus ? units : cus), dim3(SG_THREADS), SG_LDS, sa);
  return 0;
}
// int8 weights and at most 16 rows: the LDS-streamed kernel.  One tile per wavefront and x chunk (64 columns per unit)
// measured faster than two on every shape of the 8B model (lm_head 97 us against 105), although x is read twice as often.
template <int EPI> static int dispatch_stream(const GemmArgs &a, int prof_kind, bool *taken) {
  *taken = false;
  if (getenv("JSG_GEMM_NO_STREAM")) return 0;
  if constexpr (EPI == GEPI_SWIGLU) return launch_stream<EPI, 2>(a, prof_kind, taken);
  else {
    const char *pin = getenv("JSG_SG_TPW");                  // "1" or "2": tests run both
    if (!(pin && pin[0] == '2')) {
      const int rc = launch_stream<EPI, 1>(a, prof_kind, taken);
      if (*taken || rc) return rc;
    }
    return launch_stream<EPI, 2>(a, prof_kind, taken);
  }
}

// Few rows: the weight-streaming kernel when K is whole chunks.  Every block reads all of x; with two tiles of 16 weight
// rows per block that is half as often.  Measured on the lm_head (8016 tiles) the two-tile shape is no faster and moves
// more HBM bytes (1.5x the weights against 1.24x), so it is only taken when pinned.
template <int KIND, int EPI> static int dispatch_skinny(const GemmArgs &a, int prof_kind, bool *taken) {
  *taken = a.M <= 32 && a.K % SkFmt<KIND>::KC == 0 && a.K / SkFmt<KIND>::KC >= 2 && a.N % 16 == 0 && !getenv("JSG_GEMM_NO_SKINNY");
  if (!*taken) return 0;
  const char *pin = getenv("JSG_GEMM_SKINNY_TILES");     // "1" or "2": tests run small matrices through both
  const bool two = a.N % 32 == 0 && pin && pin[0] == '2';
  if (a.M <= 16) return two ? launch_skinny<KIND, EPI, 1, 2>(a, prof_kind) : launch_skinny<KIND, EPI, 1, 1>(a, prof_kind);
  return two ? launch_skinny<KIND, EPI, 2, 2>(a, prof_kind) : launch_skinny<KIND, EPI, 2, 1>(a, prof_kind);
}

template <int KIND, int EPI, int WGM, int WGN, int TM, int TN, bool DB = false> static int launch_gemm(const GemmArgs &a, int prof_kind) {
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  const int out_per_tile = EPI == GEPI_SWIGLU ? BN / 2 : BN;
  const int tiles = ((a.M + BM - 1) / BM) * (a.N / out_per_tile);
  constexpr size_t lds = (size_t)(DB ? 2 : 1) * (BM + BN) * GEMM_LDS_STRIDE * sizeof(_Float16) + 32 + (KIND == JSGRAD_W_NF4 ? 1024 : 0);
  static_assert(lds <= 160 * 1024, "LDS of one compute unit");
  if constexpr (lds > 64 * 1024) {
    static bool raised = false;   // one process, one device, one thread: set once per instantiation
    if (!raised) {
      JSG_HIP(hipFuncSetAttribute((const void *)gemm_kernel<KIND, EPI, WGM, WGN, TM, TN, DB>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      raised = true;
    }
  }
  JSG_LAUNCH(prof_kind, (gemm_kernel<KIND, EPI, WGM, WGN, TM, TN, DB>), dim3(tiles), dim3(GEMM_THREADS), lds, a);
  return 0;
}

template <int EPI> static int dispatch_gemm(int kind, const GemmArgs &a, int prof_kind) {
  // tall inputs: 256x256 block tiles out of two LDS buffers when the output is wide enough, else 256x128 out of one; short
  // ones (batched decode): 32 rows x 128 columns per block.
  // JSG_GEMM_TILE pins a shape for tests and measurements: "db", "wide" (256x256, one buffer), "tall" (256x128), "small".
  const bool tall = a.M > 64;
  const int n_out = EPI == GEPI_SWIGLU ? 2 * a.N : a.N;
  const char *pin = getenv("JSG_GEMM_TILE");
  const bool can256 = tall && n_out % 256 == 0;
  // unpinned: the largest block shape that still gives (nearly) every CU a block; a prompt of a few hundred rows is better off with
  // 128x128 blocks on all CUs than with 256x256 blocks on a quarter of them
  const int cus = state().cu_count;
  auto blocks_of = [&](int bm, int bn) { return ((a.M + bm - 1) / bm) * (n_out / bn); };
  const bool piped = can256 && (pin ? !strcmp(pin, "db") : 4 * blocks_of(256, 256) >= 3 * cus);
  const bool wide = can256 && pin && !strcmp(pin, "wide");
  const bool small = tall && (pin ? !strcmp(pin, "small") : (!piped && blocks_of(256, 128) < cus));
  bool taken = false;
  if (kind == JSGRAD_W_F16) { const int rc = dispatch_skinny<JSGRAD_W_F16, EPI>(a, prof_kind, &taken); if (taken) return rc; }
  // int8, at most 16 rows: the LDS-streamed kernel, except for matrices so small that its K parts cost more than they bring
  // (wo of the 8B shape, 16.8 MB: 9.7 us against 8.5 us with the direct-operand kernel; wq|wk|wv, 25 MB: 12.3 against 13.5)
  static const size_t stream_min = getenv("JSG_SG_MIN_BYTES") ? (size_t)atoll(getenv("JSG_SG_MIN_BYTES")) : (size_t)20 << 20;
  const bool small_matrix = EPI == GEPI_STORE && (size_t)a.N * (size_t)a.K < stream_min;
  if (kind == JSGRAD_W_I8 && !small_matrix) { const int rc = dispatch_stream<EPI>(a, prof_kind, &taken); if (taken || rc) return rc; }
  if (kind == JSGRAD_W_I8) { const int rc = dispatch_skinny<JSGRAD_W_I8, EPI>(a, prof_kind, &taken); if (taken) return rc; }
  if (kind == JSGRAD_W_NF4) { const int rc = dispatch_skinny<JSGRAD_W_NF4, EPI>(a, prof_kind, &taken); if (taken) return rc; }
#define JSG_CASE(K)                                                                                                    \
  case K:                                                                                                              \
    if (piped) return launch_gemm<K, EPI, 2, 2, 4, 4, true>(a, prof_kind);                                            \
    if (wide) return launch_gemm<K, EPI, 2, 2, 4, 4>(a, prof_kind);                                                   \
    if (small) return launch_gemm<K, EPI, 2, 2, 2, 2>(a, prof_kind);                                                  \
    return tall ? launch_gemm<K, EPI, 2, 2, 4, 2>(a, prof_kind) : launch_gemm<K, EPI, 1, 4, 1, EPI == GEPI_SWIGLU ? 2 : 1>(a, prof_kind);
  switch (kind) {
    JSG_CASE(JSGRAD_W_F16)
    JSG_CASE(JSGRAD_W_I8)
    JSG_CASE(JSGRAD_W_NF4)
  }
#undef JSG_CASE
  return fail("jsgrad_hip_gemm: weight kind %d is not built for several rows (fp16, int8 and nf4 are)", kind);
}

// largest column tile any configuration uses: output widths must be multiples of it
constexpr int GEMM_N_ALIGN = 128;

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

static int check_gemm(const char *who, int kind, int rows, int in_f) {
  JSG_REQUIRE(kind == JSGRAD_W_F16 || kind == JSGRAD_W_I8 || kind == JSGRAD_W_NF4, "%s: weight kind %d is not built for several rows (fp16, int8 and nf4 are)", who, kind);
  JSG_REQUIRE(rows > 0, "%s: %d rows", who, rows);
  JSG_REQUIRE(in_f > 0 && in_f % GEMM_BK == 0, "%s: in_features %d must be a positive multiple of %d", who, in_f, GEMM_BK);
  return 0;
}

}  // namespace jsg

using namespace jsg;

extern "C" {

int jsgrad_hip_gemm(int kind, const void *w, const void *scale, int out_f, int in_f, const void *x, int rows, void *y, const void *residual) {
  JSG_READY();
  if (int rc = check_gemm("jsgrad_hip_gemm", kind, rows, in_f)) return rc;
  JSG_REQUIRE(w && x && y, "jsgrad_hip_gemm: null pointer argument");
  JSG_REQUIRE(kind == JSGRAD_W_F16 || scale, "jsgrad_hip_gemm: quantised weights need their scales");
  JSG_REQUIRE(out_f > 0 && out_f % GEMM_N_ALIGN == 0, "jsgrad_hip_gemm: out_features %d must be a positive multiple of %d", out_f, GEMM_N_ALIGN);
  JSG_REQUIRE(aligned16(w) && aligned16(x) && aligned16(y) && aligned16(residual), "jsgrad_hip_gemm: w, x, y and residual must be 16-byte aligned");
  GemmArgs a = {};
  a.w0 = w; a.s0 = (const _Float16 *)scale; a.n0 = out_f;
  a.M = rows; a.N = out_f; a.K = in_f;
  a.x = (const _Float16 *)x; a.y = (_Float16 *)y; a.residual = (const _Float16 *)residual;
  return dispatch_gemm<GEPI_STORE>(kind, a, PROF_GEMM);
}

int jsgrad_hip_gemm_qkv_rope(int kind, const void *wq, const void *sq, const void *wk, const void *sk, const void *wv, const void *sv, const void *x,
                             int rows, int seq_len, int start_pos, const void *rope_table, void *q_out, void *cache_k, void *cache_v, int dim,
                             int n_heads, int n_kv_heads, int head_dim, int max_context) {
  JSG_READY();
  if (int rc = check_gemm("jsgrad_hip_gemm_qkv_rope", kind, rows, dim)) return rc;
  JSG_REQUIRE(wq && wk && wv && x && rope_table && q_out && cache_k && cache_v, "jsgrad_hip_gemm_qkv_rope: null pointer argument");
  JSG_REQUIRE(kind == JSGRAD_W_F16 || (sq && sk && sv), "jsgrad_hip_gemm_qkv_rope: quantised weights need their scales");
  JSG_REQUIRE(head_dim > 0 && head_dim % 8 == 0 && n_heads > 0 && n_kv_heads > 0, "jsgrad_hip_gemm_qkv_rope: bad head geometry (head_dim a multiple of 8)");
  JSG_REQUIRE(aligned16(wq) && aligned16(wk) && aligned16(wv) && aligned16(x) && aligned16(rope_table) && aligned16(q_out) && aligned16(cache_k) && aligned16(cache_v),
              "jsgrad_hip_gemm_qkv_rope: weights, x, rope_table, q_out and the caches must be 16-byte aligned");
  const int nq = n_heads * head_dim, nkv = n_kv_heads * head_dim;
  JSG_REQUIRE(nq % GEMM_N_ALIGN == 0 && nkv % GEMM_N_ALIGN == 0, "jsgrad_hip_gemm_qkv_rope: n_heads*head_dim %d and n_kv_heads*head_dim %d must be multiples of %d", nq, nkv,
              GEMM_N_ALIGN);
  JSG_REQUIRE(seq_len > 0 && rows % seq_len == 0, "jsgrad_hip_gemm_qkv_rope: %d rows are not whole sequences of %d", rows, seq_len);
  JSG_REQUIRE(start_pos >= 0 && start_pos + seq_len <= max_context, "jsgrad_hip_gemm_qkv_rope: positions [%d, %d) outside the cache of %d", start_pos,
              start_pos + seq_len, max_context);
  GemmArgs a = {};
  a.w0 = wq; a.w1 = wk; a.w2 = wv;
  a.s0 = (const _Float16 *)sq; a.s1 = (const _Float16 *)sk; a.s2 = (const _Float16 *)sv;
  a.n0 = nq; a.n1 = nkv; a.n2 = nkv;
  a.M = rows; a.N = nq + 2 * nkv; a.K = dim;
  a.x = (const _Float16 *)x; a.y = (_Float16 *)q_out;
  a.rope_table = (const _Float16 *)rope_table; a.cache_k = (_Float16 *)cache_k; a.cache_v = (_Float16 *)cache_v;
  a.seq_len = seq_len; a.start_pos = start_pos; a.head_dim = head_dim; a.max_context = max_context;
  return dispatch_gemm<GEPI_ROPE_KV>(kind, a, PROF_GEMM);
}

int jsgrad_hip_gemm_ffn_gate(int kind, const void *w1, const void *s1, const void *w3, const void *s3, const void *x, int rows, void *y, int dim,
                             int hidden) {
  JSG_READY();
  if (int rc = check_gemm("jsgrad_hip_gemm_ffn_gate", kind, rows, dim)) return rc;
  JSG_REQUIRE(w1 && w3 && x && y, "jsgrad_hip_gemm_ffn_gate: null pointer argument");
  JSG_REQUIRE(kind == JSGRAD_W_F16 || (s1 && s3), "jsgrad_hip_gemm_ffn_gate: quantised weights need their scales");
  JSG_REQUIRE(hidden > 0 && hidden % GEMM_N_ALIGN == 0, "jsgrad_hip_gemm_ffn_gate: hidden_dim %d must be a positive multiple of %d", hidden, GEMM_N_ALIGN);
  JSG_REQUIRE(aligned16(w1) && aligned16(w3) && aligned16(x) && aligned16(y), "jsgrad_hip_gemm_ffn_gate: w1, w3, x and g must be 16-byte aligned");
  GemmArgs a = {};
  a.w0 = w1; a.w1 = w3; a.s0 = (const _Float16 *)s1; a.s1 = (const _Float16 *)s3;
  a.n0 = hidden; a.n1 = hidden;
  a.M = rows; a.N = hidden; a.K = dim;
  a.x = (const _Float16 *)x; a.y = (_Float16 *)y;
  return dispatch_gemm<GEPI_SWIGLU>(kind, a, PROF_GEMM);
}

}  // extern "C"
