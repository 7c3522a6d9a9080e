/*
 * jsgrad_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C CPU restatement of the arithmetic that jsgrad's CLANG device performs for
 * Llama-3 inference.  One thread unless or_set_threads() says otherwise (the reference's
 * CLANG device is single-threaded; threads only split independent outputs among them,
 * every output is computed by the same sequence of operations either way).  It exists only as the checker for the HIP
 * path (tests, the smoke check and the cpu_baseline leg of the benchmark); the
 * product library never links, loads or calls it.
 *
 * jsgrad cannot run where this is built (no Deno/Bun, Node too old), so this file is
 * a restatement from reading the reference sources.  Citations are
 * /root/reference/<file>:<line>.
 *
 * Rounding model (what jsgrad's generated C does, renderer/cstyle.ts:116-193,203-219):
 *   R1  buffers hold their dtype: `__fp16` for half tensors, float for float tensors;
 *   R2  inside one generated kernel every ALU expression is evaluated in `float`
 *       (C promotes `__fp16` operands); rounding to fp16 happens at explicit CAST
 *       uops, at SSA variables that have more than one use (typed `__fp16`), at
 *       half constants (rendered `(__fp16)(<x>f)`, cstyle.ts:35) and at stores;
 *   R3  sums of half tensors accumulate in float (dtype.ts:243-248, tensor.ts:1967-1970)
 *       and are cast back to half;
 *   R4  EXP2 / SIN are the polynomial versions of ops.ts:1625-1676 because
 *       ClangRenderer drops the native ops (cstyle.ts:215);
 *   R5  kernel boundaries (= where R1 applies) follow the scheduler rules
 *       "realise before expand" and "one reduce per kernel" (engine/schedule.ts:283-297,
 *       472-483) as listed next to each function below.
 * Accumulation order: one accumulator per output, sequential over the reduce axis
 * (codegen/kernel.ts:609-633 upcasts outputs by 4 and unrolls the reduce by 4, which
 * keeps one chain per output).  Compiled with -ffp-contract=off so no FMA is formed.
 *
 * Parity status per function (see also the pinning tests in tests/test_oracle_*.py):
 *   pinned by closed form / brute force / an independent fp64 implementation:
 *     fp16 conversion, or_xexp2f, or_xsinf, or_freqs_cis, int8 + nf4 dequant,
 *     int8 quantise invariants, nf4 quantise (nearest code), linear, rmsnorm, rope,
 *     attention (incl. GQA map and the cache-vs-full-sequence invariant), silu,
 *     argmax tie rule, embedding gather.
 *   parity unpinned (only a jsgrad run could pin; inside the 1e-2 budget):
 *     the exact fp16 rounding points of activations that depend on fusion decisions
 *     (R5), the exact int8 code where the scaled weight lands on a .5 boundary, the
 *     low bits of sums (accumulation order), FMA contraction under -march=native.
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
static inline int omp_thread(void) { return omp_get_thread_num(); }
#else
static inline int omp_thread(void) { return 0; }
#endif

/* ------------------------------------------------------------------ fp16 <-> fp32 */

static inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }
static inline float rn16(float f) { return h2f(f2h(f)); }
/* round to the activation dtype: fp16 (act16=1) or identity for float tensors */
static inline float rn_act(float f, int act16) { return act16 ? rn16(f) : f; }

/* Software IEEE binary16 round-to-nearest-even conversion, independent of F16C; the
 * tests check it against the hardware path over all 2^16 halves and many floats. */
uint16_t or_f2h_soft(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t mag = x & 0x7fffffffu;
  if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u | ((mag >> 13) & 0x3ffu) : 0));
  if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (mag < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 rounds to 0 */
  int32_t e = (int32_t)(mag >> 23) - 127;
  uint32_t m = (mag & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (e < -14) { shift = 13 + (-14 - e); base = 0; }
  else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
  uint32_t q = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
  uint32_t r = base + q;
  if (rem > half || (rem == half && (r & 1u))) r++;
  return (uint16_t)(sign | r);
}
float or_h2f_soft(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3ffu, x;
  if (e == 31) x = sign | 0x7f800000u | (m << 13);
  else if (e == 0) {
    if (m == 0) x = sign;
    else { int k = 0; while (!(m & 0x400u)) { m <<= 1; k++; } x = sign | ((uint32_t)(113 - k) << 23) | ((m & 0x3ffu) << 13); }
  } else x = sign | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &x, 4);
  return f;
}
void or_f32_to_f16(const float *src, uint16_t *dst, long n) { for (long i = 0; i < n; i++) dst[i] = f2h(src[i]); }
void or_f16_to_f32(const uint16_t *src, float *dst, long n) { for (long i = 0; i < n; i++) dst[i] = h2f(src[i]); }

/* ------------------------------------------------------------------ transcendentals */

/* rintk, ops.ts:1467-1470: add +-0.5 then C cast (truncation). */
static inline int32_t rintk(float d) {
  float t = d + (d < 0.0f ? -0.5f : 0.5f);
  if (!(t > -2147483000.0f)) return INT32_MIN; /* out-of-range casts only occur where the result is masked */
  if (!(t < 2147483000.0f)) return INT32_MIN;
  return (int32_t)t;
}
/* pow2if, ops.ts:1473-1476: build 2^q from the exponent field. */
static inline float pow2if(int32_t q) {
  uint32_t b = (uint32_t)(q + 127) << 23;
  float f;
  memcpy(&f, &b, 4);
  return f;
}
/* ldexp2k, ops.ts:1493-1496. */
static inline float ldexp2k(float d, int32_t e) { return (d * pow2if(e >> 1)) * pow2if(e - (e >> 1)); }

/* _lazy_map_numbers(d, 0, 0, 0, d), ops.ts:1455 */
static inline float mask_nonfinite(float d) { return (d != INFINITY) ? ((d != d) ? 0.0f : ((d != -INFINITY) ? d : 0.0f)) : 0.0f; }

/* xexp2 for float32, ops.ts:1650-1673.  polyN is Horner from the first coefficient
 * (helpers/helpers.ts:810). */
float or_xexp2f(float d) {
  static const float c[7] = {0.1535920892e-3f, 0.1339262701e-2f, 0.9618384764e-2f, 0.5550347269e-1f, 0.2402264476e+0f, 0.6931471825e+0f, 1.0f};
  float x = mask_nonfinite(d);
  int32_t q = rintk(x);
  float s = x - (float)q;
  float u = c[0];
  for (int i = 1; i < 7; i++) u = u * s + c[i];
  u = ldexp2k(u, q);
  if (d >= 128.0f) u = INFINITY;
  if (d < -150.0f) u = 0.0f;
  if (d != d) u = NAN;
  return u;
}
/* xexp2 when the tensor dtype is half (ops.ts:1650-1673 with d.dtype == float16): the
 * argument is an fp16 value, the coefficients are half constants (rounded to fp16 by the
 * renderer, R2), the Horner chain itself is a float expression, and the saturation
 * bounds are [23, -22].  `d` must already be an fp16-representable float. */
float or_xexp2h(float d) {
  static const float c32[7] = {0.1535920892e-3f, 0.1339262701e-2f, 0.9618384764e-2f, 0.5550347269e-1f, 0.2402264476e+0f, 0.6931471825e+0f, 1.0f};
  float x = mask_nonfinite(d);
  int32_t q = rintk(x); /* int16 in the reference; |x| <= 65504 so no overflow before masking matters */
  float s = x - (float)q;
  float u = rn16(c32[0]);
  for (int i = 1; i < 7; i++) u = u * s + rn16(c32[i]);
  if (q > 60) q = 60;   /* masked below; keeps pow2if in range */
  if (q < -60) q = -60;
  u = ldexp2k(u, q);
  if (d >= 23.0f) u = INFINITY;
  if (d < -22.0f) u = 0.0f;
  if (d != d) u = NAN;
  return u;
}

/* sin_poly for float32, ops.ts:1609-1615 */
static inline float sin_poly(float d) {
  static const float c[5] = {2.6083159809786593541503e-06f, -0.0001981069071916863322258f, 0.00833307858556509017944336f, -0.166666597127914428710938f, 1.0f};
  float d2 = d * d, u = c[0];
  for (int i = 1; i < 5; i++) u = u * d2 + c[i];
  return d * u;
}
/* cody_waite_reduction, float32 branch, ops.ts:1577-1604 */
static inline void cody_waite(float d, float *r, int32_t *q) {
  const float m_1_pi = 0.318309886183790671537767526745028724f;
  int32_t quad = rintk(d * m_1_pi);
  float qf = (float)quad;
  float x = d;
  x = qf * -3.1414794921875f + x;
  x = qf * -0.00011315941810607910156f + x;
  x = qf * -1.9841872589410058936e-09f + x;
  x = qf * -1.2154201256553420762e-10f + x;
  *r = x;
  *q = quad;
}
/* payne_hanek_reduction for float32, ops.ts:1528-1571 */
static inline void payne_hanek(float d, float *r_out, int32_t *q_out) {
  static const uint32_t two_over_pi_f[7] = {0x00000000u, 0x28be60dbu, 0x9391054au, 0x7f09d5f4u, 0x7d4d3770u, 0x36d8a566u, 0x4f10e410u};
  uint32_t bits;
  memcpy(&bits, &d, 4);
  /* frexp, ops.ts:1498-1510 */
  uint32_t expo = (bits >> 23) & 255u;
  uint32_t mb = (bits & 0x807FFFFFu) | 0x3F000000u;
  float f;
  memcpy(&f, &mb, 4);
  int32_t e = (int32_t)expo - 127 + 1;
  uint64_t ia = (uint64_t)(f * 4.294967296e9f);
  uint64_t i = ((uint64_t)(int64_t)e) >> 5;
  int32_t es = e & 31;
  int32_t offset = 32 - es;
  uint32_t a[4];
  for (int k = 0; k < 4; k++) { /* _take, ops.ts:1547-1552: table[i+k] while the index stays below len-1 */
    a[k] = 0;
    for (int count = 0; count + k < 6; count++)
      if (i == (uint64_t)count) { a[k] = two_over_pi_f[count + k]; break; }
  }
#define SHL_LAZY(x, y) ((uint32_t)((uint64_t)(x) * (uint64_t)pow2if(y)))
#define SHR_LAZY(x, y) ((uint32_t)((uint64_t)(x) / (uint64_t)pow2if(y)))
  uint32_t hi = SHL_LAZY(a[0], es) | SHR_LAZY(a[1], offset);
  uint32_t mi = SHL_LAZY(a[1], es) | SHR_LAZY(a[2], offset);
  uint32_t lo = SHL_LAZY(a[2], es) | SHR_LAZY(a[3], offset);
#undef SHL_LAZY
#undef SHR_LAZY
  uint64_t p = ((ia * (uint64_t)hi) << 32) + ia * (uint64_t)mi + ((ia * (uint64_t)lo) >> 32);
  int32_t q = (int32_t)(p >> 62);
  p &= 0x3fffffffffffffffull;
  float r = (float)p * 3.4061215800865545e-19f;
  if (f < 0.5f) { *r_out = r; *q_out = q; }
  else { *r_out = r - 1.5707963267948966f; *q_out = q + 1; }
}
/* xsin for float32, ops.ts:1625-1644 (fast=false, switch_over=30) */
float or_xsinf(float d) {
  float x = mask_nonfinite(d);
  float x_sign = (x != 0.0f) ? (x < 0.0f ? -1.0f : 1.0f) : 0.0f;
  float x_abs = x * x_sign;
  float result;
  if (x_abs < 30.0f) { /* sin_poly_small, ops.ts:1617-1620 */
    float r; int32_t q;
    cody_waite(x_abs, &r, &q);
    result = sin_poly(r) * ((q & 1) ? -1.0f : 1.0f);
  } else {             /* sin_poly_large, ops.ts:1622-1625 */
    float r; int32_t q;
    payne_hanek(x_abs, &r, &q);
    result = sin_poly(r + ((q & 1) ? 1.5707963267948966f : 0.0f)) * ((q & 2) ? -1.0f : 1.0f);
  }
  result = result * x_sign;
  if (!(d == d) || d == INFINITY || d == -INFINITY) result = NAN;
  return result;
}
void or_xexp2f_vec(const float *x, float *y, long n) { for (long i = 0; i < n; i++) y[i] = or_xexp2f(x[i]); }
void or_xexp2h_vec(const float *x, float *y, long n) { for (long i = 0; i < n; i++) y[i] = or_xexp2h(x[i]); }
void or_xsinf_vec(const float *x, float *y, long n) { for (long i = 0; i < n; i++) y[i] = or_xsinf(x[i]); }

/* Tensor.exp for float tensors: tensor.ts:147-154 (x * (1/ln2)).exp2() */
static inline float exp_f32(float x) { return or_xexp2f(x * 1.4426950408889634f); }

/* silu(a) = a * sigmoid(a), tensor.ts:2909-2911, 3210-3226.
 * float tensors:  1 / (1 + exp2(a * (-1/ln2)))
 * half tensors :  the argument of exp2 has several uses inside xexp2, so it is an
 *                 `__fp16` SSA variable (R2): d = RN16(a * RN16(-1/ln2)). */
static inline float silu_act(float a, int act16) {
  float u;
  if (act16) u = or_xexp2h(rn16(a * rn16(-1.4426950408889634f)));
  else u = or_xexp2f(a * -1.4426950408889634f);
  return a * (1.0f / (1.0f + u));
}
void or_silu_vec(const float *x, float *y, long n, int act16) { for (long i = 0; i < n; i++) y[i] = silu_act(x[i], act16); }

/* ------------------------------------------------------------------ RoPE table */

/* precompute_freqs_cis, models/llama.ts:10-14, all float32:
 *   freqs_i = 1 / theta^(2i/dim)      via pow(theta, reverse) = exp(t*ln(theta)) (tensor.ts:3709)
 *   table[pos][i] = (cos(pos*freqs_i), sin(pos*freqs_i)),  cos(x) = sin(pi/2 - x) (tensor.ts:2964-2966)
 * out is [end][dim/2][2]. */
void or_freqs_cis(int dim, int end, float theta, float *out) {
  int half = dim / 2;
  float inv_dim = (float)(1.0 / (double)dim);
  float ln_theta = (float)log((double)theta);
  float *fr = (float *)malloc(sizeof(float) * (size_t)half);
  for (int i = 0; i < half; i++) {
    float t = (float)(2 * i) * inv_dim;
    float p = exp_f32(t * ln_theta);
    fr[i] = 1.0f * (1.0f / p);
  }
  for (int pos = 0; pos < end; pos++)
    for (int i = 0; i < half; i++) {
      float a = (float)pos * fr[i];
      out[((size_t)pos * half + i) * 2 + 0] = or_xsinf(1.5707963267948966f - a);
      out[((size_t)pos * half + i) * 2 + 1] = or_xsinf(a);
    }
  free(fr);
}

/* ------------------------------------------------------------------ quantisers */

/* Tensor.round, tensor.ts:3054-3057: half-to-even built from trunc/ceil/floor. */
static inline float round_half_even(float x) {
  int32_t ti = (int32_t)x;
  float b = (float)ti * 0.5f;
  int even = ((float)(int32_t)b == b);
  float y;
  if ((x > 0.0f) == even) { /* ceil(x - 0.5) */
    float v = x - 0.5f, t = (float)(int32_t)v;
    y = (v > t) ? t + 1.0f : t;
  } else {                  /* floor(x + 0.5) */
    float v = x + 0.5f, t = (float)(int32_t)v;
    y = (v < t) ? t - 1.0f : t;
  }
  return y;
}
void or_round_vec(const float *x, float *y, long n) { for (long i = 0; i < n; i++) y[i] = round_half_even(x[i]); }

/* Int8Linear.quantize, models/llama3.ts:37-60, for one [out,in] matrix.
 *   v      = w.cast(half)
 *   scale  = RN16( absmax_row * RN16(1/127) )            (half constant, R2)
 *   code   = round( RN16( v * (1/scale) ) ).cast(int8)   (the scaled value has several
 *            uses inside round(), so it is an `__fp16` SSA variable, R2)
 * A zero row gives scale 0 and codes from 0*inf = nan; the reference has the same hole,
 * here such rows get code 0. */
void or_int8_quantize(const float *w, int out_f, int in_f, int8_t *q, uint16_t *scale) {
  const float c127 = rn16((float)(1.0 / 127.0));
  for (int o = 0; o < out_f; o++) {
    const float *row = w + (size_t)o * in_f;
    float amax = 0.0f;
    for (int k = 0; k < in_f; k++) { float a = fabsf(rn16(row[k])); if (a > amax) amax = a; }
    uint16_t sh = f2h(amax * c127);
    float s = h2f(sh);
    scale[o] = sh;
    float inv = 1.0f / s;
    for (int k = 0; k < in_f; k++) {
      float t = rn16(rn16(row[k]) * inv);
      float r = (s == 0.0f) ? 0.0f : round_half_even(t);
      q[(size_t)o * in_f + k] = (int8_t)(int32_t)r;
    }
  }
}
/* materialised Int8 dequantisation, llama3.ts:35,75: RN16( float(code) * float(scale) ),
 * one exact float product rounded once. */
void or_int8_dequant(const int8_t *q, const uint16_t *scale, int out_f, int in_f, uint16_t *w16) {
  for (int o = 0; o < out_f; o++) {
    float s = h2f(scale[o]);
    for (int k = 0; k < in_f; k++) w16[(size_t)o * in_f + k] = f2h((float)q[(size_t)o * in_f + k] * s);
  }
}

/* NF4 code book, llama3.ts:80-81 (values are rounded to fp16 when the CODE tensor is built) */
static const float NF4_CODE[16] = {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f, -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
                                   0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};
void or_nf4_code(float *out16) { for (int i = 0; i < 16; i++) out16[i] = rn16(NF4_CODE[i]); }

/* NF4Linear.quantize, llama3.ts:98-114, block = 64 consecutive elements of the
 * flattened [out,in] weight: scale = absmax (kept in fp16), code = argmin |x/scale - CODE|
 * with ties to the lowest index (argmin -> argmax first-index rule, tensor.ts:2314-2320),
 * two codes per byte: even element in the high nibble, odd element in the low nibble (:105). */
void or_nf4_quantize(const float *w, long n, uint8_t *packed, uint16_t *scale) {
  float code[16];
  or_nf4_code(code);
  long nblk = n / 64;
  for (long b = 0; b < nblk; b++) {
    const float *x = w + b * 64;
    float amax = 0.0f;
    for (int k = 0; k < 64; k++) { float a = fabsf(x[k]); if (a > amax) amax = a; }
    scale[b] = f2h(amax);
    float inv = 1.0f / amax;
    uint8_t c[64];
    for (int k = 0; k < 64; k++) {
      float r = x[k] * inv, best = INFINITY;
      int bi = 0;
      for (int j = 0; j < 16; j++) { float dlt = fabsf(r - code[j]); if (dlt < best) { best = dlt; bi = j; } }
      c[k] = (uint8_t)bi;
    }
    for (int k = 0; k < 32; k++) packed[b * 32 + k] = (uint8_t)(c[2 * k] * 16 + c[2 * k + 1]);
  }
}
/* NF4Linear.call dequantisation, llama3.ts:91-96: RN16( CODE16[nibble] * scale[block] ). */
void or_nf4_dequant(const uint8_t *packed, const uint16_t *scale, long n, uint16_t *w16) {
  float code[16];
  or_nf4_code(code);
  for (long i = 0; i < n / 2; i++) {
    float s = h2f(scale[(2 * i) / 64]);
    w16[2 * i] = f2h(code[packed[i] >> 4] * s);
    w16[2 * i + 1] = f2h(code[packed[i] & 15] * s);
  }
}

/* ------------------------------------------------------------------ layers */

enum { OR_W_F32 = 0, OR_W_F16 = 1, OR_W_I8 = 2, OR_W_NF4 = 3 };
typedef struct {
  int kind, out_f, in_f;
  const void *w;         /* float / uint16 / int8 [out][in], or packed nf4 [out*in/2] */
  const uint16_t *scale; /* i8: [out]; nf4: [out*in/64] */
} or_linear_t;

/* Linear.call nn/index.ts:411 -> Tensor.linear tensor.ts:3800 -> dot :2593-2605;
 * Int8Linear.call llama3.ts:35; NF4Linear.call llama3.ts:91-97.
 * y[o] = RN_act( sum_k float(x[k]) * W[o][k] ), float accumulation, sequential in k.
 *   f32/f16 : W[o][k] as stored.
 *   int8/nf4, one input row (materialised=0): multiplying by the scale is an elementwise
 *             op on a tensor that is not expanded, so it fuses into the reduce kernel
 *             (schedule.ts:472-483): term = x * (float(code)*scale); the inner product is
 *             exact in float (8+11 / 11+11 significant bits), the outer one rounds to float (R2).
 *             (For nf4 the CODE gather is a reduce of its own and is realised first, but it
 *             only yields the exact fp16 code values.)
 *   int8/nf4, several input rows (materialised=1): the weight is expanded over the rows,
 *             which realises the dequantised matrix in fp16 first: W = RN16(float(code)*scale). */
static int g_threads = 1;
/* Threads for the loops over independent outputs (rows of a Linear, heads of the attention).  1 = the reference's way. */
void or_set_threads(int n) { g_threads = n < 1 ? 1 : n; }

/* The order in which a one-row Linear adds its products is not fixed by anything this file can check (see "parity
 * unpinned" at the top).  0 (the default) is the restatement's reading of the reference: one accumulator, sequential over
 * the reduce axis.  1 is another legitimate order of the SAME products: eight interleaved accumulators (element k goes to
 * accumulator k % 8) added pairwise at the end, the shape a vectorised loop has.  It exists so that tests can measure how
 * far two float summation orders drift apart through a deep model, and hold the HIP path (whose order is a third one:
 * lanes, then a tree) to that yardstick; it is never the reference arithmetic. */
static int g_sum_order = 0;
void or_set_sum_order(int mode) { g_sum_order = mode ? 1 : 0; }

/* one weight row as the floats the products use: W[o][k] as stored, code*scale, or RN16(code*scale) */
static void weight_row(const or_linear_t *L, int o, int materialised, const float *code, float *wrow) {
  const int in_f = L->in_f;
  switch (L->kind) {
    case OR_W_F32: memcpy(wrow, (const float *)L->w + (size_t)o * in_f, sizeof(float) * (size_t)in_f); break;
    case OR_W_F16: { const uint16_t *w = (const uint16_t *)L->w + (size_t)o * in_f; for (int k = 0; k < in_f; k++) wrow[k] = h2f(w[k]); break; }
    case OR_W_I8: {
      const int8_t *w = (const int8_t *)L->w + (size_t)o * in_f;
      const float s = h2f(L->scale[o]);
      if (materialised) for (int k = 0; k < in_f; k++) wrow[k] = rn16((float)w[k] * s);
      else for (int k = 0; k < in_f; k++) wrow[k] = (float)w[k] * s;
      break;
    }
    default: {
      const uint8_t *w = (const uint8_t *)L->w + ((size_t)o * in_f) / 2;
      const uint16_t *sc = L->scale + ((size_t)o * in_f) / 64;
      for (int k = 0; k < in_f; k += 2) {
        float s = h2f(sc[k / 64]);
        uint8_t b = w[k / 2];
        float w0 = code[b >> 4] * s, w1 = code[b & 15] * s;
        if (materialised) { w0 = rn16(w0); w1 = rn16(w1); }
        wrow[k] = w0; wrow[k + 1] = w1;
      }
    }
  }
}

void or_linear_ex(const or_linear_t *L, const float *x, float *y, int act16, int materialised) {
  const int in_f = L->in_f;
  float code[16];
  or_nf4_code(code);
  if (g_sum_order == 1) {
#pragma omp parallel num_threads(g_threads) if (g_threads > 1)
    {
      float *wrow = (float *)malloc(sizeof(float) * (size_t)in_f);
#pragma omp for schedule(static)
      for (int o = 0; o < L->out_f; o++) {
        weight_row(L, o, materialised, code, wrow);
        float a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        for (int k = 0; k < in_f; k++) a[k & 7] = a[k & 7] + x[k] * wrow[k];
        y[o] = rn_act(((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7])), act16);
      }
      free(wrow);
    }
    return;
  }
#pragma omp parallel for schedule(static) num_threads(g_threads) if (g_threads > 1)
  for (int o = 0; o < L->out_f; o++) {
    float acc = 0.0f;
    switch (L->kind) {
      case OR_W_F32: { const float *w = (const float *)L->w + (size_t)o * in_f; for (int k = 0; k < in_f; k++) acc = acc + x[k] * w[k]; break; }
      case OR_W_F16: { const uint16_t *w = (const uint16_t *)L->w + (size_t)o * in_f; for (int k = 0; k < in_f; k++) acc = acc + x[k] * h2f(w[k]); break; }
      case OR_W_I8: {
        const int8_t *w = (const int8_t *)L->w + (size_t)o * in_f;
        const float s = h2f(L->scale[o]);
        if (materialised) for (int k = 0; k < in_f; k++) acc = acc + x[k] * rn16((float)w[k] * s);
        else for (int k = 0; k < in_f; k++) acc = acc + x[k] * ((float)w[k] * s);
        break;
      }
      default: {
        const uint8_t *w = (const uint8_t *)L->w + ((size_t)o * in_f) / 2;
        const uint16_t *sc = L->scale + ((size_t)o * in_f) / 64;
        for (int k = 0; k < in_f; k += 2) {
          float s = h2f(sc[k / 64]);
          uint8_t b = w[k / 2];
          float w0 = code[b >> 4] * s, w1 = code[b & 15] * s;
          if (materialised) { w0 = rn16(w0); w1 = rn16(w1); }
          acc = acc + x[k] * w0;
          acc = acc + x[k + 1] * w1;
        }
      }
    }
    y[o] = rn_act(acc, act16);
  }
}
void or_linear(const or_linear_t *L, const float *x, float *y, int act16) { or_linear_ex(L, x, y, act16, 0); }

/* The same Linear for S input rows x[S][in_f] -> y[S][out_f].  Every y[s][o] is the sum or_linear_ex forms (one float
 * accumulator, sequential in k, a rounded product added at every step); only the organisation differs: a weight row is
 * turned into floats once, and OR_TILE input rows advance through k side by side (their accumulators are independent, so
 * the compiler may keep them in one vector register: IEEE multiply and add per lane, no contraction). */
#define OR_TILE 32
void or_linear_rows(const or_linear_t *L, const float *x, int S, float *y, int act16, int materialised) {
  if (S == 1) { or_linear_ex(L, x, y, act16, materialised); return; }
  const int in_f = L->in_f, out_f = L->out_f;
  const int ntile = (S + OR_TILE - 1) / OR_TILE;
  /* xt[tile][k][OR_TILE]: the input transposed inside tiles of rows (rows past S are zero and never stored) */
  float *xt = (float *)calloc((size_t)ntile * in_f * OR_TILE, sizeof(float));
  for (int s = 0; s < S; s++)
    for (int k = 0; k < in_f; k++) xt[((size_t)(s / OR_TILE) * in_f + k) * OR_TILE + s % OR_TILE] = x[(size_t)s * in_f + k];
  float code[16];
  or_nf4_code(code);
#pragma omp parallel num_threads(g_threads) if (g_threads > 1)
  {
    float *wrow = (float *)malloc(sizeof(float) * (size_t)in_f);
#pragma omp for schedule(static)
    for (int o = 0; o < out_f; o++) {
      weight_row(L, o, materialised, code, wrow);
      for (int t = 0; t < ntile; t++) {
        const float *xp = xt + (size_t)t * in_f * OR_TILE;
        float acc[OR_TILE];
        for (int i = 0; i < OR_TILE; i++) acc[i] = 0.0f;
        for (int k = 0; k < in_f; k++) {
          const float wk = wrow[k];
          for (int i = 0; i < OR_TILE; i++) acc[i] = acc[i] + xp[(size_t)k * OR_TILE + i] * wk;
        }
        for (int i = 0; i < OR_TILE && t * OR_TILE + i < S; i++) y[(size_t)(t * OR_TILE + i) * out_f + o] = rn_act(acc[i], act16);
      }
    }
    free(wrow);
  }
  free(xt);
}
/* ctypes-friendly wrapper for n_rows input rows: more than one row sees the weight expanded over the rows (materialised) */
void or_linear_call(int kind, int out_f, int in_f, const void *w, const void *scale, const float *x, int n_rows, float *y, int act16) {
  or_linear_t L = {kind, out_f, in_f, w, (const uint16_t *)scale};
  or_linear_rows(&L, x, n_rows, y, act16, n_rows > 1);
}
/* the row-by-row evaluation of the same call (what or_linear_rows must reproduce bit for bit; used by the tests) */
void or_linear_call_rowwise(int kind, int out_f, int in_f, const void *w, const void *scale, const float *x, int n_rows, float *y, int act16) {
  or_linear_t L = {kind, out_f, in_f, w, (const uint16_t *)scale};
  for (int r = 0; r < n_rows; r++) or_linear_ex(&L, x + (size_t)r * in_f, y + (size_t)r * out_f, act16, n_rows > 1);
}

/* RMSNorm.call nn/index.ts:586-588: (x.float() * sqrt(1/(mean(x^2)+eps))).cast(dtype) * weight.
 * Two kernels (R5): the sum of squares, then the scale. mean = sum * RN32(1/d) (tensor.ts:2113-2117,
 * 3576-3579); rsqrt = reciprocal().sqrt() (tensor.ts:2944-2946) = sqrtf(1/v). */
void or_rmsnorm(const float *x, const float *w, int d, float eps, int act16, float *y) {
  float ss = 0.0f;
  for (int i = 0; i < d; i++) ss = ss + x[i] * x[i];
  float m = ss * (float)(1.0 / (double)d);
  float r = sqrtf(1.0f / (m + eps));
  for (int i = 0; i < d; i++) y[i] = rn_act(rn_act(x[i] * r, act16) * w[i], act16);
}

/* apply_rotary_emb + complex_mult, models/llama.ts:17-32: interleaved pairs
 * (x[2i], x[2i+1]) * (c_i + i s_i); one kernel per tensor, stored in the activation dtype.
 * fc = table row for this position, [hd/2][2], already cast to the activation dtype (llama.ts:205). */
static void rope_rows(float *x, int n_heads, int hd, const float *fc, int act16) {
  for (int h = 0; h < n_heads; h++)
    for (int i = 0; i < hd / 2; i++) {
      float a = x[h * hd + 2 * i], b = x[h * hd + 2 * i + 1];
      float c = fc[2 * i], d = fc[2 * i + 1];
      x[h * hd + 2 * i] = rn_act(a * c - b * d, act16);
      x[h * hd + 2 * i + 1] = rn_act(a * d + b * c, act16);
    }
}
void or_rope(float *x, int n_heads, int hd, const float *fc, int act16) { rope_rows(x, n_heads, hd, fc, act16); }

/* argmax, tensor.ts:2314-2320: lowest index among the maxima. */
int or_argmax(const float *x, int n) {
  float m = x[0];
  for (int i = 1; i < n; i++) if (x[i] > m) m = x[i];
  for (int i = 0; i < n; i++) if (x[i] == m) return i;
  return n; /* all-NaN input: the reference returns n as well (idx.max() == 0) */
}

/* ------------------------------------------------------------------ model */

typedef struct {
  or_linear_t wq, wk, wv, wo, w1, w2, w3;
  const float *attention_norm, *ffn_norm; /* values in the activation dtype */
} or_layer_t;

typedef struct {
  int dim, hidden, n_heads, n_kv_heads, n_layers, vocab, max_context, head_dim, act16;
  int batched;               /* the call carries several sequences: weights are expanded over the rows even when S == 1 */
  float norm_eps, rope_theta;
  int embed_kind;            /* OR_W_F32 / OR_W_F16 / OR_W_I8 */
  const void *tok_emb;
  const uint16_t *tok_scale; /* Int8Embedding row scales */
  or_linear_t output;
  const float *norm;
  or_layer_t *layers;
  float *freqs;              /* [2*max_context][hd/2][2], float32 table (llama.ts:198) */
  float *cache_k, *cache_v;  /* [L][max_context][KV][hd], values in the activation dtype (llama.ts:79) */
} or_model_t;

or_model_t *or_model_new(int dim, int hidden, int n_heads, int n_kv_heads, int n_layers, int vocab, int max_context, float norm_eps, float rope_theta, int act16) {
  or_model_t *m = (or_model_t *)calloc(1, sizeof(or_model_t));
  m->dim = dim; m->hidden = hidden; m->n_heads = n_heads; m->n_kv_heads = n_kv_heads; m->n_layers = n_layers;
  m->vocab = vocab; m->max_context = max_context; m->head_dim = dim / n_heads; m->act16 = act16;
  m->norm_eps = norm_eps; m->rope_theta = rope_theta;
  m->layers = (or_layer_t *)calloc((size_t)n_layers, sizeof(or_layer_t));
  m->freqs = (float *)malloc(sizeof(float) * (size_t)2 * max_context * m->head_dim);
  or_freqs_cis(m->head_dim, 2 * max_context, rope_theta, m->freqs);
  size_t csz = (size_t)n_layers * max_context * n_kv_heads * m->head_dim;
  m->cache_k = (float *)calloc(csz, sizeof(float));
  m->cache_v = (float *)calloc(csz, sizeof(float));
  return m;
}
void or_model_free(or_model_t *m) {
  free(m->layers); free(m->freqs); free(m->cache_k); free(m->cache_v); free(m);
}
void or_model_reset_cache(or_model_t *m) {
  size_t csz = (size_t)m->n_layers * m->max_context * m->n_kv_heads * m->head_dim;
  memset(m->cache_k, 0, csz * sizeof(float));
  memset(m->cache_v, 0, csz * sizeof(float));
}
/* which: 0 wq 1 wk 2 wv 3 wo 4 w1 5 w2 6 w3; layer -1 = output (lm_head) */
void or_model_set_linear(or_model_t *m, int layer, int which, int kind, int out_f, int in_f, const void *w, const void *scale) {
  or_linear_t L = {kind, out_f, in_f, w, (const uint16_t *)scale};
  if (layer < 0) { m->output = L; return; }
  or_layer_t *l = &m->layers[layer];
  or_linear_t *dst[7] = {&l->wq, &l->wk, &l->wv, &l->wo, &l->w1, &l->w2, &l->w3};
  *dst[which] = L;
}
/* which: 0 attention_norm 1 ffn_norm; layer -1 = final norm */
void or_model_set_norm(or_model_t *m, int layer, int which, const float *w) {
  if (layer < 0) { m->norm = w; return; }
  if (which == 0) m->layers[layer].attention_norm = w; else m->layers[layer].ffn_norm = w;
}
/* Several sequences per call (tokens [B, S], B > 1): every Linear sees more than one input row, so quantised weights
 * are realised in fp16 first (see or_linear_ex) even for S == 1.  The sequences themselves are independent; the caller
 * runs them one after the other through or_model_forward with this flag set. */
void or_model_set_batched(or_model_t *m, int batched) { m->batched = batched; }
void or_model_set_embedding(or_model_t *m, int kind, const void *table, const void *scale) {
  m->embed_kind = kind; m->tok_emb = table; m->tok_scale = (const uint16_t *)scale;
}
const float *or_model_freqs(const or_model_t *m) { return m->freqs; }
const float *or_model_cache_k(const or_model_t *m) { return m->cache_k; }
const float *or_model_cache_v(const or_model_t *m) { return m->cache_v; }

/* Embedding.call nn/index.ts:607-619 / Int8Embedding.call llama3.ts:71-77: the one-hot
 * compare * table summed over the vocabulary has one non-zero term, i.e. a row gather;
 * the int8 variant gathers RN16(float(code) * scale[row]). */
static void embed_row(const or_model_t *m, int tok, float *h) {
  int d = m->dim;
  if (m->embed_kind == OR_W_F32) memcpy(h, (const float *)m->tok_emb + (size_t)tok * d, sizeof(float) * (size_t)d);
  else if (m->embed_kind == OR_W_F16) for (int i = 0; i < d; i++) h[i] = h2f(((const uint16_t *)m->tok_emb)[(size_t)tok * d + i]);
  else { float s = h2f(m->tok_scale[tok]); for (int i = 0; i < d; i++) h[i] = rn16((float)((const int8_t *)m->tok_emb)[(size_t)tok * d + i] * s); }
}
void or_embed(const or_model_t *m, int tok, float *h) { embed_row(m, tok, h); }

/* Attention.call models/llama.ts:61-97 for S new positions starting at start_pos, one
 * sequence.  xn: [S][dim] normed input.  out: [S][dim] = wo(attn).
 * Kernels (R5): wq, wk, wv | rope(q) | rope(k) and v -> cache assign (:87) |
 * scores = (q.k) * RN32(1/sqrt(hd)) + mask, float32 (tensor.ts:3923) | row max | row sum of
 * exp | p = (e * (1/sum)).cast(dtype) (tensor.ts:2211-2214, :3933) | p.v (float acc) | wo.
 * GQA: query head h reads kv head h / n_rep (repeat_kv, llama.ts:34-39). */
static void attention(or_model_t *m, int layer, const float *xn, int S, int start_pos, float *out) {
  const or_layer_t *l = &m->layers[layer];
  const int H = m->n_heads, KV = m->n_kv_heads, hd = m->head_dim, n_rep = H / KV, act16 = m->act16;
  const int T = start_pos + S;
  const int mat = S > 1 || m->batched;
  const float scale = (float)(1.0 / sqrt((double)hd));
  float *attn = (float *)malloc(sizeof(float) * (size_t)S * H * hd);
  float *qs = (float *)malloc(sizeof(float) * (size_t)S * H * hd);
  float *sc_all = (float *)malloc(sizeof(float) * (size_t)T * (size_t)g_threads);   /* one score row per thread */
  float *fc = (float *)malloc(sizeof(float) * (size_t)hd);
  float *ck = m->cache_k + (size_t)layer * m->max_context * KV * hd;
  float *cv = m->cache_v + (size_t)layer * m->max_context * KV * hd;
  /* all new rows enter the cache before any query reads it (assign is realised first, :87) */
  float *ks = (float *)malloc(sizeof(float) * (size_t)S * KV * hd);
  or_linear_rows(&l->wq, xn, S, qs, act16, mat);
  or_linear_rows(&l->wk, xn, S, ks, act16, mat);
  or_linear_rows(&l->wv, xn, S, cv + (size_t)start_pos * KV * hd, act16, mat);
  for (int s = 0; s < S; s++) {
    int pos = start_pos + s;
    for (int i = 0; i < hd; i++) fc[i] = rn_act(m->freqs[(size_t)pos * hd + i], act16); /* llama.ts:205 cast */
    rope_rows(qs + (size_t)s * H * hd, H, hd, fc, act16);
    rope_rows(ks + (size_t)s * KV * hd, KV, hd, fc, act16);
    memcpy(ck + (size_t)pos * KV * hd, ks + (size_t)s * KV * hd, sizeof(float) * (size_t)KV * hd);
  }
  free(ks);
#pragma omp parallel for schedule(dynamic) num_threads(g_threads) if (g_threads > 1)
  for (int sh = 0; sh < S * H; sh++) {
    const int s = sh / H, h = sh % H;
    float *sc = sc_all + (size_t)omp_thread() * T;
    {
      int vis = start_pos + s + 1; /* causal mask triu(start_pos+1), llama.ts:208: keys t <= start_pos+s */
      const int g = h / n_rep;
      const float *qh = qs + ((size_t)s * H + h) * hd;
      for (int t = 0; t < T; t++) {
        float acc = 0.0f;
        const float *kt = ck + ((size_t)t * KV + g) * hd;
        for (int i = 0; i < hd; i++) acc = acc + qh[i] * kt[i];
        acc = acc * scale;
        if (S > 1) acc = acc + (t >= vis ? -INFINITY : 0.0f);
        sc[t] = acc;
      }
      float mx = sc[0];
      for (int t = 1; t < T; t++) if (sc[t] > mx) mx = sc[t];
      float sum = 0.0f;
      for (int t = 0; t < T; t++) sum = sum + exp_f32(sc[t] - mx);
      float rs = 1.0f / sum;
      for (int t = 0; t < T; t++) sc[t] = rn_act(exp_f32(sc[t] - mx) * rs, act16);
      float *o = attn + ((size_t)s * H + h) * hd;
      for (int i = 0; i < hd; i++) {
        float acc = 0.0f;
        for (int t = 0; t < T; t++) acc = acc + sc[t] * cv[((size_t)t * KV + g) * hd + i];
        o[i] = rn_act(acc, act16);
      }
    }
  }
  or_linear_rows(&l->wo, attn, S, out, act16, mat);
  free(attn); free(qs); free(sc_all); free(fc);
}

/* FeedForward.call models/llama.ts:108-110: w2( silu(w1 x) * (w3 x) ).
 * Kernels (R5): w1 -> buffer; w3 with the epilogue silu(a)*RN_act(dot) -> buffer; w2. */
static void feed_forward(const or_model_t *m, const or_layer_t *l, const float *xn, int S, float *out, int mat) {
  const int F = m->hidden, act16 = m->act16;
  float *a = (float *)malloc(sizeof(float) * (size_t)S * F), *u = (float *)malloc(sizeof(float) * (size_t)S * F);
  or_linear_rows(&l->w1, xn, S, a, act16, mat);
  or_linear_rows(&l->w3, xn, S, u, act16, mat);
  for (long i = 0; i < (long)S * F; i++) a[i] = rn_act(silu_act(a[i], act16) * u[i], act16);
  or_linear_rows(&l->w2, a, S, out, act16, mat);
  free(a); free(u);
}

/* Transformer.forward models/llama.ts:201-213 with temperature 0 (sample -> argmax, :137):
 * returns the greedy token of the last position and, if logits != NULL, its float logits
 * (:210 `.float()` of the activation-dtype lm_head output). */
int or_model_forward(or_model_t *m, const int *tokens, int S, int start_pos, float *logits) {
  const int d = m->dim, act16 = m->act16;
  float *h = (float *)malloc(sizeof(float) * (size_t)S * d);
  float *xn = (float *)malloc(sizeof(float) * (size_t)S * d);
  float *t = (float *)malloc(sizeof(float) * (size_t)S * d);
  for (int s = 0; s < S; s++) embed_row(m, tokens[s], h + (size_t)s * d);
  for (int L = 0; L < m->n_layers; L++) {
    const or_layer_t *l = &m->layers[L];
    /* TransformerBlock.call llama.ts:124-127: h = x + attention(attention_norm(x)); out = h + ffn(ffn_norm(h)).
     * The residual add is the epilogue of the wo / w2 kernel: RN_act(x + RN_act(dot)). */
    for (int s = 0; s < S; s++) or_rmsnorm(h + (size_t)s * d, l->attention_norm, d, m->norm_eps, act16, xn + (size_t)s * d);
    attention(m, L, xn, S, start_pos, t);
    for (long i = 0; i < (long)S * d; i++) h[i] = rn_act(h[i] + t[i], act16);
    for (int s = 0; s < S; s++) or_rmsnorm(h + (size_t)s * d, l->ffn_norm, d, m->norm_eps, act16, xn + (size_t)s * d);
    feed_forward(m, l, xn, S, t, S > 1 || m->batched);
    for (long i = 0; i < (long)S * d; i++) h[i] = rn_act(h[i] + t[i], act16);
  }
  float *lg = logits ? logits : (float *)malloc(sizeof(float) * (size_t)m->vocab);
  or_rmsnorm(h + (size_t)(S - 1) * d, m->norm, d, m->norm_eps, act16, xn);
  /* the lm_head runs on all S rows before the last one is selected (llama.ts:210), so it too sees several rows */
  or_linear_ex(&m->output, xn, lg, act16, S > 1 || m->batched);
  int tok = or_argmax(lg, m->vocab);
  if (!logits) free(lg);
  free(h); free(xn); free(t);
  return tok;
}

/* Llama3._prefill + the chat loop, models/llama3.ts:284-312: token-serial prefill, then
 * greedy decode feeding each token back.  Returns the start_pos after the last step. */
int or_model_generate(or_model_t *m, const int *prompt, int n_prompt, int start_pos, int n_new, int *out_tokens) {
  int tok = 0;
  for (int i = 0; i < n_prompt; i++) { tok = or_model_forward(m, &prompt[i], 1, start_pos, NULL); start_pos++; }
  for (int i = 0; i < n_new; i++) {
    out_tokens[i] = tok;
    if (i + 1 < n_new) { tok = or_model_forward(m, &tok, 1, start_pos, NULL); start_pos++; }
  }
  return start_pos;
}
