// GGML blocks -> float32 values on the device: `ggml_data_to_tensor` of the reference
// (/root/reference/jsgrad/nn/state.ts:192-223) for the quantised types it supports, Q4_0 (2), Q4_1 (3), Q8_0 (8) and
// Q6_K (14).  The reference spells the bit layout with reshapes and transposes of byte tensors; element e of a block is
//   Q4_0  (18 B / 32):  d = f16 @0;            q = nibble(e);              value = (q - 8) * d
//   Q4_1  (20 B / 32):  d = f16 @0, m = f16 @2; q = nibble(e);              value = q * d + m
//   Q8_0  (34 B / 32):  d = f16 @0;            q = int8 @(2 + e);          value = d * q
//   Q6_K (210 B / 256): ql @0 (128), qh @128 (64), int8 scales @192 (16), d = f16 @208; with h = e / 128, r = e % 128:
//                       low 4 bits = ql[64h + r % 64] >> (r < 64 ? 0 : 4), high 2 bits = qh[32h + r % 32] >> (2 * (r / 32)),
//                       q = (6-bit code) - 32;  value = (d * q) * scales[e / 16]
// where nibble(e) of a 32-element block is byte e % 16 of the 16 code bytes, low half for e < 16, high half otherwise.
// All products are float32 in the order written (the build keeps a*b+c unfused); d * q and q * d are exact.
//
// This is byte work bound by the float32 it writes (4 bytes out for 0.56 to 1.06 bytes in): a thread makes four
// consecutive elements (they share the shift of their codes and their scale) and stores them as one 16-byte vector; the
// few bytes of a block that its threads share come from L1.
#include <type_traits>

#include "common.h"

namespace jsg {

template <int TYPE> struct GgmlFmt;
template <> struct GgmlFmt<2> { static constexpr int NE = 32, NB = 18; };
template <> struct GgmlFmt<3> { static constexpr int NE = 32, NB = 20; };
template <> struct GgmlFmt<8> { static constexpr int NE = 32, NB = 34; };
template <> struct GgmlFmt<14> { static constexpr int NE = 256, NB = 210; };

__device__ __forceinline__ float ggml_f16(const uint8_t *p) { return (float)*(const _Float16 *)p; }   // even offsets of 2-byte aligned blocks
// four consecutive bytes at an even offset of a block (blocks are 2-byte aligned, not 4)
__device__ __forceinline__ uint32_t ggml_ld4(const uint8_t *p) { return (uint32_t)*(const uint16_t *)p | ((uint32_t)*(const uint16_t *)(p + 2) << 16); }

// elements e .. e+3 of a block, e a multiple of 4: they share the shift of their codes and (Q6_K) their scale
template <int TYPE> __device__ __forceinline__ f4_t ggml_value4(const uint8_t *blk, int e) {
  f4_t o;
  if constexpr (TYPE == 2) {
    const uint32_t w = ggml_ld4(blk + 2 + (e & 15)) >> (e < 16 ? 0 : 4);
    const float d = ggml_f16(blk);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (float)((int)((w >> (8 * i)) & 15) - 8) * d;
  } else if constexpr (TYPE == 3) {
    const uint32_t w = ggml_ld4(blk + 4 + (e & 15)) >> (e < 16 ? 0 : 4);
    const float d = ggml_f16(blk), m = ggml_f16(blk + 2);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (float)((w >> (8 * i)) & 15) * d + m;
  } else if constexpr (TYPE == 8) {
    const uint32_t w = ggml_ld4(blk + 2 + e);
    const float d = ggml_f16(blk);
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = d * (float)(int8_t)(w >> (8 * i));
  } else {
    const int h = e >> 7, r = e & 127;
    const uint32_t lo = ggml_ld4(blk + 64 * h + (r & 63)) >> (r < 64 ? 0 : 4);
    const uint32_t hi = ggml_ld4(blk + 128 + 32 * h + (r & 31)) >> (2 * (r >> 5));
    const float d = ggml_f16(blk + 208), sc = (float)(int8_t)blk[192 + (e >> 4)];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int q = (int)(((lo >> (8 * i)) & 15) | (((hi >> (8 * i)) & 3) << 4)) - 32;
      o[i] = (d * (float)q) * sc;
    }
  }
  return o;
}

template <int TYPE> __global__ __launch_bounds__(256) void ggml_dequant_kernel(const uint8_t *blocks, size_t n, float *out) {
  constexpr int NE = GgmlFmt<TYPE>::NE, NB = GgmlFmt<TYPE>::NB;
  const size_t stride = (size_t)gridDim.x * blockDim.x, n4 = n / 4;   // n is whole blocks of 32 or 256 elements
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    const size_t b = (4 * i) / NE;
    __builtin_nontemporal_store(ggml_value4<TYPE>(blocks + b * NB, (int)(4 * i - b * NE)), (f4_t *)out + i);
  }
}

// ---- dtype casts on the way in: `v.cast(float16)` (llama3.ts:234) and fix_bf16's bfloat16 -> float32 -> float16
// (models/llama.ts:275).  A bfloat16 is the upper half of a float32, so the first step is exact.
enum { CAST_F32 = 0, CAST_F16 = 1, CAST_BF16 = 2 };
template <int SRC> __device__ __forceinline__ float cast_ld(const void *src, size_t i) {
  if constexpr (SRC == CAST_F32) return ((const float *)src)[i];
  else if constexpr (SRC == CAST_F16) return (float)((const _Float16 *)src)[i];
  else return __uint_as_float((uint32_t)((const uint16_t *)src)[i] << 16);
}
template <int DST> __device__ __forceinline__ void cast_st(void *dst, size_t i, float v) {
  if constexpr (DST == CAST_F32) ((float *)dst)[i] = v;
  else ((_Float16 *)dst)[i] = (_Float16)v;
}
// eight elements per thread and trip (the compiler merges the eight loads and stores of a thread into wide ones when the
// pointers are 16-byte aligned, which device allocations are); the last n % 8 elements one by one
template <int SRC, int DST> __global__ __launch_bounds__(256) void cast_kernel(const void *src, void *dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x, n8 = n / 8;
  typedef typename std::conditional<SRC == CAST_F32, float, uint16_t>::type S;
  typedef typename std::conditional<DST == CAST_F32, float, uint16_t>::type D;
  typedef S SV __attribute__((ext_vector_type(8)));
  typedef D DV __attribute__((ext_vector_type(8)));
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
    const SV v = ((const SV *)src)[i];
    DV o;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      float f;
      if constexpr (SRC == CAST_F32) f = v[e];
      else if constexpr (SRC == CAST_F16) f = (float)__builtin_bit_cast(_Float16, (uint16_t)v[e]);
      else f = __uint_as_float((uint32_t)v[e] << 16);
      if constexpr (DST == CAST_F32) o[e] = f;
      else o[e] = __builtin_bit_cast(uint16_t, (_Float16)f);
    }
    ((DV *)dst)[i] = o;
  }
  for (size_t i = n8 * 8 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) cast_st<DST>(dst, i, cast_ld<SRC>(src, i));
}

// ---- the q_proj / k_proj row permutation of convert_from_huggingface (models/llama.ts:225-227):
// reshape(n_heads, 2, hd/2, in).transpose(1, 2): output row h*hd + 2*i + j is input row h*hd + j*(hd/2) + i.
// 16-byte pieces of a row per thread; in_bytes is a multiple of 16.
__global__ __launch_bounds__(256) void hf_permute_kernel(const u4_t *src, u4_t *dst, int rows, int hd, int pieces) {
  const size_t total = (size_t)rows * pieces, stride = (size_t)gridDim.x * blockDim.x;
  for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
    const int r = (int)(t / pieces), c = (int)(t % pieces);
    const int h = r / hd, o = r % hd;
    const int from = h * hd + (o & 1) * (hd / 2) + (o >> 1);
    dst[t] = src[(size_t)from * pieces + c];
  }
}

}  // namespace jsg

using namespace jsg;

extern "C" {

size_t jsgrad_hip_ggml_nbytes(int ggml_type, size_t n) {
  switch (ggml_type) {
    case 2: return n / 32 * 18;
    case 3: return n / 32 * 20;
    case 8: return n / 32 * 34;
    case 14: return n / 256 * 210;
  }
  return 0;
}

int jsgrad_hip_ggml_dequant(int ggml_type, const void *blocks, size_t n, void *out_f32) {
  JSG_READY();
  JSG_REQUIRE(ggml_type == 2 || ggml_type == 3 || ggml_type == 8 || ggml_type == 14, "GGML type '%d' is not supported!", ggml_type);
  const size_t ne = ggml_type == 14 ? 256 : 32;
  JSG_REQUIRE(n % ne == 0, "jsgrad_hip_ggml_dequant: %zu elements are not whole blocks of %zu", n, ne);
  if (n == 0) return 0;
  JSG_REQUIRE(blocks && out_f32 && (uintptr_t)blocks % 2 == 0 && (uintptr_t)out_f32 % 16 == 0, "jsgrad_hip_ggml_dequant: null, odd (blocks) or unaligned (output, 16 bytes) pointer");
  const size_t want = (n / 4 + 255) / 256, cap = (size_t)state().cu_count * 32;
  const dim3 grid((unsigned)(want < cap ? want : cap)), block(256);
  const uint8_t *src = (const uint8_t *)blocks;
  float *dst = (float *)out_f32;
  switch (ggml_type) {
    case 2: hipLaunchKernelGGL(ggml_dequant_kernel<2>, grid, block, 0, state().stream, src, n, dst); break;
    case 3: hipLaunchKernelGGL(ggml_dequant_kernel<3>, grid, block, 0, state().stream, src, n, dst); break;
    case 8: hipLaunchKernelGGL(ggml_dequant_kernel<8>, grid, block, 0, state().stream, src, n, dst); break;
    default: hipLaunchKernelGGL(ggml_dequant_kernel<14>, grid, block, 0, state().stream, src, n, dst); break;
  }
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n) {
  JSG_READY();
  JSG_REQUIRE(src_dtype >= 0 && src_dtype <= 2 && (dst_dtype == 0 || dst_dtype == 1), "jsgrad_hip_cast: dtype %d -> %d", src_dtype, dst_dtype);
  if (n == 0) return 0;
  JSG_REQUIRE(src && dst && (uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0, "jsgrad_hip_cast: null or unaligned pointer (16 bytes)");
  const size_t want = (n + 255) / 256, cap = (size_t)state().cu_count * 32;
  const dim3 grid((unsigned)(want < cap ? want : cap)), block(256);
#define JSG_CAST(S, D) \
  if (src_dtype == S && dst_dtype == D) hipLaunchKernelGGL((cast_kernel<S, D>), grid, block, 0, state().stream, src, dst, n);
  JSG_CAST(0, 0) JSG_CAST(0, 1) JSG_CAST(1, 0) JSG_CAST(1, 1) JSG_CAST(2, 0) JSG_CAST(2, 1)
#undef JSG_CAST
  JSG_LAUNCHED();
  return 0;
}

int jsgrad_hip_hf_permute(const void *src, void *dst, int rows, int row_bytes, int n_heads) {
  JSG_READY();
  JSG_REQUIRE(src && dst && src != dst, "jsgrad_hip_hf_permute: null pointer or in place");
  JSG_REQUIRE(rows > 0 && n_heads > 0 && rows % n_heads == 0 && (rows / n_heads) % 2 == 0, "jsgrad_hip_hf_permute: %d rows do not make %d heads of even size", rows, n_heads);
  JSG_REQUIRE(row_bytes > 0 && row_bytes % 16 == 0, "jsgrad_hip_hf_permute: rows of %d bytes (a multiple of 16 is built)", row_bytes);
  const int pieces = row_bytes / 16;
  const size_t want = ((size_t)rows * pieces + 255) / 256, cap = (size_t)state().cu_count * 32;
  hipLaunchKernelGGL(hf_permute_kernel, dim3((unsigned)(want < cap ? want : cap)), dim3(256), 0, state().stream, (const u4_t *)src, (u4_t *)dst, rows, rows / n_heads, pieces);
  JSG_LAUNCHED();
  return 0;
}

}  // extern "C"
