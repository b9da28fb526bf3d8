// 16-bit models on a matrix packed with fp32 meta entries - bfloat16 models, and fp16 models whose zero points are in
// the activation type - on the matrix cores (tile GEMM: mnb_gemm256.hip, few rows: mnb_skinny.hip).
#pragma once
#include "mnb_buffer.hip.h"
#include "mnb_device.hip.h"

namespace {

// ---- bfloat16 models.  The packed matrix is the fp32 models' (meta entries {float scale[, float zero point]}, which
// also holds zero points that are not integers); activations, bias and output are bfloat16.  A weight is
// float(q) * scale - zp * scale in fp32 (one fused multiply-add), narrowed to bfloat16 (round to nearest even) as the
// matrix core's operand; the products accumulate in fp32.
typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t bf16_pair(float lo, float hi) {
  const bf2_t p = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ float bf16_widen(uint16_t bits) { return __builtin_bit_cast(float, (uint32_t)bits << 16); }

__device__ __forceinline__ uint32_t f16_pair(float lo, float hi) {
  const h2_t p = {(_Float16)lo, (_Float16)hi};  // one v_cvt_pk_f16_f32, round to nearest even
  return __builtin_bit_cast(uint32_t, p);
}

// Packed weights of one lane and slab -> 8 weights in k order, fma(float(q), s, c) with c = -zp * s, narrowed to
// bfloat16 (BF16) or fp16.
template <int BITS, bool BF16>
__device__ __forceinline__ h8_t dequant_word_wide(uint32_t w0, uint32_t w1, float s, float c) {
  auto pair = [](float lo, float hi) { return BF16 ? bf16_pair(lo, hi) : f16_pair(lo, hi); };
  uint32_t b0, b1;  // bytes: 4-bit e0 e4 e1 e5 | e2 e6 e3 e7 (the packed nibble order); 8-bit e0 e1 e2 e3 | e4 e5 e6 e7
  if constexpr (BITS == 4) {
    b0 = w0 & 0x0F0F0F0Fu;
    b1 = (w0 >> 4) & 0x0F0F0F0Fu;
  } else {
    b0 = w0;
    b1 = w1;
  }
  // opaque: otherwise the byte selects below are folded back into a shift and a mask per element
  asm volatile("" : "+v"(b0), "+v"(b1));
  auto f = [&](uint32_t b, int byte) { return __builtin_fmaf((float)((b >> (8 * byte)) & 0xffu), s, c); };
  u4_t o;
  if constexpr (BITS == 4) {
    o = u4_t{pair(f(b0, 0), f(b0, 2)), pair(f(b1, 0), f(b1, 2)), pair(f(b0, 1), f(b0, 3)), pair(f(b1, 1), f(b1, 3))};
  } else {
    o = u4_t{pair(f(b0, 0), f(b0, 1)), pair(f(b0, 2), f(b0, 3)), pair(f(b1, 0), f(b1, 1)), pair(f(b1, 2), f(b1, 3))};
  }
  return __builtin_bit_cast(h8_t, o);
}

// v_mfma_f32_16x16x32_bf16 / v_mfma_f32_32x32x16_bf16 on operands held as 8 halves' worth of bits
__device__ __forceinline__ f4_t mfma16_bf16(h8_t a, h8_t b, f4_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, a), __builtin_bit_cast(bf8_t, b), c, 0, 0, 0);
#else
  (void)a, (void)b;
  return c;
#endif
}

// the model's 16-bit type travels as _Float16 bits in the kernels' parameter blocks
__device__ __forceinline__ float widen16(_Float16 v, bool bf16) {
  return bf16 ? bf16_widen(__builtin_bit_cast(uint16_t, v)) : (float)v;
}
__device__ __forceinline__ _Float16 narrow16(float v, bool bf16) {
  return bf16 ? __builtin_bit_cast(_Float16, (__bf16)v) : (_Float16)v;
}

}  // namespace
