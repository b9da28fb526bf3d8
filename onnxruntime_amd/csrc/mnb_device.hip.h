// Device-side helpers shared by every kernel: vector types, meta access and the nibble/byte unpack.
//
// The unpack produces EXACT small integers (q - zp) in the arithmetic type of the model; the scale is applied
// afterwards with a single multiply, which is what makes the dequantised weights bit-identical to the reference
// definition  W = float(q - zp) * scale  (onnxruntime/core/mlas/lib/q4_dq.cpp:624-637):
//   fp16 model: (q | 0x6400) is the half 1024+q; subtracting 1024+zp is exact; the product with the scale
//               rounds once (RNE), the same bits as rounding the exact fp32 product to half.
//   fp32 model: float(q) - float(zp) is exact; one fp32 multiply.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mnb_layout.h"

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ h2_t mnb_as_h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
__device__ __forceinline__ uint32_t mnb_as_u32(h2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ h2_t mnb_h2(_Float16 a) { return h2_t{a, a}; }

constexpr uint32_t kMagic = 0x64006400u;  // two halves of value 1024

// ---- zero-point constants of one block, fp16 model ---------------------------------------------------
struct ZpH {
  h2_t lo;  // -(1024 + zp): for magic halves 1024 + q
  h2_t hi;  // -(64 + zp):   for magic halves (1024 + 16 q) / 16
};

__device__ __forceinline__ ZpH mnb_zp_h(_Float16 neg_1024_plus_zp) {
  ZpH z;
  z.lo = mnb_h2(neg_1024_plus_zp);
  z.hi = mnb_h2(neg_1024_plus_zp + (_Float16)960.0f);  // exact: both are integers below 2048
  return z;
}

// 4-bit, fp16: 8 nibbles of one word -> (q - zp) as 4 half pairs in k order (e0,e1)(e2,e3)(e4,e5)(e6,e7).
__device__ __forceinline__ void mnb_unpack4_h(uint32_t w, const ZpH& z, h2_t out[4]) {
  const h2_t sixteenth = mnb_h2((_Float16)0.0625f);
  uint32_t w8 = w >> 8;
  h2_t p0 = mnb_as_h2((w & 0x000F000Fu) | kMagic);
  h2_t p1 = mnb_as_h2((w & 0x00F000F0u) | kMagic);
  h2_t p2 = mnb_as_h2((w8 & 0x000F000Fu) | kMagic);
  h2_t p3 = mnb_as_h2((w8 & 0x00F000F0u) | kMagic);
  out[0] = p0 + z.lo;
  out[1] = __builtin_elementwise_fma(p1, sixteenth, z.hi);
  out[2] = p2 + z.lo;
  out[3] = __builtin_elementwise_fma(p3, sixteenth, z.hi);
}

// 8-bit, fp16: 4 bytes of one word -> (q - zp) as 2 half pairs in k order.
__device__ __forceinline__ void mnb_unpack8_h(uint32_t w, const ZpH& z, h2_t out[2]) {
  // v_perm_b32 byte selectors: 0-3 pick bytes of the second operand, 4-7 bytes of the first.
  h2_t p0 = mnb_as_h2(__builtin_amdgcn_perm(kMagic, w, 0x07010700u));  // [b0, 0x64, b1, 0x64]
  h2_t p1 = mnb_as_h2(__builtin_amdgcn_perm(kMagic, w, 0x07030702u));  // [b2, 0x64, b3, 0x64]
  out[0] = p0 + z.lo;
  out[1] = p1 + z.lo;
}

// fp32 model: element order inside a 4-bit word follows the interleave e0 e2 e4 e6 e1 e3 e5 e7.
__device__ __forceinline__ void mnb_unpack4_f(uint32_t w, float zp, float out[8]) {
  out[0] = (float)(w & 0xFu) - zp;
  out[2] = (float)((w >> 4) & 0xFu) - zp;
  out[4] = (float)((w >> 8) & 0xFu) - zp;
  out[6] = (float)((w >> 12) & 0xFu) - zp;
  out[1] = (float)((w >> 16) & 0xFu) - zp;
  out[3] = (float)((w >> 20) & 0xFu) - zp;
  out[5] = (float)((w >> 24) & 0xFu) - zp;
  out[7] = (float)(w >> 28) - zp;
}

__device__ __forceinline__ void mnb_unpack8_f(uint32_t w, float zp, float out[4]) {
  out[0] = (float)(w & 0xFFu) - zp;
  out[1] = (float)((w >> 8) & 0xFFu) - zp;
  out[2] = (float)((w >> 16) & 0xFFu) - zp;
  out[3] = (float)(w >> 24) - zp;
}

// ---- meta access ---------------------------------------------------------------------------------------
// fp16 model
template <bool HAS_ZP, int BITS>
__device__ __forceinline__ void mnb_load_meta_h(const uint8_t* meta, int64_t idx, _Float16& scale, ZpH& z) {
  if constexpr (HAS_ZP) {
    h2_t m = mnb_as_h2(reinterpret_cast<const uint32_t*>(meta)[idx]);
    scale = m.x;
    z = mnb_zp_h(m.y);
  } else {
    scale = reinterpret_cast<const _Float16*>(meta)[idx];
    z = mnb_zp_h((_Float16)(-(1024.0f + (float)(1 << (BITS - 1)))));
  }
}

// fp32 model
template <bool HAS_ZP, int BITS>
__device__ __forceinline__ void mnb_load_meta_f(const uint8_t* meta, int64_t idx, float& scale, float& zp) {
  if constexpr (HAS_ZP) {
    float2 m = reinterpret_cast<const float2*>(meta)[idx];
    scale = m.x;
    zp = m.y;
  } else {
    scale = reinterpret_cast<const float*>(meta)[idx];
    zp = (float)(1 << (BITS - 1));
  }
}

// Dequantise one 16-byte group of column n to the model type, k order, scale applied (one rounding).
// 4-bit: 32 values; 8-bit: 16 values.  block_of_k(kk) = block index of element kk of the group.
template <int BITS, bool HAS_ZP>
__device__ __forceinline__ void mnb_dequant_group_h(const uint4& v, const uint8_t* meta, int64_t g, int64_t n,
                                                    int64_t Npad, int bs, _Float16* out) {
  constexpr int GK = 128 / BITS;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  const int64_t k0 = g * GK;
  // a group spans one block, or two when 4-bit and bs == 16
  const int nblk = (bs < GK) ? GK / bs : 1;
  for (int b = 0; b < nblk; ++b) {
    _Float16 s;
    ZpH z;
    mnb_load_meta_h<HAS_ZP, BITS>(meta, ((k0 + b * bs) / bs) * Npad + mnb_meta_col(n), s, z);
    const h2_t s2 = mnb_h2(s);
    const int words = 4 / nblk;
    for (int i = 0; i < words; ++i) {
      const int wi = b * words + i;
      if constexpr (BITS == 4) {
        h2_t d[4];
        mnb_unpack4_h(w[wi], z, d);
        for (int j = 0; j < 4; ++j) {
          h2_t r = d[j] * s2;
          out[wi * 8 + 2 * j] = r.x;
          out[wi * 8 + 2 * j + 1] = r.y;
        }
      } else {
        h2_t d[2];
        mnb_unpack8_h(w[wi], z, d);
        for (int j = 0; j < 2; ++j) {
          h2_t r = d[j] * s2;
          out[wi * 4 + 2 * j] = r.x;
          out[wi * 4 + 2 * j + 1] = r.y;
        }
      }
    }
  }
}

template <int BITS, bool HAS_ZP>
__device__ __forceinline__ void mnb_dequant_group_f(const uint4& v, const uint8_t* meta, int64_t g, int64_t n,
                                                    int64_t Npad, int bs, float* out) {
  constexpr int GK = 128 / BITS;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  const int64_t k0 = g * GK;
  const int nblk = (bs < GK) ? GK / bs : 1;
  for (int b = 0; b < nblk; ++b) {
    float s, zp;
    mnb_load_meta_f<HAS_ZP, BITS>(meta, ((k0 + b * bs) / bs) * Npad + mnb_meta_col(n), s, zp);
    const int words = 4 / nblk;
    for (int i = 0; i < words; ++i) {
      const int wi = b * words + i;
      if constexpr (BITS == 4) {
        float d[8];
        mnb_unpack4_f(w[wi], zp, d);
        for (int j = 0; j < 8; ++j) out[wi * 8 + j] = d[j] * s;
      } else {
        float d[4];
        mnb_unpack8_f(w[wi], zp, d);
        for (int j = 0; j < 4; ++j) out[wi * 4 + j] = d[j] * s;
      }
    }
  }
}
