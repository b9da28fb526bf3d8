// Pieces shared by the matrix-core kernels that feed packed weights to v_mfma_f32_16x16x32_f16 straight from
// registers (mnb_skinny.hip for M <= 16, mnb_mid.hip for 16 < M): kernel parameters, the nibble/byte to "magic half"
// conversion, the per-chunk register block with its loads, and the constant operands of the correction MFMAs.
#pragma once
#include "mnb_bf16.hip.h"
#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

// Where the finished tiles go (wave-uniform, evaluated once per workgroup at the very end).
struct EpiParams {
  int kind;                // kMnbFusedNone: C[m * ldc + n];  kMnbFusedMlp: silu(gate) * up;  kMnbFusedQkv: three outputs
  int start1, start2;      // qkv: first packed column of the second and third output
  int n0, n1, n2;          // columns of each output (mlp: n0)
  _Float16* out1;          // qkv: second and third output (the first is C / ldc)
  _Float16* out2;
  int64_t ld1, ld2;
};

struct SkinnyParams {
  const _Float16* A;
  const uint4* W;
  const uint8_t* meta;
  const _Float16* bias;
  _Float16* C;
  int64_t lda, ldc, Npad;
  int M, N, K;
  int bs_shift;
  int chunks;       // chunks that hold elements below K
  int phase_chunks; // chunks staged in LDS at a time
  int mtr;          // rows of A staged (power of two >= M, <= 16)
  int a_vec_ok;     // A allows 16-byte loads
  int io_bf16;      // A, bias and C hold bfloat16 bits (MODE 2)
  EpiParams epi;
};

constexpr int kLdsPad = 8;  // halves of padding per staged row

// The four constants of the nibble unpack.  Written as plain literals the compiler emits v_and_b32 + v_or_b32 (VOP3
// encodings of this ISA family take no literal); held in registers it selects the single v_and_or_b32.  They are
// materialised by opaque moves (an SGPR for each mask, a VGPR for each magic: one SGPR operand per VALU instruction),
// which the optimiser cannot fold back into literals and which depend on nothing, not even the kernel arguments.
struct UnpackConsts {
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;  // 0x000F000F, 0x00F000F0, 0x64006400 (1024), 0x54005400 (64)
};

__device__ __forceinline__ UnpackConsts make_unpack_consts() {
  UnpackConsts u;
  asm("s_mov_b32 %0, 0x000F000F" : "=s"(u.mask_lo));
  asm("s_mov_b32 %0, 0x00F000F0" : "=s"(u.mask_hi));
  asm("v_mov_b32 %0, 0x64006400" : "=v"(u.magic_lo));
  asm("v_mov_b32 %0, 0x54005400" : "=v"(u.magic_hi));
  return u;
}

// raw magic halves of one 32-bit word: 4-bit -> 8 halves {1024+e0,1024+e1,64+e2,64+e3,1024+e4,1024+e5,64+e6,64+e7}
__device__ __forceinline__ h8_t raw4(uint32_t w, const UnpackConsts& u) {
  const uint32_t w8 = w >> 8;
  uint4 r;
  r.x = (w & u.mask_lo) | u.magic_lo;
  r.y = (w & u.mask_hi) | u.magic_hi;
  r.z = (w8 & u.mask_lo) | u.magic_lo;
  r.w = (w8 & u.mask_hi) | u.magic_hi;
  return __builtin_bit_cast(h8_t, r);
}
// 2-bit weights in their own width (the W2 section of the packed matrix): a 32-bit word holds 16 weights, the
// operands of two matrix instructions.  Bits 0..7 of each half carry four fields; or-ing a field at bit 2 f into the
// half whose unit in the last place is 2^(-2 f) gives 1024 + q, 256 + q, 64 + q, 16 + q (magic halves 0x6400, 0x5C00,
// 0x5400, 0x4C00) -- one v_and_or_b32 per pair of weights, as for nibbles.  The second operand of a word is the same
// on w >> 8.  Masks in SGPRs, magics in VGPRs (one SGPR operand per VALU instruction), by opaque moves.
struct UnpackConsts2 {
  uint32_t mask[4], magic[4];
};

__device__ __forceinline__ UnpackConsts2 make_unpack_consts2() {
  UnpackConsts2 u;
  asm("s_mov_b32 %0, 0x00030003" : "=s"(u.mask[0]));
  asm("s_mov_b32 %0, 0x000C000C" : "=s"(u.mask[1]));
  asm("s_mov_b32 %0, 0x00300030" : "=s"(u.mask[2]));
  asm("s_mov_b32 %0, 0x00C000C0" : "=s"(u.mask[3]));
  asm("v_mov_b32 %0, 0x64006400" : "=v"(u.magic[0]));
  asm("v_mov_b32 %0, 0x5C005C00" : "=v"(u.magic[1]));
  asm("v_mov_b32 %0, 0x54005400" : "=v"(u.magic[2]));
  asm("v_mov_b32 %0, 0x4C004C00" : "=v"(u.magic[3]));
  return u;
}

// raw magic halves of the low bytes of one word: {1024+e0,1024+e1,256+e2,256+e3,64+e4,64+e5,16+e6,16+e7}
__device__ __forceinline__ h8_t raw2(uint32_t w, const UnpackConsts2& u) {
  u4_t r;
#pragma unroll
  for (int f = 0; f < 4; ++f) r[f] = (w & u.mask[f]) | u.magic[f];
  return __builtin_bit_cast(h8_t, r);
}

// 8-bit: two words -> 8 halves 1024+b
__device__ __forceinline__ h8_t raw8(uint32_t w0, uint32_t w1) {
  uint4 r;
  r.x = __builtin_amdgcn_perm(kMagic, w0, 0x07010700u);
  r.y = __builtin_amdgcn_perm(kMagic, w0, 0x07030702u);
  r.z = __builtin_amdgcn_perm(kMagic, w1, 0x07010700u);
  r.w = __builtin_amdgcn_perm(kMagic, w1, 0x07030702u);
  return __builtin_bit_cast(h8_t, r);
}

// ---- registers of one chunk: weights, meta and (direct variant) the A operands ---------------------------------
template <int BITS, int T>
struct ChunkRegs {
  uint4 w[T];
  uint32_t m0[T];  // meta entry of the lane's (first) block: raw bits (32 with zero points, else 16)
  uint32_t m1[T];  // MODE 1, 4-bit only: entry of the second half vector (differs when block_size is 16)
  uint32_t z0[T];  // MODE 2 to 5: m0 / m1 hold the bits of the fp32 scale, z0 / z1 those of the fp32 zero point
  uint32_t z1[T];
};

// T adjacent meta entries (2 or 4 bytes each) with one load; dst holds the raw bits of each entry
template <bool HAS_ZP, int T>
__device__ __forceinline__ void load_meta_vec(const uint8_t* __restrict__ meta, int64_t first, uint32_t* dst) {
  if constexpr (HAS_ZP) {
    const uint32_t* q = reinterpret_cast<const uint32_t*>(meta) + first;
    if constexpr (T == 4) {
      const uint4 v = *reinterpret_cast<const uint4*>(q);
      dst[0] = v.x, dst[1] = v.y, dst[2] = v.z, dst[3] = v.w;
    } else if constexpr (T == 2) {
      const uint2 v = *reinterpret_cast<const uint2*>(q);
      dst[0] = v.x, dst[1] = v.y;
    } else {
      dst[0] = *q;
    }
  } else {
    const uint16_t* q = reinterpret_cast<const uint16_t*>(meta) + first;
    if constexpr (T == 4) {
      const uint2 v = *reinterpret_cast<const uint2*>(q);
      dst[0] = v.x & 0xFFFFu, dst[1] = v.x >> 16, dst[2] = v.y & 0xFFFFu, dst[3] = v.y >> 16;
    } else if constexpr (T == 2) {
      const uint32_t v = *reinterpret_cast<const uint32_t*>(q);
      dst[0] = v & 0xFFFFu, dst[1] = v >> 16;
    } else {
      dst[0] = *q;
    }
  }
}

// The same for a matrix packed with fp32 entries ({scale, zero point}: 8 bytes, or {scale}: 4 bytes).
template <bool HAS_ZP, int T>
__device__ __forceinline__ void load_meta_vec_f32(const uint8_t* __restrict__ meta, int64_t first, uint32_t* s,
                                                  uint32_t* z) {
  if constexpr (HAS_ZP) {
    const uint2* q = reinterpret_cast<const uint2*>(meta) + first;
    if constexpr (T == 4) {
      const uint4 v0 = *reinterpret_cast<const uint4*>(q), v1 = *reinterpret_cast<const uint4*>(q + 2);
      s[0] = v0.x, z[0] = v0.y, s[1] = v0.z, z[1] = v0.w, s[2] = v1.x, z[2] = v1.y, s[3] = v1.z, z[3] = v1.w;
    } else if constexpr (T == 2) {
      const uint4 v = *reinterpret_cast<const uint4*>(q);
      s[0] = v.x, z[0] = v.y, s[1] = v.z, z[1] = v.w;
    } else {
      const uint2 v = *q;
      s[0] = v.x, z[0] = v.y;
    }
  } else {
    const uint32_t* q = reinterpret_cast<const uint32_t*>(meta) + first;
    if constexpr (T == 4) {
      const uint4 v = *reinterpret_cast<const uint4*>(q);
      s[0] = v.x, s[1] = v.y, s[2] = v.z, s[3] = v.w;
    } else if constexpr (T == 2) {
      const uint2 v = *reinterpret_cast<const uint2*>(q);
      s[0] = v.x, s[1] = v.y;
    } else {
      s[0] = *q;
    }
  }
}

// col0 = first column of the workgroup + j; the T tiles of a lane are columns col0 + 16 t.
template <int BITS, bool HAS_ZP, int MODE, int T>
__device__ __forceinline__ void load_chunk(const SkinnyParams& p, int c, int kq, int64_t col0, ChunkRegs<BITS, T>& R) {
  constexpr int GK = 128 / BITS;
  constexpr int CK = 4 * GK;
  // small loads first: memory returns in issue order, and the weights are waited for tile by tile
  const int64_t mcol = mnb_meta_col(col0);  // entries of columns col0 + 16 t follow at mcol + t
  if constexpr (MODE == 0 || MODE == 6) {
    const int64_t kb = ((int64_t)c * CK) >> p.bs_shift;
    load_meta_vec<HAS_ZP, T>(p.meta, kb * p.Npad + mcol, R.m0);
    // MODE 6 (2-bit, blocks of 128): the second half of the chunk lies in the next block
    if constexpr (MODE == 6) load_meta_vec<HAS_ZP, T>(p.meta, (kb + 1) * p.Npad + mcol, R.m1);
  } else if constexpr (MODE == 4 || MODE == 5) {
    const int64_t kb = ((int64_t)c * CK) >> p.bs_shift;
    load_meta_vec_f32<HAS_ZP, T>(p.meta, kb * p.Npad + mcol, R.m0, R.z0);
  } else if constexpr (MODE >= 2) {
    const int64_t k0 = ((int64_t)c * 4 + kq) * GK;
    load_meta_vec_f32<HAS_ZP, T>(p.meta, (k0 >> p.bs_shift) * p.Npad + mcol, R.m0, R.z0);
    if constexpr (BITS == 4) load_meta_vec_f32<HAS_ZP, T>(p.meta, ((k0 + 16) >> p.bs_shift) * p.Npad + mcol, R.m1, R.z1);
  } else {
    // first k of the lane's vector; 2-bit vectors hold 32 k of each half of the chunk (mnb_w2_k)
    const int64_t k0 = BITS == 2 ? (int64_t)c * CK + kq * 32 : ((int64_t)c * 4 + kq) * GK;
    load_meta_vec<HAS_ZP, T>(p.meta, (k0 >> p.bs_shift) * p.Npad + mcol, R.m0);
    if constexpr (BITS == 4) load_meta_vec<HAS_ZP, T>(p.meta, ((k0 + 16) >> p.bs_shift) * p.Npad + mcol, R.m1);
    if constexpr (BITS == 2) load_meta_vec<HAS_ZP, T>(p.meta, ((k0 + 128) >> p.bs_shift) * p.Npad + mcol, R.m1);
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
#if defined(MNB_ABLATE_NO_LOADS)
    R.w[t] = make_uint4((uint32_t)c, (uint32_t)kq, (uint32_t)t, 0x12345678u);  // calibration builds: no weight stream
#else
    R.w[t] = p.W[((int64_t)c * 4 + kq) * p.Npad + col0 + t * 16];
#endif
  }
}

// The same loads for slabs that do not start at a multiple of 64 columns (the meta entries of a lane's tiles are then
// not adjacent): colw[t] is the lane's packed column in tile t, mcol[t] the position of its meta entry.
template <int BITS, bool HAS_ZP, int MODE, int T>
__device__ __forceinline__ void load_chunk_cols(const SkinnyParams& p, int c, int kq, const int32_t* colw,
                                                const int32_t* mcol, ChunkRegs<BITS, T>& R) {
  constexpr int GK = 128 / BITS;
  constexpr int CK = 4 * GK;
  if constexpr (MODE == 0 || MODE == 6) {
    const int64_t kb = ((int64_t)c * CK) >> p.bs_shift;
#pragma unroll
    for (int t = 0; t < T; ++t) load_meta_vec<HAS_ZP, 1>(p.meta, kb * p.Npad + mcol[t], &R.m0[t]);
    if constexpr (MODE == 6) {
#pragma unroll
      for (int t = 0; t < T; ++t) load_meta_vec<HAS_ZP, 1>(p.meta, (kb + 1) * p.Npad + mcol[t], &R.m1[t]);
    }
  } else if constexpr (MODE == 4 || MODE == 5) {
    const int64_t kb = ((int64_t)c * CK) >> p.bs_shift;
#pragma unroll
    for (int t = 0; t < T; ++t) load_meta_vec_f32<HAS_ZP, 1>(p.meta, kb * p.Npad + mcol[t], &R.m0[t], &R.z0[t]);
  } else if constexpr (MODE >= 2) {
    const int64_t k0 = ((int64_t)c * 4 + kq) * GK;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      load_meta_vec_f32<HAS_ZP, 1>(p.meta, (k0 >> p.bs_shift) * p.Npad + mcol[t], &R.m0[t], &R.z0[t]);
      if constexpr (BITS == 4)
        load_meta_vec_f32<HAS_ZP, 1>(p.meta, ((k0 + 16) >> p.bs_shift) * p.Npad + mcol[t], &R.m1[t], &R.z1[t]);
    }
  } else {
    const int64_t k0 = BITS == 2 ? (int64_t)c * CK + kq * 32 : ((int64_t)c * 4 + kq) * GK;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      load_meta_vec<HAS_ZP, 1>(p.meta, (k0 >> p.bs_shift) * p.Npad + mcol[t], &R.m0[t]);
      if constexpr (BITS == 4)
        load_meta_vec<HAS_ZP, 1>(p.meta, ((k0 + 16) >> p.bs_shift) * p.Npad + mcol[t], &R.m1[t]);
      if constexpr (BITS == 2)
        load_meta_vec<HAS_ZP, 1>(p.meta, ((k0 + 128) >> p.bs_shift) * p.Npad + mcol[t], &R.m1[t]);
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t) R.w[t] = p.W[((int64_t)c * 4 + kq) * p.Npad + colw[t]];
}

template <int BITS, bool HAS_ZP>
__device__ __forceinline__ void decode_meta(uint32_t raw, _Float16& s, _Float16& neg_1024_plus_zp) {
  if constexpr (HAS_ZP) {
    const h2_t m = mnb_as_h2(raw);
    s = m.x;
    neg_1024_plus_zp = m.y;
  } else {
    s = __builtin_bit_cast(_Float16, (uint16_t)raw);
    neg_1024_plus_zp = (_Float16)(-(1024.0f + (float)(1 << (BITS - 1))));
  }
}

// constant MFMA B operands (identical in every lane) that turn the A operands into the correction terms
struct BConst {
  h8_t off;  // -(offset of the raw half at each of the 8 positions of a word [+ default zero point])
  h8_t one;  // -1
};

template <int BITS, bool HAS_ZP>
__device__ __forceinline__ BConst make_bconst() {
  // offsets the raw halves carry: 1024 (low nibbles, bytes) and 64 (high nibbles); without zero points the
  // default zero point 2^(bits-1) is folded in.  All values are integers below 2048: exact in fp16.
  const float zp = HAS_ZP ? 0.f : (float)(1 << (BITS - 1));
  const _Float16 lo = (_Float16)(-(1024.0f + zp));
  const _Float16 hi = (_Float16)(-((BITS == 4 ? 64.0f : 1024.0f) + zp));
  const _Float16 m1 = (_Float16)(-1.0f);
  BConst bc;
  if constexpr (BITS == 2) {  // 1024, 256, 64, 16 by field (raw2)
    const _Float16 o1 = (_Float16)(-(256.0f + zp)), o2 = (_Float16)(-(64.0f + zp)), o3 = (_Float16)(-(16.0f + zp));
    bc.off = h8_t{lo, lo, o1, o1, o2, o2, o3, o3};
    bc.one = h8_t{m1, m1, m1, m1, m1, m1, m1, m1};
    return bc;
  }
  bc.off = h8_t{lo, lo, hi, hi, lo, lo, hi, hi};
  bc.one = h8_t{m1, m1, m1, m1, m1, m1, m1, m1};
  return bc;
}

// The same for bfloat16 models (MODE 4): every raw operand is the bfloat16 128 + q (see raw4_bf16).
template <bool HAS_ZP>
__device__ __forceinline__ BConst make_bconst_bf16() {
  const float zp = HAS_ZP ? 0.f : 8.f;
  const uint32_t off2 = bf16_pair(-(128.0f + zp), -(128.0f + zp)), one2 = bf16_pair(-1.0f, -1.0f);  // exact
  const u4_t off = {off2, off2, off2, off2}, one = {one2, one2, one2, one2};
  BConst bc;
  bc.off = __builtin_bit_cast(h8_t, off);
  bc.one = __builtin_bit_cast(h8_t, one);
  return bc;
}

// raw bfloat16 operands of one 4-bit word: 128 + e0 ... 128 + e7 in k order.  bfloat16 keeps 8 significant bits: 128 + q
// is exact for q < 128, and a nibble fits the mantissa only at bit 0 of a half, hence the shifts (7 operations per 8
// weights; 8-bit weights do not fit at all and take MODE 2).
__device__ __forceinline__ h8_t raw4_bf16(uint32_t w, const UnpackConsts& u, uint32_t magic) {
  u4_t r;
  r[0] = (w & u.mask_lo) | magic;
  r[1] = ((w >> 4) & u.mask_lo) | magic;
  r[2] = ((w >> 8) & u.mask_lo) | magic;
  r[3] = ((w >> 12) & u.mask_lo) | magic;
  return __builtin_bit_cast(h8_t, r);
}

// Sum the per-wavefront partial tiles (red[(w * T * 4 + t * 4 + r) * 64 + lane], written by NW wavefronts) in
// wavefront order and write the result.  Lane l, register r of tile t is row m_base + 4 * (l / 16) + r, packed column
// n0 + 16 t + l % 16.  bias is indexed by packed column.
// `first` / `step`: the threads that share this slab of T tiles number themselves first, first + step, ... (by default
// the whole workgroup: thread index, NW * 64).
template <int T, int NW>
__device__ __forceinline__ void reduce_and_store_tiles(const SkinnyParams& p, const float* red, int m_base,
                                                       int64_t n0, int first = threadIdx.x, int step = NW * 64) {
  auto total = [&](int tr, int l) {
    float sum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) sum += red[(w2 * T * 4 + tr) * 64 + l];
    return sum;
  };
  const bool bf16 = p.io_bf16 != 0;
  if (p.epi.kind == kMnbFusedMlp) {
    // adjacent tiles (2u, 2u + 1) are gate and up of output columns [n0 / 2 + 16 u, +16)
    if constexpr (T >= 2) {
      for (int i = first; i < (T / 2) * 4 * 64; i += step) {
        const int l = i & 63, ur = i >> 6;
        const int u = ur >> 2, r = ur & 3;
        const int m = m_base + 4 * (l >> 4) + r;
        const int64_t n_out = (n0 >> 1) + u * 16 + (l & 15);
        if (m >= p.M || n_out >= p.epi.n0) continue;
        const int64_t ng = n0 + u * 32 + (l & 15);
        const float g = total((2 * u) * 4 + r, l) + widen16(p.bias[ng], bf16);
        const float up = total((2 * u + 1) * 4 + r, l) + widen16(p.bias[ng + 16], bf16);
        p.C[(int64_t)m * p.ldc + n_out] = narrow16(g / (1.0f + __expf(-g)) * up, bf16);
      }
    }
    return;
  }
  for (int i = first; i < T * 4 * 64; i += step) {
    const int l = i & 63, tr = i >> 6;
    const int t = tr >> 2, r = tr & 3;
    const int m = m_base + 4 * (l >> 4) + r;
    const int64_t n = n0 + t * 16 + (l & 15);
    if (m >= p.M || n >= p.N) continue;
    float sum = total(tr, l);
    if (p.bias) sum += widen16(p.bias[n], bf16);
    if (p.epi.kind == kMnbFusedQkv) {
      if (n >= p.epi.start2) {
        if (n - p.epi.start2 < p.epi.n2) p.epi.out2[(int64_t)m * p.epi.ld2 + (n - p.epi.start2)] = narrow16(sum, bf16);
      } else if (n >= p.epi.start1) {
        if (n - p.epi.start1 < p.epi.n1) p.epi.out1[(int64_t)m * p.epi.ld1 + (n - p.epi.start1)] = narrow16(sum, bf16);
      } else if (n < p.epi.n0) {
        p.C[(int64_t)m * p.ldc + n] = narrow16(sum, bf16);
      }
    } else {
      p.C[(int64_t)m * p.ldc + n] = narrow16(sum, bf16);
    }
  }
}

}  // namespace
