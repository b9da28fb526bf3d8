// Blockwise quantiser: the producer of the MatMulNBits weight format, on the device.
//
// Restates BlockwiseQuantizer::quantizeAndTranspose for column-wise blocks
// (onnxruntime/core/mlas/lib/q4_dq.cpp:468-574) with range2scalezp / range2scale (:347-386):
//   asymmetric  min = min(min, 0), max = max(max, 0); scale = (max - min) / (2^bits - 1);
//               zp = clamp(roundf(-min / scale)) (min itself when the scale is 0);
//   symmetric   s = the extreme with the larger magnitude; scale = -s / 2^(bits-1); zp = 2^(bits-1);
//   q = clamp(roundf(v * (1 / stored scale) + zp), 0, 2^bits - 1), all in fp32, no fused multiply-add.
// fp16 models widen every element to fp32 and store the scale rounded to fp16; the reciprocal is taken from the
// stored scale, the zero point from the unrounded one.  Output is the canonical operand layout of the operator.
// Positions k >= K of the last block (left unwritten by the reference) receive the zero point: they dequantise to 0.
//
// A workgroup owns 128 neighbouring columns and the 8/bits consecutive blocks that share one zero-point byte.  Each
// block is first copied to LDS with 16-byte loads (rows of the source are contiguous across the 128 columns: 256-byte
// pieces of fp16 rows; 128-byte pieces - 64 columns - were measured 8 % slower, 512-byte pieces 20 % slower), so the
// source is read from HBM exactly once.  Four threads per column take one quarter of the block each: a thread reads
// its quarter from LDS, keeps it widened to fp32 in registers across the range scan, and quantises from there
// (the block size is a template parameter for that reason; quarters of 16 and more elements are read a second time
// instead).  Whole blocks - all but a ragged last one - run without per-element conditions.  (Reading a thread's
// elements straight from global memory into registers - no LDS tile, one barrier per block - was measured at less
// than half the speed: 2-byte loads per lane put too few bytes in flight.)  Blocks of 64 and fewer elements run on a
// second kernel that lays several blocks of a column side by side in one workgroup (mnb_quantize_small_kernel).
#include <hip/hip_runtime.h>

#include "mnb_internal.h"

namespace {

constexpr int kCols = 128;     // columns per workgroup
constexpr int kQuarters = 4;   // threads per column (each takes one quarter of the block)

// QROWS = block size / 4: the elements of a thread's quarter.  A compile-time constant so that the quarter, widened
// to fp32, stays in registers between the range scan and the quantisation (each element leaves LDS once).
template <typename T, int BITS, int QROWS>
__global__ void __launch_bounds__(kCols * kQuarters) mnb_quantize_kernel(uint8_t* __restrict__ B, T* __restrict__ scales,
                                                                         uint8_t* __restrict__ zp,
                                                                         const T* __restrict__ src, int64_t K, int64_t N,
                                                                         int64_t ld, int vec_ok, int nsub) {
  constexpr int PER_BYTE = 8 / BITS;  // blocks per zero-point byte, elements per weight byte
  constexpr int MAXQ = (1 << BITS) - 1;
  constexpr int MID = 1 << (BITS - 1);
  constexpr int VEC = 16 / (int)sizeof(T);  // elements per 16-byte load
  constexpr int bs = QROWS * kQuarters;
  constexpr int blob = bs * BITS / 8;
  constexpr int QBITS = QROWS * BITS;       // bits a thread produces per block: 8 (2-bit, block 16), 16, or words
  constexpr int QWORDS = (QBITS + 31) / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);                                    // [bs][kCols]
  float* red = reinterpret_cast<float*>(smem + (size_t)bs * kCols * sizeof(T));  // [2][kQuarters][kCols]

  const int tid = threadIdx.x;
  const int c = tid % kCols, qr = tid / kCols;
  const int64_t n0 = (int64_t)blockIdx.x * kCols;
  const int64_t n = n0 + c;
  const int64_t kbc = (K + bs - 1) / bs;
  const int64_t zrow = (kbc * BITS + 7) / 8;
  const int64_t kb0 = (int64_t)blockIdx.y * nsub;
  const int nb = (int)(kbc - kb0 < nsub ? kbc - kb0 : nsub);  // blocks of this workgroup, consecutive along K
  const bool full_cols = n0 + kCols <= N;
  const bool fast = vec_ok && full_cols;
  const int q0 = qr * QROWS;
  uint32_t zbyte = 0;

  // The next block travels from global memory into registers while the current one is worked on from LDS.
  constexpr int CH = kCols / VEC;                                // 16-byte chunks per row
  constexpr int PRE = (bs * CH + kCols * kQuarters - 1) / (kCols * kQuarters);  // chunks per thread and block
  // chunk u of a thread: row (tid + 256 u) / CH of the block (rows beyond the block's last re-read that row and are
  // never used, so that no load sits under a condition), 16-byte piece (tid + 256 u) % CH of the strip
  auto chunk_ptr = [&](int64_t kb, int u) -> const uint4* {
    const int64_t k0 = kb * bs;
    const int rows = (int)(k0 + bs < K ? bs : K - k0);
    const int i = tid + u * kCols * kQuarters;
    const int r = i / CH < rows ? i / CH : rows - 1;
    return reinterpret_cast<const uint4*>(src + (k0 + r) * ld + n0 + (i % CH) * VEC);
  };
  uint4 pre[PRE];
#pragma unroll
  for (int u = 0; u < PRE; ++u) pre[u] = fast ? *chunk_ptr(kb0, u) : make_uint4(0u, 0u, 0u, 0u);

  for (int sb = 0; sb < nb; ++sb) {
    const int sub = sb % PER_BYTE;
    const int64_t kb = kb0 + sb;
    const int64_t k0 = kb * bs;
    const int rows = (int)(k0 + bs < K ? bs : K - k0);
    __syncthreads();  // the previous block's tile is no longer read
    if (fast) {
#pragma unroll
      for (int u = 0; u < PRE; ++u) {
        const int i = tid + u * kCols * kQuarters;
        if (bs * CH % (kCols * kQuarters) == 0 || i < bs * CH)
          *reinterpret_cast<uint4*>(tile + (i / CH) * kCols + (i % CH) * VEC) = pre[u];
      }
      if (sb + 1 < nb) {
#pragma unroll
        for (int u = 0; u < PRE; ++u) pre[u] = *chunk_ptr(kb + 1, u);
      }
    } else {
      for (int i = tid; i < rows * kCols; i += kCols * kQuarters) {
        const int r = i / kCols, cc = i % kCols;
        tile[r * kCols + cc] = n0 + cc < N ? src[(k0 + r) * ld + n0 + cc] : (T)0.0f;
      }
    }
    __syncthreads();
    // range of this thread's quarter, then of the whole block
    const int mine = rows - q0 < QROWS ? rows - q0 : QROWS;  // rows of the quarter that exist (may be <= 0)
    const bool whole = rows == bs;  // every block but a ragged last one: no per-element conditions (uniform)
    // blocks of 64 and more elements read the tile a second time when they quantise instead of holding their
    // quarter in registers (which, with the registers of the load in flight, keeps wavefronts off the SIMD)
    constexpr bool kHold = QROWS < 16;
    float held[kHold ? QROWS : 1];
    float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
    if (whole) {
#pragma unroll
      for (int e = 0; e < QROWS; ++e) {
        const float v = (float)tile[(q0 + e) * kCols + c];
        mn = __builtin_fminf(v, mn);  // one instruction each; like the comparisons below they skip a NaN
        mx = __builtin_fmaxf(v, mx);
        if constexpr (kHold) held[e] = v;
      }
      // The reference's scan (if (v < min) min = v) keeps the first zero it meets, whatever its sign, where the
      // minimum instruction prefers -0.  Only an all-zero block shows it (the sign of its stored scale, taken from
      // the block's first element): restore the first element there.
      if (mn == 0.f && mx == 0.f) mn = mx = (float)tile[q0 * kCols + c];
    } else {
#pragma unroll
      for (int e = 0; e < QROWS; ++e) {
        float v = 0.f;
        if (e < mine) {
          v = (float)tile[(q0 + e) * kCols + c];
          mn = v < mn ? v : mn;
          mx = v > mx ? v : mx;
        }
        if constexpr (kHold) held[e] = v;
      }
    }
    red[qr * kCols + c] = mn;
    red[(kQuarters + qr) * kCols + c] = mx;
    __syncthreads();
#pragma unroll
    for (int q2 = 0; q2 < kQuarters; ++q2) {
      const float a = red[q2 * kCols + c], b = red[(kQuarters + q2) * kCols + c];
      mn = a < mn ? a : mn;
      mx = b > mx ? b : mx;
    }
    float scale;
    int z;
    if (zp) {
      mn = mn < 0.f ? mn : 0.f;
      mx = mx > 0.f ? mx : 0.f;
      scale = (mx - mn) / (float)MAXQ;
      float zf = mn;
      if (scale != 0.f) zf = 0.f - mn / scale;
      zf = zf < 0.f ? 0.f : zf;
      zf = zf > (float)MAXQ ? (float)MAXQ : zf;
      z = (int)roundf(zf);
    } else {
      const float smax = fabsf(mx) > fabsf(mn) ? mx : mn;
      scale = -smax / (float)MID;
      z = MID;
    }
    zbyte |= (uint32_t)z << (sub * BITS);
    if (zp && (sub == PER_BYTE - 1 || kb == kbc - 1)) {
      // the unused part of the last zero-point byte keeps the reference's filler, the default zero point
      for (int f = sub + 1; f < PER_BYTE; ++f) zbyte |= (uint32_t)MID << (f * BITS);
      if (n < N && qr == 0) zp[n * zrow + kb / PER_BYTE] = (uint8_t)zbyte;
      zbyte = 0;
    }
    const T stored = (T)scale;
    const float sf = (float)stored;
    const float rscale = sf != 0.f ? 1.0f / sf : 0.f;
    const float zf32 = (float)z;
    if (n < N) {
      if (qr == 0) scales[n * kbc + kb] = stored;
      uint32_t word[QWORDS];
#pragma unroll
      for (int w = 0; w < QWORDS; ++w) word[w] = 0;
      // clamp(roundf(t), 0, MAXQ), roundf rounding halves away from zero: for t >= 0 that is trunc(t + 0.49999997f)
      // (the largest float below one half: a sum that lands exactly between two floats rounds to the even one,
      // which is the integer, only when t itself is a tie), everything below 0.5 ends at 0 either way, and the clamp
      // commutes with the truncation because its bounds are integers.
      auto quantise = [&](float v) -> uint32_t {
        float t = v * rscale;  // separate statements: the product is rounded before the addition
        t = t + zf32;
        t = t + 0.49999997f;
        t = __builtin_amdgcn_fmed3f(t, 0.f, (float)MAXQ);
        return (uint32_t)t;
      };
      if (whole) {
#pragma unroll
        for (int e = 0; e < QROWS; ++e) {
          const float v = kHold ? held[e] : (float)tile[(q0 + e) * kCols + c];
          word[(e * BITS) / 32] |= quantise(v) << ((e * BITS) % 32);
        }
      } else {
#pragma unroll
        for (int e = 0; e < QROWS; ++e) {
          const uint32_t q = e < mine ? quantise(kHold ? held[e] : (float)tile[(q0 + e) * kCols + c]) : (uint32_t)z;
          word[(e * BITS) / 32] |= q << ((e * BITS) % 32);
        }
      }
      uint8_t* out = B + (n * kbc + kb) * blob + qr * (QBITS / 8);
      if constexpr (QBITS == 8) {
        *out = (uint8_t)word[0];
      } else if constexpr (QBITS == 16) {
        *reinterpret_cast<uint16_t*>(out) = (uint16_t)word[0];
      } else if constexpr (QWORDS % 4 == 0) {
        // 16-byte stores (the quarter starts at a multiple of 16 bytes of a 16-byte aligned blob)
#pragma unroll
        for (int w = 0; w < QWORDS; w += 4)
          *reinterpret_cast<uint4*>(out + 4 * w) = make_uint4(word[w], word[w + 1], word[w + 2], word[w + 3]);
      } else {
#pragma unroll
        for (int w = 0; w < QWORDS; ++w) *reinterpret_cast<uint32_t*>(out + 4 * w) = word[w];
      }
    }
  }
}

// Blocks of 16, 32 and 64 elements: with one block per workgroup the tile is a few KiB, a thread has four to sixteen
// elements between three barriers, and a column's output arrives in pieces of 2 to 8 bytes (measured 52 us for
// blocks of 32 where blocks of 128 take 29 us on the same matrix).  Here a workgroup owns 128 columns x BPW blocks
// side by side along K (128 rows; 64 rows for blocks of 16): a thread takes a whole block of its column (half of a
// block of 64), so blocks of up to 32 need no exchange of ranges at all, the source is still read in 256-byte pieces
// of 64 or 128 rows, a column's BPW blobs are contiguous in B, and the zero points of the blocks that share a byte
// meet in LDS.  One pass per workgroup; the arithmetic is that of the kernel above, statement for statement.
// SLOTS = threads per column
template <typename T, int BITS, int BS, int TPB, int SLOTS>
__global__ void __launch_bounds__(kCols * SLOTS) mnb_quantize_small_kernel(uint8_t* __restrict__ B, T* __restrict__ scales,
                                                                            uint8_t* __restrict__ zp,
                                                                            const T* __restrict__ src, int64_t K,
                                                                            int64_t N, int64_t ld, int vec_ok) {
  constexpr int PER_BYTE = 8 / BITS;
  constexpr int MAXQ = (1 << BITS) - 1;
  constexpr int MID = 1 << (BITS - 1);
  constexpr int VEC = 16 / (int)sizeof(T);
  constexpr int EPT = BS / TPB;        // elements per thread
  constexpr int BPW = SLOTS / TPB;    // blocks per workgroup
  constexpr int ROWS = BPW * BS;
  constexpr int blob = BS * BITS / 8;
  constexpr int QWORDS = EPT * BITS / 32;
  static_assert(EPT * BITS % 32 == 0 && BPW % PER_BYTE == 0,
                "a thread writes whole words; a zero-point byte stays in one workgroup");
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);                                              // [ROWS][kCols]
  float* red = reinterpret_cast<float*>(smem + (size_t)ROWS * kCols * sizeof(T));    // [2][SLOTS][kCols]
  uint32_t* zs = reinterpret_cast<uint32_t*>(red + 2 * SLOTS * kCols);              // [BPW][kCols]

  const int tid = threadIdx.x;
  const int c = tid % kCols, slot = tid / kCols;
  const int bi = slot / TPB, part = slot % TPB;
  const int64_t n0 = (int64_t)blockIdx.x * kCols;
  const int64_t n = n0 + c;
  const int64_t kbc = (K + BS - 1) / BS;
  const int64_t zrow = (kbc * BITS + 7) / 8;
  const int64_t kb0 = (int64_t)blockIdx.y * BPW;
  const int64_t k0 = kb0 * BS;
  const int rows = (int)(k0 + ROWS < K ? ROWS : K - k0);  // rows of the tile that exist (>= 1)
  const bool whole = rows == ROWS;

  if (vec_ok && n0 + kCols <= N) {
    constexpr int CH = kCols / VEC;                       // 16-byte chunks per row
    constexpr int PRE = ROWS * CH / (kCols * SLOTS);     // chunks per thread
    static_assert(ROWS * CH % (kCols * SLOTS) == 0, "whole chunks per thread");
    uint4 pre[PRE];
#pragma unroll
    for (int u = 0; u < PRE; ++u) {
      const int i = tid + u * kCols * SLOTS;
      const int r = i / CH < rows ? i / CH : rows - 1;    // rows beyond K re-read the last one and are never used
      pre[u] = *reinterpret_cast<const uint4*>(src + (k0 + r) * ld + n0 + (i % CH) * VEC);
    }
#pragma unroll
    for (int u = 0; u < PRE; ++u) {
      const int i = tid + u * kCols * SLOTS;
      *reinterpret_cast<uint4*>(tile + (i / CH) * kCols + (i % CH) * VEC) = pre[u];
    }
  } else {
    for (int i = tid; i < rows * kCols; i += kCols * SLOTS) {
      const int r = i / kCols, cc = i % kCols;
      tile[r * kCols + cc] = n0 + cc < N ? src[(k0 + r) * ld + n0 + cc] : (T)0.0f;
    }
  }
  __syncthreads();

  const int64_t kb = kb0 + bi;
  const bool exists = kb < kbc;
  const int e0 = bi * BS + part * EPT;                               // first row of this thread's elements
  const int mine = rows - e0 < EPT ? rows - e0 : EPT;                // how many of them exist (may be <= 0)
  float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
  if (whole) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const float v = (float)tile[(e0 + e) * kCols + c];
      mn = __builtin_fminf(v, mn);
      mx = __builtin_fmaxf(v, mx);
    }
    if (mn == 0.f && mx == 0.f) mn = mx = (float)tile[e0 * kCols + c];  // see the kernel above: the first zero's sign
  } else {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      if (e < mine) {
        const float v = (float)tile[(e0 + e) * kCols + c];
        mn = v < mn ? v : mn;
        mx = v > mx ? v : mx;
      }
    }
  }
  if constexpr (TPB > 1) {
    red[slot * kCols + c] = mn;
    red[(SLOTS + slot) * kCols + c] = mx;
    __syncthreads();
#pragma unroll
    for (int q2 = 0; q2 < TPB; ++q2) {
      const float a = red[(bi * TPB + q2) * kCols + c], b = red[(SLOTS + bi * TPB + q2) * kCols + c];
      mn = a < mn ? a : mn;
      mx = b > mx ? b : mx;
    }
  }
  float scale;
  int z;
  if (zp) {
    mn = mn < 0.f ? mn : 0.f;
    mx = mx > 0.f ? mx : 0.f;
    scale = (mx - mn) / (float)MAXQ;
    float zf = mn;
    if (scale != 0.f) zf = 0.f - mn / scale;
    zf = zf < 0.f ? 0.f : zf;
    zf = zf > (float)MAXQ ? (float)MAXQ : zf;
    z = (int)roundf(zf);
  } else {
    const float smax = fabsf(mx) > fabsf(mn) ? mx : mn;
    scale = -smax / (float)MID;
    z = MID;
  }
  if (zp) {
    // blocks beyond the last one leave the reference's filler, the default zero point, in their part of the byte
    if (part == 0) zs[bi * kCols + c] = exists ? (uint32_t)z : (uint32_t)MID;
    __syncthreads();
    if (part == 0 && bi % PER_BYTE == 0 && exists && n < N) {
      uint32_t zbyte = 0;
#pragma unroll
      for (int f = 0; f < PER_BYTE; ++f) zbyte |= zs[(bi + f) * kCols + c] << (f * BITS);
      zp[n * zrow + kb / PER_BYTE] = (uint8_t)zbyte;
    }
  }
  if (!exists || n >= N) return;
  const T stored = (T)scale;
  const float sf = (float)stored;
  const float rscale = sf != 0.f ? 1.0f / sf : 0.f;
  const float zf32 = (float)z;
  if (part == 0) scales[n * kbc + kb] = stored;
  auto quantise = [&](float v) -> uint32_t {  // clamp(roundf(v * rscale + zp), 0, MAXQ): see the kernel above
    float t = v * rscale;
    t = t + zf32;
    t = t + 0.49999997f;
    t = __builtin_amdgcn_fmed3f(t, 0.f, (float)MAXQ);
    return (uint32_t)t;
  };
  uint32_t word[QWORDS];
#pragma unroll
  for (int w = 0; w < QWORDS; ++w) word[w] = 0;
  if (whole) {
#pragma unroll
    for (int e = 0; e < EPT; ++e)
      word[(e * BITS) / 32] |= quantise((float)tile[(e0 + e) * kCols + c]) << ((e * BITS) % 32);
  } else {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const uint32_t q = e < mine ? quantise((float)tile[(e0 + e) * kCols + c]) : (uint32_t)z;
      word[(e * BITS) / 32] |= q << ((e * BITS) % 32);
    }
  }
  uint8_t* out = B + (n * kbc + kb) * blob + part * (EPT * BITS / 8);
  if constexpr (QWORDS % 4 == 0) {
#pragma unroll
    for (int w = 0; w < QWORDS; w += 4)
      *reinterpret_cast<uint4*>(out + 4 * w) = make_uint4(word[w], word[w + 1], word[w + 2], word[w + 3]);
  } else if constexpr (QWORDS % 2 == 0) {
#pragma unroll
    for (int w = 0; w < QWORDS; w += 2) *reinterpret_cast<uint2*>(out + 4 * w) = make_uint2(word[w], word[w + 1]);
  } else {
#pragma unroll
    for (int w = 0; w < QWORDS; ++w) *reinterpret_cast<uint32_t*>(out + 4 * w) = word[w];
  }
}

template <typename T, int BITS, int BS>
hipError_t launch_small(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld,
                        hipStream_t s) {
  constexpr int TPB = (BS == 64 && BITS != 2) ? 2 : 1;  // 2-bit blocks of 64: four blocks share a zero-point byte
  constexpr int SLOTS = 4;  // (eight for blocks of 16 - 128 rows again - was measured: no difference)
  constexpr int BPW = SLOTS / TPB, ROWS = BPW * BS;
  const auto kernel = mnb_quantize_small_kernel<T, BITS, BS, TPB, SLOTS>;
  const size_t smem = (size_t)ROWS * kCols * sizeof(T) + 2 * SLOTS * kCols * sizeof(float) + (size_t)BPW * kCols * 4;
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  const int64_t kbc = (K + BS - 1) / BS;
  dim3 grid((unsigned)((N + kCols - 1) / kCols), (unsigned)((kbc + BPW - 1) / BPW)), blk(kCols * SLOTS);
  const int vec_ok = (reinterpret_cast<uintptr_t>(src) % 16 == 0) && (ld % (16 / sizeof(T)) == 0);
  kernel<<<grid, blk, smem, s>>>((uint8_t*)B, (T*)scales, (uint8_t*)zp, (const T*)src, K, N, ld, vec_ok);
  return hipGetLastError();
}

template <typename T, int BITS, int QROWS>
hipError_t launch_k(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld, hipStream_t s) {
  constexpr int bs = QROWS * kQuarters;
  const auto kernel = mnb_quantize_kernel<T, BITS, QROWS>;
  const size_t smem = (size_t)bs * kCols * sizeof(T) + 2 * kQuarters * kCols * sizeof(float);
  // fp32 sources with 256-deep blocks need 66 KiB of LDS: above the default limit, within the CU's 160 KiB
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) return e;
  }
  const int64_t kbc = (K + bs - 1) / bs;
  // Blocks per workgroup: the 8/bits blocks of one zero-point byte when zero points are written, else one.  Many
  // small workgroups beat few long ones here: [4096, 14336] fp16 to 4 bits, blocks of 128, took 36 us with one
  // block per workgroup, 41 us with two and 44-46 us with four to eight (64-column workgroups).
  const int nsub = zp ? 8 / BITS : 1;
  const int64_t strips = (N + kCols - 1) / kCols;
  dim3 grid((unsigned)strips, (unsigned)((kbc + nsub - 1) / nsub)), blk(kCols * kQuarters);
  const int vec_ok = (reinterpret_cast<uintptr_t>(src) % 16 == 0) && (ld % (16 / sizeof(T)) == 0);
  kernel<<<grid, blk, smem, s>>>((uint8_t*)B, (T*)scales, (uint8_t*)zp, (const T*)src, K, N, ld, vec_ok, nsub);
  return hipGetLastError();
}

template <typename T, int BITS>
hipError_t launch_b(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld, int bs,
                    hipStream_t s) {
  switch (bs) {
    case 16: return launch_small<T, BITS, 16>(B, scales, zp, src, K, N, ld, s);
    case 32: return launch_small<T, BITS, 32>(B, scales, zp, src, K, N, ld, s);
    case 64:
      // measured on [4096, 14336]: the side-by-side kernel is 3-25 % faster, except for fp16 sources to 8 bits
      // (5-7 % slower)
      if constexpr (BITS == 8 && sizeof(T) == 2) return launch_k<T, BITS, 16>(B, scales, zp, src, K, N, ld, s);
      else return launch_small<T, BITS, 64>(B, scales, zp, src, K, N, ld, s);
    case 128: return launch_k<T, BITS, 32>(B, scales, zp, src, K, N, ld, s);
    case 256: return launch_k<T, BITS, 64>(B, scales, zp, src, K, N, ld, s);
    default: return hipErrorInvalidValue;
  }
}

template <typename T>
hipError_t launch_t(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld, int bits,
                    int bs, hipStream_t s) {
  if (bits == 2) return launch_b<T, 2>(B, scales, zp, src, K, N, ld, bs, s);
  return bits == 4 ? launch_b<T, 4>(B, scales, zp, src, K, N, ld, bs, s) : launch_b<T, 8>(B, scales, zp, src, K, N, ld, bs, s);
}

}  // namespace

hipError_t mnb_launch_quantize(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld,
                               int bits, int bs, int dtype, hipStream_t s) {
  if (K == 0 || N == 0) return hipSuccess;
  return dtype == kMnbDtypeFloat16 ? launch_t<_Float16>(B, scales, zp, src, K, N, ld, bits, bs, s)
                                   : launch_t<float>(B, scales, zp, src, K, N, ld, bits, bs, s);
}
