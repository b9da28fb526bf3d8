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
// A workgroup owns 64 neighbouring columns and the 8/bits consecutive blocks that share one zero-point byte.  Each
// block is first copied to LDS with 16-byte loads (rows of the source are contiguous across the 64 columns), so the
// source is read from HBM exactly once; the range scan and the quantisation then work from LDS, four threads per
// column (one quarter of the block each).  (Reading a thread's elements straight from global memory into registers -
// no LDS tile, one barrier per block - was measured at less than half the speed: 2-byte loads per lane put too few
// bytes in flight.)
#include <hip/hip_runtime.h>

#include "mnb_internal.h"

namespace {

constexpr int kCols = 64;      // columns per workgroup
constexpr int kQuarters = 4;   // threads per column (each takes one quarter of the block)

template <typename T, int BITS>
__global__ void __launch_bounds__(kCols * kQuarters) mnb_quantize_kernel(uint8_t* __restrict__ B, T* __restrict__ scales,
                                                                         uint8_t* __restrict__ zp,
                                                                         const T* __restrict__ src, int64_t K, int64_t N,
                                                                         int64_t ld, int bs, int vec_ok) {
  constexpr int PER_BYTE = 8 / BITS;  // blocks per zero-point byte, elements per weight byte
  constexpr int MAXQ = (1 << BITS) - 1;
  constexpr int MID = 1 << (BITS - 1);
  constexpr int VEC = 16 / (int)sizeof(T);  // elements per 16-byte load
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);                                    // [bs][kCols]
  float* red = reinterpret_cast<float*>(smem + (size_t)bs * kCols * sizeof(T));  // [2][kQuarters][kCols]

  const int tid = threadIdx.x;
  const int c = tid % kCols, qr = tid / kCols;
  const int64_t n0 = (int64_t)blockIdx.x * kCols;
  const int64_t n = n0 + c;
  const int64_t kbc = (K + bs - 1) / bs;
  const int64_t blob = (int64_t)bs * BITS / 8;
  const int64_t zrow = (kbc * BITS + 7) / 8;
  const int64_t kb0 = (int64_t)blockIdx.y * PER_BYTE;
  const bool full_cols = n0 + kCols <= N;
  uint32_t zbyte = 0;

  for (int sub = 0; sub < PER_BYTE; ++sub) {
    const int64_t kb = kb0 + sub;
    if (kb >= kbc) {
      // the unused part of the last zero-point byte keeps the reference's filler, the default zero point
      zbyte |= (uint32_t)MID << (sub * BITS);
      continue;
    }
    const int64_t k0 = kb * bs;
    const int rows = (int)(k0 + bs < K ? bs : K - k0);
    __syncthreads();  // the previous block's tile is no longer read
    if (vec_ok && full_cols) {
      constexpr int CH = kCols / VEC;  // 16-byte chunks per row
      for (int i = tid; i < rows * CH; i += kCols * kQuarters) {
        const int r = i / CH, ch = i % CH;
        *reinterpret_cast<uint4*>(tile + r * kCols + ch * VEC) =
            *reinterpret_cast<const uint4*>(src + (k0 + r) * ld + n0 + ch * VEC);
      }
    } else {
      for (int i = tid; i < rows * kCols; i += kCols * kQuarters) {
        const int r = i / kCols, cc = i % kCols;
        tile[r * kCols + cc] = n0 + cc < N ? src[(k0 + r) * ld + n0 + cc] : (T)0.0f;
      }
    }
    __syncthreads();
    // range of this thread's quarter, then of the whole block
    const int qrows = bs / kQuarters;
    const int r0 = qr * qrows;
    const int r1 = r0 + qrows < rows ? r0 + qrows : rows;
    float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
    for (int r = r0; r < r1; ++r) {
      const float v = (float)tile[r * kCols + c];
      mn = v < mn ? v : mn;
      mx = v > mx ? v : mx;
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
    const T stored = (T)scale;
    const float sf = (float)stored;
    const float rscale = sf != 0.f ? 1.0f / sf : 0.f;
    const float zf32 = (float)z;
    if (n < N) {
      if (qr == 0) scales[n * kbc + kb] = stored;
      auto quant = [&](int r) -> uint32_t {
        if (r >= rows) return (uint32_t)z;
        const float v = (float)tile[r * kCols + c];
        float t = v * rscale;  // separate statements: the product is rounded before the addition
        t = t + zf32;
        // roundf (halves away from zero) followed by the clamp to [0, MAXQ]: round to nearest even, then push the
        // upward ties up.  Negative ties need no care, everything below 0.5 ends at 0 either way.
        const float rn = __builtin_rintf(t);
        const float up = (t - rn == 0.5f) ? 1.0f : 0.0f;  // the difference is exact
        t = __builtin_amdgcn_fmed3f(rn + up, 0.f, (float)MAXQ);
        return (uint32_t)(int)t;
      };
      uint8_t* out = B + (n * kbc + kb) * blob + (int64_t)r0 / PER_BYTE;
      const int qbytes = qrows / PER_BYTE;  // 1 (2-bit, block 16), 2 (4-bit block 16, 2-bit block 32) or a multiple of 4
      auto quant_word = [&](int w) -> uint32_t {
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < 4 * PER_BYTE; ++e) word |= quant(r0 + w * 4 * PER_BYTE + e) << (e * BITS);
        return word;
      };
      if (qbytes >= 16 && (blob % 16) == 0) {
        // 16-byte stores (the quarter starts at a multiple of 16 bytes of a 16-byte aligned blob)
        for (int w = 0; w < qbytes / 16; ++w) {
          const uint4 v = make_uint4(quant_word(4 * w), quant_word(4 * w + 1), quant_word(4 * w + 2), quant_word(4 * w + 3));
          *reinterpret_cast<uint4*>(out + 16 * w) = v;
        }
      } else if (qbytes >= 4) {
        for (int w = 0; w < qbytes / 4; ++w) *reinterpret_cast<uint32_t*>(out + 4 * w) = quant_word(w);
      } else {
        uint32_t word = 0;
        for (int e = 0; e < qrows; ++e) word |= quant(r0 + e) << (e * BITS);
        if (qbytes == 1)
          *out = (uint8_t)word;  // 2-bit, block 16: four elements per thread
        else
          *reinterpret_cast<uint16_t*>(out) = (uint16_t)word;
      }
    }
  }
  if (zp && n < N && qr == 0) zp[n * zrow + blockIdx.y] = (uint8_t)zbyte;
}

template <typename T>
hipError_t launch_t(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld, int bits,
                    int bs, hipStream_t s) {
  const int64_t kbc = (K + bs - 1) / bs;
  const int per_byte = 8 / bits;
  dim3 grid((unsigned)((N + kCols - 1) / kCols), (unsigned)((kbc + per_byte - 1) / per_byte)), blk(kCols * kQuarters);
  const size_t smem = (size_t)bs * kCols * sizeof(T) + 2 * kQuarters * kCols * sizeof(float);
  const int vec_ok = (reinterpret_cast<uintptr_t>(src) % 16 == 0) && (ld % (16 / sizeof(T)) == 0);
  auto launch = [&](auto kernel) -> hipError_t {
    // fp32 sources with 256-deep blocks need 66 KiB of LDS: above the default limit, within the CU's 160 KiB
    if (smem > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) return e;
    }
    kernel<<<grid, blk, smem, s>>>((uint8_t*)B, (T*)scales, (uint8_t*)zp, (const T*)src, K, N, ld, bs, vec_ok);
    return hipGetLastError();
  };
  if (bits == 2) return launch(mnb_quantize_kernel<T, 2>);
  return bits == 4 ? launch(mnb_quantize_kernel<T, 4>) : launch(mnb_quantize_kernel<T, 8>);
}

}  // namespace

hipError_t mnb_launch_quantize(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld,
                               int bits, int bs, int dtype, hipStream_t s) {
  if (K == 0 || N == 0) return hipSuccess;
  return dtype == kMnbDtypeFloat16 ? launch_t<_Float16>(B, scales, zp, src, K, N, ld, bits, bs, s)
                                   : launch_t<float>(B, scales, zp, src, K, N, ld, bits, bs, s);
}
