/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for com.microsoft::MatMulNBits.
 *
 * A plain-C restatement of the reference's arithmetic contract for the op at
 * accuracy_level 0 (and, in a section of its own, of the int8-activation
 * contract of accuracy_level 4).  It is the checker used by tests/,
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py.  Nothing in the shipped library or the
 * Python host package may link, import or call it.
 *
 * What each function follows in the reference (onnxruntime 1.30.0):
 *   layout + dequantisation   onnxruntime/core/mlas/lib/q4_dq.cpp:587-641
 *                             (BlockwiseQuantizer::dequantize, column-wise blocks)
 *   default zero point        onnxruntime/core/mlas/lib/q4_dq.cpp:323,634 (kMid = 2^(bits-1))
 *   zero-point row length     onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_helper.h:33-35
 *   fp32 op semantics         onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:940-1065
 *   fp16 op semantics         onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:1069-1180
 *                             (A, scales, bias widened to fp32; fp32 accumulate; one RNE narrowing of Y)
 *   bias                      onnxruntime/core/mlas/lib/qnbitgemm.cpp:500-524 (added once per output)
 *   fp16 <-> fp32             onnxruntime/core/mlas/inc/mlas_float16.h:46-86 (round to nearest even,
 *                             NaN -> 0x7e00, overflow -> Inf); restated here from IEEE-754, not copied
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   mnbo_f16_to_f32 / mnbo_f32_to_f16   pinned: exhaustive over all 65536 halves and against numpy's
 *                                       independent float16 conversion on edge + random floats
 *   mnbo_dequantize_{f32,f16}           pinned: the reference's own 23 op-test vectors (through the matmul),
 *                                       exhaustive (q, zp) tables against integer arithmetic, unit-vector
 *                                       recovery, and an independent numpy implementation
 *   mnbo_matmul_{f32,f16,f64}           pinned: the 23 vectors (exact), integer special cases against
 *                                       numpy int64 matmul, linearity, fp64 agreement
 *   mnbo_quantize_*                     see the header comment of that section
 *   mnbo_variant_dequantize_f32         typed zero points / g_idx (the reference's "very rare" route,
 *                                       onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_impl.cc:19-75 and
 *                                       onnxruntime/core/mlas/lib/q4_dq.cpp:2187-2241).  Pinned by mathematics only
 *                                       (the reference's tests recompute their expectations and its dequantiser for
 *                                       this route does not build without the whole runtime): exact cases where no
 *                                       operation rounds, equality with mnbo_dequantize_f32 on the inputs where both
 *                                       routes are defined and exact, group selection read back through power-of-two
 *                                       scales, closeness to the fp64 value, and the last place of the three-rounding
 *                                       formula against exact rational arithmetic rounded to fp32 after each
 *                                       operation (tests/test_oracle_variants.py), on inputs where a contracted
 *                                       multiply-add and the one-rounding form both differ from it.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ fp16 */

float mnbo_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t mnbo_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);   /* NaN -> quiet NaN */
  if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);  /* >= 65536 (or Inf) -> Inf */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  if (ax < 0x33000000u) return sign;         /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
  int shift;                                 /* bits to drop from the 24-bit significand */
  uint32_t base;
  if (e < -14) { /* result is subnormal: value = m * 2^(e-23); unit = 2^-24 */
    shift = -e - 1; /* 13 + (-14 - e) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  uint32_t r = base + q; /* a carry out of the mantissa correctly bumps the exponent */
  if (r >= 0x7c00u) r = 0x7c00u;
  return (uint16_t)(sign | r);
}

void mnbo_f16_to_f32_buffer(const uint16_t* src, float* dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = mnbo_f16_to_f32(src[i]);
}

void mnbo_f32_to_f16_buffer(const float* src, uint16_t* dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = mnbo_f32_to_f16(src[i]);
}

/* ------------------------------------------------------------------ layout */

static inline int64_t k_blocks_of(int64_t K, int64_t bs) { return (K + bs - 1) / bs; }
static inline int64_t blob_of(int64_t bs, int64_t bits) { return bs * bits / 8; }
static inline int64_t zp_row_of(int64_t kb, int64_t bits) { return (kb * bits + 7) / 8; }

/* quantised element (n, k): 4-bit packs two per byte, low nibble = even k; 8-bit one per byte */
static inline int q_at(const uint8_t* B, int64_t n, int64_t k, int64_t kb_count, int64_t bs, int bits) {
  int64_t kb = k / bs, r = k % bs;
  const uint8_t* blob = B + (n * kb_count + kb) * blob_of(bs, bits);
  if (bits == 8) return blob[r];
  if (bits == 4) return (blob[r >> 1] >> ((r & 1) * 4)) & 0xf;
  return (blob[r >> 2] >> ((r & 3) * 2)) & 0x3; /* bits == 2 */
}

/* zero point of block (n, kb): packed like the weights, row length ceil(kb_count*bits/8); absent -> 2^(bits-1) */
static inline int zp_at(const uint8_t* zp, int64_t n, int64_t kb, int64_t kb_count, int bits) {
  if (!zp) return 1 << (bits - 1);
  const uint8_t* row = zp + n * zp_row_of(kb_count, bits);
  if (bits == 8) return row[kb];
  if (bits == 4) return (row[kb >> 1] >> ((kb & 1) * 4)) & 0xf;
  return (row[kb >> 2] >> ((kb & 3) * 2)) & 0x3;
}

/* ------------------------------------------------------------------ dequantise */

/* dst is column-major [N][K] (stride K): dst[n*K + k] = (q - zp) * scale, one fp32 rounding. */
void mnbo_dequantize_f32(float* dst, const uint8_t* B, const float* scales, const uint8_t* zp, int64_t N, int64_t K,
                         int bits, int64_t bs) {
  int64_t kbc = k_blocks_of(K, bs);
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      int64_t kb = k / bs;
      int d = q_at(B, n, k, kbc, bs, bits) - zp_at(zp, n, kb, kbc, bits);
      volatile float v = (float)d * scales[n * kbc + kb];
      dst[n * K + k] = v;
    }
}

/* fp16 model: the fp32 product of an integer |d| <= 255 and a widened half is exact; one RNE narrowing. */
void mnbo_dequantize_f16(uint16_t* dst, const uint8_t* B, const uint16_t* scales, const uint8_t* zp, int64_t N,
                         int64_t K, int bits, int64_t bs) {
  int64_t kbc = k_blocks_of(K, bs);
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      int64_t kb = k / bs;
      int d = q_at(B, n, k, kbc, bs, bits) - zp_at(zp, n, kb, kbc, bits);
      volatile float v = (float)d * mnbo_f16_to_f32(scales[n * kbc + kb]);
      dst[n * K + k] = mnbo_f32_to_f16(v);
    }
}

/* Typed zero points and/or a group index: dst[n*K + k] = float(q) * scale + (-scale * zp), every operation rounded to
 * fp32 by itself (matmul_nbits_impl.cc:66-73 for T = float; 2 bits: q4_dq.cpp:2227-2238 hands scale and -scale*zp to
 * a kernel that computes q*scale + that).  Scales and typed zero points arrive widened to fp32 (the fp16 operator
 * widens them first, matmul_nbits.cc:1352-1366).  block index = g_idx[k] when a group index is given, else k / bs.
 * zp_kind: 0 none (2^(bits-1)), 1 packed uint8, 2 float [N][k_blocks].
 * honour_u8_zp_with_g_idx = 0 restates the reference's CPU code literally: with a group index, packed uint8 zero
 * points are read and then ignored in favour of 8 (matmul_nbits_impl.cc:56-66); 1 applies them, as the operator's
 * schema defines and as the reference does without a group index. */
void mnbo_variant_dequantize_f32(float* dst, const uint8_t* B, const float* scales, int zp_kind, const void* zp,
                                 const int32_t* g_idx, int64_t N, int64_t K, int bits, int64_t bs,
                                 int honour_u8_zp_with_g_idx) {
  int64_t kbc = k_blocks_of(K, bs);
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      int64_t b = g_idx ? g_idx[k] : k / bs;
      float s = scales[n * kbc + b];
      float z = (float)(1 << (bits - 1));
      if (zp_kind == 2)
        z = ((const float*)zp)[n * kbc + b];
      else if (zp_kind == 1 && (!g_idx || honour_u8_zp_with_g_idx))
        z = (float)zp_at((const uint8_t*)zp, n, b, kbc, bits);
      volatile float adjust = -s * z;
      volatile float prod = (float)q_at(B, n, k, kbc, bs, bits) * s;
      volatile float v = prod + adjust;
      dst[n * K + k] = v;
    }
}

/* ------------------------------------------------------------------ matmul */

typedef struct {
  const float* A;
  const uint8_t* B;
  const float* scales;
  const uint8_t* zp;
  const float* bias;
  float* Y;
  double* Y64;
  double* bound;
  int64_t M, N, K, bs, lda, ldc;
  int bits;
  int64_t n0, n1;
} mm_job;

/* One output column slice [n0, n1): dequantise the column once, reuse it for every row of A. */
static void* mm_worker(void* p) {
  mm_job* j = (mm_job*)p;
  int64_t kbc = k_blocks_of(j->K, j->bs);
  float* w = (float*)malloc((size_t)(kbc * j->bs) * sizeof(float));
  for (int64_t n = j->n0; n < j->n1; ++n) {
    for (int64_t kb = 0; kb < kbc; ++kb) {
      int z = zp_at(j->zp, n, kb, kbc, j->bits);
      float s = j->scales[n * kbc + kb];
      const uint8_t* blob = j->B + (n * kbc + kb) * blob_of(j->bs, j->bits);
      float* wb = w + kb * j->bs;
      if (j->bits == 4) {
        for (int64_t r = 0; r < j->bs / 2; ++r) {
          wb[2 * r] = (float)((blob[r] & 0xf) - z) * s;
          wb[2 * r + 1] = (float)((blob[r] >> 4) - z) * s;
        }
      } else if (j->bits == 8) {
        for (int64_t r = 0; r < j->bs; ++r) wb[r] = (float)(blob[r] - z) * s;
      } else {
        for (int64_t r = 0; r < j->bs; ++r) wb[r] = (float)(((blob[r >> 2] >> ((r & 3) * 2)) & 3) - z) * s;
      }
    }
    for (int64_t m = 0; m < j->M; ++m) {
      const float* a = j->A + m * j->lda;
      if (j->Y) {
        float acc = 0.f;
        for (int64_t k = 0; k < j->K; ++k) acc += a[k] * w[k];
        if (j->bias) acc += j->bias[n];
        j->Y[m * j->ldc + n] = acc;
      }
      if (j->Y64) {
        double acc = 0.0, bnd = 0.0;
        for (int64_t k = 0; k < j->K; ++k) {
          double t = (double)a[k] * (double)w[k];
          acc += t;
          bnd += fabs(t);
        }
        if (j->bias) {
          acc += (double)j->bias[n];
          bnd += fabs((double)j->bias[n]);
        }
        j->Y64[m * j->ldc + n] = acc;
        if (j->bound) j->bound[m * j->ldc + n] = bnd;
      }
    }
  }
  free(w);
  return NULL;
}

static void mm_run(mm_job base, int nthreads) {
  if (nthreads < 1) nthreads = 1;
  if (nthreads > 256) nthreads = 256;
  if ((int64_t)nthreads > base.N) nthreads = (int)(base.N > 0 ? base.N : 1);
  pthread_t th[256];
  mm_job jobs[256];
  int64_t per = (base.N + nthreads - 1) / nthreads;
  int started = 0;
  for (int t = 0; t < nthreads; ++t) {
    jobs[t] = base;
    jobs[t].n0 = t * per;
    jobs[t].n1 = (t + 1) * per < base.N ? (t + 1) * per : base.N;
    if (jobs[t].n0 >= jobs[t].n1) break;
    if (nthreads == 1) {
      mm_worker(&jobs[t]);
    } else {
      pthread_create(&th[t], NULL, mm_worker, &jobs[t]);
      ++started;
    }
  }
  for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
}

/* Y[m][n] = sum_k A[m][k] * W[k][n] (+ bias[n]); fp32 accumulation in k order; elements k >= K ignored. */
void mnbo_matmul_f32(const float* A, const uint8_t* B, const float* scales, const uint8_t* zp, const float* bias,
                     float* Y, int64_t M, int64_t N, int64_t K, int bits, int64_t bs, int nthreads) {
  mm_job j = {A, B, scales, zp, bias, Y, NULL, NULL, M, N, K, bs, K, N, bits, 0, N};
  mm_run(j, nthreads);
}

/* fp64 accumulation of the same fp32 products, plus the row bound sum_k |a*w| (+|bias|) used by the error gate. */
void mnbo_matmul_f64(const float* A, const uint8_t* B, const float* scales, const uint8_t* zp, const float* bias,
                     double* Y64, double* bound, int64_t M, int64_t N, int64_t K, int bits, int64_t bs,
                     int nthreads) {
  mm_job j = {A, B, scales, zp, bias, NULL, Y64, bound, M, N, K, bs, K, N, bits, 0, N};
  mm_run(j, nthreads);
}

/* fp16 model on the reference's x64 path: widen A/scales/bias, compute in fp32, narrow Y once (RNE). */
void mnbo_matmul_f16(const uint16_t* A, const uint8_t* B, const uint16_t* scales, const uint8_t* zp,
                     const uint16_t* bias, uint16_t* Y, int64_t M, int64_t N, int64_t K, int bits, int64_t bs,
                     int nthreads) {
  int64_t kbc = k_blocks_of(K, bs);
  float* a32 = (float*)malloc((size_t)(M * K) * sizeof(float));
  float* s32 = (float*)malloc((size_t)(N * kbc) * sizeof(float));
  float* b32 = bias ? (float*)malloc((size_t)N * sizeof(float)) : NULL;
  float* y32 = (float*)malloc((size_t)(M * N) * sizeof(float));
  mnbo_f16_to_f32_buffer(A, a32, (size_t)(M * K));
  mnbo_f16_to_f32_buffer(scales, s32, (size_t)(N * kbc));
  if (bias) mnbo_f16_to_f32_buffer(bias, b32, (size_t)N);
  mnbo_matmul_f32(a32, B, s32, zp, b32, y32, M, N, K, bits, bs, nthreads);
  mnbo_f32_to_f16_buffer(y32, Y, (size_t)(M * N));
  free(a32);
  free(s32);
  free(b32);
  free(y32);
}

/* ------------------------------------------------------------------ int8 activations (accuracy_level 4)
 *
 * The reference's own scalar statement of the SQNBIT_CompInt8 contract, which its kernels are tested against
 * (onnxruntime/test/mlas/unittest/test_sqnbitgemm.cpp:94-170, QuantizeA and CallReferenceGemm_CompInt8; the
 * dispatcher is SQ4BitGemm_CompInt8, onnxruntime/core/mlas/lib/qnbitgemm.cpp:883-1086):
 *   A, per row and block of bs elements along k (the weights' block size):
 *       scale = max|a| / 127;  q = clamp(roundf(a * (scale != 0 ? 1 / scale : 0)), -128, 127)
 *       (elements k >= K of the last block count as 0)
 *   Y[m][n] = bias[n] (or 0);  for every block in k order:
 *       qsum = sum_k qa * (qb - zp)           exact, int32
 *       Y   += float(qsum) * a_scale * b_scale   evaluated left to right, every operation rounded to fp32
 * 4-bit weights only (test_sqnbitgemm.cpp:160).  fp16 models widen A, scales and bias first and narrow Y once.
 * Parity (tests/test_oracle_int8.py): the quantiser against hand-written integers on grids where the scale is a
 * power of two (ties included: half away from zero); the product against numpy's exact int64 matmul where every
 * scale is 1; against an independent numpy restatement that rounds to fp32 after every operation; against the
 * accuracy_level-0 result within the analytic bound of the activation rounding, sum over blocks of
 * (a_scale / 2) * sum |w|.
 */
void mnbo_quantize_a_int8(int8_t* qa, float* a_scale, const float* A, int64_t M, int64_t K, int64_t bs) {
  int64_t kbc = k_blocks_of(K, bs);
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t kb = 0; kb < kbc; ++kb) {
      int64_t len = K - kb * bs < bs ? K - kb * bs : bs;
      const float* a = A + m * K + kb * bs;
      float amax = 0.0f;
      for (int64_t r = 0; r < len; ++r) {
        float v = fabsf(a[r]);
        if (v > amax) amax = v;
      }
      const float scale = amax / 127.0f;
      const float recip = scale != 0.0f ? 1.0f / scale : 0.0f;
      a_scale[m * kbc + kb] = scale;
      for (int64_t r = 0; r < bs; ++r) {
        float q = r < len ? roundf(a[r] * recip) : 0.0f;
        if (q < -128.0f) q = -128.0f;
        if (q > 127.0f) q = 127.0f;
        qa[(m * kbc + kb) * bs + r] = (int8_t)q;
      }
    }
  }
}

typedef struct {
  const int8_t* qa;
  const float* a_scale;
  const uint8_t* B;
  const float* scales;
  const uint8_t* zp;
  const float* bias;
  float* Y;
  int64_t M, N, K, bs, n0, n1;
} i8_job;

static void* i8_worker(void* p) {
  i8_job* j = (i8_job*)p;
  int64_t kbc = k_blocks_of(j->K, j->bs);
  for (int64_t m = 0; m < j->M; ++m) {
    for (int64_t n = j->n0; n < j->n1; ++n) {
      float sum = j->bias ? j->bias[n] : 0.0f;
      for (int64_t kb = 0; kb < kbc; ++kb) {
        int64_t len = j->K - kb * j->bs < j->bs ? j->K - kb * j->bs : j->bs;
        const int z = zp_at(j->zp, n, kb, kbc, 4);
        const int8_t* a = j->qa + (m * kbc + kb) * j->bs;
        int32_t qsum = 0;
        for (int64_t r = 0; r < len; ++r) qsum += (int32_t)a[r] * (q_at(j->B, n, kb * j->bs + r, kbc, j->bs, 4) - z);
        float t = (float)qsum * j->a_scale[m * kbc + kb];
        t = t * j->scales[n * kbc + kb];
        sum = sum + t;
      }
      j->Y[m * j->N + n] = sum;
    }
  }
  return NULL;
}

/* A fp32 [M][K]; 4-bit canonical B / scales / zero points; Y fp32 [M][N]. */
void mnbo_matmul_int8_f32(const float* A, const uint8_t* B, const float* scales, const uint8_t* zp, const float* bias,
                          float* Y, int64_t M, int64_t N, int64_t K, int64_t bs, int nthreads) {
  int64_t kbc = k_blocks_of(K, bs);
  int8_t* qa = (int8_t*)malloc((size_t)(M * kbc * bs));
  float* as = (float*)malloc((size_t)(M * kbc) * sizeof(float));
  mnbo_quantize_a_int8(qa, as, A, M, K, bs);
  if (nthreads < 1) nthreads = 1;
  if (nthreads > 256) nthreads = 256;
  if ((int64_t)nthreads > N) nthreads = (int)(N > 0 ? N : 1);
  pthread_t th[256];
  i8_job jobs[256];
  int64_t per = (N + nthreads - 1) / nthreads;
  int started = 0;
  for (int t = 0; t < nthreads; ++t) {
    i8_job jb = {qa, as, B, scales, zp, bias, Y, M, N, K, bs, t * per, (t + 1) * per < N ? (t + 1) * per : N};
    jobs[t] = jb;
    if (jobs[t].n0 >= jobs[t].n1) break;
    if (nthreads == 1) {
      i8_worker(&jobs[t]);
    } else {
      pthread_create(&th[t], NULL, i8_worker, &jobs[t]);
      ++started;
    }
  }
  for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
  free(qa);
  free(as);
}

/* fp16 model: widen A, scales and bias, compute as above, narrow Y once (RNE). */
void mnbo_matmul_int8_f16(const uint16_t* A, const uint8_t* B, const uint16_t* scales, const uint8_t* zp,
                          const uint16_t* bias, uint16_t* Y, int64_t M, int64_t N, int64_t K, int64_t bs,
                          int nthreads) {
  int64_t kbc = k_blocks_of(K, bs);
  float* a32 = (float*)malloc((size_t)(M * K) * sizeof(float));
  float* s32 = (float*)malloc((size_t)(N * kbc) * sizeof(float));
  float* b32 = bias ? (float*)malloc((size_t)N * sizeof(float)) : NULL;
  float* y32 = (float*)malloc((size_t)(M * N) * sizeof(float));
  mnbo_f16_to_f32_buffer(A, a32, (size_t)(M * K));
  mnbo_f16_to_f32_buffer(scales, s32, (size_t)(N * kbc));
  if (bias) mnbo_f16_to_f32_buffer(bias, b32, (size_t)N);
  mnbo_matmul_int8_f32(a32, B, s32, zp, b32, y32, M, N, K, bs, nthreads);
  mnbo_f32_to_f16_buffer(y32, Y, (size_t)(M * N));
  free(a32);
  free(s32);
  free(b32);
  free(y32);
}

/* ------------------------------------------------------------------ quantise (producer of the format)
 *
 * Follows BlockwiseQuantizer::quantizeAndTranspose with column-wise blocks
 * (onnxruntime/core/mlas/lib/q4_dq.cpp:468-574) and range2scalezp / range2scale (:347-386):
 *   asymmetric: min = min(min, 0), max = max(max, 0); scale = (max - min) / (2^bits - 1);
 *               zp = clamp(round(-min / scale)) (0 when scale is 0); q = clamp(round(v / scale + zp))
 *   symmetric : s = max if |max| > |min| else min; scale = -s / 2^(bits-1);
 *               zp = 2^(bits-1); q = clamp(round(v / scale + zp))  (computed with the reciprocal of scale)
 * src is row-major [K][N].  Rounding is roundf (half away from zero), as in the reference.  fp16 models: elements
 * are widened to fp32, the scale is computed in fp32 and stored as fp16 (RNE); the zero point comes from the
 * unrounded scale, the reciprocal from the stored one.  Positions k >= K of the last block, which the reference
 * leaves unwritten, hold the zero point here (they dequantise to 0).
 * Parity: pinned by round-trip and closed-form properties and an independent numpy restatement
 * (tests/test_oracle_quantize.py); rounding of exact .5 values, of elements and of the zero point, is pinned by
 * grids on which scale, zero point and every expected integer are a closed form of roundf (x + 0.5 -> x + 1 for even
 * and odd x: tests/tie_cases.py), which a round-half-to-even quantiser fails.
 */
static void quantize_core(uint8_t* B, float* scales, uint8_t* zp, const float* src, int64_t K, int64_t N, int bits,
                          int64_t bs, int symmetric, int scale_is_f16) {
  int64_t kbc = k_blocks_of(K, bs);
  int64_t blob = blob_of(bs, bits);
  int64_t zrow = zp_row_of(kbc, bits);
  const int maxq = (1 << bits) - 1;
  const int mid = 1 << (bits - 1);
  memset(B, 0, (size_t)(N * kbc * blob));
  /* unused slots of the last zero-point byte keep the reference's filler, the default zero point (:493) */
  if (zp) memset(zp, bits == 8 ? 0 : bits == 4 ? 0x88 : 0xAA, (size_t)(N * zrow));
  for (int64_t n = 0; n < N; ++n)
    for (int64_t kb = 0; kb < kbc; ++kb) {
      int64_t k0 = kb * bs, k1 = k0 + bs < K ? k0 + bs : K;
      float scale, rscale;
      int z;
      if (!symmetric) {
        float mn = 0.f, mx = 0.f;
        for (int64_t k = k0; k < k1; ++k) {
          float v = src[k * N + n];
          if (v < mn) mn = v;
          if (v > mx) mx = v;
        }
        scale = (mx - mn) / (float)maxq;
        float zf = scale == 0.f ? mn : -mn / scale;
        if (zf < 0.f) zf = 0.f;
        if (zf > (float)maxq) zf = (float)maxq;
        z = (int)roundf(zf);
      } else {
        float mn = 3.402823466e+38f, mx = -3.402823466e+38f;
        for (int64_t k = k0; k < k1; ++k) {
          float v = src[k * N + n];
          if (v < mn) mn = v;
          if (v > mx) mx = v;
        }
        float smax = fabsf(mx) > fabsf(mn) ? mx : mn; /* the larger half maps to [-2^(bits-1), 0] */
        scale = -smax / (float)mid;
        z = mid;
      }
      /* the scale is stored in the model's type; the reciprocal is taken from the stored value (:552-553) */
      if (scale_is_f16) scale = mnbo_f16_to_f32(mnbo_f32_to_f16(scale));
      rscale = scale == 0.f ? 0.f : 1.f / scale;
      scales[n * kbc + kb] = scale;
      if (zp) {
        uint8_t* row = zp + n * zrow;
        if (bits == 8) row[kb] = (uint8_t)z;
        else if (bits == 4) row[kb >> 1] = (uint8_t)((row[kb >> 1] & ~(0xF << ((kb & 1) * 4))) | (z << ((kb & 1) * 4)));
        else row[kb >> 2] = (uint8_t)((row[kb >> 2] & ~(0x3 << ((kb & 3) * 2))) | (z << ((kb & 3) * 2)));
      }
      uint8_t* out = B + (n * kbc + kb) * blob;
      for (int64_t k = k0; k < k0 + bs; ++k) {
        float v = k < k1 ? src[k * N + n] : 0.f;
        float qf = roundf(v * rscale + (float)z);
        if (qf < 0.f) qf = 0.f;
        if (qf > (float)maxq) qf = (float)maxq;
        int q = k < k1 ? (int)qf : z; /* padding dequantises to 0 */
        int64_t r = k - k0;
        if (bits == 8) out[r] = (uint8_t)q;
        else if (bits == 4) out[r >> 1] |= (uint8_t)(q << ((r & 1) * 4));
        else out[r >> 2] |= (uint8_t)(q << ((r & 3) * 2));
      }
    }
}

void mnbo_quantize_f32(uint8_t* B, float* scales, uint8_t* zp, const float* src, int64_t K, int64_t N, int bits,
                       int64_t bs, int symmetric) {
  quantize_core(B, scales, zp, src, K, N, bits, bs, symmetric, 0);
}

void mnbo_quantize_f16(uint8_t* B, uint16_t* scales, uint8_t* zp, const uint16_t* src, int64_t K, int64_t N, int bits,
                       int64_t bs, int symmetric) {
  int64_t kbc = k_blocks_of(K, bs);
  float* src32 = (float*)malloc(sizeof(float) * (size_t)(K * N));
  float* s32 = (float*)malloc(sizeof(float) * (size_t)(N * kbc));
  mnbo_f16_to_f32_buffer(src, src32, (size_t)(K * N));
  quantize_core(B, s32, zp, src32, K, N, bits, bs, symmetric, 1);
  mnbo_f32_to_f16_buffer(s32, scales, (size_t)(N * kbc));
  free(src32);
  free(s32);
}

/* ------------------------------------------------------------------ prologue of the fused projections
 *
 * SimplifiedLayerNormalization / SkipSimplifiedLayerNormalization of the activation, the optional first stage of
 * com.microsoft::MatMulNBitsMlp and MatMulNBitsQkv (onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3851-3877).
 * Follows the CPU kernel, onnxruntime/contrib_ops/cpu/skip_layer_norm.cc:44-97 (fp32 job; the fp16 job widens
 * input, skip, gamma and bias to fp32, runs the same arithmetic and narrows both outputs once):
 *   val = input + skip (+ bias);  sum_out = val;  out = val / sqrt(sum(val^2) / K + epsilon) * gamma
 * with fp32 accumulation in k order; row m of the input uses skip row m % skip_rows (:56, offset % skip_size).
 * skip == NULL gives SimplifiedLayerNormalization (onnxruntime/core/providers/cpu/nn/layer_norm_impl.cc:65-73,87-89:
 * the same formula without the addition).  `bias` exists only so that the reference's own test vector with a bias
 * (onnxruntime/test/contrib_ops/skiplayernorm_op_test.cc:996-1048) can be replayed; the fused operators have none.
 * Parity: pinned by that vector and by :954-993 of the same file (tests/test_oracle_fused.py), plus closed forms.
 */
void mnbo_skip_simplified_layer_norm_f32(float* out, float* sum_out, const float* input, const float* skip,
                                         int64_t skip_rows, const float* gamma, const float* bias, float epsilon,
                                         int64_t M, int64_t K) {
  for (int64_t m = 0; m < M; ++m) {
    const float* x = input + m * K;
    const float* s = skip ? skip + (m % (skip_rows > 0 ? skip_rows : M)) * K : NULL;
    float* o = out + m * K;
    float mean_square = 0.0f;
    for (int64_t h = 0; h < K; ++h) {
      float val = x[h];
      if (s) val = val + s[h];
      if (bias) val = val + bias[h];
      if (sum_out) sum_out[m * K + h] = val;
      o[h] = val;
      float sq = val * val;
      mean_square = mean_square + sq;
    }
    float denom = sqrtf(mean_square / (float)K + epsilon);
    for (int64_t h = 0; h < K; ++h) {
      float q = o[h] / denom;
      o[h] = q * gamma[h];
    }
  }
}

void mnbo_skip_simplified_layer_norm_f16(uint16_t* out, uint16_t* sum_out, const uint16_t* input, const uint16_t* skip,
                                         int64_t skip_rows, const uint16_t* gamma, const uint16_t* bias, float epsilon,
                                         int64_t M, int64_t K) {
  int64_t srows = skip_rows > 0 ? skip_rows : M;
  float* in32 = (float*)malloc(sizeof(float) * (size_t)(M * K));
  float* sk32 = skip ? (float*)malloc(sizeof(float) * (size_t)(srows * K)) : NULL;
  float* g32 = (float*)malloc(sizeof(float) * (size_t)K);
  float* b32 = bias ? (float*)malloc(sizeof(float) * (size_t)K) : NULL;
  float* o32 = (float*)malloc(sizeof(float) * (size_t)(M * K));
  float* s32 = sum_out ? (float*)malloc(sizeof(float) * (size_t)(M * K)) : NULL;
  mnbo_f16_to_f32_buffer(input, in32, (size_t)(M * K));
  if (skip) mnbo_f16_to_f32_buffer(skip, sk32, (size_t)(srows * K));
  mnbo_f16_to_f32_buffer(gamma, g32, (size_t)K);
  if (bias) mnbo_f16_to_f32_buffer(bias, b32, (size_t)K);
  mnbo_skip_simplified_layer_norm_f32(o32, s32, in32, sk32, srows, g32, b32, epsilon, M, K);
  mnbo_f32_to_f16_buffer(o32, out, (size_t)(M * K));
  if (sum_out) mnbo_f32_to_f16_buffer(s32, sum_out, (size_t)(M * K));
  free(in32);
  free(sk32);
  free(g32);
  free(b32);
  free(o32);
  free(s32);
}
