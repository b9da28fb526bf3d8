// fp32 models with few rows (5 <= M <= 64, and beyond while the tile GEMM's grid stays small) on the fp32 matrix cores.
//
// Between the VALU kernel for very few rows (mnb_gemv.hip: the rows of A ride in scalar registers, which run out
// beyond eight rows) and the tile GEMM for many (mnb_gemm32.hip: 64 x 128 tiles, N / 128 workgroups - a chip mostly
// idle and one long round of 185 us and more for a few dozen rows) the work is still one pass over the weights, as in
// the reference's decode loop (MlasQ4GemmKernelBlkLen32PlusAvx512f,
// onnxruntime/core/mlas/lib/sqnbitgemm_kernel_avx_common_fp32.h:288-639): Y = A x dequant(B)^T (+ bias), everything
// in fp32.
//
// Same mapping as the fp16 decode kernel (mnb_skinny.hip): a workgroup owns 16 T output columns and 16 rows, K is
// split over its wavefronts and reduced through LDS in a fixed order (nothing is split over workgroups).  Lane
// (j = lane % 16, kq = lane / 16) reads ONE 16-byte weight vector of column j, k-group 4 c + kq of chunk c, and the GK
// activations of row j that face it.  v_mfma_f32_16x16x4_f32 contracts over four k at a time, one per kq; the
// contraction index may be permuted freely as long as A and B agree, so instruction (i, e) takes element e of word i
// of every lane's own vector: lane (j, kq) supplies weight and activation of k = GK (4 c + kq) + 8 i + e (4-bit) or
// + 4 i + e (8-bit).  The weights are dequantised in registers as (float(q) - zp) * scale: the subtraction is exact,
// so this is the reference's fp32 dequantisation bit for bit (MlasDequantizeBlockwise).  The fp32 matrix
// instruction takes 32 cycles for 64 weights of a wavefront, more than twice the vector unit's work per weight, so the
// kernel is bound by the matrix cores: one byte of 4-bit weights per SIMD and cycle, about 2.4 TB/s over the chip.
// More than 16 rows are blocks of 16 in grid.y; the blocks of one column slab re-read its weights from the caches.
#include <cstdio>
#include <cstdlib>

#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

struct Rows16Params {
  const float* A;
  const uint4* W;
  const uint8_t* meta;
  const float* bias;
  float* C;
  int64_t lda, ldc, Npad;
  int M, N;
  int bs_shift;
  int KG;      // k-groups (K is a whole number of them)
  int chunks;  // chunks of four k-groups that hold a k-group below KG
};

__device__ __forceinline__ f4_t mfma_16x16x4_f32(float a, float b, f4_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
#else
  (void)a, (void)b;
  return c;
#endif
}

// registers of one chunk: the lane's weight vectors and meta entries of T column tiles, and its activations
template <int BITS, int T>
struct Rows16Regs {
  uint4 w[T];
  float s0[T], z0[T];  // scale and zero point of the vector's (first) block
  float s1[T], z1[T];  // 4-bit with blocks of 16: of its second half
  float4 a[(128 / BITS) / 4];
};

template <int BITS, bool HAS_ZP, bool SMALL_BS, int T, int NW>
__global__ void __launch_bounds__(NW * 64) mnb_rows16_f32_kernel(Rows16Params p) {
  constexpr int GK = 128 / BITS;  // k of one 16-byte vector: 32 or 16
  constexpr int NV = GK / 4;      // 16-byte pieces of A per vector
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, kq = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * (16 * T);
  const int64_t col0 = n0 + j;  // the lane's column in tile t is col0 + 16 t (below Npad: Npad is a multiple of 256)
  const int m0 = blockIdx.y * 16;
  const int row = m0 + j < p.M ? m0 + j : p.M - 1;  // rows beyond M re-read the last row and are never stored
  const float* a_row = p.A + (int64_t)row * p.lda;
  const int64_t mcol = mnb_meta_col(col0);  // the entries of columns col0 + 16 t follow at mcol + t

  f4_t y[T];
#pragma unroll
  for (int t = 0; t < T; ++t) y[t] = f4_t{0.f, 0.f, 0.f, 0.f};

  // A k-group beyond KG (the last chunk of a K that is not a whole number of chunks) is clamped to the last one for
  // the loads and contributes nothing: its activations are replaced by zeros.
  auto load = [&](int c, Rows16Regs<BITS, T>& R) {
    const int g_raw = 4 * c + kq;
    const bool live = g_raw < p.KG;
    const int g = live ? g_raw : p.KG - 1;
    const int64_t k0 = (int64_t)g * GK;
    const int64_t kb = k0 >> p.bs_shift;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      mnb_load_meta_f<HAS_ZP, BITS>(p.meta, kb * p.Npad + mcol + t, R.s0[t], R.z0[t]);
      if constexpr (SMALL_BS) mnb_load_meta_f<HAS_ZP, BITS>(p.meta, (kb + 1) * p.Npad + mcol + t, R.s1[t], R.z1[t]);
    }
#pragma unroll
    for (int t = 0; t < T; ++t) R.w[t] = p.W[(int64_t)g * p.Npad + col0 + t * 16];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const float4 a = *reinterpret_cast<const float4*>(a_row + k0 + 4 * v);
      R.a[v] = live ? a : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };

  auto compute = [&](const Rows16Regs<BITS, T>& R) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const uint32_t wd[4] = {R.w[t].x, R.w[t].y, R.w[t].z, R.w[t].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool second = SMALL_BS && i >= 2;
        const float s = second ? R.s1[t] : R.s0[t];
        const float zp = second ? R.z1[t] : R.z0[t];
        if constexpr (BITS == 4) {
          // bytes of b0: nibbles 0 2 4 6 = elements 0 4 1 5; of b1: nibbles 1 3 5 7 = elements 2 6 3 7
          const uint32_t b0 = wd[i] & 0x0F0F0F0Fu, b1 = (wd[i] >> 4) & 0x0F0F0F0Fu;
          const float q[8] = {(float)(b0 & 0xffu),         (float)((b0 >> 16) & 0xffu), (float)(b1 & 0xffu),
                              (float)((b1 >> 16) & 0xffu), (float)((b0 >> 8) & 0xffu),  (float)(b0 >> 24),
                              (float)((b1 >> 8) & 0xffu),  (float)(b1 >> 24)};
          const float4 a_lo = R.a[2 * i], a_hi = R.a[2 * i + 1];
          const float a[8] = {a_lo.x, a_lo.y, a_lo.z, a_lo.w, a_hi.x, a_hi.y, a_hi.z, a_hi.w};
#pragma unroll
          for (int e = 0; e < 8; ++e) y[t] = mfma_16x16x4_f32(a[e], (q[e] - zp) * s, y[t]);
        } else {
          const uint32_t w = wd[i];
          const float q[4] = {(float)(w & 0xffu), (float)((w >> 8) & 0xffu), (float)((w >> 16) & 0xffu),
                              (float)(w >> 24)};
          const float4 av = R.a[i];
          const float a[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) y[t] = mfma_16x16x4_f32(a[e], (q[e] - zp) * s, y[t]);
        }
      }
    }
  };

  // two chunks in flight per wavefront; a prefetch beyond the last chunk is clamped to it and never used
  Rows16Regs<BITS, T> R0, R1;
  const int last = p.chunks - 1;
  int c = wave;
  if (c < p.chunks) {
    load(c, R0);
    for (; c + NW < p.chunks; c += 2 * NW) {
      load(c + NW, R1);
      compute(R0);
      load(c + 2 * NW < p.chunks ? c + 2 * NW : last, R0);
      compute(R1);
    }
    if (c < p.chunks) compute(R0);
  }

  // reduce over the wavefronts in wavefront order: lane (j, kq), register r of y[t] holds row m0 + 4 kq + r, column
  // n0 + 16 t + j
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[(wave * T * 4 + t * 4 + r) * 64 + lane] = y[t][r];
  __syncthreads();
  for (int i = threadIdx.x; i < T * 4 * 64; i += NW * 64) {
    const int l = i & 63, tr = i >> 6;
    const int t = tr >> 2, r = tr & 3;
    const int m = m0 + 4 * (l >> 4) + r;
    const int64_t n = n0 + t * 16 + (l & 15);
    if (m >= p.M || n >= p.N) continue;
    float sum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) sum += red[(w2 * T * 4 + tr) * 64 + l];
    if (p.bias) sum += p.bias[n];
    p.C[(int64_t)m * p.ldc + n] = sum;
  }
}

template <int BITS, bool HAS_ZP, bool SMALL_BS, int T>
hipError_t launch_nw(const Rows16Params& p, int nw, hipStream_t s) {
  const dim3 grid((unsigned)((p.N + 16 * T - 1) / (16 * T)), (unsigned)((p.M + 15) / 16));
  // two chunks of 4-bit weights for four tiles do not fit the 128 registers of sixteen wavefronts: eight there
  if (BITS == 4 && T == 4 && nw == 16) nw = 8;
  const size_t smem = (size_t)nw * T * 4 * 64 * sizeof(float);
  if constexpr (!(BITS == 4 && T == 4)) {
    if (nw == 16) {
      mnb_rows16_f32_kernel<BITS, HAS_ZP, SMALL_BS, T, 16><<<grid, dim3(1024), smem, s>>>(p);
      return hipGetLastError();
    }
  }
  if (nw >= 8)
    mnb_rows16_f32_kernel<BITS, HAS_ZP, SMALL_BS, T, 8><<<grid, dim3(512), smem, s>>>(p);
  else
    mnb_rows16_f32_kernel<BITS, HAS_ZP, SMALL_BS, T, 4><<<grid, dim3(256), smem, s>>>(p);
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP, bool SMALL_BS>
hipError_t launch_t(const Rows16Params& p, int t, int nw, hipStream_t s) {
  if (t == 4) return launch_nw<BITS, HAS_ZP, SMALL_BS, 4>(p, nw, s);
  if (t == 2) return launch_nw<BITS, HAS_ZP, SMALL_BS, 2>(p, nw, s);
  return launch_nw<BITS, HAS_ZP, SMALL_BS, 1>(p, nw, s);
}

template <int BITS, bool HAS_ZP>
hipError_t launch_bs(const Rows16Params& p, int bs, int t, int nw, hipStream_t s) {
  if constexpr (BITS == 4) {
    if (bs == 16) return launch_t<BITS, HAS_ZP, true>(p, t, nw, s);
  }
  return launch_t<BITS, HAS_ZP, false>(p, t, nw, s);
}

}  // namespace

// Rows of A 16-byte aligned, K a whole number of k-groups; from 5 rows (fewer: the VALU kernel streams the weights as
// fast and wastes no matrix-core rows) up to where the tile GEMM's 64 x 128 tiles fill the chip: both kernels run the
// fp32 matrix cores at the same rate once busy (measured 87-89 TFLOP/s), but the tile GEMM pays a whole round of
// workgroups (183 us at K = 4096) however few of them there are; the two meet at about one and a half rounds.
bool mnb_rows16_f32_applicable(const MnbGemmArgs& a) {
  int64_t min_m = 5, max_m = 64;
  const int64_t tile_gemm_wgs = ((a.M + 63) / 64) * ((a.L.N + 127) / 128);
  if (tile_gemm_wgs * 2 <= (int64_t)mnb_device_info().cus * 3) max_m = a.M;
  if (const char* e = mnb_tuning_env("MNB_ROWS16_M")) {  // calibration: "<min>,<max>"
    long long lo = 0, hi = 0;
    if (sscanf(e, "%lld,%lld", &lo, &hi) == 2) min_m = lo, max_m = hi;
  }
  return a.L.dtype == kMnbDtypeFloat && a.io == kMnbIoModel && a.M >= min_m && a.M <= max_m && a.L.K % a.L.group_k == 0 &&
         reinterpret_cast<uintptr_t>(a.A) % 16 == 0 && (a.lda * 4) % 16 == 0;
}

hipError_t mnb_launch_rows16_f32(const MnbGemmArgs& a, hipStream_t s) {
  if (!mnb_rows16_f32_applicable(a) || a.epi.kind != kMnbFusedNone) return hipErrorInvalidValue;
  const MnbLayout& L = a.L;
  Rows16Params p{};
  p.A = reinterpret_cast<const float*>(a.A);
  p.W = reinterpret_cast<const uint4*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + L.meta_off;
  p.bias = reinterpret_cast<const float*>(a.bias);
  p.C = reinterpret_cast<float*>(a.C);
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.Npad = L.Npad;
  p.M = (int)a.M;
  p.N = (int)L.N;
  p.bs_shift = mnb_log2i(L.bs);
  p.KG = (int)(L.K / L.group_k);
  p.chunks = (p.KG + 3) / 4;
  // Column tiles per workgroup: wide slabs re-read the activations less often (every workgroup reads its 16 rows of
  // A once); the grid has to give every compute unit a workgroup first.
  const int64_t tiles = (L.N + 15) / 16, row_blocks = (a.M + 15) / 16;
  int t = 1;
  if (tiles * row_blocks >= 4 * 224) t = 4;
  else if (tiles * row_blocks >= 2 * 224) t = 2;
  if (const char* e = mnb_tuning_env("MNB_ROWS16_T")) t = atoi(e) == 4 ? 4 : atoi(e) == 2 ? 2 : 1;  // calibration
  // wavefronts: at least four chunks each (measured: sixteen wavefronts pay only for K beyond 8192 or so), and four
  // when the grid brings several workgroups per compute unit anyway
  int nw = p.chunks >= 64 ? 16 : p.chunks >= 16 ? 8 : 4;
  if (((tiles + t - 1) / t) * row_blocks >= 512) nw = 4;
  if (const char* e = mnb_tuning_env("MNB_ROWS16_NW")) nw = atoi(e) == 16 ? 16 : atoi(e) == 8 ? 8 : 4;
  if (L.bits == 4) return L.has_zp ? launch_bs<4, true>(p, L.bs, t, nw, s) : launch_bs<4, false>(p, L.bs, t, nw, s);
  return L.has_zp ? launch_bs<8, true>(p, L.bs, t, nw, s) : launch_bs<8, false>(p, L.bs, t, nw, s);
}
