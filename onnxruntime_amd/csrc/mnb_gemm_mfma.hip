// Dequant-in-LDS MFMA GEMM for fp16 models, M > 16.
//
// Device counterpart of the reference's prefill loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:
// 563-732: dequantise a strip of B into a panel buffer, then run the float GEMM kernel over it).  Here a workgroup
// dequantises a BN x BK tile of B to fp16 into LDS once per k-step (bit-identical to the reference's fp16
// dequantisation) and every wavefront feeds it, together with the A tile, to v_mfma_f32_32x32x16_f16 with fp32
// accumulation.  Bias add and the single fp32 -> fp16 narrowing happen in the epilogue.
#include "mnb_device.cuh"
#include "mnb_internal.h"

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // halves; 16 bytes of padding per row keep ds_read_b128 conflict-free
constexpr int THREADS = 256;

struct GemmParams {
  const _Float16* A;
  const uint4* W;
  const uint8_t* meta;
  const _Float16* bias;
  _Float16* C;
  int64_t lda, ldc, Npad;
  int M, N, K, bs;
  int ksteps;  // Kpad / BK
};

template <int BITS, bool HAS_ZP>
__global__ void __launch_bounds__(THREADS) mnb_gemm_mfma_kernel(GemmParams p) {
  constexpr int GK = 128 / BITS;               // k per 16-byte group
  constexpr int GPK = BK / GK;                 // groups per column per k-step: 2 (4-bit) or 4 (8-bit)
  constexpr int B_LOADS = BN * GPK / THREADS;  // 16-byte weight loads per thread per k-step: 1 or 2
  constexpr int A_LOADS = BM * (BK / 8) / THREADS;  // 16-byte activation loads per thread per k-step: 4

  __shared__ __align__(16) _Float16 As[BM * LDS_STRIDE];
  __shared__ __align__(16) _Float16 Bs[BN * LDS_STRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 wavefronts, 64 x 64 outputs each
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;

  f16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 a_reg[A_LOADS];
  uint4 b_reg[B_LOADS];

  auto load_global = [&](int ks) {
    const int k0 = ks * BK;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int c = tid + i * THREADS;
      const int row = c >> 3, kc = c & 7;
      // unconditional load from a clamped address, then a select: a predicated load would serialise the loop
      int m = m0 + row;
      m = m < p.M ? m : p.M - 1;
      const int k = k0 + kc * 8;
      const int kc_safe = k < p.K ? k : p.K - 8;
      uint4 v = *reinterpret_cast<const uint4*>(p.A + (int64_t)m * p.lda + kc_safe);
      if (k >= p.K) v = make_uint4(0, 0, 0, 0);
      a_reg[i] = v;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int c = tid + i * THREADS;
      const int col = c % BN, gi = c / BN;
      b_reg[i] = p.W[(int64_t)(ks * GPK + gi) * p.Npad + n0 + col];
    }
  };

  auto store_lds = [&](int ks) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int c = tid + i * THREADS;
      const int row = c >> 3, kc = c & 7;
      *reinterpret_cast<uint4*>(&As[row * LDS_STRIDE + kc * 8]) = a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int c = tid + i * THREADS;
      const int col = c % BN, gi = c / BN;
      __align__(16) _Float16 out[GK];
      mnb_dequant_group_h<BITS, HAS_ZP>(b_reg[i], p.meta, (int64_t)ks * GPK + gi, n0 + col, p.Npad, p.bs, out);
      uint4* dst = reinterpret_cast<uint4*>(&Bs[col * LDS_STRIDE + gi * GK]);
#pragma unroll
      for (int j = 0; j < GK / 8; ++j) dst[j] = reinterpret_cast<const uint4*>(out)[j];
    }
  };

  load_global(0);
  for (int ks = 0; ks < p.ksteps; ++ks) {
    __syncthreads();  // LDS free
    store_lds(ks);
    __syncthreads();  // LDS full
    if (ks + 1 < p.ksteps) load_global(ks + 1);
    const int li = lane & 31, kq = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      h8_t af[2], bf[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        af[t] = *reinterpret_cast<const h8_t*>(&As[(wm * 64 + t * 32 + li) * LDS_STRIDE + kk * 16 + kq * 8]);
        bf[t] = *reinterpret_cast<const h8_t*>(&Bs[(wn * 64 + t * 32 + li) * LDS_STRIDE + kk * 16 + kq * 8]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue: D[i][j], lane holds column j = lane % 32 and rows 8*(r/4) + 4*(lane/32) + r%4
  const int li = lane & 31, kq = lane >> 5;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + li;
    if (n >= p.N) continue;
    const float b = p.bias ? (float)p.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + kq * 4 + (r & 3);
        if (m < p.M) p.C[(int64_t)m * p.ldc + n] = (_Float16)(acc[i][j][r] + b);
      }
    }
  }
}

template <int BITS, bool HAS_ZP>
hipError_t launch(const GemmParams& p, hipStream_t s) {
  dim3 grid((unsigned)((p.N + BN - 1) / BN), (unsigned)((p.M + BM - 1) / BM)), blk(THREADS);
  mnb_gemm_mfma_kernel<BITS, HAS_ZP><<<grid, blk, 0, s>>>(p);
  return hipGetLastError();
}

}  // namespace

hipError_t mnb_launch_gemm_mfma(const MnbGemmArgs& a, hipStream_t s) {
  GemmParams p{};
  p.A = reinterpret_cast<const _Float16*>(a.A);
  p.W = reinterpret_cast<const uint4*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + a.L.meta_off;
  p.bias = reinterpret_cast<const _Float16*>(a.bias);
  p.C = reinterpret_cast<_Float16*>(a.C);
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.Npad = a.L.Npad;
  p.M = (int)a.M;
  p.N = (int)a.L.N;
  p.K = (int)a.L.K;
  p.bs = a.L.bs;
  p.ksteps = (int)((a.L.K + BK - 1) / BK);
  if (a.L.bits == 4) return a.L.has_zp ? launch<4, true>(p, s) : launch<4, false>(p, s);
  return a.L.has_zp ? launch<8, true>(p, s) : launch<8, false>(p, s);
}
