// fp32 models, M > 16: tiled GEMM on the fp32 matrix cores.
//
// Device counterpart of the reference's prefill loop for float activations (SQ4BitGemm_CompFp32,
// onnxruntime/core/mlas/lib/qnbitgemm.cpp:563-732: dequantise a strip of B to fp32, then run the float GEMM kernel
// over it) and of the dequantise-then-SGEMM route (MatMulNBits<T>::ComputeBUnpacked,
// onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:1184-1333), which is also what typed zero points and
// bfloat16 activations run on after widening (mnb_variant.hip).
//
// 128 x 128 output tile per workgroup of four wavefronts (2 x 2), each owning 64 x 64 as 2 x 2
// v_mfma_f32_32x32x2_f32 accumulators (64 x 128 with 32 x 64 per wavefront while such tiles fit the chip in one round).  Per k-step of 32:
//   * every thread fetches 4 x 16 B of A and 8 bytes (4-bit) or 16 bytes (8-bit) of packed weights for the NEXT step
//     into registers while the matrix cores work on the current one;
//   * the weights are dequantised to fp32 in registers - float(q) - zp, one multiply by the scale: the bits of
//     MlasDequantizeBlockwise<float> (onnxruntime/core/mlas/lib/q4_dq.cpp:587-641) - and written to LDS next to the
//     A tile (rows padded by 16 B: conflict-free 16-byte reads);
//   * lane (r = lane % 32, h = lane / 32) feeds MFMA i of the step with k = 16 h + i of row / column r, so its
//     sixteen A and B operands are 64 contiguous bytes of LDS (the contraction index of a matrix instruction may be
//     permuted freely as long as A and B use the same permutation).
// One LDS buffer, two barriers per step: a step is 64 matrix instructions of 64 cycles per wavefront, so the barriers
// are noise.  The kernel is bound by the fp32 matrix cores (157 TFLOP/s peak), an order of magnitude above the VALU
// kernel it replaces for these shapes.
#include <cstdlib>

#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

typedef float f16v_t __attribute__((ext_vector_type(16)));
typedef float f4v_t __attribute__((ext_vector_type(4)));

constexpr int BN = 128, BK = 32;  // rows of the tile: 64 TM, TM = 32-row matrix-core tiles per wavefront (2, or 1 for M <= 64)
constexpr int THREADS = 256;
constexpr int STRIDE = BK + 4;  // floats per staged row

struct Gemm32Params {
  const float* A;
  const uint8_t* W;  // packed weights, byte addressed
  const uint8_t* meta;
  const float* bias;
  float* C;
  int64_t lda, ldc, Npad;
  int M, N, K, bs_shift;
  int ksteps;
  int tiles_n;
  int a_vec_ok;  // A allows 16-byte loads: aligned base, row pitch and K multiples of 4 floats
};

template <int BITS, bool HAS_ZP, int TM>
__global__ void __launch_bounds__(THREADS) mnb_gemm32_kernel(Gemm32Params p) {
  constexpr int BM = 64 * TM;
  constexpr int A_LOADS = 2 * TM;  // 16-byte activation loads per thread and step
  __shared__ __align__(16) float As[BM * STRIDE];
  __shared__ __align__(16) float Bs[BN * STRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 31, h = lane >> 5;
  const int m0 = (blockIdx.x / p.tiles_n) * BM;
  const int n0 = (blockIdx.x % p.tiles_n) * BN;

  f16v_t acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  // ---- this thread's share of the tiles
  // A: rows a_row + 32 i (i < A_LOADS), floats [a_kc, a_kc + 4) of the step; rows beyond M repeat row M - 1 (never
  // stored)
  const int a_row = tid >> 3, a_kc = (tid & 7) * 4;
  const float* a_ptr[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    int m = m0 + a_row + 32 * i;
    m = m < p.M ? m : p.M - 1;
    a_ptr[i] = p.A + (int64_t)m * p.lda + a_kc;
  }
  // B: column b_col, sixteen k of the step: half b_half of the column's 16-byte vector (4-bit: one vector covers the
  // step) or vector b_half of the step (8-bit: two vectors of sixteen)
  const int b_col = tid >> 1, b_half = tid & 1;
  const int64_t col = n0 + b_col;  // < Npad: the padding columns hold zero weights and zero scales
  const int64_t mcol = mnb_meta_col(col);

  f4v_t ra[A_LOADS];
  uint32_t rw[4];
  float rs = 0.f, rz = 0.f;

  auto load_step = [&](int ks) {
    const int k0 = ks * BK;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const float* src = a_ptr[i] + k0;
      if (p.a_vec_ok) {  // K is a multiple of 4: a chunk lies wholly below K or wholly beyond it
        ra[i] = (k0 + a_kc < p.K) ? *reinterpret_cast<const f4v_t*>(src) : f4v_t{0.f, 0.f, 0.f, 0.f};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) ra[i][e] = (k0 + a_kc + e < p.K) ? src[e] : 0.f;
      }
    }
    int64_t kfirst;  // first k of this thread's sixteen weights
    if constexpr (BITS == 4) {
      const uint8_t* v = p.W + ((int64_t)ks * p.Npad + col) * 16 + b_half * 8;
      const uint2 w = *reinterpret_cast<const uint2*>(v);
      rw[0] = w.x, rw[1] = w.y, rw[2] = 0u, rw[3] = 0u;
      kfirst = (int64_t)k0 + 16 * b_half;
    } else {
      const uint8_t* v = p.W + (((int64_t)ks * 2 + b_half) * p.Npad + col) * 16;
      const uint4 w = *reinterpret_cast<const uint4*>(v);
      rw[0] = w.x, rw[1] = w.y, rw[2] = w.z, rw[3] = w.w;
      kfirst = (int64_t)k0 + 16 * b_half;
    }
    mnb_load_meta_f<HAS_ZP, BITS>(p.meta, (kfirst >> p.bs_shift) * p.Npad + mcol, rs, rz);
  };

  auto store_step = [&]() {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      *reinterpret_cast<f4v_t*>(&As[(a_row + 32 * i) * STRIDE + a_kc]) = ra[i];
    float wv[16];
    if constexpr (BITS == 4) {
      float d[8];
      mnb_unpack4_f(rw[0], rz, d);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] = d[e] * rs;
      mnb_unpack4_f(rw[1], rz, d);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[8 + e] = d[e] * rs;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float d[4];
        mnb_unpack8_f(rw[i], rz, d);
#pragma unroll
        for (int e = 0; e < 4; ++e) wv[4 * i + e] = d[e] * rs;
      }
    }
    float* dst = &Bs[b_col * STRIDE + 16 * b_half];
#pragma unroll
    for (int c = 0; c < 4; ++c)
      *reinterpret_cast<f4v_t*>(dst + 4 * c) = f4v_t{wv[4 * c], wv[4 * c + 1], wv[4 * c + 2], wv[4 * c + 3]};
  };

  load_step(0);
  for (int ks = 0; ks < p.ksteps; ++ks) {
    __syncthreads();  // the previous step's operands have been read
    store_step();
    __syncthreads();
    if (ks + 1 < p.ksteps) load_step(ks + 1);
    const float* a_base = &As[(wm * 32 * TM + r) * STRIDE + 16 * h];
    const float* b_base = &Bs[(wn * 64 + r) * STRIDE + 16 * h];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      f4v_t a4[TM], b4[2];
#pragma unroll
      for (int t = 0; t < TM; ++t) a4[t] = *reinterpret_cast<const f4v_t*>(a_base + t * 32 * STRIDE + 4 * c);
#pragma unroll
      for (int t = 0; t < 2; ++t) b4[t] = *reinterpret_cast<const f4v_t*>(b_base + t * 32 * STRIDE + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[i][e], b4[j][e], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue.  D of a 32 x 32 tile: lane holds column r, rows 8 (q / 4) + 4 h + q % 4.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + r;
    if (n >= p.N) continue;
    const float b = p.bias ? p.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int m = m0 + wm * 32 * TM + i * 32 + (q >> 2) * 8 + h * 4 + (q & 3);
        if (m < p.M) p.C[(int64_t)m * p.ldc + n] = acc[i][j][q] + b;
      }
    }
  }
}

template <int BITS, bool HAS_ZP>
hipError_t launch(const Gemm32Params& p, int64_t row_tiles, int tm, hipStream_t s) {
  const dim3 grid((unsigned)(row_tiles * p.tiles_n)), blk(THREADS);
  if (tm == 1)
    mnb_gemm32_kernel<BITS, HAS_ZP, 1><<<grid, blk, 0, s>>>(p);
  else
    mnb_gemm32_kernel<BITS, HAS_ZP, 2><<<grid, blk, 0, s>>>(p);
  return hipGetLastError();
}

}  // namespace

bool mnb_gemm32_applicable(const MnbGemmArgs& a) {
  static const bool disabled = [] {
    const char* e = mnb_tuning_env("MNB_GEMM32");  // tuning override: "0" sends fp32 problems to the VALU tile kernel
    return e != nullptr && e[0] == '0';
  }();
  return !disabled && a.L.dtype == kMnbDtypeFloat && a.M > 16;
}

hipError_t mnb_launch_gemm32(const MnbGemmArgs& a, hipStream_t s) {
  const MnbLayout& L = a.L;
  Gemm32Params p{};
  p.A = reinterpret_cast<const float*>(a.A);
  p.W = reinterpret_cast<const uint8_t*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + L.meta_off;
  p.bias = reinterpret_cast<const float*>(a.bias);
  p.C = reinterpret_cast<float*>(a.C);
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.Npad = L.Npad;
  p.M = (int)a.M;
  p.N = (int)L.N;
  p.K = (int)L.K;
  p.bs_shift = mnb_log2i(L.bs);
  p.ksteps = (int)((L.K + BK - 1) / BK);  // <= Kpad / 32: steps past K read zero weights
  p.tiles_n = (int)((L.N + BN - 1) / BN);
  p.a_vec_ok = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 4 == 0) && (L.K % 4 == 0);
  // 64-row tiles while they still fit the 256 compute units in one round: half the latency of a round
  const int64_t rows64 = (a.M + 63) / 64;
  const int tm = rows64 * p.tiles_n <= 256 ? 1 : 2;
  const int64_t row_tiles = (a.M + 64 * tm - 1) / (64 * tm);
  if (L.bits == 4) return L.has_zp ? launch<4, true>(p, row_tiles, tm, s) : launch<4, false>(p, row_tiles, tm, s);
  return L.has_zp ? launch<8, true>(p, row_tiles, tm, s) : launch<8, false>(p, row_tiles, tm, s);
}
