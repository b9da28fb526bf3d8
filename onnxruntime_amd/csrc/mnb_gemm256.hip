// Dequant-in-LDS MFMA GEMM for fp16 models and large M: 256 x 256 output tile per workgroup.
//
// Device counterpart of the reference's prefill loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:
// 563-732).  Four wavefronts (2 x 2), each owning a 128 x 128 block of the tile as 4 x 4 v_mfma_f32_32x32x16_f16
// accumulators (256 accumulator registers per lane).  Per k-step of 64:
//   * every thread fetches 8 x 16 B of A and 2 (4-bit) or 4 (8-bit) x 16 B of packed weights for the NEXT step
//     into registers while the matrix cores work on the current one;
//   * the weights are dequantised to fp16 in registers (exact (q - zp), one rounding by the scale: bit-identical
//     to the reference's fp16 dequantisation) and written, with the A rows, into the other LDS buffer;
//   * one barrier per step.
// LDS rows are padded by 16 bytes so both the 16-byte staging writes and the ds_read_b128 operand fetches are
// bank-conflict free.  Bias add and the single fp32 -> fp16 narrowing happen in the epilogue.
#include "mnb_device.cuh"
#include "mnb_internal.h"

namespace {

typedef uint32_t u4_t __attribute__((ext_vector_type(4)));  // plain register quad (HIP's uint4 struct resists SROA)

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // halves per staged row
constexpr int THREADS = 256;
constexpr int STAGE_HALVES = (BM + BN) * LDS_STRIDE;  // one buffer: A rows then B rows

struct Gemm256Params {
  const _Float16* A;
  const uint4* W;
  const uint8_t* meta;
  const _Float16* bias;
  _Float16* C;
  int64_t lda, ldc, Npad;
  int M, N, K, bs_shift;
  int ksteps;
};

template <int BITS, bool HAS_ZP, bool SMALL_BS>
__global__ void __launch_bounds__(THREADS, 1) mnb_gemm256_kernel(Gemm256Params p) {
  constexpr int GK = 128 / BITS;                    // k per 16-byte group
  constexpr int GPK = BK / GK;                      // groups per column per k-step: 2 or 4
  constexpr int A_LOADS = BM * (BK / 8) / THREADS;  // 8
  extern __shared__ __align__(16) _Float16 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // XCD-aware tile order: consecutive workgroups go to different XCDs, so give each XCD a contiguous band of rows
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  const int li = lane & 31, kq = lane >> 5;

  f16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  u4_t a_reg[A_LOADS];
  u4_t b_reg[GPK];
  uint32_t m_reg[GPK * (SMALL_BS ? 2 : 1)];

  const int a_row = tid >> 3, a_kc = tid & 7;  // thread's first A chunk: row a_row (+32 per load), k chunk a_kc
  const _Float16* a_ptr[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    int m = m0 + a_row + i * 32;
    m = m < p.M ? m : p.M - 1;
    a_ptr[i] = p.A + (int64_t)m * p.lda + a_kc * 8;
  }
  const int64_t bcol = n0 + tid;
  const int64_t mcol = mnb_meta_col(bcol);

  auto meta_at = [&](int64_t idx) -> uint32_t {
    if constexpr (HAS_ZP)
      return reinterpret_cast<const uint32_t*>(p.meta)[idx];
    else
      return reinterpret_cast<const uint16_t*>(p.meta)[idx];
  };

  auto load_global = [&](int ks) {
    const int k0 = ks * BK;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      // unconditional loads (a predicated load serialises on its own zero fill): rows beyond M re-read row M-1
      // and are never stored; K is a multiple of BK for this kernel
      a_reg[i] = *reinterpret_cast<const u4_t*>(a_ptr[i] + k0);
    }
#pragma unroll
    for (int g = 0; g < GPK; ++g) {
      const int64_t kg = (int64_t)ks * GPK + g;
      b_reg[g] = *reinterpret_cast<const u4_t*>(p.W + kg * p.Npad + bcol);
      if constexpr (SMALL_BS) {
        m_reg[2 * g] = meta_at((kg * 2) * p.Npad + mcol);
        m_reg[2 * g + 1] = meta_at((kg * 2 + 1) * p.Npad + mcol);
      } else {
        m_reg[g] = meta_at(((kg * GK) >> p.bs_shift) * p.Npad + mcol);
      }
    }
  };

  auto decode = [&](uint32_t raw, h2_t& s2, ZpH& z) {
    if constexpr (HAS_ZP) {
      const h2_t m = mnb_as_h2(raw);
      s2 = mnb_h2(m.x);
      z = mnb_zp_h(m.y);
    } else {
      s2 = mnb_h2(__builtin_bit_cast(_Float16, (uint16_t)raw));
      z = mnb_zp_h((_Float16)(-(1024.0f + (float)(1 << (BITS - 1)))));
    }
  };

  // dequantise group g of this thread's column and write its GK halves to buffer `buf`
  auto store_b_group = [&](int buf, int g) {
    _Float16* brow = lds + buf * STAGE_HALVES + (BM + tid) * LDS_STRIDE + g * GK;
    const uint32_t wd[4] = {b_reg[g][0], b_reg[g][1], b_reg[g][2], b_reg[g][3]};
    h2_t s2a, s2b;
    ZpH za, zb;
    if constexpr (SMALL_BS) {
      decode(m_reg[2 * g], s2a, za);
      decode(m_reg[2 * g + 1], s2b, zb);
    } else {
      decode(m_reg[g], s2a, za);
      s2b = s2a;
      zb = za;
    }
    if constexpr (BITS == 4) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        h2_t d[4];
        mnb_unpack4_h(wd[i], i < 2 ? za : zb, d);
        const h2_t s2 = i < 2 ? s2a : s2b;
        const u4_t o = {mnb_as_u32(d[0] * s2), mnb_as_u32(d[1] * s2), mnb_as_u32(d[2] * s2), mnb_as_u32(d[3] * s2)};
        *reinterpret_cast<u4_t*>(brow + i * 8) = o;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        h2_t d[4];
        mnb_unpack8_h(wd[2 * i], za, d);
        mnb_unpack8_h(wd[2 * i + 1], za, d + 2);
        const u4_t o = {mnb_as_u32(d[0] * s2a), mnb_as_u32(d[1] * s2a), mnb_as_u32(d[2] * s2a),
                        mnb_as_u32(d[3] * s2a)};
        *reinterpret_cast<u4_t*>(brow + i * 8) = o;
      }
    }
  };

  auto store_a = [&](int buf, int i) {
    *reinterpret_cast<u4_t*>(lds + buf * STAGE_HALVES + (a_row + i * 32) * LDS_STRIDE + a_kc * 8) = a_reg[i];
  };

  auto mfma_slab = [&](int buf, int kk) {
    const _Float16* As = lds + buf * STAGE_HALVES;
    const _Float16* Bs = As + BM * LDS_STRIDE;
    h8_t af[4], bf[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      af[t] = *reinterpret_cast<const h8_t*>(As + (wm * 128 + t * 32 + li) * LDS_STRIDE + kk * 16 + kq * 8);
      bf[t] = *reinterpret_cast<const h8_t*>(Bs + (wn * 128 + t * 32 + li) * LDS_STRIDE + kk * 16 + kq * 8);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
  };

  // ---- prologue: stage k-step 0 into buffer 0
  load_global(0);
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) store_a(0, i);
#pragma unroll
  for (int g = 0; g < GPK; ++g) store_b_group(0, g);
  __syncthreads();

  for (int ks = 0; ks < p.ksteps; ++ks) {
    const int cur = ks & 1, nxt = cur ^ 1;
    const bool more = ks + 1 < p.ksteps;
    if (more) load_global(ks + 1);
    // four k-slabs of MFMAs; the staging of the next step is spread between them
    mfma_slab(cur, 0);
    if (more) {
#pragma unroll
      for (int i = 0; i < A_LOADS / 2; ++i) store_a(nxt, i);
    }
    mfma_slab(cur, 1);
    if (more) {
#pragma unroll
      for (int i = A_LOADS / 2; i < A_LOADS; ++i) store_a(nxt, i);
    }
    mfma_slab(cur, 2);
    if (more) {
#pragma unroll
      for (int g = 0; g < GPK / 2; ++g) store_b_group(nxt, g);
    }
    mfma_slab(cur, 3);
    if (more) {
#pragma unroll
      for (int g = GPK / 2; g < GPK; ++g) store_b_group(nxt, g);
    }
    __syncthreads();
  }

  // ---- epilogue: D[i][j] of a 32x32 tile: lane holds column j = lane % 32, rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + wn * 128 + j * 32 + li;
    if (n >= p.N) continue;
    const float b = p.bias ? (float)p.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 128 + i * 32 + (r >> 2) * 8 + kq * 4 + (r & 3);
        if (m < p.M) p.C[(int64_t)m * p.ldc + n] = (_Float16)(acc[i][j][r] + b);
      }
    }
  }
}

int log2i(int v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

template <int BITS, bool HAS_ZP, bool SMALL_BS>
hipError_t launch(const Gemm256Params& p, hipStream_t s) {
  const size_t smem = (size_t)2 * STAGE_HALVES * sizeof(_Float16);  // 147456 bytes
  static bool configured = false;  // per instantiation; the attribute is sticky for the function
  auto kernel = mnb_gemm256_kernel<BITS, HAS_ZP, SMALL_BS>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    configured = true;
  }
  dim3 grid((unsigned)((p.N + BN - 1) / BN), (unsigned)((p.M + BM - 1) / BM)), blk(THREADS);
  kernel<<<grid, blk, smem, s>>>(p);
  return hipGetLastError();
}

}  // namespace

hipError_t mnb_launch_gemm256(const MnbGemmArgs& a, hipStream_t s) {
  Gemm256Params p{};
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
  p.bs_shift = log2i(a.L.bs);
  p.ksteps = (int)((a.L.K + BK - 1) / BK);
  if (a.L.bits == 4) {
    if (a.L.bs == 16) return a.L.has_zp ? launch<4, true, true>(p, s) : launch<4, false, true>(p, s);
    return a.L.has_zp ? launch<4, true, false>(p, s) : launch<4, false, false>(p, s);
  }
  return a.L.has_zp ? launch<8, true, false>(p, s) : launch<8, false, false>(p, s);
}
