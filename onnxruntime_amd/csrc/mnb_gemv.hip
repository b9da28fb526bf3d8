// Dequantising GEMV for M <= 16 and the shape-agnostic fallback kernel.
//
// Device counterpart of the reference's decode hot loop (MlasQ4GemmKernelBlkLen32PlusAvx512f,
// onnxruntime/core/mlas/lib/sqnbitgemm_kernel_avx_common_fp32.h:288-639): unpack -> (q - zp) -> dot with A -> times
// scale -> accumulate in fp32 -> (+ bias) -> narrow once.
//
// Mapping: the 64 lanes of a wavefront own 64 neighbouring output columns and read one 16-byte vector each per
// k-group (1 KiB contiguous per wavefront in the k-group-major layout).  The activations of a k-group are the same
// for every lane: their address is wave-uniform, so they travel through the scalar cache into SGPRs and feed
// v_dot2_f32_f16 / v_fma_f32 as scalar operands -- no LDS, no VGPRs, no cross-lane reduction.
// K is split over the wavefronts of a workgroup and reduced through LDS in a fixed order.  It is NOT split over
// workgroups: device-scope release/acquire between workgroups writes back and invalidates the per-XCD L2 and cost
// 20x the kernel itself when measured.  fp16 models use the matrix-core kernel in mnb_skinny.hip instead; this
// kernel serves fp32 models.
#include <cstdio>
#include <cstdlib>

#include "mnb_device.cuh"
#include "mnb_internal.h"

struct GemvParams {
  const void* A;
  const uint4* W;
  const uint8_t* meta;
  const void* bias;
  void* C;
  int64_t lda, ldc;
  int M, N, K;
  int64_t Npad;
  int bs, bs_shift;
  int KG;      // k-groups that hold elements below K
};

template <typename T>
__device__ __forceinline__ float mnb_to_float(T v) {
  return (float)v;
}

// ---- one k-group of one column against MT rows of A -----------------------------------------------------------
// a_grp points at A[0][g*GK] and is wave-uniform.
template <typename T, int BITS, bool HAS_ZP, bool SMALL_BS, int MT>
__device__ __forceinline__ void mnb_gemv_group(const uint4& wv, const uint8_t* __restrict__ meta, int64_t midx,
                                               int64_t Npad, const T* __restrict__ a_grp, int64_t lda, int M,
                                               float* acc) {
  constexpr int GK = 128 / BITS;
  constexpr int NBLK = SMALL_BS ? 2 : 1;   // quantisation blocks inside one group
  constexpr int WORDS = 4 / NBLK;          // 32-bit words per block
  const uint32_t wd[4] = {wv.x, wv.y, wv.z, wv.w};
  if constexpr (sizeof(T) == 2) {
    constexpr int PPW = (BITS == 4) ? 4 : 2;  // half pairs per word
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      _Float16 s;
      ZpH z;
      mnb_load_meta_h<HAS_ZP, BITS>(meta, midx + b * Npad, s, z);
      h2_t d[WORDS * PPW];
#pragma unroll
      for (int i = 0; i < WORDS; ++i) {
        if constexpr (BITS == 4)
          mnb_unpack4_h(wd[b * WORDS + i], z, &d[i * PPW]);
        else
          mnb_unpack8_h(wd[b * WORDS + i], z, &d[i * PPW]);
      }
      const float sf = (float)s;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const h2_t* a2 = reinterpret_cast<const h2_t*>(a_grp + (m < M ? m : M - 1) * lda) + b * WORDS * PPW;
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < WORDS * PPW; ++j) part = __builtin_amdgcn_fdot2(d[j], a2[j], part, false);
        acc[m] = __builtin_fmaf(part, sf, acc[m]);
      }
    }
  } else {
    constexpr int EPW = (BITS == 4) ? 8 : 4;  // elements per word
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      float s, zp;
      mnb_load_meta_f<HAS_ZP, BITS>(meta, midx + b * Npad, s, zp);
      float part[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) part[m] = 0.f;
#pragma unroll
      for (int i = 0; i < WORDS; ++i) {
        float d[EPW];
        if constexpr (BITS == 4)
          mnb_unpack4_f(wd[b * WORDS + i], zp, d);
        else
          mnb_unpack8_f(wd[b * WORDS + i], zp, d);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const T* a = a_grp + (m < M ? m : M - 1) * lda + (b * WORDS + i) * EPW;
#pragma unroll
          for (int j = 0; j < EPW; ++j) part[m] = __builtin_fmaf(a[j], d[j], part[m]);
        }
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[m] = __builtin_fmaf(part[m], s, acc[m]);
    }
  }
}

// Requirements checked by the host: K % GK == 0, A 16-byte aligned with a 16-byte aligned row pitch.
// Rows [M, MT) of the register tile re-read row M-1 and are never stored.
template <typename T, int BITS, bool HAS_ZP, bool SMALL_BS, int MT, int NW, int U>
__global__ void __launch_bounds__(NW * 64) mnb_gemv_kernel(GemvParams p) {
  constexpr int GK = 128 / BITS;
  __shared__ float red[NW * MT * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t n = (int64_t)blockIdx.x * 64 + lane;  // < Npad always
  const int kg0 = 0;
  const int kg1 = p.KG;
  const T* __restrict__ A = reinterpret_cast<const T*>(p.A);
  const uint4* __restrict__ W = p.W;
  const uint8_t* __restrict__ meta = p.meta;

  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;

  for (int c = kg0 + wave * U; c < kg1; c += NW * U) {
    uint4 w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = c + u;
      w[u] = (g < kg1) ? W[(int64_t)g * p.Npad + n] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = c + u;
      if (g < kg1) {
        const int64_t kb = SMALL_BS ? (int64_t)g * 2 : (((int64_t)g * GK) >> p.bs_shift);
        mnb_gemv_group<T, BITS, HAS_ZP, SMALL_BS, MT>(w[u], meta, kb * p.Npad + mnb_meta_col(n), p.Npad, A + (int64_t)g * GK, p.lda,
                                                      p.M, acc);
      }
    }
  }

  // ---- reduce over the wavefronts of the workgroup
  if constexpr (NW > 1) {
#pragma unroll
    for (int m = 0; m < MT; ++m) red[(wave * MT + m) * 64 + lane] = acc[m];
    __syncthreads();
  }
  const int64_t bx = blockIdx.x;
  auto finish = [&](int m, int l, float sum) {
    const int64_t nn = bx * 64 + l;
    if (m < p.M && nn < p.N) {
      if (p.bias) sum += mnb_to_float(reinterpret_cast<const T*>(p.bias)[nn]);
      reinterpret_cast<T*>(p.C)[(int64_t)m * p.ldc + nn] = (T)sum;
    }
  };
  for (int i = threadIdx.x; i < MT * 64; i += NW * 64) {
    const int m = i >> 6, l = i & 63;
    float sum = 0.f;
    if constexpr (NW > 1) {
#pragma unroll
      for (int w2 = 0; w2 < NW; ++w2) sum += red[(w2 * MT + m) * 64 + l];
    } else {
      sum = acc[m];
    }
    finish(m, l, sum);
  }
}

// ------------------------------------------------------------------------------------------------ generic
// Any M, N, K, lda, alignment.  One wavefront per 64 columns x MT rows; sequential k, fp32 accumulation of
// a * (d * scale) exactly as the reference's scalar definition.  Slow; used when the fast kernels' alignment
// requirements do not hold, and for fp32 models with M > 16.
template <typename T, int BITS, bool HAS_ZP, bool SMALL_BS, int MT>
__global__ void __launch_bounds__(64) mnb_gemm_generic_kernel(GemvParams p) {
  constexpr int GK = 128 / BITS;
  constexpr int NBLK = SMALL_BS ? 2 : 1;
  constexpr int WORDS = 4 / NBLK;
  constexpr int EPW = GK / 4;  // elements per word
  const int lane = threadIdx.x;
  const int64_t n = (int64_t)blockIdx.x * 64 + lane;
  const int m0 = blockIdx.y * MT;
  const T* A = reinterpret_cast<const T*>(p.A);
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;
  for (int g = 0; g < p.KG; ++g) {
    const uint4 v = p.W[(int64_t)g * p.Npad + n];
    const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
    const int64_t kb = SMALL_BS ? (int64_t)g * 2 : (((int64_t)g * GK) >> p.bs_shift);
    float wv[GK];
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      const int64_t midx = (kb + b) * p.Npad + mnb_meta_col(n);
      if constexpr (sizeof(T) == 2) {
        // exact integers times the widened scale: the fp32 product is exact, as on the reference's x64 path
        _Float16 s;
        ZpH z;
        mnb_load_meta_h<HAS_ZP, BITS>(p.meta, midx, s, z);
        const float sf = (float)s;
#pragma unroll
        for (int i = 0; i < WORDS; ++i) {
          const int wi = b * WORDS + i;
          h2_t d[EPW / 2];
          if constexpr (BITS == 4)
            mnb_unpack4_h(wd[wi], z, d);
          else
            mnb_unpack8_h(wd[wi], z, d);
#pragma unroll
          for (int j = 0; j < EPW / 2; ++j) {
            wv[wi * EPW + 2 * j] = (float)d[j].x * sf;
            wv[wi * EPW + 2 * j + 1] = (float)d[j].y * sf;
          }
        }
      } else {
        float s, zp;
        mnb_load_meta_f<HAS_ZP, BITS>(p.meta, midx, s, zp);
#pragma unroll
        for (int i = 0; i < WORDS; ++i) {
          const int wi = b * WORDS + i;
          float d[EPW];
          if constexpr (BITS == 4)
            mnb_unpack4_f(wd[wi], zp, d);
          else
            mnb_unpack8_f(wd[wi], zp, d);
#pragma unroll
          for (int j = 0; j < EPW; ++j) wv[wi * EPW + j] = d[j] * s;
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m0 + m < p.M) {
        const T* a = A + (int64_t)(m0 + m) * p.lda + (int64_t)g * GK;
#pragma unroll
        for (int j = 0; j < GK; ++j) {
          const int64_t k = (int64_t)g * GK + j;
          const float av = (k < p.K) ? (float)a[j] : 0.f;
          acc[m] = __builtin_fmaf(av, wv[j], acc[m]);
        }
      }
    }
  }
  if (n >= p.N) return;
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    if (m0 + m < p.M) {
      float sum = acc[m];
      if (p.bias) sum += mnb_to_float(reinterpret_cast<const T*>(p.bias)[n]);
      reinterpret_cast<T*>(p.C)[(int64_t)(m0 + m) * p.ldc + n] = (T)sum;
    }
  }
}

// ------------------------------------------------------------------------------------------------ host side
namespace {

int gemv_mt(int64_t M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16; }

constexpr int kGemvU = 4;

// wavefronts per workgroup: enough that every wavefront still walks a few k-groups
int gemv_nw(const MnbLayout& L) {
  const int64_t KG = (L.K + L.group_k - 1) / L.group_k;
  return KG >= 64 ? 16 : 4;
}

bool gemv_fast_ok(const MnbGemmArgs& a) {
  const int es = a.L.dtype == kMnbDtypeFloat16 ? 2 : 4;
  return a.L.K % a.L.group_k == 0 && reinterpret_cast<uintptr_t>(a.A) % 16 == 0 && (a.lda * es) % 16 == 0;
}

template <typename T, int BITS, bool HAS_ZP, bool SMALL_BS, int MT, int NW>
hipError_t launch_gemv_nw(const GemvParams& p, int64_t col_groups, hipStream_t s) {
  dim3 grid((unsigned)col_groups), blk(NW * 64);
  mnb_gemv_kernel<T, BITS, HAS_ZP, SMALL_BS, MT, NW, kGemvU><<<grid, blk, 0, s>>>(p);
  return hipGetLastError();
}

template <typename T, int BITS, bool HAS_ZP, bool SMALL_BS, int MT>
hipError_t launch_gemv_mt(const GemvParams& p, int nw, int64_t col_groups, hipStream_t s) {
  if (nw == 16) return launch_gemv_nw<T, BITS, HAS_ZP, SMALL_BS, MT, 16>(p, col_groups, s);
  return launch_gemv_nw<T, BITS, HAS_ZP, SMALL_BS, MT, 4>(p, col_groups, s);
}

template <typename T, int BITS, bool HAS_ZP, bool SMALL_BS>
hipError_t launch_gemv_sb(const GemvParams& p, int mt, int nw, int64_t col_groups, hipStream_t s) {
  switch (mt) {
    case 1: return launch_gemv_mt<T, BITS, HAS_ZP, SMALL_BS, 1>(p, nw, col_groups, s);
    case 2: return launch_gemv_mt<T, BITS, HAS_ZP, SMALL_BS, 2>(p, nw, col_groups, s);
    case 4: return launch_gemv_mt<T, BITS, HAS_ZP, SMALL_BS, 4>(p, nw, col_groups, s);
    case 8: return launch_gemv_mt<T, BITS, HAS_ZP, SMALL_BS, 8>(p, nw, col_groups, s);
    default: return launch_gemv_mt<T, BITS, HAS_ZP, SMALL_BS, 16>(p, nw, col_groups, s);
  }
}

template <typename T, int BITS, bool HAS_ZP>
hipError_t launch_gemv_zp(const GemvParams& p, int mt, int nw, int64_t col_groups, hipStream_t s) {
  if constexpr (BITS == 4) {
    if (p.bs == 16) return launch_gemv_sb<T, BITS, HAS_ZP, true>(p, mt, nw, col_groups, s);
  }
  return launch_gemv_sb<T, BITS, HAS_ZP, false>(p, mt, nw, col_groups, s);
}

template <typename T, int BITS, bool HAS_ZP>
hipError_t launch_generic_zp(const GemvParams& p, hipStream_t s) {
  constexpr int MT = 4;
  dim3 grid((unsigned)((p.N + 63) / 64), (unsigned)((p.M + MT - 1) / MT)), blk(64);
  if constexpr (BITS == 4) {
    if (p.bs == 16) {
      mnb_gemm_generic_kernel<T, BITS, HAS_ZP, true, MT><<<grid, blk, 0, s>>>(p);
      return hipGetLastError();
    }
  }
  mnb_gemm_generic_kernel<T, BITS, HAS_ZP, false, MT><<<grid, blk, 0, s>>>(p);
  return hipGetLastError();
}

int log2i(int v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

GemvParams make_params(const MnbGemmArgs& a) {
  GemvParams p{};
  p.A = a.A;
  p.W = reinterpret_cast<const uint4*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + a.L.meta_off;
  p.bias = a.bias;
  p.C = a.C;
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.M = (int)a.M;
  p.N = (int)a.L.N;
  p.K = (int)a.L.K;
  p.Npad = a.L.Npad;
  p.bs = a.L.bs;
  p.bs_shift = log2i(a.L.bs);
  p.KG = (int)((a.L.K + a.L.group_k - 1) / a.L.group_k);
  return p;
}

}  // namespace

#define MNB_DISPATCH(FN, ...)                                                                      \
  (a.L.dtype == kMnbDtypeFloat16                                                                    \
       ? (a.L.bits == 4 ? (a.L.has_zp ? FN<_Float16, 4, true>(__VA_ARGS__) : FN<_Float16, 4, false>(__VA_ARGS__)) \
                        : (a.L.has_zp ? FN<_Float16, 8, true>(__VA_ARGS__) : FN<_Float16, 8, false>(__VA_ARGS__))) \
       : (a.L.bits == 4 ? (a.L.has_zp ? FN<float, 4, true>(__VA_ARGS__) : FN<float, 4, false>(__VA_ARGS__))       \
                        : (a.L.has_zp ? FN<float, 8, true>(__VA_ARGS__) : FN<float, 8, false>(__VA_ARGS__))))

bool mnb_gemv_applicable(const MnbGemmArgs& a) {
  return a.L.dtype == kMnbDtypeFloat && a.M >= 1 && a.M <= 16 && gemv_fast_ok(a);
}

hipError_t mnb_launch_gemv(const MnbGemmArgs& a, hipStream_t s) {
  GemvParams p = make_params(a);
  const int64_t col_groups = (a.L.N + 63) / 64;
  const int mt = gemv_mt(a.M), nw = gemv_nw(a.L);
  if (a.L.bits == 4)
    return a.L.has_zp ? launch_gemv_zp<float, 4, true>(p, mt, nw, col_groups, s)
                      : launch_gemv_zp<float, 4, false>(p, mt, nw, col_groups, s);
  return a.L.has_zp ? launch_gemv_zp<float, 8, true>(p, mt, nw, col_groups, s)
                    : launch_gemv_zp<float, 8, false>(p, mt, nw, col_groups, s);
}

hipError_t mnb_launch_gemm_generic(const MnbGemmArgs& a, hipStream_t s) {
  GemvParams p = make_params(a);
  return MNB_DISPATCH(launch_generic_zp, p, s);
}
