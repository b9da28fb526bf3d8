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

#include "mnb_device.hip.h"
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

// What a wavefront needs to issue its first loads comes as leading scalar kernel arguments, which the build asks the
// compiler to have preloaded into SGPRs at wavefront start (no scalar load in front of the first weight load); the
// parameter block carries the rest and is fetched where it is used.
#define MNB_GEMV_HOT_PARAMS                                                                                    \
  const uint4 *hot_W, int64_t hot_Npad, const void *hot_A, int64_t hot_lda, const uint8_t *hot_meta, int hot_M, \
      int hot_KG, int hot_bs_shift
#define MNB_GEMV_HOT_ARGS(p) (p).W, (p).Npad, (p).A, (p).lda, (p).meta, (p).M, (p).KG, (p).bs_shift
#define MNB_GEMV_HOT_NAMES hot_W, hot_Npad, hot_A, hot_lda, hot_meta, hot_M, hot_KG, hot_bs_shift

__device__ __forceinline__ GemvParams with_hot_params(GemvParams p, MNB_GEMV_HOT_PARAMS) {
  p.W = hot_W;
  p.Npad = hot_Npad;
  p.A = hot_A;
  p.lda = hot_lda;
  p.meta = hot_meta;
  p.M = hot_M;
  p.KG = hot_KG;
  p.bs_shift = hot_bs_shift;
  return p;
}

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
__global__ void __launch_bounds__(NW * 64) mnb_gemv_kernel(MNB_GEMV_HOT_PARAMS, GemvParams rest) {
  const GemvParams p = with_hot_params(rest, MNB_GEMV_HOT_NAMES);
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

// ------------------------------------------------------------------------------------------------ fp32, few rows
// fp32 models with M <= 4.  The kernel above gives every workgroup 64 columns, i.e. N / 64 workgroups: a K = N = 4096
// projection occupies a quarter of the chip.  Here a workgroup owns 16 columns: lane (j = lane % 16, kq = lane / 16)
// takes k-group 4c + kq of chunk c for column j, so a wavefront still reads four 256-byte runs of the packed weights
// per load.  The activations are no longer wave-uniform; they are staged once per workgroup in LDS (fp32, one
// padded row of 36 floats per k-group of 32: the four kq segments of a ds_read_b128 hit different banks) and read as
// 16-byte broadcasts.  Arithmetic per weight is that of the kernel above: float(q) - zp, fused multiply-add with the
// activation, the block sum times the scale.  The four kq partial sums meet through two cross-lane exchanges, the
// wavefronts (K split) through LDS in a fixed order.
constexpr int kG16Pad = 4;         // floats of padding per staged k-group
constexpr int kG16PhaseK = 2048;   // k staged at a time (x MT rows x 4 B <= 36 KiB)

template <int BITS, bool HAS_ZP, bool SMALL_BS, int MT, int NW>
__global__ void __launch_bounds__(NW * 64) mnb_gemv16_kernel(MNB_GEMV_HOT_PARAMS, GemvParams rest) {
  const GemvParams p = with_hot_params(rest, MNB_GEMV_HOT_NAMES);
  constexpr int GK = 128 / BITS;                // k per 16-byte vector
  constexpr int GS = GK + kG16Pad;              // staged floats per k-group
  constexpr int PH_GROUPS = kG16PhaseK / GK;    // k-groups per phase
  constexpr int NBLK = SMALL_BS ? 2 : 1;
  constexpr int WORDS = 4 / NBLK;
  constexpr int EPW = (BITS == 4) ? 8 : 4;
  __shared__ __align__(16) float As[MT * PH_GROUPS * GS];
  __shared__ float red[NW * MT * 16];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, kq = lane >> 4;
  const int64_t n = (int64_t)blockIdx.x * 16 + j;  // < Npad always
  const float* __restrict__ A = reinterpret_cast<const float*>(p.A);
  const int64_t mcol = mnb_meta_col(n);

  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;

  for (int g0 = 0; g0 < p.KG; g0 += PH_GROUPS) {
    const int g1 = g0 + PH_GROUPS < p.KG ? g0 + PH_GROUPS : p.KG;
    const int groups = g1 - g0;
    // chunks of 4 k-groups; wavefront w takes chunks w, w + NW, ...; two vectors in flight per lane.  The first
    // weight loads go out before the activations are staged, so the two latencies overlap.
    const int chunks = (groups + 3) / 4;
    int c = wave;
    uint4 w0 = make_uint4(0, 0, 0, 0), w1 = w0;
    auto gl = [&](int cc) { return g0 + cc * 4 + kq; };
    if (c < chunks && gl(c) < g1) w0 = p.W[(int64_t)gl(c) * p.Npad + n];
    if (c + NW < chunks && gl(c + NW) < g1) w1 = p.W[(int64_t)gl(c + NW) * p.Npad + n];
    __syncthreads();  // the previous phase is no longer read
    for (int i = threadIdx.x; i < MT * groups * (GK / 4); i += NW * 64) {
      const int q4 = i % (GK / 4), g = (i / (GK / 4)) % groups, m = i / ((GK / 4) * groups);
      const int mm = m < p.M ? m : p.M - 1;  // rows >= M repeat the last row and are never stored
      const float4 v = *reinterpret_cast<const float4*>(A + (int64_t)mm * p.lda + (int64_t)(g0 + g) * GK + q4 * 4);
      *reinterpret_cast<float4*>(&As[(m * PH_GROUPS + g) * GS + q4 * 4]) = v;
    }
    __syncthreads();
    for (; c < chunks; c += NW) {
      const uint4 wv = w0;
      w0 = w1;
      if (c + 2 * NW < chunks && gl(c + 2 * NW) < g1) w1 = p.W[(int64_t)gl(c + 2 * NW) * p.Npad + n];
      const int g = gl(c);
      if (g >= g1) continue;  // ragged last chunk of the phase
      const uint32_t wd[4] = {wv.x, wv.y, wv.z, wv.w};
      const int64_t kb = SMALL_BS ? (int64_t)g * 2 : (((int64_t)g * GK) >> p.bs_shift);
      const float* a_grp = &As[(g - g0) * GS];
#pragma unroll
      for (int b = 0; b < NBLK; ++b) {
        float sc, zp;
        mnb_load_meta_f<HAS_ZP, BITS>(p.meta, (kb + b) * p.Npad + mcol, sc, zp);
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
            const float* a = a_grp + m * PH_GROUPS * GS + (b * WORDS + i) * EPW;
#pragma unroll
            for (int e4 = 0; e4 < EPW / 4; ++e4) {
              const float4 av = *reinterpret_cast<const float4*>(a + e4 * 4);
              part[m] = __builtin_fmaf(av.x, d[e4 * 4 + 0], part[m]);
              part[m] = __builtin_fmaf(av.y, d[e4 * 4 + 1], part[m]);
              part[m] = __builtin_fmaf(av.z, d[e4 * 4 + 2], part[m]);
              part[m] = __builtin_fmaf(av.w, d[e4 * 4 + 3], part[m]);
            }
          }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = __builtin_fmaf(part[m], sc, acc[m]);
      }
    }
  }
  // the four kq partial sums of a column, then the wavefronts
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    acc[m] += __shfl_xor(acc[m], 16, 64);
    acc[m] += __shfl_xor(acc[m], 32, 64);
  }
  if (kq == 0) {
#pragma unroll
    for (int m = 0; m < MT; ++m) red[(wave * MT + m) * 16 + j] = acc[m];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < MT * 16; i += NW * 64) {
    const int m = i >> 4, l = i & 15;
    const int64_t nn = (int64_t)blockIdx.x * 16 + l;
    if (m >= p.M || nn >= p.N) continue;
    float sum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) sum += red[(w2 * MT + m) * 16 + l];
    if (p.bias) sum += reinterpret_cast<const float*>(p.bias)[nn];
    reinterpret_cast<float*>(p.C)[(int64_t)m * p.ldc + nn] = sum;
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

int gemv_mt(int64_t M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : 8; }

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
  mnb_gemv_kernel<T, BITS, HAS_ZP, SMALL_BS, MT, NW, kGemvU><<<grid, blk, 0, s>>>(MNB_GEMV_HOT_ARGS(p), p);
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
    default: return launch_gemv_mt<T, BITS, HAS_ZP, SMALL_BS, 8>(p, nw, col_groups, s);
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

template <int BITS, bool HAS_ZP, bool SMALL_BS, int MT>
hipError_t launch_gemv16_nw(const GemvParams& p, hipStream_t s) {
  dim3 grid((unsigned)((p.N + 15) / 16));
  const int chunks = (p.KG + 3) / 4;
  // K split over 4, 8 or 16 wavefronts; sixteen while the grid has at most two workgroups per compute unit (measured:
  // N = K = 4096 M = 1/2/4: 7.1 -> 6.8, 8.5 -> 7.6, 11.3 -> 9.6 us; K = 14336: 20.4 -> 16.3 us; N = 11008: 11.1 -> 12.0)
  int nw = chunks >= 32 ? (grid.x <= 2u * (unsigned)mnb_device_info().cus ? 16 : 8) : 4;
  if (const char* e = mnb_tuning_env("MNB_GEMV16_NW")) nw = atoi(e);
  if (nw == 16) {
    mnb_gemv16_kernel<BITS, HAS_ZP, SMALL_BS, MT, 16><<<grid, dim3(1024), 0, s>>>(MNB_GEMV_HOT_ARGS(p), p);
  } else if (nw == 8) {
    mnb_gemv16_kernel<BITS, HAS_ZP, SMALL_BS, MT, 8><<<grid, dim3(512), 0, s>>>(MNB_GEMV_HOT_ARGS(p), p);
  } else {
    mnb_gemv16_kernel<BITS, HAS_ZP, SMALL_BS, MT, 4><<<grid, dim3(256), 0, s>>>(MNB_GEMV_HOT_ARGS(p), p);
  }
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP>
hipError_t launch_gemv16(const GemvParams& p, hipStream_t s) {
  const bool small = (BITS == 4) && p.bs == 16;
#define MNB_G16(MT_)                                                                         \
  return small ? launch_gemv16_nw<BITS, HAS_ZP, (BITS == 4), MT_>(p, s)                      \
               : launch_gemv16_nw<BITS, HAS_ZP, false, MT_>(p, s)
  if (p.M <= 1) { MNB_G16(1); }
  if (p.M <= 2) { MNB_G16(2); }
  MNB_G16(4);
#undef MNB_G16
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
  p.bs_shift = mnb_log2i(a.L.bs);
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
  // few rows and too few 64-column slabs to fill the chip: 16-column workgroups
  if (a.M <= 4 && col_groups < 192) {
    if (a.L.bits == 4) return a.L.has_zp ? launch_gemv16<4, true>(p, s) : launch_gemv16<4, false>(p, s);
    return a.L.has_zp ? launch_gemv16<8, true>(p, s) : launch_gemv16<8, false>(p, s);
  }
  // Rows go eight at a time: the rows of A are wave-uniform and travel through scalar registers, and a register tile of
  // sixteen rows needs more of them than a wavefront has (measured: one pass of 16 rows 144 us where two passes of 8
  // take 46 us, K = N = 4096, 4-bit).
  const int nw = gemv_nw(a.L);
  for (int64_t m0 = 0; m0 < a.M; m0 += 8) {
    const int64_t rows = a.M - m0 < 8 ? a.M - m0 : 8;
    p.A = reinterpret_cast<const float*>(a.A) + m0 * a.lda;
    p.C = reinterpret_cast<float*>(a.C) + m0 * a.ldc;
    p.M = (int)rows;
    const int mt = gemv_mt(rows);
    hipError_t e;
    if (a.L.bits == 4)
      e = a.L.has_zp ? launch_gemv_zp<float, 4, true>(p, mt, nw, col_groups, s)
                     : launch_gemv_zp<float, 4, false>(p, mt, nw, col_groups, s);
    else
      e = a.L.has_zp ? launch_gemv_zp<float, 8, true>(p, mt, nw, col_groups, s)
                     : launch_gemv_zp<float, 8, false>(p, mt, nw, col_groups, s);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t mnb_launch_gemm_generic(const MnbGemmArgs& a, hipStream_t s) {
  GemvParams p = make_params(a);
  return MNB_DISPATCH(launch_generic_zp, p, s);
}
