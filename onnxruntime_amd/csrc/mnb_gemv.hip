// Dequantising GEMV for M <= 16 and the shape-agnostic fallback kernel.
//
// Device counterpart of the reference's decode hot loop (MlasQ4GemmKernelBlkLen32PlusAvx512f,
// onnxruntime/core/mlas/lib/sqnbitgemm_kernel_avx_common_fp32.h:288-639): unpack -> (q - zp) -> dot with A -> times
// scale -> accumulate in fp32 -> (+ bias) -> narrow once.
//
// Mapping: the 64 lanes of a wavefront own 64 neighbouring output columns and read one 16-byte vector each per
// k-group (1 KiB contiguous per wavefront, k-group-major layout).  The activations of a k-group are the same for
// every lane, so they are staged once per workgroup in LDS and read with wave-uniform (broadcast) addresses.
// K is split over the wavefronts of a workgroup (reduced through LDS) and optionally over workgroups (partial sums
// in a workspace, reduced by a second tiny kernel in a fixed order, so results are run-to-run deterministic).
#include "mnb_device.cuh"
#include "mnb_internal.h"

struct GemvParams {
  const void* A;
  const uint4* W;
  const uint8_t* meta;
  const void* bias;
  void* C;
  float* partial;
  int64_t lda, ldc;
  int M, N, K;
  int64_t Npad;
  int bs;
  int KG;      // k-groups in the packed matrix
  int gpb;     // k-groups per workgroup (blockIdx.y slice)
  int ksplit;  // gridDim.y
};

template <typename T>
__device__ __forceinline__ float mnb_to_float(T v) {
  return (float)v;
}

// sum_j a[j] * d[j] over one k-group for one row, d exact integers.  fp16: v_dot2_f32_f16 with fp32 accumulation.
template <int BITS>
__device__ __forceinline__ float mnb_dot_group_h(const h2_t* d, const _Float16* a_lds, int first_pair, int npairs) {
  float part = 0.f;
  const h2_t* a2 = reinterpret_cast<const h2_t*>(a_lds);
#pragma unroll
  for (int j = 0; j < npairs; ++j) part = __builtin_amdgcn_fdot2(d[first_pair + j], a2[first_pair + j], part, false);
  return part;
}

template <typename T, int BITS, bool HAS_ZP, int MT, int NW>
__global__ void __launch_bounds__(NW * 64) mnb_gemv_kernel(GemvParams p) {
  constexpr int GK = 128 / BITS;   // k per 16-byte group
  constexpr int U = 4;             // groups in flight per wavefront
  constexpr int CHUNK = NW * U;    // groups per workgroup iteration
  extern __shared__ __align__(16) unsigned char smem[];
  T* As = reinterpret_cast<T*>(smem);                                            // [MT][CHUNK*GK]
  float* red = reinterpret_cast<float*>(smem + sizeof(T) * MT * CHUNK * GK);      // [NW][MT][64]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t n = (int64_t)blockIdx.x * 64 + lane;  // < Npad always
  const int kg0 = blockIdx.y * p.gpb;
  const int kg1 = min(kg0 + p.gpb, p.KG);
  const T* A = reinterpret_cast<const T*>(p.A);

  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;

  for (int c0 = kg0; c0 < kg1; c0 += CHUNK) {
    // ---- issue this wavefront's weight loads first (they are the long-latency part)
    uint4 w[U];
    const int gbase = c0 + wave * U;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = gbase + u;
      w[u] = (g < kg1) ? p.W[(int64_t)g * p.Npad + n] : make_uint4(0, 0, 0, 0);
    }
    // ---- stage the activations of the chunk (zero beyond M and K)
    __syncthreads();  // previous chunk fully consumed
    const int kbase = c0 * GK;
    for (int i = threadIdx.x; i < MT * CHUNK * GK; i += NW * 64) {
      const int m = i / (CHUNK * GK);
      const int kk = i % (CHUNK * GK);
      const int k = kbase + kk;
      As[i] = (m < p.M && k < p.K) ? A[(int64_t)m * p.lda + k] : (T)0;
    }
    __syncthreads();
    // ---- consume
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = gbase + u;
      if (g >= kg1) break;
      const T* a_grp = As + (wave * U + u) * GK;
      const uint32_t wd[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
      const int64_t k0 = (int64_t)g * GK;
      const int nblk = (p.bs < GK) ? GK / p.bs : 1;  // 2 only for 4-bit with block_size 16
      const int words = 4 / nblk;
      for (int b = 0; b < nblk; ++b) {
        const int64_t midx = ((k0 + b * p.bs) / p.bs) * p.Npad + n;
        if constexpr (sizeof(T) == 2) {
          _Float16 s;
          ZpH z;
          mnb_load_meta_h<HAS_ZP, BITS>(p.meta, midx, s, z);
          constexpr int PPW = (BITS == 4) ? 4 : 2;  // half pairs per word
          h2_t d[4 * PPW];
          for (int i = 0; i < words; ++i) {
            const int wi = b * words + i;
            if constexpr (BITS == 4)
              mnb_unpack4_h(wd[wi], z, &d[wi * PPW]);
            else
              mnb_unpack8_h(wd[wi], z, &d[wi * PPW]);
          }
          const float sf = (float)s;
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const float part = mnb_dot_group_h<BITS>(d, a_grp + m * CHUNK * GK, b * words * PPW, words * PPW);
            acc[m] = __builtin_fmaf(part, sf, acc[m]);
          }
        } else {
          float s, zp;
          mnb_load_meta_f<HAS_ZP, BITS>(p.meta, midx, s, zp);
          constexpr int EPW = (BITS == 4) ? 8 : 4;  // elements per word
          for (int i = 0; i < words; ++i) {
            const int wi = b * words + i;
            float d[EPW];
            if constexpr (BITS == 4)
              mnb_unpack4_f(wd[wi], zp, d);
            else
              mnb_unpack8_f(wd[wi], zp, d);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const T* a = a_grp + m * CHUNK * GK + wi * EPW;
              float part = 0.f;
#pragma unroll
              for (int j = 0; j < EPW; ++j) part = __builtin_fmaf(a[j], d[j], part);
              acc[m] = __builtin_fmaf(part, s, acc[m]);
            }
          }
        }
      }
    }
  }

  // ---- reduce over the wavefronts of the workgroup
  __syncthreads();
#pragma unroll
  for (int m = 0; m < MT; ++m) red[(wave * MT + m) * 64 + lane] = acc[m];
  __syncthreads();
  for (int i = threadIdx.x; i < MT * 64; i += NW * 64) {
    const int m = i >> 6, l = i & 63;
    float sum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) sum += red[(w2 * MT + m) * 64 + l];
    const int64_t nn = (int64_t)blockIdx.x * 64 + l;
    if (p.ksplit > 1) {
      p.partial[((int64_t)blockIdx.y * MT + m) * p.Npad + nn] = sum;
    } else if (m < p.M && nn < p.N) {
      if (p.bias) sum += mnb_to_float(reinterpret_cast<const T*>(p.bias)[nn]);
      reinterpret_cast<T*>(p.C)[(int64_t)m * p.ldc + nn] = (T)sum;
    }
  }
}

// Second pass of a split-K GEMV: fixed-order sum of the partials, bias, one narrowing.
template <typename T, int MT>
__global__ void __launch_bounds__(256) mnb_gemv_reduce_kernel(GemvParams p) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n = idx % p.Npad;
  const int m = (int)(idx / p.Npad);
  if (m >= p.M || n >= p.N) return;
  float sum = 0.f;
  for (int s = 0; s < p.ksplit; ++s) sum += p.partial[((int64_t)s * MT + m) * p.Npad + n];
  if (p.bias) sum += mnb_to_float(reinterpret_cast<const T*>(p.bias)[n]);
  reinterpret_cast<T*>(p.C)[(int64_t)m * p.ldc + n] = (T)sum;
}

// ------------------------------------------------------------------------------------------------ generic
// Any M, N, K, lda, alignment.  One wavefront per 64 columns x MT rows; sequential k, fp32 accumulation of
// a * (d * scale) exactly as the reference's scalar definition.  Slow; used when the fast kernels' alignment
// requirements do not hold, and for fp32 models with M > 16.
template <typename T, int BITS, bool HAS_ZP, int MT>
__global__ void __launch_bounds__(64) mnb_gemm_generic_kernel(GemvParams p) {
  constexpr int GK = 128 / BITS;
  const int lane = threadIdx.x;
  const int64_t n = (int64_t)blockIdx.x * 64 + lane;
  const int m0 = blockIdx.y * MT;
  const T* A = reinterpret_cast<const T*>(p.A);
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;
  const int kg_end = (p.K + GK - 1) / GK;
  for (int g = 0; g < kg_end; ++g) {
    const uint4 v = p.W[(int64_t)g * p.Npad + n];
    float wv[GK];
    if constexpr (sizeof(T) == 2) {
      // exact integers times the widened scale: the fp32 product is exact, as on the reference's x64 path
      const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
      const int nblk = (p.bs < GK) ? GK / p.bs : 1;
      const int words = 4 / nblk;
      for (int b = 0; b < nblk; ++b) {
        _Float16 s;
        ZpH z;
        mnb_load_meta_h<HAS_ZP, BITS>(p.meta, (((int64_t)g * GK + b * p.bs) / p.bs) * p.Npad + n, s, z);
        const float sf = (float)s;
        for (int i = 0; i < words; ++i) {
          const int wi = b * words + i;
          if constexpr (BITS == 4) {
            h2_t d[4];
            mnb_unpack4_h(wd[wi], z, d);
            for (int j = 0; j < 4; ++j) {
              wv[wi * 8 + 2 * j] = (float)d[j].x * sf;
              wv[wi * 8 + 2 * j + 1] = (float)d[j].y * sf;
            }
          } else {
            h2_t d[2];
            mnb_unpack8_h(wd[wi], z, d);
            for (int j = 0; j < 2; ++j) {
              wv[wi * 4 + 2 * j] = (float)d[j].x * sf;
              wv[wi * 4 + 2 * j + 1] = (float)d[j].y * sf;
            }
          }
        }
      }
    } else {
      mnb_dequant_group_f<BITS, HAS_ZP>(v, p.meta, g, n, p.Npad, p.bs, wv);
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (m0 + m >= p.M) break;
      const T* a = A + (int64_t)(m0 + m) * p.lda + (int64_t)g * GK;
      for (int j = 0; j < GK; ++j) {
        const int64_t k = (int64_t)g * GK + j;
        if (k < p.K) acc[m] = __builtin_fmaf((float)a[j], wv[j], acc[m]);
      }
    }
  }
  if (n >= p.N) return;
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    if (m0 + m >= p.M) break;
    float sum = acc[m];
    if (p.bias) sum += mnb_to_float(reinterpret_cast<const T*>(p.bias)[n]);
    reinterpret_cast<T*>(p.C)[(int64_t)(m0 + m) * p.ldc + n] = (T)sum;
  }
}

// ------------------------------------------------------------------------------------------------ host side
namespace {

constexpr int kGemvNW = 4;

struct GemvPlan {
  int mt;      // rows held per lane: 1, 2, 4, 8 or 16
  int gpb;     // k-groups per workgroup
  int ksplit;  // workgroups along k
};

int gemv_mt(int64_t M) { return M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16; }

GemvPlan gemv_plan(const MnbLayout& L, int64_t M, size_t workspace_bytes) {
  GemvPlan pl;
  pl.mt = gemv_mt(M);
  const int64_t col_groups = (L.N + 63) / 64;
  const int chunk = kGemvNW * 4;
  // aim for about four workgroups per compute unit
  int64_t want = (1024 + col_groups - 1) / col_groups;
  int64_t max_split = (L.KG + chunk - 1) / chunk;
  if (want > max_split) want = max_split;
  if (want < 1) want = 1;
  int64_t gpb = (L.KG + want - 1) / want;
  gpb = (gpb + chunk - 1) / chunk * chunk;
  int64_t ksplit = (L.KG + gpb - 1) / gpb;
  if (ksplit > 1 && (size_t)(ksplit * pl.mt * L.Npad * 4) > workspace_bytes) {
    ksplit = 1;
    gpb = L.KG;
  }
  pl.gpb = (int)gpb;
  pl.ksplit = (int)ksplit;
  return pl;
}

template <typename T, int BITS, bool HAS_ZP, int MT>
hipError_t launch_gemv_mt(const GemvParams& p, int64_t col_groups, hipStream_t s) {
  constexpr int GK = 128 / BITS;
  constexpr int CHUNK = kGemvNW * 4;
  const size_t smem = sizeof(T) * MT * CHUNK * GK + sizeof(float) * kGemvNW * MT * 64;
  dim3 grid((unsigned)col_groups, (unsigned)p.ksplit), blk(kGemvNW * 64);
  mnb_gemv_kernel<T, BITS, HAS_ZP, MT, kGemvNW><<<grid, blk, smem, s>>>(p);
  if (p.ksplit > 1) {
    const int64_t total = (int64_t)p.M * p.Npad;
    mnb_gemv_reduce_kernel<T, MT><<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s>>>(p);
  }
  return hipGetLastError();
}

template <typename T, int BITS, bool HAS_ZP>
hipError_t launch_gemv_zp(const GemvParams& p, int mt, int64_t col_groups, hipStream_t s) {
  switch (mt) {
    case 1: return launch_gemv_mt<T, BITS, HAS_ZP, 1>(p, col_groups, s);
    case 2: return launch_gemv_mt<T, BITS, HAS_ZP, 2>(p, col_groups, s);
    case 4: return launch_gemv_mt<T, BITS, HAS_ZP, 4>(p, col_groups, s);
    case 8: return launch_gemv_mt<T, BITS, HAS_ZP, 8>(p, col_groups, s);
    default: return launch_gemv_mt<T, BITS, HAS_ZP, 16>(p, col_groups, s);
  }
}

template <typename T, int BITS, bool HAS_ZP>
hipError_t launch_generic_zp(const GemvParams& p, hipStream_t s) {
  constexpr int MT = 4;
  dim3 grid((unsigned)((p.N + 63) / 64), (unsigned)((p.M + MT - 1) / MT)), blk(64);
  mnb_gemm_generic_kernel<T, BITS, HAS_ZP, MT><<<grid, blk, 0, s>>>(p);
  return hipGetLastError();
}

GemvParams make_params(const MnbGemmArgs& a) {
  GemvParams p{};
  p.A = a.A;
  p.W = reinterpret_cast<const uint4*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + a.L.meta_off;
  p.bias = a.bias;
  p.C = a.C;
  p.partial = reinterpret_cast<float*>(a.workspace);
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.M = (int)a.M;
  p.N = (int)a.L.N;
  p.K = (int)a.L.K;
  p.Npad = a.L.Npad;
  p.bs = a.L.bs;
  p.KG = (int)a.L.KG;
  p.gpb = (int)a.L.KG;
  p.ksplit = 1;
  return p;
}

}  // namespace

#define MNB_DISPATCH(FN, ...)                                                                      \
  (a.L.dtype == kMnbDtypeFloat16                                                                    \
       ? (a.L.bits == 4 ? (a.L.has_zp ? FN<_Float16, 4, true>(__VA_ARGS__) : FN<_Float16, 4, false>(__VA_ARGS__)) \
                        : (a.L.has_zp ? FN<_Float16, 8, true>(__VA_ARGS__) : FN<_Float16, 8, false>(__VA_ARGS__))) \
       : (a.L.bits == 4 ? (a.L.has_zp ? FN<float, 4, true>(__VA_ARGS__) : FN<float, 4, false>(__VA_ARGS__))       \
                        : (a.L.has_zp ? FN<float, 8, true>(__VA_ARGS__) : FN<float, 8, false>(__VA_ARGS__))))

size_t mnb_gemv_workspace_bytes(const MnbLayout& L, int64_t M) {
  if (M < 1 || M > 16) return 0;
  GemvPlan pl = gemv_plan(L, M, (size_t)-1);
  return pl.ksplit > 1 ? (size_t)pl.ksplit * pl.mt * L.Npad * 4 : 0;
}

hipError_t mnb_launch_gemv(const MnbGemmArgs& a, hipStream_t s) {
  GemvParams p = make_params(a);
  GemvPlan pl = gemv_plan(a.L, a.M, a.workspace ? a.workspace_bytes : 0);
  p.gpb = pl.gpb;
  p.ksplit = pl.ksplit;
  const int64_t col_groups = (a.L.N + 63) / 64;
  return MNB_DISPATCH(launch_gemv_zp, p, pl.mt, col_groups, s);
}

hipError_t mnb_launch_gemm_generic(const MnbGemmArgs& a, hipStream_t s) {
  GemvParams p = make_params(a);
  return MNB_DISPATCH(launch_generic_zp, p, s);
}
