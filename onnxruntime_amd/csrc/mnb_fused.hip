// Kernels around the operators that run several MatMulNBits projections behind one activation
// (MatMulNBitsMlp / MatMulNBitsQkv, onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3851-4090; the only kernels the
// reference ships for them are WebGPU shaders, contrib_ops/webgpu/quantization/matmul_nbits_mlp.cc:241-543 and
// matmul_nbits_qkv.cc):
//
//   * the optional prologue, SimplifiedLayerNormalization / SkipSimplifiedLayerNormalization of the activation
//     (onnxruntime/contrib_ops/cpu/skip_layer_norm.cc:44-97: x = input + skip, y = x / sqrt(mean(x^2) + eps) * scale,
//     fp32 arithmetic, one narrowing of each output);
//   * the finishing pass for the GEMM kernels that cannot write the operator's outputs themselves: they produce the
//     plain product over the packed columns, and this pass applies silu(gate) * up or splits Q, K and V.
#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

constexpr int kNormThreads = 512;

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < kNormThreads / 64; ++w) s += red[w];  // same order in every thread
  return s;
}

struct NormParams {
  const void* A;
  const void* skip;
  const void* scale;
  void* out;
  void* sum_out;
  int64_t lda, ld_skip, skip_rows, ld_sum;
  int M, K;
  float eps;
};

// fp16, rows addressable with 16-byte loads, K <= 8 * kNormThreads * VPT: one pass, the row stays in registers.
template <int VPT>
__global__ void __launch_bounds__(kNormThreads) mnb_rmsnorm_h_vec_kernel(NormParams p) {
  __shared__ float red[kNormThreads / 64];
  const int m = blockIdx.x;
  const _Float16* a = reinterpret_cast<const _Float16*>(p.A) + (int64_t)m * p.lda;
  const _Float16* sk = p.skip ? reinterpret_cast<const _Float16*>(p.skip) + (int64_t)(m % p.skip_rows) * p.ld_skip : nullptr;
  const _Float16* sc = reinterpret_cast<const _Float16*>(p.scale);
  _Float16* out = reinterpret_cast<_Float16*>(p.out) + (int64_t)m * p.K;
  _Float16* so = p.sum_out ? reinterpret_cast<_Float16*>(p.sum_out) + (int64_t)m * p.ld_sum : nullptr;
  float x[VPT][8];
  h8_t g[VPT];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int k = (v * kNormThreads + threadIdx.x) * 8;
    if (k < p.K) {
      const h8_t av = *reinterpret_cast<const h8_t*>(a + k);
      g[v] = *reinterpret_cast<const h8_t*>(sc + k);
      h8_t sv;
      if (sk) sv = *reinterpret_cast<const h8_t*>(sk + k);
      h8_t sum_h;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float val = (float)av[e];
        if (sk) val += (float)sv[e];
        x[v][e] = val;
        sum_h[e] = (_Float16)val;
        ss += val * val;
      }
      if (so) *reinterpret_cast<h8_t*>(so + k) = sum_h;
    }
  }
  const float denom = sqrtf(block_sum(ss, red) / (float)p.K + p.eps);
#pragma unroll
  for (int v = 0; v < VPT; ++v) {
    const int k = (v * kNormThreads + threadIdx.x) * 8;
    if (k < p.K) {
      h8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (_Float16)(x[v][e] / denom * (float)g[v][e]);
      *reinterpret_cast<h8_t*>(out + k) = o;
    }
  }
}

// any type, alignment and K: two passes over the row
template <typename T>
__global__ void __launch_bounds__(kNormThreads) mnb_rmsnorm_generic_kernel(NormParams p) {
  __shared__ float red[kNormThreads / 64];
  const int m = blockIdx.x;
  const T* a = reinterpret_cast<const T*>(p.A) + (int64_t)m * p.lda;
  const T* sk = p.skip ? reinterpret_cast<const T*>(p.skip) + (int64_t)(m % p.skip_rows) * p.ld_skip : nullptr;
  const T* sc = reinterpret_cast<const T*>(p.scale);
  T* out = reinterpret_cast<T*>(p.out) + (int64_t)m * p.K;
  T* so = p.sum_out ? reinterpret_cast<T*>(p.sum_out) + (int64_t)m * p.ld_sum : nullptr;
  float ss = 0.f;
  for (int k = threadIdx.x; k < p.K; k += kNormThreads) {
    float val = (float)a[k];
    if (sk) val += (float)sk[k];
    if (so) so[k] = (T)val;
    ss += val * val;
  }
  const float denom = sqrtf(block_sum(ss, red) / (float)p.K + p.eps);
  for (int k = threadIdx.x; k < p.K; k += kNormThreads) {
    float val = (float)a[k];
    if (sk) val += (float)sk[k];
    out[k] = (T)(val / denom * (float)sc[k]);
  }
}

struct FinishParams {
  const void* tmp;
  int64_t ld_tmp;
  int M;
  int kind;
  int64_t start[3], n[3], ld[3];
  void* out[3];
};

template <typename T>
__global__ void __launch_bounds__(256) mnb_fused_finish_kernel(FinishParams p) {
  const T* tmp = reinterpret_cast<const T*>(p.tmp);
  if (p.kind == kMnbFusedMlp) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.M * p.n[0]) return;
    const int64_t m = idx / p.n[0], n = idx % p.n[0];
    const int64_t ng = (n >> 4) * 32 + (n & 15);  // packed column of gate; up follows 16 columns later
    const float g = (float)tmp[m * p.ld_tmp + ng];
    const float up = (float)tmp[m * p.ld_tmp + ng + 16];
    reinterpret_cast<T*>(p.out[0])[m * p.ld[0] + n] = (T)(g / (1.0f + expf(-g)) * up);
  } else {
    const int64_t width = p.n[0] + p.n[1] + p.n[2];
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.M * width) return;
    const int64_t m = idx / width;
    int64_t n = idx % width;
    int s = 0;
    if (n >= p.n[0]) {
      n -= p.n[0];
      s = 1;
      if (n >= p.n[1]) {
        n -= p.n[1];
        s = 2;
      }
    }
    reinterpret_cast<T*>(p.out[s])[m * p.ld[s] + n] = tmp[m * p.ld_tmp + p.start[s] + n];
  }
}

}  // namespace

hipError_t mnb_launch_rmsnorm(void* a_norm, void* sum_out, int64_t ld_sum, const void* A, int64_t lda, const void* skip,
                              int64_t ld_skip, int64_t skip_rows, const void* scale, float epsilon, int64_t M, int64_t K,
                              int dtype, hipStream_t s) {
  if (M == 0 || K == 0) return hipSuccess;
  NormParams p{};
  p.A = A;
  p.skip = skip;
  p.scale = scale;
  p.out = a_norm;
  p.sum_out = sum_out;
  p.lda = lda;
  p.ld_skip = ld_skip;
  p.skip_rows = skip_rows > 0 ? skip_rows : M;
  p.ld_sum = ld_sum;
  p.M = (int)M;
  p.K = (int)K;
  p.eps = epsilon;
  const dim3 grid((unsigned)M), blk(kNormThreads);
  if (dtype == kMnbDtypeFloat16) {
    auto al16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    const bool vec = K % 8 == 0 && al16(A) && lda % 8 == 0 && al16(scale) && al16(a_norm) &&
                     (!skip || (al16(skip) && ld_skip % 8 == 0)) && (!sum_out || (al16(sum_out) && ld_sum % 8 == 0));
    const int64_t per_round = 8 * kNormThreads;
    if (vec && K <= per_round)
      mnb_rmsnorm_h_vec_kernel<1><<<grid, blk, 0, s>>>(p);
    else if (vec && K <= 2 * per_round)
      mnb_rmsnorm_h_vec_kernel<2><<<grid, blk, 0, s>>>(p);
    else if (vec && K <= 4 * per_round)
      mnb_rmsnorm_h_vec_kernel<4><<<grid, blk, 0, s>>>(p);
    else
      mnb_rmsnorm_generic_kernel<_Float16><<<grid, blk, 0, s>>>(p);
  } else {
    mnb_rmsnorm_generic_kernel<float><<<grid, blk, 0, s>>>(p);
  }
  return hipGetLastError();
}

hipError_t mnb_launch_fused_finish(const MnbEpilogue& epi, const void* tmp, int64_t ld_tmp, int64_t M, int dtype,
                                   hipStream_t s) {
  FinishParams p{};
  p.tmp = tmp;
  p.ld_tmp = ld_tmp;
  p.M = (int)M;
  p.kind = epi.kind;
  for (int i = 0; i < 3; ++i) {
    p.start[i] = epi.start[i];
    p.n[i] = epi.n[i];
    p.ld[i] = epi.ld[i];
    p.out[i] = epi.out[i];
  }
  const int64_t width = epi.kind == kMnbFusedMlp ? epi.n[0] : epi.n[0] + epi.n[1] + epi.n[2];
  const int64_t total = M * width;
  if (total == 0) return hipSuccess;
  const dim3 grid((unsigned)((total + 255) / 256)), blk(256);
  if (dtype == kMnbDtypeFloat16)
    mnb_fused_finish_kernel<_Float16><<<grid, blk, 0, s>>>(p);
  else
    mnb_fused_finish_kernel<float><<<grid, blk, 0, s>>>(p);
  return hipGetLastError();
}
