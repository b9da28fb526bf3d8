// The operand variants the reference serves through its dequantise-everything route and calls "very rare"
// (MatMulNBits<T>::ComputeBUnpacked, onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:1184-1333 and
// :1336-1510): zero points in the activation type, a group index g_idx, and bfloat16 activations.
//
// Nothing here computes a product.  The variants are turned into problems the ordinary kernels run:
//   * g_idx[k] names the block whose scale and zero point element k uses (Dequantize4BitsKernelReOrder,
//     onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_impl.cc:19-75).  Sorting k by group makes the members of
//     a group adjacent: whole blocks of the operator's block size when every group has a multiple of it (act-order
//     permutations), otherwise of the largest power of two that divides every group, otherwise - after padding every
//     group to a multiple of 16 - of 16, the smallest block size the kernels know.  The weights are packed in that
//     order once; per call the activation columns are gathered into the same order, with zeros in the padding (so
//     the padded weights never count).
//   * zero points in the activation type are not integers (HQQ-style quantisers produce them), so they cannot ride
//     in the fp16 kernels' integer offset: scales and zero points are widened to fp32, exactly, at pack time (the
//     matrix is packed as an fp32 model's).  fp32 models run the fp32 kernels on it.  The widened route for 16-bit
//     models does the same on a widened copy of the activations and narrows the fp32 result plus bias once - the
//     reference's own arithmetic for this input (fp32 SGEMM on widened operands).  It is the yardstick the
//     matrix-core routes below were measured against and runs in calibration builds only (MNB_NATIVE_ROUTE=wide).
//   * 16-bit models on such a matrix - bfloat16 (always packed this way), fp16 with zero points in the activation
//     type - skip the widened route: the decode kernel (up to 16 rows), the streaming kernel and the tile GEMM
//     (beyond) dequantise the weights in fp32, narrow them to the activation type for the
//     matrix cores (what the reference's GPU provider multiplies:
//     onnxruntime/contrib_ops/cuda/quantization/matmul_nbits.cc:844-975 dequantises B into the activation type and
//     calls a GEMM of that type), accumulate in fp32, and add bias and narrow in the epilogue.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/mnb_mi355x.h"
#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

constexpr int kSrcF32 = 0, kSrcF16 = 1, kSrcBf16 = 2;
constexpr int kMinPackedBlock = 16;  // smallest block size of a matrix packed in g_idx order

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  return mnb_report_error(code, buf);
}

int hip_fail(hipError_t e, const char* what) { return fail(MNB_EP_FAIL, "%s: %s", what, hipGetErrorString(e)); }

int src_kind(int dtype) { return dtype == MNB_DTYPE_FLOAT ? kSrcF32 : dtype == MNB_DTYPE_FLOAT16 ? kSrcF16 : kSrcBf16; }
size_t elem_size(int dtype) { return dtype == MNB_DTYPE_FLOAT ? 4 : 2; }
size_t round256(size_t v) { return (v + 255) / 256 * 256; }

__device__ __forceinline__ float widen(const void* p, int64_t i, int kind) {
  if (kind == kSrcF32) return reinterpret_cast<const float*>(p)[i];
  if (kind == kSrcF16) return (float)reinterpret_cast<const _Float16*>(p)[i];
  return __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p)[i] << 16);  // bfloat16: the top half of a float
}

// round-to-nearest-even to bfloat16; NaN stays NaN (quiet)
__device__ __forceinline__ uint16_t narrow_bf16(float v) {
  const uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// ---------------------------------------------------------------------------------------------------- pack
// Weights in gather order, 4 bits: one thread per (column, 16-byte group); element j of the packed column is element
// gather[j] of the canonical one, 0 where gather[j] < 0.
__global__ void __launch_bounds__(256) mnb_variant_pack_weights_kernel(const uint8_t* __restrict__ B,
                                                                       const int32_t* __restrict__ gather,
                                                                       int64_t src_col_bytes, uint4* __restrict__ W,
                                                                       MnbLayout L) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n = idx / L.KG;
  const int64_t g = idx % L.KG;
  if (n >= L.Npad) return;
  uint32_t w[4] = {0, 0, 0, 0};
  if (n < L.N) {
    const uint8_t* src = B + n * src_col_bytes;
    for (int i = 0; i < 4; ++i) {
      uint32_t r = 0;
      for (int e = 0; e < 8; ++e) {
        const int64_t j = g * 32 + i * 8 + e;
        const int32_t k = j < L.K ? gather[j] : -1;
        const uint32_t q = k >= 0 ? (src[k >> 1] >> ((k & 1) * 4)) & 0xFu : 0u;
        const int pos = (e & 1) ? 4 + (e >> 1) : (e >> 1);  // nibble order e0 e2 e4 e6 e1 e3 e5 e7
        r |= q << (4 * pos);
      }
      w[i] = r;
    }
  }
  W[g * L.Npad + n] = make_uint4(w[0], w[1], w[2], w[3]);
}

struct MetaParams {
  const void* scales;
  const void* zp;
  const int32_t* block_group;  // packed block -> source block, or NULL (identity)
  uint8_t* meta;
  int64_t src_k_blocks;
  int src_kind;  // element type of scales and typed zero points
  int zp_kind;
  int src_bits;
  MnbLayout L;
};

// One thread per (packed block, column).
__global__ void __launch_bounds__(256) mnb_variant_pack_meta_kernel(MetaParams p) {
  const MnbLayout& L = p.L;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= L.KBp * L.Npad) return;
  const int64_t kb = idx / L.Npad;
  const int64_t n = idx % L.Npad;
  const int64_t dst = kb * L.Npad + mnb_meta_col(n);
  const bool valid = n < L.N && kb < L.k_blocks;
  float s = 0.f, z = 0.f;
  if (valid) {
    const int64_t sb = p.block_group ? p.block_group[kb] : kb;
    s = widen(p.scales, n * p.src_k_blocks + sb, p.src_kind);
    if (p.zp_kind == MNB_ZP_TYPED) {
      z = widen(p.zp, n * p.src_k_blocks + sb, p.src_kind);
    } else if (p.zp_kind == MNB_ZP_UINT8) {
      const uint8_t* zp = reinterpret_cast<const uint8_t*>(p.zp);
      const int64_t row = (p.src_k_blocks * p.src_bits + 7) / 8;
      if (p.src_bits == 8)
        z = (float)zp[n * row + sb];
      else if (p.src_bits == 4)
        z = (float)((zp[n * row + (sb >> 1)] >> ((sb & 1) * 4)) & 0xF);
      else
        z = (float)((zp[n * row + (sb >> 2)] >> ((sb & 3) * 2)) & 0x3);
    } else {
      z = (float)(1 << (p.src_bits - 1));
    }
  }
  if (L.dtype == kMnbDtypeFloat16) {  // scales are fp16 already, zero points are integers
    if (L.has_zp) {
      h2_t m;
      m.x = (_Float16)s;
      m.y = (_Float16)(-(1024.0f + z));
      reinterpret_cast<uint32_t*>(p.meta)[dst] = mnb_as_u32(m);
    } else {
      reinterpret_cast<_Float16*>(p.meta)[dst] = (_Float16)s;
    }
  } else {
    if (L.has_zp)
      reinterpret_cast<float2*>(p.meta)[dst] = make_float2(s, z);
    else
      reinterpret_cast<float*>(p.meta)[dst] = s;
  }
}

// ---------------------------------------------------------------------------------------------------- per call
// A'[m][j] = A[m][gather[j]] (0 in the padding), widened to the compute type when that differs.
template <typename TO>
__global__ void __launch_bounds__(256) mnb_variant_stage_a_kernel(const void* __restrict__ A, int64_t lda, int in_kind,
                                                                  const int32_t* __restrict__ gather,
                                                                  TO* __restrict__ out, int64_t ld_out, int64_t K_in) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (j >= ld_out) return;
  const int64_t k = gather ? gather[j] : (j < K_in ? j : -1);
  out[m * ld_out + j] = k >= 0 ? (TO)widen(A, m * lda + k, in_kind) : (TO)0;
}

// The same for 16-bit activations that stay as they are (bfloat16 for the tile GEMM): a gathered or re-pitched copy.
__global__ void __launch_bounds__(256) mnb_variant_stage_a16_kernel(const uint16_t* __restrict__ A, int64_t lda,
                                                                    const int32_t* __restrict__ gather,
                                                                    uint16_t* __restrict__ out, int64_t ld_out,
                                                                    int64_t K_in) {
  const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (j >= ld_out) return;
  const int64_t k = gather ? gather[j] : (j < K_in ? j : -1);
  out[m * ld_out + j] = k >= 0 ? A[m * lda + k] : (uint16_t)0;
}

// Y[m][n] = narrow(Y32[m][n] + bias[n])
__global__ void __launch_bounds__(256) mnb_variant_finish_kernel(const float* __restrict__ y32, int64_t ld32,
                                                                 const void* __restrict__ bias, void* __restrict__ y,
                                                                 int64_t ldy, int64_t N, int out_kind) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (n >= N) return;
  float v = y32[m * ld32 + n];
  if (bias) v += widen(bias, n, out_kind);
  if (out_kind == kSrcF16)
    reinterpret_cast<_Float16*>(y)[m * ldy + n] = (_Float16)v;
  else
    reinterpret_cast<uint16_t*>(y)[m * ldy + n] = narrow_bf16(v);
}

// The reference's dequantiser for these inputs: float(q) * scale + (-scale * zp), every operation rounded by itself.
__global__ void __launch_bounds__(256) mnb_variant_dequant_kernel(float* __restrict__ dst, const uint8_t* __restrict__ B,
                                                                  const void* __restrict__ scales,
                                                                  const void* __restrict__ zp, int zp_kind,
                                                                  const int32_t* __restrict__ g_idx, int64_t N,
                                                                  int64_t K, int bits, int bs, int kind) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= N * K) return;
  const int64_t n = idx / K, k = idx % K;
  const int64_t kbc = (K + bs - 1) / bs;
  const uint8_t* col = B + n * (kbc * bs * bits / 8);
  const float q = bits == 4 ? (float)((col[k >> 1] >> ((k & 1) * 4)) & 0xF) : (float)((col[k >> 2] >> ((k & 3) * 2)) & 0x3);
  int64_t b = g_idx ? g_idx[k] : k / bs;
  if (b < 0 || b >= kbc) {
    // a group index outside [0, k_blocks) lives on the device, where the host cannot vet it: nothing is read through
    // it and the element becomes NaN, which no valid input produces
    dst[idx] = __builtin_nanf("");
    return;
  }
  const float s = widen(scales, n * kbc + b, kind);
  float z = (float)(1 << (bits - 1));
  if (zp_kind == MNB_ZP_TYPED) {
    z = widen(zp, n * kbc + b, kind);
  } else if (zp_kind == MNB_ZP_UINT8) {
    const uint8_t* zr = reinterpret_cast<const uint8_t*>(zp) + n * ((kbc * bits + 7) / 8);
    z = bits == 4 ? (float)((zr[b >> 1] >> ((b & 1) * 4)) & 0xF) : (float)((zr[b >> 2] >> ((b & 3) * 2)) & 0x3);
  }
  const float adjust = __fmul_rn(-s, z);
  dst[idx] = __fadd_rn(__fmul_rn(q, s), adjust);
}

// ---------------------------------------------------------------------------------------------------- planning
struct GroupOrder {
  bool trivial = true;
  int packed_block = 0;  // block size of the packed matrix
  int64_t packed_k = 0;
  std::vector<int32_t> gather;       // packed k -> canonical k, -1 in the padding
  std::vector<int32_t> block_group;  // packed block of 16 -> source block
};

// Sorts k by group (stable) and pads every group to whole blocks.  The packed block size is the operator's when every
// group has a multiple of it (GPTQ act-order: a permutation, every group keeps block_size members), else the largest
// power of two >= 16 that divides every group, else 16 with padding.
int order_by_group(const int32_t* g_idx, size_t len, int64_t K, int bs, bool tables, GroupOrder* out) {
  const int64_t k_blocks = (K + bs - 1) / bs;
  if ((int64_t)len != K && (int64_t)len != k_blocks * bs)
    return fail(MNB_INVALID_ARGUMENT, "Input 'group_index' is expected to have shape {%lld} or {%lld}, got {%zu}",
                (long long)K, (long long)(k_blocks * bs), len);
  std::vector<int64_t> count((size_t)k_blocks, 0);
  out->trivial = true;
  // every entry is checked, the padded tail beyond K included, with the reference's message
  // (matmul_nbits_helper.h:92-103)
  for (int64_t k = 0; k < (int64_t)len; ++k) {
    const int64_t g = g_idx[k];
    if (g < 0 || g >= k_blocks)
      return fail(MNB_INVALID_ARGUMENT, "group_index value at index %lld is %lld, which is out of valid range [0, %lld)",
                  (long long)k, (long long)g, (long long)k_blocks);
    if (k >= K) continue;  // padding: validated, not used
    if (g != k / bs) out->trivial = false;
    ++count[(size_t)g];
  }
  if (out->trivial) {
    out->packed_k = K;
    out->packed_block = bs;
    return MNB_OK;
  }
  int pb = bs;
  for (int64_t g = 0; g < k_blocks && pb > kMinPackedBlock; ++g)
    while (pb > kMinPackedBlock && count[(size_t)g] % pb != 0) pb >>= 1;
  out->packed_block = pb;
  std::vector<int64_t> start((size_t)k_blocks, 0);
  int64_t total = 0;
  for (int64_t g = 0; g < k_blocks; ++g) {
    start[(size_t)g] = total;
    total += (count[(size_t)g] + pb - 1) / pb * pb;
  }
  out->packed_k = total;
  if (!tables) return MNB_OK;
  out->gather.assign((size_t)total, -1);
  out->block_group.assign((size_t)(total / pb), 0);
  for (int64_t g = 0; g < k_blocks; ++g) {
    const int64_t blocks = (count[(size_t)g] + pb - 1) / pb;
    for (int64_t b = 0; b < blocks; ++b) out->block_group[(size_t)(start[(size_t)g] / pb + b)] = (int32_t)g;
  }
  std::vector<int64_t> next(start);
  for (int64_t k = 0; k < K; ++k) out->gather[(size_t)next[(size_t)g_idx[k]]++] = (int32_t)k;
  return MNB_OK;
}

// leading dimension of the staged activations: whole 16-byte vectors in either compute type
int64_t staged_ld(const MnbVariantPlan& p) { return (p.packed_k + 7) / 8 * 8; }

MnbLayout packed_layout(const MnbVariantPlan& p) {
  return mnb_make_layout(p.N, p.packed_k, p.bits, p.packed_block_size, p.compute_dtype, p.zp_kind != MNB_ZP_NONE, false);
}

int check_plan(const char* fn, const MnbVariantPlan* p) {
  if (p == nullptr) return fail(MNB_INVALID_ARGUMENT, "%s: plan must not be NULL", fn);
  if (p->packed_bytes == 0 || p->packed_k <= 0 || p->N <= 0)
    return fail(MNB_INVALID_ARGUMENT, "%s: the plan was not filled by MnbVariantMakePlan", fn);
  return MNB_OK;
}

}  // namespace

extern "C" {

int MnbVariantMakePlan(size_t N, size_t K, int bits, int block_size, int a_dtype, int zp_kind,
                       const int32_t* g_idx_host, size_t g_idx_len, MnbVariantPlan* plan) {
  if (plan == nullptr) return fail(MNB_INVALID_ARGUMENT, "MnbVariantMakePlan: plan must not be NULL");
  *plan = MnbVariantPlan{};
  if (bits != 2 && bits != 4 && bits != 8)
    return fail(MNB_INVALID_ARGUMENT,
                "MnbVariantMakePlan: Only 2b, 4b and 8b quantization is supported for MatMulNBits op, additional bits "
                "support is planned.");
  if (!(block_size == 16 || block_size == 32 || block_size == 64 || block_size == 128 || block_size == 256))
    return fail(MNB_INVALID_ARGUMENT,
                "MnbVariantMakePlan: Only block sizes 16, 32, 64, 128, and 256 are supported for MatMulNBits op, got: %d",
                block_size);
  if (a_dtype != MNB_DTYPE_FLOAT && a_dtype != MNB_DTYPE_FLOAT16 && a_dtype != MNB_DTYPE_BFLOAT16)
    return fail(MNB_NOT_IMPLEMENTED, "MnbVariantMakePlan: element type %d has no MI355X kernel", a_dtype);
  if (zp_kind != MNB_ZP_NONE && zp_kind != MNB_ZP_UINT8 && zp_kind != MNB_ZP_TYPED)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantMakePlan: unknown zero-point kind %d", zp_kind);
  if (N == 0 || K == 0) return fail(MNB_INVALID_ARGUMENT, "MnbVariantMakePlan: N and K must be positive");
  if (N > 0x7fffffff || K > 0x7fffffff)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantMakePlan: N and K must fit in 31 bits");
  // the reference's limits for these inputs (matmul_nbits.cc:1249-1252, :1258-1259)
  if (zp_kind == MNB_ZP_TYPED && bits == 8)
    return fail(MNB_NOT_IMPLEMENTED, "Only 2b and 4b quantization is supported for unpacked compute for now");
  if (g_idx_host != nullptr && bits != 4)
    return fail(MNB_NOT_IMPLEMENTED, "g_idx (reorder index) is supported for 4-bit quantization only");

  GroupOrder order;
  order.packed_k = (int64_t)K;
  order.packed_block = block_size;
  if (g_idx_host != nullptr)
    if (int rc = order_by_group(g_idx_host, g_idx_len, (int64_t)K, block_size, false, &order)) return rc;

  plan->N = (int64_t)N;
  plan->K = (int64_t)K;
  plan->bits = bits;
  plan->block_size = block_size;
  plan->a_dtype = a_dtype;
  plan->zp_kind = zp_kind;
  plan->has_g_idx = order.trivial ? 0 : 1;
  plan->compute_dtype = (a_dtype == MNB_DTYPE_FLOAT16 && zp_kind != MNB_ZP_TYPED) ? MNB_DTYPE_FLOAT16 : MNB_DTYPE_FLOAT;
  plan->packed_k = order.packed_k;
  plan->packed_block_size = plan->has_g_idx ? order.packed_block : block_size;
  const MnbLayout L = packed_layout(*plan);
  plan->gather_offset = (uint64_t)L.total_bytes;
  plan->packed_bytes = (uint64_t)L.total_bytes;
  if (plan->has_g_idx) {
    // the gather table (staged_ld entries) and the block -> group table, used only while packing
    plan->packed_bytes += round256((size_t)staged_ld(*plan) * sizeof(int32_t));
  }
  return MNB_OK;
}

int MnbVariantPack(const MnbVariantPlan* plan, const void* b_dev, const void* scales_dev, const void* zero_points_dev,
                   const int32_t* g_idx_host, size_t g_idx_len, void* packed_dev, void* stream) {
  if (int rc = check_plan("MnbVariantPack", plan)) return rc;
  if (!b_dev || !scales_dev || !packed_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantPack: B, scales and the packed buffer must not be NULL");
  if ((plan->zp_kind != MNB_ZP_NONE) != (zero_points_dev != nullptr))
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantPack: zero points do not match the plan's zero-point kind");
  if (reinterpret_cast<uintptr_t>(packed_dev) % 256 != 0)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantPack: the packed buffer must be 256-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const MnbLayout L = packed_layout(*plan);
  const int64_t src_k_blocks = (plan->K + plan->block_size - 1) / plan->block_size;
  uint8_t* packed = reinterpret_cast<uint8_t*>(packed_dev);

  MetaParams mp{};
  mp.scales = scales_dev;
  mp.zp = zero_points_dev;
  mp.meta = packed + L.meta_off;
  mp.src_k_blocks = src_k_blocks;
  mp.src_kind = src_kind(plan->a_dtype);
  mp.zp_kind = plan->zp_kind;
  mp.src_bits = plan->bits;
  mp.L = L;
  const int64_t mn = L.KBp * L.Npad;
  const dim3 blk(256), mgrid((unsigned)((mn + 255) / 256));

  if (!plan->has_g_idx) {
    hipError_t e = mnb_launch_pack_weights(L, b_dev, packed_dev, s);
    if (e != hipSuccess) return hip_fail(e, "MnbVariantPack");
    mnb_variant_pack_meta_kernel<<<mgrid, blk, 0, s>>>(mp);
    e = hipGetLastError();
    return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbVariantPack");
  }

  if (g_idx_host == nullptr) return fail(MNB_INVALID_ARGUMENT, "MnbVariantPack: the plan was made with a g_idx");
  GroupOrder order;
  if (int rc = order_by_group(g_idx_host, g_idx_len, plan->K, plan->block_size, true, &order)) return rc;
  if (order.trivial || order.packed_k != plan->packed_k || order.packed_block != plan->packed_block_size)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantPack: g_idx is not the one the plan was made from");
  const int64_t ld = staged_ld(*plan);
  order.gather.resize((size_t)ld, -1);
  int32_t* gather_dev = reinterpret_cast<int32_t*>(packed + plan->gather_offset);
  int32_t* block_group_dev = nullptr;
  hipError_t e = hipMemcpyAsync(gather_dev, order.gather.data(), (size_t)ld * sizeof(int32_t), hipMemcpyHostToDevice, s);
  if (e == hipSuccess) e = hipMallocAsync(reinterpret_cast<void**>(&block_group_dev), order.block_group.size() * sizeof(int32_t), s);
  if (e != hipSuccess) return hip_fail(e, "MnbVariantPack");
  e = hipMemcpyAsync(block_group_dev, order.block_group.data(), order.block_group.size() * sizeof(int32_t),
                     hipMemcpyHostToDevice, s);
  if (e == hipSuccess) {
    const int64_t wn = L.Npad * L.KG;
    const dim3 wgrid((unsigned)((wn + 255) / 256));
    const int64_t src_col_bytes = src_k_blocks * plan->block_size / 2;
    mnb_variant_pack_weights_kernel<<<wgrid, blk, 0, s>>>(reinterpret_cast<const uint8_t*>(b_dev), gather_dev,
                                                          src_col_bytes, reinterpret_cast<uint4*>(packed_dev), L);
    mp.block_group = block_group_dev;
    mnb_variant_pack_meta_kernel<<<mgrid, blk, 0, s>>>(mp);
    e = hipGetLastError();
  }
  const hipError_t e_free = hipFreeAsync(block_group_dev, s);
  // the host tables above are pageable memory that goes away with this call
  const hipError_t e_sync = hipStreamSynchronize(s);
  if (e != hipSuccess) return hip_fail(e, "MnbVariantPack");
  if (e_free != hipSuccess) return hip_fail(e_free, "MnbVariantPack");
  return e_sync == hipSuccess ? MNB_OK : hip_fail(e_sync, "MnbVariantPack");
}

}  // extern "C"

namespace {

// [staged activations][fp32 result][workspace of the inner GEMM]
struct VariantWorkspace {
  size_t staged, y32, inner;
  size_t total() const { return staged + y32 + inner; }
};

// 16-bit activations on a matrix packed with fp32 entries - bfloat16 models, and fp16 models whose zero points are in
// the activation type - run on the matrix cores in their own type (weights dequantised in fp32 and narrowed): up to
// 16 rows on the decode kernel, beyond on the streaming kernel or the tile GEMM, chosen as for fp16 models.  The
// widened route serves calibration builds only.  Measured against it on (N, K) = (14336, 4096), bfloat16:
// 5 to 14 times faster from 17 rows up, 1.4 to 6 times up to 16 rows.
enum NativeRoute { kNativeNone, kNativeDecode, kNativeMid, kNativeTile };

// kMnbIoModel when the plan's kernels run in the compute type (fp32 models, fp16 models with integer zero points)
int native_io(const MnbVariantPlan& p) {
  if (p.a_dtype == MNB_DTYPE_BFLOAT16) return kMnbIoBf16;
  if (p.a_dtype == MNB_DTYPE_FLOAT16 && p.compute_dtype == MNB_DTYPE_FLOAT) return kMnbIoF16Wide;  // typed zero points
  return kMnbIoModel;
}

NativeRoute native_route(const MnbVariantPlan& p, size_t M) {
  if (native_io(p) == kMnbIoModel) return kNativeNone;
  if (const char* e = mnb_tuning_env("MNB_NATIVE_ROUTE")) {  // calibration: "wide" switches the native kernels off
    if (e[0] == 'w') return kNativeNone;
    if (e[0] == 't' && p.packed_k % 128 == 0) return kNativeTile;
    if (e[0] == 'm') return kNativeMid;
  }
  if (M <= 16) return kNativeDecode;
  return mnb_prefer_gemm256(packed_layout(p), (int64_t)M) ? kNativeTile : kNativeMid;  // (false unless k % 128 == 0)
}

// The tile GEMM reads A through 16-byte loads at 32-bit offsets: a caller's A that is not aligned for that is copied
// first.  (The other two kernels take any alignment.)  Columns that have to be gathered are copied for all three.
bool native_needs_copy(const MnbVariantPlan& p, NativeRoute route, const void* a, size_t lda) {
  if (p.has_g_idx) return true;
  if (route != kNativeTile) return false;
  return reinterpret_cast<uintptr_t>(a) % 16 != 0 || lda % 8 != 0 ||
         !mnb_gemm256_addressable((int64_t)lda, packed_layout(p).Npad);
}

VariantWorkspace variant_workspace(const MnbVariantPlan& p, size_t M) {
  VariantWorkspace w{};
  if (const NativeRoute route = native_route(p, M); route != kNativeNone) {
    // the tile GEMM gets room for the copy whether or not a call needs it: alignment and pitch are not known here
    if (route == kNativeTile || p.has_g_idx) w.staged = round256(M * (size_t)staged_ld(p) * sizeof(uint16_t));
    if (route == kNativeTile)
      w.inner = round256(mnb_gemm256_plan(packed_layout(p), (int64_t)M, true, native_io(p)).workspace_bytes);
    if (route == kNativeMid) w.inner = round256(mnb_mid_workspace_bytes(packed_layout(p), (int64_t)M));
    return w;
  }
  const bool widened = p.compute_dtype != p.a_dtype;
  if (p.has_g_idx || widened) w.staged = round256(M * (size_t)staged_ld(p) * elem_size(p.compute_dtype));
  if (widened) w.y32 = round256(M * (size_t)p.N * sizeof(float));
  w.inner = round256(MnbGemmWorkspaceSize(M, (size_t)p.N, (size_t)p.packed_k, p.bits, p.packed_block_size,
                                          p.zp_kind != MNB_ZP_NONE, p.compute_dtype));
  return w;
}

}  // namespace

extern "C" {

size_t MnbVariantGemmWorkspaceSize(const MnbVariantPlan* plan, size_t M) {
  if (plan == nullptr || plan->packed_bytes == 0 || M == 0) return 0;
  return variant_workspace(*plan, M).total();
}

int MnbVariantGemm(const MnbVariantPlan* plan, size_t M, const void* a_dev, size_t lda, const void* packed_dev,
                   const void* bias_dev, void* y_dev, size_t ldy, void* workspace_dev, size_t workspace_bytes,
                   void* stream) {
  if (int rc = check_plan("MnbVariantGemm", plan)) return rc;
  const MnbVariantPlan& p = *plan;
  if (M == 0) return MNB_OK;
  if (!a_dev || !packed_dev || !y_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantGemm: A, packed B and Y must not be NULL");
  if (lda < (size_t)p.K || ldy < (size_t)p.N)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantGemm: lda (%zu) < K (%lld) or ldy (%zu) < N (%lld)", lda,
                (long long)p.K, ldy, (long long)p.N);
  if (M > 65535) return fail(MNB_NOT_IMPLEMENTED, "MnbVariantGemm: at most 65535 rows per call");
  const VariantWorkspace w = variant_workspace(p, M);
  if (w.total() > 0 && (!workspace_dev || workspace_bytes < w.total()))
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantGemm: workspace of %zu bytes needed (MnbVariantGemmWorkspaceSize), %zu given",
                w.total(), workspace_dev ? workspace_bytes : (size_t)0);
  if (workspace_dev && reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantGemm: the workspace must be 256-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  uint8_t* ws = reinterpret_cast<uint8_t*>(workspace_dev);
  const bool widened = p.compute_dtype != p.a_dtype;
  const int in_kind = src_kind(p.a_dtype);

  if (const NativeRoute route = native_route(p, M); route != kNativeNone) {
    MnbGemmArgs a{};
    a.L = packed_layout(p);
    a.io = native_io(p);
    a.M = (int64_t)M;
    a.A = a_dev;
    a.lda = (int64_t)lda;
    if (native_needs_copy(p, route, a_dev, lda)) {
      const int64_t ld = staged_ld(p);
      const int32_t* gather =
          p.has_g_idx ? reinterpret_cast<const int32_t*>(reinterpret_cast<const uint8_t*>(packed_dev) + p.gather_offset)
                      : nullptr;
      const dim3 grid((unsigned)((ld + 255) / 256), (unsigned)M), blk(256);
      mnb_variant_stage_a16_kernel<<<grid, blk, 0, s>>>(reinterpret_cast<const uint16_t*>(a_dev), (int64_t)lda, gather,
                                                        reinterpret_cast<uint16_t*>(ws), ld, p.K);
      if (hipError_t e = hipGetLastError(); e != hipSuccess) return hip_fail(e, "MnbVariantGemm");
      a.A = ws;
      a.lda = ld;
    }
    a.packed = packed_dev;
    a.bias = bias_dev;
    a.C = y_dev;
    a.ldc = (int64_t)ldy;
    a.workspace = w.inner > 0 ? ws + w.staged : nullptr;
    a.workspace_bytes = w.inner;
    const hipError_t e = route == kNativeTile  ? mnb_launch_gemm256(a, s)
                         : route == kNativeMid ? mnb_launch_mid(a, s)
                                               : mnb_launch_skinny(a, s);
    return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbVariantGemm");
  }

  const void* a_in = a_dev;
  size_t ld_in = lda;
  if (w.staged > 0) {
    const int64_t ld = staged_ld(p);
    const int32_t* gather =
        p.has_g_idx ? reinterpret_cast<const int32_t*>(reinterpret_cast<const uint8_t*>(packed_dev) + p.gather_offset)
                    : nullptr;
    const dim3 grid((unsigned)((ld + 255) / 256), (unsigned)M), blk(256);
    if (p.compute_dtype == MNB_DTYPE_FLOAT16)
      mnb_variant_stage_a_kernel<_Float16><<<grid, blk, 0, s>>>(a_dev, (int64_t)lda, in_kind, gather,
                                                               reinterpret_cast<_Float16*>(ws), ld, p.K);
    else
      mnb_variant_stage_a_kernel<float><<<grid, blk, 0, s>>>(a_dev, (int64_t)lda, in_kind, gather,
                                                            reinterpret_cast<float*>(ws), ld, p.K);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return hip_fail(e, "MnbVariantGemm");
    a_in = ws;
    ld_in = (size_t)ld;
  }
  void* y_out = widened ? static_cast<void*>(ws + w.staged) : y_dev;
  const size_t ld_out = widened ? (size_t)p.N : ldy;
  if (int rc = MnbGemm(M, (size_t)p.N, (size_t)p.packed_k, p.bits, p.packed_block_size, p.zp_kind != MNB_ZP_NONE,
                       p.compute_dtype, a_in, ld_in, packed_dev, widened ? nullptr : bias_dev, y_out, ld_out,
                       w.inner > 0 ? ws + w.staged + w.y32 : nullptr, w.inner, stream))
    return rc;
  if (widened) {
    const dim3 grid((unsigned)((p.N + 255) / 256), (unsigned)M), blk(256);
    mnb_variant_finish_kernel<<<grid, blk, 0, s>>>(reinterpret_cast<const float*>(y_out), p.N, bias_dev, y_dev,
                                                   (int64_t)ldy, p.N, in_kind);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return hip_fail(e, "MnbVariantGemm");
  }
  return MNB_OK;
}

const char* MnbVariantGemmKernelName(const MnbVariantPlan* plan, size_t M) {
  if (plan == nullptr || plan->packed_bytes == 0 || M == 0) return "none";
  if (const NativeRoute route = native_route(*plan, M); route != kNativeNone)
    return route == kNativeTile ? "mnb_gemm256_kernel" : route == kNativeMid ? "mnb_mid_kernel" : "mnb_skinny_kernel";
  return MnbGemmKernelName(M, (size_t)plan->N, (size_t)plan->packed_k, plan->bits, plan->packed_block_size,
                           plan->compute_dtype);
}

int MnbVariantDequantize(float* dst_dev, const void* b_dev, const void* scales_dev, const void* zero_points_dev,
                         int zp_kind, const int32_t* g_idx_dev, size_t N, size_t K, int bits, int block_size,
                         int a_dtype, void* stream) {
  if (bits != 2 && bits != 4)
    return fail(MNB_NOT_IMPLEMENTED, "Only 2b and 4b quantization is supported for unpacked compute for now");
  if (!(block_size == 16 || block_size == 32 || block_size == 64 || block_size == 128 || block_size == 256))
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantDequantize: unsupported block size %d", block_size);
  if (a_dtype != MNB_DTYPE_FLOAT && a_dtype != MNB_DTYPE_FLOAT16 && a_dtype != MNB_DTYPE_BFLOAT16)
    return fail(MNB_NOT_IMPLEMENTED, "MnbVariantDequantize: element type %d is not supported", a_dtype);
  if (g_idx_dev != nullptr && bits != 4)
    return fail(MNB_NOT_IMPLEMENTED, "g_idx (reorder index) is supported for 4-bit quantization only");
  if ((zp_kind != MNB_ZP_NONE) != (zero_points_dev != nullptr))
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantDequantize: zero points do not match the zero-point kind");
  if (N == 0 || K == 0) return MNB_OK;
  if (!dst_dev || !b_dev || !scales_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbVariantDequantize: dst, B and scales must not be NULL");
  const int64_t total = (int64_t)N * (int64_t)K;
  const dim3 grid((unsigned)((total + 255) / 256)), blk(256);
  mnb_variant_dequant_kernel<<<grid, blk, 0, (hipStream_t)stream>>>(dst_dev, reinterpret_cast<const uint8_t*>(b_dev),
                                                                    scales_dev, zero_points_dev, zp_kind, g_idx_dev,
                                                                    (int64_t)N, (int64_t)K, bits, block_size,
                                                                    src_kind(a_dtype));
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbVariantDequantize");
}

}  // extern "C"
