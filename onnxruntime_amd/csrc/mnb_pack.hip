// PrePack and dequantise kernels.
//
// PrePack replaces the CPU-specific nibble interleave of the reference
// (onnxruntime/core/mlas/lib/sqnbitgemm_kernel_avx_common.h:39-115) with the gfx950 k-group-major layout described
// in mnb_layout.h.  The dequantise kernels restate BlockwiseQuantizer::dequantize
// (onnxruntime/core/mlas/lib/q4_dq.cpp:587-641) on the device.
#include "mnb_device.hip.h"
#include "mnb_internal.h"

// ------------------------------------------------------------------------------------------------ pack weights
// One thread per (column n, group g).  Consecutive threads take consecutive groups of one column, so the reads of
// the canonical matrix are contiguous; the 16-byte writes are strided by Npad.
// The canonical operands of up to three matrices that share one packed buffer (one matrix for MatMulNBits itself).
struct MnbPackSrc {
  const uint8_t* B[3];
  const void* scales[3];
  const void* bias[3];
  MnbColMap map;  // packed column -> (matrix, column)
};

template <int BITS>
__global__ void __launch_bounds__(256) mnb_pack_weights_kernel(MnbPackSrc S, uint4* __restrict__ W, MnbLayout L) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n = idx / L.KG;
  const int64_t g = idx % L.KG;
  if (n >= L.Npad) return;
  uint32_t w[4] = {0, 0, 0, 0};
  const int64_t col_bytes = L.k_blocks * L.bs * BITS / 8;  // bytes of one canonical column
  int m;
  int64_t col;
  if constexpr (BITS == 2) {
    // 32 two-bit elements = 8 source bytes become one 16-byte vector of nibbles (same nibble order as below)
    if (mnb_map_col(S.map, n, &m, &col)) {
      const uint8_t* src = S.B[m] + col * col_bytes;
      for (int i = 0; i < 4; ++i) {
        uint32_t r = 0;
        for (int e = 0; e < 8; ++e) {
          const int64_t off = g * 8 + i * 2 + (e >> 2);
          const uint32_t byte = off < col_bytes ? src[off] : 0u;
          const uint32_t q = (byte >> (2 * (e & 3))) & 0x3u;
          const int pos = (e & 1) ? 4 + (e >> 1) : (e >> 1);
          r |= q << (4 * pos);
        }
        w[i] = r;
      }
    }
    W[g * L.Npad + n] = make_uint4(w[0], w[1], w[2], w[3]);
    return;
  }
  if (mnb_map_col(S.map, n, &m, &col)) {
    const uint8_t* src = S.B[m] + col * col_bytes + g * 16;
    for (int i = 0; i < 4; ++i) {
      uint32_t v = 0;
      for (int b = 0; b < 4; ++b) {
        int64_t off = g * 16 + i * 4 + b;
        uint32_t byte = off < col_bytes ? src[i * 4 + b] : 0u;
        v |= byte << (8 * b);
      }
      if constexpr (BITS == 4) {
        // canonical nibble i of the word holds element e_i; store e0 e2 e4 e6 e1 e3 e5 e7
        uint32_t r = 0;
        for (int e = 0; e < 8; ++e) {
          uint32_t q = (v >> (4 * e)) & 0xFu;
          int pos = (e & 1) ? 4 + (e >> 1) : (e >> 1);
          r |= q << (4 * pos);
        }
        v = r;
      }
      w[i] = v;
    }
  }
  W[g * L.Npad + n] = make_uint4(w[0], w[1], w[2], w[3]);
}

// The native copy of a 2-bit source for the decode kernel (W2 of mnb_layout.h): one thread per (column, vector).
// Vector g = 4 c + kq belongs to lane quarter kq of chunk c (256 k); its operand i (8 weights, i = 0..7) covers
// k = 256 c + 128 (i / 4) + 32 kq + 8 (i % 4) .. + 7 (mnb_w2_k).
__global__ void __launch_bounds__(256) mnb_pack_weights2_native_kernel(MnbPackSrc S, uint4* __restrict__ W2, MnbLayout L) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t groups = L.Kpad / 64;
  const int64_t n = idx / groups, g = idx % groups;
  if (n >= L.Npad) return;
  uint32_t w[4] = {0, 0, 0, 0};
  const int64_t col_bytes = L.k_blocks * L.bs / 4;  // bytes of one canonical column
  int m;
  int64_t col;
  if (mnb_map_col(S.map, n, &m, &col)) {
    const uint8_t* src = S.B[m] + col * col_bytes;
    for (int j = 0; j < 4; ++j) {
      uint32_t r = 0;
      for (int e = 0; e < 16; ++e) {
        const int64_t k = mnb_w2_k(g, 2 * j + (e >> 3)) + (e & 7);
        const uint32_t byte = (k >> 2) < col_bytes ? src[k >> 2] : 0u;
        const uint32_t q = (byte >> (2 * (k & 3))) & 0x3u;
        r |= q << (((e & 1) ? 16 : 0) + 2 * (e >> 1));
      }
      w[j] = r;
    }
  }
  W2[g * L.Npad + n] = make_uint4(w[0], w[1], w[2], w[3]);
}

// The same transformation as a tiled transpose, for 4- and 8-bit sources whose columns are whole 16-byte groups at
// 16-byte aligned addresses (every block size but 16 with an odd block count).  In the kernel above a wavefront reads
// 64 x 16 single bytes and writes 64 vectors to 64 different cache lines; here a workgroup moves a tile of 32 columns
// x 32 groups through LDS: 16-byte loads with the lanes along a column (512-byte runs of the canonical matrix),
// 16-byte stores with the lanes along the columns (512-byte runs of the packed one).  LDS rows are padded by one
// vector, so the transposed reads are free of bank conflicts.
constexpr int kPackTile = 32;

// canonical nibble i of a word holds element e_i; the packed word holds e0 e2 e4 e6 e1 e3 e5 e7
__device__ __forceinline__ uint32_t mnb_pack_nibble_order(uint32_t v) {
  uint32_t lo = v & 0x0F0F0F0Fu, hi = (v >> 4) & 0x0F0F0F0Fu;  // even / odd elements, one per byte
  lo = (lo | (lo >> 4)) & 0x00FF00FFu;
  hi = (hi | (hi >> 4)) & 0x00FF00FFu;
  lo = (lo | (lo >> 8)) & 0x0000FFFFu;
  hi = (hi | (hi >> 8)) & 0x0000FFFFu;
  return lo | (hi << 16);
}

template <int BITS>
__global__ void __launch_bounds__(256) mnb_pack_weights_tiled_kernel(MnbPackSrc S, uint4* __restrict__ W, MnbLayout L) {
  static_assert(BITS == 4 || BITS == 8, "2-bit sources take the element-wise kernel");
  __shared__ uint4 tile[kPackTile][kPackTile + 1];
  const int64_t n0 = (int64_t)blockIdx.x * kPackTile, g0 = (int64_t)blockIdx.y * kPackTile;
  const int64_t col_groups = L.k_blocks * L.bs * BITS / 128;  // whole 16-byte groups of one canonical column
#pragma unroll
  for (int r = 0; r < kPackTile * kPackTile / 256; ++r) {
    const int i = threadIdx.x + 256 * r;
    const int gl = i % kPackTile, nl = i / kPackTile;
    const int64_t g = g0 + gl;
    int m;
    int64_t col;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (g < col_groups && mnb_map_col(S.map, n0 + nl, &m, &col))
      v = reinterpret_cast<const uint4*>(S.B[m])[col * col_groups + g];
    if constexpr (BITS == 4) {
      v.x = mnb_pack_nibble_order(v.x);
      v.y = mnb_pack_nibble_order(v.y);
      v.z = mnb_pack_nibble_order(v.z);
      v.w = mnb_pack_nibble_order(v.w);
    }
    tile[nl][gl] = v;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kPackTile * kPackTile / 256; ++r) {
    const int i = threadIdx.x + 256 * r;
    const int nl = i % kPackTile, gl = i / kPackTile;
    if (g0 + gl < L.KG) W[(g0 + gl) * L.Npad + n0 + nl] = tile[nl][gl];  // Npad is a multiple of the tile
  }
}

// Launches the weight repacking: the tiled kernel where its alignment conditions hold, else the element-wise one.
static void mnb_pack_weights_dispatch(const MnbPackSrc& S, uint4* W, const MnbLayout& L, hipStream_t s) {
  const int64_t wn = L.Npad * L.KG;
  const dim3 grid((unsigned)((wn + 255) / 256)), blk(256);
  if (L.src_bits == 2) {
    mnb_pack_weights_kernel<2><<<grid, blk, 0, s>>>(S, W, L);
    if (L.w2_bytes > 0) {
      const int64_t vecs = L.Npad * (L.Kpad / 64);
      mnb_pack_weights2_native_kernel<<<dim3((unsigned)((vecs + 255) / 256)), blk, 0, s>>>(
          S, reinterpret_cast<uint4*>(reinterpret_cast<unsigned char*>(W) + L.w2_off), L);
    }
    return;
  }
  bool tiled = (L.k_blocks * L.bs * L.bits) % 128 == 0 && L.Npad % kPackTile == 0;
  for (int m = 0; m < 3; ++m) tiled = tiled && reinterpret_cast<uintptr_t>(S.B[m]) % 16 == 0;
  const dim3 tgrid((unsigned)(L.Npad / kPackTile), (unsigned)((L.KG + kPackTile - 1) / kPackTile));
  if (L.bits == 4) {
    if (tiled)
      mnb_pack_weights_tiled_kernel<4><<<tgrid, blk, 0, s>>>(S, W, L);
    else
      mnb_pack_weights_kernel<4><<<grid, blk, 0, s>>>(S, W, L);
  } else {
    if (tiled)
      mnb_pack_weights_tiled_kernel<8><<<tgrid, blk, 0, s>>>(S, W, L);
    else
      mnb_pack_weights_kernel<8><<<grid, blk, 0, s>>>(S, W, L);
  }
}

// ------------------------------------------------------------------------------------------------ pack meta
// One thread per (block kb, column n).
template <typename T, int BITS, bool HAS_ZP>
__global__ void __launch_bounds__(256) mnb_pack_meta_kernel(MnbPackSrc S, const uint8_t* __restrict__ zp,
                                                            uint8_t* __restrict__ meta, MnbLayout L) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= L.KBp * L.Npad) return;
  const int64_t kb = idx / L.Npad;
  const int64_t n = idx % L.Npad;
  const int64_t dst = kb * L.Npad + mnb_meta_col(n);
  int m;
  int64_t col;
  const bool valid = mnb_map_col(S.map, n, &m, &col) && kb < L.k_blocks;
  T s = valid ? reinterpret_cast<const T*>(S.scales[m])[col * L.k_blocks + kb] : (T)0;
  int z = 0;
  if constexpr (HAS_ZP) {  // zero points exist only for a single matrix: col == n
    if (valid) {
      const int64_t row = (L.k_blocks * BITS + 7) / 8;
      if (zp == nullptr) {
        z = 1 << (BITS - 1);  // 2-bit weights without zero points: the default is stored explicitly
      } else if constexpr (BITS == 8) {
        z = zp[col * row + kb];
      } else if constexpr (BITS == 4) {
        z = (zp[col * row + (kb >> 1)] >> ((kb & 1) * 4)) & 0xF;
      } else {
        z = (zp[col * row + (kb >> 2)] >> ((kb & 3) * 2)) & 0x3;
      }
    }
  }
  if constexpr (sizeof(T) == 2) {
    if constexpr (HAS_ZP) {
      h2_t m;
      m.x = s;
      m.y = (_Float16)(-(1024.0f + (float)z));
      reinterpret_cast<uint32_t*>(meta)[dst] = mnb_as_u32(m);
    } else {
      reinterpret_cast<_Float16*>(meta)[dst] = s;
    }
  } else {
    if constexpr (HAS_ZP) {
      reinterpret_cast<float2*>(meta)[dst] = make_float2(s, (float)z);
    } else {
      reinterpret_cast<float*>(meta)[dst] = s;
    }
  }
}

// One bias value per packed column (zero for padding columns and absent biases).
template <typename T>
__global__ void __launch_bounds__(256) mnb_pack_bias_kernel(MnbPackSrc S, T* __restrict__ dst) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= S.map.Np) return;
  int m;
  int64_t col;
  T v = (T)0;
  if (mnb_map_col(S.map, n, &m, &col) && S.bias[m]) v = reinterpret_cast<const T*>(S.bias[m])[col];
  dst[n] = v;
}

// ------------------------------------------------------------------------------------------------ dequantise
// Canonical operands -> dst[n*K + k].  One thread per element.
template <typename T, int BITS>
__global__ void __launch_bounds__(256) mnb_dequant_canonical_kernel(T* __restrict__ dst, const uint8_t* __restrict__ B,
                                                                    const T* __restrict__ scales,
                                                                    const uint8_t* __restrict__ zp, int64_t N,
                                                                    int64_t K, int bs) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= N * K) return;
  const int64_t n = idx / K, k = idx % K;
  const int64_t kbc = (K + bs - 1) / bs;
  const int64_t kb = k / bs, r = k % bs;
  const uint8_t* blob = B + (n * kbc + kb) * (bs * BITS / 8);
  int q, z = 1 << (BITS - 1);
  if constexpr (BITS == 8) {
    q = blob[r];
    if (zp) z = zp[n * kbc + kb];
  } else if constexpr (BITS == 4) {
    q = (blob[r >> 1] >> ((r & 1) * 4)) & 0xF;
    if (zp) z = (zp[n * ((kbc + 1) / 2) + (kb >> 1)] >> ((kb & 1) * 4)) & 0xF;
  } else {
    q = (blob[r >> 2] >> ((r & 3) * 2)) & 0x3;
    if (zp) z = (zp[n * ((kbc + 3) / 4) + (kb >> 2)] >> ((kb & 3) * 2)) & 0x3;
  }
  const T s = scales[n * kbc + kb];
  if constexpr (sizeof(T) == 2) {
    dst[idx] = (_Float16)(q - z) * s;  // exact integer half times half: one RNE rounding
  } else {
    dst[idx] = (float)(q - z) * s;
  }
}

// The same for K % 8 == 0 and aligned operands: one thread per 8 consecutive k of one column (they share a block,
// block sizes being multiples of 16): one 2-, 4- or 8-byte load of weights, 16- or 32-byte stores, consecutive
// threads on consecutive addresses of both.  Arithmetic per element as above.
template <typename T, int BITS>
__global__ void __launch_bounds__(256) mnb_dequant_canonical_vec_kernel(T* __restrict__ dst,
                                                                        const uint8_t* __restrict__ B,
                                                                        const T* __restrict__ scales,
                                                                        const uint8_t* __restrict__ zp, int64_t N,
                                                                        int64_t K, int bs) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // 8-element unit
  const int64_t upr = K / 8;                                            // units per row of dst
  if (idx >= N * upr) return;
  const int64_t n = idx / upr, k = (idx % upr) * 8;
  const int64_t kbc = (K + bs - 1) / bs;
  const int64_t kb = k / bs, r = k % bs;
  const uint8_t* src = B + (n * kbc + kb) * (bs * BITS / 8) + r * BITS / 8;
  int q[8], z = 1 << (BITS - 1);
  if constexpr (BITS == 8) {
    const uint2 w = *reinterpret_cast<const uint2*>(src);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      q[e] = (w.x >> (8 * e)) & 0xFF;
      q[4 + e] = (w.y >> (8 * e)) & 0xFF;
    }
    if (zp) z = zp[n * kbc + kb];
  } else if constexpr (BITS == 4) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = (w >> (4 * e)) & 0xF;
    if (zp) z = (zp[n * ((kbc + 1) / 2) + (kb >> 1)] >> ((kb & 1) * 4)) & 0xF;
  } else {
    const uint32_t w = *reinterpret_cast<const uint16_t*>(src);
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = (w >> (2 * e)) & 0x3;
    if (zp) z = (zp[n * ((kbc + 3) / 4) + (kb >> 2)] >> ((kb & 3) * 2)) & 0x3;
  }
  const T s = scales[n * kbc + kb];
  __align__(16) T out[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if constexpr (sizeof(T) == 2)
      out[e] = (_Float16)(q[e] - z) * s;  // exact integer half times half: one RNE rounding
    else
      out[e] = (float)(q[e] - z) * s;
  }
  uint4* d = reinterpret_cast<uint4*>(dst + n * K + k);
  const uint4* o = reinterpret_cast<const uint4*>(out);
#pragma unroll
  for (int v = 0; v < (int)(8 * sizeof(T) / 16); ++v) d[v] = o[v];
}

// Packed buffer -> dst[n*K + k], through the same unpack code the GEMV/GEMM kernels use.
template <typename T, int BITS, bool HAS_ZP>
__global__ void __launch_bounds__(256) mnb_dequant_packed_kernel(T* __restrict__ dst, const uint8_t* __restrict__ packed,
                                                                 MnbLayout L, int vec_ok) {
  constexpr int GK = 128 / BITS;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t g = idx / L.Npad;
  const int64_t n = idx % L.Npad;
  if (g >= L.KG || n >= L.N) return;
  const uint4 v = reinterpret_cast<const uint4*>(packed)[g * L.Npad + n];
  const uint8_t* meta = packed + L.meta_off;
  __align__(16) T out[GK];
  if constexpr (sizeof(T) == 2) {
    mnb_dequant_group_h<BITS, HAS_ZP>(v, meta, g, n, L.Npad, L.bs, out);
  } else {
    mnb_dequant_group_f<BITS, HAS_ZP>(v, meta, g, n, L.Npad, L.bs, out);
  }
  if (vec_ok && (g + 1) * GK <= L.K) {
    // whole group inside the row, 16-byte aligned (K % 8 == 0, aligned dst): 16-byte stores
    uint4* d = reinterpret_cast<uint4*>(dst + n * L.K + g * GK);
    const uint4* o = reinterpret_cast<const uint4*>(out);
#pragma unroll
    for (int i = 0; i < (int)(GK * sizeof(T) / 16); ++i) d[i] = o[i];
    return;
  }
  for (int i = 0; i < GK; ++i) {
    const int64_t k = g * GK + i;
    if (k < L.K) dst[n * L.K + k] = out[i];
  }
}

// ------------------------------------------------------------------------------------------------ launchers
template <typename T>
static hipError_t pack_t(const MnbLayout& L, const MnbPackSrc& S, const void* zp, void* packed, hipStream_t s) {
  uint4* W = reinterpret_cast<uint4*>(packed);
  uint8_t* meta = reinterpret_cast<uint8_t*>(packed) + L.meta_off;
  const int64_t mn = L.KBp * L.Npad;
  dim3 blk(256);
  const dim3 mgrid((unsigned)((mn + 255) / 256));
  const uint8_t* z = (const uint8_t*)zp;
  mnb_pack_weights_dispatch(S, W, L, s);
  if (L.src_bits == 2) {
    mnb_pack_meta_kernel<T, 2, true><<<mgrid, blk, 0, s>>>(S, z, meta, L);  // z may be NULL: default stored
  } else if (L.bits == 4) {
    if (zp)
      mnb_pack_meta_kernel<T, 4, true><<<mgrid, blk, 0, s>>>(S, z, meta, L);
    else
      mnb_pack_meta_kernel<T, 4, false><<<mgrid, blk, 0, s>>>(S, nullptr, meta, L);
  } else {
    if (zp)
      mnb_pack_meta_kernel<T, 8, true><<<mgrid, blk, 0, s>>>(S, z, meta, L);
    else
      mnb_pack_meta_kernel<T, 8, false><<<mgrid, blk, 0, s>>>(S, nullptr, meta, L);
  }
  return hipGetLastError();
}

hipError_t mnb_launch_pack_weights(const MnbLayout& L, const void* B, void* packed, hipStream_t s) {
  MnbPackSrc S{};
  S.B[0] = reinterpret_cast<const uint8_t*>(B);
  S.map.kind = kMnbFusedNone;
  S.map.nsrc = 1;
  S.map.n[0] = L.N;
  S.map.Np = L.N;
  mnb_pack_weights_dispatch(S, reinterpret_cast<uint4*>(packed), L, s);
  return hipGetLastError();
}

hipError_t mnb_launch_pack(const MnbLayout& L, const void* B, const void* scales, const void* zp, void* packed,
                           hipStream_t s) {
  MnbPackSrc S{};
  S.B[0] = reinterpret_cast<const uint8_t*>(B);
  S.scales[0] = scales;
  S.map.kind = kMnbFusedNone;
  S.map.nsrc = 1;
  S.map.n[0] = L.N;
  S.map.Np = L.N;
  return L.dtype == kMnbDtypeFloat16 ? pack_t<_Float16>(L, S, zp, packed, s) : pack_t<float>(L, S, zp, packed, s);
}

hipError_t mnb_launch_pack_fused(const MnbFusedLayout& F, const void* const* B, const void* const* scales,
                                 const void* const* bias, void* packed, hipStream_t s) {
  MnbPackSrc S{};
  for (int i = 0; i < F.map.nsrc; ++i) {
    S.B[i] = reinterpret_cast<const uint8_t*>(B[i]);
    S.scales[i] = scales[i];
    S.bias[i] = bias[i];
  }
  S.map = F.map;
  hipError_t e = F.L.dtype == kMnbDtypeFloat16 ? pack_t<_Float16>(F.L, S, nullptr, packed, s)
                                               : pack_t<float>(F.L, S, nullptr, packed, s);
  if (e != hipSuccess) return e;
  uint8_t* bias_dst = reinterpret_cast<uint8_t*>(packed) + F.bias_off;
  const dim3 grid((unsigned)((F.map.Np + 255) / 256)), blk(256);
  if (F.L.dtype == kMnbDtypeFloat16)
    mnb_pack_bias_kernel<_Float16><<<grid, blk, 0, s>>>(S, reinterpret_cast<_Float16*>(bias_dst));
  else
    mnb_pack_bias_kernel<float><<<grid, blk, 0, s>>>(S, reinterpret_cast<float*>(bias_dst));
  return hipGetLastError();
}

template <typename T, int BITS>
static hipError_t dequant_canonical_t(void* dst, const void* B, const void* scales, const void* zp, int64_t N, int64_t K,
                                      int bs, hipStream_t s) {
  const dim3 blk(256);
  // vector kernel: 8 k per thread; needs whole units per row and naturally aligned loads and stores
  const bool vec = K % 8 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % BITS == 0;
  if (vec) {
    const int64_t units = N * (K / 8);
    mnb_dequant_canonical_vec_kernel<T, BITS><<<dim3((unsigned)((units + 255) / 256)), blk, 0, s>>>(
        (T*)dst, (const uint8_t*)B, (const T*)scales, (const uint8_t*)zp, N, K, bs);
  } else {
    const int64_t total = N * K;
    mnb_dequant_canonical_kernel<T, BITS><<<dim3((unsigned)((total + 255) / 256)), blk, 0, s>>>(
        (T*)dst, (const uint8_t*)B, (const T*)scales, (const uint8_t*)zp, N, K, bs);
  }
  return hipGetLastError();
}

hipError_t mnb_launch_dequant_canonical(void* dst, const void* B, const void* scales, const void* zp, int64_t N,
                                        int64_t K, int bits, int bs, int dtype, hipStream_t s) {
  if (N * K == 0) return hipSuccess;
  if (dtype == kMnbDtypeFloat16) {
    if (bits == 2) return dequant_canonical_t<_Float16, 2>(dst, B, scales, zp, N, K, bs, s);
    if (bits == 4) return dequant_canonical_t<_Float16, 4>(dst, B, scales, zp, N, K, bs, s);
    return dequant_canonical_t<_Float16, 8>(dst, B, scales, zp, N, K, bs, s);
  }
  if (bits == 2) return dequant_canonical_t<float, 2>(dst, B, scales, zp, N, K, bs, s);
  if (bits == 4) return dequant_canonical_t<float, 4>(dst, B, scales, zp, N, K, bs, s);
  return dequant_canonical_t<float, 8>(dst, B, scales, zp, N, K, bs, s);
}

template <typename T>
static hipError_t dequant_packed_t(void* dst, const void* packed, const MnbLayout& L, hipStream_t s) {
  const int64_t total = L.KG * L.Npad;
  dim3 grid((unsigned)((total + 255) / 256)), blk(256);
  const uint8_t* p = (const uint8_t*)packed;
  const int vec_ok = L.K % 8 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
  if (L.bits == 4) {
    if (L.has_zp)
      mnb_dequant_packed_kernel<T, 4, true><<<grid, blk, 0, s>>>((T*)dst, p, L, vec_ok);
    else
      mnb_dequant_packed_kernel<T, 4, false><<<grid, blk, 0, s>>>((T*)dst, p, L, vec_ok);
  } else {
    if (L.has_zp)
      mnb_dequant_packed_kernel<T, 8, true><<<grid, blk, 0, s>>>((T*)dst, p, L, vec_ok);
    else
      mnb_dequant_packed_kernel<T, 8, false><<<grid, blk, 0, s>>>((T*)dst, p, L, vec_ok);
  }
  return hipGetLastError();
}

hipError_t mnb_launch_dequant_packed(void* dst, const void* packed, const MnbLayout& L, hipStream_t s) {
  if (L.N == 0 || L.K == 0) return hipSuccess;
  return L.dtype == kMnbDtypeFloat16 ? dequant_packed_t<_Float16>(dst, packed, L, s)
                                     : dequant_packed_t<float>(dst, packed, L, s);
}
