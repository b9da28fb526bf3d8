// Dequant-in-LDS MFMA GEMM for fp16 models and large M: 256 x 256 output tile per workgroup.
//
// Device counterpart of the reference's prefill loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:
// 563-732).  Eight wavefronts (4 x 2, two per SIMD so that one can issue its staging work while the other owns the
// matrix core), each owning a 64 x 128 block of the tile as 2 x 4 v_mfma_f32_32x32x16_f16 accumulators (128
// accumulator registers per lane).  Per k-step of 64:
//   * every thread fetches 4 x 16 B of A and 1 (4-bit) or 2 (8-bit) x 16 B of packed weights two steps ahead
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
constexpr int THREADS = 512;
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

// Scheduling pipeline of one slab section (8 MFMAs): after every MFMA a few of the other instructions of the
// section, so they run in the MFMA's shadow; the 6 fragment reads go behind the first 6 MFMAs.  The closing
// sched_barrier keeps the scheduler from mixing the MFMAs of different slabs (they reuse the same accumulators).
template <bool VMEM, int VALU, int LDS_WRITE_EVERY>
__device__ __forceinline__ void slab_pipeline() {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                        // 1 MFMA
    if (i < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);             // 1 LDS read
    if (VMEM && i < 7) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);     // 1 VMEM read
    if constexpr (VALU > 0) __builtin_amdgcn_sched_group_barrier(0x002, VALU, 0);
    if constexpr (LDS_WRITE_EVERY > 0) {
      if (i % LDS_WRITE_EVERY == LDS_WRITE_EVERY - 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // 1 LDS write
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

template <int BITS, bool HAS_ZP, bool SMALL_BS>
__global__ void __launch_bounds__(THREADS, 2) mnb_gemm256_kernel(Gemm256Params p) {
  constexpr int GK = 128 / BITS;                    // k per 16-byte group
  constexpr int GPK = BK / GK;                      // groups per column per k-step: 2 or 4
  constexpr int B_LOADS = BN * GPK / THREADS;       // 16-byte weight loads per thread per k-step: 1 or 2
  constexpr int A_LOADS = BM * (BK / 8) / THREADS;  // 4
  extern __shared__ __align__(16) _Float16 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 4 x 2 wavefronts: rows wm*64, columns wn*128
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  const int li = lane & 31, kq = lane >> 5;

  f16_t acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // two register sets for the global prefetch (distance: two k-steps), two fragment sets for the LDS prefetch
  struct Stage {
    u4_t a[A_LOADS];
    u4_t b[B_LOADS];
    uint32_t m[B_LOADS * (SMALL_BS ? 2 : 1)];
  };
  Stage R0, R1;
  struct Frags {
    h8_t a[2], b[4];
  };
  Frags F0, F1;

  const int a_row = tid >> 3, a_kc = tid & 7;  // thread's first A chunk: row a_row (+64 per load), k chunk a_kc
  const _Float16* a_ptr[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    // rows beyond M re-read row M-1 and are never stored (a predicated load would serialise the loop)
    int m = m0 + a_row + i * 64;
    m = m < p.M ? m : p.M - 1;
    a_ptr[i] = p.A + (int64_t)m * p.lda + a_kc * 8;
  }
  const int b_col = tid & (BN - 1), b_g0 = tid >> 8;  // thread's weight column and first group (+2 per load)
  const int64_t bcol = n0 + b_col;
  const int64_t mcol = mnb_meta_col(bcol);
  const int last_step = p.ksteps - 1;

  auto meta_at = [&](int64_t idx) -> uint32_t {
    if constexpr (HAS_ZP)
      return reinterpret_cast<const uint32_t*>(p.meta)[idx];
    else
      return reinterpret_cast<const uint16_t*>(p.meta)[idx];
  };

  // k-steps past the end are clamped to the last one: the loop body stays branch free, the data is never used
  auto load_global = [&](int ks_raw, Stage& R) {
    const int ks = ks_raw < last_step ? ks_raw : last_step;
    const int k0 = ks * BK;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) R.a[i] = *reinterpret_cast<const u4_t*>(a_ptr[i] + k0);
#pragma unroll
    for (int g = 0; g < B_LOADS; ++g) {
      const int64_t kg = (int64_t)ks * GPK + b_g0 + 2 * g;
      R.b[g] = *reinterpret_cast<const u4_t*>(p.W + kg * p.Npad + bcol);
      if constexpr (SMALL_BS) {
        R.m[2 * g] = meta_at((kg * 2) * p.Npad + mcol);
        R.m[2 * g + 1] = meta_at((kg * 2 + 1) * p.Npad + mcol);
      } else {
        R.m[g] = meta_at(((kg * GK) >> p.bs_shift) * p.Npad + mcol);
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

  // dequantise the thread's g-th group and write its GK halves to buffer `buf`
  auto store_b_group = [&](int buf, int g, const Stage& R) {
    _Float16* brow = lds + buf * STAGE_HALVES + (BM + b_col) * LDS_STRIDE + (b_g0 + 2 * g) * GK;
    const uint32_t wd[4] = {R.b[g][0], R.b[g][1], R.b[g][2], R.b[g][3]};
    h2_t s2a, s2b;
    ZpH za, zb;
    if constexpr (SMALL_BS) {
      decode(R.m[2 * g], s2a, za);
      decode(R.m[2 * g + 1], s2b, zb);
    } else {
      decode(R.m[g], s2a, za);
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

  auto store_a = [&](int buf, int i, const Stage& R) {
    *reinterpret_cast<u4_t*>(lds + buf * STAGE_HALVES + (a_row + i * 64) * LDS_STRIDE + a_kc * 8) = R.a[i];
  };

  auto read_frags = [&](int buf, int kk, Frags& F) {
    const _Float16* As = lds + buf * STAGE_HALVES;
    const _Float16* Bs = As + BM * LDS_STRIDE;
#pragma unroll
    for (int t = 0; t < 2; ++t)
      F.a[t] = *reinterpret_cast<const h8_t*>(As + (wm * 64 + t * 32 + li) * LDS_STRIDE + kk * 16 + kq * 8);
#pragma unroll
    for (int t = 0; t < 4; ++t)
      F.b[t] = *reinterpret_cast<const h8_t*>(Bs + (wn * 128 + t * 32 + li) * LDS_STRIDE + kk * 16 + kq * 8);
  };

  auto mfma_slab = [&](const Frags& F) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(F.a[i], F.b[j], acc[i][j], 0, 0, 0);
  };

  // staging work of one k-step in three parts (one per MFMA slab it hides behind)
  auto store_third = [&](int buf, int q, const Stage& R) {
    if (q == 0) {
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) store_a(buf, i, R);
    } else if (q - 1 < B_LOADS) {
      store_b_group(buf, q - 1, R);
    }
  };

  // One k-step.  On entry: LDS buffer `cur` holds step ks, F0 holds its slab 0, Rn holds (or is receiving) step
  // ks+1.  Slabs 0-2: MFMAs with, in their shadow, the global loads of step ks+2 (into Rf), the fragment reads of
  // the following slab and the staging of step ks+1 into the other buffer.  Then the barrier: every wavefront has
  // finished writing the other buffer and has its slab-3 fragments in registers, so buffer `cur` is free again.
  // Slab 3 runs after the barrier, with the first fragments of step ks+1 fetched in its shadow.
  auto k_step = [&](int ks, Stage& Rf, Stage& Rn) {
    const int cur = ks & 1, nxt = cur ^ 1;
    // slab 0: global loads of step ks+2, fragments of slab 1, the A vectors of step ks+1 into the other buffer
    load_global(ks + 2, Rf);
    read_frags(cur, 1, F1);
    mfma_slab(F0);
    store_third(nxt, 0, Rn);
    slab_pipeline<true, 3, 2>();
    // slab 1: fragments of slab 2, first half of the weights of step ks+1
    read_frags(cur, 2, F0);
    mfma_slab(F1);
    store_third(nxt, 1, Rn);
    slab_pipeline<false, 9, 2>();
    // slab 2: fragments of slab 3, second half of the weights
    read_frags(cur, 3, F1);
    mfma_slab(F0);
    store_third(nxt, 2, Rn);
    slab_pipeline<false, 9, 2>();
    __syncthreads();
    // slab 3, behind the barrier: first fragments of step ks+1
    read_frags(nxt, 0, F0);
    mfma_slab(F1);
    slab_pipeline<false, 0, 0>();
  };

  // ---- prologue: steps 0 and 1 in flight, step 0 staged
  load_global(0, R0);
  load_global(1, R1);
#pragma unroll
  for (int q = 0; q < 3; ++q) store_third(0, q, R0);
  __syncthreads();
  read_frags(0, 0, F0);

  for (int ks = 0; ks < p.ksteps; ks += 2) {  // ksteps is even
    k_step(ks, R0, R1);
    k_step(ks + 1, R1, R0);
  }

  // ---- epilogue: D[i][j] of a 32x32 tile: lane holds column j = lane % 32, rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + wn * 128 + j * 32 + li;
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
  p.ksteps = (int)(a.L.K / BK);  // K is a multiple of 2 * BK
  if (a.L.bits == 4) {
    if (a.L.bs == 16) return a.L.has_zp ? launch<4, true, true>(p, s) : launch<4, false, true>(p, s);
    return a.L.has_zp ? launch<4, true, false>(p, s) : launch<4, false, false>(p, s);
  }
  return a.L.has_zp ? launch<8, true, false>(p, s) : launch<8, false, false>(p, s);
}
