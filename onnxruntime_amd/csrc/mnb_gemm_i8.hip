// int8 activations x int4 weights on the int8 matrix cores: the accuracy_level-4 route of the operator.
//
// Device counterpart of the reference's SQ4BitGemm_CompInt8 (onnxruntime/core/mlas/lib/qnbitgemm.cpp:883-1086) with
// the arithmetic of the scalar statement its kernels are tested against
// (onnxruntime/test/mlas/unittest/test_sqnbitgemm.cpp:94-170):
//   * the activations are quantised per row and block of block_size elements along k: scale = max|a| / 127,
//     q = clamp(roundf(a / scale)) (mnb_quantize_a_kernel; the reference's QuantizeARow_CompInt8 step);
//   * per block the dot product of the int8 activations with the 4-bit weights is exact integer arithmetic
//     (v_mfma_i32_32x32x32_i8), and the block's int32 sum joins the fp32 result as
//     float(sum) * a_scale * b_scale, every operation rounded on its own, blocks in k order, starting from the bias.
// Because every output is accumulated by one lane in that order, results are the bits of the scalar statement.
//
// Zero points: sum_k qa (qb - zp) = sum_k qa qb - zp sum_k qa.  The nibbles go to the matrix core as they are
// (0 ... 15 are valid int8) and the quantiser also leaves sum_k qa per row and block, so the correction is one integer
// multiply-subtract per output and block (the reference's packed kernels apply the same identity in floating point,
// qnbitgemm.cpp:903-928; here it stays in integers and is exact).
//
// A workgroup of four wavefronts (2 x 2) owns a 128 x 128 tile of the output, each wavefront 64 x 64 as 2 x 2 matrix-
// core tiles.  Per step of 128 k: the quantised activations (128 rows x 128 bytes), their scales and their sums go
// from global memory straight into one of two LDS stages (buffer_load ... lds, the same XOR-swizzled rows as the fp16
// tile GEMM); the weights never touch LDS: lane (column, k half) loads the 8 bytes of each 16-byte vector that hold
// its 16 k and splits them into bytes with two AND and one shift per word.  The k order inside a lane's 16 elements
// is the packed layout's nibble order (e0 e4 e1 e5 e2 e6 e3 e7 per word); the quantiser writes the activations in the
// same order, so no permutation happens in the loop.
//
// This route is slower than the fp16 one on this hardware for every block size and is therefore never chosen by the
// dispatcher: it runs when the caller asks for it (MnbGemmInt8).  The per-block rescale costs five vector
// instructions per output (integer correction, conversion, two multiplies, one add) against one matrix instruction
// per 32 x 32 x 32 products: with 128-wide blocks 20 instructions per matrix instruction, with 64-wide blocks 40; the
// fp16 route folds the scale into the weights and pays 3.5 per matrix instruction of half the depth.
// Blocks of 32 are declined (MNB_NOT_IMPLEMENTED): every matrix instruction would be followed by the rescale of its
// 16 sums, 80 vector instructions -- 320 issue cycles against the 32 the matrix instruction takes.  The contract fixes
// one fp32 multiply-add chain per output and block, so no arrangement of the loop removes them; the instantiation
// that existed took 4.0 ms where the full-accuracy route takes 0.21 ms (M = 2048, N = 14336, K = 4096).
#include <hip/hip_runtime.h>

#include "mnb_buffer.hip.h"
#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

typedef int i4_t __attribute__((ext_vector_type(4)));
typedef int i16_t __attribute__((ext_vector_type(16)));

constexpr int TILE = 128;                     // rows and columns of a workgroup's tile
constexpr int STEP_K = 128;                   // k per step = bytes per staged row of quantised activations
constexpr int A_STAGE = TILE * STEP_K;        // 16 KiB
constexpr int S_STAGE = 2 * 4 * TILE * 4;     // scales, then sums, of up to four blocks x 128 rows: 4 KiB
constexpr int STAGE = A_STAGE + S_STAGE;
constexpr int QUANT_THREADS = 256;

// ------------------------------------------------------------------------------------------------ quantiser of A
struct QuantAParams {
  const _Float16* A;
  int64_t lda;
  int M, K, bs;
  int64_t Mpad, Kpad;  // rows rounded up to 128, k rounded up as in the packed weights
  int8_t* qa;          // [Mpad][Kpad], k permuted inside groups of 8 (0 4 1 5 2 6 3 7)
  float* a_scale;      // [KBp][Mpad]
  int32_t* a_sum;      // [KBp][Mpad]
  int vec_ok;          // rows of A are 16-byte aligned
};

// One workgroup per row; a thread owns 8 consecutive k, the bs / 8 threads of a block reduce over lanes.
__global__ void __launch_bounds__(QUANT_THREADS) mnb_quantize_a_kernel(QuantAParams p) {
  const int row = blockIdx.x, tid = threadIdx.x;
  const int lanes = p.bs >> 3;  // threads per block: 4 ... 32, a power of two
  const _Float16* a_row = p.A + (int64_t)(row < p.M ? row : 0) * p.lda;
  for (int64_t base = 0; base < p.Kpad; base += QUANT_THREADS * 8) {
    const int64_t k0 = base + tid * 8;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.f;
    if (row < p.M && k0 < p.K) {
      if (p.vec_ok && k0 + 8 <= p.K) {
        const h8_t h = *reinterpret_cast<const h8_t*>(a_row + k0);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (float)h[e];
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (k0 + e < p.K) v[e] = (float)a_row[k0 + e];
      }
    }
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[e]));
    for (int o = 1; o < lanes; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const float scale = __fdiv_rn(amax, 127.0f);
    const float recip = scale != 0.f ? __fdiv_rn(1.0f, scale) : 0.f;
    int q[8], sum = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float r = roundf(__fmul_rn(v[e], recip));
      r = fminf(fmaxf(r, -128.f), 127.f);
      q[e] = (int)r;
      sum += q[e];
    }
    for (int o = 1; o < lanes; o <<= 1) sum += __shfl_xor(sum, o);
    if (k0 < p.Kpad) {
      auto b = [&](int e) { return (uint32_t)(q[e] & 0xff); };
      u2_t out;
      out[0] = b(0) | (b(4) << 8) | (b(1) << 16) | (b(5) << 24);
      out[1] = b(2) | (b(6) << 8) | (b(3) << 16) | (b(7) << 24);
      *reinterpret_cast<u2_t*>(p.qa + (int64_t)row * p.Kpad + k0) = out;
      if ((tid & (lanes - 1)) == 0) {
        const int64_t blk = k0 / p.bs;
        p.a_scale[blk * p.Mpad + row] = scale;
        p.a_sum[blk * p.Mpad + row] = sum;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ the GEMM
struct GemmI8Params {
  const int8_t* qa;
  const float* a_scale;  // the sums follow the scales: a_sum = a_scale + KBp * Mpad (as int32)
  const uint8_t* W;
  const uint8_t* meta;
  const _Float16* bias;
  _Float16* C;
  int64_t Mpad, Kpad, KBp, Npad, ldc;
  int M, N;
};

// BS_SLABS = block_size / 32: matrix instructions (32 k each) per block.
template <bool HAS_ZP, int BS_SLABS>
__global__ void __launch_bounds__(256) mnb_gemm_i8_kernel(GemmI8Params p) {
  constexpr int NB = BS_SLABS >= 4 ? 1 : 4 / BS_SLABS;  // blocks that end inside a step
  constexpr int META_BYTES = HAS_ZP ? 4 : 2;
  __shared__ __align__(16) unsigned char lds[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, kq = lane >> 5;
  const int m0 = blockIdx.y * TILE, n0 = blockIdx.x * TILE;
  const int steps = (int)(p.Kpad / STEP_K);

  // ---- loads into LDS.  Activations: instruction i of a wavefront fills rows (4 i + wave) * 8 + [0, 8); the lane at
  // chunk position lane & 7 of row r fetches chunk (lane & 7) ^ ((r >> 1) & 7).
  uint32_t a_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (4 * i + wave) * 8 + (lane >> 3);
    a_off[i] = (uint32_t)((int64_t)r * p.Kpad + (((lane & 7) ^ ((r >> 1) & 7)) * 16));
  }
  const uint8_t* a_tile = reinterpret_cast<const uint8_t*>(p.qa) + (int64_t)m0 * p.Kpad;
  // Scales and sums: thread u fetches 16 bytes: array u / 128 (scales, sums), block u % 128 / 32 of the step, rows
  // 4 * (u % 32) + [0, 4).  A step with fewer than four blocks re-reads its last one.
  const int su = wave * 64 + lane;
  const int s_blk = ((su & 127) >> 5) < NB ? ((su & 127) >> 5) : NB - 1;
  const uint32_t s_off =
      (uint32_t)((((int64_t)(su >> 7) * p.KBp + s_blk) * p.Mpad + m0) * 4 + (su & 31) * 16);  // from block 0 of the step
  const uint8_t* s_base = reinterpret_cast<const uint8_t*>(p.a_scale);

  auto first_block = [&](int step) { return BS_SLABS >= 4 ? step / (BS_SLABS / 4) : step * NB; };
  auto dma = [&](int step, int stage) {
    const rsrc_t ra = mnb_rsrc(a_tile + (int64_t)step * STEP_K);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      mnb_buffer_load_lds_b128(ra, a_off[i], (lds_ptr_t)(lds + stage * STAGE + (4 * i + wave) * 8 * STEP_K));
    const rsrc_t rs = mnb_rsrc(s_base + (int64_t)first_block(step) * p.Mpad * 4);
    mnb_buffer_load_lds_b128(rs, s_off, (lds_ptr_t)(lds + stage * STAGE + A_STAGE + wave * 1024));
  };

  // ---- weights: this lane's column of each column tile, its 8 bytes of every 16-byte vector; meta entries as the
  // aligned 32-bit word that holds them
  struct BRegs {
    u2_t w[4][2];
    uint32_t m[NB][2];
  };
  uint32_t w_off[2], m_off[2], m_shift[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = n0 + wn * 64 + j * 32 + li;
    w_off[j] = (uint32_t)col * 16 + kq * 8;
    const uint32_t mb = (uint32_t)mnb_meta_col(col) * META_BYTES;
    m_off[j] = mb & ~3u;
    m_shift[j] = (mb & 2u) * 8;
  }
  auto load_b = [&](int step, BRegs& R) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const rsrc_t r = mnb_rsrc(p.W + ((int64_t)step * 4 + s) * p.Npad * 16);
#pragma unroll
      for (int j = 0; j < 2; ++j) R.w[s][j] = mnb_buffer_load_b64(r, w_off[j]);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const rsrc_t r = mnb_rsrc(p.meta + ((int64_t)first_block(step) + b) * p.Npad * META_BYTES);
#pragma unroll
      for (int j = 0; j < 2; ++j) R.m[b][j] = mnb_buffer_load_b32(r, m_off[j]);
    }
  };

  // ---- accumulators: fp32 results start from the bias, int32 block sums from zero
  f16_t accf[2][2];
  i16_t acci[2][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = n0 + wn * 64 + j * 32 + li;
    const float b0 = (p.bias != nullptr && col < p.N) ? (float)p.bias[col] : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        accf[i][j][r] = b0;
        acci[i][j][r] = 0;
      }
  }

  // the block that ends with slab `slab` of the step staged at `stage`: its int32 sums join the fp32 results
  auto rescale = [&](int b, int stage, const BRegs& R) {
    const unsigned char* sc = lds + stage * STAGE + A_STAGE + b * (TILE * 4);
    float bs[2];
    int zp[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (HAS_ZP) {
        const h2_t m = mnb_as_h2(R.m[b][j]);
        bs[j] = (float)m.x;
        zp[j] = -(int)(float)m.y - 1024;  // the entry holds -(1024 + zp)
      } else {
        bs[j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(R.m[b][j] >> m_shift[j]));
        zp[j] = 8;
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int row = wm * 64 + i * 32 + 8 * g + 4 * kq;
        const f4_t as = *reinterpret_cast<const f4_t*>(sc + row * 4);
        const i4_t sm = *reinterpret_cast<const i4_t*>(sc + 4 * TILE * 4 + row * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int r = 4 * g + e;
            const int q = acci[i][j][r] - zp[j] * sm[e];
            const float t = __fmul_rn(__fmul_rn((float)q, as[e]), bs[j]);
            accf[i][j][r] = __fadd_rn(accf[i][j][r], t);
            acci[i][j][r] = 0;
          }
      }
  };

  BRegs B0, B1;
  auto step_body = [&](int step, int stage, const BRegs& Bc, BRegs& Bn) {
    // this wavefront's loads of the step have landed; the barrier makes that true of everybody's, and everybody has
    // finished reading the other stage
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lds0(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (step + 1 < steps) {
      dma(step + 1, stage ^ 1);
      load_b(step + 1, Bn);
    }
    const unsigned char* at = lds + stage * STAGE;
#pragma unroll
    for (int slab = 0; slab < 4; ++slab) {
      i4_t a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = wm * 64 + i * 32 + li;
        a[i] = *reinterpret_cast<const i4_t*>(at + row * STEP_K + (((2 * slab + kq) ^ ((row >> 1) & 7)) * 16));
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const u2_t w = Bc.w[slab][j];
        b[j] = i4_t{(int)(w[0] & 0x0F0F0F0Fu), (int)((w[0] >> 4) & 0x0F0F0F0Fu), (int)(w[1] & 0x0F0F0F0Fu),
                    (int)((w[1] >> 4) & 0x0F0F0F0Fu)};
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#if defined(__HIP_DEVICE_COMPILE__)
          acci[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acci[i][j], 0, 0, 0);
#else
          acci[i][j][0] += a[i][0] * b[j][0];  // the host pass only needs this to parse
#endif
      if constexpr (BS_SLABS <= 4) {
        if ((slab + 1) % BS_SLABS == 0) rescale((slab + 1) / BS_SLABS - 1, stage, Bc);
      } else {
        if (slab == 3 && (step & 1) == 1) rescale(0, stage, Bc);
      }
    }
  };

  dma(0, 0);
  load_b(0, B0);
  for (int step = 0; step < steps; step += 2) {
    step_body(step, 0, B0, B1);
    if (step + 1 < steps) step_body(step + 1, 1, B1, B0);
  }

  // ---- epilogue: one narrowing
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + li;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
        if (row < p.M && col < p.N) p.C[(int64_t)row * p.ldc + col] = (_Float16)accf[i][j][r];
      }
    }
}

template <bool HAS_ZP>
hipError_t launch_bs(const GemmI8Params& p, int bs, dim3 grid, hipStream_t s) {
  switch (bs) {
    case 64: mnb_gemm_i8_kernel<HAS_ZP, 2><<<grid, dim3(256), 0, s>>>(p); break;
    case 128: mnb_gemm_i8_kernel<HAS_ZP, 4><<<grid, dim3(256), 0, s>>>(p); break;
    case 256: mnb_gemm_i8_kernel<HAS_ZP, 8><<<grid, dim3(256), 0, s>>>(p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

// the kernel's 32-bit offsets into the activation scales and sums reach every row of this problem
static bool offsets_fit(const MnbLayout& L, int64_t Mpad) { return 2 * L.KBp * Mpad * 4 < ((int64_t)1 << 32); }

bool mnb_gemm_i8_supported(const MnbLayout& L, int64_t M) {
  // 8-bit weights do not fit the signed int8 operand as they are; blocks below 64 are declined (file header)
  return L.src_bits == 4 && L.bits == 4 && L.dtype == kMnbDtypeFloat16 && L.bs >= 64 && L.bs <= 256 &&
         L.Kpad < ((int64_t)1 << 24) && offsets_fit(L, mnb_round_up(M, TILE));
}

size_t mnb_gemm_i8_workspace_bytes(const MnbLayout& L, int64_t M) {
  const int64_t Mpad = mnb_round_up(M, TILE);
  return (size_t)mnb_round_up(Mpad * L.Kpad, 256) + (size_t)(2 * L.KBp * Mpad * 4);
}

hipError_t mnb_launch_gemm_i8(const MnbGemmArgs& a, hipStream_t s) {
  const MnbLayout& L = a.L;
  const int64_t Mpad = mnb_round_up(a.M, TILE);
  if (!mnb_gemm_i8_supported(L, a.M) || a.workspace == nullptr ||
      a.workspace_bytes < mnb_gemm_i8_workspace_bytes(L, a.M) || reinterpret_cast<uintptr_t>(a.workspace) % 16 != 0)
    return hipErrorInvalidValue;  // the caller checks before coming here
  QuantAParams q{};
  q.A = reinterpret_cast<const _Float16*>(a.A);
  q.lda = a.lda;
  q.M = (int)a.M;
  q.K = (int)L.K;
  q.bs = L.bs;
  q.Mpad = Mpad;
  q.Kpad = L.Kpad;
  q.qa = reinterpret_cast<int8_t*>(a.workspace);
  q.a_scale = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.workspace) + mnb_round_up(Mpad * L.Kpad, 256));
  q.a_sum = reinterpret_cast<int32_t*>(q.a_scale + L.KBp * Mpad);
  q.vec_ok = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0);
  mnb_quantize_a_kernel<<<dim3((unsigned)Mpad), dim3(QUANT_THREADS), 0, s>>>(q);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;

  GemmI8Params p{};
  p.qa = q.qa;
  p.a_scale = q.a_scale;
  p.W = reinterpret_cast<const uint8_t*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + L.meta_off;
  p.bias = reinterpret_cast<const _Float16*>(a.bias);
  p.C = reinterpret_cast<_Float16*>(a.C);
  p.Mpad = Mpad;
  p.Kpad = L.Kpad;
  p.KBp = L.KBp;
  p.Npad = L.Npad;
  p.ldc = a.ldc;
  p.M = (int)a.M;
  p.N = (int)L.N;
  const dim3 grid((unsigned)((L.N + TILE - 1) / TILE), (unsigned)(Mpad / TILE));
  return L.has_zp ? launch_bs<true>(p, L.bs, grid, s) : launch_bs<false>(p, L.bs, grid, s);
}
