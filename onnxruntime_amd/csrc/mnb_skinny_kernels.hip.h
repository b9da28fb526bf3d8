// fp16 decode kernel for 1 <= M <= 16: dequantising "skinny" GEMM on the matrix cores.
//
// Same contract as the reference's decode loop (MlasQ4GemmKernelBlkLen32PlusAvx512f,
// onnxruntime/core/mlas/lib/sqnbitgemm_kernel_avx_common_fp32.h:288-639): Y = A x dequant(B)^T (+ bias), fp32
// accumulation, one narrowing of Y.  The job is HBM-bound; the point of this design is to spend as few VALU
// instructions per weight byte as possible so the load pipe never waits for arithmetic:
//
//  * v_mfma_f32_16x16x32_f16 does the dot products: rows = the (up to 16) rows of A, columns = 16 output columns.
//    Lane (j = lane%16, kq = lane/16) reads ONE 16-byte vector of column j, k-group kq of a chunk of 4 k-groups, and
//    each of its 32-bit words is the B operand of one MFMA (the contraction index may be permuted freely as long
//    as A uses the same permutation).
//  * MODE 0 (block_size >= chunk): the B operand is the raw "magic" half 1024+q (low nibbles, bytes) or 64+q (high
//    nibbles: (w & 0x00F000F0) | 0x5400 is the half 64+q) -- 5 bit operations per 8 weights, no subtraction, no
//    multiplication.  The offsets and the zero point are removed afterwards, exactly, per (row, column, block):
//        sum_k a_k (q_k - zp) = D - C1 - zp * C2,   C1 = sum_k off_k a_k,  C2 = sum_k a_k
//    where -C1 and -C2 come out of MFMAs of the same A operands against constant operands (-off_k and -1 in every
//    lane, so each lane receives the values of its own rows), -C1 seeds the accumulator of the weight MFMAs, and
//    the scale is applied to the block sum in fp32.
//  * MODE 1 (smaller blocks): exact (q - zp) halves times the fp16 scale (bit-identical to the reference's fp16
//    dequantisation), accumulated across blocks by the MFMA.
//  * MODE 2 (bfloat16 models, whose matrix is packed with fp32 {scale, zero point} entries): weights dequantised in
//    fp32, fma(float(q), scale, -zp * scale), narrowed to bfloat16 and multiplied by v_mfma_f32_16x16x32_bf16; A,
//    bias and Y hold bfloat16 bits.
//  * MODE 3 (fp16 models with zero points in the activation type, packed the same way): as MODE 2 with the weights
//    narrowed to fp16 and the fp16 matrix instruction.
//  * MODE 4 (bfloat16 models, 4-bit weights, block_size >= chunk): MODE 0's scheme on bfloat16 - the raw operand is
//    the bfloat16 128 + q, exact in its 8 significant bits.
//  * MODE 5 (fp16 models with zero points in the activation type, block_size >= chunk): MODE 0 with the block's
//    fp32 scale and zero point - the zero point enters the fp32 correction unrounded.
//  * 2-bit weights stream from a copy in their own width (mnb_layout.h, W2): a vector holds 64 weights, the operands
//    of eight matrix instructions, a chunk is 256 k.  MODE 0 for blocks of 256, MODE 1 for blocks of 32 and 64, MODE 6
//    for blocks of 128: MODE 0 with the two halves of a chunk (operands 0..3 and 4..7) in different blocks, each with
//    its own corrections, block sum and meta entry.
//  * The A operands come straight from global memory (L2 hits after the first workgroup) when the rows of A are
//    16-byte aligned -- every load of a wavefront's first two chunks is issued before anything is waited for;
//    otherwise the rows are staged in LDS phase by phase (zero-filled beyond K, any alignment).
//  * K is split over the wavefronts of a workgroup and reduced through LDS in a fixed order; nothing is split over
//    workgroups, so there is no cross-workgroup synchronisation and no workspace.
// (The kernels, the plan and the launch ladder of the decode kernel: included by mnb_skinny.hip, which plans and
// dispatches, and by mnb_skinny_w4.hip, mnb_skinny_w4zp.hip, mnb_skinny_w8.hip and mnb_skinny_w2.hip, which each
// instantiate the kernels of one weight format -- four translation units compile side by side.)
#pragma once
#include <cstdio>
#include <cstdlib>

#include "mnb_mfma16_common.hip.h"

#if defined(MNB_STAMPS)
// Calibration builds (-DMNB_STAMPS): every wavefront of the direct decode kernels reads the constant 100 MHz counter
// at seven points of its life and leaves the readings in a device array, [workgroup][wavefront][point], which
// MnbCalibrationReadStamps_<unit> (MNB_STAMPS_READER below, one per translation unit that holds kernels) copies out: 0 entry, 1 all loads of the first chunks issued, 2 first chunk computed,
// 3 last chunk computed, 4 partial sums written to LDS, 5 past the barrier, 6 sums read back and stores issued.
// (The scheduling barriers around a reading keep it where it is written; they also keep the load block in front of
// the arithmetic, which the product build leaves to the scheduler -- measured: no difference in time.)
constexpr int kStampPoints = 8, kStampWaves = 16, kStampGroups = 4096;
static __device__ unsigned long long mnb_stamps[kStampGroups * kStampWaves * kStampPoints];
#define MNB_STAMP_PARAM , unsigned long long* stamp
#define MNB_STAMP_ARG , stamp
#define MNB_STAMP(i)                                      \
  do {                                                    \
    __builtin_amdgcn_sched_barrier(0);                    \
    stamp[i] = __builtin_amdgcn_s_memrealtime();          \
    __builtin_amdgcn_sched_barrier(0);                    \
  } while (0)
#else
#define MNB_STAMP_PARAM
#define MNB_STAMP_ARG
#define MNB_STAMP(i)
#endif

namespace {

template <int BITS, bool HAS_ZP, int MODE>
__device__ __forceinline__ BConst bconst_of_mode() {
  if constexpr (MODE == 4) return make_bconst_bf16<HAS_ZP>();
  else return make_bconst<BITS, HAS_ZP>();
}

// One chunk: T column tiles x (4 k-groups) against the 16-row A operands af[].
// the B operand i of a lane's vector as raw magic halves (MODE 0)
template <int BITS>
__device__ __forceinline__ h8_t raw_operand(const uint32_t* wd, int i, const UnpackConsts& uc, const UnpackConsts2& uc2) {
  if constexpr (BITS == 4) return raw4(wd[i], uc);
  else if constexpr (BITS == 8) return raw8(wd[2 * i], wd[2 * i + 1]);
  else return raw2((i & 1) ? wd[i >> 1] >> 8 : wd[i >> 1], uc2);
}

template <int BITS, bool HAS_ZP, int MODE, int T>
__device__ __forceinline__ void compute_chunk(const ChunkRegs<BITS, T>& R, const h8_t* af, const BConst& bc,
                                              const UnpackConsts& uc, const UnpackConsts2& uc2, f4_t* y) {
  constexpr int NI = (128 / BITS) / 8;
  static_assert(BITS != 2 || MODE <= 1 || MODE == 6, "2-bit weights in their own width: fp16 models only");
#if defined(MNB_ABLATE_NO_MATH)
  // calibration builds: the loads are waited for and nothing is computed (what the arithmetic costs a launch)
#pragma unroll
  for (int t = 0; t < T; ++t) {
    asm volatile("; keep %0 %1 %2 %3 %4" ::"v"(R.w[t].x), "v"(R.w[t].y), "v"(R.w[t].z), "v"(R.w[t].w), "v"(R.m0[t]));
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) asm volatile("; keep %0" ::"v"(__builtin_bit_cast(u4_t, af[i])));
  return;
#endif
  if constexpr (MODE == 0 || MODE == 5 || MODE == 6) {
    // init[m] = -sum_k (off_k + zp) a[m][k] (no zero points) or -sum_k off_k a[m][k]; nc2[m] = -sum_k a[m][k].
    // The constant operands are the same in every lane, so every lane receives the value of its own rows.
    // MODE 6 (2-bit weights in blocks of 128): a chunk is 256 k and its halves of 128 (operands 0..3 and 4..7) lie in
    // different blocks, so each half has its own corrections, block sum and meta entry (m0, m1).
    static_assert(MODE != 6 || BITS == 2, "two blocks per chunk: 2-bit weights only");
    constexpr int SUB = MODE == 6 ? 2 : 1, PER = NI / SUB;
    const f4_t zero = f4_t{0.f, 0.f, 0.f, 0.f};
    f4_t init[SUB], nc2[SUB];
#pragma unroll
    for (int h = 0; h < SUB; ++h) {
      init[h] = zero;
      nc2[h] = zero;
#pragma unroll
      for (int i = h * PER; i < (h + 1) * PER; ++i)
        init[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], bc.off, init[h], 0, 0, 0);
      if constexpr (HAS_ZP) {
#pragma unroll
        for (int i = h * PER; i < (h + 1) * PER; ++i)
          nc2[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], bc.one, nc2[h], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const uint32_t wd[4] = {R.w[t].x, R.w[t].y, R.w[t].z, R.w[t].w};
#pragma unroll
      for (int h = 0; h < SUB; ++h) {
        float sf, zp;  // scale and zero point of the block
        if constexpr (MODE == 5) {
          sf = __uint_as_float(R.m0[t]);
          zp = __uint_as_float(R.z0[t]);
        } else {
          _Float16 sc, nz;
          decode_meta<BITS, HAS_ZP>(h == 0 ? R.m0[t] : R.m1[t], sc, nz);
          sf = (float)sc;
          zp = -(float)nz - 1024.0f;
        }
        f4_t d = init[h];
#pragma unroll
        for (int i = h * PER; i < (h + 1) * PER; ++i)
          d = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], raw_operand<BITS>(wd, i, uc, uc2), d, 0, 0, 0);
        if constexpr (HAS_ZP) {
#pragma unroll
          for (int r = 0; r < 4; ++r) y[t][r] = __builtin_fmaf(sf, __builtin_fmaf(zp, nc2[h][r], d[r]), y[t][r]);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) y[t][r] = __builtin_fmaf(sf, d[r], y[t][r]);
        }
      }
    }
  } else if constexpr (MODE == 4) {
    // MODE 0 on bfloat16: raw operands 128 + q, offsets and zero points removed through the correction MFMAs
    static_assert(MODE != 4 || BITS == 4, "8-bit weights do not fit a bfloat16 mantissa");
    const f4_t zero = f4_t{0.f, 0.f, 0.f, 0.f};
    f4_t init = zero, nc2 = zero;
#pragma unroll
    for (int i = 0; i < NI; ++i) init = mfma16_bf16(af[i], bc.off, init);
    if constexpr (HAS_ZP) {
#pragma unroll
      for (int i = 0; i < NI; ++i) nc2 = mfma16_bf16(af[i], bc.one, nc2);
    }
    uint32_t magic;
    asm("v_mov_b32 %0, 0x43004300" : "=v"(magic));  // two bfloat16 128.0 (held in a register: see UnpackConsts)
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const float sf = __uint_as_float(R.m0[t]);
      const uint32_t wd[4] = {R.w[t].x, R.w[t].y, R.w[t].z, R.w[t].w};
      f4_t d = init;
#pragma unroll
      for (int i = 0; i < NI; ++i) d = mfma16_bf16(af[i], raw4_bf16(wd[i], uc, magic), d);
      if constexpr (HAS_ZP) {
        const float zp = __uint_as_float(R.z0[t]);
#pragma unroll
        for (int r = 0; r < 4; ++r) y[t][r] = __builtin_fmaf(sf, __builtin_fmaf(zp, nc2[r], d[r]), y[t][r]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) y[t][r] = __builtin_fmaf(sf, d[r], y[t][r]);
      }
    }
  } else if constexpr (MODE >= 2) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const uint32_t wd[4] = {R.w[t].x, R.w[t].y, R.w[t].z, R.w[t].w};
      const float dzp = (float)(1 << (BITS - 1));
      const float s0 = __uint_as_float(R.m0[t]), s1 = BITS == 4 ? __uint_as_float(R.m1[t]) : s0;
      const float c0 = -(HAS_ZP ? __uint_as_float(R.z0[t]) : dzp) * s0;
      const float c1 = BITS == 4 ? -(HAS_ZP ? __uint_as_float(R.z1[t]) : dzp) * s1 : c0;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const bool second = (BITS == 4) && i >= 2;
        const h8_t b = BITS == 4 ? dequant_word_wide<BITS, MODE == 2>(wd[i], 0u, second ? s1 : s0, second ? c1 : c0)
                                 : dequant_word_wide<BITS, MODE == 2>(wd[(2 * i) & 3], wd[(2 * i + 1) & 3], s0, c0);
        if constexpr (MODE == 2)
          y[t] = mfma16_bf16(af[i], b, y[t]);
        else
          y[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], b, y[t], 0, 0, 0);
      }
    }
  } else {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const uint32_t wd[4] = {R.w[t].x, R.w[t].y, R.w[t].z, R.w[t].w};
      _Float16 s0, s1, nz0, nz1;
      decode_meta<BITS, HAS_ZP>(R.m0[t], s0, nz0);
      if constexpr (BITS == 4 || BITS == 2) {
        decode_meta<BITS, HAS_ZP>(R.m1[t], s1, nz1);
      } else {
        s1 = s0;
        nz1 = nz0;
      }
      const ZpH z0 = mnb_zp_h(nz0), z1 = mnb_zp_h(nz1);
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        h2_t d[4];
        // words 2, 3 of a 4-bit vector may belong to the next block; operands 4..7 of a 2-bit vector lie in the other
        // half of the chunk
        const bool second = (BITS == 4 && i >= 2) || (BITS == 2 && i >= 4);
        const ZpH& z = second ? z1 : z0;
        const h2_t s2 = mnb_h2(second ? s1 : s0);
        if constexpr (BITS == 2) {
          // -(256 + zp) and -(16 + zp) beside z.lo = -(1024 + zp) and z.hi = -(64 + zp); exact (integers below 2048)
          const _Float16 nz = second ? nz1 : nz0;
          const u4_t p = __builtin_bit_cast(u4_t, raw2((i & 1) ? wd[i >> 1] >> 8 : wd[i >> 1], uc2));
          d[0] = mnb_as_h2(p[0]) + z.lo;
          d[1] = mnb_as_h2(p[1]) + mnb_h2(nz + (_Float16)768.0f);
          d[2] = mnb_as_h2(p[2]) + z.hi;
          d[3] = mnb_as_h2(p[3]) + mnb_h2(nz + (_Float16)1008.0f);
        } else if constexpr (BITS == 4) {
          mnb_unpack4_h(wd[i], z, d);
        } else {
          mnb_unpack8_h(wd[2 * i], z, d);
          mnb_unpack8_h(wd[2 * i + 1], z, d + 2);
        }
        uint4 bw;
        bw.x = mnb_as_u32(d[0] * s2);
        bw.y = mnb_as_u32(d[1] * s2);
        bw.z = mnb_as_u32(d[2] * s2);
        bw.w = mnb_as_u32(d[3] * s2);
        y[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], __builtin_bit_cast(h8_t, bw), y[t], 0, 0, 0);
      }
    }
  }
  if constexpr (T == 1) {
    // With a single tile nothing separates the last matrix instruction from the first read of its result, and the
    // compiler sinks that read behind the branches of the chunk loop, where its hazard handling loses track of the
    // matrix instruction (seen as wrong rows 4 kq + 3).  Eight idle issue cycles cover the result latency
    // (the check in tests/test_isa_hazards.py scans the generated code for reads that come too early).
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 7");
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Reduce the per-wavefront tiles through LDS in wavefront order and write Y.
// Lane (j, kq), register r of tile t holds row 4*kq + r, column n0 + 16 t + j; only rows < M travel.
template <int T, int NW>
__device__ __forceinline__ void skinny_epilogue(const SkinnyParams& p, float* red, const f4_t* y, int wave, int lane,
                                                int64_t n0 MNB_STAMP_PARAM) {
  const int kq = lane >> 4;
#if defined(MNB_ABLATE_NO_REDUCE)
  // calibration builds: no exchange through LDS, no barrier; the first wavefront stores its own partial sums (what the
  // reduction costs a launch; the result is wrong)
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t n = n0 + t * 16 + (lane & 15);
        if (4 * kq + r < p.M && n < p.N) p.C[(int64_t)(4 * kq + r) * p.ldc + n] = (_Float16)y[t][r];
      }
  }
  return;
#endif
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (4 * kq + r < p.M) red[(wave * T * 4 + t * 4 + r) * 64 + lane] = y[t][r];
  MNB_STAMP(4);
  __syncthreads();
  MNB_STAMP(5);
  reduce_and_store_tiles<T, NW>(p, red, 0, n0);
  MNB_STAMP(6);
}

// ---- activations through LDS for 4 < M <= 16 -----------------------------------------------------------------------
// Lane (j, kq) needs 16 bytes of row j at a 64-byte stride between the kq: read straight from A, one load
// instruction of a wavefront touches two cache lines per row -- 8 lines for up to four rows, 32 for sixteen -- and the
// vector cache looks lines up one after the other.  For more than four rows a wavefront therefore reads its chunk of
// A row-contiguously (64 lanes x 16 bytes = 4 rows x 256 bytes: 8 lines per instruction whatever M is), passes it
// through a private 4 KiB of LDS and picks its operands up from there.  No barrier is involved: the region belongs
// to one wavefront and LDS executes a wavefront's accesses in order.  16-byte pieces are XOR-swizzled with the row
// so that both the row-contiguous writes and the operand reads are free of bank conflicts.
// Up to four rows take the same road for another reason: read straight from A, a chunk costs a wavefront one load
// instruction per operand (four for 4-bit weights) that all fetch the same few bytes sixteen times over, and on
// single- and two-tile slabs those instructions outnumber the weight loads and fill the memory pipeline (measured
// without them: N = 4096, K = 14336 10.4 -> 8.7 us at one row, 11.3 -> 8.8 us at four).  With ROWS = 4 one
// instruction fetches the chunk of all four rows (two for 2-bit weights) and LDS hands the operands out.
template <int BITS, int ROWS = 16>
struct AStage {
  static constexpr int GK = 128 / BITS, NI = GK / 8;
  static constexpr int PIECES = 4 * NI;     // 16-byte pieces per row of a chunk
  static constexpr int RPI = 64 / PIECES;   // rows per load instruction; 16 / RPI == NI instructions
  static constexpr int LOADS = (ROWS + RPI - 1) / RPI;  // load instructions per chunk
  static constexpr int HELD = LOADS * RPI < 16 ? LOADS * RPI : 16;  // rows that pass through LDS
  static __device__ __forceinline__ int swz(int row) { return PIECES == 16 ? row : (row >> 1); }

  // global -> registers: g[I] = piece (lane % PIECES) of row I * RPI + lane / PIECES (rows >= M re-read row M - 1)
  static __device__ __forceinline__ void fetch(const SkinnyParams& p, int c, int lane, h8_t* g) {
    const int piece = lane % PIECES, r0 = lane / PIECES;
#pragma unroll
    for (int I = 0; I < LOADS; ++I) {
      int row = I * RPI + r0;
      row = row < p.M ? row : p.M - 1;
      g[I] = *reinterpret_cast<const h8_t*>(p.A + (int64_t)row * p.lda + (int64_t)c * 4 * GK + piece * 8);
    }
  }
  // registers -> LDS -> operands of lane (j, kq); rows the matrix instruction has beyond those held repeat them
  // (they are never stored)
  static __device__ __forceinline__ void pass(h8_t* mine, const h8_t* g, int lane, h8_t* af) {
    const int piece = lane % PIECES, r0 = lane / PIECES;
    const int j = (lane & 15) % HELD, kq = lane >> 4;
#pragma unroll
    for (int I = 0; I < LOADS; ++I) {
      const int row = I * RPI + r0;
      mine[row * PIECES + (piece ^ swz(row))] = g[I];
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      // the 16-byte piece of the row's chunk that holds operand i of lane quarter kq (2-bit: mnb_w2_k)
      const int piece = BITS == 2 ? (i >> 2) * 16 + kq * 4 + (i & 3) : kq * NI + i;
      af[i] = mine[j * PIECES + (piece ^ swz(j))];
    }
  }
};

// ---- direct variants: A operands from global memory (16-byte aligned rows), no barrier before the end -----------
// The chunk pipeline of a wavefront; `load_w(c, R)` issues the weight and meta loads of chunk c.
// CPW = chunks per wavefront when that is 1 or 2 for every wavefront (chunks == CPW * NW): everything is loaded up
// front in straight-line code, so the compiler's s_waitcnt counts are exact and each tile is processed as soon as
// its own vector has landed.  CPW = 0: general loop with two chunks in flight.
template <int BITS, bool HAS_ZP, int MODE, int T, int NW, int CPW, int A_LDS, class LoadW>
__device__ __forceinline__ void skinny_chunks(const SkinnyParams& p, unsigned char* smem, int wave, int lane,
                                              const LoadW& load_w, f4_t* y MNB_STAMP_PARAM) {
  constexpr int GK = 128 / BITS;
  constexpr int NI = GK / 8;
  using Stage = AStage<BITS, A_LDS == 0 ? 16 : A_LDS>;  // A_LDS: rows of a chunk that pass through LDS (4, 8, 16), 0 = operands straight from A
  const int j = lane & 15, kq = lane >> 4;
  const int arow = j < p.M ? j : p.M - 1;  // rows >= M of the MFMA A operand re-read row M-1: they are never stored
  // first k of the lane's operands inside a chunk: kq GK, or for 2-bit vectors 32 kq in each half of the chunk
  const _Float16* arow_ptr = p.A + (int64_t)arow * p.lda + kq * (BITS == 2 ? 32 : GK);
  h8_t* mine = reinterpret_cast<h8_t*>(smem) + wave * (16 * Stage::PIECES);  // A_LDS only
  const BConst bconst = bconst_of_mode<BITS, HAS_ZP, MODE>();
  const UnpackConsts uc = make_unpack_consts();
  const UnpackConsts2 uc2 = make_unpack_consts2();  // (2-bit weights; unused moves are dropped)

  // the activation loads of chunk c: the operands themselves, or the row-contiguous pieces that pass through LDS
  auto fetch_a = [&](int c, h8_t* a) {
    if constexpr (A_LDS != 0) {
      Stage::fetch(p, c, lane, a);
    } else {
#if defined(MNB_ABLATE_NO_A_LOADS)
      // calibration builds: no activation loads (what they cost a launch; the result is wrong)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const uint32_t v = 0x3c003c00u + (uint32_t)c;
        a[i] = __builtin_bit_cast(h8_t, u4_t{v, v, v, v});
      }
#else
#pragma unroll
      for (int i = 0; i < NI; ++i)
        a[i] = *reinterpret_cast<const h8_t*>(arow_ptr + (int64_t)c * 4 * GK +
                                              (BITS == 2 ? (i >> 2) * 128 + (i & 3) * 8 : 8 * i));
#endif
    }
  };
  auto run = [&](const ChunkRegs<BITS, T>& R, const h8_t* a) {
    if constexpr (A_LDS != 0) {
      h8_t af[NI];
      Stage::pass(mine, a, lane, af);
      compute_chunk<BITS, HAS_ZP, MODE, T>(R, af, bconst, uc, uc2, y);
    } else {
      compute_chunk<BITS, HAS_ZP, MODE, T>(R, a, bconst, uc, uc2, y);
    }
  };

  if constexpr (CPW > 0) {
    ChunkRegs<BITS, T> R[CPW];
    h8_t a[CPW][NI];
#pragma unroll
    for (int q = 0; q < CPW; ++q) fetch_a(wave + q * NW, a[q]);
#pragma unroll
    for (int q = 0; q < CPW; ++q) load_w(wave + q * NW, R[q]);
    MNB_STAMP(1);
    if constexpr (A_LDS != 0) {
      h8_t af[CPW][NI];
#pragma unroll
      for (int q = 0; q < CPW; ++q) Stage::pass(mine, a[q], lane, af[q]);
#pragma unroll
      for (int q = 0; q < CPW; ++q) compute_chunk<BITS, HAS_ZP, MODE, T>(R[q], af[q], bconst, uc, uc2, y);
    } else {
#pragma unroll
      for (int q = 0; q < CPW; ++q) {
        compute_chunk<BITS, HAS_ZP, MODE, T>(R[q], a[q], bconst, uc, uc2, y);
        if (q == 0) MNB_STAMP(2);
      }
    }
    MNB_STAMP(3);
  } else if constexpr (T <= 2 || (BITS == 4 && NW <= 8)) {
    // Two chunks in flight.  Loads under a run-time condition would leave the compiler unable to count the
    // outstanding loads at the join, and every wait of the loop would then be for all of them, the prefetch issued
    // a moment earlier included.  So the steady state and each possible tail are straight-line code, and the two
    // loads in front of the loop are clamped to the last chunk instead of skipped (valid memory, not used).
    ChunkRegs<BITS, T> R0, R1;
    h8_t a0[NI], a1[NI];
    auto load = [&](int c, h8_t* a, ChunkRegs<BITS, T>& R) {
      __builtin_amdgcn_sched_barrier(0);  // the loads stay between the two chunks they are written between
      fetch_a(c, a);
      load_w(c, R);
      __builtin_amdgcn_sched_barrier(0);
    };
    const int last = p.chunks - 1;
    const int own = wave < p.chunks ? (p.chunks - wave + NW - 1) / NW : 0;  // chunks of this wavefront
    int c = wave;
    load(min(c, last), a0, R0);
    load(min(c + NW, last), a1, R1);
    int q = 0;
    for (; q + 3 < own; q += 2, c += 2 * NW) {
      run(R0, a0);
      load(c + 2 * NW, a0, R0);
      run(R1, a1);
      load(c + 3 * NW, a1, R1);
    }
    const int left = own - q;  // 0 .. 3
    if (left == 3) {
      run(R0, a0);
      load(c + 2 * NW, a0, R0);
      run(R1, a1);
      run(R0, a0);
    } else if (left == 2) {
      run(R0, a0);
      run(R1, a1);
    } else if (left == 1) {
      run(R0, a0);
    }
  } else {
    // Wide slabs keep the loop with conditional prefetches where registers are short: the straight-line form needs
    // 30-50 registers more, which 16 wavefronts do not have (measured 11 % slower for T = 4; 2-9 % faster for
    // T = 1, 2).  Workgroups of four or eight wavefronts have them: 4-bit weights gain 6-7 % there (N = 28672,
    // K = 4096 14.6 -> 13.6 us at one row, 15.4 -> 14.5 at eight, blocks of 32 17.7 -> 16.7; N = 14336, K = 8192
    // 13.5 -> 12.6 us), 8-bit weights lose 2-5 % (23.0 -> 23.5 us) and stay here.
    ChunkRegs<BITS, T> R0, R1;
    h8_t a0[NI], a1[NI];
    int c = wave;
    if (c < p.chunks) {
      fetch_a(c, a0);
      load_w(c, R0);
    }
    if (c + NW < p.chunks) {
      fetch_a(c + NW, a1);
      load_w(c + NW, R1);
    }
    for (; c < p.chunks; c += 2 * NW) {
      run(R0, a0);
      if (c + 2 * NW < p.chunks) {
        fetch_a(c + 2 * NW, a0);
        load_w(c + 2 * NW, R0);
      }
      if (c + NW < p.chunks) {
        run(R1, a1);
        if (c + 3 * NW < p.chunks) {
          fetch_a(c + 3 * NW, a1);
          load_w(c + 3 * NW, R1);
        }
      }
    }
  }
  if constexpr (A_LDS != 0) __syncthreads();  // the reduction buffer overlays the staging regions of all wavefronts
}

// What a wavefront needs to issue its first loads comes as leading scalar kernel arguments, which the build asks the
// compiler to have preloaded into SGPRs when the wavefront starts (kernarg preload: no scalar load, about 0.4 us, in
// front of the first weight load); everything else stays in the parameter block and is fetched where it is used.
#define MNB_SKINNY_HOT_PARAMS                                                                                 \
  const uint4 *hot_W, int64_t hot_Npad, const _Float16 *hot_A, int64_t hot_lda, const uint8_t *hot_meta, int hot_M, \
      int hot_chunks, int hot_bs_shift
#define MNB_SKINNY_HOT_ARGS(p) (p).W, (p).Npad, (p).A, (p).lda, (p).meta, (p).M, (p).chunks, (p).bs_shift

__device__ __forceinline__ SkinnyParams with_hot_params(SkinnyParams p, MNB_SKINNY_HOT_PARAMS) {
  p.W = hot_W;
  p.Npad = hot_Npad;
  p.A = hot_A;
  p.lda = hot_lda;
  p.meta = hot_meta;
  p.M = hot_M;
  p.chunks = hot_chunks;
  p.bs_shift = hot_bs_shift;
  return p;
}
#define MNB_SKINNY_HOT_NAMES hot_W, hot_Npad, hot_A, hot_lda, hot_meta, hot_M, hot_chunks, hot_bs_shift

template <int BITS, bool HAS_ZP, int MODE, int T, int NW, int CPW, int A_LDS>
__global__ void __launch_bounds__(NW * 64) mnb_skinny_direct_kernel(MNB_SKINNY_HOT_PARAMS, SkinnyParams rest) {
  const SkinnyParams p = with_hot_params(rest, MNB_SKINNY_HOT_NAMES);
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kq = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * (16 * T);
  const int64_t col0 = n0 + (lane & 15);
  f4_t y[T];
#pragma unroll
  for (int t = 0; t < T; ++t) y[t] = f4_t{0.f, 0.f, 0.f, 0.f};
#if defined(MNB_STAMPS)
  unsigned long long stamp[kStampPoints] = {};
  MNB_STAMP(0);
#endif
  skinny_chunks<BITS, HAS_ZP, MODE, T, NW, CPW, A_LDS>(
      p, smem, wave, lane,
      [&](int c, ChunkRegs<BITS, T>& R) { load_chunk<BITS, HAS_ZP, MODE, T>(p, c, kq, col0, R); }, y MNB_STAMP_ARG);
  skinny_epilogue<T, NW>(p, reinterpret_cast<float*>(smem), y, wave, lane, n0 MNB_STAMP_ARG);
#if defined(MNB_STAMPS)
  if (lane == 0 && blockIdx.x < kStampGroups && wave < kStampWaves)
#pragma unroll
    for (int i = 0; i < kStampPoints; ++i)
      mnb_stamps[((size_t)blockIdx.x * kStampWaves + wave) * kStampPoints + i] = stamp[i];
#endif
}

// ---- direct variant for slabs of three tiles ----------------------------------------------------------------------
// A workgroup's run time is a fixed part plus a part proportional to its tiles, and hardly depends on how many of the
// 256 compute units are busy, so 513..768 column tiles are best cut into slabs of three (at most 256 workgroups, one
// round) rather than two (up to 384): N = 12288 runs 12 % faster.  Slabs of 48 columns are not aligned to the 64-column
// groups in which the meta entries of a lane's tiles are adjacent, so the tiles are addressed one by one.
// (Slabs with half a tile at the end - 56 columns for N = 14336, which would put exactly one workgroup on every
// compute unit - were measured too: the half tile costs the instructions of a whole one, and the run time did not
// improve.)
template <int BITS, bool HAS_ZP, int MODE, int T, int NW, int CPW, int A_LDS>
__global__ void __launch_bounds__(NW * 64) mnb_skinny_slab_kernel(MNB_SKINNY_HOT_PARAMS, SkinnyParams rest) {
  const SkinnyParams p = with_hot_params(rest, MNB_SKINNY_HOT_NAMES);
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, kq = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * (16 * T);
  int32_t colw[T], mcol[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int64_t col = n0 + 16 * t + j;
    col = col < p.Npad ? col : p.Npad - 1;  // beyond the matrix: padding, never stored
    colw[t] = (int32_t)col;
    mcol[t] = (int32_t)mnb_meta_col(col);
  }
  f4_t y[T];
#pragma unroll
  for (int t = 0; t < T; ++t) y[t] = f4_t{0.f, 0.f, 0.f, 0.f};
#if defined(MNB_STAMPS)
  unsigned long long stamp[kStampPoints] = {};  // (only the kernel above keeps its readings)
#endif
  skinny_chunks<BITS, HAS_ZP, MODE, T, NW, CPW, A_LDS>(
      p, smem, wave, lane,
      [&](int c, ChunkRegs<BITS, T>& R) { load_chunk_cols<BITS, HAS_ZP, MODE, T>(p, c, kq, colw, mcol, R); },
      y MNB_STAMP_ARG);
  skinny_epilogue<T, NW>(p, reinterpret_cast<float*>(smem), y, wave, lane, n0 MNB_STAMP_ARG);
}

// ---- staged variant: any alignment of A; rows staged in LDS phase by phase -------------------------------------
template <int BITS, bool HAS_ZP, int MODE, int T, int NW>
__global__ void __launch_bounds__(NW * 64) mnb_skinny_staged_kernel(SkinnyParams p) {
  constexpr int GK = 128 / BITS;  // k per 16-byte vector: 32 or 16
  constexpr int NI = GK / 8;      // MFMAs per vector: 4 or 2
  constexpr int CK = 4 * GK;      // k per chunk: 128 or 64
  extern __shared__ __align__(16) unsigned char smem[];
  _Float16* As = reinterpret_cast<_Float16*>(smem);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, kq = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * (16 * T);
  const int64_t col0 = n0 + j;
  const int row_stride = p.phase_chunks * CK + kLdsPad;  // halves
  const int arow = j & (p.mtr - 1);                      // staged row this lane feeds to the MFMA A operand

  f4_t y[T];
#pragma unroll
  for (int t = 0; t < T; ++t) y[t] = f4_t{0.f, 0.f, 0.f, 0.f};
  const BConst bconst = bconst_of_mode<BITS, HAS_ZP, MODE>();
  const UnpackConsts uc = make_unpack_consts();
  const UnpackConsts2 uc2 = make_unpack_consts2();

  for (int ph0 = 0; ph0 < p.chunks; ph0 += p.phase_chunks) {
    const int ph1 = min(ph0 + p.phase_chunks, p.chunks);
    // this wavefront's first weight loads go out before the staging barrier
    const int c_first = ph0 + wave;
    ChunkRegs<BITS, T> Rn;
    if (c_first < ph1) load_chunk<BITS, HAS_ZP, MODE, T>(p, c_first, kq, col0, Rn);
    // stage rows [0, mtr) of A for k in [ph0*CK, ph1*CK): zero beyond K, rows >= M repeat row M-1
    __syncthreads();
    {
      const int kbase = ph0 * CK;
      const int kext = (ph1 - ph0) * CK;
      for (int i = threadIdx.x; i < p.mtr * kext; i += NW * 64) {
        const int r = i / kext, kk = i % kext;
        const int k = kbase + kk;
        const int rr = r < p.M ? r : p.M - 1;
        As[r * row_stride + kk] = (k < p.K) ? p.A[(int64_t)rr * p.lda + k] : (_Float16)0.0f;
      }
    }
    __syncthreads();
    for (int c = c_first; c < ph1; c += NW) {
      const ChunkRegs<BITS, T> Rc = Rn;
      if (c + NW < ph1) load_chunk<BITS, HAS_ZP, MODE, T>(p, c + NW, kq, col0, Rn);
      h8_t af[NI];
      const _Float16* abase = As + arow * row_stride + ((c - ph0) * 4 + kq) * GK;
#pragma unroll
      for (int i = 0; i < NI; ++i) af[i] = *reinterpret_cast<const h8_t*>(abase + 8 * i);
      compute_chunk<BITS, HAS_ZP, MODE, T>(Rc, af, bconst, uc, uc2, y);
    }
  }
  __syncthreads();
#if defined(MNB_STAMPS)
  unsigned long long stamp[kStampPoints] = {};
#endif
  skinny_epilogue<T, NW>(p, reinterpret_cast<float*>(smem), y, wave, lane, n0 MNB_STAMP_ARG);
}

struct SkinnyPlan {
  int mode, t, nw, phase_chunks, mtr;
  int a_lds;   // rows of a chunk of the activations that pass through LDS: 0 (operands read straight from A), 4, 8 or 16
  size_t smem;
};

int pow2_ceil(int v) {
  int r = 1;
  while (r < v) r <<= 1;
  return r;
}

SkinnyPlan skinny_plan(const MnbLayout& L, int io, int64_t M, bool direct, int min_t) {
  SkinnyPlan pl;
  const int GK = L.group_k, CK = 4 * GK;
  const int chunks = (int)((L.K + CK - 1) / CK);
  // raw operands need every matrix instruction inside one block: a whole chunk, or half of a 2-bit chunk (mode 6)
  pl.mode = (L.bs >= CK) ? 0 : (L.bits == 2 && L.bs == 128) ? 6 : 1;
  if (const char* e = mnb_tuning_env("MNB_SKINNY_MODE")) pl.mode = e[0] == '1' ? 1 : pl.mode;  // calibration: exact halves
  if (io != kMnbIoModel) {  // fp32 meta entries: raw operands where a chunk lies inside a block, else exact weights
    const bool raw = L.bits == 4 && L.bs >= CK;
    pl.mode = io == kMnbIoBf16 ? (raw ? 4 : 2) : (raw ? 5 : 3);
    if (const char* e = mnb_tuning_env("MNB_SKINNY_WIDE_EXACT"))  // calibration: exact weights everywhere
      if (e[0] == '1') pl.mode = io == kMnbIoBf16 ? 2 : 3;
  }
  pl.mtr = pow2_ceil((int)M);
  // workgroups: as many column slabs as fill the chip; wide slabs (T = 4) amortise the A operands best
  const int64_t tiles = (L.N + 15) / 16;
  pl.t = tiles >= 800 ? 4 : tiles >= 320 ? 2 : 1;  // measured: N = 6144 prefers 2 (192 workgroups), N = 4096 prefers 1
  // wavefronts per workgroup: aim for >= 2 chunks per wavefront
  pl.nw = chunks >= 32 ? 16 : chunks >= 16 ? 8 : 4;
  // 2-bit chunks are 256 k, twice the arithmetic of the others: one per wavefront already pays (measured at K = 4096,
  // M = 1, blocks of 128: N = 14336 8.2 -> 7.3 us, N = 6144 5.6 -> 5.0 us; blocks of 64: 9.2 -> 8.0 us)
  if (L.bits == 2) pl.nw = chunks >= 16 ? 16 : chunks >= 8 ? 8 : 4;
  // More four-tile slabs than compute units: sixteen-wavefront workgroups run one per unit, in rounds that each pay
  // their own first-load latency and reduction, and the last round is partly empty.  Smaller workgroups share a unit
  // and overlap these (measured at K = 4096 and 8192, N = 20480 ... 57344, M = 1, 8, 16: 3-26 % faster; 4-bit
  // prefers four wavefronts with the general loop, 8-bit eight; up to 1.6 rounds two-tile slabs balance best).
  const int64_t slabs4 = (tiles + 3) / 4, cus = mnb_device_info().cus;
  if (direct && pl.nw == 16 && slabs4 > cus) {
    if (slabs4 * 5 <= cus * 8) {
      pl.t = 2;
      pl.nw = M >= 9 ? 4 : 8;
    } else {
      pl.nw = L.bits == 4 ? 4 : 8;
    }
  }
  const char* const plan_override = mnb_tuning_env("MNB_SKINNY_PLAN");  // calibration builds: "<T>,<NW>"
  if (const char* e = plan_override) {
    int t = 0, nw = 0;
    if (sscanf(e, "%d,%d", &t, &nw) == 2 && (t == 1 || t == 2 || t == 4) && (nw == 4 || nw == 8 || nw == 16)) {
      pl.t = t;
      pl.nw = nw;
    }
  }
  if (pl.t < min_t) pl.t = min_t;  // gate/up pairs live in one workgroup
  // three tiles per workgroup (slab kernel): one round of at most 256 workgroups where two tiles would need up to 384
  if (direct && min_t == 1 && tiles > 512 && tiles <= 768 && plan_override == nullptr) pl.t = 3;
  // Eight wavefronts of twice the chunks instead of sixteen (fp16 models; measured on K = 4096 ... 14336):
  //  * single-tile slabs (N < 5120), up to eight rows or K up to 64 chunks: 2-9 % (N = K = 4096 int4 M = 1:
  //    4.5 -> 4.1 us; 8-bit K >= 8192: 4-7 %);
  //  * two-tile slabs at K = 4096, 8-bit weights or raw 4-bit operands: 1-6 %, M = 1 even; three-tile slabs of raw
  //    4-bit operands at K = 4096 from four rows on: 0-10 % (at K = 8192 they lose 1-4 %);
  //  * raw 4-bit operands on slabs of two or four tiles with five to eight rows of A read straight from memory (two
  //    cache lines per row and load), and four-tile slabs with K >= 8192: 0-11 %, most with zero points.
  //  * raw 4-bit operands with zero points on four-tile slabs, up to four rows: the corrections of the zero points
  //    leave sixteen wavefronts short of registers, and eight run the straight-line chunk loop (K = 4096, blocks of
  //    128: N = 14336 at 1 / 2 / 4 rows 8.5 -> 7.9, 8.3 -> 7.9, 8.4 -> 8.1 us; N = 16384 9.0 -> 8.3; blocks of 256,
  //    N = 13312 8.0 -> 7.5; without zero points 7.8 / 7.9 us either way: the C2 plan stays).
  // Exact 4-bit operands (blocks of 32 and 64) on two-tile slabs do not gain.
  if (plan_override == nullptr && direct && pl.nw == 16 && pl.mode <= 1) {
    const bool raw4 = L.bits == 4 && pl.mode == 0;
    if (pl.t == 1 ? (M <= 8 || chunks <= 64)
                  : (pl.t == 2 && ((L.bits == 8 && chunks <= 64) || (raw4 && chunks <= 32))) ||
                        (pl.t == 3 && raw4 && chunks <= 32 && M >= 4) ||
                        (raw4 && (pl.t == 2 || pl.t == 4) && M <= 8 && (M >= 5 || (pl.t == 4 && chunks >= 64))) ||
                        (raw4 && pl.t == 4 && L.has_zp && M <= 4))
      pl.nw = 8;
  }
  // 16-bit models on fp32 entries: only raw operands on single-tile slabs with up to four rows gain (N = K = 4096
  // M = 1: 5.0 -> 4.6 us); every other shape of the sweep was equal or slower with eight wavefronts
  if (plan_override == nullptr && direct && pl.nw == 16 && (pl.mode == 4 || pl.mode == 5) && pl.t == 1 && M <= 4 &&
      chunks <= 32)
    pl.nw = 8;
  if (const char* e = mnb_tuning_env("MNB_SKINNY_NW")) {  // tuning override of the wavefront count alone
    const int nw = atoi(e);
    if (nw == 4 || nw == 8 || nw == 16) pl.nw = nw;
  }
  // Activations through LDS (see AStage) pay from nine rows on, for single-tile slabs from five (measured: at
  // M = 8 the wider slabs gain or lose a few per cent either way; at M = 16 everything gains 10-35 % except the
  // general loop of four-tile slabs).  The general loop needs one more operand set for it, which sixteen wavefronts
  // of 4-bit weights cannot hold in their 128 registers: those run with eight (K = 14336, M = 16: 20 -> 13 us).
  static const int a_lds_from = mnb_tuning_env("MNB_SKINNY_ALDS_FROM") ? atoi(mnb_tuning_env("MNB_SKINNY_ALDS_FROM")) : 5;
  const bool up_front = chunks == pl.nw || chunks == 2 * pl.nw;  // everything loaded before the first wait
  // (four-tile slabs have an LDS form where all chunks are loaded up front, and in the straight-line chunk loop of
  // 4-bit weights in workgroups of four or eight wavefronts)
  const bool t4_hook = !(mnb_tuning_env("MNB_SKINNY_T4LDS") && mnb_tuning_env("MNB_SKINNY_T4LDS")[0] == '0');
  // K beyond 4096 on four-tile slabs of 4-bit weights (fp16 models): sixteen wavefronts run the loop with conditional
  // prefetches, eight the straight-line one, with room for the LDS form.  Measured, N = 14336 unless noted:
  //   nine rows and more: K = 8192 at 12 / 16 rows 15.7 -> 14.2, 16.7 -> 14.6 us; K = 14336 at 16 rows 27.6 -> 23.2 us;
  //     exact operands (blocks of 64, N = 16384, K = 8192, 9 rows) 18.0 -> 16.7 us with eight wavefronts and 18.2 us
  //     with the LDS form on top, so they go without it;
  //   up to eight rows, exact operands (blocks of 32 and 64; N = 14336 and 16384, K = 8192, 11008, 14336, 1 / 4 / 8
  //     rows: 36 cases): 2-9 % faster in every one (K = 8192, blocks of 64: 16.1 -> 14.8, 16.6 -> 15.2, 17.1 -> 16.0 us);
  //   up to eight rows, raw operands below 64 chunks (K = 5120 ... 7168): 0-5 % (K = 6144: 10.7 -> 10.3 us, four rows
  //     11.1 -> 10.5 us).
  if (t4_hook && direct && L.bits == 4 && pl.t == 4 && pl.nw == 16 && !up_front && pl.mode <= 1) pl.nw = 8;
  // Three-tile slabs likewise up to 64 chunks (N = 11008, K = 8192: 12.0 -> 11.0 us, four rows 12.8 -> 11.4, blocks of
  // 64 15.8 -> 13.2; N = 12288, blocks of 32, four rows 17.0 -> 15.6; N = 9216, K = 6144 9.4 -> 8.5 us); beyond that
  // sixteen wavefronts keep more chunks in flight (N = 12288, K = 14336: 19.6 us against 22.6 with eight).
  if (t4_hook && direct && L.bits == 4 && pl.t == 3 && pl.nw == 16 && !up_front && pl.mode <= 1 && chunks <= 64) pl.nw = 8;
  const bool t4_loop_lds = t4_hook && L.bits == 4 && pl.nw <= 8 && pl.mode == 0 && (M >= 13 || chunks > 32);
  pl.a_lds = direct && M >= a_lds_from && (M >= 9 || pl.t == 1) && (up_front || pl.t < 4 || t4_loop_lds) ? 16 : 0;
  if (pl.a_lds && !up_front && pl.nw == 16 && L.bits == 4) pl.nw = 8;
  // the fp32 scales and zero points of modes 2 to 4 do not fit the 128 registers of sixteen wavefronts in the general loop
  if (pl.mode >= 2 && !up_front && pl.nw == 16) pl.nw = 8;
  // Up to eight rows on single- and two-tile slabs: read straight from A, a chunk costs a wavefront one load
  // instruction per operand, and on these slabs those loads outnumber the weight loads and fill the memory pipeline.
  // AStage with four or eight rows fetches the chunk of all rows with one or two instructions and hands the operands
  // out through LDS; bit-identical results.  Measured, weights from HBM, zero points, 4-bit blocks of 128 unless noted:
  //   N = 4096, K = 14336   1 / 2 / 4 rows 10.4 / 10.6 / 11.3 -> 9.0 us; 5 / 8 rows (were sixteen rows through LDS)
  //                         10.7 -> 9.6, 10.8 -> 10.2; blocks of 64 11.9 -> 9.9 (8 rows 12.1 -> 11.0); 2-bit 9.3 -> 7.3
  //                         (8 rows 11.0 -> 9.0); 8-bit 13.8 -> 13.5 (4 rows 14.3 -> 13.6, 8 rows 14.3 -> 14.1)
  //   N = 4096, K = 11008   8.6 -> 7.5 (8 rows 9.0 -> 8.6)
  //   N = K = 4096          4.6 -> 4.3 (4 rows 5.2 -> 4.5, 8 rows 5.0 -> 4.7); blocks of 32 5.3 -> 5.1
  //   N = 6144, K = 4096    5.6 -> 5.2 (4 rows 5.8 -> 5.2, 8 rows 6.3 -> 5.7); 8-bit 6.8 -> 6.7 (8 rows 7.7 -> 7.2)
  //   raw 4-bit operands over more than 32 chunks on two-tile slabs, which ran sixteen wavefronts (no LDS form in
  //   their 128 registers), with eight: N = K = 8192 8.8 -> 8.5 (4 rows 9.1 -> 8.7), N = 6144 8.0 -> 7.3,
  //   N = 5120, K = 14336 12.0 -> 10.2, N = 8192, K = 28672 24.0 -> 23.4.
  // Four-tile slabs do not gain (C2 without any activation load: 7.8 -> 7.7 us): there the weight loads dominate.
  const bool few_rows = !(mnb_tuning_env("MNB_SKINNY_A4") && mnb_tuning_env("MNB_SKINNY_A4")[0] == '0');
  if (few_rows && direct && pl.t <= 2 && M <= 8) {
    const bool no_lds_form = L.bits == 4 && pl.nw == 16 && !up_front;  // (the general loop of sixteen 4-bit wavefronts)
    if (pl.a_lds == 16) {
      pl.a_lds = 8;  // (single-tile slabs, five to eight rows)
    } else if (M <= 4) {
      if (no_lds_form && pl.mode == 0) pl.nw = 8;
      if (!(L.bits == 4 && pl.nw == 16 && !up_front)) pl.a_lds = 4;
    } else if (!no_lds_form) {
      pl.a_lds = 8;  // (two-tile slabs, five to eight rows)
    }
  }
  // Three-tile slabs, and four-tile slabs whose chunks are all loaded up front (the only LDS forms they have), from
  // two rows on: the activation loads cost less there, but still N = 11008, K = 4096 8.0 -> 6.8 us at one row and
  // N = 14336 9.0 -> 8.3 us at four when they are left out altogether.
  if (few_rows && direct && M <= 8 && !pl.a_lds) {
    const bool all_rows_of_c2 = mnb_tuning_env("MNB_SKINNY_A4") && mnb_tuning_env("MNB_SKINNY_A4")[0] == '3';
    if (pl.t == 3 && !(L.bits == 4 && pl.nw == 16 && !up_front)) pl.a_lds = M <= 4 ? 4 : 8;
    // (in the chunk loop of four-tile slabs the forms for up to eight rows do not pay: N = 28672, K = 4096 at 2 / 4 / 6
    // rows 13.8 -> 14.1, 14.1 -> 14.2, 14.1 -> 14.3 us, at 8 rows 14.7 -> 14.3 on one box and 14.6 -> 15.5 on another)
    // (2-bit weights take eight activation loads per chunk when read straight from A: one row gains too - N = 14336,
    // K = 4096, blocks of 128 7.4 -> 6.2 us, blocks of 256 6.8 -> 6.1, N = 16384 7.6 -> 6.5, K = 2048 5.6 -> 5.1)
    if (pl.t == 4 && up_front && (M >= 2 || L.bits == 2 || all_rows_of_c2)) pl.a_lds = M <= 4 ? 4 : 8;
  }
  // LDS: staged A rows (<= 48 KiB per phase) and, afterwards, the reduction buffer (<= 64 KiB)
  const int max_phase = (48 * 1024 / 2 / pl.mtr - kLdsPad) / CK;  // >= 11 chunks for 16 rows
  pl.phase_chunks = chunks < max_phase ? chunks : max_phase;
  if (!direct) pl.nw = 4;
  const size_t a_bytes = direct ? 0 : (size_t)pl.mtr * (pl.phase_chunks * CK + kLdsPad) * 2;
  const size_t red_bytes = (size_t)pl.nw * pl.t * 4 * 64 * 4;
  pl.smem = a_bytes > red_bytes ? a_bytes : red_bytes;
  if (pl.a_lds) {
    const size_t stage_bytes = (size_t)pl.nw * GK * 128;  // 16 rows x one chunk of halves per wavefront
    if (stage_bytes > pl.smem) pl.smem = stage_bytes;
  }
  return pl;
}

// the LDS form of a launch for the rows the plan passes through LDS (4, 8 or 16)
#define MNB_LDS_ROWS(LAUNCH, NW_, CPW_) \
  do {                                  \
    if (pl.a_lds == 4)                  \
      LAUNCH(NW_, CPW_, 4);             \
    else if (pl.a_lds == 8)             \
      LAUNCH(NW_, CPW_, 8);             \
    else                                \
      LAUNCH(NW_, CPW_, 16);            \
  } while (0)

template <int BITS, bool HAS_ZP, int MODE, int T>
hipError_t launch_slab(const SkinnyParams& p, const SkinnyPlan& pl, hipStream_t s) {
  constexpr int CW = 16 * T;
  dim3 grid((unsigned)((p.N + CW - 1) / CW));
  const int cpw = (p.chunks == pl.nw) ? 1 : (p.chunks == 2 * pl.nw) ? 2 : 0;
  // the plan never asks for the LDS route in the general loop of sixteen wavefronts on 4-bit weights: not instantiated
  if (pl.a_lds && cpw == 0 && BITS == 4 && pl.nw == 16) return hipErrorInvalidConfiguration;
  if (MODE >= 2 && cpw == 0 && pl.nw == 16) return hipErrorInvalidConfiguration;  // (nor the fp32-entry modes at all)
#define MNB_SLAB_LAUNCH(NW_, CPW_, LDS_) \
  mnb_skinny_slab_kernel<BITS, HAS_ZP, MODE, T, NW_, CPW_, LDS_>                  \
      <<<grid, dim3(NW_ * 64), pl.smem, s>>>(MNB_SKINNY_HOT_ARGS(p), p)
#define MNB_SLAB_CPW(NW_)                                           \
  do {                                                              \
    if (pl.a_lds) {                                                 \
      if (cpw == 1)                                                 \
        MNB_LDS_ROWS(MNB_SLAB_LAUNCH, NW_, 1);                      \
      else if (cpw == 2)                                            \
        MNB_LDS_ROWS(MNB_SLAB_LAUNCH, NW_, 2);                      \
      else if constexpr (!(BITS == 4 && NW_ == 16))                 \
        MNB_LDS_ROWS(MNB_SLAB_LAUNCH, NW_, 0);                      \
    } else {                                                        \
      if (cpw == 1)                                                 \
        MNB_SLAB_LAUNCH(NW_, 1, 0);                                 \
      else if (cpw == 2)                                            \
        MNB_SLAB_LAUNCH(NW_, 2, 0);                                 \
      else if constexpr (!(MODE >= 2 && NW_ == 16))                 \
        MNB_SLAB_LAUNCH(NW_, 0, 0);                                 \
    }                                                               \
  } while (0)
  switch (pl.nw) {
    case 16: MNB_SLAB_CPW(16); break;
    case 8: MNB_SLAB_CPW(8); break;
    default: MNB_SLAB_CPW(4); break;
  }
#undef MNB_SLAB_CPW
#undef MNB_SLAB_LAUNCH
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP, int MODE, int T>
hipError_t launch_t(const SkinnyParams& p, const SkinnyPlan& pl, hipStream_t s) {
  dim3 grid((unsigned)((p.N + 16 * T - 1) / (16 * T)));
  if (p.a_vec_ok) {
    const int cpw = (p.chunks == pl.nw) ? 1 : (p.chunks == 2 * pl.nw) ? 2 : 0;
    // not instantiated, never planned: LDS route in the general loop of four-tile slabs or of sixteen 4-bit wavefronts
    if (pl.a_lds && cpw == 0 && ((T == 4 && !(BITS == 4 && pl.nw <= 8)) || (BITS == 4 && pl.nw == 16)))
      return hipErrorInvalidConfiguration;
    if (MODE >= 2 && cpw == 0 && pl.nw == 16) return hipErrorInvalidConfiguration;  // (nor the fp32-entry modes at all)
#define MNB_SKINNY_LAUNCH(NW_, CPW_, LDS_) \
  mnb_skinny_direct_kernel<BITS, HAS_ZP, MODE, T, NW_, CPW_, LDS_>                \
      <<<grid, dim3(NW_ * 64), pl.smem, s>>>(MNB_SKINNY_HOT_ARGS(p), p)
#define MNB_SKINNY_CPW(NW_)                                         \
  do {                                                              \
    if (pl.a_lds) {                                                 \
      if (cpw == 1)                                                 \
        MNB_LDS_ROWS(MNB_SKINNY_LAUNCH, NW_, 1);                    \
      else if (cpw == 2)                                            \
        MNB_LDS_ROWS(MNB_SKINNY_LAUNCH, NW_, 2);                    \
      else if constexpr (!(BITS == 4 && NW_ == 16) && (T < 4 || (BITS == 4 && NW_ <= 8))) \
        MNB_LDS_ROWS(MNB_SKINNY_LAUNCH, NW_, 0);                    \
    } else {                                                        \
      if (cpw == 1)                                                 \
        MNB_SKINNY_LAUNCH(NW_, 1, 0);                               \
      else if (cpw == 2)                                            \
        MNB_SKINNY_LAUNCH(NW_, 2, 0);                               \
      else if constexpr (!(MODE >= 2 && NW_ == 16))                 \
        MNB_SKINNY_LAUNCH(NW_, 0, 0);                               \
    }                                                               \
  } while (0)
    switch (pl.nw) {
      case 16: MNB_SKINNY_CPW(16); break;
      case 8: MNB_SKINNY_CPW(8); break;
      default: MNB_SKINNY_CPW(4); break;
    }
#undef MNB_SKINNY_CPW
#undef MNB_SKINNY_LAUNCH
  } else {
    // rare: A not 16-byte aligned or K not a multiple of 8 -- one configuration is enough
    if constexpr (BITS != 2) mnb_skinny_staged_kernel<BITS, HAS_ZP, MODE, T, 4><<<grid, dim3(256), pl.smem, s>>>(p);
    else return hipErrorInvalidValue;  // (the native 2-bit copy is only taken with aligned activations)
  }
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP, int MODE>
hipError_t launch_mode(const SkinnyParams& p, const SkinnyPlan& pl, hipStream_t s) {
  if (pl.t == 3) return launch_slab<BITS, HAS_ZP, MODE, 3>(p, pl, s);  // offered to the direct variant only
  switch (pl.t) {
    case 4: return launch_t<BITS, HAS_ZP, MODE, 4>(p, pl, s);
    case 2: return launch_t<BITS, HAS_ZP, MODE, 2>(p, pl, s);
    default: return launch_t<BITS, HAS_ZP, MODE, 1>(p, pl, s);
  }
}

template <int BITS, bool HAS_ZP>
hipError_t launch_zp(const SkinnyParams& p, const SkinnyPlan& pl, hipStream_t s) {
  if (pl.mode == 4) {
    if constexpr (BITS == 4) return launch_mode<BITS, HAS_ZP, 4>(p, pl, s);
    else return hipErrorInvalidValue;
  }
  if (pl.mode == 5) {
    if constexpr (BITS == 4 && HAS_ZP) return launch_mode<BITS, HAS_ZP, 5>(p, pl, s);
    else return hipErrorInvalidValue;
  }
  if (pl.mode == 2) {
    if constexpr (BITS != 2) return launch_mode<BITS, HAS_ZP, 2>(p, pl, s);
    else return hipErrorInvalidValue;  // (2-bit weights in their own width: fp16 models only)
  }
  if (pl.mode == 3) {
    if constexpr (BITS == 4 && HAS_ZP) return launch_mode<BITS, HAS_ZP, 3>(p, pl, s);
    else return hipErrorInvalidValue;  // zero points in the activation type: 4-bit with zero points
  }
  if (pl.mode == 6) {
    if constexpr (BITS == 2) return launch_mode<BITS, HAS_ZP, 6>(p, pl, s);
    else return hipErrorInvalidValue;
  }
  return pl.mode == 0 ? launch_mode<BITS, HAS_ZP, 0>(p, pl, s) : launch_mode<BITS, HAS_ZP, 1>(p, pl, s);
}

}  // namespace

// One translation unit per weight format instantiates the kernels.  The parameter block and the plan cross the
// boundary as untyped pointers (both are types of this header, the same in every unit).
hipError_t mnb_skinny_launch_w4(const void* params, const void* plan, hipStream_t s);    // 4-bit, no zero points
hipError_t mnb_skinny_launch_w4zp(const void* params, const void* plan, hipStream_t s);  // 4-bit, zero points
hipError_t mnb_skinny_launch_w8(const void* params, const void* plan, bool has_zp, hipStream_t s);
hipError_t mnb_skinny_launch_w2(const void* params, const void* plan, hipStream_t s);    // the native 2-bit copy

#if defined(MNB_STAMPS)
// Copies the readings of the unit's last direct decode launch out (count = number of 64-bit values, at most the
// array's).
#define MNB_STAMPS_READER(name)                                                                                   \
  extern "C" __attribute__((visibility("default"))) int name(unsigned long long* dst, size_t count) {             \
    if (!dst || count > (size_t)kStampGroups * kStampWaves * kStampPoints) return 2;                              \
    if (hipDeviceSynchronize() != hipSuccess) return 1;                                                           \
    return hipMemcpyFromSymbol(dst, HIP_SYMBOL(mnb_stamps), count * sizeof(unsigned long long), 0,                \
                               hipMemcpyDeviceToHost) == hipSuccess ? 0 : 1;                                      \
  }
#else
#define MNB_STAMPS_READER(name)
#endif
