// MFMA GEMM for fp16 models and large M: 256 x 256 output tile per workgroup, weights dequantised in registers.
//
// Device counterpart of the reference's prefill loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:
// 563-732: dequantise a strip of B, then run the float GEMM kernel over it).
//
// Eight wavefronts (2 x 4, two per SIMD), each owning a 128 x 64 block of the tile as 4 x 2
// v_mfma_f32_32x32x16_f16 accumulators.  Per k-step of 64:
//   * A (activations): every thread fetches 4 x 16 B two steps ahead into registers and writes them to the other
//     LDS buffer; wavefronts read their A operands with ds_read_b128 (rows padded by 16 B: conflict free).
//     8-bit weights need the registers of the second A set, so there the fetch follows the LDS write of the previous
//     tile into the same registers (one step ahead).
//   * B (weights) never touches LDS.  Lane (column j = lane%32, half kq = lane/32) of a wavefront loads, two steps
//     ahead, exactly the 8 bytes of packed weights it will feed to the matrix core: the two 32-bit words of its
//     column's 16-byte vector that belong to its half.  Each word is dequantised in registers to 8 halves -- exact
//     (q - zp), one rounding by the scale, bit-identical to the reference's fp16 dequantisation -- and IS the MFMA
//     B operand of one k-slab.  (The contraction index of an MFMA may be permuted freely as long as A uses the same
//     permutation: for 4-bit weights slab 2g takes k = 32g + 16kq + [0,8) and slab 2g+1 takes 32g + 16kq + [8,16).)
//     LDS traffic is what bounded the design that staged a dequantised B tile in LDS (every wavefront re-read it);
//     the price here is that the two wavefront rows dequantise the same columns.
//   * one barrier per step; the dequantisation of slab s+1 and the A staging run in the shadow of slab s's MFMAs.
// Bias add and the single fp32 -> fp16 narrowing happen in the epilogue.
#include <cstdlib>

#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

typedef uint32_t u4_t __attribute__((ext_vector_type(4)));  // plain register quad (HIP's uint4 struct resists SROA)
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));

constexpr int BN = 256, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // halves per staged A row
constexpr int THREADS = 512;
// Rows of the tile: 64 * TM, TM = 32-row matrix-core tiles per wavefront (4: 256 x 256, 2: 128 x 256 for grids that
// leave most of the chip idle with the large tile).  The dynamic LDS allocation is that of TM = 4 for both: the
// epilogue stages 64 x 64 outputs per wavefront in it.
constexpr int SMEM_HALVES = 2 * 256 * LDS_STRIDE;
// cost of a k-step of the 128-row tile relative to the 256-row one (measured)
constexpr double kMnbGemm128StepRatio = 0.88;

struct Gemm256Params {
  const _Float16* A;
  const uint8_t* W;  // packed weights, byte addressed
  const uint8_t* meta;
  const _Float16* bias;
  _Float16* C;
  int64_t lda, ldc, Npad;
  int M, N, K, bs_shift;
  int ksteps;
  int tiles_m, tiles_n;
  int tile_rows;  // 256 or 128
  int c_vec_ok;  // C allows 16-byte stores of 8 columns: aligned base and pitch, N a multiple of 8
  uint32_t uc[4];  // unpack constants (see UnpackConsts)
  // several matrices packed as one (mnb_layout.h); these kinds always take the 16-byte store path
  int epi_kind;            // kMnbFusedNone / kMnbFusedMlp: C[M][n_out0] = silu(gate) * up / kMnbFusedQkv: three outputs
  int start1, start2;      // qkv: first packed column of the second and third output
  int n_out0, n_out1, n_out2;
  _Float16* out1;
  _Float16* out2;
  int64_t ld1, ld2;
};

// The constants of the nibble unpack, passed as kernel arguments: with literals the compiler emits
// v_and_b32 + v_or_b32 (VOP3 takes no literal on this ISA family); with register operands, one v_and_or_b32.
struct UnpackConsts {
  uint32_t mask_lo, mask_hi, magic;  // 0x000F000F, 0x00F000F0, 0x64006400 (two halves of 1024)
};

__device__ __forceinline__ UnpackConsts make_unpack_consts(const uint32_t* k) {
  UnpackConsts u;
  u.mask_lo = k[0];
  u.mask_hi = k[1];
  // one SGPR operand per VALU instruction: the magic lives in a VGPR (an opaque move, so it is not folded back)
  asm volatile("v_mov_b32 %0, %1" : "=v"(u.magic) : "s"(k[2]));
  return u;
}

// Packed weights of one lane and slab -> 8 dequantised halves in k order: the B operand of one MFMA.
// 4-bit: one word (w1 unused); 8-bit: two words.
template <int BITS>
__device__ __forceinline__ h8_t dequant_word(uint32_t w0, uint32_t w1, const UnpackConsts& uc, const ZpH& z,
                                             h2_t s2) {
  h2_t d[4];
  if constexpr (BITS == 4) {
    const h2_t sixteenth = mnb_h2((_Float16)0.0625f);
    const uint32_t w8 = w0 >> 8;
    const h2_t p0 = mnb_as_h2((w0 & uc.mask_lo) | uc.magic);
    const h2_t p1 = mnb_as_h2((w0 & uc.mask_hi) | uc.magic);
    const h2_t p2 = mnb_as_h2((w8 & uc.mask_lo) | uc.magic);
    const h2_t p3 = mnb_as_h2((w8 & uc.mask_hi) | uc.magic);
    d[0] = p0 + z.lo;
    d[1] = __builtin_elementwise_fma(p1, sixteenth, z.hi);
    d[2] = p2 + z.lo;
    d[3] = __builtin_elementwise_fma(p3, sixteenth, z.hi);
  } else {
    mnb_unpack8_h(w0, z, d);
    mnb_unpack8_h(w1, z, d + 2);
  }
  const u4_t o = {mnb_as_u32(d[0] * s2), mnb_as_u32(d[1] * s2), mnb_as_u32(d[2] * s2), mnb_as_u32(d[3] * s2)};
  return __builtin_bit_cast(h8_t, o);
}

// Scheduling pipeline of one slab section (NM MFMAs): after every MFMA a few of the other instructions of the
// section, so they run in the MFMA's shadow.  The closing sched_barrier keeps the scheduler from mixing the MFMAs
// of different slabs (they reuse the same accumulators).
template <int NM, int LDS_READS, int VMEM, int VALU, int LDS_WRITE_EVERY>
__device__ __forceinline__ void slab_pipeline() {
#pragma unroll
  for (int i = 0; i < NM; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                             // 1 MFMA
    if (i < LDS_READS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);          // 1 LDS read
    if (i < VMEM) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);               // 2 VMEM reads
    if constexpr (VALU > 0) __builtin_amdgcn_sched_group_barrier(0x002, VALU, 0);  // VALU
    if constexpr (LDS_WRITE_EVERY > 0) {
      if (i % LDS_WRITE_EVERY == LDS_WRITE_EVERY - 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // 1 LDS write
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

// Slab 0 of a k-step when the activations share one register set: the four LDS writes of the next A tile go first,
// the four global loads that refill their registers follow (the loads must not overtake the writes that still read
// those registers).
template <int TM>
__device__ __forceinline__ void slab0_shared_a_pipeline() {
#pragma unroll
  for (int i = 0; i < 2 * TM; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // 1 MFMA
    if (i < TM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 LDS read
    __builtin_amdgcn_sched_group_barrier(0x002, 32 / (2 * TM), 0);  // VALU
    if (i < TM)
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);            // 1 LDS write
    else if (i < TM + TM / 2)
      __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);            // 2 VMEM reads
  }
  __builtin_amdgcn_sched_barrier(0);
}

// MPS: meta entries (scale, zero point) a lane keeps per k-step and column tile.  A k-step of 64 spans 64 / block_size
// blocks; 4-bit vectors cover 32 k, so two entries serve every block size (16-wide blocks through the lane's half
// kq); 8-bit vectors cover 16 k: 4 entries for blocks of 16, 2 for blocks of 32 and more.
template <int BITS, bool HAS_ZP, int MPS, int TM>
__global__ void __launch_bounds__(THREADS, 2) mnb_gemm256_kernel(Gemm256Params p) {
  constexpr int BM = 64 * TM;                       // rows of the tile
  constexpr int STAGE_HALVES = BM * LDS_STRIDE;     // one A buffer
  constexpr int NM = 2 * TM;                        // MFMAs per slab
  constexpr int VALU_PER_MFMA = 32 / NM;            // the slab's dequantisation spread over its MFMAs
  constexpr int A_LOADS = BM * (BK / 8) / THREADS;  // 16-byte activation loads per thread per k-step: TM
  // 4-bit: a 16-byte vector spans two slabs (one word each per lane); 8-bit: one slab (two words per lane)
  constexpr int VEC_PER_STEP = (BITS == 4) ? 2 : 4;  // 8-byte weight loads per lane, column tile and k-step
  constexpr int GK = 128 / BITS;
  extern __shared__ __align__(16) _Float16 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 wavefronts: rows wm*32*TM, columns wn*64
  // column-fastest tile order: the workgroups resident at one time share a few 256-row slabs of A
  const int m0 = (blockIdx.x / p.tiles_n) * BM;
  const int n0 = (blockIdx.x % p.tiles_n) * BN;
  const int li = lane & 31, kq = lane >> 5;

  f16_t acc[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Two register sets for the global prefetch (distance: two k-steps).  8-bit weights take twice the registers of
  // 4-bit ones, so there the activations share ONE set (RA): the tile of step ks+1 leaves it for LDS in slab 0 of
  // step ks and the loads of step ks+2 refill it right behind those writes.  With 4-bit weights the loads go first,
  // into the set that was staged a step earlier: measured 5 % faster, and the registers are there.
  constexpr bool SHARED_A = BITS == 8;
  struct Stage {
    u4_t a[SHARED_A ? 1 : A_LOADS];
    u2_t b[VEC_PER_STEP][2];      // [vector of the k-step][column tile]
    uint32_t m[MPS][2];           // meta entries of the blocks of the k-step
  };
  Stage R0, R1;
  u4_t RA[A_LOADS];
  h8_t FA0[TM], FA1[TM];  // A operands, double buffered over slabs
  h8_t FB0[2], FB1[2];  // B operands, double buffered over slabs

  const UnpackConsts uc = make_unpack_consts(p.uc);

  // Addressing: every global access is  uniform base (SGPRs, advanced per k-step)  +  32-bit per-lane offset (a VGPR
  // computed once), so the loads cost no VALU work inside the loop.
  // The tile's first row is part of the uniform base, so a lane's offset spans at most 255 rows: it fits 32 bits
  // for every M as long as 512 * lda does (mnb_gemm256_addressable; larger pitches take the streaming kernel).
  const int a_row = tid >> 3, a_kc = tid & 7;  // thread's first A chunk: row a_row (+64 per load), k chunk a_kc
  const _Float16* a_tile = p.A + (int64_t)m0 * p.lda;
  uint32_t a_off[A_LOADS];                     // byte offsets from a_tile + k0
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    // rows beyond M re-read row M-1 and are never stored (a predicated load would serialise the loop)
    int r = a_row + i * 64;
    r = m0 + r < p.M ? r : p.M - 1 - m0;
    a_off[i] = (uint32_t)(((int64_t)r * p.lda + a_kc * 8) * 2);
  }
  // this lane's weight columns (one per column tile): its 8 bytes inside each 16-byte vector, and its meta entries.
  // The block of a lane's half vector is (k-group base >> bs_shift), plus kq when 4-bit blocks are 16 wide.
  constexpr int META_BYTES = HAS_ZP ? 4 : 2;
  const bool small_bs = (BITS == 4) && p.bs_shift == 4;
  uint32_t w_off[2], m_off[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t col = n0 + wn * 64 + j * 32 + li;
    w_off[j] = (uint32_t)(col * 16 + kq * 8);
    m_off[j] = (uint32_t)((mnb_meta_col(col) + (small_bs ? kq * p.Npad : 0)) * META_BYTES);
  }
  const int last_step = p.ksteps - 1;
  const int64_t vec_pitch = p.Npad * 16;               // bytes between consecutive k-groups
  const int64_t meta_pitch = p.Npad * META_BYTES;      // bytes between consecutive blocks

  // k-steps past the end are clamped to the last one: the loop body stays branch free, the data is never used
  auto load_a = [&](int ks_raw, Stage& R) {
    const int ks = ks_raw < last_step ? ks_raw : last_step;
    const uint8_t* base = reinterpret_cast<const uint8_t*>(a_tile + (int64_t)ks * BK);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const u4_t v = *reinterpret_cast<const u4_t*>(base + a_off[i]);
      if constexpr (SHARED_A)
        RA[i] = v;
      else
        R.a[i] = v;
    }
  };
  auto load_b = [&](int ks_raw, Stage& R) {
    const int ks = ks_raw < last_step ? ks_raw : last_step;
#pragma unroll
    for (int v = 0; v < VEC_PER_STEP; ++v) {
      const int64_t kg = (int64_t)ks * VEC_PER_STEP + v;  // k-group of the vector
      const int64_t kb = (kg * GK) >> p.bs_shift;         // block of the vector's first element
      const uint8_t* wbase = p.W + kg * vec_pitch;
      const uint8_t* mbase = p.meta + kb * meta_pitch;
      constexpr int VEC_PER_META = VEC_PER_STEP / MPS;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        R.b[v][j] = *reinterpret_cast<const u2_t*>(wbase + w_off[j]);
        if (v % VEC_PER_META == 0) {
          if constexpr (HAS_ZP)
            R.m[v / VEC_PER_META][j] = *reinterpret_cast<const uint32_t*>(mbase + m_off[j]);
          else
            R.m[v / VEC_PER_META][j] = *reinterpret_cast<const uint16_t*>(mbase + m_off[j]);
        }
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

  // B operands of slab kk (0..3) of the k-step held in R
  auto make_b = [&](int kk, const Stage& R, h8_t* FB) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      h2_t s2;
      ZpH z;
      if constexpr (BITS == 4) {
        const int v = kk >> 1;
        decode(R.m[v][j], s2, z);
        FB[j] = dequant_word<4>(R.b[v][j][kk & 1], 0u, uc, z, s2);
      } else {
        decode(R.m[kk * MPS / 4][j], s2, z);
        FB[j] = dequant_word<8>(R.b[kk][j][0], R.b[kk][j][1], uc, z, s2);
      }
    }
  };

  auto store_a = [&](int buf, int i, const Stage& R) {
    u4_t v;
    if constexpr (SHARED_A)
      v = RA[i];
    else
      v = R.a[i];
    *reinterpret_cast<u4_t*>(lds + buf * STAGE_HALVES + (a_row + i * 64) * LDS_STRIDE + a_kc * 8) = v;
  };

  // A operands of slab kk: lane (row li, half kq).  The k permutation matches the weights' (see the file header).
  auto read_a = [&](int buf, int kk, h8_t* FA) {
    const int koff = (BITS == 4) ? 32 * (kk >> 1) + 16 * kq + 8 * (kk & 1) : 16 * kk + 8 * kq;
    const _Float16* As = lds + buf * STAGE_HALVES + (wm * 32 * TM + li) * LDS_STRIDE + koff;
#pragma unroll
    for (int t = 0; t < TM; ++t) FA[t] = *reinterpret_cast<const h8_t*>(As + t * 32 * LDS_STRIDE);
  };

  auto mfma_slab = [&](const h8_t* FA, const h8_t* FB) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(FA[i], FB[j], acc[i][j], 0, 0, 0);
  };

  // One k-step.  On entry: LDS buffer `cur` holds the A tile of step ks, FA0/FB0 hold the operands of its slab 0,
  // Rc holds the weights of step ks (its A registers are already staged, hence free), Rn holds (or is receiving)
  // A and weights of step ks+1.
  auto k_step = [&](int ks, Stage& Rc, Stage& Rn) {
    const int cur = ks & 1, nxt = cur ^ 1;
    // slab 0: operands of slab 1; global loads of A for step ks+2; A of step ks+1 into the other buffer
    if constexpr (!SHARED_A) load_a(ks + 2, Rc);
    read_a(cur, 1, FA1);
    make_b(1, Rc, FB1);
    mfma_slab(FA0, FB0);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) store_a(nxt, i, Rn);
    if constexpr (SHARED_A) {
      load_a(ks + 2, Rc);
      slab0_shared_a_pipeline<TM>();
    } else {
      slab_pipeline<NM, TM, TM / 2, VALU_PER_MFMA, 2>();
    }
    // slab 1: operands of slab 2
    read_a(cur, 2, FA0);
    make_b(2, Rc, FB0);
    mfma_slab(FA1, FB1);
    slab_pipeline<NM, TM, 0, VALU_PER_MFMA, 0>();
    // slab 2: operands of slab 3; after that the weight registers of Rc are free: weights of step ks+2
    read_a(cur, 3, FA1);
    make_b(3, Rc, FB1);
    mfma_slab(FA0, FB0);
    load_b(ks + 2, Rc);
    slab_pipeline<NM, TM, 4, VALU_PER_MFMA, 0>();
    __syncthreads();
    // slab 3, behind the barrier: operands of slab 0 of step ks+1
    read_a(nxt, 0, FA0);
    make_b(0, Rn, FB0);
    mfma_slab(FA1, FB1);
    slab_pipeline<NM, TM, 0, VALU_PER_MFMA, 0>();
  };

  // ---- prologue: steps 0 and 1 in flight, A of step 0 staged, operands of slab 0 ready
  load_a(0, R0);
  load_b(0, R0);
  if constexpr (!SHARED_A) load_a(1, R1);
  load_b(1, R1);
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) store_a(0, i, R0);
  if constexpr (SHARED_A) load_a(1, R1);
  __syncthreads();
  read_a(0, 0, FA0);
  make_b(0, R0, FB0);

  for (int ks = 0; ks < p.ksteps; ks += 2) {  // ksteps is even
    k_step(ks, R0, R1);
    k_step(ks + 1, R1, R0);
  }

  // ---- epilogue.  D[i][j] of a 32x32 tile: lane holds column j = lane % 32, rows 8*(r/4) + 4*(lane/32) + r%4.
  // Stored straight from the accumulators that is 2 bytes per lane and 64-byte row segments; instead each wavefront
  // transposes its block through its own slice of the (now idle) A buffers, 64 rows at a time, and writes whole
  // 128-byte rows with 16-byte stores.
  float bcol[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + li;
    bcol[j] = (p.bias && n < p.N) ? (float)p.bias[n] : 0.f;
  }
  if (p.c_vec_ok) {
    constexpr int EP_STRIDE = 72;  // halves per staged row: 16-byte aligned rows, conflict-free 16-byte reads
    __syncthreads();               // every wavefront is done with the A tiles
    _Float16* ep = lds + wave * (64 * EP_STRIDE);
    const int erow = lane >> 3, ecol = (lane & 7) * 8;
    const int n_out = n0 + wn * 64 + ecol;
#pragma unroll
    for (int h = 0; h < TM / 2; ++h) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            ep[(ii * 32 + (r >> 2) * 8 + kq * 4 + (r & 3)) * EP_STRIDE + j * 32 + li] =
                (_Float16)(acc[2 * h + ii][j][r] + bcol[j]);
      // LDS operations of one wavefront complete in issue order: the reads below see the writes above
      if (p.epi_kind == kMnbFusedMlp) {
        // a staged row is gate0 up0 gate1 up1 (16 columns each) = 32 output columns: four lanes per row, each reads
        // its 8 gate and 8 up values (narrowed to fp16, as the two separate products would be) and writes 8 outputs
        const int grow = lane >> 2, q = lane & 3;
        const int gcol = (q >> 1) * 32 + (q & 1) * 8;
        const int n_glu = ((n0 + wn * 64) >> 1) + q * 8;
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
          const int row = ps * 16 + grow;
          const h8_t g = *reinterpret_cast<const h8_t*>(ep + row * EP_STRIDE + gcol);
          const h8_t u = *reinterpret_cast<const h8_t*>(ep + row * EP_STRIDE + gcol + 16);
          h8_t y;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float gf = (float)g[e];
            y[e] = (_Float16)(gf / (1.0f + __expf(-gf)) * (float)u[e]);
          }
          const int m = m0 + wm * 32 * TM + h * 64 + row;
          if (m < p.M && n_glu < p.n_out0) *reinterpret_cast<h8_t*>(p.C + (int64_t)m * p.ldc + n_glu) = y;
        }
      } else {
        // the 8 columns of a lane lie inside one 16-column tile, hence inside one output
        _Float16* dst = p.C;
        int64_t ld = p.ldc;
        int n_loc = n_out, n_lim = p.N;
        if (p.epi_kind == kMnbFusedQkv) {
          n_lim = p.n_out0;
          if (n_out >= p.start2) {
            dst = p.out2, ld = p.ld2, n_loc = n_out - p.start2, n_lim = p.n_out2;
          } else if (n_out >= p.start1) {
            dst = p.out1, ld = p.ld1, n_loc = n_out - p.start1, n_lim = p.n_out1;
          }
        }
#pragma unroll
        for (int ps = 0; ps < 8; ++ps) {
          const int row = ps * 8 + erow;
          const u4_t v = *reinterpret_cast<const u4_t*>(ep + row * EP_STRIDE + ecol);
          const int m = m0 + wm * 32 * TM + h * 64 + row;
          if (m < p.M && n_loc < n_lim) *reinterpret_cast<u4_t*>(dst + (int64_t)m * ld + n_loc) = v;
        }
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + li;
      if (n >= p.N) continue;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * 32 * TM + i * 32 + (r >> 2) * 8 + kq * 4 + (r & 3);
          if (m < p.M) p.C[(int64_t)m * p.ldc + n] = (_Float16)(acc[i][j][r] + bcol[j]);
        }
      }
    }
  }
}

template <int BITS, bool HAS_ZP, int MPS, int TM>
hipError_t launch_tm(const Gemm256Params& p, hipStream_t s) {
  const size_t smem = (size_t)SMEM_HALVES * sizeof(_Float16);  // 73728 bytes
  auto kernel = mnb_gemm256_kernel<BITS, HAS_ZP, MPS, TM>;
  // The attribute belongs to the function on the current device, so it is set on every launch (a host-side table
  // update, no device work): callers on several threads or devices need no shared flag.
  if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      e != hipSuccess)
    return e;
  dim3 grid((unsigned)(p.tiles_n * p.tiles_m)), blk(THREADS);
  kernel<<<grid, blk, smem, s>>>(p);
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP, int MPS>
hipError_t launch(const Gemm256Params& p, hipStream_t s) {
  return p.tile_rows == 128 ? launch_tm<BITS, HAS_ZP, MPS, 2>(p, s) : launch_tm<BITS, HAS_ZP, MPS, 4>(p, s);
}

}  // namespace

// Rows of the tile for a problem: the 128-row tile when its grid fills the 256 compute units in fewer, or at the
// measured step costs cheaper, rounds than the 256-row one.
int mnb_gemm256_tile_rows(const MnbLayout& L, int64_t M, double* seconds) {
  const MnbDeviceInfo& dev = mnb_device_info();
  const int64_t tiles_n = (L.N + BN - 1) / BN;
  const double ksteps = (double)(L.K / BK);
  // cycles of one 64-deep k-step of a 256-row tile with the whole chip busy (4-bit; 8-bit; 8-bit with 16-wide blocks,
  // whose four meta entries per step spill): properties of the kernel's instruction schedule
  const double cycles256 = L.bits == 4 ? 3480.0 : (L.bs >= 32 ? 3960.0 : 7080.0);
  const double step256 = cycles256 / dev.clock_hz;
  const double step128 = step256 * kMnbGemm128StepRatio;
  const int64_t cus = dev.cus;
  const double t256 = (double)((((M + 255) / 256) * tiles_n + cus - 1) / cus) * ksteps * step256;
  const double t128 = (double)((((M + 127) / 128) * tiles_n + cus - 1) / cus) * ksteps * step128;
  static const int forced = [] {
    const char* e = getenv("MNB_GEMM256_TILE_ROWS");  // tuning override: 128 or 256
    return e ? atoi(e) : 0;
  }();
  const bool small = forced ? forced == 128 : t128 < t256;
  if (seconds) *seconds = small ? t128 : t256;
  return small ? 128 : 256;
}

// Per-lane offsets of the tile GEMM are 32-bit byte counts from a base that moves with the tile: activations span
// 255 rows of lda halves plus one k-step (mnb_gemm256_max_lane_offset), weights one k-group row of Npad columns x 16
// bytes, meta entries two block rows of Npad x 4 bytes.  Problems beyond that take the streaming kernel, whose
// addressing is 64-bit throughout.
uint64_t mnb_gemm256_max_lane_offset(int64_t lda) { return ((uint64_t)255 * (uint64_t)lda + 7 * 8 + 7) * 2 + 1; }

bool mnb_gemm256_addressable(int64_t lda, int64_t Npad) {
  return mnb_gemm256_max_lane_offset(lda) < ((uint64_t)1 << 32) && (uint64_t)Npad * 16 + 16 <= ((uint64_t)1 << 32);
}

// The fused outputs are written with 16-byte stores of 8 columns: every output 16-byte aligned, with a pitch and a
// width that are multiples of 8 elements.
bool mnb_gemm256_fused_ok(const MnbEpilogue& e) {
  const int nout = e.kind == kMnbFusedQkv ? 3 : 1;
  for (int i = 0; i < nout; ++i)
    if (reinterpret_cast<uintptr_t>(e.out[i]) % 16 != 0 || e.ld[i] % 8 != 0 || e.n[i] % 8 != 0) return false;
  return true;
}

hipError_t mnb_launch_gemm256(const MnbGemmArgs& a, hipStream_t s) {
  if (!mnb_gemm256_addressable(a.lda, a.L.Npad)) return hipErrorInvalidValue;  // the dispatcher never sends these
  Gemm256Params p{};
  p.A = reinterpret_cast<const _Float16*>(a.A);
  p.W = reinterpret_cast<const uint8_t*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + a.L.meta_off;
  p.bias = reinterpret_cast<const _Float16*>(a.bias);
  p.C = reinterpret_cast<_Float16*>(a.C);
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.Npad = a.L.Npad;
  p.M = (int)a.M;
  p.N = (int)a.L.N;
  p.K = (int)a.L.K;
  p.bs_shift = mnb_log2i(a.L.bs);
  p.ksteps = (int)(a.L.K / BK);  // K is a multiple of 2 * BK
  p.tile_rows = mnb_gemm256_tile_rows(a.L, a.M, nullptr);
  p.tiles_m = (int)((a.M + p.tile_rows - 1) / p.tile_rows);
  p.tiles_n = (int)((a.L.N + BN - 1) / BN);
  p.uc[0] = 0x000F000Fu;
  p.uc[1] = 0x00F000F0u;
  p.uc[2] = 0x64006400u;
  p.uc[3] = 0;
  p.c_vec_ok = (reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.ldc % 8 == 0) && (a.L.N % 8 == 0);
  p.epi_kind = a.epi.kind;
  if (a.epi.kind != kMnbFusedNone) {
    if (!mnb_gemm256_fused_ok(a.epi)) return hipErrorInvalidValue;  // the caller checks before choosing this kernel
    p.C = reinterpret_cast<_Float16*>(a.epi.out[0]);
    p.ldc = a.epi.ld[0];
    p.c_vec_ok = 1;
    p.start1 = (int)a.epi.start[1];
    p.start2 = (int)a.epi.start[2];
    p.n_out0 = (int)a.epi.n[0];
    p.n_out1 = (int)a.epi.n[1];
    p.n_out2 = (int)a.epi.n[2];
    p.out1 = reinterpret_cast<_Float16*>(a.epi.out[1]);
    p.out2 = reinterpret_cast<_Float16*>(a.epi.out[2]);
    p.ld1 = a.epi.ld[1];
    p.ld2 = a.epi.ld[2];
  }
  if (a.L.bits == 4) return a.L.has_zp ? launch<4, true, 2>(p, s) : launch<4, false, 2>(p, s);
  // 8-bit: two entries per k-step fit the register file without spills (also for blocks of 64 and more, where both
  // entries name the same block); blocks of 16 need four and spill
  if (a.L.bs >= 32) return a.L.has_zp ? launch<8, true, 2>(p, s) : launch<8, false, 2>(p, s);
  return a.L.has_zp ? launch<8, true, 4>(p, s) : launch<8, false, 4>(p, s);
}
