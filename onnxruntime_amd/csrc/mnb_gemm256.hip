// MFMA GEMM for fp16 models and large M: 256 x 256 output tile per workgroup, weights dequantised in registers.
//
// Device counterpart of the reference's prefill loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:
// 563-732: dequantise a strip of B, then run the float GEMM kernel over it).
//
// Eight wavefronts (2 x 4, two per SIMD), each owning a 128 x 64 block of the tile as 4 x 2
// v_mfma_f32_32x32x16_f16 accumulators.  Per k-step of 64:
//   * A (activations) goes from global memory straight into LDS (global_load_lds_dwordx4: no registers, no LDS
//     store instructions), two k-steps ahead, into one of three staged tiles.  Such a load puts the 16 bytes of lane
//     L at (wave-uniform LDS base) + 16 L, so a wavefront fills 8 rows x 128 bytes with one instruction; the rows are
//     not padded, instead the lane that fills chunk position p of row r fetches chunk p ^ (r & 7) of that row, and the
//     readers (ds_read_b128, lane = row) apply the same XOR: conflict free.
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
//
// Work distribution ("stream-K").  The work of a problem is its tiles x k-steps, counted in units of two k-steps and
// numbered tile by tile.  With a workspace the grid is one workgroup per compute unit and workgroup w takes the
// w-th equal share of the units -- a tile whose units fall into several shares is computed in parts (the reference
// partitions M and N only, qnbitgemm.cpp:1600-1809; 448 tiles on 256 compute units would otherwise run as two rounds
// of which the second is three quarters full, and 64 tiles would leave three quarters of the chip idle).  A
// workgroup walks its share from the top down.  The part that holds a tile's last unit finalises the tile: it adds
// the partial sums of the parts below it and writes C.  Every other part writes its fp32 accumulators to its
// workgroup's slot in the workspace and raises its flags (one per wavefront: a wavefront's accumulators are read back
// by the wavefront of the same index, so no barrier is involved on either side).  A workgroup writes at most one
// partial (its topmost part, computed first) and waits only for workgroups with smaller indices (dispatched before
// it): the waits cannot deadlock.  The partial of a workgroup that went on to other tiles was written long before it
// is needed: the finalising part starts from it instead of from zero (no burst of reads when all workgroups finish
// together).  Partials of workgroups whose whole share lies inside the tile arrive as late as the finalising part
// itself ends and are added then, nearest first.  The order of summation is fixed by the shares, so results are the
// same from run to run.  Partials and flags travel with device-scope atomic stores and loads (write-through, no
// cache maintenance); the flags are cleared by a small kernel in front of the launch.
// Without a workspace the grid is one workgroup per tile and nothing is split.
#include <cstdlib>

#include "mnb_device.hip.h"
#include "mnb_internal.h"

namespace {

typedef uint32_t u4_t __attribute__((ext_vector_type(4)));  // plain register quad (HIP's uint4 struct resists SROA)
typedef uint32_t u2_t __attribute__((ext_vector_type(2)));

constexpr int BN = 256, BK = 64;
constexpr int ROW_BYTES = BK * 2;  // bytes per staged A row (eight 16-byte chunks, XOR-swizzled with the row)
constexpr int THREADS = 512;
// Rows of the tile: 64 * TM, TM = 32-row matrix-core tiles per wavefront (4: 256 x 256, 2: 128 x 256 for grids that
// leave most of the chip idle with the large tile).  The dynamic LDS allocation is that of TM = 4 for both: three
// staged A tiles of 32 KiB; the epilogue stages 64 x 64 outputs per wavefront in it (72 KiB).
constexpr int SMEM_BYTES = 3 * 256 * ROW_BYTES;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt immediate that waits until at most VM vector-memory operations are outstanding and every LDS operation
// of the wavefront has completed (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14).
constexpr int waitcnt_vm_lds0(int vm) { return (vm & 15) | (7 << 4) | (0 << 8) | ((vm >> 4) << 14); }
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
  // work distribution: `units` = tiles x ksteps / 2 split over the grid; workgroup w takes
  // [w * share_q + min(w, share_r), (w + 1) * share_q + min(w + 1, share_r))
  int upt;                  // units per tile
  int64_t share_q, share_r;
  uint64_t* partials;       // one slot of tile_rows x 256 floats per workgroup (NULL: grid == tiles, nothing is split)
  uint32_t* flags;          // one word per workgroup and wavefront, zero when the kernel starts
  int spin_limit;           // polls of a flag before the wait gives up and the tile is poisoned with NaN
  int c_vec_ok;  // C allows 16-byte stores of 8 columns: aligned base and pitch, N a multiple of 8
  // several matrices packed as one (mnb_layout.h); these kinds always take the 16-byte store path
  int epi_kind;            // kMnbFusedNone / kMnbFusedMlp: C[M][n_out0] = silu(gate) * up / kMnbFusedQkv: three outputs
  int start1, start2;      // qkv: first packed column of the second and third output
  int n_out0, n_out1, n_out2;
  _Float16* out1;
  _Float16* out2;
  int64_t ld1, ld2;
};

// The constants of the nibble unpack.  Written as plain literals the compiler emits v_and_b32 + v_or_b32 (VOP3 takes
// no literal on this ISA family); held in registers, one v_and_or_b32.  Opaque moves materialise them (the masks in
// SGPRs, the magic in a VGPR: one SGPR operand per VALU instruction) so that they are not folded back.
struct UnpackConsts {
  uint32_t mask_lo, mask_hi, magic;  // 0x000F000F, 0x00F000F0, 0x64006400 (two halves of 1024)
};

__device__ __forceinline__ UnpackConsts make_unpack_consts() {
  UnpackConsts u;
  asm("s_mov_b32 %0, 0x000F000F" : "=s"(u.mask_lo));
  asm("s_mov_b32 %0, 0x00F000F0" : "=s"(u.mask_hi));
  asm("v_mov_b32 %0, 0x64006400" : "=v"(u.magic));
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

// MPS: meta entries (scale, zero point) a lane keeps per k-step and column tile.  A k-step of 64 spans 64 / block_size
// blocks; 4-bit vectors cover 32 k, so two entries serve every block size (16-wide blocks through the lane's half
// kq); 8-bit vectors cover 16 k: 4 entries for blocks of 16, 2 for blocks of 32 and more.
template <int BITS, bool HAS_ZP, int MPS, int TM>
__global__ void __launch_bounds__(THREADS, 2) mnb_gemm256_kernel(Gemm256Params p) {
  constexpr int BM = 64 * TM;                       // rows of the tile
  constexpr int STAGE_BYTES = BM * ROW_BYTES;       // one staged A tile
  constexpr int NM = 2 * TM;                        // MFMAs per slab
  constexpr int VALU_PER_MFMA = 32 / NM;            // the slab's dequantisation spread over its MFMAs
  constexpr int A_LOADS = BM * (BK / 8) / THREADS;  // 16-byte activation loads per thread per k-step: TM
  // 4-bit: a 16-byte vector spans two slabs (one word each per lane); 8-bit: one slab (two words per lane)
  constexpr int VEC_PER_STEP = (BITS == 4) ? 2 : 4;  // 8-byte weight loads per lane, column tile and k-step
  constexpr int GK = 128 / BITS;
  constexpr int ACC_PAIRS = TM * 2 * 8;              // 8-byte pairs of accumulators per lane
  // vector-memory operations a wavefront issues per k-step for the weights (vectors and meta entries)
  constexpr int B_LOADS = VEC_PER_STEP * 2 + MPS * 2;
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  _Float16* const lds = reinterpret_cast<_Float16*>(lds_bytes);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 wavefronts: rows wm*32*TM, columns wn*64
  const int li = lane & 31, kq = lane >> 5;

  f16_t acc[TM][2];

  // Two register sets for the weight prefetch (distance: two k-steps); the activations need none.
  struct Stage {
    u2_t b[VEC_PER_STEP][2];      // [vector of the k-step][column tile]
    uint32_t m[MPS][2];           // meta entries of the blocks of the k-step
  };
  Stage R0, R1;
  h8_t FA0[TM], FA1[TM];  // A operands, double buffered over slabs
  h8_t FB0[2], FB1[2];  // B operands, double buffered over slabs

  const UnpackConsts uc = make_unpack_consts();

  // Addressing: every global access is  uniform base (SGPRs: the tile's corner, advanced per k-step)  +  32-bit
  // per-lane offset (a VGPR), so the loads cost no VALU work inside the loop.  The tile's first row and column are
  // part of the uniform base, so a lane's offsets span at most 255 rows of A and 256 columns of weights: they fit
  // 32 bits for every M and N as long as 512 * lda does (mnb_gemm256_addressable).
  // Load i of a wavefront fills rows i * 64 + wave * 8 + [0, 8) of the staged tile; the lane at chunk position
  // lane & 7 of row lane >> 3 fetches chunk (lane & 7) ^ (row & 7).
  const int a_row = tid >> 3, a_kc = (tid & 7) ^ ((tid >> 3) & 7);
  uint32_t a_off[A_LOADS];                     // byte offsets from a_tile + k0; set per tile (rows beyond M)
  // this lane's weight columns (one per column tile): its 8 bytes inside each 16-byte vector, and its meta entries.
  // The block of a lane's half vector is (k-group base >> bs_shift), plus kq when 4-bit blocks are 16 wide.
  constexpr int META_BYTES = HAS_ZP ? 4 : 2;
  const bool small_bs = (BITS == 4) && p.bs_shift == 4;
  uint32_t w_off[2], m_off[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = wn * 64 + j * 32 + li;  // within the tile; tiles start at multiples of 256 columns
    w_off[j] = (uint32_t)(col * 16 + kq * 8);
    m_off[j] = (uint32_t)((mnb_meta_col(col) + (small_bs ? kq * p.Npad : 0)) * META_BYTES);
  }
  const int last_step = p.ksteps - 1;
  const int64_t vec_pitch = p.Npad * 16;               // bytes between consecutive k-groups
  const int64_t meta_pitch = p.Npad * META_BYTES;      // bytes between consecutive blocks

  // the current tile (uniform)
  int m0 = 0, n0 = 0;
  const _Float16* a_tile = p.A;
  const uint8_t* w_tile = p.W;
  const uint8_t* meta_tile = p.meta;

  // k-steps past the end are clamped to the last one: the loop body stays branch free, the data is never used
  auto load_a = [&](int ks_raw, int stage_off) {
    const int ks = ks_raw < last_step ? ks_raw : last_step;
    const uint8_t* base = reinterpret_cast<const uint8_t*>(a_tile + (int64_t)ks * BK);
    // (The host pass of the compiler knows the builtin but not the target feature it needs, and silently drops the
    // whole kernel, launch stub included, if it meets the call: the call is for the device pass only.)
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
#if defined(__HIP_DEVICE_COMPILE__)
      __builtin_amdgcn_global_load_lds(base + a_off[i],
                                       (lds_ptr_t)(lds_bytes + stage_off + (i * 64 + wave * 8) * ROW_BYTES), 16, 0, 0);
#else
      (void)base;
      (void)stage_off;
#endif
    }
  };
  auto load_b = [&](int ks_raw, Stage& R) {
    const int ks = ks_raw < last_step ? ks_raw : last_step;
#pragma unroll
    for (int v = 0; v < VEC_PER_STEP; ++v) {
      const int64_t kg = (int64_t)ks * VEC_PER_STEP + v;  // k-group of the vector
      const int64_t kb = (kg * GK) >> p.bs_shift;         // block of the vector's first element
      const uint8_t* wbase = w_tile + kg * vec_pitch;
      const uint8_t* mbase = meta_tile + kb * meta_pitch;
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

  // A operands of slab kk: lane (row li, half kq).  The k permutation matches the weights' (see the file header);
  // a_rd[kk] is the lane's byte offset inside a staged tile, chunk swizzle included.
  uint32_t a_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    const int chunk = (BITS == 4) ? 4 * (kk >> 1) + 2 * kq + (kk & 1) : 2 * kk + kq;
    a_rd[kk] = (uint32_t)((wm * 32 * TM + li) * ROW_BYTES + ((chunk ^ (li & 7)) * 16));
  }
  auto read_a = [&](int stage_off, int kk, h8_t* FA) {
    const unsigned char* As = lds_bytes + stage_off + a_rd[kk];
#pragma unroll
    for (int t = 0; t < TM; ++t) FA[t] = *reinterpret_cast<const h8_t*>(As + t * 32 * ROW_BYTES);
  };

  auto mfma_slab = [&](const h8_t* FA, const h8_t* FB) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(FA[i], FB[j], acc[i][j], 0, 0, 0);
  };

  // One k-step.  On entry: the staged tile at `cur` holds A of step ks, the one at `nxt` is receiving A of step ks+1,
  // the one at `nn` is free (its readers passed the barrier of step ks-1); FA0/FB0 hold the operands of slab 0, Rc
  // holds the weights of step ks, Rn holds (or is receiving) those of step ks+1.
  auto k_step = [&](int ks, Stage& Rc, Stage& Rn, int cur, int nxt, int nn) {
    // slab 0: operands of slab 1; A of step ks+2 on its way into the free tile
    load_a(ks + 2, nn);
    read_a(cur, 1, FA1);
    make_b(1, Rc, FB1);
    mfma_slab(FA0, FB0);
    slab_pipeline<NM, TM, TM / 2, VALU_PER_MFMA, 0>();
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
    // The barrier of the step.  Before it a wavefront makes sure that its own part of A of step ks+1 has landed in
    // LDS: those loads are older than the weights fetched in slab 2 of step ks-1, and younger than those are exactly
    // the A loads of slab 0 and the weight loads of slab 2 above, so "at most A_LOADS + B_LOADS outstanding" covers
    // them (and nothing issued in this step).  Its LDS reads have completed too, so the tile at `cur` may be
    // overwritten from the next step on.  No fence: the fence of __syncthreads would wait for every outstanding
    // load, the weight prefetch included.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lds0(A_LOADS + B_LOADS));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // slab 3, behind the barrier: operands of slab 0 of step ks+1
    read_a(nxt, 0, FA0);
    make_b(0, Rn, FB0);
    mfma_slab(FA1, FB1);
    slab_pipeline<NM, TM, 0, VALU_PER_MFMA, 0>();
  };

  // ---- this workgroup's share of the units, walked from the top down
  const int64_t wg = blockIdx.x;
  const int64_t share_lo = wg * p.share_q + (wg < p.share_r ? wg : p.share_r);
  int64_t u_hi = share_lo + p.share_q + (wg < p.share_r ? 1 : 0);
  // A partial slot holds the accumulators as pairs [wave][pair][lane]: 512 contiguous bytes per instruction, and
  // every address is a uniform base plus the lane's 8-byte offset plus an immediate.
  constexpr size_t SLOT_PAIRS = (size_t)BM * BN / 2;
  const size_t wave_pairs = (size_t)wave * ACC_PAIRS * 64;

  // Adds workgroup w's partial to the accumulators: this wavefront's own portion, once w's wavefront of the same
  // index has raised its flag.  A wait that gives up poisons the tile: the failure is loud, the kernel still ends.
  auto add_partial = [&](int64_t w) {
    const uint32_t* flag = p.flags + w * 8 + wave;
    int ok = 1, polls = 0;
    while (__builtin_amdgcn_readfirstlane((int)__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) == 0) {
      if (++polls > p.spin_limit) {
        ok = 0;
        break;
      }
      __builtin_amdgcn_s_sleep(16);
    }
    uint32_t lane_here = lane;
    asm volatile("" : "+v"(lane_here));  // no address arithmetic in front of the loop over the parts (see the store)
    const uint64_t* src = p.partials + (size_t)w * SLOT_PAIRS + wave_pairs;
    // half of the partial at a time: all its loads are issued before the first is waited for (the registers of the
    // k-loop's prefetch stages are free here), so the pass costs a few round trips, not one per group
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint64_t t[ACC_PAIRS / 2];
#pragma unroll
      for (int g = 0; g < ACC_PAIRS / 2; ++g) {
        const int pair = half * (ACC_PAIRS / 2) + g;
        t[g] = __hip_atomic_load(src + (size_t)(pair / 8) * 8 * 64 + (pair % 8) * 64 + lane_here, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int g = 0; g < ACC_PAIRS / 2; ++g) {
        const int pair = half * (ACC_PAIRS / 2) + g;
        const int i = pair / 16, j = (pair / 8) % 2, q = pair % 8;
        const float lo = __builtin_bit_cast(float, (uint32_t)t[g]), hi = __builtin_bit_cast(float, (uint32_t)(t[g] >> 32));
        acc[i][j][2 * q] = ok ? acc[i][j][2 * q] + lo : __builtin_nanf("");
        acc[i][j][2 * q + 1] = ok ? acc[i][j][2 * q + 1] + hi : __builtin_nanf("");
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto share_begin = [&](int64_t w) { return w * p.share_q + (w < p.share_r ? w : p.share_r); };

  while (u_hi > share_lo) {
    const int tile = (int)((u_hi - 1) / p.upt);
    const int64_t tile_lo = (int64_t)tile * p.upt;
    const int64_t part_lo = share_lo > tile_lo ? share_lo : tile_lo;
    const int ks_begin = (int)(part_lo - tile_lo) * 2, ks_end = (int)(u_hi - tile_lo) * 2;
    const bool finalises = ks_end == p.ksteps;  // this part holds the tile's last unit
    u_hi = part_lo;

    // column-fastest tile order: the workgroups at work on neighbouring tiles share a slab of A
    m0 = (tile / p.tiles_n) * BM;
    n0 = (tile % p.tiles_n) * BN;
    a_tile = p.A + (int64_t)m0 * p.lda;
    w_tile = p.W + (int64_t)n0 * 16;
    meta_tile = p.meta + (int64_t)n0 * META_BYTES;  // meta entries are permuted inside 64-column slabs only
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      // rows beyond M re-read row M-1 and are never stored (a predicated load would serialise the loop)
      int r = a_row + i * 64;
      r = m0 + r < p.M ? r : p.M - 1 - m0;
      a_off[i] = (uint32_t)(((int64_t)r * p.lda + a_kc * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // ---- prologue: two steps in flight, A of the first landed, operands of slab 0 ready
    load_b(ks_begin, R0);
    load_b(ks_begin + 1, R1);
    // The parts below this one belong to workgroups wg-1, wg-2, ... down to the one whose share holds the tile's first
    // unit.  If that one's share begins below the tile, it computed its part first and went on: start from its sums.
    int64_t w_first = wg;  // lowest workgroup with a part of this tile
    if (finalises && ks_begin > 0) {
      do --w_first;
      while (share_begin(w_first) > tile_lo);
      if (share_begin(w_first) < tile_lo) add_partial(w_first);
    }
    __syncthreads();  // the previous part's epilogue is done with LDS
    int st0 = 0, st1 = STAGE_BYTES, st2 = 2 * STAGE_BYTES;  // staged tiles of steps ks, ks+1, ks+2
    load_a(ks_begin, st0);
    load_a(ks_begin + 1, st1);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lds0(0));
    __syncthreads();
    read_a(st0, 0, FA0);
    make_b(0, R0, FB0);

    for (int ks = ks_begin; ks < ks_end; ks += 2) {  // parts begin and end at even k-steps
      k_step(ks, R0, R1, st0, st1, st2);
      k_step(ks + 1, R1, R0, st1, st2, st0);
      const int t = st0;  // two steps on: (st0, st1, st2) <- (st2, st0, st1)
      st0 = st2;
      st2 = st1;
      st1 = t;
    }

    if (!finalises) {
      // ---- a lower part of a tile: the accumulators go to this workgroup's slot as they are, then the flag is raised
      // The lane offset is made opaque here: otherwise the compiler computes the 64 per-lane store addresses once, in
      // front of the loop over the parts, and spills them around the k-loop (128 registers).
      uint32_t lane_here = lane;
      asm volatile("" : "+v"(lane_here));
      uint64_t* dst = p.partials + (size_t)wg * SLOT_PAIRS + wave_pairs;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          uint64_t* grp = dst + (size_t)((i * 2 + j) * 8) * 64;  // uniform
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            // (copies first: a bit cast applied to a vector element expression reads the vector's first element)
            const float f_lo = acc[i][j][2 * q], f_hi = acc[i][j][2 * q + 1];
            const uint64_t v = (uint64_t)__builtin_bit_cast(uint32_t, f_lo) | ((uint64_t)__builtin_bit_cast(uint32_t, f_hi) << 32);
            __hip_atomic_store(grp + q * 64 + lane_here, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      __builtin_amdgcn_s_waitcnt(0);  // every store of this wavefront has been acknowledged by the memory system
      if (lane == 0) __hip_atomic_store(p.flags + wg * 8 + wave, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      continue;
    }

    if (ks_begin > 0) {
      // ---- the parts of workgroups whose whole share lies inside this tile end when this one does: nearest first
      for (int64_t w = wg - 1; w >= w_first; --w)
        if (share_begin(w) >= tile_lo) add_partial(w);
    }

    // ---- epilogue.  D[i][j] of a 32x32 tile: lane holds column j = lane % 32, rows 8*(r/4) + 4*(lane/32) + r%4.
    // Stored straight from the accumulators that is 2 bytes per lane and 64-byte row segments; instead each wavefront
    // transposes its block through its own slice of the (now idle) A buffers, 64 rows at a time, and writes whole
    // 128-byte rows with 16-byte stores.
    // Everything the epilogue derives from the lane index is derived here, from an opaque copy: computed once in
    // front of the loop over the parts it would stay in registers across the k-loop, which has none to spare.
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int li_e = lane_e & 31, kq_e = lane_e >> 5;
    float bcol[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + li_e;
      bcol[j] = (p.bias && n < p.N) ? (float)p.bias[n] : 0.f;
    }
    if (p.c_vec_ok) {
      constexpr int EP_STRIDE = 72;  // halves per staged row: 16-byte aligned rows, conflict-free 16-byte reads
      __syncthreads();               // every wavefront is done with the A tiles
      _Float16* ep = lds + wave * (64 * EP_STRIDE);
      const int erow = lane_e >> 3, ecol = (lane_e & 7) * 8;
      const int n_out = n0 + wn * 64 + ecol;
#pragma unroll
      for (int h = 0; h < TM / 2; ++h) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              ep[(ii * 32 + (r >> 2) * 8 + kq_e * 4 + (r & 3)) * EP_STRIDE + j * 32 + li_e] =
                  (_Float16)(acc[2 * h + ii][j][r] + bcol[j]);
        // LDS operations of one wavefront complete in issue order: the reads below see the writes above
        if (p.epi_kind == kMnbFusedMlp) {
          // a staged row is gate0 up0 gate1 up1 (16 columns each) = 32 output columns: four lanes per row, each reads
          // its 8 gate and 8 up values (narrowed to fp16, as the two separate products would be) and writes 8 outputs
          const int grow = lane_e >> 2, q = lane_e & 3;
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
        const int n = n0 + wn * 64 + j * 32 + li_e;
        if (n >= p.N) continue;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * 32 * TM + i * 32 + (r >> 2) * 8 + kq_e * 4 + (r & 3);
            if (m < p.M) p.C[(int64_t)m * p.ldc + n] = (_Float16)(acc[i][j][r] + bcol[j]);
          }
        }
      }
    }
  }
}

// Clears the flags of a split launch (a kernel, not a memset: callers may be capturing a HIP graph).
__global__ void __launch_bounds__(256) mnb_gemm256_clear_flags_kernel(uint32_t* flags, int n) {
  for (int i = threadIdx.x; i < n; i += 256) flags[i] = 0u;
}

template <int BITS, bool HAS_ZP, int MPS, int TM>
hipError_t launch_tm(const Gemm256Params& p, unsigned grid, hipStream_t s) {
  const size_t smem = (size_t)SMEM_BYTES;  // 98304 bytes
  auto kernel = mnb_gemm256_kernel<BITS, HAS_ZP, MPS, TM>;
  // The attribute belongs to the function on the current device, so it is set on every launch (a host-side table
  // update, no device work): callers on several threads or devices need no shared flag.
  if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      e != hipSuccess)
    return e;
  kernel<<<dim3(grid), dim3(THREADS), smem, s>>>(p);
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP, int MPS>
hipError_t launch(const Gemm256Params& p, unsigned grid, hipStream_t s) {
  return p.tile_rows == 128 ? launch_tm<BITS, HAS_ZP, MPS, 2>(p, grid, s) : launch_tm<BITS, HAS_ZP, MPS, 4>(p, grid, s);
}

size_t round256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

// How the tile GEMM would run a problem: rows of the tile (the 128-row tile when its grid fills the compute units in
// fewer, or at the kernel's step costs cheaper, rounds), the grid, whether tiles are split along K across workgroups
// (only with a workspace, and only when the tiles leave at least half of the compute units idle), the workspace that
// takes, and the estimated run time.  The kernel itself takes any division of the units into contiguous shares.
MnbGemm256Plan mnb_gemm256_plan(const MnbLayout& L, int64_t M, bool with_workspace) {
  const MnbDeviceInfo& dev = mnb_device_info();
  const int64_t tiles_n = (L.N + BN - 1) / BN;
  const int64_t ksteps = L.K / BK, upt = ksteps / 2;
  // cycles of one 64-deep k-step of a 256-row tile with the whole chip busy (4-bit; 8-bit; 8-bit with 16-wide blocks,
  // whose four meta entries per step spill): properties of the kernel's instruction schedule
  const double cycles256 = L.bits == 4 ? 3480.0 : (L.bs >= 32 ? 3960.0 : 7080.0);
  const int64_t cus = dev.cus;
  MnbGemm256Plan best{};
  for (int rows = 256; rows >= 128; rows -= 128) {
    const double step = cycles256 / dev.clock_hz * (rows == 256 ? 1.0 : kMnbGemm128StepRatio);
    const int64_t tiles = ((M + rows - 1) / rows) * tiles_n;
    MnbGemm256Plan pl{};
    pl.tile_rows = rows;
    pl.grid = tiles;
    pl.seconds = (double)((tiles + cus - 1) / cus) * (double)ksteps * step;
    if (with_workspace && tiles * 4 <= cus && M > 768) {
      // Few tiles of a tall problem: every tile is cut into `parts` equal ranges of k (2 ... 4, each at least 32
      // k-steps deep), one workgroup per part.  The finishing pass -- every lower part writes its sums, the top part
      // waits for them and adds them one after the other -- costs about 8 us for two parts plus 8 us for each further
      // one (256-row tiles), and a part its k-steps at about 1.15 of the steady-state step.  Measured on the
      // Llama-3-8B projections (M = 1024, N = 4096): K = 4096 in two parts 49 us against 51 us on the streaming kernel
      // and 59 us unsplit; K = 14336 in four parts 134 us against 141 us and 191 us; 8-bit weights 139 us against
      // 151 us.  With a quarter of the compute units or more already busy the split loses (96 ... 128 tiles in two
      // parts: 66 against 63 us, 80 against 76 us), and with whole rounds of tiles equal shares bring nothing either:
      // the chip is power-limited there, a balanced schedule runs at a lower clock for the same total time
      // (M = 2048, N = 14336: 223 us of arithmetic in equal shares against 225 us in two unequal rounds, plus the
      // finishing pass).
      int64_t parts = cus / tiles < 4 ? cus / tiles : 4;
      while (parts > 1 && (upt % parts != 0 || ksteps / parts < 32)) --parts;
      if (parts > 1) {
        const double pass = rows == 256 ? 8e-6 : 4e-6;
        const double t = (double)(ksteps / parts) * step * 1.15 + pass * (double)(parts - 1);
        if (t < pl.seconds) {
          pl.seconds = t;
          pl.grid = tiles * parts;
          pl.split = true;
          pl.workspace_bytes =
              round256((size_t)pl.grid * 8 * sizeof(uint32_t)) + (size_t)pl.grid * rows * BN * sizeof(float);
        }
      }
    }
    if (rows == 256 || pl.seconds < best.seconds) best = pl;
  }
  return best;
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
  const MnbGemm256Plan plan_ws = mnb_gemm256_plan(a.L, a.M, true);
  const bool ws_ok = plan_ws.split && a.workspace != nullptr && a.workspace_bytes >= plan_ws.workspace_bytes &&
                     reinterpret_cast<uintptr_t>(a.workspace) % 8 == 0;
  const MnbGemm256Plan plan = ws_ok ? plan_ws : mnb_gemm256_plan(a.L, a.M, false);
  p.tile_rows = plan.tile_rows;
  p.tiles_m = (int)((a.M + p.tile_rows - 1) / p.tile_rows);
  p.tiles_n = (int)((a.L.N + BN - 1) / BN);
  p.upt = p.ksteps / 2;
  const int64_t units = (int64_t)p.tiles_m * p.tiles_n * p.upt;
  if ((int64_t)p.tiles_m * p.tiles_n > 0x7fffffff) return hipErrorInvalidValue;
  p.share_q = units / plan.grid;
  p.share_r = units % plan.grid;
  p.spin_limit = 1 << 20;  // polls half a microsecond apart: seconds, where a healthy wait takes microseconds
  if (plan.split) {
    p.flags = reinterpret_cast<uint32_t*>(a.workspace);
    p.partials = reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(a.workspace) +
                                             round256((size_t)plan.grid * 8 * sizeof(uint32_t)));
    mnb_gemm256_clear_flags_kernel<<<dim3(1), dim3(256), 0, s>>>(p.flags, (int)plan.grid * 8);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  }
  const unsigned grid = (unsigned)plan.grid;
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
  if (a.L.bits == 4) return a.L.has_zp ? launch<4, true, 2>(p, grid, s) : launch<4, false, 2>(p, grid, s);
  // 8-bit: two entries per k-step fit the register file without spills (also for blocks of 64 and more, where both
  // entries name the same block); blocks of 16 need four and spill
  if (a.L.bs >= 32) return a.L.has_zp ? launch<8, true, 2>(p, grid, s) : launch<8, false, 2>(p, grid, s);
  return a.L.has_zp ? launch<8, true, 4>(p, grid, s) : launch<8, false, 4>(p, grid, s);
}
