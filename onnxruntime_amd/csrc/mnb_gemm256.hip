// MFMA GEMM for fp16 models and large M: 256 x 256 output tile per workgroup, weights dequantised in registers.
//
// Device counterpart of the reference's prefill loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:
// 563-732: dequantise a strip of B, then run the float GEMM kernel over it).
//
// Eight wavefronts (1 x 8, two per SIMD), each owning all 256 rows and 32 columns of the tile as 8 x 1
// v_mfma_f32_32x32x16_f16 accumulators (WM below; the 2 x 4 arrangement the kernel started with is kept for
// calibration builds).  Per k-step of 64:
//   * A (activations) goes from global memory straight into LDS (buffer_load_dwordx4 ... lds: no registers, no LDS
//     store instructions), two k-steps ahead, into one of three staged tiles.  Such a load puts the 16 bytes of lane
//     L at (wave-uniform LDS base) + 16 L, so a wavefront fills 8 rows x 128 bytes with one instruction; the rows are
//     not padded, instead the lane that fills chunk position p of row r fetches chunk p ^ ((r >> 1) & 7) of that
//     row, and the readers (ds_read_b128, lane = row) apply the same XOR.  The LDS serves such a read 16 lanes at a
//     time from 64 banks: 16 consecutive rows must start in 16 different 16-byte bank groups, and rows r, r+2, ... r+14 (same
//     half of the 256 bytes that two rows span) get the 8 different chunk positions: conflict free.
//   * B (weights) never touches LDS.  Lane (column j = lane%32, half kq = lane/32) of a wavefront loads, two steps
//     ahead (each register is reloaded right after its last use, and the loop states its own exact waits: see
//     LoadPlan), exactly the 8 bytes of packed weights it will feed to the matrix core: the two 32-bit words of its
//     column's 16-byte vector that belong to its half.  Each word is dequantised in registers to 8 halves -- exact
//     (q - zp), one rounding by the scale, bit-identical to the reference's fp16 dequantisation -- and IS the MFMA
//     B operand of one k-slab.  (The contraction index of an MFMA may be permuted freely as long as A uses the same
//     permutation: for 4-bit weights slab 2g takes k = 32g + 16kq + [0,8) and slab 2g+1 takes 32g + 16kq + [8,16).)
//     LDS traffic is what bounded the design that staged a dequantised B tile in LDS (every wavefront re-read it).
//     With the 1 x 8 arrangement every column is dequantised exactly once per workgroup.
//   * one barrier per step; the dequantisation of slab s+1 is issued among slab s's MFMAs (on this hardware vector
//     and matrix instructions of a SIMD overlap only partly: a k-step costs close to the sum of the two).
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
// same from run to run.
// The hand-over of a partial.  Every access to partials and flags is a relaxed device-scope atomic, which on this
// hardware is an access that bypasses the per-XCD caches (sc1: stores write through to, and loads are served from,
// the level all XCDs share); no fence instruction is involved.  What orders data before flag:
//   writer: s_waitcnt vmcnt(0) between the partial's stores and the flag's store -- a write-through store is counted
//           as outstanding until that shared level has acknowledged it, so the flag cannot become visible first;
//   reader: the partial's loads are issued behind the branch that leaves the polling loop, and the branch needs the
//           flag's value: a wavefront issues in order and never speculates past a branch, so no load of the partial
//           is in flight before a poll has returned 1.
// The compiler is held to the same order by signal fences (no instructions) on both sides.  Device-scope release /
// acquire fences in their place (MNB_SPLIT_FENCES=1: the writer's becomes a write-back of its XCD's L2, the reader's
// an invalidation) were measured at +12 to +18 us per launch on every split shape (M = 1024, N = 4096, K = 14336:
// 134.2 against 119.7 us; M = 512, N = K = 8192: 90.0 against 73.5 us) with bit-identical results, and are not used.
// Progress.  A workgroup waits only for workgroups with smaller indices, and the plan never splits into more than
// two rounds of workgroups: what is relied on is that workgroup w is not dispatched before workgroups 0 .. w-1
// (one-dimensional grids are dispatched in index order).  Should that ever fail, a wait ends after spin_limit polls:
// it poisons its tile with NaN and sets the status word behind the flags, which MnbGemmWorkspaceStatus reads back.
// Flags and status word are cleared by a small kernel in front of the launch, so a workspace must not be shared by
// launches that may overlap.
// Without a workspace the grid is one workgroup per tile and nothing is split.
#include <cstdlib>
#include <type_traits>

#include "mnb_bf16.hip.h"
#include "mnb_buffer.hip.h"
#include "mnb_device.hip.h"
#include "mnb_internal.h"

#if !defined(MNB_SPLIT_FENCES)
#define MNB_SPLIT_FENCES 0  // 1 (calibration builds): device-scope release / acquire fences around the flag hand-over
#endif

namespace {

constexpr int BK = 64;
constexpr int ROW_BYTES = BK * 2;  // bytes per staged A row (eight 16-byte chunks, XOR-swizzled with the row)
// Rows of the tile: 64 * TM (TM = 4: 256 x 256; TM = 2: 128 x 256 for grids that leave most of the chip idle with
// the large tile).  The dynamic LDS allocation is that of TM = 4 for both: three staged A tiles of 32 KiB; the
// epilogue stages 64 rows of each wavefront's columns in it (40 KiB).
constexpr int SMEM_BYTES = 3 * 256 * ROW_BYTES;
// Order in which a wavefront issues its vector-memory operations in a k-step of the tile GEMM, and what each wait
// of the step may leave outstanding.  The k-loop states its waits itself (the one in front of the barrier has to: the
// compiler does not know that other wavefronts read what this one's loads put into LDS; the others pin the weights'
// two k-steps of latency whatever the scheduler does with the loads).  They are exact as long as the issue order
// below is the one in the generated code; tests/test_isa_tile_gemm.py checks that, and that the compiler saw no need
// to add a wait of its own.
//   slot 0: the A loads into LDS for step s+2 (first thing in slab 0)
//   slot q = 1, 2, 3: the weight registers last read when the operands of slab q were made (that happens in the
//           section of slab q-1; the reload follows at once), for step s+2
//   slot 4: those last read when the operands of slab 0 of step s+1 were made (behind the barrier), for step s+3
// 4-bit: a vector serves two slabs and has a meta entry of its own; 8-bit: one vector per slab, a meta entry serves
// 4 / MPS slabs.  A register is reloaded right after its last use, so every datum has about two k-steps to arrive.
template <int KK>
struct Slab {
  static constexpr int value = KK;
};

template <int BITS, int MPS, int A_LOADS, int CT>
struct LoadPlan {
  static constexpr int VPS = (BITS == 4) ? 2 : 4;
  static constexpr int slot_after(int kk) { return kk == 0 ? 4 : kk; }  // slot that follows make_b(kk)
  static constexpr int vec_of_slab(int kk) { return BITS == 4 ? kk >> 1 : kk; }
  static constexpr int meta_of_slab(int kk) { return BITS == 4 ? kk >> 1 : kk * MPS / 4; }
  static constexpr int vec_slot(int v) { return slot_after(BITS == 4 ? 2 * v + 1 : v); }
  static constexpr int meta_slot(int e) { return slot_after(BITS == 4 ? 2 * e + 1 : (e + 1) * 4 / MPS - 1); }
  static constexpr int size(int q) {
    if (q == 0) return A_LOADS;
    int n = 0;
    for (int v = 0; v < VPS; ++v) n += vec_slot(v) == q ? CT : 0;  // one load per column tile of the wavefront
    for (int e = 0; e < MPS; ++e) n += meta_slot(e) == q ? CT : 0;
    return n;
  }
  static constexpr int before(int q) {  // operations of a step in front of slot q
    int n = 0;
    for (int i = 0; i < q; ++i) n += size(i);
    return n;
  }
  static constexpr int per_step() { return before(5); }
  // operations younger than the group of slot q issued `steps` k-steps earlier, seen from in front of slot q_now
  static constexpr int younger(int q, int steps, int q_now) {
    return steps * per_step() + before(q_now) - before(q) - size(q);
  }
  // what the wait in front of make_b(kk) may leave outstanding.  The data of step u sit in slots 1..3 of step u-2 or
  // in slot 4 of step u-3; make_b(0) prepares step s+1 during step s, the others step s.
  static constexpr int wait_of_slab(int kk) {
    const int ahead = kk == 0 ? 1 : 0, q_now = slot_after(kk);
    const int qv = vec_slot(vec_of_slab(kk)), qm = meta_slot(meta_of_slab(kk));
    const int yv = younger(qv, (qv == 4 ? 3 : 2) - ahead, q_now);
    const int ym = younger(qm, (qm == 4 ? 3 : 2) - ahead, q_now);
    return yv < ym ? yv : ym;
  }
  // the barrier of step s: A of step s+1 (slot 0 of step s-1) has landed, and slab 0's weights of step s+1 are there
  static constexpr int wait_of_barrier() {
    const int ya = younger(0, 1, 4), yb = wait_of_slab(0);
    return ya < yb ? ya : yb;
  }
  // a slab whose weights the previous slab's wait has already covered needs none
  static constexpr bool slab_waits(int kk) { return !(BITS == 4 && (kk & 1)); }
};

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
  int tile_cols;  // 256, or 128 with 128 rows
  // work distribution: `units` = tiles x ksteps / 2 split over the grid; workgroup w takes
  // [w * share_q + min(w, share_r), (w + 1) * share_q + min(w + 1, share_r))
  int upt;                  // units per tile
  int64_t share_q, share_r;
  uint64_t* partials;       // one slot of tile_rows x tile_cols floats per workgroup (NULL: grid == tiles, nothing is split)
  uint32_t* flags;          // one word per workgroup and wavefront, zero when the kernel starts
  uint32_t* status;         // one word behind the flags, zero when the kernel starts: set to 1 by a wait that gave up
  int spin_limit;           // polls of a flag before the wait gives up and the tile is poisoned with NaN
  int test_drop_odd_lower;  // test builds only: the lower parts of odd-numbered tiles are not computed (their flags
                            // stay zero, so the finalising parts of those tiles run into the bounded wait)
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

// End of one slab section (its matrix instructions, the LDS reads and the dequantisation of the next slab's operands,
// a group of loads).  Inside a section the compiler's scheduler interleaves freely; it does that slightly better than
// a hand-written order of "one MFMA, one LDS read, two loads, n VALU" per matrix instruction (measured: 1-2 % on every
// shape).  A fence between sections keeps it from pulling the next slab's work forward, which pays everywhere (1-4 %)
// except in the 256-row 4-bit kernel, where letting it mix the sections of a k-step is worth another 2 %.
template <bool FENCE, int INTERLEAVE = 0>
__device__ __forceinline__ void slab_end() {
  // INTERLEAVE matrix instructions, each followed by up to three vector instructions (one wavefront per SIMD: the
  // dequantisation of the next slab has to sit between this slab's matrix instructions, nobody else fills the gaps)
  if constexpr (INTERLEAVE > 0) {
#pragma unroll
    for (int k = 0; k < INTERLEAVE; ++k) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
    }
  }
  if constexpr (FENCE) __builtin_amdgcn_sched_barrier(0);
}

// MPS: meta entries (scale, zero point) a lane keeps per k-step and column tile.  A k-step of 64 spans 64 / block_size
// blocks; 4-bit vectors cover 32 k, so two entries serve every block size (16-wide blocks through the lane's half
// kq); 8-bit vectors cover 16 k: 4 entries for blocks of 16, 2 for blocks of 32 and more.
// WM: rows of the 2-D arrangement of the eight wavefronts over the tile.  WM = 2 (2 x 4): a wavefront owns
// 32 TM rows x 64 columns, and the two wavefront rows dequantise the same columns.  WM = 1 (1 x 8): a wavefront owns
// all 64 TM rows x 32 columns: every column is dequantised once per workgroup (half the vector instructions) and
// every wavefront reads the whole staged A tile (twice the LDS reads).
// DT: 0 = fp16 model (packed with fp16 meta entries); on a matrix packed with fp32 meta entries: 1 = bfloat16 model,
// 2 = fp16 model with zero points in the activation type.
// NWV: wavefronts of the workgroup, 8 (256 columns) or 4 (128 columns: twice the tiles for problems whose 256-column
// tiles leave compute units idle; same work per wavefront).
// CTW: 32-column matrix-core tiles per wavefront.  WM for the eight-wavefront arrangements; 2 with four wavefronts side by
// side (1 x 4: a wavefront owns all 64 TM rows x 64 columns, one wavefront per SIMD with the accumulators in the
// second half of its register file: every column is still dequantised once, and the staged A tile is read four times
// instead of eight).  The 1 x 4 arrangement exists in calibration builds only: bit-identical results, half the LDS
// reads (4.66 M instead of 8.34 M per launch of M = 2048, N = 14336, K = 4096), but a single wavefront per SIMD leaves
// the matrix pipe idle while it issues its own vector instructions: 3217 cycles per k-step against 2460, 231.5 us
// against 212.0 us on the same box although the power limit then allows 2.10 instead of 1.82 GHz; with the order inside a
// slab section stated by hand (one matrix instruction, two vector instructions, one LDS read, one load) 244.7 us.
// With the LDS reads of the next slab pinned to the head of each slab section and the dequantisation placed between
// the matrix instructions by scheduling groups (what a wavefront that is alone on its SIMD needs; both apply to this
// arrangement only) 1 x 4 comes to 229.3 against 210.9 us: 481 K against 389 K cycles per launch, 45 % of a
// wavefront's cycles still spent in waits.
// What bounds the launch is energy, not issue slots.  A loop of nothing but the kernel's mix (mnb_probe.hip: per
// matrix instruction two vector instructions and one 1 KB LDS operand read issued a whole iteration ahead, two
// wavefronts per SIMD, constant operands) runs at 29.0 ns per matrix instruction and wavefront against 27.05 ns for
// the matrix instructions alone: the mix costs 7 % of the issue slots.  Ablation builds of this kernel on C4 (results
// wrong on purpose) keep its cycle count and change its clock: complete 385 K cycles per launch in 208.7 us
// (1.85 GHz); without the LDS operand reads 378 K in 186.2 us (2.03 GHz); without the dequantisation arithmetic
// 382 K in 180.0 us (2.12 GHz); without both 361 K in 154.0 us (2.35 GHz, the time the complete kernel needs on
// all-zero activations); without the step's barrier 372 K in 206.9 us.  The matrix cores on random fp16 operands
// take most of the power budget; every LDS read and vector instruction beside them is paid for in clock.
// Raising the priority of a wavefront around its matrix instructions (s_setprio 1 or 3) costs 1.5 to 2 % on every
// shape.
template <int BITS, bool HAS_ZP, int MPS, int TM, int WM, int DT, int NWV, int CTW = WM>
__global__ void __launch_bounds__(64 * NWV, (2 * TM / WM) * CTW * 16 > 128 ? 1 : 2) mnb_gemm256_kernel(Gemm256Params p) {
  constexpr int THREADS = 64 * NWV;
  constexpr int WN = NWV / WM;       // wavefront columns
  constexpr int CT = CTW;            // 32-column matrix-core tiles per wavefront
  constexpr int BN = 32 * CT * WN;   // columns of the tile
  constexpr int ROWS_PER_LOAD = THREADS / 8;  // rows of A one load instruction of the workgroup stages
  constexpr int RT = 2 * TM / WM;    // 32-row matrix-core tiles per wavefront
  constexpr int WCOLS = 32 * CT;     // columns of a wavefront
  constexpr int BM = 64 * TM;                       // rows of the tile
  constexpr int STAGE_BYTES = BM * ROW_BYTES;       // one staged A tile
  constexpr bool SLAB_FENCE = !(TM == 4 && (BITS == 4 || MPS == 4));  // (8-bit with four meta entries: fenced it spills)
  constexpr int A_LOADS = BM * (BK / 8) / THREADS;  // 16-byte activation loads per thread per k-step: TM
  // 4-bit: a 16-byte vector spans two slabs (one word each per lane); 8-bit: one slab (two words per lane)
  constexpr int VEC_PER_STEP = (BITS == 4) ? 2 : 4;  // 8-byte weight loads per lane, column tile and k-step
  constexpr int ACC_PAIRS = RT * CT * 8;             // 8-byte pairs of accumulators per lane
  using Plan = LoadPlan<BITS, MPS, A_LOADS, CT>;
  extern __shared__ __align__(16) unsigned char lds_bytes[];
  _Float16* const lds = reinterpret_cast<_Float16*>(lds_bytes);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;  // rows wm * 32 RT, columns wn * WCOLS
  const int li = lane & 31, kq = lane >> 5;

  f16_t acc[RT][CT];

  // Two register sets for the weight prefetch (distance: two k-steps); the activations need none.
  constexpr bool WIDE = DT != 0;                                          // fp32 meta entries
  using meta_t = std::conditional_t<WIDE && HAS_ZP, u2_t, uint32_t>;  // fp16 entries: {scale, zp} halves; fp32: floats
  struct Stage {
    u2_t b[VEC_PER_STEP][CT];     // [vector of the k-step][column tile]
    meta_t m[MPS][CT];            // meta entries of the blocks of the k-step (see m_off)
  };
  Stage R0, R1;
  h8_t FA0[RT], FA1[RT];  // A operands, double buffered over slabs
  h8_t FB0[CT], FB1[CT];  // B operands, double buffered over slabs

  const UnpackConsts uc = make_unpack_consts();

  // Addressing: every global access is a buffer access:  uniform base (a resource in SGPRs: the tile's corner,
  // advanced per k-step)  +  32-bit per-lane offset (a VGPR), so the loads cost no VALU work inside the loop.  (The
  // flat form of the load into LDS is also what makes the compiler wait for all outstanding loads wherever it needs
  // one of them; with the buffer form its waits are exact.)  The tile's first row and column are
  // part of the uniform base, so a lane's offsets span at most 255 rows of A and 256 columns of weights: they fit
  // 32 bits for every M and N as long as 512 * lda does (mnb_gemm256_addressable).
  // Load i of a wavefront fills rows i * ROWS_PER_LOAD + wave * 8 + [0, 8) of the staged tile; the lane at chunk position
  // lane & 7 of row lane >> 3 fetches chunk (lane & 7) ^ ((row >> 1) & 7).
  const int a_row = tid >> 3, a_kc = (tid & 7) ^ ((tid >> 4) & 7);
  uint32_t a_off[A_LOADS];                     // byte offsets from a_tile + k0; set per tile (rows beyond M)
  // this lane's weight columns (one per column tile): its 8 bytes inside each 16-byte vector, and its meta entries.
  // The block of a lane's half vector is (k-group base >> bs_shift), plus kq when 4-bit blocks are 16 wide.
  constexpr int META_BYTES = (WIDE ? 2 : 1) * (HAS_ZP ? 4 : 2);
  const bool small_bs = (BITS == 4) && p.bs_shift == 4;
  // Without zero points an entry is a 16-bit scale.  A 16-bit load would be zero-extended, or packed with its
  // neighbour, right behind the load, which needs the data at once and defeats the prefetch: the lane loads the
  // aligned 32-bit word that holds its scale and shifts by m_shift (0 or 16) when it uses it.
  uint32_t w_off[CT], m_off[CT], m_shift[CT];
#pragma unroll
  for (int j = 0; j < CT; ++j) {
    const int col = wn * WCOLS + j * 32 + li;  // within the tile; tiles start at multiples of 256 columns
    w_off[j] = (uint32_t)(col * 16 + kq * 8);
    const uint32_t m_byte = (uint32_t)((mnb_meta_col(col) + (small_bs ? kq * p.Npad : 0)) * META_BYTES);
    m_off[j] = WIDE ? m_byte : (m_byte & ~3u);
    m_shift[j] = (m_byte & 2u) * 8;
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
    const rsrc_t r = mnb_rsrc(a_tile + (int64_t)ks * BK);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      mnb_buffer_load_lds_b128(r, a_off[i],
                               (lds_ptr_t)(lds_bytes + stage_off + (i * ROWS_PER_LOAD + wave * 8) * ROW_BYTES));
  };
  // One issue group of the weight prefetch: the loads of issue slot `slot` (see LoadPlan) for k-step ks_raw.
  auto load_b_slot = [&](int ks_raw, Stage& R, int slot) {
    const int ks = ks_raw < last_step ? ks_raw : last_step;
#pragma unroll
    for (int v = 0; v < VEC_PER_STEP; ++v) {
      if (Plan::vec_slot(v) != slot) continue;
      const int64_t kg = (int64_t)ks * VEC_PER_STEP + v;  // k-group of the vector
      const rsrc_t r = mnb_rsrc(w_tile + kg * vec_pitch);
#pragma unroll
      for (int j = 0; j < CT; ++j) R.b[v][j] = mnb_buffer_load_b64(r, w_off[j]);
    }
#pragma unroll
    for (int e = 0; e < MPS; ++e) {
      if (Plan::meta_slot(e) != slot) continue;
      const int64_t kb = ((int64_t)ks * BK + e * (BK / MPS)) >> p.bs_shift;  // block of the entry's first element
      const rsrc_t r = mnb_rsrc(meta_tile + kb * meta_pitch);
#pragma unroll
      for (int j = 0; j < CT; ++j) {
        if constexpr (WIDE && HAS_ZP)
          R.m[e][j] = mnb_buffer_load_b64(r, m_off[j]);
        else
          R.m[e][j] = mnb_buffer_load_b32(r, m_off[j]);
      }
    }
  };
  auto load_b = [&](int ks_raw, Stage& R) {
#pragma unroll
    for (int slot = 1; slot <= 4; ++slot) load_b_slot(ks_raw, R, slot);
  };
  // Waits until the weights that slab kk of a k-step needs have arrived (`vm`: the number of younger vector-memory
  // operations, from LoadPlan), and ties the registers to the wait: no use of them can be scheduled in front of it.
  auto await_b = [&](auto slab, Stage& R) {
    constexpr int kk = decltype(slab)::value;
    constexpr int vm = kk == 0 ? Plan::wait_of_barrier() : Plan::wait_of_slab(kk);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(vm));
    constexpr int v = Plan::vec_of_slab(kk), e = Plan::meta_of_slab(kk);
#pragma unroll
    for (int j = 0; j < CT; ++j) {
      asm volatile("; b %0" : "+v"(R.b[v][j]));
      asm volatile("; m %0" : "+v"(R.m[e][j]));
    }
  };

  auto decode = [&](auto raw_any, int j, h2_t& s2, ZpH& z) {  // fp16 models only
    const uint32_t raw = (uint32_t)raw_any;
    if constexpr (HAS_ZP) {
      const h2_t m = mnb_as_h2(raw);
      s2 = mnb_h2(m.x);
      z = mnb_zp_h(m.y);
    } else {
      s2 = mnb_h2(__builtin_bit_cast(_Float16, (uint16_t)(raw >> m_shift[j])));
      z = mnb_zp_h((_Float16)(-(1024.0f + (float)(1 << (BITS - 1)))));
    }
  };

  // B operands of slab kk (0..3) of the k-step held in R
  auto make_b = [&](int kk, const Stage& R, h8_t* FB) {
#pragma unroll
    for (int j = 0; j < CT; ++j) {
      const int v = BITS == 4 ? kk >> 1 : kk;           // the vector of the slab
      const int e = BITS == 4 ? kk >> 1 : kk * MPS / 4;  // its meta entry
      const uint32_t w0 = BITS == 4 ? R.b[v][j][kk & 1] : R.b[v][j][0];
      const uint32_t w1 = BITS == 4 ? 0u : R.b[v][j][1];
      if constexpr (WIDE) {
        float sc, zp;
        if constexpr (HAS_ZP) {
          const uint32_t sc_bits = R.m[e][j][0], zp_bits = R.m[e][j][1];  // (a bit cast straight from a vector
          sc = __builtin_bit_cast(float, sc_bits);                        // element reads element 0 for both)
          zp = __builtin_bit_cast(float, zp_bits);
        } else {
          sc = __builtin_bit_cast(float, R.m[e][j]);
          zp = (float)(1 << (BITS - 1));
        }
        FB[j] = dequant_word_wide<BITS, DT == 1>(w0, w1, sc, -zp * sc);
      } else {
#if defined(MNB_ABLATE_NO_DEQUANT)  // (calibration builds: the packed bits go to the matrix cores as they are)
        const u4_t raw = {w0, w1, (uint32_t)R.m[e][j], w0};
        FB[j] = __builtin_bit_cast(h8_t, raw);
#else
        h2_t s2;
        ZpH z;
        decode(R.m[e][j], j, s2, z);
        FB[j] = dequant_word<BITS>(w0, w1, uc, z, s2);
#endif
      }
    }
  };

  // A operands of slab kk: lane (row li, half kq).  The k permutation matches the weights' (see the file header);
  // a_rd[kk] is the lane's byte offset inside a staged tile, chunk swizzle included.
  uint32_t a_rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    const int chunk = (BITS == 4) ? 4 * (kk >> 1) + 2 * kq + (kk & 1) : 2 * kk + kq;
    a_rd[kk] = (uint32_t)((wm * 32 * RT + li) * ROW_BYTES + ((chunk ^ ((li >> 1) & 7)) * 16));
  }
  auto read_a = [&](int stage_off, int kk, h8_t* FA) {
#if defined(MNB_ABLATE_NO_LDS_READS)  // (calibration builds: the A operands keep whatever the registers hold)
#pragma unroll
    for (int t = 0; t < RT; ++t) asm volatile("; keep %0" : "+v"(FA[t]));
    return;
#endif
    const unsigned char* As = lds_bytes + stage_off + a_rd[kk];
#pragma unroll
    for (int t = 0; t < RT; ++t) FA[t] = *reinterpret_cast<const h8_t*>(As + t * 32 * ROW_BYTES);
  };

  auto mfma_slab = [&](const h8_t* FA, const h8_t* FB) {
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < CT; ++j)
        if constexpr (DT == 1) {
#if defined(__HIP_DEVICE_COMPILE__)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8_t, FA[i]),
                                                               __builtin_bit_cast(bf8_t, FB[j]), acc[i][j], 0, 0, 0);
#endif
        } else {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(FA[i], FB[j], acc[i][j], 0, 0, 0);
        }
  };

  // One k-step.  On entry: the staged tile at `cur` holds A of step ks, the one at `nxt` is receiving A of step ks+1,
  // the one at `nn` is free (its readers passed the barrier of step ks-1); FA0/FB0 hold the operands of slab 0, Rc
  // holds the weights of step ks, Rn holds (or is receiving) those of step ks+1.
  // One wavefront per SIMD (four wavefronts) has nobody to hide an LDS wait behind: the reads of the next slab's A
  // operands stay where they are written, at the head of the section, a slab ahead of their use (left alone the
  // scheduler sinks them to just in front of it to save registers).
  auto reads_stay_here = [] {
    if constexpr (NWV == 4 && CTW == 2) __builtin_amdgcn_sched_barrier(0);
  };
  auto k_step = [&](int ks, Stage& Rc, Stage& Rn, int cur, int nxt, int nn) {
    // slab 0: operands of slab 1; A of step ks+2 on its way into the free tile
    load_a(ks + 2, nn);
    read_a(cur, 1, FA1);
    reads_stay_here();
    if constexpr (Plan::slab_waits(1)) await_b(Slab<1>{}, Rc);
    make_b(1, Rc, FB1);
    mfma_slab(FA0, FB0);
    load_b_slot(ks + 2, Rc, 1);
    slab_end<SLAB_FENCE || (NWV == 4 && CTW == 2), (NWV == 4 && CTW == 2) ? RT * CT : 0>();
    // slab 1: operands of slab 2
    read_a(cur, 2, FA0);
    reads_stay_here();
    if constexpr (Plan::slab_waits(2)) await_b(Slab<2>{}, Rc);
    make_b(2, Rc, FB0);
    mfma_slab(FA1, FB1);
    load_b_slot(ks + 2, Rc, 2);
    slab_end<SLAB_FENCE || (NWV == 4 && CTW == 2), (NWV == 4 && CTW == 2) ? RT * CT : 0>();
    // slab 2: operands of slab 3
    read_a(cur, 3, FA1);
    reads_stay_here();
    if constexpr (Plan::slab_waits(3)) await_b(Slab<3>{}, Rc);
    make_b(3, Rc, FB1);
    mfma_slab(FA0, FB0);
    load_b_slot(ks + 2, Rc, 3);
    slab_end<SLAB_FENCE || (NWV == 4 && CTW == 2), (NWV == 4 && CTW == 2) ? RT * CT : 0>();
    // The barrier of the step.  Before it a wavefront makes sure that its own part of A of step ks+1 has landed in
    // LDS (issued in slab 0 of step ks-1) and that the weights of slab 0 of step ks+1 are there; LoadPlan counts the
    // operations younger than both.  The wavefront's LDS reads have completed too, so the tile at `cur` may be
    // overwritten from the next step on.  No fence: the fence of __syncthreads would wait for every outstanding load.
    // Nothing may move across: a dequantisation step of slab 3 hoisted above the wait would need a wait of its own.
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lds0(Plan::wait_of_barrier()));
#if !defined(MNB_ABLATE_NO_BARRIER)  // (calibration builds: what the step's barrier costs; results are then wrong)
    __builtin_amdgcn_s_barrier();
#endif
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // slab 3, behind the barrier: operands of slab 0 of step ks+1
    read_a(nxt, 0, FA0);
    reads_stay_here();
    await_b(Slab<0>{}, Rn);
    make_b(0, Rn, FB0);
    mfma_slab(FA1, FB1);
    load_b_slot(ks + 3, Rn, 4);
    slab_end<SLAB_FENCE || (NWV == 4 && CTW == 2), (NWV == 4 && CTW == 2) ? RT * CT : 0>();
  };

  // bias and output in the model's 16-bit type (the pointers are typed _Float16 for both: bfloat16 travels as bits)
  auto widen_elem = [](_Float16 v) {
    if constexpr (DT == 1) return bf16_widen(__builtin_bit_cast(uint16_t, v));
    else return (float)v;
  };
  auto narrow_elem = [](float v) {
    if constexpr (DT == 1) return __builtin_bit_cast(_Float16, (__bf16)v);
    else return (_Float16)v;
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
    if (!ok && lane == 0) __hip_atomic_store(p.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);  // the compiler keeps the partial's loads behind the loop (file header)
#if MNB_SPLIT_FENCES
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#endif
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
        const int i = pair / 8 / CT, j = pair / 8 % CT, q = pair % 8;
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
#if defined(MNB_TEST_HOOKS)
    if (!finalises && p.test_drop_odd_lower && (tile & 1)) continue;
#endif

    // column-fastest tile order: the workgroups at work on neighbouring tiles share a slab of A
    m0 = (tile / p.tiles_n) * BM;
    n0 = (tile % p.tiles_n) * BN;
    a_tile = p.A + (int64_t)m0 * p.lda;
    w_tile = p.W + (int64_t)n0 * 16;
    meta_tile = p.meta + (int64_t)n0 * META_BYTES;  // meta entries are permuted inside 64-column slabs only
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      // rows beyond M re-read row M-1 and are never stored (a predicated load would serialise the loop)
      int r = a_row + i * ROWS_PER_LOAD;
      r = m0 + r < p.M ? r : p.M - 1 - m0;
      a_off[i] = (uint32_t)(((int64_t)r * p.lda + a_kc * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < CT; ++j)
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
    load_b_slot(ks_begin + 2, R0, 4);  // the loop's issue order from here on (LoadPlan)

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
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < CT; ++j) {
          uint64_t* grp = dst + (size_t)((i * CT + j) * 8) * 64;  // uniform
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            // (copies first: a bit cast applied to a vector element expression reads the vector's first element)
            const float f_lo = acc[i][j][2 * q], f_hi = acc[i][j][2 * q + 1];
            const uint64_t v = (uint64_t)__builtin_bit_cast(uint32_t, f_lo) | ((uint64_t)__builtin_bit_cast(uint32_t, f_hi) << 32);
            __hip_atomic_store(grp + q * 64 + lane_here, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      // release: every store of this wavefront is visible to the device before the flag is
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
#if MNB_SPLIT_FENCES
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#else
      __builtin_amdgcn_s_waitcnt(0);  // every store of this wavefront has been acknowledged by the memory system
#endif
      __atomic_signal_fence(__ATOMIC_SEQ_CST);
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
    float bcol[CT];
#pragma unroll
    for (int j = 0; j < CT; ++j) {
      const int n = n0 + wn * WCOLS + j * 32 + li_e;
      bcol[j] = (p.bias && n < p.N) ? widen_elem(p.bias[n]) : 0.f;
    }
    if (p.c_vec_ok) {
      // a wavefront stages 64 rows x WCOLS columns at a time
      constexpr int EP_STRIDE = WCOLS + 8;  // halves per staged row: 16-byte aligned rows, conflict-free 16-byte reads
      constexpr int LPR = WCOLS / 8;        // lanes per staged row in the plain store: 8 columns each
      __syncthreads();                      // every wavefront is done with the A tiles
      _Float16* ep = lds + wave * (64 * EP_STRIDE);
      const int erow = lane_e / LPR, ecol = (lane_e % LPR) * 8;
      const int n_out = n0 + wn * WCOLS + ecol;
#pragma unroll
      for (int h = 0; h < RT / 2; ++h) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
          for (int j = 0; j < CT; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              ep[(ii * 32 + (r >> 2) * 8 + kq_e * 4 + (r & 3)) * EP_STRIDE + j * 32 + li_e] =
                  narrow_elem(acc[2 * h + ii][j][r] + bcol[j]);
        // LDS operations of one wavefront complete in issue order: the reads below see the writes above
        if (p.epi_kind == kMnbFusedMlp) {
          // a staged row is gate0 up0 [gate1 up1] (16 columns each) = 16 CT output columns: 2 CT lanes per row, each
          // reads its 8 gate and 8 up values (narrowed to fp16, as the two separate products would be) and writes 8
          // outputs
          constexpr int GL = 2 * CT;  // lanes per staged row
          const int grow = lane_e / GL, q = lane_e % GL;
          const int gcol = (q >> 1) * 32 + (q & 1) * 8;
          const int n_glu = ((n0 + wn * WCOLS) >> 1) + q * 8;
#pragma unroll
          for (int ps = 0; ps < GL; ++ps) {
            const int row = ps * (64 / GL) + grow;
            const h8_t g = *reinterpret_cast<const h8_t*>(ep + row * EP_STRIDE + gcol);
            const h8_t u = *reinterpret_cast<const h8_t*>(ep + row * EP_STRIDE + gcol + 16);
            h8_t y;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float gf = widen_elem(g[e]);
              y[e] = narrow_elem(gf / (1.0f + __expf(-gf)) * widen_elem(u[e]));
            }
            const int m = m0 + wm * 32 * RT + h * 64 + row;
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
          for (int ps = 0; ps < LPR; ++ps) {
            const int row = ps * (64 / LPR) + erow;
            const u4_t v = *reinterpret_cast<const u4_t*>(ep + row * EP_STRIDE + ecol);
            const int m = m0 + wm * 32 * RT + h * 64 + row;
            if (m < p.M && n_loc < n_lim) *reinterpret_cast<u4_t*>(dst + (int64_t)m * ld + n_loc) = v;
          }
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < CT; ++j) {
        const int n = n0 + wn * WCOLS + j * 32 + li_e;
        if (n >= p.N) continue;
#pragma unroll
        for (int i = 0; i < RT; ++i) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * 32 * RT + i * 32 + (r >> 2) * 8 + kq_e * 4 + (r & 3);
            if (m < p.M) p.C[(int64_t)m * p.ldc + n] = narrow_elem(acc[i][j][r] + bcol[j]);
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

template <int BITS, bool HAS_ZP, int MPS, int TM, int WM, int DT, int NWV = 8, int CTW = WM>
hipError_t launch_wm(const Gemm256Params& p, unsigned grid, hipStream_t s) {
  // eight wavefronts: 98304 bytes whatever the tile height (one workgroup per compute unit either way); four: the
  // three staged tiles of the 128-row tile, so that three workgroups share a compute unit
  const size_t smem = NWV == 8 ? (size_t)SMEM_BYTES : (size_t)3 * 64 * TM * ROW_BYTES;
  auto kernel = mnb_gemm256_kernel<BITS, HAS_ZP, MPS, TM, WM, DT, NWV, CTW>;
  // The attribute belongs to the function on the current device, so it is set on every launch (a host-side table
  // update, no device work): callers on several threads or devices need no shared flag.
  if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      e != hipSuccess)
    return e;
  kernel<<<dim3(grid), dim3(64 * NWV), smem, s>>>(p);
  return hipGetLastError();
}

// The 1 x 8 arrangement of the wavefronts is faster on every shape and block size measured (0.84 ... 0.98 of the
// 2 x 4 arrangement's time, bit-identical results): matrix and vector instructions hardly overlap on a SIMD, so the
// halved dequantisation work counts in full.  The 2 x 4 arrangement is compiled into calibration builds only.
template <int BITS, bool HAS_ZP, int MPS, int TM, int DT>
hipError_t launch_tm(const Gemm256Params& p, unsigned grid, hipStream_t s) {
#if defined(MNB_TUNING_HOOKS)
  if (const char* e = mnb_tuning_env("MNB_GEMM256_WAVE_ROWS"); e != nullptr && e[0] == '2')
    return launch_wm<BITS, HAS_ZP, MPS, TM, 2, DT>(p, grid, s);
  if constexpr (TM == 4 && DT == 0 && BITS == 4)
    if (const char* e = mnb_tuning_env("MNB_GEMM256_WAVES"); e != nullptr && e[0] == '4')
      return launch_wm<BITS, HAS_ZP, MPS, TM, 1, DT, 4, 2>(p, grid, s);  // 1 x 4, one wavefront per SIMD
#endif
  return launch_wm<BITS, HAS_ZP, MPS, TM, 1, DT>(p, grid, s);
}

// bfloat16 with four 8-byte meta entries per column and k-step (8-bit weights in blocks of 16 with zero points) does not
// fit the register file at 256 rows: that model runs on 128-row tiles only (mnb_gemm256_plan knows).
template <bool HAS_ZP, int MPS>
constexpr bool kBf16Has256Rows = !(HAS_ZP && MPS == 4);

// 128- or 256-row tiles of element type DT (HAS_256: whether the 256-row member exists); 128 x 128 tiles for fp16 and
// bfloat16 models
template <int BITS, bool HAS_ZP, int MPS, int DT, bool HAS_256 = true>
hipError_t launch_rows(const Gemm256Params& p, unsigned grid, hipStream_t s) {
  if (p.tile_cols == 128) {
#if defined(MNB_TUNING_HOOKS)
    // calibration only: 64 x 128 tiles for 16 < M <= 256 measured no faster than the streaming kernel (one tile per
    // workgroup leaves the k loop latency-bound: 29.5 us on M=64 N=28672 K=4096 against 25.5 us)
    if constexpr (DT == 0) {
      if (p.tile_rows == 64) return launch_wm<BITS, HAS_ZP, MPS, 1, 1, DT, 4>(p, grid, s);
    }
#endif
    if constexpr (DT == 0 || DT == 1)
      return p.tile_rows == 128 ? launch_wm<BITS, HAS_ZP, MPS, 2, 1, DT, 4>(p, grid, s) : hipErrorInvalidValue;
    else
      return hipErrorInvalidValue;
  }
  if (p.tile_rows == 128) return launch_tm<BITS, HAS_ZP, MPS, 2, DT>(p, grid, s);
  if constexpr (HAS_256)
    return launch_tm<BITS, HAS_ZP, MPS, 4, DT>(p, grid, s);
  else
    return hipErrorInvalidValue;
}

template <int BITS, bool HAS_ZP, int MPS>
hipError_t launch(const Gemm256Params& p, unsigned grid, int io, hipStream_t s) {
  if (io == kMnbIoF16Wide) {  // zero points in the activation type exist for 4-bit (and 2-bit, packed as 4-bit) only
    if constexpr (BITS == 4 && HAS_ZP)
      return launch_rows<BITS, HAS_ZP, MPS, 2>(p, grid, s);
    else
      return hipErrorInvalidValue;
  }
  if (io == kMnbIoBf16) return launch_rows<BITS, HAS_ZP, MPS, 1, kBf16Has256Rows<HAS_ZP, MPS>>(p, grid, s);
  return launch_rows<BITS, HAS_ZP, MPS, 0>(p, grid, s);
}

size_t round256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

// How the tile GEMM would run a problem: rows of the tile, the grid, whether tiles are split along K across
// workgroups (only with a workspace), the workspace that takes, and the estimated run time.  The kernel itself takes
// any division of the units into contiguous shares.
// ---- the plan: tile height and split, from a cost model calibrated on the device
// Measured behaviour (all shapes of M = 256 ... 4096, N = 4096 ... 28672, K = 4096 / 8192 / 14336, every tile height
// and number of parts):
//   * a workgroup that has its compute unit to itself on a chip at most half busy runs its k-steps at a fixed pace
//     (step: 2530 cycles for a 256-row 4-bit tile, of which the 64 matrix instructions of a SIMD take 2048 and the
//     vector instructions most of the rest -- the two hardly overlap on a SIMD), after a fixed start-up (start:
//     launch, prologue, epilogue);
//   * the chip is power-limited: with more than half of the compute units busy every workgroup slows down, by
//     load[...] at 3/4, 7/8 and all of them (a full chip does 1.2 times the work of half a chip per second, not 2);
//     kernels that are bound by the vector unit (8-bit weights, 128-row tiles) slow down less;
//   * more workgroups than compute units run as rounds (128-row tiles share a compute unit in pairs, which costs
//     what two rounds cost);
//   * cutting the tiles into `parts` ranges of k costs kFixCycles[0] + parts * kFixCycles[1] for the finishing pass
//     (the lower parts write their sums, the top part waits for them and adds them one after the other).
// Times are in cycles of the device's nominal clock.  Variants: 4-bit; 8-bit; 8-bit with 16-wide blocks.
namespace plan_model {
struct Variant {
  double start[2];    // [0]: 256-row tiles, [1]: 128-row tiles
  double step[2];
  double load[2][3];  // slow-down at 3/4, 7/8 and all compute units busy (1.0 up to half)
  double full[2];     // slow-down of a full round when there are several
};
constexpr Variant kVariants[3] = {
    {{18000, 13440}, {2530, 1478}, {{1.31, 1.465, 1.66}, {1.216, 1.365, 1.535}}, {1.67, 1.57}},
    {{18480, 15120}, {2545, 1582}, {{1.333, 1.48, 1.665}, {1.17, 1.313, 1.476}}, {1.69, 1.544}},
    {{18480, 15120}, {3105, 1905}, {{1.16, 1.30, 1.47}, {1.10, 1.20, 1.35}}, {1.47, 1.37}},
};
constexpr double kFixCycles[2][2] = {{3120, 9600}, {2400, 6720}};  // [tile height][constant, per part]

inline double load_factor(const double (&at)[3], double busy) {  // busy: fraction of the compute units with a workgroup
  if (busy <= 0.5) return 1.0;
  if (busy <= 0.75) return 1.0 + (at[0] - 1.0) * (busy - 0.5) / 0.25;
  if (busy <= 0.875) return at[0] + (at[1] - at[0]) * (busy - 0.75) / 0.125;
  return at[1] + (at[2] - at[1]) * (busy > 1.0 ? 1.0 : (busy - 0.875) / 0.125);
}

// cycles for `grid` workgroups of `steps` k-steps each (the finishing pass of a split does not slow down with load)
inline double cycles(const Variant& v, int h, int64_t grid, int64_t steps, int parts, int64_t cus) {
  const double part = (double)steps * v.step[h];
  const double fix = parts > 1 ? kFixCycles[h][0] + parts * kFixCycles[h][1] : 0.0;
  const int64_t rounds = grid / cus, rest = grid % cus;
  double t = v.start[h];
  if (rounds > 0) t += (double)rounds * (part * (rounds + (rest ? 1 : 0) > 1 ? v.full[h] : v.load[h][2]) + fix);
  if (rest > 0) t += part * load_factor(v.load[h], (double)rest / (double)cus) + fix;
  return t;
}
// 128 x 128 tiles (four wavefronts).  Measured: a workgroup alone on its compute unit (one wavefront per SIMD) needs
// 1100 cycles per k-step (4-bit) and slows down by only 1.19 when every compute unit has one - a single wavefront
// per SIMD does not draw the power two do; k workgroups on a compute unit share its matrix cores, k x 1222 cycles per
// step with the chip full, less when only some compute units hold k.  They pay exactly where the 256-column tiles
// leave half the chip idle and a split along K would need its finishing pass: 5 to 11 % on those shapes.
constexpr double kNarrowStart[3] = {12000, 13000, 13000};
constexpr double kNarrowStepAlone[3] = {1100, 1166, 1289};
constexpr double kNarrowLoad[3] = {1.06, 1.12, 1.19};
constexpr double kNarrowStepShared[3] = {1222, 1282, 1410};
inline double cycles_narrow(int vi, int64_t grid, int64_t steps, int64_t cus) {
  const int64_t k = (grid + cus - 1) / cus;
  double step;
  if (k <= 1)
    step = kNarrowStepAlone[vi] * load_factor(kNarrowLoad, (double)grid / (double)cus);
  else
    step = (double)k * kNarrowStepShared[vi] * (0.5 + 0.5 * (double)grid / (double)(k * cus));
  return kNarrowStart[vi] + (double)steps * step;
}
}  // namespace plan_model

namespace {
// [flags: 8 per workgroup][status word] rounded up to 256 bytes, then one partial tile per workgroup
size_t split_flag_bytes(int64_t grid) { return round256(((size_t)grid * 8 + 1) * sizeof(uint32_t)); }
size_t split_workspace_bytes(int64_t grid, int rows, int cols) {
  return split_flag_bytes(grid) + (size_t)grid * rows * cols * sizeof(float);
}
}  // namespace

MnbGemm256Plan mnb_gemm256_plan(const MnbLayout& L, int64_t M, bool with_workspace, int io) {
  const MnbDeviceInfo& dev = mnb_device_info();
  const int64_t ksteps = L.K / BK, upt = ksteps / 2;
  const int vi = L.bits == 4 ? 0 : (L.bs >= 32 ? 1 : 2);
  const plan_model::Variant& v = plan_model::kVariants[vi];
  const int64_t cus = dev.cus;
  // a matrix packed for an fp32 model is run by the bfloat16 instantiations, whose 8-bit / block 16 / zero-point
  // member has no 256-row form (see kBf16Has256Rows)
  const bool only_128_rows = L.dtype == kMnbDtypeFloat && L.bits == 8 && L.bs < 32 && L.has_zp;
  // 128 x 128 tiles exist for fp16 and bfloat16 models; a matrix packed with fp32 entries may also belong to an fp16
  // model with zero points in the activation type (4-bit with zero points), which has none
  const bool narrow_ok = L.dtype == kMnbDtypeFloat16 || io == kMnbIoBf16;
  auto tiles_of = [&](int rows, int cols) { return ((M + rows - 1) / rows) * ((L.N + cols - 1) / cols); };
  MnbGemm256Plan best{};
  for (int h = 0; h < 3; ++h) {
    const int rows = h == 0 ? 256 : 128, cols = h == 2 ? 128 : 256;
    if ((rows == 256 && only_128_rows) || (h == 2 && !narrow_ok)) continue;
    const int64_t tiles = tiles_of(rows, cols);
    for (int parts = 1; parts <= 8; ++parts) {
      // parts are whole units (two k-steps) of at least 16 k-steps, and never more than two rounds of workgroups:
      // a part waits for the parts below it, which must not sit in a later round than the model assumes
      if (upt % parts != 0 || (parts > 1 && (!with_workspace || ksteps / parts < 16 || tiles * parts > 2 * cus))) continue;
      if (h == 2 && parts > 1) continue;  // narrow tiles are the alternative to a split, not its companion
      MnbGemm256Plan pl{};
      pl.tile_rows = rows;
      pl.tile_cols = cols;
      pl.grid = tiles * parts;
      pl.split = parts > 1;
      pl.seconds = (h == 2 ? plan_model::cycles_narrow(vi, pl.grid, ksteps, cus)
                           : plan_model::cycles(v, h, pl.grid, ksteps / parts, parts, cus)) /
                   dev.clock_hz;
      if (pl.split) pl.workspace_bytes = split_workspace_bytes(pl.grid, rows, cols);
      if (best.grid == 0 || pl.seconds < best.seconds) best = pl;
    }
  }
  if (const char* e = mnb_tuning_env("MNB_GEMM256_PLAN")) {  // calibration: "<tile rows>,<parts>[,<tile columns>]"
    int rows = 0, parts = 0, cols = 256;
    const int got = sscanf(e, "%d,%d,%d", &rows, &parts, &cols);
    if (got >= 2 && (rows == 128 || (rows == 256 && !only_128_rows) || (rows == 64 && cols == 128 && io == kMnbIoModel)) &&
        parts >= 1 && parts <= 8 && upt % parts == 0 && (parts == 1 || with_workspace) &&
        (cols == 256 || (cols == 128 && rows <= 128 && narrow_ok))) {
      best = MnbGemm256Plan{};
      best.tile_rows = rows;
      best.tile_cols = cols;
      best.grid = tiles_of(rows, cols) * parts;
      best.split = parts > 1;
      best.workspace_bytes = parts > 1 ? split_workspace_bytes(best.grid, rows, cols) : 0;
    }
  }
  return best;
}

// Per-lane offsets of the tile GEMM are 32-bit byte counts from a base that moves with the tile: activations span
// 255 rows of lda halves plus one k-step (mnb_gemm256_max_lane_offset), weights one k-group row of Npad columns x 16
// bytes, meta entries two block rows of Npad x 4 bytes.  Problems beyond that take the streaming kernel, whose
// addressing is 64-bit throughout.
uint64_t mnb_gemm256_max_lane_offset(int64_t lda) { return ((uint64_t)255 * (uint64_t)lda + 7 * 8 + 7) * 2 + 1; }

bool mnb_gemm256_addressable(int64_t lda, int64_t Npad) {
  return mnb_gemm256_max_lane_offset(lda) < ((uint64_t)1 << 32) - 1 && (uint64_t)Npad * 16 + 16 <= ((uint64_t)1 << 32);
}

// The fused outputs are written with 16-byte stores of 8 columns: every output 16-byte aligned, with a pitch and a
// width that are multiples of 8 elements.
bool mnb_gemm256_fused_ok(const MnbEpilogue& e) {
  const int nout = e.kind == kMnbFusedQkv ? 3 : 1;
  for (int i = 0; i < nout; ++i)
    if (reinterpret_cast<uintptr_t>(e.out[i]) % 16 != 0 || e.ld[i] % 8 != 0 || e.n[i] % 8 != 0) return false;
  return true;
}

#if defined(MNB_TEST_HOOKS)
// Test builds (tests/hooks): the host chooses the bound of the cross-workgroup wait and may leave the lower parts of
// odd-numbered tiles uncomputed, so that the give-up path runs with every kernel still ending normally.
static int g_test_spin_limit = 0;
static int g_test_drop_odd_lower = 0;
extern "C" __attribute__((visibility("default"))) void MnbTestSetSplitHooks(int spin_limit, int drop_odd_lower) {
  g_test_spin_limit = spin_limit;
  g_test_drop_odd_lower = drop_odd_lower;
}
#endif

// Device address of the status word of a split launch's workspace (NULL when this problem's plan does not split or
// the workspace is too small for it): 1 after a launch in which a cross-workgroup wait gave up.
const uint32_t* mnb_gemm256_status_word(const MnbLayout& L, int64_t M, int io, const void* workspace,
                                        size_t workspace_bytes) {
  const MnbGemm256Plan plan = mnb_gemm256_plan(L, M, true, io);
  if (!plan.split || workspace == nullptr || workspace_bytes < plan.workspace_bytes ||
      reinterpret_cast<uintptr_t>(workspace) % 8 != 0)
    return nullptr;
  return reinterpret_cast<const uint32_t*>(workspace) + plan.grid * 8;
}

hipError_t mnb_launch_gemm256(const MnbGemmArgs& a, hipStream_t s) {
  if (!mnb_gemm256_addressable(a.lda, a.L.Npad)) return hipErrorInvalidValue;  // the dispatcher never sends these
  // a matrix packed for an fp32 model is run in a 16-bit type named by a.io; fused outputs exist for fp16 models only
  if ((a.io != kMnbIoModel) != (a.L.dtype == kMnbDtypeFloat) || (a.io != kMnbIoModel && a.epi.kind != kMnbFusedNone))
    return hipErrorInvalidValue;
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
  const MnbGemm256Plan plan_ws = mnb_gemm256_plan(a.L, a.M, true, a.io);
  const bool ws_ok = plan_ws.split && a.workspace != nullptr && a.workspace_bytes >= plan_ws.workspace_bytes &&
                     reinterpret_cast<uintptr_t>(a.workspace) % 8 == 0;
  const MnbGemm256Plan plan = ws_ok ? plan_ws : mnb_gemm256_plan(a.L, a.M, false, a.io);
  p.tile_rows = plan.tile_rows;
  p.tile_cols = plan.tile_cols;
  p.tiles_m = (int)((a.M + p.tile_rows - 1) / p.tile_rows);
  p.tiles_n = (int)((a.L.N + p.tile_cols - 1) / p.tile_cols);
  p.upt = p.ksteps / 2;
  const int64_t units = (int64_t)p.tiles_m * p.tiles_n * p.upt;
  if ((int64_t)p.tiles_m * p.tiles_n > 0x7fffffff) return hipErrorInvalidValue;
  p.share_q = units / plan.grid;
  p.share_r = units % plan.grid;
  p.spin_limit = 1 << 20;  // polls half a microsecond apart: seconds, where a healthy wait takes microseconds
#if defined(MNB_TEST_HOOKS)
  if (g_test_spin_limit > 0) p.spin_limit = g_test_spin_limit;
  p.test_drop_odd_lower = g_test_drop_odd_lower;
#endif
  if (plan.split) {
    p.flags = reinterpret_cast<uint32_t*>(a.workspace);
    p.status = p.flags + plan.grid * 8;
    p.partials = reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(a.workspace) + split_flag_bytes(plan.grid));
    mnb_gemm256_clear_flags_kernel<<<dim3(1), dim3(256), 0, s>>>(p.flags, (int)plan.grid * 8 + 1);
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
  if (a.L.bits == 4) return a.L.has_zp ? launch<4, true, 2>(p, grid, a.io, s) : launch<4, false, 2>(p, grid, a.io, s);
  // 8-bit: two entries per k-step (also for blocks of 64 and more, where both name the same block); blocks of 16 need four
  if (a.L.bs >= 32) return a.L.has_zp ? launch<8, true, 2>(p, grid, a.io, s) : launch<8, false, 2>(p, grid, a.io, s);
  return a.L.has_zp ? launch<8, true, 4>(p, grid, a.io, s) : launch<8, false, 4>(p, grid, a.io, s);
}
