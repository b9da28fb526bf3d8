// fp16 kernel for 16 < M <= a few hundred rows: the regime between decode and prefill, where the reference runs its
// strip-wise dequantise + SGEMM loop (SQ4BitGemm_CompFp32, onnxruntime/core/mlas/lib/qnbitgemm.cpp:563-732) and the
// work is still dominated by streaming the weights once.
//
// Same structure as the decode kernel (mnb_skinny.hip): a workgroup owns 16*T output columns and a block of 16*MT rows,
// K is split over its wavefronts (reduced through LDS at the end, fixed order), and every lane feeds its own 16-byte
// weight vector to v_mfma_f32_16x16x32_f16 as the B operand -- no LDS on the weight path.  The difference is that each
// dequantised operand is used by MT row tiles, so the weights are dequantised exactly ((q - zp) * scale in fp16, the
// reference's fp16 dequantisation bit for bit) and the matrix cores accumulate across blocks; the VALU cost of the
// dequantisation is amortised over MT * 4 matrix instructions per word.
//
// 16-bit models on a matrix packed with fp32 meta entries (IO = kMnbIoBf16, kMnbIoF16Wide: bfloat16, and fp16 with zero
// points in the activation type) run the same kernel: the weights are dequantised in fp32, fma(float(q), scale,
// -zp * scale), narrowed to the activation type, and multiplied by the matrix instruction of that type.
//
// The A operand of lane (j, kq) is 16 bytes of row j at a 64-byte stride between lanes -- read from the row-major
// activations, one load instruction would touch 64 cache lines.  A small staging kernel therefore first rewrites A
// into operand order in the caller's workspace, [chunk][word i][row tile][kq][j] in 16-byte units (zero-filled beyond
// M and K, any alignment of the source), so that every operand load of a wavefront is 1 KiB contiguous.  The staged
// copy is M x K halves (at most a few MB) and is re-read from L2 by every workgroup.
#include <atomic>

#include "mnb_mfma16_common.hip.h"

namespace {

struct MidParams {
  SkinnyParams s;
  const uint4* As;  // staged activations
  int row_tiles;    // 16-row tiles in the staged copy (multiple of the kernel's MT)
};

// A (row-major, lda) -> operand order.  One thread per 16-byte unit.
template <int BITS>
__global__ void __launch_bounds__(256) mnb_mid_stage_a_kernel(const _Float16* __restrict__ A, int64_t lda, int M, int K,
                                                              int chunks, int row_tiles, int vec_ok,
                                                              uint4* __restrict__ As) {
  constexpr int GK = 128 / BITS, NI = GK / 8, CK = 4 * GK;
  const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)chunks * NI * row_tiles * 64;
  if (u >= total) return;
  const int j = (int)(u & 15), kq = (int)((u >> 4) & 3);
  const int64_t v = u >> 6;
  const int rt = (int)(v % row_tiles);
  const int i = (int)((v / row_tiles) % NI);
  const int c = (int)(v / ((int64_t)row_tiles * NI));
  const int row = rt * 16 + j;
  const int k0 = c * CK + kq * GK + 8 * i;
  uint4 out = make_uint4(0u, 0u, 0u, 0u);
  if (row < M && k0 < K) {
    const _Float16* src = A + (int64_t)row * lda + k0;
    if (vec_ok && k0 + 8 <= K) {
      out = *reinterpret_cast<const uint4*>(src);
    } else {
      __align__(16) _Float16 tmp[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) tmp[e] = (k0 + e < K) ? src[e] : (_Float16)0.0f;
      out = *reinterpret_cast<const uint4*>(tmp);
    }
  }
  As[u] = out;
}

// exact (q - zp) * scale for the 8 weights of one 4-bit word / the 8 weights of two 8-bit words
template <int BITS>
__device__ __forceinline__ h8_t dequant_word(uint32_t w0, uint32_t w1, const UnpackConsts& uc, h2_t z_lo, h2_t z_hi,
                                             h2_t s2) {
  uint4 r;
  if constexpr (BITS == 4) {
    const uint32_t w8 = w0 >> 8;
    const h2_t p0 = mnb_as_h2((w0 & uc.mask_lo) | uc.magic_lo);  // 1024 + q
    const h2_t p1 = mnb_as_h2((w0 & uc.mask_hi) | uc.magic_hi);  //   64 + q
    const h2_t p2 = mnb_as_h2((w8 & uc.mask_lo) | uc.magic_lo);
    const h2_t p3 = mnb_as_h2((w8 & uc.mask_hi) | uc.magic_hi);
    r.x = mnb_as_u32((p0 + z_lo) * s2);
    r.y = mnb_as_u32((p1 + z_hi) * s2);
    r.z = mnb_as_u32((p2 + z_lo) * s2);
    r.w = mnb_as_u32((p3 + z_hi) * s2);
  } else {
    const h2_t p0 = mnb_as_h2(__builtin_amdgcn_perm(kMagic, w0, 0x07010700u));
    const h2_t p1 = mnb_as_h2(__builtin_amdgcn_perm(kMagic, w0, 0x07030702u));
    const h2_t p2 = mnb_as_h2(__builtin_amdgcn_perm(kMagic, w1, 0x07010700u));
    const h2_t p3 = mnb_as_h2(__builtin_amdgcn_perm(kMagic, w1, 0x07030702u));
    r.x = mnb_as_u32((p0 + z_lo) * s2);
    r.y = mnb_as_u32((p1 + z_lo) * s2);
    r.z = mnb_as_u32((p2 + z_lo) * s2);
    r.w = mnb_as_u32((p3 + z_lo) * s2);
  }
  return __builtin_bit_cast(h8_t, r);
}

// One chunk: word step i of every column tile against the MT row tiles, then -- the A operands of step i being dead --
// their reload for the wavefront's next chunk (a_next, when NEXT_A).  The activations are thus prefetched
// three quarters of a chunk ahead without a second register set.  NEXT_A is a compile-time flag on purpose: a load
// under a run-time condition makes the number of outstanding loads unknown to the compiler at the join, and every
// later wait then degenerates to "wait for all loads", the weight prefetch issued just before included.
template <int BITS, bool HAS_ZP, int T, int MT, bool NEXT_A, int IO>
__device__ __forceinline__ void mid_compute_chunk(const ChunkRegs<BITS, T>& R, h8_t (*af)[(128 / BITS) / 8],
                                                  const uint4* a_next, int64_t a_step, const UnpackConsts& uc,
                                                  f4_t (*y)[T]) {
  constexpr int NI = (128 / BITS) / 8;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const bool second = (BITS == 4) && i >= 2;  // words 2, 3 of a 4-bit vector may belong to the next block
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const uint32_t wd[4] = {R.w[t].x, R.w[t].y, R.w[t].z, R.w[t].w};
      h8_t b;
      if constexpr (IO != kMnbIoModel) {
        const float sc = __uint_as_float(second ? R.m1[t] : R.m0[t]);
        const float zp = HAS_ZP ? __uint_as_float(second ? R.z1[t] : R.z0[t]) : (float)(1 << (BITS - 1));
        b = BITS == 4 ? dequant_word_wide<BITS, IO == kMnbIoBf16>(wd[i], 0u, sc, -zp * sc)
                      : dequant_word_wide<BITS, IO == kMnbIoBf16>(wd[(2 * i) & 3], wd[(2 * i + 1) & 3], sc, -zp * sc);
      } else {
        _Float16 sc, nz;
        decode_meta<BITS, HAS_ZP>(second ? R.m1[t] : R.m0[t], sc, nz);
        const h2_t s2 = mnb_h2(sc);
        const h2_t z_lo = mnb_h2(nz);                     // -(1024 + zp)
        const h2_t z_hi = mnb_h2(nz + (_Float16)960.0f);  // -(64 + zp), exact
        b = BITS == 4 ? dequant_word<4>(wd[i], 0u, uc, z_lo, z_hi, s2)
                      : dequant_word<8>(wd[(2 * i) & 3], wd[(2 * i + 1) & 3], uc, z_lo, z_hi, s2);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (IO == kMnbIoBf16)
          y[mt][t] = mfma16_bf16(af[mt][i], b, y[mt][t]);
        else
          y[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[mt][i], b, y[mt][t], 0, 0, 0);
      }
    }
    // Nothing moves across the end of a word step: loads hoisted above the matrix instructions that still read
    // af[.][i] would need a second register set, and so would dequantised operands prepared steps ahead.
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NEXT_A) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt][i] = __builtin_bit_cast(h8_t, a_next[i * a_step + mt * 64]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// What a wavefront needs to issue its first loads comes as leading scalar kernel arguments, which the build asks the
// compiler to have preloaded into SGPRs at wavefront start; the parameter block carries the rest.
// DIRECT: the activations are read from the caller's row-major A (16-byte aligned rows, K a whole number of chunks) and
// brought into operand order inside the kernel, so the staging pass and its launch drop out: a wavefront reads its
// chunk of a 16-row tile row-contiguously (64 lanes x 16 bytes = 4 rows x 256 bytes with 4-bit weights: 8 cache lines
// per instruction), passes it through a private 4 KiB of LDS and picks its operands up from there, tile after tile (LDS
// executes a wavefront's accesses in order: no barrier).  The loads of the next chunk are issued before the current one
// is computed and wait in registers (MT x NI vectors).
template <int BITS, bool HAS_ZP, int T, int MT, int NW, int IO, bool DIRECT>
__global__ void __launch_bounds__(NW * 64) mnb_mid_kernel(const uint4* hot_W, int64_t hot_Npad, const uint4* hot_As,
                                                          const uint8_t* hot_meta, int hot_row_tiles, int hot_chunks,
                                                          int hot_bs_shift, MidParams rest) {
  MidParams mp = rest;
  mp.s.W = hot_W;
  mp.s.Npad = hot_Npad;
  mp.As = hot_As;
  mp.s.meta = hot_meta;
  mp.row_tiles = hot_row_tiles;
  mp.s.chunks = hot_chunks;
  mp.s.bs_shift = hot_bs_shift;
  const SkinnyParams& p = mp.s;
  constexpr int GK = 128 / BITS;
  constexpr int NI = GK / 8;
  constexpr int LOAD_MODE = IO == kMnbIoModel ? 1 : 2;  // which meta entries a chunk's loads fetch (load_chunk)
  extern __shared__ __align__(16) unsigned char smem[];
  float* red = reinterpret_cast<float*>(smem);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, kq = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * (16 * T);
  const int64_t col0 = n0 + j;
  const int m0 = blockIdx.y * (16 * MT);

  // staged A: unit index = (((c * NI + i) * row_tiles + rt) * 4 + kq) * 16 + j
  const uint4* a_lane = mp.As + ((int64_t)blockIdx.y * MT * 4 + kq) * 16 + j;
  const int64_t a_step = (int64_t)mp.row_tiles * 64;  // units between consecutive (c, i)
  f4_t y[MT][T];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < T; ++t) y[mt][t] = f4_t{0.f, 0.f, 0.f, 0.f};
  const UnpackConsts uc = make_unpack_consts();

  h8_t af[MT][NI];
  auto load_a = [&](int c) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < NI; ++i)
        af[mt][i] = __builtin_bit_cast(h8_t, a_lane[((int64_t)c * NI + i) * a_step + mt * 64]);
  };
  // DIRECT: 16-byte pieces of a chunk's row: PIECES; rows one load instruction covers: RPI (16 / RPI == NI instructions
  // per 16-row tile).  Pieces are XOR-swizzled with the row so that neither the row-contiguous writes nor the operand
  // reads conflict on LDS banks.
  constexpr int PIECES = 4 * NI, RPI = 64 / PIECES;
  const int piece = lane % PIECES, r0 = lane / PIECES;
  auto swz = [](int row) { return PIECES == 16 ? row : (row >> 1); };
  h8_t* const mine = reinterpret_cast<h8_t*>(smem + (size_t)NW * T * 4 * 64 * sizeof(float)) + wave * (16 * PIECES);
  h8_t g[MT][NI];  // the next chunk's activations on their way (DIRECT)
  auto fetch_a = [&](int c) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int I = 0; I < NI; ++I) {
        int row = m0 + mt * 16 + I * RPI + r0;
        row = row < p.M ? row : p.M - 1;  // rows beyond M re-read the last row and are never stored
        g[mt][I] = *reinterpret_cast<const h8_t*>(p.A + (int64_t)row * p.lda + (int64_t)c * 4 * GK + piece * 8);
      }
  };
  auto pass_a = [&]() {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int I = 0; I < NI; ++I) {
        const int row = I * RPI + r0;
        mine[row * PIECES + (piece ^ swz(row))] = g[mt][I];
      }
#pragma unroll
      for (int i = 0; i < NI; ++i) af[mt][i] = mine[j * PIECES + ((kq * NI + i) ^ swz(j))];
    }
  };

  // Weights two chunks ahead (double buffer), activations reloaded word step by word step inside the chunk.  No load
  // of the loop sits under a condition, so every wait counts exactly the loads it needs and leaves the younger
  // prefetches in flight; a prefetch beyond the wavefront's last chunk is clamped to the last chunk of the matrix
  // instead of skipped (valid memory that another wavefront of the workgroup is reading anyway, never used here).
  auto a_of = [&](int c) -> const uint4* { return a_lane + (int64_t)c * NI * a_step; };
  ChunkRegs<BITS, T> R0, R1;
  const int last = p.chunks - 1;
  int c = wave;
  if constexpr (DIRECT) {
    // weights two chunks ahead, activations one: fetched into g before a chunk is computed, passed through LDS after
    load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c, last), kq, col0, R0);
    fetch_a(min(c, last));
    load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c + NW, last), kq, col0, R1);
    pass_a();
    __builtin_amdgcn_sched_barrier(0);
    for (; c + NW < p.chunks; c += 2 * NW) {
      fetch_a(c + NW);
      __builtin_amdgcn_sched_barrier(0);
      mid_compute_chunk<BITS, HAS_ZP, T, MT, false, IO>(R0, af, nullptr, a_step, uc, y);
      load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c + 2 * NW, last), kq, col0, R0);
      __builtin_amdgcn_sched_barrier(0);
      pass_a();
      fetch_a(min(c + 2 * NW, last));
      __builtin_amdgcn_sched_barrier(0);
      mid_compute_chunk<BITS, HAS_ZP, T, MT, false, IO>(R1, af, nullptr, a_step, uc, y);
      load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c + 3 * NW, last), kq, col0, R1);
      __builtin_amdgcn_sched_barrier(0);
      pass_a();
    }
    if (c < p.chunks) mid_compute_chunk<BITS, HAS_ZP, T, MT, false, IO>(R0, af, nullptr, a_step, uc, y);
  } else {
    load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c, last), kq, col0, R0);
    load_a(min(c, last));
    load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c + NW, last), kq, col0, R1);
    __builtin_amdgcn_sched_barrier(0);
    for (; c + NW < p.chunks; c += 2 * NW) {
      mid_compute_chunk<BITS, HAS_ZP, T, MT, true, IO>(R0, af, a_of(c + NW), a_step, uc, y);
      load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c + 2 * NW, last), kq, col0, R0);
      __builtin_amdgcn_sched_barrier(0);
      mid_compute_chunk<BITS, HAS_ZP, T, MT, true, IO>(R1, af, a_of(min(c + 2 * NW, last)), a_step, uc, y);
      load_chunk<BITS, HAS_ZP, LOAD_MODE, T>(p, min(c + 3 * NW, last), kq, col0, R1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (c < p.chunks) mid_compute_chunk<BITS, HAS_ZP, T, MT, false, IO>(R0, af, nullptr, a_step, uc, y);
  }

  // reduce over the wavefronts, one row tile at a time: lane (j, kq), register r of y[mt][t] holds
  // row m0 + 16 mt + 4 kq + r, column n0 + 16 t + j
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (mt > 0) __syncthreads();
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[(wave * T * 4 + t * 4 + r) * 64 + lane] = y[mt][t][r];
    __syncthreads();
    reduce_and_store_tiles<T, NW>(p, red, m0 + mt * 16, n0);
  }
}

// ---- activations shared through LDS ---------------------------------------------------------------------------------
// The kernel above re-reads the activations once per 16 T columns: every workgroup walks all of K, and its wavefronts,
// which split K between them, share nothing.  For wide matrices that stream is several times the weights' (64 rows,
// K = 4096, N = 28672, 64 columns per workgroup: 448 x 512 KB = 229 MB against 59 MB of weights) and it is the level-2
// caches, busy 70 % of the launch, that set the pace.  Here a workgroup's eight wavefronts form KGS = 4 teams of NG = 2:
// the teams split K as before, the two wavefronts of a team own neighbouring slabs of 16 T columns and walk the same
// chunks, and the chunk's activations (16 MT rows x 256 bytes) are fetched ONCE per team, from the caller's row-major A
// straight into LDS (buffer_load ... lds, 16-byte pieces XOR-swizzled with the row so that neither the row-contiguous
// fills nor the operand reads conflict on banks), one round ahead of the arithmetic, into one of two buffers.  Per
// round: wait for the own fills of this round, barrier, start the fills of the next round, pick the operands up from
// LDS, compute, reload the weight registers for the round after next.  No staged copy of A, no staging launch.
// Needs K a whole number of chunks and 16-byte aligned rows of A; everything else takes the kernel above.
// Anatomy of a round (64 rows, N = 28672, K = 4096, 4-bit, time stamps of the shader clock in a calibration build):
// the older wavefront of a SIMD needs 2800 cycles for its arithmetic (64 matrix instructions, 1024 cycles of the matrix
// pipe, and 320 vector instructions, 1280 issue cycles), the younger one, which gets the issue slots the older
// leaves, 4250; then both wait about 1300 cycles for the fills they issued when the round began -- every workgroup
// fills at the same moment, 22 MB per round chip-wide through level-2 caches that deliver about 11 TB/s, 2 us, against
// 1.8 us of arithmetic.  A third buffer (fills two rounds ahead) does not fit the 160 KB of LDS, and would not lift
// the bandwidth bound; the ablations agree: without the arithmetic the launch takes 16.0 us, without fills, operand
// reads and arithmetic 10.9 us (the weights alone), all together 29.7 us.
// Tried on top and not kept: dequantising the next operand between the matrix instructions of the current one (a
// software pipeline inside mid_compute_chunk, also with the order forced by scheduling groups) -- bit-identical
// results and the same times (+-1 %) on eight shapes of both kernels; cutting K into parts across workgroups for
// matrices too narrow to fill the chip (fp32 partial tiles, an arrival counter per tile, the last workgroup to arrive
// adds the parts in part order) -- correct, and slower than the kernel above on every narrow shape (N = 4096,
// K = 14336, 64 rows: 27.5 against 19.7 us; K = 4096: 18.6 against 7.9 us), because a round costs 2.0 to 2.3 us
// whatever the grid (the same with 32 workgroups as with 224) on top of about 8 us per launch.
template <int BITS, bool HAS_ZP, int T, int MT, int KGS, int NG>
__global__ void __launch_bounds__(KGS * NG * 64) mnb_mid_shared_kernel(const uint4* hot_W, int64_t hot_Npad,
                                                                        const _Float16* hot_A, const uint8_t* hot_meta,
                                                                        int64_t hot_lda, int hot_chunks,
                                                                        int hot_bs_shift, MidParams rest) {
  MidParams mp = rest;
  mp.s.W = hot_W;
  mp.s.Npad = hot_Npad;
  mp.s.A = hot_A;
  mp.s.meta = hot_meta;
  mp.s.lda = hot_lda;
  mp.s.chunks = hot_chunks;
  mp.s.bs_shift = hot_bs_shift;
  const SkinnyParams& p = mp.s;
  constexpr int NW = KGS * NG;
  constexpr int GK = 128 / BITS, NI = GK / 8, CK = 4 * GK;
  constexpr int PIECES = 4 * NI;                   // 16-byte pieces per row of a chunk
  constexpr int ROWS = 16 * MT;                    // rows of A a workgroup works on
  constexpr int CHUNK_BYTES = ROWS * PIECES * 16;  // one team's activations of one chunk
  constexpr int RPI = 64 / PIECES;                 // rows one fill instruction covers
  constexpr int A_PER_WAVE = ROWS / RPI / NG;      // fill instructions per wavefront and round
  constexpr int W_LOADS = T + (BITS == 4 ? 2 : 1); // vector-memory instructions of load_chunk (MODE 1)
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kg = wave / NG, ng = wave % NG;
  const int j = lane & 15, kq = lane >> 4;
  const int64_t n0 = ((int64_t)blockIdx.x * NG + ng) * (16 * T);
  const int64_t col0 = n0 + j;
  const int m0 = blockIdx.y * ROWS;
  auto swz = [](int row) { return PIECES == 16 ? (row & 15) : ((row >> 1) & 7); };

  // this wavefront's share of a round's fills: instruction q covers rows q * RPI + lane / PIECES
  uint32_t a_off[A_PER_WAVE];
#pragma unroll
  for (int u = 0; u < A_PER_WAVE; ++u) {
    const int row = (ng * A_PER_WAVE + u) * RPI + lane / PIECES;
    const int piece = (lane % PIECES) ^ swz(row);
    const int grow = m0 + row < p.M ? m0 + row : p.M - 1;  // rows beyond M re-read the last row and are never stored
    a_off[u] = (uint32_t)(((int64_t)grow * p.lda + piece * 8) * 2);
  }
  unsigned char* const team = smem + kg * CHUNK_BYTES;  // buffer b of the team: team + b * KGS * CHUNK_BYTES
  auto fill = [&](int c, int b) {
    const rsrc_t r = mnb_rsrc(p.A + (int64_t)c * CK);
#pragma unroll
    for (int u = 0; u < A_PER_WAVE; ++u)
      mnb_buffer_load_lds_b128(r, a_off[u],
                               (lds_ptr_t)(team + b * (KGS * CHUNK_BYTES) + (ng * A_PER_WAVE + u) * RPI * PIECES * 16));
  };
  f4_t y[MT][T];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < T; ++t) y[mt][t] = f4_t{0.f, 0.f, 0.f, 0.f};
  const UnpackConsts uc = make_unpack_consts();
  h8_t af[MT][NI];
  auto pick = [&](int b) {
    const unsigned char* buf = team + b * (KGS * CHUNK_BYTES);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int row = mt * 16 + j;
        af[mt][i] = *reinterpret_cast<const h8_t*>(buf + (row * PIECES + ((kq * NI + i) ^ swz(row))) * 16);
      }
  };

  const int last = p.chunks - 1;
  const int rounds = (p.chunks + KGS - 1) / KGS;
  auto chunk_of = [&](int r) { return r * KGS + kg; };
  ChunkRegs<BITS, T> R0, R1;
  // One round.  On entry the fills of round r (issued a round earlier) are followed in issue order by exactly one
  // set of weight loads, so "at most W_LOADS outstanding" means they have landed; the barrier makes that true of the
  // team-mate's share, and tells everybody that the other buffer's readers are done with it.
  auto round = [&](int r, ChunkRegs<BITS, T>& R, int b) {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(W_LOADS));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    fill(min(chunk_of(r + 1), last), b ^ 1);
    __builtin_amdgcn_sched_barrier(0);
    pick(b);
    if (chunk_of(r) < p.chunks) mid_compute_chunk<BITS, HAS_ZP, T, MT, false, kMnbIoModel>(R, af, nullptr, 0, uc, y);
    __builtin_amdgcn_sched_barrier(0);
    load_chunk<BITS, HAS_ZP, 1, T>(p, min(chunk_of(r + 2), last), kq, col0, R);
    __builtin_amdgcn_sched_barrier(0);
  };
  load_chunk<BITS, HAS_ZP, 1, T>(p, min(chunk_of(0), last), kq, col0, R0);
  __builtin_amdgcn_sched_barrier(0);
  fill(min(chunk_of(0), last), 0);
  __builtin_amdgcn_sched_barrier(0);
  load_chunk<BITS, HAS_ZP, 1, T>(p, min(chunk_of(1), last), kq, col0, R1);
  for (int r = 0; r < rounds; r += 2) {
    round(r, R0, 0);
    round(r + 1, R1, 1);  // (past the end: loads of valid memory, a barrier everybody reaches, no arithmetic)
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lds0(0));  // the last prefetches write LDS the reduction is about to reuse
  __syncthreads();

  // reduce over the teams, one row tile at a time; the KGS wavefronts that share a slab do its sums
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (mt > 0) __syncthreads();
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[((ng * KGS + kg) * T * 4 + t * 4 + r) * 64 + lane] = y[mt][t][r];
    __syncthreads();
    reduce_and_store_tiles<T, KGS>(p, red + ng * KGS * T * 4 * 64, m0 + mt * 16, n0, kg * 64 + lane, KGS * 64);
  }
}

struct MidPlan {
  int t, mt, nw;
};

MidPlan mid_plan(const MnbLayout& L, int64_t M, int min_t = 1) {
  MidPlan pl;
  const int CK = 4 * L.group_k;
  const int chunks = (int)((L.K + CK - 1) / CK);
  const int64_t tiles = (L.N + 15) / 16;
  // A workgroup's tile of 16 T columns x 16 MT rows decides how often a dequantised weight (MT) and a loaded
  // activation operand (T) are reused; the grid has to give every CU a workgroup first.  Among the shapes that
  // reach 192 workgroups the largest tile wins, at equal area the wider one (measured: the activations are the
  // larger stream); if none does, the shape with the most workgroups.
  int64_t best_wgs = -1;
  int best_area = 0;
  pl.t = min_t;
  pl.mt = 2;
  for (int t = 4; t >= min_t; t >>= 1) {
    for (int mt = M <= 32 ? 2 : 4; mt >= 2; mt >>= 1) {
      const int64_t wgs = ((tiles + t - 1) / t) * ((M + 16 * mt - 1) / (16 * mt));
      const int area = t * mt;
      const bool full = wgs >= 192, best_full = best_wgs >= 192;
      const bool better = best_wgs < 0 || (full && !best_full) || (full && best_full && area > best_area) ||
                          (!full && !best_full && (wgs > best_wgs || (wgs == best_wgs && area > best_area)));
      if (better) {
        best_wgs = wgs;
        best_area = area;
        pl.t = t;
        pl.mt = mt;
      }
    }
  }
  // eight wavefronts split K further and hide more latency in a single round of workgroups; with several rounds of
  // the largest tile, two workgroups of four wavefronts share a CU instead
  pl.nw = chunks < 16 || (best_area == 16 && best_wgs >= 384) ? 4 : 8;
  if (const char* e = mnb_tuning_env("MNB_MID_PLAN")) {  // calibration builds: "<T>,<MT>,<NW>"
    int t = 0, mt = 0, nw = 0;
    if (sscanf(e, "%d,%d,%d", &t, &mt, &nw) == 3 && (t == 1 || t == 2 || t == 4) && (mt == 2 || mt == 4) &&
        (nw == 4 || nw == 8)) {
      pl.t = t;
      pl.mt = mt;
      pl.nw = nw;
    }
  }
  if (pl.t < min_t) pl.t = min_t;  // gate/up pairs live in one workgroup
  return pl;
}

// whether the direct form of an instantiation exists: the widest tiles have no registers left for the activations in
// flight
template <int BITS, int T, int MT>
constexpr bool kMidHasDirect = !(MT == 4 && T == 4);

template <int BITS, bool HAS_ZP, int T, int MT, int IO>
hipError_t launch_nw(const MidParams& mp, const MidPlan& pl, bool direct, hipStream_t s) {
  const SkinnyParams& p = mp.s;
  dim3 grid((unsigned)((p.N + 16 * T - 1) / (16 * T)), (unsigned)((p.M + 16 * MT - 1) / (16 * MT)));
  const size_t red = (size_t)pl.nw * T * 4 * 64 * sizeof(float);
  if constexpr (kMidHasDirect<BITS, T, MT>) {
    if (direct) {
      const size_t smem = red + (size_t)pl.nw * 16 * (128 / BITS / 2) * 16;  // + 16 rows of one chunk per wavefront
      if (pl.nw == 8)
        mnb_mid_kernel<BITS, HAS_ZP, T, MT, 8, IO, true><<<grid, dim3(512), smem, s>>>(
            p.W, p.Npad, mp.As, p.meta, mp.row_tiles, p.chunks, p.bs_shift, mp);
      else
        mnb_mid_kernel<BITS, HAS_ZP, T, MT, 4, IO, true><<<grid, dim3(256), smem, s>>>(
            p.W, p.Npad, mp.As, p.meta, mp.row_tiles, p.chunks, p.bs_shift, mp);
      return hipGetLastError();
    }
  }
  if (pl.nw == 8)
    mnb_mid_kernel<BITS, HAS_ZP, T, MT, 8, IO, false><<<grid, dim3(512), red, s>>>(p.W, p.Npad, mp.As, p.meta, mp.row_tiles,
                                                                               p.chunks, p.bs_shift, mp);
  else
    mnb_mid_kernel<BITS, HAS_ZP, T, MT, 4, IO, false><<<grid, dim3(256), red, s>>>(p.W, p.Npad, mp.As, p.meta, mp.row_tiles,
                                                                               p.chunks, p.bs_shift, mp);
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP, int T, int IO>
hipError_t launch_mt(const MidParams& p, const MidPlan& pl, bool direct, hipStream_t s) {
  return pl.mt == 2 ? launch_nw<BITS, HAS_ZP, T, 2, IO>(p, pl, direct, s) : launch_nw<BITS, HAS_ZP, T, 4, IO>(p, pl, direct, s);
}

template <int BITS, bool HAS_ZP, int IO>
hipError_t launch_t(const MidParams& p, const MidPlan& pl, bool direct, hipStream_t s) {
  switch (pl.t) {
    case 4: return launch_mt<BITS, HAS_ZP, 4, IO>(p, pl, direct, s);
    case 2: return launch_mt<BITS, HAS_ZP, 2, IO>(p, pl, direct, s);
    default: return launch_mt<BITS, HAS_ZP, 1, IO>(p, pl, direct, s);
  }
}

template <int BITS, bool HAS_ZP>
hipError_t launch_io(const MidParams& p, const MidPlan& pl, int io, bool direct, hipStream_t s) {
  if (io == kMnbIoBf16) return launch_t<BITS, HAS_ZP, kMnbIoBf16>(p, pl, direct, s);
  if (io == kMnbIoF16Wide) {  // zero points in the activation type: 4-bit with zero points
    if constexpr (BITS == 4 && HAS_ZP) return launch_t<BITS, HAS_ZP, kMnbIoF16Wide>(p, pl, direct, s);
    else return hipErrorInvalidValue;
  }
  return launch_t<BITS, HAS_ZP, kMnbIoModel>(p, pl, direct, s);
}

int mid_row_tiles(int64_t M, int mt) { return (int)((M + 16 * mt - 1) / (16 * mt)) * mt; }

// ---- the kernel with activations shared through LDS: when it applies, and its launch
constexpr int kSharedT = 4, kSharedKgs = 4, kSharedNg = 2;  // 128 columns per workgroup, eight wavefronts

bool mid_shared_applies(const MnbGemmArgs& a) {
  const MnbLayout& L = a.L;
  if (a.io != kMnbIoModel || L.dtype != kMnbDtypeFloat16 || a.M <= 16) return false;
  const int CK = 4 * L.group_k;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0);
  // the fills address A with 32-bit byte offsets from the chunk's first column
  const bool reach = (uint64_t)a.M * (uint64_t)a.lda * 2 + 512 < ((uint64_t)1 << 32);
  if (!vec_ok || !reach || L.K % CK != 0) return false;
  bool use;
  if (const char* e = mnb_tuning_env("MNB_MID_SHARED")) {
    use = e[0] != '0';
  } else {
    // A workgroup here needs the same time whatever the grid (eight rounds of 2 - 3 us at K = 4096), so the kernel pays
    // where its 128-column slabs make one well-filled round of workgroups -- which is also where the activations'
    // stream through the level-2 caches is largest.  Measured against the kernel above (K = 4096, 4-bit):
    // N = 28672: M = 17 21.9 -> 17.7 us, M = 32 22.8 -> 17.6, M = 64 28.5 -> 25.5; N = 14336, M = 128 28.1 -> 24.8;
    // N = 11008, M = 128 30.2 -> 25.2; N = 6144, M = 256 27.4 -> 24.0; with fewer workgroups than 5/8 of the compute
    // units, or more than all of them, it loses (N = 14336, M = 64: 16.9 -> 24.0; N = 28672, M = 256: 82 -> 100).
    const int64_t slabs = (L.N + 16 * kSharedT * kSharedNg - 1) / (16 * kSharedT * kSharedNg);
    const int rows = a.M <= 32 ? 32 : 64;
    const int64_t wgs = slabs * ((a.M + rows - 1) / rows), cus = mnb_device_info().cus;
    use = wgs * 8 >= cus * 5 && wgs <= cus && L.K / CK >= 2 * kSharedKgs;
  }
  return use;
}

template <int BITS, bool HAS_ZP, int MT>
hipError_t launch_shared_mt(const MidParams& mp, hipStream_t s) {
  const SkinnyParams& p = mp.s;
  constexpr int T = kSharedT, KGS = kSharedKgs, NG = kSharedNg, NW = KGS * NG;
  constexpr size_t chunk_bytes = (size_t)16 * MT * (128 / BITS / 2) * 16;
  constexpr size_t fills = 2 * KGS * chunk_bytes, red = (size_t)NW * T * 4 * 64 * sizeof(float);
  constexpr size_t smem = fills > red ? fills : red;
  auto kernel = mnb_mid_shared_kernel<BITS, HAS_ZP, T, MT, KGS, NG>;
  // more than 64 KB of dynamic LDS has to be asked for, once per device (the attribute is kept per device)
  static std::atomic<unsigned long long> asked{0};
  int device = 0;
  if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
  if (device >= 64 || !((asked.load(std::memory_order_relaxed) >> device) & 1ull)) {
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        e != hipSuccess)
      return e;
    if (device < 64) asked.fetch_or(1ull << device, std::memory_order_relaxed);
  }
  const dim3 grid((unsigned)((p.N + 16 * T * NG - 1) / (16 * T * NG)), (unsigned)((p.M + 16 * MT - 1) / (16 * MT)));
  kernel<<<grid, dim3(NW * 64), smem, s>>>(p.W, p.Npad, p.A, p.meta, p.lda, p.chunks, p.bs_shift, mp);
  return hipGetLastError();
}

template <int BITS, bool HAS_ZP>
hipError_t launch_shared(const MidParams& mp, hipStream_t s) {
  return mp.s.M <= 32 ? launch_shared_mt<BITS, HAS_ZP, 2>(mp, s) : launch_shared_mt<BITS, HAS_ZP, 4>(mp, s);
}

}  // namespace

bool mnb_mid_applicable(const MnbGemmArgs& a) {
  // fp16 models, and 16-bit ones (a.io) on a matrix packed with fp32 meta entries
  return (a.io != kMnbIoModel ? a.L.dtype == kMnbDtypeFloat : a.L.dtype == kMnbDtypeFloat16) && a.M >= 1;
}

// bytes of the staged copy of A
size_t mnb_mid_workspace_bytes(const MnbLayout& L, int64_t M) {
  const int CK = 4 * L.group_k;
  const int64_t chunks = (L.K + CK - 1) / CK;
  return (size_t)chunks * (L.group_k / 8) * mid_row_tiles(M, 4) * 64 * 16;  // the larger of the two row blockings
}

// Activations straight from A when its rows allow 16-byte loads and K is a whole number of chunks (the kernel then
// reorders them itself, and no workspace is touched); otherwise, and for the widest tiles, a staging pass writes them
// in operand order first.
bool mnb_mid_shared(const MnbGemmArgs& a) { return mid_shared_applies(a); }


bool mnb_mid_direct(const MnbGemmArgs& a) {
  if (mid_shared_applies(a)) return true;  // (reads A in place as well)
  const MidPlan pl = mid_plan(a.L, a.M, a.epi.kind == kMnbFusedMlp ? 2 : 1);
  const bool vec_ok = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0);
  bool direct = vec_ok && a.L.K % (4 * a.L.group_k) == 0 && !(pl.mt == 4 && pl.t == 4);
  if (const char* e = mnb_tuning_env("MNB_MID_DIRECT")) direct = direct && e[0] != '0';  // calibration
  return direct;
}

hipError_t mnb_launch_mid(const MnbGemmArgs& a, hipStream_t s) {
  const MnbLayout& L = a.L;
  if (!mnb_mid_applicable(a) || (a.io != kMnbIoModel && a.epi.kind != kMnbFusedNone)) return hipErrorInvalidValue;
  const MidPlan pl = mid_plan(L, a.M, a.epi.kind == kMnbFusedMlp ? 2 : 1);
  const int CK = 4 * L.group_k;
  MidParams mp{};
  SkinnyParams& p = mp.s;
  p.A = reinterpret_cast<const _Float16*>(a.A);
  p.W = reinterpret_cast<const uint4*>(a.packed);
  p.meta = reinterpret_cast<const uint8_t*>(a.packed) + L.meta_off;
  p.bias = reinterpret_cast<const _Float16*>(a.bias);
  p.C = reinterpret_cast<_Float16*>(a.C);
  p.lda = a.lda;
  p.ldc = a.ldc;
  p.Npad = L.Npad;
  p.M = (int)a.M;
  p.N = (int)L.N;
  p.K = (int)L.K;
  p.bs_shift = mnb_log2i(L.bs);
  p.chunks = (int)((L.K + CK - 1) / CK);
  p.io_bf16 = a.io == kMnbIoBf16;
  p.epi.kind = a.epi.kind;
  if (a.epi.kind != kMnbFusedNone) {
    p.C = reinterpret_cast<_Float16*>(a.epi.out[0]);
    p.ldc = a.epi.ld[0];
    p.epi.start1 = (int)a.epi.start[1];
    p.epi.start2 = (int)a.epi.start[2];
    p.epi.n0 = (int)a.epi.n[0];
    p.epi.n1 = (int)a.epi.n[1];
    p.epi.n2 = (int)a.epi.n[2];
    p.epi.out1 = reinterpret_cast<_Float16*>(a.epi.out[1]);
    p.epi.out2 = reinterpret_cast<_Float16*>(a.epi.out[2]);
    p.epi.ld1 = a.epi.ld[1];
    p.epi.ld2 = a.epi.ld[2];
  }
  if (mid_shared_applies(a)) {
    if (L.bits == 4) return L.has_zp ? launch_shared<4, true>(mp, s) : launch_shared<4, false>(mp, s);
    return L.has_zp ? launch_shared<8, true>(mp, s) : launch_shared<8, false>(mp, s);
  }
  mp.As = reinterpret_cast<const uint4*>(a.workspace);
  mp.row_tiles = mid_row_tiles(a.M, pl.mt);
  const int vec_ok = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0);
  const bool direct = mnb_mid_direct(a);
  if (!direct) {
    if (a.workspace == nullptr || a.workspace_bytes < mnb_mid_workspace_bytes(L, a.M)) return hipErrorInvalidValue;
    const int64_t units = (int64_t)p.chunks * (L.group_k / 8) * mp.row_tiles * 64;
    const dim3 sgrid((unsigned)((units + 255) / 256));
    uint4* staged = reinterpret_cast<uint4*>(a.workspace);
    if (L.bits == 4)
      mnb_mid_stage_a_kernel<4><<<sgrid, dim3(256), 0, s>>>(p.A, p.lda, p.M, p.K, p.chunks, mp.row_tiles, vec_ok, staged);
    else
      mnb_mid_stage_a_kernel<8><<<sgrid, dim3(256), 0, s>>>(p.A, p.lda, p.M, p.K, p.chunks, mp.row_tiles, vec_ok, staged);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  }
  if (L.bits == 4)
    return L.has_zp ? launch_io<4, true>(mp, pl, a.io, direct, s) : launch_io<4, false>(mp, pl, a.io, direct, s);
  return L.has_zp ? launch_io<8, true>(mp, pl, a.io, direct, s) : launch_io<8, false>(mp, pl, a.io, direct, s);
}
