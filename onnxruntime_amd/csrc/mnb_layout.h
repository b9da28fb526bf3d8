// Packed (gfx950) layout of one MatMulNBits weight matrix, shared by host and device code.
//
// The canonical operand layout (contrib_defs.cc:3782-3849 of the reference) keeps each output column contiguous
// along K.  The kernels here want the opposite: the 64 lanes of a wavefront own 64 neighbouring columns and read
// one 128-bit vector each, so PrePack turns the matrix into "k-group major" order:
//
//   W   [KG][Npad][16 B]      one 16-byte vector = 32 (4-bit) or 16 (8-bit) consecutive k of one column.
//                             4-bit: inside every 32-bit word the nibbles of elements e0..e7 are stored in the
//                             order e0 e2 e4 e6 e1 e3 e5 e7 (LSB first), so that (w & 0x000F000F), (w & 0x00F000F0),
//                             ((w>>8) & ...) yield the pairs (e0,e1) (e2,e3) (e4,e5) (e6,e7) as fp16 lanes.
//                             8-bit: bytes stay in k order.
//   meta[KBp][Npad]           per (block, column): fp16 model {half scale, half -(1024+zp)} (4 B) or {half scale}
//                             (2 B) when there are no zero points; fp32 model {float scale, float zp} (8 B) or
//                             {float scale} (4 B).  Inside every slab of 64 columns the entries are stored in the
//                             order (n%16)*4 + (n%64)/16, so that the four 16-column tiles a matrix-core lane
//                             works on are adjacent and arrive with one vector load (mnb_meta_col).
//
//   W2  [Kpad/64][Npad][16 B] 2-bit sources of fp16 models with blocks of 32 and more only, behind everything else: the
//                             weights once more in their own width for the decode kernel (M <= 16 streams half the
//                             bytes).  One 16-byte vector = 64 k of one column, the operands of eight matrix
//                             instructions: vector 4 c + kq holds, as operand i, k = 256 c + 128 (i / 4) + 32 kq +
//                             8 (i % 4) .. + 7 (mnb_w2_k), so that every matrix instruction of a wavefront -- it sums
//                             over the four kq -- stays inside one block of 128; inside every 32-bit word
//                             the fields of elements e0..e15 are stored e0 e2 .. e14 in the low half and e1 e3 .. e15
//                             in the high half (LSB first), so that (w & 0x00030003), (w & 0x000C000C), (w & 0x00300030),
//                             (w & 0x00C000C0) yield the pairs (e0,e1) (e2,e3) (e4,e5) (e6,e7) and the same masks on
//                             w >> 8 the pairs (e8,e9) .. (e14,e15).  The meta entries are shared with W.
//
//   Npad = N rounded up to 256, Kpad = k_blocks*block_size rounded up to 128, KG = Kpad*bits/128, KBp = Kpad/bs.
//   Padding columns and padding k hold zero weights and zero scales, so loads never need a bounds check.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __HIPCC__
#define MNB_HD __host__ __device__ inline
#else
#define MNB_HD inline
#endif

constexpr int kMnbDtypeFloat = 1;
constexpr int kMnbDtypeFloat16 = 10;
constexpr int kMnbColAlign = 256;
constexpr int kMnbKAlign = 128;

struct MnbLayout {
  int64_t N, K;
  int bits, bs, dtype, has_zp;  // of the PACKED matrix (2-bit weights are stored as 4-bit ones with zero points)
  int src_bits;                 // bits of the canonical operands
  int64_t k_blocks;   // ceil(K / bs)
  int64_t Npad, Kpad; // padded extents
  int64_t KG;         // 16-byte groups along k
  int64_t KBp;        // blocks along padded k
  int group_k;        // k covered by one 16-byte group: 32 (4-bit) or 16 (8-bit)
  int meta_bytes;     // bytes of one meta entry
  int64_t w_bytes, meta_off, total_bytes;
  int64_t w2_off, w2_bytes;  // the native 2-bit copy for the decode kernel (0, 0: none)
};

MNB_HD int64_t mnb_round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// log2 of a power of two (block sizes)
MNB_HD int mnb_log2i(int v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

// first k of operand i (0..7) of vector g of the native 2-bit copy
MNB_HD int64_t mnb_w2_k(int64_t g, int i) { return (g >> 2) * 256 + (int64_t)(i >> 2) * 128 + (g & 3) * 32 + (i & 3) * 8; }

// position of column n inside a meta row
MNB_HD int64_t mnb_meta_col(int64_t n) { return (n & ~(int64_t)63) | ((n & 15) << 2) | ((n >> 4) & 3); }

// native2: 2-bit sources also get the W2 section (the variant layouts do without)
MNB_HD MnbLayout mnb_make_layout(int64_t N, int64_t K, int bits, int bs, int dtype, int has_zp, bool native2 = true) {
  MnbLayout L;
  L.N = N;
  L.K = K;
  L.src_bits = bits;
  if (bits == 2) {
    // 2-bit weights are widened to nibbles when packed, so every 4-bit kernel runs them unchanged (at the 4-bit
    // kernels' byte rate); their default zero point 2 is not the 4-bit kernels' 8, so it is always stored
    bits = 4;
    has_zp = 1;
  }
  L.bits = bits;
  L.bs = bs;
  L.dtype = dtype;
  L.has_zp = has_zp ? 1 : 0;
  L.k_blocks = (K + bs - 1) / bs;
  L.Npad = mnb_round_up(N, kMnbColAlign);
  L.Kpad = mnb_round_up(L.k_blocks * bs, kMnbKAlign);
  L.group_k = 128 / bits;
  L.KG = L.Kpad / L.group_k;
  L.KBp = L.Kpad / bs;
  int scale_bytes = dtype == kMnbDtypeFloat16 ? 2 : 4;
  L.meta_bytes = has_zp ? 2 * scale_bytes : scale_bytes;
  L.w_bytes = L.KG * L.Npad * 16;
  L.meta_off = mnb_round_up(L.w_bytes, 256);
  L.total_bytes = mnb_round_up(L.meta_off + L.KBp * L.Npad * L.meta_bytes, 256);
  L.w2_off = 0;
  L.w2_bytes = 0;
  if (native2 && L.src_bits == 2 && dtype == kMnbDtypeFloat16 && bs >= 32) {
    L.w2_off = L.total_bytes;
    L.w2_bytes = (L.Kpad / 64) * L.Npad * 16;
    L.total_bytes += mnb_round_up(L.w2_bytes, 256);
  }
  return L;
}

// ---- several weight matrices behind one activation (MatMulNBitsMlp, MatMulNBitsQkv; contrib_defs.cc:3851-4090) ----
// The matrices share K, bits and block size and have no zero points.  They are packed as ONE matrix of Np columns so
// that a single launch streams all of them:
//   kMnbFusedMlp  gate and up interleaved by 16-column tiles: packed tile 2u = gate columns [16u, 16u+16), packed
//                 tile 2u+1 = the same columns of up.  A workgroup that owns an even number of adjacent tiles holds
//                 both operands of  silu(gate) * up  for its columns.
//   kMnbFusedQkv  Q, K and V side by side, each segment padded to a multiple of 16 columns, so that a 16-column tile
//                 never straddles two outputs.
// Behind the packed matrix the buffer holds one bias value per packed column (zero where the operator has no bias).
constexpr int kMnbFusedNone = 0;
constexpr int kMnbFusedMlp = 1;
constexpr int kMnbFusedQkv = 2;

struct MnbColMap {
  int kind;          // kMnbFused*
  int nsrc;          // matrices: 2 (mlp) or 3 (qkv)
  int64_t n[3];      // columns of each matrix
  int64_t start[3];  // qkv: first packed column of each segment
  int64_t Np;        // packed columns
};

struct MnbFusedLayout {
  MnbLayout L;  // the packed matrix: N = Np
  MnbColMap map;
  int64_t bias_off;
  int64_t total_bytes;
};

// packed column -> (matrix, column); false for padding columns
MNB_HD bool mnb_map_col(const MnbColMap& m, int64_t np, int* src, int64_t* col) {
  if (m.kind == kMnbFusedMlp) {
    const int64_t tile = np >> 4;
    *src = (int)(tile & 1);
    *col = (tile >> 1) * 16 + (np & 15);
    return np < m.Np && *col < m.n[0];
  }
  if (m.kind == kMnbFusedQkv) {
    const int s = np >= m.start[2] ? 2 : np >= m.start[1] ? 1 : 0;
    *src = s;
    *col = np - m.start[s];
    return np < m.Np && *col < m.n[s];
  }
  *src = 0;
  *col = np;
  return np < m.n[0];
}

MNB_HD MnbFusedLayout mnb_make_fused_layout(int kind, int64_t n0, int64_t n1, int64_t K, int bits, int bs, int dtype) {
  MnbFusedLayout F;
  MnbColMap& m = F.map;
  m.kind = kind;
  if (kind == kMnbFusedMlp) {  // n0 = N of gate and up
    m.nsrc = 2;
    m.n[0] = m.n[1] = n0;
    m.n[2] = 0;
    m.start[0] = m.start[1] = m.start[2] = 0;
    m.Np = 2 * mnb_round_up(n0, 16);
  } else {  // n0 = Nq, n1 = Nkv
    m.nsrc = 3;
    m.n[0] = n0;
    m.n[1] = m.n[2] = n1;
    m.start[0] = 0;
    m.start[1] = mnb_round_up(n0, 16);
    m.start[2] = m.start[1] + mnb_round_up(n1, 16);
    m.Np = m.start[2] + mnb_round_up(n1, 16);
  }
  F.L = mnb_make_layout(m.Np, K, bits, bs, dtype, 0);
  F.bias_off = F.L.total_bytes;
  F.total_bytes = F.bias_off + mnb_round_up(m.Np * (dtype == kMnbDtypeFloat16 ? 2 : 4), 256);
  return F;
}
