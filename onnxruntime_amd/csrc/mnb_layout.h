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
  int bits, bs, dtype, has_zp;
  int64_t k_blocks;   // ceil(K / bs)
  int64_t Npad, Kpad; // padded extents
  int64_t KG;         // 16-byte groups along k
  int64_t KBp;        // blocks along padded k
  int group_k;        // k covered by one 16-byte group: 32 (4-bit) or 16 (8-bit)
  int meta_bytes;     // bytes of one meta entry
  int64_t w_bytes, meta_off, total_bytes;
};

MNB_HD int64_t mnb_round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// position of column n inside a meta row
MNB_HD int64_t mnb_meta_col(int64_t n) { return (n & ~(int64_t)63) | ((n & 15) << 2) | ((n >> 4) & 3); }

MNB_HD MnbLayout mnb_make_layout(int64_t N, int64_t K, int bits, int bs, int dtype, int has_zp) {
  MnbLayout L;
  L.N = N;
  L.K = K;
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
  return L;
}
