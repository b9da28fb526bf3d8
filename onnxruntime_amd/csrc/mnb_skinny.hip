// fp16 decode kernel for 1 <= M <= 16: which calls it serves, its plan and the dispatch to the translation unit that
// holds the kernels of the call's weight format.  The design is described at the top of mnb_skinny_kernels.hip.h.
#include "mnb_skinny_kernels.hip.h"

bool mnb_skinny_applicable(const MnbGemmArgs& a) {
  // fp16 models, and 16-bit ones (a.io) on a matrix packed with fp32 meta entries
  return (a.io != kMnbIoModel ? a.L.dtype == kMnbDtypeFloat : a.L.dtype == kMnbDtypeFloat16) && a.M >= 1 && a.M <= 16;
}

bool mnb_skinny_native2(const MnbGemmArgs& a) {
  const MnbLayout& L = a.L;
  return L.src_bits == 2 && L.w2_bytes > 0 && a.io == kMnbIoModel && a.M <= 16 &&
         (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0) && (L.K % 256 == 0);
}

hipError_t mnb_launch_skinny(const MnbGemmArgs& a, hipStream_t s) {
  const MnbLayout& L = a.L;
  if (!mnb_skinny_applicable(a) || (a.io != kMnbIoModel && a.epi.kind != kMnbFusedNone)) return hipErrorInvalidValue;
  // direct variant: 16-byte loads of whole chunks of A
  const bool a_vec_ok = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0) && (L.K % (4 * L.group_k) == 0);
  // 2-bit sources: the copy in their own width (half the bytes to stream) when the matrix has one and whole chunks
  // of 256 k can be read straight from aligned activations; else the nibble copy
  const bool native2 = mnb_skinny_native2(a);
  MnbLayout L2 = L;
  if (native2) {
    L2.bits = 2;
    L2.group_k = 64;
  }
  SkinnyPlan pl = skinny_plan(native2 ? L2 : L, a.io, a.M, a_vec_ok, a.epi.kind == kMnbFusedMlp ? 2 : 1);
  SkinnyParams p{};
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
  const int CK = 4 * (native2 ? L2.group_k : L.group_k);
  p.chunks = (int)((L.K + CK - 1) / CK);
  if (native2) p.W = reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(a.packed) + L.w2_off);
  p.phase_chunks = pl.phase_chunks;
  p.mtr = pl.mtr;
  p.a_vec_ok = a_vec_ok;
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
  if (native2) return mnb_skinny_launch_w2(&p, &pl, s);
  if (L.bits == 4) return L.has_zp ? mnb_skinny_launch_w4zp(&p, &pl, s) : mnb_skinny_launch_w4(&p, &pl, s);
  return mnb_skinny_launch_w8(&p, &pl, L.has_zp, s);
}
