// Launchers implemented in the .hip translation units; called by the C ABI in mnb_api.hip.
#pragma once
#include <cstdlib>
#include <hip/hip_runtime.h>

#include "mnb_layout.h"

// Destination of a GEMM over several matrices packed as one (mnb_layout.h): kMnbFusedNone writes C / ldc.
struct MnbEpilogue {
  int kind;          // kMnbFused*
  int64_t start[3];  // qkv: first packed column of each output
  int64_t n[3];      // columns of each output (mlp: n[0])
  void* out[3];      // qkv: the three outputs; mlp: out[0]
  int64_t ld[3];
};

// Element type of A, bias and C when it is not the packed matrix's own (MnbGemmArgs::io).
constexpr int kMnbIoModel = 0;    // L.dtype
constexpr int kMnbIoBf16 = 1;     // bfloat16 on a matrix packed with fp32 {scale, zero point} entries
constexpr int kMnbIoF16Wide = 2;  // fp16 on such a matrix (zero points in the activation type: 4-bit with zero points)

struct MnbGemmArgs {
  MnbLayout L;
  int64_t M;
  const void* A;
  int64_t lda;
  const void* packed;
  const void* bias;
  void* C;
  int64_t ldc;
  void* workspace;
  size_t workspace_bytes;
  MnbEpilogue epi;  // kind != kMnbFusedNone: C / ldc are unused, bias is indexed by packed column
  int io = 0;       // tile GEMM and decode kernel: kMnbIoModel, or A, bias and C in a 16-bit type on a matrix packed for
                    // an fp32 model (L.dtype is float): kMnbIoBf16, kMnbIoF16Wide
};

enum MnbKernelKind {
  kMnbKernelNone = 0,
  kMnbKernelSkinny,     // fp16, M <= 16: dequantising skinny GEMM on the matrix cores
  kMnbKernelGemv,       // fp32, M <= 16: dequantising GEMV (VALU dot products, activations in SGPRs)
  kMnbKernelMid,        // fp16, M > 16: weights from registers to the matrix cores, K split over waves (any shape)
  kMnbKernelGemm256,    // fp16, MFMA GEMM with 256 x 256 tiles: large M, enough tiles to fill the chip
  kMnbKernelGemm32,     // fp32, many rows: tile GEMM on the fp32 matrix cores
  kMnbKernelRows16F32,  // fp32, 5 <= M <= 64: weights from registers to the fp32 matrix cores, K split over waves
  kMnbKernelGemmGeneric // any shape: simple tile kernel (fallback)
};

MnbKernelKind mnb_select_kernel(const MnbGemmArgs& a);
const char* mnb_kernel_name(MnbKernelKind k, const MnbLayout& L);

// records `message` as the calling thread's last error (MnbGetLastErrorMessage) and returns `code`
int mnb_report_error(int code, const char* message);

// weights only, one source matrix (the meta part of the packed buffer is written by the caller)
hipError_t mnb_launch_pack_weights(const MnbLayout& L, const void* B, void* packed, hipStream_t s);
hipError_t mnb_launch_pack(const MnbLayout& L, const void* B, const void* scales, const void* zp, void* packed,
                           hipStream_t s);
hipError_t mnb_launch_pack_fused(const MnbFusedLayout& F, const void* const* B, const void* const* scales,
                                 const void* const* bias, void* packed, hipStream_t s);
hipError_t mnb_launch_dequant_canonical(void* dst, const void* B, const void* scales, const void* zp, int64_t N,
                                        int64_t K, int bits, int bs, int dtype, hipStream_t s);
hipError_t mnb_launch_quantize(void* B, void* scales, void* zp, const void* src, int64_t K, int64_t N, int64_t ld,
                               int bits, int bs, int dtype, hipStream_t s);
hipError_t mnb_launch_dequant_packed(void* dst, const void* packed, const MnbLayout& L, hipStream_t s);

bool mnb_skinny_applicable(const MnbGemmArgs& a);
hipError_t mnb_launch_skinny(const MnbGemmArgs& a, hipStream_t s);
bool mnb_mid_applicable(const MnbGemmArgs& a);
hipError_t mnb_launch_mid(const MnbGemmArgs& a, hipStream_t s);
bool mnb_rows16_f32_applicable(const MnbGemmArgs& a);
hipError_t mnb_launch_rows16_f32(const MnbGemmArgs& a, hipStream_t s);
size_t mnb_mid_workspace_bytes(const MnbLayout& L, int64_t M);  // staged copy of A
bool mnb_mid_direct(const MnbGemmArgs& a);  // this call reads A in place: no staged copy, no workspace
bool mnb_skinny_native2(const MnbGemmArgs& a);  // a decode call that streams the native copy of 2-bit weights
bool mnb_mid_shared(const MnbGemmArgs& a);  // ... through the variant whose wavefront pairs share the activations in LDS
// 16 < M: whether the tile GEMM's plan beats the streaming kernel's estimate for this shape (needs K % 128 == 0)
bool mnb_prefer_gemm256(const MnbLayout& L, int64_t M);
bool mnb_gemv_applicable(const MnbGemmArgs& a);
hipError_t mnb_launch_gemv(const MnbGemmArgs& a, hipStream_t s);
hipError_t mnb_launch_gemm256(const MnbGemmArgs& a, hipStream_t s);
// compute units and engine clock (Hz) of the current device; asked once per device (mnb_api.hip)
// Environment overrides of the launch planners exist only in builds made with -DMNB_TUNING_HOOKS (calibration runs);
// the shipped library reads no environment variable: mnb_tuning_env returns nullptr there.
#if defined(MNB_TUNING_HOOKS)
inline const char* mnb_tuning_env(const char* name) { return getenv(name); }
#else
inline const char* mnb_tuning_env(const char*) { return nullptr; }
#endif

struct MnbDeviceInfo {
  int cus;
  double clock_hz;
};
const MnbDeviceInfo& mnb_device_info();
// how the tile GEMM would run a problem (mnb_gemm256.hip)
struct MnbGemm256Plan {
  int tile_rows;           // 256 or 128
  int tile_cols;           // 256, or 128 (with 128 rows, fp16 models)
  int64_t grid;            // workgroups: the tiles, or one per compute unit when tiles are split along K
  bool split;              // tiles are computed in parts by several workgroups (needs workspace_bytes of scratch)
  size_t workspace_bytes;  // flags + one partial tile per workgroup; 0 without a split
  double seconds;          // estimate, for the choice between kernels
};
// io: element type of the activations when it is not the packed matrix's own (MnbGemmArgs::io)
MnbGemm256Plan mnb_gemm256_plan(const MnbLayout& L, int64_t M, bool with_workspace, int io = kMnbIoModel);
// device address of the status word in a split launch's workspace; NULL when the plan for this problem does not split
const uint32_t* mnb_gemm256_status_word(const MnbLayout& L, int64_t M, int io, const void* workspace,
                                        size_t workspace_bytes);
bool mnb_gemm256_fused_ok(const MnbEpilogue& e);  // outputs allow the tile GEMM's 16-byte stores
// the tile GEMM's 32-bit per-lane offsets reach every element of this problem
uint64_t mnb_gemm256_max_lane_offset(int64_t lda);
bool mnb_gemm256_addressable(int64_t lda, int64_t Npad);
hipError_t mnb_launch_gemm_generic(const MnbGemmArgs& a, hipStream_t s);
// int8 activations (accuracy_level 4; mnb_gemm_i8.hip): 4-bit weights, fp16 model, block sizes 64 ... 256, M rows
// within the reach of the kernel's 32-bit offsets
bool mnb_gemm_i8_supported(const MnbLayout& L, int64_t M);
size_t mnb_gemm_i8_workspace_bytes(const MnbLayout& L, int64_t M);
hipError_t mnb_launch_gemm_i8(const MnbGemmArgs& a, hipStream_t s);
bool mnb_gemm32_applicable(const MnbGemmArgs& a);
hipError_t mnb_launch_gemm32(const MnbGemmArgs& a, hipStream_t s);

// kernels around the fused operators (mnb_fused.hip)
// A (+ skip) -> A_norm = x / sqrt(mean(x^2) + eps) * scale per row; sum_out (optional) = A + skip
hipError_t mnb_launch_rmsnorm(void* a_norm, void* sum_out, int64_t ld_sum, const void* A, int64_t lda, const void* skip,
                              int64_t ld_skip, int64_t skip_rows, const void* scale, float epsilon, int64_t M, int64_t K,
                              int dtype, hipStream_t s);
// tmp[M][Np] (plain GEMM over the packed matrix, bias included) -> the operator's outputs
hipError_t mnb_launch_fused_finish(const MnbEpilogue& epi, const void* tmp, int64_t ld_tmp, int64_t M, int dtype,
                                   hipStream_t s);

