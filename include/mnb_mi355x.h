/*
 * mnb_mi355x.h -- C ABI of libmnb_mi355x.so: com.microsoft::MatMulNBits for AMD Instinct MI355X (gfx950).
 *
 * The library is the device-side replacement of the routines the reference CPU kernel
 * (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc) calls in MLAS.  Every entry point takes plain
 * pointers and sizes; pointers named *_dev are HIP device pointers on the current device, `stream` is a
 * hipStream_t passed as void* (NULL = the default stream).  All functions are asynchronous with respect to the
 * host unless stated otherwise, return 0 on success or an MnbStatus code, and leave a message retrievable with
 * MnbGetLastErrorMessage() (thread local) on failure.  No function throws.
 *
 * Canonical (on-disk) operand layout, as defined by the operator schema
 * (onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3782-3849):
 *   k_blocks = ceil(K / block_size)
 *   B           u8 [N][k_blocks][block_size*bits/8]   2-bit: element e of a byte in bits 2e..2e+1;  4-bit: low nibble =
 *                                                     even k;  8-bit: one byte per element
 *   scales      T  [N][k_blocks]                       T = fp32 or fp16, same as A
 *   zero_points u8 [N][ceil(k_blocks*bits/8)]          packed like B; absent -> 2^(bits-1)
 *   bias        T  [N]
 *   W[k][n] = (q - zp) * scale;  Y[m][n] = sum_k A[m][k] * W[k][n] (+ bias[n]);  k >= K is ignored.
 */
#ifndef MNB_MI355X_H_
#define MNB_MI355X_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MNB_API __attribute__((visibility("default")))

/* Status codes; numeric values are those of OrtErrorCode
 * (include/onnxruntime/core/session/onnxruntime_error_code.h) so a caller inside an execution provider can
 * forward them to OrtApi::CreateStatus unchanged. */
typedef enum MnbStatus {
  MNB_OK = 0,
  MNB_FAIL = 1,
  MNB_INVALID_ARGUMENT = 2,
  MNB_NOT_IMPLEMENTED = 9,
  MNB_EP_FAIL = 11
} MnbStatus;

/* Element types; numeric values are those of ONNXTensorElementDataType
 * (include/onnxruntime/core/session/onnxruntime_c_api.h:195-222). */
typedef enum MnbDataType {
  MNB_DTYPE_FLOAT = 1,
  MNB_DTYPE_UINT8 = 2,
  MNB_DTYPE_INT32 = 6,
  MNB_DTYPE_FLOAT16 = 10,
  MNB_DTYPE_BFLOAT16 = 16 /* activations of the rare-variant entry points only (MnbVariant*) */
} MnbDataType;

/* Shape of one operator input for MnbCheckInputs; dims == NULL means the optional input is absent. */
typedef struct MnbTensorInfo {
  const int64_t* dims;
  size_t rank;
  int dtype; /* MnbDataType */
} MnbTensorInfo;

/* Message of the last failure on the calling thread ("" if none). The pointer stays valid until the next
 * failing call on the same thread. */
MNB_API const char* MnbGetLastErrorMessage(void);

/* Library ABI version (bumped when a signature or the packed layout changes). */
MNB_API int MnbGetVersion(void);

/* Number of usable gfx950 devices seen by HIP, or 0. Never fails. */
MNB_API int MnbGetDeviceCount(void);

/* Replaces MlasIsQNBitGemmAvailable (onnxruntime/core/mlas/inc/mlas_qnbit.h:134-139).
 * 1 if (bits, block_size, a_dtype) has a device kernel: bits in {2, 4, 8}, block_size in {16,32,64,128,256},
 * a_dtype in {MNB_DTYPE_FLOAT, MNB_DTYPE_FLOAT16}; else 0. */
MNB_API int MnbIsAvailable(int bits, int block_size, int a_dtype);

/* Replaces matmul_nbits_helper::CheckInputs
 * (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_helper.h:38-109): validates the shapes of the
 * operator inputs against the attributes, with the same messages. quantized_weight may be absent (already
 * packed). group_index values are not inspected (they live on the device). */
MNB_API int MnbCheckInputs(const MnbTensorInfo* quantized_weight, const MnbTensorInfo* scales,
                           const MnbTensorInfo* zero_points, const MnbTensorInfo* group_index,
                           const MnbTensorInfo* bias, int64_t n, int64_t k, int64_t block_size, int64_t bits);

/* Replaces MlasQNBitGemmPackQuantBDataSize (mlas_qnbit.h:206-215): bytes of the packed buffer that holds
 * weights, scales and zero points of one [N, K] matrix in the gfx950 tiled layout; 0 if unsupported.
 * has_zero_points: 1 if the operator has a zero_points input (the packed meta then carries them).
 * 2-bit weights are stored widened to nibbles (every 4-bit kernel runs them) with their zero points always explicit;
 * float16 models with blocks of 32 and more also keep a copy in the weights' own width, N * K / 4 bytes, which the
 * decode kernel streams for up to 16 rows when K is a multiple of 256 and the activations are 16-byte aligned. */
MNB_API size_t MnbPackQuantBDataSize(size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype);

/* Replaces MlasQNBitGemmPackQuantBData (mlas_qnbit.h:244-258): repacks canonical B, scales and zero points
 * (all on the device) into packed_dev (MnbPackQuantBDataSize bytes, 256-byte aligned). zero_points_dev may be
 * NULL (default zero point; has_zero_points = 0 everywhere else). The inputs may be freed once the stream has run
 * the call. */
MNB_API int MnbPackQuantBData(size_t N, size_t K, int bits, int block_size, int a_dtype, const void* b_dev,
                              const void* scales_dev, const void* zero_points_dev, void* packed_dev, void* stream);

/* Replaces MlasQNBitGemmBatchWorkspaceSize (mlas_qnbit.h:178-189): bytes of per-call device scratch MnbGemm needs for
 * this problem.  Non-zero only for fp16 activations: (a) shapes that select the weight-streaming kernel (M > 16 below
 * the tile GEMM's range, or M <= 16 with K not a multiple of 128 (4-bit) / 64 (8-bit)): a copy of A in matrix-core
 * operand order, about M*K*2 bytes, which that kernel needs unless A is 16-byte aligned with a pitch that is a
 * multiple of 8 and K is a whole number of 128 (4-bit) / 64 (8-bit) elements - such activations are read in place
 * (except by the widest tile, 64 rows x 64 columns, which large N with more than 32 rows selects) and the call is
 * then served without the scratch; (b) tall problems with few output tiles on
 * the tile GEMM, which then cuts every tile along K across workgroups: flags plus one fp32 partial tile per workgroup,
 * up to about 64 MiB.  Without (or with less than) the scratch of (b) the tile GEMM runs uncut. */
MNB_API size_t MnbGemmWorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                                    int a_dtype);

/* Replaces MlasQNBitGemmBatch at SQNBIT_CompFp32 (mlas_qnbit.h:111-125) for one B matrix:
 *   C[M][N] (ldc) = A[M][K] (lda) x dequant(packed)^T (+ bias[N]).
 * a_dev, bias_dev (optional) and c_dev have element type a_dtype; lda and ldc count elements. M <= 16 runs the
 * dequantising GEMV; larger M the weight-streaming matrix-core kernel or, once 256 x 256 tiles fill the chip, the
 * tiled MFMA GEMM (fp16), or the fp32 tile kernel. M == 0 or N == 0 is a
 * no-op. workspace_dev / workspace_bytes: per-call scratch of MnbGemmWorkspaceSize bytes (may be NULL / 0 when
 * that size is 0); it must not be shared by calls that may overlap. */
MNB_API int MnbGemm(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                    const void* a_dev, size_t lda, const void* packed_dev, const void* bias_dev, void* c_dev,
                    size_t ldc, void* workspace_dev, size_t workspace_bytes, void* stream);

/* Health of the last MnbGemm launch that used this workspace for the same problem.  No counterpart in the reference.
 * Only the tile GEMM's cut along K (case (b) of MnbGemmWorkspaceSize) has anything to report: its workgroups hand
 * partial sums to one another through the workspace and wait for one another with a bound; a wait that gave up has
 * written NaN into its output tile and set a word in the workspace.  *gave_up = 1 then, else 0 (also for problems and
 * workspaces that do not take the cut).  The call waits for `stream`.  The word is cleared by the next launch that
 * uses the workspace. */
MNB_API int MnbGemmWorkspaceStatus(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                                   int a_dtype, const void* workspace_dev, size_t workspace_bytes, void* stream,
                                   int* gave_up);

/* MnbGemm for callers that cannot allocate or carry device memory of their own: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and results
 * as MnbGemm (bit for bit) minus the workspace: the scratch MnbGemm would ask for lives in a device array inside the
 * library (MnbGemmStaticScratchCapacity bytes, 32 MiB + 64 KiB, held on every device the library runs on until the process
 * ends).  The call allocates and frees nothing.  A problem whose MnbGemmWorkspaceSize exceeds the capacity is rejected
 * with MNB_INVALID_ARGUMENT, unless the kernel that serves the call without a workspace needs none: the tile GEMM then
 * runs without its optional cut of tiles along K (the same sums in another fp32 order).  Every call on a device shares that device's array: calls that may overlap on one device
 * (different streams, several threads) race on it and must be serialised by the caller. */
MNB_API size_t MnbGemmStaticScratchCapacity(void);
MNB_API int MnbGemmStaticScratch(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                                 int a_dtype, const void* a_dev, size_t lda, const void* packed_dev,
                                 const void* bias_dev, void* c_dev, size_t ldc, void* stream);

/* Workspace bytes MnbGemmUnpacked needs (packed copy + MnbGemmWorkspaceSize). */
MNB_API size_t MnbGemmUnpackedWorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size,
                                            int has_zero_points, int a_dtype);

/* The Compute path when the weights were not packed at session initialisation (session.disable_prepacking, or B
 * not a constant initializer): counterpart of MatMulNBits<T1>::ComputeBUnpacked
 * (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:1184-1333). Packs into workspace_dev on the stream,
 * then runs MnbGemm. */
MNB_API int MnbGemmUnpacked(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, const void* a_dev,
                            size_t lda, const void* b_dev, const void* scales_dev, const void* zero_points_dev,
                            const void* bias_dev, void* c_dev, size_t ldc, void* workspace_dev,
                            size_t workspace_bytes, void* stream);

/* Replaces MlasDequantizeBlockwise<T, bits> with column-wise blocks (onnxruntime/core/mlas/inc/mlas_q4.h:352-362,
 * definition onnxruntime/core/mlas/lib/q4_dq.cpp:587-641): dst_dev[n*K + k] = (q - zp) * scale in a_dtype.
 * fp32: one multiply; fp16: round-to-nearest-even of the exact product. */
MNB_API int MnbDequantizeBlockwise(void* dst_dev, const void* b_dev, const void* scales_dev,
                                   const void* zero_points_dev, int block_size, int bits, size_t K, size_t N,
                                   int a_dtype, void* stream);

/* Same output as MnbDequantizeBlockwise, read back from a packed buffer: proves that packing loses nothing. */
MNB_API int MnbDequantizePacked(void* dst_dev, const void* packed_dev, size_t N, size_t K, int bits, int block_size,
                                int has_zero_points, int a_dtype, void* stream);

/* Replaces MlasQuantizeBlockwise<T, bits> with column-wise blocks (onnxruntime/core/mlas/inc/mlas_q4.h:315-328,
 * definition onnxruntime/core/mlas/lib/q4_dq.cpp:468-574): quantises src_dev, a row-major [K][leading_dimension]
 * matrix of a_dtype elements of which the first N columns are used, into the canonical operands b_dev
 * u8[N][k_blocks][block_size*bits/8] and scales_dev T[N][k_blocks], plus zero_points_dev u8[N][ceil(k_blocks*bits/8)]
 * for asymmetric quantisation; zero_points_dev == NULL selects symmetric quantisation (zero point 2^(bits-1)).
 * Every byte of the outputs is written. Elements k >= K of the last block are stored as the zero point. */
MNB_API int MnbQuantizeBlockwise(void* b_dev, void* scales_dev, void* zero_points_dev, const void* src_dev,
                                 int block_size, int bits, size_t K, size_t N, size_t leading_dimension, int a_dtype,
                                 void* stream);

/* ---- several projections behind one activation ------------------------------------------------------------------
 * com.microsoft::MatMulNBitsMlp and MatMulNBitsQkv (onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3851-3975 and
 * :3977-4090; the reference's only kernels for them are the WebGPU ones,
 * onnxruntime/contrib_ops/webgpu/quantization/matmul_nbits_mlp.cc:241-543 and matmul_nbits_qkv.cc:150-392).
 * The weight matrices share K, bits and block_size, have no zero points, and are packed into ONE buffer so that one
 * launch streams all of them; the biases (NULL = absent) are folded into that buffer at pack time. */

/* Optional prologue of both operators: SimplifiedLayerNormalization (skip_dev == NULL) or
 * SkipSimplifiedLayerNormalization of the activation
 * (onnxruntime/contrib_ops/cpu/skip_layer_norm.cc:44-97): x = A + skip, A_norm = x / sqrt(mean_k(x^2) + epsilon) *
 * norm_scale, computed in fp32 and narrowed once.  norm_scale_dev == NULL: no prologue (skip must be NULL too). */
typedef struct MnbNormPrologue {
  const void* norm_scale_dev; /* T[K] */
  const void* skip_dev;       /* optional T[skip_rows][ld_skip]; row m of A is added to skip row m % skip_rows */
  size_t ld_skip;
  size_t skip_rows;           /* 0 = one skip row per row of A */
  void* skip_sum_dev;         /* optional output T[M][ld_skip_sum]: A + skip (the operators' input_skip_bias_sum) */
  size_t ld_skip_sum;
  float epsilon;
} MnbNormPrologue;

#define MNB_ACTIVATION_SILU 0 /* the only activation the operator defines (matmul_nbits_mlp.cc:24-31) */

/* MatMulNBitsMlp: Y[M][N] = silu(A' x gate^T + gate_bias) * (A' x up^T + up_bias), A' = A or its normalisation.
 * Gate/up products and the activation are evaluated in fp32; Y is narrowed once. */
MNB_API size_t MnbMlpPackSize(size_t N, size_t K, int bits, int block_size, int a_dtype);
MNB_API int MnbMlpPack(size_t N, size_t K, int bits, int block_size, int a_dtype, const void* gate_b_dev,
                       const void* gate_scales_dev, const void* gate_bias_dev, const void* up_b_dev,
                       const void* up_scales_dev, const void* up_bias_dev, void* packed_dev, void* stream);
MNB_API size_t MnbMlpWorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, int has_norm);
MNB_API int MnbMlpGemm(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, const void* a_dev,
                       size_t lda, const MnbNormPrologue* norm, const void* packed_dev, int activation, void* y_dev,
                       size_t ldc, void* workspace_dev, size_t workspace_bytes, void* stream);

/* MatMulNBitsQkv: Q[M][Nq], K[M][Nkv], V[M][Nkv] = A' x {q,k,v}^T + bias. */
MNB_API size_t MnbQkvPackSize(size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype);
MNB_API int MnbQkvPack(size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype, const void* q_b_dev,
                       const void* q_scales_dev, const void* q_bias_dev, const void* k_b_dev,
                       const void* k_scales_dev, const void* k_bias_dev, const void* v_b_dev,
                       const void* v_scales_dev, const void* v_bias_dev, void* packed_dev, void* stream);
MNB_API size_t MnbQkvWorkspaceSize(size_t M, size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype,
                                   int has_norm);
MNB_API int MnbQkvGemm(size_t M, size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype,
                       const void* a_dev, size_t lda, const MnbNormPrologue* norm, const void* packed_dev, void* q_dev,
                       size_t ldq, void* k_dev, size_t ldk, void* v_dev, size_t ldv, void* workspace_dev,
                       size_t workspace_bytes, void* stream);

/* The prologue alone (what the fused calls run first): a_norm_dev T[M][K], dense. */
MNB_API int MnbSimplifiedLayerNorm(size_t M, size_t K, int a_dtype, const void* a_dev, size_t lda,
                                   const MnbNormPrologue* norm, void* a_norm_dev, void* stream);

/* ---- rare operand variants -----------------------------------------------------------------------------------------
 * The inputs the reference kernel serves through its dequantise-everything route and calls "very rare"
 * (MatMulNBits<T>::ComputeBUnpacked, onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:1184-1333, fp16
 * :1336-1510): zero points in the activation type (input zero_points of type T1, shape [N][k_blocks]), a group index
 * (input g_idx, int32[K] or [k_blocks*block_size]: element k of every column uses scale and zero point of block
 * g_idx[k]; dequantisation onnxruntime/contrib_ops/cpu/quantization/matmul_nbits_impl.cc:19-75), and bfloat16
 * activations (type constraint T1 of the schema, contrib_defs.cc:3782-3849; the reference has no CPU kernel for it).
 *
 * They run on the same GEMM kernels as MnbGemm after a transformation made once, at pack time:
 *   g_idx            the k index is permuted so that the elements of one group are adjacent and the matrix is packed
 *                    in that order: with the operator's block size when every group has a multiple of it (act-order
 *                    permutations), else with the largest power of two >= 16 that divides every group, else with
 *                    block size 16 and every group padded to a multiple of 16.  The activation columns are gathered
 *                    into that order (zeros in the padding) in front of every GEMM.  A g_idx equal to
 *                    k / block_size is recognised and dropped.
 *   typed zero points:  scales and zero points are widened to fp32 (exactly) at pack time and the matrix is packed
 *                    as an fp32 model's; fp32 models run the fp32 kernels on it (the reference's own arithmetic for
 *                    these inputs: fp32 SGEMM on dequantised operands, :1336-1510).
 *   16-bit models on such a matrix (bfloat16, always packed this way; fp16 with typed zero points):  the matrix-core
 *                    kernels run on it in the activation type instead - the decode kernel up to 16 rows, the
 *                    streaming kernel or the tile GEMM beyond, chosen as for fp16 models:
 *                    w = fma(float(q), scale, -zp * scale) in fp32, narrowed to the activation type (round to nearest
 *                    even), products accumulated in fp32, bias added and the sum narrowed in the epilogue.  This is
 *                    what the reference's GPU provider multiplies (B dequantised into the activation type, then a
 *                    GEMM of that type: onnxruntime/contrib_ops/cuda/quantization/matmul_nbits.cc:844-975); the CPU
 *                    provider has no bfloat16 kernel.  The tile GEMM reads activations in place when they are 16-byte
 *                    aligned with a pitch that is a multiple of 8 and there is no g_idx, else from a copy in the
 *                    workspace; the other two take any alignment.
 *                    One exception, with different (tighter) arithmetic: 4-bit weights in blocks of 128 and more on
 *                    the decode kernel (M <= 16).  There no weight is narrowed to the activation type.  The matrix
 *                    instruction multiplies the activations by the raw operand r = c + q, which is exact in the
 *                    activation type (bfloat16: c = 128; float16: c = 1024, or 64 for the nibbles taken from bits
 *                    4..7), two more matrix instructions per block against constant operands give S_c = sum(c * a) and
 *                    S_1 = sum(a), and the block contributes  scale * (sum(a * r) - S_c - zp * S_1)  with every sum, the
 *                    scale and the zero point in fp32 (scale and zp are the unrounded fp32 meta entries).  The result
 *                    differs from the formula above by the weight rounding that formula contains and this one does
 *                    not (relative L2 against float64: 1.7e-3 against 2.2e-3 for bfloat16, both dominated by the
 *                    narrowing of Y), so the same model rounds slightly differently at M <= 16 than at M > 16; both
 *                    are inside the operator's tolerance, and the reference holds no bfloat16 vectors to pin either.
 * Zero points are honoured together with g_idx for both zero-point types, as the schema defines; the reference's CPU
 * dequantiser reads uint8 zero points in that combination but then uses 8 (matmul_nbits_impl.cc:56-66).
 * Supported: g_idx with bits = 4; typed zero points with bits = 2 or 4 (the reference rejects 8, :1251-1252). */
typedef enum MnbZeroPointKind {
  MNB_ZP_NONE = 0,  /* no zero_points input: 2^(bits-1) */
  MNB_ZP_UINT8 = 1, /* packed uint8, [N][ceil(k_blocks*bits/8)] */
  MNB_ZP_TYPED = 2  /* activation type, [N][k_blocks] */
} MnbZeroPointKind;

/* Filled by MnbVariantMakePlan; plain data the caller keeps next to the packed buffer. */
typedef struct MnbVariantPlan {
  int64_t N, K;
  int bits, block_size; /* of the operator */
  int a_dtype;          /* MNB_DTYPE_FLOAT, MNB_DTYPE_FLOAT16 or MNB_DTYPE_BFLOAT16 */
  int zp_kind;          /* MnbZeroPointKind */
  int has_g_idx;        /* a g_idx that is not k / block_size: activations are gathered per call */
  int compute_dtype;    /* element type the GEMM kernels run in: a_dtype or MNB_DTYPE_FLOAT */
  int64_t packed_k;     /* k extent of the packed matrix (K without g_idx) */
  int packed_block_size;
  int reserved;
  uint64_t gather_offset; /* byte offset of the int32 gather table inside the packed buffer */
  uint64_t packed_bytes;  /* size of the packed buffer */
} MnbVariantPlan;

/* g_idx_host: HOST pointer to g_idx_len int32 values, or NULL.  Fails with MNB_INVALID_ARGUMENT when a value lies
 * outside [0, k_blocks) and with MNB_NOT_IMPLEMENTED for a combination without kernels. */
MNB_API int MnbVariantMakePlan(size_t N, size_t K, int bits, int block_size, int a_dtype, int zp_kind,
                               const int32_t* g_idx_host, size_t g_idx_len, MnbVariantPlan* plan);
/* Packs the canonical operands (device pointers; scales and typed zero points in a_dtype) into packed_dev
 * (plan->packed_bytes, 256-byte aligned).  g_idx_host must be the array the plan was made from.  Synchronises the
 * stream when the plan has a g_idx (the gather table is uploaded from pageable host memory). */
MNB_API int MnbVariantPack(const MnbVariantPlan* plan, const void* b_dev, const void* scales_dev,
                           const void* zero_points_dev, const int32_t* g_idx_host, size_t g_idx_len, void* packed_dev,
                           void* stream);
MNB_API size_t MnbVariantGemmWorkspaceSize(const MnbVariantPlan* plan, size_t M);
/* Y[M][ldy] = A[M][lda] x W (+ bias), A, bias and Y in plan->a_dtype. */
MNB_API int MnbVariantGemm(const MnbVariantPlan* plan, size_t M, const void* a_dev, size_t lda, const void* packed_dev,
                           const void* bias_dev, void* y_dev, size_t ldy, void* workspace_dev, size_t workspace_bytes,
                           void* stream);
/* Name of the GEMM kernel MnbVariantGemm would run for M rows (static string; for logs and profiles). */
MNB_API const char* MnbVariantGemmKernelName(const MnbVariantPlan* plan, size_t M);
/* The reference's dequantiser for these inputs, dst_dev float[N][K] whatever a_dtype is
 * (Dequantize4BitsKernelReOrder, matmul_nbits_impl.cc:19-75; 2 bits: MlasDequantizeBlockwiseFpZeroPoint,
 * onnxruntime/core/mlas/lib/q4_dq.cpp:2187-2241): scales and zero points widened to fp32,
 * w = float(q) * scale + (-scale * zp), each operation rounded on its own.  g_idx_dev: device pointer or NULL. */
MNB_API int MnbVariantDequantize(float* dst_dev, const void* b_dev, const void* scales_dev,
                                 const void* zero_points_dev, int zp_kind, const int32_t* g_idx_dev, size_t N,
                                 size_t K, int bits, int block_size, int a_dtype, void* stream);

/* int8 activations (the reference's accuracy_level 4: SQ4BitGemm_CompInt8,
 * onnxruntime/core/mlas/lib/qnbitgemm.cpp:883-1086, with the arithmetic of the scalar statement its kernels are
 * tested against, onnxruntime/test/mlas/unittest/test_sqnbitgemm.cpp:94-170).  A is quantised per row and block of
 * block_size elements (scale = max|a| / 127, round half away from zero), every block's dot product with the 4-bit
 * weights is exact integer arithmetic, and Y = bias + sum over blocks of float(dot) * a_scale * b_scale in fp32,
 * blocks in k order, narrowed once.  Same packed weights as MnbGemm.  Implemented for bits = 4, a_dtype float16,
 * block sizes 64 ... 256 and M * K / block_size below 2^29 (MNB_NOT_IMPLEMENTED otherwise).  Blocks of 32 -- the block
 * size the reference's own int8 kernels are built around -- are declined on purpose: the contract fixes one fp32
 * multiply-add chain per output and 32-deep block, 80 vector instructions behind every matrix instruction, which ran
 * 19 times slower than MnbGemm on a prefill shape.  accuracy_level is a permission, not a demand: MnbGemm computes the
 * same nodes at full accuracy and is faster for every block size (measured on prefill shapes: 1.2 times at blocks of
 * 128, 1.5 at 256), so nothing chooses this entry point by itself.  The workspace (16-byte aligned,
 * MnbGemmInt8WorkspaceSize bytes, 0 = not implemented for these arguments) receives the quantised activations. */
MNB_API size_t MnbGemmInt8WorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                                        int a_dtype);
MNB_API int MnbGemmInt8(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                        const void* a_dev, size_t lda, const void* packed_dev, const void* bias_dev, void* c_dev,
                        size_t ldc, void* workspace_dev, size_t workspace_bytes, void* stream);

/* Name of the kernel MnbGemm would run for this problem (static string; for logs and profiles). */
MNB_API const char* MnbGemmKernelName(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype);
/* The same for activations with a row pitch of lda elements (MnbGemmKernelName assumes K rounded up to 8).  The tile
 * GEMM addresses a tile's activations with 32-bit byte offsets from the tile's first row, 255 * lda + 63 elements at
 * most; pitches beyond that range select the streaming kernel, whose addressing is 64-bit. */
MNB_API const char* MnbGemmKernelNameStrided(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype,
                                             size_t lda);
/* How the tile GEMM would cut this problem when MnbGemm runs it with the workspace MnbGemmWorkspaceSize asks for: rows and
 * columns of a tile (256 x 256, 128 x 256 or 128 x 128) and the number of parts a tile is cut into along K; zeros when
 * another kernel takes the problem.  For logs, profiles and tests. */
MNB_API int MnbGemmTilePlan(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                            int* tile_rows, int* tile_cols, int* parts);

#ifdef __cplusplus
}
#endif
#endif /* MNB_MI355X_H_ */
