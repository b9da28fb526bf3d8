// C ABI of libmnb_mi355x.so (declared in include/mnb_mi355x.h): argument validation, error reporting and kernel
// selection.  No exception leaves this file.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "../../include/mnb_mi355x.h"
#include "mnb_internal.h"

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(MNB_EP_FAIL, "%s: %s", what, hipGetErrorString(e));
}

bool supported(int bits, int bs, int dtype) {
  const bool b = bits == 2 || bits == 4 || bits == 8;
  const bool s = bs == 16 || bs == 32 || bs == 64 || bs == 128 || bs == 256;
  const bool d = dtype == MNB_DTYPE_FLOAT || dtype == MNB_DTYPE_FLOAT16;
  return b && s && d;
}

int check_config(const char* fn, int bits, int bs, int dtype) {
  // Same wording as the reference kernel's constructor (matmul_nbits.cc:130-135).
  if (bits != 2 && bits != 4 && bits != 8)
    return fail(MNB_INVALID_ARGUMENT,
                "%s: Only 2b, 4b and 8b quantization is supported for MatMulNBits op, additional bits support is "
                "planned.", fn);
  if (!(bs == 16 || bs == 32 || bs == 64 || bs == 128 || bs == 256))
    return fail(MNB_INVALID_ARGUMENT,
                "%s: Only block sizes 16, 32, 64, 128, and 256 are supported for MatMulNBits op, got: %d", fn, bs);
  if (dtype != MNB_DTYPE_FLOAT && dtype != MNB_DTYPE_FLOAT16)
    return fail(MNB_NOT_IMPLEMENTED, "%s: element type %d has no MI355X kernel (float and float16 only)", fn, dtype);
  return MNB_OK;
}

std::string shape_str(const int64_t* d, size_t r) {
  std::string s = "{";
  for (size_t i = 0; i < r; ++i) {
    if (i) s += ",";
    s += std::to_string(d[i]);
  }
  return s + "}";
}

bool shape_is(const MnbTensorInfo* t, std::initializer_list<int64_t> want) {
  if (t->rank != want.size()) return false;
  size_t i = 0;
  for (int64_t w : want)
    if (t->dims[i++] != w) return false;
  return true;
}

std::string want_str(std::initializer_list<int64_t> want) {
  std::string s = "{";
  bool first = true;
  for (int64_t w : want) {
    if (!first) s += ",";
    s += std::to_string(w);
    first = false;
  }
  return s + "}";
}

bool present(const MnbTensorInfo* t) { return t != nullptr && t->dims != nullptr; }

}  // namespace

int mnb_report_error(int code, const char* message) {
  g_last_error = message;
  return code;
}

extern "C" {

const char* MnbGetLastErrorMessage(void) { return g_last_error.c_str(); }

int MnbGetVersion(void) { return 1; }

int MnbGetDeviceCount(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  int usable = 0;
  for (int i = 0; i < n; ++i) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, i) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0) ++usable;
  }
  return usable;
}

int MnbIsAvailable(int bits, int block_size, int a_dtype) { return supported(bits, block_size, a_dtype) ? 1 : 0; }

int MnbCheckInputs(const MnbTensorInfo* quantized_weight, const MnbTensorInfo* scales,
                   const MnbTensorInfo* zero_points, const MnbTensorInfo* group_index, const MnbTensorInfo* bias,
                   int64_t n, int64_t k, int64_t block_size, int64_t bits) {
  if (bits != 2 && bits != 4 && bits != 8)
    return fail(MNB_INVALID_ARGUMENT, "bits should be 2, 4 or 8, got %lld", (long long)bits);
  if (block_size < 16 || (block_size & (block_size - 1)) != 0)
    return fail(MNB_INVALID_ARGUMENT, "block_size must be a power of 2, and >= 16. Got %lld", (long long)block_size);
  const int64_t k_blocks = (k + block_size - 1) / block_size;
  const int64_t blob_size = block_size * bits / 8;

  auto mismatch1 = [&](const char* name, const MnbTensorInfo* t, std::initializer_list<int64_t> want) {
    return fail(MNB_INVALID_ARGUMENT, "Input '%s' is expected to have shape %s, got %s", name, want_str(want).c_str(),
                shape_str(t->dims, t->rank).c_str());
  };
  auto mismatch2 = [&](const char* name, const MnbTensorInfo* t, std::initializer_list<int64_t> w1,
                       std::initializer_list<int64_t> w2) {
    return fail(MNB_INVALID_ARGUMENT, "Input '%s' is expected to have shape %s or %s, got %s", name,
                want_str(w1).c_str(), want_str(w2).c_str(), shape_str(t->dims, t->rank).c_str());
  };

  if (present(quantized_weight) && !shape_is(quantized_weight, {n, k_blocks, blob_size}))
    return mismatch1("quantized_weight", quantized_weight, {n, k_blocks, blob_size});
  if (present(scales) && !shape_is(scales, {n * k_blocks}) && !shape_is(scales, {n, k_blocks}))
    return mismatch2("scales", scales, {n * k_blocks}, {n, k_blocks});
  if (present(zero_points)) {
    if (zero_points->dtype == MNB_DTYPE_UINT8) {
      const int64_t zb = (k_blocks * bits + 7) / 8;
      if (!shape_is(zero_points, {n * zb}) && !shape_is(zero_points, {n, zb}))
        return mismatch2("zero_points", zero_points, {n * zb}, {n, zb});
    } else {
      if (present(scales) && zero_points->dtype != scales->dtype)
        return fail(MNB_INVALID_ARGUMENT,
                    "Input 'zero_points' and 'scales' should have the same data type when zero_points is not uint8");
      if (!shape_is(zero_points, {n * k_blocks}) && !shape_is(zero_points, {n, k_blocks}))
        return mismatch2("zero_points", zero_points, {n * k_blocks}, {n, k_blocks});
    }
  }
  if (present(group_index) && !shape_is(group_index, {k}) && !shape_is(group_index, {k_blocks * block_size}))
    return mismatch2("group_index", group_index, {k}, {k_blocks * block_size});
  if (present(bias) && !shape_is(bias, {n})) return mismatch1("bias", bias, {n});
  return MNB_OK;
}

size_t MnbPackQuantBDataSize(size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype) {
  if (!supported(bits, block_size, a_dtype) || N == 0 || K == 0) return 0;
  return (size_t)mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points).total_bytes;
}

int MnbPackQuantBData(size_t N, size_t K, int bits, int block_size, int a_dtype, const void* b_dev,
                      const void* scales_dev, const void* zero_points_dev, void* packed_dev, void* stream) {
  if (int rc = check_config("MnbPackQuantBData", bits, block_size, a_dtype)) return rc;
  if (N == 0 || K == 0) return MNB_OK;
  if (!b_dev || !scales_dev || !packed_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbPackQuantBData: B, scales and the packed buffer must not be NULL");
  if (reinterpret_cast<uintptr_t>(packed_dev) % 256 != 0)
    return fail(MNB_INVALID_ARGUMENT, "MnbPackQuantBData: the packed buffer must be 256-byte aligned");
  MnbLayout L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, zero_points_dev != nullptr);
  hipError_t e = mnb_launch_pack(L, b_dev, scales_dev, zero_points_dev, packed_dev, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbPackQuantBData");
}

}  // extern "C"

// ------------------------------------------------------------------------------------------------ device facts
// Compute units and engine clock of the current device, asked once per device and process.  The kernel-choice
// estimates below are stated in cycles and per compute unit and scaled by these, so they follow the part the library
// runs on.  Without a usable device (a host that only asks for kernel names) the MI355X figures stand in.
const MnbDeviceInfo& mnb_device_info() {
  constexpr int kMaxDevices = 64;
  static MnbDeviceInfo info[kMaxDevices];
  static std::once_flag once[kMaxDevices];
  static const MnbDeviceInfo fallback{256, 2.4e9};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return fallback;
  }
  std::call_once(once[dev], [dev] {
    int cus = 0, khz = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, dev) != hipSuccess || khz <= 0) khz = 2400000;
    (void)hipGetLastError();
    info[dev] = MnbDeviceInfo{cus, (double)khz * 1e3};
  });
  return info[dev];
}

// ------------------------------------------------------------------------------------------------ kernel choice
// fp16, M > 16: the weight-streaming kernel (mnb_mid.hip) takes any shape; the tile GEMM wins once its tiles occupy
// enough of the chip.  The estimate compares the tile GEMM's plan (mnb_gemm256_plan) with the streaming kernel's
// measured behaviour over the same range of shapes: a fixed 8 us (at 2.4 GHz) plus 2MNK at 1286 flop per compute unit
// and cycle for 4-bit weights (790 Tflop/s on 256 compute units), 1156 for 8-bit.
constexpr double kMnbMidStartCycles = 19200.0;
constexpr double kMnbMidFlopsPerCuCycle[2] = {1286.0, 1156.0};

bool mnb_prefer_gemm256(const MnbLayout& L, int64_t M) {
  if (L.K % 128 != 0) return false;
  if (const char* e = mnb_tuning_env("MNB_MID_MAX_M")) return M > (int64_t)atoll(e);  // calibration: M up to this streams
  if (M <= 64) return false;  // (64-row tiles were measured: never ahead of the streaming kernel)
  const MnbDeviceInfo& dev = mnb_device_info();
  const double t_mid = (kMnbMidStartCycles + 2.0 * (double)M * (double)L.N * (double)L.K /
                                                 (kMnbMidFlopsPerCuCycle[L.bits == 4 ? 0 : 1] * dev.cus)) /
                       dev.clock_hz;
  // a caller that follows MnbGemmWorkspaceSize hands over the workspace the split needs
  return mnb_gemm256_plan(L, M, true).seconds < t_mid;
}

MnbKernelKind mnb_select_kernel(const MnbGemmArgs& a) {
  if (mnb_skinny_applicable(a)) {
    // The decode kernel reads activations 16 bytes at a time; when K is not a whole number of its chunks (or A is
    // misaligned) its fallback stages A element by element.  The streaming kernel's staged copy of A (zero-padded,
    // any alignment) is the faster route whenever the caller's workspace allows it.
    const bool direct = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0) &&
                        (a.L.K % (4 * a.L.group_k) == 0);
    if (!direct && a.workspace_bytes >= mnb_mid_workspace_bytes(a.L, a.M)) return kMnbKernelMid;  // (staged there too)
    return kMnbKernelSkinny;
  }
  if (mnb_rows16_f32_applicable(a)) return kMnbKernelRows16F32;
  if (mnb_gemv_applicable(a)) return kMnbKernelGemv;
  if (mnb_gemm32_applicable(a)) return kMnbKernelGemm32;
  if (a.L.dtype == kMnbDtypeFloat16) {
    // the tile GEMM loads activations 16 bytes at a time: base and row pitch aligned
    // and addresses them with 32-bit offsets from a per-tile base
    const bool aligned = (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) && (a.lda % 8 == 0) &&
                         mnb_gemm256_addressable(a.lda, a.L.Npad);
    if (aligned && mnb_prefer_gemm256(a.L, a.M)) return kMnbKernelGemm256;
    // the workspace is sized for the streaming kernel only when the shape alone selects it
    if (!mnb_prefer_gemm256(a.L, a.M) || a.workspace_bytes >= mnb_mid_workspace_bytes(a.L, a.M) || mnb_mid_direct(a))
      return kMnbKernelMid;
  }
  return kMnbKernelGemmGeneric;
}

const char* mnb_kernel_name(MnbKernelKind k, const MnbLayout&) {
  switch (k) {
    case kMnbKernelSkinny: return "mnb_skinny_kernel";
    case kMnbKernelGemv: return "mnb_gemv_kernel";
    case kMnbKernelMid: return "mnb_mid_kernel";
    case kMnbKernelGemm256: return "mnb_gemm256_kernel";
    case kMnbKernelGemm32: return "mnb_gemm32_kernel";
    case kMnbKernelRows16F32: return "mnb_rows16_f32_kernel";
    case kMnbKernelGemmGeneric: return "mnb_gemm_generic_kernel";
    default: return "none";
  }
}

extern "C" {

size_t MnbGemmWorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                            int a_dtype) {
  if (!supported(bits, block_size, a_dtype) || N == 0 || K == 0 || M == 0) return 0;
  // only the mid-M fp16 kernel needs scratch: a copy of A in matrix-core operand order
  if (a_dtype == kMnbDtypeFloat16) {
    const MnbLayout L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
    // M <= 16 needs it only when K is not a whole number of the decode kernel's chunks
    const bool wants = M > 16 ? !mnb_prefer_gemm256(L, (int64_t)M) : (K % (size_t)(4 * L.group_k) != 0);
    if (wants) return mnb_mid_workspace_bytes(L, (int64_t)M);
    // the tile GEMM: partial tiles and flags when it splits tiles along K across workgroups
    if (M > 16) return mnb_gemm256_plan(L, (int64_t)M, true).workspace_bytes;
  }
  return 0;
}

// Validation and dispatch shared by MnbGemm and MnbGemmStaticScratch.
static int gemm_checked(const char* fn, size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                        int a_dtype, const void* a_dev, size_t lda, const void* packed_dev, const void* bias_dev,
                        void* c_dev, size_t ldc, void* workspace_dev, size_t workspace_bytes, void* stream) {
  if (int rc = check_config(fn, bits, block_size, a_dtype)) return rc;
  if (M == 0 || N == 0) return MNB_OK;  // empty output: nothing to compute (matmul_nbits.cc:1533-1536)
  if (K == 0) return fail(MNB_INVALID_ARGUMENT, "%s: K must be positive", fn);
  if (!a_dev || !packed_dev || !c_dev) return fail(MNB_INVALID_ARGUMENT, "%s: A, packed B and C must not be NULL", fn);
  if (lda < K || ldc < N)
    return fail(MNB_INVALID_ARGUMENT, "%s: lda (%zu) < K (%zu) or ldc (%zu) < N (%zu)", fn, lda, K, ldc, N);
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff)
    return fail(MNB_INVALID_ARGUMENT, "%s: M, N and K must fit in 31 bits", fn);
  MnbGemmArgs a{};  // epi: plain output
  a.L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
  a.M = (int64_t)M;
  a.A = a_dev;
  a.lda = (int64_t)lda;
  a.packed = packed_dev;
  a.bias = bias_dev;
  a.C = c_dev;
  a.ldc = (int64_t)ldc;
  a.workspace = workspace_dev;
  a.workspace_bytes = workspace_dev ? workspace_bytes : 0;
  hipStream_t s = (hipStream_t)stream;
  hipError_t e;
  switch (mnb_select_kernel(a)) {
    case kMnbKernelSkinny: e = mnb_launch_skinny(a, s); break;
    case kMnbKernelGemv: e = mnb_launch_gemv(a, s); break;
    case kMnbKernelMid: {
      const size_t need = mnb_mid_workspace_bytes(a.L, a.M);
      if (a.workspace_bytes < need && !mnb_mid_direct(a))  // (aligned activations are read in place)
        return fail(MNB_INVALID_ARGUMENT, "%s: workspace of %zu bytes needed (MnbGemmWorkspaceSize), %zu given", fn, need,
                    a.workspace_bytes);
      e = mnb_launch_mid(a, s);
      break;
    }
    case kMnbKernelGemm256: e = mnb_launch_gemm256(a, s); break;
    case kMnbKernelGemm32: e = mnb_launch_gemm32(a, s); break;
    case kMnbKernelRows16F32: e = mnb_launch_rows16_f32(a, s); break;
    default: e = mnb_launch_gemm_generic(a, s); break;
  }
  return e == hipSuccess ? MNB_OK : hip_fail(e, fn);
}

int MnbGemm(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
            const void* a_dev, size_t lda, const void* packed_dev, const void* bias_dev, void* c_dev, size_t ldc,
            void* workspace_dev, size_t workspace_bytes, void* stream) {
  return gemm_checked("MnbGemm", M, N, K, bits, block_size, has_zero_points, a_dtype, a_dev, lda, packed_dev, bias_dev,
                      c_dev, ldc, workspace_dev, workspace_bytes, stream);
}

int MnbGemmWorkspaceStatus(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                           const void* workspace_dev, size_t workspace_bytes, void* stream, int* gave_up) {
  const char* fn = "MnbGemmWorkspaceStatus";
  if (!gave_up) return fail(MNB_INVALID_ARGUMENT, "%s: gave_up must not be NULL", fn);
  *gave_up = 0;
  if (int rc = check_config(fn, bits, block_size, a_dtype)) return rc;
  if (M == 0 || N == 0 || K == 0 || a_dtype != kMnbDtypeFloat16 || M <= 16) return MNB_OK;
  const MnbLayout L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
  if (!mnb_prefer_gemm256(L, (int64_t)M)) return MNB_OK;  // another kernel: its workspace holds no status
  const uint32_t* word = mnb_gemm256_status_word(L, (int64_t)M, kMnbIoModel, workspace_dev, workspace_bytes);
  if (word == nullptr) return MNB_OK;  // the launch ran uncut
  uint32_t v = 0;
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = hipMemcpyAsync(&v, word, sizeof(v), hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  if (e != hipSuccess) return hip_fail(e, fn);
  *gave_up = v != 0;
  return MNB_OK;
}

size_t MnbGemmInt8WorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                                int a_dtype) {
  if (check_config("MnbGemmInt8WorkspaceSize", bits, block_size, a_dtype) != MNB_OK || M == 0 || N == 0 || K == 0) return 0;
  const MnbLayout L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
  return mnb_gemm_i8_supported(L, (int64_t)M) ? mnb_gemm_i8_workspace_bytes(L, (int64_t)M) : 0;
}

int MnbGemmInt8(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                const void* a_dev, size_t lda, const void* packed_dev, const void* bias_dev, void* c_dev, size_t ldc,
                void* workspace_dev, size_t workspace_bytes, void* stream) {
  const char* fn = "MnbGemmInt8";
  if (int rc = check_config(fn, bits, block_size, a_dtype)) return rc;
  if (M == 0 || N == 0) return MNB_OK;
  if (K == 0) return fail(MNB_INVALID_ARGUMENT, "%s: K must be positive", fn);
  if (!a_dev || !packed_dev || !c_dev) return fail(MNB_INVALID_ARGUMENT, "%s: A, packed B and C must not be NULL", fn);
  if (lda < K || ldc < N)
    return fail(MNB_INVALID_ARGUMENT, "%s: lda (%zu) < K (%zu) or ldc (%zu) < N (%zu)", fn, lda, K, ldc, N);
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff)
    return fail(MNB_INVALID_ARGUMENT, "%s: M, N and K must fit in 31 bits", fn);
  MnbGemmArgs a{};
  a.L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
  if (!mnb_gemm_i8_supported(a.L, (int64_t)M))
    return fail(MNB_NOT_IMPLEMENTED,
                "%s: int8 activations are implemented for 4-bit weights, float16 models, block sizes 64 to 256 and "
                "M * K / block_size below 2^29 (got M=%zu, K=%zu, bits=%d, block_size=%d, a_dtype=%d); MnbGemm "
                "computes these at full accuracy",
                fn, M, K, bits, block_size, a_dtype);
  const size_t need = mnb_gemm_i8_workspace_bytes(a.L, (int64_t)M);
  if (!workspace_dev || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace_dev) % 16 != 0)
    return fail(MNB_INVALID_ARGUMENT, "%s: a 16-byte aligned workspace of %zu bytes is needed (MnbGemmInt8WorkspaceSize), %zu given",
                fn, need, workspace_dev ? workspace_bytes : (size_t)0);
  a.M = (int64_t)M;
  a.A = a_dev;
  a.lda = (int64_t)lda;
  a.packed = packed_dev;
  a.bias = bias_dev;
  a.C = c_dev;
  a.ldc = (int64_t)ldc;
  a.workspace = workspace_dev;
  a.workspace_bytes = workspace_bytes;
  const hipError_t e = mnb_launch_gemm_i8(a, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, fn);
}

}  // extern "C"

// ---- the entry point that allocates nothing ---------------------------------------------------------------------------
// The per-call scratch of MnbGemm (the streaming kernel's copy of A in matrix-core operand order) as a file-scope
// device array: every device the library runs on holds its own copy, at its own address, until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
// 32 MiB of partial tiles (128 workgroups x 256 KiB, the usual cut of a tall problem along K) plus their flags
constexpr size_t kMnbStaticScratchBytes = ((size_t)32 << 20) + ((size_t)64 << 10);
static __device__ __align__(256) unsigned char scratch[kMnbStaticScratchBytes];

namespace {

// Device address of `scratch` on the current device; asked once per device, with that device current.
int static_scratch_address(void** out) {
  constexpr int kMaxDevices = 64;
  static void* address[kMaxDevices];
  static hipError_t status[kMaxDevices];
  static std::once_flag once[kMaxDevices];
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return hip_fail(e, "MnbGemmStaticScratch: hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices)
    return fail(MNB_NOT_IMPLEMENTED, "MnbGemmStaticScratch: device ordinal %d is beyond the %d this entry point tracks", dev,
                kMaxDevices);
  std::call_once(once[dev], [dev] {
    void* p = nullptr;
    status[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    address[dev] = status[dev] == hipSuccess ? p : nullptr;
  });
  if (status[dev] != hipSuccess) return hip_fail(status[dev], "MnbGemmStaticScratch: hipGetSymbolAddress");
  if (address[dev] == nullptr) return fail(MNB_EP_FAIL, "MnbGemmStaticScratch: the scratch array has no device address");
  *out = address[dev];
  return MNB_OK;
}

}  // namespace

extern "C" {

size_t MnbGemmStaticScratchCapacity(void) { return kMnbStaticScratchBytes; }

int MnbGemmStaticScratch(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                         const void* a_dev, size_t lda, const void* packed_dev, const void* bias_dev, void* c_dev,
                         size_t ldc, void* stream) {
  if (int rc = check_config("MnbGemmStaticScratch", bits, block_size, a_dtype)) return rc;
  if (M == 0 || N == 0) return MNB_OK;
  size_t need = MnbGemmWorkspaceSize(M, N, K, bits, block_size, has_zero_points, a_dtype);
  if (need > kMnbStaticScratchBytes) {
    // The tile GEMM uses scratch only to cut tiles along K across workgroups and runs without it otherwise, and the
    // kernels a call without a workspace falls back to need none; only the streaming kernel's staged copy of the
    // activations is indispensable.
    MnbGemmArgs probe{};
    probe.L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
    probe.M = (int64_t)M;
    probe.A = a_dev;
    probe.lda = (int64_t)lda;  // (no workspace: the kernel this call would run without one)
    if (mnb_select_kernel(probe) == kMnbKernelMid && !mnb_mid_direct(probe))
      return fail(MNB_INVALID_ARGUMENT,
                  "MnbGemmStaticScratch: this problem needs %zu bytes of scratch, the static array holds %zu; use "
                  "MnbGemm with a workspace of MnbGemmWorkspaceSize bytes",
                  need, kMnbStaticScratchBytes);
    need = 0;
  }
  void* ws = nullptr;
  if (need > 0)
    if (int rc = static_scratch_address(&ws)) return rc;
  // The kernels that use the scratch write every byte they later read (the staging pass covers the whole operand
  // copy, padding included), so nothing of an earlier call's contents has to be cleared.
  return gemm_checked("MnbGemmStaticScratch", M, N, K, bits, block_size, has_zero_points, a_dtype, a_dev, lda,
                      packed_dev, bias_dev, c_dev, ldc, ws, need, stream);
}

size_t MnbGemmUnpackedWorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points,
                                    int a_dtype) {
  const size_t pack = MnbPackQuantBDataSize(N, K, bits, block_size, has_zero_points, a_dtype);
  if (pack == 0) return 0;
  return pack + MnbGemmWorkspaceSize(M, N, K, bits, block_size, has_zero_points, a_dtype);
}

int MnbGemmUnpacked(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, const void* a_dev, size_t lda,
                    const void* b_dev, const void* scales_dev, const void* zero_points_dev, const void* bias_dev,
                    void* c_dev, size_t ldc, void* workspace_dev, size_t workspace_bytes, void* stream) {
  if (int rc = check_config("MnbGemmUnpacked", bits, block_size, a_dtype)) return rc;
  if (M == 0 || N == 0) return MNB_OK;
  const int has_zp = zero_points_dev != nullptr;
  const size_t pack = MnbPackQuantBDataSize(N, K, bits, block_size, has_zp, a_dtype);
  if (!workspace_dev || workspace_bytes < pack)
    return fail(MNB_INVALID_ARGUMENT, "MnbGemmUnpacked: workspace of %zu bytes needed, %zu given", pack,
                workspace_dev ? workspace_bytes : (size_t)0);
  if (int rc = MnbPackQuantBData(N, K, bits, block_size, a_dtype, b_dev, scales_dev, zero_points_dev, workspace_dev,
                                 stream))
    return rc;
  return MnbGemm(M, N, K, bits, block_size, has_zp, a_dtype, a_dev, lda, workspace_dev, bias_dev, c_dev, ldc,
                 static_cast<char*>(workspace_dev) + pack, workspace_bytes - pack, stream);
}

// ---------------------------------------------------------------------------------------- fused projections
}  // extern "C"

namespace {

size_t round256(size_t v) { return (v + 255) / 256 * 256; }
size_t elem_size(int dtype) { return dtype == kMnbDtypeFloat16 ? 2 : 4; }

// bytes of [normalised A][plain product over the packed columns][workspace of the GEMM kernel]
struct FusedWorkspace {
  size_t a_norm, tmp, inner;
  size_t total() const { return a_norm + tmp + inner; }
};

// true when every output of the operator is a multiple of 8 columns wide (the tile GEMM's 16-byte stores)
bool widths_allow_vector_stores(const MnbFusedLayout& F) {
  for (int i = 0; i < F.map.nsrc; ++i)
    if (F.map.n[i] % 8 != 0) return false;
  return true;
}

FusedWorkspace fused_workspace(const MnbFusedLayout& F, size_t M, int has_norm) {
  FusedWorkspace w{};
  const MnbLayout& L = F.L;
  w.a_norm = has_norm ? round256(M * (size_t)L.K * elem_size(L.dtype)) : 0;
  w.inner = MnbGemmWorkspaceSize(M, (size_t)L.N, (size_t)L.K, L.bits, L.bs, 0, L.dtype);
  if (L.dtype == kMnbDtypeFloat16) {
    // fp16: the decode and streaming kernels write the operator's outputs themselves, and so does the tile GEMM when
    // the outputs allow 16-byte stores.  Where the shape selects the tile GEMM, the streaming kernel's scratch is
    // reserved as well: it takes over when the caller's pointers turn out not to be aligned.
    // (The shape alone decides: MnbGemmWorkspaceSize is non-zero for the tile GEMM too, when its plan cuts tiles
    // along K, so its value says nothing about which kernel runs.)
    const bool tile_gemm = M > 16 && mnb_prefer_gemm256(L, (int64_t)M);
    if (tile_gemm && widths_allow_vector_stores(F)) {
      const size_t mid = mnb_mid_workspace_bytes(L, (int64_t)M);
      if (w.inner < mid) w.inner = mid;
    }
    w.tmp = (tile_gemm && !widths_allow_vector_stores(F)) ? round256(M * (size_t)L.N * elem_size(L.dtype)) : 0;
  } else {
    w.tmp = round256(M * (size_t)L.N * elem_size(L.dtype));
  }
  return w;
}

int check_norm(const char* fn, const MnbNormPrologue* norm, size_t K) {
  if (!norm) return MNB_OK;
  if (!norm->norm_scale_dev) {
    if (norm->skip_dev || norm->skip_sum_dev)
      return fail(MNB_INVALID_ARGUMENT, "%s: norm_scale input must be present when skip input is provided", fn);
    return MNB_OK;
  }
  if (norm->skip_dev && norm->ld_skip < K) return fail(MNB_INVALID_ARGUMENT, "%s: ld_skip (%zu) < K (%zu)", fn, norm->ld_skip, K);
  if (norm->skip_sum_dev && !norm->skip_dev)
    return fail(MNB_INVALID_ARGUMENT, "%s: skip input must be present when input_skip_bias_sum output is requested", fn);
  if (norm->skip_sum_dev && norm->ld_skip_sum < K)
    return fail(MNB_INVALID_ARGUMENT, "%s: ld_skip_sum (%zu) < K (%zu)", fn, norm->ld_skip_sum, K);
  if (!(norm->epsilon >= 0.f)) return fail(MNB_INVALID_ARGUMENT, "%s: epsilon must not be negative", fn);
  return MNB_OK;
}

hipError_t run_norm(const MnbNormPrologue* n, const void* a, size_t lda, void* a_norm, size_t M, size_t K, int dtype,
                    hipStream_t s) {
  return mnb_launch_rmsnorm(a_norm, n->skip_sum_dev, (int64_t)n->ld_skip_sum, a, (int64_t)lda, n->skip_dev,
                            (int64_t)n->ld_skip, (int64_t)n->skip_rows, n->norm_scale_dev, n->epsilon, (int64_t)M,
                            (int64_t)K, dtype, s);
}

// One GEMM over the packed matrices of F, outputs as epi describes.
int fused_gemm(const char* fn, const MnbFusedLayout& F, size_t M, const void* a_dev, size_t lda,
               const MnbNormPrologue* norm, const void* packed_dev, MnbEpilogue epi, void* workspace_dev,
               size_t workspace_bytes, hipStream_t s) {
  const MnbLayout& L = F.L;
  const bool has_norm = norm && norm->norm_scale_dev;
  if (int rc = check_norm(fn, norm, (size_t)L.K)) return rc;
  if (lda < (size_t)L.K) return fail(MNB_INVALID_ARGUMENT, "%s: lda (%zu) < K (%lld)", fn, lda, (long long)L.K);
  if (M > 0x7fffffff || L.N > 0x7fffffff || L.K > 0x7fffffff)
    return fail(MNB_INVALID_ARGUMENT, "%s: M, N and K must fit in 31 bits", fn);
  if (!workspace_dev) workspace_bytes = 0;
  if (reinterpret_cast<uintptr_t>(workspace_dev) % 256 != 0)
    return fail(MNB_INVALID_ARGUMENT, "%s: the workspace must be 256-byte aligned", fn);
  const FusedWorkspace w = fused_workspace(F, M, has_norm);
  if (workspace_bytes < w.total())
    return fail(MNB_INVALID_ARGUMENT, "%s: workspace of %zu bytes needed, %zu given", fn, w.total(), workspace_bytes);
  char* ws = static_cast<char*>(workspace_dev);
  const void* act = a_dev;
  size_t ld_act = lda;
  if (has_norm) {
    hipError_t e = run_norm(norm, a_dev, lda, ws, M, (size_t)L.K, L.dtype, s);
    if (e != hipSuccess) return hip_fail(e, fn);
    act = ws;
    ld_act = (size_t)L.K;
  }
  MnbGemmArgs a{};
  a.L = L;
  a.M = (int64_t)M;
  a.A = act;
  a.lda = (int64_t)ld_act;
  a.packed = packed_dev;
  a.bias = static_cast<const char*>(packed_dev) + F.bias_off;
  a.workspace = w.inner ? ws + w.a_norm + w.tmp : nullptr;
  a.workspace_bytes = w.inner ? workspace_bytes - w.a_norm - w.tmp : 0;
  MnbKernelKind k = mnb_select_kernel(a);
  if (k == kMnbKernelGemm256 && w.tmp == 0 && !mnb_gemm256_fused_ok(epi)) k = kMnbKernelMid;  // scratch reserved above
  const bool direct = k == kMnbKernelSkinny || k == kMnbKernelMid || (k == kMnbKernelGemm256 && w.tmp == 0);
  if (direct) {
    a.epi = epi;
  } else {
    // plain product over the packed columns, then the finishing pass
    if (w.tmp == 0) return fail(MNB_FAIL, "%s: no scratch for the product planned for this shape", fn);
    a.C = ws + w.a_norm;
    a.ldc = L.N;
  }
  hipError_t e;
  switch (k) {
    case kMnbKernelSkinny: e = mnb_launch_skinny(a, s); break;
    case kMnbKernelGemv: e = mnb_launch_gemv(a, s); break;
    case kMnbKernelMid: e = mnb_launch_mid(a, s); break;
    case kMnbKernelGemm256: e = mnb_launch_gemm256(a, s); break;
    case kMnbKernelGemm32: e = mnb_launch_gemm32(a, s); break;
    case kMnbKernelRows16F32: e = mnb_launch_rows16_f32(a, s); break;
    default: e = mnb_launch_gemm_generic(a, s); break;
  }
  if (e != hipSuccess) return hip_fail(e, fn);
  if (!direct) {
    e = mnb_launch_fused_finish(epi, a.C, a.ldc, (int64_t)M, L.dtype, s);
    if (e != hipSuccess) return hip_fail(e, fn);
  }
  return MNB_OK;
}

}  // namespace

extern "C" {

size_t MnbMlpPackSize(size_t N, size_t K, int bits, int block_size, int a_dtype) {
  if (!supported(bits, block_size, a_dtype) || N == 0 || K == 0) return 0;
  return (size_t)mnb_make_fused_layout(kMnbFusedMlp, (int64_t)N, 0, (int64_t)K, bits, block_size, a_dtype).total_bytes;
}

int MnbMlpPack(size_t N, size_t K, int bits, int block_size, int a_dtype, const void* gate_b_dev,
               const void* gate_scales_dev, const void* gate_bias_dev, const void* up_b_dev, const void* up_scales_dev,
               const void* up_bias_dev, void* packed_dev, void* stream) {
  if (int rc = check_config("MnbMlpPack", bits, block_size, a_dtype)) return rc;
  if (N == 0 || K == 0) return MNB_OK;
  if (!gate_b_dev || !gate_scales_dev || !up_b_dev || !up_scales_dev || !packed_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbMlpPack: B and scales of both projections and the packed buffer must not be NULL");
  if (reinterpret_cast<uintptr_t>(packed_dev) % 256 != 0)
    return fail(MNB_INVALID_ARGUMENT, "MnbMlpPack: the packed buffer must be 256-byte aligned");
  const MnbFusedLayout F = mnb_make_fused_layout(kMnbFusedMlp, (int64_t)N, 0, (int64_t)K, bits, block_size, a_dtype);
  const void* B[3] = {gate_b_dev, up_b_dev, nullptr};
  const void* S[3] = {gate_scales_dev, up_scales_dev, nullptr};
  const void* bias[3] = {gate_bias_dev, up_bias_dev, nullptr};
  hipError_t e = mnb_launch_pack_fused(F, B, S, bias, packed_dev, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbMlpPack");
}

size_t MnbMlpWorkspaceSize(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, int has_norm) {
  if (!supported(bits, block_size, a_dtype) || N == 0 || K == 0 || M == 0) return 0;
  const MnbFusedLayout F = mnb_make_fused_layout(kMnbFusedMlp, (int64_t)N, 0, (int64_t)K, bits, block_size, a_dtype);
  return fused_workspace(F, M, has_norm).total();
}

int MnbMlpGemm(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, const void* a_dev, size_t lda,
               const MnbNormPrologue* norm, const void* packed_dev, int activation, void* y_dev, size_t ldc,
               void* workspace_dev, size_t workspace_bytes, void* stream) {
  if (int rc = check_config("MnbMlpGemm", bits, block_size, a_dtype)) return rc;
  if (activation != MNB_ACTIVATION_SILU)
    return fail(MNB_INVALID_ARGUMENT, "MatMulNBitsMlp: activation %d is not supported.", activation);
  if (M == 0 || N == 0) return MNB_OK;
  if (K == 0) return fail(MNB_INVALID_ARGUMENT, "MnbMlpGemm: K must be positive");
  if (!a_dev || !packed_dev || !y_dev) return fail(MNB_INVALID_ARGUMENT, "MnbMlpGemm: A, the packed weights and Y must not be NULL");
  if (ldc < N) return fail(MNB_INVALID_ARGUMENT, "MnbMlpGemm: ldc (%zu) < N (%zu)", ldc, N);
  const MnbFusedLayout F = mnb_make_fused_layout(kMnbFusedMlp, (int64_t)N, 0, (int64_t)K, bits, block_size, a_dtype);
  MnbEpilogue epi{};
  epi.kind = kMnbFusedMlp;
  epi.n[0] = (int64_t)N;
  epi.out[0] = y_dev;
  epi.ld[0] = (int64_t)ldc;
  return fused_gemm("MnbMlpGemm", F, M, a_dev, lda, norm, packed_dev, epi, workspace_dev, workspace_bytes,
                    (hipStream_t)stream);
}

size_t MnbQkvPackSize(size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype) {
  if (!supported(bits, block_size, a_dtype) || Nq == 0 || Nkv == 0 || K == 0) return 0;
  return (size_t)mnb_make_fused_layout(kMnbFusedQkv, (int64_t)Nq, (int64_t)Nkv, (int64_t)K, bits, block_size, a_dtype)
      .total_bytes;
}

int MnbQkvPack(size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype, const void* q_b_dev,
               const void* q_scales_dev, const void* q_bias_dev, const void* k_b_dev, const void* k_scales_dev,
               const void* k_bias_dev, const void* v_b_dev, const void* v_scales_dev, const void* v_bias_dev,
               void* packed_dev, void* stream) {
  if (int rc = check_config("MnbQkvPack", bits, block_size, a_dtype)) return rc;
  if (Nq == 0 || Nkv == 0 || K == 0) return MNB_OK;
  if (!q_b_dev || !q_scales_dev || !k_b_dev || !k_scales_dev || !v_b_dev || !v_scales_dev || !packed_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbQkvPack: B and scales of the three projections and the packed buffer must not be NULL");
  if (reinterpret_cast<uintptr_t>(packed_dev) % 256 != 0)
    return fail(MNB_INVALID_ARGUMENT, "MnbQkvPack: the packed buffer must be 256-byte aligned");
  const MnbFusedLayout F =
      mnb_make_fused_layout(kMnbFusedQkv, (int64_t)Nq, (int64_t)Nkv, (int64_t)K, bits, block_size, a_dtype);
  const void* B[3] = {q_b_dev, k_b_dev, v_b_dev};
  const void* S[3] = {q_scales_dev, k_scales_dev, v_scales_dev};
  const void* bias[3] = {q_bias_dev, k_bias_dev, v_bias_dev};
  hipError_t e = mnb_launch_pack_fused(F, B, S, bias, packed_dev, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbQkvPack");
}

size_t MnbQkvWorkspaceSize(size_t M, size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype,
                           int has_norm) {
  if (!supported(bits, block_size, a_dtype) || Nq == 0 || Nkv == 0 || K == 0 || M == 0) return 0;
  const MnbFusedLayout F =
      mnb_make_fused_layout(kMnbFusedQkv, (int64_t)Nq, (int64_t)Nkv, (int64_t)K, bits, block_size, a_dtype);
  return fused_workspace(F, M, has_norm).total();
}

int MnbQkvGemm(size_t M, size_t Nq, size_t Nkv, size_t K, int bits, int block_size, int a_dtype, const void* a_dev,
               size_t lda, const MnbNormPrologue* norm, const void* packed_dev, void* q_dev, size_t ldq, void* k_dev,
               size_t ldk, void* v_dev, size_t ldv, void* workspace_dev, size_t workspace_bytes, void* stream) {
  if (int rc = check_config("MnbQkvGemm", bits, block_size, a_dtype)) return rc;
  if (M == 0) return MNB_OK;
  if (Nq == 0 || Nkv == 0 || K == 0) return fail(MNB_INVALID_ARGUMENT, "MnbQkvGemm: Nq, Nkv and K must be positive");
  if (!a_dev || !packed_dev || !q_dev || !k_dev || !v_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbQkvGemm: A, the packed weights and the three outputs must not be NULL");
  if (ldq < Nq || ldk < Nkv || ldv < Nkv)
    return fail(MNB_INVALID_ARGUMENT, "MnbQkvGemm: an output pitch is smaller than its width");
  const MnbFusedLayout F =
      mnb_make_fused_layout(kMnbFusedQkv, (int64_t)Nq, (int64_t)Nkv, (int64_t)K, bits, block_size, a_dtype);
  MnbEpilogue epi{};
  epi.kind = kMnbFusedQkv;
  void* outs[3] = {q_dev, k_dev, v_dev};
  const size_t lds[3] = {ldq, ldk, ldv};
  for (int i = 0; i < 3; ++i) {
    epi.start[i] = F.map.start[i];
    epi.n[i] = F.map.n[i];
    epi.out[i] = outs[i];
    epi.ld[i] = (int64_t)lds[i];
  }
  return fused_gemm("MnbQkvGemm", F, M, a_dev, lda, norm, packed_dev, epi, workspace_dev, workspace_bytes,
                    (hipStream_t)stream);
}

int MnbSimplifiedLayerNorm(size_t M, size_t K, int a_dtype, const void* a_dev, size_t lda, const MnbNormPrologue* norm,
                           void* a_norm_dev, void* stream) {
  if (a_dtype != MNB_DTYPE_FLOAT && a_dtype != MNB_DTYPE_FLOAT16)
    return fail(MNB_NOT_IMPLEMENTED, "MnbSimplifiedLayerNorm: element type %d has no MI355X kernel", a_dtype);
  if (M == 0 || K == 0) return MNB_OK;
  if (!norm || !norm->norm_scale_dev || !a_dev || !a_norm_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbSimplifiedLayerNorm: A, norm_scale and the output must not be NULL");
  if (int rc = check_norm("MnbSimplifiedLayerNorm", norm, K)) return rc;
  if (lda < K) return fail(MNB_INVALID_ARGUMENT, "MnbSimplifiedLayerNorm: lda (%zu) < K (%zu)", lda, K);
  hipError_t e = run_norm(norm, a_dev, lda, a_norm_dev, M, K, a_dtype, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbSimplifiedLayerNorm");
}

int MnbQuantizeBlockwise(void* b_dev, void* scales_dev, void* zero_points_dev, const void* src_dev, int block_size,
                         int bits, size_t K, size_t N, size_t leading_dimension, int a_dtype, void* stream) {
  if (int rc = check_config("MnbQuantizeBlockwise", bits, block_size, a_dtype)) return rc;
  if (N == 0 || K == 0) return MNB_OK;
  if (!b_dev || !scales_dev || !src_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbQuantizeBlockwise: B, scales and src must not be NULL");
  if (leading_dimension < N)
    return fail(MNB_INVALID_ARGUMENT, "MnbQuantizeBlockwise: leading_dimension (%zu) < N (%zu)", leading_dimension, N);
  hipError_t e = mnb_launch_quantize(b_dev, scales_dev, zero_points_dev, src_dev, (int64_t)K, (int64_t)N,
                                     (int64_t)leading_dimension, bits, block_size, a_dtype, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbQuantizeBlockwise");
}

int MnbDequantizeBlockwise(void* dst_dev, const void* b_dev, const void* scales_dev, const void* zero_points_dev,
                           int block_size, int bits, size_t K, size_t N, int a_dtype, void* stream) {
  if (int rc = check_config("MnbDequantizeBlockwise", bits, block_size, a_dtype)) return rc;
  if (N == 0 || K == 0) return MNB_OK;
  if (!dst_dev || !b_dev || !scales_dev)
    return fail(MNB_INVALID_ARGUMENT, "MnbDequantizeBlockwise: dst, B and scales must not be NULL");
  hipError_t e = mnb_launch_dequant_canonical(dst_dev, b_dev, scales_dev, zero_points_dev, (int64_t)N, (int64_t)K,
                                              bits, block_size, a_dtype, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbDequantizeBlockwise");
}

int MnbDequantizePacked(void* dst_dev, const void* packed_dev, size_t N, size_t K, int bits, int block_size,
                        int has_zero_points, int a_dtype, void* stream) {
  if (int rc = check_config("MnbDequantizePacked", bits, block_size, a_dtype)) return rc;
  if (N == 0 || K == 0) return MNB_OK;
  if (!dst_dev || !packed_dev) return fail(MNB_INVALID_ARGUMENT, "MnbDequantizePacked: dst and packed must not be NULL");
  MnbLayout L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
  hipError_t e = mnb_launch_dequant_packed(dst_dev, packed_dev, L, (hipStream_t)stream);
  return e == hipSuccess ? MNB_OK : hip_fail(e, "MnbDequantizePacked");
}

const char* MnbGemmKernelNameStrided(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype, size_t lda) {
  if (!supported(bits, block_size, a_dtype) || lda < K) return "none";
  MnbGemmArgs a{};
  a.L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, 0);
  a.M = (int64_t)M;
  a.lda = (int64_t)lda;
  a.A = nullptr;  // an aligned base
  a.workspace_bytes = ~(size_t)0;  // a caller that follows MnbGemmWorkspaceSize
  const MnbKernelKind kind = mnb_select_kernel(a);
  if (kind == kMnbKernelMid && mnb_mid_shared(a)) return "mnb_mid_shared_kernel";
  return mnb_kernel_name(kind, a.L);
}

const char* MnbGemmKernelName(size_t M, size_t N, size_t K, int bits, int block_size, int a_dtype) {
  return MnbGemmKernelNameStrided(M, N, K, bits, block_size, a_dtype, (K + 7) / 8 * 8);  // the usual aligned rows
}

int MnbGemmTilePlan(size_t M, size_t N, size_t K, int bits, int block_size, int has_zero_points, int a_dtype,
                    int* tile_rows, int* tile_cols, int* parts) {
  if (tile_rows) *tile_rows = 0;
  if (tile_cols) *tile_cols = 0;
  if (parts) *parts = 0;
  if (!supported(bits, block_size, a_dtype) || M == 0 || N == 0 || K == 0) return MNB_OK;
  if (std::string(MnbGemmKernelName(M, N, K, bits, block_size, a_dtype)) != "mnb_gemm256_kernel") return MNB_OK;
  const MnbLayout L = mnb_make_layout((int64_t)N, (int64_t)K, bits, block_size, a_dtype, has_zero_points);
  const MnbGemm256Plan pl = mnb_gemm256_plan(L, (int64_t)M, true);
  const int64_t tiles = (((int64_t)M + pl.tile_rows - 1) / pl.tile_rows) * (((int64_t)N + pl.tile_cols - 1) / pl.tile_cols);
  if (tile_rows) *tile_rows = pl.tile_rows;
  if (tile_cols) *tile_cols = pl.tile_cols;
  if (parts) *parts = (int)(pl.grid / tiles);
  return MNB_OK;
}

}  // extern "C"
