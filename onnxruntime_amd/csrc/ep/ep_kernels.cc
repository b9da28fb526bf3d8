// Kernels the MI355X plugin EP registers with ONNX Runtime
// (OrtKernelImpl, include/onnxruntime/core/session/onnxruntime_ep_c_api.h:730-862):
//   com.microsoft::MatMulNBits (opset 1, fp32 and fp16 activations)  -- the operator this provider exists for
//   MemcpyFromHost / MemcpyToHost (onnx domain)                        -- the copies ONNX Runtime inserts around nodes
//                                                                          of a provider with its own memory
// The MatMulNBits kernel mirrors contrib::MatMulNBits<T1> of the reference
// (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc): attribute checks in the constructor (:100-138),
// PrePack of B together with constant scales / zero points (:252-724), Compute = CheckInputs, output shape, early
// return on an empty output, then the packed or the unpacked route (:1513-1570).
#include "ep_kernel_util.h"

namespace mi355x_ep {

namespace {

enum InputIndex : size_t { kA = 0, kB = 1, kScales = 2, kZeroPoints = 3, kGIdx = 4, kBias = 5 };

// =========================================================================================== MatMulNBits
struct MatMulNBitsKernel : OrtKernelImpl {
  Apis apis;
  int64_t K = 0, N = 0, block_size = 0, bits = 4, accuracy_level = 0;
  // constant initializers seen at kernel creation (owned by the session; valid until they are reported packed)
  const OrtValue* const_scales = nullptr;
  const OrtValue* const_zero_points = nullptr;
  const OrtValue* const_g_idx = nullptr;  // host memory (the kernel definition asks for input 4 on the CPU)
  bool has_zp_arg = false;    // the node has a zero_points input, constant or not
  bool has_g_idx = false;
  // Inputs the reference serves through its dequantise-everything route (matmul_nbits.cc:1248-1295): a group index,
  // zero points in the activation type, and bfloat16 activations.  They run through the library's variant entry
  // points; the plan describes the transformed problem.
  bool variant = false;
  MnbVariantPlan plan{};
  // packed weights (weights + scales + zero points in the device layout)
  void* packed = nullptr;
  OrtAllocator* packed_allocator = nullptr;
  int packed_dtype = 0;
  bool packed_has_zp = false;
  // session configuration entry "ep.mi355x.int8_activations" = "1" and accuracy_level = 4: quantise A to int8
  bool int8_activations = false;
};

MatMulNBitsKernel* Self(OrtKernelImpl* p) { return static_cast<MatMulNBitsKernel*>(p); }

void ORT_API_CALL MatMulNBitsRelease(OrtKernelImpl* this_ptr) noexcept {
  MatMulNBitsKernel* k = Self(this_ptr);
  if (k->packed != nullptr) {
    if (k->packed_allocator != nullptr)
      k->packed_allocator->Free(k->packed_allocator, k->packed);
    else
      (void)hipFree(k->packed);
  }
  delete k;
}

// ---- variant route -------------------------------------------------------------------------------------------
int ZpKind(const TensorDesc* zp) {
  if (zp == nullptr) return MNB_ZP_NONE;
  return zp->type == ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8 ? MNB_ZP_UINT8 : MNB_ZP_TYPED;
}

// g_idx values in host memory: the tensor's own storage, or a copy when it lives on the device after all.
OrtStatus* HostGroupIndex(const Apis& a, const OrtValue* g_idx, std::vector<int32_t>* copy, const int32_t** out,
                          size_t* len) {
  *out = nullptr;
  *len = 0;
  if (g_idx == nullptr) return nullptr;
  TensorDesc d;
  MI_RETURN_IF_ERROR(Describe(a, g_idx, &d));
  if (d.type != ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: g_idx must be an int32 tensor");
  }
  const void* p = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(g_idx, &p));
  *len = static_cast<size_t>(d.count());
  if (OnHost(a, g_idx)) {
    *out = static_cast<const int32_t*>(p);
    return nullptr;
  }
  copy->resize(*len);
  MI_RETURN_IF_HIP(a, hipMemcpy(copy->data(), p, *len * sizeof(int32_t), hipMemcpyDeviceToHost));
  *out = copy->data();
  return nullptr;
}

// Validates the operands, plans the transformed problem and packs it into `*packed` (allocated by `alloc`).
template <typename Alloc>
OrtStatus* VariantPack(MatMulNBitsKernel& k, const OrtValue* b, const OrtValue* scales, const OrtValue* zp,
                       const OrtValue* g_idx, hipStream_t stream, Alloc alloc, MnbVariantPlan* plan, void** packed) {
  const Apis& a = k.apis;
  *packed = nullptr;
  TensorDesc b_desc, s_desc, z_desc, g_desc;
  MI_RETURN_IF_ERROR(Describe(a, b, &b_desc));
  MI_RETURN_IF_ERROR(Describe(a, scales, &s_desc));
  if (zp != nullptr) MI_RETURN_IF_ERROR(Describe(a, zp, &z_desc));
  if (g_idx != nullptr) MI_RETURN_IF_ERROR(Describe(a, g_idx, &g_desc));
  MnbTensorInfo bi = ToMnb(&b_desc), si = ToMnb(&s_desc), zi = ToMnb(zp ? &z_desc : nullptr),
                gi = ToMnb(g_idx ? &g_desc : nullptr), none = ToMnb(nullptr);
  MI_RETURN_IF_ERROR(StatusFromMnb(a, MnbCheckInputs(&bi, &si, &zi, &gi, &none, k.N, k.K, k.block_size, k.bits)));
  std::vector<int32_t> g_copy;
  const int32_t* g_host = nullptr;
  size_t g_len = 0;
  MI_RETURN_IF_ERROR(HostGroupIndex(a, g_idx, &g_copy, &g_host, &g_len));
  MI_RETURN_IF_ERROR(StatusFromMnb(
      a, MnbVariantMakePlan(static_cast<size_t>(k.N), static_cast<size_t>(k.K), static_cast<int>(k.bits),
                            static_cast<int>(k.block_size), static_cast<int>(s_desc.type),
                            ZpKind(zp ? &z_desc : nullptr), g_host, g_len, plan)));
  DeviceView b_dev, s_dev, z_dev;
  MI_RETURN_IF_ERROR(b_dev.Init(a, b));
  MI_RETURN_IF_ERROR(s_dev.Init(a, scales));
  if (zp != nullptr) MI_RETURN_IF_ERROR(z_dev.Init(a, zp));
  void* buffer = nullptr;
  MI_RETURN_IF_ERROR(alloc(static_cast<size_t>(plan->packed_bytes), &buffer));
  *packed = buffer;  // the caller frees it, also on failure below
  MI_RETURN_IF_ERROR(StatusFromMnb(a, MnbVariantPack(plan, b_dev.get(), s_dev.get(), z_dev.get(), g_host, g_len, buffer,
                                                     stream)));
  MI_RETURN_IF_HIP(a, hipStreamSynchronize(stream));  // the temporary device copies go away with this scope
  return nullptr;
}

void FreePacked(MatMulNBitsKernel& k) {
  if (k.packed == nullptr) return;
  if (k.packed_allocator != nullptr)
    k.packed_allocator->Free(k.packed_allocator, k.packed);
  else
    (void)hipFree(k.packed);
  k.packed = nullptr;
}

OrtStatus* VariantPrePack(MatMulNBitsKernel& k, const OrtValue* tensor, int input_index, OrtAllocator* allocator,
                          bool* is_packed) {
  const Apis& a = k.apis;
  if (input_index == static_cast<int>(kScales) || input_index == static_cast<int>(kZeroPoints) ||
      input_index == static_cast<int>(kGIdx)) {
    *is_packed = k.packed != nullptr;  // consumed by the B call
    return nullptr;
  }
  if (input_index != static_cast<int>(kB)) return nullptr;
  // everything the packed buffer depends on must be a constant initializer; otherwise Compute packs per call
  if (k.const_scales == nullptr) return nullptr;
  if (k.has_zp_arg && k.const_zero_points == nullptr) return nullptr;
  if (k.has_g_idx && k.const_g_idx == nullptr) return nullptr;
  OrtAllocator* owner = allocator;
  auto alloc = [&](size_t bytes, void** out) -> OrtStatus* {
    *out = allocator != nullptr ? allocator->Alloc(allocator, bytes) : nullptr;
    if (*out == nullptr) {
      owner = nullptr;
      MI_RETURN_IF_HIP(a, hipMalloc(out, bytes));
    }
    return nullptr;
  };
  void* buffer = nullptr;
  OrtStatus* st = VariantPack(k, tensor, k.const_scales, k.const_zero_points, k.const_g_idx, nullptr, alloc, &k.plan,
                              &buffer);
  k.packed = buffer;
  k.packed_allocator = owner;
  if (st != nullptr) {
    FreePacked(k);
    return st;
  }
  *is_packed = true;
  return nullptr;
}

OrtStatus* VariantCompute(MatMulNBitsKernel& k, OrtKernelContext* ctx) {
  const Apis& a = k.apis;
  size_t num_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInputCount(ctx, &num_inputs));
  const OrtValue* in[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  for (size_t i = 0; i < 6 && i < num_inputs; ++i) {
    if (k.packed != nullptr && (i == kB || i == kScales || i == kZeroPoints || i == kGIdx)) continue;
    MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInput(ctx, i, &in[i]));
  }
  if (in[kA] == nullptr) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: input A is missing");
  TensorDesc ad, bias_desc;
  MI_RETURN_IF_ERROR(Describe(a, in[kA], &ad));
  if (in[kBias] != nullptr) {
    MI_RETURN_IF_ERROR(Describe(a, in[kBias], &bias_desc));
    if (bias_desc.dims.size() != 1 || bias_desc.dims[0] != k.N) {
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "bias must be a 1D tensor with shape [N]");
    }
  }
  if (ad.dims.empty() || ad.dims.back() != k.K) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMul dimension mismatch");
  }
  std::vector<int64_t> y_dims(ad.dims.begin(), ad.dims.end() - 1);
  y_dims.push_back(k.N);
  int64_t M = 1;
  for (size_t i = 0; i + 1 < ad.dims.size(); ++i) M *= ad.dims[i];
  OrtValue* y = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetOutput(ctx, 0, y_dims.data(), y_dims.size(), &y));
  if (M == 0 || k.N == 0) return nullptr;

  void* stream = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetGPUComputeStream(ctx, &stream));
  hipStream_t hs = static_cast<hipStream_t>(stream);

  // operands fed per run (or prepacking disabled): plan and pack per call into scratch memory of the session
  CallScratch pack_scratch, gemm_scratch;
  MnbVariantPlan call_plan{};
  const MnbVariantPlan* plan = &k.plan;
  void* call_packed = nullptr;
  const void* packed = k.packed;
  if (packed == nullptr) {
    if (in[kB] == nullptr || in[kScales] == nullptr) {
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: B and scales are required when B was not prepacked");
    }
    auto alloc = [&](size_t bytes, void** out) -> OrtStatus* {
      MI_RETURN_IF_ERROR(pack_scratch.Acquire(a, ctx, y, bytes, hs));
      *out = pack_scratch.get();
      return nullptr;
    };
    MI_RETURN_IF_ERROR(VariantPack(k, in[kB], in[kScales], in[kZeroPoints], in[kGIdx], hs, alloc, &call_plan, &call_packed));
    plan = &call_plan;
    packed = call_packed;
  }
  OrtStatus* result = nullptr;
  if (static_cast<int>(ad.type) != plan->a_dtype) {
    result = a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: A and scales must have the same element type");
  } else {
    const void* a_ptr = nullptr;
    const void* bias_ptr = nullptr;
    void* y_ptr = nullptr;
    result = a.ort->GetTensorData(in[kA], &a_ptr);
    if (result == nullptr && in[kBias] != nullptr) result = a.ort->GetTensorData(in[kBias], &bias_ptr);
    if (result == nullptr) result = a.ort->GetTensorMutableData(y, &y_ptr);
    if (result == nullptr) {
      const size_t Mz = static_cast<size_t>(M);
      const size_t ws_bytes = MnbVariantGemmWorkspaceSize(plan, Mz);
      result = gemm_scratch.Acquire(a, ctx, y, ws_bytes, hs);
      if (result == nullptr) {
        KernelTimer timer(hs, "MatMulNBits", plan->has_g_idx ? "gather + MatMulNBits" : "MatMulNBits (widened)", M,
                          k.N, k.K);
        const int rc = MnbVariantGemm(plan, Mz, a_ptr, static_cast<size_t>(k.K), packed, bias_ptr, y_ptr,
                                      static_cast<size_t>(k.N), gemm_scratch.get(), ws_bytes, stream);
        result = StatusFromMnb(a, rc);
      }
    }
  }
  return result;  // (the scratch objects hand their buffers back)
}

// PrePack(B) folds the constant scales and zero points into one device buffer in the gfx950 layout, the way the
// reference folds them into its packed buffer on the B call (matmul_nbits.cc:252-330).  The later calls for scales
// and zero points then only report those inputs as consumed.
OrtStatus* ORT_API_CALL MatMulNBitsPrePack(OrtKernelImpl* this_ptr, const OrtValue* tensor, int input_index,
                                           OrtAllocator* allocator, OrtSharedPrePackedWeightCache* /*cache*/,
                                           bool* is_packed) noexcept {
  MatMulNBitsKernel& k = *Self(this_ptr);
  const Apis& a = k.apis;
  *is_packed = false;
  if (k.variant) return VariantPrePack(k, tensor, input_index, allocator, is_packed);

  if (input_index == static_cast<int>(kScales) || input_index == static_cast<int>(kZeroPoints)) {
    // consumed by the B call: ONNX Runtime may drop the initializer
    *is_packed = k.packed != nullptr;
    return nullptr;
  }
  if (input_index != static_cast<int>(kB)) return nullptr;
  // Packing needs the scales now; zero points must be constant as well, or absent.
  if (k.const_scales == nullptr) return nullptr;
  if (k.has_zp_arg && k.const_zero_points == nullptr) return nullptr;

  TensorDesc b_desc, s_desc, z_desc;
  MI_RETURN_IF_ERROR(Describe(a, tensor, &b_desc));
  MI_RETURN_IF_ERROR(Describe(a, k.const_scales, &s_desc));
  if (k.const_zero_points != nullptr) MI_RETURN_IF_ERROR(Describe(a, k.const_zero_points, &z_desc));
  if (z_desc.type != ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8 && k.const_zero_points != nullptr) return nullptr;
  const int dtype = static_cast<int>(s_desc.type);
  if (!MnbIsAvailable(static_cast<int>(k.bits), static_cast<int>(k.block_size), dtype)) return nullptr;

  MnbTensorInfo bi = ToMnb(&b_desc), si = ToMnb(&s_desc), zi = ToMnb(k.const_zero_points ? &z_desc : nullptr),
                none = ToMnb(nullptr);
  MI_RETURN_IF_ERROR(StatusFromMnb(a, MnbCheckInputs(&bi, &si, &zi, &none, &none, k.N, k.K, k.block_size, k.bits)));

  const size_t bytes = MnbPackQuantBDataSize(static_cast<size_t>(k.N), static_cast<size_t>(k.K),
                                             static_cast<int>(k.bits), static_cast<int>(k.block_size),
                                             k.const_zero_points != nullptr, dtype);
  if (bytes == 0) return nullptr;
  DeviceView b_dev, s_dev, z_dev;
  MI_RETURN_IF_ERROR(b_dev.Init(a, tensor));
  MI_RETURN_IF_ERROR(s_dev.Init(a, k.const_scales));
  if (k.const_zero_points != nullptr) MI_RETURN_IF_ERROR(z_dev.Init(a, k.const_zero_points));

  void* buffer = allocator != nullptr ? allocator->Alloc(allocator, bytes) : nullptr;
  OrtAllocator* owner = allocator;
  if (buffer == nullptr) {
    owner = nullptr;
    MI_RETURN_IF_HIP(a, hipMalloc(&buffer, bytes));
  }
  int rc = MnbPackQuantBData(static_cast<size_t>(k.N), static_cast<size_t>(k.K), static_cast<int>(k.bits),
                             static_cast<int>(k.block_size), dtype, b_dev.get(), s_dev.get(), z_dev.get(), buffer,
                             /*stream*/ nullptr);
  hipError_t sync = rc == MNB_OK ? hipStreamSynchronize(nullptr) : hipSuccess;  // inputs may be freed on return
  if (rc != MNB_OK || sync != hipSuccess) {
    if (owner != nullptr)
      owner->Free(owner, buffer);
    else
      (void)hipFree(buffer);
    if (rc != MNB_OK) return StatusFromMnb(a, rc);
    return a.ort->CreateStatus(ORT_EP_FAIL, hipGetErrorString(sync));
  }
  k.packed = buffer;
  k.packed_allocator = owner;
  k.packed_dtype = dtype;
  k.packed_has_zp = k.const_zero_points != nullptr;
  *is_packed = true;
  return nullptr;
}

OrtStatus* ORT_API_CALL MatMulNBitsCompute(OrtKernelImpl* this_ptr, OrtKernelContext* ctx) noexcept {
  MatMulNBitsKernel& k = *Self(this_ptr);
  const Apis& a = k.apis;
  if (k.variant) return VariantCompute(k, ctx);
  size_t num_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInputCount(ctx, &num_inputs));
  const OrtValue* in[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  for (size_t i = 0; i < 6 && i < num_inputs; ++i) {
    // inputs that PrePack consumed are gone from the context
    if (k.packed != nullptr && (i == kB || i == kScales || i == kZeroPoints)) continue;
    MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInput(ctx, i, &in[i]));
  }
  if (in[kA] == nullptr) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: input A is missing");

  TensorDesc d[6];
  const TensorDesc* present[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  for (size_t i = 0; i < 6; ++i) {
    if (in[i] == nullptr) continue;
    MI_RETURN_IF_ERROR(Describe(a, in[i], &d[i]));
    present[i] = &d[i];
  }
  MnbTensorInfo bi = ToMnb(present[kB]), si = ToMnb(present[kScales]), zi = ToMnb(present[kZeroPoints]),
                gi = ToMnb(present[kGIdx]), biasi = ToMnb(present[kBias]);
  if (k.packed == nullptr && present[kScales] == nullptr) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: scales are required when B was not prepacked");
  }
  // With packed weights the scales / zero points were validated at PrePack time and are no longer inputs.
  if (k.packed == nullptr) {
    MI_RETURN_IF_ERROR(StatusFromMnb(a, MnbCheckInputs(&bi, &si, &zi, &gi, &biasi, k.N, k.K, k.block_size, k.bits)));
  } else if (present[kBias] != nullptr) {
    if (d[kBias].dims.size() != 1 || d[kBias].dims[0] != k.N) {
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "bias must be a 1D tensor with shape [N]");
    }
  }
  if (present[kGIdx] != nullptr) {
    return a.ort->CreateStatus(ORT_NOT_IMPLEMENTED, "MatMulNBits with g_idx has no MI355X kernel");
  }

  const TensorDesc& ad = d[kA];
  const int dtype = static_cast<int>(ad.type);
  if (dtype != MNB_DTYPE_FLOAT && dtype != MNB_DTYPE_FLOAT16) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: A must be float or float16");
  }
  if (ad.dims.empty() || ad.dims.back() != k.K) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMul dimension mismatch");  // MatMulComputeHelper
  }
  std::vector<int64_t> y_dims(ad.dims.begin(), ad.dims.end() - 1);
  y_dims.push_back(k.N);
  int64_t M = 1;
  for (size_t i = 0; i + 1 < ad.dims.size(); ++i) M *= ad.dims[i];

  OrtValue* y = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetOutput(ctx, 0, y_dims.data(), y_dims.size(), &y));
  if (M == 0 || k.N == 0) return nullptr;  // empty output (matmul_nbits.cc:1533-1536)

  const void* a_ptr = nullptr;
  const void* bias_ptr = nullptr;
  void* y_ptr = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kA], &a_ptr));
  if (in[kBias] != nullptr) MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kBias], &bias_ptr));
  MI_RETURN_IF_ERROR(a.ort->GetTensorMutableData(y, &y_ptr));
  void* stream = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetGPUComputeStream(ctx, &stream));

  const size_t Mz = static_cast<size_t>(M), Nz = static_cast<size_t>(k.N), Kz = static_cast<size_t>(k.K);
  const int bits = static_cast<int>(k.bits), bs = static_cast<int>(k.block_size);
  if (k.packed != nullptr) {
    if (dtype != k.packed_dtype) {
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: A and scales must have the same element type");
    }
    hipStream_t gs = static_cast<hipStream_t>(stream);
    if (k.int8_activations) {
      // accuracy_level 4 with the session's consent: the reference's int8-activation arithmetic, where implemented
      const size_t ws8 = MnbGemmInt8WorkspaceSize(Mz, Nz, Kz, bits, bs, k.packed_has_zp, dtype);
      if (ws8 > 0) {
        CallScratch scratch8;
        MI_RETURN_IF_ERROR(scratch8.Acquire(a, ctx, y, ws8, gs));
        KernelTimer timer(gs, "MatMulNBits", "mnb_gemm_i8_kernel", M, k.N, k.K);
        const int rc8 = MnbGemmInt8(Mz, Nz, Kz, bits, bs, k.packed_has_zp, dtype, a_ptr, Kz, k.packed, bias_ptr, y_ptr, Nz,
                                    scratch8.get(), ws8, stream);
        const hipError_t free8 = scratch8.Release();
        MI_RETURN_IF_ERROR(StatusFromMnb(a, rc8));
        MI_RETURN_IF_HIP(a, free8);
        return nullptr;
      }
    }
    // per-call scratch: concurrent Run() calls never share it (CallScratch)
    const size_t gemm_ws = MnbGemmWorkspaceSize(Mz, Nz, Kz, bits, bs, k.packed_has_zp, dtype);
    CallScratch gemm_scratch;
    MI_RETURN_IF_ERROR(gemm_scratch.Acquire(a, ctx, y, gemm_ws, gs));
    KernelTimer timer(gs, "MatMulNBits", MnbGemmKernelName(Mz, Nz, Kz, bits, bs, dtype), M, k.N, k.K);
    const int gemm_rc = MnbGemm(Mz, Nz, Kz, bits, bs, k.packed_has_zp, dtype, a_ptr, Kz, k.packed, bias_ptr, y_ptr, Nz,
                                gemm_scratch.get(), gemm_ws, stream);
    const hipError_t gemm_free = gemm_scratch.Release();
    MI_RETURN_IF_ERROR(StatusFromMnb(a, gemm_rc));
    MI_RETURN_IF_HIP(a, gemm_free);
    return nullptr;
  }

  // B was not packed at session initialisation (prepacking disabled, or B / scales / zero points are not constant
  // initializers): pack into per-call scratch memory, then run the same kernels (matmul_nbits.cc:1184-1333).
  if (in[kB] == nullptr) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: input B is missing");
  if (static_cast<int>(d[kScales].type) != dtype) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: A and scales must have the same element type");
  }
  if (present[kZeroPoints] != nullptr && d[kZeroPoints].type != ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8) {
    return a.ort->CreateStatus(ORT_NOT_IMPLEMENTED, "MatMulNBits: only uint8 zero points have an MI355X kernel");
  }
  const void* b_ptr = nullptr;
  const void* s_ptr = nullptr;
  const void* z_ptr = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kB], &b_ptr));
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kScales], &s_ptr));
  if (in[kZeroPoints] != nullptr) MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kZeroPoints], &z_ptr));
  const size_t ws_bytes = MnbGemmUnpackedWorkspaceSize(Mz, Nz, Kz, bits, bs, z_ptr != nullptr, dtype);
  if (ws_bytes == 0) return a.ort->CreateStatus(ORT_NOT_IMPLEMENTED, "MatMulNBits: configuration has no MI355X kernel");
  hipStream_t hs = static_cast<hipStream_t>(stream);
  CallScratch ws;
  MI_RETURN_IF_ERROR(ws.Acquire(a, ctx, y, ws_bytes, hs));
  KernelTimer timer(hs, "MatMulNBits", "pack + MatMulNBits", M, k.N, k.K);
  int rc = MnbGemmUnpacked(Mz, Nz, Kz, bits, bs, dtype, a_ptr, Kz, b_ptr, s_ptr, z_ptr, bias_ptr, y_ptr, Nz, ws.get(),
                           ws_bytes, stream);
  hipError_t free_err = ws.Release();
  MI_RETURN_IF_ERROR(StatusFromMnb(a, rc));
  MI_RETURN_IF_HIP(a, free_err);
  return nullptr;
}

OrtStatus* ORT_API_CALL CreateMatMulNBits(void* state, const OrtKernelInfo* info, OrtKernelImpl** kernel_out) noexcept {
  const Apis& a = *static_cast<const Apis*>(state);
  *kernel_out = nullptr;
  std::unique_ptr<MatMulNBitsKernel> k(new (std::nothrow) MatMulNBitsKernel{});
  if (!k) return a.ort->CreateStatus(ORT_FAIL, "out of memory creating the MatMulNBits kernel");
  k->ort_version_supported = ORT_API_VERSION;
  k->flags = 0;
  k->Compute = MatMulNBitsCompute;
  k->Release = MatMulNBitsRelease;
  k->PrePackWeight = MatMulNBitsPrePack;
  k->SetSharedPrePackedWeight = nullptr;  // device buffers are never shared through the host-side cache
  k->apis = a;
  MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "K", &k->K));
  MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "N", &k->N));
  MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "block_size", &k->block_size));
  if (OrtStatus* st = a.ort->KernelInfoGetAttribute_int64(info, "bits", &k->bits)) {
    a.ort->ReleaseStatus(st);
    k->bits = 4;  // schema default
  }
  if (OrtStatus* st = a.ort->KernelInfoGetAttribute_int64(info, "accuracy_level", &k->accuracy_level)) {
    a.ort->ReleaseStatus(st);
    k->accuracy_level = 0;
  }
  if (k->accuracy_level == 4 && a.ort->KernelInfo_GetConfigEntries != nullptr) {
    // accuracy_level permits int8 activations, it does not ask for them, and the full-accuracy route is the faster
    // one here: the int8 route is taken only when the session says so
    OrtKeyValuePairs* entries = nullptr;
    if (OrtStatus* st = a.ort->KernelInfo_GetConfigEntries(info, &entries)) {
      a.ort->ReleaseStatus(st);
    } else if (entries != nullptr) {
      const char* v = a.ort->GetKeyValue(entries, "ep.mi355x.int8_activations");
      k->int8_activations = v != nullptr && v[0] == '1' && v[1] == '\0';
      a.ort->ReleaseKeyValuePairs(entries);
    }
  }
  if (k->bits != 2 && k->bits != 4 && k->bits != 8) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT,
                               "Only 2b, 4b and 8b quantization is supported for MatMulNBits op, additional bits "
                               "support is planned.");
  }
  if (k->block_size != 16 && k->block_size != 32 && k->block_size != 64 && k->block_size != 128 &&
      k->block_size != 256) {
    std::string msg = "Only block sizes 16, 32, 64, 128, and 256 are supported for MatMulNBits op, got: " +
                      std::to_string(k->block_size);
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, msg.c_str());
  }
  size_t count = 0;
  MI_RETURN_IF_ERROR(a.ort->KernelInfo_GetInputCount(info, &count));
  k->has_zp_arg = InputExists(a, info, kZeroPoints, count);
  k->has_g_idx = InputExists(a, info, kGIdx, count);
  int is_constant = 0;
  const OrtValue* value = nullptr;
  if (count > kScales) {
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetConstantInput_tensor(info, kScales, &is_constant, &value));
    if (is_constant) k->const_scales = value;
  }
  if (k->has_zp_arg) {
    is_constant = 0;
    value = nullptr;
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetConstantInput_tensor(info, kZeroPoints, &is_constant, &value));
    if (is_constant) k->const_zero_points = value;
  }
  if (k->has_g_idx) {
    is_constant = 0;
    value = nullptr;
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetConstantInput_tensor(info, kGIdx, &is_constant, &value));
    if (is_constant) k->const_g_idx = value;
  }
  // The element types are read from the constant initializers: GetCapability claims a node with typed zero points
  // or bfloat16 activations only when scales and zero points are constant.
  bool typed_zp = false;
  if (k->const_zero_points != nullptr) {
    TensorDesc z;
    MI_RETURN_IF_ERROR(Describe(a, k->const_zero_points, &z));
    typed_zp = z.type != ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8;
  }
  bool bf16 = false;
  if (k->const_scales != nullptr) {
    TensorDesc sd;
    MI_RETURN_IF_ERROR(Describe(a, k->const_scales, &sd));
    bf16 = sd.type == ONNX_TENSOR_ELEMENT_DATA_TYPE_BFLOAT16;
  }
  k->variant = k->has_g_idx || typed_zp || bf16;
  *kernel_out = k.release();
  return nullptr;
}

// =========================================================================================== Memcpy
struct MemcpyKernel : OrtKernelImpl {
  Apis apis;
};

void ORT_API_CALL MemcpyRelease(OrtKernelImpl* this_ptr) noexcept { delete static_cast<MemcpyKernel*>(this_ptr); }

OrtStatus* ORT_API_CALL MemcpyCompute(OrtKernelImpl* this_ptr, OrtKernelContext* ctx) noexcept {
  const Apis& a = static_cast<MemcpyKernel*>(this_ptr)->apis;
  const OrtValue* x = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInput(ctx, 0, &x));
  if (x == nullptr) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "Memcpy: input tensor is missing");
  TensorDesc xd;
  MI_RETURN_IF_ERROR(Describe(a, x, &xd));
  OrtValue* y = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetOutput(ctx, 0, xd.dims.data(), xd.dims.size(), &y));
  size_t bytes = 0;
  MI_RETURN_IF_ERROR(a.ort->GetTensorSizeInBytes(x, &bytes));
  if (bytes == 0) return nullptr;
  const void* src = nullptr;
  void* dst = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(x, &src));
  MI_RETURN_IF_ERROR(a.ort->GetTensorMutableData(y, &dst));
  if (src == dst) return nullptr;
  const bool src_host = OnHost(a, x), dst_host = OnHost(a, y);
  hipMemcpyKind kind = src_host ? (dst_host ? hipMemcpyHostToHost : hipMemcpyHostToDevice)
                                : (dst_host ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice);
  void* stream = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetGPUComputeStream(ctx, &stream));
  hipStream_t hs = static_cast<hipStream_t>(stream);
  MI_RETURN_IF_HIP(a, hipMemcpyAsync(dst, src, bytes, kind, hs));
  // The consumer of a MemcpyToHost output is a CPU kernel that reads the bytes as soon as this returns.
  if (dst_host) MI_RETURN_IF_HIP(a, hipStreamSynchronize(hs));
  return nullptr;
}

OrtStatus* ORT_API_CALL CreateMemcpy(void* state, const OrtKernelInfo*, OrtKernelImpl** kernel_out) noexcept {
  const Apis& a = *static_cast<const Apis*>(state);
  auto* k = new (std::nothrow) MemcpyKernel{};
  *kernel_out = k;
  if (k == nullptr) return a.ort->CreateStatus(ORT_FAIL, "out of memory creating a Memcpy kernel");
  k->ort_version_supported = ORT_API_VERSION;
  k->flags = 0;
  k->Compute = MemcpyCompute;
  k->Release = MemcpyRelease;
  k->PrePackWeight = nullptr;
  k->SetSharedPrePackedWeight = nullptr;
  k->apis = a;
  return nullptr;
}

// =========================================================================================== registration
OrtStatus* AddMatMulNBits(const Apis& a, const Apis* state, const char* ep_name, OrtKernelRegistry* registry,
                          ONNXTensorElementDataType t1) {
  DefBuilder db(a);
  MI_RETURN_IF_ERROR(a.ep->CreateKernelDefBuilder(&db.b));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetOperatorType(db.b, "MatMulNBits"));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetDomain(db.b, kMsDomain));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetSinceVersion(db.b, 1, 1));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetExecutionProvider(db.b, ep_name));
  std::vector<const OrtDataType*> types;
  MI_RETURN_IF_ERROR(TypeList(a, {t1}, &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T1", types.data(), types.size()));
  MI_RETURN_IF_ERROR(TypeList(a, {ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8}, &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T2", types.data(), types.size()));
  // zero points: packed uint8, or the activation type (the reference's "unquantized zero point" route)
  MI_RETURN_IF_ERROR(TypeList(a, {ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8, t1}, &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T3", types.data(), types.size()));
  // the group index is analysed on the host when the weights are packed
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetInputMemType(db.b, kGIdx, OrtMemTypeCPUInput));
  MI_RETURN_IF_ERROR(TypeList(a, {ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32}, &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T4", types.data(), types.size()));
  OrtKernelDef* def = nullptr;
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_Build(db.b, &def));
  OrtStatus* st = a.ep->KernelRegistry_AddKernel(registry, def, CreateMatMulNBits, const_cast<Apis*>(state));
  a.ep->ReleaseKernelDef(def);
  return st;
}

OrtStatus* AddMemcpy(const Apis& a, const Apis* state, const char* ep_name, OrtKernelRegistry* registry,
                     bool from_host) {
  DefBuilder db(a);
  MI_RETURN_IF_ERROR(a.ep->CreateKernelDefBuilder(&db.b));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetOperatorType(db.b, from_host ? "MemcpyFromHost" : "MemcpyToHost"));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetDomain(db.b, kOnnxDomain));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetSinceVersion(db.b, 1, 1));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetExecutionProvider(db.b, ep_name));
  if (from_host)
    MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetInputMemType(db.b, 0, OrtMemTypeCPUInput));
  else
    MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetOutputMemType(db.b, 0, OrtMemTypeCPUOutput));
  // Only the tensor types that can reach or leave a MatMulNBits node cross the boundary of this provider.
  std::vector<const OrtDataType*> types;
  MI_RETURN_IF_ERROR(TypeList(a,
                              {ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16,
                               ONNX_TENSOR_ELEMENT_DATA_TYPE_BFLOAT16, ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8,
                               ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32},
                              &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T", types.data(), types.size()));
  OrtKernelDef* def = nullptr;
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_Build(db.b, &def));
  OrtStatus* st = a.ep->KernelRegistry_AddKernel(registry, def, CreateMemcpy, const_cast<Apis*>(state));
  a.ep->ReleaseKernelDef(def);
  return st;
}

}  // namespace

OrtStatus* CreateKernelRegistry(const Apis& apis, const char* ep_name, OrtKernelRegistry** out) {
  *out = nullptr;
  // Kernel create functions receive this pointer as their state; it outlives every session of the process.
  static const Apis* state = new Apis(apis);
  OrtKernelRegistry* registry = nullptr;
  MI_RETURN_IF_ERROR(apis.ep->CreateKernelRegistry(&registry));
  OrtStatus* st = AddMatMulNBits(apis, state, ep_name, registry, ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT);
  if (st == nullptr) st = AddMatMulNBits(apis, state, ep_name, registry, ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16);
  if (st == nullptr) st = AddMatMulNBits(apis, state, ep_name, registry, ONNX_TENSOR_ELEMENT_DATA_TYPE_BFLOAT16);
  if (st == nullptr) st = AddFusedProjectionKernels(apis, state, ep_name, registry);
  if (st == nullptr) st = AddMemcpy(apis, state, ep_name, registry, /*from_host*/ true);
  if (st == nullptr) st = AddMemcpy(apis, state, ep_name, registry, /*from_host*/ false);
  if (st != nullptr) {
    apis.ep->ReleaseKernelRegistry(registry);
    return st;
  }
  *out = registry;
  return nullptr;
}

}  // namespace mi355x_ep
