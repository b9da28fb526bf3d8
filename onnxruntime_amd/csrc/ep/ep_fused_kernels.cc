// com.microsoft::MatMulNBitsMlp and com.microsoft::MatMulNBitsQkv for the MI355X plugin EP
// (schemas: onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3851-3975 and :3977-4090).  The reference registers
// kernels for these two operators only in its WebGPU provider
// (onnxruntime/contrib_ops/webgpu/quantization/matmul_nbits_mlp.cc:230-543, matmul_nbits_qkv.cc:150-392); this file
// mirrors their contract: attribute and input checks, optional (Skip)SimplifiedLayerNormalization of A, the
// projections, and the optional input_skip_bias_sum output.
//
// Inputs:  0 A, 1 skip (optional), 2 norm_scale (optional for Mlp), then per projection B, scales, bias (optional):
//          Mlp  3..5 gate, 6..8 up;   Qkv  3..5 q, 6..8 k, 9..11 v.
// Outputs: Mlp  0 Y, 1 input_skip_bias_sum (optional);   Qkv  0 Q, 1 K, 2 V, 3 input_skip_bias_sum (optional).
//
// PrePack folds all projections (weights, scales, biases) into one device buffer when they are constant initializers;
// otherwise Compute packs per call into stream-ordered scratch memory.
#include "ep_kernel_util.h"

namespace mi355x_ep {

namespace {

constexpr size_t kInA = 0, kInSkip = 1, kInNormScale = 2, kFirstWeight = 3, kMaxInputs = 12;

struct FusedKernel : OrtKernelImpl {
  Apis apis;
  bool is_qkv = false;
  int nproj = 2;
  int64_t K = 0, n[3] = {0, 0, 0}, bits = 4, block_size = 0, accuracy_level = 0;
  float epsilon = 1e-5f;
  size_t num_inputs = 0;
  bool exists[kMaxInputs] = {};               // the node has this input
  const OrtValue* constant[kMaxInputs] = {};  // constant initializers seen at kernel creation
  void* packed = nullptr;
  OrtAllocator* packed_allocator = nullptr;
  int packed_dtype = 0;

  const char* op() const { return is_qkv ? "MatMulNBitsQkv" : "MatMulNBitsMlp"; }
  size_t num_weight_inputs() const { return kFirstWeight + 3 * static_cast<size_t>(nproj); }
};

FusedKernel* Self(OrtKernelImpl* p) { return static_cast<FusedKernel*>(p); }

void ORT_API_CALL FusedRelease(OrtKernelImpl* this_ptr) noexcept {
  FusedKernel* k = Self(this_ptr);
  if (k->packed != nullptr) {
    if (k->packed_allocator != nullptr)
      k->packed_allocator->Free(k->packed_allocator, k->packed);
    else
      (void)hipFree(k->packed);
  }
  delete k;
}

// Shape checks of one projection, with MatMulNBits' own rules and messages (matmul_nbits_helper.h:57-106).
OrtStatus* CheckProjection(const FusedKernel& k, int p, const TensorDesc& b, const TensorDesc& s,
                           const TensorDesc* bias) {
  MnbTensorInfo bi = ToMnb(&b), si = ToMnb(&s), none = ToMnb(nullptr), biasi = ToMnb(bias);
  return StatusFromMnb(k.apis, MnbCheckInputs(&bi, &si, &none, &none, &biasi, k.n[p], k.K, k.block_size, k.bits));
}

// Packs the projections given as device pointers {B, scales, bias} x nproj into `dst`.
int PackProjections(const FusedKernel& k, int dtype, const void* const* w, void* dst, void* stream) {
  const size_t K = static_cast<size_t>(k.K);
  const int bits = static_cast<int>(k.bits), bs = static_cast<int>(k.block_size);
  if (k.is_qkv)
    return MnbQkvPack(static_cast<size_t>(k.n[0]), static_cast<size_t>(k.n[1]), K, bits, bs, dtype, w[0], w[1], w[2],
                      w[3], w[4], w[5], w[6], w[7], w[8], dst, stream);
  return MnbMlpPack(static_cast<size_t>(k.n[0]), K, bits, bs, dtype, w[0], w[1], w[2], w[3], w[4], w[5], dst, stream);
}

size_t PackBytes(const FusedKernel& k, int dtype) {
  const int bits = static_cast<int>(k.bits), bs = static_cast<int>(k.block_size);
  return k.is_qkv ? MnbQkvPackSize(static_cast<size_t>(k.n[0]), static_cast<size_t>(k.n[1]),
                                   static_cast<size_t>(k.K), bits, bs, dtype)
                  : MnbMlpPackSize(static_cast<size_t>(k.n[0]), static_cast<size_t>(k.K), bits, bs, dtype);
}

OrtStatus* ORT_API_CALL FusedPrePack(OrtKernelImpl* this_ptr, const OrtValue* tensor, int input_index,
                                     OrtAllocator* allocator, OrtSharedPrePackedWeightCache* /*cache*/,
                                     bool* is_packed) noexcept {
  FusedKernel& k = *Self(this_ptr);
  const Apis& a = k.apis;
  *is_packed = false;
  const size_t idx = static_cast<size_t>(input_index);
  if (input_index < 0 || idx < kFirstWeight || idx >= k.num_weight_inputs()) return nullptr;  // A, skip, norm_scale
  if (idx != kFirstWeight) {
    *is_packed = k.packed != nullptr;  // consumed by the call for the first B
    return nullptr;
  }
  // every weight input of every projection must be a constant initializer
  const OrtValue* w[9] = {};
  for (int p = 0; p < k.nproj; ++p) {
    for (int j = 0; j < 3; ++j) {
      const size_t i = kFirstWeight + 3 * p + j;
      const OrtValue* v = (i == kFirstWeight) ? tensor : k.constant[i];
      if (j < 2 && v == nullptr) return nullptr;                     // B or scales not constant
      if (j == 2 && k.exists[i] && v == nullptr) return nullptr;     // bias given but not constant
      w[3 * p + j] = v;
    }
  }
  TensorDesc d[9];
  for (int i = 0; i < 3 * k.nproj; ++i)
    if (w[i] != nullptr) MI_RETURN_IF_ERROR(Describe(a, w[i], &d[i]));
  const int dtype = static_cast<int>(d[1].type);
  if (!MnbIsAvailable(static_cast<int>(k.bits), static_cast<int>(k.block_size), dtype)) return nullptr;
  for (int p = 0; p < k.nproj; ++p) {
    if (static_cast<int>(d[3 * p + 1].type) != dtype || (w[3 * p + 2] != nullptr && static_cast<int>(d[3 * p + 2].type) != dtype))
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "scales and biases of all projections must have one element type");
    MI_RETURN_IF_ERROR(CheckProjection(k, p, d[3 * p], d[3 * p + 1], w[3 * p + 2] ? &d[3 * p + 2] : nullptr));
  }
  const size_t bytes = PackBytes(k, dtype);
  if (bytes == 0) return nullptr;
  DeviceView views[9];
  const void* ptrs[9] = {};
  for (int i = 0; i < 3 * k.nproj; ++i) {
    if (w[i] == nullptr) continue;
    MI_RETURN_IF_ERROR(views[i].Init(a, w[i]));
    ptrs[i] = views[i].get();
  }
  void* buffer = allocator != nullptr ? allocator->Alloc(allocator, bytes) : nullptr;
  OrtAllocator* owner = allocator;
  if (buffer == nullptr) {
    owner = nullptr;
    MI_RETURN_IF_HIP(a, hipMalloc(&buffer, bytes));
  }
  const int rc = PackProjections(k, dtype, ptrs, buffer, /*stream*/ nullptr);
  const hipError_t sync = rc == MNB_OK ? hipStreamSynchronize(nullptr) : hipSuccess;  // inputs may be freed on return
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
  *is_packed = true;
  return nullptr;
}

OrtStatus* ORT_API_CALL FusedCompute(OrtKernelImpl* this_ptr, OrtKernelContext* ctx) noexcept {
  FusedKernel& k = *Self(this_ptr);
  const Apis& a = k.apis;
  size_t num_inputs = 0, num_outputs = 0;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInputCount(ctx, &num_inputs));
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetOutputCount(ctx, &num_outputs));
  const OrtValue* in[kMaxInputs] = {};
  TensorDesc d[kMaxInputs];
  for (size_t i = 0; i < kMaxInputs && i < num_inputs; ++i) {
    if (k.packed != nullptr && i >= kFirstWeight) continue;  // consumed by PrePack
    MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInput(ctx, i, &in[i]));
    if (in[i] != nullptr) MI_RETURN_IF_ERROR(Describe(a, in[i], &d[i]));
  }
  auto invalid = [&](const std::string& msg) { return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, msg.c_str()); };
  if (in[kInA] == nullptr) return invalid(std::string(k.op()) + ": input A is missing");
  const TensorDesc& ad = d[kInA];
  const int dtype = static_cast<int>(ad.type);
  if (dtype != MNB_DTYPE_FLOAT && dtype != MNB_DTYPE_FLOAT16)
    return invalid(std::string(k.op()) + ": A must be float or float16");
  if (ad.dims.empty() || ad.dims.back() != k.K) return invalid("MatMul dimension mismatch");
  int64_t M = 1;
  for (size_t i = 0; i + 1 < ad.dims.size(); ++i) M *= ad.dims[i];

  // prologue inputs (matmul_nbits_mlp.cc:252-253, matmul_nbits_qkv.cc:46,190)
  if (in[kInSkip] != nullptr && in[kInNormScale] == nullptr)
    return invalid(std::string(k.op()) + " requires norm_scale when skip is present.");
  if (k.is_qkv && in[kInNormScale] == nullptr) return invalid("MatMulNBitsQkv: norm_scale input is missing");
  MnbNormPrologue norm{};
  if (in[kInNormScale] != nullptr) {
    if (d[kInNormScale].count() != k.K || static_cast<int>(d[kInNormScale].type) != dtype)
      return invalid("norm_scale must have shape [K].");
    MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kInNormScale], &norm.norm_scale_dev));
    norm.epsilon = k.epsilon;
    if (in[kInSkip] != nullptr) {
      const TensorDesc& sd = d[kInSkip];
      const int64_t rows = sd.dims.empty() || sd.dims.back() != k.K ? 0 : sd.count() / k.K;
      if (rows == 0 || M % rows != 0 || static_cast<int>(sd.type) != dtype)
        return invalid(std::string(k.op()) + ": skip must have the type of A and broadcast over its rows");
      MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kInSkip], &norm.skip_dev));
      norm.ld_skip = static_cast<size_t>(k.K);
      norm.skip_rows = static_cast<size_t>(rows);
    }
  }

  // outputs
  const int nout = k.is_qkv ? 3 : 1;
  void* out_ptr[3] = {nullptr, nullptr, nullptr};
  const OrtValue* first_output = nullptr;  // names the device memory the call's scratch comes from
  int64_t out_elems = 0;
  for (int o = 0; o < nout; ++o) {
    std::vector<int64_t> dims(ad.dims.begin(), ad.dims.end() - 1);
    dims.push_back(k.n[o]);
    OrtValue* y = nullptr;
    MI_RETURN_IF_ERROR(a.ort->KernelContext_GetOutput(ctx, static_cast<size_t>(o), dims.data(), dims.size(), &y));
    if (y == nullptr) return invalid(std::string(k.op()) + ": an output is missing");
    MI_RETURN_IF_ERROR(a.ort->GetTensorMutableData(y, &out_ptr[o]));
    if (o == 0) first_output = y;
    out_elems += M * k.n[o];
  }
  if (num_outputs > static_cast<size_t>(nout)) {
    OrtValue* sum = nullptr;
    MI_RETURN_IF_ERROR(a.ort->KernelContext_GetOutput(ctx, static_cast<size_t>(nout), ad.dims.data(), ad.dims.size(), &sum));
    if (sum != nullptr) {
      if (in[kInSkip] == nullptr)
        return invalid("skip input must be present when input_skip_bias_sum output is requested");
      MI_RETURN_IF_ERROR(a.ort->GetTensorMutableData(sum, &norm.skip_sum_dev));
      norm.ld_skip_sum = static_cast<size_t>(k.K);
    }
  }
  if (out_elems == 0) return nullptr;  // empty output

  const void* a_ptr = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[kInA], &a_ptr));
  void* stream = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetGPUComputeStream(ctx, &stream));
  hipStream_t hs = static_cast<hipStream_t>(stream);
  const size_t Mz = static_cast<size_t>(M), Kz = static_cast<size_t>(k.K);
  const size_t n0 = static_cast<size_t>(k.n[0]), n1 = static_cast<size_t>(k.n[1]);
  const int bits = static_cast<int>(k.bits), bs = static_cast<int>(k.block_size);
  const int has_norm = norm.norm_scale_dev != nullptr;

  // scratch: [weights packed per call, when PrePack did not run][workspace of the GEMM]
  size_t pack_bytes = 0;
  const void* w_ptr[9] = {};
  if (k.packed == nullptr) {
    for (int p = 0; p < k.nproj; ++p) {
      const size_t ib = kFirstWeight + 3 * p;
      if (in[ib] == nullptr || in[ib + 1] == nullptr)
        return invalid(std::string(k.op()) + ": B and scales of every projection are required");
      if (static_cast<int>(d[ib + 1].type) != dtype || (in[ib + 2] != nullptr && static_cast<int>(d[ib + 2].type) != dtype))
        return invalid(std::string(k.op()) + ": A, scales and biases must have the same element type");
      MI_RETURN_IF_ERROR(CheckProjection(k, p, d[ib], d[ib + 1], in[ib + 2] != nullptr ? &d[ib + 2] : nullptr));
      for (int j = 0; j < 3; ++j)
        if (in[ib + j] != nullptr) MI_RETURN_IF_ERROR(a.ort->GetTensorData(in[ib + j], &w_ptr[3 * p + j]));
    }
    pack_bytes = PackBytes(k, dtype);
    if (pack_bytes == 0)
      return a.ort->CreateStatus(ORT_NOT_IMPLEMENTED, (std::string(k.op()) + ": configuration has no MI355X kernel").c_str());
  } else if (dtype != k.packed_dtype) {
    return invalid(std::string(k.op()) + ": A and scales must have the same element type");
  }
  const size_t ws_bytes = k.is_qkv ? MnbQkvWorkspaceSize(Mz, n0, n1, Kz, bits, bs, dtype, has_norm)
                                   : MnbMlpWorkspaceSize(Mz, n0, Kz, bits, bs, dtype, has_norm);
  pack_bytes = (pack_bytes + 255) / 256 * 256;  // the workspace behind it is 256-byte aligned
  CallScratch call_scratch;
  MI_RETURN_IF_ERROR(call_scratch.Acquire(a, ctx, first_output, pack_bytes + ws_bytes, hs));
  char* scratch = static_cast<char*>(call_scratch.get());
  int rc = MNB_OK;
  const void* packed = k.packed;
  if (k.packed == nullptr) {
    rc = PackProjections(k, dtype, w_ptr, scratch, stream);
    packed = scratch;
  }
  void* ws = ws_bytes > 0 ? scratch + pack_bytes : nullptr;
  if (rc == MNB_OK) {
    KernelTimer timer(hs, k.op(), has_norm ? "norm + fused projections" : "fused projections", static_cast<int64_t>(Mz),
                      static_cast<int64_t>(k.is_qkv ? n0 + 2 * n1 : 2 * n0), static_cast<int64_t>(Kz));
    if (k.is_qkv)
      rc = MnbQkvGemm(Mz, n0, n1, Kz, bits, bs, dtype, a_ptr, Kz, has_norm ? &norm : nullptr, packed, out_ptr[0], n0,
                      out_ptr[1], n1, out_ptr[2], n1, ws, ws_bytes, stream);
    else
      rc = MnbMlpGemm(Mz, n0, Kz, bits, bs, dtype, a_ptr, Kz, has_norm ? &norm : nullptr, packed, MNB_ACTIVATION_SILU,
                      out_ptr[0], n0, ws, ws_bytes, stream);
  }
  const hipError_t free_err = call_scratch.Release();
  MI_RETURN_IF_ERROR(StatusFromMnb(a, rc));
  MI_RETURN_IF_HIP(a, free_err);
  return nullptr;
}

OrtStatus* CreateFused(const Apis& a, const OrtKernelInfo* info, bool is_qkv, OrtKernelImpl** kernel_out) {
  *kernel_out = nullptr;
  std::unique_ptr<FusedKernel> k(new (std::nothrow) FusedKernel{});
  if (!k) return a.ort->CreateStatus(ORT_FAIL, "out of memory creating a fused MatMulNBits kernel");
  k->ort_version_supported = ORT_API_VERSION;
  k->flags = 0;
  k->Compute = FusedCompute;
  k->Release = FusedRelease;
  k->PrePackWeight = FusedPrePack;
  k->SetSharedPrePackedWeight = nullptr;
  k->apis = a;
  k->is_qkv = is_qkv;
  k->nproj = is_qkv ? 3 : 2;
  MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "K", &k->K));
  if (is_qkv) {
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "Nq", &k->n[0]));
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "Nkv", &k->n[1]));
    k->n[2] = k->n[1];
  } else {
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "N", &k->n[0]));
    k->n[1] = k->n[0];
  }
  MI_RETURN_IF_ERROR(a.ort->KernelInfoGetAttribute_int64(info, "block_size", &k->block_size));
  if (OrtStatus* st = a.ort->KernelInfoGetAttribute_int64(info, "bits", &k->bits)) {
    a.ort->ReleaseStatus(st);
    k->bits = 4;  // schema default
  }
  if (OrtStatus* st = a.ort->KernelInfoGetAttribute_int64(info, "accuracy_level", &k->accuracy_level)) {
    a.ort->ReleaseStatus(st);
    k->accuracy_level = 0;
  }
  k->epsilon = is_qkv ? 1e-6f : 1e-5f;  // schema defaults
  if (OrtStatus* st = a.ort->KernelInfoGetAttribute_float(info, "epsilon", &k->epsilon)) a.ort->ReleaseStatus(st);
  if (!is_qkv) {
    char act[32] = {};
    size_t size = sizeof(act);
    if (OrtStatus* st = a.ort->KernelInfoGetAttribute_string(info, "activation", act, &size)) {
      a.ort->ReleaseStatus(st);
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBitsMlp: the activation attribute is missing or not supported.");
    }
    if (std::strcmp(act, "silu") != 0) {  // matmul_nbits_mlp.cc:24-31
      const std::string msg = std::string("MatMulNBitsMlp: activation '") + act + "' is not supported.";
      return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, msg.c_str());
    }
  }
  if (k->bits != 2 && k->bits != 4 && k->bits != 8)
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT,
                               "Only 2b, 4b and 8b quantization is supported for MatMulNBits op, additional bits "
                               "support is planned.");
  if (k->block_size != 16 && k->block_size != 32 && k->block_size != 64 && k->block_size != 128 &&
      k->block_size != 256) {
    const std::string msg = "Only block sizes 16, 32, 64, 128, and 256 are supported for MatMulNBits op, got: " +
                            std::to_string(k->block_size);
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, msg.c_str());
  }
  MI_RETURN_IF_ERROR(a.ort->KernelInfo_GetInputCount(info, &k->num_inputs));
  for (size_t i = 0; i < kMaxInputs; ++i) k->exists[i] = InputExists(a, info, i, k->num_inputs);
  for (size_t i = kFirstWeight; i < k->num_weight_inputs() && i < k->num_inputs; ++i) {
    if (!k->exists[i]) continue;
    int is_constant = 0;
    const OrtValue* value = nullptr;
    MI_RETURN_IF_ERROR(a.ort->KernelInfoGetConstantInput_tensor(info, i, &is_constant, &value));
    if (is_constant) k->constant[i] = value;
  }
  *kernel_out = k.release();
  return nullptr;
}

OrtStatus* ORT_API_CALL CreateMlp(void* state, const OrtKernelInfo* info, OrtKernelImpl** out) noexcept {
  return CreateFused(*static_cast<const Apis*>(state), info, /*is_qkv*/ false, out);
}

OrtStatus* ORT_API_CALL CreateQkv(void* state, const OrtKernelInfo* info, OrtKernelImpl** out) noexcept {
  return CreateFused(*static_cast<const Apis*>(state), info, /*is_qkv*/ true, out);
}

OrtStatus* AddOne(const Apis& a, const Apis* state, const char* ep_name, OrtKernelRegistry* registry, bool is_qkv,
                  ONNXTensorElementDataType t1) {
  DefBuilder db(a);
  MI_RETURN_IF_ERROR(a.ep->CreateKernelDefBuilder(&db.b));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetOperatorType(db.b, is_qkv ? "MatMulNBitsQkv" : "MatMulNBitsMlp"));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetDomain(db.b, kMsDomain));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetSinceVersion(db.b, 1, 1));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_SetExecutionProvider(db.b, ep_name));
  std::vector<const OrtDataType*> types;
  MI_RETURN_IF_ERROR(TypeList(a, {t1}, &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T1", types.data(), types.size()));
  MI_RETURN_IF_ERROR(TypeList(a, {ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8}, &types));
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_AddTypeConstraint(db.b, "T2", types.data(), types.size()));
  OrtKernelDef* def = nullptr;
  MI_RETURN_IF_ERROR(a.ep->KernelDefBuilder_Build(db.b, &def));
  OrtStatus* st = a.ep->KernelRegistry_AddKernel(registry, def, is_qkv ? CreateQkv : CreateMlp, const_cast<Apis*>(state));
  a.ep->ReleaseKernelDef(def);
  return st;
}

}  // namespace

OrtStatus* AddFusedProjectionKernels(const Apis& a, const Apis* state, const char* ep_name, OrtKernelRegistry* registry) {
  for (bool is_qkv : {false, true})
    for (ONNXTensorElementDataType t : {ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT, ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16})
      MI_RETURN_IF_ERROR(AddOne(a, state, ep_name, registry, is_qkv, t));
  return nullptr;
}

}  // namespace mi355x_ep
