// The one subgraph the MI355X plugin EP compiles instead of running node by node: MatMulNBits followed by an Add of
// a constant [N] vector.  ONNX Runtime's own MatMulNBitsFusion rewrites that pair into the operator's bias input, but
// is registered for its CPU and CUDA providers only (onnxruntime/core/optimizer/graph_transformer_utils.cc:343-344,459;
// the pattern itself: onnxruntime/core/optimizer/matmul_nbits_fusion.cc), so a plugin provider meets the pair
// un-fused.  GetCapability claims it with EpGraphSupportInfo_AddNodesToFuse (ep.cc); ONNX Runtime then hands the pair
// to OrtEp::Compile as one fused node whose only runtime input is the activation, because constant initializers are
// dropped from the fused node (OrtNodeFusionOptions::drop_constant_initializers,
// include/onnxruntime/core/session/onnxruntime_ep_c_api.h:268-301).  Compile packs weights, scales and zero points
// into the gfx950 layout, keeps the bias on the device, and Compute is a single GEMM launch with the bias in its
// epilogue (OrtNodeComputeInfo, onnxruntime_ep_c_api.h:303-356).
//
// Arithmetic: the accumulator receives the bias in fp32 and is narrowed once, as the operator's own bias input does
// (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:1313-1333); the un-fused pair narrows the product to
// fp16 first and adds in fp16.  ONNX Runtime's fusion makes the same trade.
#include <cstring>

#include "ep_kernel_util.h"

namespace mi355x_ep {

namespace {

struct CompiledMatMulNBitsAdd : OrtNodeComputeInfo {
  Apis apis;
  int64_t K = 0, N = 0, block_size = 0, bits = 4;
  int dtype = 0;
  bool has_zp = false;
  void* packed = nullptr;  // hipMalloc
  void* bias = nullptr;    // hipMalloc, N elements of the activation type

  ~CompiledMatMulNBitsAdd() {
    if (packed != nullptr) (void)hipFree(packed);
    if (bias != nullptr) (void)hipFree(bias);
  }
};

CompiledMatMulNBitsAdd* Self(OrtNodeComputeInfo* p) { return static_cast<CompiledMatMulNBitsAdd*>(p); }

OrtStatus* ORT_API_CALL CreateStateImpl(OrtNodeComputeInfo* this_ptr, OrtNodeComputeContext* /*context*/,
                                        void** compute_state) noexcept {
  *compute_state = this_ptr;  // everything a run needs was built at Compile and is immutable afterwards
  return nullptr;
}

void ORT_API_CALL ReleaseStateImpl(OrtNodeComputeInfo*, void*) noexcept {}

OrtStatus* ORT_API_CALL ComputeImpl(OrtNodeComputeInfo* this_ptr, void* /*compute_state*/,
                                    OrtKernelContext* ctx) noexcept {
  CompiledMatMulNBitsAdd& k = *Self(this_ptr);
  const Apis& a = k.apis;
  size_t num_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInputCount(ctx, &num_inputs));
  if (num_inputs != 1) {
    return a.ort->CreateStatus(ORT_EP_FAIL, "MatMulNBits+Add: the compiled node takes the activation as its only input");
  }
  const OrtValue* x = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetInput(ctx, 0, &x));
  if (x == nullptr) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: input A is missing");
  TensorDesc ad;
  MI_RETURN_IF_ERROR(Describe(a, x, &ad));
  if (static_cast<int>(ad.type) != k.dtype) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: A and scales must have the same element type");
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

  const void* a_ptr = nullptr;
  void* y_ptr = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(x, &a_ptr));
  MI_RETURN_IF_ERROR(a.ort->GetTensorMutableData(y, &y_ptr));
  void* stream = nullptr;
  MI_RETURN_IF_ERROR(a.ort->KernelContext_GetGPUComputeStream(ctx, &stream));
  hipStream_t hs = static_cast<hipStream_t>(stream);

  const size_t Mz = static_cast<size_t>(M), Nz = static_cast<size_t>(k.N), Kz = static_cast<size_t>(k.K);
  const int bits = static_cast<int>(k.bits), bs = static_cast<int>(k.block_size);
  const size_t ws_bytes = MnbGemmWorkspaceSize(Mz, Nz, Kz, bits, bs, k.has_zp, k.dtype);
  CallScratch ws;  // per call: concurrent runs never share it
  MI_RETURN_IF_ERROR(ws.Acquire(a, ctx, y, ws_bytes, hs));
  KernelTimer timer(hs, "MatMulNBits+Add", MnbGemmKernelName(Mz, Nz, Kz, bits, bs, k.dtype), M, k.N, k.K);
  const int rc = MnbGemm(Mz, Nz, Kz, bits, bs, k.has_zp, k.dtype, a_ptr, Kz, k.packed, k.bias, y_ptr, Nz, ws.get(),
                         ws_bytes, stream);
  const hipError_t free_err = ws.Release();
  MI_RETURN_IF_ERROR(StatusFromMnb(a, rc));
  MI_RETURN_IF_HIP(a, free_err);
  return nullptr;
}

OrtStatus* InitializerOf(const Apis& a, const OrtValueInfo* info, const char* what, const OrtValue** value) {
  *value = nullptr;
  if (info == nullptr) return nullptr;
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetInitializerValue(info, value));
  if (*value == nullptr) {
    const std::string msg = std::string("MatMulNBits+Add: ") + what + " is not a constant initializer";
    return a.ort->CreateStatus(ORT_EP_FAIL, msg.c_str());
  }
  return nullptr;
}

OrtStatus* CompileOne(const Apis& a, const OrtGraph* graph, std::unique_ptr<CompiledMatMulNBitsAdd>* out) {
  size_t num_nodes = 0;
  MI_RETURN_IF_ERROR(a.ort->Graph_GetNumNodes(graph, &num_nodes));
  if (num_nodes != 2) return a.ort->CreateStatus(ORT_EP_FAIL, "MI355X EP compiles MatMulNBits+Add pairs only");
  const OrtNode* nodes[2] = {nullptr, nullptr};
  MI_RETURN_IF_ERROR(a.ort->Graph_GetNodes(graph, nodes, 2));
  const OrtNode* mm = nullptr;
  const OrtNode* add = nullptr;
  for (const OrtNode* n : nodes) {
    const char* op = nullptr;
    MI_RETURN_IF_ERROR(a.ort->Node_GetOperatorType(n, &op));
    if (std::strcmp(op, "MatMulNBits") == 0) mm = n;
    if (std::strcmp(op, "Add") == 0) add = n;
  }
  if (mm == nullptr || add == nullptr) {
    return a.ort->CreateStatus(ORT_EP_FAIL, "MI355X EP compiles MatMulNBits+Add pairs only");
  }

  auto k = std::make_unique<CompiledMatMulNBitsAdd>();
  k->apis = a;
  bool found = false;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "K", &k->K, &found));
  if (!found) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: attribute K is required");
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "N", &k->N, &found));
  if (!found) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: attribute N is required");
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "block_size", &k->block_size, &found));
  if (!found) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: attribute block_size is required");
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "bits", &k->bits, &found));
  if (!found) k->bits = 4;

  size_t num_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->Node_GetNumInputs(mm, &num_inputs));
  std::vector<const OrtValueInfo*> in(num_inputs, nullptr);
  MI_RETURN_IF_ERROR(a.ort->Node_GetInputs(mm, in.data(), num_inputs));
  if (num_inputs < 3) return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits: A, B and scales are required");
  const OrtValue* b = nullptr;
  const OrtValue* scales = nullptr;
  const OrtValue* zp = nullptr;
  MI_RETURN_IF_ERROR(InitializerOf(a, in[1], "B", &b));
  MI_RETURN_IF_ERROR(InitializerOf(a, in[2], "scales", &scales));
  if (num_inputs > 3) MI_RETURN_IF_ERROR(InitializerOf(a, in[3], "zero_points", &zp));

  // the Add input that is not the product
  const OrtValueInfo* y_info = nullptr;
  MI_RETURN_IF_ERROR(a.ort->Node_GetOutputs(mm, &y_info, 1));
  const char* y_name = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetValueInfoName(y_info, &y_name));
  const OrtValueInfo* add_in[2] = {nullptr, nullptr};
  MI_RETURN_IF_ERROR(a.ort->Node_GetInputs(add, add_in, 2));
  const OrtValueInfo* bias_info = nullptr;
  for (int i = 0; i < 2; ++i) {
    const char* name = nullptr;
    if (add_in[i] == nullptr) continue;
    MI_RETURN_IF_ERROR(a.ort->GetValueInfoName(add_in[i], &name));
    if (std::strcmp(name, y_name) != 0) bias_info = add_in[i];
  }
  const OrtValue* bias = nullptr;
  MI_RETURN_IF_ERROR(InitializerOf(a, bias_info, "the Add operand", &bias));
  if (bias == nullptr) return a.ort->CreateStatus(ORT_EP_FAIL, "MatMulNBits+Add: Add does not consume the product");

  TensorDesc b_desc, s_desc, z_desc, bias_desc;
  MI_RETURN_IF_ERROR(Describe(a, b, &b_desc));
  MI_RETURN_IF_ERROR(Describe(a, scales, &s_desc));
  if (zp != nullptr) MI_RETURN_IF_ERROR(Describe(a, zp, &z_desc));
  MI_RETURN_IF_ERROR(Describe(a, bias, &bias_desc));
  k->dtype = static_cast<int>(s_desc.type);
  k->has_zp = zp != nullptr;
  const int bits = static_cast<int>(k->bits), bs = static_cast<int>(k->block_size);
  if (!MnbIsAvailable(bits, bs, k->dtype)) {
    return a.ort->CreateStatus(ORT_NOT_IMPLEMENTED, "MatMulNBits: configuration has no MI355X kernel");
  }
  if (bias_desc.type != s_desc.type) {
    return a.ort->CreateStatus(ORT_INVALID_ARGUMENT, "MatMulNBits+Add: the Add operand must have the activation type");
  }
  MnbTensorInfo bi = ToMnb(&b_desc), si = ToMnb(&s_desc), zi = ToMnb(zp != nullptr ? &z_desc : nullptr),
                none = ToMnb(nullptr), biasi = ToMnb(&bias_desc);
  MI_RETURN_IF_ERROR(StatusFromMnb(a, MnbCheckInputs(&bi, &si, &zi, &none, &biasi, k->N, k->K, k->block_size, k->bits)));

  const size_t Nz = static_cast<size_t>(k->N), Kz = static_cast<size_t>(k->K);
  const size_t bytes = MnbPackQuantBDataSize(Nz, Kz, bits, bs, k->has_zp, k->dtype);
  if (bytes == 0) return a.ort->CreateStatus(ORT_NOT_IMPLEMENTED, "MatMulNBits: configuration has no MI355X kernel");
  DeviceView b_dev, s_dev, z_dev;
  MI_RETURN_IF_ERROR(b_dev.Init(a, b));
  MI_RETURN_IF_ERROR(s_dev.Init(a, scales));
  if (zp != nullptr) MI_RETURN_IF_ERROR(z_dev.Init(a, zp));
  MI_RETURN_IF_HIP(a, hipMalloc(&k->packed, bytes));
  MI_RETURN_IF_ERROR(StatusFromMnb(a, MnbPackQuantBData(Nz, Kz, bits, bs, k->dtype, b_dev.get(), s_dev.get(), z_dev.get(),
                                                        k->packed, /*stream*/ nullptr)));
  const void* bias_ptr = nullptr;
  size_t bias_bytes = 0;
  MI_RETURN_IF_ERROR(a.ort->GetTensorData(bias, &bias_ptr));
  MI_RETURN_IF_ERROR(a.ort->GetTensorSizeInBytes(bias, &bias_bytes));
  if (bias_bytes > 0) {
    MI_RETURN_IF_HIP(a, hipMalloc(&k->bias, bias_bytes));
    MI_RETURN_IF_HIP(a, hipMemcpy(k->bias, bias_ptr, bias_bytes, OnHost(a, bias) ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice));
  }
  MI_RETURN_IF_HIP(a, hipStreamSynchronize(nullptr));  // the temporary device copies go away with this scope

  k->ort_version_supported = ORT_API_VERSION;
  k->CreateState = CreateStateImpl;
  k->Compute = ComputeImpl;
  k->ReleaseState = ReleaseStateImpl;
  *out = std::move(k);
  return nullptr;
}

}  // namespace

OrtStatus* CompileFusedNodes(const Apis& a, const OrtGraph** graphs, const OrtNode** /*fused_nodes*/, size_t count,
                             OrtNodeComputeInfo** node_compute_infos) {
  std::vector<std::unique_ptr<CompiledMatMulNBitsAdd>> built;
  for (size_t i = 0; i < count; ++i) {
    std::unique_ptr<CompiledMatMulNBitsAdd> k;
    MI_RETURN_IF_ERROR(CompileOne(a, graphs[i], &k));  // on failure `built` frees what earlier graphs allocated
    built.push_back(std::move(k));
  }
  for (size_t i = 0; i < count; ++i) node_compute_infos[i] = built[i].release();
  return nullptr;
}

void ReleaseFusedNode(OrtNodeComputeInfo* info) { delete Self(info); }

}  // namespace mi355x_ep
