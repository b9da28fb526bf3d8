// OrtEp of the MI355X plugin EP: a kernel-registry based provider
// (include/onnxruntime/core/session/onnxruntime_ep_c_api.h:2164-2550).  GetCapability claims every node for which
// the registry holds a kernel and whose static attributes the device library supports; everything else stays with
// ONNX Runtime's CPU provider, which is what makes the library a drop-in for the MatMulNBits path and nothing else.
#include "ep_kernel_util.h"

namespace mi355x_ep {

namespace {

struct Ep : OrtEp {
  Ep(Factory& f, const Apis& a, int dev) : OrtEp{}, factory(f), apis(a), device(dev) {}
  Factory& factory;
  const Apis apis;
  const int device;
};

Ep* Self(OrtEp* p) { return static_cast<Ep*>(p); }

const char* ORT_API_CALL GetNameImpl(const OrtEp*) noexcept { return kEpName; }

}  // namespace

// Reads an integer attribute of a node; `found` is false when the attribute is unset.
OrtStatus* ReadIntAttr(const Apis& a, const OrtNode* node, const char* name, int64_t* value, bool* found) {
  *found = false;
  const OrtOpAttr* attr = nullptr;
  OrtStatus* st = a.ort->Node_GetAttributeByName(node, name, &attr);
  if (st != nullptr) {
    // ORT_NOT_FOUND: the schema has no such attribute in this opset; treat like unset
    a.ort->ReleaseStatus(st);
    return nullptr;
  }
  if (attr == nullptr) return nullptr;
  size_t used = 0;
  MI_RETURN_IF_ERROR(a.ort->ReadOpAttr(attr, ORT_OP_ATTR_INT, value, sizeof(*value), &used));
  *found = true;
  return nullptr;
}

namespace {

bool IsConstant(const Apis& a, const OrtValueInfo* v) {
  bool c = false;
  if (v == nullptr) return false;
  if (OrtStatus* st = a.ort->ValueInfo_IsConstantInitializer(v, &c)) {
    a.ort->ReleaseStatus(st);
    return false;
  }
  return c;
}

// Element type of a tensor value; UNDEFINED when the value is not a tensor.
OrtStatus* ElementTypeOf(const Apis& a, const OrtValueInfo* v, ONNXTensorElementDataType* type) {
  *type = ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED;
  const OrtTypeInfo* info = nullptr;
  MI_RETURN_IF_ERROR(a.ort->GetValueInfoTypeInfo(v, &info));
  const OrtTensorTypeAndShapeInfo* tensor = nullptr;
  MI_RETURN_IF_ERROR(a.ort->CastTypeInfoToTensorInfo(info, &tensor));
  if (tensor == nullptr) return nullptr;
  return a.ort->GetTensorElementType(tensor, type);
}

// Static screening of one MatMulNBits node: the conditions under which the reference kernel itself would not run
// its fast path are kept on the CPU provider instead of failing at run time on the device
// (onnxruntime/contrib_ops/cpu/quantization/matmul_nbits.cc:112-139 for the attribute checks).
OrtStatus* MatMulNBitsNodeSupported(const Apis& a, const OrtNode* node, bool* supported) {
  *supported = false;
  int64_t bits = 4, block_size = 0;
  bool found = false;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, node, "bits", &bits, &found));
  if (!found) bits = 4;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, node, "block_size", &block_size, &found));
  if (!found) return nullptr;
  // weight_prepacked != 0 says that B already is in a CUDA-specific layout (1: SM80, 2: SM90 fpA_intB,
  // onnxruntime/core/graph/contrib_ops/contrib_defs.cc:3800-3805), not in the canonical one this provider repacks:
  // such a node is left to a provider that knows that layout.
  int64_t weight_prepacked = 0;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, node, "weight_prepacked", &weight_prepacked, &found));
  if (found && weight_prepacked != 0) return nullptr;
  size_t num_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->Node_GetNumInputs(node, &num_inputs));
  if (num_inputs < 3) return nullptr;
  std::vector<const OrtValueInfo*> inputs(num_inputs, nullptr);
  MI_RETURN_IF_ERROR(a.ort->Node_GetInputs(node, inputs.data(), num_inputs));
  if (inputs[0] == nullptr || inputs[1] == nullptr || inputs[2] == nullptr) return nullptr;
  // Both plain activation types have kernels for every (bits, block).
  if (!MnbIsAvailable(static_cast<int>(bits), static_cast<int>(block_size), MNB_DTYPE_FLOAT16)) return nullptr;

  // A group index, zero points in the activation type and bfloat16 activations - the inputs the reference serves
  // through its dequantise-everything route (matmul_nbits.cc:1248-1295) - are transformed once, when the weights are
  // packed, so everything the packed buffer depends on has to be a constant initializer; the limits on bits are the
  // reference's own (:1251-1252, :1258-1259).
  const OrtValueInfo* zp = num_inputs > 3 ? inputs[3] : nullptr;
  const OrtValueInfo* g_idx = num_inputs > 4 ? inputs[4] : nullptr;
  ONNXTensorElementDataType t1 = ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED;
  ONNXTensorElementDataType t3 = ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8;
  MI_RETURN_IF_ERROR(ElementTypeOf(a, inputs[0], &t1));
  if (zp != nullptr) MI_RETURN_IF_ERROR(ElementTypeOf(a, zp, &t3));
  const bool typed_zp = t3 != ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8;
  const bool bf16 = t1 == ONNX_TENSOR_ELEMENT_DATA_TYPE_BFLOAT16;
  if (g_idx != nullptr || typed_zp || bf16) {
    if (typed_zp && (t3 != t1 || (bits != 2 && bits != 4))) return nullptr;
    if (g_idx != nullptr && bits != 4) return nullptr;
    if (!IsConstant(a, inputs[1]) || !IsConstant(a, inputs[2])) return nullptr;
    if (zp != nullptr && !IsConstant(a, zp)) return nullptr;
    if (g_idx != nullptr && !IsConstant(a, g_idx)) return nullptr;
  }
  *supported = true;
  return nullptr;
}

// MatMulNBitsMlp / MatMulNBitsQkv: the same (bits, block_size) support as MatMulNBits, and the one activation the
// operator defines (onnxruntime/contrib_ops/webgpu/quantization/matmul_nbits_mlp.cc:24-31).
OrtStatus* FusedProjectionNodeSupported(const Apis& a, const OrtNode* node, bool is_mlp, bool* supported) {
  *supported = false;
  int64_t bits = 4, block_size = 0;
  bool found = false;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, node, "bits", &bits, &found));
  if (!found) bits = 4;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, node, "block_size", &block_size, &found));
  if (!found) return nullptr;
  if (is_mlp) {
    const OrtOpAttr* attr = nullptr;
    if (OrtStatus* st = a.ort->Node_GetAttributeByName(node, "activation", &attr)) {
      a.ort->ReleaseStatus(st);
      return nullptr;
    }
    if (attr == nullptr) return nullptr;
    char act[16] = {};
    size_t used = 0;
    if (OrtStatus* st = a.ort->ReadOpAttr(attr, ORT_OP_ATTR_STRING, act, sizeof(act) - 1, &used)) {
      a.ort->ReleaseStatus(st);  // longer than any supported name
      return nullptr;
    }
    if (std::strncmp(act, "silu", sizeof(act)) != 0) return nullptr;
  }
  *supported = MnbIsAvailable(static_cast<int>(bits), static_cast<int>(block_size), MNB_DTYPE_FLOAT16) != 0;
  return nullptr;
}

// MatMulNBits -> Add(constant [N]) is the pair ONNX Runtime's MatMulNBitsFusion folds into the operator's bias input,
// but only for its own CPU and CUDA providers (onnxruntime/core/optimizer/graph_transformer_utils.cc:343-344,459;
// matmul_nbits_fusion.cc).  For this provider the Add would stay behind as a CPU node with a device-to-host copy in
// front of it, so the pair is claimed as one fused node instead and compiled to a single GEMM launch with bias
// (OrtEp::Compile, ep_compile.cc).  Conditions: the MatMulNBits node has no bias of its own, constant weights /
// scales / zero points (they are packed at compile time), its output feeds this Add and nothing else, and the
// other Add input is a constant 1-D tensor of N elements in the activation type.
OrtStatus* FindBiasAdd(const Apis& a, const OrtNode* mm, const OrtNode** add_out) {
  *add_out = nullptr;
  int64_t N = 0;
  bool found = false;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "N", &N, &found));
  if (!found) return nullptr;
  size_t num_inputs = 0, num_outputs = 0;
  MI_RETURN_IF_ERROR(a.ort->Node_GetNumInputs(mm, &num_inputs));
  std::vector<const OrtValueInfo*> in(num_inputs, nullptr);
  MI_RETURN_IF_ERROR(a.ort->Node_GetInputs(mm, in.data(), num_inputs));
  if (num_inputs > 5 && in[5] != nullptr) return nullptr;               // already has a bias
  if (num_inputs > 4 && in[4] != nullptr) return nullptr;               // group index: the kernel's variant route
  if (num_inputs < 3 || !IsConstant(a, in[1]) || !IsConstant(a, in[2])) return nullptr;
  if (num_inputs > 3 && in[3] != nullptr && !IsConstant(a, in[3])) return nullptr;
  MI_RETURN_IF_ERROR(a.ort->Node_GetNumOutputs(mm, &num_outputs));
  if (num_outputs != 1) return nullptr;
  const OrtValueInfo* y = nullptr;
  MI_RETURN_IF_ERROR(a.ort->Node_GetOutputs(mm, &y, 1));
  bool is_graph_output = false;
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_IsGraphOutput(y, &is_graph_output));
  size_t consumers = 0;
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetValueNumConsumers(y, &consumers));
  if (is_graph_output || consumers != 1) return nullptr;
  const OrtNode* add = nullptr;
  int64_t index = -1;
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetValueConsumers(y, &add, &index, 1));
  if (add == nullptr || (index != 0 && index != 1)) return nullptr;
  const char* op = nullptr;
  const char* domain = nullptr;
  MI_RETURN_IF_ERROR(a.ort->Node_GetOperatorType(add, &op));
  MI_RETURN_IF_ERROR(a.ort->Node_GetDomain(add, &domain));
  if (std::strcmp(op, "Add") != 0 || (domain[0] != 0 && std::strcmp(domain, "ai.onnx") != 0)) return nullptr;
  size_t add_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->Node_GetNumInputs(add, &add_inputs));
  if (add_inputs != 2) return nullptr;
  const OrtValueInfo* ain[2] = {nullptr, nullptr};
  MI_RETURN_IF_ERROR(a.ort->Node_GetInputs(add, ain, 2));
  const OrtValueInfo* bias = ain[1 - index];
  if (!IsConstant(a, bias)) return nullptr;
  const OrtValue* bias_value = nullptr;
  const OrtValue* scales_value = nullptr;
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetInitializerValue(bias, &bias_value));
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetInitializerValue(in[2], &scales_value));
  if (bias_value == nullptr || scales_value == nullptr) return nullptr;
  TensorDesc bd, sd;
  MI_RETURN_IF_ERROR(Describe(a, bias_value, &bd));
  MI_RETURN_IF_ERROR(Describe(a, scales_value, &sd));
  if (bd.dims.size() != 1 || bd.dims[0] != N || bd.type != sd.type) return nullptr;
  // Compile must not fail on this pair: screen here everything it validates.  A pair that does not pass stays
  // un-fused, and the MatMulNBits kernel reports the problem at run time the way the reference kernel does.
  int64_t K = 0, block_size = 0, bits = 4;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "K", &K, &found));
  if (!found) return nullptr;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "block_size", &block_size, &found));
  if (!found) return nullptr;
  MI_RETURN_IF_ERROR(ReadIntAttr(a, mm, "bits", &bits, &found));
  if (!found) bits = 4;
  if (!MnbIsAvailable(static_cast<int>(bits), static_cast<int>(block_size), static_cast<int>(sd.type))) return nullptr;
  const OrtValue* b_value = nullptr;
  const OrtValue* zp_value = nullptr;
  MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetInitializerValue(in[1], &b_value));
  if (b_value == nullptr) return nullptr;
  TensorDesc b_desc, z_desc;
  MI_RETURN_IF_ERROR(Describe(a, b_value, &b_desc));
  if (num_inputs > 3 && in[3] != nullptr) {
    MI_RETURN_IF_ERROR(a.ort->ValueInfo_GetInitializerValue(in[3], &zp_value));
    if (zp_value == nullptr) return nullptr;
    MI_RETURN_IF_ERROR(Describe(a, zp_value, &z_desc));
    if (z_desc.type != ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8) return nullptr;  // typed zero points: unpacked route only
  }
  MnbTensorInfo bi = ToMnb(&b_desc), si = ToMnb(&sd), zi = ToMnb(zp_value != nullptr ? &z_desc : nullptr),
                none = ToMnb(nullptr), biasi = ToMnb(&bd);
  if (MnbCheckInputs(&bi, &si, &zi, &none, &biasi, N, K, block_size, bits) != MNB_OK) return nullptr;
  *add_out = add;
  return nullptr;
}

OrtStatus* ORT_API_CALL GetCapabilityImpl(OrtEp* this_ptr, const OrtGraph* graph,
                                          OrtEpGraphSupportInfo* graph_support_info) noexcept {
  Ep& ep = *Self(this_ptr);
  const Apis& a = ep.apis;
  size_t num_nodes = 0;
  MI_RETURN_IF_ERROR(a.ort->Graph_GetNumNodes(graph, &num_nodes));
  if (num_nodes == 0) return nullptr;
  std::vector<const OrtNode*> nodes(num_nodes, nullptr);
  MI_RETURN_IF_ERROR(a.ort->Graph_GetNodes(graph, nodes.data(), num_nodes));
  for (const OrtNode* node : nodes) {
    const OrtKernelDef* def = nullptr;
    MI_RETURN_IF_ERROR(a.ep->EpGraphSupportInfo_LookUpKernel(graph_support_info, node, &def));
    if (def == nullptr) continue;  // no registered kernel matches op, domain, version and types
    const char* op_type = nullptr;
    MI_RETURN_IF_ERROR(a.ort->Node_GetOperatorType(node, &op_type));
    if (std::strcmp(op_type, "MatMulNBits") == 0) {
      bool ok = false;
      MI_RETURN_IF_ERROR(MatMulNBitsNodeSupported(a, node, &ok));
      if (!ok) continue;
      const OrtNode* add = nullptr;
      MI_RETURN_IF_ERROR(FindBiasAdd(a, node, &add));
      if (add != nullptr) {
        const OrtNode* pair[2] = {node, add};
        OrtNodeFusionOptions options{};
        options.ort_version_supported = ORT_API_VERSION;
        options.drop_constant_initializers = true;  // everything constant is packed into device memory at Compile
        MI_RETURN_IF_ERROR(a.ep->EpGraphSupportInfo_AddNodesToFuse(graph_support_info, pair, 2, &options));
        continue;
      }
    } else if (std::strcmp(op_type, "MatMulNBitsMlp") == 0 || std::strcmp(op_type, "MatMulNBitsQkv") == 0) {
      bool ok = false;
      MI_RETURN_IF_ERROR(FusedProjectionNodeSupported(a, node, op_type[11] == 'M', &ok));
      if (!ok) continue;
    }
    MI_RETURN_IF_ERROR(a.ep->EpGraphSupportInfo_AddSingleNode(graph_support_info, node));
  }
  return nullptr;
}

OrtStatus* ORT_API_CALL GetKernelRegistryImpl(OrtEp* this_ptr, const OrtKernelRegistry** kernel_registry) noexcept {
  *kernel_registry = nullptr;
  return Self(this_ptr)->factory.GetKernelRegistry(kernel_registry);
}

OrtStatus* ORT_API_CALL CreateAllocatorImpl(OrtEp* this_ptr, const OrtMemoryInfo* memory_info,
                                            OrtAllocator** allocator) noexcept {
  Ep& ep = *Self(this_ptr);
  return ep.factory.CreateAllocator(&ep.factory, memory_info, nullptr, allocator);
}

OrtStatus* ORT_API_CALL CreateSyncStreamForDeviceImpl(OrtEp* this_ptr, const OrtMemoryDevice* memory_device,
                                                      OrtSyncStreamImpl** stream) noexcept {
  Ep& ep = *Self(this_ptr);
  return ep.factory.CreateSyncStreamForDevice(&ep.factory, memory_device, nullptr, stream);
}

OrtStatus* ORT_API_CALL IsConcurrentRunSupportedImpl(OrtEp*, bool* is_supported) noexcept {
  // Kernels keep no mutable per-call state: packed weights are read-only after session initialisation and
  // scratch memory is allocated in stream order per call.
  *is_supported = true;
  return nullptr;
}

OrtStatus* ORT_API_CALL CompileImpl(OrtEp* this_ptr, const OrtGraph** graphs, const OrtNode** fused_nodes, size_t count,
                                    OrtNodeComputeInfo** node_compute_infos, OrtNode** /*ep_context_nodes*/) noexcept {
  return CompileFusedNodes(Self(this_ptr)->apis, graphs, fused_nodes, count, node_compute_infos);
}

void ORT_API_CALL ReleaseNodeComputeInfosImpl(OrtEp*, OrtNodeComputeInfo** infos, size_t count) noexcept {
  for (size_t i = 0; i < count; ++i) ReleaseFusedNode(infos[i]);
}

OrtStatus* ORT_API_CALL CreateProfilerImpl(OrtEp* this_ptr, OrtEpProfilerImpl** profiler) noexcept {
  return CreateEpProfiler(Self(this_ptr)->apis, profiler);
}

OrtStatus* ORT_API_CALL SyncImpl(OrtEp* this_ptr) noexcept {
  Ep& ep = *Self(this_ptr);
  MI_RETURN_IF_HIP(ep.apis, hipSetDevice(ep.device));
  MI_RETURN_IF_HIP(ep.apis, hipDeviceSynchronize());
  return nullptr;
}

}  // namespace

OrtEp* CreateEp(Factory& factory, const Apis& apis, int device) {
  Ep* ep = new (std::nothrow) Ep(factory, apis, device);
  if (ep == nullptr) return nullptr;
  ep->ort_version_supported = ORT_API_VERSION;
  ep->GetName = GetNameImpl;
  ep->GetCapability = GetCapabilityImpl;
  ep->GetKernelRegistry = GetKernelRegistryImpl;
  ep->CreateAllocator = CreateAllocatorImpl;
  ep->CreateSyncStreamForDevice = CreateSyncStreamForDeviceImpl;
  ep->IsConcurrentRunSupported = IsConcurrentRunSupportedImpl;
  ep->Sync = SyncImpl;
  // the only subgraph the provider compiles is MatMulNBits + Add(bias); everything else runs registered kernels
  ep->CreateProfiler = CreateProfilerImpl;
  ep->Compile = CompileImpl;
  ep->ReleaseNodeComputeInfos = ReleaseNodeComputeInfosImpl;
  return ep;
}

void DestroyEp(OrtEp* ep) { delete static_cast<Ep*>(ep); }

}  // namespace mi355x_ep
