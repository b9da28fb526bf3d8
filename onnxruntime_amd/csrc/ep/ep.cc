// OrtEp of the MI355X plugin EP: a kernel-registry based provider
// (include/onnxruntime/core/session/onnxruntime_ep_c_api.h:2164-2550).  GetCapability claims every node for which
// the registry holds a kernel and whose static attributes the device library supports; everything else stays with
// ONNX Runtime's CPU provider, which is what makes the library a drop-in for the MatMulNBits path and nothing else.
#include "ep_common.h"

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
  size_t num_inputs = 0;
  MI_RETURN_IF_ERROR(a.ort->Node_GetNumInputs(node, &num_inputs));
  if (num_inputs < 3) return nullptr;
  std::vector<const OrtValueInfo*> inputs(num_inputs, nullptr);
  MI_RETURN_IF_ERROR(a.ort->Node_GetInputs(node, inputs.data(), num_inputs));
  if (num_inputs > 4 && inputs[4] != nullptr) return nullptr;  // g_idx: no device kernel
  // The activation type decides the kernel family; both registered types have kernels for every (bits, block).
  *supported = MnbIsAvailable(static_cast<int>(bits), static_cast<int>(block_size), MNB_DTYPE_FLOAT16) != 0;
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
  // Compile / ReleaseNodeComputeInfos stay NULL: the provider registers kernels and never fuses subgraphs.
  return ep;
}

void DestroyEp(OrtEp* ep) { delete static_cast<Ep*>(ep); }

}  // namespace mi355x_ep
