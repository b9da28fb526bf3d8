// Test double of the ONNX Runtime side of the plugin-EP C ABI.
//
// No ONNX Runtime binary exists in the build image, so the tests load libonnxruntime_mi355x_ep.so into this host
// instead.  It is compiled against the same public headers as the plugin (onnxruntime_c_api.h /
// onnxruntime_ep_c_api.h, found on the include path), defines the opaque Ort* types itself, fills the OrtApi /
// OrtEpApi tables with the entries the plugin uses (every other entry stays NULL, so a call the host does not model
// crashes the test instead of passing silently) and then walks a session's life the way ONNX Runtime does:
//   CreateEpFactories -> GetSupportedDevices -> CreateEp -> GetKernelRegistry -> GetCapability on a one-node graph
//   -> allocator / data transfer / stream from the factory -> initializers copied to the device -> kernel creation
//   -> PrePackWeight per constant input (packed initializers are freed) -> MemcpyFromHost -> Compute ->
//   MemcpyToHost -> release of everything.
// It is test infrastructure only; nothing in the product links to it.
#include <dlfcn.h>

#include <cstdarg>
#include <cstdio>
#include <chrono>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "onnxruntime_c_api.h"

// ------------------------------------------------------------------------------------------- opaque types
struct OrtStatus {
  OrtErrorCode code;
  std::string msg;
};
struct OrtMemoryDevice {
  OrtMemoryInfoDeviceType type;
  OrtDeviceMemoryType mem_type;
  uint32_t vendor;
  uint32_t device_id;
};
struct OrtMemoryInfo {
  std::string name;
  OrtMemoryDevice dev;
  size_t alignment;
  OrtAllocatorType alloc_type;
};
struct OrtValue {
  std::vector<int64_t> dims;
  ONNXTensorElementDataType type = ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED;
  void* data = nullptr;
  size_t bytes = 0;
  const OrtMemoryInfo* mem = nullptr;
  OrtAllocator* owner = nullptr;  // frees `data`; NULL = borrowed or malloc'ed host memory
  bool host_owned = false;
  ~OrtValue() {
    if (data == nullptr) return;
    if (owner != nullptr)
      owner->Free(owner, data);
    else if (host_owned)
      free(data);
  }
};
struct OrtTensorTypeAndShapeInfo {
  std::vector<int64_t> dims;
  ONNXTensorElementDataType type;
};
struct OrtHardwareDevice {
  OrtHardwareDeviceType type;
  uint32_t vendor_id;
  uint32_t device_id;
};
struct OrtEpDevice {
  OrtEpFactory* factory;
  const OrtHardwareDevice* hw;
  std::vector<const OrtMemoryInfo*> mem_infos;
};
struct OrtDataType {
  ONNXTensorElementDataType elem;
};
struct OrtKernelDef {
  std::string op, domain, ep;
  int start = 1, end = 1;
  std::map<std::string, std::vector<ONNXTensorElementDataType>> constraints;
  std::map<size_t, OrtMemType> input_mem, output_mem;
};
struct OrtKernelDefBuilder {
  OrtKernelDef def;
};
struct OrtKernelRegistry {
  struct Entry {
    OrtKernelDef def;
    OrtKernelCreateFunc fn;
    void* state;
  };
  std::vector<Entry> entries;
};
struct OrtOpAttr {
  std::string name;
  int64_t value;
  int kind = 0;  // 0 int, 1 float, 2 string
  float f = 0.f;
  std::string s;
};
struct OrtTypeInfo {
  OrtTensorTypeAndShapeInfo tensor;
};
struct OrtValueInfo {
  std::string name;
  OrtTypeInfo type_info = {{{}, ONNX_TENSOR_ELEMENT_DATA_TYPE_UNDEFINED}};
  const OrtValue* initializer = nullptr;  // host tensor of a constant initializer
  bool is_graph_output = false;
  std::vector<std::pair<const OrtNode*, int64_t>> consumers = {};  // (node, input index)
};
struct OrtNode {
  std::string op, domain, name;
  int since_version = 1;
  std::vector<std::unique_ptr<OrtValueInfo>> inputs;  // NULL entry = omitted optional input
  std::vector<std::unique_ptr<OrtValueInfo>> outputs = {};
  std::vector<OrtOpAttr> attrs;
  std::vector<std::string> schema_attrs;                     // attribute names the operator schema knows
  std::map<std::string, ONNXTensorElementDataType> types;    // type-constraint name -> bound element type
};
struct OrtGraph {
  std::vector<const OrtNode*> nodes;
};
struct OrtEpGraphSupportInfo {
  const OrtKernelRegistry* registry;
  std::string ep_name;
  std::vector<const OrtNode*> claimed;
  std::vector<std::vector<const OrtNode*>> fused = {};  // groups handed to EpGraphSupportInfo_AddNodesToFuse
  std::vector<bool> fused_drops_constants = {};
};
struct OrtNodeComputeContext {
  std::string node_name;
};
struct OrtProfilingEvent {
  OrtProfilingEventCategory category;
  int32_t pid, tid;
  std::string name;
  int64_t timestamp_us, duration_us;
  std::vector<std::pair<std::string, std::string>> args;
};
struct OrtProfilingEventsContainer {
  std::vector<OrtProfilingEvent> events;
};
struct OrtKernelInfo {
  const OrtNode* node;
  std::map<size_t, const OrtValue*> constants;
};
struct OrtKeyValuePairs {
  std::map<std::string, std::string> kv;
};
struct OrtSyncStream {
  OrtSyncStreamImpl* impl;
};
// What the session's allocator and the scratch calls saw during the last run on this thread (EpHostLastRunStats).
struct EpHostRunStats {
  uint64_t scratch_requests;     // KernelContext_GetScratchBuffer calls
  uint64_t scratch_served;       // ... that returned memory
  uint64_t scratch_bytes_max;    // largest request
  uint64_t allocator_requests;   // KernelContext_GetAllocator calls
  uint64_t allocators_released;  // ReleaseAllocator calls on those allocators
  uint64_t scratch_freed;        // scratch buffers handed back through such an allocator
  uint64_t ep_allocs;            // Alloc calls that reached the plugin's own OrtAllocator (arena misses)
  uint64_t arena_allocs;         // Alloc calls on the session's arena (outputs, scratch, PrePack)
  double host_us_per_compute;    // timing mode: host time of one Compute call (mean), stream kept busy
  double wall_us_per_compute;    // ... wall time per call including the final stream flush
  double device_us_per_compute;  // ... device time per call between two events on the compute stream (-1: no HIP)
  uint64_t timed_computes;
};
thread_local EpHostRunStats tl_stats{};
// 0: scratch requests are served from the arena; 1: KernelContext_GetScratchBuffer fails with a status;
// 2: it succeeds with a NULL buffer; 3: it returns memory that is only 64-byte aligned
thread_local int tl_scratch_mode = 0;

// The session's device allocator: ONNX Runtime puts an arena in front of the provider's OrtAllocator, so in steady
// state an output or a scratch buffer of a size seen before costs no call into the provider.  Modelled as exact-size
// free lists over 256-byte multiples.
struct ArenaAllocator : OrtAllocator {
  OrtAllocator* inner = nullptr;
  std::mutex mutex;
  std::map<size_t, std::vector<void*>> free_lists;
  std::map<void*, size_t> live;
  explicit ArenaAllocator(OrtAllocator* ep_allocator) : inner(ep_allocator) {
    version = ORT_API_VERSION;
    Alloc = [](OrtAllocator* self, size_t size) noexcept -> void* {
      auto* a = static_cast<ArenaAllocator*>(self);
      const size_t rounded = (size + 255) / 256 * 256;
      std::lock_guard<std::mutex> lock(a->mutex);
      ++tl_stats.arena_allocs;
      void* p = nullptr;
      auto& fl = a->free_lists[rounded];
      if (!fl.empty()) {
        p = fl.back();
        fl.pop_back();
      } else {
        ++tl_stats.ep_allocs;
        p = a->inner->Alloc(a->inner, rounded);
      }
      if (p != nullptr) a->live[p] = rounded;
      return p;
    };
    Free = [](OrtAllocator* self, void* p) noexcept {
      if (p == nullptr) return;
      auto* a = static_cast<ArenaAllocator*>(self);
      std::lock_guard<std::mutex> lock(a->mutex);
      auto it = a->live.find(p);
      if (it == a->live.end()) return;  // not ours: a protocol error the tests see as a leak of `live`
      a->free_lists[it->second].push_back(p);
      a->live.erase(it);
    };
    Info = [](const OrtAllocator* self) noexcept -> const OrtMemoryInfo* {
      auto* a = static_cast<const ArenaAllocator*>(self);
      return a->inner->Info(a->inner);
    };
    Reserve = nullptr;
    GetStats = nullptr;
    AllocOnStream = nullptr;
  }
  ~ArenaAllocator() {
    for (auto& kv : free_lists)
      for (void* p : kv.second) inner->Free(inner, p);
    for (auto& kv : live) inner->Free(inner, kv.first);
  }
};

// What KernelContext_GetAllocator hands out: a handle onto the session's arena that ReleaseAllocator deletes.
struct AllocatorHandle : OrtAllocator {
  OrtAllocator* arena = nullptr;
  explicit AllocatorHandle(OrtAllocator* a) : arena(a) {
    version = ORT_API_VERSION;
    Alloc = [](OrtAllocator* self, size_t size) noexcept -> void* {
      auto* h = static_cast<AllocatorHandle*>(self);
      return h->arena->Alloc(h->arena, size);
    };
    Free = [](OrtAllocator* self, void* p) noexcept {
      auto* h = static_cast<AllocatorHandle*>(self);
      if (p != nullptr) ++tl_stats.scratch_freed;
      h->arena->Free(h->arena, p);
    };
    Info = [](const OrtAllocator* self) noexcept -> const OrtMemoryInfo* {
      auto* h = static_cast<const AllocatorHandle*>(self);
      return h->arena->Info(h->arena);
    };
    Reserve = nullptr;
    GetStats = nullptr;
    AllocOnStream = nullptr;
  }
};

struct OrtKernelContext {
  std::vector<const OrtValue*> inputs;
  std::vector<std::unique_ptr<OrtValue>> outputs;
  std::vector<bool> output_on_host;
  OrtAllocator* device_allocator;
  const OrtMemoryInfo* cpu_mem;
  OrtSyncStream* stream;
  std::vector<bool> output_skipped = {};  // optional outputs the graph does not use: GetOutput yields NULL
};

namespace {

// configuration entries of the (one) session this host stands for
std::map<std::string, std::string>& SessionConfig() {
  static std::map<std::string, std::string> config;
  return config;
}

size_t ElemSize(ONNXTensorElementDataType t) {
  switch (t) {
    case ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT:
    case ONNX_TENSOR_ELEMENT_DATA_TYPE_INT32:
      return 4;
    case ONNX_TENSOR_ELEMENT_DATA_TYPE_FLOAT16:
    case ONNX_TENSOR_ELEMENT_DATA_TYPE_BFLOAT16:
      return 2;
    case ONNX_TENSOR_ELEMENT_DATA_TYPE_UINT8:
      return 1;
    default:
      return 0;
  }
}

size_t ByteSize(const std::vector<int64_t>& dims, ONNXTensorElementDataType t) {
  size_t n = ElemSize(t);
  for (int64_t d : dims) n *= static_cast<size_t>(d);
  return n;
}

OrtStatus* MakeStatus(OrtErrorCode code, const char* msg) { return new OrtStatus{code, msg ? msg : ""}; }

const OrtKernelRegistry::Entry* LookUp(const OrtKernelRegistry& reg, const std::string& ep, const OrtNode& node) {
  for (const auto& e : reg.entries) {
    const OrtKernelDef& d = e.def;
    if (d.op != node.op || d.domain != node.domain || d.ep != ep) continue;
    if (node.since_version < d.start || node.since_version > d.end) continue;
    bool ok = true;
    for (const auto& c : d.constraints) {
      auto it = node.types.find(c.first);
      if (it == node.types.end()) continue;  // the node does not use that formal parameter
      bool found = false;
      for (auto t : c.second) found = found || t == it->second;
      ok = ok && found;
    }
    if (ok) return &e;
  }
  return nullptr;
}

// ------------------------------------------------------------------------------------------- API tables
OrtApi g_ort{};
OrtEpApi g_ep{};
OrtDataType g_types[32];

void FillApisOnce() {
  for (int i = 0; i < 32; ++i) g_types[i].elem = static_cast<ONNXTensorElementDataType>(i);

  // ---- OrtApi
  g_ort.CreateStatus = [](OrtErrorCode code, const char* msg) noexcept -> OrtStatus* { return MakeStatus(code, msg); };
  g_ort.GetErrorCode = [](const OrtStatus* s) noexcept { return s->code; };
  g_ort.GetErrorMessage = [](const OrtStatus* s) noexcept { return s->msg.c_str(); };
  g_ort.ReleaseStatus = [](OrtStatus* s) noexcept { delete s; };
  g_ort.GetEpApi = []() noexcept -> const OrtEpApi* { return &g_ep; };
  g_ort.HardwareDevice_Type = [](const OrtHardwareDevice* d) noexcept { return d->type; };
  g_ort.HardwareDevice_VendorId = [](const OrtHardwareDevice* d) noexcept { return d->vendor_id; };
  g_ort.HardwareDevice_DeviceId = [](const OrtHardwareDevice* d) noexcept { return d->device_id; };
  g_ort.CreateMemoryInfo_V2 = [](const char* name, OrtMemoryInfoDeviceType type, uint32_t vendor, int32_t device_id,
                                 OrtDeviceMemoryType mem_type, size_t alignment, OrtAllocatorType alloc_type,
                                 OrtMemoryInfo** out) noexcept -> OrtStatus* {
    *out = new OrtMemoryInfo{name, {type, mem_type, vendor, static_cast<uint32_t>(device_id)}, alignment, alloc_type};
    return nullptr;
  };
  g_ort.ReleaseMemoryInfo = [](OrtMemoryInfo* m) noexcept { delete m; };
  g_ort.KernelInfoGetAttribute_int64 = [](const OrtKernelInfo* info, const char* name, int64_t* out) noexcept
      -> OrtStatus* {
    for (const auto& a : info->node->attrs)
      if (a.name == name) {
        *out = a.value;
        return nullptr;
      }
    return MakeStatus(ORT_FAIL, (std::string("No attribute with name:'") + name + "'is defined.").c_str());
  };
  g_ort.KernelInfoGetAttribute_float = [](const OrtKernelInfo* info, const char* name, float* out) noexcept
      -> OrtStatus* {
    for (const auto& a : info->node->attrs)
      if (a.name == name && a.kind == 1) {
        *out = a.f;
        return nullptr;
      }
    return MakeStatus(ORT_FAIL, (std::string("No attribute with name:'") + name + "'is defined.").c_str());
  };
  g_ort.KernelInfoGetAttribute_string = [](const OrtKernelInfo* info, const char* name, char* out,
                                           size_t* size) noexcept -> OrtStatus* {
    for (const auto& a : info->node->attrs)
      if (a.name == name && a.kind == 2) {
        const size_t need = a.s.size() + 1;
        if (out == nullptr) {
          *size = need;
          return nullptr;
        }
        if (*size < need) {
          *size = need;
          return MakeStatus(ORT_INVALID_ARGUMENT, "Result buffer is not large enough");
        }
        std::memcpy(out, a.s.c_str(), need);
        *size = need;
        return nullptr;
      }
    return MakeStatus(ORT_FAIL, (std::string("No attribute with name:'") + name + "'is defined.").c_str());
  };
  // session configuration entries (OrtSessionOptions::AddConfigEntry in a real session; EpHostSetSessionConfig here)
  g_ort.KernelInfo_GetConfigEntries = [](const OrtKernelInfo*, OrtKeyValuePairs** out) noexcept -> OrtStatus* {
    auto* kv = new OrtKeyValuePairs();
    kv->kv = SessionConfig();
    *out = kv;
    return nullptr;
  };
  g_ort.GetKeyValue = [](const OrtKeyValuePairs* kvps, const char* key) noexcept -> const char* {
    auto it = kvps->kv.find(key);
    return it == kvps->kv.end() ? nullptr : it->second.c_str();
  };
  g_ort.ReleaseKeyValuePairs = [](OrtKeyValuePairs* kvps) noexcept { delete kvps; };
  g_ort.KernelContext_GetOutputCount = [](const OrtKernelContext* c, size_t* out) noexcept -> OrtStatus* {
    *out = c->outputs.size();
    return nullptr;
  };
  g_ort.KernelInfo_GetInputCount = [](const OrtKernelInfo* info, size_t* out) noexcept -> OrtStatus* {
    *out = info->node->inputs.size();
    return nullptr;
  };
  g_ort.KernelInfo_GetInputName = [](const OrtKernelInfo* info, size_t index, char* out, size_t* size) noexcept
      -> OrtStatus* {
    if (index >= info->node->inputs.size())
      return MakeStatus(ORT_INVALID_ARGUMENT, "::OrtKernelInfo input index is out of bounds");
    const std::string name = info->node->inputs[index] ? info->node->inputs[index]->name : std::string();
    const size_t need = name.size() + 1;
    if (out == nullptr) {
      *size = need;
      return nullptr;
    }
    if (*size < need) {
      *size = need;
      return MakeStatus(ORT_INVALID_ARGUMENT, "Output buffer is not large enough for ::OrtKernelInfo input name");
    }
    std::memcpy(out, name.c_str(), need);
    *size = need;
    return nullptr;
  };
  g_ort.KernelInfoGetConstantInput_tensor = [](const OrtKernelInfo* info, size_t index, int* is_constant,
                                               const OrtValue** out) noexcept -> OrtStatus* {
    auto it = info->constants.find(index);
    *is_constant = it != info->constants.end();
    *out = *is_constant ? it->second : nullptr;
    return nullptr;
  };
  g_ort.GetTensorTypeAndShape = [](const OrtValue* v, OrtTensorTypeAndShapeInfo** out) noexcept -> OrtStatus* {
    *out = new OrtTensorTypeAndShapeInfo{v->dims, v->type};
    return nullptr;
  };
  g_ort.ReleaseTensorTypeAndShapeInfo = [](OrtTensorTypeAndShapeInfo* i) noexcept { delete i; };
  g_ort.GetDimensionsCount = [](const OrtTensorTypeAndShapeInfo* i, size_t* out) noexcept -> OrtStatus* {
    *out = i->dims.size();
    return nullptr;
  };
  g_ort.GetDimensions = [](const OrtTensorTypeAndShapeInfo* i, int64_t* dims, size_t n) noexcept -> OrtStatus* {
    for (size_t k = 0; k < n && k < i->dims.size(); ++k) dims[k] = i->dims[k];
    return nullptr;
  };
  g_ort.GetTensorElementType = [](const OrtTensorTypeAndShapeInfo* i, ONNXTensorElementDataType* out) noexcept
      -> OrtStatus* {
    *out = i->type;
    return nullptr;
  };
  g_ort.GetTensorData = [](const OrtValue* v, const void** out) noexcept -> OrtStatus* {
    *out = v->data;
    return nullptr;
  };
  g_ort.GetTensorMutableData = [](OrtValue* v, void** out) noexcept -> OrtStatus* {
    *out = v->data;
    return nullptr;
  };
  g_ort.GetTensorSizeInBytes = [](const OrtValue* v, size_t* out) noexcept -> OrtStatus* {
    *out = v->bytes;
    return nullptr;
  };
  g_ort.KernelContext_GetInputCount = [](const OrtKernelContext* c, size_t* out) noexcept -> OrtStatus* {
    *out = c->inputs.size();
    return nullptr;
  };
  g_ort.KernelContext_GetInput = [](const OrtKernelContext* c, size_t index, const OrtValue** out) noexcept
      -> OrtStatus* {
    *out = index < c->inputs.size() ? c->inputs[index] : nullptr;
    return nullptr;
  };
  g_ort.KernelContext_GetOutput = [](OrtKernelContext* c, size_t index, const int64_t* dims, size_t rank,
                                     OrtValue** out) noexcept -> OrtStatus* {
    if (index >= c->outputs.size()) return MakeStatus(ORT_INVALID_ARGUMENT, "output index out of range");
    if (index < c->output_skipped.size() && c->output_skipped[index]) {
      *out = nullptr;
      return nullptr;
    }
    if (!c->outputs[index]) {
      auto v = std::make_unique<OrtValue>();
      v->dims.assign(dims, dims + rank);
      v->type = c->inputs[0]->type;  // every kernel modelled here produces the type of its first input
      v->bytes = ByteSize(v->dims, v->type);
      if (c->output_on_host[index]) {
        v->mem = c->cpu_mem;
        v->data = v->bytes ? malloc(v->bytes) : nullptr;
        v->host_owned = true;
      } else {
        v->mem = c->device_allocator->Info(c->device_allocator);
        v->owner = c->device_allocator;
        v->data = v->bytes ? c->device_allocator->Alloc(c->device_allocator, v->bytes) : nullptr;
        if (v->bytes && v->data == nullptr) return MakeStatus(ORT_FAIL, "device allocation of an output failed");
      }
      c->outputs[index] = std::move(v);
    }
    *out = c->outputs[index].get();
    return nullptr;
  };
  g_ort.GetTensorMemoryInfo = [](const OrtValue* v, const OrtMemoryInfo** out) noexcept -> OrtStatus* {
    *out = v->mem;
    return nullptr;
  };
  // custom_ops.cc:219-232: the session's allocator for the device of mem_info, wrapped; the caller releases the wrapper
  g_ort.KernelContext_GetAllocator = [](const OrtKernelContext* c, const OrtMemoryInfo* mem,
                                        OrtAllocator** out) noexcept -> OrtStatus* {
    ++tl_stats.allocator_requests;
    *out = nullptr;
    const OrtMemoryInfo* dev = c->device_allocator->Info(c->device_allocator);
    if (mem == nullptr || mem->dev.type != dev->dev.type || mem->dev.device_id != dev->dev.device_id ||
        mem->dev.mem_type != dev->dev.mem_type)
      return MakeStatus(ORT_INVALID_ARGUMENT, "No requested allocator available");
    *out = new AllocatorHandle(c->device_allocator);
    return nullptr;
  };
  g_ort.ReleaseAllocator = [](OrtAllocator* a) noexcept {
    ++tl_stats.allocators_released;
    delete static_cast<AllocatorHandle*>(a);
  };
  // custom_ops.cc:901-913: a buffer from that allocator, tied to the compute stream; the caller frees it through the
  // allocator.  A request for 0 bytes yields NULL.
  g_ort.KernelContext_GetScratchBuffer = [](const OrtKernelContext* c, const OrtMemoryInfo* mem, size_t bytes,
                                            void** out) noexcept -> OrtStatus* {
    ++tl_stats.scratch_requests;
    if (bytes > tl_stats.scratch_bytes_max) tl_stats.scratch_bytes_max = bytes;
    *out = nullptr;
    if (bytes == 0) return nullptr;
    const OrtMemoryInfo* dev = c->device_allocator->Info(c->device_allocator);
    if (mem == nullptr || mem->dev.type != dev->dev.type || mem->dev.device_id != dev->dev.device_id ||
        mem->dev.mem_type != dev->dev.mem_type)
      return MakeStatus(ORT_INVALID_ARGUMENT, "No requested allocator available");
    if (tl_scratch_mode == 1) return MakeStatus(ORT_FAIL, "the host declines scratch requests (test mode)");
    if (tl_scratch_mode == 2) return nullptr;
    if (tl_scratch_mode == 3) {
      // a misaligned address inside a block the arena never sees again until the session ends (freed as not-ours)
      char* block = static_cast<char*>(c->device_allocator->Alloc(c->device_allocator, bytes + 256));
      *out = block ? block + 64 : nullptr;
      if (block) ++tl_stats.scratch_served;
      return nullptr;
    }
    *out = c->device_allocator->Alloc(c->device_allocator, bytes);
    if (*out == nullptr) return MakeStatus(ORT_FAIL, "device allocation of a scratch buffer failed");
    ++tl_stats.scratch_served;
    return nullptr;
  };
  g_ort.KernelContext_GetGPUComputeStream = [](const OrtKernelContext* c, void** out) noexcept -> OrtStatus* {
    *out = c->stream ? c->stream->impl->GetHandle(c->stream->impl) : nullptr;
    return nullptr;
  };
  g_ort.SyncStream_GetHandle = [](OrtSyncStream* s) noexcept -> void* { return s->impl->GetHandle(s->impl); };
  g_ort.Graph_GetNumNodes = [](const OrtGraph* g, size_t* n) noexcept -> OrtStatus* {
    *n = g->nodes.size();
    return nullptr;
  };
  g_ort.Graph_GetNodes = [](const OrtGraph* g, const OrtNode** nodes, size_t n) noexcept -> OrtStatus* {
    for (size_t i = 0; i < n && i < g->nodes.size(); ++i) nodes[i] = g->nodes[i];
    return nullptr;
  };
  g_ort.Node_GetOperatorType = [](const OrtNode* n, const char** out) noexcept -> OrtStatus* {
    *out = n->op.c_str();
    return nullptr;
  };
  g_ort.Node_GetDomain = [](const OrtNode* n, const char** out) noexcept -> OrtStatus* {
    *out = n->domain.c_str();
    return nullptr;
  };
  g_ort.Node_GetName = [](const OrtNode* n, const char** out) noexcept -> OrtStatus* {
    *out = n->name.c_str();
    return nullptr;
  };
  g_ort.Node_GetNumInputs = [](const OrtNode* n, size_t* out) noexcept -> OrtStatus* {
    *out = n->inputs.size();
    return nullptr;
  };
  g_ort.Node_GetInputs = [](const OrtNode* n, const OrtValueInfo** inputs, size_t count) noexcept -> OrtStatus* {
    for (size_t i = 0; i < count && i < n->inputs.size(); ++i) inputs[i] = n->inputs[i].get();
    return nullptr;
  };
  g_ort.Node_GetNumOutputs = [](const OrtNode* n, size_t* out) noexcept -> OrtStatus* {
    *out = n->outputs.size();
    return nullptr;
  };
  g_ort.Node_GetOutputs = [](const OrtNode* n, const OrtValueInfo** outputs, size_t count) noexcept -> OrtStatus* {
    for (size_t i = 0; i < count && i < n->outputs.size(); ++i) outputs[i] = n->outputs[i].get();
    return nullptr;
  };
  g_ort.GetValueInfoName = [](const OrtValueInfo* v, const char** out) noexcept -> OrtStatus* {
    *out = v->name.c_str();
    return nullptr;
  };
  g_ort.GetValueInfoTypeInfo = [](const OrtValueInfo* v, const OrtTypeInfo** out) noexcept -> OrtStatus* {
    *out = &v->type_info;
    return nullptr;
  };
  g_ort.CastTypeInfoToTensorInfo = [](const OrtTypeInfo* t, const OrtTensorTypeAndShapeInfo** out) noexcept
      -> OrtStatus* {
    *out = &t->tensor;
    return nullptr;
  };
  g_ort.ValueInfo_IsConstantInitializer = [](const OrtValueInfo* v, bool* out) noexcept -> OrtStatus* {
    *out = v->initializer != nullptr;
    return nullptr;
  };
  g_ort.ValueInfo_GetInitializerValue = [](const OrtValueInfo* v, const OrtValue** out) noexcept -> OrtStatus* {
    *out = v->initializer;  // NULL when the value is not an initializer, like the real call
    return nullptr;
  };
  g_ort.ValueInfo_IsGraphOutput = [](const OrtValueInfo* v, bool* out) noexcept -> OrtStatus* {
    *out = v->is_graph_output;
    return nullptr;
  };
  g_ort.ValueInfo_GetValueNumConsumers = [](const OrtValueInfo* v, size_t* out) noexcept -> OrtStatus* {
    *out = v->consumers.size();
    return nullptr;
  };
  g_ort.ValueInfo_GetValueConsumers = [](const OrtValueInfo* v, const OrtNode** nodes, int64_t* indices,
                                         size_t count) noexcept -> OrtStatus* {
    if (count < v->consumers.size()) return MakeStatus(ORT_INVALID_ARGUMENT, "consumer buffers are too small");
    for (size_t i = 0; i < v->consumers.size(); ++i) {
      nodes[i] = v->consumers[i].first;
      indices[i] = v->consumers[i].second;
    }
    return nullptr;
  };
  g_ort.Node_GetAttributeByName = [](const OrtNode* n, const char* name, const OrtOpAttr** out) noexcept
      -> OrtStatus* {
    *out = nullptr;
    for (const auto& a : n->attrs)
      if (a.name == name) {
        *out = &a;
        return nullptr;
      }
    for (const auto& s : n->schema_attrs)
      if (s == name) return nullptr;  // optional attribute left unset
    return MakeStatus(ORT_NOT_FOUND, "attribute not found");
  };
  g_ort.ReadOpAttr = [](const OrtOpAttr* a, OrtOpAttrType type, void* data, size_t len, size_t* out) noexcept
      -> OrtStatus* {
    if (type == ORT_OP_ATTR_INT && a->kind == 0 && len >= sizeof(int64_t)) {
      *static_cast<int64_t*>(data) = a->value;
      *out = sizeof(int64_t);
      return nullptr;
    }
    if (type == ORT_OP_ATTR_FLOAT && a->kind == 1 && len >= sizeof(float)) {
      *static_cast<float*>(data) = a->f;
      *out = sizeof(float);
      return nullptr;
    }
    if (type == ORT_OP_ATTR_STRING && a->kind == 2) {
      *out = a->s.size();
      if (len < a->s.size()) return MakeStatus(ORT_INVALID_ARGUMENT, "Size of data not large enough to hold the string");
      std::memcpy(data, a->s.data(), a->s.size());  // not NUL-terminated, like the real call
      return nullptr;
    }
    return MakeStatus(ORT_INVALID_ARGUMENT, "bad ReadOpAttr");
  };

  // ---- OrtEpApi
  g_ep.CreateEpDevice = [](OrtEpFactory* f, const OrtHardwareDevice* hw, const OrtKeyValuePairs*,
                           const OrtKeyValuePairs*, OrtEpDevice** out) noexcept -> OrtStatus* {
    *out = new OrtEpDevice{f, hw, {}};
    return nullptr;
  };
  g_ep.ReleaseEpDevice = [](OrtEpDevice* d) noexcept { delete d; };
  g_ep.EpDevice_AddAllocatorInfo = [](OrtEpDevice* d, const OrtMemoryInfo* m) noexcept -> OrtStatus* {
    d->mem_infos.push_back(m);
    return nullptr;
  };
  g_ep.EpGraphSupportInfo_AddSingleNode = [](OrtEpGraphSupportInfo* g, const OrtNode* n) noexcept -> OrtStatus* {
    g->claimed.push_back(n);
    return nullptr;
  };
  g_ep.EpGraphSupportInfo_AddNodesToFuse = [](OrtEpGraphSupportInfo* g, const OrtNode* const* nodes, size_t n,
                                             const OrtNodeFusionOptions* options) noexcept -> OrtStatus* {
    if (n == 0 || nodes == nullptr) return MakeStatus(ORT_INVALID_ARGUMENT, "Must specify a valid array of nodes");
    g->fused.emplace_back(nodes, nodes + n);
    g->fused_drops_constants.push_back(options != nullptr && options->drop_constant_initializers);
    return nullptr;
  };
  g_ep.CreateProfilingEvent = [](OrtProfilingEventCategory category, int32_t pid, int32_t tid, const char* name,
                                 int64_t timestamp_us, int64_t duration_us, const char* const* keys,
                                 const char* const* values, size_t num_args, OrtProfilingEvent** out) noexcept
      -> OrtStatus* {
    if (name == nullptr) return MakeStatus(ORT_INVALID_ARGUMENT, "event_name must not be NULL");
    auto* e = new OrtProfilingEvent{category, pid, tid, name, timestamp_us, duration_us, {}};
    for (size_t i = 0; i < num_args; ++i) e->args.emplace_back(keys[i], values[i]);
    *out = e;
    return nullptr;
  };
  g_ep.ReleaseProfilingEvent = [](OrtProfilingEvent* e) noexcept { delete e; };
  g_ep.ProfilingEventsContainer_AddEvents = [](OrtProfilingEventsContainer* c, const OrtProfilingEvent* const* events,
                                               size_t n) noexcept -> OrtStatus* {
    if (n == 0) return MakeStatus(ORT_INVALID_ARGUMENT, "num_events must be greater than 0");
    for (size_t i = 0; i < n; ++i) c->events.push_back(*events[i]);  // ORT copies the event data
    return nullptr;
  };
  g_ep.EpGraphSupportInfo_LookUpKernel = [](OrtEpGraphSupportInfo* g, const OrtNode* n,
                                            const OrtKernelDef** out) noexcept -> OrtStatus* {
    const auto* e = LookUp(*g->registry, g->ep_name, *n);
    *out = e ? &e->def : nullptr;
    return nullptr;
  };
  g_ep.MemoryInfo_GetMemoryDevice = [](const OrtMemoryInfo* m) noexcept -> const OrtMemoryDevice* { return &m->dev; };
  g_ep.Value_GetMemoryDevice = [](const OrtValue* v) noexcept -> const OrtMemoryDevice* { return &v->mem->dev; };
  g_ep.MemoryDevice_AreEqual = [](const OrtMemoryDevice* a, const OrtMemoryDevice* b) noexcept {
    return a->type == b->type && a->mem_type == b->mem_type && a->vendor == b->vendor &&
           a->device_id == b->device_id;
  };
  g_ep.MemoryDevice_GetDeviceType = [](const OrtMemoryDevice* d) noexcept { return d->type; };
  g_ep.MemoryDevice_GetMemoryType = [](const OrtMemoryDevice* d) noexcept { return d->mem_type; };
  g_ep.MemoryDevice_GetVendorId = [](const OrtMemoryDevice* d) noexcept { return d->vendor; };
  g_ep.MemoryDevice_GetDeviceId = [](const OrtMemoryDevice* d) noexcept { return d->device_id; };
  g_ep.CreateKernelRegistry = [](OrtKernelRegistry** out) noexcept -> OrtStatus* {
    *out = new OrtKernelRegistry{};
    return nullptr;
  };
  g_ep.ReleaseKernelRegistry = [](OrtKernelRegistry* r) noexcept { delete r; };
  g_ep.KernelRegistry_AddKernel = [](OrtKernelRegistry* r, const OrtKernelDef* def, OrtKernelCreateFunc fn,
                                     void* state) noexcept -> OrtStatus* {
    r->entries.push_back({*def, fn, state});
    return nullptr;
  };
  g_ep.CreateKernelDefBuilder = [](OrtKernelDefBuilder** out) noexcept -> OrtStatus* {
    *out = new OrtKernelDefBuilder{};
    return nullptr;
  };
  g_ep.ReleaseKernelDefBuilder = [](OrtKernelDefBuilder* b) noexcept { delete b; };
  g_ep.KernelDefBuilder_SetOperatorType = [](OrtKernelDefBuilder* b, const char* v) noexcept -> OrtStatus* {
    b->def.op = v;
    return nullptr;
  };
  g_ep.KernelDefBuilder_SetDomain = [](OrtKernelDefBuilder* b, const char* v) noexcept -> OrtStatus* {
    b->def.domain = v;
    return nullptr;
  };
  g_ep.KernelDefBuilder_SetSinceVersion = [](OrtKernelDefBuilder* b, int s, int e) noexcept -> OrtStatus* {
    if (s < 1) return MakeStatus(ORT_INVALID_ARGUMENT, "Start version must be >= 1");
    if (e < s) return MakeStatus(ORT_INVALID_ARGUMENT, "End version must be >= to the start version");
    b->def.start = s;
    b->def.end = e;
    return nullptr;
  };
  g_ep.KernelDefBuilder_SetExecutionProvider = [](OrtKernelDefBuilder* b, const char* v) noexcept -> OrtStatus* {
    b->def.ep = v;
    return nullptr;
  };
  g_ep.KernelDefBuilder_SetInputMemType = [](OrtKernelDefBuilder* b, size_t i, OrtMemType t) noexcept -> OrtStatus* {
    b->def.input_mem[i] = t;
    return nullptr;
  };
  g_ep.KernelDefBuilder_SetOutputMemType = [](OrtKernelDefBuilder* b, size_t i, OrtMemType t) noexcept
      -> OrtStatus* {
    b->def.output_mem[i] = t;
    return nullptr;
  };
  g_ep.KernelDefBuilder_AddTypeConstraint = [](OrtKernelDefBuilder* b, const char* name,
                                               const OrtDataType* const* types, size_t n) noexcept -> OrtStatus* {
    auto& v = b->def.constraints[name];
    v.clear();
    for (size_t i = 0; i < n; ++i) v.push_back(types[i]->elem);
    return nullptr;
  };
  g_ep.KernelDefBuilder_Build = [](OrtKernelDefBuilder* b, OrtKernelDef** out) noexcept -> OrtStatus* {
    if (b->def.op.empty() || b->def.ep.empty())
      return MakeStatus(ORT_INVALID_ARGUMENT, "kernel def needs an operator type and an execution provider");
    *out = new OrtKernelDef(b->def);
    return nullptr;
  };
  g_ep.ReleaseKernelDef = [](OrtKernelDef* d) noexcept { delete d; };
  g_ep.GetTensorDataType = [](ONNXTensorElementDataType t, const OrtDataType** out) noexcept -> OrtStatus* {
    if (static_cast<int>(t) < 0 || static_cast<int>(t) >= 32) return MakeStatus(ORT_INVALID_ARGUMENT, "bad type");
    *out = &g_types[static_cast<int>(t)];
    return nullptr;
  };
}

void FillApis() {
  static std::once_flag once;
  std::call_once(once, FillApisOnce);
}

const OrtApi* ORT_API_CALL GetApi(uint32_t version) NO_EXCEPTION {
  return version <= ORT_API_VERSION ? &g_ort : nullptr;
}
const char* ORT_API_CALL GetVersionString(void) NO_EXCEPTION { return "ort-host-shim"; }
const OrtApiBase g_base{GetApi, GetVersionString};

// ------------------------------------------------------------------------------------------- session walk
struct Trace {
  char* buf;
  size_t len;
  size_t used = 0;
  void add(const char* fmt, ...) {
    if (buf == nullptr || used >= len) return;
    va_list ap;
    va_start(ap, fmt);
    int n = vsnprintf(buf + used, len - used, fmt, ap);
    va_end(ap);
    if (n > 0) used += static_cast<size_t>(n) < len - used ? static_cast<size_t>(n) : len - used - 1;
  }
};

struct Plugin {
  void* handle = nullptr;
  CreateEpApiFactoriesFn create = nullptr;
  ReleaseEpApiFactoryFn release = nullptr;
};

Plugin* LoadPlugin(const char* path, std::string* error) {
  static std::mutex mutex;  // sessions may be driven from several test threads
  std::lock_guard<std::mutex> lock(mutex);
  static std::map<std::string, Plugin> loaded;
  auto it = loaded.find(path);
  if (it != loaded.end()) return &it->second;
  Plugin p;
  p.handle = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (p.handle == nullptr) {
    *error = std::string("dlopen failed: ") + dlerror();
    return nullptr;
  }
  p.create = reinterpret_cast<CreateEpApiFactoriesFn>(dlsym(p.handle, "CreateEpFactories"));
  p.release = reinterpret_cast<ReleaseEpApiFactoryFn>(dlsym(p.handle, "ReleaseEpFactory"));
  if (p.create == nullptr || p.release == nullptr) {
    *error = "the library does not export CreateEpFactories / ReleaseEpFactory";
    return nullptr;
  }
  return &(loaded[path] = p);
}

// Set by EpHostProfileNextRun: the next RunNode on this thread drives the plugin's profiler the way ONNX Runtime's
// session profiling does and writes one line per reported event into the buffer.
thread_local char* tl_profile_buf = nullptr;
thread_local size_t tl_profile_len = 0;
// Set by EpHostTimeNextRun: after its functional repeats the next RunNode on this thread calls Compute `warmup` +
// `iters` more times on the same device inputs and reports what one call costs (EpHostLastRunStats).
thread_local int tl_timing_iters = 0;
thread_local int tl_timing_warmup = 0;

// HIP events for the device-side figure of the timing mode, looked up at run time so that this host double links
// against nothing of the GPU stack.
struct HipEvents {
  using Create = int (*)(void**);
  using Record = int (*)(void*, void*);
  using Sync = int (*)(void*);
  using Elapsed = int (*)(float*, void*, void*);
  using Destroy = int (*)(void*);
  Create create = nullptr;
  Record record = nullptr;
  Sync sync = nullptr;
  Elapsed elapsed = nullptr;
  Destroy destroy = nullptr;
  bool ok = false;
  HipEvents() {
    void* h = dlopen("libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
    if (h == nullptr) return;
    create = reinterpret_cast<Create>(dlsym(h, "hipEventCreate"));
    record = reinterpret_cast<Record>(dlsym(h, "hipEventRecord"));
    sync = reinterpret_cast<Sync>(dlsym(h, "hipEventSynchronize"));
    elapsed = reinterpret_cast<Elapsed>(dlsym(h, "hipEventElapsedTime"));
    destroy = reinterpret_cast<Destroy>(dlsym(h, "hipEventDestroy"));
    ok = create && record && sync && elapsed && destroy;
  }
};
constexpr int64_t kProfilingStartOffsetNs = 5000000;  // pretend ORT's profiling began 5 ms before the EP's

int Fail(OrtStatus* st, const char* where, char* err, size_t err_len) {
  int code = st->code == ORT_OK ? ORT_FAIL : static_cast<int>(st->code);
  if (err != nullptr && err_len > 0) snprintf(err, err_len, "%s: %s", where, st->msg.c_str());
  delete st;
  return code;
}

int HostFail(int code, const std::string& msg, char* err, size_t err_len) {
  if (err != nullptr && err_len > 0) snprintf(err, err_len, "%s", msg.c_str());
  return code;
}

}  // namespace

extern "C" {

// One operator input handed in by the test: host data + shape. data == NULL: the optional input is absent.
struct EpHostTensor {
  const void* data;
  const int64_t* dims;
  size_t rank;
  int dtype;  // ONNXTensorElementDataType
};

enum {
  EP_HOST_NOT_CLAIMED = -1,   // GetCapability left the node to the CPU provider
  EP_HOST_LOAD_FAILED = -2,
  EP_HOST_NO_DEVICE = -3,     // the factory offered no OrtEpDevice
  EP_HOST_PROTOCOL = -4,      // the plugin broke an expectation of the host
  EP_HOST_NOT_FUSED = -5      // a MatMulNBits + Add pair was offered and the plugin did not ask to fuse it
};

// Sets (value != NULL) or removes a session configuration entry for the sessions created afterwards.
__attribute__((visibility("default"))) void EpHostSetSessionConfig(const char* key, const char* value) {
  if (value != nullptr)
    SessionConfig()[key] = value;
  else
    SessionConfig().erase(key);
}

// Factory-level queries that need no GPU. Writes "name|vendor|vendor_id|version|num_ep_devices" into `out`.
__attribute__((visibility("default"))) int EpHostProbeFactory(const char* plugin_path, int offer_amd_gpu, char* out,
                                                             size_t out_len, char* err, size_t err_len) {
  FillApis();
  std::string error;
  Plugin* plugin = LoadPlugin(plugin_path, &error);
  if (plugin == nullptr) return HostFail(EP_HOST_LOAD_FAILED, error, err, err_len);
  OrtEpFactory* factory = nullptr;
  size_t n = 0;
  if (OrtStatus* st = plugin->create("mi355x", &g_base, nullptr, &factory, 1, &n))
    return Fail(st, "CreateEpFactories", err, err_len);
  if (n != 1 || factory == nullptr) return HostFail(EP_HOST_PROTOCOL, "expected exactly one factory", err, err_len);
  OrtHardwareDevice cpu{OrtHardwareDeviceType_CPU, 0x8086, 0};
  OrtHardwareDevice nv{OrtHardwareDeviceType_GPU, 0x10DE, 1};
  OrtHardwareDevice amd{OrtHardwareDeviceType_GPU, 0x1002, 0x75A3};
  std::vector<const OrtHardwareDevice*> hw{&cpu, &nv};
  if (offer_amd_gpu) hw.push_back(&amd);
  OrtEpDevice* devs[4] = {nullptr, nullptr, nullptr, nullptr};
  size_t num = 0;
  if (OrtStatus* st = factory->GetSupportedDevices(factory, hw.data(), hw.size(), devs, 4, &num)) {
    plugin->release(factory);
    return Fail(st, "GetSupportedDevices", err, err_len);
  }
  snprintf(out, out_len, "%s|%s|0x%04x|%s|%zu|%d", factory->GetName(factory), factory->GetVendor(factory),
           factory->GetVendorId(factory), factory->GetVersion(factory), num,
           static_cast<int>(factory->IsStreamAware(factory)));
  for (size_t i = 0; i < num; ++i) delete devs[i];
  plugin->release(factory);
  return 0;
}

// One attribute of the node under test.
struct EpHostAttr {
  const char* name;
  int kind;  // 0 int, 1 float, 2 string
  int64_t i;
  float f;
  const char* s;
};

// Description of the node under test: operator, attributes, and for each input its name and type-constraint name.
struct EpHostNodeSpec {
  const char* op_type;
  const EpHostAttr* attrs;
  size_t num_attrs;
  const char* const* schema_attrs;  // every attribute name the operator schema defines
  size_t num_schema_attrs;
  const char* const* input_names;
  const char* const* input_types;
  size_t num_inputs;
  size_t num_outputs;               // outputs of the schema
  int skipped_output_mask;          // bit o: optional output o is not used by the graph
};

// An Add node behind output 0 of the node under test (the graph ONNX Runtime's MatMulNBitsFusion would rewrite).
struct EpHostAddSpec {
  EpHostTensor operand;         // the other Add input
  int operand_is_constant;      // it is a constant initializer
  int product_input_index;      // which Add input (0 or 1) the product feeds
  int product_is_graph_output;  // the product is also a graph output
  int extra_consumer;           // a second node consumes the product as well
};

// One output buffer of the caller.
struct EpHostOutput {
  void* data;
  size_t capacity;
  int64_t dims[8];
  size_t rank;
  int produced;
};

}  // extern "C"

namespace {

// Runs one node through the plugin.  `inputs` has spec.num_inputs entries in operator order; input 0 is the
// activation and is fed per run from host memory through MemcpyFromHost.  Bit i of `constant_mask` marks input i as
// a constant initializer (the host then offers it to PrePackWeight), the other inputs are fed per run as device
// tensors.  Compute is called `repeat` times; the outputs of the last call are copied to `outs`.
// Returns 0, an OrtErrorCode reported by the plugin, or a negative EP_HOST_* code; `trace` receives a short log
// ("claimed=1 prepacked=1,2,3 ...").
//
// With `add` the graph has a second node, Add(product, operand) in either input order.  The plugin is then expected
// to claim both nodes as one group (EpGraphSupportInfo_AddNodesToFuse); the host calls OrtEp::Compile on that group
// and runs the OrtNodeComputeInfo it returns, feeding only the non-constant inputs as ONNX Runtime does when the
// group was fused with drop_constant_initializers.  A pair the plugin leaves un-fused ends with EP_HOST_NOT_FUSED.
int RunNode(const char* plugin_path, const EpHostNodeSpec& spec, const EpHostTensor* inputs, int constant_mask,
            EpHostOutput* outs, int repeat, char* trace_buf, size_t trace_len, char* err, size_t err_len,
            const EpHostAddSpec* add = nullptr) {
  const size_t NI = spec.num_inputs;
  FillApis();
  Trace trace{trace_buf, trace_len};
  if (trace_buf && trace_len) trace_buf[0] = 0;
  std::string error;
  Plugin* plugin = LoadPlugin(plugin_path, &error);
  if (plugin == nullptr) return HostFail(EP_HOST_LOAD_FAILED, error, err, err_len);

  OrtEpFactory* factory = nullptr;
  size_t num_factories = 0;
  if (OrtStatus* st = plugin->create("mi355x", &g_base, nullptr, &factory, 1, &num_factories))
    return Fail(st, "CreateEpFactories", err, err_len);
  struct FactoryGuard {
    Plugin* p;
    OrtEpFactory* f;
    ~FactoryGuard() { p->release(f); }
  } factory_guard{plugin, factory};

  OrtHardwareDevice cpu{OrtHardwareDeviceType_CPU, 0x8086, 0};
  OrtHardwareDevice amd{OrtHardwareDeviceType_GPU, 0x1002, 0x75A3};
  const OrtHardwareDevice* hw[2] = {&cpu, &amd};
  OrtEpDevice* ep_devices[2] = {nullptr, nullptr};
  size_t num_ep_devices = 0;
  if (OrtStatus* st = factory->GetSupportedDevices(factory, hw, 2, ep_devices, 2, &num_ep_devices))
    return Fail(st, "GetSupportedDevices", err, err_len);
  if (num_ep_devices == 0) return HostFail(EP_HOST_NO_DEVICE, "the factory offered no device", err, err_len);
  std::unique_ptr<OrtEpDevice> ep_device(ep_devices[0]);
  const OrtMemoryInfo* device_mem = nullptr;
  for (const OrtMemoryInfo* m : ep_device->mem_infos)
    if (m->dev.mem_type == OrtDeviceMemoryType_DEFAULT) device_mem = m;
  if (device_mem == nullptr) return HostFail(EP_HOST_PROTOCOL, "no default device memory info", err, err_len);
  OrtMemoryInfo cpu_mem{"Cpu", {OrtMemoryInfoDeviceType_CPU, OrtDeviceMemoryType_DEFAULT, 0, 0}, 0, OrtDeviceAllocator};

  OrtEp* ep = nullptr;
  const OrtHardwareDevice* chosen = ep_device->hw;
  const OrtKeyValuePairs* no_meta = nullptr;
  if (OrtStatus* st = factory->CreateEp(factory, &chosen, &no_meta, 1, nullptr, nullptr, &ep))
    return Fail(st, "CreateEp", err, err_len);
  struct EpGuard {
    OrtEpFactory* f;
    OrtEp* e;
    ~EpGuard() { f->ReleaseEp(f, e); }
  } ep_guard{factory, ep};
  const std::string ep_name = ep->GetName(ep);

  // ---- optional: follow the run with the plugin's profiler (OrtEp::CreateProfiler)
  char* profile_buf = tl_profile_buf;
  const size_t profile_len = tl_profile_len;
  tl_profile_buf = nullptr;
  OrtEpProfilerImpl* profiler = nullptr;
  struct ProfilerGuard {
    OrtEpProfilerImpl*& p;
    ~ProfilerGuard() {
      if (p != nullptr) p->Release(p);
    }
  } profiler_guard{profiler};
  if (profile_buf != nullptr) {
    profile_buf[0] = 0;
    if (ep->CreateProfiler == nullptr) return HostFail(EP_HOST_PROTOCOL, "the plugin has no CreateProfiler", err, err_len);
    if (OrtStatus* st = ep->CreateProfiler(ep, &profiler)) return Fail(st, "CreateProfiler", err, err_len);
    if (profiler == nullptr) return HostFail(EP_HOST_PROTOCOL, "CreateProfiler returned NULL", err, err_len);
    if (profiler->ort_version_supported < 25 || profiler->Release == nullptr || profiler->StartProfiling == nullptr ||
        profiler->EndProfiling == nullptr)
      return HostFail(EP_HOST_PROTOCOL, "OrtEpProfilerImpl lacks a required member", err, err_len);
    if (OrtStatus* st = profiler->StartProfiling(profiler, kProfilingStartOffsetNs))
      return Fail(st, "StartProfiling", err, err_len);
  }

  const OrtKernelRegistry* registry = nullptr;
  if (OrtStatus* st = ep->GetKernelRegistry(ep, &registry)) return Fail(st, "GetKernelRegistry", err, err_len);
  if (registry == nullptr) return HostFail(EP_HOST_PROTOCOL, "GetKernelRegistry returned NULL", err, err_len);
  trace.add("kernels=%zu ", registry->entries.size());

  // ---- host views of the caller's tensors (initializers stay host tensors, as in a loaded model)
  auto host_view = [&](const EpHostTensor& t) {
    auto v = std::make_unique<OrtValue>();
    v->dims.assign(t.dims, t.dims + t.rank);
    v->type = static_cast<ONNXTensorElementDataType>(t.dtype);
    v->bytes = ByteSize(v->dims, v->type);
    v->data = const_cast<void*>(t.data);
    v->mem = &cpu_mem;
    return v;
  };
  std::vector<std::unique_ptr<OrtValue>> host_values(NI), device_values(NI);
  for (size_t i = 0; i < NI; ++i)
    if (inputs[i].data != nullptr) host_values[i] = host_view(inputs[i]);
  std::unique_ptr<OrtValue> add_operand_value;
  if (add != nullptr && add->operand.data != nullptr) add_operand_value = host_view(add->operand);

  // ---- the graph: the node under test, optionally followed by an Add
  OrtNode node;
  node.op = spec.op_type;
  node.domain = "com.microsoft";
  node.name = "node0";
  node.since_version = 1;
  for (size_t i = 0; i < spec.num_schema_attrs; ++i) node.schema_attrs.push_back(spec.schema_attrs[i]);
  for (size_t i = 0; i < spec.num_attrs; ++i) {
    OrtOpAttr at;
    at.name = spec.attrs[i].name;
    at.value = spec.attrs[i].i;
    at.kind = spec.attrs[i].kind;
    at.f = spec.attrs[i].f;
    at.s = spec.attrs[i].s ? spec.attrs[i].s : "";
    node.attrs.push_back(at);
  }
  const char* const* kInputNames = spec.input_names;
  const char* const* kInputTypes = spec.input_types;
  size_t last = 0;
  for (size_t i = 0; i < NI; ++i)
    if (inputs[i].data != nullptr || i == 0) last = i;
  for (size_t i = 0; i <= last; ++i) {
    if (inputs[i].data == nullptr && i != 0) {
      node.inputs.emplace_back(nullptr);
      continue;
    }
    node.inputs.emplace_back(new OrtValueInfo{kInputNames[i]});
    if (i != 0 && ((constant_mask >> i) & 1)) node.inputs.back()->initializer = host_values[i].get();
    auto t = static_cast<ONNXTensorElementDataType>(inputs[i].dtype);
    node.inputs.back()->type_info.tensor = {host_values[i]->dims, t};
    auto it = node.types.find(kInputTypes[i]);
    if (it == node.types.end()) node.types[kInputTypes[i]] = t;
  }
  for (size_t o = 0; o < spec.num_outputs; ++o) {
    node.outputs.emplace_back(new OrtValueInfo{"out" + std::to_string(o)});
    node.outputs.back()->is_graph_output = true;
  }
  OrtNode add_node, other_consumer;
  OrtGraph graph;
  graph.nodes.push_back(&node);
  if (add != nullptr) {
    OrtValueInfo& product = *node.outputs[0];
    const int pi = add->product_input_index ? 1 : 0;
    product.is_graph_output = add->product_is_graph_output != 0;
    product.consumers.emplace_back(&add_node, pi);
    if (add->extra_consumer) product.consumers.emplace_back(&other_consumer, 0);
    add_node.op = "Add";
    add_node.domain = "";
    add_node.name = "add0";
    add_node.since_version = 14;
    add_node.inputs.resize(2);
    add_node.inputs[pi].reset(new OrtValueInfo{product.name});
    add_node.inputs[1 - pi].reset(new OrtValueInfo{"add_operand"});
    if (add->operand_is_constant) add_node.inputs[1 - pi]->initializer = add_operand_value.get();
    add_node.outputs.emplace_back(new OrtValueInfo{"sum"});
    add_node.outputs.back()->is_graph_output = true;
    add_node.types["T"] = static_cast<ONNXTensorElementDataType>(inputs[0].dtype);
    graph.nodes.push_back(&add_node);
    if (add->extra_consumer) {
      other_consumer.op = "Identity";
      other_consumer.domain = "";
      other_consumer.name = "identity0";
      other_consumer.since_version = 14;
      other_consumer.inputs.emplace_back(new OrtValueInfo{product.name});
      other_consumer.outputs.emplace_back(new OrtValueInfo{"copy"});
      other_consumer.outputs.back()->is_graph_output = true;
      other_consumer.types["T"] = add_node.types["T"];
      graph.nodes.push_back(&other_consumer);
    }
  }
  OrtEpGraphSupportInfo support{registry, ep_name, {}};
  if (OrtStatus* st = ep->GetCapability(ep, &graph, &support)) return Fail(st, "GetCapability", err, err_len);
  trace.add("claimed=%zu fused=%zu ", support.claimed.size(), support.fused.size());
  if (support.claimed.empty() && support.fused.empty())
    return HostFail(EP_HOST_NOT_CLAIMED, "node not claimed", err, err_len);
  // A node may be claimed once: singly or in one fused group.
  for (const auto& group : support.fused)
    for (const OrtNode* n : group)
      for (const OrtNode* c : support.claimed)
        if (c == n) return HostFail(EP_HOST_PROTOCOL, "a node was claimed both singly and in a fused group", err, err_len);
  const bool compiled = add != nullptr && support.fused.size() == 1 && support.fused[0].size() == 2 &&
                        support.fused[0][0] == &node && support.fused[0][1] == &add_node;
  if (add != nullptr && !compiled) {
    if (!support.fused.empty()) return HostFail(EP_HOST_PROTOCOL, "unexpected fused group", err, err_len);
    return HostFail(EP_HOST_NOT_FUSED, "the MatMulNBits + Add pair was not fused", err, err_len);
  }
  if (add == nullptr && !support.fused.empty())
    return HostFail(EP_HOST_PROTOCOL, "a fused group in a graph of one node", err, err_len);

  // ---- session resources
  OrtAllocator* ep_allocator = nullptr;
  if (OrtStatus* st = ep->CreateAllocator(ep, device_mem, &ep_allocator)) return Fail(st, "CreateAllocator", err, err_len);
  struct AllocGuard {
    OrtEpFactory* f;
    OrtAllocator* a;
    ~AllocGuard() { f->ReleaseAllocator(f, a); }
  } alloc_guard{factory, ep_allocator};
  // every device value below dies before the arena (declared later = destroyed earlier), the arena before the
  // plugin's allocator
  ArenaAllocator arena(ep_allocator);
  OrtAllocator* allocator = &arena;
  struct ValuesGuard {  // device tensors go back to the arena before it is destroyed
    std::vector<std::unique_ptr<OrtValue>>& v;
    ~ValuesGuard() {
      for (auto& x : v) x.reset();
    }
  } values_guard{device_values};
  const int timing_iters = tl_timing_iters, timing_warmup = tl_timing_warmup;
  tl_timing_iters = 0;
  tl_stats = EpHostRunStats{};
  tl_stats.device_us_per_compute = -1.0;
  OrtDataTransferImpl* transfer = nullptr;
  if (OrtStatus* st = factory->CreateDataTransfer(factory, &transfer)) return Fail(st, "CreateDataTransfer", err, err_len);
  struct TransferGuard {
    OrtDataTransferImpl* t;
    ~TransferGuard() { t->Release(t); }
  } transfer_guard{transfer};
  if (!transfer->CanCopy(transfer, &cpu_mem.dev, &device_mem->dev) ||
      !transfer->CanCopy(transfer, &device_mem->dev, &cpu_mem.dev))
    return HostFail(EP_HOST_PROTOCOL, "data transfer refuses host<->device copies", err, err_len);
  OrtSyncStreamImpl* stream_impl = nullptr;
  if (OrtStatus* st = ep->CreateSyncStreamForDevice(ep, &device_mem->dev, &stream_impl))
    return Fail(st, "CreateSyncStreamForDevice", err, err_len);
  struct StreamGuard {
    OrtSyncStreamImpl* s;
    ~StreamGuard() { s->Release(s); }
  } stream_guard{stream_impl};
  OrtSyncStream stream{stream_impl};

  // ---- values. Host copies wrap the caller's memory; constants go to the device through the data transfer.
  auto to_device = [&](size_t i, bool with_stream) -> OrtStatus* {
    auto d = std::make_unique<OrtValue>();
    d->dims = host_values[i]->dims;
    d->type = host_values[i]->type;
    d->bytes = host_values[i]->bytes;
    d->mem = device_mem;
    d->owner = allocator;
    d->data = d->bytes ? allocator->Alloc(allocator, d->bytes) : nullptr;
    if (d->bytes && d->data == nullptr) return MakeStatus(ORT_FAIL, "device allocation failed");
    const OrtValue* src = host_values[i].get();
    OrtValue* dst = d.get();
    OrtSyncStream* s = with_stream ? &stream : nullptr;
    OrtStatus* st = transfer->CopyTensors(transfer, &src, &dst, &s, 1);
    device_values[i] = std::move(d);
    return st;
  };
  for (size_t i = 1; i < NI && !compiled; ++i) {
    if (!host_values[i]) continue;
    // initializers are copied without a stream at session initialisation, run inputs on the run's stream
    if (OrtStatus* st = to_device(i, !((constant_mask >> i) & 1))) return Fail(st, "CopyTensors", err, err_len);
  }

  // ---- the compiled route: OrtEp::Compile on the fused group
  struct ComputeInfoGuard {
    OrtEp* e;
    OrtNodeComputeInfo* info = nullptr;
    void* state = nullptr;
    bool has_state = false;
    ~ComputeInfoGuard() {
      if (info == nullptr) return;
      if (has_state) info->ReleaseState(info, state);
      e->ReleaseNodeComputeInfos(e, &info, 1);
    }
  } compute_info{ep};
  if (compiled) {
    if (!support.fused_drops_constants[0])
      return HostFail(EP_HOST_PROTOCOL, "this host models fused nodes without their constant initializers only", err, err_len);
    if (ep->Compile == nullptr || ep->ReleaseNodeComputeInfos == nullptr)
      return HostFail(EP_HOST_PROTOCOL, "nodes were fused but OrtEp::Compile is not implemented", err, err_len);
    OrtGraph subgraph;
    subgraph.nodes = support.fused[0];
    OrtNode fused_node;
    fused_node.op = ep_name + "_fused_0";
    fused_node.name = fused_node.op;
    fused_node.inputs.emplace_back(new OrtValueInfo{kInputNames[0]});
    fused_node.outputs.emplace_back(new OrtValueInfo{"sum"});
    const OrtGraph* graphs[1] = {&subgraph};
    const OrtNode* fused_nodes[1] = {&fused_node};
    OrtNodeComputeInfo* infos[1] = {nullptr};
    OrtNode* ep_context_nodes[1] = {nullptr};
    if (OrtStatus* st = ep->Compile(ep, graphs, fused_nodes, 1, infos, ep_context_nodes)) return Fail(st, "Compile", err, err_len);
    if (infos[0] == nullptr) return HostFail(EP_HOST_PROTOCOL, "Compile returned no OrtNodeComputeInfo", err, err_len);
    compute_info.info = infos[0];
    OrtNodeComputeContext node_context{fused_node.name};
    if (OrtStatus* st = infos[0]->CreateState(infos[0], &node_context, &compute_info.state))
      return Fail(st, "CreateState", err, err_len);
    compute_info.has_state = true;
    trace.add("compiled=1 ");
  }

  // ---- kernel creation + PrePack
  struct KernelGuard {
    OrtKernelImpl* k;
    ~KernelGuard() {
      if (k != nullptr) k->Release(k);
    }
  };
  const auto* entry = compiled ? nullptr : LookUp(*registry, ep_name, node);
  if (!compiled && entry == nullptr) return HostFail(EP_HOST_PROTOCOL, "claimed node without a kernel", err, err_len);
  // inputs the kernel definition wants in host memory (OrtMemTypeCPUInput) are never copied to the device
  auto wants_host = [&](size_t i) {
    if (entry == nullptr) return false;
    auto it = entry->def.input_mem.find(i);
    return it != entry->def.input_mem.end() && it->second == OrtMemTypeCPUInput;
  };
  for (size_t i = 1; i < NI; ++i)
    if (device_values[i] && wants_host(i)) device_values[i].reset();
  auto fed_value = [&](size_t i) -> const OrtValue* {
    return wants_host(i) ? host_values[i].get() : device_values[i].get();
  };
  OrtKernelInfo info{&node, {}};
  for (size_t i = 1; i < NI; ++i)
    if (fed_value(i) && ((constant_mask >> i) & 1)) info.constants[i] = fed_value(i);
  OrtKernelImpl* kernel = nullptr;
  if (!compiled) {
    if (OrtStatus* st = entry->fn(entry->state, &info, &kernel)) return Fail(st, "kernel creation", err, err_len);
    if (kernel == nullptr) return HostFail(EP_HOST_PROTOCOL, "kernel creation returned NULL", err, err_len);
  }
  KernelGuard kernel_guard{kernel};
  if (kernel != nullptr && kernel->flags != 0)
    return HostFail(EP_HOST_PROTOCOL, "OrtKernelImpl::flags must start as 0", err, err_len);
  trace.add("prepacked=");
  std::vector<bool> packed(NI, false);
  if (kernel != nullptr && kernel->PrePackWeight != nullptr) {
    for (size_t i = 1; i < NI; ++i) {
      if (!info.constants.count(i)) continue;
      bool is_packed = false;
      if (OrtStatus* st = kernel->PrePackWeight(kernel, fed_value(i), static_cast<int>(i), allocator, nullptr,
                                                &is_packed))
        return Fail(st, "PrePackWeight", err, err_len);
      packed[i] = is_packed;
      if (is_packed) trace.add("%zu,", i);
    }
    // Like ONNX Runtime, drop the initializers the kernel took over - after all PrePack calls of the node.
    for (size_t i = 1; i < NI; ++i)
      if (packed[i]) device_values[i].reset();
  }
  std::vector<bool> dropped = packed;  // initializers the kernel took over are gone, host-side ones included
  trace.add(" ");

  // ---- Memcpy kernels around the node
  auto memcpy_kernel = [&](const char* op, ONNXTensorElementDataType t, OrtKernelImpl** out) -> OrtStatus* {
    OrtNode n;
    n.op = op;
    n.domain = "";
    n.since_version = 1;
    n.inputs.emplace_back(new OrtValueInfo{"X"});
    n.types["T"] = t;
    const auto* e = LookUp(*registry, ep_name, n);
    if (e == nullptr) return MakeStatus(ORT_FAIL, (std::string("no kernel registered for ") + op).c_str());
    OrtKernelInfo ki{&n, {}};
    return e->fn(e->state, &ki, out);
  };

  int rc = 0;
  for (int r = 0; r < (repeat < 1 ? 1 : repeat) && rc == 0; ++r) {
    // A: host -> device through MemcpyFromHost
    OrtKernelImpl* from_host = nullptr;
    if (OrtStatus* st = memcpy_kernel("MemcpyFromHost", host_values[0]->type, &from_host))
      return Fail(st, "MemcpyFromHost creation", err, err_len);
    KernelGuard from_guard{from_host};
    OrtKernelContext copy_in{{host_values[0].get()}, {}, {false}, allocator, &cpu_mem, &stream};
    copy_in.outputs.resize(1);
    if (OrtStatus* st = from_host->Compute(from_host, &copy_in)) return Fail(st, "MemcpyFromHost", err, err_len);

    OrtKernelContext ctx{{}, {}, {}, allocator, &cpu_mem, &stream};
    ctx.outputs.resize(spec.num_outputs);
    ctx.output_on_host.assign(spec.num_outputs, false);
    ctx.output_skipped.assign(spec.num_outputs, false);
    for (size_t o = 0; o < spec.num_outputs; ++o) ctx.output_skipped[o] = (spec.skipped_output_mask >> o) & 1;
    const uint64_t correlation = 1700000000000000ull + static_cast<uint64_t>(r);  // epoch-based, like ORT's
    if (profiler != nullptr && profiler->StartEvent != nullptr)
      if (OrtStatus* st = profiler->StartEvent(profiler, correlation)) return Fail(st, "StartEvent", err, err_len);
    struct EventGuard {
      OrtEpProfilerImpl* p;
      uint64_t id;
      ~EventGuard() {
        if (p == nullptr || p->StopEvent == nullptr) return;
        OrtProfilingEvent node_event{OrtProfilingEventCategory_NODE, -1, -1, "node0_kernel_time", 0, 0, {}};
        if (OrtStatus* st = p->StopEvent(p, id, &node_event)) delete st;
      }
    } event_guard{profiler, correlation};
    if (compiled) {
      ctx.inputs.assign(1, copy_in.outputs[0].get());  // the fused node's only non-constant input
      if (OrtStatus* st = compute_info.info->Compute(compute_info.info, compute_info.state, &ctx))
        return Fail(st, "compiled Compute", err, err_len);
    } else {
      ctx.inputs.assign(node.inputs.size(), nullptr);
      ctx.inputs[0] = copy_in.outputs[0].get();
      for (size_t i = 1; i < node.inputs.size(); ++i)
        if (!dropped[i] && fed_value(i)) ctx.inputs[i] = fed_value(i);
      if (OrtStatus* st = kernel->Compute(kernel, &ctx)) return Fail(st, "Compute", err, err_len);
    }
    for (size_t o = 0; o < spec.num_outputs; ++o) {
      outs[o].produced = 0;
      if (ctx.output_skipped[o]) continue;
      if (!ctx.outputs[o]) return HostFail(EP_HOST_PROTOCOL, "Compute produced no output", err, err_len);
      OrtKernelImpl* to_host = nullptr;
      if (OrtStatus* st = memcpy_kernel("MemcpyToHost", ctx.outputs[o]->type, &to_host))
        return Fail(st, "MemcpyToHost creation", err, err_len);
      KernelGuard to_guard{to_host};
      OrtKernelContext copy_out{{ctx.outputs[o].get()}, {}, {true}, allocator, &cpu_mem, &stream};
      copy_out.outputs.resize(1);
      if (OrtStatus* st = to_host->Compute(to_host, &copy_out)) return Fail(st, "MemcpyToHost", err, err_len);
      if (OrtStatus* st = stream_impl->Flush(stream_impl)) return Fail(st, "stream Flush", err, err_len);
      const OrtValue& out = *copy_out.outputs[0];
      if (out.bytes > outs[o].capacity)
        return HostFail(EP_HOST_PROTOCOL, "output larger than the caller's buffer", err, err_len);
      if (out.bytes) std::memcpy(outs[o].data, out.data, out.bytes);
      outs[o].rank = out.dims.size() < 8 ? out.dims.size() : 8;
      for (size_t i = 0; i < outs[o].rank; ++i) outs[o].dims[i] = out.dims[i];
      outs[o].produced = 1;
    }
  }
  // ---- timing mode: the cost of one Compute call as ONNX Runtime's executor sees it.  The activation stays on the
  // device (what the previous node would have produced), every call gets a fresh context whose output comes from the
  // arena, and nothing synchronises between the calls.
  if (rc == 0 && timing_iters > 0) {
    OrtKernelImpl* from_host = nullptr;
    if (OrtStatus* st = memcpy_kernel("MemcpyFromHost", host_values[0]->type, &from_host))
      return Fail(st, "MemcpyFromHost creation", err, err_len);
    KernelGuard from_guard{from_host};
    OrtKernelContext copy_in{{host_values[0].get()}, {}, {false}, allocator, &cpu_mem, &stream};
    copy_in.outputs.resize(1);
    if (OrtStatus* st = from_host->Compute(from_host, &copy_in)) return Fail(st, "MemcpyFromHost", err, err_len);
    auto one_compute = [&]() -> OrtStatus* {
      OrtKernelContext ctx{{}, {}, {}, allocator, &cpu_mem, &stream};
      ctx.outputs.resize(spec.num_outputs);
      ctx.output_on_host.assign(spec.num_outputs, false);
      ctx.output_skipped.assign(spec.num_outputs, false);
      for (size_t o = 0; o < spec.num_outputs; ++o) ctx.output_skipped[o] = (spec.skipped_output_mask >> o) & 1;
      if (compiled) {
        ctx.inputs.assign(1, copy_in.outputs[0].get());
        return compute_info.info->Compute(compute_info.info, compute_info.state, &ctx);
      }
      ctx.inputs.assign(node.inputs.size(), nullptr);
      ctx.inputs[0] = copy_in.outputs[0].get();
      for (size_t i = 1; i < node.inputs.size(); ++i)
        if (!dropped[i] && fed_value(i)) ctx.inputs[i] = fed_value(i);
      return kernel->Compute(kernel, &ctx);
    };
    for (int i = 0; i < timing_warmup; ++i)
      if (OrtStatus* st = one_compute()) return Fail(st, "Compute (warm-up)", err, err_len);
    if (OrtStatus* st = stream_impl->Flush(stream_impl)) return Fail(st, "stream Flush", err, err_len);
    static HipEvents hip;
    void* e0 = nullptr;
    void* e1 = nullptr;
    void* handle = stream_impl->GetHandle(stream_impl);
    const bool events = hip.ok && hip.create(&e0) == 0 && hip.create(&e1) == 0;
    const uint64_t ep_allocs_before = tl_stats.ep_allocs;
    const auto t0 = std::chrono::steady_clock::now();
    if (events) hip.record(e0, handle);
    for (int i = 0; i < timing_iters; ++i)
      if (OrtStatus* st = one_compute()) return Fail(st, "Compute (timed)", err, err_len);
    if (events) hip.record(e1, handle);
    const auto t1 = std::chrono::steady_clock::now();
    if (OrtStatus* st = stream_impl->Flush(stream_impl)) return Fail(st, "stream Flush", err, err_len);
    const auto t2 = std::chrono::steady_clock::now();
    tl_stats.timed_computes = static_cast<uint64_t>(timing_iters);
    tl_stats.host_us_per_compute = std::chrono::duration<double, std::micro>(t1 - t0).count() / timing_iters;
    tl_stats.wall_us_per_compute = std::chrono::duration<double, std::micro>(t2 - t0).count() / timing_iters;
    if (events) {
      float ms = 0.f;
      if (hip.sync(e1) == 0 && hip.elapsed(&ms, e0, e1) == 0) tl_stats.device_us_per_compute = ms * 1e3 / timing_iters;
      hip.destroy(e0);
      hip.destroy(e1);
    }
    trace.add("timed=%d ep_allocs_while_timed=%llu ", timing_iters,
              static_cast<unsigned long long>(tl_stats.ep_allocs - ep_allocs_before));
  }
  if (profiler != nullptr) {
    OrtProfilingEventsContainer container;
    if (OrtStatus* st = profiler->EndProfiling(profiler, &container)) return Fail(st, "EndProfiling", err, err_len);
    size_t used = 0;
    for (const auto& e : container.events) {
      std::string line = std::to_string(static_cast<int>(e.category)) + "|" + e.name + "|" +
                         std::to_string(e.timestamp_us) + "|" + std::to_string(e.duration_us);
      for (const auto& kv : e.args) line += "|" + kv.first + "=" + kv.second;
      line += "\n";
      if (used + line.size() + 1 > profile_len) break;
      std::memcpy(profile_buf + used, line.c_str(), line.size() + 1);
      used += line.size();
    }
  }
  if (OrtStatus* st = ep->Sync(ep)) return Fail(st, "OrtEp::Sync", err, err_len);
  bool concurrent = false;
  if (OrtStatus* st = ep->IsConcurrentRunSupported(ep, &concurrent)) return Fail(st, "IsConcurrentRunSupported", err, err_len);
  trace.add("concurrent=%d", static_cast<int>(concurrent));
  return rc;
}

}  // namespace

extern "C" {

// The next EpHostRun* call on the calling thread is profiled: CreateProfiler, StartProfiling, StartEvent / StopEvent
// around every Compute, EndProfiling; `buf` receives "category|name|timestamp_us|duration_us|key=value..." lines.
__attribute__((visibility("default"))) void EpHostProfileNextRun(char* buf, size_t len) {
  tl_profile_buf = len > 0 ? buf : nullptr;
  tl_profile_len = len;
}

// The next EpHostRun* call on the calling thread ends with `warmup` untimed and `iters` timed Compute calls on
// device-resident inputs; EpHostLastRunStats then holds what one call cost.
__attribute__((visibility("default"))) void EpHostTimeNextRun(int warmup, int iters) {
  tl_timing_warmup = warmup;
  tl_timing_iters = iters;
}

// How the next sessions on this thread answer KernelContext_GetScratchBuffer: 0 serve (default), 1 fail with a
// status, 2 succeed with a NULL buffer, 3 return a buffer that is only 64-byte aligned.
__attribute__((visibility("default"))) void EpHostSetScratchMode(int mode) { tl_scratch_mode = mode; }

// Allocator and scratch statistics (and the timing figures) of the last EpHostRun* call on the calling thread.
__attribute__((visibility("default"))) void EpHostLastRunStats(EpHostRunStats* out) { *out = tl_stats; }

// Any operator of the com.microsoft domain the plugin registers (MatMulNBitsMlp, MatMulNBitsQkv, ...).
__attribute__((visibility("default"))) int EpHostRunNode(const char* plugin_path, const EpHostNodeSpec* spec,
                                                        const EpHostTensor* inputs, int constant_mask,
                                                        EpHostOutput* outs, int repeat, char* trace_buf,
                                                        size_t trace_len, char* err, size_t err_len) {
  return RunNode(plugin_path, *spec, inputs, constant_mask, outs, repeat, trace_buf, trace_len, err, err_len);
}

// com.microsoft::MatMulNBits followed by Add(product, operand): the pair the plugin is expected to fuse and compile.
// `inputs` as for EpHostRunMatMulNBits; the sum is copied to `y`.
__attribute__((visibility("default"))) int EpHostRunMatMulNBitsAdd(
    const char* plugin_path, int64_t N, int64_t K, int64_t bits, int64_t block_size, const EpHostTensor* inputs,
    int constant_mask, const EpHostAddSpec* add, void* y, size_t y_bytes, int64_t* y_dims, size_t* y_rank, int repeat,
    char* trace_buf, size_t trace_len, char* err, size_t err_len) {
  const EpHostAttr attrs[4] = {{"K", 0, K, 0.f, nullptr},
                               {"N", 0, N, 0.f, nullptr},
                               {"bits", 0, bits, 0.f, nullptr},
                               {"block_size", 0, block_size, 0.f, nullptr}};
  static const char* kSchemaAttrs[5] = {"K", "N", "bits", "block_size", "accuracy_level"};
  static const char* kInputNames[6] = {"A", "B", "scales", "zero_points", "g_idx", "bias"};
  static const char* kInputTypes[6] = {"T1", "T2", "T1", "T3", "T4", "T1"};
  const EpHostNodeSpec spec{"MatMulNBits", attrs, 4, kSchemaAttrs, 5, kInputNames, kInputTypes, 6, 1, 0};
  EpHostOutput out{};
  out.data = y;
  out.capacity = y_bytes;
  const int rc =
      RunNode(plugin_path, spec, inputs, constant_mask, &out, repeat, trace_buf, trace_len, err, err_len, add);
  if (rc == 0) {
    *y_rank = out.rank;
    for (size_t i = 0; i < out.rank; ++i) y_dims[i] = out.dims[i];
  }
  return rc;
}

// One com.microsoft::MatMulNBits node; `inputs` has six entries (A, B, scales, zero_points, g_idx, bias).  The result
// of the last Compute call is copied to `y` (y_bytes capacity) and its shape to y_dims / y_rank (capacity 8).
__attribute__((visibility("default"))) int EpHostRunMatMulNBits(
    const char* plugin_path, int64_t N, int64_t K, int64_t bits, int64_t block_size, int64_t accuracy_level,
    const EpHostTensor* inputs, int constant_mask, void* y, size_t y_bytes, int64_t* y_dims, size_t* y_rank,
    int repeat, char* trace_buf, size_t trace_len, char* err, size_t err_len) {
  const EpHostAttr attrs[5] = {{"K", 0, K, 0.f, nullptr},
                               {"N", 0, N, 0.f, nullptr},
                               {"bits", 0, bits, 0.f, nullptr},
                               {"block_size", 0, block_size, 0.f, nullptr},
                               {"accuracy_level", 0, accuracy_level, 0.f, nullptr}};
  static const char* kSchemaAttrs[5] = {"K", "N", "bits", "block_size", "accuracy_level"};
  static const char* kInputNames[6] = {"A", "B", "scales", "zero_points", "g_idx", "bias"};
  static const char* kInputTypes[6] = {"T1", "T2", "T1", "T3", "T4", "T1"};
  const EpHostNodeSpec spec{"MatMulNBits", attrs, 5, kSchemaAttrs, 5, kInputNames, kInputTypes, 6, 1, 0};
  EpHostOutput out{};
  out.data = y;
  out.capacity = y_bytes;
  const int rc = RunNode(plugin_path, spec, inputs, constant_mask, &out, repeat, trace_buf, trace_len, err, err_len);
  if (rc == 0) {
    *y_rank = out.rank;
    for (size_t i = 0; i < out.rank; ++i) y_dims[i] = out.dims[i];
  }
  return rc;
}

}  // extern "C"
